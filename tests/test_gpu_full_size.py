"""The five BASELINE configurations at their full sizes, and two tensors whose codes exceed the Infinity Cache.

The CPU oracle checks a band of rows of each tensor bit for bit; the whole tensor
is checked through properties that do not depend on size:
  * out_scale == the scale rule applied to an independent torch abs-max reduction;
  * fused dynamic quantize == compute_scales + quantize (codes and scales, all words);
  * every code lies in the value's range, dequant == F(scale*code) by independent torch arithmetic,
    and |dequant - x| <= scale/2 (+ the rounding of quotient and product in 16-bit types);
  * quantize(dequantize(codes)) with the same scales returns the same codes (idempotence);
  * dequantize is linear in the scales: doubling every (power-of-two exact) scale doubles the output.
"""
import numpy as np
import pytest

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef)
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu

CONFIGS = [
    ("cfg1", (1024, 1024), ElemType.F32, QuantValue.Q8S, None, "normal1", 1),
    ("cfg2", (4096, 4096), ElemType.BF16, QuantValue.Q8S, 32, "normal_outliers", 2),
    ("cfg3", (14336, 4096), ElemType.BF16, QuantValue.Q4S, 32, "normal", 3),
    ("cfg4", (8192, 8192), ElemType.F32, QuantValue.Q2S, 64, "laplace", 4),
    ("cfg5", (28672, 8192), ElemType.BF16, QuantValue.E2M1, 32, "normal_t3", 5),
    # codes + scales above 192 MiB: the quantize kernels stream such outputs past the caches, where the five
    # configurations above (and every small test) write theirs through to the Infinity Cache
    ("large_output_block32", (16384, 12800), ElemType.BF16, QuantValue.Q8S, 32, "normal", 6),
    ("large_output_per_tensor", (16384, 12800), ElemType.BF16, QuantValue.Q8S, None, "normal1", 7),
]


def _unpack_codes(torch, codes, bits):
    """int32 words [rows, cols/nq] -> int32 codes [rows, cols] (sign-extended fields)."""
    nq = 32 // bits
    shifts = torch.arange(nq, device=codes.device, dtype=torch.int32) * bits
    fields = (codes.unsqueeze(-1) >> shifts) & ((1 << bits) - 1)
    fields = torch.where(fields >= (1 << (bits - 1)), fields - (1 << bits), fields)
    return fields.reshape(codes.shape[0], -1)


@pytest.mark.parametrize("name,shape,elem,value,block,dist,seed", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_full_size_config(oracle, name, shape, elem, value, block, dist, seed):
    import torch

    import bench

    w = dict(shape=shape, elem=elem.name, value=value.name, block=block, dist=dist, seed=seed)
    x = bench.make_input(torch, w)
    rows, cols = shape
    level = QuantLevel.Tensor if block is None else QuantLevel.block([block])
    scheme = QuantScheme.default().with_value(value).with_level(level)
    lo, hi = value.range()
    bits = value.size_bits()
    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    sshape = scheme.scales_shape(shape)
    codes = torch.zeros(scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
    scales = torch.zeros(sshape, dtype=torch.float32, device="cuda")
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")

    print(f"{name}: dynamic quantize", flush=True)
    qz.launch_dynamic(client, h(x), h(codes), h(scales), scheme, elem, ws.data_ptr(), 1024)
    torch.cuda.synchronize()

    # --- scales against an independent reduction (torch), same f32 formula
    xf = x.float()
    if block is None:
        amax = xf.abs().max().reshape(1)
    else:
        amax = xf.abs().reshape(rows, cols // block, block).amax(dim=2)
    want = (2.0 * amax) / (hi - lo)
    if elem != ElemType.F32:
        want = want.to(x.dtype).float()  # the scale is rounded to the input type first
    assert torch.equal(scales.reshape(want.shape), want)

    # --- two-step path gives the same words and scales
    print(f"{name}: compute_scales + quantize", flush=True)
    in_scales = torch.zeros(sshape, dtype=x.dtype, device="cuda")
    qz.compute_scales(client, h(x), h(in_scales), scheme, elem, ws.data_ptr(), 1024)
    codes2 = torch.zeros_like(codes)
    scales2 = torch.zeros_like(scales)
    qz.launch_ref(client, h(x), h(codes2), h(in_scales), h(scales2), scheme, elem)
    torch.cuda.synchronize()
    assert torch.equal(codes, codes2) and torch.equal(scales, scales2)

    # --- oracle on a band of rows (first, middle, last), bit for bit
    band = max(1, min(rows // 3, (1 << 20) // cols))
    if block is not None:
        for r0 in (0, rows // 2, rows - band):
            xs = x[r0:r0 + band].contiguous()
            xs_np = xs.cpu().numpy() if elem == ElemType.F32 else xs.view(torch.int16).cpu().numpy().view(np.uint16)
            s_ref = oracle.compute_scales(xs_np, elem, (band, cols), scheme)
            w_ref, os_ref = oracle.quantize(xs_np, elem, (band, cols), s_ref, scheme, threads=8)
            assert np.array_equal(codes[r0:r0 + band].cpu().numpy().view(np.uint32), w_ref)
            assert np.array_equal(scales[r0:r0 + band].cpu().numpy().reshape(-1), os_ref.reshape(-1))
    else:
        x_np = x.cpu().numpy() if elem == ElemType.F32 else x.view(torch.int16).cpu().numpy().view(np.uint16)
        s_ref = oracle.compute_scales(x_np, elem, shape, scheme)
        w_ref, os_ref = oracle.quantize(x_np, elem, shape, s_ref, scheme, threads=8)
        assert np.array_equal(codes.cpu().numpy().view(np.uint32), w_ref)
        assert np.array_equal(scales.cpu().numpy().reshape(-1), os_ref.reshape(-1))

    # --- dequantize, range and error bound over the whole tensor
    print(f"{name}: dequantize", flush=True)
    y = torch.zeros_like(x)
    dq.launch_ref(client, h(codes), h(y), h(scales), scheme, elem)
    torch.cuda.synchronize()
    c = _unpack_codes(torch, codes, bits)
    assert int(c.min()) >= lo and int(c.max()) <= hi
    s_full = scales.reshape(1, 1).expand(rows, cols) if block is None else scales.repeat_interleave(block, dim=1)
    # y == F(scale * code) exactly (independent torch arithmetic in the tensor's dtype)
    assert torch.equal(y, (s_full.to(x.dtype) * c.to(x.dtype)))
    err = (y.float() - xf).abs()
    # f32: the reference's bound, scale/2*(1+1e-4).  bf16 computes the quotient and the product
    # in the tensor's type (8 significant bits): with P = the power of two above |q|max, the
    # quotient is off by up to P*2^-9 steps and the product by up to |q|*2^-8 <= 2*P*2^-9 steps.
    pow2 = 2.0 ** np.ceil(np.log2(max(abs(lo), abs(hi))))
    bound = s_full * (0.5 * (1 + 1e-4) if elem == ElemType.F32 else 0.5 + 3 * pow2 * 2.0 ** -9)
    assert bool((err <= bound + 1e-30).all())
    del err, c

    # --- idempotence: quantizing the dequantized tensor with the same scales is a fixed point
    print(f"{name}: idempotence + linearity", flush=True)
    codes3 = torch.zeros_like(codes)
    qz.launch_ref(client, h(y), h(codes3), h(in_scales), h(scales2), scheme, elem)
    torch.cuda.synchronize()
    assert torch.equal(codes3, codes)

    # --- linearity in the scales: doubling is exact in binary floating point
    y2 = torch.zeros_like(x)
    scales_x2 = scales * 2.0
    dq.launch_ref(client, h(codes), h(y2), h(scales_x2), scheme, elem)
    torch.cuda.synchronize()
    assert torch.equal(y2.float(), y.float() * 2.0)
