"""A tensor whose byte offsets do not fit 32 bits (bf16 [36864, 65536]: 2.4 G elements, 4.8 GB).

Every kernel family has to carry 64-bit offsets through: the flat kernels (contiguous), the row
kernels (pitched rows), the transposed kernels, the reductions.  The CPU oracle checks bands of rows
at the start, in the middle and at the very end (beyond 4 GiB); whole-tensor checks are equalities
between independent GPU paths and torch reductions."""
import numpy as np
import pytest

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef)
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz
from cubek_amd import reduce as cq_reduce

pytestmark = pytest.mark.gpu
ROWS, COLS, BLOCK = 36864, 65536, 32
ELEM = ElemType.BF16


def bits_of(t):
    import torch

    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def test_offsets_beyond_32_bits(oracle):
    import torch

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([BLOCK]))
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    x = torch.empty((ROWS, COLS), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, ROWS, 2048):  # chunked: bounds the f32 temporary
        x[r0:r0 + 2048] = torch.randn((2048, COLS), generator=g, device="cuda").mul_(0.03).to(torch.bfloat16)
    assert x.numel() * 2 > 1 << 32

    print("contiguous: fused dynamic quantize, two-step, dequantize", flush=True)
    codes = torch.zeros((ROWS, COLS // 8), dtype=torch.int32, device="cuda")
    scales = torch.zeros((ROWS, COLS // BLOCK), dtype=torch.float32, device="cuda")
    qz.launch_dynamic(client, h(x), h(codes), h(scales), scheme, ELEM)
    in_scales = torch.zeros((ROWS, COLS // BLOCK), dtype=torch.bfloat16, device="cuda")
    qz.compute_scales(client, h(x), h(in_scales), scheme, ELEM)
    codes2 = torch.zeros_like(codes)
    scales2 = torch.zeros_like(scales)
    qz.launch_ref(client, h(x), h(codes2), h(in_scales), h(scales2), scheme, ELEM)
    y = torch.zeros_like(x)
    dq.launch_ref(client, h(codes), h(y), h(scales), scheme, ELEM)
    torch.cuda.synchronize()
    assert torch.equal(codes, codes2) and torch.equal(scales, scales2)
    del codes2, scales2

    band = 16
    refs = {}
    for r0 in (0, ROWS // 2, ROWS - band):
        xs = bits_of(x[r0:r0 + band])
        s_ref = oracle.compute_scales(xs, ELEM, (band, COLS), scheme)
        w_ref, os_ref = oracle.quantize(xs, ELEM, (band, COLS), s_ref, scheme, threads=8)
        y_ref = oracle.dequantize(w_ref, (band, COLS), os_ref, ELEM, scheme)
        refs[r0] = (w_ref, os_ref, y_ref)
        assert np.array_equal(codes[r0:r0 + band].cpu().numpy().view(np.uint32), w_ref), r0
        assert np.array_equal(scales[r0:r0 + band].cpu().numpy().reshape(-1), os_ref.reshape(-1)), r0
        assert np.array_equal(bits_of(y[r0:r0 + band]).reshape(-1), y_ref.reshape(-1)), r0

    print("reductions against torch", flush=True)
    for axis in (0, 1):
        out = torch.zeros((1, COLS) if axis == 0 else (ROWS, 1), dtype=torch.bfloat16, device="cuda")
        nbytes = cq_reduce.workspace_bytes(h(x), axis, ELEM)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        cq_reduce.max_abs(client, h(x), h(out), axis, ELEM, ws.data_ptr() if nbytes else 0, nbytes)
        torch.cuda.synchronize()
        want = torch.stack([x[r0:r0 + 4096].abs().amax(dim=axis, keepdim=True) for r0 in range(0, ROWS, 4096)])
        want = want.amax(dim=0) if axis == 0 else want.reshape(ROWS, 1)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), axis
        del out, ws, want

    print("pitched rows (row kernels)", flush=True)
    pc = COLS - 64  # the view [ROWS, COLS - 64] of the same buffer: rows keep their pitch
    hx = TensorHandleRef(h(x).handle, (ROWS, pc), (COLS, 1), 2)
    pcodes = torch.zeros((ROWS, pc // 8), dtype=torch.int32, device="cuda")
    pscales = torch.zeros((ROWS, pc // BLOCK), dtype=torch.float32, device="cuda")
    qz.launch_dynamic(client, hx, h(pcodes), h(pscales), scheme, ELEM)
    py = torch.full((ROWS, COLS), 7.0, dtype=torch.bfloat16, device="cuda")
    dq.launch_ref(client, h(pcodes), TensorHandleRef(h(py).handle, (ROWS, pc), (COLS, 1), 2), h(pscales), scheme, ELEM)
    torch.cuda.synchronize()
    assert torch.equal(pcodes, codes[:, :pc // 8]) and torch.equal(pscales, scales[:, :pc // BLOCK])
    assert torch.equal(py[:, :pc].view(torch.int16), y[:, :pc].view(torch.int16))
    assert bool((py[:, pc:] == 7.0).all())
    del pcodes, pscales, py

    print("transposed floats", flush=True)
    xt = torch.empty((COLS, ROWS), dtype=torch.bfloat16, device="cuda")
    for c0 in range(0, COLS, 8192):
        xt[c0:c0 + 8192] = x[:, c0:c0 + 8192].t()
    hxt = TensorHandleRef(h(xt).handle, (ROWS, COLS), (1, ROWS), 2)
    tcodes = torch.zeros_like(codes)
    tscales = torch.zeros_like(scales)
    qz.launch_dynamic(client, hxt, h(tcodes), h(tscales), scheme, ELEM)
    torch.cuda.synchronize()
    assert torch.equal(tcodes, codes) and torch.equal(tscales, scales)
    del tcodes, tscales
    xt.fill_(7.0)
    dq.launch_ref(client, h(codes), hxt, h(scales), scheme, ELEM)
    torch.cuda.synchronize()
    for c0 in range(0, COLS, 8192):
        assert torch.equal(xt[c0:c0 + 8192].t().contiguous().view(torch.int16),
                           y[:, c0:c0 + 8192].contiguous().view(torch.int16)), c0
