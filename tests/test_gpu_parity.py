"""Parity of the HIP path (through the C ABI) with the CPU oracle and with the
committed exact-rational fixtures.  Integer codes, scales and dequantized bits
must be identical; the only tolerance anywhere is NaN payloads (NaN == NaN)."""
import numpy as np
import pytest

import golden_cases as gc
from cubek_amd import (ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue)

pytestmark = pytest.mark.gpu

RAMPS = gc.load("ref_ramps.npz")
TYPED = gc.load("typed_small.npz")
NATIVE = gc.load("typed_native.npz")
ALL_VALUES = list(QuantValue)
INT_VALUES = [QuantValue.Q8F, QuantValue.Q8S, QuantValue.Q4F, QuantValue.Q4S, QuantValue.Q2F, QuantValue.Q2S]
ELEMS = [ElemType.F32, ElemType.BF16, ElemType.F16]


@pytest.fixture(scope="module")
def gpu():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a device"
    import gpu_harness

    return gpu_harness


def same_floats(a, b, elem):
    """Bit equality, except that any NaN matches any NaN."""
    a = np.ascontiguousarray(a).reshape(-1)
    b = np.ascontiguousarray(b).reshape(-1)
    if a.dtype == np.float32:
        a, b = a.view(np.uint32), np.ascontiguousarray(b, dtype=np.float32).view(np.uint32)
        nan_a, nan_b = (a & 0x7FFFFFFF) > 0x7F800000, (b & 0x7FFFFFFF) > 0x7F800000
    elif elem == ElemType.BF16:
        nan_a, nan_b = (a & 0x7FFF) > 0x7F80, (b & 0x7FFF) > 0x7F80
    else:
        nan_a, nan_b = (a & 0x7FFF) > 0x7C00, (b & 0x7FFF) > 0x7C00
    return a.shape == b.shape and np.array_equal(nan_a, nan_b) and np.array_equal(a[~nan_a], b[~nan_b])


def rand_input(rng, shape, elem, oracle, sigma=0.02, outliers=0.001):
    x = rng.normal(0, sigma, shape).astype(np.float32)
    if outliers:
        x[rng.random(shape) < outliers] *= 50
    return oracle.to_bits(x, elem)


# ---------------------------------------------------------------- fixtures

@pytest.mark.parametrize("case", RAMPS + TYPED + NATIVE, ids=lambda c: c.name)
def test_golden_fixtures(gpu, case):
    sshape = (1,) if case.scheme.level.is_tensor else case.scheme.scales_shape(case.shape)
    strides = (1,) if case.scheme.level.is_tensor else case.scale_strides
    words, out_scale = gpu.quantize(case.x, case.elem, case.shape, case.scale, case.scheme,
                                    scale_shape=sshape, scale_strides=strides)
    assert gc.bits_equal(words, case.words)
    assert gc.bits_equal(out_scale, case.out_scale)
    deq = gpu.dequantize(words, case.shape, out_scale, case.elem, case.scheme,
                         scale_shape=sshape, scale_strides=strides)
    assert gc.bits_equal(deq, case.deq)


@pytest.mark.parametrize("case", RAMPS, ids=lambda c: c.name)
def test_reference_round_trip(gpu, case):
    """The reference's own test: quantize -> dequantize into a fresh buffer,
    |x^ - x| <= scale/2*(1+1e-4) (tests/suite/symmetric.rs:99-140, :240-283)."""
    words, out_scale = gpu.quantize(case.x, case.elem, case.shape, case.scale, case.scheme)
    deq = gpu.dequantize(words, case.shape, out_scale, case.elem, case.scheme)
    x = case.x.reshape(case.shape)
    if case.scheme.level.is_tensor:
        tol = case.scale[0] / 2 * (1 + 1e-4)
    else:
        b = case.scheme.level.block_size.dims[-1]
        tol = np.repeat(case.scale.reshape(case.shape[0], -1), b, axis=1) / 2 * (1 + 1e-4)
    assert deq.shape == x.shape and np.all(np.abs(deq - x) <= tol)


# ---------------------------------------------------------------- seeded, vs oracle

@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("value", ALL_VALUES, ids=lambda v: v.name)
@pytest.mark.parametrize("block", [None, 16, 32, 64, 128], ids=lambda b: f"b{b}")
def test_seeded_vs_oracle(gpu, oracle, elem, value, block):
    rng = np.random.default_rng(hash((int(elem), int(value), block or 0)) % 2**32)
    shape = (96, 512)
    x = rand_input(rng, shape, elem, oracle)
    level = QuantLevel.Tensor if block is None else QuantLevel.block([block])
    scheme = QuantScheme.default().with_value(value).with_level(level)
    # scales: oracle rule == GPU compute_scales
    s_ref = oracle.compute_scales(x, elem, shape, scheme)
    s_gpu = gpu.compute_scales(x, elem, shape, scheme)
    assert same_floats(s_gpu, s_ref, elem)
    # quantize with given scales
    w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
    w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
    assert np.array_equal(w_gpu, w_ref)
    assert same_floats(os_gpu, os_ref, ElemType.F32)
    # fused dynamic == two-step
    w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
    assert np.array_equal(w_dyn, w_ref)
    assert same_floats(os_dyn, os_ref, ElemType.F32)
    # dequantize
    d_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
    d_gpu = gpu.dequantize(w_ref, shape, os_ref, elem, scheme)
    assert same_floats(d_gpu, d_ref, elem)


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("param", [QuantParam.F16, QuantParam.BF16], ids=lambda p: p.name)
def test_param_dtypes(gpu, oracle, elem, param):
    rng = np.random.default_rng(int(elem) * 7 + int(param))
    shape = (64, 256)
    x = rand_input(rng, shape, elem, oracle, sigma=1.0)
    for value, level in ((QuantValue.Q8S, QuantLevel.block([32])), (QuantValue.Q4S, QuantLevel.Tensor),
                         (QuantValue.E2M1, QuantLevel.block([64]))):
        scheme = QuantScheme.default().with_value(value).with_level(level).with_param(param)
        s_ref = oracle.compute_scales(x, elem, shape, scheme)
        w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
        pe = gpu.param_elem(scheme)
        assert np.array_equal(w_gpu, w_ref) and same_floats(os_gpu, os_ref, pe)
        w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
        assert np.array_equal(w_dyn, w_ref) and same_floats(os_dyn, os_ref, pe)
        assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                           oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem)


@pytest.mark.parametrize("elem", [ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_params_typed_like_the_tensor_on_whole_tiles(gpu, oracle, elem):
    """bf16 scales of a bf16 tensor, f16 of f16: a contiguous tensor runs kernels compiled for that parameter
    type over its whole tiles (four of them here) and the lane-wise kernels over the ragged rest."""
    param = QuantParam.BF16 if elem == ElemType.BF16 else QuantParam.F16
    rng = np.random.default_rng(4100 + int(elem))
    shape = (33, 1024)
    x = rand_input(rng, shape, elem, oracle, sigma=2.0)
    for value, level, store in ((QuantValue.Q8S, QuantLevel.block([32]), QuantStore.U32),
                                (QuantValue.Q4S, QuantLevel.block([16]), QuantStore.U32),
                                (QuantValue.Q2S, QuantLevel.block([64]), QuantStore.U32),
                                (QuantValue.E2M1, QuantLevel.block([32]), QuantStore.U32),
                                (QuantValue.Q4F, QuantLevel.block([128]), QuantStore.U32),
                                (QuantValue.Q8F, QuantLevel.Tensor, QuantStore.U32),
                                (QuantValue.E4M3, QuantLevel.block([32]), QuantStore.Native),
                                (QuantValue.E5M2, QuantLevel.block([128]), QuantStore.Native),
                                (QuantValue.E2M1, QuantLevel.block([32]), QuantStore.Native),
                                (QuantValue.Q8S, QuantLevel.block([8]), QuantStore.Native)):
        scheme = QuantScheme.default().with_value(value).with_level(level).with_store(store).with_param(param)
        pe = gpu.param_elem(scheme)
        s_ref = oracle.compute_scales(x, elem, shape, scheme)
        w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
        assert np.array_equal(w_gpu, w_ref) and same_floats(os_gpu, os_ref, pe), (value, level)
        w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
        assert np.array_equal(w_dyn, w_ref) and same_floats(os_dyn, os_ref, pe), (value, level)
        assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                           oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem), (value, level)


# ---------------------------------------------------------------- adversarial arithmetic

def test_bf16_all_significand_pairs(gpu, oracle):
    """The bf16 kernel multiplies by a reciprocal; its proof says the rounded
    quotient is the same for every pair of 8-bit significands.  Enumerate all
    128 x 128 pairs at several exponent offsets, in both signs."""
    sig = np.arange(128, 256, dtype=np.uint32)
    for scale_exp, x_exp_offsets in ((127, (0, 3, 5, 6, 7)), (120, (2, 6)), (100, (5,)), (140, (6,))):
        for off in x_exp_offsets:
            # x = significand i at exponent scale_exp+off ; scale = significand j at scale_exp
            xb = (((scale_exp + off) << 7) | (sig & 0x7F)).astype(np.uint16)
            sb = ((scale_exp << 7) | (sig & 0x7F)).astype(np.uint16)
            x = np.repeat(xb[None, :], 128, axis=0)           # row j: all x significands
            x = np.concatenate([x, x | 0x8000], axis=1)        # both signs -> [128, 256]
            shape = x.shape
            for value in (QuantValue.Q8S, QuantValue.Q8F, QuantValue.Q4S, QuantValue.E2M1):
                scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([128]))
                scales = np.repeat(sb[:, None], 2, axis=1).copy()  # [128, 2]
                w_ref, os_ref = oracle.quantize(x, ElemType.BF16, shape, scales, scheme)
                w_gpu, os_gpu = gpu.quantize(x, ElemType.BF16, shape, scales, scheme)
                assert np.array_equal(w_gpu, w_ref), (scale_exp, off, value)
                assert np.array_equal(os_gpu.reshape(-1), os_ref.reshape(-1))


def test_f32_near_ties(gpu, oracle):
    """f32 quotients on and next to half-integers, where x*rcp(d) and x/d may
    land on different sides: the kernel has to fall back to IEEE division."""
    rng = np.random.default_rng(99)
    for value in (QuantValue.Q8S, QuantValue.Q8F, QuantValue.Q4S, QuantValue.Q2S, QuantValue.E2M1, QuantValue.E4M3):
        lo, hi = value.range()
        scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([64]))
        rows = 256
        scales = rng.uniform(0.001, 3.0, (rows, 1)).astype(np.float32)
        k = rng.integers(int(max(lo, -300)) - 1, int(min(hi, 300)) + 1, (rows, 64)).astype(np.float32) + 0.5
        x = (k * scales).astype(np.float32)
        nudge = rng.integers(-3, 4, x.shape).astype(np.int32)
        x = (x.view(np.int32) + nudge).view(np.float32)
        w_ref, _ = oracle.quantize(x, ElemType.F32, x.shape, scales, scheme)
        w_gpu, _ = gpu.quantize(x, ElemType.F32, x.shape, scales, scheme)
        assert np.array_equal(w_gpu, w_ref), value
        w_dyn, os_dyn = gpu.quantize_dynamic(x, ElemType.F32, x.shape, scheme)
        s2 = oracle.compute_scales(x, ElemType.F32, x.shape, scheme)
        w2, os2 = oracle.quantize(x, ElemType.F32, x.shape, s2, scheme)
        assert np.array_equal(w_dyn, w2) and np.array_equal(os_dyn.reshape(-1), os2.reshape(-1))


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_special_values_and_scales(gpu, oracle, elem):
    """Quiet NaN, infinities, zeros, denormal / huge / zero / negative / NaN scales.
    (Decisions of this build where the reference is silent: NaN quotient -> q_max,
    abs-max skips NaN.)"""
    specials = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, -1e-40, 3e38, -3e38, 1.0, -1.0,
                         0.5, 1.5, 2.5, -0.5, -1.5, 1e-20, 65504.0, 1e10, -7.25, 127.5, -127.5,
                         128.5, 6.5, 5.5, 4.5, 448.0, 1e-30, 3.0, -3.0, 1e30, 1e-10], dtype=np.float32)
    x32 = np.tile(specials, (16, 2))                      # [16, 64]
    with np.errstate(over="ignore"):
        x = oracle.to_bits(x32, elem)
    shape = x32.shape
    scale_vals = np.array([1.0, 0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40, 1e-38, 3e38, -1.0, 0.5, 3.0,
                           1e-30, 1e30, 2.0 ** -120, 2.0 ** 110], dtype=np.float32)
    for value in (QuantValue.Q8S, QuantValue.Q4F, QuantValue.Q2S, QuantValue.E2M1):
        scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([32]))
        with np.errstate(over="ignore"):
            scales = oracle.to_bits(np.repeat(scale_vals[:, None], 2, axis=1), elem)   # [16, 2]
        w_ref, os_ref = oracle.quantize(x, elem, shape, scales, scheme)
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, scales, scheme)
        assert np.array_equal(w_gpu, w_ref), value
        assert same_floats(os_gpu, os_ref, ElemType.F32)
        assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                           oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem)
        # dynamic: blocks containing NaN/inf, and an all-zero block
        xz = x.copy()
        xz[3, :32] = 0
        s_ref = oracle.compute_scales(xz, elem, shape, scheme)
        assert same_floats(gpu.compute_scales(xz, elem, shape, scheme), s_ref, elem)
        w2, os2 = oracle.quantize(xz, elem, shape, s_ref, scheme)
        w_dyn, os_dyn = gpu.quantize_dynamic(xz, elem, shape, scheme)
        assert np.array_equal(w_dyn, w2) and same_floats(os_dyn, os2, ElemType.F32)
        # per tensor
        st = QuantScheme.default().with_value(value)
        xf = oracle.to_bits(np.where(np.isfinite(x32), x32, 1.0).astype(np.float32), elem)
        s_t = oracle.compute_scales(xf, elem, shape, st)
        assert same_floats(gpu.compute_scales(xf, elem, shape, st), s_t, elem)
        wt, ost = oracle.quantize(xf, elem, shape, s_t, st)
        wd, osd = gpu.quantize_dynamic(xf, elem, shape, st)
        assert np.array_equal(wd, wt) and same_floats(osd, ost, ElemType.F32)


# ---------------------------------------------------------------- layouts

def test_nd_blocks_and_strided_scales(gpu, oracle):
    rng = np.random.default_rng(5)
    for elem in ELEMS:
        for shape, block, value in (((4, 6, 32), (2, 3, 16), QuantValue.Q4S), ((4, 6, 32), (3, 8), QuantValue.Q8S),
                                    ((8, 96), (24,), QuantValue.Q8S), ((2, 3, 4, 64), (3, 2, 16), QuantValue.Q2S),
                                    ((6, 40), (3, 8), QuantValue.Q4F), ((5, 48), (5, 48), QuantValue.Q8F)):
            scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block(block))
            x = rand_input(rng, shape, elem, oracle, sigma=1.0)
            s_ref = oracle.compute_scales(x, elem, shape, scheme)
            assert same_floats(gpu.compute_scales(x, elem, shape, scheme), s_ref, elem)
            w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
            w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
            assert np.array_equal(w_gpu, w_ref) and same_floats(os_gpu, os_ref, ElemType.F32)
            w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
            assert np.array_equal(w_dyn, w_ref) and same_floats(os_dyn, os_ref, ElemType.F32)
            assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                               oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem)
    # column-major scales in a padded buffer, out_scale with yet another layout
    elem, shape = ElemType.BF16, (8, 128)
    scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([32]))
    x = rand_input(rng, shape, elem, oracle)
    s = oracle.compute_scales(x, elem, shape, scheme)          # [8, 4]
    buf = np.zeros(64, dtype=np.uint16)
    in_strides, out_strides = (1, 8), (6, 1)                  # column-major / padded rows
    for r in range(8):
        for c in range(4):
            buf[r * in_strides[0] + c * in_strides[1]] = s[r, c]
    w_ref, os_ref = oracle.quantize(x, elem, shape, buf, scheme, scale_strides=in_strides,
                                    out_scale_strides=out_strides)
    w_gpu, os_gpu = gpu.quantize(x, elem, shape, buf, scheme, scale_shape=(8, 4), scale_strides=in_strides,
                                 out_scale_strides=out_strides)
    assert np.array_equal(w_gpu, w_ref) and np.array_equal(os_gpu.reshape(-1), os_ref.reshape(-1))
    d_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme, scale_strides=out_strides)
    d_gpu = gpu.dequantize(w_ref, shape, os_ref, elem, scheme, scale_shape=(8, 4), scale_strides=out_strides)
    assert same_floats(d_gpu, d_ref, elem)


def test_ragged_per_tensor_sizes(gpu, oracle):
    """Element counts that are a multiple of num_quants but not of a 16-byte
    chunk, tiny tensors, rank 1 and rank 4."""
    rng = np.random.default_rng(8)
    for elem in ELEMS:
        for value in (QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q2S):
            nq = 32 // value.size_bits()
            for shape in ((nq,), (3, nq), (7, 5 * nq), (1, 1, 3, 11 * nq), (33, 3 * nq)):
                scheme = QuantScheme.default().with_value(value)
                x = rand_input(rng, shape, elem, oracle, sigma=2.0)
                s_ref = oracle.compute_scales(x, elem, shape, scheme)
                assert same_floats(gpu.compute_scales(x, elem, shape, scheme), s_ref, elem)
                w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
                w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
                assert np.array_equal(w_gpu, w_ref) and same_floats(os_gpu, os_ref, ElemType.F32)
                w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
                assert np.array_equal(w_dyn, w_ref) and same_floats(os_dyn, os_ref, ElemType.F32)
                assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                                   oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem)


def test_unaligned_base_pointers(gpu, oracle):
    """A float tensor that starts 4 bytes into an allocation cannot use 16-byte
    loads; results must not change."""
    import torch
    from cubek_amd import ComputeClient, TensorHandleRef
    from cubek_amd import dequantize as dq, quantize as qz

    rng = np.random.default_rng(3)
    shape = (16, 256)
    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))
    x = rng.normal(0, 1, shape).astype(np.float32)
    s_ref = oracle.compute_scales(x, ElemType.F32, shape, scheme)
    w_ref, os_ref = oracle.quantize(x, ElemType.F32, shape, s_ref, scheme)
    buf = torch.zeros(x.size + 1, dtype=torch.float32, device="cuda")
    buf[1:] = torch.from_numpy(x.reshape(-1)).cuda()
    view = buf[1:].view(shape)
    assert view.data_ptr() % 16 == 4
    out = torch.zeros(scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
    os_ = torch.zeros(scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
    client = ComputeClient.current()
    qz.launch_dynamic(client, TensorHandleRef.from_torch(view), TensorHandleRef.from_torch(out),
                      TensorHandleRef.from_torch(os_), scheme, ElemType.F32)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), w_ref)
    assert np.array_equal(os_.cpu().numpy().reshape(-1), os_ref.reshape(-1))
    back = torch.zeros(x.size + 1, dtype=torch.float32, device="cuda")
    dq.launch_ref(client, TensorHandleRef.from_torch(out), TensorHandleRef.from_torch(back[1:].view(shape)),
                  TensorHandleRef.from_torch(os_), scheme, ElemType.F32)
    torch.cuda.synchronize()
    d_ref = oracle.dequantize(w_ref, shape, os_ref, ElemType.F32, scheme)
    assert np.array_equal(back[1:].cpu().numpy().reshape(shape), d_ref)
    # per tensor on the same unaligned view: the grid abs-max must not assume alignment
    pt = QuantScheme.default().with_value(QuantValue.Q8S)
    s_t = oracle.compute_scales(x, ElemType.F32, shape, pt)
    wt, ost = oracle.quantize(x, ElemType.F32, shape, s_t, pt)
    out_t = torch.zeros(pt.packed_shape(shape), dtype=torch.int32, device="cuda")
    os_t = torch.zeros((1,), dtype=torch.float32, device="cuda")
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")
    qz.launch_dynamic(client, TensorHandleRef.from_torch(view), TensorHandleRef.from_torch(out_t),
                      TensorHandleRef.from_torch(os_t), pt, ElemType.F32, ws.data_ptr(), 1024)
    sc_t = torch.zeros((1,), dtype=torch.float32, device="cuda")
    qz.compute_scales(client, TensorHandleRef.from_torch(view), TensorHandleRef.from_torch(sc_t), pt, ElemType.F32,
                      ws.data_ptr(), 1024)
    torch.cuda.synchronize()
    assert np.array_equal(out_t.cpu().numpy().view(np.uint32), wt)
    assert os_t.cpu().numpy()[0] == ost.reshape(-1)[0] == sc_t.cpu().numpy()[0]


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_dequantize_blocks_that_split_a_word(gpu, oracle, elem):
    """The reference's dequantize launchers take any block size (src/dequantize.rs:231-280 has no
    check_block_size_compat).  A block smaller than a packed word then gives the whole word the scale of
    the word's first element (src/dequantize.rs:70-76); native bytes take the scale of their own block."""
    rng = np.random.default_rng(77 + int(elem))
    shape = (6, 96)
    for value, block, store in ((QuantValue.Q8S, [2], QuantStore.U32), (QuantValue.Q4S, [4], QuantStore.U32),
                                (QuantValue.Q2F, [8], QuantStore.U32), (QuantValue.Q4F, [2, 12], QuantStore.U32),
                                (QuantValue.Q8S, [3], QuantStore.Native), (QuantValue.E2M1, [1], QuantStore.Native),
                                (QuantValue.E4M3, [2, 3], QuantStore.Native)):
        scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block(block)).with_store(store)
        n_stored = int(np.prod(scheme.packed_shape(shape)))
        if store == QuantStore.U32:
            stored = rng.integers(0, 2**32, n_stored, dtype=np.uint64).astype(np.uint32)
        else:
            stored = rng.integers(0, 256, n_stored, dtype=np.uint64).astype(np.uint8)
            if value == QuantValue.E4M3:
                stored[(stored & 0x7F) == 0x7F] = 0x3A  # no NaN codes
        scales = rng.uniform(0.01, 2.0, scheme.scales_shape(shape)).astype(np.float32)
        got = gpu.dequantize(stored, shape, scales, elem, scheme)
        want = oracle.dequantize(stored, shape, scales, elem, scheme)
        assert same_floats(got, want, elem), (value.name, block, store.name)


# ---------------------------------------------------------------- native store

@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("value", [QuantValue.Q8F, QuantValue.Q8S, QuantValue.E4M3, QuantValue.E5M2, QuantValue.E2M1],
                         ids=lambda v: v.name)
def test_native_store(gpu, oracle, elem, value):
    rng = np.random.default_rng(int(elem) * 31 + int(value))
    shape = (32, 256)
    for level in (QuantLevel.Tensor, QuantLevel.block([32]), QuantLevel.block([2, 16])):
        scheme = QuantScheme.default().with_value(value).with_level(level).with_store(QuantStore.Native)
        x = rand_input(rng, shape, elem, oracle, sigma=1.0)
        s_ref = oracle.compute_scales(x, elem, shape, scheme)
        assert same_floats(gpu.compute_scales(x, elem, shape, scheme), s_ref, elem)
        w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
        assert np.array_equal(w_gpu, w_ref) and same_floats(os_gpu, os_ref, ElemType.F32)
        w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
        assert np.array_equal(w_dyn, w_ref) and same_floats(os_dyn, os_ref, ElemType.F32)
        assert same_floats(gpu.dequantize(w_ref, shape, os_ref, elem, scheme),
                           oracle.dequantize(w_ref, shape, os_ref, elem, scheme), elem)
    if value in (QuantValue.E4M3, QuantValue.E5M2):
        # every integer the clamp can produce goes through the hardware fp8 conversion
        lo, hi = value.range()
        ints = np.arange(lo, hi + 1, dtype=np.float32)
        if ints.size > 4096:
            ints = np.concatenate([ints[:2048], ints[-2048:], np.arange(-4096, 4096, dtype=np.float32) * 13])
        pad = (-ints.size) % 64
        xi = np.concatenate([ints, np.zeros(pad, np.float32)]).reshape(-1, 64)
        sch = QuantScheme.default().with_value(value).with_store(QuantStore.Native)
        one = np.array([1.0], np.float32)
        w_ref, _ = oracle.quantize(xi, ElemType.F32, xi.shape, one, sch)
        w_gpu, _ = gpu.quantize(xi, ElemType.F32, xi.shape, one, sch)
        assert np.array_equal(w_gpu, w_ref)


# ---------------------------------------------------------------- errors

def test_error_codes(gpu):
    import torch
    from cubek_amd import ComputeClient, QuantError, TensorHandleRef, _ffi
    from cubek_amd import dequantize as dq, quantize as qz

    client = ComputeClient.current()
    x = torch.zeros((8, 64), dtype=torch.float32, device="cuda")
    out = torch.zeros((8, 16), dtype=torch.int32, device="cuda")
    sc = torch.ones((8, 2), dtype=torch.float32, device="cuda")
    h = TensorHandleRef.from_torch
    ok = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([32]))
    qz.launch_ref(client, h(x), h(out), h(sc), h(sc.clone()), ok, ElemType.F32)

    def status(fn):
        with pytest.raises(QuantError) as e:
            fn()
        return e.value.status

    # block size not a multiple of num_quants: the reference asserts (src/lib.rs:28-31)
    bad_block = ok.with_level(QuantLevel.block([2]))
    sc2 = torch.ones((8, 32), dtype=torch.float32, device="cuda")
    assert status(lambda: qz.launch_ref(client, h(x), h(out), h(sc2), h(sc2.clone()), bad_block, ElemType.F32)) \
        == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    # Q4/Q2 have no native store: the reference panics (src/quantize.rs:213-219)
    native_q4 = QuantScheme.default().with_value(QuantValue.Q4S).with_store(QuantStore.Native)
    out8 = torch.zeros((8, 64), dtype=torch.uint8, device="cuda")
    one = torch.ones((1,), dtype=torch.float32, device="cuda")
    assert status(lambda: qz.launch_ref(client, h(x), h(out8), h(one), h(one.clone()), native_q4, ElemType.F32)) \
        == _ffi.ERR_UNSUPPORTED_SCHEME
    assert status(lambda: dq.launch_ref(client, h(out8), h(x), h(one), native_q4, ElemType.F32)) \
        == _ffi.ERR_UNSUPPORTED_SCHEME
    # packed shape that does not match
    out_bad = torch.zeros((8, 15), dtype=torch.int32, device="cuda")
    assert status(lambda: qz.launch_ref(client, h(x), h(out_bad), h(sc), h(sc.clone()), ok, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH
    # scales of the wrong shape
    sc_bad = torch.ones((8, 3), dtype=torch.float32, device="cuda")
    assert status(lambda: qz.launch_ref(client, h(x), h(out), h(sc_bad), h(sc_bad.clone()), ok, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH
    # per-tensor dynamic without workspace
    pt = QuantScheme.default().with_value(QuantValue.Q8S)
    assert status(lambda: qz.launch_dynamic(client, h(x), h(out), h(one), pt, ElemType.F32)) \
        == _ffi.ERR_WORKSPACE_TOO_SMALL
    # wrong element size for the declared dtype
    assert status(lambda: qz.launch_ref(client, h(x), h(out), h(sc), h(sc.clone()), ok, ElemType.BF16)) \
        == _ffi.ERR_SHAPE_MISMATCH


def test_scale_division_all_significands(gpu):
    """The kernels divide 2*absmax by the range width with a reciprocal and one
    residual correction.  Every f32 significand, at three exponents, for every
    value type, against numpy's IEEE division."""
    import torch
    from cubek_amd import ComputeClient, TensorHandleRef
    from cubek_amd import quantize as qz

    client = ComputeClient.current()
    sig = np.arange(1 << 23, dtype=np.uint32)
    for value in ALL_VALUES:
        lo, hi = value.range()
        width = np.float32(hi - lo)
        nq = 32 // value.size_bits()
        scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([nq]))
        for exp_field in (127, 100, 140):
            amax = (sig | np.uint32(exp_field << 23)).view(np.float32)
            want = (amax + amax) / width
            slices = nq // 4
            per = (1 << 23) // slices
            for k in range(slices):
                a = torch.from_numpy(amax[k * per:(k + 1) * per]).cuda()
                x = torch.zeros((per, nq), dtype=torch.float32, device="cuda")
                x[:, 1] = a            # the block's abs-max ...
                x[:, nq - 1] = -a / 2  # ... and a smaller negative value
                scales = torch.zeros((per, 1), dtype=torch.float32, device="cuda")
                qz.compute_scales(client, TensorHandleRef.from_torch(x), TensorHandleRef.from_torch(scales),
                                  scheme, ElemType.F32)
                codes = torch.zeros((per, 1), dtype=torch.int32, device="cuda")
                out_scale = torch.zeros((per, 1), dtype=torch.float32, device="cuda")
                qz.launch_dynamic(client, TensorHandleRef.from_torch(x), TensorHandleRef.from_torch(codes),
                                  TensorHandleRef.from_torch(out_scale), scheme, ElemType.F32)
                torch.cuda.synchronize()
                ref = want[k * per:(k + 1) * per]
                assert np.array_equal(scales.cpu().numpy().reshape(-1).view(np.uint32), ref.view(np.uint32)), \
                    (value, exp_field, k)
                assert np.array_equal(out_scale.cpu().numpy().reshape(-1).view(np.uint32), ref.view(np.uint32)), \
                    (value, exp_field, k)


@pytest.mark.parametrize("value", [QuantValue.E5M2, QuantValue.Q2S, QuantValue.Q4S, QuantValue.Q8F], ids=lambda v: v.name)
def test_f16_every_input_every_divisor(gpu, oracle, value):
    """The f16 kernels replace the division by a reciprocal and one residual step, and for fields
    that hold the whole range (Q2 / Q4 / Q8) round, clamp and pack in packed f16 arithmetic.  All
    65536 x 65536 (element, divisor) bit patterns, NaN, infinities, zeros and subnormals
    included, against the oracle's IEEE division; a wide clamp range and the three field widths."""
    import torch
    from cubek_amd import ComputeClient
    from cubek_amd import quantize as qz

    client = ComputeClient.current()
    rows = 2048
    x = np.ascontiguousarray(np.broadcast_to(np.arange(65536, dtype=np.uint16), (rows, 65536)))
    dx = gpu.to_dev(x)
    scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([128]))
    pshape = scheme.packed_shape((rows, 65536))
    for d0 in range(0, 65536, rows):
        d = np.arange(d0, d0 + rows, dtype=np.uint16)
        scale = np.ascontiguousarray(np.broadcast_to(d[:, None], (rows, 512)))
        dout = torch.zeros(pshape, dtype=torch.int32, device="cuda")
        dos = torch.zeros((rows, 512), dtype=torch.float32, device="cuda")
        dscale = gpu.to_dev(scale)  # the handle only borrows it
        qz.launch_ref(client, gpu.handle(dx), gpu.handle(dout), gpu.handle(dscale), gpu.handle(dos),
                      scheme, ElemType.F16)
        torch.cuda.synchronize()
        want, _ = oracle.quantize(x, ElemType.F16, (rows, 65536), scale, scheme, threads=16)
        assert np.array_equal(gpu.to_host(dout).reshape(-1), want.reshape(-1)), (value.name, d0)


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_negative_zero_survives_every_dequantize_path(gpu, oracle, elem):
    """-0 codes (fp8 / fp4 sign bit with zero magnitude) and zero codes under a negative scale
    dequantize to -0, whichever kernel takes the layout: contiguous, pitched rows, transposed,
    transposed with an odd pitch (per-element)."""
    import torch
    from cubek_amd import ComputeClient
    from cubek_amd import dequantize as dq

    client = ComputeClient.current()
    rows, cols = 64, 64
    cases = [(QuantValue.E4M3, QuantStore.Native, np.uint8, 0x80, 0.5), (QuantValue.E5M2, QuantStore.Native, np.uint8, 0x80, 0.5),
             (QuantValue.E2M1, QuantStore.Native, np.uint8, 0x88, 0.5), (QuantValue.Q8S, QuantStore.U32, np.uint32, 0, -0.5),
             (QuantValue.Q4S, QuantStore.U32, np.uint32, 0, -0.5)]
    for value, store, sdt, code, scale in cases:
        scheme = QuantScheme.default().with_value(value).with_store(store)
        pshape = scheme.packed_shape((rows, cols))
        codes = np.full(pshape, code, dtype=sdt)
        params = np.array([scale], dtype=np.float32)
        want = oracle.dequantize(codes, (rows, cols), params, elem, scheme).reshape(rows, cols)
        assert np.signbit(oracle.from_bits(want, elem)).all()
        for name, fstr in (("contiguous", (cols, 1)), ("pitched", (cols + 8, 1)), ("transposed", (1, rows)),
                           ("transposed_odd_pitch", (1, rows + 1))):
            n = 1 + (rows - 1) * fstr[0] + (cols - 1) * fstr[1]
            d_y = torch.full((n,), 7.0, dtype={ElemType.F32: torch.float32, ElemType.BF16: torch.bfloat16,
                                               ElemType.F16: torch.float16}[elem], device="cuda")
            d_codes, d_params = gpu.to_dev(codes), gpu.to_dev(params)  # the handles only borrow: keep them alive
            dq.launch_ref(client, gpu.handle(d_codes), gpu.handle(d_y, (rows, cols), fstr), gpu.handle(d_params),
                          scheme, elem)
            torch.cuda.synchronize()
            raw = d_y.view(torch.int32 if elem == ElemType.F32 else torch.int16)
            got = torch.as_strided(raw, (rows, cols), fstr).cpu().numpy()
            bits = np.uint32 if elem == ElemType.F32 else np.uint16
            assert np.array_equal(got.view(bits), np.ascontiguousarray(want).view(bits)), (value.name, elem.name, name)
