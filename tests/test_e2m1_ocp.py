"""The extension value E2M1_OCP: OCP microscaling FP4 rounded ONCE from the quotient (0.5 and 1.5 occur), e2m1
nibbles in both stores.  The reference has no such value (its E2M1 rounds to an integer first,
crates/cubek-quant/src/quantize.rs:33-43), so nothing here is reference parity: the oracle's arm is pinned against
the exact-rational model (tests/golden/typed_ocp.npz), a hand-written known answer and a nearest-value search, and
the kernels are compared with the oracle bit for bit."""
import numpy as np
import pytest

import golden_cases as gc
from cubek_amd.scheme import (ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue)

OCP = gc.load("typed_ocp.npz")
E2M1_GRID = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
ELEMS = [ElemType.BF16, ElemType.F16, ElemType.F32]


def ocp(store=QuantStore.U32, block=None, param=QuantParam.F32):
    level = QuantLevel.Tensor if block is None else QuantLevel.block(list(block))
    return QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_store(store).with_param(param).with_level(level)


def as_u32(case):
    """The same case with the U32 store: eight nibbles per word are the native store's four bytes."""
    return case.scheme.with_store(QuantStore.U32), case.words.view(np.uint32)


def nibbles(stored: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(stored).view(np.uint8).reshape(-1)
    return np.stack([b & 0xF, b >> 4], axis=1).reshape(-1)


# ---------------------------------------------------------------- host side and oracle (no GPU)

def test_scheme_functions():
    assert QuantValue.E2M1_OCP.size_bits() == 4 and QuantValue.E2M1_OCP.range() == (-6.0, 6.0)
    assert ocp().num_quants() == 8 and ocp(QuantStore.Native).num_quants() == 2
    assert ocp(block=[32]).packed_shape((4, 64)) == (4, 8)
    assert ocp(QuantStore.Native, block=[32]).packed_shape((4, 64)) == (4, 32)
    assert int(QuantValue.E2M1_OCP) == 9 and int(QuantValue.E2M1) == 6  # a value of its own, never E2M1


def test_library_scheme_functions():
    from cubek_amd import _ffi

    L = _ffi.lib()
    assert L.cq_value_size_bits(9) == 4
    assert L.cq_scheme_num_quants(ocp().to_c()) == 8 and L.cq_scheme_num_quants(ocp(QuantStore.Native).to_c()) == 2


@pytest.mark.parametrize("case", OCP, ids=lambda c: c.name)
def test_oracle_matches_exact_model(oracle, case):
    for scheme, want in ((case.scheme, case.words), as_u32(case)):
        words, out_scale = oracle.quantize(case.x, case.elem, case.shape, case.scale, scheme,
                                           scale_strides=case.scale_strides)
        assert gc.bits_equal(words, want)
        assert gc.bits_equal(out_scale, case.out_scale)
        deq = oracle.dequantize(words, case.shape, out_scale, case.elem, scheme, scale_strides=case.scale_strides)
        assert gc.bits_equal(deq, case.deq)


def test_oracle_known_answer(oracle):
    """Every midpoint of the e2m1 grid goes to the even code, the clamp saturates at +-6, a quotient below 1/4 keeps
    its sign on a zero; element 2k sits in the low nibble."""
    x = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.5,
                  1.5, -0.25, -0.3, 7.0, -7.0, 0.26, 0.74, -0.0], np.float32).reshape(1, 16)
    want = [0x0, 0x2, 0x2, 0x4, 0x4, 0x6, 0x6, 0x1,
            0x3, 0x8, 0x9, 0x7, 0xF, 0x1, 0x1, 0x8]
    codes, _ = oracle.quantize(x, ElemType.F32, (1, 16), np.array([1.0], np.float32), ocp(QuantStore.Native))
    assert nibbles(codes).tolist() == want
    words, _ = oracle.quantize(x, ElemType.F32, (1, 16), np.array([1.0], np.float32), ocp())
    assert words.reshape(-1).tolist() == [sum(n << (4 * i) for i, n in enumerate(want[:8])),
                                          sum(n << (4 * i) for i, n in enumerate(want[8:]))]
    y = oracle.dequantize(words, (1, 16), np.array([0.5], np.float32), ElemType.F32, ocp())
    sign = np.where(np.array(want) & 8, -1.0, 1.0)
    assert np.array_equal(y.reshape(-1), (sign * E2M1_GRID[np.array(want) & 7] * 0.5).astype(np.float32))
    assert np.signbit(y.reshape(-1)[9]) and np.signbit(y.reshape(-1)[15])


def test_oracle_is_the_nearest_grid_value(oracle):
    """Independent of the oracle's cast: the stored magnitude is a grid value nearest to clamp(x / d) (computed in
    float64 from the f32 quotient), and off the midpoints it is the only one."""
    rng = np.random.default_rng(7)
    x = rng.normal(0, 2.5, (64, 256)).astype(np.float32)
    d = np.float32(0.37)
    codes, _ = oracle.quantize(x, ElemType.F32, x.shape, np.array([d], np.float32), ocp(QuantStore.Native))
    n = nibbles(codes)
    q = np.clip((x.reshape(-1) / d).astype(np.float32).astype(np.float64), -6, 6)
    dist = np.abs(np.abs(q)[:, None] - E2M1_GRID[None, :])
    assert np.array_equal(dist[np.arange(q.size), n & 7], dist.min(axis=1))
    assert np.array_equal((n & 8) != 0, np.signbit(q))
    assert {0x1, 0x3, 0x9, 0xB} <= set(n.tolist())  # the halves occur: this is not the reference's E2M1


def test_differs_from_the_reference_value(oracle):
    """1.5 / 1 stays 1.5 here; the reference's E2M1 rounds it to 2 first."""
    x = np.full((1, 8), 1.5, np.float32)
    s = np.array([1.0], np.float32)
    w_ocp, _ = oracle.quantize(x, ElemType.F32, (1, 8), s, ocp())
    w_ref, _ = oracle.quantize(x, ElemType.F32, (1, 8), s, QuantScheme.default().with_value(QuantValue.E2M1))
    assert w_ocp[0] == 0x33333333 and w_ref[0] == 0x22222222
    assert np.all(oracle.dequantize(w_ocp, (1, 8), s, ElemType.F32, ocp()) == 1.5)


# ---------------------------------------------------------------- kernels against the oracle

@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def same_bits(a, b):
    a, b = np.ascontiguousarray(a).reshape(-1), np.ascontiguousarray(b).reshape(-1)
    return a.shape == b.shape and np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("case", OCP, ids=lambda c: c.name)
def test_gpu_fixtures(gpu, case):
    sshape = (1,) if case.scheme.level.is_tensor else case.scheme.scales_shape(case.shape)
    strides = (1,) if case.scheme.level.is_tensor else case.scale_strides
    for scheme, want in ((case.scheme, case.words), as_u32(case)):
        words, out_scale = gpu.quantize(case.x, case.elem, case.shape, case.scale, scheme,
                                        scale_shape=sshape, scale_strides=strides)
        assert gc.bits_equal(words, want), scheme.store
        assert gc.bits_equal(out_scale, case.out_scale)
        deq = gpu.dequantize(words, case.shape, out_scale, case.elem, scheme, scale_shape=sshape, scale_strides=strides)
        assert gc.bits_equal(deq, case.deq), scheme.store


@pytest.mark.gpu
@pytest.mark.parametrize("elem", [ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_gpu_every_16_bit_input(gpu, oracle, elem):
    """All 65 536 bit patterns of a 16-bit type as inputs (NaNs and infinities included) under divisors that are tame,
    tiny, huge, negative and not a power of two; streaming kernels (blocks of 32) and the per-tensor path."""
    x = np.arange(65536, dtype=np.uint16).reshape(64, 1024)
    for d in (1.0, 0.3, 3.0e-5, 1.7e4, -0.75, 2.0 ** -110):
        for store in (QuantStore.U32, QuantStore.Native):
            for block in ([32], None):
                scheme = ocp(store, block)
                s = oracle.to_bits(np.full(scheme.scales_shape(x.shape), d, np.float32), elem)
                w_ref, os_ref = oracle.quantize(x, elem, x.shape, s, scheme)
                w_gpu, os_gpu = gpu.quantize(x, elem, x.shape, s, scheme)
                assert same_bits(w_gpu, w_ref) and same_bits(os_gpu, os_ref), (d, store, block)
    y_ref = oracle.dequantize(w_ref, x.shape, os_ref, elem, scheme)
    assert same_bits(gpu.dequantize(w_ref, x.shape, os_ref, elem, scheme), y_ref)


@pytest.mark.gpu
def test_gpu_f32_near_midpoints(gpu, oracle):
    """f32 quotients one ulp either side of every midpoint of the grid (and on it), under several divisors."""
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0], np.float32)
    q = np.concatenate([np.nextafter(mids, np.float32(0)), mids, np.nextafter(mids, np.float32(9))])
    q = np.concatenate([q, -q])
    rng = np.random.default_rng(11)
    for d in (np.float32(1.0), np.float32(0.1), np.float32(3.3e-3), np.float32(-7.0)):
        x = np.resize((q * d).astype(np.float32), (32, 64))
        x[20:] = rng.normal(0, 3 * abs(d), (12, 64)).astype(np.float32)
        for store in (QuantStore.U32, QuantStore.Native):
            scheme = ocp(store, [64])
            s = np.full(scheme.scales_shape(x.shape), d, np.float32)
            w_ref, _ = oracle.quantize(x, ElemType.F32, x.shape, s, scheme)
            w_gpu, _ = gpu.quantize(x, ElemType.F32, x.shape, s, scheme)
            assert same_bits(w_gpu, w_ref), (d, store)


@pytest.mark.gpu
@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("block", [None, (16,), (32,), (128,), (24,), (4, 32), (2, 3, 16)], ids=str)
def test_gpu_seeded_vs_oracle(gpu, oracle, elem, block):
    """Contiguous tensors on every kernel family that a block shape selects (whole tiles, lanes, odd blocks, 2-D blocks,
    per element), both stores, given scales, fused dynamic quantize and dequantize."""
    shape = (6, 96, 768) if block and len(block) == 3 else (192, 768)
    rng = np.random.default_rng(len(shape) * 131 + int(elem) + (sum(block) if block else 0))
    x32 = rng.normal(0, 1.0, shape).astype(np.float32)
    x32[rng.random(shape) < 0.002] *= 40
    x32.reshape(-1)[:128] = 0.0
    x = oracle.to_bits(x32, elem)
    for store in (QuantStore.U32, QuantStore.Native):
        for param in (QuantParam.F32, QuantParam.BF16):
            scheme = ocp(store, block, param)
            s_ref = oracle.compute_scales(x, elem, shape, scheme)
            w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
            w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
            assert same_bits(w_gpu, w_ref) and same_bits(os_gpu, os_ref), (store, param, "given")
            w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
            assert same_bits(w_dyn, w_ref) and same_bits(os_dyn, os_ref), (store, param, "dynamic")
            y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
            assert same_bits(gpu.dequantize(w_ref, shape, os_ref, elem, scheme), y_ref), (store, param)
            if store == QuantStore.U32:
                assert {1, 3} <= set((nibbles(w_ref) & 7).tolist())
