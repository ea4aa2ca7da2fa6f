"""cq_gemv_quantized (y = dequantize(W) @ x from the packed weights) against the GEMV over the ORACLE's
dequantized weights, computed in float64.  Tolerance, stated once: the kernels accumulate in f32, at most
~260 sequential additions per lane followed by a 6-step tree, each rounding 2^-24 relative, so
|y - y_ref| <= 2e-5 * sum|w * x|; an output of a 16-bit type is the f32 sum rounded once (checked bit for
bit against the f32 output)."""
import numpy as np
import pytest

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue,
                       TensorHandleRef, _ffi, matvec)

pytestmark = pytest.mark.gpu

CASES = [
    # elem, value, block, param, rows, cols, word pitch (None: contiguous)     -- the streaming kernel unless noted
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 1000, 4096, None),
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 77, 2048, None),
    (ElemType.BF16, QuantValue.E2M1, [32], QuantParam.F32, 130, 11008, None),     # last strip partly idle
    (ElemType.F16, QuantValue.Q4F, [32], QuantParam.F32, 333, 8192, None),
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 64, 4096, 520),         # pitched rows of words
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 50, 8448, None),        # four strips and an eighth
    (ElemType.F16, QuantValue.Q4S, [32], QuantParam.F32, 21, 16480, None),        # eight waves per workgroup
    (ElemType.BF16, QuantValue.Q4F, [32], QuantParam.F32, 1, 32768, None),        # one row, the longest it takes
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 9, 32, None),           # one block per row
    (ElemType.BF16, QuantValue.E2M1_OCP, [32], QuantParam.F32, 37, 2048, None),   # the extension value: e2m1 nibbles in u32 words
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 11, 53248, None),       # rows longer than the LDS holds of x
    (ElemType.F16, QuantValue.Q8S, [64], QuantParam.F16, 5, 40000, None),         # ... 8-bit codes, two segments
    (ElemType.F16, QuantValue.Q4S, [128], QuantParam.F16, 33, 4224, None),        # four units under one f16 scale
    (ElemType.BF16, QuantValue.Q8S, [32], QuantParam.F32, 45, 2080, None),        # 8-bit codes, two units per block
    (ElemType.BF16, QuantValue.Q4F, [64], QuantParam.BF16, 19, 16448, 2060),      # bf16 scales, eight waves, pitched
    (ElemType.F16, QuantValue.Q8F, [16], QuantParam.F32, 70, 1040, None),         # 8-bit codes, a scale per unit
    (ElemType.BF16, QuantValue.Q2S, [64], QuantParam.F32, 52, 4160, None),        # 2-bit codes
    (ElemType.F16, QuantValue.Q2F, [128], QuantParam.F16, 17, 8192, None),        # 2-bit codes, two units per block
    (ElemType.BF16, QuantValue.Q4S, [128], QuantParam.F16, 12, 1024, None),       # f16 scales under bf16 x
    (ElemType.F16, QuantValue.Q8S, [64], QuantParam.BF16, 31, 2112, None),        # bf16 scales under f16 x
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.BF16, 100, 1024, None),
    (ElemType.F16, QuantValue.Q8S, [64], QuantParam.F16, 50, 512, None),
    (ElemType.F32, QuantValue.Q2S, [64], QuantParam.F32, 96, 1024, None),          # x in f32: streaming again
    (ElemType.F32, QuantValue.Q4S, [32], QuantParam.F32, 75, 4160, 524),
    (ElemType.F32, QuantValue.Q8F, [16], QuantParam.F32, 31, 17008, None),         # ... rows too long for the LDS
    (ElemType.F32, QuantValue.Q4S, [32], QuantParam.BF16, 20, 1024, None),         # f32 x under bf16 scales: general kernel
    (ElemType.F32, QuantValue.Q8F, None, QuantParam.F32, 33, 260, None),          # general: 260 values are not whole units
    (ElemType.BF16, QuantValue.Q4S, [4, 16], QuantParam.F32, 64, 256, None),      # blocks narrower than a unit
    (ElemType.BF16, QuantValue.Q8S, None, QuantParam.F32, 29, 2064, None),        # streaming again: one scale per tensor
    (ElemType.F16, QuantValue.Q4F, None, QuantParam.F16, 11, 4128, None),
    (ElemType.BF16, QuantValue.Q4S, [6, 64], QuantParam.F32, 66, 4160, None),     # blocks of six rows
    (ElemType.F16, QuantValue.Q8S, [128, 128], QuantParam.F32, 256, 1024, None),  # 128 x 128 weight blocks
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 40, 1056, None),        # cols not a multiple of 64 blocks
]


def _id(c):
    elem, value, block, param, rows, cols, pitch = c
    return f"{elem.name}-{value.name}-{'x'.join(map(str, block)) if block else 'tensor'}-{param.name}-{rows}x{cols}" + \
        ("-pitched" if pitch else "")


def check_case(oracle, case, seed, native=False, vectors=1):
    import torch

    elem, value, block, param, rows, cols, pitch = case
    level = QuantLevel.Tensor if block is None else QuantLevel.block(block)
    scheme = QuantScheme.default().with_value(value).with_level(level).with_param(param)
    if native:
        scheme = scheme.with_store(QuantStore.Native)
    rng = np.random.default_rng(seed)
    w32 = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    w32[rng.random((rows, cols)) < 0.002] *= 20
    wb = oracle.to_bits(w32, elem)
    scales = oracle.compute_scales(wb, elem, (rows, cols), scheme)
    words, out_scale = oracle.quantize(wb, elem, (rows, cols), scales, scheme)
    deq = oracle.from_bits(oracle.dequantize(words, (rows, cols), out_scale, elem, scheme), elem).astype(np.float64)
    xb = oracle.to_bits(rng.normal(0, 1, (vectors, cols)).astype(np.float32), elem).reshape(vectors, cols)
    x64 = oracle.from_bits(xb, elem).astype(np.float64).reshape(vectors, cols)
    want = x64 @ deq.T           # [vectors, rows]
    mag = np.abs(x64) @ np.abs(deq).T

    nq = scheme.num_quants()
    wpr = cols // nq
    pitch = pitch or wpr
    buf = np.zeros((rows, pitch), np.uint8 if native else np.uint32)  # native: stored elements are bytes
    buf[:, :wpr] = words.reshape(rows, wpr)
    d_words = torch.from_numpy(buf if native else buf.view(np.int32)).cuda()
    to16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda() if a.dtype == np.uint16 \
        else torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_scales, d_x = to16(out_scale), to16(xb)
    sshape = (1,) if block is None else tuple(d_scales.shape)
    h_words = TensorHandleRef(d_words.data_ptr(), (rows, wpr), (pitch, 1), 1 if native else 4)
    h_scales = TensorHandleRef(d_scales.data_ptr(), sshape, tuple(d_scales.stride()) if block else (1,),
                               d_scales.element_size())
    # one right-hand side as a vector, several as the rows of a matrix
    h_x = TensorHandleRef.from_torch(d_x) if vectors > 1 else TensorHandleRef.from_torch(d_x[0])
    client = ComputeClient.current()
    y32 = torch.full((vectors, rows), float("nan"), dtype=torch.float32, device="cuda")
    h_y = lambda t: TensorHandleRef.from_torch(t) if vectors > 1 else TensorHandleRef.from_torch(t[0])
    matvec.launch_ref(client, h_words, h_scales, scheme, h_x, h_y(y32), elem, ElemType.F32)
    torch.cuda.synchronize()
    got = y32.cpu().numpy().astype(np.float64)
    assert np.all(np.abs(got - want) <= 2e-5 * mag + 1e-30), (case, vectors, float(np.max(np.abs(got - want) / (mag + 1e-30))))
    if elem != ElemType.F32:  # the same sums, rounded once to the 16-bit type
        y16 = torch.zeros((vectors, rows), dtype=torch.int16, device="cuda")
        matvec.launch_ref(client, h_words, h_scales, scheme, h_x, h_y(y16), elem, elem)
        torch.cuda.synchronize()
        assert np.array_equal(y16.cpu().numpy().view(np.uint16).reshape(-1), oracle.to_bits(y32.cpu().numpy().reshape(-1), elem)), \
            (case, vectors)


@pytest.mark.parametrize("case", CASES, ids=_id)
def test_gemv_matches_oracle_dequantized_weights(oracle, case):
    elem, value, block, param, rows, cols, pitch = case
    check_case(oracle, case, rows * 7 + cols)


NATIVE_CASES = [
    # the native store: e4m3 / e5m2 / i8 bytes (16 values per 16-byte unit), e2m1 pairs (32 values)
    (ElemType.BF16, QuantValue.E4M3, [32], QuantParam.F32, 77, 4128, None),
    (ElemType.F16, QuantValue.E4M3, [128, 128], QuantParam.F32, 256, 2048, None),   # 128 x 128 weight blocks
    (ElemType.BF16, QuantValue.E5M2, [16], QuantParam.BF16, 30, 2064, 2096),        # a scale per unit, pitched rows
    (ElemType.F16, QuantValue.E5M2, None, QuantParam.F16, 21, 16400, None),         # per tensor, eight waves
    (ElemType.BF16, QuantValue.E2M1, [32], QuantParam.F32, 53, 8448, None),         # e2m1 pairs, a scale per unit
    (ElemType.F16, QuantValue.E2M1, [64], QuantParam.F16, 18, 1088, None),
    (ElemType.BF16, QuantValue.Q8S, [32], QuantParam.F32, 45, 2080, None),          # i8 bytes: the 8-bit fields
    (ElemType.F16, QuantValue.Q8F, [16], QuantParam.BF16, 9, 16, None),             # one unit per row
    (ElemType.F32, QuantValue.E4M3, [32], QuantParam.F32, 37, 2080, None),          # x in f32
    (ElemType.F32, QuantValue.E2M1, [64], QuantParam.F32, 12, 4160, None),
    (ElemType.BF16, QuantValue.E2M1_OCP, [32], QuantParam.F32, 41, 4160, None),     # the extension value: e2m1 pairs
]


@pytest.mark.parametrize("case", NATIVE_CASES, ids=_id)
def test_gemv_native_store_matches_oracle_dequantized_weights(oracle, case):
    elem, value, block, param, rows, cols, pitch = case
    check_case(oracle, case, rows * 11 + cols, native=True)


# 4-bit fields on blocks of 32 with f32 scales, rows of whole groups of 128 values: two to four vectors at once go to
# the matrix-core kernel (rows in runs of 2048 or 4096 values; a last run cut short; rows not a multiple of 16; pitched
# rows; more vectors than four in turns, a last single one on the streaming kernel)
MATRIX_CORE_CASES = [
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 64, 4096, None),
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 77, 4224, None),
    (ElemType.F16, QuantValue.Q4F, [32], QuantParam.F32, 333, 8192, None),
    (ElemType.BF16, QuantValue.E2M1, [32], QuantParam.F32, 130, 11008, None),
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 50, 8448, 1060),
    (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, 21, 16512, None),
    (ElemType.F16, QuantValue.Q4S, [32], QuantParam.F32, 5, 6144, None),
    (ElemType.BF16, QuantValue.Q4F, [32], QuantParam.F32, 1, 4096, None),
]


@pytest.mark.parametrize("vectors", [2, 3, 4, 5, 9])
@pytest.mark.parametrize("case", MATRIX_CORE_CASES, ids=_id)
def test_gemv_on_the_matrix_cores(oracle, case, vectors):
    check_case(oracle, case, 3 + vectors, vectors=vectors)


@pytest.mark.parametrize("vectors", [2, 3, 4, 7, 8, 11])
@pytest.mark.parametrize("kind", ["q4-b32", "q8-b64-f16", "e4m3-native", "q4-general", "q4-wide", "e2m1-native-wide",
                                  "e5m2-native", "q2-in-turns"])
def test_gemv_with_several_right_hand_sides(oracle, kind, vectors):
    """x [vectors, cols] -> y [vectors, rows]: every row of y is the product with that row of x, whichever way the
    vectors are taken (up to four or eight at once by the streaming kernel, in turns otherwise)."""
    import torch

    elem, value, block, param, native, rows, cols = {
        "q4-b32": (ElemType.BF16, QuantValue.Q4S, [32], QuantParam.F32, False, 70, 4160),
        "q8-b64-f16": (ElemType.F16, QuantValue.Q8S, [64], QuantParam.F16, False, 33, 2112),
        "e4m3-native": (ElemType.BF16, QuantValue.E4M3, [32], QuantParam.F32, True, 41, 1056),
        "q4-general": (ElemType.BF16, QuantValue.Q4S, [8], QuantParam.F32, False, 20, 512),   # blocks narrower than a unit
        "e5m2-native": (ElemType.F16, QuantValue.E5M2, [64], QuantParam.F32, True, 26, 2112),
        "q2-in-turns": (ElemType.BF16, QuantValue.Q2S, [64], QuantParam.F32, False, 14, 1088),   # 2-bit: one vector per launch
        "q4-wide": (ElemType.BF16, QuantValue.Q4S, [64], QuantParam.BF16, False, 19, 18560),   # five segments of x, the last short
        "e2m1-native-wide": (ElemType.F16, QuantValue.E2M1, [32], QuantParam.F32, True, 10, 10304),
    }[kind]
    scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block(block)).with_param(param)
    if native:
        scheme = scheme.with_store(QuantStore.Native)
    rng = np.random.default_rng(vectors * 100 + cols)
    w32 = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    wb = oracle.to_bits(w32, elem)
    scales = oracle.compute_scales(wb, elem, (rows, cols), scheme)
    words, out_scale = oracle.quantize(wb, elem, (rows, cols), scales, scheme)
    deq = oracle.from_bits(oracle.dequantize(words, (rows, cols), out_scale, elem, scheme), elem).astype(np.float64)
    xpitch = cols + 8 * int(rng.integers(0, 3))  # rows of x on 16-byte boundaries, sometimes pitched
    xb = np.zeros((vectors, xpitch), np.uint16)
    xb[:, :cols] = oracle.to_bits(rng.normal(0, 1, (vectors, cols)).astype(np.float32), elem).reshape(vectors, cols)
    x64 = oracle.from_bits(xb[:, :cols].copy(), elem).astype(np.float64).reshape(vectors, cols)
    want, mag = x64 @ deq.T, np.abs(x64) @ np.abs(deq).T
    wpr = cols // scheme.num_quants()
    stored = words.reshape(rows, wpr)
    d_words = torch.from_numpy(stored if native else stored.view(np.int32)).cuda()
    to16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda() if a.dtype == np.uint16 \
        else torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_scales, d_x = to16(out_scale), to16(xb)
    h = TensorHandleRef.from_torch
    h_x = TensorHandleRef(d_x.data_ptr(), (vectors, cols), (xpitch, 1), 2)
    y = torch.full((vectors, rows + 3), float("nan"), dtype=torch.float32, device="cuda")
    h_y = TensorHandleRef(y.data_ptr(), (vectors, rows), (rows + 3, 1), 4)
    matvec.launch_ref(ComputeClient.current(), h(d_words), h(d_scales), scheme, h_x, h_y, elem, ElemType.F32)
    torch.cuda.synchronize()
    got = y.cpu().numpy().astype(np.float64)
    assert np.all(np.isnan(got[:, rows:]))  # nothing written between the rows of y
    assert np.all(np.abs(got[:, :rows] - want) <= 2e-5 * mag + 1e-30), float(np.max(np.abs(got[:, :rows] - want) / (mag + 1e-30)))


def test_gemv_random_configurations(oracle):
    """Sixty drawn cases (CQ_RANDOM_GEMV=N: N) of the streaming kernel's domain and its edges: every code width,
    block extents from one 16-byte unit up (also over rows), one scale per tensor, every scale type, ragged strips,
    pitched words, one to six right-hand sides, both stores, x in all three float types."""
    import os

    rng = np.random.default_rng(2024)
    values = {2: [QuantValue.Q2S, QuantValue.Q2F], 4: [QuantValue.Q4S, QuantValue.Q4F, QuantValue.E2M1],
              8: [QuantValue.Q8S, QuantValue.Q8F]}
    for i in range(int(os.environ.get("CQ_RANDOM_GEMV", "60"))):
        bits = int(rng.choice([2, 4, 8]))
        unit = 128 // bits
        elem = [ElemType.BF16, ElemType.F16, ElemType.BF16, ElemType.F32][int(rng.integers(4))]
        param = [QuantParam.F32, QuantParam.F16, QuantParam.BF16][int(rng.integers(3))]
        if elem == ElemType.F32 and rng.random() < 0.8:
            param = QuantParam.F32  # (f32 x streams under f32 scales; the rest goes to the general kernel)
        kind = int(rng.integers(4))
        units_per_block = int(2 ** rng.integers(0, 3))
        bc = unit * units_per_block
        if bc > 255:  # block extents are bytes in the scheme
            bc, units_per_block = unit, 1
        blocks = int(rng.integers(1, max(2, 6000 // bc)))
        cols = bc * blocks
        rows = int(rng.integers(1, 70))
        block = [bc]
        if kind == 0:
            block = None
        elif kind == 1:
            br = int(rng.choice([2, 3, 5]))
            rows = br * int(rng.integers(1, 20))
            block = [br, bc]
        value = values[bits][int(rng.integers(len(values[bits])))]
        wpr = cols // (32 // bits)
        pitch = None if rng.random() < 0.6 else wpr + 4 * int(rng.integers(1, 5))
        vectors = int(rng.choice([1, 1, 1, 2, 4, 5, 6]))
        # every third case in the native store, where the value has one (bytes: the pitch counts bytes)
        native = i % 3 == 2 and value in (QuantValue.Q8S, QuantValue.Q8F, QuantValue.E2M1)
        if native and elem == ElemType.F32:
            param = QuantParam.F32  # the native store only streams, and f32 x streams under f32 scales
        if native:
            pitch = None if pitch is None else (cols // (2 if value == QuantValue.E2M1 else 1)) + 16 * int(rng.integers(1, 4))
        check_case(oracle, (elem, value, block, param, rows, cols, pitch), 1000 + i, native=native, vectors=vectors)


@pytest.mark.parametrize("elem", [ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_gemv_scales_of_every_kind(oracle, elem):
    """Negative, zero, tiny and huge scales among ordinary ones (the streaming kernel sends their lanes down a
    plain path): same tolerance against the oracle's dequantized weights."""
    import torch

    rows, cols = 96, 4096
    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))
    rng = np.random.default_rng(5)
    words = rng.integers(0, 2**32, (rows, cols // 8), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.001, 0.02, (rows, cols // 32)).astype(np.float32)
    odd = rng.random(scales.shape) < 0.05
    scales[odd] = rng.choice(np.array([-0.01, 0.0, -0.0, 1e-36, -3.0, 2.0 ** -110, 3000.0, -1e-30], np.float32), int(odd.sum()))
    deq = oracle.from_bits(oracle.dequantize(words, (rows, cols), scales, elem, scheme), elem).astype(np.float64)
    assert np.all(np.isfinite(deq))
    d_words = torch.from_numpy(words.view(np.int32)).cuda()
    d_scales = torch.from_numpy(scales).cuda()
    h = TensorHandleRef.from_torch
    for vectors in (1, 3):  # one right-hand side, and three at once
        xb = oracle.to_bits(rng.normal(0, 1, (vectors, cols)).astype(np.float32), elem).reshape(vectors, cols)
        x64 = oracle.from_bits(xb, elem).astype(np.float64).reshape(vectors, cols)
        want, mag = x64 @ deq.T, np.abs(x64) @ np.abs(deq).T
        d_x = torch.from_numpy(xb.view(np.int16)).cuda()
        y = torch.zeros((vectors, rows), dtype=torch.float32, device="cuda")
        hx, hy = (h(d_x), h(y)) if vectors > 1 else (h(d_x[0]), h(y[0]))
        matvec.launch_ref(ComputeClient.current(), h(d_words), h(d_scales), scheme, hx, hy, elem, ElemType.F32)
        torch.cuda.synchronize()
        got = y.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - want) <= 2e-5 * mag + 1e-30), (vectors, float(np.max(np.abs(got - want) / (mag + 1e-30))))


def test_gemv_scales_with_strides(oracle):
    """The scales of a [rows, blocks] layout stored column by column (strides (1, rows)) and with a row pitch:
    the streaming kernel addresses them through both strides."""
    import torch

    rows, cols = 37, 2304
    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))
    rng = np.random.default_rng(11)
    words = rng.integers(0, 2**32, (rows, cols // 8), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.001, 0.02, (rows, cols // 32)).astype(np.float32)
    deq = oracle.from_bits(oracle.dequantize(words, (rows, cols), scales, ElemType.BF16, scheme), ElemType.BF16).astype(np.float64)
    xb = oracle.to_bits(rng.normal(0, 1, cols).astype(np.float32), ElemType.BF16)
    x64 = oracle.from_bits(xb, ElemType.BF16).astype(np.float64)
    want, mag = deq @ x64, np.abs(deq) @ np.abs(x64)
    d_words = torch.from_numpy(words.view(np.int32)).cuda()
    d_x = torch.from_numpy(xb.view(np.int16)).cuda()
    h = TensorHandleRef.from_torch
    nb = cols // 32
    col_major = torch.from_numpy(np.ascontiguousarray(scales.T)).cuda()           # [blocks, rows]
    pitched = torch.zeros((rows, nb + 5), dtype=torch.float32, device="cuda")
    pitched[:, :nb] = torch.from_numpy(scales).cuda()
    for name, h_scales in (("column-major", TensorHandleRef(col_major.data_ptr(), (rows, nb), (1, rows), 4)),
                           ("pitched", TensorHandleRef(pitched.data_ptr(), (rows, nb), (nb + 5, 1), 4))):
        y = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
        matvec.launch_ref(ComputeClient.current(), h(d_words), h_scales, scheme, h(d_x), h(y), ElemType.BF16, ElemType.F32)
        torch.cuda.synchronize()
        got = y.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - want) <= 2e-5 * mag + 1e-30), name


@pytest.mark.parametrize("kind", ["e4m3-native", "q4-f32-x", "q4-bf16", "q4-bf16-four-vectors"])
def test_gemv_infinite_scale_in_a_rows_last_unit(oracle, kind):
    """Rows whose last strip is partly filled (cols / values per unit is not a multiple of 64), with an infinite scale
    on the last block of one row and +-0 codes elsewhere in it: the lanes past the row's end must contribute nothing
    (they hold the last unit again against zeros of x, and Inf * 0 is NaN).  The row with the infinite scale sums to
    +-Inf or NaN exactly where the float64 product over the oracle's dequantized weights does; every other row is
    finite and within the tolerance."""
    import torch

    native = kind == "e4m3-native"
    elem = ElemType.F32 if kind == "q4-f32-x" else ElemType.BF16
    vectors = 4 if kind.endswith("four-vectors") else 1
    value = QuantValue.E4M3 if native else QuantValue.Q4S
    scheme = QuantScheme.default().with_value(value).with_level(QuantLevel.block([32]))
    if native:
        scheme = scheme.with_store(QuantStore.Native)
    rows, cols = 6, 2080   # 65 units of 32 values (130 of 16 for the bytes): the last strip holds one or two units
    rng = np.random.default_rng(21)
    nq = scheme.num_quants()
    if native:
        stored = rng.integers(0, 120, (rows, cols), dtype=np.uint8) | (rng.integers(0, 2, (rows, cols), dtype=np.uint8) << 7)
    else:
        stored = rng.integers(0, 2**32, (rows, cols // nq), dtype=np.uint64).astype(np.uint32)
    scales = rng.uniform(0.001, 0.02, (rows, cols // 32)).astype(np.float32)
    scales[2, -1] = np.inf
    # that block's codes are all +3 (e4m3: 1.0) and x is +1 there, so row 2 sums to +Inf, not to NaN
    if native:
        stored[2, -32:] = 0x38
    else:
        stored[2, -(32 // nq):] = 0x33333333
    deq = oracle.from_bits(oracle.dequantize(stored, (rows, cols), scales, elem, scheme), elem).astype(np.float64)
    xb = oracle.to_bits(rng.normal(0, 1, (vectors, cols)).astype(np.float32), elem).reshape(vectors, cols)
    xb[:, -32:] = oracle.to_bits(np.ones(32, np.float32), elem)
    x64 = oracle.from_bits(xb, elem).astype(np.float64).reshape(vectors, cols)
    with np.errstate(invalid="ignore", over="ignore"):
        want, mag = x64 @ deq.T, np.abs(x64) @ np.abs(deq).T
    d_stored = torch.from_numpy(stored if native else stored.view(np.int32)).cuda()
    d_scales = torch.from_numpy(scales).cuda()
    d_x = torch.from_numpy(xb.view(np.int16) if elem != ElemType.F32 else xb).cuda()
    h = TensorHandleRef.from_torch
    y = torch.zeros((vectors, rows), dtype=torch.float32, device="cuda")
    hx, hy = (h(d_x), h(y)) if vectors > 1 else (h(d_x[0]), h(y[0]))
    matvec.launch_ref(ComputeClient.current(), h(d_stored), h(d_scales), scheme, hx, hy, elem, ElemType.F32)
    torch.cuda.synchronize()
    got = y.cpu().numpy().astype(np.float64)
    finite = np.isfinite(want)
    assert np.all(want[:, 2] == np.inf) and finite[:, [0, 1, 3, 4, 5]].all()
    assert np.all(np.abs(got - want)[finite] <= (2e-5 * mag + 1e-30)[finite]), kind
    assert np.array_equal(np.isnan(got), np.isnan(want)), (kind, got[:, 2], want[:, 2])
    assert np.array_equal(got[~finite & ~np.isnan(want)], want[~finite & ~np.isnan(want)]), (kind, got[:, 2], want[:, 2])


def test_gemv_without_columns_gives_zeros():
    """cols == 0: every sum is empty, y is written with zeros (one vector and three)."""
    import torch

    scheme = QuantScheme.default().with_value(QuantValue.Q4S)
    h = TensorHandleRef
    w = torch.zeros(4, dtype=torch.int32, device="cuda")
    s = torch.ones(1, dtype=torch.float32, device="cuda")
    x = torch.zeros(4, dtype=torch.bfloat16, device="cuda")
    for vectors in (1, 3):
        y = torch.full((vectors, 7), float("nan"), dtype=torch.float32, device="cuda")
        h_x = h(x.data_ptr(), (0,), (1,), 2) if vectors == 1 else h(x.data_ptr(), (vectors, 0), (0, 1), 2)
        h_y = h.from_torch(y[0]) if vectors == 1 else h.from_torch(y)
        matvec.launch_ref(ComputeClient.current(), h(w.data_ptr(), (7, 0), (0, 1), 4), h.from_torch(s), scheme, h_x, h_y,
                          ElemType.BF16, ElemType.F32)
        torch.cuda.synchronize()
        assert torch.equal(y, torch.zeros_like(y)), vectors


def test_gemv_argument_checks():
    import torch

    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))
    w = torch.zeros((8, 16), dtype=torch.int32, device="cuda")
    s = torch.ones((8, 4), dtype=torch.float32, device="cuda")
    x = torch.zeros(128, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(8, dtype=torch.float32, device="cuda")
    h = TensorHandleRef.from_torch
    client = ComputeClient.current()
    matvec.launch_ref(client, h(w), h(s), scheme, h(x), h(y), ElemType.BF16, ElemType.F32)

    def status(fn):
        with pytest.raises(_ffi.QuantError) as e:
            fn()
        return e.value.status

    assert status(lambda: matvec.launch_ref(client, h(w), h(s), scheme, h(x[:64]), h(y), ElemType.BF16, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: matvec.launch_ref(client, h(w), h(s[:, :3]), scheme, h(x), h(y), ElemType.BF16, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: matvec.launch_ref(client, h(w), h(s), scheme, h(x), h(y), ElemType.F32, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH  # x is not f32
    from cubek_amd import QuantStore
    assert status(lambda: matvec.launch_ref(client, h(w), h(s), scheme.with_store(QuantStore.Native), h(x), h(y),
                                            ElemType.BF16, ElemType.F32)) == _ffi.ERR_UNSUPPORTED_SCHEME
    assert status(lambda: matvec.launch_ref(client, h(w.t()), h(s), scheme, h(x), h(y), ElemType.BF16, ElemType.F32)) \
        in (_ffi.ERR_NON_CONTIGUOUS, _ffi.ERR_SHAPE_MISMATCH)
