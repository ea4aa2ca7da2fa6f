"""cq_into_contiguous_packed (through the C ABI) against the CPU oracle, bit for bit."""
import numpy as np
import pytest

from cubek_amd import ComputeClient, QuantError, _ffi
from cubek_amd import contiguous as cq_contiguous
from repack_cases import CASES, pack_last, scatter_packed

pytestmark = pytest.mark.gpu

BIG = [
    ("u32x8_transposed_big", np.uint32, 8, (1024, 768), 0, (1, 0)),
    ("u32x4_transposed_ragged_tiles", np.uint32, 4, (528, 1008), 0, (1, 0)),
    ("u32x8_transposed_ragged_tiles", np.uint32, 8, (2080, 2336), 0, (1, 0)),
    ("u32x16_transposed_ragged_tiles", np.uint32, 16, (320, 1088), 0, (1, 0)),
    ("u32x8_rank4_batched_transposed", np.uint32, 8, (2, 3, 64, 96), 2, (1, 0, 3, 2)),
    ("u32x8_batch_between", np.uint32, 8, (64, 5, 128), 0, (1, 2, 0)),
    ("u32x16_transposed_big", np.uint32, 16, (512, 2048), 0, (1, 0)),
    ("u32x8_batched_transposed_big", np.uint32, 8, (3, 256, 640), 1, (0, 2, 1)),
    ("u32x8_rows_pitched_big", np.uint32, 8, (300, 4096), 1, (0, 1)),
    ("u8x2_transposed_big", np.uint8, 2, (512, 384), 0, (1, 0)),
    ("u8x2_transposed_ragged_tiles", np.uint8, 2, (2080, 1312), 0, (1, 0)),
    ("u8x2_batched_transposed_big", np.uint8, 2, (3, 256, 640), 1, (0, 2, 1)),
    ("u8x2_transposed_not_word_multiple", np.uint8, 2, (516, 388), 0, (1, 0)),
    # packed along the contiguous last dimension: copies of strided rows
    ("u32x8_rows_heads_swapped", np.uint32, 8, (2, 6, 40, 128), 3, (0, 2, 1, 3)),
    ("u32x8_rows_leading_swapped", np.uint32, 8, (5, 3, 2048), 2, (1, 0, 2)),
    ("u8x2_rows_pitched_big", np.uint8, 2, (300, 4096), 1, (0, 1)),
    ("u8x2_rows_heads_swapped", np.uint8, 2, (2, 6, 40, 96), 3, (0, 2, 1, 3)),
]


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def run(gpu, buf, dtype, packing, shape, in_strides, packed_dim):
    import torch

    in_shape = tuple(s // packing if d == packed_dim else s for d, s in enumerate(shape))
    out_shape = tuple(shape[:-1]) + (shape[-1] // packing,)
    d_in = gpu.to_dev(buf)
    d_out = torch.zeros(out_shape, dtype=torch.int32 if dtype == np.uint32 else torch.uint8, device="cuda")
    cq_contiguous.into_contiguous_packed_ref(ComputeClient.current(), gpu.handle(d_in, in_shape, in_strides),
                                             gpu.handle(d_out), shape, packing)
    torch.cuda.synchronize()
    return gpu.to_host(d_out).view(dtype)


@pytest.mark.parametrize("pad", [0, 3, 4], ids=lambda p: f"pad{p}")
@pytest.mark.parametrize("case", CASES + BIG, ids=[c[0] for c in CASES + BIG])
def test_into_contiguous_packed(gpu, oracle, case, pad):
    # pad 0 / 4 keep the rows 16-byte aligned (tiled transposition where it applies),
    # pad 3 does not (per-element kernel)
    name, dtype, packing, shape, packed_dim, order = case
    rng = np.random.default_rng(len(name) * 5 + packing)
    bits = 8 * np.dtype(dtype).itemsize // packing
    logical = rng.integers(0, 1 << bits, size=shape, dtype=np.uint64)
    buf, in_strides = scatter_packed(logical, dtype, packing, packed_dim, order, rng, pad)
    want = oracle.into_contiguous_packed(buf, packing, shape, in_strides, packed_dim)
    assert np.array_equal(want, pack_last(logical, dtype, packing))
    got = run(gpu, buf, dtype, packing, shape, in_strides, packed_dim)
    assert np.array_equal(got, want)


def test_quantize_transposed_then_repack_equals_quantize_of_transpose(gpu, oracle):
    """The use cubek-matmul makes of it: weights quantized as [N, K] (per-tensor scale),
    viewed transposed as [K, N], re-packed, must equal the packed codes of the
    transposed weights."""
    from cubek_amd import ElemType, QuantScheme, QuantValue

    rng = np.random.default_rng(2)
    n, k = 96, 64
    scheme = QuantScheme.default().with_value(QuantValue.Q4S)
    w = rng.normal(0, 1, (n, k)).astype(np.float32)
    s = oracle.compute_scales(w, ElemType.F32, (n, k), scheme)
    codes_nk, _ = gpu.quantize(w, ElemType.F32, (n, k), s, scheme)            # [n, k/8] words
    codes_kn, _ = gpu.quantize(np.ascontiguousarray(w.T), ElemType.F32, (k, n), s, scheme)  # [k, n/8]
    # transposed view of codes_nk: logical [k, n], packed along dim 0 (stride 1), dim 1 stride k/8
    got = run(gpu, codes_nk.reshape(-1), np.uint32, 8, (k, n), (1, k // 8), 0)
    assert np.array_equal(got, codes_kn.reshape(k, n // 8))


def test_into_contiguous_packed_errors(gpu):
    import torch

    client = ComputeClient.current()
    src = torch.zeros((16, 4), dtype=torch.int32, device="cuda")
    dst = torch.zeros((16, 4), dtype=torch.int32, device="cuda")

    def status(fn):
        with pytest.raises(QuantError) as e:
            fn()
        return e.value.status

    h = gpu.handle
    assert status(lambda: cq_contiguous.into_contiguous_packed_ref(client, h(src), h(dst), (16, 30), 8)) \
        == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: cq_contiguous.into_contiguous_packed_ref(client, h(src), h(dst), (16, 32), 5)) \
        == _ffi.ERR_INVALID_ARGUMENT
    assert status(lambda: cq_contiguous.into_contiguous_packed_ref(client, h(src), h(dst, (16, 4), (8, 1)), (16, 32), 8)) \
        == _ffi.ERR_NON_CONTIGUOUS


@pytest.mark.parametrize("seed", range(6))
def test_into_contiguous_packed_random(gpu, oracle, seed):
    """Seeded random rank / shape / packed dimension / memory order / padding."""
    rng = np.random.default_rng(500 + seed)
    for _ in range(10):
        dtype, packing = [(np.uint32, 4), (np.uint32, 8), (np.uint32, 16), (np.uint8, 2)][int(rng.integers(4))]
        rank = int(rng.integers(1, 5))
        shape = [int(rng.choice([1, 2, 3, 5, 8, 12])) for _ in range(rank)]
        packed_dim = int(rng.integers(rank))
        mult = packing * (4 if rng.random() < 0.5 else 1)  # word-quad multiples reach the tiled kernel
        shape[packed_dim] = mult * int(rng.integers(1, 12))
        shape[-1] = (mult if packed_dim != rank - 1 else shape[-1]) * (int(rng.integers(1, 12)) if packed_dim != rank - 1 else 1)
        shape = tuple(shape)
        # memory order: the packed dimension is the fastest one (stride 1)
        lead = [d for d in range(rank) if d != packed_dim]
        rng.shuffle(lead)
        order = tuple(lead + [packed_dim])
        pad = int(rng.choice([0, 3, 4]))
        bits = 8 * np.dtype(dtype).itemsize // packing
        logical = rng.integers(0, 1 << bits, size=shape, dtype=np.uint64)
        buf, in_strides = scatter_packed(logical, dtype, packing, packed_dim, order, rng, pad)
        # the library finds the packed dimension itself: the rightmost one with stride 1
        in_shape = tuple(s // packing if d == packed_dim else s for d, s in enumerate(shape))
        rightmost = max(d for d in range(rank) if in_strides[d] == 1)
        if rightmost != packed_dim:
            continue  # another dimension of extent 1 also has stride 1: ambiguous by construction
        want = oracle.into_contiguous_packed(buf, packing, shape, in_strides, packed_dim)
        assert np.array_equal(want, pack_last(logical, dtype, packing))
        got = run(gpu, buf, dtype, packing, shape, in_strides, packed_dim)
        assert np.array_equal(got, want), (dtype.__name__, packing, shape, packed_dim, order, pad)
