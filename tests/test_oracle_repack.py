"""cqo_into_contiguous_packed against its definition stated the other way round: scatter
a logical array of small integers into a strided tensor packed along `packed_dim`,
and expect the gather to return the same array packed along the last dimension."""
import numpy as np
import pytest

from repack_cases import CASES, pack_last, scatter_packed


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_into_contiguous_packed_matches_definition(oracle, case):
    name, dtype, packing, shape, packed_dim, order = case
    rng = np.random.default_rng(len(name) * 7 + packing)
    bits = 8 * np.dtype(dtype).itemsize // packing
    logical = rng.integers(0, 1 << bits, size=shape, dtype=np.uint64)
    buf, in_strides = scatter_packed(logical, dtype, packing, packed_dim, order, rng)
    got = oracle.into_contiguous_packed(buf, packing, shape, in_strides, packed_dim)
    assert np.array_equal(got, pack_last(logical, dtype, packing))


def test_already_contiguous_is_a_copy(oracle):
    rng = np.random.default_rng(1)
    words = rng.integers(0, 1 << 32, size=(5, 3, 4), dtype=np.uint64).astype(np.uint32)
    got = oracle.into_contiguous_packed(words.reshape(-1), 8, (5, 3, 32), (12, 4, 1), 2)
    assert np.array_equal(got, words)


def test_repacking_a_transposed_quantized_tensor_gives_the_directly_quantized_one(oracle):
    """Ties the field order to the quantize path (which the golden vectors pin): quantize x^T, view
    the result as the logical x packed along its first dimension, re-pack -> the words of quantize(x)."""
    from cubek_amd import ElemType, QuantScheme, QuantValue

    rng = np.random.default_rng(5)
    rows, cols = 16, 48
    for value, nq in ((QuantValue.Q4S, 8), (QuantValue.Q2F, 16), (QuantValue.Q8S, 4)):
        if rows % nq:
            continue
        scheme = QuantScheme.default().with_value(value)
        x = rng.normal(0, 1, (rows, cols)).astype(np.float32)
        scale = oracle.compute_scales(x, ElemType.F32, (rows, cols), scheme)
        direct, _ = oracle.quantize(x, ElemType.F32, (rows, cols), scale, scheme)
        xt = np.ascontiguousarray(x.T)
        of_transposed, _ = oracle.quantize(xt, ElemType.F32, (cols, rows), scale, scheme)   # [cols, rows / nq]
        # stored element (i, c) of the logical [rows, cols] tensor packed along dim 0 sits at c * (rows / nq) + i
        got = oracle.into_contiguous_packed(of_transposed.reshape(-1), nq, (rows, cols), (1, rows // nq), 0)
        assert np.array_equal(got, direct.reshape(rows, cols // nq)), value
