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
