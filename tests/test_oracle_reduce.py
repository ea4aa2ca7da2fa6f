"""cqo_reduce_max_abs against numpy's abs().max() (library routine) and its invariants."""
import numpy as np
import pytest

from cubek_amd import ElemType


@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_reduce_max_abs_matches_numpy(oracle, elem):
    rng = np.random.default_rng(int(elem) + 40)
    for shape in ((7,), (5, 9), (3, 4, 6), (2, 3, 4, 5), (4, 1, 8)):
        x32 = rng.normal(0, 3, shape).astype(np.float32)
        x = oracle.to_bits(x32, elem)
        vals = oracle.from_bits(x, elem).reshape(shape)
        for axis in range(len(shape)):
            got = oracle.from_bits(oracle.reduce_max_abs(x, elem, shape, axis), elem)
            want = np.abs(vals).max(axis=axis, keepdims=True)
            assert got.shape == want.shape and np.array_equal(got, want)


def test_reduce_max_abs_strides_nan_and_empty_axis(oracle):
    rng = np.random.default_rng(3)
    base = rng.normal(0, 1, (6, 10)).astype(np.float32)
    # transposed view [10, 6] of the buffer: strides (1, 10)
    got = oracle.reduce_max_abs(base.reshape(-1), ElemType.F32, (10, 6), 0, in_strides=(1, 10))
    assert np.array_equal(got.reshape(-1), np.abs(base).max(axis=1))
    x = np.array([[np.nan, -2.0, 1.0], [np.nan, np.nan, np.nan]], np.float32)
    assert oracle.reduce_max_abs(x, ElemType.F32, (2, 3), 1).reshape(-1).tolist() == [2.0, 0.0]
    # permutation along the axis does not change the result; the axis of extent 1 is |x|
    y = rng.normal(0, 1, (4, 7)).astype(np.float32)
    p = rng.permutation(7)
    assert np.array_equal(oracle.reduce_max_abs(y, ElemType.F32, (4, 7), 1),
                          oracle.reduce_max_abs(np.ascontiguousarray(y[:, p]), ElemType.F32, (4, 7), 1))
    assert np.array_equal(oracle.reduce_max_abs(y.reshape(4, 1, 7), ElemType.F32, (4, 1, 7), 1).reshape(4, 7), np.abs(y))
