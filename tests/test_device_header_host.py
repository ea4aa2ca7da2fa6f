"""Host-side parts of include/cubek_quant_device.hpp (no GPU): the multiply-and-shift divider and
ScalesLayout::{to_source_pos, is_block_start} against plain integer arithmetic and the oracle."""
import numpy as np

import device_header as dh
from cubek_amd.scheme import QuantLevel, QuantScheme


def test_fast_divmod_equals_integer_division():
    L = dh.lib()
    rng = np.random.default_rng(5)
    divisors = list(range(1, 300)) + [1000, 4096, 4097, 14336, 28672, 65535, 65536, 1 << 20, (1 << 31) - 1] + \
        [int(v) for v in rng.integers(1, 1 << 31, 60)]
    for d in divisors:
        ns = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 31) - 1, (1 << 31) - d] + \
             [int(v) for v in rng.integers(0, 1 << 31, 40)]
        for n in ns:
            if 0 <= n < (1 << 31):
                assert L.dh_host_fast_div(n, d) == n // d, (n, d)


def test_scales_layout_matches_brute_force_and_oracle(oracle):
    """Unravel the element index, divide each coordinate by its block extent (values_shape is the quantized
    tensor's shape: its last dimension is multiplied by num_quants, src/layout/scales.rs:246-258)."""
    L = dh.lib()
    rng = np.random.default_rng(12)
    for shape, block, nq in (((4, 8), (4,), 4), ((4, 8), (2, 4), 4), ((3, 4, 16), (2, 8), 8), ((2, 3, 4, 16), (3, 2, 16), 16),
                             ((5, 6, 8), (5, 2, 4), 4), ((6, 24), (1, 24), 8)):
        scheme = QuantScheme.default().with_level(QuantLevel.block(block))
        blk = (1,) * (len(shape) - len(block)) + tuple(block)
        strides = tuple(int(v) for v in rng.integers(1, 50, len(shape)))
        vshape = tuple(shape[:-1]) + (shape[-1] // nq,)
        args = (dh.u64(vshape), len(shape), nq, dh.u64(strides), dh.u8(block), len(block))
        for e in range(int(np.prod(shape))):
            coords = np.unravel_index(e, shape)
            want = sum((c // b) * s for c, b, s in zip(coords, blk, strides))
            assert L.dh_host_scale_pos(*args, e) == want == oracle.scale_index(scheme, shape, strides, e)
            assert bool(L.dh_host_is_block_start(*args, e)) == all(c % b == 0 for c, b in zip(coords, blk))
    # per tensor
    none = (dh.u64((4, 2)), 2, 4, dh.u64((0, 0)), dh.u8(()), 0)
    assert L.dh_host_scale_pos(*none, 17) == 0 and L.dh_host_is_block_start(*none, 0) and not L.dh_host_is_block_start(*none, 4)
    # positions at and beyond 2^31 take the 64-bit branch
    big = (dh.u64((1 << 20, 1 << 10)), 2, 4, dh.u64((128, 1)), dh.u8((32,)), 1)
    for e in ((1 << 31) - 1, 1 << 31, (1 << 32) - 5, (1 << 32) - 1):
        assert L.dh_host_scale_pos(*big, e) == (e // 4096) * 128 + (e % 4096) // 32


def test_scales_layout_of_an_empty_tensor_is_built_without_dividing_by_zero():
    """A zero-sized dimension must not reach the magic-number division on the host (1 << k) / 0; such a layout is
    never indexed, and a divisor of 0 stands for the division by 1."""
    L = dh.lib()
    assert L.dh_host_fast_div(12345, 0) == 12345
    empty = (dh.u64((0, 8)), 2, 4, dh.u64((1, 1)), dh.u8((32,)), 1)
    assert L.dh_host_scale_pos(*empty, 0) == 0
    empty_last = (dh.u64((4, 0)), 2, 4, dh.u64((1, 1)), dh.u8((32,)), 1)
    assert L.dh_host_scale_pos(*empty_last, 0) == 0
