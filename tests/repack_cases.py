"""Shared by the CPU and GPU tests of into_contiguous_packed: cases and a numpy model
that builds the strided, packed input from a logical array (the inverse direction)."""
import numpy as np

# (name, stored dtype, packing, logical shape, packed_dim, memory order of the input's dims
#  from slowest to fastest)
CASES = [
    ("u32x4_rows_pitched", np.uint32, 4, (6, 32), 1, (0, 1)),
    ("u32x8_transposed", np.uint32, 8, (16, 24), 0, (1, 0)),
    ("u32x4_transposed", np.uint32, 4, (64, 128), 0, (1, 0)),
    ("u32x16_transposed", np.uint32, 16, (32, 48), 0, (1, 0)),
    ("u32x8_batched_transposed", np.uint32, 8, (3, 16, 40), 1, (0, 2, 1)),
    ("u32x8_batch_swapped", np.uint32, 8, (3, 4, 16), 2, (1, 0, 2)),
    ("u32x4_rank4_mixed", np.uint32, 4, (2, 8, 3, 12), 1, (2, 0, 3, 1)),
    ("u8x2_transposed", np.uint8, 2, (10, 6), 0, (1, 0)),
    ("u8x2_batched_transposed", np.uint8, 2, (2, 8, 12), 1, (0, 2, 1)),
    ("u32x8_vector", np.uint32, 8, (64,), 0, (0,)),
]


def pack_last(logical: np.ndarray, dtype, packing: int) -> np.ndarray:
    bits = 8 * np.dtype(dtype).itemsize // packing
    g = logical.reshape(logical.shape[:-1] + (logical.shape[-1] // packing, packing)).astype(np.uint64)
    out = np.zeros(g.shape[:-1], dtype=np.uint64)
    for k in range(packing):
        out |= g[..., k] << np.uint64(k * bits)
    return out.astype(dtype)


def scatter_packed(logical: np.ndarray, dtype, packing: int, packed_dim: int, order, rng, pad: int = 3):
    """Pack `logical` along packed_dim and lay the result out in memory with the dims
    ordered `order` (slowest first); the rows of the fastest dim get `pad` extra elements.  Returns (buffer, strides in elements)."""
    moved = np.moveaxis(logical, packed_dim, -1)
    packed = np.moveaxis(pack_last(moved, dtype, packing), -1, packed_dim)  # shape with packed_dim / packing
    in_shape = packed.shape
    strides = [0] * len(in_shape)
    acc = 1
    for i, d in enumerate(reversed(order)):
        strides[d] = acc
        acc *= in_shape[d] + (pad if i == 0 else 0)  # pad the pitch of the fastest dim
    reach = 1 + sum((n - 1) * st for n, st in zip(in_shape, strides))
    info = np.iinfo(dtype)
    buf = rng.integers(0, int(info.max) + 1, size=reach, dtype=np.uint64).astype(dtype)  # garbage in the gaps
    view = np.lib.stride_tricks.as_strided(buf, in_shape, tuple(s * buf.itemsize for s in strides))
    view[...] = packed
    return buf, tuple(strides)
