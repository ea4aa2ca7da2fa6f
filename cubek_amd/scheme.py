"""Quantization scheme options: the Python mirror of the types the reference
re-exports as ``cubek_quant::scheme`` (crates/cubek-quant/src/lib.rs:14) and
builds in its tests with ``QuantScheme::default().with_level(..).with_value(..)``
(crates/cubek-quant/tests/suite/symmetric.rs:60-66, :201-207).

Pure host logic: nothing here touches the GPU or loads the native library.
"""
from __future__ import annotations

import ctypes
import enum
import functools
from dataclasses import dataclass, replace
from typing import Sequence, Tuple

MAX_BLOCK_DIMS = 5  # BlockSize storage of the reference's scheme type


class QuantValue(enum.IntEnum):
    Q8F = 0
    Q8S = 1
    Q4F = 2
    Q4S = 3
    Q2F = 4
    Q2S = 5
    E2M1 = 6
    E4M3 = 7
    E5M2 = 8
    #: extension without a counterpart in the reference: OCP FP4 rounded once, straight to the e2m1 grid
    #: (0.5 and 1.5 occur), e2m1 nibbles in either store; never what the E2M1 value of the reference produces
    E2M1_OCP = 9

    def size_bits(self) -> int:
        """Bits of one quantized value (call sites src/quantize.rs:62)."""
        if self in (QuantValue.Q8F, QuantValue.Q8S, QuantValue.E4M3, QuantValue.E5M2):
            return 8
        if self in (QuantValue.Q4F, QuantValue.Q4S, QuantValue.E2M1, QuantValue.E2M1_OCP):
            return 4
        return 2

    def range(self) -> Tuple[float, float]:
        """(q_min, q_max) as used at src/quantize.rs:243,296 and by the scale
        rule ``2*absmax/(q_max-q_min)`` (tests/suite/symmetric.rs:35-37)."""
        return _RANGES[self]

    def is_symmetric(self) -> bool:
        lo, hi = self.range()
        return lo == -hi


_RANGES = {
    QuantValue.Q8F: (-128.0, 127.0),
    QuantValue.Q8S: (-127.0, 127.0),
    QuantValue.Q4F: (-8.0, 7.0),
    QuantValue.Q4S: (-7.0, 7.0),
    QuantValue.Q2F: (-2.0, 1.0),
    QuantValue.Q2S: (-1.0, 1.0),
    QuantValue.E2M1: (-6.0, 6.0),
    QuantValue.E4M3: (-448.0, 448.0),
    QuantValue.E5M2: (-57344.0, 57344.0),
    QuantValue.E2M1_OCP: (-6.0, 6.0),
}


class QuantParam(enum.IntEnum):
    F32 = 0
    F16 = 1
    BF16 = 2


class QuantStore(enum.IntEnum):
    U32 = 0
    Native = 1

    def size_bits(self, value: QuantValue) -> int:
        """Bits of one stored element (call site src/dequantize.rs:92)."""
        return 32 if self == QuantStore.U32 else value.size_bits()


class QuantMode(enum.IntEnum):
    Symmetric = 0


class ElemType(enum.IntEnum):
    """Float element types of value tensors (the reference passes
    ``ElemType``/``StorageType``; Flex32 is stored as f32)."""

    F32 = 0
    F16 = 1
    BF16 = 2
    Flex32 = 0  # alias: same storage and arithmetic as F32 here

    @property
    def size(self) -> int:
        return 4 if self == ElemType.F32 else 2


@dataclass(frozen=True)
class BlockSize:
    """Block extents for the trailing dimensions, at most 5 entries of u8."""

    dims: Tuple[int, ...]

    def __post_init__(self):
        if not 1 <= len(self.dims) <= MAX_BLOCK_DIMS:
            raise ValueError(f"block size needs 1..{MAX_BLOCK_DIMS} dimensions, got {self.dims}")
        for d in self.dims:
            if not 1 <= int(d) <= 255:
                raise ValueError(f"block extents are u8 values in 1..255, got {self.dims}")

    def as_slice(self) -> Tuple[int, ...]:
        return self.dims

    def to_dim_vec(self, rank: int) -> Tuple[int, ...]:
        """Left-pad with 1s to ``rank`` entries (src/layout/scales.rs:239)."""
        if rank < len(self.dims):
            raise ValueError(f"block rank {len(self.dims)} exceeds tensor rank {rank}")
        return (1,) * (rank - len(self.dims)) + tuple(self.dims)

    def num_elements(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n


@dataclass(frozen=True)
class QuantLevel:
    """``QuantLevel::Tensor`` or ``QuantLevel::Block(block_size)``."""

    block_size: BlockSize | None = None

    Tensor = None  # filled in below

    @staticmethod
    def block(values: Sequence[int]) -> "QuantLevel":
        return QuantLevel(BlockSize(tuple(int(v) for v in values)))

    @property
    def is_tensor(self) -> bool:
        return self.block_size is None


QuantLevel.Tensor = QuantLevel(None)


class _CScheme(ctypes.Structure):
    """Binary layout of ``cq_scheme`` (include/cubek_quant.h)."""

    _fields_ = [
        ("value", ctypes.c_uint8),
        ("param", ctypes.c_uint8),
        ("store", ctypes.c_uint8),
        ("level", ctypes.c_uint8),
        ("mode", ctypes.c_uint8),
        ("block_rank", ctypes.c_uint8),
        ("block", ctypes.c_uint8 * MAX_BLOCK_DIMS),
        ("reserved", ctypes.c_uint8),
    ]


@dataclass(frozen=True)
class QuantScheme:
    """Default = Q8F / F32 params / U32 store / per-tensor / symmetric."""

    value: QuantValue = QuantValue.Q8F
    param: QuantParam = QuantParam.F32
    store: QuantStore = QuantStore.U32
    level: QuantLevel = QuantLevel.Tensor
    mode: QuantMode = QuantMode.Symmetric

    @staticmethod
    def default() -> "QuantScheme":
        return QuantScheme()

    def with_level(self, level: QuantLevel) -> "QuantScheme":
        return replace(self, level=level)

    def with_mode(self, mode: QuantMode) -> "QuantScheme":
        return replace(self, mode=mode)

    def with_value(self, value: QuantValue) -> "QuantScheme":
        return replace(self, value=value)

    def with_store(self, store: QuantStore) -> "QuantScheme":
        return replace(self, store=store)

    def with_param(self, param: QuantParam) -> "QuantScheme":
        return replace(self, param=param)

    def size_bits_stored(self) -> int:
        return self.store.size_bits(self.value)

    def size_bits_value(self) -> int:
        return self.value.size_bits()

    def native_packing(self) -> int:
        """Values per stored element of the native store (2 for e2m1 bytes)."""
        return 2 if (self.store == QuantStore.Native and self.value in (QuantValue.E2M1, QuantValue.E2M1_OCP)) else 1

    def num_quants(self) -> int:
        """Values per stored element: 32/size_bits for the U32 store
        (src/quantize.rs:290,305; tests/suite/symmetric.rs:69)."""
        if self.store == QuantStore.U32:
            return 32 // self.value.size_bits()
        return self.native_packing()

    def to_c(self) -> _CScheme:
        """The ``cq_scheme`` struct (cached per scheme value; treat it as read-only)."""
        return _scheme_to_c(self)

    def _build_c(self) -> _CScheme:
        c = _CScheme()
        c.value, c.param, c.store = int(self.value), int(self.param), int(self.store)
        c.level = 0 if self.level.is_tensor else 1
        c.mode = int(self.mode)
        dims = () if self.level.is_tensor else self.level.block_size.dims
        c.block_rank = len(dims)
        for i, d in enumerate(dims):
            c.block[i] = d
        c.reserved = 0
        return c

    # ---- host-side shape helpers used by callers and tests ----


    def packed_shape(self, shape: Sequence[int]) -> Tuple[int, ...]:
        """Shape of the quantized tensor in stored elements: last dim / num_quants."""
        nq = self.num_quants()
        if shape[-1] % nq:
            raise ValueError(f"last dimension {shape[-1]} is not a multiple of num_quants={nq}")
        return tuple(shape[:-1]) + (shape[-1] // nq,)

    def scales_shape(self, shape: Sequence[int]) -> Tuple[int, ...]:
        """[1] per tensor, else one scale per block (tests/suite/symmetric.rs:159)."""
        if self.level.is_tensor:
            return (1,)
        blk = self.level.block_size.to_dim_vec(len(shape))
        out = []
        for s, b in zip(shape, blk):
            if s % b:
                raise ValueError(f"dimension {s} is not a multiple of its block size {b}")
            out.append(s // b)
        return tuple(out)


@functools.lru_cache(maxsize=256)
def _scheme_to_c(scheme: QuantScheme) -> _CScheme:
    return scheme._build_c()
