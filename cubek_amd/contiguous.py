"""Re-packing of strided quantized tensors: ``into_contiguous_packed`` of cubecl-std as
cubek-matmul calls it on quantized operands (crates/cubek-matmul/src/base.rs:505-529).
Executed by gfx950 kernels behind the C ABI; the caller provides the output.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

from . import _ffi
from .tensor import ComputeClient, TensorHandleRef


def into_contiguous_packed_ref(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
                               shape: Sequence[int], packing: int) -> None:
    """``shape`` is the logical (unpacked) shape; ``input`` holds ``packing`` values per
    stored element along its rightmost stride-1 dimension, ``output`` is contiguous with
    the last dimension of ``shape`` divided by ``packing``."""
    c_shape = (ctypes.c_uint64 * len(shape))(*shape)
    rc = _ffi.lib().cq_into_contiguous_packed(client.stream, input.as_c(), output.as_c(), c_shape, len(shape),
                                              packing)
    if rc:
        _ffi.check(rc)
