"""Abs-max along an axis: the ``reduce::<R, MaxAbs>`` call of the reference's
``cubek-reduce`` crate (crates/cubek-reduce/src/lib.rs:93-131 with
src/instructions/maxabs.rs), which callers run in front of quantize to obtain
per-row / per-channel maxima.  Executed by gfx950 kernels behind the C ABI.
"""
from __future__ import annotations

from . import _ffi
from .scheme import ElemType
from .tensor import ComputeClient, TensorHandleRef


def workspace_bytes(input: TensorHandleRef, axis: int, elem: ElemType) -> int:
    return int(_ffi.lib().cq_reduce_workspace_bytes(input.as_c(), axis, int(elem)))


def max_abs(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef, axis: int,
            elem: ElemType, workspace: int = 0, workspace_size: int = 0) -> None:
    """``output`` has the input's shape with extent 1 on ``axis`` (else QuantError
    ERR_SHAPE_MISMATCH, the reference's ReduceError::MismatchShape; an axis >= rank
    gives ERR_INVALID_AXIS, its ReduceError::InvalidAxis)."""
    rc = _ffi.lib().cq_reduce_max_abs(client.stream, input.as_c(), output.as_c(), axis, int(elem),
                                      workspace, workspace_size)
    if rc:
        _ffi.check(rc)
