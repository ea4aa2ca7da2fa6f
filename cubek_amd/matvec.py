"""A consumer of the packed format: ``y = dequantize(W) @ x`` with the weights read once in their
quantized form (the matrix-vector case of the reference matmul's quantized operand,
crates/cubek-matmul/src/base.rs:309-317)."""
from __future__ import annotations

from . import _ffi
from .scheme import ElemType, QuantScheme
from .tensor import ComputeClient, TensorHandleRef


def launch_ref(client: ComputeClient, values: TensorHandleRef, params: TensorHandleRef, scheme: QuantScheme,
               x: TensorHandleRef, y: TensorHandleRef, elem: ElemType, y_elem: ElemType) -> None:
    """``values``: packed [rows, cols / num_quants]; ``params``: the scales; ``x``: [cols] of ``elem``;
    ``y``: [rows] of ``y_elem``.  Each weight enters as the value dequantize would store for ``elem``."""
    rc = _ffi.lib().cq_gemv_quantized(client.stream, values.as_c(), params.as_c(), scheme.to_c(), x.as_c(), y.as_c(),
                                      int(elem), int(y_elem))
    if rc:
        _ffi.check(rc)
