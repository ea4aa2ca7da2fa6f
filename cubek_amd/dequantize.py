"""``cubek_quant::dequantize`` for MI355X (crates/cubek-quant/src/dequantize.rs:171-178)."""
from __future__ import annotations

from . import _ffi
from .scheme import ElemType, QuantScheme
from .tensor import ComputeClient, TensorHandleRef


def launch_ref(client: ComputeClient, values: TensorHandleRef, output: TensorHandleRef,
               params: TensorHandleRef, scheme: QuantScheme, input_dtype: ElemType) -> None:
    """Convert the quantized ``values`` back to floats of type ``input_dtype``
    (the reference names the output float type ``input_dtype``)."""
    rc = _ffi.lib().cq_dequantize(client.stream, values.as_c(), output.as_c(), params.as_c(),
                                  scheme.to_c(), int(input_dtype))
    if rc:
        _ffi.check(rc)
