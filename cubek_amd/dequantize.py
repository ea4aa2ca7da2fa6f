"""``cubek_quant::dequantize`` for MI355X (crates/cubek-quant/src/dequantize.rs:171-178)."""
from __future__ import annotations

import ctypes

from . import _ffi
from .scheme import ElemType, QuantScheme
from .tensor import ComputeClient, TensorHandleRef


def launch_ref(client: ComputeClient, values: TensorHandleRef, output: TensorHandleRef,
               params: TensorHandleRef, scheme: QuantScheme, input_dtype: ElemType) -> None:
    """Convert the quantized ``values`` back to floats of type ``input_dtype``
    (the reference names the output float type ``input_dtype``)."""
    L = _ffi.lib()
    cv, k1 = _ffi.make_tensor(values.handle, values.shape, values.strides, values.elem_size)
    co, k2 = _ffi.make_tensor(output.handle, output.shape, output.strides, output.elem_size)
    cp, k3 = _ffi.make_tensor(params.handle, params.shape, params.strides, params.elem_size)
    cs = scheme.to_c()
    _ffi.check(L.cq_dequantize(ctypes.c_void_p(client.stream), ctypes.byref(cv), ctypes.byref(co),
                               ctypes.byref(cp), ctypes.byref(cs), int(input_dtype)))
