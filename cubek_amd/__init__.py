"""cubek_amd — the quantize/dequantize path of tracel-ai/cubek's ``cubek-quant``
crate, rebuilt for MI355X (gfx950): hand-written HIP kernels behind a C ABI
(include/cubek_quant.h) and a host layer that keeps the crate's API surface.

    cubek_amd.scheme      QuantScheme / QuantValue / QuantStore / QuantLevel / QuantParam
    cubek_amd.quantize    launch_ref, compute_scales, launch_dynamic
    cubek_amd.dequantize  launch_ref
    cubek_amd.reduce      max_abs (abs-max along an axis, the step in front of quantize)
    cubek_amd.contiguous  into_contiguous_packed_ref (strided quantized tensor -> contiguous)
    cubek_amd.matvec      launch_ref (y = dequantize(W) @ x straight from the packed weights)

Importing the package does not load the native library; the first call does and
raises if it has not been built.
"""
from . import contiguous, dequantize, matvec, quantize, reduce, scheme  # noqa: F401
from ._ffi import QuantError  # noqa: F401
from .scheme import (BlockSize, ElemType, QuantLevel, QuantMode, QuantParam, QuantScheme,  # noqa: F401
                     QuantStore, QuantValue)
from .tensor import ComputeClient, TensorHandleRef  # noqa: F401

__all__ = ["quantize", "dequantize", "reduce", "contiguous", "matvec", "scheme", "QuantError", "BlockSize", "ElemType", "QuantLevel",
           "QuantMode", "QuantParam", "QuantScheme", "QuantStore", "QuantValue", "ComputeClient",
           "TensorHandleRef"]
