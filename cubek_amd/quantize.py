"""``cubek_quant::quantize`` for MI355X: same entry point, same argument
meaning as crates/cubek-quant/src/quantize.rs:174-182, executed by hand-written
gfx950 kernels behind the C ABI.  Conditions on which the reference panics
raise :class:`cubek_amd.QuantError` with the matching status code.
"""
from __future__ import annotations

import ctypes

from . import _ffi
from .scheme import ElemType, QuantScheme
from .tensor import ComputeClient, TensorHandleRef


def _ct(t: TensorHandleRef):
    return _ffi.make_tensor(t.handle, t.shape, t.strides, t.elem_size)


def launch_ref(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
               scale: TensorHandleRef, out_scale: TensorHandleRef, scheme: QuantScheme,
               input_elem: ElemType) -> None:
    """Quantize ``input`` with the given ``scale`` tensor (typed like the input)
    into ``output`` and copy the scales, cast to ``scheme.param``, into ``out_scale``."""
    L = _ffi.lib()
    cin, k1 = _ct(input)
    cout, k2 = _ct(output)
    csc, k3 = _ct(scale)
    cos, k4 = _ct(out_scale)
    cs = scheme.to_c()
    _ffi.check(L.cq_quantize(ctypes.c_void_p(client.stream), ctypes.byref(cin), ctypes.byref(cout),
                             ctypes.byref(csc), ctypes.byref(cos), ctypes.byref(cs), int(input_elem)))


def workspace_bytes(scheme: QuantScheme, num_elements: int) -> int:
    cs = scheme.to_c()
    return int(_ffi.lib().cq_workspace_bytes(ctypes.byref(cs), num_elements))


def compute_scales(client: ComputeClient, input: TensorHandleRef, scales: TensorHandleRef,
                   scheme: QuantScheme, input_elem: ElemType, workspace: int = 0,
                   workspace_bytes: int = 0) -> None:
    """scale = 2*absmax/(q_max-q_min) per block or tensor, typed like the input
    (the rule of crates/cubek-quant/tests/suite/symmetric.rs:35-38,156-179)."""
    L = _ffi.lib()
    cin, k1 = _ct(input)
    csc, k2 = _ct(scales)
    cs = scheme.to_c()
    _ffi.check(L.cq_compute_scales(ctypes.c_void_p(client.stream), ctypes.byref(cin), ctypes.byref(csc),
                                   ctypes.byref(cs), int(input_elem), ctypes.c_void_p(workspace),
                                   workspace_bytes))


def launch_dynamic(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
                   out_scale: TensorHandleRef, scheme: QuantScheme, input_elem: ElemType,
                   workspace: int = 0, workspace_bytes: int = 0) -> None:
    """Fused abs-max + scale + quantize; same results as compute_scales + launch_ref."""
    L = _ffi.lib()
    cin, k1 = _ct(input)
    cout, k2 = _ct(output)
    cos, k3 = _ct(out_scale)
    cs = scheme.to_c()
    _ffi.check(L.cq_quantize_dynamic(ctypes.c_void_p(client.stream), ctypes.byref(cin), ctypes.byref(cout),
                                     ctypes.byref(cos), ctypes.byref(cs), int(input_elem),
                                     ctypes.c_void_p(workspace), workspace_bytes))
