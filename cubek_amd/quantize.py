"""``cubek_quant::quantize`` for MI355X: same entry point, same argument
meaning as crates/cubek-quant/src/quantize.rs:174-182, executed by hand-written
gfx950 kernels behind the C ABI.  Conditions on which the reference panics
raise :class:`cubek_amd.QuantError` with the matching status code.
"""
from __future__ import annotations

from . import _ffi
from .scheme import ElemType, QuantScheme
from .tensor import ComputeClient, TensorHandleRef


def launch_ref(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
               scale: TensorHandleRef, out_scale: TensorHandleRef, scheme: QuantScheme,
               input_elem: ElemType) -> None:
    """Quantize ``input`` with the given ``scale`` tensor (typed like the input)
    into ``output`` and copy the scales, cast to ``scheme.param``, into ``out_scale``."""
    rc = _ffi.lib().cq_quantize(client.stream, input.as_c(), output.as_c(), scale.as_c(), out_scale.as_c(),
                                scheme.to_c(), int(input_elem))
    if rc:
        _ffi.check(rc)


def workspace_bytes(scheme: QuantScheme, num_elements: int) -> int:
    return int(_ffi.lib().cq_workspace_bytes(scheme.to_c(), num_elements))


def compute_scales(client: ComputeClient, input: TensorHandleRef, scales: TensorHandleRef,
                   scheme: QuantScheme, input_elem: ElemType, workspace: int = 0,
                   workspace_bytes: int = 0) -> None:
    """scale = 2*absmax/(q_max-q_min) per block or tensor, typed like the input
    (the rule of crates/cubek-quant/tests/suite/symmetric.rs:35-38,156-179)."""
    rc = _ffi.lib().cq_compute_scales(client.stream, input.as_c(), scales.as_c(), scheme.to_c(),
                                      int(input_elem), workspace, workspace_bytes)
    if rc:
        _ffi.check(rc)


def launch_dynamic(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
                   out_scale: TensorHandleRef, scheme: QuantScheme, input_elem: ElemType,
                   workspace: int = 0, workspace_bytes: int = 0) -> None:
    """Fused abs-max + scale + quantize; same results as compute_scales + launch_ref."""
    rc = _ffi.lib().cq_quantize_dynamic(client.stream, input.as_c(), output.as_c(), out_scale.as_c(),
                                        scheme.to_c(), int(input_elem), workspace, workspace_bytes)
    if rc:
        _ffi.check(rc)


def launch_dynamic_static(client: ComputeClient, input: TensorHandleRef, output: TensorHandleRef,
                          out_scale: TensorHandleRef, scheme: QuantScheme, input_elem: ElemType) -> None:
    """launch_dynamic for callers that cannot allocate a workspace: the scratch memory is an array
    inside the library (one per GPU, shared by all calls on that GPU)."""
    rc = _ffi.lib().cq_quantize_dynamic_static(client.stream, input.as_c(), output.as_c(), out_scale.as_c(),
                                               scheme.to_c(), int(input_elem))
    if rc:
        _ffi.check(rc)
