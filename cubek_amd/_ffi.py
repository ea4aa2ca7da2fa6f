"""ctypes binding of the C ABI declared in include/cubek_quant.h.

The native library is mandatory: there is no Python or CPU fallback.  If
``libcubek_quant_hip.so`` is missing, every entry point raises ``RuntimeError``
telling the user to build it (``python -c 'import __graft_entry__ as g; g.build()'``
or ``make -C cubek_amd/csrc``).
"""
from __future__ import annotations

import ctypes
import os
from typing import Sequence

from .scheme import _CScheme

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libcubek_quant_hip.so")

#: every symbol include/cubek_quant.h declares
EXPORTED_SYMBOLS = (
    "cq_value_size_bits", "cq_scheme_num_quants", "cq_value_range", "cq_quantize", "cq_dequantize",
    "cq_compute_scales", "cq_quantize_dynamic", "cq_workspace_bytes", "cq_strerror",
    "cq_last_hip_error", "cq_abi_version", "cq_reduce_max_abs", "cq_reduce_workspace_bytes",
    "cq_into_contiguous_packed", "cq_quantize_dynamic_static",
    "cq_gemv_quantized", "cq_plan_kind",
)


class CTensor(ctypes.Structure):
    """Binary layout of ``cq_tensor``."""

    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("shape", ctypes.POINTER(ctypes.c_uint64)),
        ("strides", ctypes.POINTER(ctypes.c_uint64)),
        ("rank", ctypes.c_uint32),
        ("elem_size", ctypes.c_uint32),
    ]


class QuantError(RuntimeError):
    """A non-zero cq_status.  ``status`` holds the code (include/cubek_quant.h)."""

    def __init__(self, status: int, message: str):
        super().__init__(f"cq_status {status}: {message}")
        self.status = status


# status codes (mirrors enum cq_status)
OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED_SCHEME, ERR_BLOCK_NOT_DIVISIBLE, ERR_SHAPE_MISMATCH, \
    ERR_NON_CONTIGUOUS, ERR_WORKSPACE_TOO_SMALL, ERR_HIP, ERR_TOO_LARGE, ERR_INVALID_AXIS, \
    ERR_SCRATCH_TOO_SMALL = range(11)

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"native library not built: {LIB_PATH} is missing; there is no fallback path. "
            "Build it with `make -C cubek_amd/csrc` (needs hipcc).")
    L = ctypes.CDLL(LIB_PATH)
    tp = ctypes.POINTER(CTensor)
    sp = ctypes.POINTER(_CScheme)
    L.cq_abi_version.restype = ctypes.c_uint32
    L.cq_abi_version.argtypes = []
    L.cq_last_hip_error.restype = ctypes.c_int
    L.cq_last_hip_error.argtypes = []
    L.cq_strerror.restype = ctypes.c_char_p
    L.cq_strerror.argtypes = [ctypes.c_int]
    L.cq_value_size_bits.restype = ctypes.c_uint32
    L.cq_value_size_bits.argtypes = [ctypes.c_uint8]
    L.cq_scheme_num_quants.restype = ctypes.c_uint32
    L.cq_scheme_num_quants.argtypes = [sp]
    L.cq_value_range.restype = ctypes.c_int
    L.cq_value_range.argtypes = [ctypes.c_uint8, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
    L.cq_workspace_bytes.restype = ctypes.c_size_t
    L.cq_workspace_bytes.argtypes = [sp, ctypes.c_uint64]
    L.cq_quantize.restype = ctypes.c_int
    L.cq_quantize.argtypes = [ctypes.c_void_p, tp, tp, tp, tp, sp, ctypes.c_int]
    L.cq_dequantize.restype = ctypes.c_int
    L.cq_dequantize.argtypes = [ctypes.c_void_p, tp, tp, tp, sp, ctypes.c_int]
    L.cq_compute_scales.restype = ctypes.c_int
    L.cq_compute_scales.argtypes = [ctypes.c_void_p, tp, tp, sp, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]
    L.cq_quantize_dynamic.restype = ctypes.c_int
    L.cq_quantize_dynamic.argtypes = [ctypes.c_void_p, tp, tp, tp, sp, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]
    L.cq_quantize_dynamic_static.restype = ctypes.c_int
    L.cq_quantize_dynamic_static.argtypes = [ctypes.c_void_p, tp, tp, tp, sp, ctypes.c_int]
    L.cq_plan_kind.restype = ctypes.c_int
    L.cq_plan_kind.argtypes = [ctypes.c_int, tp, tp, tp, tp, sp, ctypes.c_int, ctypes.POINTER(ctypes.c_uint32)]
    L.cq_gemv_quantized.restype = ctypes.c_int
    L.cq_gemv_quantized.argtypes = [ctypes.c_void_p, tp, tp, sp, tp, tp, ctypes.c_int, ctypes.c_int]
    L.cq_reduce_max_abs.restype = ctypes.c_int
    L.cq_reduce_max_abs.argtypes = [ctypes.c_void_p, tp, tp, ctypes.c_uint32, ctypes.c_int, ctypes.c_void_p,
                                    ctypes.c_size_t]
    L.cq_reduce_workspace_bytes.restype = ctypes.c_size_t
    L.cq_reduce_workspace_bytes.argtypes = [tp, ctypes.c_uint32, ctypes.c_int]
    L.cq_into_contiguous_packed.restype = ctypes.c_int
    L.cq_into_contiguous_packed.argtypes = [ctypes.c_void_p, tp, tp, ctypes.POINTER(ctypes.c_uint64), ctypes.c_uint32,
                                            ctypes.c_uint32]
    _lib = L
    return L


def check(status: int) -> None:
    if status != OK:
        msg = lib().cq_strerror(status).decode()
        if status == ERR_HIP:
            msg += f" (hipError_t {lib().cq_last_hip_error()})"
        raise QuantError(status, msg)


def make_tensor(ptr: int, shape: Sequence[int], strides: Sequence[int], elem_size: int):
    """Returns (CTensor, keepalive) — keep the second value alive during the call."""
    rank = len(shape)
    shp = (ctypes.c_uint64 * rank)(*[int(s) for s in shape])
    strd = (ctypes.c_uint64 * rank)(*[int(s) for s in strides])
    t = CTensor(ctypes.c_void_p(ptr), shp, strd, rank, elem_size)
    return t, (shp, strd)


#: enum cq_kernel_family
FAMILY_NONE, FAMILY_FLAT, FAMILY_FLAT_ROWS, FAMILY_FLAT_LANES, FAMILY_ROWS, FAMILY_BLOCKS, FAMILY_TRANSPOSED, \
    FAMILY_PER_ELEMENT, FAMILY_STAGED = range(9)
FAMILY_NAMES = ("none", "flat", "flat_rows", "flat_lanes", "rows", "blocks", "transposed", "per_element", "staged")
#: enum cq_op
OP_QUANTIZE, OP_QUANTIZE_DYNAMIC, OP_DEQUANTIZE, OP_COMPUTE_SCALES, OP_GEMV = range(5)


def plan_kind(op: int, floats, values, scale, out_scale, scheme, elem) -> str:
    """Name of the kernel family a call would run on (``cq_plan_kind``); tensors are ``TensorHandleRef`` or None."""
    fam = ctypes.c_uint32(0)
    c = lambda t: t.as_c() if t is not None else None
    rc = lib().cq_plan_kind(op, c(floats), c(values), c(scale), c(out_scale), scheme.to_c(), int(elem), ctypes.byref(fam))
    if rc:
        check(rc)
    return FAMILY_NAMES[fam.value]
