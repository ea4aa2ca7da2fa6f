"""ctypes front end of tests/cpp/libcq_device_header_test.so: consumer kernels built on
include/cubek_quant_device.hpp alone (built by cubek_amd/csrc/Makefile)."""
from __future__ import annotations

import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "libcq_device_header_test.so")
_lib = None
_u64p = ctypes.POINTER(ctypes.c_uint64)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_vp = ctypes.c_void_p


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        assert os.path.exists(LIB_PATH), "tests/cpp/libcq_device_header_test.so is not built (make -C cubek_amd/csrc)"
        L = ctypes.CDLL(LIB_PATH)
        layout = [_u64p, ctypes.c_uint32, _u64p, _u8p, ctypes.c_uint32]
        L.dh_dequantize_packed.restype = ctypes.c_int
        L.dh_dequantize_packed.argtypes = [ctypes.c_int] * 4 + [_vp, _vp] + layout + [ctypes.c_uint64, _vp]
        L.dh_dequantize_native.restype = ctypes.c_int
        L.dh_dequantize_native.argtypes = [ctypes.c_int] * 3 + [_vp, _vp] + layout + [ctypes.c_uint64, _vp]
        L.dh_dequantize_native_pairs.restype = ctypes.c_int
        L.dh_dequantize_native_pairs.argtypes = [ctypes.c_int] * 3 + [_vp, _vp] + layout + [ctypes.c_uint64, _vp]
        L.dh_global_scale_pos.restype = ctypes.c_int
        L.dh_global_scale_pos.argtypes = [ctypes.c_uint32] * 8 + [_vp]
        with_nq = [_u64p, ctypes.c_uint32, ctypes.c_uint32, _u64p, _u8p, ctypes.c_uint32]
        L.dh_scales_layout.restype = ctypes.c_int
        L.dh_scales_layout.argtypes = with_nq + [ctypes.c_uint64, _vp, _vp]
        L.dh_host_scale_pos.restype = ctypes.c_uint64
        L.dh_host_scale_pos.argtypes = with_nq + [ctypes.c_uint64]
        L.dh_host_is_block_start.restype = ctypes.c_int
        L.dh_host_is_block_start.argtypes = with_nq + [ctypes.c_uint64]
        L.dh_host_fast_div.restype = ctypes.c_uint32
        L.dh_host_fast_div.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        _lib = L
    return _lib


def u64(seq):
    return (ctypes.c_uint64 * len(seq))(*[int(v) for v in seq])


def u8(seq):
    return (ctypes.c_uint8 * max(len(seq), 1))(*[int(v) for v in seq])
