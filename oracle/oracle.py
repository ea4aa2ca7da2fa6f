"""ctypes front end of the CPU oracle (oracle/cq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark — never by the shipped package.

Arrays are numpy; 16-bit floats travel as ``uint16`` bit patterns together with
an ``ElemType`` tag.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Sequence

import numpy as np

from cubek_amd.scheme import ElemType, QuantParam, QuantScheme, _CScheme

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcq_oracle.so")
_lib = None


def build() -> str:
    """Compile the oracle with gcc (a few seconds)."""
    subprocess.run(["make", "-C", _HERE, "-B", "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_u64p = ctypes.POINTER(ctypes.c_uint64)
_vp = ctypes.c_void_p
_sp = ctypes.POINTER(_CScheme)


def _declare(L):
    L.cqo_bf16_to_f32.restype = ctypes.c_float
    L.cqo_bf16_to_f32.argtypes = [ctypes.c_uint16]
    L.cqo_f32_to_bf16.restype = ctypes.c_uint16
    L.cqo_f32_to_bf16.argtypes = [ctypes.c_float]
    L.cqo_f16_to_f32.restype = ctypes.c_float
    L.cqo_f16_to_f32.argtypes = [ctypes.c_uint16]
    L.cqo_f32_to_f16.restype = ctypes.c_uint16
    L.cqo_f32_to_f16.argtypes = [ctypes.c_float]
    for name in ("e4m3", "e5m2", "e2m1"):
        enc = getattr(L, f"cqo_f32_to_{name}")
        enc.restype, enc.argtypes = ctypes.c_uint8, [ctypes.c_float]
        dec = getattr(L, f"cqo_{name}_to_f32")
        dec.restype, dec.argtypes = ctypes.c_float, [ctypes.c_uint8]
    L.cqo_value_size_bits.restype = ctypes.c_uint32
    L.cqo_value_size_bits.argtypes = [ctypes.c_uint8]
    L.cqo_num_quants.restype = ctypes.c_uint32
    L.cqo_num_quants.argtypes = [_sp]
    L.cqo_value_range.restype = ctypes.c_int
    L.cqo_value_range.argtypes = [ctypes.c_uint8, ctypes.POINTER(ctypes.c_float),
                                  ctypes.POINTER(ctypes.c_float)]
    L.cqo_scale_index.restype = ctypes.c_uint64
    L.cqo_scale_index.argtypes = [_sp, ctypes.c_uint32, _u64p, _u64p, ctypes.c_uint64]
    L.cqo_is_block_start.restype = ctypes.c_int
    L.cqo_is_block_start.argtypes = [_sp, ctypes.c_uint32, _u64p, ctypes.c_uint64]
    L.cqo_pack_word.restype = ctypes.c_uint32
    L.cqo_pack_word.argtypes = [ctypes.POINTER(ctypes.c_int32), ctypes.c_uint32]
    L.cqo_unpack_word.restype = None
    L.cqo_unpack_word.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_int32)]
    q_args = [_vp, ctypes.c_int, ctypes.c_uint32, _u64p, _vp, _u64p, _vp, _u64p, _vp, _sp,
              ctypes.c_uint64, ctypes.c_uint64]
    d_args = [_vp, ctypes.c_uint32, _u64p, _vp, _u64p, _vp, ctypes.c_int, _sp,
              ctypes.c_uint64, ctypes.c_uint64]
    for n in ("cqo_quantize_packed", "cqo_quantize_native"):
        getattr(L, n).restype, getattr(L, n).argtypes = ctypes.c_int, q_args
    for n in ("cqo_dequantize_packed", "cqo_dequantize_native"):
        getattr(L, n).restype, getattr(L, n).argtypes = ctypes.c_int, d_args
    L.cqo_quantize_packed_mt.restype = ctypes.c_int
    L.cqo_quantize_packed_mt.argtypes = q_args + [ctypes.c_int]
    L.cqo_dequantize_packed_mt.restype = ctypes.c_int
    L.cqo_dequantize_packed_mt.argtypes = d_args + [ctypes.c_int]
    L.cqo_reduce_max_abs.restype = ctypes.c_int
    L.cqo_reduce_max_abs.argtypes = [_vp, ctypes.c_int, ctypes.c_uint32, _u64p, _u64p, ctypes.c_uint32, _vp, _u64p]
    L.cqo_into_contiguous_packed.restype = ctypes.c_int
    L.cqo_into_contiguous_packed.argtypes = [_vp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, _u64p, _u64p,
                                             ctypes.c_uint32, _vp]
    L.cqo_compute_scales.restype = ctypes.c_int
    L.cqo_compute_scales.argtypes = [_vp, ctypes.c_int, ctypes.c_uint32, _u64p, _vp, _sp]


# ---------------------------------------------------------------- helpers

def np_dtype(elem: ElemType):
    return np.float32 if elem == ElemType.F32 else np.uint16


def param_elem(param: QuantParam) -> ElemType:
    return {QuantParam.F32: ElemType.F32, QuantParam.F16: ElemType.F16,
            QuantParam.BF16: ElemType.BF16}[param]


def _u64(seq: Sequence[int]):
    return (ctypes.c_uint64 * len(seq))(*[int(v) for v in seq])


def contiguous_strides(shape: Sequence[int]):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_vp)


def to_bits(a: np.ndarray, elem: ElemType) -> np.ndarray:
    """f32 array -> storage array of ``elem`` (uint16 bit patterns for 16-bit types)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if elem == ElemType.F32:
        return a
    if elem == ElemType.F16:
        return a.astype(np.float16).view(np.uint16)
    u = a.view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def from_bits(a: np.ndarray, elem: ElemType) -> np.ndarray:
    """storage array -> f32 values."""
    if elem == ElemType.F32:
        return np.asarray(a, dtype=np.float32)
    if elem == ElemType.F16:
        return a.view(np.float16).astype(np.float32)
    return (a.astype(np.uint32) << 16).view(np.float32)


def _check_footprint(scheme: QuantScheme, shape, strides, available: int) -> None:
    """The C side trusts its pointers: refuse scale buffers smaller than the layout reaches."""
    if scheme.level.is_tensor:
        assert available >= 1
        return
    reach = 1 + sum((n - 1) * st for n, st in zip(scheme.scales_shape(shape), strides))
    assert reach <= available, f"scale buffer of {available} entries, layout reaches {reach}"


# ---------------------------------------------------------------- entry points

def scale_index(scheme: QuantScheme, shape, scale_strides, elem: int) -> int:
    c = scheme.to_c()
    return int(lib().cqo_scale_index(ctypes.byref(c), len(shape), _u64(shape),
                                     _u64(scale_strides), elem))


def is_block_start(scheme: QuantScheme, shape, elem: int) -> bool:
    c = scheme.to_c()
    return bool(lib().cqo_is_block_start(ctypes.byref(c), len(shape), _u64(shape), elem))


def compute_scales(x: np.ndarray, elem: ElemType, shape, scheme: QuantScheme) -> np.ndarray:
    """Scales typed like the input (``elem``), contiguous, one per block or [1]."""
    c = scheme.to_c()
    sshape = scheme.scales_shape(shape)
    out = np.zeros(sshape, dtype=np_dtype(elem))
    x = np.ascontiguousarray(x)
    rc = lib().cqo_compute_scales(_ptr(x), int(elem), len(shape), _u64(shape), _ptr(out),
                                  ctypes.byref(c))
    if rc:
        raise RuntimeError(f"cqo_compute_scales failed: {rc}")
    return out


def quantize(x: np.ndarray, elem: ElemType, shape, scale: np.ndarray, scheme: QuantScheme,
             scale_strides=None, threads: int = 0, out_scale_strides=None):
    """Returns (stored values, out_scale).  ``scale`` is typed ``elem``; out_scale
    is typed scheme.param, as large as ``scale``, addressed with
    ``out_scale_strides`` (default: the strides of ``scale``)."""
    from cubek_amd.scheme import QuantStore

    c = scheme.to_c()
    x = np.ascontiguousarray(x)
    n = int(np.prod(shape))
    if scale_strides is None:
        scale_strides = (1,) if scheme.level.is_tensor else contiguous_strides(scheme.scales_shape(shape))
    if scheme.level.is_tensor:
        scale_strides = (0,) * len(shape)
    if out_scale_strides is None or scheme.level.is_tensor:
        out_scale_strides = scale_strides
    _check_footprint(scheme, shape, scale_strides, scale.size)
    _check_footprint(scheme, shape, out_scale_strides, scale.size)
    assert x.size == n and x.dtype == np_dtype(elem), "input array does not match shape/dtype"
    out_scale = np.zeros(scale.size, dtype=np_dtype(param_elem(scheme.param)))
    nq = scheme.num_quants()
    if scheme.store == QuantStore.U32:
        out = np.zeros(n // nq, dtype=np.uint32)
        if threads > 0:
            rc = lib().cqo_quantize_packed_mt(_ptr(x), int(elem), len(shape), _u64(shape),
                                              _ptr(scale), _u64(scale_strides), _ptr(out_scale),
                                              _u64(out_scale_strides), _ptr(out), ctypes.byref(c),
                                              0, n // nq, threads)
        else:
            rc = lib().cqo_quantize_packed(_ptr(x), int(elem), len(shape), _u64(shape),
                                           _ptr(scale), _u64(scale_strides), _ptr(out_scale),
                                           _u64(out_scale_strides), _ptr(out), ctypes.byref(c),
                                           0, n // nq)
        out = out.reshape(scheme.packed_shape(shape))
    else:
        out = np.zeros(n // nq, dtype=np.uint8)
        rc = lib().cqo_quantize_native(_ptr(x), int(elem), len(shape), _u64(shape), _ptr(scale),
                                       _u64(scale_strides), _ptr(out_scale),
                                       _u64(out_scale_strides), _ptr(out), ctypes.byref(c), 0, n)
        out = out.reshape(scheme.packed_shape(shape))
    if rc:
        raise RuntimeError(f"oracle quantize failed: {rc}")
    return out, out_scale.reshape(scale.shape)


def dequantize(values: np.ndarray, shape, params: np.ndarray, elem: ElemType,
               scheme: QuantScheme, scale_strides=None, threads: int = 0) -> np.ndarray:
    """``shape`` is the unpacked shape; returns storage array of ``elem``."""
    from cubek_amd.scheme import QuantStore

    c = scheme.to_c()
    values = np.ascontiguousarray(values)
    n = int(np.prod(shape))
    if scale_strides is None:
        scale_strides = (1,) if scheme.level.is_tensor else contiguous_strides(scheme.scales_shape(shape))
    if scheme.level.is_tensor:
        scale_strides = (0,) * len(shape)
    _check_footprint(scheme, shape, scale_strides, params.size)
    out = np.zeros(n, dtype=np_dtype(elem))
    nq = scheme.num_quants()
    assert values.size == n // nq, "stored array does not match shape"
    if scheme.store == QuantStore.U32:
        args = (_ptr(values), len(shape), _u64(shape), _ptr(params), _u64(scale_strides),
                _ptr(out), int(elem), ctypes.byref(c), 0, n // nq)
        rc = (lib().cqo_dequantize_packed_mt(*args, threads) if threads > 0
              else lib().cqo_dequantize_packed(*args))
    else:
        rc = lib().cqo_dequantize_native(_ptr(values), len(shape), _u64(shape), _ptr(params),
                                         _u64(scale_strides), _ptr(out), int(elem),
                                         ctypes.byref(c), 0, n)
    if rc:
        raise RuntimeError(f"oracle dequantize failed: {rc}")
    return out.reshape(shape)


def reduce_max_abs(x: np.ndarray, elem: ElemType, shape, axis: int, in_strides=None) -> np.ndarray:
    """max |x| along ``axis`` (kept with extent 1); ``x`` is the raw buffer when strides are given."""
    x = np.ascontiguousarray(x)
    if in_strides is None:
        in_strides = contiguous_strides(shape)
    out_shape = tuple(1 if d == axis else s for d, s in enumerate(shape))
    out = np.zeros(out_shape, dtype=np_dtype(elem))
    rc = lib().cqo_reduce_max_abs(_ptr(x), int(elem), len(shape), _u64(shape), _u64(in_strides), axis,
                                  _ptr(out), _u64(contiguous_strides(out_shape)))
    if rc:
        raise RuntimeError(f"cqo_reduce_max_abs failed: {rc}")
    return out


def into_contiguous_packed(buf: np.ndarray, packing: int, shape, in_strides, packed_dim: int) -> np.ndarray:
    """Strided stored tensor (``buf`` uint32 or uint8, ``packing`` values per element along
    ``packed_dim``) -> contiguous tensor packed along the last dimension of the logical ``shape``."""
    buf = np.ascontiguousarray(buf)
    assert buf.dtype in (np.uint32, np.uint8)
    in_shape = tuple(s // packing if d == packed_dim else s for d, s in enumerate(shape))
    assert 1 + sum((n - 1) * st for n, st in zip(in_shape, in_strides)) <= buf.size
    out_shape = tuple(shape[:-1]) + (shape[-1] // packing,)
    out = np.zeros(out_shape, dtype=buf.dtype)
    rc = lib().cqo_into_contiguous_packed(_ptr(buf), buf.itemsize, packing, len(shape), _u64(shape),
                                          _u64(in_strides), packed_dim, _ptr(out))
    if rc:
        raise RuntimeError(f"cqo_into_contiguous_packed failed: {rc}")
    return out
