"""The shared library loads without a GPU and exports every symbol that
include/cubek_quant.h declares; host-only entry points behave (no compute calls)."""
import ctypes
import os
import re

import pytest

from cubek_amd import QuantLevel, QuantScheme, QuantStore, QuantValue, _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cubek_quant.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_ffi.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _ffi.lib()
    for sym in declared_symbols():
        assert getattr(lib, sym) is not None
    assert lib.cq_abi_version() == 1


def test_scheme_helpers_match_python_mirror():
    lib = _ffi.lib()
    for value in QuantValue:
        assert lib.cq_value_size_bits(int(value)) == value.size_bits()
        lo, hi = ctypes.c_float(), ctypes.c_float()
        assert lib.cq_value_range(int(value), ctypes.byref(lo), ctypes.byref(hi)) == 0
        assert (lo.value, hi.value) == value.range()
        for store in QuantStore:
            s = QuantScheme.default().with_value(value).with_store(store)
            c = s.to_c()
            assert lib.cq_scheme_num_quants(ctypes.byref(c)) == s.num_quants()
    assert lib.cq_value_size_bits(99) == 0
    lo, hi = ctypes.c_float(), ctypes.c_float()
    assert lib.cq_value_range(99, ctypes.byref(lo), ctypes.byref(hi)) == _ffi.ERR_INVALID_ARGUMENT


def test_workspace_and_messages():
    lib = _ffi.lib()
    per_tensor = QuantScheme.default().to_c()
    per_block = QuantScheme.default().with_level(QuantLevel.block([32])).to_c()
    assert lib.cq_workspace_bytes(ctypes.byref(per_tensor), 1 << 20) == 1024
    assert lib.cq_workspace_bytes(ctypes.byref(per_block), 1 << 20) == 0
    msgs = {lib.cq_strerror(i).decode() for i in range(11)}
    assert len(msgs) == 11 and "success" in msgs
    assert ctypes.sizeof(_ffi.CTensor) == 32 and ctypes.sizeof(type(per_tensor)) == 12


def test_argument_validation_needs_no_gpu():
    """NULL tensors and bad schemes are rejected before anything touches the device."""
    lib = _ffi.lib()
    s = QuantScheme.default().to_c()
    assert lib.cq_quantize(None, None, None, None, None, ctypes.byref(s), 0) == _ffi.ERR_INVALID_ARGUMENT
    assert lib.cq_dequantize(None, None, None, None, ctypes.byref(s), 0) == _ffi.ERR_INVALID_ARGUMENT
    assert lib.cq_quantize(None, None, None, None, None, None, 0) == _ffi.ERR_INVALID_ARGUMENT
    bad = QuantScheme.default().with_value(QuantValue.Q4S).with_store(QuantStore.Native).to_c()
    assert lib.cq_quantize(None, None, None, None, None, ctypes.byref(bad), 0) == _ffi.ERR_UNSUPPORTED_SCHEME
    with pytest.raises(_ffi.QuantError):
        _ffi.check(_ffi.ERR_SHAPE_MISMATCH)
