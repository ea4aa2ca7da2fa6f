"""Host-side validation of the C ABI: every refusal below is decided before a kernel
is launched, so these run without a GPU (the pointers are never dereferenced)."""
import ctypes

import pytest

from cubek_amd import ElemType, QuantLevel, QuantScheme, QuantStore, QuantValue, TensorHandleRef, _ffi
from cubek_amd import contiguous as cq_contiguous
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz
from cubek_amd import reduce as cq_reduce
from cubek_amd.tensor import ComputeClient

FAKE = 0x7F0000001000  # a non-NULL "device pointer"; validation must fail before it is used
CLIENT = ComputeClient(0)


def t(shape, elem_size, strides=None, ptr=FAKE):
    if strides is None:
        strides, acc = [], 1
        for n in reversed(shape):
            strides.append(acc)
            acc *= n
        strides = tuple(reversed(strides))
    return TensorHandleRef(ptr, tuple(shape), tuple(strides), elem_size)


def status(fn):
    with pytest.raises(_ffi.QuantError) as e:
        fn()
    return e.value.status


Q8_B32 = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([32]))


def test_quantize_shape_and_size_checks():
    x, out, sc = t((8, 64), 4), t((8, 16), 4), t((8, 2), 4)
    run = lambda **k: qz.launch_ref(CLIENT, k.get("x", x), k.get("out", out), k.get("sc", sc), k.get("os", sc),
                                    k.get("scheme", Q8_B32), k.get("elem", ElemType.F32))
    assert status(lambda: run(out=t((8, 15), 4))) == _ffi.ERR_SHAPE_MISMATCH       # packed shape
    assert status(lambda: run(out=t((8, 16), 1))) == _ffi.ERR_SHAPE_MISMATCH       # u32 store needs 4-byte elements
    assert status(lambda: run(sc=t((8, 3), 4))) == _ffi.ERR_SHAPE_MISMATCH         # one scale per block
    assert status(lambda: run(sc=t((16,), 4))) == _ffi.ERR_SHAPE_MISMATCH          # scales keep the tensor's rank
    assert status(lambda: run(elem=ElemType.BF16)) == _ffi.ERR_SHAPE_MISMATCH      # element size vs dtype
    assert status(lambda: run(out=t((4, 2, 16), 4))) == _ffi.ERR_SHAPE_MISMATCH    # rank
    # block size not a multiple of the values per word: the reference asserts (src/lib.rs:28-31)
    bad = Q8_B32.with_level(QuantLevel.block([2]))
    assert status(lambda: run(scheme=bad, sc=t((8, 32), 4))) == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    # shape not a multiple of the block
    b48 = Q8_B32.with_level(QuantLevel.block([48]))
    assert status(lambda: run(scheme=b48, sc=t((8, 1), 4))) == _ffi.ERR_SHAPE_MISMATCH
    # more block dimensions than tensor dimensions
    b3 = Q8_B32.with_level(QuantLevel.block([1, 2, 32]))
    assert status(lambda: run(scheme=b3)) == _ffi.ERR_SHAPE_MISMATCH
    # NULL data pointer, rank 0
    assert status(lambda: run(x=t((8, 64), 4, ptr=0))) == _ffi.ERR_INVALID_ARGUMENT
    assert status(lambda: run(x=t((), 4))) == _ffi.ERR_INVALID_ARGUMENT


def test_native_store_and_scheme_checks():
    x, sc = t((8, 64), 4), t((1,), 4)
    native_q4 = QuantScheme.default().with_value(QuantValue.Q4S).with_store(QuantStore.Native)
    assert status(lambda: qz.launch_ref(CLIENT, x, t((8, 64), 1), sc, sc, native_q4, ElemType.F32)) \
        == _ffi.ERR_UNSUPPORTED_SCHEME                                             # src/quantize.rs:213-219
    assert status(lambda: dq.launch_ref(CLIENT, t((8, 64), 1), x, sc, native_q4, ElemType.F32)) \
        == _ffi.ERR_UNSUPPORTED_SCHEME
    e2m1 = QuantScheme.default().with_value(QuantValue.E2M1).with_store(QuantStore.Native)
    assert status(lambda: qz.launch_ref(CLIENT, x, t((8, 64), 1), sc, sc, e2m1, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH                                                 # two nibbles per byte: [8, 32]
    e4m3 = QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)
    assert status(lambda: qz.launch_ref(CLIENT, x, t((8, 64), 4), sc, sc, e4m3, ElemType.F32)) \
        == _ffi.ERR_SHAPE_MISMATCH                                                 # native store is bytes
    raw = type(QuantScheme.default().to_c()).from_buffer_copy(QuantScheme.default().to_c())  # to_c() is cached
    raw.reserved = 1
    assert _ffi.lib().cq_quantize(None, x.as_c(), x.as_c(), sc.as_c(), sc.as_c(), ctypes.byref(raw), 0) \
        == _ffi.ERR_INVALID_ARGUMENT
    raw = type(raw).from_buffer_copy(QuantScheme.default().to_c())
    raw.value = 42
    assert _ffi.lib().cq_dequantize(None, x.as_c(), x.as_c(), sc.as_c(), ctypes.byref(raw), 0) \
        == _ffi.ERR_INVALID_ARGUMENT


def test_block_divisibility_is_asserted_where_the_reference_asserts_it():
    """check_block_size_compat (src/lib.rs:20-33) guards the reference's quantize launchers only
    (src/quantize.rs:260,305); its dequantize launchers take any block size.  Without a GPU an accepted
    call goes on to its launch and fails there, with a HIP error."""
    x, out = t((8, 64), 4), t((8, 16), 4)
    b2 = Q8_B32.with_level(QuantLevel.block([2]))
    sc = t((8, 32), 4)
    assert status(lambda: qz.launch_ref(CLIENT, x, out, sc, sc, b2, ElemType.F32)) == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    assert status(lambda: qz.launch_dynamic(CLIENT, x, out, sc, b2, ElemType.F32)) == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    passed_validation = (_ffi.OK, _ffi.ERR_HIP)

    def outcome(fn):
        try:
            fn()
            return _ffi.OK
        except _ffi.QuantError as e:
            return e.status

    assert outcome(lambda: dq.launch_ref(CLIENT, out, x, sc, b2, ElemType.F32)) in passed_validation
    assert outcome(lambda: qz.compute_scales(CLIENT, x, sc, b2, ElemType.F32)) in passed_validation
    # native store: the divisor is the line size the reference picks for the input tensor: at most 16 bytes,
    # dividing the last dimension and the smallest stride above 1; 1 when the last dimension is strided
    i8 = QuantScheme.default().with_value(QuantValue.Q8S).with_store(QuantStore.Native)
    n2 = i8.with_level(QuantLevel.block([2]))
    bytes_out = t((8, 64), 1)
    assert status(lambda: qz.launch_ref(CLIENT, x, bytes_out, sc, sc, n2, ElemType.F32)) == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    x_odd_pitch = t((8, 64), 4, (66, 1))   # rows 66 elements apart: line size 2
    assert outcome(lambda: qz.launch_ref(CLIENT, x_odd_pitch, bytes_out, sc, sc, n2, ElemType.F32)) in passed_validation
    x_transposed = t((8, 64), 4, (1, 8))   # last dimension strided: line size 1
    n1 = i8.with_level(QuantLevel.block([1]))
    assert outcome(lambda: qz.launch_ref(CLIENT, x_transposed, bytes_out, t((8, 64), 4), t((8, 64), 4), n1,
                                         ElemType.F32)) in passed_validation
    assert status(lambda: qz.launch_ref(CLIENT, x, bytes_out, t((8, 64), 4), t((8, 64), 4), n1, ElemType.F32)) \
        == _ffi.ERR_BLOCK_NOT_DIVISIBLE                                            # contiguous: line size 4
    assert outcome(lambda: dq.launch_ref(CLIENT, bytes_out, x, sc, n2, ElemType.F32)) in passed_validation


def test_per_tensor_dynamic_needs_its_workspace():
    scheme = QuantScheme.default().with_value(QuantValue.Q8S)
    x, out, one = t((8, 64), 4), t((8, 16), 4), t((1,), 4)
    assert qz.workspace_bytes(scheme, 512) == 1024 and qz.workspace_bytes(Q8_B32, 512) == 0
    assert status(lambda: qz.launch_dynamic(CLIENT, x, out, one, scheme, ElemType.F32)) == _ffi.ERR_WORKSPACE_TOO_SMALL
    assert status(lambda: qz.launch_dynamic(CLIENT, x, out, one, scheme, ElemType.F32, FAKE, 512)) \
        == _ffi.ERR_WORKSPACE_TOO_SMALL
    assert status(lambda: qz.compute_scales(CLIENT, x, one, scheme, ElemType.F32)) == _ffi.ERR_WORKSPACE_TOO_SMALL
    assert status(lambda: qz.compute_scales(CLIENT, t((8, 62), 4), one, scheme, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH


def test_reduce_checks():
    x = t((4, 8), 4)
    assert status(lambda: cq_reduce.max_abs(CLIENT, x, t((4, 1), 4), 2, ElemType.F32)) == _ffi.ERR_INVALID_AXIS
    assert status(lambda: cq_reduce.max_abs(CLIENT, x, t((4, 2), 4), 1, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: cq_reduce.max_abs(CLIENT, x, t((4,), 4), 1, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: cq_reduce.max_abs(CLIENT, x, t((4, 1), 2), 1, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH
    # enough rows already: only the room for a contiguous result, should the output tensor be strided
    assert cq_reduce.workspace_bytes(t((8192, 8192), 2), 1, ElemType.BF16) == 8192 * 2
    assert cq_reduce.workspace_bytes(t((64, 1 << 20), 2), 1, ElemType.BF16) > 256         # rows cut into slices
    assert cq_reduce.workspace_bytes(t((64, 1 << 20), 2), 1, ElemType.BF16) <= (64 << 21) // 32


def test_into_contiguous_packed_checks():
    src, dst = t((16, 4), 4), t((16, 4), 4)
    run = lambda **k: cq_contiguous.into_contiguous_packed_ref(CLIENT, k.get("src", src), k.get("dst", dst),
                                                               k.get("shape", (16, 32)), k.get("packing", 8))
    assert status(lambda: run(shape=(16, 30))) == _ffi.ERR_SHAPE_MISMATCH       # last dim not a multiple of packing
    assert status(lambda: run(packing=5)) == _ffi.ERR_INVALID_ARGUMENT          # 32 bits / 5
    assert status(lambda: run(dst=t((16, 4), 4, (8, 1)))) == _ffi.ERR_NON_CONTIGUOUS
    assert status(lambda: run(dst=t((16, 4), 1))) == _ffi.ERR_SHAPE_MISMATCH    # element types differ
    assert status(lambda: run(shape=(16, 4, 8))) == _ffi.ERR_SHAPE_MISMATCH     # rank
    # transposed source: logical [32, 16] packed along dim 0 (stride 1): source shape must be [4, 16]
    assert status(lambda: run(src=t((32, 2), 4, (1, 4)), dst=t((32, 2), 4), shape=(32, 16))) == _ffi.ERR_SHAPE_MISMATCH


def test_element_counts_beyond_64_bit_products_are_refused():
    scheme = QuantScheme.default().with_value(QuantValue.Q8S)
    big = 1 << 31
    x, out, one = t((big, big, 4), 4), t((big, big, 1), 4), t((1,), 4)
    assert status(lambda: qz.launch_ref(CLIENT, x, out, one, one, scheme, ElemType.F32)) == _ffi.ERR_TOO_LARGE
    assert status(lambda: dq.launch_ref(CLIENT, out, x, one, scheme, ElemType.F32)) == _ffi.ERR_TOO_LARGE


def test_empty_tensors_are_a_no_op():
    """Zero elements: nothing to launch, success (shapes still have to agree)."""
    x, out, sc = t((0, 64), 4), t((0, 16), 4), t((0, 2), 4)
    qz.launch_ref(CLIENT, x, out, sc, sc, Q8_B32, ElemType.F32)
    dq.launch_ref(CLIENT, out, x, sc, Q8_B32, ElemType.F32)
    qz.launch_dynamic(CLIENT, x, out, sc, Q8_B32, ElemType.F32)
    qz.compute_scales(CLIENT, x, sc, Q8_B32, ElemType.F32)
    assert status(lambda: qz.launch_ref(CLIENT, x, t((0, 15), 4), sc, sc, Q8_B32, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH
    cq_reduce.max_abs(CLIENT, t((0, 8), 4), t((0, 1), 4), 1, ElemType.F32)   # no outputs
    cq_contiguous.into_contiguous_packed_ref(CLIENT, t((0, 4), 4), t((0, 4), 4), (0, 32), 8)


def test_argument_checks_walked_over_every_scheme_and_layout():
    """tests/cpp/plan_walk.cpp: 5.5 million cq_plan_kind calls over operation x float type x value x parameter type
    x store x block shape x tensor shape x layout, valid, invalid and damaged descriptors alike: no crash, every
    status a known one, a kernel family named whenever the answer is CQ_OK."""
    import os
    import subprocess

    binary = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "plan_walk")
    assert os.path.exists(binary), "tests/cpp/plan_walk is not built (make -C cubek_amd/csrc)"
    proc = subprocess.run([binary], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:]
    last = proc.stdout.strip().splitlines()[-1]
    counts = {int(k): int(v) for k, v in (f[1:].split("]=") for f in last.split()[2:])}
    assert sum(counts.values()) > 5_000_000 and counts[0] > 100_000, last   # plenty of valid calls among them
    assert all(counts[k] == 0 for k in (5, 6, 7, 9, 10, 11, 12, 13, 14, 15)), last  # nothing launched, nothing unknown
