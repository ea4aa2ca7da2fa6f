"""The streaming kernels that stage values or scales through LDS (cq_kernels_staged.hip), bit for bit against
the oracle through the C ABI:

* blocks that are not a power-of-two number of 16-byte chunks (24, 40, 48, 72, 120 ... values): fused dynamic
  quantize on the pieces kernel, given scales and dequantize lane by lane with a division by the block's chunks;
* scale tensors with any two strides (stored column by column, padded, with a column stride), on tiles of
  16 rows x 64 chunks whose edges are cut short both ways.

Every case also checks that nothing outside the outputs' views is written."""
import numpy as np
import pytest

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue,
                       TensorHandleRef, _ffi)
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu

ELEMS = [ElemType.BF16, ElemType.F16, ElemType.F32]


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def same_bits(a, b):
    a, b = np.ascontiguousarray(a).reshape(-1), np.ascontiguousarray(b).reshape(-1)
    return a.shape == b.shape and np.array_equal(a.view(np.uint8), b.view(np.uint8))


def scheme_of(value, store, block, param=QuantParam.F32):
    return (QuantScheme.default().with_value(value).with_store(store).with_param(param)
            .with_level(QuantLevel.block(list(block))))


def plan_family(op, scheme, elem, floats, values, scale, out_scale=None):
    return _ffi.plan_kind(op, floats, values, scale, out_scale, scheme, elem)


# (shape, block, value, store): blocks of 3, 5, 6, 7, 9, 12, 15, 17 and 31 chunks of a 16-bit type; rows that make the
# last wave ragged; several workgroups
PIECES = [
    ((64, 4104), (24,), QuantValue.Q8S, QuantStore.U32),
    ((7, 33, 120), (40,), QuantValue.Q4S, QuantStore.U32),
    ((1000, 48), (48,), QuantValue.Q2S, QuantStore.U32),
    ((129, 1008), (56,), QuantValue.E2M1, QuantStore.U32),
    ((31, 2160), (72,), QuantValue.Q8F, QuantStore.U32),
    ((300, 96), (96,), QuantValue.Q4F, QuantStore.U32),
    ((77, 1080), (120,), QuantValue.E4M3, QuantStore.Native),
    ((50, 2040), (136,), QuantValue.E5M2, QuantStore.Native),
    ((9, 4960), (248,), QuantValue.E2M1, QuantStore.Native),
    ((33, 1320), (40,), QuantValue.E2M1_OCP, QuantStore.U32),
    ((21, 1440), (72,), QuantValue.E2M1_OCP, QuantStore.Native),
    ((2000, 24), (24,), QuantValue.Q8S, QuantStore.Native),
    ((5, 240), (80,), QuantValue.Q2F, QuantStore.U32),
]


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("case", PIECES, ids=lambda c: f"{c[2].name}_{c[3].name}_b{c[1][0]}")
def test_blocks_of_an_odd_number_of_chunks(gpu, oracle, elem, case):
    shape, block, value, store = case
    rng = np.random.default_rng(sum(shape) + block[0] + int(elem))
    for param in (QuantParam.F32, QuantParam.F16 if elem == ElemType.BF16 else QuantParam.BF16):
        scheme = scheme_of(value, store, block, param)
        x32 = rng.normal(0, 1.5, shape).astype(np.float32)
        x32[rng.random(shape) < 0.002] = np.nan
        x32.reshape(-1)[:block[0]] = 0.0           # an all-zero block: scale 0, 0/0 -> q_max
        x = oracle.to_bits(x32, elem)
        s_ref = oracle.compute_scales(x, elem, shape, scheme)
        w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
        w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
        assert same_bits(w_dyn, w_ref) and same_bits(os_dyn, os_ref), (param, "dynamic")
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
        assert same_bits(w_gpu, w_ref) and same_bits(os_gpu, os_ref), (param, "given")
        y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
        y_gpu = gpu.dequantize(w_ref, shape, os_ref, elem, scheme)
        ok = ~np.isnan(oracle.from_bits(y_ref, elem)).reshape(-1)
        assert same_bits(y_gpu.reshape(-1)[ok], y_ref.reshape(-1)[ok]), (param, "dequantize")
        assert np.isnan(oracle.from_bits(y_gpu, elem)).reshape(-1)[~ok].all()


def test_odd_blocks_take_the_staged_and_the_lane_wise_kernels():
    """cq_plan_kind: contiguous bf16 [512, 4104] with blocks of 24: quantize (fused or with given scales) runs on
    the staged family, dequantize lane by lane; f32 blocks of 252 values (63 chunks: more than a wave's LDS share holds)
    stay with the block kernel."""
    import torch

    h = TensorHandleRef.from_torch
    for elem, dt, shape, block, dynamic, given in ((ElemType.BF16, torch.bfloat16, (512, 4104), 24, "staged", "staged"),
                                                   (ElemType.F32, torch.float32, (64, 2520), 252, "blocks", "flat_lanes")):
        scheme = scheme_of(QuantValue.Q8S, QuantStore.U32, (block,))
        x = torch.zeros(shape, dtype=dt, device="cuda")
        w = torch.zeros(scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
        s = torch.zeros(scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
        sf = torch.zeros(scheme.scales_shape(shape), dtype=dt, device="cuda")
        assert plan_family(_ffi.OP_QUANTIZE_DYNAMIC, scheme, elem, h(x), h(w), None, h(s)) == dynamic
        assert plan_family(_ffi.OP_QUANTIZE, scheme, elem, h(x), h(w), h(sf), h(s)) == given
        assert plan_family(_ffi.OP_DEQUANTIZE, scheme, elem, h(x), h(w), h(s)) == "flat_lanes"


def test_pieces_with_unaligned_codes_and_more_than_one_workgroup(gpu, oracle):
    """The stored tensor starts 4 bytes into its allocation (no 16-byte stores), 70 000 blocks of 24 bf16 values
    (274 waves of the pieces kernel, the last one ragged)."""
    import torch

    elem, shape = ElemType.BF16, (70000, 24)
    scheme = scheme_of(QuantValue.Q4S, QuantStore.U32, (24,))
    rng = np.random.default_rng(77)
    x = oracle.to_bits(rng.normal(0, 0.3, shape).astype(np.float32), elem)
    s_ref = oracle.compute_scales(x, elem, shape, scheme)
    w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
    pshape = scheme.packed_shape(shape)
    buf = torch.full((int(np.prod(pshape)) + 2,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    view = buf[1:-1].view(pshape)
    assert view.data_ptr() % 16 == 4
    os_ = torch.zeros(scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
    dx = gpu.to_dev(x.reshape(shape))
    h = TensorHandleRef.from_torch
    qz.launch_dynamic(ComputeClient.current(), h(dx), h(view), h(os_), scheme, elem)
    torch.cuda.synchronize()
    got = buf.cpu().numpy().view(np.uint32)
    assert got[0] == 0x5A5A5A5A and got[-1] == 0x5A5A5A5A
    assert np.array_equal(got[1:-1], w_ref.reshape(-1))
    assert same_bits(os_.cpu().numpy(), os_ref)


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("value,block,cols", [(QuantValue.Q4S, 24, 1176), (QuantValue.Q8S, 40, 4120), (QuantValue.Q2S, 48, 96)],
                         ids=["q4s_b24", "q8s_b40", "q2s_b48"])
def test_odd_blocks_on_pitched_rows(gpu, oracle, elem, value, block, cols):
    """Rows with a pitch of their own in all three tensors: given scales and dequantize run lane by lane with the
    division by the block's chunks, the fused quantize on the block kernel.  The padding keeps its bytes."""
    import torch

    rows = 37
    scheme = scheme_of(value, QuantStore.U32, (block,))
    nq, nb = scheme.num_quants(), cols // block
    rng = np.random.default_rng(block + cols + int(elem))
    x = oracle.to_bits(rng.normal(0, 1, (rows, cols)).astype(np.float32), elem)
    s_ref = oracle.compute_scales(x, elem, (rows, cols), scheme)
    w_ref, os_ref = oracle.quantize(x, elem, (rows, cols), s_ref, scheme)
    y_ref = oracle.dequantize(w_ref, (rows, cols), os_ref, elem, scheme)
    esz = 4 if elem == ElemType.F32 else 2
    pad = 32 // esz
    fill = np.float32(777.0) if elem == ElemType.F32 else np.uint16(0x7777)
    xbuf = np.full((rows, cols + pad), fill, dtype=x.dtype)
    xbuf[:, :cols] = x.reshape(rows, cols)
    sbuf = np.full((rows, nb + 3), fill, dtype=x.dtype)
    sbuf[:, :nb] = np.asarray(s_ref).reshape(rows, nb)
    d_x, d_s = gpu.to_dev(xbuf), gpu.to_dev(sbuf)
    wcols = cols // nq
    d_w = torch.full((rows, wcols + 4), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    d_os = torch.full((rows, nb + 1), -5.0, dtype=torch.float32, device="cuda")
    hx = TensorHandleRef(d_x.data_ptr(), (rows, cols), (cols + pad, 1), esz)
    hs = TensorHandleRef(d_s.data_ptr(), (rows, nb), (nb + 3, 1), esz)
    hw = TensorHandleRef(d_w.data_ptr(), (rows, wcols), (wcols + 4, 1), 4)
    hos = TensorHandleRef(d_os.data_ptr(), (rows, nb), (nb + 1, 1), 4)
    client = ComputeClient.current()
    assert plan_family(_ffi.OP_QUANTIZE, scheme, elem, hx, hw, hs, hos) == "flat_lanes"
    assert plan_family(_ffi.OP_DEQUANTIZE, scheme, elem, hx, hw, hos) == "flat_lanes"

    def check_stored(what):
        got_w = d_w.cpu().numpy().view(np.uint32)
        assert np.array_equal(got_w[:, :wcols], w_ref.reshape(rows, -1)) and np.all(got_w[:, wcols:] == 0x5A5A5A5A), what
        got_s = d_os.cpu().numpy()
        assert same_bits(got_s[:, :nb], os_ref) and np.all(got_s[:, nb:] == -5.0), what

    qz.launch_ref(client, hx, hw, hs, hos, scheme, elem)
    torch.cuda.synchronize()
    check_stored("given")
    d_w.fill_(0x5A5A5A5A)
    d_os.fill_(-5.0)
    qz.launch_dynamic(client, hx, hw, hos, scheme, elem)
    torch.cuda.synchronize()
    check_stored("dynamic")
    d_y = gpu.to_dev(np.full((rows, cols + pad), fill, dtype=x.dtype))
    dq.launch_ref(client, hw, TensorHandleRef(d_y.data_ptr(), (rows, cols), (cols + pad, 1), esz), hos, scheme, elem)
    torch.cuda.synchronize()
    got_y = gpu.to_host(d_y)
    assert same_bits(got_y[:, :cols], y_ref.reshape(rows, cols)) and np.all(got_y[:, cols:] == fill)


# ---- scale tensors with two strides ----------------------------------------------------------------------------

def strided_buffer(rng, shape, strides, fill, dtype):
    """A buffer that holds a [rows, cols] view with the given strides (elements), filled with `fill` elsewhere."""
    reach = 1 + sum((n - 1) * st for n, st in zip(shape, strides))
    return np.full(reach, fill, dtype=dtype)


def place(buf, values, strides):
    rows, cols = values.shape
    idx = (np.arange(rows)[:, None] * strides[0] + np.arange(cols)[None, :] * strides[1]).reshape(-1)
    buf[idx] = values.reshape(-1)
    return idx


SCALE_LAYOUTS = {
    "column_major": lambda rows, nb: (1, rows),
    "column_major_padded": lambda rows, nb: (1, rows + 3),
    "column_stride_2": lambda rows, nb: (2 * nb + 1, 2),
    "both_strided": lambda rows, nb: (3, 3 * rows + 2),
}
# (rows, cols, block, value, store): tiles cut short along rows (33, 70, 5) and along the row (cols / chunk not a
# multiple of 64), every width of codes
TILE_CASES = [
    (70, 1056, 32, QuantValue.E2M1, QuantStore.U32),
    (33, 2048, 64, QuantValue.Q8S, QuantStore.U32),
    (128, 512, 16, QuantValue.Q4S, QuantStore.U32),
    (5, 4160, 32, QuantValue.Q2S, QuantStore.U32),
    (40, 1280, 128, QuantValue.E4M3, QuantStore.Native),
    (64, 640, 32, QuantValue.E2M1, QuantStore.Native),
    (45, 1088, 32, QuantValue.E2M1_OCP, QuantStore.U32),
    (20, 1024, 64, QuantValue.E2M1_OCP, QuantStore.Native),
    (37, 768, 128, QuantValue.Q8F, QuantStore.Native),
]


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("layout", sorted(SCALE_LAYOUTS))
@pytest.mark.parametrize("case", TILE_CASES, ids=lambda c: f"{c[3].name}_{c[4].name}_{c[0]}x{c[1]}_b{c[2]}")
def test_scale_tensors_with_two_strides(gpu, oracle, elem, layout, case):
    import torch

    rows, cols, block, value, store = case
    if elem == ElemType.F32 and block > 128:
        block = 128  # 32 lanes of four values at most
    shape = (rows, cols)
    nb = cols // block
    rng = np.random.default_rng(rows * 31 + cols + int(elem))
    param = {ElemType.BF16: QuantParam.F32, ElemType.F16: QuantParam.F16, ElemType.F32: QuantParam.BF16}[elem]
    scheme = scheme_of(value, store, (block,), param)
    pe = gpu.param_elem(scheme)
    x32 = rng.normal(0, 0.7, shape).astype(np.float32)
    x32[rng.random(shape) < 0.001] = np.nan
    x = oracle.to_bits(x32, elem)
    s_ref = oracle.compute_scales(x, elem, shape, scheme)                  # [rows, nb], typed elem
    w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)         # out_scale typed param
    y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
    sstr = SCALE_LAYOUTS[layout](rows, nb)
    ostr = SCALE_LAYOUTS["column_major" if layout != "column_major" else "column_stride_2"](rows, nb)
    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    hs = lambda t, strides: TensorHandleRef(t.data_ptr(), (rows, nb), tuple(strides), t.element_size())
    stored_np = np.uint32 if store == QuantStore.U32 else np.uint8
    pshape = scheme.packed_shape(shape)
    dx = gpu.to_dev(x.reshape(shape))
    sent16, sent32 = np.uint16(0x7B7B), np.float32(-777.0)
    sent = lambda e: sent32 if e == ElemType.F32 else sent16
    np_of = lambda e: np.float32 if e == ElemType.F32 else np.uint16

    def fresh_out_scale(strides):
        buf = strided_buffer(rng, (rows, nb), strides, sent(pe), np_of(pe))
        return gpu.to_dev(buf)

    def check_out_scale(t, strides, what):
        got = gpu.to_host(t)
        want = strided_buffer(rng, (rows, nb), strides, sent(pe), np_of(pe))
        place(want, np.asarray(os_ref).reshape(rows, nb), strides)
        assert same_bits(got, want), (layout, what)

    # the plan: nothing of this runs one thread per element or on the row kernels
    sin_buf = strided_buffer(rng, (rows, nb), sstr, sent(elem), np_of(elem))
    place(sin_buf, np.asarray(s_ref).reshape(rows, nb), sstr)
    d_sin = gpu.to_dev(sin_buf)
    d_w = torch.zeros(pshape, dtype=torch.int32 if store == QuantStore.U32 else torch.uint8, device="cuda")
    d_os = fresh_out_scale(ostr)
    assert plan_family(_ffi.OP_QUANTIZE, scheme, elem, h(dx), h(d_w), hs(d_sin, sstr), hs(d_os, ostr)) == "staged"
    assert plan_family(_ffi.OP_QUANTIZE_DYNAMIC, scheme, elem, h(dx), h(d_w), None, hs(d_os, ostr)) == "staged"
    assert plan_family(_ffi.OP_DEQUANTIZE, scheme, elem, h(dx), h(d_w), hs(d_os, ostr)) == "staged"

    # given scales in one layout, out_scale in another
    qz.launch_ref(client, h(dx), h(d_w), hs(d_sin, sstr), hs(d_os, ostr), scheme, elem)
    torch.cuda.synchronize()
    assert same_bits(gpu.to_host(d_w).view(stored_np), w_ref), (layout, "given")
    check_out_scale(d_os, ostr, "given out_scale")

    # fused abs-max, out_scale in the first layout
    d_w2 = torch.zeros_like(d_w)
    d_os2 = fresh_out_scale(sstr)
    qz.launch_dynamic(client, h(dx), h(d_w2), hs(d_os2, sstr), scheme, elem)
    torch.cuda.synchronize()
    assert same_bits(gpu.to_host(d_w2).view(stored_np), w_ref), (layout, "dynamic")
    check_out_scale(d_os2, sstr, "dynamic out_scale")

    # dequantize from either
    for t, strides in ((d_os, ostr), (d_os2, sstr)):
        d_y = torch.zeros(shape, dtype=gpu.storage_dtype(elem), device="cuda")
        dq.launch_ref(client, h(d_w), h(d_y), hs(t, strides), scheme, elem)
        torch.cuda.synchronize()
        y_gpu = gpu.to_host(d_y)
        ok = ~np.isnan(oracle.from_bits(y_ref, elem)).reshape(-1)
        assert same_bits(y_gpu.reshape(-1)[ok], y_ref.reshape(-1)[ok]), (layout, "dequantize")
        assert np.isnan(oracle.from_bits(y_gpu, elem)).reshape(-1)[~ok].all()


def test_scale_tiles_on_pitched_rows(gpu, oracle):
    """Value tensors with a row pitch of their own (a [100, 1024] view of [100, 1040] floats, codes in rows of 136
    words) under scales stored column by column: the padding keeps its bytes."""
    import torch

    elem, rows, cols, block = ElemType.BF16, 100, 1024, 32
    scheme = scheme_of(QuantValue.Q4S, QuantStore.U32, (block,))
    nb = cols // block
    rng = np.random.default_rng(9)
    x = oracle.to_bits(rng.normal(0, 1, (rows, cols)).astype(np.float32), elem)
    s_ref = oracle.compute_scales(x, elem, (rows, cols), scheme)
    w_ref, os_ref = oracle.quantize(x, elem, (rows, cols), s_ref, scheme)
    y_ref = oracle.dequantize(w_ref, (rows, cols), os_ref, elem, scheme)
    xbuf = np.full((rows, cols + 16), 0x7F7F, dtype=np.uint16)
    xbuf[:, :cols] = x.reshape(rows, cols)
    d_x = gpu.to_dev(xbuf)
    d_w = torch.full((rows, 136), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    d_os = torch.full((nb, rows), -5.0, dtype=torch.float32, device="cuda")
    hx = TensorHandleRef(d_x.data_ptr(), (rows, cols), (cols + 16, 1), 2)
    hw = TensorHandleRef(d_w.data_ptr(), (rows, cols // 8), (136, 1), 4)
    hos = TensorHandleRef(d_os.data_ptr(), (rows, nb), (1, rows), 4)
    client = ComputeClient.current()
    assert plan_family(_ffi.OP_QUANTIZE_DYNAMIC, scheme, elem, hx, hw, None, hos) == "staged"
    qz.launch_dynamic(client, hx, hw, hos, scheme, elem)
    torch.cuda.synchronize()
    got_w = d_w.cpu().numpy().view(np.uint32)
    assert np.array_equal(got_w[:, :cols // 8], w_ref.reshape(rows, -1)) and np.all(got_w[:, cols // 8:] == 0x5A5A5A5A)
    assert same_bits(d_os.cpu().numpy().T, os_ref)
    d_y = torch.full((rows, cols + 16), 0x7777, dtype=torch.int16, device="cuda")
    hy = TensorHandleRef(d_y.data_ptr(), (rows, cols), (cols + 16, 1), 2)
    dq.launch_ref(client, hw, hy, hos, scheme, elem)
    torch.cuda.synchronize()
    got_y = d_y.cpu().numpy().view(np.uint16)
    assert np.array_equal(got_y[:, :cols], y_ref.reshape(rows, cols)) and np.all(got_y[:, cols:] == 0x7777)


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("value,block", [(QuantValue.Q8S, 32), (QuantValue.E2M1, 64), (QuantValue.Q2S, 128)],
                         ids=["q8s_b32", "e2m1_b64", "q2s_b128"])
@pytest.mark.parametrize("v_layout", ["transposed", "transposed_padded", "column_stride_3"])
def test_stored_tensor_whose_last_dimension_is_not_contiguous(gpu, oracle, elem, value, block, v_layout):
    """Words of the U32 store with a stride along the last dimension (the stored tensor transposed in memory, with
    padded columns, or every third word of its rows): the codes of a tile pass through LDS.  70 rows x 4224 columns:
    tiles cut short both ways.  Quantize (fused and with given scales) and dequantize against the oracle; the bytes
    between the words keep their value."""
    import torch

    rows, cols = 70, 4224
    if elem == ElemType.F32 and block == 128:
        block = 64
    scheme = scheme_of(value, QuantStore.U32, (block,))
    nq, nb = scheme.num_quants(), cols // block
    wcols = cols // nq
    vstr = {"transposed": (1, rows), "transposed_padded": (1, rows + 5), "column_stride_3": (3 * wcols + 2, 3)}[v_layout]
    rng = np.random.default_rng(rows + block + int(elem))
    x = oracle.to_bits(rng.normal(0, 1, (rows, cols)).astype(np.float32), elem)
    s_ref = oracle.compute_scales(x, elem, (rows, cols), scheme)
    w_ref, os_ref = oracle.quantize(x, elem, (rows, cols), s_ref, scheme)
    y_ref = oracle.dequantize(w_ref, (rows, cols), os_ref, elem, scheme)
    reach = 1 + (rows - 1) * vstr[0] + (wcols - 1) * vstr[1]
    idx = (np.arange(rows)[:, None] * vstr[0] + np.arange(wcols)[None, :] * vstr[1]).reshape(-1)
    want_buf = np.full(reach, 0x5A5A5A5A, dtype=np.uint32)
    want_buf[idx] = np.asarray(w_ref).reshape(-1)
    d_x, d_s = gpu.to_dev(x.reshape(rows, cols)), gpu.to_dev(np.asarray(s_ref).reshape(rows, nb))
    h = TensorHandleRef.from_torch
    client = ComputeClient.current()
    for what in ("dynamic", "given"):
        d_w = torch.full((reach,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
        d_os = torch.zeros((rows, nb), dtype=torch.float32, device="cuda")
        hw = TensorHandleRef(d_w.data_ptr(), (rows, wcols), vstr, 4)
        if what == "dynamic":
            assert plan_family(_ffi.OP_QUANTIZE_DYNAMIC, scheme, elem, h(d_x), hw, None, h(d_os)) == "staged"
            qz.launch_dynamic(client, h(d_x), hw, h(d_os), scheme, elem)
        else:
            assert plan_family(_ffi.OP_QUANTIZE, scheme, elem, h(d_x), hw, h(d_s), h(d_os)) == "staged"
            qz.launch_ref(client, h(d_x), hw, h(d_s), h(d_os), scheme, elem)
        torch.cuda.synchronize()
        assert np.array_equal(d_w.cpu().numpy().view(np.uint32), want_buf), (v_layout, what)
        assert same_bits(d_os.cpu().numpy(), os_ref), (v_layout, what)
    d_y = torch.zeros((rows, cols), dtype=gpu.storage_dtype(elem), device="cuda")
    assert plan_family(_ffi.OP_DEQUANTIZE, scheme, elem, h(d_y), hw, h(d_os)) == "staged"
    dq.launch_ref(client, hw, h(d_y), h(d_os), scheme, elem)
    torch.cuda.synchronize()
    assert same_bits(gpu.to_host(d_y), y_ref), v_layout


@pytest.mark.parametrize("what", ["blocks_of_24", "column_major_scales"])
def test_staged_kernels_at_full_size_match_the_flat_kernels(gpu, what):
    """bf16 [28672, 8184] with blocks of 24 and [28672, 8192] with scales stored column by column: thousands of
    workgroups.  Given scales / dequantize of the odd blocks run lane by lane and were checked against the oracle
    above; here the fused quantize must give the same codes and scales as that path, and the column-major launches
    the same as the contiguous-scale (flat) ones."""
    import torch

    h = TensorHandleRef.from_torch
    client = ComputeClient.current()
    g = torch.Generator(device="cuda").manual_seed(5)
    if what == "blocks_of_24":
        rows, cols, block = 28672, 8184, 24
        scheme = scheme_of(QuantValue.Q4S, QuantStore.U32, (block,))
        x = torch.randn((rows, cols), generator=g, device="cuda", dtype=torch.float32).mul_(0.02).to(torch.bfloat16)
        w1 = torch.zeros(scheme.packed_shape((rows, cols)), dtype=torch.int32, device="cuda")
        s1 = torch.zeros(scheme.scales_shape((rows, cols)), dtype=torch.float32, device="cuda")
        qz.launch_dynamic(client, h(x), h(w1), h(s1), scheme, ElemType.BF16)
        # the same scales, given (typed like the input: they are bf16 values already)
        w2, s2 = torch.zeros_like(w1), torch.zeros_like(s1)
        qz.launch_ref(client, h(x), h(w2), h(s1.to(torch.bfloat16)), h(s2), scheme, ElemType.BF16)
        torch.cuda.synchronize()
        assert torch.equal(w1, w2) and torch.equal(s1.view(torch.int32), s2.view(torch.int32))
        # scales against torch: F(2 * absmax / 14) with the division in f32
        amax = x.view(rows, cols // block, block).abs().amax(dim=2).float()
        want = ((2 * amax) / 14.0).to(torch.bfloat16).float()
        assert torch.equal(s1, want)
        # codes and dequantized values against the same formulas in torch (bf16 arithmetic = the f32 operation rounded
        # once): clamp(rint(bf16(x / d)), -7, 7) and bf16(scale * code)
        y = torch.empty_like(x)
        dq.launch_ref(client, h(w1), h(y), h(s1), scheme, ElemType.BF16)
        torch.cuda.synchronize()
        shifts = torch.arange(8, device="cuda", dtype=torch.int32) * 4
        codes = (w1.unsqueeze(-1) >> shifts) & 15
        codes = torch.where(codes >= 8, codes - 16, codes).reshape(rows, cols)
        d = s1.repeat_interleave(block, dim=1)
        want_codes = (x.float() / d).to(torch.bfloat16).float().round().clamp(-7, 7).to(torch.int32)
        assert torch.equal(codes, want_codes)
        assert torch.equal((codes.float() * d).to(torch.bfloat16).view(torch.int16), y.view(torch.int16))
    else:
        rows, cols, block = 28672, 8192, 32
        scheme = scheme_of(QuantValue.E2M1, QuantStore.U32, (block,))
        nb = cols // block
        x = torch.randn((rows, cols), generator=g, device="cuda", dtype=torch.float32).mul_(0.02).to(torch.bfloat16)
        w1 = torch.zeros(scheme.packed_shape((rows, cols)), dtype=torch.int32, device="cuda")
        s1 = torch.zeros((rows, nb), dtype=torch.float32, device="cuda")
        qz.launch_dynamic(client, h(x), h(w1), h(s1), scheme, ElemType.BF16)         # flat
        col = lambda t: TensorHandleRef(t.data_ptr(), (rows, nb), (1, rows), t.element_size())
        w2 = torch.zeros_like(w1)
        s2 = torch.zeros((nb, rows), dtype=torch.float32, device="cuda")
        qz.launch_dynamic(client, h(x), h(w2), col(s2), scheme, ElemType.BF16)       # tiles
        torch.cuda.synchronize()
        assert torch.equal(w1, w2) and torch.equal(s1.view(torch.int32), s2.t().contiguous().view(torch.int32))
        w3 = torch.zeros_like(w1)
        s3 = torch.zeros((nb, rows), dtype=torch.float32, device="cuda")
        sin = s2.to(torch.bfloat16)
        qz.launch_ref(client, h(x), h(w3), col(sin), col(s3), scheme, ElemType.BF16)
        y1, y2 = torch.empty_like(x), torch.empty_like(x)
        dq.launch_ref(client, h(w1), h(y1), h(s1), scheme, ElemType.BF16)
        dq.launch_ref(client, h(w1), h(y2), col(s2), scheme, ElemType.BF16)
        torch.cuda.synchronize()
        assert torch.equal(w1, w3) and torch.equal(s2.view(torch.int32), s3.view(torch.int32))
        assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
