"""Non-contiguous value tensors through the C ABI.  The reference addresses its
tensors through linear views built from shape and strides
(crates/cubek-quant/src/quantize.rs:309-317, src/dequantize.rs:261-270), so a
strided tensor must give what its contiguous copy gives: the oracle runs on the
copy, the GPU on the strided buffers, and the logical views are compared bit
for bit.  Elements of the destination buffers outside the views must stay untouched."""
import zlib

import numpy as np
import pytest
from numpy.lib.stride_tricks import as_strided

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantScheme, QuantStore, QuantValue, TensorHandleRef)
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def reach(shape, strides):
    return 1 + sum((n - 1) * st for n, st in zip(shape, strides))


def view(buf, shape, strides):
    assert reach(shape, strides) <= buf.size
    return as_strided(buf, shape, tuple(st * buf.itemsize for st in strides))


def layouts(shape, per):
    """(name, float strides, stored strides) for logical `shape`, `per` values per stored element."""
    pshape = shape[:-1] + (shape[-1] // per,)
    rank = len(shape)

    def contiguous(sh, pad=0):
        st, acc = [], 1
        for i, n in enumerate(reversed(sh)):
            st.append(acc)
            acc *= n + (pad if i == 0 else 0)
        return tuple(reversed(st))

    def permuted(sh):
        # memory order = reversed logical order (a transposed tensor)
        st, acc = [], 1
        for n in sh:
            st.append(acc)
            acc *= n
        return tuple(st)

    out = [("contiguous", contiguous(shape), contiguous(pshape)),
           ("pitched", contiguous(shape, 5), contiguous(pshape, 3)),
           ("pitched_aligned", contiguous(shape, 64), contiguous(pshape, 8)),
           # rows that start on multiples of 4 bytes only: 16-byte loads and 8-byte stores off their alignment
           ("pitched_words", contiguous(shape, 6), contiguous(pshape, 1)),
           ("transposed_floats", permuted(shape), contiguous(pshape)),
           ("transposed_stored", contiguous(shape), permuted(pshape)),
           ("both", permuted(shape), permuted(pshape))]
    if rank >= 2:
        # last two dimensions swapped in memory (rows of the buffer = logical columns), padded pitch,
        # leading dimensions outermost: the transposed-float kernels
        def swapped(sh, pad):
            st = [0] * len(sh)
            st[-2] = 1
            st[-1] = sh[-2] + pad
            acc = st[-1] * sh[-1]
            for d in range(len(sh) - 3, -1, -1):
                st[d] = acc
                acc *= sh[d]
            return tuple(st)

        out.append(("last_two_swapped", swapped(shape, 0), contiguous(pshape)))
        out.append(("last_two_swapped_pitched", swapped(shape, 6), contiguous(pshape, 3)))
        out.append(("every_other_row", tuple(s * (2 if d == 0 else 1) for d, s in enumerate(contiguous(shape))),
                    tuple(s * (2 if d == 0 else 1) for d, s in enumerate(contiguous(pshape)))))
    if rank >= 3:
        # the first two dimensions swapped in memory, pitched rows: groups of rows with a pitch of their own
        def leading_swapped(sh, pad):
            st = contiguous((sh[1], sh[0]) + tuple(sh[2:]), pad)
            return (st[1], st[0]) + tuple(st[2:])

        out.append(("leading_swapped", leading_swapped(shape, 64), leading_swapped(pshape, 8)))
        out.append(("leading_swapped_floats", leading_swapped(shape, 0), contiguous(pshape)))
    if rank >= 4:
        # dimensions 1 and 2 swapped in memory (heads and positions of an attention tensor): short rows
        # behind three levels of strides
        def middle_swapped(sh):
            st = contiguous((sh[0], sh[2], sh[1]) + tuple(sh[3:]))
            return (st[0], st[2], st[1]) + tuple(st[3:])

        out.append(("middle_swapped", middle_swapped(shape), middle_swapped(pshape)))
        out.append(("middle_swapped_floats", middle_swapped(shape), contiguous(pshape)))
    return pshape, out


SCHEMES = [
    ("q8s_tensor", QuantScheme.default().with_value(QuantValue.Q8S)),
    ("q4s_block32", QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))),
    ("q2f_block_2x16", QuantScheme.default().with_value(QuantValue.Q2F).with_level(QuantLevel.block([2, 16]))),
    ("e2m1_u32_block16", QuantScheme.default().with_value(QuantValue.E2M1).with_level(QuantLevel.block([16]))),
    ("q8f_native_block16", QuantScheme.default().with_value(QuantValue.Q8F).with_store(QuantStore.Native)
     .with_level(QuantLevel.block([16]))),
    ("e4m3_native_tensor", QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)),
    ("e2m1_native_block32", QuantScheme.default().with_value(QuantValue.E2M1).with_store(QuantStore.Native)
     .with_level(QuantLevel.block([32]))),
    # the extension value (e2m1 nibbles rounded once, in either store)
    ("ocp_u32_block32", QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_level(QuantLevel.block([32]))),
    ("ocp_native_block16", QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_store(QuantStore.Native)
     .with_level(QuantLevel.block([16]))),
    # blocks of 64 / 128 columns: on transposed floats, lanes share a block
    ("q8s_block64", QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([64]))),
    ("q4s_block128", QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([128]))),
    ("e4m3_native_block64", QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)
     .with_level(QuantLevel.block([64]))),
    # value ranges wider than their 8-bit field in the u32 store: the codes wrap (src/quantize.rs:75)
    ("e4m3_u32_block32", QuantScheme.default().with_value(QuantValue.E4M3).with_level(QuantLevel.block([32]))),
    ("e5m2_u32_tensor", QuantScheme.default().with_value(QuantValue.E5M2)),
]


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_strided_value_tensors(gpu, oracle, elem, name, scheme):
    check_layouts(gpu, oracle, elem, name, scheme, ((6, 64), (2, 4, 96), (3, 70, 128), (2, 72, 256)), None)


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_long_pitched_rows(gpu, oracle, elem, name, scheme):
    """Rows of many steps of the streaming kernels (whole steps, and a partial last step per row),
    with 1-D blocks and with blocks over the last two dimensions."""
    check_layouts(gpu, oracle, elem, name, scheme, ((4, 16384), (2, 2, 16384 + 4096 + 512)),
                  ("contiguous", "pitched", "pitched_aligned", "every_other_row", "leading_swapped", "leading_swapped_floats"))


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_pitched_rows_of_a_few_steps(gpu, oracle, elem, name, scheme):
    """Rows of 256 - 896 sixteen-byte chunks: the streaming kernels take them as steps of 256 chunks,
    so one workgroup's steps lie in up to four rows (also rows of a block that share their scales),
    a row's last step may be partial, and the launch ends on a workgroup with fewer steps than the others."""
    check_layouts(gpu, oracle, elem, name, scheme,
                  ((4, 4096), (6, 5120), (2, 2, 7168), (4, 2560), (6, 2048), (6, 1024), (10, 1280), (3, 2, 2048), (2, 3, 2, 2560)),
                  ("pitched", "pitched_aligned", "pitched_words", "every_other_row", "leading_swapped", "leading_swapped_floats"))


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_short_rows_behind_permuted_dimensions(gpu, oracle, elem, name, scheme):
    """[batch, heads, positions, head dimension] views of [batch, positions, heads, head dimension] buffers,
    and short pitched rows: every lane of the streaming kernels finds its own row."""
    check_layouts(gpu, oracle, elem, name, scheme, ((2, 3, 6, 128), (2, 5, 8, 64), (2, 4, 8, 128), (1, 12, 24, 64), (1, 2, 300, 256), (3, 2, 2, 1024)),
                  ("middle_swapped", "middle_swapped_floats", "pitched_aligned", "pitched_words", "every_other_row", "leading_swapped"))


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_short_rows_behind_a_long_innermost_dimension(gpu, oracle, elem, name, scheme):
    """Attention-shaped views whose position axis is longer than the rows one workgroup spans: the lanes step
    from their workgroup's first row, with a carry through one, two and three outer dimensions, and the last
    workgroup runs past the end."""
    check_layouts(gpu, oracle, elem, name, scheme, ((2, 3, 1100, 128), (1, 2, 2102, 64), (2, 2, 3, 302, 64)),
                  ("middle_swapped", "middle_swapped_floats", "leading_swapped"))


@pytest.mark.parametrize("name,scheme", SCHEMES, ids=[n for n, _ in SCHEMES])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_long_rows_behind_permuted_dimensions_in_whole_tiles(gpu, oracle, elem, name, scheme):
    """Attention-shaped views with rows of 512 bytes and more whose position axis is a whole number of workgroup
    tiles: the launch reads them head by head (its workgroups take their tiles in another order than they are
    numbered in)."""
    check_layouts(gpu, oracle, elem, name, scheme, ((2, 3, 1024, 256), (1, 5, 512, 512), (2, 2, 3, 256, 256)),
                  ("middle_swapped", "middle_swapped_floats"))


BLOCKS_OF_ROWS = [
    ("q8s_block_16x32", QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([16, 32]))),
    ("q4s_block_8x64", QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([8, 64]))),
    ("e4m3_native_block_32x32", QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)
     .with_level(QuantLevel.block([32, 32]))),
    ("q2s_block_64x64", QuantScheme.default().with_value(QuantValue.Q2S).with_level(QuantLevel.block([64, 64]))),
]


@pytest.mark.parametrize("name,scheme", BLOCKS_OF_ROWS, ids=[n for n, _ in BLOCKS_OF_ROWS])
@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_blocks_of_rows_on_short_rows(gpu, oracle, elem, name, scheme):
    """Blocks of 8 - 64 rows on rows of at most 1 KiB: the fused abs-max + quantize runs as two launches (the
    scales, then the streaming kernel lane by lane reading them back); given scales and dequantize take the
    same lane-wise kernels."""
    check_layouts(gpu, oracle, elem, name, scheme, ((2, 4, 64, 128), (192, 256), (3, 128, 64), (2, 64, 192)),
                  ("contiguous", "pitched_aligned", "pitched_words", "every_other_row", "middle_swapped", "leading_swapped"))


def test_half_words_of_codes_per_row(gpu, oracle):
    """f32 rows of 12 and 20 values as e2m1 bytes: a row ends in the middle of a 32-bit word of codes, so the
    kernels whose lanes pair up to store a word must leave such rows (and a tensor of 3 x 4 values, whose
    codes end half a word in) to the kernels that store bytes."""
    scheme = QuantScheme.default().with_value(QuantValue.E2M1).with_store(QuantStore.Native).with_level(QuantLevel.block([4]))
    check_layouts(gpu, oracle, ElemType.F32, "e2m1_native_block4", scheme, ((6, 12), (5, 3, 20), (3, 4), (1, 12)),
                  ("contiguous", "pitched_aligned", "pitched_words", "every_other_row"))


def check_layouts(gpu, oracle, elem, name, scheme, shapes, only):
    import torch

    rng = np.random.default_rng(zlib.crc32(name.encode()) % 1000 + int(elem))
    client = ComputeClient.current()
    per = scheme.num_quants()
    stored_np = np.uint32 if scheme.store == QuantStore.U32 else np.uint8
    pe = gpu.param_elem(scheme)
    for shape in shapes:
        if scheme.level.block_size is not None and shape[-1] % scheme.level.block_size.dims[-1]:
            continue
        pshape, cases = layouts(shape, per)
        sshape = scheme.scales_shape(shape)
        for case, fstr, vstr in cases:
            if only is not None and case not in only:
                continue
            fbuf = oracle.to_bits(rng.normal(0, 1, reach(shape, fstr)).astype(np.float32), elem)
            xc = np.ascontiguousarray(view(fbuf, shape, fstr))
            s_ref = oracle.compute_scales(xc, elem, shape, scheme)
            w_ref, os_ref = oracle.quantize(xc, elem, shape, s_ref, scheme)
            y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
            tag = (name, elem.name, shape, case)

            d_f = gpu.to_dev(fbuf)
            h_f = gpu.handle(d_f, shape, fstr)
            sentinel = 0xA5 if stored_np == np.uint8 else 0xA5A5A5A5
            vbuf0 = np.full(reach(pshape, vstr), sentinel, dtype=stored_np)

            def stored_handle():
                d = gpu.to_dev(vbuf0)
                return d, gpu.handle(d, pshape, vstr)

            def check_stored(d_v, what):
                got = gpu.to_host(d_v).view(stored_np)
                assert np.array_equal(view(got, pshape, vstr), w_ref.reshape(pshape)), tag + (what,)
                mask = np.ones(got.size, dtype=bool)
                view(mask, pshape, vstr)[...] = False
                assert np.all(got[mask] == sentinel), tag + (what, "wrote outside the view")

            # scales from the strided floats
            d_s = torch.zeros(sshape, dtype=gpu.storage_dtype(elem), device="cuda")
            ws, nbytes = gpu.workspace(scheme, int(np.prod(shape)))
            qz.compute_scales(client, h_f, gpu.handle(d_s), scheme, elem, ws.data_ptr(), nbytes)
            assert np.array_equal(gpu.to_host(d_s).reshape(-1), s_ref.reshape(-1)), tag + ("scales",)

            # quantize with given scales
            d_v, h_v = stored_handle()
            d_os = torch.zeros(sshape, dtype=gpu.storage_dtype(pe), device="cuda")
            qz.launch_ref(client, h_f, h_v, gpu.handle(d_s), gpu.handle(d_os), scheme, elem)
            torch.cuda.synchronize()
            check_stored(d_v, "quantize")
            assert np.array_equal(gpu.to_host(d_os).reshape(-1), os_ref.reshape(-1)), tag + ("out_scale",)

            # fused dynamic quantize
            d_v2, h_v2 = stored_handle()
            d_os2 = torch.zeros(sshape, dtype=gpu.storage_dtype(pe), device="cuda")
            qz.launch_dynamic(client, h_f, h_v2, gpu.handle(d_os2), scheme, elem, ws.data_ptr(), nbytes)
            torch.cuda.synchronize()
            check_stored(d_v2, "dynamic")
            assert np.array_equal(gpu.to_host(d_os2).reshape(-1), os_ref.reshape(-1)), tag + ("dynamic out_scale",)

            # dequantize strided stored -> strided floats
            fill = np.float32(777.0) if elem == ElemType.F32 else np.uint16(0x7777)
            ybuf0 = np.full(fbuf.size, fill, dtype=fbuf.dtype)
            d_y = gpu.to_dev(ybuf0)
            dq.launch_ref(client, h_v, gpu.handle(d_y, shape, fstr), gpu.handle(d_os), scheme, elem)
            torch.cuda.synchronize()
            got = gpu.to_host(d_y).view(fbuf.dtype)
            lhs, rhs = view(got, shape, fstr), y_ref.reshape(shape)
            if elem == ElemType.F32:
                lhs, rhs = lhs.view(np.uint32), rhs.view(np.uint32)
            assert np.array_equal(lhs, rhs), tag + ("dequantize",)
            mask = np.ones(got.size, dtype=bool)
            view(mask, shape, fstr)[...] = False
            assert np.all(got[mask] == fill), tag + ("dequantize wrote outside the view",)


LARGE_TRANSPOSED_SCHEMES = {
    "q4s_block32": QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32])),
    "q8s_tensor": QuantScheme.default().with_value(QuantValue.Q8S),
    "e4m3_native_block32": (QuantScheme.default().with_value(QuantValue.E4M3).with_store(QuantStore.Native)
                            .with_level(QuantLevel.block([32]))),
    "e2m1_block32": QuantScheme.default().with_value(QuantValue.E2M1).with_level(QuantLevel.block([32])),
    "ocp_u32_block32": QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_level(QuantLevel.block([32])),
    "ocp_native_block64": (QuantScheme.default().with_value(QuantValue.E2M1_OCP).with_store(QuantStore.Native)
                           .with_level(QuantLevel.block([64]))),
    "q2s_block32": QuantScheme.default().with_value(QuantValue.Q2S).with_level(QuantLevel.block([32])),
    "q8s_block32": QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([32])),
    "q4s_block64": QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([64])),
    "e5m2_native_tensor": QuantScheme.default().with_value(QuantValue.E5M2).with_store(QuantStore.Native),
    "q4s_block96": QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([96])),
    "q8s_block96": QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([96])),
    "q8s_block160": QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([160])),
    "q2s_block192": QuantScheme.default().with_value(QuantValue.Q2S).with_level(QuantLevel.block([192])),
}


@pytest.mark.parametrize("elem,rows,cols", [(ElemType.BF16, 12288, 8192), (ElemType.F32, 6144, 8192)],
                         ids=["bf16", "f32"])
def test_large_transposed_floats_match_the_contiguous_path(gpu, elem, rows, cols):
    """A transposed float tensor of 192 MiB (grids of thousands of workgroups, offsets beyond
    32 bits in bytes): codes, scales and dequantized values must equal what the contiguous
    kernels, checked against the oracle elsewhere, give for the same logical tensor."""
    transposed_against_contiguous(gpu, elem, rows, cols, ("q4s_block32", "q8s_tensor", "e4m3_native_block32"))


@pytest.mark.parametrize("elem,rows,cols,names", [
    (ElemType.BF16, 4104, 32864, ("q4s_block32", "e2m1_block32", "q2s_block32", "e5m2_native_tensor")),
    (ElemType.F16, 2056, 32832, ("q8s_block32", "q4s_block64", "e4m3_native_block32")),
    (ElemType.F32, 2052, 16416, ("q4s_block32", "q8s_block32")),
    (ElemType.BF16, 4096, 65536, ("q2s_block32",)),
], ids=["bf16", "f16", "f32", "bf16_2bit"])
def test_transposed_tiles_with_ragged_edges_match_the_contiguous_path(gpu, elem, rows, cols, names):
    """Transposed float tensors of thousands of 64 x 256-byte tiles whose last tiles are cut short along both
    axes (the sizes at which whole tiles go through shared memory), against the contiguous kernels."""
    transposed_against_contiguous(gpu, elem, rows, cols, names)


@pytest.mark.parametrize("elem,rows,cols,names", [
    (ElemType.BF16, 4128, 8640, ("q4s_block96", "q8s_block96", "q8s_block160", "q2s_block192")),
    (ElemType.F32, 2064, 8640, ("q4s_block96", "q8s_block160")),
], ids=["bf16", "f32"])
def test_large_transposed_floats_with_blocks_that_straddle_tiles(gpu, elem, rows, cols, names):
    """Blocks of 96, 160 and 192 columns on transposed tensors of more than a thousand tiles: these extents do not
    divide the 128 / 256 / 512 columns of a tile, so a block may start in one tile and end in the next.  out_scale
    (given scales) and the codes must equal the contiguous path's."""
    transposed_against_contiguous(gpu, elem, rows, cols, names)


def transposed_against_contiguous(gpu, elem, rows, cols, names):
    import torch

    client = ComputeClient.current()
    tdt = {ElemType.F32: torch.float32, ElemType.BF16: torch.bfloat16, ElemType.F16: torch.float16}[elem]
    eb = 4 if elem == ElemType.F32 else 2
    g = torch.Generator(device="cuda")
    g.manual_seed(rows + int(elem))
    x = torch.randn((rows, cols), generator=g, device="cuda", dtype=torch.float32).mul_(0.05).to(tdt)
    x[5, 7] = -0.0
    xt = x.t().contiguous()                      # memory [cols, rows]
    h = TensorHandleRef.from_torch
    h_x = h(x)
    h_xt = TensorHandleRef(h(xt).handle, (rows, cols), (1, rows), eb)
    for name in names:
        scheme = LARGE_TRANSPOSED_SCHEMES[name]
        print(name, elem.name, rows, cols, flush=True)
        native = scheme.store == QuantStore.Native
        pshape = scheme.packed_shape((rows, cols)) if not native else (rows, cols)
        sshape = scheme.scales_shape((rows, cols))
        ws, nbytes = gpu.workspace(scheme, rows * cols)
        outs = []
        for hx in (h_x, h_xt):
            codes = torch.full(pshape, 0x5A, dtype=torch.uint8 if native else torch.int32, device="cuda")
            scales = torch.zeros(sshape, dtype=torch.float32, device="cuda")
            qz.launch_dynamic(client, hx, h(codes), h(scales), scheme, elem, ws.data_ptr(), nbytes)
            outs.append((codes, scales))
        torch.cuda.synchronize()
        assert torch.equal(outs[0][0], outs[1][0]), (name, "codes")
        assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32)), (name, "scales")
        # given scales (the launch_ref form), transposed input
        codes2 = torch.zeros_like(outs[0][0])
        os2 = torch.zeros_like(outs[0][1])
        s_in = outs[0][1].to(tdt)
        qz.launch_ref(client, h_xt, h(codes2), h(s_in), h(os2), scheme, elem)
        codes3 = torch.zeros_like(outs[0][0])
        os3 = torch.zeros_like(outs[0][1])
        qz.launch_ref(client, h_x, h(codes3), h(s_in), h(os3), scheme, elem)
        torch.cuda.synchronize()
        assert torch.equal(codes2, codes3), (name, "codes, given scales")
        assert torch.equal(os2.view(torch.int32), os3.view(torch.int32)), (name, "out_scale, given scales")
        # dequantize into a transposed and into a contiguous tensor
        y = torch.empty_like(x)
        yt = torch.empty_like(xt)
        dq.launch_ref(client, h(outs[0][0]), h(y), h(outs[0][1]), scheme, elem)
        dq.launch_ref(client, h(outs[0][0]), TensorHandleRef(h(yt).handle, (rows, cols), (1, rows), eb), h(outs[0][1]),
                      scheme, elem)
        torch.cuda.synchronize()
        bits = torch.int32 if elem == ElemType.F32 else torch.int16
        assert torch.equal(yt.t().contiguous().view(bits), y.view(bits)), (name, "dequantize")
        del outs, codes2, codes3, y, yt


def test_more_pitched_rows_than_one_grid_dimension_holds(gpu):
    """70000 pitched rows: the row index of the streaming kernels spills from the grid's y into z.
    Codes, scales and dequantized values must equal those of the contiguous copy."""
    import torch

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    rows, cols, pad = 70000, 8192, 64
    scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block([32]))
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    buf = torch.empty((rows, cols + pad), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, rows, 10000):
        buf[r0:r0 + 10000] = torch.randn((min(10000, rows - r0), cols + pad), generator=g, device="cuda").mul_(0.1).to(torch.bfloat16)
    xc = buf[:, :cols].contiguous()
    hp = TensorHandleRef(h(buf).handle, (rows, cols), (cols + pad, 1), 2)
    outs = []
    for hx in (h(xc), hp):
        codes = torch.zeros((rows, cols // 8), dtype=torch.int32, device="cuda")
        scales = torch.zeros((rows, cols // 32), dtype=torch.float32, device="cuda")
        qz.launch_dynamic(client, hx, h(codes), h(scales), scheme, ElemType.BF16)
        outs.append((codes, scales))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    y = torch.empty_like(xc)
    dq.launch_ref(client, h(outs[0][0]), h(y), h(outs[0][1]), scheme, ElemType.BF16)
    ybuf = torch.full_like(buf, 7.0)
    dq.launch_ref(client, h(outs[0][0]), TensorHandleRef(h(ybuf).handle, (rows, cols), (cols + pad, 1), 2), h(outs[0][1]),
                  scheme, ElemType.BF16)
    torch.cuda.synchronize()
    assert torch.equal(ybuf[:, :cols].contiguous().view(torch.int16), y.view(torch.int16))
    assert bool((ybuf[:, cols:] == 7.0).all())


@pytest.mark.parametrize("cols", [64, 16384], ids=["short_rows", "long_rows"])
def test_broadcast_rows_read_like_their_copies(gpu, cols):
    """A float input whose rows are one row repeated (row stride 0) quantizes like its materialised copy."""
    import torch

    client = ComputeClient.current()
    h = TensorHandleRef.from_torch
    rows = 6
    scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([32]))
    g = torch.Generator(device="cuda")
    g.manual_seed(cols)
    row = torch.randn((1, cols), generator=g, device="cuda").to(torch.bfloat16)
    full = row.expand(rows, cols).contiguous()
    outs = []
    for hx in (h(full), TensorHandleRef(h(row).handle, (rows, cols), (0, 1), 2)):
        codes = torch.zeros((rows, cols // 4), dtype=torch.int32, device="cuda")
        scales = torch.zeros((rows, cols // 32), dtype=torch.float32, device="cuda")
        qz.launch_dynamic(client, hx, h(codes), h(scales), scheme, ElemType.BF16)
        in_scales = torch.zeros((rows, cols // 32), dtype=torch.bfloat16, device="cuda")
        qz.compute_scales(client, hx, h(in_scales), scheme, ElemType.BF16)
        codes2 = torch.zeros_like(codes)
        scales2 = torch.zeros_like(scales)
        qz.launch_ref(client, hx, h(codes2), h(in_scales), h(scales2), scheme, ElemType.BF16)
        outs.append((codes, scales, codes2, scales2))
    torch.cuda.synchronize()
    for a, b in zip(outs[0], outs[1]):
        assert torch.equal(a, b)
    assert torch.equal(outs[0][0], outs[0][2])


LARGE_VIEWS = {
    # a [4, 3584, 8192] slice of a [4, 4096, 8256] buffer: rows in groups with a pitch of their own
    "sliced_batches": ((4, 3584, 8192), (4, 4096, 8256), (4096 * 8256, 8256, 1)),
    # [batch, heads, positions, head dimension] out of [batch, positions, heads, head dimension]
    "permuted_heads": ((8, 32, 2048, 128), (8, 2048, 32, 128), (2048 * 32 * 128, 128, 32 * 128, 1)),
    # short pitched rows
    "short_pitched_rows": ((65536, 512), (65536, 576), (576, 1)),
}


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(LARGE_VIEWS))
@pytest.mark.parametrize("elem", [ElemType.BF16, ElemType.F32], ids=lambda e: e.name)
def test_large_strided_views_match_the_contiguous_path(gpu, elem, case):
    """Strided views with a contiguous last dimension at sizes of thousands of workgroups: codes, scales and
    dequantized values must equal what the contiguous kernels, checked against the oracle elsewhere, give for
    a contiguous copy; what the view does not cover stays as it was."""
    import torch

    client = ComputeClient.current()
    tdt = torch.float32 if elem == ElemType.F32 else torch.bfloat16
    eb = 4 if elem == ElemType.F32 else 2
    shape, bufshape, strides = LARGE_VIEWS[case]
    g = torch.Generator(device="cuda")
    g.manual_seed(77 + int(elem))
    buf = torch.randn(bufshape, generator=g, device="cuda", dtype=torch.float32).mul_(0.05).to(tdt)
    x = torch.as_strided(buf, shape, strides).contiguous()
    h = TensorHandleRef.from_torch
    strided = lambda t: TensorHandleRef(h(t).handle, shape, strides, eb)
    for name, scheme in (("e2m1_block32", QuantScheme.default().with_value(QuantValue.E2M1).with_level(QuantLevel.block([32]))),
                         ("q8s_tensor", QuantScheme.default().with_value(QuantValue.Q8S)),
                         ("e4m3_native_block64", QuantScheme.default().with_value(QuantValue.E4M3)
                          .with_store(QuantStore.Native).with_level(QuantLevel.block([64])))):
        print(case, name, elem.name, flush=True)
        native = scheme.store == QuantStore.Native
        pshape = scheme.packed_shape(shape) if not native else shape
        sshape = scheme.scales_shape(shape)
        ws, nbytes = gpu.workspace(scheme, x.numel())
        outs = []
        for hx in (h(x), strided(buf)):
            codes = torch.full(pshape, 0x5A, dtype=torch.uint8 if native else torch.int32, device="cuda")
            scales = torch.zeros(sshape, dtype=torch.float32, device="cuda")
            qz.launch_dynamic(client, hx, h(codes), h(scales), scheme, elem, ws.data_ptr(), nbytes)
            outs.append((codes, scales))
        torch.cuda.synchronize()
        assert torch.equal(outs[0][0], outs[1][0]), (name, "codes")
        assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32)), (name, "scales")
        bits = torch.int16 if eb == 2 else torch.int32
        # block scales from the strided tensor, then quantize with them given
        if scheme.level.block_size is not None:
            s_in = [torch.zeros(sshape, dtype=tdt, device="cuda") for _ in range(2)]
            qz.compute_scales(client, h(x), h(s_in[0]), scheme, elem)
            qz.compute_scales(client, strided(buf), h(s_in[1]), scheme, elem)
            torch.cuda.synchronize()
            assert torch.equal(s_in[0].view(bits), s_in[1].view(bits)), (name, "compute_scales")
        else:
            s_in = [outs[0][1].to(tdt)] * 2
        codes2, os2 = torch.zeros_like(outs[0][0]), torch.zeros_like(outs[0][1])
        qz.launch_ref(client, strided(buf), h(codes2), h(s_in[1]), h(os2), scheme, elem)
        codes3, os3 = torch.zeros_like(outs[0][0]), torch.zeros_like(outs[0][1])
        qz.launch_ref(client, h(x), h(codes3), h(s_in[0]), h(os3), scheme, elem)
        torch.cuda.synchronize()
        assert torch.equal(codes2, codes3), (name, "codes, given scales")
        assert torch.equal(os2.view(torch.int32), os3.view(torch.int32)), (name, "out_scale, given scales")
        # dequantize into a contiguous tensor and into the view of a buffer full of a sentinel
        y = torch.empty_like(x)
        ybuf = torch.full(bufshape, 3.0, dtype=tdt, device="cuda")
        dq.launch_ref(client, h(outs[0][0]), h(y), h(outs[0][1]), scheme, elem)
        dq.launch_ref(client, h(outs[0][0]), strided(ybuf), h(outs[0][1]), scheme, elem)
        torch.cuda.synchronize()
        yv = torch.as_strided(ybuf, shape, strides)
        assert torch.equal(yv.contiguous().view(bits), y.view(bits)), (name, "dequantized")
        covered = torch.zeros(bufshape, dtype=torch.bool, device="cuda")
        torch.as_strided(covered, shape, strides).fill_(True)
        assert bool((ybuf[~covered] == 3.0).all()), (name, "wrote outside the view")
        del outs, codes2, codes3, os2, os3, y, ybuf, yv, covered
