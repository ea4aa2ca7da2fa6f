"""cq_reduce_max_abs (through the C ABI) against the CPU oracle: every kernel
variant (lane groups, wave per row, sliced rows, columns, sliced columns,
strided fallback), bit for bit, plus the reference's error cases."""
import numpy as np
import pytest

from cubek_amd import ComputeClient, ElemType, QuantError, TensorHandleRef, _ffi
from cubek_amd import reduce as cq_reduce

pytestmark = pytest.mark.gpu
ELEMS = [ElemType.F32, ElemType.BF16, ElemType.F16]


def run(torch, gpu, x_np, elem, shape, axis, use_workspace=True, in_strides=None, out_strides=None):
    dx = gpu.to_dev(x_np.reshape(-1))
    out_shape = tuple(1 if d == axis else s for d, s in enumerate(shape))
    n_out = int(np.prod(out_shape))
    hin = gpu.handle(dx, shape, in_strides if in_strides is not None else gpu.contiguous_strides(shape))
    ostr = out_strides if out_strides is not None else gpu.contiguous_strides(out_shape)
    reach = 1 + sum((n - 1) * st for n, st in zip(out_shape, ostr))
    dout = torch.zeros(max(reach, 1), dtype=gpu.storage_dtype(elem), device="cuda")
    hout = gpu.handle(dout, out_shape, ostr)
    nbytes = cq_reduce.workspace_bytes(hin, axis, elem) if use_workspace else 0
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    cq_reduce.max_abs(ComputeClient.current(), hin, hout, axis, elem, ws.data_ptr() if nbytes else 0, nbytes)
    torch.cuda.synchronize()
    return gpu.to_host(dout), n_out


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_reduce_contiguous_all_paths(gpu, oracle, elem):
    import torch

    rng = np.random.default_rng(int(elem) + 7)
    cases = [
        ((64, 32), 1), ((300, 8), 1), ((33, 512), 1),          # lane groups (1..64 chunks per row)
        ((40, 4096), 1), ((3, 100000), 1), ((1, 1 << 20), 1),  # wave per row, sliced rows
        ((5000, 1000), 1),                                      # odd chunk count per row
        ((512, 256), 0), ((4096, 64), 0), ((20000, 16), 0),     # columns, sliced columns
        ((6, 50, 128), 1), ((4, 3, 8, 64), 2), ((2, 7, 24), 0),
        ((10, 7), 1), ((10, 7), 0), ((5, 3, 2), 1),             # not chunk-aligned: fallback
        ((8, 1, 64), 1),
        ((100000, 64), 0), ((3000, 24), 0), ((2, 4000, 40), 1), ((1, 300, 1024), 1),  # tiles of chunk columns
        ((3, 600, 520), 1), ((70000, 8), 0), ((5, 9, 16), 1),
        ((300, 1001), 1), ((1001, 300), 0), ((9, 4097), 1),     # long odd axes: wave per output
    ]
    for shape, axis in cases:
        x32 = rng.normal(0, 2, shape).astype(np.float32)
        x32[rng.random(shape) < 0.01] = np.nan
        x = oracle.to_bits(x32, elem)
        want = oracle.reduce_max_abs(x, elem, shape, axis).reshape(-1)
        for use_ws in (True, False):
            got, n_out = run(torch, gpu, x, elem, shape, axis, use_workspace=use_ws)
            assert np.array_equal(got[:n_out].view(np.uint8), want.view(np.uint8)), (shape, axis, use_ws)


def test_reduce_strided_views_and_errors(gpu, oracle):
    import torch

    rng = np.random.default_rng(11)
    base = rng.normal(0, 1, (48, 40)).astype(np.float32)
    # transposed view [40, 48] (strides 1, 40), both axes; output written with a padded stride
    for axis in (0, 1):
        want = oracle.reduce_max_abs(base.reshape(-1), ElemType.F32, (40, 48), axis, in_strides=(1, 40)).reshape(-1)
        out_shape = (1, 48) if axis == 0 else (40, 1)
        ostr = (0, 2) if axis == 0 else (3, 0)
        got, n_out = run(torch, gpu, base, ElemType.F32, (40, 48), axis, in_strides=(1, 40), out_strides=ostr)
        step = 2 if axis == 0 else 3
        assert np.array_equal(got[::step][:n_out], want)
    x = torch.zeros((4, 8), dtype=torch.float32, device="cuda")
    h = TensorHandleRef.from_torch
    client = ComputeClient.current()

    def status(fn):
        with pytest.raises(QuantError) as e:
            fn()
        return e.value.status

    good = torch.zeros((4, 1), dtype=torch.float32, device="cuda")
    bad = torch.zeros((4, 2), dtype=torch.float32, device="cuda")
    assert status(lambda: cq_reduce.max_abs(client, h(x), h(good), 2, ElemType.F32)) == _ffi.ERR_INVALID_AXIS
    assert status(lambda: cq_reduce.max_abs(client, h(x), h(bad), 1, ElemType.F32)) == _ffi.ERR_SHAPE_MISMATCH
    assert status(lambda: cq_reduce.max_abs(client, h(x), h(good), 1, ElemType.BF16)) == _ffi.ERR_SHAPE_MISMATCH


def test_reduce_feeds_per_channel_scales(gpu, oracle):
    """The use the reference's callers make of MaxAbs: per-row abs-max -> scale by the
    test's rule -> quantize with those scales.  A [rows, 128] tensor with block [128]
    has exactly one block per row, so the two routes must agree."""
    import torch
    from cubek_amd import QuantLevel, QuantScheme, QuantValue

    rng = np.random.default_rng(5)
    shape = (256, 128)
    x = rng.normal(0, 1, shape).astype(np.float32)
    amax, _ = run(torch, gpu, x, ElemType.F32, shape, 1)
    scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_level(QuantLevel.block([128]))
    s_blocks = gpu.compute_scales(x, ElemType.F32, shape, scheme).reshape(-1)
    assert np.array_equal((2 * amax[:256]) / np.float32(254.0), s_blocks)


# shape / strides / axis of the reference's reduce suite
# (crates/cubek-reduce/tests/suite/mod.rs:134-230); it runs Sum/Mean/Prod/ArgMax/ArgMin
# over this matrix, here it is MaxAbs.
REFERENCE_MATRIX = [
    ((22,), (1,), 0), ((1024,), (1,), 0),
    ((4, 8), (8, 1), 1), ((4, 8), (8, 1), 0),
    ((8, 256), (256, 1), 1), ((8, 256), (256, 1), 0),
    ((16, 16, 16), (1, 256, 16), 0), ((16, 16, 16), (1, 256, 16), 1),
    ((11, 12, 13), (156, 13, 1), 2),
    ((4, 4, 4, 4), (1, 16, 64, 4), 0), ((4, 4, 4, 4), (1, 16, 64, 4), 1),
    ((4, 4, 4, 4), (64, 16, 4, 1), 3),
    ((8, 8), (64, 1), 1), ((8, 8), (64, 1), 0),
    ((4, 32), (0, 1), 0),
]


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_reduce_reference_matrix(gpu, oracle, elem):
    import torch

    rng = np.random.default_rng(int(elem) + 91)
    for shape, strides, axis in REFERENCE_MATRIX:
        reach = 1 + sum((n - 1) * st for n, st in zip(shape, strides))
        x = oracle.to_bits(rng.uniform(-1, 1, reach).astype(np.float32), elem)
        want = oracle.reduce_max_abs(x, elem, shape, axis, in_strides=strides).reshape(-1)
        got, n_out = run(torch, gpu, x, elem, shape, axis, in_strides=strides)
        assert np.array_equal(got[:n_out].view(np.uint8), want.view(np.uint8)), (shape, strides, axis)


@pytest.mark.parametrize("seed", range(8))
def test_reduce_random_shapes_axes_and_layouts(gpu, oracle, seed):
    """Seeded random rank / shape / axis / strides / float type, with and without workspace."""
    import torch

    rng = np.random.default_rng(1000 + seed)
    for _ in range(12):
        rank = int(rng.integers(1, 5))
        shape = [int(rng.choice([1, 2, 3, 5, 8, 16, 24, 33, 64, 100, 256, 1000, 4096])) for _ in range(rank)]
        while int(np.prod(shape)) > (1 << 20):
            shape[int(np.argmax(shape))] //= 2
        shape = tuple(shape)
        axis = int(rng.integers(rank))
        elem = ELEMS[int(rng.integers(3))]
        order = list(range(rank))
        kind = int(rng.integers(3))
        if kind == 2:
            rng.shuffle(order)
        strides, acc = [0] * rank, 1
        for i, d in enumerate(reversed(order)):
            strides[d] = acc
            acc *= shape[d] + (4 if kind == 1 and i == 0 else 0)
        reach = 1 + sum((n - 1) * st for n, st in zip(shape, strides))
        x32 = rng.normal(0, 1, reach).astype(np.float32)
        x32[rng.random(reach) < 0.01] = np.nan
        x = oracle.to_bits(x32, elem)
        want = oracle.reduce_max_abs(x, elem, shape, axis, in_strides=strides).reshape(-1)
        for use_ws in (True, False):
            got, n_out = run(torch, gpu, x, elem, shape, axis, use_workspace=use_ws, in_strides=strides)
            assert np.array_equal(got[:n_out].view(np.uint8), want.view(np.uint8)), (shape, strides, axis, elem.name, use_ws)


# shape, input strides (elements): strided inputs whose last dimension is contiguous
ROWWISE_STRIDED = [
    ((96, 4096), (4160, 1)),                                   # pitched rows, long
    ((2048, 64), (72, 1)),                                     # pitched rows, short
    ((300, 1024), (2048, 1)),                                  # every other row
    ((2, 6, 40, 128), (6 * 40 * 128, 128, 6 * 128, 1)),        # heads and positions swapped in memory
    ((3, 5, 2048), (2048, 3 * 2048, 1)),                       # leading dimensions swapped
    ((4, 700, 256), (1024 * 320, 320, 1)),                     # a slice of a larger batch, pitched
    ((1, 9000, 8), (0, 16, 1)),                                # rows of one 16-byte chunk (two for f32) at a pitch
    ((300, 1024), (1030, 1)),                                  # rows that start on multiples of 4 bytes only (bf16 / f16)
    ((5, 64, 256), (64 * 258 + 2, 258, 1)),                    # the same behind a batch dimension
    ((256, 4096), (1, 256)),                                   # a transposed matrix: reduced in the order of its strides
    ((48, 40, 64), (1, 48, 48 * 40)),                          # all dimensions reversed in memory
    ((6, 512, 64), (512 * 64, 1, 512)),                        # last two dimensions swapped in memory
]


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
def test_reduce_strided_inputs_with_contiguous_rows(gpu, oracle, elem):
    """Every axis of pitched, sliced and permuted inputs (the kernels that look up each row or column
    dimension by dimension), with and without the workspace for partial maxima, NaN elements ignored."""
    import torch

    rng = np.random.default_rng(4242 + int(elem))
    for shape, strides in ROWWISE_STRIDED:
        reach = 1 + sum((n - 1) * st for n, st in zip(shape, strides))
        x32 = rng.normal(0, 1, reach).astype(np.float32)
        x32[rng.random(reach) < 0.01] = np.nan
        x = oracle.to_bits(x32, elem)
        for axis in range(len(shape)):
            want = oracle.reduce_max_abs(x, elem, shape, axis, in_strides=strides).reshape(-1)
            for use_ws in (True, False):
                got, n_out = run(torch, gpu, x, elem, shape, axis, use_workspace=use_ws, in_strides=strides)
                assert np.array_equal(got[:n_out].view(np.uint8), want.view(np.uint8)), (shape, strides, axis, use_ws)


@pytest.mark.parametrize("case", ["permuted_heads", "pitched_rows"])
def test_reduce_large_strided_views_match_their_contiguous_copies(gpu, case):
    """Full-size strided inputs (thousands of workgroups, sliced reductions with a fold) against the
    contiguous kernels, which the other tests check against the oracle, on a contiguous copy."""
    import torch

    from cubek_amd import TensorHandleRef

    shape, bufshape, strides = {
        "permuted_heads": ((8, 32, 2048, 128), (8, 2048, 32, 128), (2048 * 32 * 128, 128, 32 * 128, 1)),
        "pitched_rows": ((14336, 8192), (14336, 8256), (8256, 1)),
    }[case]
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    buf = torch.randn(bufshape, generator=g, device="cuda", dtype=torch.bfloat16)
    buf.view(-1)[::4099] = float("nan")
    x = torch.as_strided(buf, shape, strides).contiguous()
    h = TensorHandleRef.from_torch
    client = ComputeClient.current()
    for axis in range(len(shape)):
        oshape = tuple(1 if d == axis else n for d, n in enumerate(shape))
        outs = []
        for hin in (h(x), TensorHandleRef(h(buf).handle, shape, strides, 2)):
            o = torch.full(oshape, -1.0, device="cuda", dtype=torch.bfloat16)
            nbytes = cq_reduce.workspace_bytes(hin, axis, ElemType.BF16)
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
            cq_reduce.max_abs(client, hin, h(o), axis, ElemType.BF16, ws.data_ptr() if nbytes else 0, nbytes)
            torch.cuda.synchronize()
            outs.append(o)
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)), (case, axis)
        ref = torch.nan_to_num(x.float(), nan=0.0).abs().amax(dim=axis, keepdim=True).to(torch.bfloat16)
        assert torch.equal(outs[1].view(torch.int16), ref.view(torch.int16)), (case, axis, "torch")


def test_reduce_over_an_empty_axis_writes_the_identity(gpu):
    """No elements along the axis: every output is the identity of max-abs, 0."""
    import torch

    for elem in ELEMS:
        dt = gpu.storage_dtype(elem)
        din = torch.zeros(16, dtype=dt, device="cuda")
        dout = torch.ones(32, dtype=dt, device="cuda")   # 1.0f / the bits 0x0001: anything but zero
        hin = gpu.handle(din, (4, 0, 8), (8, 8, 1))
        hout = gpu.handle(dout, (4, 1, 8), (8, 8, 1))
        cq_reduce.max_abs(ComputeClient.current(), hin, hout, 1, elem, 0, 0)
        torch.cuda.synchronize()
        assert not dout.view(torch.uint8).any().item(), elem
