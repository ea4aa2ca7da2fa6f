"""cq_plan_kind: which kernel family a call would run on.  Nothing is launched and no pointer is
dereferenced, so this runs without a GPU.  Every BASELINE configuration must land on the streaming kernels,
and every layout the design names must land on the family the design claims for it."""
import pytest

from cubek_amd import ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue, TensorHandleRef, _ffi

BASE = 0x7F0000000000  # 4 KiB aligned fake device addresses, far apart
F32, BF16 = ElemType.F32, ElemType.BF16


def t(shape, elem_size, strides=None, offset=0, slot=0):
    if strides is None:
        strides, acc = [], 1
        for n in reversed(shape):
            strides.append(acc)
            acc *= n
        strides = tuple(reversed(strides))
    return TensorHandleRef(BASE + slot * (1 << 36) + offset, tuple(shape), tuple(strides), elem_size)


def kinds(scheme, elem, shape, f_strides=None, v_strides=None, s_strides=None, f_offset=0, ops=None):
    esz = 4 if elem == F32 else 2
    floats = t(shape, esz, f_strides, f_offset, 0)
    values = t(scheme.packed_shape(shape), 4 if scheme.store == QuantStore.U32 else 1, v_strides, 0, 1)
    sshape = scheme.scales_shape(shape)
    psz = 4 if scheme.param == QuantParam.F32 else 2
    scale_in = t(sshape, esz, s_strides, 0, 2)        # typed like the input
    params = t(sshape, psz, s_strides, 0, 3)          # typed scheme.param
    out = {}
    for name, op, sc, osc in (("quantize", _ffi.OP_QUANTIZE, scale_in, params),
                              ("dynamic", _ffi.OP_QUANTIZE_DYNAMIC, None, params),
                              ("dequantize", _ffi.OP_DEQUANTIZE, params, None),
                              ("scales", _ffi.OP_COMPUTE_SCALES, scale_in, None)):
        if ops is None or name in ops:
            out[name] = _ffi.plan_kind(op, floats, values, sc, osc, scheme, elem)
    return out


def scheme_of(value, block=None, store=QuantStore.U32, param=QuantParam.F32):
    level = QuantLevel.Tensor if block is None else QuantLevel.block(block)
    return QuantScheme.default().with_value(value).with_level(level).with_store(store).with_param(param)


@pytest.mark.parametrize("name,elem,value,block,shape", [
    ("cfg1", F32, QuantValue.Q8S, None, (1024, 1024)),
    ("cfg2", BF16, QuantValue.Q8S, [32], (4096, 4096)),
    ("cfg3", BF16, QuantValue.Q4S, [32], (14336, 4096)),
    ("cfg4", F32, QuantValue.Q2S, [64], (8192, 8192)),
    ("cfg5", BF16, QuantValue.E2M1, [32], (28672, 8192)),
])
def test_baseline_configurations_take_the_streaming_kernels(name, elem, value, block, shape):
    got = kinds(scheme_of(value, block), elem, shape)
    assert got == {"quantize": "flat", "dynamic": "flat", "dequantize": "flat", "scales": "flat"}, name


def test_layouts_land_on_the_family_the_design_claims():
    e2m1 = scheme_of(QuantValue.E2M1, [32])
    rows, cols = 28672, 8192
    # pitched rows of whole 4 KiB steps: the flat kernels over row steps
    got = kinds(e2m1, BF16, (rows, cols), f_strides=(cols + 64, 1))
    assert got == {"quantize": "flat_rows", "dynamic": "flat_rows", "dequantize": "flat_rows", "scales": "flat_rows"}
    # ragged pitched rows (576 chunks = 2.25 steps), short rows: lane by lane
    assert set(kinds(e2m1, BF16, (32768, 4608), f_strides=(4672, 1)).values()) == {"flat_lanes"}
    assert set(kinds(e2m1, BF16, (262144, 256), f_strides=(320, 1)).values()) == {"flat_lanes"}
    # parameters typed like the tensor (bf16 scales of a bf16 tensor): whole tiles on a contiguous run; any other
    # 16-bit parameter type, and pitched rows, lane by lane (scale production has no stored parameters)
    got = kinds(scheme_of(QuantValue.E2M1, [32], param=QuantParam.BF16), BF16, (rows, cols))
    assert got == {"quantize": "flat", "dynamic": "flat", "dequantize": "flat", "scales": "flat"}
    got = kinds(scheme_of(QuantValue.E2M1, [32], param=QuantParam.F16), BF16, (rows, cols))
    assert got == {"quantize": "flat_lanes", "dynamic": "flat_lanes", "dequantize": "flat_lanes", "scales": "flat"}
    got = kinds(scheme_of(QuantValue.E2M1, [32], param=QuantParam.BF16), BF16, (rows, cols), f_strides=(cols + 64, 1))
    assert got == {"quantize": "flat_lanes", "dynamic": "flat_lanes", "dequantize": "flat_lanes", "scales": "flat_rows"}
    # attention layout: [batch, heads, positions, head dimension] view of a [batch, positions, heads, head dimension] buffer
    nb, nh, ns, nd = 8, 32, 4096, 128
    got = kinds(e2m1, BF16, (nb, nh, ns, nd), f_strides=(ns * nh * nd, nd, nh * nd, 1))
    assert set(got.values()) == {"flat_lanes"}
    # a tensor too small for a whole tile
    assert kinds(e2m1, BF16, (4, 64), ops=("dynamic",)) == {"dynamic": "flat_lanes"}
    # 128 x 128 weight blocks, e4m3 bytes: fused block kernel; given scales: the flat kernels over row steps
    blocks = scheme_of(QuantValue.E4M3, [128, 128], store=QuantStore.Native)
    got = kinds(blocks, BF16, (rows, cols))
    assert got == {"quantize": "flat_rows", "dynamic": "blocks", "dequantize": "flat_rows", "scales": "rows"}
    # transposed float tensor
    got = kinds(e2m1, BF16, (rows, cols), f_strides=(1, rows))
    assert got == {"quantize": "transposed", "dynamic": "transposed", "dequantize": "transposed", "scales": "transposed"}
    # blocks that are not a power-of-two number of lanes: quantize stages its floats through LDS so that a lane holds
    # a whole piece of its block; dequantize (and quantize on pitched rows) runs lane by lane and divides by the block
    got = kinds(scheme_of(QuantValue.Q4S, [24]), BF16, (8192, 8184))
    assert got == {"quantize": "staged", "dynamic": "staged", "dequantize": "flat_lanes", "scales": "rows"}
    # ... on pitched rows the fused quantize stays with the block kernel
    got = kinds(scheme_of(QuantValue.Q4S, [24]), BF16, (8192, 8184), f_strides=(8192, 1))
    assert got == {"quantize": "flat_lanes", "dynamic": "blocks", "dequantize": "flat_lanes", "scales": "rows"}
    # scales stored column-major: tiles of 32 rows whose scales pass through LDS
    got = kinds(e2m1, BF16, (8192, 8192), s_strides=(1, 8192), ops=("quantize", "dynamic", "dequantize"))
    assert got == {"quantize": "staged", "dynamic": "staged", "dequantize": "staged"}
    # ... also on pitched rows; 2-D blocks under such scales stay with the row kernels
    got = kinds(e2m1, BF16, (8192, 8192), f_strides=(8256, 1), s_strides=(1, 8192), ops=("quantize", "dynamic", "dequantize"))
    assert got == {"quantize": "staged", "dynamic": "staged", "dequantize": "staged"}
    got = kinds(scheme_of(QuantValue.E2M1, [4, 32]), BF16, (8192, 8192), s_strides=(1, 2048), ops=("quantize", "dequantize"))
    assert got == {"quantize": "rows", "dequantize": "rows"}


def gemv_kind(scheme, elem, rows, cols, pitch=None, s_strides=None, x_offset=0):
    esz = 4 if elem == F32 else 2
    wpr = cols // scheme.num_quants()
    values = t((rows, wpr), 4, (pitch or wpr, 1), 0, 1)
    sshape = scheme.scales_shape((rows, cols))
    params = t(sshape, 4 if scheme.param == QuantParam.F32 else 2, s_strides, 0, 3)
    return _ffi.plan_kind(_ffi.OP_GEMV, t((cols,), esz, None, x_offset, 0), values, params, t((rows,), esz, None, 0, 2), scheme, elem)


def test_matrix_vector_products_that_stream():
    F16 = ElemType.F16
    # configuration 3's weights and the other shapes of the benchmark
    for rows, cols in ((14336, 4096), (4096, 14336), (28672, 8192), (4096, 11008), (8192, 28672)):
        assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), BF16, rows, cols) == "flat", (rows, cols)
    # 2-, 4- and 8-bit codes, larger blocks, scales typed like x, blocks over rows, one scale per tensor, pitched rows
    assert gemv_kind(scheme_of(QuantValue.Q4S, [128], param=QuantParam.F16), F16, 4096, 4096) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q4F, [64], param=QuantParam.BF16), BF16, 4096, 4096, pitch=520) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q8S, [16]), BF16, 100, 2064) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q2S, [64]), F16, 100, 4160) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q8S, [128, 128]), BF16, 256, 1024) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q4S, None), BF16, 64, 32768) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), BF16, 64, 4096, s_strides=(1, 64)) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), BF16, 64, 53248) == "flat"  # rows longer than the LDS holds of x
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32], param=QuantParam.F16), BF16, 64, 4096) == "flat"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), F32, 64, 4096) == "flat"  # x in f32 (with f32 scales)
    # the general kernel: f32 x with 16-bit scales, blocks narrower than 16 bytes of codes or not a power of two
    # of them, words or x off 16-byte boundaries
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32], param=QuantParam.F16), F32, 64, 4096) == "rows"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [16]), BF16, 64, 4096) == "rows"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [96]), BF16, 64, 4032) == "rows"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), BF16, 64, 4096, pitch=513) == "rows"
    assert gemv_kind(scheme_of(QuantValue.Q4S, [32]), BF16, 64, 4096, x_offset=2) == "rows"


def test_matrix_vector_product_with_several_right_hand_sides():
    scheme = scheme_of(QuantValue.Q4S, [32])
    rows, cols = 512, 4096
    values, params = t((rows, cols // 8), 4, None, 0, 1), t((rows, cols // 32), 4, None, 0, 3)
    x, y = t((5, cols), 2, None, 0, 0), t((5, rows), 2, None, 0, 2)
    assert _ffi.plan_kind(_ffi.OP_GEMV, x, values, params, y, scheme, BF16) == "flat"
    with pytest.raises(_ffi.QuantError) as e:  # as many rows of y as of x
        _ffi.plan_kind(_ffi.OP_GEMV, x, values, params, t((4, rows), 2, None, 0, 2), scheme, BF16)
    assert e.value.status == _ffi.ERR_SHAPE_MISMATCH
    with pytest.raises(_ffi.QuantError) as e:  # a vector against a batch
        _ffi.plan_kind(_ffi.OP_GEMV, x, values, params, t((rows,), 2, None, 0, 2), scheme, BF16)
    assert e.value.status == _ffi.ERR_SHAPE_MISMATCH


def test_slow_paths_are_reported():
    e2m1 = scheme_of(QuantValue.E2M1, [32])
    # rows that start on odd multiples of 2 bytes: lane by lane (16-byte accesses off their alignment); rows that are
    # not whole words of codes stay per element
    got = kinds(e2m1, BF16, (8192, 8192), f_strides=(8193, 1), ops=("quantize", "dynamic", "dequantize"))
    assert set(got.values()) == {"flat_lanes"}
    got = kinds(scheme_of(QuantValue.Q8S), BF16, (8192, 8196), f_strides=(8197, 1), ops=("quantize", "dynamic", "dequantize"))
    assert set(got.values()) == {"per_element"}
    # a quantized tensor whose last dimension is not the contiguous one: words of the u32 store pass through LDS
    # (the staged tiles); bytes of the native store go one thread per element
    got = kinds(e2m1, BF16, (4096, 4096), v_strides=(1, 4096), ops=("quantize", "dynamic", "dequantize"))
    assert set(got.values()) == {"staged"}
    native = scheme_of(QuantValue.E4M3, [32], store=QuantStore.Native)
    got = kinds(native, BF16, (4096, 4096), v_strides=(1, 4096), ops=("quantize", "dequantize"))
    assert set(got.values()) == {"per_element"}
    # E4M3 / E5M2 in the u32 store (codes wrap their 8-bit field): quantize lane by lane, streaming dequantize; under
    # layouts of the other families (a transposed float tensor) per element
    for value in (QuantValue.E4M3, QuantValue.E5M2):
        got = kinds(scheme_of(value, [32]), BF16, (4096, 4096), ops=("quantize", "dynamic", "dequantize"))
        assert got == {"quantize": "flat_lanes", "dynamic": "flat_lanes", "dequantize": "flat"}
        got = kinds(scheme_of(value), F32, (4096, 4096), f_strides=(4160, 1), ops=("quantize", "dynamic", "dequantize"))
        assert got == {"quantize": "flat_lanes", "dynamic": "flat_lanes", "dequantize": "flat_rows"}
        got = kinds(scheme_of(value, [32]), BF16, (4096, 4096), f_strides=(1, 4096), ops=("quantize", "dynamic", "dequantize"))
        assert got == {"quantize": "per_element", "dynamic": "per_element", "dequantize": "transposed"}
    # blocks smaller than a packed word on dequantize
    got = kinds(scheme_of(QuantValue.Q8S, [2]), BF16, (4096, 4096), ops=("dequantize",))
    assert got == {"dequantize": "per_element"}


def test_plan_kind_validates_like_the_entry_points():
    s = scheme_of(QuantValue.Q8S, [32])
    with pytest.raises(_ffi.QuantError) as e:
        _ffi.plan_kind(_ffi.OP_QUANTIZE, t((8, 64), 4), t((8, 15), 4), t((8, 2), 4), t((8, 2), 4), s, F32)
    assert e.value.status == _ffi.ERR_SHAPE_MISMATCH
    bad = scheme_of(QuantValue.Q8S, [2])
    with pytest.raises(_ffi.QuantError) as e:
        _ffi.plan_kind(_ffi.OP_QUANTIZE, t((8, 64), 4), t((8, 16), 4), t((8, 32), 4), t((8, 32), 4), bad, F32)
    assert e.value.status == _ffi.ERR_BLOCK_NOT_DIVISIBLE
    # an empty tensor launches nothing
    assert _ffi.plan_kind(_ffi.OP_DEQUANTIZE, t((0, 64), 4), t((0, 16), 4), t((0, 2), 4), None, s, F32) == "none"


def test_extension_value_runs_on_the_streaming_kernels():
    """E2M1_OCP (no counterpart in the reference) takes the same families as the native e2m1 encoding, in both stores."""
    for store in (QuantStore.U32, QuantStore.Native):
        got = kinds(scheme_of(QuantValue.E2M1_OCP, [32], store=store), BF16, (28672, 8192))
        assert set(got.values()) == {"flat"}, (store, got)
