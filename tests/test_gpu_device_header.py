"""include/cubek_quant_device.hpp on the GPU, against the committed exact-rational fixtures (their
expected dequantized bits), never against the library's own dequantize: every function of the header,
three float types, three scale storage types, the packed store and the four native encodings."""
import numpy as np
import pytest

import device_header as dh
import golden_cases as gc
from cubek_amd import ElemType, QuantStore, QuantValue

pytestmark = pytest.mark.gpu

RAMPS = gc.load("ref_ramps.npz")
TYPED = gc.load("typed_small.npz")
NATIVE = gc.load("typed_native.npz")
_NATIVE_ID = {QuantValue.Q8F: 0, QuantValue.Q8S: 0, QuantValue.E4M3: 1, QuantValue.E5M2: 2, QuantValue.E2M1: 3}


def _dev(a):
    import torch

    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def _layout_args(case):
    vshape = case.scheme.packed_shape(case.shape)
    block = [] if case.scheme.level.is_tensor else list(case.scheme.level.block_size.dims)
    strides = case.scale_strides if not case.scheme.level.is_tensor else (0,) * len(case.shape)
    return dh.u64(vshape), len(case.shape), dh.u64(strides), dh.u8(block), len(block)


def _out(case):
    import torch

    n = int(np.prod(case.shape))
    return torch.zeros(n, dtype=torch.float32 if case.elem == ElemType.F32 else torch.int16, device="cuda")


def _bits(t, elem):
    a = t.cpu().numpy()
    return a.view(np.uint32) if elem == ElemType.F32 else a.view(np.uint16)


@pytest.mark.parametrize("case", RAMPS + TYPED, ids=lambda c: c.name)
def test_packed_functions_reproduce_the_fixtures(case):
    """dequantize_symmetric_packed_values (-> _value_at -> _value -> unpack_q, dequantize_symmetric) and, for
    the 16-bit float types, dequantize_symmetric_packed_value_pairs."""
    words, scales = _dev(case.words), _dev(case.out_scale)
    want = case.deq.view(np.uint32) if case.elem == ElemType.F32 else case.deq
    for pairs in ((0,) if case.elem == ElemType.F32 else (0, 1)):
        out = _out(case)
        rc = dh.lib().dh_dequantize_packed(int(case.elem), case.scheme.value.size_bits(), int(case.scheme.param), pairs,
                                           words.data_ptr(), scales.data_ptr(), *_layout_args(case), words.numel(),
                                           out.data_ptr())
        assert rc == 0
        assert np.array_equal(_bits(out, case.elem), want.reshape(-1)), ("pairs" if pairs else "values")


@pytest.mark.parametrize("case", NATIVE, ids=lambda c: c.name)
def test_native_functions_reproduce_the_fixtures(case):
    """dequantize_symmetric_native_values (-> _value -> decode_native) for i8 / e4m3 / e5m2 / e2m1x2 bytes."""
    assert case.scheme.store == QuantStore.Native and case.words.size % 4 == 0
    words, scales = _dev(case.words.view(np.uint32)), _dev(case.out_scale)
    out = _out(case)
    rc = dh.lib().dh_dequantize_native(int(case.elem), _NATIVE_ID[case.scheme.value], int(case.scheme.param),
                                       words.data_ptr(), scales.data_ptr(), *_layout_args(case), words.numel(),
                                       out.data_ptr())
    assert rc == 0
    want = case.deq.view(np.uint32) if case.elem == ElemType.F32 else case.deq
    assert np.array_equal(_bits(out, case.elem), want.reshape(-1))


def test_pairs_equal_values_for_every_word_pattern():
    """The fast path against the plain one over scales of every kind (tiny, huge, negative, zero, NaN-free
    specials) and random words, bf16 and f16, 2 / 4 / 8 bits: identical bits."""
    import torch

    rng = np.random.default_rng(3)
    n_words = 1 << 14
    words = rng.integers(0, 2**32, n_words, dtype=np.uint64).astype(np.uint32)
    words[:256] = np.arange(256, dtype=np.uint32) * 0x01010101  # every byte value in every position
    scales = rng.normal(0, 1, n_words // 8).astype(np.float32)
    scales[:12] = [0.0, -0.0, 1e-38, 1e-30, 3e38, 1e30, -1.5, 65504.0, 6e-8, 2.0 ** -100, 2.0 ** 100, 2.0 ** -14]
    dw, ds = _dev(words), _dev(scales)
    for elem in (ElemType.BF16, ElemType.F16):
        for bits in (2, 4, 8):
            nq = 32 // bits
            block = 8 * nq  # one scale per 8 words
            layout = (dh.u64((n_words,)), 1, dh.u64((1,)), dh.u8((block,)), 1)
            outs = []
            for pairs in (0, 1):
                out = torch.zeros(n_words * nq, dtype=torch.int16, device="cuda")
                assert dh.lib().dh_dequantize_packed(int(elem), bits, 0, pairs, dw.data_ptr(), ds.data_ptr(), *layout,
                                                     n_words, out.data_ptr()) == 0
                outs.append(out.cpu().numpy().view(np.uint16))
            assert np.array_equal(outs[0], outs[1]), (elem.name, bits)


@pytest.mark.parametrize("case", [c for c in NATIVE if c.elem != ElemType.F32 and _NATIVE_ID[c.scheme.value] != 0],
                         ids=lambda c: c.name)
def test_native_pairs_reproduce_the_fixtures(case):
    """dequantize_symmetric_native_value_pairs for e4m3 / e5m2 / e2m1x2 bytes and the 16-bit float types."""
    words, scales = _dev(case.words.view(np.uint32)), _dev(case.out_scale)
    out = _out(case)
    rc = dh.lib().dh_dequantize_native_pairs(int(case.elem), _NATIVE_ID[case.scheme.value], int(case.scheme.param),
                                             words.data_ptr(), scales.data_ptr(), *_layout_args(case), words.numel(),
                                             out.data_ptr())
    assert rc == 0
    assert np.array_equal(_bits(out, case.elem), case.deq.reshape(-1))


def test_native_pairs_equal_values_for_every_word_pattern():
    """The pair form against the plain one over scales of every kind (tiny, huge, negative, zero, infinite, NaN)
    and every byte value in every position (NaN and infinity encodings included), bf16 and f16: identical bits."""
    import torch

    rng = np.random.default_rng(4)
    n_words = 1 << 14
    words = rng.integers(0, 2**32, n_words, dtype=np.uint64).astype(np.uint32)
    words[:256] = np.arange(256, dtype=np.uint32) * 0x01010101
    scales = rng.normal(0, 1, n_words // 8).astype(np.float32)
    # the 256 patterns under an ordinary, a negative and a zero scale; the special scales over random words
    words[256:512], words[512:768] = words[:256], words[:256]
    scales[0:32], scales[32:64], scales[64:96] = 0.37, -1.5, -0.0
    scales[96:110] = [0.0, -0.0, 1e-38, 1e-30, 3e38, 1e30, -1.5, 65504.0, 6e-8, 2.0 ** -100, 2.0 ** 100, 2.0 ** -14,
                      np.inf, np.nan]
    dw, ds = _dev(words), _dev(scales)
    for elem in (ElemType.BF16, ElemType.F16):
        for native in (1, 2, 3):
            per_word = 8 if native == 3 else 4
            stored = (n_words * 4,)  # stored elements: bytes
            block = 8 * per_word     # one scale per 8 words
            layout = (dh.u64(stored), 1, dh.u64((1,)), dh.u8((block,)), 1)
            outs = []
            for fn in (dh.lib().dh_dequantize_native, dh.lib().dh_dequantize_native_pairs):
                out = torch.zeros(n_words * per_word, dtype=torch.int16, device="cuda")
                assert fn(int(elem), native, 0, dw.data_ptr(), ds.data_ptr(), *layout, n_words, out.data_ptr()) == 0
                outs.append(out.cpu().numpy().view(np.uint16))
            assert np.array_equal(outs[0], outs[1]), (elem.name, native)


def test_global_scale_layout_and_device_scales_layout(oracle):
    """GlobalScaleLayout<BR, BC>::to_source_pos(batch, row, col) == the N-D ScalesLayout of the same tensor
    == 'coordinate / block extent' in numpy; and ScalesLayout evaluated on the device."""
    import torch

    L = dh.lib()
    for br, bc, (batches, rows, cols) in ((1, 32, (2, 5, 128)), (1, 24, (1, 7, 96)), (128, 128, (2, 256, 384)),
                                          (3, 16, (3, 9, 64)), (16, 1, (1, 64, 40))):
        srows, scols = rows // br, cols // bc
        strides = (srows * scols + 3, scols + 1, 1)  # padded scales tensor
        out = torch.zeros(batches * rows * cols, dtype=torch.int32, device="cuda")
        assert L.dh_global_scale_pos(br, bc, *strides, batches, rows, cols, out.data_ptr()) == 0
        b, r, c = np.meshgrid(np.arange(batches), np.arange(rows), np.arange(cols), indexing="ij")
        want = b * strides[0] + (r // br) * strides[1] + (c // bc) * strides[2]
        assert np.array_equal(out.cpu().numpy().reshape(batches, rows, cols), want)
        # the N-D layout of the same tensor agrees, on the device
        n = batches * rows * cols
        pos = torch.zeros(n, dtype=torch.int64, device="cuda")
        start = torch.zeros(n, dtype=torch.uint8, device="cuda")
        assert L.dh_scales_layout(dh.u64((batches, rows, cols)), 3, 1, dh.u64(strides), dh.u8((br, bc)), 2, n,
                                  pos.data_ptr(), start.data_ptr()) == 0
        assert np.array_equal(pos.cpu().numpy().reshape(batches, rows, cols), want)
        assert np.array_equal(start.cpu().numpy().reshape(batches, rows, cols).astype(bool), (r % br == 0) & (c % bc == 0))
    out = torch.ones(64, dtype=torch.int32, device="cuda")
    assert L.dh_global_scale_pos(0, 0, 5, 6, 7, 1, 2, 32, out.data_ptr()) == 0 and not out.any()  # per tensor
