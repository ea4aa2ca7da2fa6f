"""The C oracle against (a) the committed exact-rational fixtures, (b) the
reference's own round-trip tolerance on its 24 cases, (c) closed forms and
brute force that a plausible mistake would break."""
import ctypes
from fractions import Fraction

import numpy as np
import pytest
import torch

import golden_cases as gc
from cubek_amd.scheme import (ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore,
                              QuantValue)

RAMPS = gc.load("ref_ramps.npz")
TYPED = gc.load("typed_small.npz")
NATIVE = gc.load("typed_native.npz")


@pytest.mark.parametrize("case", RAMPS + TYPED + NATIVE, ids=lambda c: c.name)
def test_oracle_matches_exact_model(oracle, case):
    words, out_scale = oracle.quantize(case.x, case.elem, case.shape, case.scale, case.scheme,
                                       scale_strides=case.scale_strides)
    assert gc.bits_equal(words, case.words)
    assert gc.bits_equal(out_scale, case.out_scale)
    deq = oracle.dequantize(words, case.shape, out_scale, case.elem, case.scheme,
                            scale_strides=case.scale_strides)
    assert gc.bits_equal(deq, case.deq)


@pytest.mark.parametrize("case", RAMPS, ids=lambda c: c.name)
def test_reference_round_trip_tolerance(oracle, case):
    """|dequant(quant(x)) - x| <= scale/2 * (1+1e-4), the assertion of
    crates/cubek-quant/tests/suite/symmetric.rs:130-140 and :271-283."""
    words, out_scale = oracle.quantize(case.x, case.elem, case.shape, case.scale, case.scheme)
    deq = oracle.dequantize(words, case.shape, out_scale, case.elem, case.scheme)
    x = case.x.reshape(case.shape)
    if case.scheme.level.is_tensor:
        tol = case.scale[0] / 2 * (1 + 1e-4)
    else:
        b = case.scheme.level.block_size.dims[-1]
        tol = np.repeat(case.scale.reshape(case.shape[0], -1), b, axis=1) / 2 * (1 + 1e-4)
    assert deq.shape == x.shape
    assert np.all(np.abs(deq - x) <= tol)


def test_known_answer_q2s_ramp(oracle):
    """32x32 per-tensor Q2S ramp, derivable by hand: scale = 1024/2 = 512,
    x_i = i-512, so x/scale crosses -0.5 at i=256 and +0.5 at i=768, both exact
    ties that round to the even code 0.  Codes: -1 for i<256, 0 for 256..768,
    +1 for i>768; 16 codes per word, code k at bits [2k,2k+2), -1 stored as 0b11."""
    n = 1024
    x = (np.arange(n, dtype=np.float32) - 512).reshape(32, 32)
    scheme = QuantScheme.default().with_value(QuantValue.Q2S)
    words, out_scale = oracle.quantize(x, ElemType.F32, (32, 32), np.array([512.0], np.float32), scheme)
    codes = np.where(np.arange(n) < 256, 3, np.where(np.arange(n) > 768, 1, 0)).astype(np.uint64)
    want = (codes.reshape(-1, 16) << (2 * np.arange(16, dtype=np.uint64))).sum(axis=1).astype(np.uint32)
    assert np.array_equal(words.reshape(-1), want)
    assert want[0] == 0xFFFFFFFF and want[16] == 0 and want[48] == 0x55555554 and want[63] == 0x55555555
    assert out_scale[0] == 512.0


def test_pack_unpack_exhaustive(oracle):
    """Every field value at every position: field i sits at bits [i*b,(i+1)*b),
    negative codes are two's complement, unpack inverts pack."""
    L = oracle.lib()
    for bits in (2, 4, 8):
        nq = 32 // bits
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        for pos in range(nq):
            for v in range(lo, hi + 1):
                codes = (ctypes.c_int32 * 16)(*([0] * 16))
                codes[pos] = v
                w = L.cqo_pack_word(codes, bits)
                assert w == ((v & ((1 << bits) - 1)) << (pos * bits))
                back = (ctypes.c_int32 * 16)()
                L.cqo_unpack_word(w, bits, back)
                assert list(back)[:nq] == [v if i == pos else 0 for i in range(nq)]
        rng = np.random.default_rng(bits)
        for _ in range(200):
            vals = rng.integers(lo, hi + 1, nq)
            codes = (ctypes.c_int32 * 16)(*[int(v) for v in vals], *([0] * (16 - nq)))
            w = L.cqo_pack_word(codes, bits)
            assert w == sum(((int(v) % (1 << bits)) << (i * bits)) for i, v in enumerate(vals))
            back = (ctypes.c_int32 * 16)()
            L.cqo_unpack_word(w, bits, back)
            assert list(back)[:nq] == [int(v) for v in vals]


def test_scale_index_brute_force(oracle):
    """to_source_pos / is_block_start against 'unravel, then divide each
    coordinate by its block extent' on small N-D shapes, with odd strides."""
    rng = np.random.default_rng(11)
    for shape, block in (((4, 8), (4,)), ((4, 8), (2, 4)), ((3, 4, 6), (2, 3)), ((2, 3, 4, 8), (3, 2, 4)),
                         ((5, 6), (5, 2)), ((2, 2, 2, 2, 8), (2, 1, 2, 1, 4)), ((6, 12), (1, 12))):
        scheme = QuantScheme.default().with_level(QuantLevel.block(block))
        blk = (1,) * (len(shape) - len(block)) + tuple(block)
        strides = tuple(int(v) for v in rng.integers(1, 50, len(shape)))
        n = int(np.prod(shape))
        starts = 0
        for e in range(n):
            coords = np.unravel_index(e, shape)
            want = sum((c // b) * s for c, b, s in zip(coords, blk, strides))
            assert oracle.scale_index(scheme, shape, strides, e) == want
            is_start = all(c % b == 0 for c, b in zip(coords, blk))
            assert oracle.is_block_start(scheme, shape, e) == is_start
            starts += is_start
        assert starts == int(np.prod([s // b for s, b in zip(shape, blk)]))
    tensor = QuantScheme.default()
    assert oracle.scale_index(tensor, (4, 8), (0, 0), 17) == 0
    assert oracle.is_block_start(tensor, (4, 8), 0) and not oracle.is_block_start(tensor, (4, 8), 4)


def test_config_shapes_reduce_to_row_col_formula(oracle):
    """For [rows, cols] with a 1-D block B on the last axis the index is r*(cols/B) + c/B."""
    rng = np.random.default_rng(5)
    for rows, cols, B in ((4096, 4096, 32), (14336, 4096, 32), (8192, 8192, 64), (28672, 8192, 32)):
        scheme = QuantScheme.default().with_level(QuantLevel.block([B]))
        strides = (cols // B, 1)
        for e in rng.integers(0, rows * cols, 200):
            e = int(e)
            assert oracle.scale_index(scheme, (rows, cols), strides, e) == (e // cols) * (cols // B) + (e % cols) // B
            assert oracle.is_block_start(scheme, (rows, cols), e) == (e % B == 0)


def test_bf16_arithmetic_matches_torch_cpu(oracle):
    """Library cross-check of the 'f32 op, then one rounding to bf16' model:
    torch's CPU bfloat16 divide / round / clamp / multiply on the same data."""
    rng = np.random.default_rng(17)
    rows, cols, B = 16, 256, 32
    x32 = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x32[rng.random((rows, cols)) < 0.01] *= 50
    xb = oracle.to_bits(x32, ElemType.BF16)
    for value in (QuantValue.Q8S, QuantValue.Q4S, QuantValue.E2M1, QuantValue.Q8F):
        scheme = QuantScheme.default().with_level(QuantLevel.block([B])).with_value(value)
        scales = oracle.compute_scales(xb, ElemType.BF16, (rows, cols), scheme)
        words, out_scale = oracle.quantize(xb, ElemType.BF16, (rows, cols), scales, scheme)
        xt = torch.from_numpy(xb.view(np.int16)).view(torch.bfloat16).reshape(rows, cols)
        st = torch.from_numpy(scales.view(np.int16)).view(torch.bfloat16).reshape(rows, cols // B)
        lo, hi = value.range()
        q = torch.clamp(torch.round(xt / st.repeat_interleave(B, dim=1)), lo, hi)
        codes = q.to(torch.int32).numpy().reshape(-1)
        bits = value.size_bits()
        nq = 32 // bits
        fields = (codes.astype(np.int64) & ((1 << bits) - 1)).reshape(-1, nq)
        want = (fields << (bits * np.arange(nq))).sum(axis=1).astype(np.uint32)
        assert np.array_equal(words.reshape(-1), want)
        # out_scale = f32(bf16 scale)
        assert np.array_equal(out_scale.reshape(-1), st.to(torch.float32).numpy().reshape(-1))
        deq = oracle.dequantize(words, (rows, cols), out_scale, ElemType.BF16, scheme)
        qf = q.to(torch.int32).to(torch.bfloat16)  # codes travel as integers: -0.0 becomes +0
        want_deq = (st.repeat_interleave(B, dim=1) * qf).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(deq, want_deq)


def test_scale_rule_identities(oracle):
    """2*absmax/(q_max-q_min): abs-max is order independent and exact; for the
    symmetric ranges it equals absmax/q_max bit for bit (BASELINE config 1:
    'scale = absmax/127')."""
    rng = np.random.default_rng(23)
    x = rng.normal(0, 1, (8, 64)).astype(np.float32)
    for value, qmax in ((QuantValue.Q8S, 127), (QuantValue.Q4S, 7), (QuantValue.Q2S, 1), (QuantValue.E2M1, 6)):
        s = oracle.compute_scales(x, ElemType.F32, (8, 64), QuantScheme.default().with_value(value))
        assert s.shape == (1,) and s[0] == np.float32(np.abs(x).max()) / np.float32(qmax)
        sb = oracle.compute_scales(x, ElemType.F32, (8, 64),
                                   QuantScheme.default().with_value(value).with_level(QuantLevel.block([16])))
        want = np.abs(x).reshape(8, 4, 16).max(axis=2) / np.float32(qmax)
        assert np.array_equal(sb, want.astype(np.float32))
    # asymmetric range: divisor is q_max - q_min = 255, computed from 2*absmax
    s = oracle.compute_scales(x, ElemType.F32, (8, 64), QuantScheme.default().with_value(QuantValue.Q8F))
    assert s[0] == (np.float32(2.0) * np.float32(np.abs(x).max())) / np.float32(255.0)
    # exact rational check of one value, and permutation invariance
    a = Fraction(float(np.abs(x).max()))
    import golden.exact_model as em
    assert Fraction(float(s[0])) == em.round_to_format(em.round_to_format(2 * a, "f32") / 255, "f32")
    perm = rng.permutation(x.size)
    s2 = oracle.compute_scales(x.reshape(-1)[perm].reshape(8, 64), ElemType.F32, (8, 64),
                               QuantScheme.default().with_value(QuantValue.Q8F))
    assert s2[0] == s[0]


def test_edge_semantics_fixed_by_decision(oracle):
    """Behaviour the reference's tests leave open (parity unpinned); these are
    the choices the GPU path has to reproduce: NaN quotient -> q_max, +-inf
    saturate, zero scale with zero input -> q_max, abs-max skips NaN."""
    scheme = QuantScheme.default().with_value(QuantValue.Q8S)
    x = np.array([np.nan, np.inf, -np.inf, 0.0, 1e30, -1e30, 1.0, -1.0], np.float32).reshape(1, 8)
    w, _ = oracle.quantize(x, ElemType.F32, (1, 8), np.array([1.0], np.float32), scheme)
    assert w.reshape(-1).view(np.int8).tolist() == [127, 127, -127, 0, 127, -127, 1, -1]
    w0, _ = oracle.quantize(np.zeros((1, 4), np.float32), ElemType.F32, (1, 4), np.array([0.0], np.float32), scheme)
    assert w0.reshape(-1).view(np.uint8).tolist() == [127] * 4
    xs = np.array([np.nan, -3.0, 2.0, np.nan], np.float32).reshape(1, 4)
    s = oracle.compute_scales(xs, ElemType.F32, (1, 4), scheme)
    assert s[0] == np.float32(3.0) / np.float32(127.0)


def test_param_dtype_rounds_the_divisor(oracle):
    """out_scale = FS(scale) and the divisor is F(FS(scale)) (src/quantize.rs:26-27,90):
    with f32 data and BF16 params the division uses the bf16-rounded scale."""
    x = np.array([100.0, -100.0, 33.0, 1.0], np.float32).reshape(1, 4)
    sc = np.array([1.00390625 + 2 ** -10], np.float32)  # rounds to 1.0078125 in bf16 (tie away from 1.0)
    scheme = QuantScheme.default().with_value(QuantValue.Q8S).with_param(QuantParam.BF16)
    w, out_scale = oracle.quantize(x, ElemType.F32, (1, 4), sc, scheme)
    d = np.float32(oracle.from_bits(out_scale, ElemType.BF16)[0])
    assert d != sc[0]
    want = np.clip(np.rint(x / d), -127, 127).astype(np.int8).reshape(-1)
    assert np.array_equal(w.reshape(-1).view(np.int8), want)


def test_native_fp8_store_matches_torch_composition(oracle):
    """cqo_quantize_native / cqo_dequantize_native for e4m3 and e5m2 against the same
    computation spelled with torch CPU routines: IEEE divide, round half to even, clamp,
    cast to float8; and float8 -> f32 times scale.  (That the reference's native arm means
    exactly this composition is a decision; that the oracle computes it is what this pins.)"""
    import torch
    from cubek_amd import ElemType, QuantLevel, QuantScheme, QuantStore, QuantValue

    rng = np.random.default_rng(21)
    for value, tdt, top in ((QuantValue.E4M3, torch.float8_e4m3fn, 448.0), (QuantValue.E5M2, torch.float8_e5m2, 57344.0)):
        for block in (None, 16):
            shape = (24, 64)
            level = QuantLevel.Tensor if block is None else QuantLevel.block([block])
            scheme = QuantScheme.default().with_value(value).with_store(QuantStore.Native).with_level(level)
            x = rng.normal(0, 3, shape).astype(np.float32)
            s = oracle.compute_scales(x, ElemType.F32, shape, scheme)
            codes, out_scale = oracle.quantize(x, ElemType.F32, shape, s, scheme)
            if block is None:
                s_full = np.full(shape, s.reshape(-1)[0], dtype=np.float32)
            else:
                s_full = np.repeat(s.reshape(shape[0], -1), block, axis=1)
            q = torch.clamp(torch.round(torch.from_numpy(x) / torch.from_numpy(s_full)), -top, top)
            want = q.to(tdt).view(torch.uint8).numpy()
            assert np.array_equal(codes.reshape(shape), want), value.name
            y = oracle.dequantize(codes, shape, out_scale, ElemType.F32, scheme)
            y_want = (torch.from_numpy(want).view(tdt).to(torch.float32) * torch.from_numpy(s_full)).numpy()
            assert np.array_equal(y.reshape(shape), y_want), value.name


# ---------------------------------------------------------------- native store pins

def _native(value, block=None, param=QuantParam.F32):
    level = QuantLevel.Tensor if block is None else QuantLevel.block(block)
    return QuantScheme.default().with_value(value).with_store(QuantStore.Native).with_level(level).with_param(param)


def test_native_e2m1_known_answer_bytes(oracle):
    """Hand-written: scale 1, quotients are the inputs.  e2m1 codes by the OCP FP4 table
    {0: 0, 0.5: 1, 1: 2, 1.5: 3, 2: 4, 3: 5, 4: 6, 6: 7}, sign in bit 3; the quantizer rounds to an
    integer first (src/quantize.rs:26-30), so 0.5 -> 0 and 1.5 -> 2 (ties to even), 2.5 -> 2, 5 -> tie
    between 4 and 6 -> the even code, 4; 7 clamps to 6.  Element 2k sits in the LOW nibble of byte k."""
    x = np.array([0, 1, 2, 3, 4, 5, 6, 7,
                  -1, -2, -3, -4, -5, -6, -7, 0.5,
                  1.5, 2.5, 3.5, 4.5, 5.5, -0.5, -1.5, -0.25], np.float32).reshape(1, 24)
    want_nibbles = [0x0, 0x2, 0x4, 0x5, 0x6, 0x6, 0x7, 0x7,
                    0xA, 0xC, 0xD, 0xE, 0xE, 0xF, 0xF, 0x0,
                    0x4, 0x4, 0x6, 0x6, 0x7, 0x8, 0xC, 0x8]   # 3.5 -> 4, 4.5 -> 4, 5.5 -> 6; -0.5, -0.25 -> -0
    want_bytes = [lo | (hi << 4) for lo, hi in zip(want_nibbles[0::2], want_nibbles[1::2])]
    codes, out_scale = oracle.quantize(x, ElemType.F32, (1, 24), np.array([1.0], np.float32), _native(QuantValue.E2M1))
    assert codes.reshape(-1).tolist() == want_bytes
    assert want_bytes[:4] == [0x20, 0x54, 0x66, 0x77]  # spelled out: element 0 low, element 1 high
    y = oracle.dequantize(codes, (1, 24), np.array([0.5], np.float32), ElemType.F32, _native(QuantValue.E2M1))
    mags = {0x0: 0.0, 0x2: 1.0, 0x4: 2.0, 0x5: 3.0, 0x6: 4.0, 0x7: 6.0}
    want_y = [(-0.5 if n & 8 else 0.5) * mags[n & 7] for n in want_nibbles]
    assert y.reshape(-1).tolist() == want_y
    assert np.signbit(y.reshape(-1)).tolist() == [bool(n & 8) for n in want_nibbles]  # -0 survives


def test_native_i8_known_answer_bytes(oracle):
    """Every code of the i8 store: x = k * 0.5 with scale 0.5 gives quotient k; the stored byte is k in
    two's complement (Q8S clamps -128 to -127, Q8F keeps it); dequantize returns scale * k."""
    ks = np.arange(-130, 131)
    x = np.zeros(264, np.float32)
    x[:ks.size] = ks * 0.5
    for value, lo in ((QuantValue.Q8S, -127), (QuantValue.Q8F, -128)):
        codes, _ = oracle.quantize(x.reshape(1, -1), ElemType.F32, (1, 264), np.array([0.5], np.float32), _native(value))
        want = np.clip(ks, lo, 127)
        assert codes.reshape(-1)[:ks.size].tolist() == [int(k) & 0xFF for k in want]
        assert not codes.reshape(-1)[ks.size:].any()
        y = oracle.dequantize(codes, (1, 264), np.array([0.5], np.float32), ElemType.F32, _native(value))
        assert y.reshape(-1)[:ks.size].tolist() == (want * 0.5).tolist()


@pytest.mark.parametrize("elem", [ElemType.F32, ElemType.BF16, ElemType.F16], ids=lambda e: e.name)
def test_native_store_agrees_with_packed_store(oracle, elem):
    """The two stores of one scheme hold the same codes in different containers, which ties the native
    arms to the packed path that the exact-rational fixtures pin: native i8 byte e is field e % 4 of
    packed word e / 4; a native e2m1 nibble decodes to the integer the packed E2M1 path stores, rounded
    to the e2m1 grid (5 -> 4, the only integer of [-6, 6] off the grid); dequantized values agree wherever
    the packed integer is on the grid."""
    rng = np.random.default_rng(31)
    shape = (8, 128)
    x = rng.uniform(-0.1, 0.1, shape).astype(np.float32)  # quotients spread over the whole value range
    xb = oracle.to_bits(x, elem)
    for value in (QuantValue.Q8S, QuantValue.Q8F, QuantValue.E2M1):
        for block in (None, [32], [2, 16]):
            level = QuantLevel.Tensor if block is None else QuantLevel.block(block)
            packed = QuantScheme.default().with_value(value).with_level(level)
            s = oracle.compute_scales(xb, elem, shape, packed)
            words, os_p = oracle.quantize(xb, elem, shape, s, packed)
            codes, os_n = oracle.quantize(xb, elem, shape, s, _native(value, block))
            assert gc.bits_equal(os_p, os_n)
            bits = value.size_bits()
            fields = (words.reshape(-1, 1) >> (bits * np.arange(32 // bits, dtype=np.uint32))) & ((1 << bits) - 1)
            ints = fields.reshape(-1).astype(np.int64)
            ints = np.where(ints >= 1 << (bits - 1), ints - (1 << bits), ints)
            yp = oracle.from_bits(oracle.dequantize(words, shape, os_p, elem, packed), elem).reshape(-1)
            yn = oracle.from_bits(oracle.dequantize(codes, shape, os_n, elem, _native(value, block)), elem).reshape(-1)
            if bits == 8:
                assert np.array_equal(codes.reshape(-1), fields.reshape(-1).astype(np.uint8))
                assert np.array_equal(yp, yn)
            else:
                nib = np.stack([codes.reshape(-1) & 0xF, codes.reshape(-1) >> 4], axis=1).reshape(-1)
                grid = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
                decoded = np.where(nib & 8, -1.0, 1.0) * grid[nib & 7]
                want = np.where(np.abs(ints) == 5, np.sign(ints) * 4, ints)
                assert np.array_equal(np.abs(decoded), np.abs(want)) and np.array_equal(decoded[want != 0], want[want != 0])
                assert set(np.unique(np.abs(ints))) >= {0, 1, 2, 3, 4, 5, 6}  # the data reach every integer
                on_grid = np.abs(ints) != 5
                assert np.array_equal(yp[on_grid], yn[on_grid])


@pytest.mark.parametrize("elem,value,block,shape", [
    (ElemType.F32, QuantValue.Q8S, None, (37, 52)),        # 481 words: odd, not a multiple of the 64-word slices
    (ElemType.BF16, QuantValue.Q4S, 8, (131, 72)),         # 1179 words
    (ElemType.F16, QuantValue.Q2S, 16, (5, 7, 48)),        # 105 words, rank 3
    (ElemType.BF16, QuantValue.E2M1, 32, (3, 64)),         # 24 words: fewer than one slice
], ids=["f32_q8s_tensor", "bf16_q4s_b8", "f16_q2s_b16_rank3", "bf16_e2m1_b32_tiny"])
def test_threaded_drivers_equal_the_single_threaded_functions(oracle, elem, value, block, shape):
    """cqo_quantize_packed_mt / cqo_dequantize_packed_mt cut the words into slices for 1 - 17 threads: every word
    and every out_scale entry must come out as from one call over the whole range (a dropped or doubled slice, or a
    slice that starts at the wrong word, changes the result)."""
    rng = np.random.default_rng(len(shape) * 100 + int(value))
    level = QuantLevel.Tensor if block is None else QuantLevel.block([block])
    scheme = QuantScheme.default().with_value(value).with_level(level)
    x = oracle.to_bits(rng.normal(0, 1, shape).astype(np.float32), elem)
    scale = oracle.compute_scales(x, elem, shape, scheme)
    words, out_scale = oracle.quantize(x, elem, shape, scale, scheme)
    deq = oracle.dequantize(words, shape, out_scale, elem, scheme)
    assert np.count_nonzero(words) > words.size // 2
    for threads in range(1, 18):
        w_mt, os_mt = oracle.quantize(x, elem, shape, scale, scheme, threads=threads)
        assert gc.bits_equal(w_mt, words), threads
        assert gc.bits_equal(os_mt, out_scale), threads
        d_mt = oracle.dequantize(words, shape, out_scale, elem, scheme, threads=threads)
        assert gc.bits_equal(d_mt, deq), threads
