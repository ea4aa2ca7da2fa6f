"""Writes tests/golden/*.npz: inputs and expected outputs computed with the
exact-rational model (exact_model.py), never with the C oracle or the GPU.

    python tests/golden/gen_golden.py

Cases
  ref_ramps.npz   the reference's own 24 round-trip cases
                  (crates/cubek-quant/tests/suite/mod.rs:18-52 x
                  tests/suite/symmetric.rs:24-66,143-207): shapes 32x32 and
                  16x64, six integer value types, per-tensor and per-block
                  (block = first dimension, along the last axis), f32 data ramps,
                  scales by the test's host rule.
  typed_small.npz f32/bf16/f16 inputs with many exact .5 quotients, other
                  param dtypes, N-D blocks, strided scales, E2M1/E4M3 ranges.
  typed_native.npz the native store (crates/cubek-quant/src/quantize.rs:100-126,
                  src/dequantize.rs:150-167): i8 / e4m3 / e5m2 bytes and e2m1 nibble
                  pairs for f32/bf16/f16 inputs: every integer quotient of the value
                  range and every half-integer in between, signed zeros, random data
                  with abs-max scales per tensor and per block, f16/bf16 parameters.
  typed_ocp.npz   the extension value E2M1_OCP (not in the reference): every multiple of 1/8 of
                  the e2m1 range as a quotient, random data, three float and parameter types.
"""
from __future__ import annotations

import os
import sys
from fractions import Fraction

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import exact_model as em  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def f32_bits(values):
    return np.array([em.fraction_to_bits(v, "f32") for v in values], dtype=np.uint32)


def contiguous_strides(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


def run_case(store, name, x_bits, fmt, shape, block, value, param_fmt, scale_bits=None,
             scale_strides=None, native=False):
    if scale_bits is None:
        scale_bits = em.scales_from_absmax(x_bits, fmt, shape, block, value)
    if scale_strides is None:
        scale_strides = (0,) * len(shape) if block is None else contiguous_strides(
            tuple(s // b for s, b in zip(shape, (1,) * (len(shape) - len(block)) + tuple(block))))
    quantize, dequantize = ((em.quantize_tensor_native, em.dequantize_tensor_native) if native
                            else (em.quantize_tensor, em.dequantize_tensor))
    words, out_scale = quantize(x_bits, fmt, shape, scale_bits, scale_strides, block, value, param_fmt)
    deq = dequantize(words, fmt, shape, out_scale, scale_strides, block, value, param_fmt)
    store[f"{name}/x"] = x_bits.reshape(-1)
    store[f"{name}/scale"] = scale_bits.reshape(-1)
    store[f"{name}/words"] = words
    store[f"{name}/out_scale"] = out_scale
    store[f"{name}/deq"] = deq
    store[f"{name}/meta"] = np.array(
        [fmt, value, param_fmt, ",".join(map(str, shape)),
         "" if block is None else ",".join(map(str, block)),
         ",".join(map(str, scale_strides))] + (["native"] if native else []))


def reference_ramps():
    store = {}
    for (m, n) in ((32, 32), (16, 64)):
        num = m * n
        half = Fraction(num, 2)
        for value in ("Q8F", "Q8S", "Q4F", "Q4S", "Q2F", "Q2S"):
            lo, hi = em.RANGES[value]
            # per tensor: x_i = i - N/2 ; scale = (2*half)/(q_max-q_min)   symmetric.rs:29-38
            x = f32_bits([Fraction(i) - half for i in range(num)])
            scale = f32_bits([em.round_to_format(2 * half / (hi - lo), "f32")])
            run_case(store, f"tensor_{m}x{n}_{value}", x, "f32", (m, n), None, value, "f32",
                     scale_bits=scale)
            # per block: x_i = (i - N/2)/N in f32 ; block = m on the last axis   symmetric.rs:148-179
            xb = f32_bits([em.round_to_format((Fraction(i) - half) / num, "f32") for i in range(num)])
            run_case(store, f"block_{m}x{n}_{value}", xb, "f32", (m, n), (m,), value, "f32")
    np.savez_compressed(os.path.join(HERE, "ref_ramps.npz"), **store)
    return len(store) // 6


def to_fmt_bits(values, fmt):
    """Round arbitrary Fractions to fmt and return bit patterns."""
    dt = np.uint32 if fmt == "f32" else np.uint16
    return np.array([em.fraction_to_bits(em.round_to_format(Fraction(v), fmt), fmt) for v in values],
                    dtype=dt)


def typed_small():
    rng = np.random.default_rng(20240607)
    store = {}

    def gauss(n, sigma):
        return [Fraction(float(v)) for v in rng.normal(0.0, sigma, n)]

    # exact half-integer quotients: x = (k + 1/2) * s with s a power of two / a 3-bit odd scale
    for fmt in ("f32", "bf16", "f16"):
        for value in ("Q8S", "Q4S", "Q2S", "Q8F", "Q4F", "Q2F", "E2M1"):
            lo, hi = em.RANGES[value]
            bits = em.size_bits(value)
            nq = 32 // bits
            ks = list(range(lo - 2, hi + 2))
            vals = []
            for s in (Fraction(1, 4), Fraction(3, 8)):
                vals += [(Fraction(k) + Fraction(1, 2)) * s for k in ks]
                vals += [Fraction(k) * s for k in ks]
            while len(vals) % 64:
                vals.append(Fraction(0))
            x = to_fmt_bits(vals, fmt)
            n = len(vals)
            # per-tensor with an explicit scale that makes the quotients exact ties
            sc = to_fmt_bits([Fraction(1, 4)], fmt)
            run_case(store, f"ties_{fmt}_{value}_s0.25", x, fmt, (n // 64, 64), None, value, "f32",
                     scale_bits=sc)
            sc = to_fmt_bits([Fraction(3, 8)], fmt)
            run_case(store, f"ties_{fmt}_{value}_s0.375", x, fmt, (n // 64, 64), None, value, "f32",
                     scale_bits=sc)

    # random data, scales from abs-max, every param dtype
    for fmt in ("f32", "bf16", "f16"):
        for value, block in (("Q8S", (32,)), ("Q4S", (32,)), ("Q2S", (64,)), ("E2M1", (32,)),
                             ("Q8F", (16,)), ("Q4F", (8,)), ("Q2F", (16,)), ("E4M3", (16,))):
            for param in ("f32", "f16", "bf16"):
                if param != "f32" and value not in ("Q8S", "Q4S", "E2M1"):
                    continue
                shape = (6, 128)
                x = to_fmt_bits(gauss(6 * 128, 0.02), fmt)
                run_case(store, f"rand_{fmt}_{value}_{param}", x, fmt, shape, block, value, param)
        x = to_fmt_bits(gauss(4 * 64, 1.0), fmt)
        run_case(store, f"rand_tensor_{fmt}_Q8S", x, fmt, (4, 64), None, "Q8S", "f32")

    # N-D blocks and strided scales
    shape = (4, 6, 32)
    x = to_fmt_bits(gauss(4 * 6 * 32, 0.5), "f32")
    run_case(store, "nd_f32_Q4S_2x3x16", x, "f32", shape, (2, 3, 16), "Q4S", "f32")
    run_case(store, "nd_f32_Q8S_3x8", x, "f32", shape, (3, 8), "Q8S", "f32")
    xb = to_fmt_bits(gauss(8 * 64, 0.5), "bf16")
    # scales [8,2] stored column-major inside a 16-entry buffer: strides (1,8)
    sc_contig = em.scales_from_absmax(xb, "bf16", (8, 64), (32,), "Q8S")  # [8,2]
    buf = np.zeros(16, dtype=np.uint16)
    for r in range(8):
        for c in range(2):
            buf[r * 1 + c * 8] = sc_contig[r, c]
    run_case(store, "strided_bf16_Q8S", xb, "bf16", (8, 64), (32,), "Q8S", "f32", scale_bits=buf,
             scale_strides=(1, 8))
    # negative scales (only a caller's own scales can be): the quotient changes sign, a zero code
    # dequantizes to -0
    for fmt in ("f32", "bf16", "f16"):
        vals = [(Fraction(k) + h) * Fraction(-3, 8) for k in range(-9, 9) for h in (0, Fraction(1, 2))]
        while len(vals) % 64:
            vals.append(Fraction(0))
        run_case(store, f"negscale_{fmt}_Q4S", to_fmt_bits(vals, fmt), fmt, (len(vals) // 64, 64), None, "Q4S", "f32",
                 scale_bits=to_fmt_bits([Fraction(-3, 8)], fmt))
        x = to_fmt_bits(gauss(2 * 64, 1.0), fmt)
        neg = em.scales_from_absmax(x, fmt, (2, 64), (32,), "Q8S") | (1 << (31 if fmt == "f32" else 15))
        run_case(store, f"negscale_{fmt}_Q8S_b32", x, fmt, (2, 64), (32,), "Q8S", "f32", scale_bits=neg)
    np.savez_compressed(os.path.join(HERE, "typed_small.npz"), **store)
    return len(store) // 6


def typed_native():
    rng = np.random.default_rng(20250311)
    store = {}

    def gauss(n, sigma):
        return [Fraction(float(v)) for v in rng.normal(0.0, sigma, n)]

    def with_signed_zeros(bits, fmt, where):
        """Turns the (zero) entries at ``where`` into -0."""
        bits = bits.copy()
        for i in where:
            assert bits[i] == 0
            bits[i] = 1 << (31 if fmt == "f32" else 15)
        return bits

    for fmt in ("f32", "bf16", "f16"):
        for value in ("Q8S", "Q8F", "E4M3", "E5M2", "E2M1"):
            lo, hi = em.RANGES[value]
            if value == "E5M2":  # the range is too wide to walk: its ends, the small integers, powers of two
                ks = list(range(-34, 35)) + [s * (2 ** p + o) for p in range(6, 16) for o in (-1, 0, 1) for s in (-1, 1)]
                ks += list(range(57340, 57347)) + list(range(-57346, -57339))
            else:
                ks = list(range(lo - 2, hi + 3))
            # integer and half-integer quotients under a power-of-two scale, +0 and -0, small negatives
            vals = []
            for k in ks:
                vals += [Fraction(k), Fraction(k) + Fraction(1, 2)]
            vals += [Fraction(-1, 4), Fraction(1, 4), Fraction(-3, 8), Fraction(-1, 2), Fraction(1, 2)]
            zeros_at = list(range(len(vals), len(vals) + 4))
            vals += [Fraction(0)] * 4
            while len(vals) % 64:
                vals.append(Fraction(0))
            n = len(vals)
            for tag, s in (("s0.25", Fraction(1, 4)), ("s-0.5", Fraction(-1, 2))):
                x = with_signed_zeros(to_fmt_bits([v * s for v in vals], fmt), fmt, zeros_at[:2])
                run_case(store, f"native_ties_{fmt}_{value}_{tag}", x, fmt, (n // 64, 64), None, value, "f32",
                         scale_bits=to_fmt_bits([s], fmt), native=True)
            # random data, scales from abs-max, per tensor and per block, other parameter types
            x = to_fmt_bits(gauss(4 * 128, 0.02), fmt)
            run_case(store, f"native_rand_{fmt}_{value}_tensor", x, fmt, (4, 128), None, value, "f32", native=True)
            for param in ("f32", "f16", "bf16"):
                if param != "f32" and value not in ("Q8S", "E4M3", "E2M1"):
                    continue
                x = to_fmt_bits(gauss(4 * 128, 0.02), fmt)
                run_case(store, f"native_rand_{fmt}_{value}_b32_{param}", x, fmt, (4, 128), (32,), value, param,
                         native=True)
    # N-D blocks
    x = to_fmt_bits(gauss(4 * 6 * 32, 0.5), "f32")
    run_case(store, "native_nd_f32_E2M1_2x3x16", x, "f32", (4, 6, 32), (2, 3, 16), "E2M1", "f32", native=True)
    run_case(store, "native_nd_f32_Q8S_3x8", x, "f32", (4, 6, 32), (3, 8), "Q8S", "f32", native=True)
    np.savez_compressed(os.path.join(HERE, "typed_native.npz"), **store)
    return len(store) // 6


def typed_ocp():
    """The extension value E2M1_OCP (no counterpart in the reference): e2m1 nibbles rounded once from the
    quotient.  Native-store layout; the U32 store holds the same bytes as little-endian words."""
    rng = np.random.default_rng(20240611)
    store = {}

    def gauss(n, sigma):
        return [Fraction(float(v)) for v in rng.normal(0.0, sigma, n)]

    for fmt in ("f32", "bf16", "f16"):
        # every multiple of 1/8 in [-7, 7] (all seven midpoints of the e2m1 grid, both signs, and the clamp),
        # sixteenths near zero, signed zeros
        vals = [Fraction(k, 8) for k in range(-56, 57)]
        vals += [Fraction(s * k, 16) for k in (1, 3, 5) for s in (-1, 1)]
        zeros_at = list(range(len(vals), len(vals) + 4))
        vals += [Fraction(0)] * 4
        while len(vals) % 64:
            vals.append(Fraction(0))
        n = len(vals)
        sign_bit = 1 << (31 if fmt == "f32" else 15)
        for tag, s in (("s0.25", Fraction(1, 4)), ("s-0.5", Fraction(-1, 2))):
            x = to_fmt_bits([v * s for v in vals], fmt)
            for i in zeros_at[:2]:
                assert x[i] == 0
                x[i] = sign_bit
            run_case(store, f"ocp_ties_{fmt}_{tag}", x, fmt, (n // 64, 64), None, "E2M1_OCP", "f32",
                     scale_bits=to_fmt_bits([s], fmt), native=True)
        x = to_fmt_bits(gauss(4 * 128, 0.02), fmt)
        run_case(store, f"ocp_rand_{fmt}_tensor", x, fmt, (4, 128), None, "E2M1_OCP", "f32", native=True)
        for param in ("f32", "f16", "bf16"):
            x = to_fmt_bits(gauss(4 * 128, 0.02), fmt)
            run_case(store, f"ocp_rand_{fmt}_b32_{param}", x, fmt, (4, 128), (32,), "E2M1_OCP", param, native=True)
    x = to_fmt_bits(gauss(4 * 6 * 32, 0.5), "f32")
    run_case(store, "ocp_nd_f32_2x3x16", x, "f32", (4, 6, 32), (2, 3, 16), "E2M1_OCP", "f32", native=True)
    np.savez_compressed(os.path.join(HERE, "typed_ocp.npz"), **store)
    return len(store) // 6


if __name__ == "__main__":
    a = reference_ramps()
    b = typed_small()
    c = typed_native()
    d = typed_ocp()
    print(f"wrote {a} reference ramp cases, {b} typed cases, {c} native-store cases and {d} cases of the e2m1 extension")
