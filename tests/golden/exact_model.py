"""Exact-rational statement of the quantize/dequantize arithmetic, independent
of the C oracle: every float operation is carried out on ``fractions.Fraction``
and rounded ONCE, directly to the target format, with round-half-to-even.

It is the mathematical definition the specification appeals to ("the correctly
rounded quotient in F", "round half to even", "two's-complement field i at bits
[i*b,(i+1)*b)"), written so that a dropped rounding step, a reciprocal multiply,
round-half-away, a transposed field order or a wrong scale index in the oracle
shows up as a mismatch.  Pure Python, small inputs only, finite values only.

The native store (one byte per value: i8, e4m3, e5m2; two e2m1 nibbles per byte)
is stated the same way: the minifloat formats are built from their published bit
fields (sign, exponent, mantissa, bias), "cast to Q" is "nearest value of the format,
ties to the even code, saturating", and the sign of a zero result is the sign IEEE
arithmetic gives it (sign(x) xor sign(scale)).

Specification followed: crates/cubek-quant/src/quantize.rs:19-43,61-81,100-126,
src/dequantize.rs:22-25,86-118,150-167, src/layout/scales.rs:144-160,179-194,
tests/suite/symmetric.rs:35-38,156-179.
"""
from __future__ import annotations

from fractions import Fraction
from typing import List, Sequence, Tuple

import numpy as np

# name -> (precision p incl. hidden bit, emin, emax)
FORMATS = {"f32": (24, -126, 127), "f16": (11, -14, 15), "bf16": (8, -126, 127)}


def rint_even(q: Fraction) -> int:
    """Nearest integer, ties to even."""
    fl = q.numerator // q.denominator
    rem = q - fl
    if rem > Fraction(1, 2):
        return fl + 1
    if rem < Fraction(1, 2):
        return fl
    return fl if fl % 2 == 0 else fl + 1


def round_to_format(q: Fraction, fmt: str) -> Fraction:
    """Nearest value of the binary format, ties to even mantissa; gradual
    underflow; raises on overflow (callers stay in range)."""
    p, emin, emax = FORMATS[fmt]
    if q == 0:
        return Fraction(0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    e = max(e, emin)
    quantum = Fraction(2) ** (e - p + 1)
    r = rint_even(a / quantum) * quantum
    if r >= Fraction(2) ** (emax + 1):
        raise OverflowError("result overflows the format")
    return sign * r


def bits_to_fraction(bits: int, fmt: str) -> Fraction:
    if fmt == "f32":
        v = np.array([bits], dtype=np.uint32).view(np.float32)[0]
    elif fmt == "f16":
        v = np.array([bits], dtype=np.uint16).view(np.float16)[0]
    else:
        v = np.array([bits << 16], dtype=np.uint32).view(np.float32)[0]
    assert np.isfinite(v)
    return Fraction(float(v))


def fraction_to_bits(q: Fraction, fmt: str) -> int:
    """Bit pattern of a value already representable in ``fmt`` (sign of zero: +)."""
    f = float(q)
    assert Fraction(f) == q
    if fmt == "f32":
        out = int(np.array([f], dtype=np.float32).view(np.uint32)[0])
        assert Fraction(float(np.float32(f))) == q
        return out
    if fmt == "f16":
        assert Fraction(float(np.float16(f))) == q
        return int(np.array([f], dtype=np.float16).view(np.uint16)[0])
    u = int(np.array([f], dtype=np.float32).view(np.uint32)[0])
    assert u & 0xFFFF == 0
    return u >> 16


def size_bits(value: str) -> int:
    return {"Q8F": 8, "Q8S": 8, "E4M3": 8, "E5M2": 8, "Q4F": 4, "Q4S": 4, "E2M1": 4, "E2M1_OCP": 4,
            "Q2F": 2, "Q2S": 2}[value]


RANGES = {"Q8F": (-128, 127), "Q8S": (-127, 127), "Q4F": (-8, 7), "Q4S": (-7, 7),
          "Q2F": (-2, 1), "Q2S": (-1, 1), "E2M1": (-6, 6), "E2M1_OCP": (-6, 6), "E4M3": (-448, 448),
          "E5M2": (-57344, 57344)}


def block_of(elem: int, shape: Sequence[int], block: Sequence[int]) -> Tuple[Tuple[int, ...], bool]:
    """(block coordinates, is first element of its block) from first principles:
    unravel the linear index row-major, divide each coordinate by its block extent."""
    coords = []
    rem = elem
    for s in reversed(shape):
        coords.append(rem % s)
        rem //= s
    coords.reverse()
    blk = tuple(c // b for c, b in zip(coords, block))
    start = all(c % b == 0 for c, b in zip(coords, block))
    return blk, start


def quantize_codes(x: Sequence[Fraction], d: Fraction, fmt: str, value: str) -> List[int]:
    lo, hi = RANGES[value]
    out = []
    for xi in x:
        t = round_to_format(xi / d, fmt)  # correctly rounded quotient in F
        out.append(min(max(rint_even(t), lo), hi))
    return out


def pack(codes: Sequence[int], bits: int) -> int:
    w = 0
    for i, c in enumerate(codes):
        w |= (c % (1 << bits)) << (i * bits)  # two's complement field
    return w


def unpack(word: int, bits: int) -> List[int]:
    out = []
    for i in range(32 // bits):
        raw = (word >> (i * bits)) % (1 << bits)
        out.append(raw - (1 << bits) if raw >= (1 << (bits - 1)) else raw)
    return out


def quantize_tensor(x_bits: np.ndarray, fmt: str, shape: Sequence[int], scale_bits: np.ndarray,
                    scale_strides: Sequence[int], block: Sequence[int] | None, value: str,
                    param_fmt: str):
    """Packed-u32 quantization of a contiguous tensor.
    Returns (words uint32[N/nq], out_scale bit patterns in param_fmt, same footprint as scale)."""
    bits = size_bits(value)
    nq = 32 // bits
    n = int(np.prod(shape))
    x = [bits_to_fraction(int(b), fmt) for b in x_bits.reshape(-1)]
    words = np.zeros(n // nq, dtype=np.uint32)
    out_scale = np.zeros(scale_bits.size, dtype=np.uint32 if param_fmt == "f32" else np.uint16)
    blk_vec = None if block is None else (1,) * (len(shape) - len(block)) + tuple(block)
    for p in range(n // nq):
        e0 = p * nq
        if blk_vec is None:
            si, start = 0, e0 == 0
        else:
            bc, start = block_of(e0, shape, blk_vec)
            si = sum(c * s for c, s in zip(bc, scale_strides))
        s_f = bits_to_fraction(int(scale_bits.reshape(-1)[si]), fmt)
        s_fs = round_to_format(s_f, param_fmt)
        if start:
            out_scale[si] = fraction_to_bits(s_fs, param_fmt)
        d = round_to_format(s_fs, fmt)
        words[p] = pack(quantize_codes(x[e0:e0 + nq], d, fmt, value), bits)
    return words, out_scale


def dequantize_tensor(words: np.ndarray, fmt: str, shape: Sequence[int], scale_bits: np.ndarray,
                      scale_strides: Sequence[int], block: Sequence[int] | None, value: str,
                      param_fmt: str) -> np.ndarray:
    bits = size_bits(value)
    nq = 32 // bits
    n = int(np.prod(shape))
    out = np.zeros(n, dtype=np.uint32 if fmt == "f32" else np.uint16)
    blk_vec = None if block is None else (1,) * (len(shape) - len(block)) + tuple(block)
    for p in range(n // nq):
        e0 = p * nq
        if blk_vec is None:
            si = 0
        else:
            bc, _ = block_of(e0, shape, blk_vec)
            si = sum(c * s for c, s in zip(bc, scale_strides))
        s = round_to_format(bits_to_fraction(int(scale_bits.reshape(-1)[si]), param_fmt), fmt)
        for i, c in enumerate(unpack(int(words[p]), bits)):
            # F(c) is +0 for the code 0, so the product's sign is the scale's when it is zero
            y = round_to_format(s * c, fmt)
            out[e0 + i] = (fraction_to_bits(abs(y), fmt) | (int((s < 0) != (c < 0)) << (31 if fmt == "f32" else 15))
                           if y == 0 else fraction_to_bits(y, fmt))
    return out


def scales_from_absmax(x_bits: np.ndarray, fmt: str, shape: Sequence[int],
                       block: Sequence[int] | None, value: str) -> np.ndarray:
    """scale = f32(2*absmax) / f32(q_max-q_min) rounded to f32, then to ``fmt``;
    contiguous scales, one per block (or one in total)."""
    lo, hi = RANGES[value]
    n = int(np.prod(shape))
    x = [abs(bits_to_fraction(int(b), fmt)) for b in x_bits.reshape(-1)]
    if block is None:
        sshape = (1,)
        amax = {(): max(x)}
        keys = [()]
    else:
        blk_vec = (1,) * (len(shape) - len(block)) + tuple(block)
        sshape = tuple(s // b for s, b in zip(shape, blk_vec))
        amax = {}
        for e in range(n):
            bc, _ = block_of(e, shape, blk_vec)
            amax[bc] = max(amax.get(bc, Fraction(0)), x[e])
        keys = list(np.ndindex(*sshape))
    out = np.zeros(len(keys), dtype=np.uint32 if fmt == "f32" else np.uint16)
    for i, k in enumerate(keys):
        two_a = round_to_format(2 * amax[tuple(k)], "f32")
        s32 = round_to_format(two_a / (hi - lo), "f32")
        out[i] = fraction_to_bits(round_to_format(s32, fmt), fmt)
    return out.reshape(sshape)


# ---------------------------------------------------------------- native store
# name -> (exponent bits, mantissa bits, bias): OCP 8-bit floating point (E4M3 finite-only
# with one NaN code, E5M2 IEEE-like) and OCP microscaling FP4 (E2M1, no NaN, no infinity)
MINIFLOATS = {"E4M3": (4, 3, 7), "E5M2": (5, 2, 15), "E2M1": (2, 1, 1), "E2M1_OCP": (2, 1, 1)}
#: values that share a byte in the native store (element 2k in the low nibble)
NIBBLE_VALUES = ("E2M1", "E2M1_OCP")


def minifloat_magnitudes(name: str) -> List[Fraction]:
    """Finite magnitudes of the format by magnitude code 0, 1, 2, ... (sign bit excluded)."""
    ebits, mbits, bias = MINIFLOATS[name]
    out = []
    for code in range(1 << (ebits + mbits)):
        e, f = code >> mbits, code & ((1 << mbits) - 1)
        if name == "E4M3" and code == 0x7F:
            break  # S.1111.111 is NaN
        if name == "E5M2" and e == (1 << ebits) - 1:
            break  # infinities and NaNs
        if e == 0:
            out.append(Fraction(f, 1 << mbits) * Fraction(2) ** (1 - bias))
        else:
            out.append((1 + Fraction(f, 1 << mbits)) * Fraction(2) ** (e - bias))
    return out


def minifloat_encode(mag: Fraction, name: str) -> int:
    """Magnitude code of the nearest finite value; a tie goes to the even code (the one whose
    last mantissa bit is 0); magnitudes beyond the largest finite value saturate to it."""
    table = minifloat_magnitudes(name)
    assert mag >= 0
    best = 0
    for code, v in enumerate(table):
        d, db = abs(v - mag), abs(table[best] - mag)
        if d < db or (d == db and code % 2 == 0 and best % 2 == 1):
            best = code
    return best


def sign_and_magnitude(bits: int, fmt: str) -> Tuple[bool, Fraction]:
    width = 32 if fmt == "f32" else 16
    neg = bool((bits >> (width - 1)) & 1)
    return neg, abs(bits_to_fraction(bits, fmt))


def signed_bits(neg: bool, mag: Fraction, fmt: str) -> int:
    """Bit pattern of (-1)^neg * mag, mag representable in fmt; keeps the sign of zero."""
    width = 32 if fmt == "f32" else 16
    return fraction_to_bits(mag, fmt) | (int(neg) << (width - 1))


def native_code(neg: bool, mag_q: Fraction, fmt: str, value: str) -> int:
    """Stored byte (nibble for E2M1) of one element: ``mag_q`` = |x| / |divisor| exactly,
    ``neg`` the sign of the quotient.  round to F, rint, clamp, cast to Q."""
    lo, hi = RANGES[value]
    if value == "E2M1_OCP":
        # the extension: no integer rounding; the quotient in F, clamped, is cast once to the e2m1 grid
        t = min(round_to_format(mag_q, fmt), Fraction(-lo if neg else hi))
        return (int(neg) << 3) | minifloat_encode(t, value)
    k = rint_even(round_to_format(mag_q, fmt))  # |rint(t)|: both roundings are sign-symmetric
    k = min(k, -lo) if neg else min(k, hi)
    if value in ("Q8F", "Q8S"):
        return (-k if neg else k) % 256          # i8 cast: two's complement byte, -0 -> 0
    ebits, mbits, _ = MINIFLOATS[value]
    return (int(neg) << (ebits + mbits)) | minifloat_encode(Fraction(k), value)


def native_decode(code: int, value: str) -> Tuple[bool, Fraction]:
    if value in ("Q8F", "Q8S"):
        v = code - 256 if code >= 128 else code
        return v < 0, Fraction(abs(v))
    ebits, mbits, _ = MINIFLOATS[value]
    return bool(code >> (ebits + mbits)), minifloat_magnitudes(value)[code & ((1 << (ebits + mbits)) - 1)]


def _scale_lookup(e: int, shape, blk_vec, scale_strides):
    if blk_vec is None:
        return 0, e == 0
    bc, start = block_of(e, shape, blk_vec)
    return sum(c * s for c, s in zip(bc, scale_strides)), start


def quantize_tensor_native(x_bits: np.ndarray, fmt: str, shape: Sequence[int], scale_bits: np.ndarray,
                           scale_strides: Sequence[int], block: Sequence[int] | None, value: str,
                           param_fmt: str):
    """Native-store quantization of a contiguous tensor: one byte per element, or (E2M1) two
    nibbles per byte with element 2k in the LOW nibble and element 2k+1 in the high one.
    Returns (bytes uint8, out_scale bit patterns in param_fmt)."""
    n = int(np.prod(shape))
    per_byte = 2 if value in NIBBLE_VALUES else 1
    out = np.zeros(n // per_byte, dtype=np.uint8)
    out_scale = np.zeros(scale_bits.size, dtype=np.uint32 if param_fmt == "f32" else np.uint16)
    blk_vec = None if block is None else (1,) * (len(shape) - len(block)) + tuple(block)
    flat = x_bits.reshape(-1)
    for e in range(n):
        si, start = _scale_lookup(e, shape, blk_vec, scale_strides)
        s_neg, s_mag = sign_and_magnitude(int(scale_bits.reshape(-1)[si]), fmt)
        s_fs = round_to_format(s_mag, param_fmt)
        if start:
            out_scale[si] = signed_bits(s_neg, s_fs, param_fmt)
        d = round_to_format(s_fs, fmt)
        x_neg, x_mag = sign_and_magnitude(int(flat[e]), fmt)
        code = native_code(x_neg != s_neg, x_mag / d, fmt, value)
        if per_byte == 2:
            out[e // 2] |= code << (4 * (e % 2))
        else:
            out[e] = code
    return out, out_scale


def dequantize_tensor_native(codes: np.ndarray, fmt: str, shape: Sequence[int], scale_bits: np.ndarray,
                             scale_strides: Sequence[int], block: Sequence[int] | None, value: str,
                             param_fmt: str) -> np.ndarray:
    """F(scale) * F(q), one rounding to F; a zero product keeps the sign IEEE gives it."""
    n = int(np.prod(shape))
    out = np.zeros(n, dtype=np.uint32 if fmt == "f32" else np.uint16)
    blk_vec = None if block is None else (1,) * (len(shape) - len(block)) + tuple(block)
    for e in range(n):
        si, _ = _scale_lookup(e, shape, blk_vec, scale_strides)
        s_neg, s_mag = sign_and_magnitude(int(scale_bits.reshape(-1)[si]), param_fmt)
        s = round_to_format(s_mag, fmt)
        code = int(codes[e // 2] >> (4 * (e % 2))) & 0xF if value in NIBBLE_VALUES else int(codes[e])
        q_neg, q_mag = native_decode(code, value)
        out[e] = signed_bits(s_neg != q_neg, round_to_format(s * q_mag, fmt), fmt)
    return out
