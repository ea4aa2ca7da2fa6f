"""Exact-rational statement of the quantize/dequantize arithmetic, independent
of the C oracle: every float operation is carried out on ``fractions.Fraction``
and rounded ONCE, directly to the target format, with round-half-to-even.

It is the mathematical definition the specification appeals to ("the correctly
rounded quotient in F", "round half to even", "two's-complement field i at bits
[i*b,(i+1)*b)"), written so that a dropped rounding step, a reciprocal multiply,
round-half-away, a transposed field order or a wrong scale index in the oracle
shows up as a mismatch.  Pure Python, small inputs only, finite values only.

Specification followed: crates/cubek-quant/src/quantize.rs:19-31,61-81,
src/dequantize.rs:22-25,86-118, src/layout/scales.rs:144-160,179-194,
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
    return {"Q8F": 8, "Q8S": 8, "E4M3": 8, "E5M2": 8, "Q4F": 4, "Q4S": 4, "E2M1": 4,
            "Q2F": 2, "Q2S": 2}[value]


RANGES = {"Q8F": (-128, 127), "Q8S": (-127, 127), "Q4F": (-8, 7), "Q4S": (-7, 7),
          "Q2F": (-2, 1), "Q2S": (-1, 1), "E2M1": (-6, 6), "E4M3": (-448, 448),
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
            out[e0 + i] = fraction_to_bits(round_to_format(s * c, fmt), fmt)
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
