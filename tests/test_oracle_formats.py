"""Pins the oracle's float-format helpers against library routines and tables.

bf16 <- torch's CPU conversion, f16 <- numpy's, e4m3/e5m2/e2m1 <- brute-force
nearest-value search over the decoded table (ties to even code).
"""
import ctypes

import numpy as np
import torch


def _f32_samples():
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=200_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[np.isfinite(f)]
    special = np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 5.96e-8,
                        2.98e-8, 2.9802322e-8, 6.1e-5, 6.09e-5, 3.3895314e38, 3.4e38, 1.0039062,
                        1.00390625, 1.01171875, 0.99609375], dtype=np.float32)
    # values around bf16/f16 rounding midpoints
    base = rng.normal(0, 100, 50_000).astype(np.float32)
    mid16 = (base.view(np.uint32) & 0xFFFF0000 | 0x8000).view(np.float32)
    mid13 = (base.view(np.uint32) & 0xFFFFE000 | 0x1000).view(np.float32)
    return np.concatenate([f, special, -special, base, mid16, mid13,
                           np.nextafter(mid16, np.float32(np.inf)),
                           np.nextafter(mid13, np.float32(-np.inf))])


def test_bf16_matches_torch(oracle):
    L = oracle.lib()
    f = _f32_samples()
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.cqo_f32_to_bf16(ctypes.c_float(float(v))) for v in f[:60_000]], dtype=np.uint16)
    assert np.array_equal(got, want[:60_000])
    # the vectorised numpy helper used to build test inputs agrees as well
    from cubek_amd.scheme import ElemType
    assert np.array_equal(oracle.to_bits(f, ElemType.BF16), want)
    # widening is exact for all 65536 patterns
    allb = np.arange(65536, dtype=np.uint32)
    wide = (allb << 16).view(np.float32)
    got_w = np.array([L.cqo_bf16_to_f32(int(b)) for b in range(0, 65536, 7)], dtype=np.float32)
    fin = ~np.isnan(wide[::7])  # NaN payloads do not survive the float->double ctypes hop
    assert np.array_equal(got_w.view(np.uint32)[fin], wide[::7].view(np.uint32)[fin])
    assert np.all(np.isnan(got_w[~fin]))


def test_f16_matches_numpy(oracle):
    L = oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([L.cqo_f16_to_f32(int(b)) for b in range(65536)], dtype=np.float32)
    fin = ~np.isnan(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    assert np.all(np.isnan(got[~fin]))
    f = _f32_samples()[:80_000]
    with np.errstate(over="ignore"):
        want_h = f.astype(np.float16).view(np.uint16)
    got_h = np.array([L.cqo_f32_to_f16(ctypes.c_float(float(v))) for v in f], dtype=np.uint16)
    assert np.array_equal(got_h, want_h)


def _table_encode(decode, ncodes, x):
    """Nearest representable value; ties -> even code; saturate."""
    vals = np.array([decode(c) for c in range(ncodes)], dtype=np.float64)
    best = None
    for c in range(ncodes):
        if not np.isfinite(vals[c]):
            continue
        d = abs(vals[c] - abs(x))
        if best is None or d < best[0] or (d == best[0] and c % 2 == 0 and best[1] % 2 == 1):
            best = (d, c)
    return best[1]


def test_minifloats_match_table_search(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(3)
    for name, ncodes, top in (("e4m3", 0x7F, 448.0), ("e5m2", 0x7C, 57344.0), ("e2m1", 8, 6.0)):
        enc = getattr(L, f"cqo_f32_to_{name}")
        dec = getattr(L, f"cqo_{name}_to_f32")
        # decode table is monotone and starts at 0
        vals = [dec(c) for c in range(ncodes)]
        assert vals[0] == 0.0 and all(b > a for a, b in zip(vals, vals[1:])) and vals[-1] == top
        # sign bit mirrors
        signbit = {"e4m3": 0x80, "e5m2": 0x80, "e2m1": 0x8}[name]
        assert dec(signbit | 3) == -dec(3)
        xs = list(rng.uniform(0, top * 1.05, 3000)) + [float(i) for i in range(0, int(min(top, 600)) + 2)]
        xs += [(a + b) / 2 for a, b in zip(vals, vals[1:])]  # exact midpoints
        for x in xs:
            x32 = float(np.float32(x))
            want = _table_encode(dec, ncodes, min(x32, top))
            assert enc(ctypes.c_float(x32)) == want, (name, x32)
            assert enc(ctypes.c_float(-x32)) == (want | signbit), (name, -x32)
    # published OCP values
    assert [L.cqo_e2m1_to_f32(c) for c in range(8)] == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert L.cqo_e4m3_to_f32(0x7E) == 448.0 and L.cqo_e4m3_to_f32(0x01) == 2.0 ** -9
    assert L.cqo_e5m2_to_f32(0x7B) == 57344.0 and L.cqo_e5m2_to_f32(0x01) == 2.0 ** -16


def test_fp8_matches_torch_float8(oracle):
    """e4m3 / e5m2 against torch's CPU float8 conversions (a library routine): every byte
    decodes to the same value, and in-range floats encode to the same byte."""
    import torch

    L = oracle.lib()
    rng = np.random.default_rng(8)
    for name, tdt, top in (("e4m3", torch.float8_e4m3fn, 448.0), ("e5m2", torch.float8_e5m2, 57344.0)):
        enc = getattr(L, f"cqo_f32_to_{name}")
        dec = getattr(L, f"cqo_{name}_to_f32")
        decoded = torch.arange(256, dtype=torch.uint8).view(tdt).to(torch.float32).numpy()
        for code in range(256):
            ours = dec(code)
            if np.isfinite(decoded[code]):
                assert ours == decoded[code], (name, code)
        xs = np.concatenate([rng.uniform(-top, top, 20000), rng.normal(0, 1, 20000), rng.normal(0, 2.0 ** -8, 5000),
                             np.arange(-448, 449, dtype=np.float64)]).astype(np.float32)
        xs = xs[np.abs(xs) <= top]
        want = torch.from_numpy(xs).to(tdt).view(torch.uint8).numpy()
        got = np.array([enc(ctypes.c_float(float(v))) for v in xs], dtype=np.uint8)
        # -0.0 and +0.0: both sides keep the sign of a float cast
        assert np.array_equal(got, want), (name, xs[got != want][:5], got[got != want][:5], want[got != want][:5])
