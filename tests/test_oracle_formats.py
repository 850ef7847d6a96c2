"""Pins the oracle's scalar formats (OCP E4M3, bf16) without retyping its formulas.

E4M3 decode: closed form over all 256 codes written with exact rationals, the torch CPU
view cast, and ROCm's hip_fp8.h host cast (the library the reference's host oracle calls,
projects/skinny_gemm/test.cu:33).  E4M3 encode: brute-force nearest-representable search
with ties to the even mantissa, torch's CPU cast, and hip_fp8.h's host cast
(projects/common.cuh:103 uses it with SATFINITE).  bf16: torch's CPU cast.
"""
import os
import subprocess
from fractions import Fraction

import numpy as np
import pytest
import torch


def _closed_form_table():
    vals = []
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            vals.append(None)
            continue
        if e == 0:
            v = Fraction(m, 8) * Fraction(1, 64)
        else:
            v = (1 + Fraction(m, 8)) * (Fraction(2) ** (e - 7))
        vals.append(-v if s else v)
    return vals


def test_decode_closed_form(oracle):
    got = oracle.e4m3_decode(np.arange(256, dtype=np.uint8))
    table = _closed_form_table()
    for c, v in enumerate(table):
        if v is None:
            assert np.isnan(got[c])
        else:
            assert Fraction(float(got[c])) == v, c
    assert got[0x7E] == 448.0 and got[0xFE] == -448.0
    assert got[0x38] == 1.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9
    assert np.signbit(got[0x80]) and got[0x80] == 0.0


def test_decode_matches_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = oracle.e4m3_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))


def _brute_encode(xs):
    """Nearest finite E4M3 value, ties to the code with an even mantissa, saturating."""
    table = _closed_form_table()
    pos = [(float(table[c]), c) for c in range(0x7F)]  # 0x00..0x7e ascending
    grid = np.array([p[0] for p in pos], dtype=np.float64)
    out = np.empty(xs.shape, np.uint8)
    ax = np.abs(xs.astype(np.float64))
    hi = np.searchsorted(grid, ax, side="left").clip(0, len(grid) - 1)
    lo = (hi - 1).clip(0)
    dlo, dhi = ax - grid[lo], grid[hi] - ax
    pick = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    pick = np.where(ax >= grid[-1], len(grid) - 1, pick)  # saturate (also +inf)
    out[:] = pick.astype(np.uint8)
    out |= (np.signbit(xs).astype(np.uint8) << 7)
    return out


def _sample_f32():
    rng = np.random.default_rng(1234)
    parts = [
        rng.standard_normal(300000).astype(np.float32) * 100,
        rng.standard_normal(300000).astype(np.float32),
        rng.standard_normal(200000).astype(np.float32) * 1e-2,
        (rng.random(200000).astype(np.float32) * 1000 - 500),
    ]
    # every midpoint between neighbouring codes, and its fp32 neighbours
    table = [float(v) for v in _closed_form_table()[:0x7F]]
    mids = np.array([(a + b) / 2 for a, b in zip(table[:-1], table[1:])], dtype=np.float32)
    parts += [mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)), -mids]
    parts += [np.array([0.0, -0.0, 448.0, 449.0, 463.9, 464.0, 465.0, 1e9, -1e9, np.inf, -np.inf,
                        2.0 ** -10, 1.5 * 2.0 ** -9, 17.0, 19.0, 1.0625], dtype=np.float32)]
    return np.concatenate(parts)


def test_encode_brute_force_all_bf16(oracle):
    bits = np.arange(65536, dtype=np.uint32)
    xs = (bits << 16).view(np.float32)
    finite = ~np.isnan(xs)
    got = oracle.e4m3_encode(xs)
    want = _brute_encode(xs[finite])
    assert np.array_equal(got[finite], want)
    assert np.all((got[~finite] & 0x7F) == 0x7F)


def test_encode_brute_force_fp32_sample(oracle):
    xs = _sample_f32()
    assert np.array_equal(oracle.e4m3_encode(xs), _brute_encode(xs))


def test_encode_known_ties(oracle):
    enc = lambda v: int(oracle.e4m3_encode(np.array([v], np.float32))[0])
    dec = lambda c: float(oracle.e4m3_decode(np.array([c], np.uint8))[0])
    assert dec(enc(17.0)) == 16.0      # tie -> even mantissa
    assert dec(enc(19.0)) == 20.0
    assert dec(enc(1.0625)) == 1.0
    assert dec(enc(2.0 ** -10)) == 0.0  # tie between 0 and 2^-9 -> 0
    assert dec(enc(1.5 * 2.0 ** -9)) == 2.0 ** -8
    assert enc(464.0) == 0x7E and enc(1e30) == 0x7E and enc(float("inf")) == 0x7E
    assert enc(float("-inf")) == 0xFE
    assert enc(float("nan")) & 0x7F == 0x7F


def test_encode_matches_torch_in_range(oracle):
    xs = _sample_f32()
    xs = xs[np.abs(xs) <= 448.0]
    want = torch.from_numpy(xs).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(oracle.e4m3_encode(xs), want)


def test_roundtrip_all_codes(oracle):
    codes = np.arange(256, dtype=np.uint8)
    vals = oracle.e4m3_decode(codes)
    back = oracle.e4m3_encode(vals)
    ok = (codes & 0x7F) != 0x7F
    assert np.array_equal(back[ok], codes[ok])


def _helper():
    import oracle as orc
    if not os.path.exists(orc.HIPFP8_HOST_CAST):
        orc.build()
    return orc.HIPFP8_HOST_CAST


def test_decode_matches_hip_fp8_header(oracle):
    out = subprocess.run([_helper(), "decode"], check=True, capture_output=True, text=True).stdout
    got = oracle.e4m3_decode(np.arange(256, dtype=np.uint8)).view(np.uint32)
    for line in out.strip().splitlines():
        c, bits = line.split()
        c, bits = int(c), int(bits, 16)
        if (c & 0x7F) == 0x7F:
            assert (bits & 0x7FFFFFFF) > 0x7F800000
        else:
            assert bits == int(got[c]), c


def test_encode_matches_hip_fp8_header(oracle):
    xs = _sample_f32()[::7]
    xs = xs[~np.isnan(xs)]
    text = "\n".join("%08x" % b for b in xs.view(np.uint32))
    out = subprocess.run([_helper(), "encode"], input=text, check=True, capture_output=True, text=True).stdout
    want = np.array([int(t) for t in out.split()], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3_encode(xs), want)


def test_bf16_matches_torch(oracle):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, size=500000, dtype=np.uint64).astype(np.uint32)
    edge = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F800000,
                     0xFF800000, 0x00000001, 0x80000000, 0x7F7F8000], dtype=np.uint32)
    xs = np.concatenate([bits, edge]).view(np.float32)
    xs = xs[~np.isnan(xs)]
    want = torch.from_numpy(xs).bfloat16().view(torch.int16).numpy().view(np.uint16)
    got = oracle.bf16_from_f32(xs)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.bf16_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)
    assert np.isnan(oracle.bf16_to_f32(oracle.bf16_from_f32(np.array([np.nan], np.float32))))[0]
