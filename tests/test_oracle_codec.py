"""Pins of the oracle's fp8 e4m3fn and bf16 codecs (oracle/fp8gemm_oracle.c).

Nothing here retypes the oracle's formulas: the decode table is rebuilt from the OCP bit
layout with exact Fractions, the encoder is checked against a brute-force nearest-even
search over all finite codes and against torch's float8_e4m3fn / bfloat16 casts (torch is a
library here, not the reference).
"""
from fractions import Fraction

import numpy as np
import pytest
import torch


def _decode_table_fraction():
    tab = []
    for v in range(256):
        s, e, m = v >> 7, (v >> 3) & 15, v & 7
        if e == 15 and m == 7:
            tab.append(None)
            continue
        mag = Fraction(m, 8) * Fraction(1, 64) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
        tab.append(-mag if s else mag)
    return tab


def test_decode_all_256_codes(orc):
    tab = _decode_table_fraction()
    got = orc.e4m3fn_decode(np.arange(256, dtype=np.uint8))
    for v in range(256):
        if tab[v] is None:
            assert np.isnan(got[v])
        else:
            assert Fraction(float(got[v])) == tab[v], v
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9
    assert np.signbit(got[0x80]) and got[0x80] == 0.0


def test_decode_matches_torch(orc):
    codes = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = orc.e4m3fn_decode(codes)
    assert np.array_equal(np.isnan(t), np.isnan(got))
    ok = ~np.isnan(t)
    assert np.array_equal(t[ok], got[ok])


def _brute_encode(x, finite_codes, finite_vals):
    """nearest finite code, ties to the code with even mantissa, saturating"""
    ax = abs(x)
    best, bestd = None, None
    for c, v in zip(finite_codes, finite_vals):
        d = abs(Fraction(ax) - v)
        if best is None or d < bestd or (d == bestd and (c & 1) == 0 and (best & 1) == 1):
            best, bestd = c, d
    return best | (0x80 if np.signbit(np.float32(x)) else 0)


def test_encode_brute_force(orc):
    tab = _decode_table_fraction()
    codes = [c for c in range(0x7F)]
    vals = [tab[c] for c in codes]
    rng = np.random.RandomState(3)
    xs = list(rng.standard_normal(300).astype(np.float32) * 3)
    xs += list((rng.rand(200).astype(np.float32) - 0.5) * 1000)
    xs += list((rng.rand(200).astype(np.float32) - 0.5) * 0.05)
    # every midpoint between neighbouring codes (the tie cases) and both float neighbours
    for c in range(0x7E):
        mid = np.float32(float((vals[c] + vals[c + 1]) / 2))
        xs += [mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid]
    xs += [np.float32(448), np.float32(464), np.float32(465), np.float32(1e30), np.float32(-1e30),
           np.float32(0.0), np.float32(-0.0), np.float32(2.0 ** -10), np.float32(2.0 ** -11)]
    xs = np.array(xs, np.float32)
    got = orc.e4m3fn_encode(xs)
    for x, g in zip(xs, got):
        assert g == _brute_encode(float(x), codes, vals), (x, g)


def test_encode_specials(orc):
    got = orc.e4m3fn_encode(np.array([np.inf, -np.inf, np.nan, 1e9, -1e9], np.float32))
    assert got[0] == 0x7E and got[1] == 0xFE and (got[2] & 0x7F) == 0x7F
    assert got[3] == 0x7E and got[4] == 0xFE


def test_encode_matches_torch_in_range(orc):
    rng = np.random.RandomState(5)
    x = np.concatenate([rng.standard_normal(20000) * 100, rng.standard_normal(20000) * 0.01,
                        rng.uniform(-448, 448, 20000)]).astype(np.float32)
    x = x[np.abs(x) <= 448]
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(orc.e4m3fn_encode(x), t)


def test_encode_decode_roundtrip(orc):
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    assert np.array_equal(orc.e4m3fn_encode(orc.e4m3fn_decode(codes)), codes)


def test_bf16_matches_torch(orc):
    rng = np.random.RandomState(7)
    x = np.concatenate([rng.standard_normal(50000) * 50, rng.standard_normal(1000) * 1e-30,
                        np.array([0.0, -0.0, np.inf, -np.inf, 3.0e38, 65504.0])]).astype(np.float32)
    # exact ties: low 16 bits == 0x8000, even and odd upper halves
    u = rng.randint(0, 0x7F00, 2000).astype(np.uint32) << 16 | 0x8000
    x = np.concatenate([x, u.view(np.float32)])
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.bf16_encode(x), t)
    assert np.array_equal(orc.bf16_decode(t), torch.from_numpy(t.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_bf16_nan_stays_nan(orc):
    h = orc.bf16_encode(np.array([np.nan], np.float32))
    assert np.isnan(orc.bf16_decode(h)[0])
