"""Pins the scalar formats of the oracle against what the specifications fix:
OCP FP8 E4M3 (e4m3fn), IEEE binary16 and bfloat16 -- exhaustive tables, every midpoint,
saturation and special values, plus library cross-checks (numpy float16, torch bf16 / e4m3fn)."""
from fractions import Fraction

import numpy as np
import pytest
import torch


def _e4m3_value(code):
    """OCP FP8 E4M3 straight from the format definition: S.EEEE.MMM, bias 7, no infinities,
    S.1111.111 = NaN, subnormals (E = 0) = M * 2^-9."""
    s, e, m = code >> 7, (code >> 3) & 15, code & 7
    if e == 15 and m == 7:
        return None
    v = Fraction(m, 8) * Fraction(2) ** (1 - 7) if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
    return -v if s else v


def test_e4m3_decode_exhaustive(oracle):
    dec = oracle.e4m3_decode(np.arange(256, dtype=np.uint8))
    for c in range(256):
        v = _e4m3_value(c)
        if v is None:
            assert np.isnan(dec[c])
        else:
            assert Fraction(float(dec[c])) == v, c
    assert dec[0x7E] == 448.0 and dec[0xFE] == -448.0 and dec[0x01] == 2.0 ** -9 and dec[0x08] == 2.0 ** -6


def test_e4m3_encode_identity_on_all_codes(oracle):
    codes = np.array([c for c in range(256) if _e4m3_value(c) is not None and c != 0x80], dtype=np.uint8)
    assert (oracle.e4m3_encode(oracle.e4m3_decode(codes)) == codes).all()
    assert oracle.e4m3_encode(np.float32([-0.0]))[0] == 0x80


def test_e4m3_encode_midpoints_ties_to_even_and_neighbours(oracle):
    for c in range(0x7E):  # all adjacent positive pairs (c, c+1)
        lo, hi = float(_e4m3_value(c)), float(_e4m3_value(c + 1))
        mid = np.float32((lo + hi) / 2)
        assert float(mid) == (lo + hi) / 2  # midpoints are exact in fp32
        even = c if c % 2 == 0 else c + 1
        below, above = np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9))
        got = oracle.e4m3_encode(np.array([mid, below, above, -mid, -below, -above], np.float32))
        assert list(got) == [even, c, c + 1, even | 0x80, c | 0x80, (c + 1) | 0x80], c


def test_e4m3_encode_saturation_nan_and_tiny(oracle):
    x = np.float32([448.0, 448.00003, 449.0, 463.9, 464.0, 480.0, 1e9, np.inf, -np.inf, -1e30, np.nan, 2.0 ** -10, 2.0 ** -10 * 1.0001,
                    2.0 ** -11, 1e-30, 0.0])
    want = [0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0xFE, 0x7F, 0x00, 0x01, 0x00, 0x00, 0x00]
    assert list(oracle.e4m3_encode(x)) == want


def test_e4m3_encode_matches_torch_in_range(oracle, rng):
    # torch.float8_e4m3fn is a library routine (RNE, non-saturating): it must agree wherever |x| <= 448
    x = np.concatenate([rng.uniform(-448, 448, 200000), rng.normal(0, 1, 200000), rng.normal(0, 1e-2, 100000)]).astype(np.float32)
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert (oracle.e4m3_encode(x) == t).all()


def test_f16_conversions_against_numpy(oracle, rng):
    allbits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(allbits)
    ref = allbits.view(np.float16).astype(np.float32)
    assert ((f == ref) | (np.isnan(f) & np.isnan(ref))).all()
    x = np.concatenate([rng.normal(0, 1, 300000), rng.normal(0, 300, 100000), rng.normal(0, 1e-6, 100000),
                        [65504, 65519.9, 65520, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 0.0, -0.0, np.inf]]).astype(np.float32)
    assert (oracle.f32_to_f16_bits(x) == x.astype(np.float16).view(np.uint16)).all()
    # every fp16 midpoint: exact ties must go to even
    fin = allbits[(allbits & 0x7C00) != 0x7C00]
    fin = fin[fin < 0x7BFF]
    lo, hi = fin.view(np.float16).astype(np.float64), (fin + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert (oracle.f32_to_f16_bits(mid) == np.where(fin % 2 == 0, fin, fin + 1)).all()


def test_bf16_conversions_against_torch(oracle, rng):
    x = np.concatenate([rng.normal(0, 1, 300000), rng.normal(0, 1e20, 1000), rng.normal(0, 1e-20, 1000), [0.0, -0.0, np.inf, -np.inf, 3.3895314e38]]).astype(np.float32)
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (oracle.f32_to_bf16_bits(x) == t).all()
    bits = np.arange(65536, dtype=np.uint16)
    back = oracle.bf16_bits_to_f32(bits)
    ref = (bits.astype(np.uint32) << 16).view(np.float32)
    assert ((back == ref) | (np.isnan(back) & np.isnan(ref))).all()


def test_code_index_is_monotone(oracle):
    codes = np.array([c for c in range(256) if _e4m3_value(c) is not None], dtype=np.uint8)
    vals = oracle.e4m3_decode(codes)
    idx = oracle.e4m3_code_index(codes)
    order = np.argsort(vals, kind="stable")
    assert (np.diff(idx[order]) >= 0).all()
    assert idx[codes == 0x7E][0] == 126 and idx[codes == 0xFE][0] == -126
