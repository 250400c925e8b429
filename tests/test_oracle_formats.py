"""Pins the oracle's number formats (fp8 e4m3fn and e5m2, half, bf16) against the tables
the reference's own tests hold and against closed forms that do not share code
with the oracle."""
import numpy as np

from oracle import oracle as orc


def _lut(golden):
    vals = golden["fp8e4m3fn_lut"]["values"]
    return np.array([np.nan if v == "nan" else v for v in vals], np.float64)


def test_fp8_decode_matches_reference_table(golden):
    lut = _lut(golden)
    got = orc.fp8_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(lut))
    ok = ~np.isnan(lut)
    assert np.array_equal(got[ok], lut[ok])
    # sign of zero
    assert np.signbit(got[0x80]) and not np.signbit(got[0])


def test_fp8_encode_reference_samples(golden):
    pairs = golden["fp8e4m3fn_from_float"]["pairs"]
    x = np.array([p[0] for p in pairs], np.float32)
    want = np.array([p[1] for p in pairs], np.uint8)
    got = orc.fp8_from_f32(x)
    # the reference compares through float_equal, so -0 (0x80) == +0 (0x00)
    lut = _lut(golden)
    assert np.array_equal(lut[got], lut[want])


def _rne_to_table(x, lut):
    """Definition, independent of the oracle's bit twiddling: nearest finite
    table value, ties to the even code, saturate to 448."""
    pos = lut[:0x7f]                       # 0 .. 448 ascending, codes 0..0x7e
    ax = np.abs(x.astype(np.float64))
    idx = np.searchsorted(pos, ax, side="left")          # pos[idx-1] < ax <= pos[idx]
    idx = np.clip(idx, 1, len(pos) - 1)
    lo, hi = pos[idx - 1], pos[idx]
    dlo, dhi = ax - lo, hi - ax
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((idx % 2) == 0))
    code = np.where(pick_hi, idx, idx - 1)
    code = np.where(ax >= 448.0, 0x7e, code)
    code = np.where(ax == 0.0, 0, code)
    return (code | (np.signbit(x).astype(np.int64) << 7)).astype(np.uint8)


def test_fp8_encode_is_rne_saturating(golden):
    lut = _lut(golden)
    rng = np.random.default_rng(0)
    pos = lut[:0x7f]
    mids = (pos[:-1] + pos[1:]) / 2            # every tie point is exact in float32
    adv = np.concatenate([mids, np.nextafter(mids.astype(np.float32), np.float32(0)),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)),
                          pos, [448.0, 449.0, 464.0, 512.0, 1e6, 3e38, 2.0**-10,
                                2.0**-11, 1e-30]])
    rnd = np.concatenate([rng.normal(0, 1, 200000), rng.normal(0, 100, 200000),
                          rng.uniform(-500, 500, 100000), rng.normal(0, 0.01, 100000)])
    x = np.concatenate([adv, -adv, rnd]).astype(np.float32)
    # float8_impl.hpp:228-246 clips only when the rounded exponent exceeds 15, so
    # floats in (464, 512) come out as exponent 15 / mantissa 7 = the NaN code.
    # quantizelinear and convert clamp to +-448 before the cast, so the path
    # never feeds that interval; it is left out of the property here.
    x = x[(np.abs(x) <= 464) | (np.abs(x) >= 512)]
    got = orc.fp8_from_f32(x)
    want = _rne_to_table(x, lut)
    assert np.array_equal(got, want)
    # specials: +-inf saturate, NaN keeps its sign bit with all-ones payload
    sp = np.array([np.inf, -np.inf, np.nan], np.float32)
    g = orc.fp8_from_f32(sp)
    assert g[0] == 0x7e and g[1] == 0xfe and (g[2] & 0x7f) == 0x7f


def test_fp8_round_trip_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    finite = (codes & 0x7f) != 0x7f
    back = orc.fp8_from_f32(orc.fp8_to_f32(codes))
    assert np.array_equal(back[finite], codes[finite])


def _lut_e5m2(golden):
    return np.array([float(v) for v in golden["fp8e5m2_lut"]["values"]], np.float64)


def test_bf8_decode_matches_reference_table(golden):
    lut = _lut_e5m2(golden)
    got = orc.bf8_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(lut))
    ok = ~np.isnan(lut)
    assert np.array_equal(got[ok], lut[ok])                    # +-inf at 0x7c / 0xfc included
    assert np.isinf(got[0x7c]) and np.isinf(got[0xfc]) and got[0xfc] < 0
    assert np.signbit(got[0x80]) and not np.signbit(got[0])
    # an e5m2 value is the upper byte of the half with the same value
    half = orc.half_to_f32((np.arange(256, dtype=np.uint16) << 8)).astype(np.float64)
    assert np.array_equal(got[ok], half[ok])


def test_bf8_encode_reference_samples(golden):
    pairs = golden["fp8e5m2_from_float"]["pairs"]
    x = np.array([p[0] for p in pairs], np.float32)
    want = np.array([p[1] for p in pairs], np.uint8)
    got = orc.bf8_from_f32(x)
    # test/fp8e5m2.cpp compares through float_equal; every sample but +-7.6e-06 has a non-zero
    # result, and for those two the sign of the zero is kept (test_negative_zero of that file)
    assert np.array_equal(got, want)


def test_bf8_encode_is_rne_saturating(golden):
    """Independent of the oracle's bit arithmetic: nearest finite table value, ties to the even
    code, everything at or beyond 57344 (rounded) saturates to 0x7b."""
    lut = _lut_e5m2(golden)
    pos = lut[:0x7c]                                           # 0 .. 57344 ascending
    rng = np.random.default_rng(1)
    mids = (pos[:-1] + pos[1:]) / 2
    adv = np.concatenate([mids, np.nextafter(mids.astype(np.float32), np.float32(0)),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)), pos,
                          [57344.0, 57345.0, 61439.0, 61440.0, 61441.0, 65536.0, 1e6, 3e38,
                           2.0**-17, 2.0**-18, 1e-30, 1e-45]])
    rnd = np.concatenate([rng.normal(0, 1, 200000), rng.normal(0, 1000, 200000),
                          rng.uniform(-70000, 70000, 100000), rng.normal(0, 1e-4, 100000)])
    x = np.concatenate([adv, -adv, rnd]).astype(np.float32)
    ax = np.abs(x.astype(np.float64))
    idx = np.clip(np.searchsorted(pos, ax, side="left"), 1, len(pos) - 1)
    lo, hi = pos[idx - 1], pos[idx]
    dlo, dhi = ax - lo, hi - ax
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((idx % 2) == 0))
    code = np.where(pick_hi, idx, idx - 1)
    # 61440 is the tie between 57344 (odd code 0x7b) and 65536: it rounds up and out of range,
    # and out of range clips to the largest finite value (float8_impl.hpp:228-233)
    code = np.where(ax >= 57344.0, 0x7b, code)
    want = (code | (np.signbit(x).astype(np.int64) << 7)).astype(np.uint8)
    assert np.array_equal(orc.bf8_from_f32(x), want)
    sp = np.array([np.inf, -np.inf, np.nan], np.float32)
    g = orc.bf8_from_f32(sp)
    assert g[0] == 0x7b and g[1] == 0xfb and (g[2] & 0x7f) == 0x7f


def test_bf8_round_trip_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    finite = (codes & 0x7c) != 0x7c
    back = orc.bf8_from_f32(orc.bf8_to_f32(codes))
    assert np.array_equal(back[finite], codes[finite])


def test_bf8_convert_and_quantize_follow_the_type_limits():
    """convert (op/convert.hpp:64-87): NaN -> numeric_limits::quiet_NaN (0xff), infinities go
    through the constructor (which clips), everything else clamps to +-57344."""
    x = np.array([np.nan, np.inf, -np.inf, 1e9, -1e9, 57344.0, 3.0, -0.0], np.float32)
    got = orc.convert(x, orc.F32, orc.BF8)
    assert list(got) == [0xff, 0x7b, 0xfb, 0x7b, 0xfb, 0x7b, 0x42, 0x80]
    back = orc.convert(np.array([0x7c, 0xfc, 0x7d, 0x42], np.uint8), orc.BF8, orc.F32)
    assert np.isinf(back[0]) and back[1] == -np.inf and np.isnan(back[2]) and back[3] == 3.0


def _check_lut(pairs, from_f32, to_f32):
    bits = np.array([p[0] for p in pairs], np.uint16)
    vals = np.array([float(p[1]) for p in pairs], np.float64)
    fin = np.isfinite(vals)
    got_f = to_f32(bits).astype(np.float64)
    assert np.array_equal(np.isnan(got_f), np.isnan(vals))
    # the tables hold values printed with ~16 significant digits; every entry is
    # exactly representable so float32(value) must convert back to the same bits
    assert np.array_equal(from_f32(vals[fin].astype(np.float32)), bits[fin])
    assert np.allclose(got_f[fin], vals[fin], rtol=1e-7, atol=0)
    inf = np.isinf(vals)
    assert np.array_equal(from_f32(vals[inf].astype(np.float32)), bits[inf])


def test_half_reference_table(golden):
    _check_lut(golden["half_lut"]["pairs"], orc.half_from_f32, orc.half_to_f32)


def test_bf16_reference_table(golden):
    _check_lut(golden["bf16_lut"]["pairs"], orc.bf16_from_f32, orc.bf16_to_f32)


def test_half_to_f32_is_ieee_half_for_all_codes():
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = orc.half_to_f32(codes)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_bf16_to_f32_is_high_half_of_float():
    codes = np.arange(65536, dtype=np.uint16)
    want = (codes.astype(np.uint32) << 16)
    assert np.array_equal(orc.bf16_to_f32(codes).view(np.uint32), want)


def _normal_floats(rng, n):
    x = np.concatenate([rng.normal(0, 1, n), rng.normal(0, 1e-4, n), rng.uniform(-7e4, 7e4, n),
                        rng.normal(0, 1e-7, n)]).astype(np.float32)
    return x[(np.abs(x) >= np.float32(1.1754944e-38)) | (x == 0)]


def test_half_from_f32_rounds_toward_zero():
    """generic_float shifts the mantissa out: conversion is RTZ, overflow to inf
    only from 2^16.  numpy's RNE result is stepped back where it moved away
    from zero."""
    rng = np.random.default_rng(1)
    x = _normal_floats(rng, 100000)
    x = np.concatenate([x, np.float32([1 + 1.5 * 2.0**-11, 65504, 65519, 65520, 65535.9, 65536, 1e9,
                                      -65535, -65536, 2.0**-24, 2.0**-25, 1.9 * 2.0**-24, 6e-8,
                                      6.1e-5, 6.0e-5])])
    h = x.astype(np.float16)
    away = np.abs(h.astype(np.float64)) > np.abs(x.astype(np.float64))
    h = np.where(away, np.nextafter(h, np.float16(0)), h)
    want = h.view(np.uint16).copy()
    big = np.abs(x) >= 65536.0
    want[big] = np.where(x[big] > 0, 0x7c00, 0xfc00)
    got = orc.half_from_f32(x)
    assert np.array_equal(got, want)
    assert orc.half_from_f32(np.float32([1 + 1.5 * 2.0**-11]))[0] == 0x3c00


def test_bf16_from_f32_is_truncation():
    rng = np.random.default_rng(2)
    x = _normal_floats(rng, 100000)
    want = (x.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(orc.bf16_from_f32(x), want)
    assert orc.bf16_from_f32(np.float32([1 + 1.5 * 2.0**-8]))[0] == 0x3f80


def test_convert_saturates_and_keeps_nan():
    # test/ref/convert.cpp: 2*half::max -> half::max, 2*lowest -> lowest, NaN stays NaN
    x = np.float32([2 * 65504.0, -2 * 65504.0, np.nan, np.inf, -np.inf, 1.0009765625 + 2.0**-12])
    got = orc.convert(x, orc.F32, orc.F16)
    assert got[0] == 0x7bff and got[1] == 0xfbff
    assert (got[2] & 0x7c00) == 0x7c00 and (got[2] & 0x3ff) != 0
    assert got[3] == 0x7c00 and got[4] == 0xfc00
    assert got[5] == 0x3c01
    b = orc.convert(np.float32([3.4e38, -3.4e38, 1.0, np.nan]), orc.F32, orc.BF16)
    assert b[0] == 0x7f7f and b[1] == 0xff7f and b[2] == 0x3f80 and (b[3] & 0x7f80) == 0x7f80
