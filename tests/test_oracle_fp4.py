"""The oracle's fp4 (e2m1) casts and pack/unpack against the reference's known answers
(test/ref/pack_unpack_fp4.cpp) and against what the format's definition fixes."""
import math

import numpy as np
import pytest

from oracle import oracle as orc

E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def test_reference_known_answers(golden):
    cases = {c["name"]: c for c in golden["fp4"]}
    c = cases["pack_fp4"]
    x = np.float32(c["input"]).reshape(c["lens"])
    assert orc.pack_fp4(x, c["axis"]).flatten().tolist() == c["gold_bytes"]
    c = cases["unpack_fp4"]
    b = np.uint8(c["input_bytes"]).reshape(c["lens"])
    assert orc.fp8_to_f32(orc.unpack_fp4(b, c["axis"])).flatten().tolist() == c["gold"]
    c = cases["pack_unpack_fp4"]
    x = np.float32(c["input"]).reshape(c["lens"])
    back = orc.fp8_to_f32(orc.unpack_fp4(orc.pack_fp4(x, c["axis"]), c["axis"]))
    assert back.flatten().tolist() == c["gold"]


def test_all_codes_follow_the_e2m1_definition():
    # sign, two exponent bits (bias 1), one mantissa bit; exponent 0 is the subnormal 0 / 0.5
    for code in range(16):
        s, e, m = code >> 3, (code >> 1) & 3, code & 1
        want = (m * 0.5) if e == 0 else (1 + 0.5 * m) * 2.0 ** (e - 1)
        got = orc.fp4_to_f32(code)
        assert got == (-want if s else want)
        assert math.copysign(1.0, got) == (-1.0 if s else 1.0)
        assert orc.fp4_from_f32(got) == code          # every code round-trips, -0 included


def test_rounding_is_nearest_with_ties_to_the_even_code():
    for i in range(7):
        lo, hi = E2M1[i], E2M1[i + 1]
        tie = (lo + hi) / 2
        even = i if i % 2 == 0 else i + 1
        for sign, bit in ((1.0, 0), (-1.0, 8)):
            assert orc.fp4_from_f32(sign * tie) == even | bit
            assert orc.fp4_from_f32(sign * np.nextafter(np.float32(tie), np.float32(0))) == i | bit
            assert orc.fp4_from_f32(sign * np.nextafter(np.float32(tie), np.float32(10))) == (i + 1) | bit
    # nearest neighbour on a fine grid, by brute force over the eight magnitudes
    for x in np.linspace(-7, 7, 2801, dtype=np.float32):
        code = orc.fp4_from_f32(x)
        d = [abs(abs(float(x)) - v) for v in E2M1]
        assert d[code & 7] == min(d)


def test_saturation_nan_and_signed_zero():
    assert orc.fp4_from_f32(6.0) == 7 and orc.fp4_from_f32(1e30) == 7
    assert orc.fp4_from_f32(float("inf")) == 7 and orc.fp4_from_f32(float("-inf")) == 15
    assert orc.fp4_from_f32(float("nan")) == 0
    assert orc.fp4_from_f32(-0.0) == 8 and orc.fp4_from_f32(0.0) == 0
    assert orc.fp4_from_f32(-0.2) == 8            # rounds to -0


@pytest.mark.parametrize("axis", [0, 1, -1])
def test_pack_unpack_axes(axis):
    rng = np.random.default_rng(4)
    x = rng.uniform(-7, 7, (4, 6, 8)).astype(np.float32)
    packed = orc.pack_fp4(x, axis)
    shp = list(x.shape)
    shp[axis] //= 2
    assert list(packed.shape) == shp
    un = orc.fp8_to_f32(orc.unpack_fp4(packed, axis))
    assert un.shape == x.shape
    want = np.vectorize(lambda v: orc.fp4_to_f32(orc.fp4_from_f32(v)))(x).astype(np.float32)
    assert np.array_equal(un, want)
    # low nibble = even element along the axis
    ev = np.take(x, range(0, x.shape[axis], 2), axis=axis)
    lo = np.vectorize(orc.fp4_from_f32)(ev).astype(np.uint8)
    assert np.array_equal(packed & 0xF, lo)
    with pytest.raises(ValueError):
        orc.pack_fp4(np.zeros((2, 3), np.float32), 1)
