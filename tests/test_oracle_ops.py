"""Pins the oracle's operators against the reference's own known-answer tests
(tests/golden/reference_vectors.json) and against closed forms."""
import numpy as np
import pytest

from oracle import oracle as orc


def _iota(lens, dtype, start=0):
    n = int(np.prod(lens))
    return (np.arange(n, dtype=np.int64) + start).astype(dtype).reshape(lens)


def test_quant_dot_reference_known_answers(golden):
    """test/ref/dot_op.cpp quant_dot_* (2 args, transposed views, alpha/beta via
    apply_alpha_beta.cpp:32-76, batched)."""
    assert len(golden["quant_dot"]) == 15
    for c in golden["quant_dot"]:
        a = _iota(c["a"]["lens"], np.int8)
        b = _iota(c["b"]["lens"], np.int8)
        if c["a_perm"]:
            a = a.transpose(c["a_perm"])
        if c["b_perm"]:
            b = b.transpose(c["b_perm"])
        if c["alpha"] != 1:
            # mul(alpha, A) in float, then convert back to int8 before the GEMM
            af = (np.float32(c["alpha"]) * a.astype(np.float32))
            a = orc.convert(af, orc.F32, orc.I8).reshape(a.shape)
        out = orc.quant_dot(a, b, orc.I8).astype(np.int64)
        if c["uses_c"] and c["beta"] != 0:
            cm = _iota(c["c"]["lens"], np.int32, c["iota_start"]["c"])
            bc = orc.convert(cm.astype(np.float32) * np.float32(c["beta"]), orc.F32, orc.I32)
            out = out + bc.reshape(out.shape)
        assert out.flatten().tolist() == c["gold"], c["name"]


def test_quant_dot_4args_scales(golden):
    # ref_quant_gemm 4-input form: elementwise scale in float, then float GEMM
    c = golden["quant_dot_4args_scales"]
    a = (np.float32(c["a"]) * np.float32(c["scale_a"])).reshape(c["a_lens"])
    b = (np.float32(c["b"]) * np.float32(c["scale_b"])).reshape(c["b_lens"])
    out = orc.gemm(a, b, orc.F32, orc.F32)
    assert out.flatten().tolist() == c["gold"]


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (7, 5, 3), (33, 65, 129), (64, 64, 512)])
def test_quant_dot_int8_equals_integer_matmul(m, n, k):
    rng = np.random.default_rng(m * 1000 + n)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    want = a.astype(np.int64) @ b.astype(np.int64)
    assert np.array_equal(orc.quant_dot(a, b, orc.I8), want)
    # transposed views of [K,M] / [N,K] storage give the same numbers
    at = np.ascontiguousarray(a.T).T
    bt = np.ascontiguousarray(b.T).T
    assert np.array_equal(orc.quant_dot(at, bt, orc.I8), want)


def test_quant_dot_int8_extreme_values_do_not_lose_bits():
    k = 4096
    a = np.full((2, k), -128, np.int8)
    b = np.full((k, 3), -128, np.int8)
    assert np.all(orc.quant_dot(a, b, orc.I8) == 128 * 128 * k)


def test_quant_dot_fp8_is_exact_sum_rounded_once():
    """Every e4m3fn value is an integer multiple of 2^-9, so the dot product is
    an exact integer in units of 2^-18; the reference's double accumulation
    holds it exactly and rounds once to float."""
    rng = np.random.default_rng(3)
    m, n, k = 9, 11, 1024
    codes = np.array([c for c in range(256) if (c & 0x7f) != 0x7f], np.uint8)
    a = rng.choice(codes, (m, k))
    b = rng.choice(codes, (k, n))
    ai = np.rint(orc.fp8_to_f32(a).astype(np.float64) * 512).astype(np.int64)
    bi = np.rint(orc.fp8_to_f32(b).astype(np.float64) * 512).astype(np.int64)
    exact = (ai @ bi).astype(np.float64) / 2.0**18       # < 2^53: exact
    want = exact.astype(np.float32)
    got = orc.quant_dot(a, b, orc.FP8)
    assert got.dtype == np.float32
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_quantizelinear_reference_known_answers(golden):
    for c in golden["quantizelinear"]:
        x = np.float32(c["x"]).reshape(c["lens"])
        s = np.float32(c["scale"]).reshape(c["lens"])
        if c["zp"] is not None:
            z = np.array(c["zp"], np.int8).reshape(c["lens"])
            got = orc.quantizelinear(x, s, z, orc.F32, orc.I8)
        else:
            got = orc.quantizelinear(x, s, None, orc.F32, orc.U8)   # default out type uint8
        assert got.flatten().tolist() == c["gold"], c["name"]


def test_quantizelinear_fp8_reference_case(golden):
    c = golden["quantizelinear_fp8e4m3"]
    x = np.float32(c["x"]).reshape(c["lens"])
    s = np.float32(c["scale"]).reshape(c["lens"])
    z = orc.fp8_from_f32(np.float32(c["zp_float"])).reshape(c["lens"])
    got = orc.quantizelinear(x, s, z, orc.F32, orc.FP8)
    # the reference test builds its gold as fp8(clamp(x/s + zp, -448, 448)) in double
    zf = orc.fp8_to_f32(z).astype(np.float64)
    q = np.clip(x.astype(np.float64) / s.astype(np.float64) + zf, -448, 448)
    want = orc.fp8_from_f32(q.astype(np.float32))
    assert np.array_equal(got, want)
    # hand-checked entries: 0.5/0.25 + 0.6875 = 2.6875 -> 2.75 (0x43); 0.75/0.75+0.75=1.75 (0x3e)
    assert got.flatten()[0] == 0x43 and got.flatten()[1] == 0x3e


def test_quantizelinear_fp8e5m2_reference_case(golden):
    c = golden["quantizelinear_fp8e5m2"]
    x = np.float32(c["x"]).reshape(c["lens"])
    s = np.float32(c["scale"]).reshape(c["lens"])
    z = orc.bf8_from_f32(np.float32(c["zp_float"])).reshape(c["lens"])
    got = orc.quantizelinear(x, s, z, orc.F32, orc.BF8)
    # the reference test builds its gold as fp8(clamp(x/s, -57344, 57344) + zp) in double
    zf = orc.bf8_to_f32(z).astype(np.float64)
    q = np.clip(x.astype(np.float64) / s.astype(np.float64), -57344, 57344) + zf
    want = orc.bf8_from_f32(q.astype(np.float32))
    assert np.array_equal(got, want)
    # hand-checked entries: the zero point 0.6875 is the tie between 0.625 (0x39) and 0.75 (0x3a)
    # and goes to the even code, 0.75; 0.5/0.25 + 0.75 = 2.75 is the tie between 2.5 (0x41) and
    # 3 (0x42) -> 3; 0.75/0.75 + 0.75 = 1.75 (0x3f)
    assert got.flatten()[0] == 0x42 and got.flatten()[1] == 0x3f


def test_quant_dot_fp8e5m2_is_the_exact_sum_rounded_once():
    """quant_dot over e5m2 (op/quant_dot.hpp:62-77 -> gemm in double, float out): every product of
    two e5m2 values is a multiple of 2^-32 below 2^32, so the sum is exact in Python integers."""
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (5, 48)).astype(np.uint8)
    b = rng.integers(0, 256, (48, 7)).astype(np.uint8)
    a[(a & 0x7c) == 0x7c] = 0x3c
    b[(b & 0x7c) == 0x7c] = 0xbc
    a = (a & 0xbf) | 0x20            # exponents 8..15 and 24..: keep magnitudes in a narrow range
    got = orc.quant_dot(a, b, orc.BF8)
    af, bf = orc.bf8_to_f32(a).astype(np.float64), orc.bf8_to_f32(b).astype(np.float64)
    from fractions import Fraction
    for i in range(5):
        for j in range(7):
            exact = sum(Fraction(float(af[i, k])) * Fraction(float(bf[k, j])) for k in range(48))
            assert got[i, j] == np.float32(float(exact)), (i, j)


def test_quantizelinear_int8_ties_to_even_and_true_division():
    x = np.float32([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 1e9, -1e9, 3.0])
    got = orc.quantizelinear(x, np.float32(1.0), np.int8(0), orc.F32, orc.I8)
    assert got.tolist() == [0, 2, 2, 0, -2, -2, 127, -128, 3]
    # x / s is a float division, not a multiply by the reciprocal
    rng = np.random.default_rng(4)
    x = rng.normal(0, 3, 20000).astype(np.float32)
    s = np.float32(0.0123)
    want = np.clip(np.rint(x / s).astype(np.float64), -128, 127).astype(np.int8)
    assert np.array_equal(orc.quantizelinear(x, s, np.int8(0), orc.F32, orc.I8), want)
    want5 = np.clip(np.rint(x / s).astype(np.float64) + 5, -128, 127).astype(np.int8)
    assert np.array_equal(orc.quantizelinear(x, s, np.int8(5), orc.F32, orc.I8), want5)


def test_dequantizelinear_reference_known_answers(golden):
    for c in golden["dequantizelinear"]:
        t = orc.U8 if c["x_type"] == "uint8" else orc.I8
        x = np.array(c["x"], np.uint8 if t == orc.U8 else np.int8).reshape(c["lens"])
        s = np.float32(c["scale"]).reshape(c["lens"])
        z = None if c["zp"] is None else np.array(c["zp"], x.dtype).reshape(c["lens"])
        got = orc.dequantizelinear(x, s, z, t, orc.F32)
        assert got.flatten().tolist() == c["gold"], c["name"]


def test_dequantizelinear_int32_product_is_taken_in_double():
    rng = np.random.default_rng(5)
    acc = rng.integers(-2**30, 2**30, (64, 48)).astype(np.int32)
    zp = rng.integers(-2**20, 2**20, (64, 48)).astype(np.int32)
    s = rng.uniform(1e-4, 1e-2, 48).astype(np.float32)
    got = orc.dequantizelinear(acc, s, zp, orc.I32, orc.F32)
    want = ((acc.astype(np.float64) - zp.astype(np.float64)) * s.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and it is NOT the same as a float32 product for large accumulators
    naive = (acc - zp).astype(np.float32) * s
    assert not np.array_equal(naive, want)


def _strided(c, dtype):
    """Literal of a test case.  A migraphx literal built from a vector is filled
    in logical (row-major index) order whatever its strides are
    (src/include/migraphx/literal.hpp fill), so the strides only change where the
    bytes sit in memory, which is rebuilt here to exercise strided views."""
    raw = np.array(c["data"], np.uint8)
    data = raw if dtype == np.uint8 else raw.view(np.int8)
    lens = c["shape"]["lens"]
    x = data.reshape(lens)
    strides = c["shape"].get("strides")
    if strides and len(lens) == 2 and strides[0] < strides[1]:
        x = np.ascontiguousarray(x.T).T          # same values, column-major storage
        assert [st // x.itemsize for st in x.strides] == strides
    if c["multibroadcast"]:
        x = np.broadcast_to(x, c["multibroadcast"])
    return x


def test_unpack_int4_reference_known_answers(golden):
    assert len(golden["unpack_int4"]) == 6
    for c in golden["unpack_int4"]:
        dt = np.int8 if c["shape"]["type"] == "int8" else np.uint8
        got = orc.unpack_int4(_strided(c, dt), c["axis"])
        assert got.astype(np.int64).flatten().tolist() == c["gold"], c["name"]


def test_pack_int4_reference_known_answers(golden):
    assert len(golden["pack_int4"]) == 6
    for c in golden["pack_int4"]:
        dt = np.int8 if c["shape"]["type"] == "int8" else np.uint8
        got = orc.pack_int4(_strided(c, dt), c["axis"])
        assert got.view(np.uint8).flatten().tolist() == c["gold"], c["name"]


def test_pack_unpack_round_trip_and_odd_axis():
    rng = np.random.default_rng(6)
    u = rng.integers(0, 16, (5, 12), dtype=np.uint8)
    assert np.array_equal(orc.unpack_int4(orc.pack_int4(u)), u)
    s = rng.integers(-8, 8, (5, 12)).astype(np.int8)
    assert np.array_equal(orc.unpack_int4(orc.pack_int4(s)), s)
    u4 = u[:4]
    assert np.array_equal(orc.unpack_int4(orc.pack_int4(u4, 0), 0), u4)
    with pytest.raises(ValueError):
        orc.pack_int4(np.zeros((3, 5), np.uint8))


def _matmulnbits(c):
    """The graph parse_matmulnbits.cpp:42-159 builds, evaluated op by op."""
    n, nblk, blob = c["b_lens"]
    blk = blob * 2
    a_lens = c["a_lens"]
    k = a_lens[-1]
    a = (np.arange(int(np.prod(a_lens)), dtype=np.float32) if c["a"] == "iota"
         else np.float32(c["a"])).reshape(a_lens)
    b = np.array(c["b"], np.uint8).reshape(n, -1)
    q = orc.unpack_int4(b)[:, :k]
    scales = np.float32(c["scales"]).reshape(n, -1)
    s_full = np.repeat(scales, blk, axis=1)[:, :k]
    if c["zp"] is None:
        z_full = np.full((n, k), 8, np.uint8)
    else:
        z = orc.unpack_int4(np.array(c["zp"], np.uint8).reshape(n, -1))[:, :nblk]
        z_full = np.repeat(z, blk, axis=1)[:, :k]
    w = orc.dequantizelinear(np.ascontiguousarray(q), np.ascontiguousarray(s_full),
                             np.ascontiguousarray(z_full), orc.U8, orc.F32)
    wt = w.T
    if a.ndim == 1:
        return orc.gemm(a[None, :], wt, orc.F32, orc.F32)[0]
    if a.ndim > 2:
        wt = np.broadcast_to(wt, a.shape[:-2] + wt.shape)
    return orc.gemm(a, wt, orc.F32, orc.F32)


def test_matmulnbits_reference_known_answers(golden):
    """test/onnx/verify/matmulnbits_tests.cpp: pins nibble order, block layout,
    the default zero point 8, packed zero points, runt blocks and the
    transpose feeding dot."""
    assert len(golden["matmulnbits"]) == 4
    for c in golden["matmulnbits"]:
        got = _matmulnbits(c).flatten()
        gold = np.float32(c["gold"])
        assert got.shape == gold.shape, c["name"]
        assert np.allclose(got, gold, rtol=2e-6, atol=1e-5), (c["name"], got, gold)


def test_dot_half_accumulates_in_double_and_truncates():
    rng = np.random.default_rng(7)
    m, n, k = 3, 5, 257
    a = orc.half_from_f32(rng.normal(0, 1, (m, k)).astype(np.float32))
    b = orc.half_from_f32(rng.normal(0, 1, (k, n)).astype(np.float32))
    af = orc.half_to_f32(a).astype(np.float64)
    bf = orc.half_to_f32(b).astype(np.float64)
    s = np.zeros((m, n))
    for kk in range(k):                          # same order as gemm_naive
        s += np.outer(af[:, kk], bf[kk, :])
    want = orc.half_from_f32(s.astype(np.float32))
    assert np.array_equal(orc.dot(a, b, orc.F16), want)


def test_w4a16_composite_matches_stepwise_definition():
    rng = np.random.default_rng(8)
    m, n, k, g = 2, 6, 256, 128
    wq = rng.integers(0, 16, (n, k), dtype=np.uint8)
    packed = orc.pack_int4(wq)
    scales = orc.half_from_f32(rng.uniform(0.005, 0.02, (n, k // g)).astype(np.float32))
    a = orc.half_from_f32(rng.normal(0, 1, (m, k)).astype(np.float32))
    got = orc.w4a16_matmul(a, packed, scales, 8, g)
    sf = np.repeat(orc.half_to_f32(scales), g, axis=1).astype(np.float64)
    w = orc.half_from_f32(((wq.astype(np.float64) - 8) * sf).astype(np.float32))
    want = orc.dot(a, w.T, orc.F16)
    assert np.array_equal(got, want)
