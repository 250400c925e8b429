"""GPU parity of the elementwise operators of the quantized path, through the
C ABI, against the CPU oracle.  All of them are required bit-exact."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests.gpu_util import dev, half_dev, bf16_dev, half_bits, bf16_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from amdmigraphx_amd import ops
    return ops


def _adversarial_f32(rng, n):
    x = np.concatenate([rng.standard_normal(n), rng.standard_normal(n) * 40,
                        rng.uniform(-500, 500, n), rng.standard_normal(n) * 1e-3,
                        [0.0, -0.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 1e9, -1e9, np.inf, -np.inf,
                         np.nan, 448, 449, 464, 470, -470, 1e-30, 2.0**-10, 2.0**-9]])
    return x.astype(np.float32)


def test_reference_quantizelinear_known_answers_on_gpu(ops, golden):
    for c in golden["quantizelinear"]:
        x = np.float32(c["x"]).reshape(c["lens"])
        s = np.float32(c["scale"]).reshape(c["lens"])
        if c["zp"] is not None:
            z = np.array(c["zp"], np.int8).reshape(c["lens"])
            got = ops.quantizelinear(dev(x), dev(s), dev(z), ops.DT.I8)
        else:
            got = ops.quantizelinear(dev(x), dev(s), None, ops.DT.U8)
        assert got.cpu().numpy().flatten().tolist() == c["gold"], c["name"]


def test_reference_dequantizelinear_known_answers_on_gpu(ops, golden):
    for c in golden["dequantizelinear"]:
        dt = np.uint8 if c["x_type"] == "uint8" else np.int8
        x = np.array(c["x"], dt).reshape(c["lens"])
        s = np.float32(c["scale"]).reshape(c["lens"])
        z = None if c["zp"] is None else dev(np.array(c["zp"], dt).reshape(c["lens"]))
        got = ops.dequantizelinear(dev(x), dev(s), z)
        assert got.cpu().numpy().flatten().tolist() == c["gold"], c["name"]


@pytest.mark.parametrize("scale", [1.0 / 32, 0.0123, 3.7])
@pytest.mark.parametrize("zp", [0, 5, -7])
def test_quantize_f32_to_int8(ops, scale, zp):
    rng = np.random.default_rng(0)
    x = _adversarial_f32(rng, 5000).reshape(1, -1)
    want = orc.quantizelinear(x, np.float32(scale), np.int8(zp), orc.F32, orc.I8)
    got = ops.quantizelinear(dev(x), dev(np.float32([scale])), dev(np.int8([zp])), ops.DT.I8)
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("scale,zp", [(1.0 / 32, 0), (0.0123, 5), (3.7, -7)])
def test_quantize_f32_to_int8_whole_tensor_form(ops, scale, zp):
    """A dense tensor of a multiple of 16 elements with one scale and zero point takes the
    16-elements-per-thread kernel: same answers, ties, NaN and infinities included."""
    rng = np.random.default_rng(2)
    x = _adversarial_f32(rng, 5000)
    x = x[:x.size // 64 * 64].reshape(-1, 64)
    want = orc.quantizelinear(x, np.float32(scale), np.int8(zp), orc.F32, orc.I8)
    got = ops.quantizelinear(dev(x), dev(np.float32([scale])), dev(np.int8([zp])), ops.DT.I8)
    assert np.array_equal(got.cpu().numpy(), want)
    got = ops.quantizelinear(dev(x), dev(np.float32([scale])), None, ops.DT.I8)
    assert np.array_equal(got.cpu().numpy(), orc.quantizelinear(x, np.float32(scale), np.int8(0), orc.F32, orc.I8))


def test_quantize_per_column_and_per_row(ops):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((37, 101)) * 3).astype(np.float32)
    sc = rng.uniform(0.01, 0.1, 101).astype(np.float32)
    sr = rng.uniform(0.01, 0.1, 37).astype(np.float32)
    assert np.array_equal(ops.quantizelinear(dev(x), dev(sc), None, ops.DT.I8).cpu().numpy(),
                          orc.quantizelinear(x, sc, None, orc.F32, orc.I8))
    assert np.array_equal(ops.quantizelinear(dev(x), dev(sr), None, ops.DT.I8).cpu().numpy(),
                          orc.quantizelinear(x, sr, None, orc.F32, orc.I8))


@pytest.mark.parametrize("xt", ["f32", "f16", "bf16"])
def test_quantize_to_fp8(ops, xt):
    rng = np.random.default_rng(2)
    x = _adversarial_f32(rng, 20000).reshape(1, -1)
    s = np.float32(np.nanmax(np.abs(x[np.isfinite(x)])) / 448)
    if xt == "f32":
        want = orc.quantizelinear(x, s, None, orc.F32, orc.FP8)
        got = ops.quantizelinear(dev(x), dev(np.float32([s])), None, ops.DT.FP8)
    elif xt == "f16":
        xb, sb = orc.half_from_f32(x), orc.half_from_f32(np.float32([0.37]))
        want = orc.quantizelinear(xb, sb, None, orc.F16, orc.FP8)
        got = ops.quantizelinear(half_dev(xb), half_dev(sb), None, ops.DT.FP8)
    else:
        xb, sb = orc.bf16_from_f32(x), orc.bf16_from_f32(np.float32([0.37]))
        want = orc.quantizelinear(xb, sb, None, orc.BF16, orc.FP8)
        got = ops.quantizelinear(bf16_dev(xb), bf16_dev(sb), None, ops.DT.FP8)
    assert np.array_equal(got.cpu().numpy(), want)


def test_quantize_fp8_every_tie_point(ops):
    """Exact midpoints between neighbouring e4m3fn values and their float
    neighbours: pins the hardware converter's rounding against the oracle."""
    vals = orc.fp8_to_f32(np.arange(0x7f, dtype=np.uint8)).astype(np.float64)
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
    x = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                        vals.astype(np.float32)])
    x = np.concatenate([x, -x]).reshape(1, -1)
    want = orc.quantizelinear(x, np.float32(1.0), None, orc.F32, orc.FP8)
    got = ops.quantizelinear(dev(x), dev(np.float32([1.0])), None, ops.DT.FP8)
    assert np.array_equal(got.cpu().numpy(), want)


def test_quantize_half_input_to_int8(ops):
    rng = np.random.default_rng(3)
    xb = orc.half_from_f32((rng.standard_normal((8, 999)) * 5).astype(np.float32))
    sb = orc.half_from_f32(np.float32([0.0371]))
    want = orc.quantizelinear(xb, sb, np.int8(3), orc.F16, orc.I8)
    got = ops.quantizelinear(half_dev(xb), half_dev(sb), dev(np.int8([3])), ops.DT.I8)
    assert np.array_equal(got.cpu().numpy(), want)


def test_dequantize_int32_and_u8_half(ops):
    rng = np.random.default_rng(4)
    acc = rng.integers(-2**30, 2**30, (64, 96)).astype(np.int32)
    zp = rng.integers(-2**20, 2**20, (64, 96)).astype(np.int32)
    s = rng.uniform(1e-4, 1e-2, 96).astype(np.float32)
    want = orc.dequantizelinear(acc, s, zp, orc.I32, orc.F32)
    got = ops.dequantizelinear(dev(acc), dev(s), dev(zp))
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    q = rng.integers(0, 16, (32, 256), dtype=np.uint8)
    sh = orc.half_from_f32(rng.uniform(0.005, 0.02, (32, 256)).astype(np.float32))
    z8 = np.full((32, 256), 8, np.uint8)
    want = orc.dequantizelinear(q, sh, z8, orc.U8, orc.F16)
    got = ops.dequantizelinear(dev(q), half_dev(sh), dev(z8))
    assert np.array_equal(half_bits(got), want)


def test_reference_int4_known_answers_on_gpu(ops, golden):
    """All 12 cases of test/ref/unpack_int4.cpp and pack_int4.cpp, including the transposed
    literal, the multibroadcast view and axis 0, on the device with the views' own strides."""
    assert len(golden["unpack_int4"]) + len(golden["pack_int4"]) == 12
    for c in golden["unpack_int4"] + golden["pack_int4"]:
        dt = np.int8 if c["shape"]["type"] == "int8" else np.uint8
        raw = np.array(c["data"], np.uint8)
        lens = c["shape"]["lens"]
        x = dev((raw if dt == np.uint8 else raw.view(np.int8)).reshape(lens))
        strides = c["shape"].get("strides")
        if strides and len(lens) == 2 and strides[0] < strides[1]:
            x = x.t().contiguous().t()           # same values, column-major storage
            assert list(x.stride()) == strides
        if c["multibroadcast"]:
            x = x.expand(c["multibroadcast"])    # stride 0 along the new dimension
        fn = ops.unpack_int4 if "unpack" in c["name"] else ops.pack_int4
        got = fn(x, c["axis"]).cpu().numpy()
        assert got.view(np.uint8).flatten().tolist() == (np.array(c["gold"]).astype(np.int64) & 0xff).tolist(), c["name"]


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
def test_int4_any_axis_and_views_match_oracle(ops, axis):
    rng = np.random.default_rng(50 + axis)
    for dt, lo, hi in ((np.uint8, 0, 40), (np.int8, -30, 30)):
        x = rng.integers(lo, hi, (6, 10, 14)).astype(dt)
        p = ops.pack_int4(dev(x), axis)
        assert np.array_equal(p.cpu().numpy(), orc.pack_int4(x, axis))
        u = ops.unpack_int4(p, axis)
        assert np.array_equal(u.cpu().numpy(), orc.unpack_int4(orc.pack_int4(x, axis), axis))
        # a permuted view and a broadcast view, both along the same logical axis
        xv = dev(x).permute(2, 0, 1)
        xn = np.transpose(x, (2, 0, 1))
        assert np.array_equal(ops.unpack_int4(xv, axis).cpu().numpy(), orc.unpack_int4(np.ascontiguousarray(xn), axis))
        assert np.array_equal(ops.pack_int4(xv, axis).cpu().numpy(), orc.pack_int4(np.ascontiguousarray(xn), axis))
        xb = dev(x[:, :1, :]).expand(6, 4, 14)
        xbn = np.ascontiguousarray(np.broadcast_to(x[:, :1, :], (6, 4, 14)))
        assert np.array_equal(ops.unpack_int4(xb, axis).cpu().numpy(), orc.unpack_int4(xbn, axis))


def test_pack_unpack_random(ops):
    rng = np.random.default_rng(5)
    for dt, lo, hi in ((np.uint8, 0, 40), (np.int8, -30, 30)):
        x = rng.integers(lo, hi, (17, 130)).astype(dt)
        p = ops.pack_int4(dev(x))
        assert np.array_equal(p.cpu().numpy(), orc.pack_int4(x))
        assert np.array_equal(ops.unpack_int4(p).cpu().numpy(), orc.unpack_int4(orc.pack_int4(x)))
    from amdmigraphx_amd import Mi355Error
    with pytest.raises(Mi355Error):
        ops.pack_int4(torch.zeros((3, 5), dtype=torch.uint8, device="cuda"))


def test_convert(ops):
    rng = np.random.default_rng(6)
    x = _adversarial_f32(rng, 20000)
    x = np.concatenate([x, np.float32([65504, 65519, 65520, 65536, 1e5, -1e5, 3.39e38, -3.39e38,
                                       6e-8, 6.1e-5, 5.9e-8, 1 + 1.5 * 2.0**-11])])
    got = ops.convert(dev(x), ops.DT.F16)
    assert np.array_equal(half_bits(got), orc.convert(x, orc.F32, orc.F16))
    got = ops.convert(dev(x), ops.DT.BF16)
    assert np.array_equal(bf16_bits(got), orc.convert(x, orc.F32, orc.BF16))
    got = ops.convert(dev(x), ops.DT.FP8)
    assert np.array_equal(got.cpu().numpy(), orc.convert(x, orc.F32, orc.FP8))
    hb = orc.half_from_f32(x)
    got = ops.convert(half_dev(hb), ops.DT.F32)
    want = orc.convert(hb, orc.F16, orc.F32)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_fp4_unpack_and_pack_match_oracle(ops):
    """All 256 packed bytes through unpack (fp8 e4m3fn out), and pack on every rounding boundary,
    its float neighbours, saturation, infinities, NaN and signed zeros -- bit for bit."""
    packed = np.arange(256, dtype=np.uint8).reshape(8, 32)
    got = ops.unpack_fp4(dev(packed)).cpu().numpy()
    assert np.array_equal(got, orc.unpack_fp4(packed))
    ties = np.float32([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    pts = np.concatenate([ties, np.nextafter(ties, np.float32(0)), np.nextafter(ties, np.float32(10)),
                          np.float32([0, 0.5, 1, 1.5, 2, 3, 4, 6, 6.5, 448, 1e30, np.inf, np.nan, 1e-30])])
    x = np.concatenate([pts, -pts]).astype(np.float32)
    rng = np.random.default_rng(5)
    x = np.concatenate([x, rng.uniform(-7, 7, 4096 - x.size).astype(np.float32)]).reshape(64, 64)
    got = ops.pack_fp4(dev(x)).cpu().numpy()
    assert np.array_equal(got, orc.pack_fp4(x))
    # round trip on the device equals the oracle's
    back = ops.unpack_fp4(ops.pack_fp4(dev(x))).cpu().numpy()
    assert np.array_equal(back, orc.unpack_fp4(orc.pack_fp4(x)))
    from amdmigraphx_amd import Mi355Error
    with pytest.raises(Mi355Error):
        ops.pack_fp4(dev(np.zeros((2, 3), np.float32)))
