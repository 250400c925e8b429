"""Programs built, quantized, compiled and run through the Python surface on the MI355X target,
checked against the CPU oracle."""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mgx():
    from amdmigraphx_amd import migraphx
    return migraphx


def qdq_matmul(mgx, m, k, n, w, sw):
    """X float -> Q/DQ (scale 1/32) ; W int8 -> DQ per output channel ; dot (benchmark config 1)."""
    p = mgx.program()
    mm = p.get_main_module()
    x = mm.add_parameter("x", mgx.shape(type="float", lens=[m, k]))
    sx = mm.add_literal(np.float32([1.0 / 32]))
    zx = mm.add_literal(np.int8([0]))
    bc = lambda v, lens: mm.add_instruction(mgx.op("multibroadcast", out_lens=lens), [v])
    q = mm.add_instruction(mgx.op("quantizelinear"), [x, bc(sx, [m, k]), bc(zx, [m, k])])
    dx = mm.add_instruction(mgx.op("dequantizelinear"), [q, bc(sx, [m, k]), bc(zx, [m, k])])
    wl = mm.add_literal(w)
    swl = mm.add_literal(sw)
    swb = mm.add_instruction(mgx.op("broadcast", axis=1, out_lens=[k, n]), [swl])
    dw = mm.add_instruction(mgx.op("dequantizelinear"), [wl, swb, bc(zx, [k, n])])
    mm.add_return([mm.add_instruction(mgx.op("dot"), [dx, dw])])
    return p


def test_qdq_matmul_bit_exact(mgx):
    rng = np.random.default_rng(0)
    m, k, n = 256, 1024, 1024
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (k, n), dtype=np.int8)
    sw = rng.uniform(0.001, 0.01, n).astype(np.float32)
    p = qdq_matmul(mgx, m, k, n, w, sw)
    p.compile(mgx.get_target("gpu"))
    assert p.is_compiled()
    text = repr(p)
    assert "mi355::quant_dot" in text and "mi355::dequantizelinear" not in text
    out = p.run({"x": x})
    assert len(out) == 1 and out[0].get_shape() == mgx.shape(type="float", lens=[m, n])
    xq = orc.quantizelinear(x, np.float32(1.0 / 32), np.int8(0), orc.F32, orc.I8)
    want = orc.qdq_matmul_int8(xq, w, np.float32(1.0 / 32), sw)
    assert np.array_equal(np.array(out[0]).view(np.uint32), want.view(np.uint32))
    # a second run with another input reuses the compiled program
    x2 = rng.standard_normal((m, k)).astype(np.float32)
    out2 = np.array(p.run({"x": mgx.argument(x2)})[0])
    xq2 = orc.quantizelinear(x2, np.float32(1.0 / 32), np.int8(0), orc.F32, orc.I8)
    assert np.array_equal(out2.view(np.uint32), orc.qdq_matmul_int8(xq2, w, np.float32(1.0 / 32), sw).view(np.uint32))


def test_device_arguments_without_offload_copy(mgx):
    rng = np.random.default_rng(1)
    m, k, n = 64, 256, 128
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (k, n), dtype=np.int8)
    sw = rng.uniform(0.001, 0.01, n).astype(np.float32)
    p = qdq_matmul(mgx, m, k, n, w, sw)
    q = qdq_matmul(mgx, m, k, n, w, sw)
    p.compile(mgx.get_target("gpu"), offload_copy=False)
    q.compile(mgx.get_target("gpu"))
    dx = mgx.to_gpu(mgx.argument(x))
    got = mgx.from_gpu(p.run({"x": dx})[0])
    want = q.run({"x": x})[0]
    assert got == want
    buf = mgx.allocate_gpu(mgx.shape(type="float", lens=[4, 4]))
    assert buf.get_shape().lens() == [4, 4] and buf.data_ptr() != 0


def test_int8_quantization_of_a_float_program(mgx):
    """quantize_int8 with calibration data (src/quantization.cpp:88-174), then compile: the dot runs
    as a quantized GEMM and stays close to the float result (test/quantization.cpp:1066 allows
    0.004 relative RMS for the same construction)."""
    rng = np.random.default_rng(2)
    m, k, n = 32, 512, 256
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)

    def build():
        p = mgx.program()
        mm = p.get_main_module()
        xp = mm.add_parameter("x", mgx.shape(type="float", lens=[m, k]))
        wl = mm.add_literal(w)
        mm.add_return([mm.add_instruction(mgx.op("dot"), [xp, wl])])
        return p

    t = mgx.get_target("gpu")
    p = build()
    mgx.quantize_int8(p, t, [{"x": x}])
    p.compile(t)
    assert "mi355::quant_dot" in repr(p)
    got = np.array(p.run({"x": x})[0])
    want = x.astype(np.float64) @ w.astype(np.float64)
    rms = np.sqrt(((got - want) ** 2).mean() / (want ** 2).mean())
    assert rms < 0.02, rms
    f = build()
    f.compile(t)
    ref = np.array(f.run({"x": x})[0])
    np.testing.assert_allclose(ref, want, rtol=1e-5, atol=1e-5)
