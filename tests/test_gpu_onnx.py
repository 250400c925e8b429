"""The reference's ONNX test models of the quantized-GEMM path parsed by the host layer, compiled
for the MI355X target and checked against the reference's expected outputs."""
import numpy as np
import pytest

from host_util import ensure_built, run_onnx
from test_onnx import matmulnbits_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def built():
    ensure_built()


def test_matmulnbits_models_on_device(golden, tmp_path):
    # test/onnx/verify/matmulnbits_tests.cpp; float models take the bit-exact float dot behind the
    # device's dequantization, so the tolerance is the reference's own
    for c in golden["matmulnbits"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["name"] + ".onnx", matmulnbits_inputs(c), tmp_path)
        np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=1e-5, atol=1e-4, err_msg=c["name"])


def test_blocked_quantize_dequantize_models_on_device(golden, tmp_path):
    for c in golden["onnx_qdq"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], c["inputs"], tmp_path)
        want = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == want.tolist(), c["name"]
        if c["name"].startswith("quantize"):
            assert got.tolist() == [float(v) for v in c["gold"]], c["name"]


def test_qlinearmatmul_models_on_device(golden, tmp_path):
    # uint8 operands are no quant_dot inputs of simplify_qdq (int8 and fp8 only), so these run as
    # dequantize -> float dot -> quantize on the device; the answers are the reference's
    for c in golden["onnx_qlinearmatmul"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == [float(v) for v in c["gold"]], c["name"]


def test_integer_matmul_models_on_device(golden, tmp_path):
    # test/onnx/verify/matmulinteger_*_test.cpp: uint8 operands move to int8 through half on the
    # device (convert, half add, convert), zero points are subtracted in int8, the product is the
    # int8 quant_dot -- int32 results, exact; matmulintegertofloat_*: dequantize, float dot, bias
    from test_onnx import _integer_case_inputs
    cases = [c for c in golden["onnx_integer"] if c["name"].startswith("matmulinteger")]
    assert len(cases) == 7
    for c in cases:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], _integer_case_inputs(c), tmp_path)
        want = run_onnx("oracle", c["model"], _integer_case_inputs(c), tmp_path)
        assert got.tolist() == want.tolist(), c["name"]
        gold = [float(v) for v in c["gold"]]
        assert (np.trunc(got) if c["name"].startswith("matmulintegertofloat") else got).tolist() == gold, c["name"]


def test_qlinearconv_models_on_device(golden, tmp_path):
    # test/onnx/verify/qlinearconv_*_test.cpp: uint8 tensors are no quant_convolution inputs of
    # simplify_qdq, so the layer runs as dequantize -> float convolution -> (bias) -> quantize on the
    # device, each step bit-identical to the CPU target's; the answers are the reference's
    from test_onnx import _integer_case_inputs
    cases = [c for c in golden["onnx_integer"] if c["name"].startswith("qlinearconv")]
    assert len(cases) == 5
    for c in cases:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], _integer_case_inputs(c), tmp_path)
        want = run_onnx("oracle", c["model"], _integer_case_inputs(c), tmp_path)
        assert got.tolist() == want.tolist(), c["name"]
        gold = np.float64(c["gold"])
        part = got[:len(gold)] if c.get("gold_is_prefix") else got
        assert np.abs(part - gold).max() <= 1 and (part == gold).mean() >= 0.95, c["name"]


def test_convinteger_models_on_device(tmp_path):
    # test/onnx/parse/convinteger_*.cpp models against the operator's definition: every term is an
    # int8 quant_convolution on the device, the zero-point tensors go in as dense copies
    from test_onnx import CONVINTEGER_MODELS, convinteger_case
    for case in CONVINTEGER_MODELS:
        print("onnx", case[0], flush=True)
        inputs, want = convinteger_case(*case)
        got = run_onnx("mi355", case[0], inputs, tmp_path)
        assert got.tolist() == want.flatten().astype(np.float64).tolist(), case[0]


def test_dynamicquantizelinear_models_on_device(golden, tmp_path):
    # test/onnx/verify/dynamicquantizelinear_*_test.cpp: the range (reduce_max / reduce_min over all
    # elements), the scale and zero point arithmetic and the quantization all run on the device
    for c in golden["onnx_dynamicquantizelinear"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], {"x": c["x"]}, tmp_path)
        want = run_onnx("oracle", c["model"], {"x": c["x"]}, tmp_path)
        assert got.tolist() == want.tolist(), c["name"]
        assert got[:len(c["y"])].tolist() == [float(v) for v in c["y"]], c["name"]


def test_matmulbnb4_models_on_device(golden, tmp_path):
    # test/onnx/verify/matmulbnb4_tests.cpp: codes and absmax are inputs of these models, so the
    # unpacking, the table lookup (or code / 8), the scaling and the product all run on the device;
    # every step is exact or correctly rounded, the product is the double sum of the CPU target
    for c in golden["onnx_matmulbnb4"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], c["inputs"], tmp_path)
        want = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == want.tolist(), c["name"]
        np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=2e-5, atol=1e-3, err_msg=c["name"])
    # a larger layer (N = 64, K = 128, block 64; four rows of A) with seeded inputs
    rng = np.random.default_rng(5)
    inputs = {"A": rng.standard_normal(4 * 128).astype(np.float32), "B": rng.integers(0, 256, 64 * 128 // 2),
              "absmax": (rng.random(128) + 0.5).astype(np.float32)}
    got = run_onnx("mi355", "matmulbnb4_large_test.onnx", inputs, tmp_path)
    want = run_onnx("oracle", "matmulbnb4_large_test.onnx", inputs, tmp_path)
    assert got.tolist() == want.tolist()


def test_qlinearadd_and_qlinearmul_models_on_device(golden, tmp_path):
    # test/onnx/verify/qlinear{add,mul}[_bcast]_test.cpp: dequantize, add / mul, quantize on the device
    for c in golden["onnx_qlinearbinary"]:
        print("onnx", c["name"], flush=True)
        got = run_onnx("mi355", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == [float(v) for v in c["gold"]], c["name"]


def test_written_qdq_conv_model_on_device(tmp_path):
    """A QDQ-format convolution layer written as ONNX bytes: parse, compile for mi355 (simplify_qdq
    turns it into quant_convolution with the dequantize epilogue fused), bit-identical to the CPU
    target on the same input."""
    import subprocess
    import host_util
    from test_onnx import qdq_conv_model
    rng = np.random.default_rng(3)
    data, _, _, _ = qdq_conv_model(rng)
    path = tmp_path / "qdq_conv.onnx"
    path.write_bytes(data)
    x = rng.standard_normal((2, 4, 9, 9)).astype(np.float32)
    spec = tmp_path / "in.txt"
    spec.write_text("x " + " ".join(repr(float(v)) for v in x.flatten()) + "\n")
    results = {}
    for target in ("oracle", "mi355"):
        out = tmp_path / (target + ".txt")
        # the CPU target evaluates what it is given, so it gets the graph simplify_qdq leaves
        r = subprocess.run([host_util.HOST_TESTS, "onnx", target, str(path), str(spec), str(out), "simplify_qdq"],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stdout + r.stderr
        results[target] = np.loadtxt(out)
    assert results["mi355"].tolist() == results["oracle"].tolist()


def test_written_qdq_matmul_model_on_device(tmp_path):
    """benchmark config 1 from ONNX bytes through the Python surface: one fused quant_dot launch
    (dequantize and bias in its epilogue), bit-identical to the oracle."""
    from oracle import oracle as orc
    from amdmigraphx_amd import migraphx as mgx
    from test_onnx import qdq_matmul_model
    rng = np.random.default_rng(4)
    data, w, sw, bias = qdq_matmul_model(rng, m=256, k=1024, n=1024)
    p = mgx.parse_onnx_buffer(data)
    p.compile(mgx.get_target("gpu"))
    text = repr(p)
    assert text.count("mi355::quant_dot") == 1 and "mi355::binary" not in text and "mi355::chain" not in text
    x = rng.standard_normal((256, 1024)).astype(np.float32)
    got = np.array(p.run({"x": x})[0])
    xq = orc.quantizelinear(x, np.float32(1.0 / 32), np.int8(0), orc.F32, orc.I8)
    want = orc.qdq_matmul_int8(xq, w, np.float32(1.0 / 32), sw) + bias[None, :]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_layernormalization_models_on_device(golden, tmp_path):
    """LayerNormalization over the last axis: the parser's reduce_mean / sub / mul / reduce_mean / add / rsqrt / mul /
    mul / add becomes one mi355::chain_rows, with the bits of the CPU target (the float model; its 16-bit siblings
    go through converts around the same float arithmetic)."""
    import os
    from amdmigraphx_amd import migraphx as mgx
    from host_util import ONNX_DIR
    p = mgx.parse_onnx(os.path.join(ONNX_DIR, "layer_norm_4d_test.onnx"))
    p.compile(mgx.get_target("gpu"))
    text = repr(p)
    assert text.count("mi355::chain_rows") == 1 and "mi355::reduce_mean" not in text, text
    rng = np.random.default_rng(23)
    for model, lens in (("layer_norm_4d_test.onnx", (3, 3, 3, 3)), ("layer_norm_3d_test.onnx", (1, 4, 2)),
                        ("layer_norm_2d_axis_minus_one_test.onnx", (3, 4))):
        inputs = {"x": rng.standard_normal(lens).astype(np.float32).flatten(),
                  "scale": rng.uniform(0.5, 1.5, lens[-1]).astype(np.float32),
                  "bias": rng.standard_normal(lens[-1]).astype(np.float32)}
        print("onnx", model, flush=True)
        got = run_onnx("mi355", model, inputs, tmp_path)
        want = run_onnx("oracle", model, inputs, tmp_path)
        assert got.tolist() == want.tolist(), model
    for c in golden["onnx_layernorm"]:
        n = int(np.prod(c["x_lens"]))
        got = run_onnx("mi355", c["model"], {"x": list(range(1, n + 1)), "scale": c["scale"], "bias": c["bias"]},
                       tmp_path)
        tol = 1e-5 if c["type"] == "float" else 8e-3
        np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=tol, atol=tol, err_msg=c["name"])
