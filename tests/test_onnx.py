"""The ONNX front-end slice of the host layer on the reference's own test models
(tests/golden/onnx/*.onnx are data files of test/onnx): expected outputs of test/onnx/verify,
program structure of test/onnx/parse, error messages of the negative tests.  Evaluated on the CPU
oracle target."""
import numpy as np
import pytest

from host_util import ensure_built, print_onnx, run_onnx


@pytest.fixture(scope="module", autouse=True)
def built():
    ensure_built()


def matmulnbits_inputs(c):
    a = (np.arange(int(np.prod(c["a_lens"])), dtype=np.float32) if isinstance(c["a"], str) else np.float32(c["a"]))
    inputs = {"a": a.flatten(), "b": c["b"], "scales": c["scales"]}
    if c["zp"] is not None:
        inputs["zp"] = c["zp"]
    return inputs


def test_matmulnbits_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/matmulnbits_tests.cpp
    for c in golden["matmulnbits"]:
        got = run_onnx("oracle", c["name"] + ".onnx", matmulnbits_inputs(c), tmp_path)
        np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=1e-5, atol=1e-4, err_msg=c["name"])


def test_blocked_quantize_dequantize_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/dequantizelinear_blocked_test.cpp, quantizelinear_blocked_test.cpp
    assert len(golden["onnx_qdq"]) == 5
    for c in golden["onnx_qdq"]:
        got = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        if c["name"].startswith("quantize"):
            assert got.tolist() == [float(v) for v in c["gold"]], c["name"]
        else:
            np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=1e-6, atol=1e-6, err_msg=c["name"])


def test_qlinearmatmul_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/qlinearmatmul_{1D,2D,3D,N_D_perchannel}_test.cpp: uint8 results, exact
    assert len(golden["onnx_qlinearmatmul"]) == 4
    for c in golden["onnx_qlinearmatmul"]:
        got = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == [float(v) for v in c["gold"]], c["name"]


def _integer_case_inputs(c):
    inputs = {}
    for name, v in c["inputs"].items():
        inputs[name] = [i % 256 for i in range(v["count"])] if isinstance(v, dict) else v
    return inputs


def test_integer_matmul_and_qlinearconv_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/matmulinteger_*_test.cpp, matmulintegertofloat_*.cpp, qlinearconv_*_test.cpp.
    # MatMulInteger: int32 results, exact.  MatMulIntegerToFloat: the reference test reads the float
    # result as int32 (truncating) and compares by RMS; QLinearConv: uint8 results compared by RMS
    # there -- here every value must be within one step and 95 % must be equal.
    assert len(golden["onnx_integer"]) == 12
    for c in golden["onnx_integer"]:
        got = run_onnx("oracle", c["model"], _integer_case_inputs(c), tmp_path)
        gold = np.float64(c["gold"])
        if c.get("gold_is_prefix"):
            got = got[:len(gold)]
        assert got.shape == gold.shape, c["name"]
        if c["name"].startswith("matmulinteger_"):
            assert got.tolist() == gold.tolist(), c["name"]
        elif c["name"].startswith("matmulintegertofloat"):
            assert np.trunc(got).tolist() == gold.tolist(), c["name"]
        else:
            assert np.abs(got - gold).max() <= 1 and (got == gold).mean() >= 0.95, (c["name"], got, gold)


def _conv_int64(x, w):
    n, c, h, wd = x.shape
    o, _, kh, kw = w.shape
    out = np.zeros((n, o, h - kh + 1, wd - kw + 1), np.int64)
    for r in range(kh):
        for q in range(kw):
            out += np.einsum("nchw,oc->nohw", x[:, :, r:r + out.shape[2], q:q + out.shape[3]], w[:, :, r, q])
    return out


CONVINTEGER_MODELS = [
    # test/onnx/parse/convinteger_*.cpp: (model, x type and shape, w type and shape, which zero points are inputs)
    ("convinteger_no_bias_test.onnx", np.int8, (1, 3, 5, 5), np.int8, (1, 3, 2, 2), ()),
    ("convinteger_bias_test.onnx", np.int8, (2, 3, 32, 32), np.int8, (4, 3, 5, 5), ("2",)),
    ("convinteger_dual_bias_test.onnx", np.int8, (2, 3, 10, 10), np.int8, (4, 3, 3, 3), ("2", "3")),
    ("convinteger_no_bias_uint8_test.onnx", np.uint8, (1, 3, 32, 32), np.uint8, (1, 3, 5, 5), ()),
    ("convinteger_mismatched_input_types_test.onnx", np.int8, (1, 3, 32, 32), np.uint8, (1, 3, 5, 5), ()),
]


def convinteger_case(model, xt, xs, wt, ws, zps, seed=0):
    rng = np.random.default_rng(seed + len(model))
    lim = lambda t: (0, 256) if t == np.uint8 else (-128, 128)
    x = rng.integers(*lim(xt), xs).astype(xt)
    w = rng.integers(*lim(wt), ws).astype(wt)
    inputs = {"0": x.flatten(), "1": w.flatten()}
    xz = wz = 0
    if "2" in zps:
        xz = int(rng.integers(-20, 20))
        inputs["2"] = [xz]
    if "3" in zps:
        wz = int(rng.integers(-20, 20))
        inputs["3"] = [wz]
    # uint8 tensors without a zero point are taken as they are shifted by 128 (the operator's own rule)
    xv = x.astype(np.int64) - (xz if "2" in zps else (128 if xt == np.uint8 else 0))
    wv = w.astype(np.int64) - (wz if "3" in zps else (128 if wt == np.uint8 else 0))
    return inputs, _conv_int64(xv, wv)


@pytest.mark.parametrize("case", CONVINTEGER_MODELS, ids=[c[0] for c in CONVINTEGER_MODELS])
def test_convinteger_models_against_the_definition(case, tmp_path):
    inputs, want = convinteger_case(*case)
    got = run_onnx("oracle", case[0], inputs, tmp_path)
    assert got.tolist() == want.flatten().astype(np.float64).tolist()


def test_convinteger_program_structure_and_rejections():
    # test/onnx/parse/convinteger_dual_bias_test.cpp: conv - conv(x_zp, w) - conv(x, w_zp) + conv(x_zp, w_zp)
    rc, text = print_onnx("convinteger_dual_bias_test.onnx")
    assert rc == 0 and text.count("quant_convolution[") == 4 and text.count("sub(") == 2 and text.count("add(") == 1, text
    rc, text = print_onnx("convinteger_no_bias_uint8_test.onnx")
    assert rc == 0 and text.count("quant_convolution[") == 1 and text.count("convert[target_type=5]") == 2, text
    for model in ("convinteger_mismatched_data_bias_test.onnx", "convinteger_mismatched_weight_bias_test.onnx"):
        rc, text = print_onnx(model)
        assert rc == 4 and "Zero Point must have same type" in text, text


def test_dynamicquantizelinear_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/dynamicquantizelinear_1d_test.cpp, _2d_test.cpp: y, y_scale and y_zero_point
    assert len(golden["onnx_dynamicquantizelinear"]) == 3
    for c in golden["onnx_dynamicquantizelinear"]:
        got = run_onnx("oracle", c["model"], {"x": c["x"]}, tmp_path)
        n = len(c["y"])
        assert got[:n].tolist() == [float(v) for v in c["y"]], c["name"]
        np.testing.assert_allclose(got[n], c["y_scale"][0], rtol=1e-6)
        assert got[n + 1] == c["y_zero_point"][0]


def test_per_tensor_and_per_axis_models(tmp_path):
    # test/onnx/parse/dequantizelinear_test.cpp, _zero_point_test, _axis_test, _neg_axis_test: shapes of
    # the models, values against the operator's definition
    x = np.array([3, -7, 20, 100, -128], np.int8)
    s = np.float32([0.5, 2.0, 0.25, 3.0, 1.5])
    z = np.array([1, -2, 3, 0, 5], np.int8)
    want = (x.astype(np.float64) - z) * s
    for model in ("dequantizelinear_axis_test.onnx", "dequantizelinear_neg_axis_test.onnx"):
        got = run_onnx("oracle", model, {"0": x, "1": s, "2": z}, tmp_path)
        np.testing.assert_allclose(got, want, rtol=1e-6)
    x5 = np.array([3, 7, 20, 100, 127], np.int8)
    got = run_onnx("oracle", "dequantizelinear_test.onnx", {"0": x5, "1": [0.5]}, tmp_path)
    np.testing.assert_allclose(got, x5 * 0.5)
    got = run_onnx("oracle", "dequantizelinear_zero_point_test.onnx", {"0": x5, "1": [2.0], "2": [10]}, tmp_path)
    np.testing.assert_allclose(got, (x5.astype(np.float64) - 10) * 2.0)
    xs = np.float32([0.4, -3.2, 17.5, 300.0, 2.5])
    got = run_onnx("oracle", "quantizelinear_test.onnx", {"0": xs, "1": [0.5]}, tmp_path)
    assert got.tolist() == np.clip(np.rint(xs / np.float32(0.5)), 0, 255).tolist()   # uint8 without a zero point


@pytest.mark.parametrize("model,result_shape", [
    # test/onnx/parse/matmul_*_test.cpp
    ("matmul_vv_test.onnx", "{1}"), ("matmul_vm_test.onnx", "{8}"), ("matmul_mv_test.onnx", "{6}"),
    ("matmul_vbm_test.onnx", "{5, 8}"), ("matmul_bmv_test.onnx", "{3, 6}"), ("matmul_bmbm_test.onnx", "{5, 2, 3, 6, 8}"),
])
def test_matmul_vector_and_batch_rules(model, result_shape):
    rc, text = print_onnx(model)
    assert rc == 0, text
    ret = [l for l in text.splitlines() if "@return(" in l][0]
    src = ret.split("@return(")[1].split(")")[0]
    line = [l for l in text.splitlines() if l.startswith(src + " =")][0]
    assert line.split("float_type, ")[1].startswith(result_shape), text


def test_matmul_vector_times_vector_value(tmp_path):
    a = np.arange(7, dtype=np.float32)
    b = np.arange(7, dtype=np.float32) * 0.5
    got = run_onnx("oracle", "matmul_vv_test.onnx", {"1": a, "2": b}, tmp_path)
    np.testing.assert_allclose(got, [float(a @ b)])


@pytest.mark.parametrize("model,message", [
    # test/onnx/parse/matmulnbits_negative_tests.cpp, dequantizelinear_negative_tests.cpp
    ("matmulnbits_invalid_bits_value_test.onnx", "bits only supported for value of 4, actual value 5"),
    ("matmulnbits_block_size_too_small_test.onnx", "block_size must be a power of 2 and >=16, actual value 8"),
    ("matmulnbits_block_size_not_power_of_two_test.onnx", "block_size must be a power of 2 and >=16, actual value 20"),
    ("matmulnbits_invalid_b_dims_test.onnx", "Input B does not match expected dims"),
    ("matmulnbits_invalid_scales_dims_test.onnx", "Input scales does not match expected dims"),
    ("matmulnbits_invalid_zp_dims_test.onnx", "Input zero_points does not match expected dims"),
    ("dequantizelinear_too_few_inputs_test.onnx", "must have either 2 or 3 inputs, 1 inputs provided"),
    ("dequantizelinear_too_many_inputs_test.onnx", "must have either 2 or 3 inputs, 4 inputs provided"),
    ("dequantizelinear_x_and_zp_type_mismatch_test.onnx", "x and y_zero_point must be of same type"),
    ("dequantizelinear_scale_and_zp_shape_mismatch_test.onnx", "y_scale and y_zero_point shape mismatch"),
    # test/onnx/parse/matmulbnb4_tests.cpp
    ("matmulbnb4_invalid_quant_type_test.onnx", "quant_type must be 0 (FP4) or 1 (NF4), actual value: "),
    ("matmulbnb4_invalid_block_size_test.onnx", "block_size must be a power of 2 and >= 16, actual value: "),
    ("matmulbnb4_invalid_block_size_small_test.onnx", "block_size must be a power of 2 and >= 16, actual value: "),
    ("matmulbnb4_wrong_input_count_test.onnx", "requires exactly 3 inputs (A, B, absmax)"),
    ("matmulbnb4_wrong_a_dims_test.onnx", "Input A must have at least 1 dimension"),
    ("matmulbnb4_wrong_a_inner_dim_test.onnx", "must match attribute K"),
    ("matmulbnb4_wrong_b_dims_test.onnx", "Input B does not match expected dims"),
    ("matmulbnb4_wrong_absmax_dims_test.onnx", "Input absmax does not match expected dims"),
    ("matmulbnb4_missing_n_attr_test.onnx", "Attribute N is required but missing"),
])
def test_malformed_models_are_rejected_with_the_reference_messages(model, message):
    rc, text = print_onnx(model)
    assert rc == 4 and message in text, text


def test_python_module_parses_files_and_buffers():
    import os
    from host_util import ONNX_DIR
    mgx = pytest.importorskip("amdmigraphx_amd.migraphx")
    path = os.path.join(ONNX_DIR, "matmulnbits_mm_test.onnx")
    p = mgx.parse_onnx(path)
    assert sorted(p.get_parameter_names()) == ["a", "b", "scales", "zp"]
    assert p.get_output_shapes() == [mgx.shape(type="float", lens=[2, 4])]
    with open(path, "rb") as f:
        q = mgx.parse_onnx_buffer(f.read())
    assert p == q
    with pytest.raises(RuntimeError):
        mgx.parse_onnx_buffer(b"\x3a\x7f\x01")      # a graph field that claims more bytes than there are
    with pytest.raises(RuntimeError):
        mgx.parse_onnx(os.path.join(ONNX_DIR, "no_such_file.onnx"))


def qdq_conv_model(rng):
    """x float -> Q/DQ (one scale) ; int8 weights with one scale per output channel -> DQ (axis 0) ;
    Conv with SAME_UPPER padding, stride 2 and a bias: what a QDQ-format quantized CNN layer holds."""
    import onnx_writer as ow
    w = rng.integers(-127, 128, (6, 4, 3, 3), dtype=np.int8)
    sw = rng.uniform(0.002, 0.01, 6).astype(np.float32)
    bias = rng.standard_normal(6).astype(np.float32)
    inits = [("w", w), ("sw", sw), ("zw", np.zeros(6, np.int8)), ("sx", np.float32([0.05])),
             ("zx", np.zeros(1, np.int8)), ("bias", bias)]
    nodes = [ow.node("QuantizeLinear", ["x", "sx", "zx"], ["xq"]),
             ow.node("DequantizeLinear", ["xq", "sx", "zx"], ["xd"]),
             ow.node("DequantizeLinear", ["w", "sw", "zw"], ["wd"], axis=0),
             ow.node("Conv", ["xd", "wd", "bias"], ["y"], auto_pad="SAME_UPPER", strides=[2, 2])]
    data = ow.model(nodes, [("x", ow.FLOAT, [2, 4, 9, 9])], [("y", ow.FLOAT, [2, 6, 5, 5])], inits)
    return data, w, sw, bias


def test_written_qdq_conv_model_parses_and_matches_the_definition(tmp_path):
    import os
    from oracle import oracle as orc
    rng = np.random.default_rng(3)
    data, w, sw, bias = qdq_conv_model(rng)
    path = tmp_path / "qdq_conv.onnx"
    path.write_bytes(data)
    import host_util
    x = rng.standard_normal((2, 4, 9, 9)).astype(np.float32)
    spec = tmp_path / "in.txt"
    spec.write_text("x " + " ".join(repr(float(v)) for v in x.flatten()) + "\n")
    out = tmp_path / "out.txt"
    import subprocess
    r = subprocess.run([host_util.HOST_TESTS, "onnx", "oracle", str(path), str(spec), str(out)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.loadtxt(out).reshape(2, 6, 5, 5)
    xq = orc.quantizelinear(x.reshape(-1, 9), np.float32(0.05), np.int8(0), orc.F32, orc.I8).reshape(x.shape)
    xd = xq.astype(np.float32) * np.float32(0.05)
    wd = w.astype(np.float32) * sw[:, None, None, None]
    # SAME_UPPER for 9 -> 5 with stride 2 and a 3-wide window: one zero in front, one behind
    want = orc.convolution(xd, wd, orc.F32, (1, 1, 1, 1), (2, 2)) + bias[None, :, None, None]
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("model,fragment", [
    # test/onnx/parse/conv_1d_test.cpp, conv_bias_test.cpp, conv_autopad_same_test.cpp
    ("conv_1d_test.onnx", "convolution[padding=[0],stride=[1],dilation=[1]"),
    ("conv_bias_test.onnx", "broadcast[axis=1,out_lens=[1, 1, 28, 28]]"),
    ("conv_autopad_same_test.onnx", "convolution[padding=[1, 1, 1, 1],stride=[1, 1],dilation=[1, 1]"),
])
def test_conv_models_structure(model, fragment):
    rc, text = print_onnx(model)
    assert rc == 0 and fragment in text, text


@pytest.mark.parametrize("model,message", [
    ("conv_autopad_fail_test.onnx", "auto_pad and padding cannot be specified simultaneously"),
    ("conv_attr_fail_test.onnx", "Inconsistent strides size, is: 2, should be: 1"),
    ("conv_bad_bias_test.onnx", "Types do not match"),
])
def test_malformed_conv_models_are_rejected(model, message):
    rc, text = print_onnx(model)
    assert rc == 4 and message in text, text


@pytest.mark.parametrize("model,message", [
    # test/onnx/parse/matmulinteger_zp_mismatch_error_test.cpp, matmulinteger_invalid_type_error.cpp,
    # matmulintegerToFloat_bad_{bias,scale}*_test.cpp: each must throw (messages of parse_matmul.cpp)
    ("matmulinteger_int8_uint8_one_zp_error_test.onnx", "zero point must be the same type as data"),
    ("matmulinteger_invalid_type_error.onnx", "Unsupported type"),
    ("matmulintegertofloat_bad_bias_test.onnx", "PARSE_QUANT_DOT_SCALED"),
    ("matmulintegertofloat_bad_bias_test2.onnx", "PARSE_QUANT_DOT_SCALED"),
    ("matmulintegertofloat_bad_bias_test3.onnx", "PARSE_QUANT_DOT_SCALED"),
    ("matmulintegertofloat_bad_scale_test.onnx", "Scales must be float or half_type"),
    ("matmulintegertofloat_bad_scale2_test.onnx", "PARSE_QUANT_DOT_SCALED"),
    ("matmulintegertofloat_bad_scale3_test.onnx", "PARSE_QUANT_DOT_SCALED"),
    ("matmulintegertofloat_bad_scale4_test.onnx", "Scales must be float or half_type"),
    ("matmulintegertofloat_bad_scale5_test.onnx", "Scales must be float or half_type"),
])
def test_malformed_integer_matmul_models_are_rejected(model, message):
    rc, text = print_onnx(model)
    assert rc == 4 and message in text, text


def test_integer_matmul_and_qlinearconv_program_structure():
    # test/onnx/parse/matmulinteger_test.cpp, matmulinteger_dual_zp_test.cpp, qlinearconv_test.cpp: what the
    # parsed programs consist of
    rc, text = print_onnx("matmulinteger_int8_uint8_dual_zp_test.onnx")
    assert rc == 0, text
    # the uint8 operand and its zero point move to int8 through half, each zero point is subtracted
    assert text.count("convert[target_type=1]") == 2 and text.count("convert[target_type=5]") == 2, text
    assert text.count("sub(") == 2 and text.count("quant_dot(") == 1, text
    rc, text = print_onnx("matmulinteger_int8_uint8_test.onnx")
    assert rc == 0 and text.count("sub(") == 0 and text.count("quant_dot(") == 1, text
    rc, text = print_onnx("qlinearconv_test.onnx")
    assert rc == 0 and text.count("dequantizelinear(") == 2 and text.count("convolution[") == 1 and \
        text.count("quantizelinear[") == 1, text
    rc, text = print_onnx("matmulintegertofloat_zp_bias_test.onnx")
    assert rc == 0 and text.count("dequantizelinear(") == 2 and text.count("dot(") == 1 and text.count("sub(") == 1, text


def qdq_matmul_model(rng, m=64, k=256, n=128, with_bias=True):
    """benchmark config 1 as a QDQ-format ONNX model: x float -> Q/DQ (scale 1/32) ; int8 weights with
    one scale per output column -> DQ (axis 1) ; MatMul ; Add of a bias."""
    import onnx_writer as ow
    w = rng.integers(-127, 128, (k, n), dtype=np.int8)
    sw = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    inits = [("w", w), ("sw", sw), ("zw", np.zeros(n, np.int8)), ("sx", np.float32([1.0 / 32])),
             ("zx", np.zeros(1, np.int8)), ("bias", bias)]
    nodes = [ow.node("QuantizeLinear", ["x", "sx", "zx"], ["xq"]),
             ow.node("DequantizeLinear", ["xq", "sx", "zx"], ["xd"]),
             ow.node("DequantizeLinear", ["w", "sw", "zw"], ["wd"], axis=1),
             ow.node("MatMul", ["xd", "wd"], ["mm"])]
    out = "mm"
    if with_bias:
        nodes.append(ow.node("Add", ["mm", "bias"], ["y"]))
        out = "y"
    data = ow.model(nodes, [("x", ow.FLOAT, [m, k])], [(out, ow.FLOAT, [m, n])], inits)
    return data, w, sw, bias


def test_written_qdq_matmul_model_becomes_quant_dot(tmp_path):
    from oracle import oracle as orc
    mgx = pytest.importorskip("amdmigraphx_amd.migraphx")
    rng = np.random.default_rng(4)
    data, w, sw, bias = qdq_matmul_model(rng)
    p = mgx.parse_onnx_buffer(data)
    assert p.get_parameter_shapes()["x"] == mgx.shape(type="float", lens=[64, 256])
    text = repr(p)
    assert text.count("dequantizelinear") == 2 and "dot(" in text and "quant_dot" not in text
    # on the CPU target the parsed graph gives the fake-quantized product
    import subprocess
    import host_util
    path = tmp_path / "qdq_matmul.onnx"
    path.write_bytes(data)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    spec = tmp_path / "in.txt"
    spec.write_text("x " + " ".join(repr(float(v)) for v in x.flatten()) + "\n")
    out = tmp_path / "out.txt"
    r = subprocess.run([host_util.HOST_TESTS, "onnx", "oracle", str(path), str(spec), str(out), "simplify_qdq"],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.loadtxt(out).reshape(64, 128).astype(np.float32)
    xq = orc.quantizelinear(x, np.float32(1.0 / 32), np.int8(0), orc.F32, orc.I8)
    want = orc.qdq_matmul_int8(xq, w, np.float32(1.0 / 32), sw) + bias[None, :]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


NF4_TABLE = np.float32([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
                        -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
                        0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
                        0.7229568362236023, 1.0])


def matmulbnb4_definition(a, b, absmax, n, k, block, nf4):
    """The operator's definition in numpy: low nibble first, row n of the [N, K] weight behind row n - 1,
    one absmax per block of consecutive codes; code / 8 or table[code], times absmax; A x W^T."""
    b = np.asarray(b, np.uint8)
    codes = np.stack([b & 15, b >> 4], axis=1).reshape(-1)[:n * k]
    scale = np.repeat(np.float32(absmax), block)[:n * k]
    value = NF4_TABLE[codes] if nf4 else codes.astype(np.float32) / np.float32(8)
    w = (value * scale).reshape(n, k)
    return np.float32(a).reshape(-1, k).astype(np.float64) @ w.T.astype(np.float64)


MATMULBNB4_MODELS = {
    # model: (N, K, block_size, NF4 table?) -- the attributes of test/onnx/gen_onnx.py's models
    "matmulbnb4_fp4_test.onnx": (4, 8, 16, False), "matmulbnb4_nf4_test.onnx": (8, 16, 16, True),
    "matmulbnb4_block32_test.onnx": (4, 16, 32, False), "matmulbnb4_fp4_1d_input_test.onnx": (4, 8, 16, False),
    "matmulbnb4_fp4_3d_input_test.onnx": (4, 8, 16, False),
}


def test_matmulbnb4_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/matmulbnb4_tests.cpp (compared by RMS there; its NF4 numbers have six digits)
    assert len(golden["onnx_matmulbnb4"]) == 5
    for c in golden["onnx_matmulbnb4"]:
        got = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        gold = np.float64(c["gold"])
        assert got.shape == gold.shape, c["name"]
        np.testing.assert_allclose(got, gold, rtol=2e-5, atol=1e-3, err_msg=c["name"])
        n, k, block, nf4 = MATMULBNB4_MODELS[c["model"]]
        want = matmulbnb4_definition(c["inputs"]["A"], c["inputs"]["B"], c["inputs"]["absmax"], n, k, block, nf4)
        np.testing.assert_allclose(got, want.reshape(-1), rtol=1e-6, err_msg=c["name"])


def test_matmulbnb4_structure():
    rc, text = print_onnx("matmulbnb4_nf4_test.onnx")
    assert rc == 0, text
    for op in ("unpack_int4", "gather[", "multibroadcast[", "transpose[", "dot"):
        assert op in text, (op, text)
    rc, text = print_onnx("matmulbnb4_fp4_3d_input_test.onnx")
    assert rc == 0 and "div" in text and "gather[" not in text, text
    ret = [l for l in text.splitlines() if "@return(" in l][0]
    src = ret.split("@return(")[1].split(")")[0]
    line = [l for l in text.splitlines() if l.startswith(src + " =")][0]
    assert "float_type, {2, 3, 4}" in line, text


def test_qlinearadd_and_qlinearmul_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/qlinearadd_test.cpp, qlinearadd_bcast_test.cpp, qlinearmul_test.cpp,
    # qlinearmul_bcast_test.cpp: 8-bit results (compared by RMS there; here every value must be equal)
    assert len(golden["onnx_qlinearbinary"]) == 4
    for c in golden["onnx_qlinearbinary"]:
        got = run_onnx("oracle", c["model"], c["inputs"], tmp_path)
        assert got.tolist() == [float(v) for v in c["gold"]], c["name"]


def test_qlinearbinary_rejects_mismatched_types(tmp_path):
    import onnx_writer as ow
    # A uint8, B int8: src/onnx/parse_qlinearbinary.cpp:124-125
    inits = [("sa", np.float32([0.1])), ("za", np.uint8([0])), ("sb", np.float32([0.1])), ("zb", np.int8([0])),
             ("sc", np.float32([0.1])), ("zc", np.uint8([0]))]
    nodes = [ow.node("QLinearAdd", ["A", "sa", "za", "B", "sb", "zb", "sc", "zc"], ["C"], domain="com.microsoft")]
    data = ow.model(nodes, [("A", ow.UINT8, [4]), ("B", ow.INT8, [4])], [("C", ow.UINT8, [4])], inits)
    path = tmp_path / "bad.onnx"
    path.write_bytes(data)
    rc, text = print_onnx(str(path))
    assert rc == 4 and "QLinearAdd: mismatched input types" in text, text


def test_layernormalization_models_reference_known_answers(golden, tmp_path):
    # test/onnx/verify/layer_norm_3d_test.cpp, layer_norm_3d_half_test.cpp, layer_norm_3d_bf16_test.cpp: x = 1, 2, ...
    # (compared by RMS there; 16-bit models are computed in float and rounded once at the end)
    assert len(golden["onnx_layernorm"]) == 3
    for c in golden["onnx_layernorm"]:
        n = int(np.prod(c["x_lens"]))
        got = run_onnx("oracle", c["model"], {"x": list(range(1, n + 1)), "scale": c["scale"], "bias": c["bias"]},
                       tmp_path)
        tol = 1e-5 if c["type"] == "float" else 8e-3
        np.testing.assert_allclose(got, np.float64(c["gold"]), rtol=tol, atol=tol, err_msg=c["name"])


def test_layernormalization_definition_on_the_other_models(tmp_path):
    """The models without known answers in the reference's tests, against the definition in numpy: other axes, four
    dimensions, no bias (src/onnx/parse_layernorm.cpp:103-176)."""
    rng = np.random.default_rng(17)
    for model, lens, axis, with_bias in (("layer_norm_2d_axis_zero_test.onnx", (3, 4), 0, True),
                                         ("layer_norm_2d_axis_one_test.onnx", (3, 4), 1, True),
                                         ("layer_norm_2d_axis_minus_one_test.onnx", (3, 4), -1, True),
                                         ("layer_norm_4d_test.onnx", (3, 3, 3, 3), -1, True),
                                         ("layer_norm_without_bias_test.onnx", (1, 2), -1, False)):
        x = rng.standard_normal(lens).astype(np.float32)
        norm_lens = lens[axis:]
        scale = rng.uniform(0.5, 1.5, norm_lens[:1] if len(norm_lens) > 1 and False else norm_lens[-1:] if len(norm_lens) == 1 else norm_lens).astype(np.float32)
        bias = rng.standard_normal(scale.shape).astype(np.float32)
        inputs = {"x": x.flatten(), "scale": scale.flatten()}
        if with_bias:
            inputs["bias"] = bias.flatten()
        got = run_onnx("oracle", model, inputs, tmp_path)
        axes = tuple(range(axis % len(lens), len(lens)))
        x64 = x.astype(np.float64)
        mean = x64.mean(axis=axes, keepdims=True)
        var = ((x64 - mean) ** 2).mean(axis=axes, keepdims=True)
        want = (x64 - mean) / np.sqrt(var + 1e-5) * scale.reshape((1,) * (len(lens) - scale.ndim) + scale.shape)
        if with_bias:
            want = want + bias.reshape((1,) * (len(lens) - bias.ndim) + bias.shape)
        np.testing.assert_allclose(got[:want.size], want.flatten(), rtol=2e-5, atol=2e-5, err_msg=model)


def test_layernormalization_error_messages():
    # test/onnx/parse/layer_norm_invalid_*: src/onnx/parse_layernorm.cpp:70-110, 180-200
    for model, message in (("layer_norm_invalid_axis_error_test.onnx", "PARSE_LAYERNORM: invalid axis"),
                           ("layer_norm_invalid_minus_axis_error_test.onnx", "PARSE_LAYERNORM: invalid axis"),
                           ("layer_norm_invalid_input_count_error_test.onnx", "PARSE_LAYERNORM: invalid input count"),
                           ("layer_norm_invalid_shape_error_test.onnx", "PARSE_LAYERNORM: invalid ndims=1, must be at least 2"),
                           ("layer_norm_3d_invalid_int8_test.onnx", "PARSE_LAYERNORM: Invalid type for input"),
                           ("layer_norm_3d_invalid_scale_test.onnx", "PARSE_LAYERNORM: Invalid type for scale"),
                           ("layer_norm_3d_invalid_bias_test.onnx", "PARSE_LAYERNORM: Invalid type for bias")):
        rc, text = print_onnx(model)
        assert rc == 4 and message in text, (model, text)
