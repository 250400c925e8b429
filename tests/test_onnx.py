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
