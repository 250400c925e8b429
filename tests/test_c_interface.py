"""The C interface of the host layer (amdmigraphx_amd/host/include/migraphx/migraphx.h,
libmigraphx_c.so): the library exports every function the header declares, and the C test program
tests/cpp/capi_tests.c -- shapes, arguments, operators, a QDQ matmul built, quantized, saved,
loaded, compiled and run, an ONNX model parsed with input-shape options, error statuses -- passes on
the CPU oracle target.  The same program runs on the device in test_gpu_c_interface."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from host_util import BIN, ROOT, ensure_built
from onnx_writer import model, node

CAPI_TESTS = os.path.join(BIN, "capi_tests")
HEADER = os.path.join(ROOT, "amdmigraphx_amd", "host", "include", "migraphx", "migraphx.h")
LIBRARY = os.path.join(ROOT, "amdmigraphx_amd", "lib", "libmigraphx_c.so")


def declared():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(migraphx_[a-z0-9_]+)\s*\(", text)))


def symbolic_batch_matmul(path):
    """x [batch, 8] (the batch dimension carries no value) times an 8 x 4 initializer."""
    w = np.arange(32, dtype=np.float32).reshape(8, 4)
    data = model([node("MatMul", ["x", "w"], ["y"])], [("x", 1, [0, 8])], [("y", 1, [0, 4])], [("w", w)])
    with open(path, "wb") as f:
        f.write(data)


def run_capi_tests(target, tmp_path):
    ensure_built()
    onnx = str(tmp_path / "symbolic_batch_matmul.onnx")
    symbolic_batch_matmul(onnx)
    r = subprocess.run([CAPI_TESTS, target, onnx], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip().endswith("0 failed checks")


def test_library_exports_every_declared_function():
    ensure_built()
    names = declared()
    assert len(names) > 90
    for n in ("migraphx_program_compile", "migraphx_program_run", "migraphx_quantize_int8", "migraphx_load",
              "migraphx_save", "migraphx_parse_onnx", "migraphx_operation_create"):
        assert n in names
    h = ctypes.CDLL(LIBRARY)
    for n in names:
        assert hasattr(h, n), n


def test_status_codes_and_type_numbers_follow_the_reference():
    # src/api/include/migraphx/migraphx.h:34-74: tuple 0, fp4x2 1, then the visit order of the types
    text = open(HEADER).read()
    want = ["tuple", "fp4x2", "bool", "half", "float", "double", "uint8", "int8", "uint16", "int16", "int32",
            "int64", "uint32", "uint64", "fp8e4m3fnuz", "fp8e4m3fn", "fp8e5m2", "bf16", "fp8e5m2fnuz"]
    for i, name in enumerate(want):
        assert re.search(r"migraphx_shape_%s_type\s*=\s*%d\b" % (name, i), text), name
    for name, code in (("success", 0), ("bad_param", 1), ("unknown_target", 3), ("unknown_error", 4)):
        assert re.search(r"migraphx_status_%s\s*=\s*%d\b" % (name, code), text), name


def test_c_program_on_the_cpu_oracle_target(tmp_path):
    run_capi_tests("oracle", tmp_path)
