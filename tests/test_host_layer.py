"""Host layer (C++): IR, operators, passes and the target registry, without a GPU.

The cases live in tests/cpp/host_tests.cpp; each is run here as its own pytest
case.  The MatMulNBits graph builder is additionally checked against the
reference's known answers (test/onnx/verify/matmulnbits_tests.cpp) by handing
the fixtures to the test program's `matmulnbits` tool, evaluated on the CPU
oracle target.
"""
import os
import subprocess

import numpy as np
import pytest

from host_util import HOST_TESTS, ensure_built, list_cases, run_matmulnbits

ensure_built()


@pytest.mark.parametrize("case", list_cases(HOST_TESTS))
def test_host_case(case):
    r = subprocess.run([HOST_TESTS, case], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr


def test_matmulnbits_builder_reference_known_answers(golden, tmp_path):
    assert len(golden["matmulnbits"]) == 4
    for c in golden["matmulnbits"]:
        got = run_matmulnbits("oracle", c, tmp_path)
        gold = np.float32(c["gold"])
        assert got.shape == gold.shape, c["name"]
        assert np.allclose(got, gold, rtol=2e-6, atol=1e-5), (c["name"], got, gold)


def test_host_libraries_export_target_registration():
    """libmigraphx_mi355.so depends on the kernel library and the core library only
    through their public symbols; loading it needs no GPU."""
    import ctypes
    lib = os.path.join(os.path.dirname(HOST_TESTS), "..", "..", "..", "amdmigraphx_amd", "lib")
    ctypes.CDLL(os.path.join(lib, "libmigraphx.so"), mode=ctypes.RTLD_GLOBAL)
    ctypes.CDLL(os.path.join(lib, "libmigraphx_mi355.so"), mode=ctypes.RTLD_GLOBAL)
