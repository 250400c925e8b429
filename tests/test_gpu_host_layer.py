"""The mi355 target end to end (C++): programs compiled for the CPU oracle target
and for "mi355" from the same inputs must agree (tests/cpp/gpu_tests.cpp)."""
import subprocess

import numpy as np
import pytest

from host_util import GPU_TESTS, ensure_built, list_cases, run_matmulnbits

ensure_built()

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", list_cases(GPU_TESTS))
def test_target_case(case):
    print("gpu_tests", case, flush=True)
    r = subprocess.run([GPU_TESTS, case], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr


def test_matmulnbits_reference_known_answers_on_device(golden, tmp_path):
    """The reference's MatMulNBits known answers, evaluated by the mi355 target
    (float graphs: the operator-by-operator path)."""
    for c in golden["matmulnbits"]:
        print("matmulnbits", c["name"], flush=True)
        got = run_matmulnbits("mi355", c, tmp_path)
        gold = np.float32(c["gold"])
        assert got.shape == gold.shape, c["name"]
        assert np.allclose(got, gold, rtol=2e-6, atol=1e-5), (c["name"], got, gold)
