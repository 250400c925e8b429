"""Build and drive the C++ test programs of the host layer."""
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")
HOST_TESTS = os.path.join(BIN, "host_tests")
GPU_TESTS = os.path.join(BIN, "gpu_tests")


def ensure_built():
    """Build the libraries and test programs when they are not there yet."""
    lib = os.path.join(ROOT, "amdmigraphx_amd", "lib")
    need = [os.path.join(lib, "libmi355_qgemm.so"), os.path.join(lib, "libmigraphx.so"),
            os.path.join(lib, "libmigraphx_mi355.so"), os.path.join(lib, "libmigraphx_c.so"),
            os.path.join(ROOT, "oracle", "liboracle.so"), HOST_TESTS, GPU_TESTS, os.path.join(BIN, "capi_tests")]
    if all(os.path.exists(p) for p in need):
        return
    import sys
    sys.path.insert(0, ROOT)
    import __graft_entry__
    __graft_entry__.build()


def list_cases(prog):
    ensure_built()
    out = subprocess.run([prog, "--list"], capture_output=True, text=True, check=True).stdout
    return out.split()


def run_matmulnbits(target, case, tmp_path, use_half=False):
    """Evaluate one MatMulNBits fixture (dict with a_lens, b_lens, a, b, scales, zp)."""
    n, nblk, blob = case["b_lens"]
    a_lens = list(case["a_lens"])
    a = (np.arange(int(np.prod(a_lens)), dtype=np.float32) if isinstance(case["a"], str)
         else np.float32(case["a"]))
    zp = case.get("zp")
    spec = tmp_path / (case["name"] + ".txt")
    with open(spec, "w") as f:
        f.write(f"{len(a_lens)} {' '.join(map(str, a_lens))} {n} {nblk} {blob} "
                f"{0 if zp is None else 1} {1 if use_half else 0}\n")
        f.write(" ".join(repr(float(v)) for v in a.flatten()) + "\n")
        f.write(" ".join(str(int(v)) for v in case["b"]) + "\n")
        f.write(" ".join(repr(float(v)) for v in case["scales"]) + "\n")
        if zp is not None:
            f.write(" ".join(str(int(v)) for v in zp) + "\n")
    out = tmp_path / (case["name"] + ".out")
    r = subprocess.run([HOST_TESTS, "matmulnbits", target, str(spec), str(out)],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    return np.loadtxt(out, dtype=np.float32, ndmin=1)


ONNX_DIR = os.path.join(ROOT, "tests", "golden", "onnx")


def run_onnx(target, model, inputs, tmp_path):
    """Parse tests/golden/onnx/<model> with the host layer and evaluate it on `target` with the
    given parameter values (name -> flat list); returns the outputs as one flat float64 array."""
    spec = tmp_path / (model + ".in")
    with open(spec, "w") as f:
        for name, values in inputs.items():
            f.write(name + " " + " ".join(repr(float(v)) for v in values) + "\n")
    out = tmp_path / (model + ".out")
    r = subprocess.run([HOST_TESTS, "onnx", target, os.path.join(ONNX_DIR, model), str(spec), str(out)],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    return np.loadtxt(out, dtype=np.float64, ndmin=1)


def print_onnx(model):
    """The parsed program as text, or the error message (return code 4) when parsing throws."""
    r = subprocess.run([HOST_TESTS, "onnx", "print", os.path.join(ONNX_DIR, model)],
                       capture_output=True, text=True, timeout=600)
    return r.returncode, r.stdout
