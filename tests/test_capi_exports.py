"""CPU-side checks of the drop-in boundary: the shared library loads without a
GPU and exports every function the public header declares, and the ctypes
binding covers the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mi355_qgemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for n in ("mi355_quant_dot", "mi355_quantizelinear", "mi355_dequantizelinear",
              "mi355_unpack_int4", "mi355_pack_int4", "mi355_convert", "mi355_w4a16_gemm",
              "mi355_colsum_i8", "mi355_rowsum_i8"):
        assert n in names


def test_library_exports_every_declared_symbol():
    from amdmigraphx_amd import capi
    if not os.path.exists(capi.lib_path()):
        pytest.skip("library not built in this checkout (run __graft_entry__.build())")
    h = ctypes.CDLL(capi.lib_path())
    for name in _declared():
        assert hasattr(h, name), name
    assert sorted(capi.EXPORTS) == _declared()
    assert h.mi355_version() >= 100


def test_bad_arguments_are_rejected_without_a_gpu():
    """Argument validation happens before any HIP call."""
    from amdmigraphx_amd import capi
    if not os.path.exists(capi.lib_path()):
        pytest.skip("library not built in this checkout")
    L = capi.lib()
    d = capi.QuantDotDesc(m=4, n=4, k=4, lda=4, ldb=4, ldc=4, batch=1, in_type=capi.DT.I8,
                          out_type=capi.DT.I32)
    assert L.mi355_quant_dot(ctypes.byref(d), None, None, None, None, None, None, None, None) == -1
    d.in_type = capi.DT.F16
    one = ctypes.c_void_p(16)
    assert L.mi355_quant_dot(ctypes.byref(d), one, one, one, None, None, None, None, None) == -2
    d.in_type, d.out_type = capi.DT.I8, capi.DT.F32      # bare int8 quant_dot must give int32
    assert L.mi355_quant_dot(ctypes.byref(d), one, one, one, None, None, None, None, None) == -1
    assert L.mi355_pack_int4(one, one, 0, 3, 5, None) == -1            # odd axis
    assert L.mi355_w4a16_gemm(one, 128, one, one, None, 0, 8, one, 4, 1, 4, 128, 48, None) == -2
    assert L.mi355_status_string(-2) == b"unsupported configuration"
