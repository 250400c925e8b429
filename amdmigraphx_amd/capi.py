"""ctypes binding of ``libmi355_qgemm.so`` (see ``include/mi355_qgemm.h``).

There is no fallback: if the library cannot be loaded every use raises
``Mi355Error``.  Pointers are raw device addresses (``tensor.data_ptr()``)."""
import ctypes
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_PKG, "lib", "libmi355_qgemm.so")


class Mi355Error(RuntimeError):
    pass


class DT:
    I8, U8, I32, F32, F16, BF16, FP8, FP4X2, BF8 = range(9)   # FP8: OCP e4m3fn, BF8: OCP e5m2


class QP:
    NONE, PER_TENSOR, PER_ROW, PER_COL, PER_COL_BATCH = range(5)


class W4ZP:
    SCALAR, GROUP, PACKED = range(3)


class QuantDotDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in
                ("m", "n", "k", "lda", "ldb", "ldc", "batch", "stride_a", "stride_b", "stride_c")] + \
               [(n, ctypes.c_int32) for n in
                ("trans_a", "trans_b", "in_type", "out_type", "dequant", "scale_a_mode",
                 "scale_b_mode", "zp_a", "zp_b")]


class QuantConvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in
                ("n", "c", "h", "w", "o", "kh", "kw", "pad_h", "pad_w", "stride_h", "stride_w",
                 "dil_h", "dil_w", "group", "pad_h_hi", "pad_w_hi")] + \
               [(n, ctypes.c_int32) for n in
                ("in_type", "out_type", "dequant", "scale_x_mode", "scale_w_mode")]


class QuantConv3dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("n", "c", "d", "h", "w", "o", "kd", "kh", "kw")] + \
               [(n, ctypes.c_int64 * 3) for n in ("pad", "pad_hi", "stride", "dil")] + \
               [("group", ctypes.c_int64)] + \
               [(n, ctypes.c_int32) for n in
                ("in_type", "out_type", "dequant", "scale_x_mode", "scale_w_mode")]


class MxDotDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in
                ("m", "n", "k", "batch", "lda", "ldb", "ldc", "stride_a", "stride_b", "stride_c",
                 "sa_batch", "sa_row", "sa_block", "sa_elem", "sb_batch", "sb_row", "sb_block", "sb_elem")] + \
               [(n, ctypes.c_int32) for n in ("a_type", "b_type")]


EXPORTS = {
    "mi355_quant_dot_mx_workspace_size": [ctypes.POINTER(MxDotDesc)],
    "mi355_quant_dot_mx": [ctypes.POINTER(MxDotDesc)] + [ctypes.c_void_p] * 6 + [ctypes.c_size_t, ctypes.c_void_p],
    "mi355_quant_convolution_dims": [ctypes.POINTER(QuantConvDesc), ctypes.POINTER(ctypes.c_int64),
                                     ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_size_t)],
    "mi355_quant_convolution": [ctypes.POINTER(QuantConvDesc)] + [ctypes.c_void_p] * 6 +
                               [ctypes.c_size_t, ctypes.c_void_p],
    "mi355_quant_convolution3d_dims": [ctypes.POINTER(QuantConv3dDesc), ctypes.POINTER(ctypes.c_int64),
                                       ctypes.POINTER(ctypes.c_size_t)],
    "mi355_quant_convolution3d": [ctypes.POINTER(QuantConv3dDesc)] + [ctypes.c_void_p] * 6 +
                                 [ctypes.c_size_t, ctypes.c_void_p],
    "mi355_quant_dot": [ctypes.POINTER(QuantDotDesc)] + [ctypes.c_void_p] * 8,
    "mi355_quant_dot_bias": [ctypes.POINTER(QuantDotDesc)] + [ctypes.c_void_p] * 9,
    "mi355_quant_dot_workspace_size": [ctypes.POINTER(QuantDotDesc)],
    "mi355_quant_dot_ws": [ctypes.POINTER(QuantDotDesc)] + [ctypes.c_void_p] * 9 +
                          [ctypes.c_size_t, ctypes.c_void_p],
    "mi355_quant_dot_static": [ctypes.POINTER(QuantDotDesc)] + [ctypes.c_void_p] * 9,
    "mi355_colsum_i8": [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                        ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p],
    "mi355_rowsum_i8": [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                        ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p],
    "mi355_quantizelinear": [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int64,
                             ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                             ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_int64,
                             ctypes.c_void_p],
    "mi355_dequantizelinear": [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32,
                               ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64,
                               ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                               ctypes.c_void_p],
    "mi355_unpack_int4": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                          ctypes.c_int64, ctypes.c_void_p],
    "mi355_pack_int4": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                        ctypes.c_int64, ctypes.c_void_p],
    "mi355_unpack_int4_nd": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                             ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64), ctypes.c_int32,
                             ctypes.c_void_p],
    "mi355_pack_int4_nd": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                           ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64), ctypes.c_int32,
                           ctypes.c_void_p],
    "mi355_unpack_fp4": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_pack_fp4": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_convert": [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32,
                      ctypes.c_int64, ctypes.c_void_p],
    "mi355_dot": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32] +
                 [ctypes.c_int64] * 12 + [ctypes.c_void_p],
    "mi355_dot_scaled": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32] +
                        [ctypes.c_int64] * 12 + [ctypes.c_void_p, ctypes.c_void_p],
    "mi355_dot_fp32acc": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32] +
                         [ctypes.c_int64] * 12 + [ctypes.c_void_p, ctypes.c_void_p],
    "mi355_dot_batch2": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32] +
                        [ctypes.c_int64] * 13 + [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p],
    "mi355_dot_batch2_strided": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32] +
                                [ctypes.c_int64] * 16 + [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p],
    "mi355_contiguous": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                         ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                         ctypes.c_void_p],
    "mi355_binary_f32": [ctypes.c_int32, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p,
                         ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_int32,
                         ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p],
    "mi355_chain_f32": [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p),
                        ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32), ctypes.c_int32,
                        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_chain_rows_f32": [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p),
                             ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32), ctypes.c_int32,
                             ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_chain_f32_q8": [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p),
                           ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32), ctypes.c_int32,
                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                           ctypes.c_void_p],
    "mi355_convolution_f32": [ctypes.c_void_p] * 5,
    "mi355_reduce_all_f32": [ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p],
    "mi355_binary_typed": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64),
                           ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_int32,
                           ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p],
    "mi355_binary_i32": [ctypes.c_int32, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p,
                         ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_int32,
                         ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p],
    "mi355_unary_f32": [ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p],
    "mi355_reduce_mean_f32": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_softmax_f32": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_gather_rows": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int64,
                          ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p],
    "mi355_w4a16_gemm": [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
                         ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
                         ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                         ctypes.c_int64, ctypes.c_void_p],
    "mi355_w4a16_gemm_workspace_size": [ctypes.c_int64] * 4,
    "mi355_w4a16_gemm_ws": [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
                            ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
                            ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                            ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    "mi355_quant_dot_prepacked_size": [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64],
    "mi355_quant_dot_prepack": [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p],
    "mi355_quant_dot_prepacked": [ctypes.c_void_p] * 10,
    "mi355_w4a16_prepacked_size": [ctypes.c_int64] * 3,
    "mi355_w4a16_prepacked_max_rows": [ctypes.c_int64] * 3,
    "mi355_w4a16_prepack": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_int64,
                            ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p],
    "mi355_w4a16_gemm_prepacked": [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
                                   ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_void_p],
    "mi355_status_string": [ctypes.c_int],
    "mi355_version": [],
}


def lib_path():
    return _LIB


def build_library(force=True):
    """Compile every HIP source for gfx950 into lib/libmi355_qgemm.so."""
    cmd = ["make", "-C", os.path.join(_PKG, "csrc"), "-j8"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)


_handle = None


def lib():
    """The loaded library with argument types set; raises if it is missing."""
    global _handle
    if _handle is None:
        if not os.path.exists(_LIB):
            raise Mi355Error(f"{_LIB} is not built: run __graft_entry__.build() "
                             "(make -C amdmigraphx_amd/csrc)")
        try:
            h = ctypes.CDLL(_LIB)
        except OSError as e:
            raise Mi355Error(f"cannot load {_LIB}: {e}") from e
        for name, argtypes in EXPORTS.items():
            fn = getattr(h, name)
            fn.argtypes = argtypes
            fn.restype = (ctypes.c_char_p if name == "mi355_status_string" else
                          ctypes.c_size_t if name.endswith("_workspace_size") or name.endswith("_prepacked_size")
                          else ctypes.c_int64 if name.endswith("_max_rows")
                          else ctypes.c_int)
        _handle = h
    return _handle


def check(status, what):
    if status != 0:
        raise Mi355Error(f"{what}: {lib().mi355_status_string(status).decode()} ({status})")
