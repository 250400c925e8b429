"""numpy front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Loads ``liboracle.so`` (built from ``ref_oracle.c`` by ``make -C oracle``) and
exposes the ref-target arithmetic on numpy arrays.  Only tests, the smoke
check and the benchmark's cpu_baseline leg import this module; the shipped
library never does.

Low-precision element types have no numpy dtype, so they travel as raw bits:
half and bf16 as ``uint16``, fp8 e4m3fn as ``uint8``; the ``*_type`` argument
says how the bits are to be read.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

I8, U8, I32, F32, F16, BF16, FP8, F64, BF8 = range(9)
_NP = {I8: np.int8, U8: np.uint8, I32: np.int32, F32: np.float32,
       F16: np.uint16, BF16: np.uint16, FP8: np.uint8, F64: np.float64, BF8: np.uint8}


def build():
    """Compile the oracle (used by __graft_entry__.build and by tests when the
    library is missing)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                          stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    lib.orc_gemm.argtypes = [vp, ci, vp, vp, ci] + [i64] * 10
    lib.orc_gemm.restype = None
    lib.orc_quantizelinear.argtypes = [vp, ci, vp, ci, vp, i64, i64, vp, i64, i64, i64, i64]
    lib.orc_quantizelinear.restype = None
    lib.orc_dequantizelinear.argtypes = [vp, vp, ci, vp, ci, i64, i64, vp, i64, i64, i64, i64]
    lib.orc_dequantizelinear.restype = None
    lib.orc_unpack_int4.argtypes = [vp, vp, ci, i64, i64, i64]
    lib.orc_unpack_int4.restype = None
    lib.orc_pack_int4.argtypes = [vp, vp, ci, i64, i64, i64]
    lib.orc_pack_int4.restype = None
    lib.orc_unpack_fp4.argtypes = [vp, vp, i64, i64, i64]
    lib.orc_unpack_fp4.restype = None
    lib.orc_pack_fp4.argtypes = [vp, vp, i64, i64, i64]
    lib.orc_pack_fp4.restype = None
    lib.orc_fp4_to_f32.argtypes = [ctypes.c_uint8]
    lib.orc_fp4_to_f32.restype = ctypes.c_float
    lib.orc_fp4_from_f32.argtypes = [ctypes.c_float]
    lib.orc_fp4_from_f32.restype = ctypes.c_uint8
    lib.orc_convolution.argtypes = [vp, ci, vp, vp, ci] + [i64] * 16
    lib.orc_convolution.restype = None
    lib.orc_convolution3d.argtypes = [vp, ci, vp, vp, ci, i64, i64, vp, i64, vp, vp, vp, vp, i64, vp]
    lib.orc_convolution3d.restype = None
    lib.orc_convert.argtypes = [vp, ci, vp, ci, ctypes.c_size_t]
    lib.orc_convert.restype = None
    lib.orc_mul_f32.argtypes = [vp, vp, i64, i64, vp, i64, i64, i64, i64]
    lib.orc_mul_f32.restype = None
    for name in ("half", "bf16", "fp8e4m3fn", "fp8e5m2"):
        getattr(lib, f"orc_{name}_from_f32_n").argtypes = [vp, vp, ctypes.c_size_t]
        getattr(lib, f"orc_{name}_from_f32_n").restype = None
        getattr(lib, f"orc_{name}_to_f32_n").argtypes = [vp, vp, ctypes.c_size_t]
        getattr(lib, f"orc_{name}_to_f32_n").restype = None
    return lib


_lib = _load()


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# --- scalar formats --------------------------------------------------------

def _conv(name, x, src, dst):
    x = _c(x, src)
    y = np.empty(x.shape, dst)
    getattr(_lib, name)(_p(x), _p(y), x.size)
    return y


def half_from_f32(x):
    return _conv("orc_half_from_f32_n", x, np.float32, np.uint16)


def half_to_f32(x):
    return _conv("orc_half_to_f32_n", x, np.uint16, np.float32)


def bf16_from_f32(x):
    return _conv("orc_bf16_from_f32_n", x, np.float32, np.uint16)


def bf16_to_f32(x):
    return _conv("orc_bf16_to_f32_n", x, np.uint16, np.float32)


def fp8_from_f32(x):
    return _conv("orc_fp8e4m3fn_from_f32_n", x, np.float32, np.uint8)


def fp8_to_f32(x):
    return _conv("orc_fp8e4m3fn_to_f32_n", x, np.uint8, np.float32)


def bf8_from_f32(x):
    """float -> fp8 e5m2 bits (float8.hpp:102-116)."""
    return _conv("orc_fp8e5m2_from_f32_n", x, np.float32, np.uint8)


def bf8_to_f32(x):
    return _conv("orc_fp8e5m2_to_f32_n", x, np.uint8, np.float32)


# --- ops ---------------------------------------------------------------------

def _elem_strides(a):
    return [s // a.itemsize for s in a.strides]


def gemm(a, b, ab_type, c_type):
    """C[..., M, N] = A[..., M, K] . B[..., K, N] as gemm_naive does it.

    ``a`` and ``b`` may be arbitrary strided views (transposes); all leading
    dimensions are batch dimensions and must match."""
    assert a.ndim == b.ndim and a.ndim >= 2
    assert a.shape[:-2] == b.shape[:-2] and a.shape[-1] == b.shape[-2]
    m, k = a.shape[-2:]
    n = b.shape[-1]
    batch_shape = a.shape[:-2]
    out = np.empty(batch_shape + (m, n), _NP[c_type])
    if a.ndim > 2:
        # collapse batch dims: copy only if they do not collapse to one stride
        a3 = a.reshape((-1, m, k))
        b3 = b.reshape((-1, k, n))
    else:
        a3, b3 = a[None], b[None]
    nb = a3.shape[0]
    sa, sb = _elem_strides(a3), _elem_strides(b3)
    _lib.orc_gemm(_p(out), c_type, ctypes.c_void_p(a3.ctypes.data), ctypes.c_void_p(b3.ctypes.data),
                  ab_type, m, n, k, sa[1], sa[2], sb[1], sb[2], nb, sa[0], sb[0])
    return out


def conv_out_len(in_len, k, pad, stride, dilation, pad_hi=None):
    """op/quant_convolution.hpp:113-126 (the quotient truncates toward zero)."""
    span = in_len - (1 + dilation * (k - 1)) + pad + (pad if pad_hi is None else pad_hi)
    return max(1, int(span / stride) + 1)


def convolution(x, w, x_type, padding=None, stride=None, dilation=None, group=1):
    """convolution / quant_convolution of an [N, C, spatial...] input with [O, C/group, window...]
    weights over one, two or three spatial axes: int8 -> int32, fp8 -> float (double products),
    float -> float (float products, double sum).  `padding` holds one value per axis, or the low
    values followed by the high ones."""
    x = _c(x, _NP[x_type])
    w = _c(w, _NP[x_type])
    nd = x.ndim - 2
    assert 1 <= nd <= 3 and w.ndim == x.ndim
    padding = list(padding) if padding is not None else [0] * nd
    stride = list(stride) if stride is not None else [1] * nd
    dilation = list(dilation) if dilation is not None else [1] * nd
    n, c = x.shape[:2]
    o, cg = w.shape[:2]
    assert cg * group == c and o % group == 0
    hi = padding[nd:] if len(padding) == 2 * nd else padding   # (low..., high...) form
    out_sp = [conv_out_len(x.shape[2 + i], w.shape[2 + i], padding[i], stride[i], dilation[i], hi[i])
              for i in range(nd)]
    out_type = I32 if x_type == I8 else F32
    out = np.empty((n, o, *out_sp), _NP[out_type])
    lead = 3 - nd                                              # missing leading axes have length one

    def arr(v, fill):
        return np.ascontiguousarray([fill] * lead + [int(e) for e in v[:nd]], np.int64)

    a = [arr(x.shape[2:], 1), arr(w.shape[2:], 1), arr(padding, 0), arr(stride, 1), arr(dilation, 1), arr(out_sp, 1)]
    _lib.orc_convolution3d(_p(out), out_type, _p(x), _p(w), x_type, n, c, _p(a[0]), o, _p(a[1]), _p(a[2]),
                           _p(a[3]), _p(a[4]), group, _p(a[5]))
    return out


def quant_dot(a, b, ab_type=I8):
    """quant_dot: int8/uint8 -> int32, fp8 -> float (op/quant_dot.hpp:76-77)."""
    return gemm(a, b, ab_type, I32 if ab_type in (I8, U8) else F32)


def dot(a, b, ab_type):
    return gemm(a, b, ab_type, ab_type)


def _bcast2d(p, rows, cols, dtype):
    """Return (array, row_stride, col_stride) addressing a q-param as [r, c]."""
    p = np.asarray(p, dtype=dtype)
    if p.ndim == 0 or p.size == 1:
        return np.ascontiguousarray(p.reshape(1)), 0, 0
    if p.ndim == 1:
        if p.shape[0] == cols:
            return np.ascontiguousarray(p), 0, 1
        if p.shape[0] == rows:
            return np.ascontiguousarray(p), 1, 0
        raise ValueError("1-D parameter matches neither axis")
    p = np.ascontiguousarray(np.broadcast_to(p, (rows, cols)))
    return p, cols, 1


def quantizelinear(x, scale, zp, x_type, out_type):
    x = _c(x, _NP[x_type])
    shp = x.shape
    x2 = x.reshape(-1, shp[-1]) if x.ndim > 1 else x.reshape(1, -1)
    rows, cols = x2.shape
    s, ssr, ssc = _bcast2d(np.asarray(scale).reshape(-1, cols) if np.ndim(scale) > 2 else scale,
                           rows, cols, _NP[x_type])
    out = np.empty((rows, cols), _NP[out_type])
    if zp is None:
        _lib.orc_quantizelinear(_p(out), out_type, _p(x2), x_type, _p(s), ssr, ssc,
                                None, 0, 0, rows, cols)
    else:
        z, zsr, zsc = _bcast2d(np.asarray(zp).reshape(-1, cols) if np.ndim(zp) > 2 else zp,
                               rows, cols, _NP[out_type])
        _lib.orc_quantizelinear(_p(out), out_type, _p(x2), x_type, _p(s), ssr, ssc,
                                _p(z), zsr, zsc, rows, cols)
    return out.reshape(shp)


def dequantizelinear(x, scale, zp, x_type, s_type):
    x = _c(x, _NP[x_type])
    shp = x.shape
    x2 = x.reshape(-1, shp[-1]) if x.ndim > 1 else x.reshape(1, -1)
    rows, cols = x2.shape
    s, ssr, ssc = _bcast2d(np.asarray(scale).reshape(-1, cols) if np.ndim(scale) > 2 else scale,
                           rows, cols, _NP[s_type])
    out = np.empty((rows, cols), _NP[s_type])
    if zp is None:
        _lib.orc_dequantizelinear(_p(out), _p(x2), x_type, _p(s), s_type, ssr, ssc,
                                  None, 0, 0, rows, cols)
    else:
        z, zsr, zsc = _bcast2d(np.asarray(zp).reshape(-1, cols) if np.ndim(zp) > 2 else zp,
                               rows, cols, _NP[x_type])
        _lib.orc_dequantizelinear(_p(out), _p(x2), x_type, _p(s), s_type, ssr, ssc,
                                  _p(z), zsr, zsc, rows, cols)
    return out.reshape(shp)


def _axis_split(shape, axis):
    axis = axis % len(shape)
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return axis, outer, shape[axis], inner


def unpack_int4(x, axis=-1):
    signed = x.dtype == np.int8
    xc = np.ascontiguousarray(x)
    axis, outer, alen, inner = _axis_split(xc.shape, axis)
    shp = list(xc.shape)
    shp[axis] *= 2
    out = np.empty(shp, xc.dtype)
    _lib.orc_unpack_int4(_p(out), _p(xc), int(signed), outer, alen, inner)
    return out


def pack_int4(x, axis=-1):
    signed = x.dtype == np.int8
    xc = np.ascontiguousarray(x)
    axis, outer, alen, inner = _axis_split(xc.shape, axis)
    if alen % 2:
        raise ValueError("PACK_INT4: Can not pack axis that has odd lengths")
    shp = list(xc.shape)
    shp[axis] //= 2
    out = np.empty(shp, xc.dtype)
    _lib.orc_pack_int4(_p(out), _p(xc), int(signed), outer, alen // 2, inner)
    return out


def unpack_fp4(x, axis=-1):
    """fp4x2 bytes -> fp8 e4m3fn bytes, the axis doubled (op/unpack_fp4.hpp:78-101)."""
    xc = np.ascontiguousarray(x, dtype=np.uint8)
    axis, outer, alen, inner = _axis_split(xc.shape, axis)
    shp = list(xc.shape)
    shp[axis] *= 2
    out = np.empty(shp, np.uint8)
    _lib.orc_unpack_fp4(_p(out), _p(xc), outer, alen, inner)
    return out


def pack_fp4(x, axis=-1):
    """float32 -> fp4x2 bytes, the axis halved (op/pack_fp4.hpp:82-106)."""
    xc = np.ascontiguousarray(x, dtype=np.float32)
    axis, outer, alen, inner = _axis_split(xc.shape, axis)
    if alen % 2:
        raise ValueError("PACK_FP4: Can not pack along axis of odd length")
    shp = list(xc.shape)
    shp[axis] //= 2
    out = np.empty(shp, np.uint8)
    _lib.orc_pack_fp4(_p(out), _p(xc), outer, alen // 2, inner)
    return out


def fp4_to_f32(code):
    return float(_lib.orc_fp4_to_f32(int(code) & 0xff))


def fp4_from_f32(x):
    return int(_lib.orc_fp4_from_f32(float(x)))


def convert(x, x_type, out_type):
    x = _c(x, _NP[x_type])
    out = np.empty(x.shape, _NP[out_type])
    _lib.orc_convert(_p(out), out_type, _p(x), x_type, x.size)
    return out


def mul_f32(a, b, rows, cols):
    a, asr, asc = _bcast2d(a, rows, cols, np.float32)
    b, bsr, bsc = _bcast2d(b, rows, cols, np.float32)
    out = np.empty((rows, cols), np.float32)
    _lib.orc_mul_f32(_p(out), _p(a), asr, asc, _p(b), bsr, bsc, rows, cols)
    return out


# --- the composite paths of the benchmark configs ------------------------------

def qdq_matmul_int8(x_q, w_q, s_x, s_w, zp_x=0, zp_w=0, out_type=F32):
    """What simplify_qdq leaves for DQ(x_q) . DQ(w_q) (simplify_qdq.cpp:225-289):
    quant_dot -> int32, out_scale = mul(s_x, s_w) in fp32, zero-point terms as
    three extra quant_dots, dequantizelinear, optional convert."""
    m, k = x_q.shape
    n = w_q.shape[1]
    acc = quant_dot(x_q, w_q, I8)
    scale = mul_f32(np.asarray(s_x, np.float32), np.asarray(s_w, np.float32), m, n)
    zp = None
    if zp_x != 0 or zp_w != 0:
        zp = np.zeros((m, n), np.int32)
        zx = np.full((m, k), zp_x, np.int8)
        zw = np.full((k, n), zp_w, np.int8)
        if zp_x != 0:
            zp = zp + quant_dot(zx, w_q, I8)
        if zp_w != 0:
            zp = zp + quant_dot(x_q, zw, I8)
        if zp_x != 0 and zp_w != 0:
            zp = zp - quant_dot(zx, zw, I8)
        zp = zp.astype(np.int32)
    out = dequantizelinear(acc, scale, zp, I32, F32)
    if out_type != F32:
        out = convert(out, F32, out_type)
    return out


def qdq_matmul_fp8(x_q, w_q, s_x, s_w, out_type=F32, fp8_type=FP8):
    m = x_q.shape[0]
    n = w_q.shape[1]
    acc = quant_dot(x_q, w_q, fp8_type)
    scale = mul_f32(np.asarray(s_x, np.float32), np.asarray(s_w, np.float32), m, n)
    out = dequantizelinear(acc, scale, None, F32, F32)
    if out_type != F32:
        out = convert(out, F32, out_type)
    return out


def w4a16_matmul(a_h, w_packed, scales_h, zp, group):
    """unpack_int4 -> dequantizelinear(scales, zp) -> transpose -> dot, the
    graph of parse_matmulnbits.cpp:85-159 with fp16 activations and scales.

    a_h       [M, K] half bits, w_packed [N, K/2] uint8 (low nibble = even k),
    scales_h  [N, K/group] half bits, zp scalar or [N, K/group] uint8."""
    n, kh = w_packed.shape
    k = kh * 2
    q = unpack_int4(w_packed)                               # [N, K] u8
    s_full = np.repeat(scales_h, group, axis=1)[:, :k]
    if np.ndim(zp) == 0:
        z_full = np.full((n, k), zp, np.uint8)
    else:
        z_full = np.repeat(np.asarray(zp, np.uint8), group, axis=1)[:, :k]
    w = dequantizelinear(q, s_full, z_full, U8, F16)        # [N, K] half bits
    return dot(a_h, w.T, F16)


# ---- float operators around the GEMMs of an encoder graph -------------------------------------

BIN = {"add": 0, "sub": 1, "mul": 2, "div": 3}
UN = {"erf": 0, "sqrt": 1, "rsqrt": 2, "exp": 3, "tanh": 4, "neg": 5}


def binary_f32(op, a, b):
    a, b = np.broadcast_arrays(np.float32(a), np.float32(b))
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = np.empty(a.shape, np.float32)
    _lib.orc_binary_f32(BIN[op], _p(out), _p(a), _p(b), ctypes.c_size_t(a.size))
    return out


def unary_f32(op, x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.float32)
    _lib.orc_unary_f32(UN[op], _p(out), _p(x), ctypes.c_size_t(x.size))
    return out


def _reduced_last(x, axes):
    """x with the reduced axes moved to the end and flattened: [outer, reduced]."""
    axes = sorted(a % x.ndim for a in axes)
    keep = [d for d in range(x.ndim) if d not in axes]
    xt = np.ascontiguousarray(np.transpose(x, keep + axes))
    outer = int(np.prod([x.shape[d] for d in keep], dtype=np.int64))
    return xt.reshape(outer, -1), keep, axes


def reduce_mean_f32(x, axes):
    """Mean over `axes` (kept as length-1 dimensions), accumulated in double in index order."""
    x = np.float32(x)
    flat, keep, axes = _reduced_last(x, axes)
    out = np.empty(flat.shape[0], np.float32)
    _lib.orc_reduce_mean_f32(_p(out), _p(flat), ctypes.c_int64(flat.shape[0]),
                             ctypes.c_int64(flat.shape[1]), ctypes.c_int64(1))
    shp = [1 if d in axes else x.shape[d] for d in range(x.ndim)]
    return out.reshape(shp)


def softmax_f32(x, axis):
    x = np.ascontiguousarray(x, np.float32)
    axis, outer, alen, inner = _axis_split(x.shape, axis)
    out = np.empty(x.shape, np.float32)
    _lib.orc_softmax_f32(_p(out), _p(x), ctypes.c_int64(outer), ctypes.c_int64(alen),
                         ctypes.c_int64(inner))
    return out


def gather(data, indices, axis=0):
    data = np.ascontiguousarray(data)
    idx = np.asarray(indices, np.int64)
    axis, outer, alen, inner = _axis_split(data.shape, axis)
    scalar = idx.ndim == 0
    flat = np.ascontiguousarray(idx.reshape(-1))
    out = np.empty((outer, flat.size, inner), data.dtype)
    _lib.orc_gather(_p(out), _p(data), _p(flat), ctypes.c_int64(flat.size), ctypes.c_int64(outer),
                    ctypes.c_int64(alen), ctypes.c_int64(inner), ctypes.c_int64(data.itemsize))
    shp = list(data.shape[:axis]) + ([] if scalar else list(idx.shape)) + list(data.shape[axis + 1:])
    return out.reshape(shp)
