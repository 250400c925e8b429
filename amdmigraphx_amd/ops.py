"""Torch-tensor front end over the C ABI, used by the tests, the smoke check
and the benchmark.  torch supplies device memory and streams only; every
computation goes through ``libmi355_qgemm.so``.

Operator names and argument meaning follow the MIGraphX operators they stand
for (quant_dot, quantizelinear, dequantizelinear, unpack_int4, pack_int4,
convert); low-precision tensors without a torch dtype contract travel as raw
bits (uint8 for fp8 e4m3fn, int16/uint16 views for half and bf16 are taken from
torch.float16 / torch.bfloat16 tensors directly)."""
import ctypes

import torch

from .capi import DT, QP, W4ZP, QuantDotDesc, QuantConv3dDesc, QuantConvDesc, MxDotDesc, Mi355Error, check, lib

_TORCH2DT = {torch.int8: DT.I8, torch.uint8: DT.U8, torch.int32: DT.I32, torch.float32: DT.F32,
             torch.float16: DT.F16, torch.bfloat16: DT.BF16}
_DT2TORCH = {DT.I8: torch.int8, DT.U8: torch.uint8, DT.I32: torch.int32, DT.F32: torch.float32,
             DT.F16: torch.float16, DT.BF16: torch.bfloat16, DT.FP8: torch.uint8, DT.BF8: torch.uint8}


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _require_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise Mi355Error("operands must be device tensors")


def _mat_layout(t):
    """(trans, ld, batch_stride) of a [..., R, C] view that is row-major or a
    transpose of row-major storage in its last two dims."""
    r, c = t.shape[-2:]
    sr, sc = t.stride()[-2:]
    if sc == 1 or c == 1:
        return 0, max(sr if r > 1 else c, c, 1)
    if sr == 1 or r == 1:
        return 1, max(sc if c > 1 else r, r, 1)
    raise Mi355Error("matrix is neither row-major nor a transpose view")


def quant_dot(a, b, fp8=False, scale_a=None, scale_b=None, zp_a=0, zp_b=0,
              colsum_b=None, rowsum_a=None, out_dtype=None, out=None, bias=None, workspace=None):
    """quant_dot, optionally with the fused dequantizelinear epilogue.

    a [..., M, K], b [..., K, N] int8 (or uint8 carrying fp8 e4m3fn bits with
    fp8=True, fp8 e5m2 bits with fp8="e5m2"; plain uint8 operands give the bare int32 result
    only); transposed
    views are passed as they are.  Without scales the
    bare accumulators come back (int32 / float32).  With ``scale_a`` (scalar
    or [M]) / ``scale_b`` (scalar or [N]) float32 tensors the epilogue
    (double(acc) - zp) * (scale_a*scale_b) -> out_dtype is applied; ``bias`` (float32 [N])
    is then added in float32, before the conversion to a 16-bit ``out_dtype``.
    ``workspace`` (any dense device tensor, see quant_dot_workspace_size) lets a skinny int8
    product, bare or with the epilogue, split K over the chip without atomics; the word
    ``"static"`` takes the library's own static device buffer instead (nothing is allocated,
    shapes that need more than it holds are refused)."""
    _require_cuda(a, b, scale_a, scale_b, bias, None if isinstance(workspace, str) else workspace)
    if a.dim() != b.dim() or a.dim() < 2:
        raise Mi355Error("QUANT_DOT: dot only accepts >= 2D operands of equal rank")
    if a.shape[:-2] != b.shape[:-2]:
        raise Mi355Error("QUANT_DOT: outer dimensions of A and B mismatch")
    if a.shape[-1] != b.shape[-2]:
        raise Mi355Error("QUANT_DOT: inner dimensions are not compatible")
    if a.dtype != b.dtype:
        raise Mi355Error("QUANT_DOT: operands must have the same type")
    batch_shape = a.shape[:-2]
    m, k = a.shape[-2:]
    n = b.shape[-1]
    nb = 1
    for s in batch_shape:
        nb *= s
    if a.dim() > 2:
        a3 = a.reshape((nb, m, k)) if a.dim() > 3 else a
        b3 = b.reshape((nb, k, n)) if b.dim() > 3 else b
        sa, sb = a3.stride(0), b3.stride(0)
    else:
        a3, b3, sa, sb = a, b, 0, 0
    ta, lda = _mat_layout(a3)
    tb, ldb = _mat_layout(b3)
    dequant = scale_a is not None or scale_b is not None or out_dtype is not None
    in_type = _fp8_dt(fp8, a)
    if dequant:
        odt = out_dtype or torch.float32
    else:
        odt = torch.float32 if fp8 else torch.int32
    if out is None:
        out = torch.empty(batch_shape + (m, n), dtype=odt, device=a.device)
    # C may be a row-strided view (columns contiguous, batches evenly spaced)
    if out.stride(-1) != 1 and n > 1:
        raise Mi355Error("quant_dot: the output's last dimension must be contiguous")
    ldc = out.stride(-2) if m > 1 else max(n, out.stride(-2))
    stride_c = m * ldc
    if out.dim() > 2 and nb > 1:
        if out.dim() > 3 and not out.flatten(0, -3).is_contiguous():
            raise Mi355Error("quant_dot: batch dimensions of the output must be dense")
        stride_c = out.stride(-3)
    # one vector of column scales (and one bias) per batch entry: scale_b dense [batch, N]
    cols_per_batch = (scale_b is not None and nb > 1 and scale_b.dim() >= 2 and scale_b.numel() == nb * n and
                      scale_b.is_contiguous())
    d = QuantDotDesc(m=m, n=n, k=k, lda=lda, ldb=ldb, ldc=ldc, batch=nb, stride_a=sa, stride_b=sb,
                     stride_c=stride_c, trans_a=ta, trans_b=tb, in_type=in_type,
                     out_type=_TORCH2DT[odt], dequant=int(dequant),
                     scale_a_mode=QP.NONE if scale_a is None else
                     (QP.PER_TENSOR if scale_a.numel() == 1 else QP.PER_ROW),
                     scale_b_mode=QP.NONE if scale_b is None else
                     (QP.PER_TENSOR if scale_b.numel() == 1 else
                      QP.PER_COL_BATCH if cols_per_batch else QP.PER_COL),
                     zp_a=int(zp_a), zp_b=int(zp_b))
    if scale_a is not None and scale_a.numel() not in (1, m):
        raise Mi355Error("scale_a must be a scalar or have M elements")
    if scale_b is not None and scale_b.numel() not in (1, n) and not cols_per_batch:
        raise Mi355Error("scale_b must be a scalar, have N elements, or batch x N of them (dense)")
    if bias is not None:
        if not dequant:
            raise Mi355Error("quant_dot: a bias needs the dequantizing epilogue")
        if bias.dtype != torch.float32 or bias.numel() != (nb * n if cols_per_batch else n) or \
                not bias.is_contiguous():
            raise Mi355Error("bias must be a dense float32 vector of N elements (batch x N with such scales)")
    if isinstance(workspace, str):
        if workspace != "static":
            raise Mi355Error("workspace must be a device tensor or the word 'static'")
        st = lib().mi355_quant_dot_static(ctypes.byref(d), _ptr(a3), _ptr(b3), _ptr(out), _ptr(scale_a),
                                          _ptr(scale_b), _ptr(colsum_b), _ptr(rowsum_a), _ptr(bias), _stream())
        check(st, "mi355_quant_dot_static")
    elif workspace is not None:
        if not workspace.is_contiguous():
            raise Mi355Error("the workspace must be dense")
        st = lib().mi355_quant_dot_ws(ctypes.byref(d), _ptr(a3), _ptr(b3), _ptr(out), _ptr(scale_a),
                                      _ptr(scale_b), _ptr(colsum_b), _ptr(rowsum_a), _ptr(bias), _ptr(workspace),
                                      workspace.numel() * workspace.element_size(), _stream())
        check(st, "mi355_quant_dot_ws")
    elif bias is not None:
        st = lib().mi355_quant_dot_bias(ctypes.byref(d), _ptr(a3), _ptr(b3), _ptr(out), _ptr(scale_a),
                                        _ptr(scale_b), _ptr(colsum_b), _ptr(rowsum_a), _ptr(bias), _stream())
        check(st, "mi355_quant_dot_bias")
    else:
        st = lib().mi355_quant_dot(ctypes.byref(d), _ptr(a3), _ptr(b3), _ptr(out), _ptr(scale_a),
                                   _ptr(scale_b), _ptr(colsum_b), _ptr(rowsum_a), _stream())
        check(st, "mi355_quant_dot")
    return out


def _fp8_dt(fp8, t):
    return DT.BF8 if fp8 == "e5m2" else DT.FP8 if fp8 else (DT.U8 if t.dtype == torch.uint8 else DT.I8)


def quant_dot_prepack(b, fp8=False):
    """Reorder a constant B [K, N] (any strides: a transposed view is read as it lies) once, for
    quant_dot_prepacked.  Returns None for a shape or type the reordered form does not take."""
    _require_cuda(b)
    if b.dim() != 2:
        raise Mi355Error("quant_dot_prepack: B is a matrix")
    k, n = b.shape
    it = _fp8_dt(fp8, b)
    size = lib().mi355_quant_dot_prepacked_size(it, n, k)
    if size == 0:
        return None
    out = torch.empty(size, dtype=torch.uint8, device=b.device)
    check(lib().mi355_quant_dot_prepack(_ptr(b), it, n, k, b.stride(0), b.stride(1), _ptr(out), _stream()),
          "mi355_quant_dot_prepack")
    return out


def quant_dot_prepacked(a, b_prepacked, n, fp8=False, scale_a=None, scale_b=None, zp_a=0, zp_b=0,
                        colsum_b=None, rowsum_a=None, out_dtype=None, out=None, bias=None):
    """quant_dot of a [M <= 16, K] against a B reordered by quant_dot_prepack, with the epilogue
    arguments of quant_dot; one launch, no workspace."""
    _require_cuda(a, b_prepacked, scale_a, scale_b, bias)
    if a.dim() != 2 or a.stride(1) != 1:
        raise Mi355Error("quant_dot_prepacked: A is a row-major matrix")
    m, k = a.shape
    dequant = scale_a is not None or scale_b is not None or out_dtype is not None
    odt = (out_dtype or torch.float32) if dequant else (torch.float32 if fp8 else torch.int32)
    if out is None:
        out = torch.empty((m, n), dtype=odt, device=a.device)
    d = QuantDotDesc(m=m, n=n, k=k, lda=a.stride(0) if m > 1 else max(k, a.stride(0)), ldb=n,
                     ldc=out.stride(0) if m > 1 else max(n, out.stride(0)), batch=1, stride_a=0, stride_b=0,
                     stride_c=0, trans_a=0, trans_b=0, in_type=_fp8_dt(fp8, a), out_type=_TORCH2DT[out.dtype],
                     dequant=int(dequant),
                     scale_a_mode=QP.NONE if scale_a is None else
                     (QP.PER_TENSOR if scale_a.numel() == 1 else QP.PER_ROW),
                     scale_b_mode=QP.NONE if scale_b is None else
                     (QP.PER_TENSOR if scale_b.numel() == 1 else QP.PER_COL),
                     zp_a=int(zp_a), zp_b=int(zp_b))
    check(lib().mi355_quant_dot_prepacked(ctypes.byref(d), _ptr(a), _ptr(b_prepacked), _ptr(out), _ptr(scale_a),
                                          _ptr(scale_b), _ptr(colsum_b), _ptr(rowsum_a), _ptr(bias), _stream()),
          "mi355_quant_dot_prepacked")
    return out


def quant_dot_mx(a, b_nk, scale_a, scale_b, a_fp4=False, b_fp4=False, out=None, workspace=None):
    """Four-input quant_dot of block-scaled operands: C = (float(A) * SA) . (float(B) * SB)^T.

    ``a`` [..., M, K] and ``b_nk`` [..., N, K] are uint8 tensors of e4m3fn codes, or with
    ``a_fp4`` / ``b_fp4`` of packed e2m1 pairs ([..., M, K/2], low nibble = even k).  The scales are
    float32, either of the operand's logical shape ([..., M, K], the operator's form) or compact
    ([..., M, K/32], one per block).  Returns float32 [..., M, N].  ``workspace``: a dense uint8
    device tensor to use (and keep between calls) instead of a fresh allocation."""
    _require_cuda(a, b_nk, scale_a, scale_b)
    if a.dtype != torch.uint8 or b_nk.dtype != torch.uint8:
        raise Mi355Error("quant_dot_mx: operands are uint8 tensors of fp8 codes or packed fp4 pairs")
    a, b_nk = a.contiguous(), b_nk.contiguous()
    scale_a, scale_b = scale_a.contiguous(), scale_b.contiguous()
    batch_shape = a.shape[:-2]
    if b_nk.shape[:-2] != batch_shape:
        raise Mi355Error("QUANT_DOT: outer dimensions of A and B mismatch")
    m, n = a.shape[-2], b_nk.shape[-2]
    k = a.shape[-1] * (2 if a_fp4 else 1)
    if b_nk.shape[-1] * (2 if b_fp4 else 1) != k:
        raise Mi355Error("QUANT_DOT: inner dimensions are not compatible")
    nb = 1
    for v in batch_shape:
        nb *= v

    def scale_strides(sc, rows):
        if sc.dtype != torch.float32 or sc.shape[:-1] != batch_shape + (rows,):
            raise Mi355Error("quant_dot_mx: scales must be float32 of the operand's shape or [rows, K/32]")
        cols = sc.shape[-1]
        if cols == k:
            return rows * k, k, 32, 1
        if cols * 32 == k:
            return rows * cols, cols, 1, 0
        raise Mi355Error("quant_dot_mx: scales must have K or K/32 columns")

    sab, sar, sak, sae = scale_strides(scale_a, m)
    sbb, sbr, sbk, sbe = scale_strides(scale_b, n)
    if out is None:
        out = torch.empty(batch_shape + (m, n), dtype=torch.float32, device=a.device)
    d = MxDotDesc(m=m, n=n, k=k, batch=nb, lda=a.shape[-1], ldb=b_nk.shape[-1], ldc=n,
                  stride_a=m * a.shape[-1], stride_b=n * b_nk.shape[-1], stride_c=m * n,
                  sa_batch=sab, sa_row=sar, sa_block=sak, sa_elem=sae,
                  sb_batch=sbb, sb_row=sbr, sb_block=sbk, sb_elem=sbe,
                  a_type=DT.FP4X2 if a_fp4 else DT.FP8, b_type=DT.FP4X2 if b_fp4 else DT.FP8)
    need = int(lib().mi355_quant_dot_mx_workspace_size(ctypes.byref(d)))
    ws = workspace if workspace is not None else torch.empty(max(need, 16), dtype=torch.uint8, device=a.device)
    if ws.numel() * ws.element_size() < need or not ws.is_contiguous():
        raise Mi355Error("quant_dot_mx: the workspace is too small or not dense")
    check(lib().mi355_quant_dot_mx(ctypes.byref(d), _ptr(a), _ptr(b_nk), _ptr(out), _ptr(scale_a), _ptr(scale_b),
                                   _ptr(ws), need, _stream()), "mi355_quant_dot_mx")
    return out


def dot(a, b, scale=None, fp32acc=False):
    """Float `dot` of float32 / float16 / bfloat16 tensors [..., M, K] . [..., K, N] (any strides
    inside a matrix, batches dense).  By default the reference's double sum bit for bit; with
    ``fp32acc`` (float32 only) on the fp32 matrix cores.  ``scale``: one float32 the result is
    multiplied by."""
    _require_cuda(a, b, scale)
    if a.dtype != b.dtype or a.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise Mi355Error("dot: float32, float16 or bfloat16 operands of one type")
    if a.dim() != b.dim() or a.dim() < 2 or a.shape[:-2] != b.shape[:-2] or a.shape[-1] != b.shape[-2]:
        raise Mi355Error("DOT: operands do not fit")
    m, k = a.shape[-2:]
    n = b.shape[-1]
    nb = 1
    for v in a.shape[:-2]:
        nb *= v
    a3 = a.reshape((nb, m, k)) if a.dim() != 3 else a
    b3 = b.reshape((nb, k, n)) if b.dim() != 3 else b
    out = torch.empty(a.shape[:-2] + (m, n), dtype=a.dtype, device=a.device)
    fn = lib().mi355_dot_fp32acc if fp32acc else lib().mi355_dot_scaled
    check(fn(_ptr(a3), _ptr(b3), _ptr(out), _TORCH2DT[a.dtype], m, n, k, a3.stride(1), a3.stride(2),
             b3.stride(1), b3.stride(2), n, nb, a3.stride(0) if nb > 1 else 0, b3.stride(0) if nb > 1 else 0,
             m * n, _ptr(scale), _stream()), "mi355_dot")
    return out


def quant_dot_workspace_size(m, n, k, batch=1, trans_b=False, fp8=False):
    """Bytes of workspace an int8 (or fp8) quant_dot of that shape can use (0: none)."""
    d = QuantDotDesc(m=m, n=n, k=k, batch=batch, lda=k, ldb=k if trans_b else n, ldc=n,
                     stride_a=m * k, stride_b=k * n, stride_c=m * n, trans_a=0, trans_b=int(trans_b),
                     in_type=DT.FP8 if fp8 else DT.I8, out_type=DT.F32 if fp8 else DT.I32, dequant=0)
    return int(lib().mi355_quant_dot_workspace_size(ctypes.byref(d)))


def quant_convolution(x, w, padding=None, stride=None, dilation=None, group=1, fp8=False,
                      scale_x=None, scale_w=None, out_dtype=None, out=None, workspace=None):
    """quant_convolution of a dense [N, C, spatial...] tensor with dense [O, C/group, window...]
    weights over one, two or three spatial axes (int8, or uint8 carrying fp8 e4m3fn codes with
    fp8=True), optionally with the dequantizing epilogue: ``scale_x`` one float, ``scale_w`` one
    float or one per output channel.  ``padding`` holds one value per spatial axis for both sides,
    or the low values followed by the high ones.  ``out`` (dense, of the result's shape and type)
    and ``workspace`` (a uint8 tensor of at least the size the library asks for) are allocated
    here unless the caller brings them, e.g. to reuse them from call to call."""
    _require_cuda(x, w, scale_x, scale_w)
    nd = x.dim() - 2
    if nd < 1 or nd > 3 or w.dim() != x.dim():
        raise Mi355Error("QUANT_CONVOLUTION: input and weights must have 3 to 5 dimensions, and the same number")
    if x.dtype != w.dtype:
        raise Mi355Error("QUANT_CONVOLUTION: Types do not match")
    if not x.is_contiguous() or not w.is_contiguous():
        raise Mi355Error("quant_convolution: input and weights must be dense")
    padding = list(padding) if padding is not None else [0] * nd
    stride = list(stride) if stride is not None else [1] * nd
    dilation = list(dilation) if dilation is not None else [1] * nd
    if len(padding) not in (nd, 2 * nd) or len(stride) != nd or len(dilation) != nd:
        raise Mi355Error("QUANT_CONVOLUTION: inconsistent attribute sizes")
    n, c = x.shape[:2]
    o, cg = w.shape[:2]
    if group < 1 or cg * group != c or o % group != 0:
        raise Mi355Error("QUANT_CONVOLUTION: mismatched channel numbers")
    dequant = scale_x is not None or scale_w is not None or out_dtype is not None
    odt = (out_dtype or torch.float32) if dequant else (torch.float32 if fp8 else torch.int32)
    pad_hi = padding[nd:] if len(padding) == 2 * nd else padding
    if scale_x is not None and scale_x.numel() != 1:
        raise Mi355Error("scale_x must be a single value")
    if scale_w is not None and scale_w.numel() not in (1, o):
        raise Mi355Error("scale_w must be a scalar or have one value per output channel")
    # the descriptor and the result's size depend on the shapes and attributes only: kept per
    # combination, so that a layer called again costs one library call
    key = (tuple(x.shape), tuple(w.shape), tuple(padding), tuple(stride), tuple(dilation), group, fp8, odt, dequant,
           scale_x is None, None if scale_w is None else scale_w.numel() == 1)
    plan = _CONV_PLANS.get(key)
    if plan is None:
        plan = _conv_plan(x, w, nd, n, c, o, padding, pad_hi, stride, dilation, group, fp8, odt, dequant, scale_x,
                          scale_w)
        if len(_CONV_PLANS) < 256:
            _CONV_PLANS[key] = plan
    d, out_spatial, need_bytes, run, what = plan
    shape = (n, o, *out_spatial)
    if out is None:
        out = torch.empty(shape, dtype=odt, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != odt or not out.is_contiguous() or out.device != x.device:
        raise Mi355Error("quant_convolution: out must be a dense tensor of the result's shape and type")
    if workspace is None:
        workspace = torch.empty(max(need_bytes, 16), dtype=torch.uint8, device=x.device)
    elif workspace.dtype != torch.uint8 or workspace.numel() < need_bytes or workspace.device != x.device:
        raise Mi355Error(f"quant_convolution: workspace must be a uint8 tensor of at least {need_bytes} bytes")
    check(run(ctypes.byref(d), _ptr(x), _ptr(w), _ptr(out), _ptr(scale_x), _ptr(scale_w), _ptr(workspace),
              need_bytes, _stream()), what)
    return out


_CONV_PLANS = {}


def _conv_plan(x, w, nd, n, c, o, padding, pad_hi, stride, dilation, group, fp8, odt, dequant, scale_x, scale_w):
    """(descriptor, spatial lengths of the result, workspace bytes, entry point, its name)"""
    common = dict(group=group, in_type=DT.FP8 if fp8 else DT.I8, out_type=_TORCH2DT[odt], dequant=int(dequant),
                  scale_x_mode=QP.NONE if scale_x is None else QP.PER_TENSOR,
                  scale_w_mode=QP.NONE if scale_w is None else
                  (QP.PER_TENSOR if scale_w.numel() == 1 else QP.PER_ROW))
    need = ctypes.c_size_t()
    if nd == 2:
        d = QuantConvDesc(n=n, c=c, h=x.shape[2], w=x.shape[3], o=o, kh=w.shape[2], kw=w.shape[3],
                          pad_h=padding[0], pad_w=padding[1], pad_h_hi=pad_hi[0], pad_w_hi=pad_hi[1],
                          stride_h=stride[0], stride_w=stride[1], dil_h=dilation[0], dil_w=dilation[1], **common)
        oh, ow = ctypes.c_int64(), ctypes.c_int64()
        check(lib().mi355_quant_convolution_dims(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow),
                                                 ctypes.byref(need)), "mi355_quant_convolution_dims")
        out_spatial = [oh.value, ow.value]
        run, what = lib().mi355_quant_convolution, "mi355_quant_convolution"
    else:
        # one spatial axis: a depth and a height of one in front
        lead = 3 - nd
        three = ctypes.c_int64 * 3
        sp = [1] * lead + list(x.shape[2:])
        win = [1] * lead + list(w.shape[2:])
        d = QuantConv3dDesc(n=n, c=c, d=sp[0], h=sp[1], w=sp[2], o=o, kd=win[0], kh=win[1], kw=win[2],
                            pad=three(*([0] * lead + padding[:nd])), pad_hi=three(*([0] * lead + list(pad_hi))),
                            stride=three(*([1] * lead + stride)), dil=three(*([1] * lead + dilation)), **common)
        lens = three()
        check(lib().mi355_quant_convolution3d_dims(ctypes.byref(d), lens, ctypes.byref(need)),
              "mi355_quant_convolution3d_dims")
        out_spatial = list(lens)[lead:]
        run, what = lib().mi355_quant_convolution3d, "mi355_quant_convolution3d"
    return d, out_spatial, need.value, run, what


def colsum_i8(b):
    k, n = b.shape
    tb, ldb = _mat_layout(b)
    out = torch.empty(n, dtype=torch.int32, device=b.device)
    check(lib().mi355_colsum_i8(_ptr(b), k, n, ldb, tb, _ptr(out), _stream()), "mi355_colsum_i8")
    return out


def rowsum_i8(a):
    m, k = a.shape
    ta, lda = _mat_layout(a)
    out = torch.empty(m, dtype=torch.int32, device=a.device)
    check(lib().mi355_rowsum_i8(_ptr(a), m, k, lda, ta, _ptr(out), _stream()), "mi355_rowsum_i8")
    return out


def _qparam_strides(p, rows, cols):
    if p is None:
        return 0, 0
    if p.numel() == 1:
        return 0, 0
    if p.dim() == 1 and p.numel() == cols:
        return 0, 1
    if p.dim() == 1 and p.numel() == rows:
        return 1, 0
    if p.numel() == rows * cols:
        return cols, 1
    raise Mi355Error("quantization parameter does not broadcast to the input")


def quantizelinear(x, scale, zp=None, out_type=DT.I8):
    """quantizelinear of a dense tensor (last dim = columns).  ``scale`` has
    x's dtype; ``zp`` the output's (uint8 bits for fp8)."""
    _require_cuda(x, scale, zp)
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    if scale.dtype != x.dtype:
        raise Mi355Error("QUANTIZELINEAR: Scales and input must be the same type")
    out = torch.empty(x.shape, dtype=_DT2TORCH[out_type], device=x.device)
    ssr, ssc = _qparam_strides(scale, rows, cols)
    zsr, zsc = _qparam_strides(zp, rows, cols)
    st = lib().mi355_quantizelinear(_ptr(x), _TORCH2DT[x.dtype], _ptr(scale.contiguous()), ssr, ssc,
                                    _ptr(None if zp is None else zp.contiguous()), zsr, zsc,
                                    _ptr(out), out_type, rows, cols, _stream())
    check(st, "mi355_quantizelinear")
    return out


def dequantizelinear(x, scale, zp=None, x_type=None):
    _require_cuda(x, scale, zp)
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    xt = x_type if x_type is not None else _TORCH2DT[x.dtype]
    out = torch.empty(x.shape, dtype=scale.dtype, device=x.device)
    ssr, ssc = _qparam_strides(scale, rows, cols)
    zsr, zsc = _qparam_strides(zp, rows, cols)
    st = lib().mi355_dequantizelinear(_ptr(x), xt, _ptr(scale.contiguous()), _TORCH2DT[scale.dtype],
                                      ssr, ssc, _ptr(None if zp is None else zp.contiguous()),
                                      zsr, zsc, _ptr(out), rows, cols, _stream())
    check(st, "mi355_dequantizelinear")
    return out


def unpack_fp4(x):
    """fp4x2 bytes (uint8) -> fp8 e4m3fn bits (uint8), last axis doubled."""
    _require_cuda(x)
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    out = torch.empty(x.shape[:-1] + (cols * 2,), dtype=torch.uint8, device=x.device)
    check(lib().mi355_unpack_fp4(_ptr(x), _ptr(out), rows, cols, _stream()), "mi355_unpack_fp4")
    return out


def pack_fp4(x):
    """float32 -> fp4x2 bytes (uint8), last axis halved."""
    _require_cuda(x)
    if x.dtype != torch.float32:
        raise Mi355Error("pack_fp4: float32 input")
    x = x.contiguous()
    cols = x.shape[-1]
    if cols % 2:
        raise Mi355Error("PACK_FP4: Can not pack along axis of odd length")
    rows = x.numel() // max(cols, 1)
    out = torch.empty(x.shape[:-1] + (cols // 2,), dtype=torch.uint8, device=x.device)
    check(lib().mi355_pack_fp4(_ptr(x), _ptr(out), rows, cols, _stream()), "mi355_pack_fp4")
    return out


def _int4_nd(fn_name, x, axis, out_shape):
    nd = x.dim()
    if nd > 8:
        raise Mi355Error("at most 8 dimensions")
    lens = (ctypes.c_int64 * nd)(*x.shape)
    strides = (ctypes.c_int64 * nd)(*x.stride())
    out = torch.empty(out_shape, dtype=x.dtype, device=x.device)
    check(getattr(lib(), fn_name)(_ptr(x), _ptr(out), int(x.dtype == torch.int8), nd, lens, strides,
                                  axis, _stream()), fn_name)
    return out


def unpack_int4(x, axis=-1):
    """unpack_int4 along ``axis`` of any strided view (transposed, expanded): the result is dense."""
    _require_cuda(x)
    ax = axis % x.dim()
    shp = list(x.shape)
    shp[ax] *= 2
    if ax == x.dim() - 1 and x.is_contiguous():
        cols = x.shape[-1]
        rows = x.numel() // max(cols, 1)
        out = torch.empty(shp, dtype=x.dtype, device=x.device)
        check(lib().mi355_unpack_int4(_ptr(x), _ptr(out), int(x.dtype == torch.int8), rows, cols,
                                      _stream()), "mi355_unpack_int4")
        return out
    return _int4_nd("mi355_unpack_int4_nd", x, ax, shp)


def pack_int4(x, axis=-1):
    _require_cuda(x)
    ax = axis % x.dim()
    shp = list(x.shape)
    if shp[ax] % 2:
        raise Mi355Error("PACK_INT4: Can not pack axis that has odd lengths")
    shp[ax] //= 2
    if ax == x.dim() - 1 and x.is_contiguous():
        cols = x.shape[-1]
        rows = x.numel() // max(cols, 1)
        out = torch.empty(shp, dtype=x.dtype, device=x.device)
        check(lib().mi355_pack_int4(_ptr(x), _ptr(out), int(x.dtype == torch.int8), rows, cols,
                                    _stream()), "mi355_pack_int4")
        return out
    return _int4_nd("mi355_pack_int4_nd", x, ax, shp)


def convert(x, out_type, in_type=None):
    x = x.contiguous()
    it = in_type if in_type is not None else _TORCH2DT[x.dtype]
    out = torch.empty(x.shape, dtype=_DT2TORCH[out_type], device=x.device)
    check(lib().mi355_convert(_ptr(x), it, _ptr(out), out_type, x.numel(), _stream()),
          "mi355_convert")
    return out


def w4a16_gemm(a, w_packed, scales, group, zp=8, zp_mode=None, out=None, workspace=None):
    """fp16 activations [M, K] times int4 weights packed [N, K/2] with fp16
    group scales [N, K/group]; zp is an int (per tensor) or a uint8 tensor.
    ``workspace`` (a dense device tensor, see w4a16_gemm_workspace_size) lets shapes whose
    column tiles do not fill the chip split K."""
    _require_cuda(a, w_packed, scales, workspace)
    m, k = a.shape
    n = w_packed.shape[0]
    if w_packed.shape[1] * 2 != k:
        raise Mi355Error("packed weight does not match K")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    if isinstance(zp, int):
        zptr, mode, zs = None, W4ZP.SCALAR, zp
    else:
        zptr, zs = _ptr(zp), 0
        mode = zp_mode if zp_mode is not None else W4ZP.GROUP
    if workspace is not None:
        if not workspace.is_contiguous():
            raise Mi355Error("the workspace must be dense")
        st = lib().mi355_w4a16_gemm_ws(_ptr(a), a.stride(0), _ptr(w_packed), _ptr(scales), zptr, mode, zs,
                                       _ptr(out), out.stride(0), m, n, k, group, _ptr(workspace),
                                       workspace.numel() * workspace.element_size(), _stream())
        check(st, "mi355_w4a16_gemm_ws")
        return out
    st = lib().mi355_w4a16_gemm(_ptr(a), a.stride(0), _ptr(w_packed), _ptr(scales), zptr, mode, zs,
                                _ptr(out), out.stride(0), m, n, k, group, _stream())
    check(st, "mi355_w4a16_gemm")
    return out


def w4a16_prepack(w_packed, scales, group, zp=8):
    """Reorder constant int4 weights [N, K/2] and their fp16 group scales [N, K/group] once for
    w4a16_gemm_prepacked; returns the device buffer, or None when the reordered form does not
    take the shape."""
    _require_cuda(w_packed, scales)
    n, k = w_packed.shape[0], w_packed.shape[1] * 2
    size = int(lib().mi355_w4a16_prepacked_size(n, k, group))
    if size == 0:
        return None
    if not (w_packed.is_contiguous() and scales.is_contiguous()):
        raise Mi355Error("weights and scales must be dense")
    out = torch.empty(size, dtype=torch.uint8, device=w_packed.device)
    check(lib().mi355_w4a16_prepack(_ptr(w_packed), _ptr(scales), zp, n, k, group, _ptr(out), _stream()),
          "mi355_w4a16_prepack")
    return out


def w4a16_gemm_prepacked(a, prepacked, n, out=None):
    """fp16 activations [M, K] times weights reordered by w4a16_prepack (N rows)."""
    _require_cuda(a, prepacked)
    m, k = a.shape
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=a.device)
    check(lib().mi355_w4a16_gemm_prepacked(_ptr(a), a.stride(0), _ptr(prepacked), _ptr(out), out.stride(0),
                                           m, n, k, _stream()), "mi355_w4a16_gemm_prepacked")
    return out


def w4a16_gemm_workspace_size(m, n, k, group):
    """Bytes of workspace w4a16_gemm can use for that shape (0: none)."""
    return int(lib().mi355_w4a16_gemm_workspace_size(m, n, k, group))
