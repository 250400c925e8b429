/*
 * mi355_qgemm.h -- C ABI of the MI355X (gfx950) quantized-GEMM kernels.
 *
 * This is the boundary a MIGraphX target's lowered operators call from their
 * `compute(context&, shape, args)`: plain device pointers and sizes in, a
 * status code out.  Every entry point
 *   - takes DEVICE pointers only (HBM resident operands),
 *   - launches on the hipStream_t passed as `stream` (a void*; NULL = the
 *     default stream) and returns without synchronising,
 *   - allocates nothing and keeps no state between calls (re-entrant across
 *     streams),
 *   - returns MI355_OK or a negative mi355_status; it never throws.
 *
 * Each function names the reference operator whose `ref` target arithmetic it
 * reproduces (paths relative to the MIGraphX source tree).
 */
#ifndef MI355_QGEMM_H
#define MI355_QGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mi355_status {
    MI355_OK              = 0,
    MI355_ERR_BAD_ARG     = -1, /* null pointer, negative size, bad enum */
    MI355_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for */
    MI355_ERR_LAUNCH      = -3, /* HIP reported an error at launch */
    MI355_ERR_SCRATCH_TOO_SMALL = -4 /* mi355_quant_dot_static: the split needs more than the static buffer */
} mi355_status;

/* Element types.  half / bf16 / fp8 are passed as their raw bits. */
typedef enum mi355_dtype {
    MI355_I8   = 0,
    MI355_U8   = 1,
    MI355_I32  = 2,
    MI355_F32  = 3,
    MI355_F16  = 4, /* IEEE binary16 */
    MI355_BF16 = 5,
    MI355_FP8  = 6, /* OCP e4m3fn */
    MI355_FP4X2 = 7, /* two OCP e2m1 codes per byte, low nibble = even element (block-scaled operands) */
    MI355_BF8  = 8  /* OCP e5m2 (shape::fp8e5m2_type, src/include/migraphx/float8.hpp:102-116) */
} mi355_dtype;

/* How a quantization parameter is broadcast over an [M, N] result. */
typedef enum mi355_qparam_mode {
    MI355_QP_NONE       = 0, /* absent: scale 1, zero point 0 */
    MI355_QP_PER_TENSOR = 1, /* one element */
    MI355_QP_PER_ROW    = 2, /* [M] */
    MI355_QP_PER_COL    = 3, /* [N] */
    MI355_QP_PER_COL_BATCH = 4 /* scale_b only: [batch, N], one vector of column scales per batch entry, and
                                  the bias likewise [batch, N] -- several layers that read the same
                                  activations (stride_a = 0) as one launch.  int8 with the dequantizing
                                  epilogue, N % 4 == 0, shapes of the matrix-core path; else
                                  MI355_ERR_UNSUPPORTED.  No counterpart in the reference's operator, which
                                  has no fused epilogue. */
} mi355_qparam_mode;

/*
 * Problem description of one (batched) quant_dot, optionally with the
 * dequantizelinear epilogue that simplify_qdq puts behind it.
 *
 * A is [batch, M, K]; element (b, m, k) lives at  a + b*stride_a + m*lda + k
 *   (trans_a = 0) or a + b*stride_a + k*lda + m (trans_a = 1, a transpose
 *   view of [K, M] storage).
 * B is [batch, K, N]; element (b, k, n) lives at  b + b*stride_b + k*ldb + n
 *   (trans_b = 0) or b + b*stride_b + n*ldb + k (trans_b = 1, the transpose
 *   view of [N, K] storage that simplify_qdq.cpp:49-82 produces when the
 *   weight's transpose sat between dequantizelinear and dot).
 * C is [batch, M, N] row-major with leading dimension ldc.
 * All strides are in elements.
 */
typedef struct mi355_quant_dot_desc {
    int64_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t batch;
    int64_t stride_a, stride_b, stride_c;
    int32_t trans_a, trans_b;
    int32_t in_type;  /* MI355_I8, MI355_FP8 or MI355_BF8; MI355_U8 for the bare result only */
    int32_t out_type; /* MI355_I32 / MI355_F32: bare quant_dot result (int8 / fp8).
                         With an epilogue: MI355_F32, MI355_F16 or MI355_BF16. */
    /* ---- fused dequantizelinear epilogue (all zero = bare quant_dot) ---- */
    int32_t dequant;      /* 0: store accumulators, 1: apply the epilogue     */
    int32_t scale_a_mode; /* MI355_QP_NONE / PER_TENSOR / PER_ROW             */
    int32_t scale_b_mode; /* MI355_QP_NONE / PER_TENSOR / PER_COL             */
    int32_t zp_a, zp_b;   /* zero points of the quantized A and B (int8 only) */
} mi355_quant_dot_desc;

/*
 * quant_dot (+ fused dequantizelinear).
 *
 * Replaces: ref_quant_gemm::compute (src/targets/ref/lowering.cpp:218-248) ->
 * gemm_naive (src/gemm.cpp:42-63) with the shape rules of
 * op::quant_dot::compute_shape (src/include/migraphx/op/quant_dot.hpp:51-121):
 * int8 x int8 -> int32 (exact), fp8 e4m3fn x fp8 e4m3fn -> float, fp8 e5m2 x fp8 e5m2 -> float
 * (op/quant_dot.hpp:62-66 takes every fp8 type; both operands have the same one).
 *
 * With desc->dequant it also replaces the instructions simplify_qdq.cpp:225-289
 * emits behind the quant_dot and that the ref target evaluates one by one:
 *   scale[m,n] = scale_a[m or 0] * scale_b[n or 0]            (fp32 `mul`)
 *   zp[m,n]    = zp_a*colsum_b[n] + zp_b*rowsum_a[m] - K*zp_a*zp_b
 *                (what the three extra quant_dots of :250-279 add up to)
 *   out        = float((double(acc) - double(zp)) * double(scale))
 *                (op/dequantizelinear.hpp:71-78)
 *   then `convert` to half / bf16 (op/convert.hpp:64-87: round toward zero,
 *   saturating, NaN kept) when out_type asks for it.
 * colsum_b [batch? no: N] / rowsum_a [M] are int32 sums over K of B's columns /
 * A's rows (see mi355_colsum_i8 / mi355_rowsum_i8); they are read only when
 * the matching zero point is non-zero and may be NULL otherwise.
 */
int mi355_quant_dot(const mi355_quant_dot_desc* desc,
                    const void* a,
                    const void* b,
                    void* c,
                    const float* scale_a,
                    const float* scale_b,
                    const int32_t* colsum_b,
                    const int32_t* rowsum_a,
                    void* stream);

/* The same with the bias `add` that follows the dequantizelinear of a linear layer
 * (op::add, src/include/migraphx/op/binary.hpp:60-90, of a [N] vector broadcast over the rows):
 *   out = float(dequantized) + bias[n]      one more fp32 rounding, never a fused multiply-add,
 * applied before the `convert` to a 16-bit type.  bias is [N] fp32 (batches share it); NULL gives
 * mi355_quant_dot.  Requires desc->dequant. */
int mi355_quant_dot_bias(const mi355_quant_dot_desc* desc,
                         const void* a,
                         const void* b,
                         void* c,
                         const float* scale_a,
                         const float* scale_b,
                         const int32_t* colsum_b,
                         const int32_t* rowsum_a,
                         const float* bias,
                         void* stream);

/*
 * quant_convolution (+ fused dequantizelinear) of an [N, C, H, W] tensor with [O, C/group, KH, KW]
 * weights, both dense; the result is dense [N, O, OH, OW].
 *
 * Replaces: op::quant_convolution::compute (src/include/migraphx/op/quant_convolution.hpp:142-157)
 * -> convolution (src/include/migraphx/convolution.hpp:37-100) with the shape rule of
 * quant_convolution.hpp:85-134: cross-correlation, `pad` zeros on the low side and `pad_hi` on
 * the high side of each spatial dimension (the reference's 2 * kdims padding form; equal values
 * give its kdims form), window positions stepping by the dilation; int8 x int8 -> int32 (exact), fp8 e4m3fn -> float.  A one-dimensional
 * convolution is passed with h = kh = 1.
 * With desc->dequant it also replaces what simplify_qdq.cpp:171-222 puts behind it for symmetric
 * zero points:  out = float(double(acc) * double(scale_x[0] * scale_w[o or 0]))  [-> half / bf16].
 * scale_w_mode = MI355_QP_PER_ROW means one scale per output channel ([O]).
 * workspace: device memory of at least the size mi355_quant_convolution_dims reports, 16-byte
 * aligned; it holds the window matrix and is free again when the call's work has finished.
 */
typedef struct mi355_quant_conv_desc {
    int64_t n, c, h, w;     /* input  [N, C, H, W] */
    int64_t o, kh, kw;      /* weights [O, C / group, KH, KW] */
    int64_t pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;   /* pad: zeros on the low side */
    int64_t group;
    int64_t pad_h_hi, pad_w_hi; /* zeros on the high side (enter the output size only) */
    int32_t in_type;        /* MI355_I8 or MI355_FP8 */
    int32_t out_type;       /* bare: MI355_I32 / MI355_F32; dequant: MI355_F32 / F16 / BF16 */
    int32_t dequant;
    int32_t scale_x_mode;   /* MI355_QP_NONE / PER_TENSOR */
    int32_t scale_w_mode;   /* MI355_QP_NONE / PER_TENSOR / PER_ROW (= per output channel) */
} mi355_quant_conv_desc;
int mi355_quant_convolution_dims(const mi355_quant_conv_desc* desc, int64_t* oh, int64_t* ow,
                                 size_t* workspace_bytes);
int mi355_quant_convolution(const mi355_quant_conv_desc* desc, const void* x, const void* w, void* out,
                            const float* scale_x, const float* scale_w, void* workspace,
                            size_t workspace_bytes, void* stream);

/* The same over three spatial axes: input [N, C, D, H, W], weights [O, C / group, KD, KH, KW],
 * output [N, O, OD, OH, OW]  (ref: convolution.hpp:37-100 loops over any number of spatial axes;
 * op/quant_convolution.hpp:52-157 accepts one to three).  pad / pad_hi / stride / dil hold one
 * value per spatial axis in the order depth, height, width.  The two-dimensional entry points are
 * this one with a depth of one. */
typedef struct mi355_quant_conv3d_desc {
    int64_t n, c, d, h, w;
    int64_t o, kd, kh, kw;
    int64_t pad[3], pad_hi[3], stride[3], dil[3];
    int64_t group;
    int32_t in_type, out_type, dequant, scale_x_mode, scale_w_mode;   /* as in mi355_quant_conv_desc */
} mi355_quant_conv3d_desc;
/* out_lens: OD, OH, OW */
int mi355_quant_convolution3d_dims(const mi355_quant_conv3d_desc* desc, int64_t* out_lens,
                                   size_t* workspace_bytes);
int mi355_quant_convolution3d(const mi355_quant_conv3d_desc* desc, const void* x, const void* w, void* out,
                              const float* scale_x, const float* scale_w, void* workspace,
                              size_t workspace_bytes, void* stream);

/* Float convolution of the same description (in_type = MI355_F32; out_type, dequant and the scale
 * modes are not read): op::convolution::compute (src/include/migraphx/op/convolution.hpp:208-239)
 * as the reference evaluates it -- float products added into a double over (channel, kd, kh, kw),
 * one rounding at the end -- bit for bit.  A correctness path (one thread per output) for what the
 * integer front ends leave of layers with uint8 tensors (QLinearConv) and for unquantized models. */
int mi355_convolution_f32(const mi355_quant_conv3d_desc* desc, const float* x, const float* w, float* out,
                          void* stream);

/* The same with a workspace.  A quant_dot that launches fewer workgroups than the chip has CUs
 * (a skinny or mid-size A against a large B, one image of a convolution) is split along K.
 * Without a workspace only the bare int8 product is split (the shares are added into C with
 * integer atomics); with one, the shares write partial tiles and a second kernel adds them up and
 * applies the dequantizing epilogue (no atomics, no clearing of C).  int8: the same bits as the
 * unsplit kernel, any N when B is [N, K].  fp8 (one batch, N % 4 == 0): float partial sums added
 * in a fixed order, the same bits on every call, within the fp8 tolerance of the unsplit
 * kernel's.  mi355_quant_dot_workspace_size gives the bytes that description can use (0: none);
 * a NULL or smaller workspace is not an error, the call then behaves like mi355_quant_dot_bias.
 * The workspace must be 16-byte aligned device memory and is free again when the call's work is
 * done. */
size_t mi355_quant_dot_workspace_size(const mi355_quant_dot_desc* desc);
int mi355_quant_dot_ws(const mi355_quant_dot_desc* desc, const void* a, const void* b, void* c,
                       const float* scale_a, const float* scale_b, const int32_t* colsum_b,
                       const int32_t* rowsum_a, const float* bias, void* workspace,
                       size_t workspace_bytes, void* stream);

/* quant_dot for callers that cannot allocate.  No counterpart in the reference: it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc, which can
 * neither allocate the workspace of mi355_quant_dot_ws nor keep one around.  Same arguments and
 * result as mi355_quant_dot_ws; the split-K partial sums go to a buffer of
 * MI355_QUANT_DOT_STATIC_SCRATCH_BYTES that is part of the library's device code (one copy per
 * GPU, held from module load until the process ends).  The call itself allocates and frees
 * nothing; the first call on a device looks the buffer's address up once.  A description whose
 * mi355_quant_dot_workspace_size exceeds the buffer is refused with MI355_ERR_SCRATCH_TOO_SMALL
 * (nothing is launched).  All calls on one GPU share the buffer: calls that may run at the same
 * time on one GPU (different streams, different threads) race on it and must be ordered by the
 * caller.  The buffer keeps the last call's partial sums; no call depends on its contents. */
#define MI355_QUANT_DOT_STATIC_SCRATCH_BYTES (32u << 20)
int mi355_quant_dot_static(const mi355_quant_dot_desc* desc, const void* a, const void* b, void* c,
                           const float* scale_a, const float* scale_b, const int32_t* colsum_b,
                           const int32_t* rowsum_a, const float* bias, void* stream);

/*
 * quant_dot with element-wise scales, the MX block formats' form:
 *   C[b, m, n] = float( sum_k double(float(A[b,m,k]) * SA[b,m,k]) * double(float(B[b,k,n]) * SB[b,k,n]) )
 *
 * Replaces: ref_quant_gemm::compute with four inputs (src/targets/ref/lowering.cpp:221-242:
 * float(a) * scale_a and float(b) * scale_b element by element in float, then gemm_naive,
 * src/gemm.cpp:42-63), which is what simplify_qdq.cpp:290-357 leaves of
 * unpack_fp4 -> dequantizelinear -> dot for block-quantized operands.
 *
 * A is [batch, M, K] and B is given as [batch, N, K] (K contiguous for both: the transpose view
 * the operator sees as [K, N]); each either one e4m3fn code per element (MI355_FP8) or two e2m1
 * codes per byte along K (MI355_FP4X2, what unpack_fp4 reads); lda / ldb / stride_a / stride_b count
 * BYTES of the stored operand.  C is float, row-major.  The scales are float tensors addressed as
 *   SA(b, m, k) = scale_a[b * sa_batch + m * sa_row + (k / 32) * sa_block + (k % 32) * sa_elem]
 * (element strides), so the operator's full-size scale tensor is (M*K, K, 32, 1) and a compact
 * [M, K/32] tensor of block scales is (M*K/32, K/32, 1, 0); likewise SB(b, n, k).
 * Where every block of 32 scales along K is one positive normal power of two (what the MX formats
 * store as e8m0) the product runs on v_mfma_scale_f32_16x16x128_f8f6f4 with the scales as the
 * instruction's block-scale operands; any other scale values are detected on the device and the
 * call then evaluates the formula above as written (slowly).  K must be a multiple of 32, rows
 * 16-byte aligned.  workspace: mi355_quant_dot_mx_workspace_size bytes of device memory, 16-byte
 * aligned, free again when the call's work is done.
 */
typedef struct mi355_mx_dot_desc {
    int64_t m, n, k, batch;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    int64_t sa_batch, sa_row, sa_block, sa_elem;
    int64_t sb_batch, sb_row, sb_block, sb_elem;
    int32_t a_type, b_type; /* MI355_FP8 or MI355_FP4X2 */
} mi355_mx_dot_desc;
size_t mi355_quant_dot_mx_workspace_size(const mi355_mx_dot_desc* desc);
int mi355_quant_dot_mx(const mi355_mx_dot_desc* desc, const void* a, const void* b, float* c,
                       const float* scale_a, const float* scale_b, void* workspace,
                       size_t workspace_bytes, void* stream);

/* int32 column sums of an int8 [K, N] matrix (same addressing as B above,
 * batch 1): out[n] = sum_k B[k, n].  Equals quant_dot(ones[1,K], B), the
 * zero-point term of simplify_qdq.cpp:260-266 divided by the zero point. */
int mi355_colsum_i8(const void* b, int64_t k, int64_t n, int64_t ldb, int32_t trans_b,
                    int32_t* out, void* stream);

/* int32 row sums of an int8 [M, K] matrix: out[m] = sum_k A[m, k]
 * (simplify_qdq.cpp:267-273). */
int mi355_rowsum_i8(const void* a, int64_t m, int64_t k, int64_t lda, int32_t trans_a,
                    int32_t* out, void* stream);

/*
 * quantizelinear on a dense [rows, cols] tensor.
 *
 * Replaces: op::quantizelinear::compute
 * (src/include/migraphx/op/quantizelinear.hpp:71-108).
 *   integral out: clamp(double(nearbyint(x / s)) + double(zp)), x / s divided
 *                 in x's own type, ties to even;
 *   fp8 out:      clamp(double(x)/double(s) + double(zp), -448, 448) -> fp8 e4m3fn;
 *                 the same with +-57344 for MI355_BF8 (fp8 e5m2).
 * scale has x's element type, zp (may be NULL = 0) has the output's.  Both are
 * addressed as p[r*stride_r + c*stride_c] so a per-tensor parameter uses
 * strides (0,0), a per-column one (0,1), a per-row one (1,0), a full one
 * (cols,1) -- the strides the broadcast views of the graph carry.
 */
int mi355_quantizelinear(const void* x, int32_t x_type,
                         const void* scale, int64_t scale_stride_r, int64_t scale_stride_c,
                         const void* zp, int64_t zp_stride_r, int64_t zp_stride_c,
                         void* out, int32_t out_type,
                         int64_t rows, int64_t cols, void* stream);

/*
 * dequantizelinear on a dense [rows, cols] tensor.
 *
 * Replaces: op::dequantizelinear::compute
 * (src/include/migraphx/op/dequantizelinear.hpp:60-83):
 * out = (double(x) - double(zp)) * scale, stored in the scale's type.
 * x_type in {I8, U8, I32, F32, FP8}; scale_type in {F32, F16, BF16}.
 */
int mi355_dequantizelinear(const void* x, int32_t x_type,
                           const void* scale, int32_t scale_type,
                           int64_t scale_stride_r, int64_t scale_stride_c,
                           const void* zp, int64_t zp_stride_r, int64_t zp_stride_c,
                           void* out, int64_t rows, int64_t cols, void* stream);

/*
 * unpack_int4 / pack_int4 along the last axis of a dense [rows, cols] byte
 * tensor (cols = packed length for unpack, unpacked length for pack).
 *
 * Replaces: op::unpack_int4::compute (src/include/migraphx/op/unpack_int4.hpp:75-121)
 * and op::pack_int4::compute (src/include/migraphx/op/pack_int4.hpp:79-124).
 * Low nibble = even element; is_signed selects sign extension / [-8,7] clip.
 */
int mi355_unpack_int4(const void* in, void* out, int32_t is_signed,
                      int64_t rows, int64_t cols, void* stream);
int mi355_pack_int4(const void* in, void* out, int32_t is_signed,
                    int64_t rows, int64_t cols, void* stream);

/*
 * The same along any axis of a strided view: `lens` (HOST array, ndim <= MI355_MAX_DIMS entries)
 * are the lengths of the INPUT, `in_strides` its element strides (zero = a broadcast dimension,
 * as multibroadcast views carry), `axis` the packed axis (negative counts from the end).  The
 * output is dense row-major with lens[axis] doubled (unpack) or halved (pack).
 *
 * Replaces the same two operators for every axis and for the non-standard input shapes they
 * accept (op/unpack_int4.hpp:54-73 normalises the axis, :75-121 walks the multi-index with
 * idx[axis] * 2 and idx[axis] * 2 + 1; op/pack_int4.hpp:79-124 likewise).
 */
int mi355_unpack_int4_nd(const void* in, void* out, int32_t is_signed, int32_t ndim,
                         const int64_t* lens, const int64_t* in_strides, int32_t axis, void* stream);
int mi355_pack_int4_nd(const void* in, void* out, int32_t is_signed, int32_t ndim,
                       const int64_t* lens, const int64_t* in_strides, int32_t axis, void* stream);

/*
 * unpack_fp4 / pack_fp4 along the last axis of a dense [rows, cols] tensor (cols = packed length
 * for unpack, unpacked length for pack).  fp4 is e2m1 (magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6), two
 * codes per byte, low nibble = even element.
 *
 * Replaces: op::unpack_fp4::compute (src/include/migraphx/op/unpack_fp4.hpp:78-101), which writes
 * fp8 e4m3fn, and op::pack_fp4::compute (src/include/migraphx/op/pack_fp4.hpp:82-106) with
 * cast_to_fp4 of src/include/migraphx/fp4_casts.hpp:80-100 (nearest, ties to the even code,
 * saturating at 6, NaN -> 0) for float input.
 */
int mi355_unpack_fp4(const void* in, void* out, int64_t rows, int64_t cols, void* stream);
int mi355_pack_fp4(const float* in, void* out, int64_t rows, int64_t cols, void* stream);

/*
 * convert float -> half / bf16 / fp8 and back on n dense elements; also to int8 / uint8 / int32
 * (NaN -> 0, saturating, truncating toward zero: the integral branch of op/convert.hpp:64-87).
 *
 * Replaces: op::convert::compute (src/include/migraphx/op/convert.hpp:64-87)
 * with the software-float conversions of generic_float.hpp:172-222 (half and
 * bf16: round toward zero) and float8_impl.hpp:38-247 (fp8 e4m3fn and e5m2: nearest even,
 * clipping; NaN becomes numeric_limits::quiet_NaN of the type, 0x7f and 0xff).
 */
int mi355_convert(const void* in, int32_t in_type, void* out, int32_t out_type,
                  int64_t n, void* stream);

/* Zero-point forms of the int4 weight-only GEMM. */
typedef enum mi355_w4_zp_mode {
    MI355_W4_ZP_SCALAR = 0, /* one value for the whole tensor (MatMulNBits default 8) */
    MI355_W4_ZP_GROUP  = 1, /* uint8 [N, K/group], already unpacked */
    MI355_W4_ZP_PACKED = 2  /* 4-bit pairs, uint8 [N, ceil(K/group/2)], low nibble first */
} mi355_w4_zp_mode;

/*
 * int4 weight-only GEMM / GEMV with group-wise scales:
 *   out[m, n] = half( sum_k a[m,k] * w[n,k] ),  w[n,k] = half((q[n,k] - zp) * scale[n, k/group])
 *
 * Replaces the chain the ref target runs op by op for the graph of
 * src/onnx/parse_matmulnbits.cpp:85-159:
 *   unpack_int4 (op/unpack_int4.hpp:75-121) ->
 *   dequantizelinear with block-broadcast scales / zero points
 *     (op/dequantizelinear.hpp:60-83, op/builder/.../quantize_dequantize_linear.hpp:84-152) ->
 *   transpose -> dot (op/dot.hpp:102-107, gemm_naive src/gemm.cpp:42-63).
 * a      fp16 [M, K] (lda), w_packed uint8 [N, K/2] (two nibbles per byte along K,
 * low nibble = even k), scales fp16 [N, K/group], out fp16 [M, N] (ldc).
 * K must be a multiple of `group`, group a multiple of 32.
 */
int mi355_w4a16_gemm(const void* a, int64_t lda,
                     const void* w_packed,
                     const void* scales,
                     const void* zp, int32_t zp_mode, int32_t zp_scalar,
                     void* out, int64_t ldc,
                     int64_t m, int64_t n, int64_t k, int64_t group,
                     void* stream);

/* The same with a workspace.  Where the column tiles alone do not fill the chip (more than 32
 * rows against N / 128 tiles; 2..64 rows against few 64-column tiles and K >= 8192) the kernels
 * split K over more workgroups when they have room for the float partial sums; a second kernel
 * adds them in a fixed order and converts to half.  Deterministic, within the path's fp tolerance
 * of the unsplit result (another order of fp32 additions).  mi355_w4a16_gemm_workspace_size gives
 * the bytes the shape can use (0: none); a NULL or smaller workspace is not an error.  16-byte
 * aligned device memory, free again when the call's work is done. */
size_t mi355_w4a16_gemm_workspace_size(int64_t m, int64_t n, int64_t k, int64_t group);
int mi355_w4a16_gemm_ws(const void* a, int64_t lda,
                        const void* w_packed,
                        const void* scales,
                        const void* zp, int32_t zp_mode, int32_t zp_scalar,
                        void* out, int64_t ldc,
                        int64_t m, int64_t n, int64_t k, int64_t group,
                        void* workspace, size_t workspace_bytes,
                        void* stream);

/*
 * The same product for constant weights, reordered once ahead of time (a target does this when it
 * compiles the program: the packed weights and scales of a weight-only layer are literals).
 * mi355_w4a16_prepack writes, from the operator's own tensors (w_packed uint8 [N, K/2], scales fp16
 * [N, K/128], one zero point for the tensor), a device buffer of mi355_w4a16_prepacked_size bytes
 * that holds the same nibbles and scales -- 256 bytes more than the two tensors -- in the order
 * the kernel's lanes read them; mi355_w4a16_gemm_prepacked then computes out = half(sum_k a * w)
 * with w = half((q - zp) * scale) exactly as mi355_w4a16_gemm does (same reference chain:
 * src/onnx/parse_matmulnbits.cpp:85-159, op/unpack_int4.hpp:75-121, op/dequantizelinear.hpp:60-83,
 * op/dot.hpp:102-107), within the same tolerance of the fp32 sum.
 * Shapes: group 128, N % 16 == 0, K % 512 == 0, K <= 28672, M <= mi355_w4a16_prepacked_max_rows (1 for
 * any K; up to 16 while the rows fit the LDS: 16 at K <= 4096, 8 at K <= 8192, 4 at K <= 16384; rows
 * of a 16-byte aligned with lda % 8 == 0); other M: MI355_ERR_UNSUPPORTED, the caller keeps
 * mi355_w4a16_gemm for them.  Row r of a several-row call carries the bits of the one-row call on row r.  mi355_w4a16_prepacked_size returns 0 for a shape
 * the reordered form does not take.  Any scale values are accepted; the fastest form needs
 * 2^-10 <= scale < 2^-4 and a zero point of 0, 1, 2, 4 or 8, which the reordering checks on the
 * device and records in the buffer.
 */
size_t mi355_w4a16_prepacked_size(int64_t n, int64_t k, int64_t group);
int64_t mi355_w4a16_prepacked_max_rows(int64_t n, int64_t k, int64_t group);
int mi355_w4a16_prepack(const void* w_packed, const void* scales, int32_t zp_scalar,
                        int64_t n, int64_t k, int64_t group,
                        void* prepacked, void* stream);
int mi355_w4a16_gemm_prepacked(const void* a, int64_t lda,
                               const void* prepacked,
                               void* out, int64_t ldc,
                               int64_t m, int64_t n, int64_t k,
                               void* stream);

/*
 * quant_dot (+ fused dequantizelinear) of a few rows against a constant B reordered once ahead of
 * time (a target does this when it compiles the program: the weights of a linear layer are
 * literals).  mi355_quant_dot_prepack writes B -- addressed as b[k * stride_k + n * stride_n], so
 * [K, N] and [N, K] sources need no copy -- into a device buffer of mi355_quant_dot_prepacked_size
 * bytes (the size of B) as the 16-column x 64-k operand tiles of the matrix-core instruction;
 * mi355_quant_dot_prepacked then computes what mi355_quant_dot_bias computes for the same
 * descriptor (same reference chain: src/targets/ref/lowering.cpp:218-248 -> src/gemm.cpp:42-63,
 * the epilogue of simplify_qdq.cpp:225-289) in one launch without a workspace: bit-identical for
 * int8, within the fp8 tolerance for fp8 (its own fixed summation order).  desc->trans_b, ldb and
 * stride_b are not read.
 * Shapes: M <= 16, N % 16 == 0, K % 64 == 0, one batch, A row-major with lda % 16 == 0 and a
 * 16-byte aligned base (otherwise MI355_ERR_UNSUPPORTED: the caller keeps mi355_quant_dot_bias).
 * mi355_quant_dot_prepacked_size returns 0 for an N, K or element type the reordered form does
 * not take.
 */
size_t mi355_quant_dot_prepacked_size(int32_t in_type, int64_t n, int64_t k);
int mi355_quant_dot_prepack(const void* b, int32_t in_type, int64_t n, int64_t k,
                            int64_t stride_k, int64_t stride_n,
                            void* prepacked, void* stream);
int mi355_quant_dot_prepacked(const mi355_quant_dot_desc* desc,
                              const void* a, const void* b_prepacked, void* c,
                              const float* scale_a, const float* scale_b,
                              const int32_t* colsum_b, const int32_t* rowsum_a,
                              const float* bias,
                              void* stream);

/*
 * Float dot: C[b, m, n] = T( sum_k double(A[b, m, k]) * double(B[b, k, n]) ), k ascending,
 * T in {F32, F16, BF16} for all three tensors (16-bit results truncate, as the software
 * floats do).
 *
 * Replaces: op::dot::compute (src/include/migraphx/op/dot.hpp:102-107) -> gemm_naive
 * (src/gemm.cpp:42-63).  Bit-exact with it; meant for calibration runs of the unquantized
 * graph and for the dot behind a dequantizelinear that the int4 kernel does not cover, not
 * for throughput.  A and B are addressed by element strides, so transposed and broadcast views
 * need no copy; C is row-major with leading dimension ldc.
 */
int mi355_dot(const void* a, const void* b, void* c, int32_t type,
              int64_t m, int64_t n, int64_t k,
              int64_t a_stride_m, int64_t a_stride_k, int64_t b_stride_k, int64_t b_stride_n,
              int64_t ldc, int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
              void* stream);

/* The same followed by the `mul` with one float that scales attention scores
 * (op::mul, src/include/migraphx/op/binary.hpp:60-90, of a broadcast scalar): fp32 only,
 *   C = float(sum) * scale[0]       the sum is rounded to float first, then multiplied in fp32,
 * which is what the two operators give one after the other.  scale is a DEVICE pointer; NULL gives
 * mi355_dot. */
int mi355_dot_scaled(const void* a, const void* b, void* c, int32_t type,
                     int64_t m, int64_t n, int64_t k,
                     int64_t a_stride_m, int64_t a_stride_k, int64_t b_stride_k, int64_t b_stride_n,
                     int64_t ldc, int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                     const float* scale, void* stream);

/* The same arguments (fp32 only), with the sums on the fp32 matrix cores: fp32 products and fp32
 * accumulation at twice the rate of mi355_dot_scaled.  The result is no longer the bits of the
 * reference's double sum; it stays within K * 2^-24 of sum|a||b| of it, far inside the 1e-3
 * relative the float outputs of the path are held to.  Meant for the attention products of an
 * encoder when the caller asks for speed (the mi355 target lowers `dot` to it when the environment
 * variable MIGRAPHX_MI355_FP32_DOT is set at compile time); op::dot::compute
 * (src/include/migraphx/op/dot.hpp:102-107) is the operator it stands in for. */
int mi355_dot_fp32acc(const void* a, const void* b, void* c, int32_t type,
                      int64_t m, int64_t n, int64_t k,
                      int64_t a_stride_m, int64_t a_stride_k, int64_t b_stride_k, int64_t b_stride_n,
                      int64_t ldc, int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                      const float* scale, void* stream);

/* mi355_dot_scaled (fp32acc == 0) or mi355_dot_fp32acc over TWO batch axes, each operand with a
 * stride of its own per axis: batch entry (o, i) of A starts at o * stride_a_outer + i *
 * stride_a_inner.  C is dense, [batch_outer, batch_inner, m, n].  This is how the target multiplies
 * [batch, heads, rows, k] views whose batch axes do not collapse into one stride -- the head split
 * of an attention layer, transpose(0, 2, 1, 3) of [batch, rows, heads, k] -- without copying them
 * (op::dot::compute_shape, src/include/migraphx/op/dot.hpp:43-99, takes any such view). */
int mi355_dot_batch2(const void* a, const void* b, void* c, int32_t type,
                     int64_t m, int64_t n, int64_t k,
                     int64_t a_stride_m, int64_t a_stride_k, int64_t b_stride_k, int64_t b_stride_n,
                     int64_t batch_outer, int64_t batch_inner,
                     int64_t stride_a_outer, int64_t stride_a_inner,
                     int64_t stride_b_outer, int64_t stride_b_inner,
                     const float* scale, int32_t fp32acc, void* stream);
/* The same with C as a strided set of row-major blocks: output (o, i, row, col) lies at
 * c + o * stride_c_outer + i * stride_c_inner + row * ldc + col (blocks that do not overlap).  This is how
 * the target writes the context of an attention layer, dot(probabilities, values) over [batch, heads],
 * straight into the [batch, rows, heads, width] layout the transpose(0, 2, 1, 3) + contiguous behind it
 * would produce (stride_c_inner = width, ldc = heads * width): the copy is not made
 * (src/eliminate_contiguous.cpp removes such copies where the reference's kernels take the view). */
int mi355_dot_batch2_strided(const void* a, const void* b, void* c, int32_t type,
                             int64_t m, int64_t n, int64_t k,
                             int64_t a_stride_m, int64_t a_stride_k, int64_t b_stride_k, int64_t b_stride_n,
                             int64_t ldc, int64_t batch_outer, int64_t batch_inner,
                             int64_t stride_a_outer, int64_t stride_a_inner,
                             int64_t stride_b_outer, int64_t stride_b_inner,
                             int64_t stride_c_outer, int64_t stride_c_inner,
                             const float* scale, int32_t fp32acc, void* stream);

/*
 * contiguous: gather a strided view (ndim <= MI355_MAX_DIMS, element strides, zero = broadcast)
 * into a dense row-major tensor.  lens / strides are HOST arrays.
 *
 * Replaces: op::contiguous::compute (src/include/migraphx/op/contiguous.hpp:43-83).
 */
#define MI355_MAX_DIMS 8
int mi355_contiguous(const void* in, void* out, int32_t elem_size, int32_t ndim,
                     const int64_t* lens, const int64_t* strides, void* stream);

/*
 * Float operators of the graph around the quantized GEMMs (an encoder layer's bias and residual
 * adds, layer normalisation built from reduce_mean / sub / mul / rsqrt, GELU through erf, attention
 * softmax, embedding lookup).  float32 only; not tuned.
 *
 * mi355_binary_f32   op::add / sub / mul / div (src/include/migraphx/op/binary.hpp:60-90): out is a
 *                    dense row-major tensor of `lens`; a and b are addressed through element strides
 *                    (zero = broadcast), HOST arrays of ndim entries.
 * mi355_unary_f32    op::erf / sqrt / rsqrt (1 / sqrt(x)) / exp / tanh / neg on n dense elements
 *                    (op/unary.hpp; erf.hpp, rsqrt.hpp, ...).  erf, exp and tanh use the device math
 *                    library and may differ from the host's by a few units in the last place.
 * mi355_reduce_mean_f32  op::reduce_mean over the last axis of [rows, cols] (op/reduce_mean.hpp:34-50,
 *                    reduce_op.hpp:186-202): sum in double, divided by cols, rounded to float.
 * mi355_softmax_f32  softmax over the last axis (ref_softmax, src/targets/ref/lowering.cpp:281-312):
 *                    e = float(exp(double(x) - max)), out = float(double(e) / sum_double(e)).
 * mi355_gather_rows  op::gather along axis 0 of a [table_rows, row_bytes] table with int32 or int64
 *                    indices (op/gather.hpp:100-118); row_bytes must be a multiple of 4.
 */
typedef enum mi355_binary_op {
    MI355_BIN_ADD = 0, MI355_BIN_SUB = 1, MI355_BIN_MUL = 2, MI355_BIN_DIV = 3,
    MI355_BIN_MAX = 4, MI355_BIN_MIN = 5 /* std::max / std::min (op/max.hpp, min.hpp): mi355_binary_f32 only */
} mi355_binary_op;
typedef enum mi355_unary_op {
    MI355_UN_ERF = 0, MI355_UN_SQRT = 1, MI355_UN_RSQRT = 2, MI355_UN_EXP = 3, MI355_UN_TANH = 4, MI355_UN_NEG = 5,
    MI355_UN_NEARBYINT = 6 /* op/nearbyint.hpp: ties to even */
} mi355_unary_op;
int mi355_binary_f32(int32_t op, const float* a, const int64_t* a_strides, const float* b,
                     const int64_t* b_strides, float* out, int32_t ndim, const int64_t* lens,
                     void* stream);
/* The same operators on the narrow types the integer-MatMul front end leaves in a graph
 * (src/op/builder/bias_uint8.cpp:49-100: uint8 data moved to int8 through half, zero points
 * subtracted in int8): MI355_I8 / MI355_U8 (add / sub / mul; operands promote to int, the result
 * converts back, wrapping) and MI355_F16 / MI355_BF16 (the operator on floats, the result converted
 * back toward zero: generic_float.hpp:303-326).  Addressing as mi355_binary_f32. */
int mi355_binary_typed(int32_t op, int32_t type, const void* a, const int64_t* a_strides, const void* b,
                       const int64_t* b_strides, void* out, int32_t ndim, const int64_t* lens,
                       void* stream);
/* add / sub / mul of int32 tensors (wrapping), same addressing as mi355_binary_f32: the
 * zero-point terms of src/simplify_qdq.cpp:196-222 and :250-279 when they stay in the graph. */
int mi355_binary_i32(int32_t op, const int32_t* a, const int64_t* a_strides, const int32_t* b,
                     const int64_t* b_strides, int32_t* out, int32_t ndim, const int64_t* lens,
                     void* stream);
int mi355_unary_f32(int32_t op, const float* in, float* out, int64_t n, void* stream);
/* reduce_max (op 0) / reduce_min (op 1) over all n elements into out[0] (op/reduce_max.hpp,
 * reduce_min.hpp with every axis reduced: the range DynamicQuantizeLinear needs); one workgroup. */
int mi355_reduce_all_f32(int32_t op, const float* in, float* out, int64_t n, void* stream);
int mi355_reduce_mean_f32(const float* in, float* out, int64_t rows, int64_t cols, void* stream);
int mi355_softmax_f32(const float* in, float* out, int64_t rows, int64_t cols, void* stream);
int mi355_gather_rows(const void* table, const void* ids, int32_t ids_are_int64, void* out,
                      int64_t n_ids, int64_t table_rows, int64_t row_bytes, void* stream);

/* A chain of the float operators above applied element by element in one pass over a dense
 * [rows, cols] result, so that the intermediate tensors of e.g. GELU (mul, erf, add, mul, mul) or
 * bias + residual never reach memory.  It is the device counterpart of one fused pointwise module
 * (src/fuse_pointwise.cpp:364-385 builds them for the reference's targets, which then compile each module;
 * here nothing is compiled at run time).  Each element runs a small register machine with the running
 * value and one saved value; every step is the same IEEE float operation the single operators
 * perform, in the order the steps list them, so the result equals the unfused sequence bit for bit.
 *   MI355_CH_LOAD    value = input[src]
 *   MI355_CH_BINARY  value = value (op) operand, or operand (op) value when `reversed`;
 *                    operand = input[src] for src >= 0, the saved value for MI355_CH_SAVED,
 *                    the running value itself for MI355_CH_SELF
 *   MI355_CH_UNARY   value = op(value)
 *   MI355_CH_SAVE    saved = value
 * Input i is addressed as inputs[i][row * row_strides[i] + col * col_strides[i]] with a column
 * stride of 0 (constant along the row) or 1.  The first step must be a LOAD.  All arrays are HOST
 * arrays; at most MI355_CHAIN_MAX_STEPS steps and MI355_CHAIN_MAX_INPUTS inputs. */
typedef enum mi355_chain_kind
{
    MI355_CH_LOAD     = 0,
    MI355_CH_BINARY   = 1,
    MI355_CH_UNARY    = 2,
    MI355_CH_SAVE     = 3,
    MI355_CH_ROW_MEAN = 4 /* mi355_chain_rows_f32 only */
} mi355_chain_kind;
#define MI355_CH_SAVED (-1)
#define MI355_CH_SELF (-2)
#define MI355_CHAIN_MAX_STEPS 24
#define MI355_CHAIN_MAX_INPUTS 8
#define MI355_CHAIN_ROWS_MAX_COLS 4096
typedef struct mi355_chain_step
{
    int32_t kind;     /* mi355_chain_kind */
    int32_t op;       /* mi355_binary_op or mi355_unary_op; unused for LOAD and SAVE */
    int32_t src;      /* LOAD: input index; BINARY: input index, MI355_CH_SAVED or MI355_CH_SELF */
    int32_t reversed; /* BINARY only */
} mi355_chain_step;
int mi355_chain_f32(const mi355_chain_step* steps, int32_t n_steps, const float* const* inputs,
                    const int64_t* row_strides, const int32_t* col_strides, int32_t n_inputs,
                    float* out, int64_t rows, int64_t cols, void* stream);
/* The chain with one more kind of step, for operators that reduce over the last axis between the
 * pointwise ones (layer normalisation: reduce_mean, sub, mul, reduce_mean, add, rsqrt, mul, mul, add):
 *   MI355_CH_ROW_MEAN  value = the mean of the running value over its row, in every column
 * which is reduce_mean over the last axis (src/include/migraphx/op/reduce_mean.hpp:34-50) followed by
 * the broadcast back to the row, with mi355_reduce_mean_f32's summation (double, one rounding to
 * float), so the result equals the separate operators bit for bit.  A wave holds a whole row in
 * registers: cols <= MI355_CHAIN_ROWS_MAX_COLS, else MI355_ERR_UNSUPPORTED.  The reference reaches the
 * same fusion through src/fuse_reduce.cpp:251-340, 448-470 and compiles the fused module. */
int mi355_chain_rows_f32(const mi355_chain_step* steps, int32_t n_steps, const float* const* inputs,
                         const int64_t* row_strides, const int32_t* col_strides, int32_t n_inputs,
                         float* out, int64_t rows, int64_t cols, void* stream);
/* The same chain with quantizelinear (src/include/migraphx/op/quantizelinear.hpp:71-108) as its last
 * operation: the chain's final value leaves as int8, nearbyint(value / scale[0]) + zero_point[0]
 * saturated to [-128, 127], one scale and one zero point (NULL: 0) for the whole tensor, both DEVICE
 * pointers; the float value itself is not stored.  What the target makes of a float pointwise chain
 * whose only reader is a per-tensor quantizelinear (the activations in front of a quantized layer). */
int mi355_chain_f32_q8(const mi355_chain_step* steps, int32_t n_steps, const float* const* inputs,
                       const int64_t* row_strides, const int32_t* col_strides, int32_t n_inputs,
                       const float* scale, const int8_t* zero_point, int8_t* out, int64_t rows,
                       int64_t cols, void* stream);

/* Human-readable text for a status code (static storage). */
const char* mi355_status_string(int status);

/* Library version, major*10000 + minor*100 + patch. */
int mi355_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_QGEMM_H */
