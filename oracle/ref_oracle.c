/*
 * ref_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C CPU restatement of the arithmetic that MIGraphX's `ref` target
 * performs on the quantized-GEMM path.  It exists only so that tests, the
 * smoke check and the benchmark's cpu_baseline leg have something to compare
 * the HIP kernels against.  Nothing in the shipped library links, loads or
 * calls this file.
 *
 * Every function names the reference source it follows (paths relative to
 * the reference tree).  How each function is pinned (which of the reference's
 * own known-answer vectors or which closed form checks it) is listed next to
 * it; the checks themselves live in tests/test_oracle_*.py.
 *
 *   function                      pinned by
 *   ---------------------------   -------------------------------------------
 *   orc_fp8e4m3fn_to_f32          256-entry table of test/fp8e4m3fn.cpp:34-105
 *   orc_fp8e4m3fn_from_f32        samples test/fp8e4m3fn.cpp:121-140 + brute
 *                                 force "nearest table entry, ties to even
 *                                 mantissa, saturate to 448" over random and
 *                                 adversarial floats
 *   orc_fp8e5m2_to_f32            256-entry table of test/fp8e5m2.cpp:34-292
 *   orc_fp8e5m2_from_f32          samples test/fp8e5m2.cpp:320-360 + the same
 *                                 brute force against the table, saturating
 *                                 to 57344
 *   orc_half_* / orc_bf16_*       tables test/half.cpp, test/bf16.cpp + closed
 *                                 form (mantissa shift == round toward zero,
 *                                 compared with numpy bit arithmetic)
 *   orc_quant_dot                 16 quant_dot cases test/ref/dot_op.cpp:1391-
 *                                 1865 + numpy int64 matmul + exact fixed point
 *                                 closed form for fp8
 *   orc_quantizelinear            test/ref/quantizelinear.cpp:33-168
 *   orc_dequantizelinear          test/ref/dequantizelinear.cpp:32-83
 *   orc_unpack_int4/orc_pack_int4 test/ref/unpack_int4.cpp, pack_int4.cpp,
 *                                 pack_unpack_int4.cpp
 *   orc_unpack_fp4/orc_pack_fp4   test/ref/pack_unpack_fp4.cpp:34-89 (three cases) +
 *                                 all 16 codes against the e2m1 definition
 *                                 (+-{0, .5, 1, 1.5, 2, 3, 4, 6}), nearest-even on
 *                                 every midpoint, saturation, NaN -> 0
 *   orc_dot                       test/onnx/verify/matmulnbits_tests.cpp golds
 *                                 (whole unpack -> dequantize -> dot chain)
 *   orc_convolution               test/ref/quant_convolution.cpp:33-133 (three int8
 *                                 cases: plain, padding, padding + stride);
 *                                 test/ref/convolution.cpp:674-701 (dilation) and
 *                                 :761-857 (groups) for the window indexing;
 *                                 brute force over every attribute against a
 *                                 padded-array numpy restatement
 *   orc_convert                   test/ref/convert.cpp + closed form
 *   orc_softmax_f32               test/ref/softmax.cpp:33-107 (two cases, 122
 *                                 expected values, axis inside the shape)
 *   orc_reduce_mean_f32           test/ref/reduce_mean.cpp:33-195 (axes {0,2},
 *                                 {1}, {1,2}, {2} of a 3x2x2 tensor)
 *   orc_gather                    test/ref/gather.cpp:59-214 (seven cases:
 *                                 axes 0 / 1 / -1, negative and scalar indices)
 *   orc_binary_f32, orc_unary_f32 one C operator / libm call each, which is
 *                                 also how the reference's tests form their
 *                                 expected values (test/ref/div.cpp:33-50,
 *                                 erf.cpp:33-49, rsqrt.cpp:33-46); checked
 *                                 against numpy / math.erf
 */
#include <fenv.h>
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* element type codes shared with oracle.py */
enum {
    ORC_I8   = 0,
    ORC_U8   = 1,
    ORC_I32  = 2,
    ORC_F32  = 3,
    ORC_F16  = 4,
    ORC_BF16 = 5,
    ORC_FP8  = 6, /* OCP e4m3fn */
    ORC_F64  = 7,
    ORC_BF8  = 8  /* OCP e5m2 */
};

static inline uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ------------------------------------------------------------------------
 * generic_float<M,E>::from_float / to_float
 * src/include/migraphx/generic_float.hpp:172-222 (from_float), :129-170
 * (to_float).  half = generic_float<10,5> (half.hpp:34), bf16 =
 * generic_float<7,8> (bf16.hpp:34).  The mantissa is shifted right, i.e. the
 * conversion rounds toward zero; exponent overflow gives infinity.
 * ---------------------------------------------------------------------- */
static uint32_t gf_from_f32(float x, int msize, int esize)
{
    uint32_t u        = f32_bits(x);
    uint32_t fsign    = u >> 31;
    uint32_t fexp     = (u >> 23) & 0xffu;
    uint32_t fman     = u & 0x7fffffu;
    uint32_t all_ones = (1u << esize) - 1u;
    int bias          = (1 << (esize - 1)) - 1;
    int diff          = 127 - bias;
    uint32_t e, m;
    if(fexp == 0)
    {
        e = 0;
        m = fman >> (23 - msize);
    }
    else if(fexp == 0xffu)
    {
        e = all_ones;
        m = fman >> (23 - msize);
    }
    else
    {
        int ee = (int)fexp - diff;
        if(ee >= (int)all_ones)
        {
            e = all_ones;
            m = 0;
        }
        else if(ee < 1)
        {
            int shift        = diff - (int)fexp;
            int shift_amount = shift + (23 - msize) + 1;
            e                = 0;
            if(shift_amount < 32)
                m = (fman | (1u << 23)) >> shift_amount;
            else
                m = 0;
        }
        else
        {
            e = (uint32_t)ee;
            m = fman >> (23 - msize);
        }
    }
    if(e > all_ones)
        e = all_ones;
    m &= (1u << msize) - 1u;
    return (fsign << (msize + esize)) | (e << msize) | m;
}

static float gf_to_f32(uint32_t bits, int msize, int esize)
{
    uint32_t all_ones = (1u << esize) - 1u;
    uint32_t sign     = (bits >> (msize + esize)) & 1u;
    uint32_t e        = (bits >> msize) & all_ones;
    uint32_t m        = bits & ((1u << msize) - 1u);
    int bias          = (1 << (esize - 1)) - 1;
    uint32_t fe, fm;
    if(e == 0 && esize != 8)
    {
        if(m == 0)
        {
            fe = 0;
            fm = 0;
        }
        else
        {
            /* normalise the subnormal: shift so the leading one is dropped */
            int top = 31 - __builtin_clz(m); /* index of leading one */
            int shift = msize - (top + 1);
            fm        = (m << (shift + 1)) & ((1u << msize) - 1u);
            fe        = (uint32_t)(127 - bias - shift);
            fm <<= (23 - msize);
        }
    }
    else if(e == all_ones)
    {
        fm = m << (23 - msize);
        fe = 0xffu;
    }
    else
    {
        fm = m << (23 - msize);
        fe = (uint32_t)((int)e + (127 - bias));
    }
    return bits_f32((sign << 31) | (fe << 23) | fm);
}

uint16_t orc_half_from_f32(float x) { return (uint16_t)gf_from_f32(x, 10, 5); }
float orc_half_to_f32(uint16_t h) { return gf_to_f32(h, 10, 5); }
uint16_t orc_bf16_from_f32(float x) { return (uint16_t)gf_from_f32(x, 7, 8); }
float orc_bf16_to_f32(uint16_t h) { return gf_to_f32(h, 7, 8); }

/* ------------------------------------------------------------------------
 * fp8 e4m3fn (OCP, "fn": no infinities, 0x7f/0xff are NaN, max 448)
 * cast_from_f8<3,4,float,false>  src/include/migraphx/float8_impl.hpp:249-325
 * cast_to_f8<3,4,float,false,true(clip)> float8_impl.hpp:38-247, selected by
 * float8.hpp:87-101 with MIGRAPHX_F8_DOWNCAST_CLIPPING (float8.hpp:32).
 * Round to nearest even, saturate to +-448 (0x7e/0xfe), +-inf -> +-448,
 * NaN -> 0x7f / 0xff.
 * ---------------------------------------------------------------------- */
static float f8_to_f32(uint8_t x, int wm, int we)
{
    if(x == 0)
        return 0.0f;
    if(x == 0x80)
        return bits_f32(0x80000000u);
    uint32_t sign     = x >> 7;
    uint32_t mantissa = x & ((1u << wm) - 1u);
    int exponent      = (x & 0x7f) >> wm;
    if(we == 4)
    {
        if(x == 0x7f || x == 0xff)
            return bits_f32(0x7f800001u);
    }
    else if(exponent == 31) /* e5m2: +-inf, else NaN (float8_impl.hpp:286-291) */
    {
        if(mantissa == 0)
            return bits_f32(sign ? 0xff800000u : 0x7f800000u);
        return bits_f32(0x7f800001u);
    }
    const int exp_low_cutoff = (1 << (8 - 1)) - (1 << (we - 1)) + 1; /* 121 */
    if(exponent == 0)
    {
        int sh = 1 + __builtin_clz(mantissa) - (32 - wm);
        mantissa <<= sh;
        exponent += 1 - sh;
        mantissa &= (1u << wm) - 1u;
    }
    exponent += exp_low_cutoff - 1;
    mantissa <<= 23 - wm;
    return bits_f32((sign << 31) | ((uint32_t)exponent << 23) | mantissa);
}

static uint8_t f8_from_f32(float fx, uint32_t wm, uint32_t we)
{
    const uint32_t mfmt = 23;
    uint32_t x        = f32_bits(fx);
    uint32_t head     = x & 0xFF800000u;
    uint32_t mantissa = x & 0x7FFFFFu;
    int exponent      = (int)((head >> 23) & 0xFF);
    uint32_t sign     = head >> 31;
    const int bias    = 127;

    uint32_t signed_inf      = (sign << 7) + (((1u << we) - 1u) << wm);
    uint32_t signed_all_ones = (sign << 7) + ((((1u << we) - 1u) << wm) + ((1u << wm) - 1u));
    /* float8_impl.hpp:81-83: e4m3fn max is all ones - 1, e5m2 max is all ones - 4 */
    uint32_t signed_max = wm == 2 ? signed_all_ones - 4u : signed_all_ones - 1u;

    if((x & 0x7F800000u) == 0x7F800000u)
    {
        if(mantissa == 0)
            return (uint8_t)signed_max;                      /* float8_impl.hpp:103-109 */
        return (uint8_t)(signed_inf + ((1u << wm) - 1u));    /* all-ones mantissa NaN */
    }
    if(x == 0)
        return 0;
    if(x == 0x80000000u)
        return 0x80;

    const int f8_bias                  = (1 << (we - 1u)) - 1; /* 7 | 15 */
    const int f8_denormal_act_exponent = 1 - f8_bias;          /* -6 | -14 */
    int act_exponent, f8_exponent, exponent_diff;

    if(exponent == 0 && mantissa != 0)
    {
        act_exponent  = 1 - bias;
        exponent_diff = f8_denormal_act_exponent - act_exponent;
    }
    else
    {
        act_exponent = exponent - bias;
        if(act_exponent <= f8_denormal_act_exponent)
            exponent_diff = f8_denormal_act_exponent - act_exponent;
        else
            exponent_diff = 0;
        mantissa += (1u << mfmt);
    }

    uint32_t sh1 = mfmt - wm + (uint32_t)exponent_diff;
    if(sh1 > 31u)
        sh1 = 31u;
    uint32_t sh2 = mfmt - wm + (uint32_t)exponent_diff - 1u;
    if(sh2 > 31u)
        sh2 = 31u;
    int midpoint = (mantissa & ((1u << sh1) - 1u)) == (1u << sh2);

    if(exponent_diff > 0)
    {
        uint32_t s = (uint32_t)exponent_diff;
        if(s > 31u)
            s = 31u;
        mantissa >>= s;
    }
    else if(exponent_diff == -1)
        mantissa <<= 1;
    int implicit_one = (mantissa & (1u << mfmt)) != 0;
    f8_exponent      = (act_exponent + exponent_diff) + f8_bias - (implicit_one ? 0 : 1);

    uint32_t drop_mask = (1u << (mfmt - wm)) - 1u;
    int odd            = (mantissa & (1u << (mfmt - wm))) != 0;
    mantissa += (midpoint ? (odd ? mantissa : mantissa - 1u) : mantissa) & drop_mask;

    if(f8_exponent == 0 && ((1u << mfmt) & mantissa))
        f8_exponent = 1;
    else if((1u << (mfmt + 1)) & mantissa)
    {
        mantissa >>= 1;
        f8_exponent++;
    }
    mantissa >>= (mfmt - wm);

    /* float8_impl.hpp:228: exponent 31 of e5m2 belongs to inf and NaN */
    const int max_exp = (1 << we) - (wm == 3 ? 1 : 2);
    if(f8_exponent > max_exp)
        return (uint8_t)signed_max;
    if(f8_exponent == 0 && mantissa == 0)
        return (uint8_t)(sign << 7);
    mantissa &= (1u << wm) - 1u;
    uint8_t r = (uint8_t)((sign << 7) | ((uint32_t)f8_exponent << wm) | mantissa);
    /* e4m3fn: exponent 15 with mantissa 7 is the NaN code: the clip branch above is
       reached only for f8_exponent > 15, so 0x7f can come out of the rounding
       carry; the reference returns it unchanged (float8_impl.hpp:243-246). */
    return r;
}

float orc_fp8e4m3fn_to_f32(uint8_t x) { return f8_to_f32(x, 3, 4); }
uint8_t orc_fp8e4m3fn_from_f32(float fx) { return f8_from_f32(fx, 3, 4); }

/* ------------------------------------------------------------------------
 * fp8 e5m2 (OCP: exponent 31 is +-inf with mantissa 0, NaN otherwise; max 57344 = 0x7b)
 * cast_from_f8<2,5,float,false> / cast_to_f8<2,5,float,false,true(clip)>, selected by
 * float8.hpp:102-116.  Round to nearest even, saturate to +-57344, +-inf -> +-57344,
 * NaN -> 0x7f / 0xff.
 * ---------------------------------------------------------------------- */
float orc_fp8e5m2_to_f32(uint8_t x) { return f8_to_f32(x, 2, 5); }
uint8_t orc_fp8e5m2_from_f32(float fx) { return f8_from_f32(fx, 2, 5); }

/* vector forms for the Python side */
void orc_half_from_f32_n(const float* x, uint16_t* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_half_from_f32(x[i]);
}
void orc_half_to_f32_n(const uint16_t* x, float* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_half_to_f32(x[i]);
}
void orc_bf16_from_f32_n(const float* x, uint16_t* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_bf16_from_f32(x[i]);
}
void orc_bf16_to_f32_n(const uint16_t* x, float* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_bf16_to_f32(x[i]);
}
void orc_fp8e5m2_from_f32_n(const float* x, uint8_t* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_fp8e5m2_from_f32(x[i]);
}
void orc_fp8e5m2_to_f32_n(const uint8_t* x, float* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_fp8e5m2_to_f32(x[i]);
}
void orc_fp8e4m3fn_from_f32_n(const float* x, uint8_t* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_fp8e4m3fn_from_f32(x[i]);
}
void orc_fp8e4m3fn_to_f32_n(const uint8_t* x, float* y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = orc_fp8e4m3fn_to_f32(x[i]);
}

/* ------------------------------------------------------------------------
 * typed element access: what `static_cast<double>(view[i])` and
 * `view[i] = double_value` do for each element type on the ref target.
 * ---------------------------------------------------------------------- */
static inline double load_f64(const void* p, int type, size_t i)
{
    switch(type)
    {
    case ORC_I8: return (double)((const int8_t*)p)[i];
    case ORC_U8: return (double)((const uint8_t*)p)[i];
    case ORC_I32: return (double)((const int32_t*)p)[i];
    case ORC_F32: return (double)((const float*)p)[i];
    case ORC_F16: return (double)orc_half_to_f32(((const uint16_t*)p)[i]);
    case ORC_BF16: return (double)orc_bf16_to_f32(((const uint16_t*)p)[i]);
    case ORC_FP8: return (double)orc_fp8e4m3fn_to_f32(((const uint8_t*)p)[i]);
    case ORC_BF8: return (double)orc_fp8e5m2_to_f32(((const uint8_t*)p)[i]);
    case ORC_F64: return ((const double*)p)[i];
    default: return NAN;
    }
}

/* double -> T as C++ does it for `T x = d` / `static_cast<T>(d)`:
 * integers truncate, float rounds to nearest even, half/bf16/fp8 go through
 * float first (their constructors take a float) and then apply their own
 * conversion. */
static inline void store_f64(void* p, int type, size_t i, double d)
{
    switch(type)
    {
    case ORC_I8: ((int8_t*)p)[i] = (int8_t)d; break;
    case ORC_U8: ((uint8_t*)p)[i] = (uint8_t)d; break;
    case ORC_I32: ((int32_t*)p)[i] = (int32_t)d; break;
    case ORC_F32: ((float*)p)[i] = (float)d; break;
    case ORC_F16: ((uint16_t*)p)[i] = orc_half_from_f32((float)d); break;
    case ORC_BF16: ((uint16_t*)p)[i] = orc_bf16_from_f32((float)d); break;
    case ORC_FP8: ((uint8_t*)p)[i] = orc_fp8e4m3fn_from_f32((float)d); break;
    case ORC_BF8: ((uint8_t*)p)[i] = orc_fp8e5m2_from_f32((float)d); break;
    case ORC_F64: ((double*)p)[i] = d; break;
    default: break;
    }
}

static inline double type_max(int type)
{
    switch(type)
    {
    case ORC_I8: return 127.0;
    case ORC_U8: return 255.0;
    case ORC_I32: return 2147483647.0;
    case ORC_F32: return 3.40282346638528859811704183484516925e+38;
    case ORC_F16: return 65504.0;
    case ORC_BF16: return 3.38953138925153547590470800371487867e+38;
    case ORC_FP8: return 448.0;
    case ORC_BF8: return 57344.0; /* float8.hpp:361-373 */
    default: return INFINITY;
    }
}
static inline double type_lowest(int type)
{
    if(type == ORC_U8)
        return 0.0;
    if(type == ORC_I8)
        return -128.0;
    if(type == ORC_I32)
        return -2147483648.0;
    return -type_max(type);
}

/* ------------------------------------------------------------------------
 * gemm_naive  src/gemm.cpp:42-63, reached from
 *   ref_quant_gemm::compute  src/targets/ref/lowering.cpp:218-248 (quant_dot)
 *   op::dot::compute         src/include/migraphx/op/dot.hpp:102-107
 * One output element at a time: s (double) += double(a) * double(b) for k
 * ascending, then C = static_cast<T>(s).  Strides are element strides so that
 * transposed views (simplify_qdq.cpp:49-82 re-applies transposes to the
 * quantized tensor) need no copy.  C is written row-major, batch outermost.
 * ---------------------------------------------------------------------- */
void orc_gemm(void* c,
              int c_type,
              const void* a,
              const void* b,
              int ab_type,
              int64_t m,
              int64_t n,
              int64_t k,
              int64_t a_sm,
              int64_t a_sk,
              int64_t b_sk,
              int64_t b_sn,
              int64_t batch,
              int64_t a_sb,
              int64_t b_sb)
{
    int64_t total = batch * m * n;
#pragma omp parallel for schedule(static)
    for(int64_t idx = 0; idx < total; idx++)
    {
        int64_t bi = idx / (m * n);
        int64_t r  = idx % (m * n);
        int64_t i  = r / n;
        int64_t j  = r % n;
        double s   = 0.0;
        if(ab_type == ORC_I8)
        {
            const int8_t* ap = (const int8_t*)a + bi * a_sb + i * a_sm;
            const int8_t* bp = (const int8_t*)b + bi * b_sb + j * b_sn;
            for(int64_t kk = 0; kk < k; kk++)
                s += (double)ap[kk * a_sk] * (double)bp[kk * b_sk];
        }
        else
        {
            size_t a0 = (size_t)(bi * a_sb + i * a_sm);
            size_t b0 = (size_t)(bi * b_sb + j * b_sn);
            for(int64_t kk = 0; kk < k; kk++)
                s += load_f64(a, ab_type, a0 + (size_t)(kk * a_sk)) *
                     load_f64(b, ab_type, b0 + (size_t)(kk * b_sk));
        }
        store_f64(c, c_type, (size_t)idx, s);
    }
}

/* ------------------------------------------------------------------------
 * convolution  src/include/migraphx/convolution.hpp:37-100, called by
 *   op::quant_convolution::compute  src/include/migraphx/op/quant_convolution.hpp:142-157
 *   op::convolution::compute        src/include/migraphx/op/convolution.hpp:208-239
 * Cross-correlation of an [N, C, D, H, W] input with [O, C/group, KD, KH, KW] weights (the
 * reference's loop runs over any number of spatial axes; one, two and three are what its operators
 * accept): the window of output (n, o, z, y, x) starts at (z*stride - pad, y*stride - pad,
 * x*stride - pad), steps by the dilation, and positions outside the input contribute nothing.
 * Output channel o reads the input channels of group o / (O / group).  The sum runs over
 * (channel, kd, kh, kw) in that order in a double.
 * quant_convolution converts both tensors to double first (get_all<double>), so each product is
 * a double product; the float operator multiplies in float and adds the rounded product.
 * One conversion to the output type at the end.
 * ---------------------------------------------------------------------- */
void orc_convolution3d(void* out,
                       int out_type,
                       const void* x,
                       const void* w,
                       int x_type,
                       int64_t n,
                       int64_t c,
                       const int64_t* in_lens,  /* D, H, W of the input */
                       int64_t o,
                       const int64_t* win_lens, /* KD, KH, KW */
                       const int64_t* pad,      /* zeros in front of each spatial axis */
                       const int64_t* stride,
                       const int64_t* dil,
                       int64_t group,
                       const int64_t* out_lens) /* OD, OH, OW */
{
    const int64_t cg    = c / group; /* input channels per group = weights' second dimension */
    const int64_t og    = o / group;
    const int64_t d = in_lens[0], h = in_lens[1], wd = in_lens[2];
    const int64_t kd = win_lens[0], kh = win_lens[1], kw = win_lens[2];
    const int64_t od = out_lens[0], oh = out_lens[1], ow = out_lens[2];
    const int64_t total = n * o * od * oh * ow;
#pragma omp parallel for schedule(static)
    for(int64_t idx = 0; idx < total; idx++)
    {
        const int64_t ox = idx % ow;
        const int64_t oy = (idx / ow) % oh;
        const int64_t oz = (idx / (ow * oh)) % od;
        const int64_t oc = (idx / (ow * oh * od)) % o;
        const int64_t b  = idx / (ow * oh * od * o);
        const int64_t g  = oc / og;
        double acc       = 0.0;
        for(int64_t k = 0; k < cg; k++)
        {
            const int64_t ic = g * cg + k;
            for(int64_t t = 0; t < kd; t++)
            {
                const int64_t iz = oz * stride[0] - pad[0] + t * dil[0];
                for(int64_t r = 0; r < kh; r++)
                {
                    const int64_t iy = oy * stride[1] - pad[1] + r * dil[1];
                    for(int64_t q = 0; q < kw; q++)
                    {
                        const int64_t ix = ox * stride[2] - pad[2] + q * dil[2];
                        if(iz < 0 || iz >= d || iy < 0 || iy >= h || ix < 0 || ix >= wd)
                            continue;
                        const size_t xi = (size_t)((((b * c + ic) * d + iz) * h + iy) * wd + ix);
                        const size_t wi = (size_t)((((oc * cg + k) * kd + t) * kh + r) * kw + q);
                        if(x_type == ORC_F32)
                            acc += ((const float*)x)[xi] * ((const float*)w)[wi];
                        else
                            acc += load_f64(x, x_type, xi) * load_f64(w, x_type, wi);
                    }
                }
            }
        }
        store_f64(out, out_type, (size_t)idx, acc);
    }
}

/* the two-dimensional case: a depth of one */
void orc_convolution(void* out,
                     int out_type,
                     const void* x,
                     const void* w,
                     int x_type,
                     int64_t n,
                     int64_t c,
                     int64_t h,
                     int64_t wd,
                     int64_t o,
                     int64_t kh,
                     int64_t kw,
                     int64_t pad_h,
                     int64_t pad_w,
                     int64_t stride_h,
                     int64_t stride_w,
                     int64_t dil_h,
                     int64_t dil_w,
                     int64_t group,
                     int64_t oh,
                     int64_t ow)
{
    const int64_t in_lens[3]  = {1, h, wd};
    const int64_t win_lens[3] = {1, kh, kw};
    const int64_t pad[3]      = {0, pad_h, pad_w};
    const int64_t stride[3]   = {1, stride_h, stride_w};
    const int64_t dil[3]      = {1, dil_h, dil_w};
    const int64_t out_lens[3] = {1, oh, ow};
    orc_convolution3d(out, out_type, x, w, x_type, n, c, in_lens, o, win_lens, pad, stride, dil, group, out_lens);
}

/* ------------------------------------------------------------------------
 * quantizelinear::compute  src/include/migraphx/op/quantizelinear.hpp:71-108
 * integral output:  clamp(double(nearbyint(x / s)) + double(zp)) where x / s
 *   is evaluated in the input's own type (float division for float; for half
 *   and bf16 the quotient is converted back to that type, generic_float.hpp
 *   :318-326) under FE_TONEAREST.
 * fp8 output: clamp(double(x) / double(s) + double(zp), -448, 448), then
 *   double -> float -> fp8.
 * x is a dense [rows, cols] array; scale and zero point are addressed with
 * element strides (0 = broadcast) the way the broadcast views of the graph
 * address them.  zp == NULL means the all-zero default.
 * ---------------------------------------------------------------------- */
void orc_quantizelinear(void* out,
                        int out_type,
                        const void* x,
                        int x_type,
                        const void* scale,
                        int64_t s_sr,
                        int64_t s_sc,
                        const void* zp,
                        int64_t z_sr,
                        int64_t z_sc,
                        int64_t rows,
                        int64_t cols)
{
    int old = fegetround();
    fesetround(FE_TONEAREST);
    double lo    = type_lowest(out_type);
    double hi    = type_max(out_type);
    int integral = (out_type == ORC_I8 || out_type == ORC_U8 || out_type == ORC_I32);
#pragma omp parallel for schedule(static)
    for(int64_t r = 0; r < rows; r++)
    {
        fesetround(FE_TONEAREST);
        for(int64_t c = 0; c < cols; c++)
        {
            size_t i  = (size_t)(r * cols + c);
            size_t si = (size_t)(r * s_sr + c * s_sc);
            double z  = zp ? load_f64(zp, out_type, (size_t)(r * z_sr + c * z_sc)) : 0.0;
            double q;
            if(integral)
            {
                float xv = (float)load_f64(x, x_type, i);
                float sv = (float)load_f64(scale, x_type, si);
                float d  = xv / sv;
                if(x_type == ORC_F16)
                    d = orc_half_to_f32(orc_half_from_f32(d));
                else if(x_type == ORC_BF16)
                    d = orc_bf16_to_f32(orc_bf16_from_f32(d));
                q = (double)nearbyintf(d) + z;
            }
            else
            {
                q = load_f64(x, x_type, i) / load_f64(scale, x_type, si) + z;
            }
            double v = fmax(lo, fmin(hi, q));
            store_f64(out, out_type, i, v);
        }
    }
    fesetround(old);
}

/* ------------------------------------------------------------------------
 * dequantizelinear::compute src/include/migraphx/op/dequantizelinear.hpp:60-83
 * out = (double(x) - double(zp)) * scale, product in double (the scale is
 * promoted), stored to the scale's type.
 * ---------------------------------------------------------------------- */
void orc_dequantizelinear(void* out,
                          const void* x,
                          int x_type,
                          const void* scale,
                          int s_type,
                          int64_t s_sr,
                          int64_t s_sc,
                          const void* zp,
                          int64_t z_sr,
                          int64_t z_sc,
                          int64_t rows,
                          int64_t cols)
{
#pragma omp parallel for schedule(static)
    for(int64_t r = 0; r < rows; r++)
    {
        for(int64_t c = 0; c < cols; c++)
        {
            size_t i = (size_t)(r * cols + c);
            double z = zp ? load_f64(zp, x_type, (size_t)(r * z_sr + c * z_sc)) : 0.0;
            double s = load_f64(scale, s_type, (size_t)(r * s_sr + c * s_sc));
            store_f64(out, s_type, i, (load_f64(x, x_type, i) - z) * s);
        }
    }
}

/* ------------------------------------------------------------------------
 * unpack_int4::compute  src/include/migraphx/op/unpack_int4.hpp:75-121
 * pack_int4::compute    src/include/migraphx/op/pack_int4.hpp:79-124
 * Dense tensor seen as [outer, axis_len, inner]; the axis doubles (unpack) or
 * halves (pack).  Low nibble is the even element.
 * ---------------------------------------------------------------------- */
void orc_unpack_int4(
    uint8_t* out, const uint8_t* in, int is_signed, int64_t outer, int64_t axis_len, int64_t inner)
{
    for(int64_t o = 0; o < outer; o++)
        for(int64_t a = 0; a < axis_len; a++)
            for(int64_t i = 0; i < inner; i++)
            {
                uint8_t v   = in[(o * axis_len + a) * inner + i];
                size_t lo_i = (size_t)((o * 2 * axis_len + 2 * a) * inner + i);
                size_t hi_i = lo_i + (size_t)inner;
                if(is_signed)
                {
                    int8_t v1   = (int8_t)(uint8_t)(v << 4);
                    v1          = (int8_t)(v1 >> 4);
                    int8_t v2   = (int8_t)((int8_t)v >> 4);
                    out[lo_i]   = (uint8_t)v1;
                    out[hi_i]   = (uint8_t)v2;
                }
                else
                {
                    out[lo_i] = v & 0xf;
                    out[hi_i] = v >> 4;
                }
            }
}

void orc_pack_int4(
    uint8_t* out, const uint8_t* in, int is_signed, int64_t outer, int64_t axis_len, int64_t inner)
{
    /* axis_len is the OUTPUT axis length; the input axis is 2*axis_len */
    for(int64_t o = 0; o < outer; o++)
        for(int64_t a = 0; a < axis_len; a++)
            for(int64_t i = 0; i < inner; i++)
            {
                size_t i1 = (size_t)((o * 2 * axis_len + 2 * a) * inner + i);
                size_t i2 = i1 + (size_t)inner;
                uint8_t u1, u2;
                if(is_signed)
                {
                    int8_t v1 = (int8_t)in[i1], v2 = (int8_t)in[i2];
                    v1 = v1 < -8 ? -8 : (v1 > 7 ? 7 : v1);
                    v2 = v2 < -8 ? -8 : (v2 > 7 ? 7 : v2);
                    u1 = (uint8_t)v1;
                    u2 = (uint8_t)v2;
                }
                else
                {
                    u1 = in[i1] > 15 ? 15 : in[i1];
                    u2 = in[i2] > 15 ? 15 : in[i2];
                }
                out[(o * axis_len + a) * inner + i] = (uint8_t)((u2 << 4) | (u1 & 0xf));
            }
}

/* ------------------------------------------------------------------------
 * fp4 (e2m1) casts  src/include/migraphx/fp4_casts.hpp:41-100
 * unpack_fp4::compute  src/include/migraphx/op/unpack_fp4.hpp:78-101
 * pack_fp4::compute    src/include/migraphx/op/pack_fp4.hpp:82-106
 * A code is sign (bit 3), exponent (bits 2:1), mantissa (bit 0); the eight magnitudes are
 * 0, 0.5, 1, 1.5, 2, 3, 4, 6.  float -> fp4 rounds to the nearest magnitude, a tie going to the
 * neighbour with an even code (0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4,
 * 5 -> 4); anything above 5 (infinity included) gives 6; NaN gives code 0; the sign bit is kept,
 * also for zero.  unpack writes fp8 e4m3fn (every fp4 value is one), low nibble first; pack reads
 * floats.  Dense tensor seen as [outer, axis_len, inner] as for int4.
 * ---------------------------------------------------------------------- */
static const float orc_fp4_values[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

float orc_fp4_to_f32(uint8_t code)
{
    float v = orc_fp4_values[code & 7];
    return (code & 8) ? -v : v;
}

uint8_t orc_fp4_from_f32(float x)
{
    if(isnan(x))
        return 0;
    uint8_t sign = signbit(x) ? 8 : 0;
    float a      = fabsf(x);
    uint8_t i    = 0;
    /* first magnitude whose upper tie point is not passed; the tie belongs to the even code */
    for(i = 0; i < 7; i++)
    {
        float tie = 0.5f * (orc_fp4_values[i] + orc_fp4_values[i + 1]);
        if(a < tie || (a == tie && (i & 1) == 0))
            break;
    }
    return (uint8_t)(i | sign);
}

void orc_unpack_fp4(uint8_t* out, const uint8_t* in, int64_t outer, int64_t axis_len, int64_t inner)
{
    for(int64_t o = 0; o < outer; o++)
        for(int64_t a = 0; a < axis_len; a++)
            for(int64_t i = 0; i < inner; i++)
            {
                uint8_t v   = in[(o * axis_len + a) * inner + i];
                size_t lo_i = (size_t)((o * 2 * axis_len + 2 * a) * inner + i);
                size_t hi_i = lo_i + (size_t)inner;
                out[lo_i]   = orc_fp8e4m3fn_from_f32(orc_fp4_to_f32(v & 0xf));
                out[hi_i]   = orc_fp8e4m3fn_from_f32(orc_fp4_to_f32(v >> 4));
            }
}

void orc_pack_fp4(uint8_t* out, const float* in, int64_t outer, int64_t axis_len, int64_t inner)
{
    /* axis_len is the OUTPUT axis length; the input axis is 2*axis_len */
    for(int64_t o = 0; o < outer; o++)
        for(int64_t a = 0; a < axis_len; a++)
            for(int64_t i = 0; i < inner; i++)
            {
                size_t i1 = (size_t)((o * 2 * axis_len + 2 * a) * inner + i);
                size_t i2 = i1 + (size_t)inner;
                out[(o * axis_len + a) * inner + i] =
                    (uint8_t)((orc_fp4_from_f32(in[i2]) << 4) | (orc_fp4_from_f32(in[i1]) & 0xf));
            }
}

/* ------------------------------------------------------------------------
 * convert::compute  src/include/migraphx/op/convert.hpp:64-87
 * NaN -> quiet NaN of the target, +-inf kept for float targets, values at or
 * beyond the finite range saturate to max/lowest, otherwise T(double(x)).
 * ---------------------------------------------------------------------- */
void orc_convert(void* out, int out_type, const void* x, int x_type, size_t n)
{
    int integral = (out_type == ORC_I8 || out_type == ORC_U8 || out_type == ORC_I32);
#pragma omp parallel for schedule(static)
    for(size_t i = 0; i < n; i++)
    {
        double dx = load_f64(x, x_type, i);
        if(isnan(dx))
        {
            switch(out_type)
            {
            case ORC_F32: ((float*)out)[i] = bits_f32(0x7fc00000u); break;
            case ORC_F16: ((uint16_t*)out)[i] = 0x7e00; break;
            case ORC_BF16: ((uint16_t*)out)[i] = 0x7fc0; break;
            case ORC_FP8: ((uint8_t*)out)[i] = 0x7f; break;
            case ORC_BF8: ((uint8_t*)out)[i] = 0xff; break; /* float8.hpp:364 */
            default: store_f64(out, out_type, i, 0.0); break;
            }
            continue;
        }
        if(!integral && isinf(dx))
        {
            store_f64(out, out_type, i, dx);
            continue;
        }
        if(dx >= type_max(out_type))
            dx = type_max(out_type);
        else if(dx <= type_lowest(out_type))
            dx = type_lowest(out_type);
        store_f64(out, out_type, i, dx);
    }
}

/* mul of two float tensors (op/mul.hpp via op/binary.hpp): plain IEEE float
 * product, used by simplify_qdq.cpp:243-248 to combine the two input scales.
 * a is addressed [r*a_sr + c*a_sc], same for b; out is dense. */
void orc_mul_f32(float* out,
                 const float* a,
                 int64_t a_sr,
                 int64_t a_sc,
                 const float* b,
                 int64_t b_sr,
                 int64_t b_sc,
                 int64_t rows,
                 int64_t cols)
{
    for(int64_t r = 0; r < rows; r++)
        for(int64_t c = 0; c < cols; c++)
            out[r * cols + c] = a[r * a_sr + c * a_sc] * b[r * b_sr + c * b_sc];
}

/* ------------------------------------------------------------------------
 * Float operators around the quantized GEMMs of an encoder graph.  Tensors
 * are dense; a reduced / indexed axis is described as [outer, axis_len, inner].
 * ---------------------------------------------------------------------- */

/* op::add / sub / mul / div on float tensors: op/binary.hpp:60-90 applies the
 * plain C++ operator element by element (add.hpp, sub.hpp, mul.hpp, div.hpp). */
void orc_binary_f32(int op, float* out, const float* a, const float* b, size_t n)
{
    for(size_t i = 0; i < n; i++)
    {
        switch(op)
        {
        case 0: out[i] = a[i] + b[i]; break;
        case 1: out[i] = a[i] - b[i]; break;
        case 2: out[i] = a[i] * b[i]; break;
        default: out[i] = a[i] / b[i]; break;
        }
    }
}

/* op::erf / sqrt / rsqrt / exp / tanh / neg on float tensors: op/unary.hpp with
 * the lambdas std::erf(x) (erf.hpp), std::sqrt(x) (sqrt.hpp), 1 / std::sqrt(x)
 * (rsqrt.hpp:36-39), std::exp(x), std::tanh(x), -x, each on a float argument. */
void orc_unary_f32(int op, float* out, const float* x, size_t n)
{
    for(size_t i = 0; i < n; i++)
    {
        const float v = x[i];
        switch(op)
        {
        case 0: out[i] = erff(v); break;
        case 1: out[i] = sqrtf(v); break;
        case 2: out[i] = 1 / sqrtf(v); break;
        case 3: out[i] = expf(v); break;
        case 4: out[i] = tanhf(v); break;
        default: out[i] = -v; break;
        }
    }
}

/* op::reduce_mean: op/reduce_op.hpp:186-202 accumulates the reduced elements
 * in accumulator_type<float> = double (type_traits.hpp:78-81) in index order,
 * reduce_mean.hpp:45-48 divides by double(count); the store rounds to float. */
void orc_reduce_mean_f32(float* out, const float* x, int64_t outer, int64_t axis_len, int64_t inner)
{
    for(int64_t o = 0; o < outer; o++)
        for(int64_t i = 0; i < inner; i++)
        {
            double val = 0.0;
            for(int64_t a = 0; a < axis_len; a++)
                val = (double)x[(o * axis_len + a) * inner + i] + val;
            out[o * inner + i] = (float)(val / (double)axis_len);
        }
}

/* softmax: ref_softmax::compute, src/targets/ref/lowering.cpp:281-312.  Per
 * batch: max over the axis as double; out = float(exp(double(x) - max)); the
 * sum of those floats in a double; out = float(double(out) / sum). */
void orc_softmax_f32(float* out, const float* x, int64_t outer, int64_t axis_len, int64_t inner)
{
    for(int64_t o = 0; o < outer; o++)
        for(int64_t i = 0; i < inner; i++)
        {
            double mx = -DBL_MAX;
            for(int64_t a = 0; a < axis_len; a++)
            {
                double v = (double)x[(o * axis_len + a) * inner + i];
                mx       = mx < v ? v : mx;
            }
            for(int64_t a = 0; a < axis_len; a++)
            {
                size_t idx = (size_t)((o * axis_len + a) * inner + i);
                out[idx]   = (float)exp((double)x[idx] - mx);
            }
            double sum = 0.0;
            for(int64_t a = 0; a < axis_len; a++)
                sum += (double)out[(o * axis_len + a) * inner + i];
            for(int64_t a = 0; a < axis_len; a++)
            {
                size_t idx = (size_t)((o * axis_len + a) * inner + i);
                out[idx]   = (float)((double)out[idx] / sum);
            }
        }
}

/* gather: op/gather.hpp:100-118.  data is [outer, axis_len, inner] elements of
 * elem_size bytes, the n_idx indices replace the axis; a negative index counts
 * from the end of the axis. */
void orc_gather(void* out, const void* data, const int64_t* idx, int64_t n_idx, int64_t outer,
                int64_t axis_len, int64_t inner, int64_t elem_size)
{
    const size_t run = (size_t)(inner * elem_size);
    for(int64_t o = 0; o < outer; o++)
        for(int64_t j = 0; j < n_idx; j++)
        {
            int64_t id = idx[j] < 0 ? idx[j] + axis_len : idx[j];
            memcpy((char*)out + (size_t)(o * n_idx + j) * run,
                   (const char*)data + (size_t)(o * axis_len + id) * run, run);
        }
}
