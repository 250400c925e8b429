// HBM-bound elementwise operators of the quantized path: quantizelinear,
// dequantizelinear, unpack_int4, pack_int4, convert.  Each thread handles a
// short run of consecutive elements so loads and stores are wide and
// coalesced; the arithmetic follows the ref target step by step.
#include "common.h"

namespace {

constexpr int PW_THREADS = 256;

template <int XT>
MI355_DEVINL float load_x(const void* x, int64_t i)
{
    if constexpr(XT == MI355_F32)
        return static_cast<const float*>(x)[i];
    else if constexpr(XT == MI355_F16)
        return half_to_f32(static_cast<const uint16_t*>(x)[i]);
    else
        return bf16_to_f32(static_cast<const uint16_t*>(x)[i]);
}

// x / s evaluated in x's own type (generic_float's operator/ converts the float
// quotient back to the narrow type, generic_float.hpp:318-326)
template <int XT>
MI355_DEVINL float div_in_type(float x, float s)
{
    float d = x / s;
    if constexpr(XT == MI355_F16)
        d = half_to_f32(f32_to_half_rtz(d));
    else if constexpr(XT == MI355_BF16)
        d = bf16_to_f32(f32_to_bf16_rtz(d));
    return d;
}

struct qparams
{
    const void* scale;
    int64_t s_sr, s_sc;
    const void* zp;
    int64_t z_sr, z_sc;
};

template <int XT, int OT>
__global__ __launch_bounds__(PW_THREADS) void quantizelinear_kernel(
    const void* x, qparams q, void* out, int64_t rows, int64_t cols)
{
    // 4 consecutive elements of one row per thread (cols is padded up per row)
    const int64_t cols4  = (cols + 3) / 4;
    const int64_t gid    = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if(gid >= rows * cols4)
        return;
    const int64_t r  = gid / cols4;
    const int64_t c0 = (gid - r * cols4) * 4;
    uint8_t res[4];
    const int cnt = (int)min((int64_t)4, cols - c0);
    for(int e = 0; e < cnt; e++)
    {
        const int64_t c = c0 + e;
        const float xv  = load_x<XT>(x, r * cols + c);
        const float sv  = load_x<XT>(q.scale, r * q.s_sr + c * q.s_sc);
        if constexpr(OT == MI355_FP8)
        {
            double z = 0.0;
            if(q.zp != nullptr)
                z = (double)fp8_to_f32(static_cast<const uint8_t*>(q.zp)[r * q.z_sr + c * q.z_sc]);
            double v = clamp_like_ref((double)xv / (double)sv + z, -448.0, 448.0);
            res[e]   = f32_to_fp8_rne((float)v);
        }
        else if constexpr(OT == MI355_BF8)
        {
            double z = 0.0;
            if(q.zp != nullptr)
                z = (double)bf8_to_f32(static_cast<const uint8_t*>(q.zp)[r * q.z_sr + c * q.z_sc]);
            double v = clamp_like_ref((double)xv / (double)sv + z, -57344.0, 57344.0);
            res[e]   = f32_to_bf8_rne((float)v);
        }
        else
        {
            double z = 0.0;
            if(q.zp != nullptr)
            {
                if constexpr(OT == MI355_I8)
                    z = (double)static_cast<const int8_t*>(q.zp)[r * q.z_sr + c * q.z_sc];
                else
                    z = (double)static_cast<const uint8_t*>(q.zp)[r * q.z_sr + c * q.z_sc];
            }
            double qv = (double)rintf(div_in_type<XT>(xv, sv)) + z;
            if constexpr(OT == MI355_I8)
                res[e] = (uint8_t)(int8_t)(int)clamp_like_ref(qv, -128.0, 127.0);
            else
                res[e] = (uint8_t)(int)clamp_like_ref(qv, 0.0, 255.0);
        }
    }
    uint8_t* o = static_cast<uint8_t*>(out) + r * cols + c0;
    if(cnt == 4 && ((reinterpret_cast<uintptr_t>(o) & 3) == 0))
        *reinterpret_cast<uint32_t*>(o) =
            res[0] | ((uint32_t)res[1] << 8) | ((uint32_t)res[2] << 16) | ((uint32_t)res[3] << 24);
    else
        for(int e = 0; e < cnt; e++)
            o[e] = res[e];
}

// fp32 -> int8 with one scale and one zero point for the whole tensor (activations): 16 elements
// per thread as four 16-byte loads and one 16-byte store, the same arithmetic as above.  n16 is
// the element count / 16; x and out are 16-byte aligned.
__global__ __launch_bounds__(PW_THREADS) void quantize_f32_i8_tensor_kernel(
    const v4f* x, const float* scale, const int8_t* zp, uint4* out, int64_t n16)
{
    const float sv = scale[0];
    const double z = zp != nullptr ? (double)zp[0] : 0.0;
    const int64_t step = (int64_t)gridDim.x * PW_THREADS;
    for(int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x; i < n16; i += step)
    {
        v4f v[4];
#pragma unroll
        for(int j = 0; j < 4; j++)
            v[j] = x[4 * i + j];
        uint32_t w[4];
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            w[j] = 0;
#pragma unroll
            for(int e = 0; e < 4; e++)
            {
                const double qv = (double)rintf(v[j][e] / sv) + z;
                const uint32_t b = (uint8_t)(int8_t)(int)clamp_like_ref(qv, -128.0, 127.0);
                w[j] |= b << (8 * e);
            }
        }
        out[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__global__ __launch_bounds__(PW_THREADS) void dequantizelinear_kernel(const void* x,
                                                                      int x_type,
                                                                      qparams q,
                                                                      int s_type,
                                                                      void* out,
                                                                      int64_t rows,
                                                                      int64_t cols)
{
    const int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if(i >= rows * cols)
        return;
    const int64_t r = i / cols;
    const int64_t c = i - r * cols;
    double z        = 0.0;
    if(q.zp != nullptr)
        z = load_as_f64(q.zp, x_type, r * q.z_sr + c * q.z_sc);
    const double s = load_as_f64(q.scale, s_type, r * q.s_sr + c * q.s_sc);
    const double v = (load_as_f64(x, x_type, i) - z) * s;
    // stored to the scale's type: double -> float (nearest even), then the
    // narrow type's own conversion from float (round toward zero)
    const float f = (float)v;
    if(s_type == MI355_F32)
        static_cast<float*>(out)[i] = f;
    else if(s_type == MI355_F16)
        static_cast<uint16_t*>(out)[i] = f32_to_half_rtz(f);
    else
        static_cast<uint16_t*>(out)[i] = f32_to_bf16_rtz(f);
}

// one packed byte -> two bytes; 8 packed bytes per thread where aligned
__global__ __launch_bounds__(PW_THREADS) void unpack_int4_kernel(
    const uint8_t* in, uint8_t* out, int is_signed, int64_t total)
{
    const int64_t i0 = ((int64_t)blockIdx.x * PW_THREADS + threadIdx.x) * 8;
    if(i0 >= total)
        return;
    const int cnt = (int)min((int64_t)8, total - i0);
    for(int e = 0; e < cnt; e++)
    {
        uint8_t v = in[i0 + e];
        uint8_t lo, hi;
        if(is_signed)
        {
            lo = (uint8_t)((int8_t)(uint8_t)(v << 4) >> 4);
            hi = (uint8_t)((int8_t)v >> 4);
        }
        else
        {
            lo = v & 0xf;
            hi = v >> 4;
        }
        out[2 * (i0 + e)]     = lo;
        out[2 * (i0 + e) + 1] = hi;
    }
}

// fp4 (e2m1): sign, two exponent bits, one mantissa bit; magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6.
// Their fp8 e4m3fn codes (exponent bias 7, three mantissa bits), indexed by the low three bits:
__constant__ const uint8_t fp4_as_fp8[8] = {0x00, 0x30, 0x38, 0x3c, 0x40, 0x44, 0x48, 0x4c};

// one packed byte -> two fp8 bytes, low nibble first; 8 packed bytes per thread
__global__ __launch_bounds__(PW_THREADS) void unpack_fp4_kernel(const uint8_t* in, uint8_t* out, int64_t total)
{
    const int64_t i0 = ((int64_t)blockIdx.x * PW_THREADS + threadIdx.x) * 8;
    if(i0 >= total)
        return;
    const int cnt = (int)min((int64_t)8, total - i0);
    for(int e = 0; e < cnt; e++)
    {
        const uint8_t v       = in[i0 + e];
        out[2 * (i0 + e)]     = fp4_as_fp8[v & 7] | ((v & 0x08) << 4);
        out[2 * (i0 + e) + 1] = fp4_as_fp8[(v >> 4) & 7] | (v & 0x80);
    }
}

// float -> fp4 code: nearest magnitude, a tie to the neighbour with the even code, beyond 5 -> 6
// (infinity included), NaN -> 0, sign kept (also for zero)
MI355_DEVINL uint8_t f32_to_fp4(float x)
{
    if(x != x)
        return 0;
    const uint8_t sign = (__builtin_bit_cast(uint32_t, x) >> 31) ? 8 : 0;
    const float a      = __builtin_fabsf(x);
    uint8_t i;
    if(a <= 0.25f)
        i = 0;
    else if(a < 0.75f)
        i = 1;
    else if(a <= 1.25f)
        i = 2;
    else if(a < 1.75f)
        i = 3;
    else if(a <= 2.5f)
        i = 4;
    else if(a < 3.5f)
        i = 5;
    else if(a <= 5.0f)
        i = 6;
    else
        i = 7;
    return i | sign;
}

__global__ __launch_bounds__(PW_THREADS) void pack_fp4_kernel(const float* in, uint8_t* out, int64_t total_out)
{
    const int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if(i >= total_out)
        return;
    out[i] = (uint8_t)((f32_to_fp4(in[2 * i + 1]) << 4) | f32_to_fp4(in[2 * i]));
}

__global__ __launch_bounds__(PW_THREADS) void pack_int4_kernel(
    const uint8_t* in, uint8_t* out, int is_signed, int64_t total_out)
{
    const int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if(i >= total_out)
        return;
    uint8_t u1, u2;
    if(is_signed)
    {
        int v1 = (int8_t)in[2 * i], v2 = (int8_t)in[2 * i + 1];
        v1 = max(-8, min(7, v1));
        v2 = max(-8, min(7, v2));
        u1 = (uint8_t)v1;
        u2 = (uint8_t)v2;
    }
    else
    {
        u1 = min((int)in[2 * i], 15);
        u2 = min((int)in[2 * i + 1], 15);
    }
    out[i] = (uint8_t)((u2 << 4) | (u1 & 0xf));
}

__global__ __launch_bounds__(PW_THREADS) void convert_kernel(
    const void* in, int in_type, void* out, int out_type, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x;
    if(i >= n)
        return;
    const double dx = load_as_f64(in, in_type, i);
    const float f   = (float)dx;
    switch(out_type)
    {
    case MI355_F32:
        static_cast<float*>(out)[i] = (dx != dx) ? __builtin_bit_cast(float, 0x7fc00000u) : f;
        break;
    case MI355_F16: static_cast<uint16_t*>(out)[i] = convert_f32_to_half(f); break;
    case MI355_BF16: static_cast<uint16_t*>(out)[i] = convert_f32_to_bf16(f); break;
    case MI355_FP8:
        if(dx != dx)
            static_cast<uint8_t*>(out)[i] = 0x7f;
        else
            static_cast<uint8_t*>(out)[i] =
                f32_to_fp8_rne((float)fmin(448.0, fmax(-448.0, dx)));
        break;
    case MI355_I8:
        // integral targets: NaN -> numeric_limits::quiet_NaN() = 0, saturate, then truncate toward zero
        static_cast<int8_t*>(out)[i] = dx != dx ? (int8_t)0 : (int8_t)(int)fmin(127.0, fmax(-128.0, dx));
        break;
    case MI355_U8:
        static_cast<uint8_t*>(out)[i] = dx != dx ? (uint8_t)0 : (uint8_t)(int)fmin(255.0, fmax(0.0, dx));
        break;
    case MI355_I32:
        static_cast<int32_t*>(out)[i] =
            dx != dx ? 0 : (int32_t)fmin(2147483647.0, fmax(-2147483648.0, dx));
        break;
    case MI355_BF8:
        // numeric_limits<fp8e5m2>::quiet_NaN() is 0xff (float8.hpp:364); infinities go through
        // the clipping constructor
        if(dx != dx)
            static_cast<uint8_t*>(out)[i] = 0xff;
        else
            static_cast<uint8_t*>(out)[i] =
                f32_to_bf8_rne((float)fmin(57344.0, fmax(-57344.0, dx)));
        break;
    default: break;
    }
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + PW_THREADS - 1) / PW_THREADS); }

template <int XT>
int launch_quantize(int out_type,
                    const void* x,
                    const qparams& q,
                    void* out,
                    int64_t rows,
                    int64_t cols,
                    hipStream_t s)
{
    const int64_t work = rows * ((cols + 3) / 4);
    switch(out_type)
    {
    case MI355_I8:
        hipLaunchKernelGGL((quantizelinear_kernel<XT, MI355_I8>), dim3(blocks_for(work)),
                           dim3(PW_THREADS), 0, s, x, q, out, rows, cols);
        break;
    case MI355_U8:
        hipLaunchKernelGGL((quantizelinear_kernel<XT, MI355_U8>), dim3(blocks_for(work)),
                           dim3(PW_THREADS), 0, s, x, q, out, rows, cols);
        break;
    case MI355_FP8:
        hipLaunchKernelGGL((quantizelinear_kernel<XT, MI355_FP8>), dim3(blocks_for(work)),
                           dim3(PW_THREADS), 0, s, x, q, out, rows, cols);
        break;
    case MI355_BF8:
        hipLaunchKernelGGL((quantizelinear_kernel<XT, MI355_BF8>), dim3(blocks_for(work)),
                           dim3(PW_THREADS), 0, s, x, q, out, rows, cols);
        break;
    default: return MI355_ERR_UNSUPPORTED;
    }
    return mi355_launch_status();
}

} // namespace

extern "C" int mi355_quantizelinear(const void* x,
                                    int32_t x_type,
                                    const void* scale,
                                    int64_t scale_stride_r,
                                    int64_t scale_stride_c,
                                    const void* zp,
                                    int64_t zp_stride_r,
                                    int64_t zp_stride_c,
                                    void* out,
                                    int32_t out_type,
                                    int64_t rows,
                                    int64_t cols,
                                    void* stream)
{
    if(x == nullptr || scale == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    if(rows == 0 || cols == 0)
        return MI355_OK;
    if(rows * ((cols + 3) / 4) > (int64_t)0x7fffffff * PW_THREADS)
        return MI355_ERR_UNSUPPORTED;
    qparams q{scale, scale_stride_r, scale_stride_c, zp, zp_stride_r, zp_stride_c};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t total = rows * cols;
    if(x_type == MI355_F32 && out_type == MI355_I8 && scale_stride_r == 0 && scale_stride_c == 0 &&
       (zp == nullptr || (zp_stride_r == 0 && zp_stride_c == 0)) && total % 16 == 0 &&
       reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0)
    {
        const int64_t n16 = total / 16;
        int64_t blocks    = (n16 + PW_THREADS - 1) / PW_THREADS;
        if(blocks > 256 * 32)
            blocks = 256 * 32;
        hipLaunchKernelGGL(quantize_f32_i8_tensor_kernel, dim3((unsigned)blocks), dim3(PW_THREADS), 0, s,
                           static_cast<const v4f*>(x), static_cast<const float*>(scale),
                           static_cast<const int8_t*>(zp), static_cast<uint4*>(out), n16);
        return mi355_launch_status();
    }
    switch(x_type)
    {
    case MI355_F32: return launch_quantize<MI355_F32>(out_type, x, q, out, rows, cols, s);
    case MI355_F16: return launch_quantize<MI355_F16>(out_type, x, q, out, rows, cols, s);
    case MI355_BF16: return launch_quantize<MI355_BF16>(out_type, x, q, out, rows, cols, s);
    default: return MI355_ERR_UNSUPPORTED;
    }
}

extern "C" int mi355_dequantizelinear(const void* x,
                                      int32_t x_type,
                                      const void* scale,
                                      int32_t scale_type,
                                      int64_t scale_stride_r,
                                      int64_t scale_stride_c,
                                      const void* zp,
                                      int64_t zp_stride_r,
                                      int64_t zp_stride_c,
                                      void* out,
                                      int64_t rows,
                                      int64_t cols,
                                      void* stream)
{
    if(x == nullptr || scale == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    if(x_type != MI355_I8 && x_type != MI355_U8 && x_type != MI355_I32 && x_type != MI355_F32 &&
       x_type != MI355_FP8 && x_type != MI355_BF8)
        return MI355_ERR_UNSUPPORTED;
    if(scale_type != MI355_F32 && scale_type != MI355_F16 && scale_type != MI355_BF16)
        return MI355_ERR_UNSUPPORTED;
    if(rows == 0 || cols == 0)
        return MI355_OK;
    qparams q{scale, scale_stride_r, scale_stride_c, zp, zp_stride_r, zp_stride_c};
    hipLaunchKernelGGL(dequantizelinear_kernel, dim3(blocks_for(rows * cols)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), x, x_type, q, scale_type, out, rows, cols);
    return mi355_launch_status();
}

extern "C" int mi355_unpack_int4(
    const void* in, void* out, int32_t is_signed, int64_t rows, int64_t cols, void* stream)
{
    if(in == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    const int64_t total = rows * cols;
    if(total == 0)
        return MI355_OK;
    hipLaunchKernelGGL(unpack_int4_kernel, dim3(blocks_for((total + 7) / 8)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(in),
                       static_cast<uint8_t*>(out), is_signed, total);
    return mi355_launch_status();
}

extern "C" int mi355_pack_int4(
    const void* in, void* out, int32_t is_signed, int64_t rows, int64_t cols, void* stream)
{
    if(in == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    if(cols % 2 != 0)
        return MI355_ERR_BAD_ARG; // PACK_INT4: can not pack an axis of odd length
    const int64_t total_out = rows * (cols / 2);
    if(total_out == 0)
        return MI355_OK;
    hipLaunchKernelGGL(pack_int4_kernel, dim3(blocks_for(total_out)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(in),
                       static_cast<uint8_t*>(out), is_signed, total_out);
    return mi355_launch_status();
}

// ---- int4 pack / unpack along any axis of a strided view ------------------------------------
// One thread per packed byte.  `lens` are the lengths of the packed tensor (unpack: the input,
// pack: the output); the byte with multi-index idx pairs with the elements idx[axis] * 2 and
// idx[axis] * 2 + 1 of the unpacked tensor.  The strided side (the input) is addressed through
// element strides, zero for a broadcast dimension; the output is dense row-major.
struct int4_nd_params
{
    const uint8_t* in;
    uint8_t* out;
    int64_t lens[MI355_MAX_DIMS];
    int64_t in_strides[MI355_MAX_DIMS];
    int64_t out_strides[MI355_MAX_DIMS];
    int64_t total;
    int ndim, axis, is_signed;
};

template <bool PACK>
__global__ __launch_bounds__(PW_THREADS) void int4_nd_kernel(int4_nd_params p)
{
    for(int64_t i = (int64_t)blockIdx.x * PW_THREADS + threadIdx.x; i < p.total;
        i += (int64_t)gridDim.x * PW_THREADS)
    {
        int64_t rest = i, in_off = 0, out_off = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            const int64_t idx = rest % p.lens[d];
            rest /= p.lens[d];
            // along the axis the unpacked side holds two elements per packed byte
            in_off += idx * p.in_strides[d] * ((PACK && d == p.axis) ? 2 : 1);
            out_off += idx * p.out_strides[d] * ((!PACK && d == p.axis) ? 2 : 1);
        }
        if constexpr(PACK)
        {
            const uint8_t r1 = p.in[in_off], r2 = p.in[in_off + p.in_strides[p.axis]];
            uint8_t u1, u2;
            if(p.is_signed)
            {
                u1 = (uint8_t)max(-8, min(7, (int)(int8_t)r1));
                u2 = (uint8_t)max(-8, min(7, (int)(int8_t)r2));
            }
            else
            {
                u1 = (uint8_t)min((int)r1, 15);
                u2 = (uint8_t)min((int)r2, 15);
            }
            p.out[out_off] = (uint8_t)((u2 << 4) | (u1 & 0xf));
        }
        else
        {
            const uint8_t v = p.in[in_off];
            uint8_t lo, hi;
            if(p.is_signed)
            {
                lo = (uint8_t)((int8_t)(uint8_t)(v << 4) >> 4);
                hi = (uint8_t)((int8_t)v >> 4);
            }
            else
            {
                lo = v & 0xf;
                hi = v >> 4;
            }
            p.out[out_off]                         = lo;
            p.out[out_off + p.out_strides[p.axis]] = hi;
        }
    }
}

template <bool PACK>
static int launch_int4_nd(const void* in, void* out, int32_t is_signed, int32_t ndim, const int64_t* lens,
                          const int64_t* in_strides, int32_t axis, void* stream)
{
    if(ndim < 1 || ndim > MI355_MAX_DIMS || lens == nullptr || in_strides == nullptr)
        return MI355_ERR_BAD_ARG;
    if(axis < 0)
        axis += ndim;
    if(axis < 0 || axis >= ndim)
        return MI355_ERR_BAD_ARG;
    int4_nd_params p{};
    p.total = 1;
    for(int d = 0; d < ndim; d++)
    {
        if(lens[d] < 0 || in_strides[d] < 0)
            return MI355_ERR_BAD_ARG;
        p.lens[d]       = lens[d]; // lengths of the INPUT
        p.in_strides[d] = in_strides[d];
    }
    if(PACK)
    {
        if(lens[axis] % 2 != 0)
            return MI355_ERR_BAD_ARG; // PACK_INT4: can not pack an axis of odd length
        p.lens[axis] = lens[axis] / 2; // the kernel walks the packed tensor
    }
    // dense strides of the output
    int64_t run = 1;
    for(int d = ndim - 1; d >= 0; d--)
    {
        p.out_strides[d] = run;
        run *= (!PACK && d == axis) ? p.lens[d] * 2 : p.lens[d];
        p.total *= p.lens[d];
    }
    if(p.total == 0)
        return MI355_OK;
    if(in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.in        = static_cast<const uint8_t*>(in);
    p.out       = static_cast<uint8_t*>(out);
    p.ndim      = ndim;
    p.axis      = axis;
    p.is_signed = is_signed;
    int64_t blocks = (p.total + PW_THREADS - 1) / PW_THREADS;
    if(blocks > 256 * 16)
        blocks = 256 * 16;
    hipLaunchKernelGGL(int4_nd_kernel<PACK>, dim3((unsigned)blocks), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

extern "C" int mi355_unpack_int4_nd(const void* in, void* out, int32_t is_signed, int32_t ndim,
                                    const int64_t* lens, const int64_t* in_strides, int32_t axis, void* stream)
{
    return launch_int4_nd<false>(in, out, is_signed, ndim, lens, in_strides, axis, stream);
}

extern "C" int mi355_pack_int4_nd(const void* in, void* out, int32_t is_signed, int32_t ndim,
                                  const int64_t* lens, const int64_t* in_strides, int32_t axis, void* stream)
{
    return launch_int4_nd<true>(in, out, is_signed, ndim, lens, in_strides, axis, stream);
}

extern "C" int mi355_unpack_fp4(const void* in, void* out, int64_t rows, int64_t cols, void* stream)
{
    if(in == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    const int64_t total = rows * cols;
    if(total == 0)
        return MI355_OK;
    hipLaunchKernelGGL(unpack_fp4_kernel, dim3(blocks_for((total + 7) / 8)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(in),
                       static_cast<uint8_t*>(out), total);
    return mi355_launch_status();
}

extern "C" int mi355_pack_fp4(const float* in, void* out, int64_t rows, int64_t cols, void* stream)
{
    if(in == nullptr || out == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    if(cols % 2 != 0)
        return MI355_ERR_BAD_ARG; // PACK_FP4: can not pack along an axis of odd length
    const int64_t total_out = rows * (cols / 2);
    if(total_out == 0)
        return MI355_OK;
    hipLaunchKernelGGL(pack_fp4_kernel, dim3(blocks_for(total_out)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), in, static_cast<uint8_t*>(out), total_out);
    return mi355_launch_status();
}

extern "C" int mi355_convert(
    const void* in, int32_t in_type, void* out, int32_t out_type, int64_t n, void* stream)
{
    if(in == nullptr || out == nullptr || n < 0)
        return MI355_ERR_BAD_ARG;
    if(mi355_dtype_size(in_type) == 0 || mi355_dtype_size(out_type) == 0)
        return MI355_ERR_BAD_ARG;
    if(out_type != MI355_F32 && out_type != MI355_F16 && out_type != MI355_BF16 &&
       out_type != MI355_FP8 && out_type != MI355_BF8 && out_type != MI355_I8 && out_type != MI355_U8 &&
       out_type != MI355_I32)
        return MI355_ERR_UNSUPPORTED;
    if(n == 0)
        return MI355_OK;
    hipLaunchKernelGGL(convert_kernel, dim3(blocks_for(n)), dim3(PW_THREADS), 0,
                       static_cast<hipStream_t>(stream), in, in_type, out, out_type, n);
    return mi355_launch_status();
}
