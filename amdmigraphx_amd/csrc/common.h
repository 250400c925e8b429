// Shared device/host helpers of the gfx950 quantized-GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "mi355_qgemm.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

#define MI355_DEVINL __device__ __forceinline__

static inline int mi355_launch_status()
{
    return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ERR_LAUNCH;
}

static inline size_t mi355_dtype_size(int t)
{
    switch(t)
    {
    case MI355_I8:
    case MI355_U8:
    case MI355_FP8:
    case MI355_BF8: return 1;
    case MI355_F16:
    case MI355_BF16: return 2;
    case MI355_I32:
    case MI355_F32: return 4;
    default: return 0;
    }
}

// ---------------------------------------------------------------------------
// Conversions with the ref target's semantics.
// ---------------------------------------------------------------------------

// float -> half bits, round toward zero, overflow to infinity from 2^16 on,
// as generic_float<10,5>::from_float does (generic_float.hpp:172-222).
MI355_DEVINL uint16_t f32_to_half_rtz(float x)
{
    // v_cvt_pkrtz_f16_f32 rounds toward zero, keeps subnormals and maps an
    // out-of-range finite value to the largest finite half; the software
    // conversion gives infinity for |x| >= 65536 instead.
    auto p       = __builtin_amdgcn_cvt_pkrtz(x, 0.0f);
    uint16_t h   = __builtin_bit_cast(uint32_t, p) & 0xffffu;
    uint32_t ux  = __builtin_bit_cast(uint32_t, x);
    uint32_t ax  = ux & 0x7fffffffu;
    if(ax >= 0x47800000u && ax < 0x7f800000u) // 65536 <= |x| < inf
        h = (uint16_t)(((ux >> 16) & 0x8000u) | 0x7c00u);
    // float subnormal inputs: the software path keeps exponent 0 and shifts the
    // float mantissa (fexp == 0 branch); hardware gives +-0.  Both are far
    // below half's range; follow the software result.
    if(ax != 0 && ax < 0x00800000u)
        h = (uint16_t)(((ux >> 16) & 0x8000u) | ((ux & 0x7fffffu) >> 13));
    if(ax > 0x7f800000u) // NaN: mantissa >> 13, may need a non-zero payload
        h = (uint16_t)(((ux >> 16) & 0x8000u) | 0x7c00u | ((ux & 0x7fffffu) >> 13));
    return h;
}

MI355_DEVINL float half_to_f32(uint16_t h)
{
    return (float)__builtin_bit_cast(_Float16, h);
}

MI355_DEVINL uint16_t f32_to_bf16_rtz(float x)
{
    return (uint16_t)(__builtin_bit_cast(uint32_t, x) >> 16);
}

MI355_DEVINL float bf16_to_f32(uint16_t h)
{
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}

// OCP e4m3fn decode (float8_impl.hpp:249-325); gfx950's converter is OCP.
MI355_DEVINL float fp8_to_f32(uint8_t v)
{
    return __builtin_amdgcn_cvt_f32_fp8((int)v, 0);
}

// float -> e4m3fn, nearest even.  The caller has clamped to [-448, 448]
// (quantizelinear and convert both do before the cast), so the saturation
// behaviour of the hardware converter outside that range never matters.
MI355_DEVINL uint8_t f32_to_fp8_rne(float x)
{
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(x, 0.0f, 0, false);
    return (uint8_t)(r & 0xff);
}

// OCP e5m2 decode (float8_impl.hpp:249-325 with Wm = 2, We = 5): an e5m2 code is the upper byte
// of the half with the same value, infinities and NaN included.
MI355_DEVINL float bf8_to_f32(uint8_t v)
{
    return half_to_f32((uint16_t)((uint32_t)v << 8));
}

// float -> e5m2, nearest even.  The caller has clamped to [-57344, 57344], as for e4m3fn above.
MI355_DEVINL uint8_t f32_to_bf8_rne(float x)
{
    int r = __builtin_amdgcn_cvt_pk_bf8_f32(x, 0.0f, 0, false);
    return (uint8_t)(r & 0xff);
}

// `convert` op (op/convert.hpp:64-87) from float to a 16-bit float type.
MI355_DEVINL uint16_t convert_f32_to_half(float x)
{
    // selects, not branches: the epilogues convert thousands of values per wave.  The hardware
    // conversion under round-toward-zero already gives the largest finite half for every finite
    // |x| >= 65504 and keeps infinities; what is left are NaN (one canonical result) and float
    // subnormals (the software conversion shifts the mantissa, the hardware gives +-0).
    const uint32_t ux = __builtin_bit_cast(uint32_t, x);
    const uint32_t ax = ux & 0x7fffffffu;
    const auto p      = __builtin_amdgcn_cvt_pkrtz(x, 0.0f);
    uint32_t h        = __builtin_bit_cast(uint32_t, p) & 0xffffu;
    h = (ax - 1u < 0x007fffffu) ? (((ux >> 16) & 0x8000u) | ((ux & 0x7fffffu) >> 13)) : h;
    h = x != x ? 0x7e00u : h;
    return (uint16_t)h;
}

MI355_DEVINL uint16_t convert_f32_to_bf16(float x)
{
    // toward zero: every finite value at or beyond the largest finite bf16 has that number's upper
    // half already, infinities keep theirs; NaN gets the one canonical result
    const uint32_t ux = __builtin_bit_cast(uint32_t, x);
    return (uint16_t)(x != x ? 0x7fc0u : ux >> 16);
}

// two of them side by side (lo in the low half): one v_perm_b32 takes both upper halves
MI355_DEVINL uint32_t convert_f32_to_bf16x2(float lo, float hi)
{
    const uint32_t ulo = lo != lo ? 0x7fc00000u : __builtin_bit_cast(uint32_t, lo);
    const uint32_t uhi = hi != hi ? 0x7fc00000u : __builtin_bit_cast(uint32_t, hi);
    return __builtin_amdgcn_perm(uhi, ulo, 0x07060302u);
}

// The `add` of a bias behind dequantizelinear: its own fp32 rounding, never contracted with the
// multiplication in front of it.  b = -0.0f leaves every value (signed zeros and NaN included) as
// it is, which is how "no bias" is passed.
MI355_DEVINL float add_bias(float v, float b)
{
#pragma clang fp contract(off)
    return v + b;
}

// Typed loads as double / stores from double, mirroring
// static_cast<double>(view[i]) and view[i] = d on the ref target.
MI355_DEVINL double load_as_f64(const void* p, int type, int64_t i)
{
    switch(type)
    {
    case MI355_I8: return (double)((const int8_t*)p)[i];
    case MI355_U8: return (double)((const uint8_t*)p)[i];
    case MI355_I32: return (double)((const int32_t*)p)[i];
    case MI355_F32: return (double)((const float*)p)[i];
    case MI355_F16: return (double)half_to_f32(((const uint16_t*)p)[i]);
    case MI355_BF16: return (double)bf16_to_f32(((const uint16_t*)p)[i]);
    case MI355_FP8: return (double)fp8_to_f32(((const uint8_t*)p)[i]);
    case MI355_BF8: return (double)bf8_to_f32(((const uint8_t*)p)[i]);
    default: return 0.0;
    }
}

// quantizelinear's saturation: std::max(lo, std::min(hi, q)) with std::min / std::max's comparison
// order, so a NaN ends up at hi exactly as on the reference's CPU target
// (src/include/migraphx/op/quantizelinear.hpp:95-104)
MI355_DEVINL double clamp_like_ref(double q, double lo, double hi)
{
    double v = (q < hi) ? q : hi;
    return (lo < v) ? v : lo;
}
