// 16-bit and 8-bit float element types of the host layer.
//
// half and bf16 follow generic_float<M, E> (src/include/migraphx/generic_float.hpp:172-222): the
// conversion from float shifts the mantissa right, i.e. rounds toward zero, and an exponent beyond
// the format's range gives infinity.  fp8e4m3fn follows cast_to_f8 / cast_from_f8 with clipping
// (src/include/migraphx/float8_impl.hpp:38-325): round to nearest even, saturate at +-448, NaN
// codes 0x7f / 0xff, no infinities.
#ifndef MIGRAPHX_GUARD_FLOAT_TYPES_HPP
#define MIGRAPHX_GUARD_FLOAT_TYPES_HPP

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <type_traits>

namespace migraphx {
namespace detail {

inline uint32_t float_bits(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float bits_float(uint32_t u)
{
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// float -> narrow binary float with MB mantissa bits and EB exponent bits, truncating
template <int MB, int EB>
inline uint16_t narrow_truncate(float f)
{
    const uint32_t u    = float_bits(f);
    const uint16_t sign = (u >> 31) << (MB + EB);
    const int fexp      = (u >> 23) & 0xff;
    const uint32_t man  = u & 0x7fffff;
    const int emax      = (1 << EB) - 1;
    const int bias      = (1 << (EB - 1)) - 1;
    if(fexp == 0xff)
    {
        if(man == 0)
            return sign | (emax << MB);
        return sign | (emax << MB) | (1 << (MB - 1)) | (man >> (23 - MB)); // quiet NaN
    }
    if(fexp == 0) // float zero / subnormal: far below either format's smallest subnormal
        return sign;
    int e = fexp - 127 + bias;
    if(e >= emax)
        return sign | (emax << MB); // infinity
    if(e > 0)
        return sign | (e << MB) | (man >> (23 - MB));
    // subnormal of the narrow format: shift the mantissa with its hidden bit
    const int shift = 1 - e + (23 - MB);
    if(shift > 24)
        return sign;
    return sign | ((man | 0x800000) >> shift);
}

template <int MB, int EB>
inline float widen(uint16_t h)
{
    const uint32_t sign = uint32_t(h >> (MB + EB)) << 31;
    const int emax      = (1 << EB) - 1;
    const int bias      = (1 << (EB - 1)) - 1;
    int e               = (h >> MB) & emax;
    uint32_t man        = h & ((1 << MB) - 1);
    if(e == emax)
        return bits_float(sign | 0x7f800000 | (man << (23 - MB)));
    if(e == 0)
    {
        if(man == 0)
            return bits_float(sign);
        // subnormal: man * 2^(1 - bias - MB); for bf16 this is a float subnormal
        const float v = std::ldexp(static_cast<float>(man), 1 - bias - MB);
        return sign != 0 ? -v : v;
    }
    return bits_float(sign | uint32_t(e - bias + 127) << 23 | (man << (23 - MB)));
}

} // namespace detail

template <int MB, int EB>
struct narrow_float
{
    uint16_t bits = 0;
    narrow_float() = default;
    template <class T, std::enable_if_t<std::is_arithmetic<T>{}, int> = 0>
    narrow_float(T x) : bits(detail::narrow_truncate<MB, EB>(static_cast<float>(x))) // NOLINT
    {
    }
    operator float() const { return detail::widen<MB, EB>(bits); }               // NOLINT
    static narrow_float from_bits(uint16_t b)
    {
        narrow_float r;
        r.bits = b;
        return r;
    }
};

using half = narrow_float<10, 5>;
using bf16 = narrow_float<7, 8>;

struct fp8e4m3fn
{
    uint8_t bits = 0;
    fp8e4m3fn() = default;
    template <class T, std::enable_if_t<std::is_arithmetic<T>{}, int> = 0>
    fp8e4m3fn(T x) : bits(encode(static_cast<float>(x))) // NOLINT
    {
    }
    operator float() const { return decode(bits); }               // NOLINT
    static fp8e4m3fn from_bits(uint8_t b)
    {
        fp8e4m3fn r;
        r.bits = b;
        return r;
    }

    static float decode(uint8_t b)
    {
        const int e     = (b >> 3) & 0xf;
        const int m     = b & 7;
        const float sgn = (b & 0x80) != 0 ? -1.0f : 1.0f;
        if(e == 0xf and m == 7)
            return std::numeric_limits<float>::quiet_NaN();
        if(e == 0)
            return sgn * std::ldexp(static_cast<float>(m), -9);
        return sgn * std::ldexp(static_cast<float>(8 + m), e - 10);
    }

    // nearest representable value, ties to the even code, magnitudes from 448 up (and infinities)
    // saturate to +-448
    static uint8_t encode(float f)
    {
        const uint8_t sign = std::signbit(f) ? 0x80 : 0;
        if(std::isnan(f))
            return sign | 0x7f;
        const float a = std::fabs(f);
        if(a >= 448.0f)
            return sign | 0x7e;
        // spacing of the grid around a: 2^-9 below 2^-6, else 2^(floor(log2 a) - 3)
        int ex = 0;
        std::frexp(a, &ex); // a = m * 2^ex, m in [0.5, 1)
        int step_exp = (ex - 1) - 3;
        if(step_exp < -9)
            step_exp = -9;
        const float q = std::ldexp(a, -step_exp);   // exact
        float r       = std::nearbyint(q);          // FE_TONEAREST: ties to even
        const float v = std::ldexp(r, step_exp);
        if(v >= 480.0f)
            return sign | 0x7e;
        if(v == 0.0f)
            return sign;
        int e2 = 0;
        const float m2 = std::frexp(v, &e2); // v = m2 * 2^e2
        if(e2 - 1 < -6)
            return sign | static_cast<uint8_t>(std::ldexp(v, 9));
        const int mant = static_cast<int>(std::ldexp(m2, 4)) - 8;
        return sign | static_cast<uint8_t>(((e2 - 1 + 7) << 3) | mant);
    }
};

// fp8 e5m2 (src/include/migraphx/float8.hpp:102-116 with cast_to_f8<2, 5, float, false, true> /
// cast_from_f8<2, 5, float, false>): exponent 31 is +-infinity with a zero mantissa and NaN
// otherwise; conversion from float rounds to the nearest value, ties to the even code, and clips
// everything from 57344 up (infinities included) to +-57344.
struct fp8e5m2
{
    uint8_t bits = 0;
    fp8e5m2() = default;
    template <class T, std::enable_if_t<std::is_arithmetic<T>{}, int> = 0>
    fp8e5m2(T x) : bits(encode(static_cast<float>(x))) // NOLINT
    {
    }
    operator float() const { return decode(bits); }               // NOLINT
    static fp8e5m2 from_bits(uint8_t b)
    {
        fp8e5m2 r;
        r.bits = b;
        return r;
    }

    static float decode(uint8_t b)
    {
        const int e     = (b >> 2) & 0x1f;
        const int m     = b & 3;
        const float sgn = (b & 0x80) != 0 ? -1.0f : 1.0f;
        if(e == 0x1f)
            return m == 0 ? sgn * std::numeric_limits<float>::infinity()
                          : std::numeric_limits<float>::quiet_NaN();
        if(e == 0)
            return sgn * std::ldexp(static_cast<float>(m), -16);
        return sgn * std::ldexp(static_cast<float>(4 + m), e - 17);
    }

    static uint8_t encode(float f)
    {
        const uint8_t sign = std::signbit(f) ? 0x80 : 0;
        if(std::isnan(f))
            return sign | 0x7f;
        const float a = std::fabs(f);
        if(a >= 57344.0f)
            return sign | 0x7b;
        // spacing of the grid around a: 2^-16 below 2^-14, else 2^(floor(log2 a) - 2)
        int ex = 0;
        std::frexp(a, &ex);
        int step_exp = (ex - 1) - 2;
        if(step_exp < -16)
            step_exp = -16;
        const float q = std::ldexp(a, -step_exp);   // exact
        const float r = std::nearbyint(q);          // FE_TONEAREST: ties to even
        const float v = std::ldexp(r, step_exp);
        if(v > 57344.0f)
            return sign | 0x7b;
        if(v == 0.0f)
            return sign;
        int e2 = 0;
        const float m2 = std::frexp(v, &e2);
        if(e2 - 1 < -14)
            return sign | static_cast<uint8_t>(std::ldexp(v, 16));
        const int mant = static_cast<int>(std::ldexp(m2, 3)) - 4;
        return sign | static_cast<uint8_t>(((e2 - 1 + 15) << 2) | mant);
    }
};

} // namespace migraphx

namespace std {
template <int MB, int EB>
struct numeric_limits<migraphx::narrow_float<MB, EB>>
{
    using T = migraphx::narrow_float<MB, EB>;
    static constexpr bool is_specialized = true;
    static T max() { return T::from_bits(((((1 << EB) - 2) << MB) | ((1 << MB) - 1))); }
    static T lowest() { return T::from_bits((1 << (MB + EB)) | ((((1 << EB) - 2) << MB) | ((1 << MB) - 1))); }
    static T min() { return T::from_bits(1 << MB); }
    static T epsilon() { return T(std::ldexp(1.0f, -MB)); }
};
template <>
struct numeric_limits<migraphx::fp8e4m3fn>
{
    using T = migraphx::fp8e4m3fn;
    static constexpr bool is_specialized = true;
    static T max() { return T::from_bits(0x7e); }
    static T lowest() { return T::from_bits(0xfe); }
    static T min() { return T::from_bits(0x08); }
    static T epsilon() { return T::from_bits(0x20); }
};
template <>
struct numeric_limits<migraphx::fp8e5m2> // float8.hpp:357-375
{
    using T = migraphx::fp8e5m2;
    static constexpr bool is_specialized = true;
    static T max() { return T::from_bits(0x7b); }
    static T lowest() { return T::from_bits(0xfb); }
    static T min() { return T::from_bits(0x04); }
    static T epsilon() { return T::from_bits(0x34); }
    static T infinity() { return T::from_bits(0x7c); }
    static T quiet_NaN() { return T::from_bits(0xff); } // NOLINT
};
} // namespace std

#endif
