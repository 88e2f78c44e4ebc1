// scalar_convert.hpp -- host-side conversion of one scalar between the nine element types, with
// the same rules the device kernels apply (aix_device.h: convert<S, D>): float-like -> integer
// saturates and maps NaN to 0, anything -> f16/bf16 goes through float with round-to-nearest-even,
// everything else is a plain C++ conversion (aixDeviceCPU.cpp:96-117, aixFloat16.hpp:201-252,
// 783-805).
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>

namespace aixhip::scalar {

inline uint32_t bits_of(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float float_of(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1F) return float_of(sign | 0x7F800000u | (m << 13));
    if (e == 0) {
        if (m == 0) return float_of(sign);
        e = 1;
        while (!(m & 0x400u)) { m <<= 1; --e; }        // normalise the subnormal
        m &= 0x3FFu;
        return float_of(sign | ((e + 112u) << 23) | (m << 13));
    }
    return float_of(sign | ((e + 112u) << 23) | (m << 13));
}

inline uint16_t float_to_half(float f)
{
    const uint32_t u = bits_of(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t e = (u >> 23) & 0xFFu, m = u & 0x7FFFFFu;
    if (e == 0xFF) return (uint16_t)(sign | 0x7C00u | (m ? (0x0200u | (m >> 13)) : 0u));
    const int he = (int)e - 112;
    if (he >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (he <= 0) {
        if (he < -10) return sign;
        const uint32_t full = m | 0x800000u, sh = (uint32_t)(14 - he);
        uint16_t r = (uint16_t)(sign | (full >> sh));
        const uint32_t rest = full & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rest > half || (rest == half && (r & 1u))) ++r;
        return r;
    }
    uint16_t r = (uint16_t)(sign | ((uint32_t)he << 10) | (m >> 13));
    const uint32_t rest = m & 0x1FFFu;
    if (rest > 0x1000u || (rest == 0x1000u && (r & 1u))) ++r;
    return r;
}

inline uint16_t float_to_bf16(float f)
{
    const uint32_t u = bits_of(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x7FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
inline float bf16_to_float(uint16_t b) { return float_of((uint32_t)b << 16); }

// A scalar decoded into the widest lossless carrier of its class.
struct Value {
    enum Kind { kFloat, kSigned, kUnsigned } kind{kFloat};
    long double f{0};
    int64_t i{0};
    uint64_t u{0};
};

inline Value decode(const void* p, int dtype)
{
    Value v;
    switch (dtype) {
        case 0: { double x; std::memcpy(&x, p, 8); v.f = x; break; }
        case 1: { float x; std::memcpy(&x, p, 4); v.f = x; break; }
        case 2: { uint16_t x; std::memcpy(&x, p, 2); v.f = half_to_float(x); break; }
        case 3: { uint16_t x; std::memcpy(&x, p, 2); v.f = bf16_to_float(x); break; }
        case 4: { int64_t x; std::memcpy(&x, p, 8); v.kind = Value::kSigned; v.i = x; break; }
        case 5: { int32_t x; std::memcpy(&x, p, 4); v.kind = Value::kSigned; v.i = x; break; }
        case 6: { int16_t x; std::memcpy(&x, p, 2); v.kind = Value::kSigned; v.i = x; break; }
        case 7: { int8_t x; std::memcpy(&x, p, 1); v.kind = Value::kSigned; v.i = x; break; }
        case 8: { uint8_t x; std::memcpy(&x, p, 1); v.kind = Value::kUnsigned; v.u = x; break; }
        default: break;
    }
    return v;
}

template <class D> inline D to_integer(const Value& v)
{
    if (v.kind == Value::kFloat) {
        long double x = v.f;
        if (std::isnan(x)) return 0;
        const long double lo = (long double)std::numeric_limits<D>::lowest(), hi = (long double)std::numeric_limits<D>::max();
        x = x < lo ? lo : (x > hi ? hi : x);
        return (D)x;
    }
    // integer -> integer is a plain cast (wraps), as static_cast does on the CPU device
    return v.kind == Value::kSigned ? (D)v.i : (D)v.u;
}

template <class F> inline F to_floating(const Value& v)
{
    return v.kind == Value::kFloat ? (F)v.f : v.kind == Value::kSigned ? (F)v.i : (F)v.u;
}

// Writes the converted scalar (element type `to`) at `out`; returns its size in bytes.
inline size_t encode(const Value& v, int to, void* out)
{
    switch (to) {
        case 0: { const double x = to_floating<double>(v); std::memcpy(out, &x, 8); return 8; }
        case 1: { const float x = to_floating<float>(v); std::memcpy(out, &x, 4); return 4; }
        case 2: { const uint16_t x = float_to_half(to_floating<float>(v)); std::memcpy(out, &x, 2); return 2; }
        case 3: { const uint16_t x = float_to_bf16(to_floating<float>(v)); std::memcpy(out, &x, 2); return 2; }
        case 4: { const int64_t x = to_integer<int64_t>(v); std::memcpy(out, &x, 8); return 8; }
        case 5: { const int32_t x = to_integer<int32_t>(v); std::memcpy(out, &x, 4); return 4; }
        case 6: { const int16_t x = to_integer<int16_t>(v); std::memcpy(out, &x, 2); return 2; }
        case 7: { const int8_t x = to_integer<int8_t>(v); std::memcpy(out, &x, 1); return 1; }
        case 8: { const uint8_t x = to_integer<uint8_t>(v); std::memcpy(out, &x, 1); return 1; }
        default: return 0;
    }
}

} // namespace aixhip::scalar
