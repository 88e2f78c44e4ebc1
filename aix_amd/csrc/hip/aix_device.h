// aix_device.h -- device-side element types, conversions and per-element operators.
//
// Shared by the precompiled kernels and by every runtime-generated fused kernel (the text of
// this file is the hipRTC prelude), so it includes nothing and uses only compiler builtins and
// the device math library that hipcc/hipRTC declare implicitly.
//
// Semantics mirror the reference CPU device (Targets/AIXLib/aixDeviceCPU.cpp) and its software
// 16-bit floats (Targets/AIXLib/aixFloat16.hpp):
//   * f16 / bf16 arithmetic happens in f32 and is rounded to 16 bits (RNE) after EVERY operator;
//   * integer arithmetic wraps; float -> integer conversion saturates and maps NaN to 0
//     (aixDeviceCPU.cpp:96-117);
//   * sqrt/log/exp/pow on integer element types evaluate in floating point and saturate back;
//     sin/cos/tanh on integers truncate toward zero (aixDeviceCPU.cpp:154-242);
//   * compile with -ffp-contract=off: a*b+c must stay two roundings.
#ifndef AIX_DEVICE_H
#define AIX_DEVICE_H

namespace aixd {

typedef signed char        i8;
typedef unsigned char      u8;
typedef short              i16;
typedef unsigned short     u16;
typedef int                i32;
typedef unsigned int       u32;
typedef long long          i64;
typedef unsigned long long u64;
typedef _Float16           f16;

// bfloat16 storage word.  f32 -> bf16 is the hardware conversion (v_cvt_pk_bf16_f32): round to nearest even,
// and a NaN keeps its upper payload bits and gets bit 6 set -- on every one of the 2^32 inputs the value the
// reference computes on the integer image, ((u + 0x7FFF + ((u >> 16) & 1)) >> 16, NaN: (u >> 16) | 0x40;
// aixFloat16.hpp:783-805), in one instruction instead of seven.
struct bf16 { u16 bits; };

__device__ __forceinline__ float bf16_up(bf16 v) { return __builtin_bit_cast(float, (u32)v.bits << 16); }
__device__ __forceinline__ bf16 bf16_down(float f)
{
    // through inline assembly: given the conversion as an fptrunc, this compiler's instruction selection fails on
    // some negations that feed it
    u32 packed;
    asm("v_cvt_pk_bf16_f32 %0, %1, %1" : "=v"(packed) : "v"(f));
    bf16 r;
    r.bits = (u16)packed;
    return r;
}

enum { DT_F64 = 0, DT_F32 = 1, DT_F16 = 2, DT_BF16 = 3, DT_I64 = 4, DT_I32 = 5, DT_I16 = 6, DT_I8 = 7, DT_U8 = 8 };

// ---- traits ---------------------------------------------------------------------------------
// W = type in which one operator is evaluated before rounding back to T.
template <class T> struct traits;
template <> struct traits<double> { typedef double W; enum { code = DT_F64, is_float = 1, is_int = 0 }; };
template <> struct traits<float>  { typedef float  W; enum { code = DT_F32, is_float = 1, is_int = 0 }; };
template <> struct traits<f16>    { typedef float  W; enum { code = DT_F16, is_float = 1, is_int = 0 }; };
template <> struct traits<bf16>   { typedef float  W; enum { code = DT_BF16, is_float = 1, is_int = 0 }; };
template <> struct traits<i64>    { typedef i64 W; typedef u64 U; enum { code = DT_I64, is_float = 0, is_int = 1, is_signed = 1 }; };
template <> struct traits<i32>    { typedef i32 W; typedef u32 U; enum { code = DT_I32, is_float = 0, is_int = 1, is_signed = 1 }; };
template <> struct traits<i16>    { typedef i32 W; typedef u32 U; enum { code = DT_I16, is_float = 0, is_int = 1, is_signed = 1 }; };
template <> struct traits<i8>     { typedef i32 W; typedef u32 U; enum { code = DT_I8,  is_float = 0, is_int = 1, is_signed = 1 }; };
template <> struct traits<u8>     { typedef i32 W; typedef u32 U; enum { code = DT_U8,  is_float = 0, is_int = 1, is_signed = 0 }; };

template <class T> __device__ __forceinline__ typename traits<T>::W up(T v) { return (typename traits<T>::W)v; }
template <> __device__ __forceinline__ float up<bf16>(bf16 v) { return bf16_up(v); }
template <class T> __device__ __forceinline__ T down(typename traits<T>::W v) { return (T)v; }
template <> __device__ __forceinline__ bf16 down<bf16>(float v) { return bf16_down(v); }

template <class T> __device__ __forceinline__ T zero() { return down<T>((typename traits<T>::W)0); }

// lowest(): aixDeviceCPU.cpp:130-138, aixFloat16.hpp:173-178, 767-772.
template <class T> __device__ __forceinline__ T lowest();
template <> __device__ __forceinline__ double lowest<double>() { return -1.7976931348623157e308; }
template <> __device__ __forceinline__ float  lowest<float>()  { return -3.402823466e38f; }
template <> __device__ __forceinline__ f16    lowest<f16>()    { return __builtin_bit_cast(f16, (u16)0xFBFF); }
template <> __device__ __forceinline__ bf16   lowest<bf16>()   { bf16 r; r.bits = 0xFF7F; return r; }
template <> __device__ __forceinline__ i64    lowest<i64>()    { return (i64)0x8000000000000000ull; }
template <> __device__ __forceinline__ i32    lowest<i32>()    { return (i32)0x80000000u; }
template <> __device__ __forceinline__ i16    lowest<i16>()    { return (i16)-32768; }
template <> __device__ __forceinline__ i8     lowest<i8>()     { return (i8)-128; }
template <> __device__ __forceinline__ u8     lowest<u8>()     { return (u8)0; }

// ---- conversions ----------------------------------------------------------------------------
// double -> integer with saturation, NaN -> 0.
template <class D> __device__ __forceinline__ D sat_from_double(double x);
template <> __device__ __forceinline__ i64 sat_from_double<i64>(double x)
{
    if (x != x) return 0;
    if (x >= 9223372036854775808.0) return (i64)0x7FFFFFFFFFFFFFFFull;
    if (x <= -9223372036854775808.0) return (i64)0x8000000000000000ull;
    return (i64)x;
}
template <> __device__ __forceinline__ i32 sat_from_double<i32>(double x)
{ if (x != x) return 0; x = x < -2147483648.0 ? -2147483648.0 : (x > 2147483647.0 ? 2147483647.0 : x); return (i32)x; }
template <> __device__ __forceinline__ i16 sat_from_double<i16>(double x)
{ if (x != x) return 0; x = x < -32768.0 ? -32768.0 : (x > 32767.0 ? 32767.0 : x); return (i16)(i32)x; }
template <> __device__ __forceinline__ i8 sat_from_double<i8>(double x)
{ if (x != x) return 0; x = x < -128.0 ? -128.0 : (x > 127.0 ? 127.0 : x); return (i8)(i32)x; }
template <> __device__ __forceinline__ u8 sat_from_double<u8>(double x)
{ if (x != x) return 0; x = x < 0.0 ? 0.0 : (x > 255.0 ? 255.0 : x); return (u8)(i32)x; }

// Any element type as double (exact for every type except |i64| > 2^53).
template <class S> __device__ __forceinline__ double as_double(S v) { return (double)v; }
template <> __device__ __forceinline__ double as_double<bf16>(bf16 v) { return (double)bf16_up(v); }
template <> __device__ __forceinline__ double as_double<f16>(f16 v) { return (double)(float)v; }

// convert<S, D>: the value conversion of copy / fill.  Float-like -> integer saturates;
// everything that targets a 16-bit float goes through float first (aixFloat16.hpp has only a
// float constructor), everything else is a plain C++ conversion.
template <class S, class D> struct conv {
    static __device__ __forceinline__ D run(S v)
    {
        if constexpr (traits<S>::is_float && traits<D>::is_int) return sat_from_double<D>(as_double<S>(v));
        else if constexpr (traits<D>::code == DT_BF16) {
            if constexpr (traits<S>::code == DT_BF16) return v;
            else if constexpr (traits<S>::code == DT_F16) return bf16_down((float)v);
            else return bf16_down((float)v);
        }
        else if constexpr (traits<D>::code == DT_F16) {
            if constexpr (traits<S>::code == DT_BF16) return (f16)bf16_up(v);
            else return (f16)(float)v;
        }
        else if constexpr (traits<S>::code == DT_BF16) return (D)bf16_up(v);
        else if constexpr (traits<S>::code == DT_F16) return (D)(float)v;
        else return (D)v;
    }
};
template <class S, class D> __device__ __forceinline__ D convert(S v) { return conv<S, D>::run(v); }

// ---- arithmetic -----------------------------------------------------------------------------
template <class T> __device__ __forceinline__ T e_add(T a, T b)
{
    if constexpr (traits<T>::is_int) { typedef typename traits<T>::U U; return (T)((U)a + (U)b); }
    else return down<T>(up(a) + up(b));
}
template <class T> __device__ __forceinline__ T e_sub(T a, T b)
{
    if constexpr (traits<T>::is_int) { typedef typename traits<T>::U U; return (T)((U)a - (U)b); }
    else return down<T>(up(a) - up(b));
}
template <class T> __device__ __forceinline__ T e_mul(T a, T b)
{
    if constexpr (traits<T>::is_int) { typedef typename traits<T>::U U; return (T)((U)a * (U)b); }
    else return down<T>(up(a) * up(b));
}
template <class T> __device__ __forceinline__ T e_div(T a, T b)
{
    if constexpr (traits<T>::is_int) {
        // Division by zero and lowest / -1 trap on the CPU; here they are defined: 0 and wrap.
        typedef typename traits<T>::W W;
        const W x = (W)a, y = (W)b;
        if (y == 0) return (T)0;
        if constexpr (traits<T>::is_signed) { if (y == (W)-1) { typedef typename traits<T>::U U; return (T)((U)0 - (U)a); } }
        return (T)(x / y);
    }
    else return down<T>(up(a) / up(b));
}
template <class T> __device__ __forceinline__ T e_neg(T a)
{
    if constexpr (traits<T>::is_int) { typedef typename traits<T>::U U; return (T)((U)0 - (U)a); }
    else return down<T>(-up(a));
}

// Comparisons in the evaluation type: +-0 equal, NaN unordered (aixFloat16.hpp:66-95).
template <class T> __device__ __forceinline__ bool e_gt(T a, T b) { return up(a) > up(b); }
template <class T> __device__ __forceinline__ bool e_lt(T a, T b) { return up(a) < up(b); }
template <class T> __device__ __forceinline__ bool e_isnan(T a)
{
    if constexpr (traits<T>::is_float) { const typename traits<T>::W w = up(a); return w != w; }
    else return false;
}

// ---- math -----------------------------------------------------------------------------------
enum { M_SQRT = 1, M_SIN = 2, M_COS = 3, M_TANH = 4, M_LOG = 5, M_EXP = 6 };

template <int F> __device__ __forceinline__ float math_f32(float x)
{
    if constexpr (F == M_SQRT) return sqrtf(x);
    else if constexpr (F == M_SIN) return sinf(x);
    else if constexpr (F == M_COS) return cosf(x);
    else if constexpr (F == M_TANH) return tanhf(x);
    else if constexpr (F == M_LOG) return logf(x);
    else return expf(x);
}
template <int F> __device__ __forceinline__ double math_f64(double x)
{
    if constexpr (F == M_SQRT) {
        // The library routine can be one unit off; one Newton step on the exact residual
        // (fused multiply-add) makes the result correctly rounded, as the CPU's is.
        double y = sqrt(x);
        if (x > 0.0 && x < __builtin_huge_val()) {
            const double r = __builtin_fma(-y, y, x);
            y = __builtin_fma(r, 0.5 / y, y);
        }
        return y;
    }
    else if constexpr (F == M_SIN) return sin(x);
    else if constexpr (F == M_COS) return cos(x);
    else if constexpr (F == M_TANH) return tanh(x);
    else if constexpr (F == M_LOG) return log(x);
    else return exp(x);
}

template <int F, class T> __device__ __forceinline__ T e_math(T a)
{
    if constexpr (traits<T>::code == DT_F64) return math_f64<F>(a);
    else if constexpr (traits<T>::is_float) return down<T>(math_f32<F>(up(a)));
    else {
        const double r = math_f64<F>((double)a);
        if constexpr (F == M_SIN || F == M_COS || F == M_TANH) return (T)(i32)r;   // |r| <= 1: truncation
        else return sat_from_double<T>(r);
    }
}
template <class T> __device__ __forceinline__ T e_sqrt(T a) { return e_math<M_SQRT>(a); }
template <class T> __device__ __forceinline__ T e_sin(T a)  { return e_math<M_SIN>(a); }
template <class T> __device__ __forceinline__ T e_cos(T a)  { return e_math<M_COS>(a); }
template <class T> __device__ __forceinline__ T e_tanh(T a) { return e_math<M_TANH>(a); }
template <class T> __device__ __forceinline__ T e_log(T a)  { return e_math<M_LOG>(a); }
template <class T> __device__ __forceinline__ T e_exp(T a)  { return e_math<M_EXP>(a); }

// Integer power as the saturated, truncated real value of base^e (what the CPU's long double
// evaluation followed by the saturating conversion yields): exact by repeated multiplication on
// the magnitude, clamped to the range of T; negative exponents give 0 except for bases 0, 1, -1.
template <class T> __device__ __forceinline__ T int_pow(T base, T e)
{
    const i64 b = (i64)base, n = (i64)e;
    const i64 hi = (i64)(((u64)1 << (8 * sizeof(T) - (traits<T>::is_signed ? 1 : 0))) - 1);   // max of T
    const i64 lo = traits<T>::is_signed ? -hi - 1 : 0;
    if (n == 0) return (T)1;
    if (b == 1) return (T)1;
    if (b == -1) return (T)((n & 1) ? -1 : 1);
    if (b == 0) return n > 0 ? (T)0 : (T)hi;                       // 0^negative = +inf -> max
    if (n < 0) return (T)0;                                        // |b| >= 2: |result| < 1
    const bool negative = b < 0 && (n & 1);
    const u64 mag = b < 0 ? (u64)0 - (u64)b : (u64)b;
    const u64 limit = negative ? (u64)hi + 1 : (u64)hi;            // |lo| or hi
    u64 r = 1;
    for (i64 k = 0; k < n; ++k) {
        if (r > limit / mag) { r = limit + 1; break; }             // would exceed: saturate
        r *= mag;
    }
    if (r > limit) return negative ? (T)lo : (T)hi;
    return negative ? (T)(i64)((u64)0 - r) : (T)(i64)r;
}

template <class T> __device__ __forceinline__ T e_pow(T a, T b)
{
    if constexpr (traits<T>::code == DT_F64) return pow(a, b);
    else if constexpr (traits<T>::is_float) {
        // squares and cubes (GELU's x^3 and its derivative) as products: two roundings at most, inside the 2 ulp of
        // powf, a fraction of its cost; the exponent usually is one scalar for the whole tensor, so the branch is uniform
        const float x = up(a), e = up(b);
        if (e == 2.0f) return down<T>(x * x);
        if (e == 3.0f) return down<T>(x * x * x);
        return down<T>(powf(x, e));
    }
    else return int_pow<T>(a, b);
}

// tril / triu as an elementwise predicate over the flat logical index of a tensor whose last two dims are [rows, cols]:
// tril keeps columns up to row + diagonal, triu columns from row + diagonal on.  The (row, column) of a vector's first
// element is found once per vector (two divisions, 32-bit when everything fits); its other elements step the column.
struct TriPos { i64 r, c; };
__device__ __forceinline__ TriPos tri_origin(u64 i, u64 rows, u64 cols)
{
    TriPos p;
    if (((i | rows | cols) >> 32) == 0) {
        const u32 q = (u32)i / (u32)cols;
        p.c = (i64)((u32)i - q * (u32)cols);
        p.r = (i64)(q % (u32)rows);
    } else {
        const u64 q = i / cols;
        p.c = (i64)(i - q * cols);
        p.r = (i64)(q % rows);
    }
    return p;
}
__device__ __forceinline__ bool tri_keeps(TriPos p, int e, u64 rows, u64 cols, i64 diagonal, int upper)
{
    i64 c = p.c + e, r = p.r;
    while (c >= (i64)cols) { c -= (i64)cols; if (++r == (i64)rows) r = 0; }      // the vector runs over the end of a row
    return upper ? c >= r + diagonal : c <= r + diagonal;
}

// ---- 16-byte vectors of any element type ------------------------------------------------------
template <class T, int N> struct alignas(sizeof(T) * N) vec { T v[N]; };
template <class T> struct vec16 { enum { n = 16 / sizeof(T) }; typedef vec<T, 16 / sizeof(T)> type; };

// An operand of a row-shaped kernel: the 16-byte vector at row + col, or -- the operand is broadcast along the row --
// copies of the one element *row.  Without a branch: a branch per operand makes the compiler wait for the first
// operand's data before it issues the second operand's load (two memory latencies per lane instead of one; measured
// 86 -> 74 us on x[8192, 8192] + v[8192]).  The broadcast element is fetched as the aligned 16 bytes around it (a
// naturally aligned 16-byte block holding a valid element lies in the same page: the read cannot fault) and picked
// out afterwards.
template <class T, int N> __device__ __forceinline__ const vec<T, N>* row_vec_ptr(const T* row, u64 col, bool bcast)
{
    // as an offset from `row`, so that the pointer keeps its (global) address space
    const long long off = bcast ? -(long long)((u64)row & (u64)(sizeof(T) * N - 1)) : (long long)(col * sizeof(T));
    return (const vec<T, N>*)((const char*)row + off);
}
template <class T, int N> __device__ __forceinline__ vec<T, N> row_vec_fix(vec<T, N> v, const T* row, bool bcast)
{
    const unsigned k = (unsigned)(((u64)row & (u64)(sizeof(T) * N - 1)) / sizeof(T));
    T s = v.v[0];
#pragma unroll
    for (int j = 1; j < N; ++j) s = k == (unsigned)j ? v.v[j] : s;
#pragma unroll
    for (int e = 0; e < N; ++e) v.v[e] = bcast ? s : v.v[e];
    return v;
}

// Sum / maximum of one value per lane over the LANES (64: a wave, 256: the workgroup's four waves through `red`) lanes
// that share a row, returned to every one of them.  The order is that of the stand-alone reduction kernels -- shuffle
// tree down to lane 0 of a wave, then wave 0's result combined with waves 1, 2, 3 in turn -- so that a sum formed
// inside a fused kernel has the bits of the same sum formed by itself.
template <int LANES, class W> __device__ __forceinline__ W row_sum(W v, W* red)
{
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_down(v, d, 64);
    if constexpr (LANES == 64) return __shfl(v, 0, 64);
    else {
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        return ((red[0] + red[1]) + red[2]) + red[3];
    }
}
// The place of a row's first maximum (argmaxIndicesTo along the row): every lane brings the best of its own elements --
// the largest value that is no NaN and the smallest column holding it -- and all lanes get the winner back.  A greater
// value wins, between equal values the smaller column; a lane without a candidate loses to one with.
template <int LANES, class W> __device__ __forceinline__ u32 row_first_max(W v, u32 at, bool valid, W* red, u32* redi)
{
    u32 ok = valid ? 1u : 0u;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        const W ov = __shfl_down(v, d, 64);
        const u32 oat = __shfl_down(at, d, 64), ook = __shfl_down(ok, d, 64);
        const bool take = (ok && ook) ? (ov > v || (ov == v && oat < at)) : (ook != 0 && ok == 0);
        if (take) { v = ov; at = oat; ok = ook; }
    }
    if constexpr (LANES == 64) return __shfl(at, 0, 64);
    else {
        __syncthreads();
        if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = v; redi[threadIdx.x >> 6] = at; redi[4 + (threadIdx.x >> 6)] = ok; }
        __syncthreads();
        v = red[0]; at = redi[0]; ok = redi[4];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const W ov = red[w];
            const u32 oat = redi[w], ook = redi[4 + w];
            const bool take = (ok && ook) ? (ov > v || (ov == v && oat < at)) : (ook != 0 && ok == 0);
            if (take) { v = ov; at = oat; ok = ook; }
        }
        return at;
    }
}
template <int LANES, class W> __device__ __forceinline__ W row_max(W v, W* red)
{
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) { const W o = __shfl_down(v, d, 64); v = o > v ? o : v; }
    if constexpr (LANES == 64) return __shfl(v, 0, 64);
    else {
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        W r = red[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) r = red[w] > r ? red[w] : r;
        return r;
    }
}

// Stores of values that this kernel and its neighbours will not read again.  A non-temporal store does not allocate its
// line in the caches on the way out: on results of tens of megabytes that is worth 15 % of a copy-shaped kernel's time
// (negate over 256 MiB: 87 -> 74 us; the transpose copy: 93 -> 79 us); small results are stored normally so that the
// next kernel finds them in cache.
template <class V> __device__ __forceinline__ void store_nt(V* p, const V& v)
{
    if constexpr (sizeof(V) == 16) { typedef unsigned int w4 __attribute__((ext_vector_type(4))); __builtin_nontemporal_store(__builtin_bit_cast(w4, v), (w4*)p); }
    else if constexpr (sizeof(V) == 8) __builtin_nontemporal_store(__builtin_bit_cast(unsigned long long, v), (unsigned long long*)p);
    else if constexpr (sizeof(V) == 4) __builtin_nontemporal_store(__builtin_bit_cast(unsigned int, v), (unsigned int*)p);
    else if constexpr (sizeof(V) == 2) __builtin_nontemporal_store(__builtin_bit_cast(unsigned short, v), (unsigned short*)p);
    else if constexpr (sizeof(V) == 1) __builtin_nontemporal_store(__builtin_bit_cast(unsigned char, v), (unsigned char*)p);
    else if constexpr (sizeof(V) % 16 == 0 && alignof(V) >= 16) {
        typedef unsigned int w4 __attribute__((ext_vector_type(4)));
        struct Pieces { w4 q[sizeof(V) / 16]; };
        const Pieces pieces = __builtin_bit_cast(Pieces, v);
#pragma unroll
        for (unsigned k = 0; k < sizeof(V) / 16; ++k) __builtin_nontemporal_store(pieces.q[k], (w4*)p + k);
    }
    else *p = v;
}
// The hint is a compile-time choice of the kernel: chosen at run time inside one kernel, the optimiser folds the two
// branches' stores into ONE plain store and the hint is lost (and fencing them apart with empty asm statements makes
// every wave wait for its store before it may retire: 74 -> 84 us on the row-broadcast add).
template <bool NT, class V> __device__ __forceinline__ void store_sel(V* p, const V& v)
{
    if constexpr (NT) store_nt(p, v);
    else *p = v;
}

// An address that arrives as plain data (read from a table in memory, a field of an argument block copied from one), as
// a pointer the compiler knows to be global memory.  A pointer made from a plain integer is "flat": every access through
// it is a flat_load / flat_store, which counts against the LDS counter too, so the waits before LDS operations and
// barriers then cover the global loads in flight (gemm_tile16_k's register ring degenerated to "wait for everything":
// [8192, 768] x [768, 768] 18.6 -> 22.4 us until its table addresses went through here).
template <class T> __device__ __forceinline__ T* global_ptr(u64 address)
{
    return (T*)(__attribute__((address_space(1))) T*)address;
}

} // namespace aixd
#endif
