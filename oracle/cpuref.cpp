// cpuref.cpp -- CPU oracle for the AIX device operator set.
//
// TEST INFRASTRUCTURE ONLY: loaded by tests, the smoke check and the benchmark's
// cpu_baseline leg; never by the product libraries.
//
// Every function restates the behaviour of the reference CPU device
// (Targets/AIXLib/aixDeviceCPU.cpp, cited per function) including the quirks
// its callers and tests depend on: results written flat from the base pointer,
// per-op loop bounds, accumulators of the element type, strict-greater argmax,
// saturating float->int conversion, software f16/bf16 that round after every op.
//
// What pins each group (see tests/test_oracle_*.py):
//   * all functions, all dtypes      -- differential runs against the reference's
//                                       own DeviceCPU compiled into oracle/_ref
//                                       (tests/test_oracle_vs_ref.py), bit for bit
//   * conversions f16/bf16           -- exhaustive over 65536 patterns vs numpy
//                                       float16 and a bit-level bf16 model
//   * add/sub/mul/div/neg, casts,
//     fill, data movement, argmax    -- numpy closed forms + literals from the
//                                       reference tests (tests/golden/*.json)
//   * sqrt/exp/log/pow               -- correctly rounded value via float64 math
//   * sin/cos/tanh                   -- host libm (the reference calls the same
//                                       routine), bounded against float64
//   * sum/reduceTo/matmul            -- literals, linearity/identity invariants and
//                                       float64 brute force
//   * the accuracy oracles sum_wide,
//     reduce_to_wide, matmul_wide    -- math.fsum / float64 numpy over the logical
//                                       contents of every view kind and every
//                                       destination shape; integers stored as floats
//                                       must come out exact and equal to the
//                                       reference's own sum / reduceTo
//                                       (tests/test_oracle_wide.py)
//   * ulp_hist_f32 (the 2-ulp rule)  -- hand-built pairs: +-0, neighbours across 0
//                                       and across powers of two, NaN against NaN
//                                       and against numbers (same file)
// No function of this file is "parity unpinned".

#include "cpuref.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <thread>
#include <type_traits>
#include <vector>

namespace {

// ---------------------------------------------------------------------------
// 16-bit float storage types.  Arithmetic happens in float and is rounded back
// to 16 bits after every operation (aixFloat16.hpp:104-122, 698-716).
// ---------------------------------------------------------------------------
inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

// IEEE binary16 -> binary32, exact (aixFloat16.hpp:189-199 does it by table).
inline float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t expo = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x3FFu;
    if (expo == 0x1F) return bits_f32(sign | 0x7F800000u | (mant << 13));
    if (expo != 0)    return bits_f32(sign | ((expo + 112u) << 23) | (mant << 13));
    if (mant == 0)    return bits_f32(sign);
    int e = -1;                                  // subnormal: renormalise
    do { mant <<= 1; ++e; } while ((mant & 0x400u) == 0);
    return bits_f32(sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3FFu) << 13));
}

// binary32 -> binary16, round to nearest even, NaN keeps its top payload bits and is
// quieted (aixFloat16.hpp:201-252).
inline uint16_t float_to_half(float f)
{
    const uint32_t u = f32_bits(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t expo = (u >> 23) & 0xFFu;
    const uint32_t mant = u & 0x7FFFFFu;
    if (expo == 0xFF)
        return mant ? (uint16_t)(sign | 0x7C00u | 0x0200u | (mant >> 13)) : (uint16_t)(sign | 0x7C00u);
    const int he = (int)expo - 112;              // re-biased exponent
    if (he >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (he <= 0) {
        if (he < -10) return sign;               // below half of the smallest subnormal
        const uint32_t full = mant | 0x800000u;
        const uint32_t sh = (uint32_t)(14 - he);
        uint16_t r = (uint16_t)(sign | (full >> sh));
        const uint32_t rest = full & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rest > half || (rest == half && (r & 1u))) ++r;
        return r;
    }
    uint16_t r = (uint16_t)(sign | ((uint32_t)he << 10) | (mant >> 13));
    const uint32_t rest = mant & 0x1FFFu;
    if (rest > 0x1000u || (rest == 0x1000u && (r & 1u))) ++r;   // may carry into exponent/inf
    return r;
}

// binary32 -> bfloat16 RNE; NaN is truncated and gets bit 6 set (aixFloat16.hpp:783-805).
inline uint16_t float_to_bf16(float f)
{
    const uint32_t u = f32_bits(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x7FFFFFu)) return (uint16_t)((u >> 16) | 0x40u);
    uint16_t r = (uint16_t)(u >> 16);
    const uint32_t rest = u & 0xFFFFu;
    if (rest > 0x8000u || (rest == 0x8000u && (r & 1u))) ++r;
    return r;
}
inline float bf16_to_float(uint16_t b) { return bits_f32((uint32_t)b << 16); }

struct half_t {
    uint16_t bits{0};
    half_t() = default;
    half_t(float f) : bits(float_to_half(f)) {}
    operator float() const { return half_to_float(bits); }
};
struct bhalf_t {
    uint16_t bits{0};
    bhalf_t() = default;
    bhalf_t(float f) : bits(float_to_bf16(f)) {}
    operator float() const { return bf16_to_float(bits); }
};

template <class T> struct is_half16 : std::false_type {};
template <> struct is_half16<half_t> : std::true_type {};
template <> struct is_half16<bhalf_t> : std::true_type {};
template <class T> constexpr bool is_floatlike_v = std::is_floating_point_v<T> || is_half16<T>::value;

// Arithmetic of the element type.  Integers follow C++ (promote, wrap on store);
// 16-bit floats compute in float then round.
template <class T> inline T t_add(T x, T y) { if constexpr (is_half16<T>::value) return T((float)x + (float)y); else return (T)(x + y); }
template <class T> inline T t_sub(T x, T y) { if constexpr (is_half16<T>::value) return T((float)x - (float)y); else return (T)(x - y); }
template <class T> inline T t_mul(T x, T y) { if constexpr (is_half16<T>::value) return T((float)x * (float)y); else return (T)(x * y); }
template <class T> inline T t_neg(T x)      { if constexpr (is_half16<T>::value) return T(-(float)x);           else return (T)(-x); }
template <class T> inline T t_div(T x, T y)
{
    if constexpr (is_half16<T>::value) return T((float)x / (float)y);
    else if constexpr (std::is_integral_v<T>) {
        // The reference would raise SIGFPE here; the oracle defines both cases so that
        // a test can never crash the process: x/0 -> 0, lowest/-1 -> lowest (wrapped).
        if (y == 0) return 0;
        if constexpr (std::is_signed_v<T>) if (y == (T)-1) return (T)(0 - (std::make_unsigned_t<T>)x);
        return (T)(x / y);
    }
    else return x / y;
}
template <class T> inline bool t_gt(T x, T y) { if constexpr (is_half16<T>::value) return (float)x > (float)y; else return x > y; }
template <class T> inline bool t_lt(T x, T y) { if constexpr (is_half16<T>::value) return (float)x < (float)y; else return x < y; }
template <class T> inline T t_max(T acc, T x) { return t_lt(acc, x) ? x : acc; }          // std::max<T>(acc, x)
template <class T> inline T t_zero() { if constexpr (is_half16<T>::value) return T(0.0f); else return (T)0; }

template <class T> inline T t_lowest()
{
    if constexpr (std::is_same_v<T, half_t>)  { half_t h;  h.bits = 0xFBFF; return h; }
    else if constexpr (std::is_same_v<T, bhalf_t>) { bhalf_t b; b.bits = 0xFF7F; return b; }
    else return std::numeric_limits<T>::lowest();
}

// Value conversion used by copy, fill and the long-double math results
// (aixDeviceCPU.cpp:96-117): float-like -> integer saturates and maps NaN to 0;
// everything else is a plain C++ conversion, 16-bit floats always by way of float.
template <class S, class D> inline D convert_value(S v)
{
    if constexpr (is_floatlike_v<S> && std::is_integral_v<D>) {
        long double x;
        if constexpr (is_half16<S>::value) x = (long double)(float)v; else x = (long double)v;
        if (std::isnan(x)) return 0;
        const long double lo = (long double)std::numeric_limits<D>::lowest();
        const long double hi = (long double)std::numeric_limits<D>::max();
        x = x < lo ? lo : (x > hi ? hi : x);
        return (D)x;
    }
    else if constexpr (is_half16<D>::value) {
        if constexpr (is_half16<S>::value) return D((float)v); else return D((float)v);
    }
    else if constexpr (is_half16<S>::value) return (D)(float)v;
    else return (D)v;
}

// ---------------------------------------------------------------------------
// Index helpers
// ---------------------------------------------------------------------------
// Element position of logical index i under (offset, shape, strides)
// (aixDeviceCPU.cpp:672-683).
inline uint64_t phys(const cpuref_tensor* t, uint64_t i)
{
    uint64_t pos = t->offset;
    for (int d = t->rank - 1; d >= 0; --d) {
        const uint64_t ext = t->shape[d];
        pos += (i % ext) * t->strides[d];
        i /= ext;
    }
    return pos;
}

// phys(t, i) for i = start, start + 1, ...: the same positions, produced by carrying a
// multi-index instead of dividing anew for every element.  With `weight` (one multiplier per
// dimension) it also carries sum(coordinate * weight), which is DstMap::map(i).
struct Cursor {
    const cpuref_tensor* t;
    const uint64_t* weight;
    uint64_t pos, mapped;
    uint64_t idx[CPUREF_MAX_RANK];
    Cursor(const cpuref_tensor* tensor, uint64_t start = 0, const uint64_t* w = nullptr) : t(tensor), weight(w), pos(tensor->offset), mapped(0)
    {
        for (int d = t->rank - 1; d >= 0; --d) {
            const uint64_t ext = t->shape[d];
            idx[d] = ext ? start % ext : 0;
            if (ext) start /= ext;
            pos += idx[d] * t->strides[d];
            if (weight) mapped += idx[d] * weight[d];
        }
    }
    inline void next()
    {
        for (int d = t->rank - 1; d >= 0; --d) {
            if (++idx[d] < t->shape[d]) { pos += t->strides[d]; if (weight) mapped += weight[d]; return; }
            pos -= (t->shape[d] - 1) * t->strides[d];
            if (weight) mapped -= (t->shape[d] - 1) * weight[d];
            idx[d] = 0;
        }
    }
};

// For every source dimension, the multiplier that maps its coordinate into the flat
// index of the (smaller) destination.  Same walk as aixDeviceCPU.cpp:627-649: source
// dims are scanned from the last; a destination dim is consumed when it equals the
// source extent (coordinate kept) or when it is 1 (coordinate dropped); a source dim
// that matches neither leaves the destination cursor where it is.
struct DstMap {
    uint64_t weight[CPUREF_MAX_RANK];
    void build(const uint64_t* dshape, int drank, const uint64_t* sshape, int srank)
    {
        int j = drank - 1;
        uint64_t run = 1;
        for (int i = srank - 1; i >= 0; --i) {
            weight[i] = 0;
            if (j >= 0 && dshape[j] == sshape[i])      { weight[i] = run; run *= dshape[j]; --j; }
            else if (j >= 0 && dshape[j] == 1)         { --j; }
        }
    }
    uint64_t map(uint64_t i, const uint64_t* sshape, int srank) const
    {
        uint64_t r = 0;
        for (int d = srank - 1; d >= 0; --d) { r += (i % sshape[d]) * weight[d]; i /= sshape[d]; }
        return r;
    }
};

template <class F> inline int by_dtype(int dtype, F&& f)
{
    switch (dtype) {
        case CPUREF_F64:  f(double{});   return CPUREF_OK;
        case CPUREF_F32:  f(float{});    return CPUREF_OK;
        case CPUREF_F16:  f(half_t{});   return CPUREF_OK;
        case CPUREF_BF16: f(bhalf_t{});  return CPUREF_OK;
        case CPUREF_I64:  f(int64_t{});  return CPUREF_OK;
        case CPUREF_I32:  f(int32_t{});  return CPUREF_OK;
        case CPUREF_I16:  f(int16_t{});  return CPUREF_OK;
        case CPUREF_I8:   f(int8_t{});   return CPUREF_OK;
        case CPUREF_U8:   f(uint8_t{});  return CPUREF_OK;
        default: return CPUREF_EINVAL;
    }
}

template <class T> inline long double to_ld(T v)
{
    if constexpr (is_half16<T>::value) return (long double)(float)v; else return (long double)v;
}

// One output row of the i, j, k nest reordered to i, k, j: every out[i][j] still starts from
// zero and receives a[i][k] * b[k][j] for k = 0, 1, ... in that order, each product rounded
// before it is added (no contraction), so the result is bit-identical to the nest above; only
// independent outputs are interleaved, which lets the j loop run on vector registers.
template <class T>
__attribute__((target_clones("avx2", "default")))
void matmul_row_ikj(const T* arow, uint64_t as1, const T* b, uint64_t bs0, T* orow, uint64_t n, uint64_t kk)
{
    for (uint64_t j = 0; j < n; ++j) orow[j] = T(0);
    for (uint64_t k = 0; k < kk; ++k) {
        const T x = arow[k * as1];
        const T* brow = b + k * bs0;
        for (uint64_t j = 0; j < n; ++j) orow[j] = orow[j] + x * brow[j];
    }
}

} // namespace

extern "C" {

size_t cpuref_dtype_size(int dtype)
{
    static const size_t sz[CPUREF_DTYPE_COUNT] = {8, 4, 2, 2, 8, 4, 2, 1, 1};
    return (dtype >= 0 && dtype < CPUREF_DTYPE_COUNT) ? sz[dtype] : 0;
}

// add/sub/mul/div: aixDeviceCPU.cpp:28-82 (loop over result.size, dispatch on result
// dtype :747).  pow: :229-242 (loop over a.size, long double powl, converted back).
int cpuref_binary(int op, const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out)
{
    if (op < CPUREF_ADD || op > CPUREF_POW) return CPUREF_EINVAL;
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; const T* pb = (const T*)b->data; T* po = (T*)out->data;
        Cursor ca(a), cb(b);
        if (op == CPUREF_POW) {
            for (uint64_t i = 0; i < a->size; ++i, ca.next(), cb.next())
                po[i] = convert_value<long double, T>(std::pow(to_ld(pa[ca.pos]), to_ld(pb[cb.pos])));
            return;
        }
        for (uint64_t i = 0; i < out->size; ++i, ca.next(), cb.next()) {
            const T x = pa[ca.pos], y = pb[cb.pos];
            po[i] = op == CPUREF_ADD ? t_add(x, y) : op == CPUREF_SUB ? t_sub(x, y)
                  : op == CPUREF_MUL ? t_mul(x, y) : t_div(x, y);
        }
    });
}

// negate :84-94; sqrt/log/exp through long double :154-165, 203-227; sin/cos/tanh call
// the <cmath> overload of the element type :167-201 (float -> sinf, integers -> double
// routine then implicit truncation, 16-bit floats -> float routine then rounding).
// All loop over a.size and dispatch on the result dtype.
int cpuref_unary(int op, const cpuref_tensor* a, const cpuref_tensor* out)
{
    if (op < CPUREF_NEG || op > CPUREF_EXP) return CPUREF_EINVAL;
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; T* po = (T*)out->data;
        Cursor ca(a);
        for (uint64_t i = 0; i < a->size; ++i, ca.next()) {
            const T x = pa[ca.pos];
            switch (op) {
                case CPUREF_NEG:  po[i] = t_neg(x); break;
                case CPUREF_SQRT: po[i] = convert_value<long double, T>(std::sqrt(to_ld(x))); break;
                case CPUREF_LOG:  po[i] = convert_value<long double, T>(std::log(to_ld(x)));  break;
                case CPUREF_EXP:  po[i] = convert_value<long double, T>(std::exp(to_ld(x)));  break;
                default:
                    if constexpr (is_half16<T>::value) {
                        const float f = (float)x;
                        po[i] = T(op == CPUREF_SIN ? std::sin(f) : op == CPUREF_COS ? std::cos(f) : std::tanh(f));
                    } else if constexpr (std::is_integral_v<T>) {
                        const double d = (double)x;
                        po[i] = (T)(op == CPUREF_SIN ? std::sin(d) : op == CPUREF_COS ? std::cos(d) : std::tanh(d));
                    } else {
                        po[i] = op == CPUREF_SIN ? std::sin(x) : op == CPUREF_COS ? std::cos(x) : std::tanh(x);
                    }
            }
        }
    });
}

// aixDeviceCPU.cpp:119-128, 822-842: out.size copies of the converted scalar, flat.
int cpuref_fill(const void* scalar, int scalar_dtype, const cpuref_tensor* out)
{
    int rc = CPUREF_OK;
    int r1 = by_dtype(scalar_dtype, [&](auto stag) {
        using S = decltype(stag);
        S s; std::memcpy(&s, scalar, sizeof(S));
        rc = by_dtype(out->dtype, [&](auto dtag) {
            using D = decltype(dtag);
            const D v = convert_value<S, D>(s);
            D* po = (D*)out->data;
            for (uint64_t i = 0; i < out->size; ++i) po[i] = v;
        });
    });
    return r1 ? r1 : rc;
}

// aixDeviceCPU.cpp:130-138.
int cpuref_fill_min(const cpuref_tensor* out)
{
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        T* po = (T*)out->data; const T v = t_lowest<T>();
        for (uint64_t i = 0; i < out->size; ++i) po[i] = v;
    });
}

// aixDeviceCPU.cpp:407-423, 1107-1127: flat conversion, 9x9.
int cpuref_copy(const void* src, int src_dtype, void* dst, int dst_dtype, uint64_t n)
{
    int rc = CPUREF_OK;
    int r1 = by_dtype(src_dtype, [&](auto stag) {
        using S = decltype(stag);
        rc = by_dtype(dst_dtype, [&](auto dtag) {
            using D = decltype(dtag);
            if constexpr (std::is_same_v<S, D>) { std::memcpy(dst, src, n * sizeof(S)); }
            else {
                const S* ps = (const S*)src; D* pd = (D*)dst;
                for (uint64_t i = 0; i < n; ++i) pd[i] = convert_value<S, D>(ps[i]);
            }
        });
    });
    return r1 ? r1 : rc;
}

// aixDeviceCPU.cpp:425-438 (loop over dst.size, dispatch on src dtype :1150).
int cpuref_contiguous(const cpuref_tensor* src, const cpuref_tensor* dst)
{
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        Cursor cs(src);
        for (uint64_t i = 0; i < dst->size; ++i, cs.next()) pd[i] = ps[cs.pos];
    });
}

// aixDeviceCPU.cpp:391-405: source read flat (contiguous assumed, offset ignored); the
// flat index is split by a's strides, two coordinates swap, and the element lands at the
// dot product with the result's strides.
int cpuref_transpose(const cpuref_tensor* a, const cpuref_tensor* out, uint64_t dim0, uint64_t dim1)
{
    if ((int)dim0 >= a->rank || (int)dim1 >= a->rank) return CPUREF_EINVAL;
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; T* po = (T*)out->data;
        uint64_t coord[CPUREF_MAX_RANK];
        for (uint64_t i = 0; i < a->size; ++i) {
            uint64_t rest = i;
            for (int d = 0; d < a->rank; ++d) { coord[d] = rest / a->strides[d]; rest %= a->strides[d]; }
            std::swap(coord[dim0], coord[dim1]);
            uint64_t pos = 0;
            for (int d = 0; d < a->rank; ++d) pos += coord[d] * out->strides[d];
            po[pos] = pa[i];
        }
    });
}

// aixDeviceCPU.cpp:140-152: accumulator of the element type, index order.
int cpuref_sum(const cpuref_tensor* a, const cpuref_tensor* out)
{
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data;
        T acc = t_zero<T>();
        for (uint64_t i = 0; i < a->size; ++i) acc = t_add(acc, pa[phys(a, i)]);
        *(T*)out->data = acc;
    });
}

// aixDeviceCPU.cpp:244-255.
int cpuref_max(const cpuref_tensor* a, const cpuref_tensor* out)
{
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data;
        T acc = pa[phys(a, 0)];
        for (uint64_t i = 1; i < a->size; ++i) acc = t_max(acc, pa[phys(a, i)]);
        *(T*)out->data = acc;
    });
}

// aixDeviceCPU.cpp:257-273, 1025-1046: int32 result only; first maximum wins.
int cpuref_argmax(const cpuref_tensor* a, const cpuref_tensor* out)
{
    if (out->dtype != CPUREF_I32) return CPUREF_EINVAL;
    return by_dtype(a->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data;
        T best = pa[phys(a, 0)];
        int32_t where = 0;
        for (uint64_t i = 1; i < a->size; ++i) {
            const T x = pa[phys(a, i)];
            if (t_gt(x, best)) { best = x; where = (int32_t)i; }
        }
        *(int32_t*)out->data = where;
    });
}

// aixDeviceCPU.cpp:300-318: one-hot of the first maximum over a.size int32 slots.
int cpuref_argmax_indices(const cpuref_tensor* a, const cpuref_tensor* out)
{
    if (out->dtype != CPUREF_I32) return CPUREF_EINVAL;
    return by_dtype(a->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; int32_t* po = (int32_t*)out->data;
        T best = pa[phys(a, 0)];
        uint64_t where = 0;
        po[0] = 0;
        for (uint64_t i = 1; i < a->size; ++i) {
            po[i] = 0;
            const T x = pa[phys(a, i)];
            if (t_gt(x, best)) { best = x; where = i; }
        }
        po[where] = 1;
    });
}

// aixDeviceCPU.cpp:440-453: dst[map(i)] += src[phys(i)] for all source elements in index
// order; accumulation happens in the destination, in the element type.
int cpuref_reduce_to(const cpuref_tensor* src, const cpuref_tensor* dst)
{
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        DstMap m; m.build(dst->shape, dst->rank, src->shape, src->rank);
        Cursor cs(src, 0, m.weight);
        for (uint64_t i = 0; i < src->size; ++i, cs.next()) {
            T& slot = pd[cs.mapped];
            slot = t_add(slot, ps[cs.pos]);
        }
    });
}

// aixDeviceCPU.cpp:455-466.
int cpuref_max_to(const cpuref_tensor* src, const cpuref_tensor* dst)
{
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        DstMap m; m.build(dst->shape, dst->rank, src->shape, src->rank);
        Cursor cs(src, 0, m.weight);
        for (uint64_t i = 0; i < src->size; ++i, cs.next()) {
            T& slot = pd[cs.mapped];
            slot = t_max(slot, ps[cs.pos]);
        }
    });
}

// aixDeviceCPU.cpp:275-298: the first element seen for a slot always seeds it, later ones
// replace it only when strictly greater; the stored index is
// (flat source index / src.strides[dim]) % src.shape[dim]  -- physical strides on purpose.
int cpuref_argmax_to(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim)
{
    if (dst->dtype != CPUREF_I32 || (int)dim >= src->rank) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; int32_t* pd = (int32_t*)dst->data;
        std::vector<T> best(dst->size);
        std::vector<char> seen(dst->size, 0);
        DstMap m; m.build(dst->shape, dst->rank, src->shape, src->rank);
        for (uint64_t i = 0; i < src->size; ++i) {
            const uint64_t s = m.map(i, src->shape, src->rank);
            const T x = ps[phys(src, i)];
            if (!seen[s] || t_gt(x, best[s])) {
                seen[s] = 1; best[s] = x;
                pd[s] = (int32_t)((i / src->strides[dim]) % src->shape[dim]);
            }
        }
    });
}

// aixDeviceCPU.cpp:320-360: winners are remembered by flat logical source index and a 1 is
// scattered to that position of the (pre-zeroed, contiguous) destination.
int cpuref_argmax_indices_to(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim)
{
    if (dst->dtype != CPUREF_I32 || (int)dim >= dst->rank) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; int32_t* pd = (int32_t*)dst->data;
        uint64_t rshape[CPUREF_MAX_RANK]; uint64_t slots = 1;
        for (int d = 0; d < dst->rank; ++d) { rshape[d] = (d == (int)dim) ? 1 : dst->shape[d]; slots *= rshape[d]; }
        std::vector<T> best(slots);
        std::vector<char> seen(slots, 0);
        std::vector<uint64_t> where(slots, 0);
        DstMap m; m.build(rshape, dst->rank, src->shape, src->rank);
        Cursor cs(src, 0, m.weight);
        for (uint64_t i = 0; i < src->size; ++i, cs.next()) {
            const uint64_t s = cs.mapped;
            const T x = ps[cs.pos];
            if (!seen[s] || t_gt(x, best[s])) { seen[s] = 1; best[s] = x; where[s] = i; }
        }
        for (uint64_t s = 0; s < slots; ++s) pd[(int32_t)where[s]] = 1;
    });
}

// aixDeviceCPU.cpp:362-389: i, j, k loops; accumulator of the element type starting at 0;
// operands addressed through their views, result row-major from base.
int cpuref_matmul(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out)
{
    return cpuref_matmul_rows(a, b, out, 1);
}

int cpuref_matmul_rows(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads)
{
    if (a->rank != 2 || b->rank != 2) return CPUREF_EINVAL;
    if (out->dtype == CPUREF_F32 || out->dtype == CPUREF_F64) {
        // f32 / f64: the reordered nest.  B is first copied to a dense [K, N] array if its rows are not unit-stride.
        return by_dtype(out->dtype, [&](auto tag) {
            using T = decltype(tag);
            if constexpr (std::is_same_v<T, float> || std::is_same_v<T, double>) {
                const uint64_t m = a->shape[0], n = b->shape[1], kk = a->shape[1];
                const T* pa = (const T*)a->data + a->offset; T* po = (T*)out->data;
                const T* pb = (const T*)b->data + b->offset;
                uint64_t bs0 = b->strides[0];
                std::vector<T> dense;
                if (b->strides[1] != 1 && n > 1) {
                    dense.resize(kk * n);
                    for (uint64_t k = 0; k < kk; ++k) for (uint64_t j = 0; j < n; ++j) dense[k * n + j] = pb[k * b->strides[0] + j * b->strides[1]];
                    pb = dense.data(); bs0 = n;
                }
                auto rows = [&](uint64_t r0, uint64_t r1) {
                    for (uint64_t i = r0; i < r1; ++i) matmul_row_ikj<T>(pa + i * a->strides[0], a->strides[1], pb, bs0, po + i * n, n, kk);
                };
                if (threads <= 1 || m < 2) { rows(0, m); return; }
                std::vector<std::thread> pool;
                const uint64_t per = (m + threads - 1) / threads;
                for (int t = 0; t < threads; ++t) {
                    const uint64_t r0 = std::min<uint64_t>(m, t * per), r1 = std::min<uint64_t>(m, r0 + per);
                    if (r0 < r1) pool.emplace_back(rows, r0, r1);
                }
                for (auto& th : pool) th.join();
            }
        });
    }
    return by_dtype(out->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; const T* pb = (const T*)b->data; T* po = (T*)out->data;
        const uint64_t m = a->shape[0], n = b->shape[1], kk = a->shape[1];
        auto rows = [&](uint64_t r0, uint64_t r1) {
            for (uint64_t i = r0; i < r1; ++i)
                for (uint64_t j = 0; j < n; ++j) {
                    T acc = t_zero<T>();
                    for (uint64_t k = 0; k < kk; ++k)
                        acc = t_add(acc, t_mul(pa[phys(a, i * kk + k)], pb[phys(b, k * n + j)]));
                    po[i * n + j] = acc;
                }
        };
        if (threads <= 1) { rows(0, m); return; }
        std::vector<std::thread> pool;
        const uint64_t per = (m + threads - 1) / threads;
        for (int t = 0; t < threads; ++t) {
            const uint64_t r0 = std::min<uint64_t>(m, t * per), r1 = std::min<uint64_t>(m, r0 + per);
            if (r0 < r1) pool.emplace_back(rows, r0, r1);
        }
        for (auto& th : pool) th.join();
    });
}

// aixDeviceCPU.cpp:468-496: iterate the source; coordinates are taken in the sliced shape
// and scaled by the destination's strides.
int cpuref_slice_set(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim,
                     uint64_t start, uint64_t end, uint64_t step, int honor_dst_offset)
{
    if ((int)dim >= dst->rank || step == 0) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        uint64_t sshape[CPUREF_MAX_RANK];
        for (int d = 0; d < dst->rank; ++d) sshape[d] = dst->shape[d];
        sshape[dim] = (end - start + step - 1) / step;
        for (uint64_t i = 0; i < src->size; ++i) {
            uint64_t rest = i, pos = honor_dst_offset ? dst->offset : 0;
            for (int d = dst->rank - 1; d >= 0; --d) {
                const uint64_t c = rest % sshape[d]; rest /= sshape[d];
                pos += (d == (int)dim ? start + c * step : c) * dst->strides[d];
            }
            pd[pos] = ps[phys(src, i)];
        }
    });
}

// aixDeviceCPU.cpp:566-622: masks on the last two dims; both sides addressed through
// their views; keep = col <= row + diagonal (tril) or col >= row + diagonal (triu).
static int tri_impl(const cpuref_tensor* src, const cpuref_tensor* dst, int64_t diagonal, bool lower)
{
    if (src->rank < 2) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        const uint64_t rows = src->shape[src->rank - 2], cols = src->shape[src->rank - 1];
        for (uint64_t i = 0; i < dst->size; ++i) {
            const int64_t r = (int64_t)((i / cols) % rows), c = (int64_t)(i % cols);
            const bool zero = lower ? (c > r + diagonal) : (c < r + diagonal);
            pd[phys(dst, i)] = zero ? t_zero<T>() : ps[phys(src, i)];
        }
    });
}
int cpuref_tril(const cpuref_tensor* src, const cpuref_tensor* dst, int64_t diagonal) { return tri_impl(src, dst, diagonal, true); }
int cpuref_triu(const cpuref_tensor* src, const cpuref_tensor* dst, int64_t diagonal) { return tri_impl(src, dst, diagonal, false); }

static inline int64_t index_at(const cpuref_tensor* idx, uint64_t k, int strided)
{
    return ((const int32_t*)idx->data)[strided ? phys(idx, k) : k];
}

// The reference only asserts the range of the indices on the host (aixCore.hpp:1242, 1640-1650) and then reads or
// writes out of bounds.  The oracle refuses such a call before it touches anything.
static bool indices_in_range(const cpuref_tensor* idx, int strided, uint64_t extent)
{
    for (uint64_t k = 0; k < idx->size; ++k) {
        const int64_t v = index_at(idx, k, strided);
        if (v < 0 || (uint64_t)v >= extent) return false;
    }
    return true;
}

// aixDeviceCPU.cpp:498-530: iterate dst.size; dst contiguous from base.
int cpuref_index_select(const cpuref_tensor* src, const cpuref_tensor* dst,
                        const cpuref_tensor* indices, uint64_t dim, int strided_indices)
{
    if (indices->dtype != CPUREF_I32) return CPUREF_EINVAL;
    if (!indices_in_range(indices, strided_indices, src->rank ? src->shape[dim] : 1)) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        uint64_t inner = 1;
        for (int d = (int)dim + 1; d < src->rank; ++d) inner *= src->shape[d];
        const uint64_t span = src->rank ? src->shape[dim] * inner : 0, ni = indices->size;
        for (uint64_t i = 0; i < dst->size; ++i) {
            const uint64_t e = i % inner, k = (i / inner) % ni, o = i / (ni * inner);
            const uint64_t from = o * span + (uint64_t)index_at(indices, k, strided_indices) * inner + e;
            pd[o * ni * inner + k * inner + e] = ps[phys(src, from)];
        }
    });
}

// aixDeviceCPU.cpp:532-564: iterate src.size; dst addressed flat from base.
int cpuref_index_add(const cpuref_tensor* src, const cpuref_tensor* dst,
                     const cpuref_tensor* indices, uint64_t dim, int strided_indices)
{
    if (indices->dtype != CPUREF_I32) return CPUREF_EINVAL;
    if (!indices_in_range(indices, strided_indices, dst->rank ? dst->shape[dim] : 1)) return CPUREF_EINVAL;
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data; T* pd = (T*)dst->data;
        uint64_t inner = 1;
        for (int d = (int)dim + 1; d < dst->rank; ++d) inner *= dst->shape[d];
        const uint64_t span = dst->rank ? dst->shape[dim] * inner : 0, ni = indices->size;
        for (uint64_t i = 0; i < src->size; ++i) {
            const uint64_t e = i % inner, k = (i / inner) % ni, o = i / (ni * inner);
            T& slot = pd[o * span + (uint64_t)index_at(indices, k, strided_indices) * inner + e];
            slot = t_add(slot, ps[phys(src, o * ni * inner + k * inner + e)]);
        }
    });
}

// ---------------------------------------------------------------------------
// Accuracy oracles
// ---------------------------------------------------------------------------
int cpuref_sum_wide(const cpuref_tensor* a, double* sum_out, double* abs_sum_out)
{
    return by_dtype(a->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data;
        long double s = 0, sa = 0;
        for (uint64_t i = 0; i < a->size; ++i) { const long double x = to_ld(pa[phys(a, i)]); s += x; sa += std::fabs(x); }
        if (sum_out) *sum_out = (double)s;
        if (abs_sum_out) *abs_sum_out = (double)sa;
    });
}

int cpuref_reduce_to_wide(const cpuref_tensor* src, const cpuref_tensor* dst_like, double* dst64, double* abs64)
{
    return by_dtype(src->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* ps = (const T*)src->data;
        DstMap m; m.build(dst_like->shape, dst_like->rank, src->shape, src->rank);
        for (uint64_t i = 0; i < src->size; ++i) {
            const uint64_t s = m.map(i, src->shape, src->rank);
            const double x = (double)to_ld(ps[phys(src, i)]);
            dst64[s] += x;
            if (abs64) abs64[s] += std::fabs(x);
        }
    });
}

int cpuref_matmul_stack(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads)
{
    if (a->rank < 2 || a->rank != b->rank || a->rank != out->rank) return CPUREF_EINVAL;
    const int nb = a->rank - 2;
    uint64_t count = 1;
    for (int d = 0; d < nb; ++d) {
        if (a->shape[d] != b->shape[d] || a->shape[d] != out->shape[d]) return CPUREF_EINVAL;
        count *= a->shape[d];
    }
    auto matrix = [nb](const cpuref_tensor* t) {
        cpuref_tensor m = *t;
        m.rank = 2;
        m.shape[0] = t->shape[nb]; m.shape[1] = t->shape[nb + 1];
        m.strides[0] = t->strides[nb]; m.strides[1] = t->strides[nb + 1];
        m.size = m.shape[0] * m.shape[1];
        return m;
    };
    cpuref_tensor a2 = matrix(a), b2 = matrix(b), o2 = matrix(out);
    if (a2.shape[1] != b2.shape[0]) return CPUREF_EINVAL;
    const uint64_t per = a2.shape[0] * b2.shape[1] * cpuref_dtype_size(out->dtype);
    o2.offset = 0; o2.strides[0] = b2.shape[1]; o2.strides[1] = 1;
    for (uint64_t i = 0; i < count; ++i) {
        uint64_t rest = i, oa = a->offset, ob = b->offset;
        for (int d = nb - 1; d >= 0; --d) {
            const uint64_t c = rest % a->shape[d];
            rest /= a->shape[d];
            oa += c * a->strides[d]; ob += c * b->strides[d];
        }
        a2.offset = oa; b2.offset = ob;
        o2.data = (char*)out->data + i * per;
        const int rc = cpuref_matmul_rows(&a2, &b2, &o2, threads);
        if (rc != CPUREF_OK) return rc;
    }
    return CPUREF_OK;
}

int cpuref_matmul_wide(const cpuref_tensor* a, const cpuref_tensor* b, double* out64, double* abs64, int threads)
{
    if (a->rank != 2 || b->rank != 2 || a->dtype != b->dtype) return CPUREF_EINVAL;
    return by_dtype(a->dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* pa = (const T*)a->data; const T* pb = (const T*)b->data;
        const uint64_t m = a->shape[0], n = b->shape[1], kk = a->shape[1];
        // Gather both operands once into dense double arrays (B transposed) so the inner
        // loop is a unit-stride dot product.
        std::vector<double> da(m * kk), dbt(n * kk);
        for (uint64_t i = 0; i < m; ++i) for (uint64_t k = 0; k < kk; ++k) da[i * kk + k] = (double)to_ld(pa[phys(a, i * kk + k)]);
        for (uint64_t k = 0; k < kk; ++k) for (uint64_t j = 0; j < n; ++j) dbt[j * kk + k] = (double)to_ld(pb[phys(b, k * n + j)]);
        auto rows = [&](uint64_t r0, uint64_t r1) {
            for (uint64_t i = r0; i < r1; ++i)
                for (uint64_t j = 0; j < n; ++j) {
                    const double* x = &da[i * kk]; const double* y = &dbt[j * kk];
                    double s = 0, sa = 0;
                    for (uint64_t k = 0; k < kk; ++k) { const double p = x[k] * y[k]; s += p; sa += std::fabs(p); }
                    out64[i * n + j] = s;
                    if (abs64) abs64[i * n + j] = sa;
                }
        };
        if (threads <= 1) { rows(0, m); return; }
        std::vector<std::thread> pool;
        const uint64_t per = (m + threads - 1) / threads;
        for (int t = 0; t < threads; ++t) {
            const uint64_t r0 = std::min<uint64_t>(m, t * per), r1 = std::min<uint64_t>(m, r0 + per);
            if (r0 < r1) pool.emplace_back(rows, r0, r1);
        }
        for (auto& th : pool) th.join();
    });
}

// cpuref_matmul / cpuref_matmul_stack with the products of every result element added exactly (cpuref_matmul_wide) and
// rounded ONCE to the element type: what a device that accumulates 16-bit products in a wide type computes, as opposed to
// the reference's running sum in the element type (aixDeviceCPU.cpp:362-389).  Rank 2 or stacks of matrices.
int cpuref_matmul_stack_wide(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads)
{
    if (a->rank < 2 || a->rank != b->rank || a->rank != out->rank || a->dtype != b->dtype || a->dtype != out->dtype) return CPUREF_EINVAL;
    const int nb = a->rank - 2;
    uint64_t count = 1;
    for (int d = 0; d < nb; ++d) {
        if (a->shape[d] != b->shape[d] || a->shape[d] != out->shape[d]) return CPUREF_EINVAL;
        count *= a->shape[d];
    }
    auto matrix = [nb](const cpuref_tensor* t) {
        cpuref_tensor m = *t;
        m.rank = 2;
        m.shape[0] = t->shape[nb]; m.shape[1] = t->shape[nb + 1];
        m.strides[0] = t->strides[nb]; m.strides[1] = t->strides[nb + 1];
        m.size = m.shape[0] * m.shape[1];
        return m;
    };
    cpuref_tensor a2 = matrix(a), b2 = matrix(b);
    if (a2.shape[1] != b2.shape[0]) return CPUREF_EINVAL;
    const uint64_t mn = a2.shape[0] * b2.shape[1], per = mn * cpuref_dtype_size(out->dtype);
    std::vector<double> exact(mn);
    for (uint64_t i = 0; i < count; ++i) {
        uint64_t rest = i, oa = a->offset, ob = b->offset;
        for (int d = nb - 1; d >= 0; --d) {
            const uint64_t c = rest % a->shape[d];
            rest /= a->shape[d];
            oa += c * a->strides[d]; ob += c * b->strides[d];
        }
        a2.offset = oa; b2.offset = ob;
        int rc = cpuref_matmul_wide(&a2, &b2, exact.data(), nullptr, threads);
        if (rc == CPUREF_OK) rc = cpuref_copy(exact.data(), CPUREF_F64, (char*)out->data + i * per, out->dtype, mn);     // results are written densely
        if (rc != CPUREF_OK) return rc;
    }
    return CPUREF_OK;
}

uint64_t cpuref_ulp_hist_f32(const float* x, const float* y, uint64_t n, uint64_t* hist, int nbins)
{
    auto ordered = [](float f) -> int64_t {       // monotone map float -> integer line
        const uint32_t u = f32_bits(f);
        return (u & 0x80000000u) ? -(int64_t)(u & 0x7FFFFFFFu) : (int64_t)u;
    };
    uint64_t worst = 0;
    for (uint64_t i = 0; i < n; ++i) {
        uint64_t d;
        const bool nx = std::isnan(x[i]), ny = std::isnan(y[i]);
        if (nx || ny) d = (nx && ny) ? 0 : (uint64_t)(nbins - 1);
        else { const int64_t a = ordered(x[i]), b = ordered(y[i]); d = (uint64_t)(a > b ? a - b : b - a); }
        worst = std::max(worst, d);
        if (hist && nbins > 0) hist[std::min<uint64_t>(d, (uint64_t)nbins - 1)]++;
    }
    return worst;
}

} // extern "C"
