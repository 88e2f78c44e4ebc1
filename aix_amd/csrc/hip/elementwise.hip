// elementwise.hip -- binary / unary / pow, fill, fillMin and converting copy for all nine
// element types.  HBM-bound: every kernel moves 16 bytes per lane per access where the views
// allow it.
//
// Three shapes of kernel, chosen on the host from the jointly collapsed iteration space:
//   flat    all operands unit-stride (or a broadcast scalar) and 16-byte aligned: 4 independent
//           16-byte loads per operand per lane in flight, grid-stride over tiles;
//   rows    innermost dim unit-stride-or-broadcast for every operand (row/column broadcast,
//           sliced rows): one 16-byte chunk per lane, outer coordinates decomposed once per chunk;
//   gather  anything else (transposed operands): one element per lane, full decomposition.
// Results are written contiguously from out->data (aixDeviceCPU.cpp:33-39, 87-93).

#include "common.hpp"

using namespace aixd;
using namespace aixk;

namespace {

template <int OP, class T> struct Bin {
    static __device__ __forceinline__ T run(T a, T b)
    {
        if constexpr (OP == AIXK_ADD) return e_add(a, b);
        else if constexpr (OP == AIXK_SUB) return e_sub(a, b);
        else if constexpr (OP == AIXK_MUL) return e_mul(a, b);
        else if constexpr (OP == AIXK_DIV) return e_div(a, b);
        else return e_pow(a, b);
    }
};
template <int OP, class T> struct Un {
    static __device__ __forceinline__ T run(T a)
    {
        if constexpr (OP == AIXK_NEG) return e_neg(a);
        else return e_math<OP>(a);            // AIXK_SQRT..AIXK_EXP == M_SQRT..M_EXP
    }
};
static_assert(AIXK_SQRT == M_SQRT && AIXK_SIN == M_SIN && AIXK_COS == M_COS && AIXK_TANH == M_TANH &&
              AIXK_LOG == M_LOG && AIXK_EXP == M_EXP, "unary op codes must match the math selectors");

// ---- flat ------------------------------------------------------------------------------------
// NIN = 1 or 2 inputs.  AS / BS: that input is a single broadcast element.  One 16-byte vector per
// operand per lane and one workgroup per 256 vectors: many small groups in flight overlap their
// load and compute phases better than a long per-lane loop (measured on the fused chain).
// `out` may be one of the inputs (in-place operators, aixCore.hpp:1447, 1451), so in these three kernels it
// and the inputs carry no restrict qualifier: every lane reads its elements before it writes the same addresses.
template <class F, class T, int NIN, bool AS, bool BS, bool NT>
__global__ __launch_bounds__(kBlock) void ew_flat(const T* a, const T* b, T* out, u64 n)
{
    typedef typename vec16<T>::type V;
    constexpr int VEC = vec16<T>::n;
    const u64 nvec = n / VEC;
    const V* A = (const V*)a;
    const V* B = (const V*)b;
    V* O = (V*)out;
    T sa = zero<T>(), sb = zero<T>();
    if constexpr (AS) sa = a[0];
    if constexpr (NIN == 2 && BS) sb = b[0];
    for (u64 v = (u64)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += (u64)gridDim.x * kBlock) {
        V ra, rb, r;
        if constexpr (!AS) ra = A[v];
        if constexpr (NIN == 2 && !BS) rb = B[v];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const T x = AS ? sa : ra.v[e];
            if constexpr (NIN == 2) { const T y = BS ? sb : rb.v[e]; r.v[e] = F::run(x, y); }
            else r.v[e] = F::run(x);
        }
        store_sel<NT>(O + v, r);
    }
    // tail (< VEC elements) by the first lanes of block 0
    const u64 done = nvec * VEC;
    if (blockIdx.x == 0 && done + threadIdx.x < n) {
        const u64 i = done + threadIdx.x;
        const T x = AS ? sa : a[i];
        if constexpr (NIN == 2) { const T y = BS ? sb : b[i]; out[i] = F::run(x, y); }
        else out[i] = F::run(x);
    }
}

// ---- rows ------------------------------------------------------------------------------------
// Space dims: [outer..., inner]; inner strides are 1 or 0 for inputs.  `chunks` = inner / VEC.
template <class F, class T, int NIN, class IDX, bool NT>
__global__ __launch_bounds__(kBlock) void ew_rows(const T* a, const T* b,
                                                  T* out, Space<2> sp, u64 total_chunks, IDX chunks)
{
    typedef typename vec16<T>::type V;
    constexpr int VEC = vec16<T>::n;
    const int inner = sp.rank - 1;
    for (u64 c = (u64)blockIdx.x * kBlock + threadIdx.x; c < total_chunks; c += (u64)gridDim.x * kBlock) {
        IDX row = (IDX)(c / chunks);
        const IDX col = (IDX)(c - (u64)row * chunks) * VEC;
        u64 pa = sp.offset[0], pb = sp.offset[1];
        for (int d = inner - 1; d >= 0; --d) {
            const IDX ext = (IDX)sp.shape[d];
            const IDX q = row / ext, r = row - q * ext;
            pa += (u64)r * sp.stride[0][d];
            if constexpr (NIN == 2) pb += (u64)r * sp.stride[1][d];
            row = q;
        }
        const bool a_b = sp.stride[0][inner] == 0, b_b = NIN == 2 && sp.stride[1][inner] == 0;
        V va = *row_vec_ptr<T, VEC>(a + pa, col, a_b), vb, vr;
        if constexpr (NIN == 2) vb = *row_vec_ptr<T, VEC>(b + pb, col, b_b);
        va = row_vec_fix<T, VEC>(va, a + pa, a_b);
        if constexpr (NIN == 2) vb = row_vec_fix<T, VEC>(vb, b + pb, b_b);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if constexpr (NIN == 2) vr.v[e] = F::run(va.v[e], vb.v[e]);
            else vr.v[e] = F::run(va.v[e]);
        }
        store_sel<NT>((V*)(out + c * VEC), vr);
    }
}

// [rows, cols] operands (a dense matrix with a row or a column vector, a transposed-free pair of matrices with their own
// row pitches): one vector per lane, no loop, the row strides as plain kernel arguments -- no Space to read, one
// division.  Measured on x[8192, 8192] + v[8192] (f32, non-temporal stores): 74 us against 84-90 us for ew_rows.
template <class F, class T, int NIN, bool NT>
__global__ __launch_bounds__(kBlock) void ew_rows2(const T* a, const T* b, T* out, u64 rs0, u64 rs1, u32 total_chunks, u32 chunks, u32 flags)
{
    typedef typename vec16<T>::type V;
    constexpr int VEC = vec16<T>::n;
    const u32 c = blockIdx.x * kBlock + threadIdx.x;
    if (c >= total_chunks) return;
    const u32 row = c / chunks, col = (c - row * chunks) * VEC;
    const T* ra = a + (u64)row * rs0;
    const T* rb = NIN == 2 ? b + (u64)row * rs1 : ra;
    const bool fa = flags & 1u, fb = NIN == 2 && (flags & 2u);
    V va = *row_vec_ptr<T, VEC>(ra, col, fa), vb, vr;
    if constexpr (NIN == 2) vb = *row_vec_ptr<T, VEC>(rb, col, fb);
    va = row_vec_fix<T, VEC>(va, ra, fa);
    if constexpr (NIN == 2) vb = row_vec_fix<T, VEC>(vb, rb, fb);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        if constexpr (NIN == 2) vr.v[e] = F::run(va.v[e], vb.v[e]);
        else vr.v[e] = F::run(va.v[e]);
    }
    store_sel<NT>((V*)(out + (u64)c * VEC), vr);
}

// ---- gather ----------------------------------------------------------------------------------
template <class F, class T, int NIN, class IDX>
__global__ __launch_bounds__(kBlock) void ew_gather(const T* a, const T* b,
                                                    T* out, Space<2> sp, u64 n)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) {
        IDX rest = (IDX)i;
        u64 pa = sp.offset[0], pb = sp.offset[1];
        for (int d = sp.rank - 1; d >= 0; --d) {
            const IDX ext = (IDX)sp.shape[d];
            const IDX q = rest / ext, r = rest - q * ext;
            pa += (u64)r * sp.stride[0][d];
            if constexpr (NIN == 2) pb += (u64)r * sp.stride[1][d];
            rest = q;
        }
        if constexpr (NIN == 2) out[i] = F::run(a[pa], b[pb]);
        else out[i] = F::run(a[pa]);
    }
}

// Host-side routing shared by binary and unary.
template <class F, class T, int NIN>
int launch_ew(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint64_t n)
{
    if (n == 0) return AIXK_OK;
    constexpr int VEC = vec16<T>::n;
    const uint64_t* strides[2] = {a->strides, NIN == 2 ? b->strides : a->strides};
    const uint64_t offsets[2] = {a->offset, NIN == 2 ? b->offset : a->offset};
    Space<2> sp;
    if (!collapse<2>(a->rank, a->shape, strides, offsets, &sp))
        return fail(AIXK_EINVAL, "elementwise: view does not collapse to %d dims", kMaxDims);
    const T* pa = (const T*)a->data;
    const T* pb = NIN == 2 ? (const T*)b->data : pa;
    T* po = (T*)out->data;
    const bool nt = streams_out(n * sizeof(T));       // a large result leaves through non-temporal stores
    // flat: rank 0 (single element / all-broadcast) or rank 1 with strides in {0,1}
    const bool flat_shape = sp.rank == 0 || (sp.rank == 1 && sp.stride[0][0] <= 1 && sp.stride[1][0] <= 1);
    if (flat_shape) {
        const int as = sp.rank == 0 ? (n > 1) : sp.stride[0][0] == 0;
        const int bs = sp.rank == 0 ? (n > 1) : sp.stride[1][0] == 0;
        const T* qa = pa + sp.offset[0];
        const T* qb = pb + sp.offset[1];
        if ((as || aligned16(qa)) && (bs || aligned16(qb)) && aligned16(po)) {
            const unsigned grid = grid_for(n / VEC + 1, kBlock, 1u << 22);
            const int fa = sp.rank == 0 ? 0 : as, fb = (NIN == 2 && sp.rank != 0) ? bs : 0;
#define AIXK_FLAT(AS_, BS_) do { if (nt) hipLaunchKernelGGL((ew_flat<F, T, NIN, AS_, BS_, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, qa, qb, po, (u64)n); \
                                 else hipLaunchKernelGGL((ew_flat<F, T, NIN, AS_, BS_, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, qa, qb, po, (u64)n); } while (0)
            if (fa && fb) AIXK_FLAT(true, true);
            else if (fa) AIXK_FLAT(true, false);
            else if (fb) AIXK_FLAT(false, true);
            else AIXK_FLAT(false, false);
#undef AIXK_FLAT
            AIXK_HIP(hipGetLastError());
            return AIXK_OK;
        }
    }
    const bool small = n < (1ull << 31) && view_extent(a) < (1ull << 31) && (NIN == 1 || view_extent(b) < (1ull << 31));
    // rows: inner dim unit-or-broadcast for all, inner extent and row starts multiples of VEC
    if (sp.rank >= 2 && aligned16(po)) {
        const int in = sp.rank - 1;
        bool ok = sp.shape[in] % VEC == 0;
        for (int o = 0; o < NIN && ok; ++o) {
            const T* base = (o == 0 ? pa : pb);
            if (sp.stride[o][in] > 1) ok = false;
            if (sp.stride[o][in] == 1) {
                if (!aligned16(base + sp.offset[o])) ok = false;
                for (int d = 0; d < in; ++d) if (sp.stride[o][d] % VEC) ok = false;
            }
        }
        if (ok) {
            const uint64_t chunks = sp.shape[in] / VEC, total = n / VEC;
            const unsigned grid = grid_for(total, kBlock, 1u << 22);
            const u32 flags = (sp.stride[0][in] == 0 ? 1u : 0u) | (NIN == 2 && sp.stride[1][in] == 0 ? 2u : 0u) | (sp.rank == 2 ? 4u : 0u);
            const u64 rs0 = sp.stride[0][0], rs1 = sp.stride[1][0];
            if (sp.rank == 2 && small && total <= ((uint64_t)1 << 30)) {
                const T* qa = pa + sp.offset[0];
                const T* qb = pb + sp.offset[1];
                const unsigned g2 = (unsigned)((total + kBlock - 1) / kBlock);
                if (nt) hipLaunchKernelGGL((ew_rows2<F, T, NIN, true>), dim3(g2), dim3(kBlock), 0, ctx->stream, qa, qb, po, rs0, rs1, (u32)total, (u32)chunks, flags);
                else hipLaunchKernelGGL((ew_rows2<F, T, NIN, false>), dim3(g2), dim3(kBlock), 0, ctx->stream, qa, qb, po, rs0, rs1, (u32)total, (u32)chunks, flags);
                AIXK_HIP(hipGetLastError());
                return AIXK_OK;
            }
#define AIXK_ROWS(IDX_, NT_) hipLaunchKernelGGL((ew_rows<F, T, NIN, IDX_, NT_>), dim3(grid), dim3(kBlock), 0, ctx->stream, pa, pb, po, sp, (u64)total, (IDX_)chunks)
            if (small) { if (nt) AIXK_ROWS(u32, true); else AIXK_ROWS(u32, false); }
            else { if (nt) AIXK_ROWS(u64, true); else AIXK_ROWS(u64, false); }
#undef AIXK_ROWS
            AIXK_HIP(hipGetLastError());
            return AIXK_OK;
        }
    }
    const unsigned grid = grid_for(n, kBlock, 1u << 22);
    if (small)
        hipLaunchKernelGGL((ew_gather<F, T, NIN, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, pa, pb, po, sp, (u64)n);
    else
        hipLaunchKernelGGL((ew_gather<F, T, NIN, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, pa, pb, po, sp, (u64)n);
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

template <int OP> int binary_op(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint64_t n)
{
    return by_dtype(out->dtype, [&](auto tag) { typedef decltype(tag) T; return launch_ew<Bin<OP, T>, T, 2>(ctx, a, b, out, n); });
}
template <int OP> int unary_op(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* out, uint64_t n)
{
    return by_dtype(out->dtype, [&](auto tag) { typedef decltype(tag) T; return launch_ew<Un<OP, T>, T, 1>(ctx, a, nullptr, out, n); });
}

// ---- fill / cast -----------------------------------------------------------------------------
// One lane converts K elements where K*min(sizeof) == 16 bytes.
template <class T, int K> struct alignas(16) pack { T v[K]; };

template <class S, class D, bool NT>
__global__ __launch_bounds__(kBlock) void cast_flat(const S* __restrict__ src, D* __restrict__ dst, u64 n)
{
    constexpr int K = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));
    typedef pack<S, K> PS;
    typedef pack<D, K> PD;
    const u64 nchunk = n / K;
    for (u64 c = (u64)blockIdx.x * kBlock + threadIdx.x; c < nchunk; c += (u64)gridDim.x * kBlock) {
        const PS in = ((const PS*)src)[c];
        PD o;
#pragma unroll
        for (int e = 0; e < K; ++e) o.v[e] = convert<S, D>(in.v[e]);
        store_sel<NT>((PD*)dst + c, o);
    }
    const u64 done = nchunk * K;
    if (blockIdx.x == 0 && done + threadIdx.x < n) dst[done + threadIdx.x] = convert<S, D>(src[done + threadIdx.x]);
}
template <class S, class D>
__global__ __launch_bounds__(kBlock) void cast_any(const S* __restrict__ src, D* __restrict__ dst, u64 n)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) dst[i] = convert<S, D>(src[i]);
}

// The fill scalar travels by value in its source type and is converted on the device, so the
// conversion rules are the device's own (the same code the converting copy uses).
template <class S, class D> __global__ void fill_cvt(D* __restrict__ out, S value, u64 n)
{
    const D v = convert<S, D>(value);
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) out[i] = v;
}
template <class S, class D> __global__ __launch_bounds__(kBlock) void fill_cvt_vec(D* __restrict__ out, S value, u64 n)
{
    typedef typename vec16<D>::type V;
    constexpr int VEC = vec16<D>::n;
    const D s = convert<S, D>(value);
    V v;
#pragma unroll
    for (int e = 0; e < VEC; ++e) v.v[e] = s;
    const u64 nvec = n / VEC;
    V* O = (V*)out;
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (u64)gridDim.x * kBlock) O[i] = v;
    const u64 done = nvec * VEC;
    if (blockIdx.x == 0 && done + threadIdx.x < n) out[done + threadIdx.x] = s;
}

// Small fills of one launch (aixk_fill_many): workgroup k writes item k.
struct FillItems { static constexpr int kMost = 32; u64 dst[kMost]; u64 bits[kMost]; u32 n[kMost]; u32 esz[kMost]; };
__global__ __launch_bounds__(kBlock) void fill_items_k(FillItems it)
{
    const u32 k = blockIdx.x, n = it.n[k], esz = it.esz[k];
    const u64 bits = it.bits[k];
    for (u32 i = threadIdx.x; i < n; i += kBlock) {
        if (esz == 1) global_ptr<u8>(it.dst[k])[i] = (u8)bits;
        else if (esz == 2) global_ptr<u16>(it.dst[k])[i] = (u16)bits;
        else if (esz == 4) global_ptr<u32>(it.dst[k])[i] = (u32)bits;
        else global_ptr<u64>(it.dst[k])[i] = bits;
    }
}

template <class T> __global__ void fill_min_k(T* __restrict__ out, u64 n)
{
    const T v = lowest<T>();
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) out[i] = v;
}


} // namespace

extern "C" {

int32_t aixk_binary(aixk_ctx* ctx, int op, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(b) && valid_tensor(out), "binary: bad operand descriptor");
    AIXK_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype, "binary: operands must have the result's element type");
    AIXK_REQUIRE(a->rank == b->rank && std::memcmp(a->shape, b->shape, sizeof(uint64_t) * a->rank) == 0,
                 "binary: operands must have the same logical shape");
    // loop bound: result.size for + - * /, a.size for pow (aixDeviceCPU.cpp:35, 236)
    const uint64_t n = op == AIXK_POW ? a->size : out->size;
    AIXK_REQUIRE(n == numel(a), "binary: element count %llu does not match the operand shape", (unsigned long long)n);
    switch (op) {
        case AIXK_ADD: return binary_op<AIXK_ADD>(ctx, a, b, out, n);
        case AIXK_SUB: return binary_op<AIXK_SUB>(ctx, a, b, out, n);
        case AIXK_MUL: return binary_op<AIXK_MUL>(ctx, a, b, out, n);
        case AIXK_DIV: return binary_op<AIXK_DIV>(ctx, a, b, out, n);
        case AIXK_POW: return binary_op<AIXK_POW>(ctx, a, b, out, n);
        default: return fail(AIXK_EINVAL, "binary: unknown op %d", op);
    }
}

int32_t aixk_unary(aixk_ctx* ctx, int op, const aixhip_tensor* a, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(out), "unary: bad operand descriptor");
    AIXK_REQUIRE(a->dtype == out->dtype, "unary: operand must have the result's element type");
    const uint64_t n = a->size;                      // aixDeviceCPU.cpp:90, 160
    AIXK_REQUIRE(n == numel(a), "unary: size does not match shape");
    switch (op) {
        case AIXK_NEG:  return unary_op<AIXK_NEG>(ctx, a, out, n);
        case AIXK_SQRT: return unary_op<AIXK_SQRT>(ctx, a, out, n);
        case AIXK_SIN:  return unary_op<AIXK_SIN>(ctx, a, out, n);
        case AIXK_COS:  return unary_op<AIXK_COS>(ctx, a, out, n);
        case AIXK_TANH: return unary_op<AIXK_TANH>(ctx, a, out, n);
        case AIXK_LOG:  return unary_op<AIXK_LOG>(ctx, a, out, n);
        case AIXK_EXP:  return unary_op<AIXK_EXP>(ctx, a, out, n);
        default: return fail(AIXK_EINVAL, "unary: unknown op %d", op);
    }
}

int32_t aixk_fill(aixk_ctx* ctx, const void* scalar, int scalar_dtype, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(scalar != nullptr && valid_tensor(out), "fill: bad argument");
    const uint64_t n = out->size;
    if (n == 0) return AIXK_OK;
    return by_dtype(scalar_dtype, [&](auto stag) {
        typedef decltype(stag) S;
        S s;
        std::memcpy(&s, scalar, sizeof(S));
        return by_dtype(out->dtype, [&](auto dtag) {
            typedef decltype(dtag) D;
            D* po = (D*)out->data;
            const unsigned grid = grid_for(n / vec16<D>::n + 1, kBlock, (unsigned)ctx->cus * 16u);
            if (aligned16(po)) hipLaunchKernelGGL((fill_cvt_vec<S, D>), dim3(grid), dim3(kBlock), 0, ctx->stream, po, s, (u64)n);
            else hipLaunchKernelGGL((fill_cvt<S, D>), dim3(grid), dim3(kBlock), 0, ctx->stream, po, s, (u64)n);
            AIXK_HIP(hipGetLastError());
            return (int)AIXK_OK;
        });
    });
}

int32_t aixk_fill_many(aixk_ctx* ctx, const aixk_fill_item* items, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(items != nullptr || count == 0, "fill_many: null items");
    for (uint32_t at = 0; at < count; at += FillItems::kMost) {
        FillItems it{};
        const uint32_t now = count - at < (uint32_t)FillItems::kMost ? count - at : (uint32_t)FillItems::kMost;
        for (uint32_t k = 0; k < now; ++k) {
            const aixk_fill_item& f = items[at + k];
            AIXK_REQUIRE(f.dst != nullptr && (f.element_size == 1 || f.element_size == 2 || f.element_size == 4 || f.element_size == 8) &&
                         f.elements <= 65536 && ((uintptr_t)f.dst % f.element_size) == 0, "fill_many: bad item %u", at + k);
            it.dst[k] = (u64)(uintptr_t)f.dst; it.bits[k] = f.bits; it.n[k] = f.elements; it.esz[k] = f.element_size;
        }
        hipLaunchKernelGGL(fill_items_k, dim3(now), dim3(kBlock), 0, ctx->stream, it);
        AIXK_HIP(hipGetLastError());
    }
    return AIXK_OK;
}

int32_t aixk_fill_min(aixk_ctx* ctx, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(out), "fillMin: bad argument");
    const uint64_t n = out->size;
    if (n == 0) return AIXK_OK;
    return by_dtype(out->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 16u);
        hipLaunchKernelGGL((fill_min_k<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, (T*)out->data, (u64)n);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_cast(aixk_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype, uint64_t n)
{
    AIXK_TRY(set_device(ctx));
    if (n == 0) return AIXK_OK;
    AIXK_REQUIRE(src && dst, "copy: null pointer");
    if (src_dtype == dst_dtype) {
        AIXK_REQUIRE(src_dtype >= 0 && src_dtype < AIXK_DTYPE_COUNT, "copy: unknown element type");
        AIXK_HIP(hipMemcpyAsync(dst, src, n * aixk_dtype_size(src_dtype), hipMemcpyDeviceToDevice, ctx->stream));
        return AIXK_OK;
    }
    return by_dtype(src_dtype, [&](auto stag) {
        typedef decltype(stag) S;
        return by_dtype(dst_dtype, [&](auto dtag) {
            typedef decltype(dtag) D;
            if constexpr (traits<S>::code == traits<D>::code) return (int)AIXK_OK;
            else {
                constexpr int K = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));
                const unsigned max_blocks = 1u << 22;              // one chunk per lane
                if (aligned16(src) && aligned16(dst)) {
                    if (streams_out(n * sizeof(D)))
                        hipLaunchKernelGGL((cast_flat<S, D, true>), dim3(grid_for(n / K + 1, kBlock, max_blocks)), dim3(kBlock), 0, ctx->stream, (const S*)src, (D*)dst, (u64)n);
                    else
                        hipLaunchKernelGGL((cast_flat<S, D, false>), dim3(grid_for(n / K + 1, kBlock, max_blocks)), dim3(kBlock), 0, ctx->stream, (const S*)src, (D*)dst, (u64)n);
                } else
                    hipLaunchKernelGGL((cast_any<S, D>), dim3(grid_for(n, kBlock, max_blocks)), dim3(kBlock), 0, ctx->stream,
                                       (const S*)src, (D*)dst, (u64)n);
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            }
        });
    });
}

} // extern "C"
