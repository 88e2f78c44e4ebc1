// layout.hip -- pure data movement: contiguous (gather a view into a dense tensor), the
// materialising transpose, sliceSet, tril/triu, indexSelect, indexAdd.
//
// Data movement does not look at values, so kernels are instantiated per element SIZE
// (1, 2, 4, 8 bytes), not per element type.  A 2-D (optionally batched) transposed source is
// moved through 64x64 LDS tiles so that both the HBM read and the HBM write are coalesced;
// everything else uses a strided gather with the same three shapes as the elementwise kernels.

#include "common.hpp"

#include <algorithm>
#include <utility>
#include <vector>

using namespace aixd;
using namespace aixk;

namespace {

template <int BYTES> struct word;
template <> struct word<1> { typedef u8 type; };
template <> struct word<2> { typedef u16 type; };
template <> struct word<4> { typedef u32 type; };
template <> struct word<8> { typedef u64 type; };

template <class F> int by_size(int dtype, F&& f)
{
    switch (aixk_dtype_size(dtype)) {
        case 1: return f(u8{});
        case 2: return f(u16{});
        case 4: return f(u32{});
        case 8: return f(u64{});
        default: return fail(AIXK_EINVAL, "unknown element type %d", dtype);
    }
}

struct alignas(16) u128 { u64 lo, hi; };
template <class F> int by_bytes(size_t bytes, F&& f)
{
    switch (bytes) {
        case 1: return f(u8{});
        case 2: return f(u16{});
        case 4: return f(u32{});
        case 8: return f(u64{});
        case 16: return f(u128{});
        default: return fail(AIXK_EINVAL, "no word of %zu bytes", bytes);
    }
}

// A strided copy moves words, not values, so both views may be read as arrays of wider words where their innermost runs
// allow it: `f` elements at a time if in both views the last dim is dense and a multiple of f long, every other stride and
// the offset are multiples of f and the storage is aligned to f elements -- flat logical indices then pair up f at a time
// in both views.  (A head's [512, 64] slab of 2-byte elements inside a [8192, 768] activation: 16-byte words, an eighth of
// the index arithmetic and of the memory instructions.)
inline size_t widest_factor(const aixhip_tensor* t, size_t esz)
{
    if (t->rank == 0 || t->strides[t->rank - 1] != 1) return 1;
    size_t f = 16 / esz;
    const int last = t->rank - 1;
    auto fits = [&](size_t k) {
        if (t->shape[last] % k != 0 || t->offset % k != 0 || ((uintptr_t)t->data) % (k * esz) != 0) return false;
        for (int d = 0; d < last; ++d) if (t->strides[d] % k != 0) return false;
        return true;
    };
    while (f > 1 && !fits(f)) f /= 2;
    return f;
}
inline void widen(aixhip_tensor* t, size_t f)
{
    if (f <= 1) return;
    const int last = t->rank - 1;
    t->shape[last] /= f;
    for (int d = 0; d < last; ++d) t->strides[d] /= f;
    t->offset /= f;
    t->size /= f;
}

// Position of flat logical index i inside one collapsed view.
template <class IDX> __device__ __forceinline__ u64 locate(const Space<1>& sp, IDX i) { return aixk::locate<1, IDX>(sp, 0, i); }

// ---- strided gather: dst[i] = src[view(i)] -----------------------------------------------------
template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void gather_k(const W* __restrict__ src, W* __restrict__ dst, Space<1> sp, u64 n)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock)
        dst[i] = src[locate<IDX>(sp, (IDX)i)];
}

// rows: inner dim unit stride, 16-byte chunks
template <class W, class IDX, bool NT>
__global__ __launch_bounds__(kBlock) void gather_rows_k(const W* __restrict__ src, W* __restrict__ dst, Space<1> sp,
                                                        u64 total_chunks, IDX chunks)
{
    typedef typename vec16<W>::type V;
    constexpr int VEC = vec16<W>::n;
    Space<1> outer = sp;
    outer.rank = sp.rank - 1;
    for (u64 c = (u64)blockIdx.x * kBlock + threadIdx.x; c < total_chunks; c += (u64)gridDim.x * kBlock) {
        const IDX row = (IDX)(c / chunks);
        const IDX col = (IDX)(c - (u64)row * chunks) * VEC;
        const u64 p = locate<IDX>(outer, row) + col;
        store_sel<NT>((V*)(dst + c * VEC), *(const V*)(src + p));
    }
}

// rows again, walked in the order of the SOURCE: when consecutive destination rows are far apart in the source (heads
// and positions swapped: 64 KB hops that keep landing on the same memory channel) but consecutive source rows are
// close together in the destination, the lanes follow the source and scatter whole rows instead.  dims: outermost
// first, the last one varies fastest; both offsets in elements.
struct RowWalk {
    int rank;
    u64 ext[kMaxDims], src[kMaxDims], dst[kMaxDims];
    u64 src_off;
};
template <class W, class IDX, bool NT>
__global__ __launch_bounds__(kBlock) void permute_rows_k(const W* __restrict__ src, W* __restrict__ dst, RowWalk w, u64 total_chunks, IDX chunks)
{
    typedef typename vec16<W>::type V;
    constexpr int VEC = vec16<W>::n;
    for (u64 c = (u64)blockIdx.x * kBlock + threadIdx.x; c < total_chunks; c += (u64)gridDim.x * kBlock) {
        IDX row = (IDX)(c / chunks);
        const IDX col = (IDX)(c - (u64)row * chunks) * VEC;
        u64 ps = w.src_off + col, pd = col;
        for (int d = w.rank - 1; d >= 0; --d) {
            const IDX ext = (IDX)w.ext[d], q = row / ext, k = row - q * ext;
            ps += (u64)k * w.src[d]; pd += (u64)k * w.dst[d];
            row = q;
        }
        store_sel<NT>((V*)(dst + pd), *(const V*)(src + ps));
    }
}

// ---- tiled transpose ---------------------------------------------------------------------------
// Source element (b, r, c) lives at  off + b*sb + r*1 + c*ld   (unit stride along r);
// destination is dense [B, R, C].  Tile = 64 (r) x 64 (c); 256 lanes.
// Load: lanes sweep r fastest (coalesced in the source); store: lanes sweep c fastest.
constexpr int kTile = 64;
template <class W>
__global__ __launch_bounds__(kBlock) void transpose_tiled_k(const W* __restrict__ src, W* __restrict__ dst,
                                                            u64 R, u64 C, u64 ld, u64 sb, u64 off, u32 tiles_r, u32 tiles_c)
{
    __shared__ W tile[kTile][kTile + 1];
    // XCD-friendly order: consecutive workgroups walk down r so that neighbouring groups share
    // destination rows' DRAM pages.
    const u32 t = blockIdx.x;
    const u32 tr = t % tiles_r, tc = t / tiles_r;
    const u64 b = blockIdx.y;
    const u64 r0 = (u64)tr * kTile, c0 = (u64)tc * kTile;
    const W* s = src + off + b * sb;
    W* d = dst + b * R * C;
    const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;      // 64 x 4
#pragma unroll 4
    for (int k = ly; k < kTile; k += 4) {                        // k indexes c within the tile
        const u64 r = r0 + lx, c = c0 + k;
        if (r < R && c < C) tile[k][lx] = s[r + c * ld];
    }
    __syncthreads();
#pragma unroll 4
    for (int k = ly; k < kTile; k += 4) {                        // k indexes r within the tile
        const u64 r = r0 + k, c = c0 + lx;
        if (r < R && c < C) d[r * C + c] = tile[lx][k];
    }
}

// Same tile walk with 16-byte global accesses on both sides (whole tiles only, everything
// 16-byte aligned): a lane loads VEC consecutive r of one c, scatters them into the LDS tile as
// tile[r][c], and later gathers VEC consecutive c of one r for a 16-byte store.  TR x TC is the
// tile in elements (TR along the source's contiguous dim), BLOCK the lanes of a workgroup.
// Measured on [8192,8192] f32 (us; a plain copy of the same bytes: 89, with non-temporal stores 73):
// 64 x 64 / 256 lanes 111, 128 x 64 / 256 lanes 102, 128 x 128 / 512 lanes 93 -- longer runs on both
// sides (512 bytes) and 8 loads per lane in flight -- and 79 with the result leaving through
// non-temporal stores; four tiles that are neighbours along the destination's contiguous dim are
// numbered consecutively (one tile after another along either dim: 95-103).
template <class W, int TR, int TC, int BLOCK, bool NT>
__global__ __launch_bounds__(BLOCK) void transpose_vec_k(const W* __restrict__ src, W* __restrict__ dst,
                                                         u64 R, u64 C, u64 ld, u64 sb, u64 off, u32 tiles_r, u32 tiles_c)
{
    typedef typename vec16<W>::type V;
    constexpr int VEC = vec16<W>::n;
    constexpr int LPR = TR / VEC, RPP = BLOCK / LPR;       // lanes per source row, source rows per pass
    constexpr int LPW = TC / VEC, WPP = BLOCK / LPW;       // lanes per destination row, destination rows per pass
    extern __shared__ __align__(16) unsigned char transpose_lds[];
    W (*tile)[TC + 1] = (W (*)[TC + 1])transpose_lds;
    const u32 t = blockIdx.x;
    u32 tr, tc;
    if (tiles_c % 4 == 0) { tc = (t / (4 * tiles_r)) * 4 + t % 4; tr = (t / 4) % tiles_r; }
    else { tr = t % tiles_r; tc = t / tiles_r; }
    const u64 b = blockIdx.y;
    const u64 r0 = (u64)tr * TR, c0 = (u64)tc * TC;
    const W* s = src + off + b * sb;
    W* d = dst + b * R * C;
    const int lv = (threadIdx.x % LPR) * VEC, lp = threadIdx.x / LPR;
#pragma unroll
    for (int cc = lp; cc < TC; cc += RPP) {
        const V v = *(const V*)(s + (r0 + lv) + (c0 + cc) * ld);
#pragma unroll
        for (int e = 0; e < VEC; ++e) tile[lv + e][cc] = v.v[e];
    }
    __syncthreads();
    const int wv = (threadIdx.x % LPW) * VEC, wp = threadIdx.x / LPW;
#pragma unroll
    for (int rr = wp; rr < TR; rr += WPP) {
        V v;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v.v[e] = tile[rr][wv + e];
        if constexpr (NT) store_nt((V*)(d + (r0 + rr) * C + c0 + wv), v);
        else *(V*)(d + (r0 + rr) * C + c0 + wv) = v;
    }
}

// ---- generic strided copy with both sides strided (sliceSet, transpose scatter) ---------------
template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void copy_views_k(const W* __restrict__ src, W* __restrict__ dst,
                                                       Space<1> ssp, Space<1> dsp, u64 n)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock)
        dst[locate<IDX>(dsp, (IDX)i)] = src[locate<IDX>(ssp, (IDX)i)];
}

// Several such copies in one launch: item k's views and element count come from a table in device memory, its share of
// the grid from `starts` (count + 1 ascending numbers, the last one the grid size).
struct CopyItem { u64 src, dst, n, pad; Space<1> ssp, dsp; };

template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void copy_views_many_k(const CopyItem* __restrict__ items, const u32* __restrict__ starts, u32 count)
{
    u32 lo = 0, hi = count;
    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (starts[mid] <= blockIdx.x) lo = mid; else hi = mid; }
    const CopyItem& it = items[lo];
    const u32 first = starts[lo], share = starts[lo + 1] - first;
    const W* src = global_ptr<const W>(it.src);
    W* dst = global_ptr<W>(it.dst);
    const u64 n = it.n;
    for (u64 i = (u64)(blockIdx.x - first) * kBlock + threadIdx.x; i < n; i += (u64)share * kBlock)
        dst[locate<IDX>(it.dsp, (IDX)i)] = src[locate<IDX>(it.ssp, (IDX)i)];
}

// ---- fill + sliceSet in one pass ----------------------------------------------------------------
// dst is dense: element i is (o, c, e) = (i / (D inner), (i / inner) % D, i % inner) around the sliced dim.
template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void slice_set_init_k(const W* __restrict__ src, W* __restrict__ dst, Space<1> ssp, u64 n,
                                                           u64 inner, u64 extent, u64 start, u64 end, u64 step, u64 count, W init)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) {
        const u64 q = i / inner, e = i - q * inner, o = q / extent, c = q - o * extent;
        W v = init;
        if (c >= start && c < end) {
            const u64 k = (c - start) / step;
            if (start + k * step == c) v = src[locate<IDX>(ssp, (IDX)((o * count + k) * inner + e))];
        }
        dst[i] = v;
    }
}

// ---- tril / triu -------------------------------------------------------------------------------
template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void tri_k(const W* __restrict__ src, W* __restrict__ dst, Space<1> ssp, Space<1> dsp,
                                                u64 n, u64 rows, u64 cols, i64 diagonal, int upper)
{
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) {
        const i64 r = (i64)((i / cols) % rows), c = (i64)(i % cols);
        const bool zero = upper ? (c < r + diagonal) : (c > r + diagonal);
        dst[locate<IDX>(dsp, (IDX)i)] = zero ? (W)0 : src[locate<IDX>(ssp, (IDX)i)];
    }
}

// Dense source and destination, rows of whole 16-byte vectors: a lane owns one vector (all of it in one row), reads it
// only if some of it is kept and writes 16 bytes; the zeroed triangle is never read.
template <class W>
__global__ __launch_bounds__(kBlock) void tri_vec_k(const W* __restrict__ src, W* __restrict__ dst, u64 nvec, u64 rows, u64 cols, i64 diagonal, int upper)
{
    constexpr int VEC = 16 / sizeof(W);
    typedef vec<W, VEC> V;
    const u64 v = (u64)blockIdx.x * kBlock + threadIdx.x;
    if (v >= nvec) return;
    const u64 i = v * VEC;
    const i64 r = (i64)((i / cols) % rows), c = (i64)(i % cols);
    const i64 edge = r + diagonal;                       // lower: columns above `edge` are zeroed; upper: columns below it
    const bool none = upper ? (c + VEC - 1 < edge) : (c > edge);
    V x;
    if (none) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) x.v[e] = (W)0;
    } else {
        x = *(const V*)(src + i);
#pragma unroll
        for (int e = 0; e < VEC; ++e) if (upper ? (c + e < edge) : (c + e > edge)) x.v[e] = (W)0;
    }
    *(V*)(dst + i) = x;
}

// ---- indexSelect -------------------------------------------------------------------------------
// The reference checks the range of the indices only by a host-side assert after a synchronize
// (aixCore.hpp:1242, 1640-1650).  Here an index outside [0, extent) touches no memory: indexSelect
// writes a zero for it, indexAdd skips it.
template <class W, class IDX>
__global__ __launch_bounds__(kBlock) void index_select_k(const W* __restrict__ src, W* __restrict__ dst, const i32* __restrict__ idx,
                                                         Space<1> ssp, Space<1> isp, u64 n, u64 inner, u64 ni, u64 span)
{
    // (IDX = u32 when everything fits: a 64-bit division is a hundred instructions, and there are three per element)
    const IDX per = (IDX)inner, count = (IDX)ni;
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) {
        const IDX row = (IDX)i / per, e = (IDX)i - row * per, o = row / count, k = row - o * count;
        const i32 at = idx[locate<IDX>(isp, k)];
        const u64 which = (u64)(i64)at;
        if (at < 0 || which * inner >= (span ? span : inner)) { dst[i] = (W)0; continue; }          // index outside the source: no access, a zero
        dst[i] = src[locate<IDX>(ssp, (IDX)((u64)o * span + which * inner + e))];
    }
}

// Rows of a dense source whose length is a whole number of 16-byte words (an embedding table's rows): a lane moves a
// 16-byte word, and 2^shift neighbouring lanes (the least power of two that holds a row, at most the workgroup) share a
// row: one index load per row and group of lanes, a shift and a mask instead of divisions per word (the element-wise
// kernel spent its time on those: 27 us for [8192, 768] bf16 rows, 19 us word by word with divisions, 9 us here).
template <class IDX>
__global__ __launch_bounds__(kBlock) void index_select_rows_k(const u128* __restrict__ src, u128* __restrict__ dst, const i32* __restrict__ idx,
                                                              Space<1> isp, u64 rows, u64 inner, u64 ni, u64 extent, u32 shift)
{
    const u32 lanes = 1u << shift, sub = threadIdx.x >> shift, first = threadIdx.x & (lanes - 1), per_pass = kBlock >> shift;
    for (u64 row = (u64)blockIdx.x * per_pass + sub; row < rows; row += (u64)gridDim.x * per_pass) {
        const u64 o = row / ni, k = row - o * ni;
        const i32 at = idx[locate<IDX>(isp, (IDX)k)];
        const bool inside = at >= 0 && (u64)at < extent;                                // (an index outside the source: a row of zeros)
        const u128* from = src + (o * extent + (inside ? (u64)at : 0)) * inner;
        u128* to = dst + row * inner;
        for (u64 e = first; e < inner; e += lanes) to[e] = inside ? from[e] : u128{0, 0};
    }
}

// ---- indexAdd ----------------------------------------------------------------------------------
// dst[slot] += src[i] with duplicates summed: atomics.  32/64-bit types use native atomics;
// 8/16-bit types update their containing 32-bit word with a compare-and-swap loop.
template <class T> __device__ __forceinline__ void atomic_accumulate(T* base, u64 pos, T val)
{
    if constexpr (traits<T>::code == DT_F32) atomicAdd(base + pos, val);
    else if constexpr (traits<T>::code == DT_F64) atomicAdd(base + pos, val);
    else if constexpr (traits<T>::code == DT_I32) atomicAdd((int*)base + pos, val);
    else if constexpr (traits<T>::code == DT_I64) atomicAdd((unsigned long long*)base + pos, (unsigned long long)val);
    else {
        const uintptr_t addr = (uintptr_t)(base + pos);
        u32* wordp = (u32*)(addr & ~(uintptr_t)3);
        const u32 shift = (u32)(addr & 3) * 8;
        constexpr u32 mask = sizeof(T) == 1 ? 0xFFu : 0xFFFFu;
        u32 old = *wordp, assumed;
        do {
            assumed = old;
            typedef typename word<sizeof(T)>::type Wd;
            const Wd cur_bits = (Wd)((assumed >> shift) & mask);
            const T cur = __builtin_bit_cast(T, cur_bits);
            const T nxt = e_add(cur, val);
            const u32 nxt_bits = (u32)__builtin_bit_cast(Wd, nxt);
            old = atomicCAS(wordp, assumed, (assumed & ~(mask << shift)) | (nxt_bits << shift));
        } while (old != assumed);
    }
}

template <class T, class IDX>
__global__ __launch_bounds__(kBlock) void index_add_k(const T* __restrict__ src, T* __restrict__ dst, const i32* __restrict__ idx,
                                                      Space<1> ssp, Space<1> isp, u64 n, u64 inner, u64 ni, u64 span)
{
    const IDX per = (IDX)inner, count = (IDX)ni;                   // (IDX = u32 when everything fits: no 64-bit divisions)
    for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock) {
        const IDX row = (IDX)i / per, e = (IDX)i - row * per, o = row / count, k = row - o * count;
        const i32 at = idx[locate<IDX>(isp, k)];
        const u64 which = (u64)(i64)at;
        if (at < 0 || which * inner >= (span ? span : inner)) continue;                               // index outside the destination: nothing is written
        atomic_accumulate<T>(dst, (u64)o * span + which * inner + e, src[locate<IDX>(ssp, (IDX)i)]);
    }
}

// 16-bit element types with an even inner extent: a lane owns the two elements of one 32-bit word of the
// destination and updates both in one compare-and-swap -- half the atomics, and the two halves of a word no longer
// fight each other from neighbouring lanes (the two embedding gradients of a transformer step, [8192, 768] bf16 each:
// 267 us per call before, 0.34 ms less per step with this).
template <class T, class IDX>
__global__ __launch_bounds__(kBlock) void index_add_pairs_k(const T* __restrict__ src, T* __restrict__ dst, const i32* __restrict__ idx,
                                                            Space<1> ssp, Space<1> isp, u64 n, u64 inner, u64 ni, u64 span)
{
    typedef typename word<sizeof(T)>::type Wd;
    const IDX per = (IDX)inner, count = (IDX)ni;
    for (u64 i = ((u64)blockIdx.x * kBlock + threadIdx.x) * 2; i < n; i += (u64)gridDim.x * kBlock * 2) {
        const IDX row = (IDX)i / per, e = (IDX)i - row * per, o = row / count, k = row - o * count;
        const i32 at = idx[locate<IDX>(isp, k)];
        const u64 which = (u64)(i64)at;
        if (at < 0 || which * inner >= (span ? span : inner)) continue;
        const T lo = src[locate<IDX>(ssp, (IDX)i)], hi = src[locate<IDX>(ssp, (IDX)(i + 1))];
        u32* wordp = (u32*)(dst + (u64)o * span + which * inner + e);
        u32 old = *wordp, assumed;
        do {
            assumed = old;
            const T a = __builtin_bit_cast(T, (Wd)(assumed & 0xFFFFu)), b = __builtin_bit_cast(T, (Wd)(assumed >> 16));
            const u32 next = (u32)__builtin_bit_cast(Wd, e_add(a, lo)) | ((u32)__builtin_bit_cast(Wd, e_add(b, hi)) << 16);
            old = atomicCAS(wordp, assumed, next);
        } while (old != assumed);
    }
}

// Host routing for dst(dense)[i] = src[view(i)], n elements.
int gather_into(aixk_ctx* ctx, const aixhip_tensor* src, void* dst, uint64_t n)
{
    if (n == 0) return AIXK_OK;
    Space<1> sp;
    if (!collapse1(src, &sp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const size_t esz = aixk_dtype_size(src->dtype);
    const unsigned max_blocks = (unsigned)ctx->cus * 32u;
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31);

    // dense already: plain copy
    if (sp.rank == 0 || (sp.rank == 1 && sp.stride[0][0] == 1)) {
        AIXK_HIP(hipMemcpyAsync(dst, (const char*)src->data + sp.offset[0] * esz, n * esz, hipMemcpyDeviceToDevice, ctx->stream));
        return AIXK_OK;
    }
    return by_size(src->dtype, [&](auto tag) {
        typedef decltype(tag) W;
        constexpr int VEC = vec16<W>::n;
        const W* ps = (const W*)src->data;
        W* pd = (W*)dst;
        const bool nt = streams_out(n * sizeof(W));         // a large result leaves through non-temporal stores
        // 2-D / batched 2-D transposed: [B?, R, C] with strides (sb, 1, ld)
        if ((sp.rank == 2 && sp.stride[0][0] == 1) || (sp.rank == 3 && sp.stride[0][1] == 1)) {
            const int o = sp.rank - 2;
            const uint64_t B = sp.rank == 3 ? sp.shape[0] : 1, sb = sp.rank == 3 ? sp.stride[0][0] : 0;
            const uint64_t R = sp.shape[o], C = sp.shape[o + 1], ld = sp.stride[0][o + 1];
            const uint64_t tr = (R + kTile - 1) / kTile, tc = (C + kTile - 1) / kTile;
            const bool vecok = ld != 0 && ld % VEC == 0 && sb % VEC == 0 && aligned16(ps + sp.offset[0]) && aligned16(pd) && B < 65536;
            // tile in elements: 512-byte runs on both sides where the shape allows (128 x 128 of 4 bytes, 256 x 256 of
            // 2 would not fit: 128 x 128 there too), else 64 x 64
            auto launch_t = [&](auto kernel, uint64_t TR, uint64_t TC, unsigned block) {
                const size_t lds = sizeof(W) * TR * (TC + 1);
                hipLaunchKernelGGL(kernel, dim3((unsigned)((R / TR) * (C / TC)), (unsigned)B), dim3(block), lds, ctx->stream,
                                   ps, pd, (u64)R, (u64)C, (u64)ld, (u64)sb, (u64)sp.offset[0], (u32)(R / TR), (u32)(C / TC));
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            };
            if (vecok && sizeof(W) <= 4 && sizeof(W) >= 2 && R % 128 == 0 && C % 128 == 0 && (R / 128) * (C / 128) < (1ull << 31) && (R / 128) * (C / 128) * B >= (uint64_t)ctx->cus)
            {
                if constexpr (sizeof(W) * 128 * 129 > 65536) {               // beyond the default limit of dynamic LDS: raised once
                    static bool raised = false;
                    if (!raised) {
                        AIXK_HIP(hipFuncSetAttribute((const void*)transpose_vec_k<W, 128, 128, 512, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(sizeof(W) * 128 * 129)));
                        AIXK_HIP(hipFuncSetAttribute((const void*)transpose_vec_k<W, 128, 128, 512, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(sizeof(W) * 128 * 129)));
                        raised = true;
                    }
                }
                return nt ? launch_t(transpose_vec_k<W, 128, 128, 512, true>, 128, 128, 512) : launch_t(transpose_vec_k<W, 128, 128, 512, false>, 128, 128, 512);
            }
            if (vecok && R % kTile == 0 && C % kTile == 0 && tr * tc < (1ull << 31))
                return nt ? launch_t(transpose_vec_k<W, kTile, kTile, kBlock, true>, kTile, kTile, kBlock) : launch_t(transpose_vec_k<W, kTile, kTile, kBlock, false>, kTile, kTile, kBlock);
            if (ld != 0 && tr * tc < (1ull << 31) && B < 65536) {
                hipLaunchKernelGGL((transpose_tiled_k<W>), dim3((unsigned)(tr * tc), (unsigned)B), dim3(kBlock), 0, ctx->stream,
                                   ps, pd, (u64)R, (u64)C, (u64)ld, (u64)sb, (u64)sp.offset[0], (u32)tr, (u32)tc);
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            }
        }
        // rows: inner dim unit stride and everything 16-byte aligned
        const int in = sp.rank - 1;
        if (sp.stride[0][in] == 1 && sp.shape[in] % VEC == 0 && aligned16(pd) && aligned16(ps + sp.offset[0])) {
            bool ok = true;
            for (int d = 0; d < in; ++d) if (sp.stride[0][d] % VEC) ok = false;
            if (ok) {
                const uint64_t chunks = sp.shape[in] / VEC, total = n / VEC;
                const unsigned grid = grid_for(total, kBlock, max_blocks);
                // the walk in source order, if its hop between consecutive rows (in the destination) is the shorter one
                if (in >= 2) {
                    RowWalk w{};
                    w.rank = in; w.src_off = sp.offset[0];
                    uint64_t run = sp.shape[in];
                    bool plain = true;
                    for (int d = in - 1; d >= 0; --d) { w.ext[d] = sp.shape[d]; w.src[d] = sp.stride[0][d]; w.dst[d] = run; run *= sp.shape[d]; if (sp.stride[0][d] == 0) plain = false; }
                    const uint64_t hop_here = w.src[in - 1] * sizeof(W);
                    for (int i = 1; i < in; ++i)                       // insertion sort by source stride, largest first
                        for (int j = i; j > 0 && w.src[j] > w.src[j - 1]; --j) { std::swap(w.ext[j], w.ext[j - 1]); std::swap(w.src[j], w.src[j - 1]); std::swap(w.dst[j], w.dst[j - 1]); }
                    const uint64_t hop_there = w.dst[in - 1] * sizeof(W);
                    if (plain && hop_here >= 4096 && hop_there < hop_here) {
                        if (small) { if (nt) hipLaunchKernelGGL((permute_rows_k<W, u32, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, w, (u64)total, (u32)chunks);
                                     else hipLaunchKernelGGL((permute_rows_k<W, u32, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, w, (u64)total, (u32)chunks); }
                        else { if (nt) hipLaunchKernelGGL((permute_rows_k<W, u64, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, w, (u64)total, (u64)chunks);
                               else hipLaunchKernelGGL((permute_rows_k<W, u64, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, w, (u64)total, (u64)chunks); }
                        AIXK_HIP(hipGetLastError());
                        return (int)AIXK_OK;
                    }
                }
                if (small) { if (nt) hipLaunchKernelGGL((gather_rows_k<W, u32, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)total, (u32)chunks);
                             else hipLaunchKernelGGL((gather_rows_k<W, u32, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)total, (u32)chunks); }
                else { if (nt) hipLaunchKernelGGL((gather_rows_k<W, u64, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)total, (u64)chunks);
                       else hipLaunchKernelGGL((gather_rows_k<W, u64, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)total, (u64)chunks); }
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            }
        }
        const unsigned grid = grid_for(n, kBlock, max_blocks);
        if (small) hipLaunchKernelGGL((gather_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)n);
        else hipLaunchKernelGGL((gather_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, pd, sp, (u64)n);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int copy_views(aixk_ctx* ctx, const aixhip_tensor* src_in, const aixhip_tensor* dst_in, uint64_t n)
{
    if (n == 0) return AIXK_OK;
    const size_t esz = aixk_dtype_size(src_in->dtype);
    aixhip_tensor wide_src = *src_in, wide_dst = *dst_in;
    const size_t f = n == numel(src_in) && n == numel(dst_in) ? std::min(widest_factor(src_in, esz), widest_factor(dst_in, esz)) : 1;
    widen(&wide_src, f); widen(&wide_dst, f);
    n /= f;
    const aixhip_tensor *src = &wide_src, *dst = &wide_dst;
    Space<1> ssp, dsp;
    if (!collapse1(src, &ssp) || !collapse1(dst, &dsp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31) && view_extent(dst) < (1ull << 31);
    return by_bytes(esz * f, [&](auto tag) {
        typedef decltype(tag) W;
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 32u);
        if (small) hipLaunchKernelGGL((copy_views_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, dsp, (u64)n);
        else hipLaunchKernelGGL((copy_views_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, dsp, (u64)n);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

} // namespace

extern "C" {

int32_t aixk_contiguous(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "contiguous: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "contiguous: element types differ");
    const uint64_t n = dst->size;                    // aixDeviceCPU.cpp:431
    AIXK_REQUIRE(n == numel(src), "contiguous: dst size does not match the source shape");
    return gather_into(ctx, src, dst->data, n);
}

int32_t aixk_transpose(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* out, uint64_t dim0, uint64_t dim1)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(out), "transpose: bad operand descriptor");
    AIXK_REQUIRE(a->dtype == out->dtype, "transpose: element types differ");
    AIXK_REQUIRE((int)dim0 < a->rank && (int)dim1 < a->rank && out->rank == a->rank, "transpose: dims out of range");
    // Source read through the swapped view; equals the flat read of aixDeviceCPU.cpp:391-405 for
    // the contiguous sources that function assumes.
    aixhip_tensor v = *a;
    v.shape[dim0] = a->shape[dim1]; v.shape[dim1] = a->shape[dim0];
    v.strides[dim0] = a->strides[dim1]; v.strides[dim1] = a->strides[dim0];
    uint64_t dense[AIXK_MAX_RANK];
    row_major_strides(v.rank, v.shape, dense);
    bool out_dense = true;
    for (int d = 0; d < v.rank; ++d) if (v.shape[d] > 1 && out->strides[d] != dense[d]) out_dense = false;
    if (out_dense) return gather_into(ctx, &v, out->data, a->size);
    aixhip_tensor o = *out;
    o.offset = 0;                                    // result written from base (aixDeviceCPU.cpp:395-403)
    std::memcpy(o.shape, v.shape, sizeof(v.shape));
    return copy_views(ctx, &v, &o, a->size);
}

int32_t aixk_slice_set(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                       uint64_t dim, uint64_t start, uint64_t end, uint64_t step)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "sliceSet: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "sliceSet: element types differ");
    AIXK_REQUIRE((int)dim < dst->rank && step > 0 && end >= start, "sliceSet: bad slice");
    aixhip_tensor window = *dst;                     // the strided window of dst that receives src
    window.shape[dim] = (end - start + step - 1) / step;
    window.offset = dst->offset + start * dst->strides[dim];
    window.strides[dim] = dst->strides[dim] * step;
    const uint64_t n = src->size;                    // aixDeviceCPU.cpp:477
    AIXK_REQUIRE(n == numel(&window) && n == numel(src), "sliceSet: source size does not match the slice");
    AIXK_REQUIRE(start + (window.shape[dim] ? (window.shape[dim] - 1) * step : 0) < dst->shape[dim] || n == 0,
                 "sliceSet: slice exceeds the destination");
    return copy_views(ctx, src, &window, n);
}

int32_t aixk_slice_set_many(aixk_ctx* ctx, const aixk_slice_item* items, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    if (count == 0) return AIXK_OK;
    AIXK_REQUIRE(items, "sliceSet of several items: no items");
    AIXK_REQUIRE(count <= AIXK_SLICE_ITEMS_MAX, "sliceSet of several items: more than %d items", (int)AIXK_SLICE_ITEMS_MAX);
    const size_t esz = aixk_dtype_size(items[0].src.dtype);
    const size_t table_bytes = (size_t)count * sizeof(CopyItem), all_bytes = table_bytes + ((size_t)count + 1) * sizeof(u32);
    char* host = nullptr;                            // built where the copy engine will read it
    const char* dev = nullptr;
    AIXK_TRY(table_slot(ctx, all_bytes, (void**)&host, (const void**)&dev));
    CopyItem* table = (CopyItem*)host;
    u32* starts = (u32*)(host + table_bytes);
    bool small = true;
    u32 grid = 0;
    // the windows of the destinations, and the widest word every item can be copied in
    std::vector<aixhip_tensor> windows(count);
    size_t f = 16 / esz;
    for (uint32_t k = 0; k < count; ++k) {
        const aixhip_tensor *src = &items[k].src, *dst = &items[k].dst;
        const uint64_t dim = items[k].dim, start = items[k].start, end = items[k].end, step = items[k].step;
        AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "sliceSet: bad operand descriptor");
        AIXK_REQUIRE(src->dtype == dst->dtype, "sliceSet: element types differ");
        AIXK_REQUIRE(aixk_dtype_size(src->dtype) == esz, "sliceSet of several items: element sizes differ");
        AIXK_REQUIRE((int)dim < dst->rank && step > 0 && end >= start, "sliceSet: bad slice");
        aixhip_tensor& window = windows[k];
        window = *dst;
        window.shape[dim] = (end - start + step - 1) / step;
        window.offset = dst->offset + start * dst->strides[dim];
        window.strides[dim] = dst->strides[dim] * step;
        const uint64_t n = src->size;
        AIXK_REQUIRE(n > 0 && n == numel(&window) && n == numel(src), "sliceSet: source size does not match the slice");
        AIXK_REQUIRE(start + (window.shape[dim] - 1) * step < dst->shape[dim], "sliceSet: slice exceeds the destination");
        window.size = n;
        f = std::min({f, widest_factor(src, esz), widest_factor(&window, esz)});
    }
    for (uint32_t k = 0; k < count; ++k) {
        aixhip_tensor wide_src = items[k].src;
        aixhip_tensor& window = windows[k];
        widen(&wide_src, f); widen(&window, f);
        const aixhip_tensor* src = &wide_src;
        const uint64_t n = src->size;
        CopyItem& it = table[k];
        it.src = (u64)(uintptr_t)src->data; it.dst = (u64)(uintptr_t)window.data; it.n = n; it.pad = 0;
        if (!collapse1(src, &it.ssp) || !collapse1(&window, &it.dsp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
        small = small && n < (1ull << 31) && view_extent(src) < (1ull << 31) && view_extent(&window) < (1ull << 31);
        starts[k] = grid;
        const unsigned share = grid_for(n, kBlock, (unsigned)ctx->cus * 4u);
        AIXK_REQUIRE((uint64_t)grid + share < (1ull << 31), "sliceSet of several items: grid too large");
        grid += share;
    }
    starts[count] = grid;
    AIXK_TRY(table_upload(ctx, host, dev, all_bytes));
    return by_bytes(esz * f, [&](auto tag) {
        typedef decltype(tag) W;
        if (small) hipLaunchKernelGGL((copy_views_many_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const CopyItem*)dev, (const u32*)(dev + table_bytes), (u32)count);
        else hipLaunchKernelGGL((copy_views_many_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const CopyItem*)dev, (const u32*)(dev + table_bytes), (u32)count);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_slice_set_init(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                            uint64_t dim, uint64_t start, uint64_t end, uint64_t step, uint64_t init_bits)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "sliceSet: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "sliceSet: element types differ");
    AIXK_REQUIRE((int)dim < dst->rank && step > 0 && end >= start, "sliceSet: bad slice");
    uint64_t dense[AIXK_MAX_RANK];
    row_major_strides(dst->rank, dst->shape, dense);
    bool is_dense = dst->offset == 0 && dst->size == numel(dst);
    for (int d = 0; d < dst->rank; ++d) if (dst->shape[d] != 1 && dst->strides[d] != dense[d]) is_dense = false;
    AIXK_REQUIRE(is_dense, "sliceSet with initialisation: the destination must be dense");
    const uint64_t count = (end - start + step - 1) / step;
    uint64_t window = count;
    for (int d = 0; d < dst->rank; ++d) if (d != (int)dim) window *= dst->shape[d];
    AIXK_REQUIRE(src->size == window && window == numel(src), "sliceSet: source size does not match the slice");
    AIXK_REQUIRE(count == 0 || start + (count - 1) * step < dst->shape[dim], "sliceSet: slice exceeds the destination");
    const uint64_t n = dst->size;
    if (n == 0) return AIXK_OK;
    uint64_t inner = 1;
    for (int d = (int)dim + 1; d < dst->rank; ++d) inner *= dst->shape[d];
    Space<1> ssp;
    if (!collapse1(src, &ssp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31);
    return by_size(src->dtype, [&](auto tag) {
        typedef decltype(tag) W;
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 32u);
        if (small) hipLaunchKernelGGL((slice_set_init_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, (u64)n,
                                      (u64)inner, (u64)dst->shape[dim], (u64)start, (u64)end, (u64)step, (u64)count, (W)init_bits);
        else hipLaunchKernelGGL((slice_set_init_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, (u64)n,
                                (u64)inner, (u64)dst->shape[dim], (u64)start, (u64)end, (u64)step, (u64)count, (W)init_bits);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_tri(aixk_ctx* ctx, int upper, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "tril/triu: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "tril/triu: element types differ");      // aixDeviceMetal.cpp:1160-1161
    AIXK_REQUIRE(src->rank >= 2, "tril/triu: rank must be at least 2");
    const uint64_t n = dst->size;                    // aixDeviceCPU.cpp:576
    if (n == 0) return AIXK_OK;
    AIXK_REQUIRE(n == numel(src) && n == numel(dst), "tril/triu: sizes differ");
    Space<1> ssp, dsp;
    if (!collapse1(src, &ssp) || !collapse1(dst, &dsp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const uint64_t rows = src->shape[src->rank - 2], cols = src->shape[src->rank - 1];
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31) && view_extent(dst) < (1ull << 31);
    return by_size(src->dtype, [&](auto tag) {
        typedef decltype(tag) W;
        constexpr uint64_t VEC = 16 / sizeof(W);
        const bool dense = (ssp.rank == 0 || (ssp.rank == 1 && ssp.stride[0][0] == 1)) && (dsp.rank == 0 || (dsp.rank == 1 && dsp.stride[0][0] == 1));
        const W* ps = (const W*)src->data + ssp.offset[0];
        W* pd = (W*)dst->data + dsp.offset[0];
        if (dense && cols % VEC == 0 && aligned16(ps) && aligned16(pd) && n / VEC / kBlock < (1ull << 31)) {
            hipLaunchKernelGGL((tri_vec_k<W>), dim3((unsigned)((n / VEC + kBlock - 1) / kBlock)), dim3(kBlock), 0, ctx->stream, ps, pd, (u64)(n / VEC), (u64)rows, (u64)cols, (i64)diagonal, upper);
            AIXK_HIP(hipGetLastError());
            return (int)AIXK_OK;
        }
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 32u);
        if (small) hipLaunchKernelGGL((tri_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, dsp, (u64)n, (u64)rows, (u64)cols, (i64)diagonal, upper);
        else hipLaunchKernelGGL((tri_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, ssp, dsp, (u64)n, (u64)rows, (u64)cols, (i64)diagonal, upper);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_index_select(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                          const aixhip_tensor* indices, uint64_t dim)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst) && valid_tensor(indices), "indexSelect: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "indexSelect: element types differ");
    AIXK_REQUIRE(indices->dtype == AIXK_I32, "indexSelect: indices must be int32");
    AIXK_REQUIRE((src->rank == 0 && dim == 0) || (int)dim < src->rank, "indexSelect: dim out of range");
    const uint64_t n = dst->size;                    // aixDeviceCPU.cpp:516
    if (n == 0) return AIXK_OK;
    uint64_t inner = 1;
    for (int d = (int)dim + 1; d < src->rank; ++d) inner *= src->shape[d];
    const uint64_t span = src->rank ? src->shape[dim] * inner : 0, ni = indices->size;
    AIXK_REQUIRE(ni > 0, "indexSelect: empty indices");
    Space<1> ssp, isp;
    if (!collapse1(src, &ssp) || !collapse1(indices, &isp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31) && numel(src) < (1ull << 31);
    {
        // a dense source, rows of whole 16-byte words: word by word
        const size_t esz = aixk_dtype_size(src->dtype);
        bool dense = src->rank > 0;
        uint64_t run = 1;
        for (int d = src->rank - 1; d >= 0 && dense; --d) { dense = src->shape[d] == 1 || src->strides[d] == run; run *= src->shape[d]; }
        const char* base = (const char*)src->data + src->offset * esz;
        if (dense && esz && (inner * esz) % 16 == 0 && aligned16(base) && aligned16(dst->data)) {
            const uint64_t per = inner * esz / 16, rows = n / inner;
            u32 shift = 0;
            while ((1u << shift) < per && (1u << shift) < kBlock) ++shift;
            const unsigned grid = grid_for(rows, kBlock >> shift, (unsigned)ctx->cus * 64u);
            if (small) hipLaunchKernelGGL((index_select_rows_k<u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const u128*)base, (u128*)dst->data, (const i32*)indices->data, isp, (u64)rows, (u64)per, (u64)ni, (u64)src->shape[dim], shift);
            else hipLaunchKernelGGL((index_select_rows_k<u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const u128*)base, (u128*)dst->data, (const i32*)indices->data, isp, (u64)rows, (u64)per, (u64)ni, (u64)src->shape[dim], shift);
            AIXK_HIP(hipGetLastError());
            return (int32_t)AIXK_OK;
        }
    }
    return by_size(src->dtype, [&](auto tag) {
        typedef decltype(tag) W;
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 32u);
        if (small) hipLaunchKernelGGL((index_select_k<W, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
        else hipLaunchKernelGGL((index_select_k<W, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const W*)src->data, (W*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_index_add(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                       const aixhip_tensor* indices, uint64_t dim)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst) && valid_tensor(indices), "indexAdd: bad operand descriptor");
    AIXK_REQUIRE(src->dtype == dst->dtype, "indexAdd: element types differ");
    AIXK_REQUIRE(indices->dtype == AIXK_I32, "indexAdd: indices must be int32");
    AIXK_REQUIRE((dst->rank == 0 && dim == 0) || (int)dim < dst->rank, "indexAdd: dim out of range");
    const uint64_t n = src->size;                    // aixDeviceCPU.cpp:550
    if (n == 0) return AIXK_OK;
    uint64_t inner = 1;
    for (int d = (int)dim + 1; d < dst->rank; ++d) inner *= dst->shape[d];
    const uint64_t span = dst->rank ? dst->shape[dim] * inner : 0, ni = indices->size;
    AIXK_REQUIRE(ni > 0, "indexAdd: empty indices");
    Space<1> ssp, isp;
    if (!collapse1(src, &ssp) || !collapse1(indices, &isp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const bool small = n < (1ull << 31) && view_extent(src) < (1ull << 31);
    return by_dtype(src->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if constexpr (sizeof(T) == 2) {
            if (inner % 2 == 0 && ((uintptr_t)dst->data & 3u) == 0) {
                const unsigned pairs_grid = grid_for(n / 2, kBlock, (unsigned)ctx->cus * 32u);
                if (small) hipLaunchKernelGGL((index_add_pairs_k<T, u32>), dim3(pairs_grid), dim3(kBlock), 0, ctx->stream, (const T*)src->data, (T*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
                else hipLaunchKernelGGL((index_add_pairs_k<T, u64>), dim3(pairs_grid), dim3(kBlock), 0, ctx->stream, (const T*)src->data, (T*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            }
        }
        const unsigned grid = grid_for(n, kBlock, (unsigned)ctx->cus * 32u);
        if (small) hipLaunchKernelGGL((index_add_k<T, u32>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const T*)src->data, (T*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
        else hipLaunchKernelGGL((index_add_k<T, u64>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const T*)src->data, (T*)dst->data, (const i32*)indices->data, ssp, isp, (u64)n, (u64)inner, (u64)ni, (u64)span);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

} // extern "C"

namespace aixk {
// dst (dense, n elements) = the logical contents of `src`; used by the GEMM to make operands K-contiguous.
int gather_dense(aixk_ctx* ctx, const aixhip_tensor* src, void* dst, uint64_t n) { return gather_into(ctx, src, dst, n); }
} // namespace aixk
