// reduce.hip -- sum / max / argmax over a whole tensor and over subsets of dims
// (reduceTo, maxTo, argmaxTo, argmaxIndicesTo) for all nine element types.
//
// HBM-bound streaming reductions.  Per lane: 16-byte loads, accumulation in registers in a wide
// type (f32 for f16/bf16, same-width wrap-around for integers, f32/f64 for themselves); per
// wavefront: a 64-lane shuffle tree; per workgroup: LDS combine of the 4 waves; across
// workgroups: partials in scratch, combined in a fixed order (results are run-to-run
// deterministic).
//
// Semantics kept from the reference CPU device:
//   * reduceTo / maxTo accumulate INTO dst (aixDeviceCPU.cpp:449-452, 461-465);
//   * argmax picks the first maximum in flat logical order; a NaN is never picked unless it is
//     the first element of its slot (strict '>' scan, aixDeviceCPU.cpp:263-272, 286-295);
//   * argmaxTo stores (flat / src.strides[dim]) % src.shape[dim] with the source's PHYSICAL
//     stride (aixDeviceCPU.cpp:293);
//   * max keeps a NaN only if it is the first element / already in dst (std::max, :250-254).
// The destination slot of a source element is the reference's right-aligned shape walk
// (aixDeviceCPU.cpp:627-649), expressed as per-dim weights computed on the host.

#include "common.hpp"

#include <type_traits>

#include <algorithm>

using namespace aixd;
using namespace aixk;

// Static device memory for the entry point that may not allocate (aixk_reduce_all_noalloc): the partial results of one
// whole-tensor reduction, at most 4096 workgroups x 16 bytes.  Every GPU the library runs on holds its own copy at its
// own address until the process ends.  The name is a host-side stand-in, never a device address: host code uses the
// per-device pointer hipGetSymbolAddress returns (kept in the context), and the kernels take that pointer as an
// argument like the pooled scratch.
static __device__ __align__(256) unsigned char scratch[65536];

namespace aixk {
int resolve_static_scratch(aixk_ctx* ctx)
{
    void* ptr = nullptr;
    AIXK_HIP(hipSetDevice(ctx->device));
    AIXK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    ctx->static_scratch = ptr;
    return AIXK_OK;
}
} // namespace aixk

namespace {

constexpr size_t kStaticScratchBytes = 65536;
constexpr uint64_t kStaticMaxElements = 1ull << 31;

constexpr int kWave = 64;
constexpr int kWaves = kBlock / kWave;

// ---- accumulators ------------------------------------------------------------------------------
template <class T> struct sum_acc { typedef typename traits<T>::W type; };
template <> struct sum_acc<i64> { typedef u64 type; };
template <> struct sum_acc<i32> { typedef u32 type; };
template <> struct sum_acc<i16> { typedef u32 type; };
template <> struct sum_acc<i8>  { typedef u32 type; };
template <> struct sum_acc<u8>  { typedef u32 type; };

template <class W> __device__ __forceinline__ W neg_inf();
template <> __device__ __forceinline__ double neg_inf<double>() { return -__builtin_huge_val(); }
template <> __device__ __forceinline__ float neg_inf<float>() { return -__builtin_huge_valf(); }
template <> __device__ __forceinline__ i64 neg_inf<i64>() { return lowest<i64>(); }
template <> __device__ __forceinline__ i32 neg_inf<i32>() { return lowest<i32>(); }

// flags: 1 = holds a non-NaN value, 2 = the slot's first element is NaN
// idx: flat logical index (argmax sources are limited to 2^31 elements on the host side)
template <class W> struct ArgAcc { W v; u32 idx; u32 flags; };

template <class T> struct SumOp {
    typedef typename sum_acc<T>::type Acc;
    typedef T Out;
    static constexpr bool kTracksIndex = false;
    static __device__ __forceinline__ Acc init() { return (Acc)0; }
    static __device__ __forceinline__ Acc load(T x, u64, bool) { return (Acc)up(x); }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) { return a + b; }
    static __device__ __forceinline__ void step(Acc& a, T x, u64, bool) { a += (Acc)up(x); }
    static __device__ __forceinline__ Acc shfl(Acc v, int d) { return __shfl_down(v, d, kWave); }
};
template <class T> struct MaxOp {
    typedef typename traits<T>::W Acc;
    typedef T Out;
    static constexpr bool kTracksIndex = false;
    static __device__ __forceinline__ Acc init() { return neg_inf<Acc>(); }
    static __device__ __forceinline__ Acc load(T x, u64, bool) { const Acc w = up(x); return w != w ? neg_inf<Acc>() : w; }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b) { return b > a ? b : a; }
    static __device__ __forceinline__ void step(Acc& a, T x, u64, bool) { const Acc w = up(x); if (w > a) a = w; }      // NaN: '>' is false
    static __device__ __forceinline__ Acc shfl(Acc v, int d) { return __shfl_down(v, d, kWave); }
};
template <class T> struct ArgOp {
    typedef typename traits<T>::W W;
    typedef ArgAcc<W> Acc;
    typedef i32 Out;
    static constexpr bool kTracksIndex = true;
    static __device__ __forceinline__ Acc init() { Acc a; a.v = neg_inf<W>(); a.idx = ~0u; a.flags = 0; return a; }
    // In-order scan by one lane: indices only grow, so an equal value never replaces the holder.
    static __device__ __forceinline__ void step(Acc& a, T x, u64 flat, bool first)
    {
        const W w = up(x);
        const bool nan = w != w;
        if (!nan && (!(a.flags & 1u) || w > a.v)) { a.v = w; a.idx = (u32)flat; a.flags |= 1u; }
        if (first && nan) a.flags |= 2u;
    }
    static __device__ __forceinline__ Acc load(T x, u64 flat, bool first)
    {
        Acc a; a.v = up(x); a.idx = (u32)flat;
        const bool nan = a.v != a.v;
        a.flags = nan ? (first ? 2u : 0u) : 1u;
        return a;
    }
    static __device__ __forceinline__ Acc combine(Acc a, Acc b)
    {
        const bool av = a.flags & 1u, bv = b.flags & 1u;
        bool take_b;
        if (av && bv) take_b = b.v > a.v || (b.v == a.v && b.idx < a.idx);
        else if (av != bv) take_b = bv;
        else take_b = b.idx < a.idx;
        Acc r = take_b ? b : a;
        r.flags = (r.flags & 1u) | ((a.flags | b.flags) & 2u);
        return r;
    }
    static __device__ __forceinline__ Acc shfl(Acc v, int d)
    {
        Acc r;
        r.idx = __shfl_down(v.idx, d, kWave);
        r.v = __shfl_down(v.v, d, kWave);
        r.flags = __shfl_down(v.flags, d, kWave);
        return r;
    }
};

template <class Op> __device__ __forceinline__ typename Op::Acc wave_reduce(typename Op::Acc v)
{
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v = Op::combine(v, Op::shfl(v, d));
    return v;                                  // lane 0 holds the result
}

// Result valid in thread 0.  `smem` holds kWaves accumulators.
template <class Op> __device__ __forceinline__ typename Op::Acc block_reduce(typename Op::Acc v, typename Op::Acc* smem)
{
    v = wave_reduce<Op>(v);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();                           // smem may still be in use from a previous round
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = Op::combine(v, smem[w]);
    }
    return v;
}

// ---- landing a finished accumulator --------------------------------------------------------------
struct Finish {
    int into;                // 1: combine with what dst holds (reduceTo/maxTo); 0: overwrite (sum/max);
                             // 2: combine with `init` as if dst held it everywhere (dst itself is never read)
    int onehot;              // argmax: write 1 at the winner's flat index instead of an index per slot
    u64 q_stride, q_extent;  // argmax along a dim: stored index = (flat / q_stride) % q_extent; q_stride 0: store flat
    u64 init;                // into == 2: the value, in the low bytes, in the destination's element type
};

template <class T> __device__ __forceinline__ T held(const Finish& f, const T* dst, u64 slot)
{
    if (f.into == 2) { T v; __builtin_memcpy(&v, &f.init, sizeof(T)); return v; }
    return dst[slot];
}

// `first` = value of the slot's first element (only read by max in overwrite mode);
// `first_flat` = flat logical index of the slot's first element (only read by argmax).
template <class T> __device__ __forceinline__ void land(SumOp<T>, const Finish& f, T* dst, u64 slot, typename SumOp<T>::Acc acc, T, u64)
{
    typedef typename SumOp<T>::Acc A;
    if constexpr (traits<T>::is_int) dst[slot] = f.into ? (T)((A)held(f, dst, slot) + acc) : (T)acc;
    else dst[slot] = f.into ? down<T>(up(held(f, dst, slot)) + acc) : down<T>(acc);
}
template <class T> __device__ __forceinline__ void land(MaxOp<T>, const Finish& f, T* dst, u64 slot, typename MaxOp<T>::Acc acc, T first, u64)
{
    if (f.into) { const T was = held(f, dst, slot); if (acc > up(was)) dst[slot] = down<T>(acc); else if (f.into == 2) dst[slot] = was; }   // NaN in dst: '>' is false, it stays
    else dst[slot] = e_isnan(first) ? first : down<T>(acc);                   // a leading NaN sticks
}
template <class T> __device__ __forceinline__ void land(ArgOp<T>, const Finish& f, i32* dst, u64 slot, typename ArgOp<T>::Acc acc, T, u64 first_flat)
{
    const u64 flat = (acc.flags & 2u) ? first_flat : acc.idx;
    if (f.onehot) dst[flat] = 1;
    else dst[slot] = f.q_stride ? (i32)((flat / f.q_stride) % f.q_extent) : (i32)flat;
}

// ---- whole tensor ----------------------------------------------------------------------------------
template <class Op, class T, class IDX, bool FLAT>
__global__ __launch_bounds__(kBlock) void reduce_all_k(const T* __restrict__ src, typename Op::Out* dst, Space<1> sp, u64 n,
                                                       typename Op::Acc* partials, Finish fin)
{
    typedef typename Op::Acc Acc;
    __shared__ Acc smem[kWaves];
    Acc acc = Op::init();
    if constexpr (FLAT) {
        typedef typename vec16<T>::type V;
        constexpr int VEC = vec16<T>::n;
        constexpr int U = 4;
        const T* base = src + sp.offset[0];
        const V* B = (const V*)base;
        const u64 nvec = n / VEC;
        const u64 tile = (u64)kBlock * U;
        for (u64 v0 = (u64)blockIdx.x * tile; v0 < nvec; v0 += (u64)gridDim.x * tile) {
            V r[U];
#pragma unroll
            for (int k = 0; k < U; ++k) { const u64 v = v0 + (u64)k * kBlock + threadIdx.x; if (v < nvec) r[k] = B[v]; }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const u64 v = v0 + (u64)k * kBlock + threadIdx.x;
                if (v < nvec) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) { const u64 i = v * VEC + e; Op::step(acc, r[k].v[e], i, i == 0); }
                }
            }
        }
        const u64 done = nvec * VEC;
        if (blockIdx.x == 0 && done + threadIdx.x < n) { const u64 i = done + threadIdx.x; Op::step(acc, base[i], i, i == 0); }
    } else {
        for (u64 i = (u64)blockIdx.x * kBlock + threadIdx.x; i < n; i += (u64)gridDim.x * kBlock)
            Op::step(acc, src[locate<1, IDX>(sp, 0, (IDX)i)], i, i == 0);
    }
    acc = block_reduce<Op>(acc, smem);
    if (threadIdx.x == 0) {
        if (gridDim.x == 1) land(Op{}, fin, dst, 0, acc, src[locate<1, IDX>(sp, 0, (IDX)0)], 0);
        else partials[blockIdx.x] = acc;
    }
}

// Second pass of the whole-tensor reduction: one workgroup folds the partials in index order.
// (A kernel boundary instead of an in-kernel "last group finishes" hand-off: the device-scope
// fences that hand-off needs cost more than a second launch on this multi-die part.)
template <class Op, class T, class IDX>
__global__ __launch_bounds__(kBlock) void reduce_all_finish_k(const T* __restrict__ src, typename Op::Out* dst, Space<1> sp,
                                                              const typename Op::Acc* __restrict__ partials, unsigned count, Finish fin)
{
    typedef typename Op::Acc Acc;
    __shared__ Acc smem[kWaves];
    Acc a = Op::init();
    // batches of 8 loads in flight per lane: one after the other the (up to 16) loads of a lane are a chain of memory
    // latencies, most of this kernel's time
    constexpr unsigned U = 8;
    for (unsigned i0 = threadIdx.x; i0 < count; i0 += kBlock * U) {
        Acc r[U];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < count) r[k] = partials[i0 + k * kBlock];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < count) a = Op::combine(a, r[k]);
    }
    a = block_reduce<Op>(a, smem);
    if (threadIdx.x == 0) land(Op{}, fin, dst, 0, a, src[locate<1, IDX>(sp, 0, (IDX)0)], 0);
}

// The partial sums a generated kernel left behind (one per workgroup, in the wide type of T), folded in index order and
// landed as reduceTo lands a sum: the value the destination was initialised with, widened, plus the sum, rounded once.
template <class T>
__global__ __launch_bounds__(kBlock) void sum_partials_k(const typename traits<T>::W* __restrict__ partials, unsigned count, T* dst, u64 init_bits)
{
    typedef SumOp<T> Op;
    typedef typename Op::Acc Acc;
    __shared__ Acc smem[kWaves];
    Acc a = Op::init();
    constexpr unsigned U = 8;
    for (unsigned i0 = threadIdx.x; i0 < count; i0 += kBlock * U) {
        Acc r[U];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < count) r[k] = partials[i0 + k * kBlock];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < count) a = Op::combine(a, r[k]);
    }
    a = block_reduce<Op>(a, smem);
    if (threadIdx.x == 0) {
        T init;
        __builtin_memcpy(&init, &init_bits, sizeof(T));
        *dst = down<T>(up(init) + a);
    }
}

// The same for several sums in one launch (the scalar gradients of a backward pass, which wait for each other): workgroup
// k lands item k.
struct PartialsItem { u64 partials, dst, init; u32 count, pad; };

template <class T>
__global__ __launch_bounds__(kBlock) void sum_partials_many_k(const PartialsItem* __restrict__ items)
{
    typedef SumOp<T> Op;
    typedef typename Op::Acc Acc;
    __shared__ Acc smem[kWaves];
    const PartialsItem it = items[blockIdx.x];
    const Acc* partials = global_ptr<const Acc>(it.partials);
    Acc a = Op::init();
    constexpr unsigned U = 8;
    for (unsigned i0 = threadIdx.x; i0 < it.count; i0 += kBlock * U) {
        Acc r[U];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < it.count) r[k] = partials[i0 + k * kBlock];
#pragma unroll
        for (unsigned k = 0; k < U; ++k) if (i0 + k * kBlock < it.count) a = Op::combine(a, r[k]);
    }
    a = block_reduce<Op>(a, smem);
    if (threadIdx.x == 0) {
        T init;
        __builtin_memcpy(&init, &it.init, sizeof(T));
        *global_ptr<T>(it.dst) = down<T>(up(init) + a);
    }
}

// ---- per-slot plans ------------------------------------------------------------------------------
// Kept dims address the destination slot, reduced dims are folded away.  All extents/strides are
// those of the jointly collapsed (src strides, dst weights) space; `flat` strides are the
// row-major strides of that space, which preserve the flat logical index of the original shape.
struct RedPlan {
    int nk, nr;
    u64 k_ext[kMaxDims], k_src[kMaxDims], k_dst[kMaxDims], k_flat[kMaxDims];
    u64 r_ext[kMaxDims], r_src[kMaxDims], r_flat[kMaxDims];
    u64 src_off, slots, red;
};

struct SlotPos { u64 src, dst, flat; };

// What the column sweeps need of a plan, as plain kernel arguments: read out of the (1 KB) plan in the kernel they
// cost a chain of dependent scalar loads at the head of every workgroup -- several microseconds where a workgroup
// lives for ten.  `slot0` is the position of the first leading slot; with more leading slots (gridDim.z > 1) the
// kernel still walks the plan.
struct OuterDirect { u64 C, R, r_src, r_flat, k_flat; SlotPos slot0; };

__device__ __forceinline__ SlotPos slot_pos(const RedPlan& p, u64 slot, int ndims)
{
    SlotPos s; s.src = p.src_off; s.dst = 0; s.flat = 0;
    for (int d = ndims - 1; d >= 0; --d) {
        const u64 q = slot / p.k_ext[d], c = slot - q * p.k_ext[d];
        s.src += c * p.k_src[d]; s.dst += c * p.k_dst[d]; s.flat += c * p.k_flat[d];
        slot = q;
    }
    return s;
}

// inner: exactly one reduced dim, unit source stride.  One group (wave or workgroup) per slot.
template <class Op, class T, int GROUP, bool VECT>
__global__ __launch_bounds__(kBlock) void reduce_inner_k(const T* __restrict__ src, typename Op::Out* dst, RedPlan p, Finish fin)
{
    typedef typename Op::Acc Acc;
    constexpr int per_block = kBlock / GROUP;
    __shared__ Acc smem[kWaves];
    const int g = threadIdx.x / GROUP, l = threadIdx.x % GROUP;
    const u64 L = p.r_ext[0];
    for (u64 slot0 = (u64)blockIdx.x * per_block; slot0 < p.slots; slot0 += (u64)gridDim.x * per_block) {
        const u64 slot = slot0 + g;
        const bool live = slot < p.slots;
        Acc acc = Op::init();
        SlotPos s = slot_pos(p, live ? slot : 0, p.nk);
        if (live) {
            const T* row = src + s.src;
            if constexpr (VECT) {
                typedef typename vec16<T>::type V;
                constexpr int VEC = vec16<T>::n;
                constexpr int U = 4;
                const V* R = (const V*)row;
                const u64 nvec = L / VEC;
                for (u64 v0 = 0; v0 < nvec; v0 += (u64)GROUP * U) {
                    V r[U];
#pragma unroll
                    for (int k = 0; k < U; ++k) { const u64 v = v0 + (u64)k * GROUP + l; if (v < nvec) r[k] = R[v]; }
#pragma unroll
                    for (int k = 0; k < U; ++k) {
                        const u64 v = v0 + (u64)k * GROUP + l;
                        if (v < nvec) {
#pragma unroll
                            for (int e = 0; e < VEC; ++e) { const u64 j = v * VEC + e; Op::step(acc, r[k].v[e], s.flat + j * p.r_flat[0], j == 0); }
                        }
                    }
                }
            } else {
                for (u64 j = l; j < L; j += GROUP) Op::step(acc, row[j], s.flat + j * p.r_flat[0], j == 0);
            }
        }
        if constexpr (GROUP == kBlock) acc = block_reduce<Op>(acc, smem);
        else acc = wave_reduce<Op>(acc);
        if (live && l == 0) land(Op{}, fin, dst, s.dst, acc, src[s.src], s.flat);
    }
}

// outer: one reduced dim R, innermost kept dim C with unit source stride and unit dst weight,
// optional leading kept dims (blockIdx.z).  Lanes own VEC neighbouring columns; the 4 waves of a
// workgroup take interleaved rows of the workgroup's row chunk (blockIdx.y).
template <class Op, class T, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_outer_k(const T* __restrict__ src, typename Op::Out* dst, RedPlan p,
                                                         u64 rows_per_chunk, typename Op::Acc* partials, Finish fin)
{
    typedef typename Op::Acc Acc;
    typedef vec<T, VEC> V;
    __shared__ Acc sm[kWaves][kWave * VEC];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const u64 C = p.k_ext[p.nk - 1], R = p.r_ext[0];
    const u64 c0 = ((u64)blockIdx.x * kWave + lane) * VEC;
    const SlotPos s = slot_pos(p, blockIdx.z, p.nk - 1);
    const u64 r_begin = (u64)blockIdx.y * rows_per_chunk;
    const u64 r_end = r_begin + rows_per_chunk < R ? r_begin + rows_per_chunk : R;
    Acc acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = Op::init();
    if (c0 < C) {
        const T* col = src + s.src + c0;
        constexpr int U = 4;
        for (u64 r0 = r_begin + wave; r0 < r_end; r0 += (u64)kWaves * U) {
            V x[U];
#pragma unroll
            for (int k = 0; k < U; ++k) { const u64 r = r0 + (u64)k * kWaves; if (r < r_end) x[k] = *(const V*)(col + r * p.r_src[0]); }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const u64 r = r0 + (u64)k * kWaves;
                if (r < r_end) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) Op::step(acc[e], x[k].v[e], r, r == 0);     // the row stands in for the flat index
                }
            }
        }
        // A lane scans one column with ascending rows, so the row orders candidates exactly as the
        // flat index would; the (64-bit) flat index is formed once per column, not per element.
        if constexpr (Op::kTracksIndex) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) if (acc[e].flags & 1u) acc[e].idx = (u32)(s.flat + (u64)acc[e].idx * p.r_flat[0] + (c0 + e) * p.k_flat[p.nk - 1]);
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) sm[wave][lane * VEC + e] = acc[e];
    __syncthreads();
    if (wave == 0 && c0 < C) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            Acc a = sm[0][lane * VEC + e];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) a = Op::combine(a, sm[w][lane * VEC + e]);
            const u64 c = c0 + e;
            if (partials) partials[((u64)blockIdx.z * gridDim.y + blockIdx.y) * C + c] = a;
            else land(Op{}, fin, dst, s.dst + c, a, src[s.src + c], s.flat + c * p.k_flat[p.nk - 1]);
        }
    }
}

// `outer` for wide rows: the four waves sit side by side, so a workgroup reads 256 * VEC
// consecutive columns (4 KB of f32) of each row and every lane owns its columns outright -- no
// LDS stage.  Long contiguous runs per row are what the strided walk needs to approach the
// bandwidth of the unit-stride routes.
template <class Op, class T, int VEC>
__global__ __launch_bounds__(kBlock) void reduce_outer_wide_k(const T* __restrict__ src, typename Op::Out* dst, OuterDirect d, RedPlan p,
                                                              u64 rows_per_chunk, typename Op::Acc* partials, Finish fin)
{
    typedef typename Op::Acc Acc;
    typedef vec<T, VEC> V;
    const u64 C = d.C, R = d.R;
    const u64 c0 = ((u64)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (c0 >= C) return;
    const SlotPos s = gridDim.z == 1 ? d.slot0 : slot_pos(p, blockIdx.z, p.nk - 1);
    const u64 r_begin = (u64)blockIdx.y * rows_per_chunk;
    const u64 r_end = r_begin + rows_per_chunk < R ? r_begin + rows_per_chunk : R;
    Acc acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = Op::init();
    const T* col = src + s.src + c0;
    constexpr int U = 8;
    for (u64 r0 = r_begin; r0 < r_end; r0 += U) {
        V x[U];
#pragma unroll
        for (int k = 0; k < U; ++k) if (r0 + k < r_end) x[k] = *(const V*)(col + (r0 + k) * d.r_src);
#pragma unroll
        for (int k = 0; k < U; ++k) {
            const u64 r = r0 + k;
            if (r < r_end) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) Op::step(acc[e], x[k].v[e], r, r == 0);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        const u64 c = c0 + e;
        if constexpr (Op::kTracksIndex) { if (acc[e].flags & 1u) acc[e].idx = (u32)(s.flat + (u64)acc[e].idx * d.r_flat + c * d.k_flat); }
        if (partials) partials[((u64)blockIdx.z * gridDim.y + blockIdx.y) * C + c] = acc[e];
        else land(Op{}, fin, dst, s.dst + c, acc[e], src[s.src + c], s.flat + c * d.k_flat);
    }
}

// argmaxIndicesTo over a handful of rows with the zero-initialisation of the destination folded in (the pair axis of a
// composed ReLU: fill(0) + argmaxIndicesTo on [2, 4096, 2048]): a lane owns VEC columns, finds the winning row of each
// and writes the whole one-hot column block -- R dense 16-byte stores -- instead of a fill pass plus scattered ones.
template <class T, int VEC>
__global__ __launch_bounds__(kBlock) void argmax_onehot_rows_k(const T* __restrict__ src, i32* __restrict__ dst, RedPlan p)
{
    typedef ArgOp<T> Op;
    typedef typename Op::Acc Acc;
    typedef vec<T, VEC> V;
    typedef vec<i32, VEC> O;
    const u64 C = p.k_ext[p.nk - 1], R = p.r_ext[0];
    const u64 c0 = ((u64)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (c0 >= C) return;
    const SlotPos s = slot_pos(p, blockIdx.z, p.nk - 1);
    const T* col = src + s.src + c0;
    Acc acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = Op::init();
    for (u64 r = 0; r < R; ++r) {
        const V x = *(const V*)(col + r * p.r_src[0]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) Op::step(acc[e], x.v[e], r, r == 0);
    }
    u32 winner[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) winner[e] = (acc[e].flags & 2u) ? 0u : acc[e].idx;      // a leading NaN wins (as land() has it)
    for (u64 r = 0; r < R; ++r) {
        O out;
#pragma unroll
        for (int e = 0; e < VEC; ++e) out.v[e] = winner[e] == (u32)r ? 1 : 0;
        *(O*)(dst + s.flat + r * p.r_flat[0] + c0) = out;
    }
}

// argmaxIndicesTo along a unit-stride dim with the zero-initialisation folded in (the mask of a softmax's max() backward:
// fill(0) + argmaxIndicesTo over rows of 512): a wave finds the winner of a row -- the arithmetic of
// reduce_inner_k<ArgOp, T, kWave, .> -- and writes the row's one-hot block densely, 16 bytes per lane and step.
template <class T, bool VECT>
__global__ __launch_bounds__(kBlock) void argmax_onehot_inner_k(const T* __restrict__ src, i32* __restrict__ dst, RedPlan p)
{
    typedef ArgOp<T> Op;
    typedef typename Op::Acc Acc;
    typedef typename vec16<T>::type V;
    constexpr int VEC = vec16<T>::n;
    typedef vec<i32, 4> O4;
    const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
    const u64 L = p.r_ext[0];
    for (u64 slot = (u64)blockIdx.x * kWaves + w; slot < p.slots; slot += (u64)gridDim.x * kWaves) {
        const SlotPos s = slot_pos(p, slot, p.nk);
        const T* row = src + s.src;
        Acc acc = Op::init();                                                           // candidates carry their position in the row
        if constexpr (VECT) {
            for (u64 v = l; v < L / VEC; v += kWave) {
                const V x = *(const V*)(row + v * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) { const u64 j = v * VEC + e; Op::step(acc, x.v[e], j, j == 0); }
            }
        } else {
            for (u64 j = l; j < L; j += kWave) Op::step(acc, row[j], j, j == 0);
        }
        acc = wave_reduce<Op>(acc);
        const u32 mine = (acc.flags & 2u) ? 0u : acc.idx;                               // a leading NaN wins (as land() has it)
        const u32 winner = __shfl(mine, 0, kWave);
        i32* out = dst + s.flat;                                                         // the row is contiguous in the flat order
        for (u64 j0 = (u64)l * 4; j0 < L; j0 += (u64)kWave * 4) {
            O4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v.v[e] = (u32)(j0 + e) == winner ? 1 : 0;
            *(O4*)(out + j0) = v;
        }
    }
}

// The same for several tensors of dense rows in one launch (the masks of max()'s backward, head after head): item k's
// addresses and extents come from a table in device memory, its share of the grid from `starts`.
struct OnehotItem { u64 src, dst, rows, len; };

template <class T>
__global__ __launch_bounds__(kBlock) void argmax_onehot_inner_many_k(const OnehotItem* __restrict__ items, const u32* __restrict__ starts, u32 count)
{
    typedef ArgOp<T> Op;
    typedef typename Op::Acc Acc;
    typedef typename vec16<T>::type V;
    constexpr int VEC = vec16<T>::n;
    typedef vec<i32, 4> O4;
    u32 lo = 0, hi = count;
    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (starts[mid] <= blockIdx.x) lo = mid; else hi = mid; }
    const OnehotItem it = items[lo];
    const u32 first = starts[lo], share = starts[lo + 1] - first;
    const T* src = global_ptr<const T>(it.src);
    i32* dst = global_ptr<i32>(it.dst);
    const int w = threadIdx.x / kWave, l = threadIdx.x % kWave;
    const u64 L = it.len;
    for (u64 slot = (u64)(blockIdx.x - first) * kWaves + w; slot < it.rows; slot += (u64)share * kWaves) {
        const T* row = src + slot * L;
        Acc acc = Op::init();
        for (u64 v = l; v < L / VEC; v += kWave) {
            const V x = *(const V*)(row + v * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) { const u64 j = v * VEC + e; Op::step(acc, x.v[e], j, j == 0); }
        }
        acc = wave_reduce<Op>(acc);
        const u32 mine = (acc.flags & 2u) ? 0u : acc.idx;
        const u32 winner = __shfl(mine, 0, kWave);
        i32* out = dst + slot * L;
        for (u64 j0 = (u64)l * 4; j0 < L; j0 += (u64)kWave * 4) {
            O4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v.v[e] = (u32)(j0 + e) == winner ? 1 : 0;
            *(O4*)(out + j0) = v;
        }
    }
}

// Column sums of several dense matrices in one launch (the gradients of biases and of LayerNorm's parameters: one
// reduceTo each, asked for throughout a backward pass and read only at its end).  Item k is rows x cols elements with
// `pitch` elements between rows; dst[c] = init + the sum down column c.  Stage one: a workgroup takes 256 columns (a
// lane owns 4 neighbours, the four waves take interleaved rows) of one chunk of an item's rows and leaves its sums, in
// the accumulator's type, in `partials`; stage two adds up the chunks of a column, adds the initial value, rounds once.
struct ColsumItem {
    u64 src, dst, rows, cols, pitch, init;
    u64 partials;                       // index of the item's first partial sum
    u32 first_wg, tiles, chunks, rows_per_chunk, first_col, pad;
};

template <class T>
__global__ __launch_bounds__(kBlock) void sum_columns_many_k(const ColsumItem* __restrict__ items, u32 count, typename SumOp<T>::Acc* partials)
{
    typedef SumOp<T> Op;
    typedef typename Op::Acc Acc;
    typedef vec<T, 4> V;
    __shared__ Acc sm[kWaves][kWave * 4];
    u32 lo = 0, hi = count;
    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (items[mid].first_wg <= blockIdx.x) lo = mid; else hi = mid; }
    const ColsumItem it = items[lo];
    const u32 local = blockIdx.x - it.first_wg, tile = local % it.tiles, chunk = local / it.tiles;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const u64 c0 = ((u64)tile * kWave + lane) * 4;
    const u64 r_begin = (u64)chunk * it.rows_per_chunk;
    const u64 r_end = r_begin + it.rows_per_chunk < it.rows ? r_begin + it.rows_per_chunk : it.rows;
    Acc acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = Op::init();
    if (c0 < it.cols) {                                     // cols is a multiple of 4: a lane's columns are all there or none
        const T* col = global_ptr<const T>(it.src) + c0;
        constexpr int U = 4;
        for (u64 r0 = r_begin + wave; r0 < r_end; r0 += (u64)kWaves * U) {
            V x[U];
#pragma unroll
            for (int k = 0; k < U; ++k) { const u64 r = r0 + (u64)k * kWaves; if (r < r_end) x[k] = *(const V*)(col + r * it.pitch); }
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const u64 r = r0 + (u64)k * kWaves;
                if (r < r_end) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) Op::step(acc[e], x[k].v[e], r, false);
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) sm[wave][lane * 4 + e] = acc[e];
    __syncthreads();
    if (wave == 0 && c0 < it.cols) {
        Acc* out = partials + it.partials + (u64)chunk * it.cols + c0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Acc a = sm[0][lane * 4 + e];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) a = Op::combine(a, sm[w][lane * 4 + e]);
            out[e] = a;
        }
    }
}

template <class T>
__global__ __launch_bounds__(kBlock) void sum_columns_finish_many_k(const ColsumItem* __restrict__ items, u32 count, const typename SumOp<T>::Acc* __restrict__ partials,
                                                                    u32 columns)
{
    typedef SumOp<T> Op;
    typedef typename Op::Acc Acc;
    const u32 g = blockIdx.x * kBlock + threadIdx.x;
    if (g >= columns) return;
    u32 lo = 0, hi = count;
    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (items[mid].first_col <= g) lo = mid; else hi = mid; }
    const ColsumItem it = items[lo];
    const u64 c = g - it.first_col;
    const Acc* col = partials + it.partials + c;
    Acc a = Op::init();
    u32 k = 0;
    for (; k + 4 <= it.chunks; k += 4) {                    // four loads in flight
        const Acc x0 = col[(u64)k * it.cols], x1 = col[(u64)(k + 1) * it.cols], x2 = col[(u64)(k + 2) * it.cols], x3 = col[(u64)(k + 3) * it.cols];
        a = Op::combine(Op::combine(Op::combine(Op::combine(a, x0), x1), x2), x3);
    }
    for (; k < it.chunks; ++k) a = Op::combine(a, col[(u64)k * it.cols]);
    T init;
    __builtin_memcpy(&init, &it.init, sizeof(T));
    global_ptr<T>(it.dst)[c] = down<T>((Acc)up(init) + a);
}

// argmax down the columns of wide rows with the rows split into chunks: the record a lane keeps per column is the
// pair (value, row) and the scan is a bare `x > best` -- three instructions per element against the seven of
// ArgOp::step -- and the partial records are 8 bytes instead of 12 (16 for 8-byte elements).  A strict `>` from minus
// infinity never picks a NaN and keeps the first of equal values; what it cannot tell apart -- a column chunk whose
// values are all NaN or the lowest value of the type -- is left as row = ~0 and settled by argmax_cols_finish_k.
template <class W> struct ColRec { W v; u32 row; };
template <> struct ColRec<double> { double v; u32 row; u32 pad; };
template <> struct ColRec<i64> { i64 v; u32 row; u32 pad; };

template <class T, int VEC>
__global__ __launch_bounds__(kBlock) void argmax_cols_k(const T* __restrict__ src, OuterDirect d, RedPlan p, u64 rows_per_chunk, ColRec<typename traits<T>::W>* __restrict__ partials)
{
    typedef typename traits<T>::W W;
    typedef vec<T, VEC> V;
    const u64 C = d.C, R = d.R;
    const u64 c0 = ((u64)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (c0 >= C) return;
    const SlotPos s = gridDim.z == 1 ? d.slot0 : slot_pos(p, blockIdx.z, p.nk - 1);
    const u64 r_begin = (u64)blockIdx.y * rows_per_chunk;
    const u64 r_end = r_begin + rows_per_chunk < R ? r_begin + rows_per_chunk : R;
    W best[VEC]; u32 row[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { best[e] = neg_inf<W>(); row[e] = ~0u; }
    const T* col = src + s.src + c0;
    constexpr int U = 8;
    for (u64 r0 = r_begin; r0 < r_end; r0 += U) {
        V x[U];
#pragma unroll
        for (int k = 0; k < U; ++k) if (r0 + k < r_end) x[k] = *(const V*)(col + (r0 + k) * d.r_src);
#pragma unroll
        for (int k = 0; k < U; ++k) {
            if (r0 + k < r_end) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) { const W w = up(x[k].v[e]); const bool more = w > best[e]; best[e] = more ? w : best[e]; row[e] = more ? (u32)(r0 + k) : row[e]; }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        ColRec<W> rec{};
        rec.v = best[e]; rec.row = row[e];
        partials[((u64)blockIdx.z * gridDim.y + blockIdx.y) * C + c0 + e] = rec;
    }
}

// Second stage: a lane folds the chunk records of one column in chunk order (rows ascend with the chunks, so a later
// record wins only with a strictly greater value), all its loads in flight at once, and lands the result.  A leading
// NaN wins, as everywhere in this file.  A column no chunk found anything in holds only NaNs and lowest values: if its
// first element is not a NaN it is such a lowest value and the first of them, so row 0 wins there too.
template <class T>
__global__ __launch_bounds__(kBlock) void argmax_cols_finish_k(const T* __restrict__ src, i32* dst, OuterDirect d, RedPlan p, u64 slots, unsigned chunks,
                                                               const ColRec<typename traits<T>::W>* __restrict__ partials, Finish fin)
{
    typedef typename traits<T>::W W;
    typedef ColRec<W> Rec;
    __shared__ Rec sm[kWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const u64 C = d.C;
    const u64 slot = (u64)blockIdx.x * kWave + lane;           // 64 columns per workgroup; wave w folds chunks w, w + 4, ...
    const bool live = slot < slots;
    const u64 o = live ? slot / C : 0, c = live ? slot - o * C : 0;
    W best = neg_inf<W>(); u32 row = ~0u;
    if (live) {
        const Rec* col = partials + o * chunks * C + c;
        constexpr unsigned U = 8;
        for (unsigned k0 = wave; k0 < chunks; k0 += kWaves * U) {
            Rec r[U];
#pragma unroll
            for (unsigned k = 0; k < U; ++k) if (k0 + k * kWaves < chunks) r[k] = col[(u64)(k0 + k * kWaves) * C];
#pragma unroll
            for (unsigned k = 0; k < U; ++k) if (k0 + k * kWaves < chunks && r[k].row != ~0u && (row == ~0u || r[k].v > best)) { best = r[k].v; row = r[k].row; }
        }
    }
    Rec mine{}; mine.v = best; mine.row = row;
    sm[wave][lane] = mine;
    __syncthreads();
    if (wave != 0 || !live) return;
    // the waves hold interleaved chunks: among equal values the lower row wins
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
        const Rec r = sm[w][lane];
        if (r.row != ~0u && (row == ~0u || r.v > best || (r.v == best && r.row < row))) { best = r.v; row = r.row; }
    }
    const SlotPos s = slots == C ? d.slot0 : slot_pos(p, o, p.nk - 1);
    const T* first = src + s.src + c;
    if (e_isnan(*first) || row == ~0u) row = 0;
    const u64 flat = s.flat + (u64)row * d.r_flat + c * d.k_flat;
    if (fin.onehot) dst[flat] = 1;
    else dst[s.dst + c] = fin.q_stride ? (i32)((flat / fin.q_stride) % fin.q_extent) : (i32)flat;
}

// second stage of `outer` when rows were split over several workgroups: 64 slots per workgroup,
// the four waves take every fourth chunk (independent loads in flight), LDS folds the four.
template <class Op, class T>
__global__ __launch_bounds__(kBlock) void reduce_outer_finish_k(const T* __restrict__ src, typename Op::Out* dst, RedPlan p,
                                                                unsigned chunks, const typename Op::Acc* __restrict__ partials, Finish fin)
{
    typedef typename Op::Acc Acc;
    __shared__ Acc sm[kWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const u64 C = p.k_ext[p.nk - 1];
    for (u64 base = (u64)blockIdx.x * kWave; base < p.slots; base += (u64)gridDim.x * kWave) {
        const u64 slot = base + lane;
        const bool live = slot < p.slots;
        const u64 o = live ? slot / C : 0, c = live ? slot - o * C : 0;
        Acc a = Op::init();
        if (live) {
            const Acc* col = partials + o * chunks * C + c;
            unsigned k = wave;
            for (; k + 3 * kWaves < chunks; k += 4 * kWaves) {
                const Acc x0 = col[(u64)k * C], x1 = col[(u64)(k + kWaves) * C], x2 = col[(u64)(k + 2 * kWaves) * C], x3 = col[(u64)(k + 3 * kWaves) * C];
                a = Op::combine(Op::combine(Op::combine(Op::combine(a, x0), x1), x2), x3);
            }
            for (; k < chunks; k += kWaves) a = Op::combine(a, col[(u64)k * C]);
        }
        __syncthreads();
        sm[wave][lane] = a;
        __syncthreads();
        if (wave == 0 && live) {
#pragma unroll
            for (int w = 1; w < kWaves; ++w) a = Op::combine(a, sm[w][lane]);
            const SlotPos s = slot_pos(p, o, p.nk - 1);
            land(Op{}, fin, dst, s.dst + c, a, src[s.src + c], s.flat + c * p.k_flat[p.nk - 1]);
        }
    }
}

// generic: any mix of kept / reduced dims.  group = 1 lane per slot, or a whole workgroup per slot.
template <class Op, class T>
__global__ __launch_bounds__(kBlock) void reduce_generic_k(const T* __restrict__ src, typename Op::Out* dst, RedPlan p, int block_per_slot, Finish fin)
{
    typedef typename Op::Acc Acc;
    __shared__ Acc smem[kWaves];
    const u64 groups = block_per_slot ? gridDim.x : (u64)gridDim.x * kBlock;
    const u64 gid = block_per_slot ? blockIdx.x : (u64)blockIdx.x * kBlock + threadIdx.x;
    const u64 l = block_per_slot ? threadIdx.x : 0, step = block_per_slot ? kBlock : 1;
    const u64 rounds = (p.slots + groups - 1) / groups;      // same trip count for every lane of a workgroup
    for (u64 it = 0; it < rounds; ++it) {
        const u64 slot = it * groups + gid;
        const bool live = slot < p.slots;
        const SlotPos s = slot_pos(p, live ? slot : 0, p.nk);
        Acc acc = Op::init();
        if (live) {
            for (u64 j = l; j < p.red; j += step) {
                u64 rest = j, pos = s.src, flat = s.flat;
                for (int d = p.nr - 1; d >= 0; --d) {
                    const u64 q = rest / p.r_ext[d], c = rest - q * p.r_ext[d];
                    pos += c * p.r_src[d]; flat += c * p.r_flat[d];
                    rest = q;
                }
                Op::step(acc, src[pos], flat, j == 0);
            }
        }
        if (block_per_slot) acc = block_reduce<Op>(acc, smem);
        if (live && l == 0) land(Op{}, fin, dst, s.dst, acc, src[s.src], s.flat);
    }
}

// ---- host side -------------------------------------------------------------------------------------
// Per source dim, the multiplier into the flat destination index (0 = reduced away); the walk of
// aixDeviceCPU.cpp:627-649.
void dst_weights(const uint64_t* dshape, int drank, const uint64_t* sshape, int srank, uint64_t* weight)
{
    int j = drank - 1;
    uint64_t run = 1;
    for (int i = srank - 1; i >= 0; --i) {
        weight[i] = 0;
        if (j >= 0 && dshape[j] == sshape[i]) { weight[i] = run; run *= dshape[j]; --j; }
        else if (j >= 0 && dshape[j] == 1) { --j; }
    }
}

bool make_plan(const aixhip_tensor* src, const uint64_t* weight, RedPlan* p)
{
    const uint64_t* strides[2] = {src->strides, weight};
    const uint64_t offsets[2] = {src->offset, 0};
    Space<2> sp;
    if (!collapse<2>(src->rank, src->shape, strides, offsets, &sp)) return false;
    uint64_t flat[kMaxDims];
    row_major_strides(sp.rank, sp.shape, flat);
    std::memset(p, 0, sizeof(*p));
    p->src_off = sp.offset[0];
    p->slots = 1; p->red = 1;
    for (int d = 0; d < sp.rank; ++d) {
        if (sp.stride[1][d] != 0) {
            p->k_ext[p->nk] = sp.shape[d]; p->k_src[p->nk] = sp.stride[0][d]; p->k_dst[p->nk] = sp.stride[1][d]; p->k_flat[p->nk] = flat[d];
            ++p->nk; p->slots *= sp.shape[d];
        } else {
            p->r_ext[p->nr] = sp.shape[d]; p->r_src[p->nr] = sp.stride[0][d]; p->r_flat[p->nr] = flat[d];
            ++p->nr; p->red *= sp.shape[d];
        }
    }
    for (int d = p->nk; d < kMaxDims; ++d) p->k_ext[d] = 1;
    for (int d = p->nr; d < kMaxDims; ++d) p->r_ext[d] = 1;
    return true;
}

template <class Op, class T>
int run_all(aixk_ctx* ctx, const aixhip_tensor* a, typename Op::Out* dst, const Finish& fin, void* fixed = nullptr);

// Does argmax_onehot_rows_k take this plan?  One reduced dim of fewer than 8 rows, the innermost kept dim dense on both
// sides, everything aligned for VEC-wide accesses.
// Does argmax_onehot_inner_k take this plan?  One reduced dim with unit source stride that is also the innermost dim of
// the flat order, rows of a multiple of 4 elements that start 16-byte aligned in the destination.
inline bool onehot_inner_route(const RedPlan& p, const void* dst)
{
    if (!(p.nk >= 1 && p.nr == 1 && p.r_src[0] == 1 && p.r_flat[0] == 1 && p.red >= 32 && p.red % 4 == 0 && p.red < (1ull << 31))) return false;
    if (!aligned16(dst)) return false;
    for (int d = 0; d < p.nk; ++d) if (p.k_flat[d] % 4) return false;
    return true;
}

template <class T>
bool onehot_rows_route(const RedPlan& p, const T* ps, const void* dst)
{
    constexpr int VEC16 = vec16<T>::n, VEC = VEC16 < 4 ? VEC16 : 4;
    if (!(p.nr == 1 && p.nk >= 1 && p.k_src[p.nk - 1] == 1 && p.k_dst[p.nk - 1] == 1 && p.k_flat[p.nk - 1] == 1 && p.red >= 2)) return false;
    const uint64_t C = p.k_ext[p.nk - 1], R = p.r_ext[0], O = p.slots / C;
    if (R >= 8 || O > 65535 || C % VEC != 0 || C / VEC / kBlock >= (1ull << 31)) return false;
    if (((uintptr_t)(ps + p.src_off) % (sizeof(T) * VEC)) != 0 || p.r_src[0] % VEC != 0 || p.r_flat[0] % VEC != 0 || !aligned16(dst)) return false;
    for (int d = 0; d + 1 < p.nk; ++d) if (p.k_src[d] % VEC || p.k_flat[d] % VEC) return false;
    return true;
}

inline OuterDirect outer_direct(const RedPlan& p)
{
    OuterDirect d;
    d.C = p.k_ext[p.nk - 1]; d.R = p.r_ext[0]; d.r_src = p.r_src[0]; d.r_flat = p.r_flat[0]; d.k_flat = p.k_flat[p.nk - 1];
    d.slot0.src = p.src_off; d.slot0.dst = 0; d.slot0.flat = 0;
    return d;
}

template <class Op, class T>
int run_plan(aixk_ctx* ctx, const aixhip_tensor* src, typename Op::Out* dst, const RedPlan& p, const Finish& fin)
{
    typedef typename Op::Acc Acc;
    constexpr int VEC16 = vec16<T>::n;
    const T* ps = (const T*)src->data;
    const unsigned cus = (unsigned)ctx->cus;
    hipStream_t st = ctx->stream;
    if (p.slots == 0 || p.red == 0) return AIXK_OK;

    // nothing kept: the whole source folds into dst[0]
    if (p.nk == 0) return run_all<Op, T>(ctx, src, dst, fin);

    // inner: one reduced dim with unit source stride
    if constexpr (Op::kTracksIndex) {
        if (fin.onehot == 2 && onehot_inner_route(p, dst)) {
            // a row per wave, all rows in flight at once
            bool vect = p.red % VEC16 == 0 && aligned16(ps + p.src_off);
            for (int d = 0; d < p.nk; ++d) if (p.k_src[d] % VEC16) vect = false;
            const unsigned rows_grid = grid_for(p.slots, kWaves, 1u << 30);
            if (vect) hipLaunchKernelGGL((argmax_onehot_inner_k<T, true>), dim3(rows_grid), dim3(kBlock), 0, st, ps, (i32*)dst, p);
            else hipLaunchKernelGGL((argmax_onehot_inner_k<T, false>), dim3(rows_grid), dim3(kBlock), 0, st, ps, (i32*)dst, p);
            AIXK_HIP(hipGetLastError());
            return AIXK_OK;
        }
    }
    if (p.nr == 1 && p.r_src[0] == 1 && p.red >= 32) {
        bool vect = p.red % VEC16 == 0 && aligned16(ps + p.src_off);
        for (int d = 0; d < p.nk; ++d) if (p.k_src[d] % VEC16) vect = false;
        const bool big = p.red >= 2048;
        const uint64_t per_block = big ? 1 : kWaves;
        const unsigned grid = grid_for(p.slots, (unsigned)per_block, cus * 64u);
        if (big) {
            if (vect) hipLaunchKernelGGL((reduce_inner_k<Op, T, kBlock, true>), dim3(grid), dim3(kBlock), 0, st, ps, dst, p, fin);
            else hipLaunchKernelGGL((reduce_inner_k<Op, T, kBlock, false>), dim3(grid), dim3(kBlock), 0, st, ps, dst, p, fin);
        } else {
            if (vect) hipLaunchKernelGGL((reduce_inner_k<Op, T, kWave, true>), dim3(grid), dim3(kBlock), 0, st, ps, dst, p, fin);
            else hipLaunchKernelGGL((reduce_inner_k<Op, T, kWave, false>), dim3(grid), dim3(kBlock), 0, st, ps, dst, p, fin);
        }
        AIXK_HIP(hipGetLastError());
        return AIXK_OK;
    }
    // outer: one reduced dim, innermost kept dim dense on both sides
    if (p.nr == 1 && p.nk >= 1 && p.k_src[p.nk - 1] == 1 && p.k_dst[p.nk - 1] == 1 && p.k_flat[p.nk - 1] == 1 && p.red >= 2) {
        const uint64_t C = p.k_ext[p.nk - 1], R = p.r_ext[0], O = p.slots / C;
        constexpr int VEC = VEC16 < 4 ? VEC16 : 4;
        bool vect = C % VEC == 0 && ((uintptr_t)(ps + p.src_off) % (sizeof(T) * VEC)) == 0 && p.r_src[0] % VEC == 0;
        for (int d = 0; d + 1 < p.nk; ++d) if (p.k_src[d] % VEC) vect = false;
        const int v = vect ? VEC : 1;
        // one-hot argmax over a handful of rows whose destination this call also has to zero: written densely in one pass
        if constexpr (Op::kTracksIndex) {
            if (fin.onehot == 2 && onehot_rows_route<T>(p, ps, dst)) {
                const uint64_t tiles = (C / VEC + kBlock - 1) / kBlock;
                hipLaunchKernelGGL((argmax_onehot_rows_k<T, VEC>), dim3((unsigned)tiles, 1, (unsigned)O), dim3(kBlock), 0, st, ps, (i32*)dst, p);
                AIXK_HIP(hipGetLastError());
                return AIXK_OK;
            }
        }
        // wide rows: workgroups of 256 * v columns, rows split into chunks of at least 16 (a handful of rows --
        // the pair axis of a composed ReLU, say -- is one chunk: every lane folds its columns outright)
        if (vect && C >= (uint64_t)kBlock * v * 2 && (R >= 64 || R < 8) && O <= 65535) {
            const uint64_t tiles = (C + (uint64_t)kBlock * v - 1) / ((uint64_t)kBlock * v);
            // two workgroups per compute unit: the sweep runs at the same pace from 32 to 256 chunks (41 us on [8192, 8192]
            // f32), the second stage costs a microsecond per 30 chunks, and with one workgroup per compute unit the pace
            // depends on details of the instruction stream (41 or 47-49 us for near-identical kernels)
            const uint64_t want = (uint64_t)cus * 2;
            uint64_t chunks = tiles * O < want ? std::min<uint64_t>({(want + tiles * O - 1) / (tiles * O), (R + 15) / 16, (uint64_t)65535}) : 1;
            while (chunks > 1 && chunks * O * C * sizeof(Acc) > ctx->scratch_bytes) chunks /= 2;
            uint64_t rows_per_chunk = (R + chunks - 1) / chunks;
            // The workgroups of a launch start together and walk their chunks in step.  If the chunks lie a multiple of
            // 4 MiB apart (128 rows of 32 KiB, say) all of them ask the same memory channels for different DRAM rows at
            // every step; the same happens within a few rows of such a distance.  Chunks are lengthened until their
            // distance is at least 8 rows away from every multiple of 4 MiB (measured on [8192, 8192] f32: 128 rows per
            // chunk 50 us, 127 or 129 rows 47-49 us, 136 rows 41 us).
            if (chunks > 1) {
                const uint64_t pitch = p.r_src[0] * sizeof(T), period = 4ull << 20, guard = 8 * pitch;
                if (pitch > 0 && guard * 2 < period)
                    for (int tries = 0; tries < 64; ++tries) {
                        const uint64_t phase = (rows_per_chunk * pitch) % period;
                        if (phase >= guard && phase <= period - guard) break;
                        ++rows_per_chunk;
                    }
            }
            chunks = (R + rows_per_chunk - 1) / rows_per_chunk;
            if constexpr (Op::kTracksIndex) {
                // the (value, row) sweep with its own second stage
                typedef ColRec<typename traits<T>::W> Rec;
                if (chunks > 1 && fin.onehot != 2 && R < (1ull << 32) - 1 && chunks * O * C * sizeof(Rec) <= ctx->scratch_bytes) {
                    Rec* recs = (Rec*)ctx->scratch;
                    hipLaunchKernelGGL((argmax_cols_k<T, VEC>), dim3((unsigned)tiles, (unsigned)chunks, (unsigned)O), dim3(kBlock), 0, st, ps, outer_direct(p), p, (u64)rows_per_chunk, recs);
                    AIXK_HIP(hipGetLastError());
                    hipLaunchKernelGGL((argmax_cols_finish_k<T>), dim3((unsigned)((p.slots + kWave - 1) / kWave)), dim3(kBlock), 0, st, ps, (i32*)dst, outer_direct(p), p, (u64)p.slots, (unsigned)chunks, (const Rec*)recs, fin);
                    AIXK_HIP(hipGetLastError());
                    return AIXK_OK;
                }
            }
            Acc* partials = chunks > 1 ? (Acc*)ctx->scratch : nullptr;
            hipLaunchKernelGGL((reduce_outer_wide_k<Op, T, VEC>), dim3((unsigned)tiles, (unsigned)chunks, (unsigned)O), dim3(kBlock), 0, st,
                               ps, dst, outer_direct(p), p, (u64)rows_per_chunk, partials, fin);
            AIXK_HIP(hipGetLastError());
            if (chunks > 1) {
                hipLaunchKernelGGL((reduce_outer_finish_k<Op, T>), dim3(grid_for(p.slots, kWave, cus * 8u)), dim3(kBlock), 0, st,
                                   ps, dst, p, (unsigned)chunks, (const Acc*)partials, fin);
                AIXK_HIP(hipGetLastError());
            }
            return AIXK_OK;
        }
        const uint64_t col_tiles = (C + (uint64_t)kWave * v - 1) / ((uint64_t)kWave * v);
        if (O <= 65535 && col_tiles < (1ull << 31)) {
            // split rows until the launch has enough workgroups to fill the chip
            uint64_t chunks = 1;
            const uint64_t want = (uint64_t)cus * 8;
            if (col_tiles * O < want) chunks = std::min<uint64_t>({(want + col_tiles * O - 1) / (col_tiles * O), (R + 63) / 64, (uint64_t)65535});
            if (chunks < 1) chunks = 1;
            while (chunks > 1 && chunks * O * C * sizeof(Acc) > ctx->scratch_bytes) chunks /= 2;
            const uint64_t rows_per_chunk = (R + chunks - 1) / chunks;
            chunks = (R + rows_per_chunk - 1) / rows_per_chunk;
            Acc* partials = chunks > 1 ? (Acc*)ctx->scratch : nullptr;
            const dim3 grid((unsigned)col_tiles, (unsigned)chunks, (unsigned)O);
            if (vect) hipLaunchKernelGGL((reduce_outer_k<Op, T, VEC>), grid, dim3(kBlock), 0, st, ps, dst, p, (u64)rows_per_chunk, partials, fin);
            else hipLaunchKernelGGL((reduce_outer_k<Op, T, 1>), grid, dim3(kBlock), 0, st, ps, dst, p, (u64)rows_per_chunk, partials, fin);
            AIXK_HIP(hipGetLastError());
            if (chunks > 1) {
                hipLaunchKernelGGL((reduce_outer_finish_k<Op, T>), dim3(grid_for(p.slots, kWave, cus * 8u)), dim3(kBlock), 0, st,
                                   ps, dst, p, (unsigned)chunks, (const Acc*)partials, fin);
                AIXK_HIP(hipGetLastError());
            }
            return AIXK_OK;
        }
    }
    // generic
    const int block_per_slot = p.red >= 256 && p.slots < (uint64_t)cus * 64;
    const unsigned grid = block_per_slot ? grid_for(p.slots, 1, cus * 16u) : grid_for(p.slots, kBlock, cus * 16u);
    hipLaunchKernelGGL((reduce_generic_k<Op, T>), dim3(grid), dim3(kBlock), 0, st, ps, dst, p, block_per_slot, fin);
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

// `fixed` = the per-device address of the static scratch array when the caller may not allocate (then the launch must be
// the one the pooled scratch would get, or the call is refused), else null.
template <class Op, class T>
int run_all(aixk_ctx* ctx, const aixhip_tensor* a, typename Op::Out* dst, const Finish& fin, void* fixed)
{
    typedef typename Op::Acc Acc;
    const uint64_t n = a->size;
    Space<1> sp;
    if (!collapse1(a, &sp)) return fail(AIXK_EINVAL, "view does not collapse to %d dims", kMaxDims);
    const T* ps = (const T*)a->data;
    const bool flat = (sp.rank == 0 || (sp.rank == 1 && sp.stride[0][0] == 1)) && aligned16(ps + sp.offset[0]);
    const bool small = n < (1ull << 31) && view_extent(a) < (1ull << 31);
    constexpr int VEC = vec16<T>::n;
    // with the fixed scratch the grid is cut to what it holds (4096 partial results of 16 bytes: every dtype on parts of up to
    // 256 compute units runs the grid of the allocating entry point and lands the same bits; beyond that the partial
    // sums of float types are grouped differently)
    unsigned max_blocks = (unsigned)std::min<uint64_t>((uint64_t)ctx->cus * 16, (fixed ? kStaticScratchBytes : ctx->scratch_bytes) / sizeof(Acc));
    const unsigned grid = flat ? grid_for(n / VEC + 1, kBlock * 4, max_blocks) : grid_for(n, kBlock * 4, max_blocks);
    Acc* partials = (Acc*)(fixed ? fixed : ctx->scratch);
    if (flat) hipLaunchKernelGGL((reduce_all_k<Op, T, u32, true>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, dst, sp, (u64)n, partials, fin);
    else if (small) hipLaunchKernelGGL((reduce_all_k<Op, T, u32, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, dst, sp, (u64)n, partials, fin);
    else hipLaunchKernelGGL((reduce_all_k<Op, T, u64, false>), dim3(grid), dim3(kBlock), 0, ctx->stream, ps, dst, sp, (u64)n, partials, fin);
    AIXK_HIP(hipGetLastError());
    if (grid > 1) {
        if (small) hipLaunchKernelGGL((reduce_all_finish_k<Op, T, u32>), dim3(1), dim3(kBlock), 0, ctx->stream, ps, dst, sp, (const Acc*)partials, grid, fin);
        else hipLaunchKernelGGL((reduce_all_finish_k<Op, T, u64>), dim3(1), dim3(kBlock), 0, ctx->stream, ps, dst, sp, (const Acc*)partials, grid, fin);
        AIXK_HIP(hipGetLastError());
    }
    return AIXK_OK;
}

} // namespace

extern "C" {

static int32_t reduce_all_impl(aixk_ctx* ctx, int kind, const aixhip_tensor* a, const aixhip_tensor* out, void* fixed)
{
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(out), "reduce: bad operand descriptor");
    AIXK_REQUIRE(out->data != nullptr, "reduce: null result");
    if (a->size == 0 && kind == AIXK_SUM) return aixk_zero(ctx, out->data, aixk_dtype_size(out->dtype));
    AIXK_REQUIRE(a->size > 0 && a->size == numel(a), "reduce: empty or inconsistent source");
    Finish fin{0, 0, 0, 0, 0};
    if (kind == AIXK_SUM || kind == AIXK_MAX) {
        AIXK_REQUIRE(a->dtype == out->dtype, "reduce: operand must have the result's element type");
        return by_dtype(out->dtype, [&](auto tag) {
            typedef decltype(tag) T;
            if (kind == AIXK_SUM) return run_all<SumOp<T>, T>(ctx, a, (T*)out->data, fin, fixed);
            return run_all<MaxOp<T>, T>(ctx, a, (T*)out->data, fin, fixed);
        });
    }
    AIXK_REQUIRE(kind == AIXK_ARGMAX || kind == AIXK_ARGMAX_ONEHOT, "reduce: unknown kind %d", kind);
    // aixDeviceCPU.cpp:1027-1030, 1050-1053
    AIXK_REQUIRE(out->dtype == AIXK_I32, "argmax supports only int32 data type for its result.");
    AIXK_REQUIRE(a->size < (1ull << 31), "argmax: index does not fit int32");
    if (kind == AIXK_ARGMAX_ONEHOT) {
        fin.onehot = 1;
        AIXK_TRY(aixk_zero(ctx, out->data, a->size * sizeof(int32_t)));
    }
    return by_dtype(a->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        return run_all<ArgOp<T>, T>(ctx, a, (int32_t*)out->data, fin, fixed);
    });
}

int32_t aixk_reduce_all(aixk_ctx* ctx, int kind, const aixhip_tensor* a, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    return reduce_all_impl(ctx, kind, a, out, nullptr);
}

// The same reduction for callers that may not allocate (stream capture, serving loops, harnesses that forbid
// hipMalloc): the partial results of the workgroups live in the static device array `scratch` of this file instead
// of the context's pooled scratch.  No hipMalloc / hipFree / allocating library call is made on this path.  The
// array is shared by every call on the GPU and keeps the last call's contents; each launch overwrites the partials
// it reads, so nothing has to be cleared, but two calls that overlap on one GPU (two contexts, two streams) race.
int32_t aixk_reduce_all_noalloc(aixk_ctx* ctx, int kind, const aixhip_tensor* a, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(ctx->static_scratch != nullptr, "reduce (no-allocation entry point): the static scratch of device %d was not resolved", ctx->device);
    AIXK_REQUIRE(a != nullptr && a->size <= kStaticMaxElements,
                 "reduce (no-allocation entry point): at most %llu elements per call", (unsigned long long)kStaticMaxElements);
    return reduce_all_impl(ctx, kind, a, out, ctx->static_scratch);
}

static int32_t reduce_to_impl(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst, const uint64_t* init);

int32_t aixk_reduce_to(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst)
{
    return reduce_to_impl(ctx, kind, src, dst, nullptr);
}

int32_t aixk_reduce_to_init(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst, uint64_t init_bits)
{
    return reduce_to_impl(ctx, kind, src, dst, &init_bits);
}

static int32_t reduce_to_impl(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst, const uint64_t* init)
{
    AIXK_TRY(set_device(ctx));
    if (init && src->size == 0 && valid_tensor(dst)) return aixk_fill(ctx, init, dst->dtype, dst);
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "reduceTo: bad operand descriptor");
    AIXK_REQUIRE(kind == AIXK_SUM || kind == AIXK_MAX, "reduceTo: unknown kind %d", kind);
    AIXK_REQUIRE(src->dtype == dst->dtype, "reduceTo: element types differ");          // aixDeviceMetal.cpp:787-790
    if (src->size == 0) return AIXK_OK;
    AIXK_REQUIRE(src->size == numel(src), "reduceTo: inconsistent source");
    uint64_t weight[AIXK_MAX_RANK];
    dst_weights(dst->shape, dst->rank, src->shape, src->rank, weight);
    RedPlan plan;
    if (!make_plan(src, weight, &plan)) return fail(AIXK_EINVAL, "reduceTo: view does not collapse to %d dims", kMaxDims);
    if (init && (dst->size != plan.slots || plan.red == 0)) {
        // not one landing per destination element: initialise the ordinary way, then accumulate
        AIXK_TRY(aixk_fill(ctx, init, dst->dtype, dst));
        init = nullptr;
    }
    const Finish fin{init ? 2 : 1, 0, 0, 0, init ? *init : 0};
    return by_dtype(src->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if (kind == AIXK_SUM) return run_plan<SumOp<T>, T>(ctx, src, (T*)dst->data, plan, fin);
        return run_plan<MaxOp<T>, T>(ctx, src, (T*)dst->data, plan, fin);
    });
}

int32_t aixk_argmax_to(aixk_ctx* ctx, int onehot, const aixhip_tensor* src, const aixhip_tensor* dst, uint64_t dim)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(src) && valid_tensor(dst), "argmaxTo: bad operand descriptor");
    // aixDeviceCPU.cpp:1191-1194, 1214-1217
    AIXK_REQUIRE(dst->dtype == AIXK_I32, "argmaxTo supports only int32 data type for its result.");
    AIXK_REQUIRE((int)dim < src->rank, "argmaxTo: dim out of range");
    if (src->size == 0) return AIXK_OK;
    AIXK_REQUIRE(src->size == numel(src) && src->size < (1ull << 31), "argmaxTo: inconsistent or too large source");
    uint64_t weight[AIXK_MAX_RANK];
    Finish fin{0, onehot, 0, 0};
    if (onehot) {
        AIXK_REQUIRE((int)dim < dst->rank, "argmaxIndicesTo: dim out of range");
        uint64_t rshape[AIXK_MAX_RANK];
        for (int d = 0; d < dst->rank; ++d) rshape[d] = d == (int)dim ? 1 : dst->shape[d];   // aixDeviceCPU.cpp:325-326
        dst_weights(rshape, dst->rank, src->shape, src->rank, weight);
    } else {
        AIXK_REQUIRE(src->strides[dim] != 0, "argmaxTo: zero stride along the reduced dim");
        dst_weights(dst->shape, dst->rank, src->shape, src->rank, weight);
        fin.q_stride = src->strides[dim];
        fin.q_extent = src->shape[dim];
    }
    RedPlan plan;
    if (!make_plan(src, weight, &plan)) return fail(AIXK_EINVAL, "argmaxTo: view does not collapse to %d dims", kMaxDims);
    return by_dtype(src->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if (fin.onehot == 2 && !onehot_rows_route<T>(plan, (const T*)src->data, dst->data) && !onehot_inner_route(plan, dst->data)) {
            // the zero-initialisation this call owes, as a pass of its own, then ones scattered as usual
            AIXK_TRY(aixk_zero(ctx, dst->data, src->size * sizeof(int32_t)));
            fin.onehot = 1;
        }
        return run_plan<ArgOp<T>, T>(ctx, src, (int32_t*)dst->data, plan, fin);
    });
}

int32_t aixk_argmax_onehot_many(aixk_ctx* ctx, const aixk_argmax_item* items, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    if (count == 0) return AIXK_OK;
    AIXK_REQUIRE(items, "argmaxIndicesTo of several items: no items");
    // one launch if every item is dense rows of one element type reduced along the last dim, else item by item
    bool together = count >= 2 && count <= AIXK_ARGMAX_ITEMS_MAX;
    const int dtype = items[0].src.dtype;
    for (uint32_t k = 0; k < count && together; ++k) {
        const aixhip_tensor *src = &items[k].src, *dst = &items[k].dst;
        together = valid_tensor(src) && valid_tensor(dst) && src->dtype == dtype && dst->dtype == AIXK_I32 && src->rank >= 1 &&
                   (int)items[k].dim == src->rank - 1 && dst->rank == src->rank && src->size > 0 && src->size == numel(src) && src->size < (1ull << 31) &&
                   dst->size == src->size && dst->offset == 0 && aligned16(dst->data);
        if (!together) break;
        const uint64_t L = src->shape[src->rank - 1], vec = 16 / aixk_dtype_size(dtype);
        uint64_t dense[AIXK_MAX_RANK];
        row_major_strides(src->rank, src->shape, dense);
        for (int d = 0; d < src->rank; ++d)
            if (dst->shape[d] != src->shape[d] || (src->shape[d] != 1 && (src->strides[d] != dense[d] || dst->strides[d] != dense[d]))) together = false;
        together = together && L >= 32 && L % 4 == 0 && L % vec == 0 && aligned16((const char*)src->data + src->offset * aixk_dtype_size(dtype));
    }
    if (!together) {
        for (uint32_t k = 0; k < count; ++k) AIXK_TRY(aixk_argmax_to(ctx, 2, &items[k].src, &items[k].dst, items[k].dim));
        return AIXK_OK;
    }
    const size_t table_bytes = (size_t)count * sizeof(OnehotItem), all_bytes = table_bytes + ((size_t)count + 1) * sizeof(u32);
    char* host = nullptr;
    const char* dev = nullptr;
    AIXK_TRY(table_slot(ctx, all_bytes, (void**)&host, (const void**)&dev));
    OnehotItem* table = (OnehotItem*)host;
    u32* starts = (u32*)(host + table_bytes);
    u32 grid = 0;
    for (uint32_t k = 0; k < count; ++k) {
        const aixhip_tensor *src = &items[k].src, *dst = &items[k].dst;
        const uint64_t L = src->shape[src->rank - 1], rows = src->size / L;
        table[k].src = (u64)(uintptr_t)((const char*)src->data + src->offset * aixk_dtype_size(dtype));
        table[k].dst = (u64)(uintptr_t)dst->data;
        table[k].rows = rows; table[k].len = L;
        starts[k] = grid;
        grid += grid_for(rows, kWaves, 1u << 20);
    }
    starts[count] = grid;
    AIXK_TRY(table_upload(ctx, host, dev, all_bytes));
    return by_dtype(dtype, [&](auto tag) {
        typedef decltype(tag) T;
        hipLaunchKernelGGL((argmax_onehot_inner_many_k<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const OnehotItem*)dev, (const u32*)(dev + table_bytes), (u32)count);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

int32_t aixk_sum_columns_many(aixk_ctx* ctx, const aixk_colsum_item* items, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    if (count == 0) return AIXK_OK;
    AIXK_REQUIRE(items, "column sums of several items: no items");
    // one pair of launches if every item is a dense matrix of one floating-point type summed down its columns into a
    // dense vector, else item by item
    const int dtype = items[0].src.dtype;
    bool together = count >= 2 && count <= AIXK_COLSUM_ITEMS_MAX && (dtype == AIXK_F32 || dtype == AIXK_F16 || dtype == AIXK_BF16);
    const size_t esz = aixk_dtype_size(dtype);
    uint64_t tiles_all = 0, columns = 0;
    for (uint32_t k = 0; k < count && together; ++k) {
        const aixhip_tensor *src = &items[k].src, *dst = &items[k].dst;
        together = valid_tensor(src) && valid_tensor(dst) && src->dtype == dtype && dst->dtype == dtype && src->rank >= 2 && dst->rank >= 1 && src->size > 0 &&
                   src->size == numel(src) && dst->size == numel(dst) && src->data && dst->data;
        if (!together) break;
        const uint64_t C = src->shape[src->rank - 1], R = src->size / C;
        uint64_t dense[AIXK_MAX_RANK];
        row_major_strides(src->rank, src->shape, dense);
        for (int d = 0; d < src->rank; ++d) if (src->shape[d] != 1 && src->strides[d] != dense[d]) together = false;
        together = together && dst->size == C && dst->shape[dst->rank - 1] == C && (C == 1 || dst->strides[dst->rank - 1] == 1) && R >= 2 && C % 4 == 0 &&
                   R < (1ull << 31) && C < (1ull << 31) && ((uintptr_t)((const char*)src->data + src->offset * esz) % (4 * esz)) == 0;
        tiles_all += (C + 255) / 256;
        columns += C;
    }
    together = together && columns < (1ull << 31);
    const uint64_t acc_bytes = dtype == AIXK_F32 ? sizeof(SumOp<float>::Acc) : sizeof(SumOp<bf16>::Acc);
    std::vector<ColsumItem> plan;
    u32 grid = 0;
    if (together) {
        // rows in chunks of at least 64 so that the launch has about 8 workgroups per compute unit
        const uint64_t want = (uint64_t)ctx->cus * 8;
        const uint64_t split = std::max<uint64_t>(1, (want + tiles_all - 1) / tiles_all);
        plan.resize(count);
        uint64_t partials = 0, col = 0;
        for (uint32_t k = 0; k < count; ++k) {
            const aixhip_tensor *src = &items[k].src, *dst = &items[k].dst;
            const uint64_t C = src->shape[src->rank - 1], R = src->size / C;
            uint64_t chunks = std::min<uint64_t>({split, (R + 63) / 64, (uint64_t)64});
            uint64_t rpc = ((R + chunks - 1) / chunks + 15) & ~(uint64_t)15;
            chunks = (R + rpc - 1) / rpc;
            ColsumItem& it = plan[k];
            it.src = (u64)(uintptr_t)((const char*)src->data + src->offset * esz);
            it.dst = (u64)(uintptr_t)((char*)dst->data + dst->offset * esz);
            it.rows = R; it.cols = C; it.pitch = C; it.init = items[k].init_bits;
            it.partials = partials;
            it.first_wg = grid; it.tiles = (u32)((C + 255) / 256); it.chunks = (u32)chunks; it.rows_per_chunk = (u32)rpc; it.first_col = (u32)col; it.pad = 0;
            partials += chunks * C;
            col += C;
            const uint64_t wgs = (uint64_t)it.tiles * chunks;
            if ((uint64_t)grid + wgs >= (1ull << 31)) { together = false; break; }
            grid += (u32)wgs;
        }
        together = together && partials * acc_bytes <= ctx->scratch_bytes;
    }
    if (!together) {
        for (uint32_t k = 0; k < count; ++k) AIXK_TRY(aixk_reduce_to_init(ctx, AIXK_SUM, &items[k].src, &items[k].dst, items[k].init_bits));
        return AIXK_OK;
    }
    const size_t table_bytes = (size_t)count * sizeof(ColsumItem);
    char* host = nullptr;
    const char* dev = nullptr;
    AIXK_TRY(table_slot(ctx, table_bytes, (void**)&host, (const void**)&dev));
    std::memcpy(host, plan.data(), table_bytes);
    AIXK_TRY(table_upload(ctx, host, dev, table_bytes));
    return by_dtype(dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if constexpr (std::is_same<T, float>::value || std::is_same<T, f16>::value || std::is_same<T, bf16>::value) {
            typedef typename SumOp<T>::Acc Acc;
            hipLaunchKernelGGL((sum_columns_many_k<T>), dim3(grid), dim3(kBlock), 0, ctx->stream, (const ColsumItem*)dev, (u32)count, (Acc*)ctx->scratch);
            AIXK_HIP(hipGetLastError());
            hipLaunchKernelGGL((sum_columns_finish_many_k<T>), dim3((unsigned)((columns + kBlock - 1) / kBlock)), dim3(kBlock), 0, ctx->stream, (const ColsumItem*)dev,
                               (u32)count, (const Acc*)ctx->scratch, (u32)columns);
            AIXK_HIP(hipGetLastError());
        }
        return (int)AIXK_OK;
    });
}

int32_t aixk_sum_partials(aixk_ctx* ctx, const void* partials, uint64_t count, const aixhip_tensor* dst, uint64_t init_bits)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(dst) && dst->data && dst->size == 1, "sum of partials: the result is one element");
    AIXK_REQUIRE(partials && count > 0 && count < (1ull << 31), "sum of partials: no partials, or too many");
    AIXK_REQUIRE(dst->dtype == AIXK_F64 || dst->dtype == AIXK_F32 || dst->dtype == AIXK_F16 || dst->dtype == AIXK_BF16, "sum of partials: floating-point results only");
    return by_dtype(dst->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if constexpr (std::is_same<T, double>::value || std::is_same<T, float>::value || std::is_same<T, f16>::value || std::is_same<T, bf16>::value) {
            hipLaunchKernelGGL((sum_partials_k<T>), dim3(1), dim3(kBlock), 0, ctx->stream, (const typename traits<T>::W*)partials, (unsigned)count,
                               (T*)dst->data + dst->offset, (u64)init_bits);
            AIXK_HIP(hipGetLastError());
        }
        return (int)AIXK_OK;
    });
}

int32_t aixk_sum_partials_many(aixk_ctx* ctx, const aixk_partials_item* items, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    if (count == 0) return AIXK_OK;
    AIXK_REQUIRE(items, "sums of partials: no items");
    const int dtype = items[0].dst.dtype;
    bool together = count >= 2 && count <= AIXK_PARTIALS_ITEMS_MAX && (dtype == AIXK_F64 || dtype == AIXK_F32 || dtype == AIXK_F16 || dtype == AIXK_BF16);
    for (uint32_t k = 0; k < count && together; ++k)
        together = valid_tensor(&items[k].dst) && items[k].dst.data && items[k].dst.size == 1 && items[k].dst.dtype == dtype && items[k].partials &&
                   items[k].count > 0 && items[k].count < (1ull << 31);
    if (!together) {
        for (uint32_t k = 0; k < count; ++k) AIXK_TRY(aixk_sum_partials(ctx, items[k].partials, items[k].count, &items[k].dst, items[k].init_bits));
        return AIXK_OK;
    }
    const size_t table_bytes = (size_t)count * sizeof(PartialsItem), esz = aixk_dtype_size(dtype);
    PartialsItem* host = nullptr;
    const PartialsItem* dev = nullptr;
    AIXK_TRY(table_slot(ctx, table_bytes, (void**)&host, (const void**)&dev));
    for (uint32_t k = 0; k < count; ++k) {
        host[k].partials = (u64)(uintptr_t)items[k].partials;
        host[k].dst = (u64)(uintptr_t)((char*)items[k].dst.data + items[k].dst.offset * esz);
        host[k].init = items[k].init_bits;
        host[k].count = (u32)items[k].count;
        host[k].pad = 0;
    }
    AIXK_TRY(table_upload(ctx, host, dev, table_bytes));
    return by_dtype(dtype, [&](auto tag) {
        typedef decltype(tag) T;
        if constexpr (std::is_same<T, double>::value || std::is_same<T, float>::value || std::is_same<T, f16>::value || std::is_same<T, bf16>::value) {
            hipLaunchKernelGGL((sum_partials_many_k<T>), dim3(count), dim3(kBlock), 0, ctx->stream, dev);
            AIXK_HIP(hipGetLastError());
        }
        return (int)AIXK_OK;
    });
}

} // extern "C"
