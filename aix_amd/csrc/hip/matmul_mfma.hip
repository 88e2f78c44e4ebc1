// matmul_mfma.hip -- GEMM on the matrix cores for f32 / f16 / bf16, f32 accumulation.
//
// Kernels (A is [M,K], B is [K,N]; "K-contiguous" = unit stride along K, "T form" = unit stride along M / N):
//
//   16-bit, whole tiles   gemm_nt16_direct_k: 256x256x64 workgroup tile, eight waves (two per SIMD) on
//                         v_mfma_f32_16x16x32, LDS filled by LDS-direct global loads, swizzled layout,
//                         explicit software pipeline; both operand forms;
//   16-bit, whole tiles   gemm_direct16_k: the same scheme on 128 x {128, 192, 256} x 64 tiles for results that 256 x 256
//                         tiles cannot spread over the chip; stacks and groups of products by blockIdx.y;
//   16-bit, mid-size      gemm_tile16_k: 128x128 / 128x64 / 64x64 tiles, register staging, both operand
//                         forms, stacks of matrices (blockIdx.y) and K splits over workgroups (blockIdx.z);
//   16-bit, small         gemm_small16_k: 32x32 tile, K split over the workgroup's four waves;
//   16-bit, K = 64        gemm_k64_nt_k: stacks of products with one K step (attention's scores): every wave on its
//                         own, rows to fragments and accumulators to rows through a slab of its own, no barrier;
//   16-bit, odd layouts   gemm_nt16_k: K-contiguous operands only, bounds-checked (others are gathered first);
//   f32, large            gemm_x3_k: each operand as three bf16 planes on the bf16 matrix pipe, f32 accumulation;
//   f32, very large       split_planes_k + gemm_direct16_k<PLANES>: the planes written to memory once, six plane pairs
//                         multiplied by the LDS-direct 16-bit kernel;
//   f32                   gemm_nt32_k: v_mfma_f32_32x32x2f32, 128x128 or 64x64 tile x BK=32, both operand forms.
//
// All but the first two use 4 waves in a 2x2 arrangement (gemm_small16_k: one 32x32 tile, K split; gemm_k64_nt_k: four
// independent waves) with the accumulators
// resident in the 512-entry unified register file.  Every lane feeds the 16-bit MFMA with 8 consecutive K
// values of one row; because A and B use the same lane->K assignment, the dot products are independent of
// how the instruction numbers K internally.
//
// Workgroups are numbered so that the 32 groups resident on one XCD (dispatch is round-robin over
// the 8 XCDs) cover a compact 4 x 8 block of output tiles and share A/B panels in that XCD's L2.
//
// Odd K (not a multiple of 8 elements for 16-bit, 4 for f32) falls back to the LDS-tiled kernel in
// matmul.hip.
#pragma clang fp contract(fast)

#include "common.hpp"

#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <type_traits>
#include <utility>

using namespace aixd;
using namespace aixk;

namespace aixk {
int gather_dense(aixk_ctx* ctx, const aixhip_tensor* src, void* dst, uint64_t n);     // layout.hip
}

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct GemmArgs {
    const void* a; const void* b; void* c;
    u64 M, N, K, lda, ldb;          // element strides between rows of A [M,K] and B [N,K]
    u32 tiles_m, tiles_n, swizzle;  // swizzle = 1: XCD-aware numbering is a bijection for this grid
};

// A stack of independent products in one launch: blockIdx.y numbers the matrices in row-major order of up to
// three (collapsed) leading dims; every matrix of A / B starts sa / sb elements further per step of its dim,
// results are dense, sc elements apart.  rank 0: a single product.
// `table` set: the matrices are unrelated buffers instead -- three addresses (A, B, C) per matrix in device memory, in
// the order of blockIdx.y (a group of separate matmul calls issued as one launch).
struct BatchArgs {
    u32 rank, ext[3];
    u64 sa[3], sb[3], sc;
    const u64* table;
};

// blockIdx -> output tile, XCD-aware and grouped (4 tile rows per column sweep).
__device__ __forceinline__ void tile_of(const GemmArgs& g, u32& tm, u32& tn)
{
    const u32 ntiles = g.tiles_m * g.tiles_n;
    u32 lin = blockIdx.x;
    if (g.swizzle) lin = (lin % 8u) * (ntiles / 8u) + lin / 8u;
    constexpr u32 GM = 4;
    const u32 width = GM * g.tiles_n;
    const u32 group = lin / width, first = group * GM;
    const u32 gsz = g.tiles_m - first < GM ? g.tiles_m - first : GM;
    const u32 in = lin - group * width;
    tm = first + in % gsz;
    tn = in / gsz;
}

template <class T> struct Mma16;
template <> struct Mma16<bf16> {
    static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c)
    { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0); }
    static __device__ __forceinline__ f32x4 run16(u32x4 a, u32x4 b, f32x4 c)
    { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0); }
    static __device__ __forceinline__ bf16 out(float v) { return bf16_down(v); }
    static __device__ __forceinline__ u32 pack(float lo, float hi) { return (u32)out(lo).bits | ((u32)out(hi).bits << 16); }
};
template <> struct Mma16<f16> {
    static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c)
    { return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0); }
    static __device__ __forceinline__ f32x4 run16(u32x4 a, u32x4 b, f32x4 c)
    { return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0); }
    static __device__ __forceinline__ f16 out(float v) { return (f16)v; }
    static __device__ __forceinline__ u32 pack(float lo, float hi)
    { return (u32)__builtin_bit_cast(u16, (f16)lo) | ((u32)__builtin_bit_cast(u16, (f16)hi) << 16); }
};

// ---- 16-bit operands ---------------------------------------------------------------------------
// BM x BN workgroup tile, BK = 64; LDS row = 64 elements + 8 padding = 144 bytes.
template <class T, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_nt16_k(GemmArgs g)
{
    constexpr int BK = 64, LDR = BK + 8;                 // elements per LDS row
    constexpr int WM = BM / 2, WN = BN / 2, TI = WM / 32, TJ = WN / 32;
    constexpr int CA = BM * (BK / 8) / 256, CB = BN * (BK / 8) / 256;      // 16-byte chunks per lane per step
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    u16* As = (u16*)smem;                                // [2][BM][LDR]
    u16* Bs = As + 2 * BM * LDR;                         // [2][BN][LDR]

    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const u16* A = (const u16*)g.a;
    const u16* B = (const u16*)g.b;

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    u32x4 ra[CA], rb[CB];
    auto load_global = [&](u64 k0) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            const u64 r = m0 + row, k = k0 + kc * 8;
            ra[i] = (r < g.M && k < g.K) ? *(const u32x4*)(A + r * g.lda + k) : (u32x4){0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            const u64 r = n0 + row, k = k0 + kc * 8;
            rb[i] = (r < g.N && k < g.K) ? *(const u32x4*)(B + r * g.ldb + k) : (u32x4){0, 0, 0, 0};
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            *(u32x4*)(As + (buf * BM + row) * LDR + kc * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            *(u32x4*)(Bs + (buf * BN + row) * LDR + kc * 8) = rb[i];
        }
    };

    const u64 steps = (g.K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (u64 kt = 0; kt < steps; ++kt) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < steps) load_global((kt + 1) * BK);
        const u16* as = As + (buf * BM + wm * WM + (lane & 31)) * LDR + (lane >> 5) * 8;
        const u16* bs = Bs + (buf * BN + wn * WN + (lane & 31)) * LDR + (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4 fa[TI], fb[TJ];
#pragma unroll
            for (int i = 0; i < TI; ++i) fa[i] = *(const u32x4*)(as + i * 32 * LDR + kk * 16);
#pragma unroll
            for (int j = 0; j < TJ; ++j) fb[j] = *(const u32x4*)(bs + j * 32 * LDR + kk * 16);
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) acc[i][j] = Mma16<T>::run(fa[i], fb[j], acc[i][j]);
        }
        if (kt + 1 < steps) store_lds(buf ^ 1);
        __syncthreads();
    }

    // accumulator element v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
    T* C = (T*)g.c;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const u64 col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const u64 row = m0 + wm * WM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.M && col < g.N) C[row * g.N + col] = Mma16<T>::out(acc[i][j][v]);
            }
        }
}

// ---- 16-bit operands, 256 x 256 x 64 tile fed by LDS-direct loads ---------------------------------
// For M, N multiples of 256 and K a multiple of 64.  Two 64 KB LDS stages; each wave fills its share
// of the next stage with global_load_lds_dwordx4 (16 bytes per lane straight into LDS, no staging
// registers, whole 128-byte rows per 8 lanes so every L2 request is a full line).  One load
// instruction deposits 1 KB contiguously (lane L at byte 16 L), so padding is impossible; instead
// the 16-byte k-chunk q of row r is kept in slot q ^ f(r), f(r) = ((r >> 1) & 7) ^ ((r & 1) << 2),
// which makes the ds_read_b128 fragment reads (16 consecutive rows, four slots) conflict-free for
// both 8-lane/32-bank and 16-lane/64-bank service; the producing lane applies the same
// permutation to the global address it fetches.
//
// EIGHT waves, two per SIMD, in a 2 x 4 arrangement: a wave owns 128 x 64 of the tile as 8 x 4
// tiles of 16 x 16 and multiplies with v_mfma_f32_16x16x32.  Both choices are about power, which is
// what bounds this kernel on real operands (a loop of nothing but MFMAs on U(-1,1)/64 values runs
// at 1.81 GHz and 0.68 of the nominal peak with v_mfma_f32_32x32x16, at 2.08 GHz and 0.81 with
// v_mfma_f32_16x16x32, which moves half the accumulator bits per flop; on all-zero operands both
// reach 0.91-0.92 at 2.4 GHz): the 16 x 16 x 32 instruction needs two waves per SIMD to be issued
// back to back, and with two waves the older one takes the matrix pipe whenever it can, the younger
// one whenever the older waits -- no issue slot is lost to LDS or load latency.  The price is 1.5 x
// the LDS fragment traffic of four waves with 128 x 128 each.
//
// A K-step is two slices of 32: phase A multiplies slice 0 while slice 1 is read into the other
// fragment set, the step's single barrier, phase B multiplies slice 1 while slice 0 of the other
// stage is read and ALL eight loads of the tile after next are issued (a whole K-step ahead of the
// wait that needs them: spread over both phases they left 10 us on the table at 4096^3).  Reads and
// loads sit between the MFMAs in fenced sub-blocks of eight.  The compiler does not track LDS-direct
// loads against LDS reads, so the waits before the barrier are explicit (s_waitcnt vmcnt) and the
// barrier is the bare instruction.  Results leave through LDS as non-temporal 16-byte stores (the
// product is not read again by this kernel, and at its end every L2 would have to write it back).
#define AIX_SB() __builtin_amdgcn_sched_barrier(0)
#define AIX_WAIT(VM, LGKM) __builtin_amdgcn_s_waitcnt(((VM) & 15) | (((VM) >> 4) << 14) | 0x70 | ((LGKM) << 8))
#define AIX_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define AIX_GLB(p) ((const __attribute__((address_space(1))) void*)(p))
//
// An operand may also be given the other way round -- A as [K, M] with unit stride along M (a
// transposed view, "T" form), B as [K, N] with unit stride along N (plain row-major) -- and is then
// consumed where it lies: its stage holds 64 k-rows of 512 bytes (LDS-direct chunks of 2 k-rows),
// and the MFMA fragments, which need 8 consecutive k per lane, are assembled by
// ds_read_b64_tr_b16: in every group of 16 lanes, lane j points at 4 consecutive elements
// ("row" j) and lane i receives element i & 3 of rows (i >> 2) + 4 e, e = 0..3.  With lane j
// pointing at X[k + (j >> 2)][n + 4 (j & 3) ..], lane i receives X[k .. k + 3][n + i]: four k of
// its own column; two such reads make a fragment; the wave's four groups of 16 lanes read the same
// 16 columns at k, k + 8, k + 16, k + 24.  The four k-rows of a group are 512 bytes apart (same
// banks), and so are the rows of the next group, so the 16-byte chunk c of k-row k is kept in slot
// c ^ 4 (k & 3) ^ 2 ((k >> 3) & 1): the 32 bytes that a group reads from each of its four k-rows,
// and those of the neighbouring group, fall into disjoint banks.
//
// The read is issued through inline assembly: given the builtin, the compiler orders it behind every
// LDS-direct load in flight (s_waitcnt vmcnt(0) before each read), which serialises the pipeline.
// The price is that the compiler no longer knows the result is pending, so every phase that consumes
// such fragments starts with an explicit s_waitcnt lgkmcnt(0).
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x4 tr_fragment(const unsigned char* lds_addr)
{
    const u32 addr = (u32)(size_t)(__attribute__((address_space(3))) const unsigned char*)lds_addr;
    u32x2 lo, hi;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:2048" : "=v"(hi) : "v"(addr));       // k + 4
    return u32x4{lo.x, lo.y, hi.x, hi.y};
}

template <int N> struct Const { static constexpr int v = N; };

template <class T, bool AT, bool BT>
__global__ __launch_bounds__(512) void gemm_nt16_direct_k(GemmArgs g)
{
    constexpr int BM = 256, BK = 64, STAGE = 2 * 256 * BK * 2;      // 65536 bytes: A rows then B rows
    constexpr int WGN = 4, TI = 8, TJ = 4, WCOLS = TJ * 16;          // 2 x 4 waves of 128 x 64
    constexpr int LPW = 8, LH = 4;                                   // loads per wave and tile: 4 chunks of A, 4 of B
    constexpr int NF = TI + TJ, FPB = NF / 4;                        // fragments per slice, per sub-block
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * 256, n0 = (u64)tn * 256;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), wm = wave / WGN, wn = wave % WGN;
    // producer, K-contiguous operand: wave w fills rows 32 w .. 32 w + 31, 4 chunks of 8 rows (128 B each)
    const int lr = lane >> 3;
    const int fe = (lr >> 1) ^ ((lr & 1) << 2);              // f(row) in even chunks; odd chunks: fe ^ 4
    const int q0 = (lane & 7) ^ fe, q1 = q0 ^ 4;
    // producer, T-form operand: wave w fills k-rows 8 w .. 8 w + 7, 4 chunks of 2 k-rows (512 B each); lane = (k-row
    // lane >> 5, slot lane & 31) fetches chunk slot ^ 4 (k & 3) ^ 2 ((k >> 3) & 1), k & 3 = 2 (chunk & 1) + (lane >> 5),
    // (k >> 3) & 1 = w & 1
    const int tk = lane >> 5, ts0 = (lane & 31) ^ (4 * tk) ^ (2 * (wave & 1)), ts1 = ts0 ^ 8;
    const char* A = AT ? (const char*)g.a + m0 * 2 + (u64)(wave * 8) * g.lda * 2 : (const char*)g.a + (m0 + wave * 32) * g.lda * 2;
    const char* B = BT ? (const char*)g.b + n0 * 2 + (u64)(wave * 8) * g.ldb * 2 : (const char*)g.b + (n0 + wave * 32) * g.ldb * 2;
    const u32 oa0 = AT ? (u32)((tk * g.lda + ts0 * 8) * 2) : (u32)((lr * g.lda + q0 * 8) * 2);
    const u32 oa1 = AT ? (u32)((tk * g.lda + ts1 * 8) * 2) : (u32)((lr * g.lda + q1 * 8) * 2);
    const u32 ob0 = BT ? (u32)((tk * g.ldb + ts0 * 8) * 2) : (u32)((lr * g.ldb + q0 * 8) * 2);
    const u32 ob1 = BT ? (u32)((tk * g.ldb + ts1 * 8) * 2) : (u32)((lr * g.ldb + q1 * 8) * 2);
    const u64 ca = (AT ? 4 : 16) * g.lda, cb = (BT ? 4 : 16) * g.ldb;      // bytes between chunks
    const u64 sa = AT ? (u64)BK * g.lda * 2 : (u64)BK * 2, sb = BT ? (u64)BK * g.ldb * 2 : (u64)BK * 2;   // bytes between K-steps
    const int steps = (int)(g.K / BK);
    // consumer, K-contiguous operand: lane reads row (lane & 15) of a 16-row block, k-chunk 4 s + (lane >> 4) of slice s
    const int r15 = lane & 15, grp = lane >> 4;
    const int slot0 = grp ^ (((r15 >> 1) & 7) ^ ((r15 & 1) << 2));
    // consumer, T-form operand: lane j of a 16-lane group points at k-row 32 s + 8 grp + (j >> 2) [+ 4], columns
    // 4 (j & 3) .. + 3 of the 16-column block; the block index enters by XOR (bits 5 and up of the byte address)
    const int tq = r15 >> 2;
    const int tlane = (8 * grp + tq) * 512 + 8 * (r15 & 1);
    const int tsw = (4 * tq) ^ (2 * (grp & 1));
    const int fra = AT ? tlane + (((16 * wm + ((r15 & 3) >> 1)) ^ tsw) * 16) : (wm * 128 + r15) * 128 + slot0 * 16;
    const int frb = BM * 128 + (BT ? tlane + (((8 * wn + ((r15 & 3) >> 1)) ^ tsw) * 16) : (wn * WCOLS + r15) * 128 + slot0 * 16);

    f32x4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    u32x4 fa[2][TI], fb[2][TJ];

    // load n of a tile (0..7): n < 4 is this wave's chunk n of A, otherwise chunk n - 4 of B
    auto load = [&](auto n_, u64 ki, int bo) {
        constexpr int n = decltype(n_)::v;
        if constexpr (n < LH)
            __builtin_amdgcn_global_load_lds(AIX_GLB(A + (n * ca + ki * sa) + ((n & 1) ? oa1 : oa0)), AIX_LDS(smem + bo + (wave * LH + n) * 1024), 16, 0, 0);
        else
            __builtin_amdgcn_global_load_lds(AIX_GLB(B + ((n - LH) * cb + ki * sb) + ((n & 1) ? ob1 : ob0)), AIX_LDS(smem + bo + BM * 128 + (wave * LH + n - LH) * 1024), 16, 0, 0);
    };
    // fragment f of slice s: f < 8 is A's 16-row block f, otherwise B's block f - 8
    auto read = [&](int set, int bo, int s, int f) {
        if (f < TI) {
            if constexpr (AT) fa[set][f] = tr_fragment(smem + bo + (fra ^ (f * 32)) + s * 16384);
            else fa[set][f] = *(const u32x4*)(smem + bo + (fra ^ (s * 64)) + f * 2048);
        } else {
            if constexpr (BT) fb[set][f - TI] = tr_fragment(smem + bo + (frb ^ ((f - TI) * 32)) + s * 16384);
            else fb[set][f - TI] = *(const u32x4*)(smem + bo + (frb ^ (s * 64)) + (f - TI) * 2048);
        }
    };
    // MFMAs on fragment set FC while set FN is read from stage rbo, slice S; with LOADS, the tile `ko` goes to stage lbo
    auto phase = [&](auto FC_, auto FN_, int rbo, auto S_, auto LOADS_, u64 ko, int lbo) {
        constexpr int FC = decltype(FC_)::v, FN = decltype(FN_)::v, S = decltype(S_)::v, LOADS = decltype(LOADS_)::v;
        if constexpr (AT || BT) { AIX_SB(); __builtin_amdgcn_s_waitcnt(0xC07F); AIX_SB(); }     // lgkmcnt(0): fragment set FC has arrived
        [&]<int... b>(std::integer_sequence<int, b...>) {
            ([&] {
#pragma unroll
                for (int f = b * FPB; f < (b + 1) * FPB; ++f) read(FN, rbo, S, f);
                if constexpr (LOADS) { load(Const<b>{}, ko, lbo); load(Const<b + 4>{}, ko, lbo); }
#pragma unroll
                for (int i = 2 * b; i < 2 * b + 2; ++i)
#pragma unroll
                    for (int j = 0; j < TJ; ++j) acc[i][j] = Mma16<T>::run16(fa[FC][i], fb[FC][j], acc[i][j]);
                AIX_SB();
            }(), ...);
        }(std::make_integer_sequence<int, 4>{});
    };

    // Tiles past the end re-read the last tile into a stage nobody consumes any more.
    {
        const u64 k1 = 1 < steps ? 1 : 0;
        [&]<int... n>(std::integer_sequence<int, n...>) { (load(Const<n>{}, (u64)0, 0), ...); }(std::make_integer_sequence<int, LPW>{});
        [&]<int... n>(std::integer_sequence<int, n...>) { (load(Const<n>{}, k1, STAGE), ...); }(std::make_integer_sequence<int, LPW>{});
    }
    AIX_SB();
    AIX_WAIT(LPW, 15);                                        // tile 0 has landed (the 8 loads of tile 1 may be in flight)
    __builtin_amdgcn_s_barrier();
    AIX_SB();
#pragma unroll
    for (int f = 0; f < NF; ++f) read(0, 0, 0, f);
    for (int kt = 0; kt < steps; ++kt) {
        const int bo = (kt & 1) * STAGE, nbo = bo ^ STAGE;
        const u64 k2 = (u64)(kt + 2 < steps ? kt + 2 : steps - 1);
        phase(Const<0>{}, Const<1>{}, bo, Const<1>{}, Const<0>{}, k2, nbo);
        AIX_WAIT(0, 0);                                       // tile kt+1 complete in the other stage; own reads of this stage done
        __builtin_amdgcn_s_barrier();
        AIX_SB();
        phase(Const<1>{}, Const<0>{}, nbo, Const<0>{}, Const<1>{}, k2, bo);
    }
    AIX_WAIT(0, 0);                                           // stray loads have landed before LDS is reused
    __builtin_amdgcn_s_barrier();
    AIX_SB();

    // Epilogue through LDS, each wave on its own 4.5 KB: a 16-row slab of the wave's 128 x 64 block is laid out
    // row-major (pitch 68 floats), read back as runs of 8 columns, rounded and stored with 16-byte writes (128
    // contiguous bytes per row).  Accumulator element v of lane l: row 4 (l / 16) + v, column l % 16 of its 16 x 16 tile.
    constexpr int PITCH = WCOLS + 4;
    float* slab = (float*)smem + wave * (16 * PITCH + 64);
    u16* C = (u16*)g.c;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) slab[(4 * grp + v) * PITCH + j * 16 + r15] = acc[i][j][v];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int run = lane + 64 * t, row = run >> 3, cg = run & 7;
            const f32x4 lo = *(const f32x4*)(slab + row * PITCH + cg * 8);
            const f32x4 hi = *(const f32x4*)(slab + row * PITCH + cg * 8 + 4);
            u32x4 o;
            o.x = Mma16<T>::pack(lo.x, lo.y); o.y = Mma16<T>::pack(lo.z, lo.w);
            o.z = Mma16<T>::pack(hi.x, hi.y); o.w = Mma16<T>::pack(hi.z, hi.w);
            __builtin_nontemporal_store(o, (u32x4*)(C + (m0 + wm * 128 + i * 16 + row) * g.N + n0 + wn * WCOLS + cg * 8));
        }
    }
}

// The same scheme for results that 256 x 256 tiles cannot spread over the chip: BM x BN tiles with BM = 128 and BN = 128,
// 192 or 256 (the widths of a d = 768 model are multiples of 192, not of 256), still eight waves in a 2 x 4 arrangement,
// a wave on 64 x BN / 4 as 4 x (BN / 64) tiles of 16 x 16, K-steps of 64 through two LDS stages filled by LDS-direct
// loads, both operand forms consumed where they lie.  What changes with the tile:
//  * a wave issues BM / 64 loads of A and BN / 64 of B per tile; with an odd count the parity of a load's 8-row block,
//    which picks one of the two producer swizzles, follows the wave's number (the two offsets are swapped once);
//  * a T-form stage keeps k-rows of 2 BM (2 BN) bytes, so a load covers 1024 / pitch k-rows and every load has its own
//    lane -> (k-row, chunk) map (kept in a register per load); rows of 256 and 512 bytes fall on the same banks and
//    use the slot c ^ 4 (k & 3) ^ 2 ((k >> 3) & 1) of the 256 x 256 kernel; rows of 384 bytes alternate between two
//    halves of the banks by themselves and use c ^ 4 ((k >> 1) & 1) ^ 2 ((k >> 3) & 1), which also stays inside the
//    row's 8-chunk groups (24 chunks do not hold a 16-chunk group);
//  * the T-form fragment addresses are kept per 16-column block (the block's chunk enters before the swizzle, and with
//    BN / 4 = 48 columns per wave it cannot be folded in by XOR).
template <int P> __device__ __forceinline__ int tform_swizzle(int k_low3, int k_bit3)
{
    if constexpr (P == 384) return (4 * ((k_low3 >> 1) & 1)) ^ (2 * k_bit3);
    else return (4 * (k_low3 & 3)) ^ (2 * k_bit3);
}

template <int OFF> __device__ __forceinline__ u32x4 tr_fragment_at(const unsigned char* lds_addr)
{
    const u32 addr = (u32)(size_t)(__attribute__((address_space(3))) const unsigned char*)lds_addr;
    u32x2 lo, hi;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo) : "v"(addr));
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "i"(OFF));       // k + 4
    return u32x4{lo.x, lo.y, hi.x, hi.y};
}

// K = 64 with both operands K-contiguous (A [M, 64], B given as [N, 64]: the scores q . k^T of attention and the
// gradient dO . v^T, on stacks of a few hundred matrices).  Such a product moves a byte of result per 64 flop: it is a
// stream of stores, and what a tile pipeline adds -- stages shared by a workgroup, a barrier per K step, a prologue and
// an epilogue that do not overlap -- only keeps its loads and stores from running side by side.  Here a wave is on its
// own: it loads 64 rows of A once and then STEPS blocks of 64 rows of B one after the other, the next block's loads in
// flight while this one is multiplied and stored, and never meets a barrier.  The operands are swapped in the MFMA, so
// that the four accumulators of a lane are four neighbouring columns of one row, and the B rows of two neighbouring
// column tiles are dealt out so that a lane's columns of both are eight in a row.  Rows of 128 bytes become fragments,
// and accumulators become rows, in a slab of LDS that belongs to the wave (see below).  The four waves of a workgroup
// cover 128 rows x 128 STEPS columns; what they share meets in the L1.
template <class T, int STEPS>
__global__ __launch_bounds__(256) void gemm_k64_nt_k(GemmArgs g, BatchArgs bt, u32 spread)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // workgroups go round the eight XCDs in the order of their numbers: with `spread` all tiles of a matrix are numbered
    // onto one XCD, so that its operands cross the fabric once and meet in one L2
    const u32 per = g.tiles_m * g.tiles_n;
    u32 matrix = blockIdx.x / per, tile = blockIdx.x - matrix * per;
    if (spread) {
        const u32 xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3;
        matrix = (idx / per) * 8u + xcd;
        tile = idx % per;
    }
    const u32 tn = tile % g.tiles_n, tm = tile / g.tiles_n;
    const u16* A = (const u16*)g.a;
    const u16* B = (const u16*)g.b;
    u16* C = (u16*)g.c;
    if (bt.table) {
        const u64* entry = bt.table + 3 * (u64)matrix;
        A = global_ptr<const u16>(entry[0]); B = global_ptr<const u16>(entry[1]); C = global_ptr<u16>(entry[2]);
    } else if (bt.rank) {
        u32 rest = matrix;
        for (int d = (int)bt.rank - 1; d >= 0; --d) {
            const u32 q = rest / bt.ext[d], c = rest - q * bt.ext[d];
            A += (u64)c * bt.sa[d]; B += (u64)c * bt.sb[d];
            rest = q;
        }
        C += (u64)matrix * bt.sc;
    }
    const u64 m0 = (u64)tm * 128 + (u64)(wave >> 1) * 64;
    const u64 n0 = (u64)tn * (128 * STEPS) + (u64)(wave & 1) * (64 * STEPS);
    const int r = lane & 15, kq = lane >> 4;
    // operand row r of the even tile of a pair is B row 8 (r / 4) + r % 4 of the pair's 32, of the odd tile that row + 4
    const int rb = 8 * (r >> 2) + (r & 3);
    // The wave's own slab: 32 rows of 128 bytes at a pitch of 144 (16 rows that differ in nothing else land in 16 different
    // banks).  Global memory is only ever touched by eight neighbouring lanes per 128-byte row -- a lane per row, which is
    // what the fragments and the accumulators are, costs the L1 a tag lookup per lane -- and the slab turns rows into
    // fragments and accumulators into rows.  A wave's LDS operations complete in order: no barrier anywhere.
    __shared__ __attribute__((aligned(16))) unsigned char slabs[4][32 * 144];
    unsigned char* slab = slabs[wave];
    const int lr = lane >> 3, lc = lane & 7;
    auto fetch32 = [&](const u16* base, u64 row0, u64 ld, u32x4 (&t)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) t[q] = *(const u32x4*)(base + (row0 + 8 * q + lr) * ld + 8 * lc);
    };
    auto to_slab = [&](const u32x4 (&t)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) *(u32x4*)(slab + (8 * q + lr) * 144 + 16 * lc) = t[q];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    auto fragment = [&](int row, int s) { return *(const u32x4*)(slab + row * 144 + 16 * (kq + 4 * s)); };
    u32x4 fa[4][2], fb[4][2], ta[2][4], tb[2][2][4];
    fetch32(A, m0, g.lda, ta[0]);
    fetch32(A, m0 + 32, g.lda, ta[1]);
    fetch32(B, n0, g.ldb, tb[0][0]);
    fetch32(B, n0 + 32, g.ldb, tb[0][1]);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        to_slab(ta[h]);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 2; ++s) fa[2 * h + t][s] = fragment(16 * t + r, s);
        asm volatile("" ::: "memory");
    }
#pragma unroll
    for (int step = 0; step < STEPS; ++step) {
        if (step + 1 < STEPS) {
            fetch32(B, n0 + 64 * (step + 1), g.ldb, tb[(step + 1) & 1][0]);
            fetch32(B, n0 + 64 * (step + 1) + 32, g.ldb, tb[(step + 1) & 1][1]);
        }
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            to_slab(tb[step & 1][pair]);
#pragma unroll
            for (int s = 0; s < 2; ++s) { fb[2 * pair][s] = fragment(rb, s); fb[2 * pair + 1][s] = fragment(4 + rb, s); }
            asm volatile("" ::: "memory");
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x4 acc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                acc[j] = Mma16<T>::run16(fb[j][0], fa[i][0], acc[j]);
                acc[j] = Mma16<T>::run16(fb[j][1], fa[i][1], acc[j]);
            }
            // lane (kq, r) holds row r, columns 32 p + 8 kq ... + 7 of pair p
#pragma unroll
            for (int pair = 0; pair < 2; ++pair) {
                const f32x4 lo = acc[2 * pair], hi = acc[2 * pair + 1];
                *(u32x4*)(slab + r * 144 + 64 * pair + 16 * kq) = u32x4{Mma16<T>::pack(lo.x, lo.y), Mma16<T>::pack(lo.z, lo.w), Mma16<T>::pack(hi.x, hi.y), Mma16<T>::pack(hi.z, hi.w)};
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const u32x4 v = *(const u32x4*)(slab + (lr + 8 * h) * 144 + 16 * lc);
                *(u32x4*)(C + (m0 + 16 * i + lr + 8 * h) * g.N + n0 + 64 * step + 8 * lc) = v;
            }
            asm volatile("" ::: "memory");
        }
    }
}

// PLANES: an f32 product on the bf16 pipe from operands that split_planes_k has laid out as three bf16 planes each (hi, mid,
// lo: K-contiguous, plane after plane): the K loop runs over the six plane pairs that carry the product to f32 accuracy,
// smallest terms first -- (lo, hi), (hi, lo), (mid, mid), (mid, hi), (hi, mid), (hi, hi) -- and the accumulators leave as
// f32; a lane whose accumulators hold an infinity or a NaN stores the launch's number into the flag word, as gemm_x3_k does.
struct PlanesArgs { u64 plane_a, plane_b; u32* flag; u32 seq; };      // bytes from one plane to the next

template <class T, bool AT, bool BT, int BM, int BN, bool PLANES = false>
__global__ __launch_bounds__(512) void gemm_direct16_k(GemmArgs g, BatchArgs bt, PlanesArgs pl)
{
    static_assert((BM == 128 && (BN == 128 || BN == 192 || BN == 256)) || (BM == 256 && BN == 256), "tiles this kernel is written for");
    static_assert(!PLANES || (!AT && !BT), "planes are laid out K-contiguous");
    constexpr int BK = 64, ASZ = BM * 128, BSZ = BN * 128, STAGE = ASZ + BSZ;
    constexpr int WGN = 4, TI = BM / 32, TJ = BN / 64, WROWS = TI * 16, WCOLS = TJ * 16;
    constexpr int LHA = BM / 64, LHB = BN / 64, LPW = LHA + LHB;     // loads per wave and tile
    constexpr int NF = TI + TJ, NB = 4;                              // fragments per slice; sub-blocks per phase
    constexpr int PA = 2 * BM, PB = 2 * BN;                          // bytes per k-row of a T-form stage
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), wm = wave / WGN, wn = wave % WGN;
    // blockIdx.y numbers the matrices of a stack, or the separate products of a group (addresses from a table)
    u64 base_a = (u64)(size_t)g.a, base_b = (u64)(size_t)g.b, base_c = (u64)(size_t)g.c;
    if (bt.table) {
        const u64* entry = bt.table + 3 * (u64)blockIdx.y;
        base_a = entry[0]; base_b = entry[1]; base_c = entry[2];
    } else if (bt.rank) {
        u32 rest = blockIdx.y;
        for (int d = (int)bt.rank - 1; d >= 0; --d) {
            const u32 q = rest / bt.ext[d], c = rest - q * bt.ext[d];
            base_a += (u64)c * bt.sa[d] * 2; base_b += (u64)c * bt.sb[d] * 2;
            rest = q;
        }
        base_c += (u64)blockIdx.y * bt.sc * 2;
    }
    const char* ga = global_ptr<const char>(base_a);
    const char* gb = global_ptr<const char>(base_b);

    // producer.  K-contiguous: load n of a wave fills the 8-row block wave * LH + n (128 bytes per row, 8 lanes per row);
    // T form: the wave fills k-rows 8 wave .. 8 wave + 7, load n the bytes 1024 n .. 1024 n + 1023 of them.
    const int lr = lane >> 3;
    const int fe = (lr >> 1) ^ ((lr & 1) << 2);
    u32 oa[AT ? LHA : 2], ob[BT ? LHB : 2];
    const char* A;
    const char* B;
    if constexpr (AT) {
        A = ga + m0 * 2 + (u64)(wave * 8) * g.lda * 2;
#pragma unroll
        for (int n = 0; n < LHA; ++n) {
            const int pos = n * 1024 + lane * 16, kq = pos / PA, slot = (pos % PA) / 16;
            oa[n] = (u32)((kq * g.lda + (u64)((slot ^ tform_swizzle<PA>(kq, wave & 1)) * 8)) * 2);
        }
    } else {
        A = ga + (m0 + (u64)wave * LHA * 8) * g.lda * 2;
        const int par = (LHA & 1) ? (wave & 1) : 0;                  // parity of the wave's first block
        oa[0] = (u32)((lr * g.lda + (u64)(((lane & 7) ^ fe ^ (4 * par)) * 8)) * 2);
        oa[1] = (u32)((lr * g.lda + (u64)(((lane & 7) ^ fe ^ (4 * par) ^ 4) * 8)) * 2);
    }
    if constexpr (BT) {
        B = gb + n0 * 2 + (u64)(wave * 8) * g.ldb * 2;
#pragma unroll
        for (int n = 0; n < LHB; ++n) {
            const int pos = n * 1024 + lane * 16, kq = pos / PB, slot = (pos % PB) / 16;
            ob[n] = (u32)((kq * g.ldb + (u64)((slot ^ tform_swizzle<PB>(kq, wave & 1)) * 8)) * 2);
        }
    } else {
        B = gb + (n0 + (u64)wave * LHB * 8) * g.ldb * 2;
        const int par = (LHB & 1) ? (wave & 1) : 0;
        ob[0] = (u32)((lr * g.ldb + (u64)(((lane & 7) ^ fe ^ (4 * par)) * 8)) * 2);
        ob[1] = (u32)((lr * g.ldb + (u64)(((lane & 7) ^ fe ^ (4 * par) ^ 4) * 8)) * 2);
    }
    const u64 ca = 16 * g.lda, cb = 16 * g.ldb;                                          // bytes between 8-row blocks (K-contiguous)
    const u64 sa = AT ? (u64)BK * g.lda * 2 : (u64)BK * 2, sb = BT ? (u64)BK * g.ldb * 2 : (u64)BK * 2;   // bytes between K-steps
    const int per_pair = (int)(g.K / BK), steps = PLANES ? 6 * per_pair : per_pair;
    // where K-step `ki` starts, in bytes from the operands' bases (PLANES: pair ki / per_pair, step ki % per_pair of it)
    auto step_a = [&](int ki) -> u64 {
        if constexpr (PLANES) { const int pr = ki / per_pair; return (u64)((0x052u >> (2 * pr)) & 3u) * pl.plane_a + (u64)(ki - pr * per_pair) * sa; }
        else return (u64)ki * sa;
    };
    auto step_b = [&](int ki) -> u64 {
        if constexpr (PLANES) { const int pr = ki / per_pair; return (u64)((0x118u >> (2 * pr)) & 3u) * pl.plane_b + (u64)(ki - pr * per_pair) * sb; }
        else return (u64)ki * sb;
    };

    // consumer.  K-contiguous: lane reads row (lane & 15) of a 16-row block, k-chunk 4 s + (lane >> 4) of slice s.
    // T form: lane j of a 16-lane group points at k-row 32 s + 8 grp + (j >> 2) [+ 4], columns 4 (j & 3) .. + 3 of the block.
    const int r15 = lane & 15, grp = lane >> 4, tq = r15 >> 2;
    const int slot0 = grp ^ (((r15 >> 1) & 7) ^ ((r15 & 1) << 2));
    int fra[AT ? TI : 1], frb[BT ? TJ : 1];
    if constexpr (AT) {
#pragma unroll
        for (int f = 0; f < TI; ++f)
            fra[f] = (8 * grp + tq) * PA + 8 * (r15 & 1) + (((wm * (WROWS / 8) + 2 * f + ((r15 & 3) >> 1)) ^ tform_swizzle<PA>(tq, grp & 1)) * 16);
    } else fra[0] = (wm * WROWS + r15) * 128 + slot0 * 16;
    if constexpr (BT) {
#pragma unroll
        for (int f = 0; f < TJ; ++f)
            frb[f] = ASZ + (8 * grp + tq) * PB + 8 * (r15 & 1) + (((wn * (WCOLS / 8) + 2 * f + ((r15 & 3) >> 1)) ^ tform_swizzle<PB>(tq, grp & 1)) * 16);
    } else frb[0] = ASZ + (wn * WCOLS + r15) * 128 + slot0 * 16;

    f32x4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    u32x4 fa[2][TI], fb[2][TJ];

    // load n of the tile that starts ka / kb bytes into the operands
    auto load = [&](auto n_, u64 ka, u64 kb, int bo) {
        constexpr int n = decltype(n_)::v;
        if constexpr (n < LHA) {
            const char* src = AT ? A + ka + oa[AT ? n : 0] : A + (n * ca + ka) + oa[n & 1];
            __builtin_amdgcn_global_load_lds(AIX_GLB(src), AIX_LDS(smem + bo + (wave * LHA + n) * 1024), 16, 0, 0);
        } else {
            constexpr int m = n - LHA;
            const char* src = BT ? B + kb + ob[BT ? m : 0] : B + (m * cb + kb) + ob[m & 1];
            __builtin_amdgcn_global_load_lds(AIX_GLB(src), AIX_LDS(smem + bo + ASZ + (wave * LHB + m) * 1024), 16, 0, 0);
        }
    };
    auto read = [&](int set, int bo, int s, auto f_) {
        constexpr int f = decltype(f_)::v;
        if constexpr (f < TI) {
            if constexpr (AT) fa[set][f] = tr_fragment_at<4 * PA>(smem + bo + fra[AT ? f : 0] + s * 32 * PA);
            else fa[set][f] = *(const u32x4*)(smem + bo + (fra[0] ^ (s * 64)) + f * 2048);
        } else {
            constexpr int e = f - TI;
            if constexpr (BT) fb[set][e] = tr_fragment_at<4 * PB>(smem + bo + frb[BT ? e : 0] + s * 32 * PB);
            else fb[set][e] = *(const u32x4*)(smem + bo + (frb[0] ^ (s * 64)) + e * 2048);
        }
    };
    // MFMAs on fragment set FC while set FN is read from stage rbo, slice S; with LOADS, tile `ko` goes to stage lbo
    auto phase = [&](auto FC_, auto FN_, int rbo, auto S_, auto LOADS_, u64 ka, u64 kb, int lbo) {
        constexpr int FC = decltype(FC_)::v, FN = decltype(FN_)::v, S = decltype(S_)::v, LOADS = decltype(LOADS_)::v;
        if constexpr (AT || BT) { AIX_SB(); __builtin_amdgcn_s_waitcnt(0xC07F); AIX_SB(); }     // lgkmcnt(0): fragment set FC has arrived
        auto block = [&]<int b>(Const<b>) {
            [&]<int... f>(std::integer_sequence<int, f...>) {
                (read(FN, rbo, S, Const<b * NF / NB + f>{}), ...);
            }(std::make_integer_sequence<int, (b + 1) * NF / NB - b * NF / NB>{});
            if constexpr (LOADS) {
                [&]<int... n>(std::integer_sequence<int, n...>) {
                    (load(Const<b * LPW / NB + n>{}, ka, kb, lbo), ...);
                }(std::make_integer_sequence<int, (b + 1) * LPW / NB - b * LPW / NB>{});
            }
#pragma unroll
            for (int i = b * TI / NB; i < (b + 1) * TI / NB; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) acc[i][j] = Mma16<T>::run16(fa[FC][i], fb[FC][j], acc[i][j]);
            AIX_SB();
        };
        block(Const<0>{}); block(Const<1>{}); block(Const<2>{}); block(Const<3>{});
    };

    {
        const int k1 = 1 < steps ? 1 : 0;
        const u64 a0 = step_a(0), b0 = step_b(0), a1 = step_a(k1), b1 = step_b(k1);
        [&]<int... n>(std::integer_sequence<int, n...>) { (load(Const<n>{}, a0, b0, 0), ...); }(std::make_integer_sequence<int, LPW>{});
        [&]<int... n>(std::integer_sequence<int, n...>) { (load(Const<n>{}, a1, b1, STAGE), ...); }(std::make_integer_sequence<int, LPW>{});
    }
    AIX_SB();
    AIX_WAIT(LPW, 15);                                        // tile 0 has landed (the loads of tile 1 may be in flight)
    __builtin_amdgcn_s_barrier();
    AIX_SB();
    [&]<int... f>(std::integer_sequence<int, f...>) { (read(0, 0, 0, Const<f>{}), ...); }(std::make_integer_sequence<int, NF>{});
    for (int kt = 0; kt < steps; ++kt) {
        const int bo = (kt & 1) * STAGE, nbo = bo ^ STAGE;
        const int k2 = kt + 2 < steps ? kt + 2 : steps - 1;
        const u64 a2 = step_a(k2), b2 = step_b(k2);
        phase(Const<0>{}, Const<1>{}, bo, Const<1>{}, Const<0>{}, a2, b2, nbo);
        AIX_WAIT(0, 0);                                       // tile kt+1 complete in the other stage; own reads of this stage done
        __builtin_amdgcn_s_barrier();
        AIX_SB();
        phase(Const<1>{}, Const<0>{}, nbo, Const<0>{}, Const<1>{}, a2, b2, bo);
    }
    AIX_WAIT(0, 0);                                           // stray loads have landed before LDS is reused
    __builtin_amdgcn_s_barrier();
    AIX_SB();

    // Epilogue through LDS, each wave on its own slab: 16 rows of the wave's 64 x WCOLS block row-major (pitch WCOLS + 4
    // floats), read back as runs of 8 columns, rounded and stored with 16-byte non-temporal writes.
    constexpr int PITCH = WCOLS + 4, RUNS = 16 * (WCOLS / 8);
    float* slab = (float*)smem + wave * (16 * PITCH + 64);
    if constexpr (PLANES) {
        float probe = 0.0f;                                   // x * 0 is a NaN for an infinity or a NaN, else a zero
        float* Cf = global_ptr<float>(base_c);
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) { slab[(4 * grp + v) * PITCH + j * 16 + r15] = acc[i][j][v]; probe += acc[i][j][v] * 0.0f; }
#pragma unroll
            for (int t = 0; t < (2 * RUNS + 63) / 64; ++t) {                  // runs of 4 columns: 16 bytes of f32
                const int run = lane + 64 * t, row = run / (WCOLS / 4), cg = run % (WCOLS / 4);
                if ((2 * RUNS) % 64 == 0 || run < 2 * RUNS)
                    __builtin_nontemporal_store(*(const f32x4*)(slab + row * PITCH + cg * 4),
                                                (f32x4*)(Cf + (m0 + wm * WROWS + i * 16 + row) * g.N + n0 + wn * WCOLS + cg * 4));
            }
        }
        if (probe != probe) *pl.flag = pl.seq;
        return;
    }
    u16* C = global_ptr<u16>(base_c);
#pragma unroll
    for (int i = 0; i < TI; ++i) {
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) slab[(4 * grp + v) * PITCH + j * 16 + r15] = acc[i][j][v];
#pragma unroll
        for (int t = 0; t < (RUNS + 63) / 64; ++t) {
            const int run = lane + 64 * t, row = run / (WCOLS / 8), cg = run % (WCOLS / 8);
            if (RUNS % 64 == 0 || run < RUNS) {
                const f32x4 lo = *(const f32x4*)(slab + row * PITCH + cg * 8);
                const f32x4 hi = *(const f32x4*)(slab + row * PITCH + cg * 8 + 4);
                u32x4 o;
                o.x = Mma16<T>::pack(lo.x, lo.y); o.y = Mma16<T>::pack(lo.z, lo.w);
                o.z = Mma16<T>::pack(hi.x, hi.y); o.w = Mma16<T>::pack(hi.z, hi.w);
                __builtin_nontemporal_store(o, (u32x4*)(C + (m0 + wm * WROWS + i * 16 + row) * g.N + n0 + wn * WCOLS + cg * 8));
            }
        }
    }
}
#undef AIX_GLB
#undef AIX_LDS
#undef AIX_WAIT
#undef AIX_SB

// ---- 16-bit operands, small problems --------------------------------------------------------------
// For outputs that 64 x 64 tiles cannot spread over the chip (the per-head matmuls of attention,
// [512, 64] x [64, 512] and the like): a 32 x 32 tile per workgroup and the K dimension split over the
// workgroup's four waves.  Wave w owns the 64-wide K steps w, w + 4, ...: it fetches its own operand
// tiles (8 independent 16-byte loads per lane, the next step's in flight under the current step's
// MFMAs), stages them in its own part of LDS and never waits for the other waves -- with so few
// workgroups nothing else hides the latency of a K step, so the chain is made a quarter as long --
// and the four partial tiles are added through LDS at the end.
//
// Both operands are consumed where they lie.  A K-contiguous operand is staged as [row][k] (pitch 72
// elements) and read with ds_read_b128, as in gemm_nt16_k.  A T-form operand (A given as [K, M] with
// unit stride along M, B as plain row-major [K, N]) is staged as it comes, [k][row] with a pitch of
// 96 elements, and the fragments -- 8 consecutive k per lane -- are assembled by ds_read_b64_tr_b16
// (see gemm_nt16_direct_k for the lane mapping); 192 bytes between k-rows put the four k-rows that a
// group of 16 lanes reads, and the two groups of a half-wave, into disjoint banks.
typedef short s16x4 __attribute__((ext_vector_type(4)));

template <int PT>
__device__ __forceinline__ u32x4 tr_fragment_lds(const u16* p)
{
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p + 4 * PT));     // k + 4
    const u32x2 l = __builtin_bit_cast(u32x2, lo), h = __builtin_bit_cast(u32x2, hi);
    return u32x4{l.x, l.y, h.x, h.y};
}

template <bool AT, bool BT> struct Small16 {
    static constexpr int BM = 32, BN = 32, BK = 64, PK = BK + 8, PT = 96;
    static constexpr int SA = AT ? BK * PT : BM * PK, SB = BT ? BK * PT : BN * PK;      // elements per wave
    static constexpr size_t kLds = (size_t)4 * (SA + SB) * 2 > 16384 ? (size_t)4 * (SA + SB) * 2 : 16384;   // the stages double as the reduction buffer
};

template <class T, bool AT, bool BT>
__global__ __launch_bounds__(256) void gemm_small16_k(GemmArgs g, BatchArgs bt)
{
    typedef Small16<AT, BT> S;
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, PK = S::PK, PT = S::PT, SA = S::SA, SB = S::SB;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_small[];

    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const u16* A = (const u16*)g.a;
    const u16* B = (const u16*)g.b;
    T* C = (T*)g.c;
    if (bt.table) {
        const u64* entry = bt.table + 3 * (u64)blockIdx.y;
        A = global_ptr<const u16>(entry[0]); B = global_ptr<const u16>(entry[1]); C = global_ptr<T>(entry[2]);
    } else if (bt.rank) {                                    // uniform over the workgroup: scalar arithmetic
        u32 rest = blockIdx.y;
        for (int d = (int)bt.rank - 1; d >= 0; --d) {
            const u32 q = rest / bt.ext[d], c = rest - q * bt.ext[d];
            A += (u64)c * bt.sa[d]; B += (u64)c * bt.sb[d];
            rest = q;
        }
        C += (u64)blockIdx.y * bt.sc;
    }
    u16* as = (u16*)smem_small + wave * (SA + SB);           // this wave's stage
    u16* bs = as + SA;

    // four 16-byte chunks per lane, operand and step: chunk c = lane + 64 i is (row c / 8, k 8 (c % 8)) of a
    // K-contiguous tile, (k-row c / 4, column 8 (c % 4)) of a T-form tile
    u32x4 ra[4], rb[4];
    auto load_global = [&](u64 k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = lane + 64 * i;
            if constexpr (AT) { const u64 k = k0 + (c >> 2), m = m0 + (c & 3) * 8; ra[i] = (k < g.K && m < g.M) ? *(const u32x4*)(A + k * g.lda + m) : (u32x4){0, 0, 0, 0}; }
            else { const u64 m = m0 + (c >> 3), k = k0 + (c & 7) * 8; ra[i] = (m < g.M && k < g.K) ? *(const u32x4*)(A + m * g.lda + k) : (u32x4){0, 0, 0, 0}; }
            if constexpr (BT) { const u64 k = k0 + (c >> 2), n = n0 + (c & 3) * 8; rb[i] = (k < g.K && n < g.N) ? *(const u32x4*)(B + k * g.ldb + n) : (u32x4){0, 0, 0, 0}; }
            else { const u64 n = n0 + (c >> 3), k = k0 + (c & 7) * 8; rb[i] = (n < g.N && k < g.K) ? *(const u32x4*)(B + n * g.ldb + k) : (u32x4){0, 0, 0, 0}; }
        }
    };
    auto store_lds = [&] {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = lane + 64 * i;
            *(u32x4*)(as + (AT ? (c >> 2) * PT + (c & 3) * 8 : (c >> 3) * PK + (c & 7) * 8)) = ra[i];
            *(u32x4*)(bs + (BT ? (c >> 2) * PT + (c & 3) * 8 : (c >> 3) * PK + (c & 7) * 8)) = rb[i];
        }
    };
    // fragment addresses inside a stage for the 16-wide K slice 0; slice kk adds 16 k
    const int j = lane & 15;
    const int tro = (8 * (lane >> 5) + (j >> 2)) * PT + 16 * ((lane >> 4) & 1) + 4 * (j & 3);
    const int kro = (lane & 31) * PK + (lane >> 5) * 8;

    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

    const u64 steps = (g.K + BK - 1) / BK;
    u64 kt = (u64)wave;
    if (kt < steps) load_global(kt * BK);
    for (; kt < steps; kt += 4) {
        store_lds();                                          // the wave's LDS operations execute in order: no barrier inside a wave
        if (kt + 4 < steps) load_global((kt + 4) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4 fa, fb;
            if constexpr (AT) fa = tr_fragment_lds<PT>(as + tro + kk * 16 * PT); else fa = *(const u32x4*)(as + kro + kk * 16);
            if constexpr (BT) fb = tr_fragment_lds<PT>(bs + tro + kk * 16 * PT); else fb = *(const u32x4*)(bs + kro + kk * 16);
            acc = Mma16<T>::run(fa, fb, acc);
        }
    }

    // add the four waves' partial tiles: slot e = 64 v + lane holds accumulator element v of lane `lane`
    __syncthreads();
    float* red = (float*)smem_small;
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wave * 1024 + v * 64 + lane] = acc[v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + 256 * i, v = e >> 6, l = e & 63;
        const float sum = (red[e] + red[1024 + e]) + (red[2048 + e] + red[3072 + e]);
        const u64 row = m0 + (v >> 2) * 8 + (l >> 5) * 4 + (v & 3), col = n0 + (l & 31);
        if (row < g.M && col < g.N) C[row * g.N + col] = Mma16<T>::out(sum);
    }
}

// ---- 16-bit operands, mid-size problems and stacks of matrices --------------------------------------
// Everything between the two kernels above: outputs of a few hundred tiles (a [8192, 768] activation times a
// [768, 768] weight), weight gradients with few tiles and a very long K ([768, 8192] x [8192, 768]), and stacks of
// attention-sized products.  BM x BN workgroup tile (128 x 128, 128 x 64, 64 x 64), BK = 32, four waves 2 x 2,
// two LDS stages filled from registers -- for interior tiles from a ring of register stages that keeps the global
// loads of the next 2-3 K steps in flight, for edge tiles one step ahead -- one barrier per step; 41 KB of LDS at
// most, so several workgroups share a compute unit and overlap each other's barriers and LDS reads.  Results leave
// through LDS as 16-byte stores.  Both operand forms are consumed where they lie: K-contiguous staged [row][k], unpadded, with
// the 16-byte chunks of a row XOR-swizzled (kswz below); T form staged [k][row] with a pitch of tile + 32 elements (64 or
// 192 bytes modulo 256: the four k-rows a group of 16 lanes reads with ds_read_b64_tr_b16, and the two groups of a
// half-wave, fall into disjoint banks).  SQ_LDS_BANK_CONFLICT = 0 for both.
//
// blockIdx.y numbers the matrices of a stack (BatchArgs).  blockIdx.z numbers K splits: split s multiplies K steps
// [s * per_split, (s + 1) * per_split) and, when there is more than one split, stores its f32 partial tile in
// `partial` ([split][matrix][M][N]) for splitk_finish_k to add up in split order and round once.
struct SplitArgs { float* partial; u32 splits, per_split; u64 matrices; };

// K-contiguous operands are staged without padding: row r keeps its 16-byte k-chunk q in slot q ^ kswz<BK>(r).  A group of 8
// (or 16) lanes that writes whole rows then covers 128 (256) contiguous bytes, and the fragment reads -- 32 consecutive
// rows, one chunk -- fall into disjoint banks under both an 8-lane / 32-bank and a 16-lane / 64-bank service (padded rows
// of 80 bytes read without conflicts but cost a third of the LDS cycles in write conflicts, by SQ_LDS_BANK_CONFLICT).
// Only bits 0..3 of r enter, so a row's swizzle is known from the lane that owns it.
template <int BK> __device__ __forceinline__ int kswz(int r)
{
    if constexpr (BK == 64) return ((r >> 1) & 7) ^ ((r & 1) << 2);          // 8 chunks per row (gemm_nt16_direct_k's)
    else return (r ^ (r >> 2)) & 3;                                           // 4 chunks per row
}

template <int BM, int BN, int BK_, bool AT, bool BT> struct Tile16 {
    static constexpr int BK = BK_, PA = BM + 32, PB = BN + 32;
    static constexpr int SA = AT ? BK * PA : BM * BK, SB = BT ? BK * PB : BN * BK;       // elements per stage
    static constexpr size_t kLds = (size_t)2 * (SA + SB) * 2;
};

template <class T, int BM, int BN, int BKT, bool AT, bool BT, int RING = 0>
__global__ __launch_bounds__(256) void gemm_tile16_k(GemmArgs g, BatchArgs bt, SplitArgs sk)
{
    typedef Tile16<BM, BN, BKT, AT, BT> S;
    constexpr int BK = S::BK, PA = S::PA, PB = S::PB, SA = S::SA, SB = S::SB;
    constexpr int WM = BM / 2, WN = BN / 2, TI = WM / 32, TJ = WN / 32;
    constexpr int CA = BM * (BK / 8) / 256, CB = BN * (BK / 8) / 256;        // 16-byte chunks per lane and step
    constexpr int CH = BK / 8;                                                // chunks per K-contiguous row
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_tile[];
    u16* As = (u16*)smem_tile;                            // [2][SA]
    u16* Bs = As + 2 * SA;                                // [2][SB]

    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const u16* A = (const u16*)g.a;
    const u16* B = (const u16*)g.b;
    if (bt.table) {
        const u64* entry = bt.table + 3 * (u64)blockIdx.y;
        A = global_ptr<const u16>(entry[0]); B = global_ptr<const u16>(entry[1]);
    } else if (bt.rank) {                                    // uniform over the workgroup: scalar arithmetic
        u32 rest = blockIdx.y;
        for (int d = (int)bt.rank - 1; d >= 0; --d) {
            const u32 q = rest / bt.ext[d], c = rest - q * bt.ext[d];
            A += (u64)c * bt.sa[d]; B += (u64)c * bt.sb[d];
            rest = q;
        }
    }

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // Register stages between global memory and LDS.  A tile whose rows, columns and K steps all lie inside the operands
    // ("interior") is fetched by unconditional loads, DEPTH K-steps ahead: only then can the in-order load counter tell
    // "the oldest tile has arrived" from "everything has arrived" (a load under a bounds check is a branch, and behind a
    // branch the compiler waits for every load in flight), and with 4-8 MFMAs per wave and step nothing but that distance
    // covers the latency of a load.  Edge tiles take the checked loads, one step ahead.
    constexpr int DEPTH = RING ? RING : BM * BN >= 128 * 128 ? 2 : 3;      // registers: the 128 x 128 tile keeps three waves per SIMD with 2
    u32x4 ra[DEPTH][CA], rb[DEPTH][CB];
    auto load_global = [&](u64 k0, u32x4* pa, u32x4* pb) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            if constexpr (AT) { const u64 k = k0 + c / (BM / 8), m = m0 + (c % (BM / 8)) * 8; pa[i] = (k < g.K && m < g.M) ? *(const u32x4*)(A + k * g.lda + m) : (u32x4){0, 0, 0, 0}; }
            else { const u64 m = m0 + c / (BK / 8), k = k0 + (c % (BK / 8)) * 8; pa[i] = (m < g.M && k < g.K) ? *(const u32x4*)(A + m * g.lda + k) : (u32x4){0, 0, 0, 0}; }
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            if constexpr (BT) { const u64 k = k0 + c / (BN / 8), n = n0 + (c % (BN / 8)) * 8; pb[i] = (k < g.K && n < g.N) ? *(const u32x4*)(B + k * g.ldb + n) : (u32x4){0, 0, 0, 0}; }
            else { const u64 n = n0 + c / (BK / 8), k = k0 + (c % (BK / 8)) * 8; pb[i] = (n < g.N && k < g.K) ? *(const u32x4*)(B + n * g.ldb + k) : (u32x4){0, 0, 0, 0}; }
        }
    };
    // the same without checks: the lane's part of the address once, the K step enters as a uniform offset
    const u16 *ga[CA], *gb[CB];
#pragma unroll
    for (int i = 0; i < CA; ++i) {
        const int c = tid + 256 * i;
        ga[i] = AT ? A + (u64)(c / (BM / 8)) * g.lda + m0 + (c % (BM / 8)) * 8 : A + (m0 + c / (BK / 8)) * g.lda + (c % (BK / 8)) * 8;
    }
#pragma unroll
    for (int i = 0; i < CB; ++i) {
        const int c = tid + 256 * i;
        gb[i] = BT ? B + (u64)(c / (BN / 8)) * g.ldb + n0 + (c % (BN / 8)) * 8 : B + (n0 + c / (BK / 8)) * g.ldb + (c % (BK / 8)) * 8;
    }
    const u64 ka = AT ? (u64)BK * g.lda : (u64)BK, kb = BT ? (u64)BK * g.ldb : (u64)BK;      // elements per K step
    auto load_interior = [&](u64 kt, u32x4* pa, u32x4* pb) {
#pragma unroll
        for (int i = 0; i < CA; ++i) pa[i] = *(const u32x4*)(ga[i] + kt * ka);
#pragma unroll
        for (int i = 0; i < CB; ++i) pb[i] = *(const u32x4*)(gb[i] + kt * kb);
    };
    auto store_lds = [&](int buf, const u32x4* pa, const u32x4* pb) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            *(u32x4*)(As + buf * SA + (AT ? (c / (BM / 8)) * PA + (c % (BM / 8)) * 8 : (c / CH) * BK + ((c % CH) ^ kswz<BK>(c / CH)) * 8)) = pa[i];
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            *(u32x4*)(Bs + buf * SB + (BT ? (c / (BN / 8)) * PB + (c % (BN / 8)) * 8 : (c / CH) * BK + ((c % CH) ^ kswz<BK>(c / CH)) * 8)) = pb[i];
        }
    };
    // fragment addresses inside a stage for the wave's first 32 rows: T form for the 16-wide K slice 0; K-contiguous: the
    // row's start, the chunk (lane / 32 + 2 kk) goes through the row's swizzle
    const int j16 = lane & 15, swz = kswz<BK>(lane & 31), half = lane >> 5;
    const int fa0 = AT ? (8 * (lane >> 5) + (j16 >> 2)) * PA + 16 * ((lane >> 4) & 1) + 4 * (j16 & 3) + wm * WM : (wm * WM + (lane & 31)) * BK;
    const int fb0 = BT ? (8 * (lane >> 5) + (j16 >> 2)) * PB + 16 * ((lane >> 4) & 1) + 4 * (j16 & 3) + wn * WN : (wn * WN + (lane & 31)) * BK;

    const u64 steps = (g.K + BK - 1) / BK;
    const u64 first = (u64)blockIdx.z * sk.per_split;
    const u64 last = first + sk.per_split < steps ? first + sk.per_split : steps;
    auto multiply = [&](int buf) {
        const u16* as = As + buf * SA + fa0;
        const u16* bs = Bs + buf * SB + fb0;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4 fa[TI], fb[TJ];
            const int slot = ((half + 2 * kk) ^ swz) * 8;
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                if constexpr (AT) fa[i] = tr_fragment_lds<PA>(as + i * 32 + kk * 16 * PA); else fa[i] = *(const u32x4*)(as + i * 32 * BK + slot);
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                if constexpr (BT) fb[j] = tr_fragment_lds<PB>(bs + j * 32 + kk * 16 * PB); else fb[j] = *(const u32x4*)(bs + j * 32 * BK + slot);
            }
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) acc[i][j] = Mma16<T>::run(fa[i], fb[j], acc[i][j]);
        }
    };
    // (short K: the ring's first loads would fetch the last tile over and over)
    const bool interior = m0 + BM <= g.M && n0 + BN <= g.N && g.K % BK == 0 && last - first >= 2 * DEPTH + 2;
    u64 kt = first;
    if (first < last) {
        if (interior) {
            // ring slot d holds tile t + 1 when step t = first + d (mod DEPTH) begins; tiles past the end re-read the last one
            const u64 end = last - 1;
            load_interior(first, ra[0], rb[0]);
            store_lds(0, ra[0], rb[0]);
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) { const u64 t = first + 1 + d; load_interior(t < end ? t : end, ra[d], rb[d]); }
            __syncthreads();
            // whole turns of the ring, in a loop without exits between the steps (an exit would merge states in which different
            // slots hold the youngest loads, and the wait for one slot would become a wait for all)
            for (; kt + DEPTH <= last; kt += DEPTH) {
#pragma unroll
                for (int d = 0; d < DEPTH; ++d) {
                    const u64 t = kt + d, nt = t + 1 + DEPTH;
                    const int buf = (int)((t - first) & 1);
                    store_lds(buf ^ 1, ra[d], rb[d]);                 // tile t + 1 (behind the last step: a copy nobody reads)
                    load_interior(nt < end ? nt : end, ra[d], rb[d]);
                    multiply(buf);
                    __syncthreads();
                }
            }
        } else {
            load_global(first * BK, ra[0], rb[0]);
            store_lds(0, ra[0], rb[0]);
        }
    }
    __syncthreads();
    // edge tiles, and the steps an interior tile has left after the last whole turn (its tile kt is staged already)
    for (; kt < last; ++kt) {
        const int buf = (int)((kt - first) & 1);
        if (kt + 1 < last) load_global((kt + 1) * BK, ra[0], rb[0]);
        multiply(buf);
        if (kt + 1 < last) store_lds(buf ^ 1, ra[0], rb[0]);
        __syncthreads();
    }

    // accumulator element v of lane l: row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
    const u64 plane = g.M * g.N;
    T* C = bt.table ? global_ptr<T>(bt.table[3 * (u64)blockIdx.y + 2]) : (T*)g.c + (u64)blockIdx.y * plane;
    float* P = sk.splits > 1 ? sk.partial + ((u64)blockIdx.z * sk.matrices + blockIdx.y) * plane : nullptr;
    if (!P && g.N % 8 == 0 && ((size_t)g.c & 15) == 0) {
        // Through LDS (free after the last barrier), each wave on its own 32 x 32 slab: written as the MFMA leaves it (a lane
        // = a column), read back as runs of 8 columns, rounded and stored 16 bytes per lane: an eighth of the store
        // instructions of two-byte stores straight from the accumulators (4-8 % of a [8192, 768] x [768, 768] product; the
        // f32 partial tiles of a K split gain nothing from the detour and go out directly).
        constexpr int PITCH = 36;
        static_assert((size_t)4 * 32 * PITCH * 4 <= S::kLds, "the epilogue slabs fit into the stages");
        float* slab = (float*)smem_tile + wave * (32 * PITCH);
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
#pragma unroll
                for (int v = 0; v < 16; ++v) slab[((v >> 2) * 8 + (lane >> 5) * 4 + (v & 3)) * PITCH + (lane & 31)] = acc[i][j][v];
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int grp = lane + 64 * t, r = grp >> 2, cg = grp & 3;
                    const f32x4 lo = *(const f32x4*)(slab + r * PITCH + cg * 8);
                    const f32x4 hi = *(const f32x4*)(slab + r * PITCH + cg * 8 + 4);
                    const u64 row = m0 + wm * WM + i * 32 + r, col = n0 + wn * WN + j * 32 + cg * 8;
                    if (row < g.M && col < g.N) {
                        u32x4 o;
                        o.x = Mma16<T>::pack(lo.x, lo.y); o.y = Mma16<T>::pack(lo.z, lo.w);
                        o.z = Mma16<T>::pack(hi.x, hi.y); o.w = Mma16<T>::pack(hi.z, hi.w);
                        *(u32x4*)(C + row * g.N + col) = o;
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const u64 col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const u64 row = m0 + wm * WM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.M && col < g.N) {
                    if (P) P[row * g.N + col] = acc[i][j][v];
                    else C[row * g.N + col] = Mma16<T>::out(acc[i][j][v]);
                }
            }
        }
}

// out[e] = the partial results of all K splits added in split order, rounded once.
template <class T>
__global__ __launch_bounds__(256) void splitk_finish_k(const float* __restrict__ partial, T* __restrict__ out, u64 total, u32 splits)
{
    for (u64 e = (u64)blockIdx.x * 256 + threadIdx.x; e < total; e += (u64)gridDim.x * 256) {
        float sum = partial[e];
        for (u32 s = 1; s < splits; ++s) sum += partial[(u64)s * total + e];
        out[e] = Mma16<T>::out(sum);
    }
}

// ---- f32 operands on the bf16 matrix pipe ------------------------------------------------------------
// The f32 MFMA runs at 1/16 of the bf16 rate.  An f32 value is the exact sum of three bf16 values (8 + 8 + 8
// significand bits: hi = x truncated to its upper 16 bits, mid = RNE(x - hi), lo = RNE(x - hi - mid); the exponent
// range is the same, so nothing overflows or underflows that f32 itself does not), and a product of two bf16 values
// is exact in f32.  So A . B = sum over the six plane pairs (hi hi, hi mid, mid hi, mid mid, hi lo, lo hi) of bf16
// MFMAs accumulating in f32; the three pairs left out (mid lo, lo mid, lo lo) are below 2^-23 of |a| |b| per term --
// the size of f32's own rounding of a product -- and the accumulation is the f32 accumulation of the matrix unit
// either way.  Six bf16 MFMAs cost 6/16 of one f32 MFMA of the same shape.
//
// gemm_x3_k: 128 x 128 x 32 tile, four waves 2 x 2.  The operands are read from memory as f32 (K-contiguous or T
// form, 16-byte chunks of four values), split in registers, and staged as three bf16 planes per operand with the
// layouts of gemm_tile16_k (so the fragment reads, including ds_read_b64_tr_b16 for T-form operands, are the same);
// a wave reads 12 fragments per 24 MFMAs.  One LDS stage of 48-60 KB (two workgroups per compute unit) and two barriers
// per K step: the next step's global loads are in flight during the MFMAs.  blockIdx.z numbers K splits as in
// gemm_tile16_k.
//
// Infinities and NaNs do not survive the split (inf - inf, and inf times a zero mid or lo plane of the other operand),
// but they cannot hide either: every operand element meets a nonzero hi plane or a zero, so a non-finite input leaves
// an infinity or a NaN in some accumulator of its row or column.  A lane that ends up with one stores the launch's
// number into a flag word, and the f32 MFMA kernel that is always launched right behind -- its workgroups return at
// once unless the flag carries this number -- redoes the whole product with IEEE arithmetic (which also covers sums
// that overflow on their own: the redo returns the same infinities).
//
// The planes also have f32's exponent range only down to where their last bits fall off the bf16 grid: the three planes
// of x carry its 24 significand bits as multiples of 2^(e - 23), and bf16 ends at 2^-133 (its subnormals, which the
// matrix unit takes as they are, like f32 subnormals in its products and accumulators), so an operand below 2^-110 is
// no longer the sum of its planes (2^-116: 1e-5 off, f32 subnormals: all three planes zero).  Every lane therefore
// follows the smallest nonzero magnitude among the values it splits, and one at or below 2^-100 raises the same flag:
// the product is redone in IEEE f32 arithmetic, which has no such limit (aixDeviceCPU.cpp:362-389).
constexpr u32 kX3Smallest = (127u - 100u) << 24;         // (bits << 1) - 1 of 2^-100, exclusive bound

template <bool AT, bool BT> struct TileX3 {
    static constexpr int BM = 128, BN = 128, BK = 32, PA = BM + 32, PB = BN + 32;
    static constexpr int SA = AT ? BK * PA : BM * BK, SB = BT ? BK * PB : BN * BK;       // bf16 elements per plane
    static constexpr size_t kLds = (size_t)3 * (SA + SB) * 2;
};

__device__ __forceinline__ u32 min3u(u32 a, u32 b, u32 c)
{
    u32 r;
    asm("v_min3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ u32 cvt_pk_bf16(float lo, float hi)
{
    u32 r;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}

// four f32 -> three word pairs of four bf16 (element e in bits 16 (e & 1) of word e / 2).
// `least` follows the smallest nonzero magnitude seen: (bits << 1) - 1 drops the sign and sends zeros to the top.
__device__ __forceinline__ void split3(const u32x4 x, u32x2& h, u32x2& m, u32x2& l, u32& least)
{
    const u32 xs[4] = {x.x, x.y, x.z, x.w};
    least = min3u(least, (xs[0] << 1) - 1u, (xs[1] << 1) - 1u);
    least = min3u(least, (xs[2] << 1) - 1u, (xs[3] << 1) - 1u);
    float r[4];
    u32 hb[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) { hb[e] = xs[e] & 0xFFFF0000u; r[e] = __builtin_bit_cast(float, xs[e]) - __builtin_bit_cast(float, hb[e]); }
    h.x = (hb[0] >> 16) | hb[1]; h.y = (hb[2] >> 16) | hb[3];
    m.x = cvt_pk_bf16(r[0], r[1]); m.y = cvt_pk_bf16(r[2], r[3]);
    const float s0 = r[0] - __builtin_bit_cast(float, m.x << 16), s1 = r[1] - __builtin_bit_cast(float, m.x & 0xFFFF0000u);
    const float s2 = r[2] - __builtin_bit_cast(float, m.y << 16), s3 = r[3] - __builtin_bit_cast(float, m.y & 0xFFFF0000u);
    l.x = cvt_pk_bf16(s0, s1); l.y = cvt_pk_bf16(s2, s3);
}

// The three planes of a whole operand in memory, for products large enough that gemm_direct16_k<..., PLANES> (256 x 256
// tiles, eight waves, LDS-direct loads) beats splitting in registers tile by tile: planes[p][r][k], p = hi, mid, lo, r < R,
// k < Kp with zeros from K on, always K-contiguous whatever the source's form (TR: src[k * ld + r], a T-form operand, is
// transposed through LDS on the way).  The operands that the planes cannot carry -- infinities, NaNs, magnitudes below
// 2^-100 -- are noticed here: the launch's number goes into the flag word and the IEEE kernel that stands by redoes the product.
__device__ __forceinline__ void split3_watch(const u32x4 x, u32x2& h, u32x2& m, u32x2& l, u32& least, u32& most)
{
    split3(x, h, m, l, least);
    most = max(max(most, x.x & 0x7FFFFFFFu), max(x.y & 0x7FFFFFFFu, max(x.z & 0x7FFFFFFFu, x.w & 0x7FFFFFFFu)));
}

template <bool TR>
__global__ __launch_bounds__(256) void split_planes_k(const float* __restrict__ src, u16* __restrict__ planes, u64 R, u64 K, u64 Kp, u64 ld, u32* flag, u32 seq)
{
    const int tid = threadIdx.x;
    const u64 plane = R * Kp;
    u32 least = ~0u, most = 0u;
    if constexpr (!TR) {
        // 32 rows x 64 k per workgroup; a lane splits 8 consecutive k of one row
        const u64 r = (u64)blockIdx.y * 32 + tid / 8, k = (u64)blockIdx.x * 64 + (tid % 8) * 8;
        u32x4 x0 = u32x4{0, 0, 0, 0}, x1 = u32x4{0, 0, 0, 0};
        if (k < K) x0 = *(const u32x4*)(src + r * ld + k);
        if (k + 4 < K) x1 = *(const u32x4*)(src + r * ld + k + 4);
        u32x2 h0, m0, l0, h1, m1, l1;
        split3_watch(x0, h0, m0, l0, least, most);
        split3_watch(x1, h1, m1, l1, least, most);
        u16* out = planes + r * Kp + k;
        *(u32x4*)out = u32x4{h0.x, h0.y, h1.x, h1.y};
        *(u32x4*)(out + plane) = u32x4{m0.x, m0.y, m1.x, m1.y};
        *(u32x4*)(out + 2 * plane) = u32x4{l0.x, l0.y, l1.x, l1.y};
    } else {
        // 64 k x 64 r per workgroup: 16-byte loads along r, the planes transposed in LDS, 16-byte stores along k.  A lane writes
        // one k of four neighbouring rows and its 15 neighbours write the same k of the next rows, 576 bytes apart (four
        // banks in turn): the 16-byte chunk of k is therefore kept at chunk ^ (row / 4 & 7) of its row
        __shared__ u16 tile[3][64][72];
        const u64 k0 = (u64)blockIdx.x * 64, r0 = (u64)blockIdx.y * 64;
        const int rc = tid % 16, kr = tid / 16;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int kk = pass * 16 + kr;
            u32x4 x = u32x4{0, 0, 0, 0};
            if (k0 + kk < K) x = *(const u32x4*)(src + (k0 + kk) * ld + r0 + rc * 4);
            u32x2 h, m, l;
            split3_watch(x, h, m, l, least, most);
            const u32 hv[4] = {h.x & 0xFFFFu, h.x >> 16, h.y & 0xFFFFu, h.y >> 16}, mv[4] = {m.x & 0xFFFFu, m.x >> 16, m.y & 0xFFFFu, m.y >> 16},
                      lv[4] = {l.x & 0xFFFFu, l.x >> 16, l.y & 0xFFFFu, l.y >> 16};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int at = (((kk >> 3) ^ (rc & 7)) << 3) | (kk & 7);
                tile[0][rc * 4 + e][at] = (u16)hv[e]; tile[1][rc * 4 + e][at] = (u16)mv[e]; tile[2][rc * 4 + e][at] = (u16)lv[e];
            }
        }
        __syncthreads();
        const int row = tid / 4, kc = (tid % 4) * 16;
#pragma unroll
        for (int p = 0; p < 3; ++p) {
            u16* out = planes + (u64)p * plane + (r0 + row) * Kp + k0 + kc;
            const int sw = (row >> 2) & 7;
            *(u32x4*)out = *(const u32x4*)&tile[p][row][((kc >> 3) ^ sw) << 3];
            *(u32x4*)(out + 8) = *(const u32x4*)&tile[p][row][(((kc >> 3) + 1) ^ sw) << 3];
        }
    }
    if (least < kX3Smallest || most >= 0x7F800000u) *flag = seq;
}

template <bool AT, bool BT>
__global__ __launch_bounds__(256) void gemm_x3_k(GemmArgs g, SplitArgs sk, u32* flag, u32 seq)
{
    typedef TileX3<AT, BT> S;
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, PA = S::PA, PB = S::PB, SA = S::SA, SB = S::SB;
    constexpr int WM = BM / 2, WN = BN / 2, TI = WM / 32, TJ = WN / 32;
    constexpr int CA = BM * (BK / 4) / 256, CB = BN * (BK / 4) / 256;        // 16-byte chunks (4 values) per lane and step
    constexpr int C4 = BK / 4;                                                // 4-value chunks per K-contiguous row
    // K-contiguous plane rows are unpadded and swizzled (kswz): the 4 values of chunk k4 are one half of 16-byte slot k4 / 2
    auto kplace = [](int c) { const int r = c / C4, k4 = c % C4; return r * BK + (((k4 >> 1) ^ kswz<BK>(r)) * 8) + (k4 & 1) * 4; };
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_x3[];
    u16* As = (u16*)smem_x3;                              // [3][SA]
    u16* Bs = As + 3 * SA;                                // [3][SB]

    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const float* A = (const float*)g.a;
    const float* B = (const float*)g.b;

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // smallest nonzero operand magnitude this lane has split (see split3); six vector instructions per four values, 3 % of
    // the kernel's time at 4096^3 (watching in the first workgroup of every row and column of tiles only gained nothing)
    u32 least = 0xFFFFFFFFu;
    u32x4 ra[CA], rb[CB];
    auto load_global = [&](u64 k0) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            if constexpr (AT) { const u64 k = k0 + c / (BM / 4), m = m0 + (c % (BM / 4)) * 4; ra[i] = (k < g.K && m < g.M) ? *(const u32x4*)(A + k * g.lda + m) : (u32x4){0, 0, 0, 0}; }
            else { const u64 m = m0 + c / (BK / 4), k = k0 + (c % (BK / 4)) * 4; ra[i] = (m < g.M && k < g.K) ? *(const u32x4*)(A + m * g.lda + k) : (u32x4){0, 0, 0, 0}; }
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            if constexpr (BT) { const u64 k = k0 + c / (BN / 4), n = n0 + (c % (BN / 4)) * 4; rb[i] = (k < g.K && n < g.N) ? *(const u32x4*)(B + k * g.ldb + n) : (u32x4){0, 0, 0, 0}; }
            else { const u64 n = n0 + c / (BK / 4), k = k0 + (c % (BK / 4)) * 4; rb[i] = (n < g.N && k < g.K) ? *(const u32x4*)(B + n * g.ldb + k) : (u32x4){0, 0, 0, 0}; }
        }
    };
    auto store_lds = [&] {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            const int at = AT ? (c / (BM / 4)) * PA + (c % (BM / 4)) * 4 : kplace(c);
            u32x2 h, m, l;
            split3(ra[i], h, m, l, least);
            *(u32x2*)(As + at) = h; *(u32x2*)(As + SA + at) = m; *(u32x2*)(As + 2 * SA + at) = l;
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            const int at = BT ? (c / (BN / 4)) * PB + (c % (BN / 4)) * 4 : kplace(c);
            u32x2 h, m, l;
            split3(rb[i], h, m, l, least);
            *(u32x2*)(Bs + at) = h; *(u32x2*)(Bs + SB + at) = m; *(u32x2*)(Bs + 2 * SB + at) = l;
        }
    };
    const int j16 = lane & 15, swz = kswz<BK>(lane & 31), half = lane >> 5;
    const int fa0 = AT ? (8 * (lane >> 5) + (j16 >> 2)) * PA + 16 * ((lane >> 4) & 1) + 4 * (j16 & 3) + wm * WM : (wm * WM + (lane & 31)) * BK;
    const int fb0 = BT ? (8 * (lane >> 5) + (j16 >> 2)) * PB + 16 * ((lane >> 4) & 1) + 4 * (j16 & 3) + wn * WN : (wn * WN + (lane & 31)) * BK;

    const u64 steps = (g.K + BK - 1) / BK;
    const u64 first = (u64)blockIdx.z * sk.per_split;
    const u64 last = first + sk.per_split < steps ? first + sk.per_split : steps;
    if (first < last) load_global(first * BK);
    for (u64 kt = first; kt < last; ++kt) {
        store_lds();
        __syncthreads();
        if (kt + 1 < last) load_global((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            u32x4 fa[3][TI], fb[3][TJ];
            const int slot = ((half + 2 * kk) ^ swz) * 8;
#pragma unroll
            for (int p = 0; p < 3; ++p) {
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const u16* q = As + p * SA + fa0;
                    if constexpr (AT) fa[p][i] = tr_fragment_lds<PA>(q + i * 32 + kk * 16 * PA); else fa[p][i] = *(const u32x4*)(q + i * 32 * BK + slot);
                }
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const u16* q = Bs + p * SB + fb0;
                    if constexpr (BT) fb[p][j] = tr_fragment_lds<PB>(q + j * 32 + kk * 16 * PB); else fb[p][j] = *(const u32x4*)(q + j * 32 * BK + slot);
                }
            }
            // smallest contributions first; four independent accumulators between two uses of the same one
            constexpr int pa[6] = {2, 0, 1, 1, 0, 0}, pb[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int i = 0; i < TI; ++i)
#pragma unroll
                    for (int j = 0; j < TJ; ++j) acc[i][j] = Mma16<bf16>::run(fa[pa[t]][i], fb[pb[t]][j], acc[i][j]);
        }
        __syncthreads();
    }

    const u64 plane = g.M * g.N;
    float* C = sk.splits > 1 ? sk.partial + (u64)blockIdx.z * plane : (float*)g.c;
    float probe = 0.0f;                                   // NaN as soon as one accumulator is an infinity or a NaN (x * 0)
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const u64 col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const u64 row = m0 + wm * WM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.M && col < g.N) C[row * g.N + col] = acc[i][j][v];
                probe = __builtin_fmaf(acc[i][j][v], 0.0f, probe);
            }
        }
    if (probe != probe || least < kX3Smallest) *flag = seq;
}

__global__ __launch_bounds__(256) void splitk_finish_f32_k(const float* __restrict__ partial, float* __restrict__ out, u64 total, u32 splits)
{
    for (u64 e = (u64)blockIdx.x * 256 + threadIdx.x; e < total; e += (u64)gridDim.x * 256) {
        float sum = partial[e];
        for (u32 s = 1; s < splits; ++s) sum += partial[(u64)s * total + e];
        out[e] = sum;
    }
}

// ---- f32 operands ------------------------------------------------------------------------------
// 128 x 128 (or 64 x 64) workgroup tile, BK = 32.  v_mfma_f32_32x32x2f32 takes one element per lane
// and operand -- lane l holds A[row l % 32][k l / 32] -- so both operand forms feed it directly:
//   K-contiguous (A as [M, K], B given as [N, K]): staged [row][k], 32 floats + 4 padding per row;
//     a lane reads 4 consecutive k of its row with one ds_read_b128 and spends them on 4 MFMAs;
//   T form (A given as [K, M] with unit stride along M, B as plain row-major [K, N]): staged as it
//     comes, [k][row] with a pitch of BM + 8 floats; a lane reads its column of 4 consecutive k-rows
//     with 4 ds_read_b32 (32 consecutive floats per half-wave; the other half-wave's rows k + 4 start
//     32 banks away), no transposing copy beforehand.
template <int BM, int BN, bool AT, bool BT>
__global__ __launch_bounds__(256) void gemm_nt32_k(GemmArgs g, SplitArgs sk, const u32* only_if, u32 seq)
{
    if (only_if && *only_if != seq) return;                                // stand-by launch behind gemm_x3_k: nothing to redo
    constexpr int BK = 32, LDR = BK + 4;
    constexpr int WM = BM / 2, WN = BN / 2, TI = WM / 32, TJ = WN / 32;
    constexpr int CA = BM * (BK / 4) / 256, CB = BN * (BK / 4) / 256;      // 16-byte chunks per lane, operand and step
    constexpr int PA = AT ? BM + 8 : LDR, PB = BT ? BN + 8 : LDR;          // floats per LDS row
    constexpr int SA = (AT ? BK : BM) * PA, SB = (BT ? BK : BN) * PB;      // floats per stage
    extern __shared__ __attribute__((aligned(16))) unsigned char smem32[];
    float* As = (float*)smem32;                                            // [2][SA]
    float* Bs = As + 2 * SA;                                               // [2][SB]

    u32 tm, tn;
    tile_of(g, tm, tn);
    const u64 m0 = (u64)tm * BM, n0 = (u64)tn * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const float* A = (const float*)g.a;
    const float* B = (const float*)g.b;

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // chunk c of a K-contiguous tile is (row c / 8, k 4 (c % 8)); of a T-form tile (k-row c / (B / 4), column 4 (c % (B / 4)))
    f32x4 ra[CA], rb[CB];
    auto load_global = [&](u64 k0) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            if constexpr (AT) { const u64 k = k0 + c / (BM / 4), m = m0 + (c % (BM / 4)) * 4; ra[i] = (k < g.K && m < g.M) ? *(const f32x4*)(A + k * g.lda + m) : (f32x4){0, 0, 0, 0}; }
            else { const u64 r = m0 + (c >> 3), k = k0 + (c & 7) * 4; ra[i] = (r < g.M && k < g.K) ? *(const f32x4*)(A + r * g.lda + k) : (f32x4){0, 0, 0, 0}; }
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            if constexpr (BT) { const u64 k = k0 + c / (BN / 4), n = n0 + (c % (BN / 4)) * 4; rb[i] = (k < g.K && n < g.N) ? *(const f32x4*)(B + k * g.ldb + n) : (f32x4){0, 0, 0, 0}; }
            else { const u64 r = n0 + (c >> 3), k = k0 + (c & 7) * 4; rb[i] = (r < g.N && k < g.K) ? *(const f32x4*)(B + r * g.ldb + k) : (f32x4){0, 0, 0, 0}; }
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i;
            *(f32x4*)(As + buf * SA + (AT ? (c / (BM / 4)) * PA + (c % (BM / 4)) * 4 : (c >> 3) * PA + (c & 7) * 4)) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i;
            *(f32x4*)(Bs + buf * SB + (BT ? (c / (BN / 4)) * PB + (c % (BN / 4)) * 4 : (c >> 3) * PB + (c & 7) * 4)) = rb[i];
        }
    };

    // Fragments are double buffered: the reads of the next 8-wide K slice are issued under the 16
    // MFMAs of the current one; the tile for the next step goes to the other LDS buffer under the
    // third slice; the step's barrier sits before the last slice, whose MFMAs cover the first
    // fragment reads from that buffer.  sched_barrier keeps the phases apart (left alone, the
    // compiler emits "4 reads, wait, 16 MFMAs" per slice and exposes the LDS latency each time).
    f32x4 fa[2][TI], fb[2][TJ];
    auto read_frags = [&](int set, int buf, int kk) {
        const int k = kk * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int row = wm * WM + i * 32 + (lane & 31);
            if constexpr (AT) {
#pragma unroll
                for (int e = 0; e < 4; ++e) fa[set][i][e] = As[buf * SA + (k + e) * PA + row];
            } else fa[set][i] = *(const f32x4*)(As + buf * SA + row * PA + k);
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const int row = wn * WN + j * 32 + (lane & 31);
            if constexpr (BT) {
#pragma unroll
                for (int e = 0; e < 4; ++e) fb[set][j][e] = Bs[buf * SB + (k + e) * PB + row];
            } else fb[set][j] = *(const f32x4*)(Bs + buf * SB + row * PB + k);
        }
    };
    auto mma = [&](int set) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[set][i][s], fb[set][j][s], acc[i][j], 0, 0, 0);
    };
    // blockIdx.z numbers K splits (few tiles, long K: [2048, 4096] x [4096, 10]): split s multiplies its share of the K
    // steps and stores an f32 partial tile for splitk_finish_f32_k
    const u64 steps = (g.K + BK - 1) / BK;
    const u64 first = (u64)blockIdx.z * sk.per_split;
    const u64 last = first + sk.per_split < steps ? first + sk.per_split : steps;
    load_global(first * BK);
    store_lds(0);
    __syncthreads();
    read_frags(0, 0, 0);
    for (u64 kt = first; kt < last; ++kt) {
        const int buf = (int)((kt - first) & 1);
        load_global((kt + 1 < last ? kt + 1 : kt) * BK);        // past the end: the last tile again, into a buffer nobody reads
        read_frags(1, buf, 1); mma(0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(0, buf, 2); mma(1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(1, buf, 3); store_lds(buf ^ 1); mma(0);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(0, buf ^ 1, 0); mma(1);
        __builtin_amdgcn_sched_barrier(0);
    }

    float* C = sk.splits > 1 ? sk.partial + (u64)blockIdx.z * g.M * g.N : (float*)g.c;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const u64 col = n0 + wn * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const u64 row = m0 + wm * WM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.M && col < g.N) C[row * g.N + col] = acc[i][j][v];
            }
        }
}

// Workspace for operands that have to be made K-contiguous; grows on demand, lives with the
// context (all use is ordered on the context's single stream).
int workspace(aixk_ctx* ctx, int which, size_t bytes, void** out)
{
    if (ctx->gemm_ws_bytes[which] < bytes) {
        if (ctx->capturing) return fail(AIXK_EINVAL, "matmul workspace would have to grow inside a capture: run the same step once before capturing it");
        if (ctx->gemm_ws[which]) {
            AIXK_HIP(hipStreamSynchronize(ctx->stream));
            AIXK_HIP(hipFree(ctx->gemm_ws[which]));
            ctx->gemm_ws[which] = nullptr;
            ctx->gemm_ws_bytes[which] = 0;
        }
        const size_t want = (bytes + (size_t(1) << 20)) & ~((size_t(1) << 20) - 1);
        if (hipMalloc(&ctx->gemm_ws[which], want) != hipSuccess) { (void)hipGetLastError(); ctx->gemm_ws[which] = nullptr; return fail(AIXK_ENOMEM, "matmul workspace of %zu bytes", want); }
        ctx->gemm_ws_bytes[which] = want;
    }
    *out = ctx->gemm_ws[which];
    return AIXK_OK;
}

template <class K> int set_lds(K kernel, size_t bytes)
{
    static std::unordered_map<const void*, size_t> done;          // kernel -> dynamic LDS limit already raised
    auto it = done.find((const void*)kernel);
    if (it == done.end() || it->second < bytes) {
        AIXK_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
        done[(const void*)kernel] = bytes;
    }
    return AIXK_OK;
}


// gemm_small16_k on the last two dims of a / b (rank 2 descriptors), `batch` = the joint collapsed space of the
// leading dims (operands 0, 1, 2 = a, b, out) or null for one product.  -1: a layout the kernel does not take.
int launch_small16(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>* batch, const u64* table = nullptr)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    constexpr size_t esz = 2;
    const char* qa = (const char*)a->data + a->offset * esz;
    const char* qb = (const char*)b->data + b->offset * esz;
    const bool a_k = a->strides[1] == 1 || K == 1, a_m = a->strides[0] == 1 && M % 8 == 0;
    const bool b_k = b->strides[0] == 1 || K == 1, b_n = b->strides[1] == 1 && N % 8 == 0;
    const uint64_t la = a_k ? a->strides[0] : a->strides[1], lb = b_k ? b->strides[1] : b->strides[0];
    if (!((a_k || a_m) && (b_k || b_n) && la % 8 == 0 && lb % 8 == 0 && aligned16(qa) && aligned16(qb))) return -1;
    BatchArgs bt{};
    uint64_t count = 1;
    if (batch) {
        if (batch->rank > 3) return -1;
        bt.rank = (u32)batch->rank;
        for (int d = 0; d < batch->rank; ++d) {
            if (batch->shape[d] >= (1ull << 31) || batch->stride[0][d] % 8 != 0 || batch->stride[1][d] % 8 != 0) return -1;   // every matrix 16-byte aligned
            bt.ext[d] = (u32)batch->shape[d]; bt.sa[d] = batch->stride[0][d]; bt.sb[d] = batch->stride[1][d];
            count *= batch->shape[d];
        }
        if (count > 65535) return -1;
        bt.sc = M * N;
        if (bt.rank == 0) { bt.rank = 1; bt.ext[0] = 1; }
        bt.table = table;
    }
    GemmArgs g{};
    g.a = qa; g.b = qb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = la; g.ldb = lb;
    g.tiles_m = (u32)((M + 31) / 32); g.tiles_n = (u32)((N + 31) / 32);
    const u32 n = g.tiles_m * g.tiles_n;
    g.swizzle = n % 8u == 0 ? 1u : 0u;
    const bool at = !a_k, tb = !b_k;
    auto launch = [&](auto kernel, size_t lds) {
        AIXK_TRY(set_lds(kernel, lds));
        hipLaunchKernelGGL(kernel, dim3(n, (unsigned)count), dim3(256), lds, ctx->stream, g, bt);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    };
    if (out->dtype == AIXK_BF16) {
        if (!at && !tb) return launch(gemm_small16_k<bf16, false, false>, Small16<false, false>::kLds);
        if (!at && tb) return launch(gemm_small16_k<bf16, false, true>, Small16<false, true>::kLds);
        if (at && !tb) return launch(gemm_small16_k<bf16, true, false>, Small16<true, false>::kLds);
        return launch(gemm_small16_k<bf16, true, true>, Small16<true, true>::kLds);
    }
    if (!at && !tb) return launch(gemm_small16_k<f16, false, false>, Small16<false, false>::kLds);
    if (!at && tb) return launch(gemm_small16_k<f16, false, true>, Small16<false, true>::kLds);
    if (at && !tb) return launch(gemm_small16_k<f16, true, false>, Small16<true, false>::kLds);
    return launch(gemm_small16_k<f16, true, true>, Small16<true, true>::kLds);
}


// K step of gemm_tile16_k by tile height: the 64 x 64 tile wants 64 (fewer barriers per byte; 1536^3 NT 25.7 -> 21.2 us),
// the 128-row tiles 32 (more workgroups per compute unit; the transformer's shapes are 5 % faster overall).
constexpr int tile16_bk(int bm) { return bm == 64 ? 64 : 32; }

// gemm_tile16_k on the last two dims of a / b, `batch` as for launch_small16.  tile: 0 = 64 x 64, 1 = 128 x 64,
// 2 = 128 x 128, 3 = 128 x 192, 4 = 192 x 128; splits: K splits wanted (1 = none).  -1: a layout the kernel does not take.
int launch_tile16(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>* batch,
                  int tile, uint64_t splits, const u64* table = nullptr)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    constexpr size_t esz = 2;
    const char* qa = (const char*)a->data + a->offset * esz;
    const char* qb = (const char*)b->data + b->offset * esz;
    const bool a_k = a->strides[1] == 1 || K == 1, a_m = a->strides[0] == 1 && M % 8 == 0;
    const bool b_k = b->strides[0] == 1 || K == 1, b_n = b->strides[1] == 1 && N % 8 == 0;
    const uint64_t la = a_k ? a->strides[0] : a->strides[1], lb = b_k ? b->strides[1] : b->strides[0];
    if (!((a_k || a_m) && (b_k || b_n) && la % 8 == 0 && lb % 8 == 0 && aligned16(qa) && aligned16(qb))) return -1;
    BatchArgs bt{};
    uint64_t count = 1;
    if (batch) {
        if (batch->rank > 3) return -1;
        bt.rank = (u32)batch->rank;
        for (int d = 0; d < batch->rank; ++d) {
            if (batch->shape[d] >= (1ull << 31) || batch->stride[0][d] % 8 != 0 || batch->stride[1][d] % 8 != 0) return -1;
            bt.ext[d] = (u32)batch->shape[d]; bt.sa[d] = batch->stride[0][d]; bt.sb[d] = batch->stride[1][d];
            count *= batch->shape[d];
        }
        if (count > 65535) return -1;
        bt.sc = M * N;
        bt.table = table;
    }
    const uint64_t bm = tile == 0 ? 64 : tile == 4 ? 192 : 128, bn = tile == 2 || tile == 4 ? 128 : tile == 3 ? 192 : 64;
    GemmArgs g{};
    g.a = qa; g.b = qb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = la; g.ldb = lb;
    g.tiles_m = (u32)((M + bm - 1) / bm); g.tiles_n = (u32)((N + bn - 1) / bn);
    const u32 n = g.tiles_m * g.tiles_n;
    g.swizzle = n % 8u == 0 ? 1u : 0u;
    const uint64_t bk = (uint64_t)tile16_bk((int)bm);
    const uint64_t steps = (K + bk - 1) / bk;
    if (splits > steps) splits = steps;
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    SplitArgs sk{};
    sk.per_split = (u32)((steps + splits - 1) / splits);
    sk.splits = (u32)((steps + sk.per_split - 1) / sk.per_split);
    sk.matrices = count;
    if (sk.splits > 1) {
        void* ws;
        AIXK_TRY(workspace(ctx, 2, (size_t)sk.splits * count * M * N * sizeof(float), &ws));
        sk.partial = (float*)ws;
    }
    const bool at = !a_k, tb = !b_k;
    auto launch = [&](auto kernel, size_t lds) {
        AIXK_TRY(set_lds(kernel, lds));
        hipLaunchKernelGGL(kernel, dim3(n, (unsigned)count, sk.splits), dim3(256), lds, ctx->stream, g, bt, sk);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    };
    auto by_form = [&](auto dtype_tag, auto bm_tag, auto bn_tag, auto bk_tag, auto ring_tag) {
        typedef decltype(dtype_tag) T;
        constexpr int BM = decltype(bm_tag)::value, BN = decltype(bn_tag)::value, BK = decltype(bk_tag)::value ? decltype(bk_tag)::value : tile16_bk(BM);
        constexpr int RING = decltype(ring_tag)::value;
        if (!at && !tb) return launch(gemm_tile16_k<T, BM, BN, BK, false, false, RING>, Tile16<BM, BN, BK, false, false>::kLds);
        if (!at && tb) return launch(gemm_tile16_k<T, BM, BN, BK, false, true, RING>, Tile16<BM, BN, BK, false, true>::kLds);
        if (at && !tb) return launch(gemm_tile16_k<T, BM, BN, BK, true, false, RING>, Tile16<BM, BN, BK, true, false>::kLds);
        return launch(gemm_tile16_k<T, BM, BN, BK, true, true, RING>, Tile16<BM, BN, BK, true, true>::kLds);
    };
    auto by_tile = [&](auto dtype_tag) {
        constexpr std::integral_constant<int, 0> usual{};
        if (tile == 0) return by_form(dtype_tag, std::integral_constant<int, 64>{}, std::integral_constant<int, 64>{}, usual, usual);
        if (tile == 1) return by_form(dtype_tag, std::integral_constant<int, 128>{}, std::integral_constant<int, 64>{}, usual, usual);
        if (tile == 3) return by_form(dtype_tag, std::integral_constant<int, 128>{}, std::integral_constant<int, 192>{}, usual, usual);
        if (tile == 4) return by_form(dtype_tag, std::integral_constant<int, 192>{}, std::integral_constant<int, 128>{}, usual, usual);
        return by_form(dtype_tag, std::integral_constant<int, 128>{}, std::integral_constant<int, 128>{}, usual, usual);
    };
    const int rc = out->dtype == AIXK_BF16 ? by_tile(bf16{}) : by_tile(f16{});
    if (rc != AIXK_OK || sk.splits == 1) return rc;
    const uint64_t total = count * M * N;
    const unsigned blocks = grid_for(total, 256, (unsigned)ctx->cus * 16u);
    if (out->dtype == AIXK_BF16) hipLaunchKernelGGL((splitk_finish_k<bf16>), dim3(blocks), dim3(256), 0, ctx->stream, (const float*)sk.partial, (bf16*)out->data, (u64)total, sk.splits);
    else hipLaunchKernelGGL((splitk_finish_k<f16>), dim3(blocks), dim3(256), 0, ctx->stream, (const float*)sk.partial, (f16*)out->data, (u64)total, sk.splits);
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

// Stacks and groups of K = 64 products with K-contiguous operands and whole 128 x 128 tiles (gemm_k64_nt_k).  -1: not
// for this product.
int launch_k64(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>* batch, const u64* table)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    constexpr size_t esz = 2;
    if (!(K == 64 && M % 128 == 0 && N % 128 == 0 && a->strides[1] == 1 && b->strides[0] == 1)) return -1;
    const char* qa = (const char*)a->data + a->offset * esz;
    const char* qb = (const char*)b->data + b->offset * esz;
    const uint64_t la = a->strides[0], lb = b->strides[1];
    if (!(la % 8 == 0 && lb % 8 == 0 && aligned16(qa) && aligned16(qb) && aligned16(out->data))) return -1;
    BatchArgs bt{};
    uint64_t count = 1;
    if (batch) {
        if (batch->rank > 3) return -1;
        bt.rank = (u32)batch->rank;
        for (int d = 0; d < batch->rank; ++d) {
            if (batch->shape[d] >= (1ull << 31) || batch->stride[0][d] % 8 != 0 || batch->stride[1][d] % 8 != 0) return -1;
            bt.ext[d] = (u32)batch->shape[d]; bt.sa[d] = batch->stride[0][d]; bt.sb[d] = batch->stride[1][d];
            count *= batch->shape[d];
        }
        if (count > 65535) return -1;
        bt.sc = M * N;
        bt.table = table;
    }
    // a wave sweeps STEPS blocks of 64 columns: as many as still leave three workgroups per compute unit
    int steps = 1;
    for (int cand : {2, 4, 8})
        if ((N / 128) % cand == 0 && (M / 128) * (N / 128 / cand) * count >= 3 * (uint64_t)ctx->cus) steps = cand;
    const uint64_t tiles = (M / 128) * (N / 128 / steps);
    if (tiles * count >= (1ull << 31) || (M / 128) * (N / 128) * count < 2 * (uint64_t)ctx->cus) return -1;
    GemmArgs g{};
    g.a = qa; g.b = qb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = la; g.ldb = lb;
    g.tiles_m = (u32)(M / 128); g.tiles_n = (u32)(N / 128 / steps);
    const u32 spread = count % 8 == 0 ? 1u : 0u;
    auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles * count)), dim3(256), 0, ctx->stream, g, bt, spread); };
    auto by_steps = [&](auto tag) {
        typedef decltype(tag) T;
        if (steps == 8) launch(gemm_k64_nt_k<T, 8>);
        else if (steps == 4) launch(gemm_k64_nt_k<T, 4>);
        else if (steps == 2) launch(gemm_k64_nt_k<T, 2>);
        else launch(gemm_k64_nt_k<T, 1>);
    };
    if (out->dtype == AIXK_BF16) by_steps(bf16{}); else by_steps(f16{});
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

// 16-bit products of whole 128 x {128, 192, 256} x 64 tiles, at least half a tile per compute unit: the LDS-direct kernel
// on its smaller tiles (gemm_direct16_k).  `batch` / `table` as for launch_small16 (a stack of matrices, or a group of
// separate products).  limit > 0: only if the estimated cost stays below it (the caller has another kernel to offer).
// -1: not for this product.
int launch_direct16(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>* batch, const u64* table, double limit)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    constexpr size_t esz = 2;
    if (!(M % 128 == 0 && N % 64 == 0 && K % 64 == 0)) return -1;
    const char* qa = (const char*)a->data + a->offset * esz;
    const char* qb = (const char*)b->data + b->offset * esz;
    const bool a_k = a->strides[1] == 1, a_m = a->strides[0] == 1;
    const bool b_k = b->strides[0] == 1, b_n = b->strides[1] == 1;
    const uint64_t la = a_k ? a->strides[0] : a->strides[1], lb = b_k ? b->strides[1] : b->strides[0];
    BatchArgs bt{};
    uint64_t count = 1;
    if (batch) {
        if (batch->rank > 3) return -1;
        bt.rank = (u32)batch->rank;
        for (int d = 0; d < batch->rank; ++d) {
            if (batch->shape[d] >= (1ull << 31) || batch->stride[0][d] % 8 != 0 || batch->stride[1][d] % 8 != 0) return -1;
            bt.ext[d] = (u32)batch->shape[d]; bt.sa[d] = batch->stride[0][d]; bt.sb[d] = batch->stride[1][d];
            count *= batch->shape[d];
        }
        if (count > 65535) return -1;
        bt.sc = M * N;
        bt.table = table;
    }
    // rounds of workgroups x tile area, a smaller tile's flop 1.35 times as dear as one of the 256 x 256 kernel (more
    // fragment traffic per flop; measured: 4096^3 111 us on 256 x 256 tiles, 137 on 128 x 256); the larger tile on a tie
    uint64_t bn = 0, bm = 128;
    double least = 0;
    for (uint64_t cand : {256, 192, 128}) {
        if (N % cand != 0) continue;
        const uint64_t tiles = (M / 128) * (N / cand) * count;
        const double cost = 1.35 * (double)(((tiles + (uint64_t)ctx->cus - 1) / (uint64_t)ctx->cus) * cand * 128);
        if (bn == 0 || cost < least) { bn = cand; least = cost; }
    }
    // stacks and groups also have the 256 x 256 tile of this kernel (a single product of whole 256 x 256 tiles has
    // gemm_nt16_direct_k): 24 weight gradients [768, 8192]^T x [8192, 768] are 216 such tiles, one round of the chip, where
    // 432 tiles of 128 x 256 are 1.7
    if (batch && M % 256 == 0 && N % 256 == 0) {
        const uint64_t tiles = (M / 256) * (N / 256) * count;
        const double cost = (double)(((tiles + (uint64_t)ctx->cus - 1) / (uint64_t)ctx->cus) * 65536);
        if (bn == 0 || cost < least) { bn = 256; bm = 256; least = cost; }
    }
    if (bn == 0 || (limit > 0 && least >= limit)) return -1;
    const uint64_t tiles = (M / bm) * (N / bn);
    if (tiles * count * 2 < (uint64_t)ctx->cus || tiles >= (1ull << 31)) return -1;
    // a long K under less than three quarters of a round of tiles: the kernels that split K over workgroups fill the chip
    // better ([1024, 4096] x [4096, 2048]: 128 tiles, 41 us here against 37 with K split; [768, 8192]^T x [8192, 8192]: 192
    // tiles, 131 us here against 146)
    if (!batch && K >= 4096 && tiles * 4 < (uint64_t)ctx->cus * 3) return -1;
    if (!((a_k || a_m) && (b_k || b_n) && la % 8 == 0 && lb % 8 == 0 && la < (1ull << 27) && lb < (1ull << 27) && aligned16(qa) && aligned16(qb))) return -1;
    GemmArgs g{};
    g.a = qa; g.b = qb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = la; g.ldb = lb;
    g.tiles_m = (u32)(M / bm); g.tiles_n = (u32)(N / bn);
    const u32 n = g.tiles_m * g.tiles_n;
    g.swizzle = n % 8u == 0 ? 1u : 0u;
    const size_t lds = 2 * (bm + bn) * 128;
    const bool at = !a_k, tb = !b_k;
    auto launch = [&](auto kernel) {
        AIXK_TRY(set_lds(kernel, lds));
        hipLaunchKernelGGL(kernel, dim3(n, (unsigned)count), dim3(512), lds, ctx->stream, g, bt, PlanesArgs{});
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    };
    auto by_form = [&](auto dtype_tag, auto bn_tag, auto bm_tag) {
        typedef decltype(dtype_tag) T;
        constexpr int BN = decltype(bn_tag)::value, BM = decltype(bm_tag)::value;
        if (!at && !tb) return launch(gemm_direct16_k<T, false, false, BM, BN>);
        if (!at && tb) return launch(gemm_direct16_k<T, false, true, BM, BN>);
        if (at && !tb) return launch(gemm_direct16_k<T, true, false, BM, BN>);
        return launch(gemm_direct16_k<T, true, true, BM, BN>);
    };
    auto by_tile = [&](auto dtype_tag) {
        constexpr std::integral_constant<int, 128> rows128{};
        if (bm == 256) return by_form(dtype_tag, std::integral_constant<int, 256>{}, std::integral_constant<int, 256>{});
        if (bn == 256) return by_form(dtype_tag, std::integral_constant<int, 256>{}, rows128);
        if (bn == 192) return by_form(dtype_tag, std::integral_constant<int, 192>{}, rows128);
        return by_form(dtype_tag, std::integral_constant<int, 128>{}, rows128);
    };
    return out->dtype == AIXK_BF16 ? by_tile(bf16{}) : by_tile(f16{});
}

// Which kernel multiplies 16-bit operands whose layouts are consumed in place (everything the LDS-direct kernel does
// not take).  Measured on the shapes of a d = 768 transformer step at 8192 tokens, in microseconds, old route -> new:
// [8192,768]x[768,768] 28 -> 23, [8192,3072]^T-free x [3072,768] 76 -> 67, weight gradients [768,8192]x[8192,768]
// 73 -> 32 (8 K splits) and [768,8192]x[8192,3072] 113 -> 72 (4 splits), stacks of 192 attention products
// [512,64]x[64,512] 121 -> 42, [512,512]x[512,64] 52 -> 27, [512,512]^T x [512,64] 92 -> 27.
int route16(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>* batch, const u64* table = nullptr)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    const uint64_t cus = (uint64_t)ctx->cus;
    uint64_t count = 1;
    if (batch) for (int d = 0; d < batch->rank; ++d) count *= batch->shape[d];
    const uint64_t t64 = ((M + 63) / 64) * ((N + 63) / 64), t128 = ((M + 127) / 128) * ((N + 127) / 128), t12864 = ((M + 127) / 128) * ((N + 63) / 64);
    auto splits_for = [&](uint64_t groups, uint64_t steps, uint64_t fill) {        // long K, few workgroups: split K over workgroups
        if (K < 4096 || groups >= fill * cus) return (uint64_t)1;
        return std::max<uint64_t>(1, std::min<uint64_t>(steps / 16, (fill * cus + groups - 1) / groups));
    };
    if (batch) {
        // stacks: thin results (attention's [seq, head dim]) on 128 x 64 tiles, everything else on 128 x 128
        // a group of separate products (table): no K splits -- their partial planes assume one dense stack of results
        if (M <= 64) return launch_tile16(ctx, a, b, out, batch, 0, table ? 1 : splits_for(t64 * count, (K + 63) / 64 * 2, 4), table);
        if (N <= 64) return launch_tile16(ctx, a, b, out, batch, 1, table ? 1 : splits_for(t12864 * count, (K + 31) / 32, 2), table);
        if (K == 64) {                                     // one K step: a stream of stores (gemm_k64_nt_k)
            const int rc = launch_k64(ctx, a, b, out, batch, table);
            if (rc != -1) return rc;
        }
        if (K >= 512) {                                    // whole tiles and enough K steps to pay for its prologue: the LDS-direct kernel
            const int rc = launch_direct16(ctx, a, b, out, batch, table, 0);
            if (rc != -1) return rc;
        }
        return launch_tile16(ctx, a, b, out, batch, 2, table ? 1 : splits_for(t128 * count, (K + 31) / 32, 2), table);
    }
    // Tiles and K splits by a two-term cost in units of one K step (32 deep) of a lone 128 x 128 workgroup: the steps of the
    // workgroups that share a compute unit, plus -- with K split over workgroups -- the f32 partial results to write and
    // add up.  Measured on a d = 768 transformer's products at 8192 tokens (us per step of a lone workgroup: 128 x 128 0.32-0.45
    // by operand form, 128 x 192 and 192 x 128 1.4 times that; two workgroups on one compute unit take 1.6 steps for a step
    // of each, a third and every further pair queue behind; a MB of partial result costs 2 steps):
    //   [8192, 768] x [768, 768]: 384 tiles of 128 x 128 (1.5 per unit) 20.3 us, 256 tiles of 128 x 192 18.5
    //   [8192, 3072] x [3072, 768]: 60.8 -> 51.6; [8192, 8192] x [8192, 768]: 155.8 -> 135.9 (no split; 2 splits 144)
    //   [768, 8192] x [8192, 8192]: 160 -> 139 (192 x 128); [768, 8192] x [8192, 768]: 80.8 unsplit, 27.5 with 7 splits
    //   [768, 8192] x [8192, 3072]: 86.7 unsplit, 63 (128 x 128, 3 splits) / 62 (128 x 192, 5 splits)
    // The 192-wide tiles enter where they divide the result (the widths of a d = 768 model are multiples of 192, not of
    // 256); the 128 x 128 choice stays unless another is a twentieth cheaper.
    auto sharing = [](uint64_t per_unit) { return per_unit <= 1 ? 1.0 : per_unit % 2 ? 1.6 * (double)(per_unit - 1) / 2 + 1.0 : 1.6 * (double)per_unit / 2; };
    auto cheapest = [&](uint64_t most, int* tile_out) {
        const uint64_t steps = (K + 31) / 32;
        const double mb = (double)M * (double)N * 4e-6;
        uint64_t splits = 1;
        int tile = 2;
        double least = 0.0;
        for (int cand = 2; cand <= 4; ++cand) {
            if (cand == 3 && (N % 192 != 0 || M % 128 != 0)) continue;
            if (cand == 4 && (M % 192 != 0 || N % 128 != 0)) continue;
            const uint64_t tiles = cand == 2 ? t128 : cand == 3 ? (M / 128) * (N / 192) : (M / 192) * (N / 128);
            const double weight = cand == 2 ? 1.0 : 1.4;
            for (uint64_t sp = 1; sp <= most; ++sp) {
                const double cost = weight * sharing((tiles * sp + cus - 1) / cus) * (double)((steps + sp - 1) / sp) + (sp > 1 ? 2.0 * (double)sp * mb : 0.0);
                if ((cand == 2 && sp == 1) || cost < least * (cand == tile ? 1.0 : 0.95)) { least = cost; splits = sp; tile = cand; }
            }
        }
        *tile_out = tile;
        return splits;
    };
    if (K >= 4096 && t128 < 2 * cus && M >= 128 && N >= 128) {
        // a long K and few tiles (weight gradients): K split over workgroups.  Splits shorten every workgroup's chain of K
        // steps, as long as the workgroups still find a compute unit each, and each adds an f32 copy of the result to write
        // and read back.
        int tile = 2;
        const uint64_t steps = (K + 31) / 32;
        const uint64_t splits = cheapest(std::max<uint64_t>(1, std::min<uint64_t>(steps / 16, 16)), &tile);
        return launch_tile16(ctx, a, b, out, nullptr, tile, splits);
    }
    if (t64 < 2 * cus) {
        // outputs that 64 x 64 tiles cannot spread over the chip twice: with a long K, 64 x 64 tiles and K split over
        // workgroups; from half a tile per compute unit on, 64 x 64 tiles as they are (their interior tiles prefetch three K
        // steps ahead: 1024^3 NN 12.0 -> 8.7 us, [1024,1024] x K 2048 20.3 -> 13.3, 1280^3 TN 37.5 -> 14.2); below that, 32 x 32
        // tiles with K split over the waves (512^3: 4.3 us against 5.9)
        if (K >= 4096) return launch_tile16(ctx, a, b, out, nullptr, 0, splits_for(t64, (K + 63) / 64 * 2, 4));
        if (2 * t64 > cus) return launch_tile16(ctx, a, b, out, nullptr, 0, 1);
        return launch_small16(ctx, a, b, out, nullptr);
    }
    if (2 * t128 >= cus) {                                 // (2048^3: 256 tiles of 128 x 128 27.4 us, 512 of 128 x 64 33.0; 1536^3: 144 tiles 19.6, 576 of 64 x 64 22.1)
        int tile = 2;
        (void)cheapest(1, &tile);
        return launch_tile16(ctx, a, b, out, nullptr, tile, 1);
    }
    if (t12864 >= 2 * cus) return launch_tile16(ctx, a, b, out, nullptr, 1, 1);
    return launch_tile16(ctx, a, b, out, nullptr, 0, 1);
}

} // namespace

namespace aixk {

// A stack of 16-bit products that do not fill the chip one by one, in one launch.  -1: not handled here.
int matmul_mfma_batched(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>& batch)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    if (aixk_dtype_size(out->dtype) != 2 || (out->dtype != AIXK_BF16 && out->dtype != AIXK_F16)) return -1;
    if (K % 8 != 0 || M * N < 64 * 64) return -1;                  // as for a single product
    if (((M + 63) / 64) * ((N + 63) / 64) >= (uint64_t)ctx->cus * 2) return -1;     // each product fills the chip by itself: one launch each
    return route16(ctx, a, b, out, &batch);
}

// `count` separate 16-bit products of one shape and one operand layout (only the buffers differ) in one launch: the
// kernels of the stacks, with the three addresses of every product read from a table in device memory.  -1: not
// handled here (the caller issues them one by one).
int matmul_mfma_grouped(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint32_t count)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    if (out->dtype != AIXK_BF16 && out->dtype != AIXK_F16) return -1;
    if (count < 2 || count > 65535 || K % 8 != 0 || M * N < 64 * 64) return -1;
    if (((M + 63) / 64) * ((N + 63) / 64) >= (uint64_t)ctx->cus * 3) return -1;       // each product fills the chip by itself
    for (uint32_t i = 0; i < count; ++i) {
        if (a[i].dtype != out->dtype || b[i].dtype != out->dtype || out[i].dtype != out->dtype) return -1;
        if (a[i].shape[0] != M || a[i].shape[1] != K || b[i].shape[0] != K || b[i].shape[1] != N) return -1;
        if (a[i].strides[0] != a->strides[0] || a[i].strides[1] != a->strides[1] || b[i].strides[0] != b->strides[0] || b[i].strides[1] != b->strides[1]) return -1;
        if (!aligned16((const char*)a[i].data + a[i].offset * 2) || !aligned16((const char*)b[i].data + b[i].offset * 2) || !aligned16(out[i].data)) return -1;
    }
    u64* host = nullptr;
    const u64* dev = nullptr;
    AIXK_TRY(table_slot(ctx, (size_t)count * 3 * sizeof(u64), (void**)&host, (const void**)&dev));
    for (uint32_t i = 0; i < count; ++i) {
        host[3 * i] = (u64)(uintptr_t)((const char*)a[i].data + a[i].offset * 2);
        host[3 * i + 1] = (u64)(uintptr_t)((const char*)b[i].data + b[i].offset * 2);
        host[3 * i + 2] = (u64)(uintptr_t)out[i].data;
    }
    AIXK_TRY(table_upload(ctx, host, dev, (size_t)count * 3 * sizeof(u64)));
    Space<3> batch{};
    batch.rank = 1;
    batch.shape[0] = count;
    aixhip_tensor o2 = out[0];
    o2.offset = 0; o2.strides[0] = N; o2.strides[1] = 1;
    return route16(ctx, &a[0], &b[0], &o2, &batch, dev);
}

int matmul_mfma(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    const size_t esz = aixk_dtype_size(out->dtype);
    const uint64_t kq = 16 / esz;                                 // elements per 16-byte chunk
    if (K % kq != 0 || M * N < 64 * 64) return -1;                // odd K / tiny outputs: LDS-tiled kernel
    if (((M + 63) / 64) * ((N + 63) / 64) >= (1ull << 31)) return -1;

    // 16-bit, whole 256 x 256 x 64 tiles, enough of them: every operand layout is consumed where it lies
    // (K-contiguous, or "T" form with unit stride along M / N), no gathers.
    if (esz == 2 && M % 256 == 0 && N % 256 == 0 && K % 64 == 0 && (M / 256) * (N / 256) >= (uint64_t)ctx->cus / 2 &&
        (M / 256) * (N / 256) < (1ull << 31)) {
        // unless smaller tiles fill the chip's rounds so much better that they win all the same ([8192, 768] x [768, 2304]:
        // 288 tiles are a full round and an eighth of one, 44.7 us; 768 tiles of 128 x 192 are three full rounds, 36-39 us)
        const uint64_t t256 = (M / 256) * (N / 256);
        const int rc = launch_direct16(ctx, a, b, out, nullptr, nullptr, (double)(((t256 + (uint64_t)ctx->cus - 1) / (uint64_t)ctx->cus) * 65536));
        if (rc != -1) return rc;
        const char* qa = (const char*)a->data + a->offset * esz;
        const char* qb = (const char*)b->data + b->offset * esz;
        const bool a_k = a->strides[1] == 1, a_m = a->strides[0] == 1;
        const bool b_k = b->strides[0] == 1, b_n = b->strides[1] == 1;
        const uint64_t la = a_k ? a->strides[0] : a->strides[1], lb = b_k ? b->strides[1] : b->strides[0];
        if ((a_k || a_m) && (b_k || b_n) && la % 8 == 0 && lb % 8 == 0 && la < (1ull << 27) && lb < (1ull << 27) && aligned16(qa) && aligned16(qb)) {
            GemmArgs g{};
            g.a = qa; g.b = qb; g.c = out->data;
            g.M = M; g.N = N; g.K = K; g.lda = la; g.ldb = lb;
            g.tiles_m = (u32)(M / 256); g.tiles_n = (u32)(N / 256);
            const u32 n = g.tiles_m * g.tiles_n;
            g.swizzle = n % 8u == 0 ? 1u : 0u;
            constexpr size_t lds = 2 * 65536;
            const bool at = !a_k, bt = !b_k;
            auto launch = [&](auto kernel) {
                AIXK_TRY(set_lds(kernel, lds));
                hipLaunchKernelGGL(kernel, dim3(n), dim3(512), lds, ctx->stream, g);
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            };
            if (out->dtype == AIXK_BF16) {
                if (!at && !bt) return launch(gemm_nt16_direct_k<bf16, false, false>);
                if (!at && bt) return launch(gemm_nt16_direct_k<bf16, false, true>);
                if (at && !bt) return launch(gemm_nt16_direct_k<bf16, true, false>);
                return launch(gemm_nt16_direct_k<bf16, true, true>);
            }
            if (!at && !bt) return launch(gemm_nt16_direct_k<f16, false, false>);
            if (!at && bt) return launch(gemm_nt16_direct_k<f16, false, true>);
            if (at && !bt) return launch(gemm_nt16_direct_k<f16, true, false>);
            return launch(gemm_nt16_direct_k<f16, true, true>);
        }
    }

    if (esz == 2) { const int rc = launch_direct16(ctx, a, b, out, nullptr, nullptr, 0); if (rc != -1) return rc; }

    // 16-bit, operands consumed where they lie (K-contiguous or T form): tiles and K splits by shape
    if (esz == 2) {
        const int rc = route16(ctx, a, b, out, nullptr);
        if (rc != -1) return rc;
    }

    auto grid_of = [&](GemmArgs& g, uint64_t bm, uint64_t bn) {
        g.tiles_m = (u32)((M + bm - 1) / bm);
        g.tiles_n = (u32)((N + bn - 1) / bn);
        const u32 n = g.tiles_m * g.tiles_n;
        g.swizzle = n % 8u == 0 ? 1u : 0u;
        return n;
    };
    // problems that 128 x 128 tiles cannot spread over the chip twice use 64 x 64 tiles
    const bool small_tiles = ((M + 127) / 128) * ((N + 127) / 128) < (uint64_t)ctx->cus * 2;

    // f32: either operand form is consumed where it lies (K-contiguous, or unit stride along M / N with an extent
    // that is a multiple of 4); anything else is gathered into K-contiguous scratch first
    if (out->dtype == AIXK_F32) {
        const char* pa = (const char*)a->data + a->offset * esz;
        const char* pb = (const char*)b->data + b->offset * esz;
        const bool a_k = a->strides[1] == 1 || K == 1, a_m = a->strides[0] == 1 && M % 4 == 0;
        const bool b_k = b->strides[0] == 1 || K == 1, b_n = b->strides[1] == 1 && N % 4 == 0;
        uint64_t lda = a_k ? a->strides[0] : a->strides[1], ldb = b_k ? b->strides[1] : b->strides[0];
        bool at = !a_k && a_m, bt = !b_k && b_n, gathered = false;
        if (!(a_k || a_m) || lda % 4 != 0 || !aligned16(pa)) {
            void* ws;
            gathered = true;
            AIXK_TRY(workspace(ctx, 0, M * K * esz, &ws));
            AIXK_TRY(gather_dense(ctx, a, ws, M * K));
            pa = (const char*)ws; lda = K; at = false;
        }
        if (!(b_k || b_n) || ldb % 4 != 0 || !aligned16(pb)) {
            aixhip_tensor bt_view = *b;                           // the [N,K] view of b
            bt_view.shape[0] = N; bt_view.shape[1] = K;
            bt_view.strides[0] = b->strides[1]; bt_view.strides[1] = b->strides[0];
            void* ws;
            gathered = true;
            AIXK_TRY(workspace(ctx, 1, N * K * esz, &ws));
            AIXK_TRY(gather_dense(ctx, &bt_view, ws, N * K));
            pb = (const char*)ws; ldb = K; bt = false;
        }
        GemmArgs g{};
        g.a = pa; g.b = pb; g.c = out->data;
        g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb;
        const uint64_t t128 = ((M + 127) / 128) * ((N + 127) / 128), fill = 2 * (uint64_t)ctx->cus, steps = (K + 31) / 32;
        const u32* only_if = nullptr;          // set: the launches below stand by behind a split-plane kernel
        u32 seq = 0;
        // whole 256 x 256 tiles, at least one per compute unit: the planes of both operands are written to memory once
        // (split_planes_k) and multiplied by the LDS-direct 16-bit kernel, six plane pairs deep (4096^3: 0.73 -> 0.64 ms)
        if (M % 256 == 0 && N % 256 == 0 && (M / 256) * (N / 256) >= (uint64_t)ctx->cus && (M / 256) * (N / 256) < (1ull << 31) && K >= 256 &&
            !gathered && lda < (1ull << 27) && ldb < (1ull << 27) && M / 32 <= 65535 && N / 32 <= 65535) {
            const uint64_t Kp = (K + 63) / 64 * 64;
            void *wa = nullptr, *wb = nullptr;
            // (no room for the planes -- six bytes per operand element -- is no error: gemm_x3_k below needs none)
            if (workspace(ctx, 0, 3 * M * Kp * 2, &wa) != AIXK_OK || workspace(ctx, 1, 3 * N * Kp * 2, &wb) != AIXK_OK) wa = nullptr;
            if (wa) {
            if (++ctx->gemm_seq == 0) ++ctx->gemm_seq;
            seq = ctx->gemm_seq;
            auto split = [&](const char* src, bool transposed, uint64_t rows, uint64_t ld, void* planes) {
                if (transposed) hipLaunchKernelGGL(split_planes_k<true>, dim3((unsigned)(Kp / 64), (unsigned)(rows / 64)), dim3(256), 0, ctx->stream,
                                                   (const float*)src, (u16*)planes, (u64)rows, (u64)K, (u64)Kp, (u64)ld, (u32*)ctx->counter, seq);
                else hipLaunchKernelGGL(split_planes_k<false>, dim3((unsigned)(Kp / 64), (unsigned)(rows / 32)), dim3(256), 0, ctx->stream,
                                        (const float*)src, (u16*)planes, (u64)rows, (u64)K, (u64)Kp, (u64)ld, (u32*)ctx->counter, seq);
            };
            split(pa, at, M, lda, wa);
            split(pb, bt, N, ldb, wb);
            AIXK_HIP(hipGetLastError());
            GemmArgs gp{};
            gp.a = wa; gp.b = wb; gp.c = out->data;
            gp.M = M; gp.N = N; gp.K = Kp; gp.lda = Kp; gp.ldb = Kp;
            gp.tiles_m = (u32)(M / 256); gp.tiles_n = (u32)(N / 256);
            const u32 n = gp.tiles_m * gp.tiles_n;
            gp.swizzle = n % 8u == 0 ? 1u : 0u;
            constexpr size_t lds = 2 * 65536;
            auto kernel = gemm_direct16_k<bf16, false, false, 256, 256, true>;
            AIXK_TRY(set_lds(kernel, lds));
            hipLaunchKernelGGL(kernel, dim3(n), dim3(512), lds, ctx->stream, gp, BatchArgs{}, PlanesArgs{M * Kp * 2, N * Kp * 2, (u32*)ctx->counter, seq});
            AIXK_HIP(hipGetLastError());
            only_if = (const u32*)ctx->counter;
            ctx->gemm_last_route = 1;
            }
        }
        // enough 128 x 128 tiles: on the bf16 pipe, each operand as three bf16 planes (gemm_x3_k); with few tiles and a
        // long K, K is split over workgroups
        // two workgroups per compute unit hide each other's split-and-stage phases: with fewer tiles than that, K is split
        // over workgroups if it is long enough, else the f32 MFMA kernels below take the product
        uint64_t splits = 1;
        // (as many splits as still fit one round of two workgroups per compute unit: [784, 4096]^T x [4096, 2048], 112 tiles,
        // takes 107 us with 4 splits and 131 with 5, whose 560 workgroups spill into a second round)
        if (t128 < fill && K >= 2048) {
            const uint64_t whole = fill / t128, over = (fill + t128 - 1) / t128;
            splits = std::max<uint64_t>(1, std::min<uint64_t>({steps / 16, t128 * whole >= fill - fill / 8 ? whole : over, (uint64_t)64}));
        }
        if (!only_if && t128 * splits >= fill - fill / 8 && t128 >= (uint64_t)ctx->cus / 4) {
            const u32 n = grid_of(g, 128, 128);
            SplitArgs sk{};
            sk.per_split = (u32)((steps + splits - 1) / splits);
            sk.splits = (u32)((steps + sk.per_split - 1) / sk.per_split);
            sk.matrices = 1;
            if (sk.splits > 1) {
                void* ws;
                AIXK_TRY(workspace(ctx, 2, (size_t)sk.splits * M * N * sizeof(float), &ws));
                sk.partial = (float*)ws;
            }
            if (++ctx->gemm_seq == 0) ++ctx->gemm_seq;                     // 0 is what the flag word holds at creation
            seq = ctx->gemm_seq;
            auto launch_x3 = [&](auto kernel, size_t lds) {
                AIXK_TRY(set_lds(kernel, lds));
                hipLaunchKernelGGL(kernel, dim3(n, 1, sk.splits), dim3(256), lds, ctx->stream, g, sk, (u32*)ctx->counter, seq);
                AIXK_HIP(hipGetLastError());
                return (int)AIXK_OK;
            };
            int rc;
            if (!at && !bt) rc = launch_x3(gemm_x3_k<false, false>, TileX3<false, false>::kLds);
            else if (!at && bt) rc = launch_x3(gemm_x3_k<false, true>, TileX3<false, true>::kLds);
            else if (at && !bt) rc = launch_x3(gemm_x3_k<true, false>, TileX3<true, false>::kLds);
            else rc = launch_x3(gemm_x3_k<true, true>, TileX3<true, true>::kLds);
            if (rc != AIXK_OK) return rc;
            if (sk.splits > 1) {
                const uint64_t total = M * N;
                hipLaunchKernelGGL(splitk_finish_f32_k, dim3(grid_for(total, 256, (unsigned)ctx->cus * 16u)), dim3(256), 0, ctx->stream,
                                   (const float*)sk.partial, (float*)out->data, (u64)total, sk.splits);
                AIXK_HIP(hipGetLastError());
            }
            only_if = (const u32*)ctx->counter;                            // operands the planes cannot carry: redo with IEEE arithmetic
            ctx->gemm_last_route = 1;
        }
        auto launch = [&](auto kernel, uint64_t tile, size_t lds) {
            const u32 n = grid_of(g, tile, tile);
            // few tiles and a long K (a weight gradient with ten output columns): K split over workgroups
            SplitArgs sk{};
            uint64_t ksplits = 1;
            if (!only_if && n < (u32)ctx->cus && K >= 2048) ksplits = std::max<uint64_t>(1, std::min<uint64_t>({steps / 8, (fill + n - 1) / n, (uint64_t)64}));
            sk.per_split = (u32)((steps + ksplits - 1) / ksplits);
            sk.splits = (u32)((steps + sk.per_split - 1) / sk.per_split);
            sk.matrices = 1;
            if (sk.splits > 1) {
                void* ws;
                AIXK_TRY(workspace(ctx, 2, (size_t)sk.splits * M * N * sizeof(float), &ws));
                sk.partial = (float*)ws;
            }
            AIXK_TRY(set_lds(kernel, lds));
            hipLaunchKernelGGL(kernel, dim3(n, 1, sk.splits), dim3(256), lds, ctx->stream, g, sk, only_if, seq);
            AIXK_HIP(hipGetLastError());
            if (sk.splits > 1) {
                hipLaunchKernelGGL(splitk_finish_f32_k, dim3(grid_for(M * N, 256, (unsigned)ctx->cus * 16u)), dim3(256), 0, ctx->stream,
                                   (const float*)sk.partial, (float*)out->data, (u64)(M * N), sk.splits);
                AIXK_HIP(hipGetLastError());
            }
            return (int)AIXK_OK;
        };
        // stage sizes: K-contiguous rows x 36 floats, T form 32 k-rows x (tile + 8) floats
        auto lds_of = [](size_t tile, bool ta, bool tb) { return 2 * sizeof(float) * ((ta ? 32 * (tile + 8) : tile * 36) + (tb ? 32 * (tile + 8) : tile * 36)); };
        if (small_tiles) {
            if (!at && !bt) return launch(gemm_nt32_k<64, 64, false, false>, 64, lds_of(64, false, false));
            if (!at && bt) return launch(gemm_nt32_k<64, 64, false, true>, 64, lds_of(64, false, true));
            if (at && !bt) return launch(gemm_nt32_k<64, 64, true, false>, 64, lds_of(64, true, false));
            return launch(gemm_nt32_k<64, 64, true, true>, 64, lds_of(64, true, true));
        }
        if (!at && !bt) return launch(gemm_nt32_k<128, 128, false, false>, 128, lds_of(128, false, false));
        if (!at && bt) return launch(gemm_nt32_k<128, 128, false, true>, 128, lds_of(128, false, true));
        if (at && !bt) return launch(gemm_nt32_k<128, 128, true, false>, 128, lds_of(128, true, false));
        return launch(gemm_nt32_k<128, 128, true, true>, 128, lds_of(128, true, true));
    }

    // 16-bit: A as [M,K] and B as [N,K], both with unit stride along K and 16-byte aligned rows
    const char* pa = (const char*)a->data + a->offset * esz;
    uint64_t lda = a->strides[0];
    if (!(a->strides[1] == 1 || K == 1) || lda % kq != 0 || !aligned16(pa)) {
        void* ws;
        AIXK_TRY(workspace(ctx, 0, M * K * esz, &ws));
        AIXK_TRY(gather_dense(ctx, a, ws, M * K));
        pa = (const char*)ws;
        lda = K;
    }
    const char* pb = (const char*)b->data + b->offset * esz;
    uint64_t ldb = b->strides[1];
    if (!(b->strides[0] == 1 || K == 1) || ldb % kq != 0 || !aligned16(pb)) {
        aixhip_tensor bt = *b;                                    // the [N,K] view of b
        bt.shape[0] = N; bt.shape[1] = K;
        bt.strides[0] = b->strides[1]; bt.strides[1] = b->strides[0];
        void* ws;
        AIXK_TRY(workspace(ctx, 1, N * K * esz, &ws));
        AIXK_TRY(gather_dense(ctx, &bt, ws, N * K));
        pb = (const char*)ws;
        ldb = K;
    }

    GemmArgs g{};
    g.a = pa; g.b = pb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb;
    auto grid16 = [&](uint64_t bm, uint64_t bn) { return grid_of(g, bm, bn); };
    const bool big = ((M + 255) / 256) * ((N + 255) / 256) >= (uint64_t)ctx->cus / 2;
    if (big) {
        constexpr size_t lds = 2 * (256 + 256) * 72 * 2;
        const u32 n = grid16(256, 256);
        if (out->dtype == AIXK_BF16) { AIXK_TRY(set_lds(gemm_nt16_k<bf16, 256, 256>, lds)); hipLaunchKernelGGL((gemm_nt16_k<bf16, 256, 256>), dim3(n), dim3(256), lds, ctx->stream, g); }
        else { AIXK_TRY(set_lds(gemm_nt16_k<f16, 256, 256>, lds)); hipLaunchKernelGGL((gemm_nt16_k<f16, 256, 256>), dim3(n), dim3(256), lds, ctx->stream, g); }
    } else if (small_tiles) {
        constexpr size_t lds = 2 * (64 + 64) * 72 * 2;
        const u32 n = grid16(64, 64);
        if (out->dtype == AIXK_BF16) { AIXK_TRY(set_lds(gemm_nt16_k<bf16, 64, 64>, lds)); hipLaunchKernelGGL((gemm_nt16_k<bf16, 64, 64>), dim3(n), dim3(256), lds, ctx->stream, g); }
        else { AIXK_TRY(set_lds(gemm_nt16_k<f16, 64, 64>, lds)); hipLaunchKernelGGL((gemm_nt16_k<f16, 64, 64>), dim3(n), dim3(256), lds, ctx->stream, g); }
    } else {
        constexpr size_t lds = 2 * (128 + 128) * 72 * 2;
        const u32 n = grid16(128, 128);
        if (out->dtype == AIXK_BF16) { AIXK_TRY(set_lds(gemm_nt16_k<bf16, 128, 128>, lds)); hipLaunchKernelGGL((gemm_nt16_k<bf16, 128, 128>), dim3(n), dim3(256), lds, ctx->stream, g); }
        else { AIXK_TRY(set_lds(gemm_nt16_k<f16, 128, 128>, lds)); hipLaunchKernelGGL((gemm_nt16_k<f16, 128, 128>), dim3(n), dim3(256), lds, ctx->stream, g); }
    }
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

} // namespace aixk
