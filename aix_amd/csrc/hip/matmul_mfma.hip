// matmul_mfma.hip -- GEMM on the matrix cores for f32 / f16 / bf16, f32 accumulation.
//
// One core kernel shape per precision, both operands K-contiguous in memory ("NT": A is [M,K] with
// unit stride along K, B is given as [N,K] with unit stride along K):
//
//   16-bit  v_mfma_f32_32x32x16_{bf16,f16}; workgroup tile 256x256 (or 128x128 for small
//           problems) x BK=64, 4 waves in a 2x2 arrangement, each wave 4x4 (2x2) MFMA tiles with
//           the accumulators resident in the 512-entry unified register file;
//   f32     v_mfma_f32_32x32x2f32; workgroup tile 128x128 x BK=32, each wave 2x2 MFMA tiles.
//
// Per K-step: 16-byte global loads into registers for step t+1 are issued before the MFMAs of step
// t, then written to the other LDS buffer (double buffered, one barrier per step).  LDS rows are
// padded by 16 bytes so that the 8 lanes served per LDS cycle by ds_read_b128 hit 32 distinct
// banks.  Every lane feeds the MFMA with 8 (f32: 4) consecutive K values of one row; because A and
// B use the same lane->K assignment, the dot products are independent of how the instruction
// numbers K internally.
//
// Workgroups are numbered so that the 32 groups resident on one XCD (dispatch is round-robin over
// the 8 XCDs) cover a compact 4 x 8 block of output tiles and share A/B panels in that XCD's L2.
//
// Operands that are not K-contiguous (plain row-major B, transposed-view A, sliced views) are
// first gathered into K-contiguous scratch by the tiled transpose; odd K (not a multiple of 8
// elements for 16-bit, 4 for f32) falls back to the LDS-tiled kernel in matmul.hip.
#pragma clang fp contract(fast)

#include "common.hpp"

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
    static __device__ __forceinline__ bf16 out(float v) { return bf16_down(v); }
};
template <> struct Mma16<f16> {
    static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c)
    { return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0); }
    static __device__ __forceinline__ f16 out(float v) { return (f16)v; }
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

// ---- f32 operands ------------------------------------------------------------------------------
// 128 x 128 workgroup tile, BK = 32; LDS row = 32 floats + 4 padding = 144 bytes.  A lane reads 4
// consecutive K of its row with one ds_read_b128 and spends them on 4 successive 32x32x2 MFMAs.
__global__ __launch_bounds__(256) void gemm_nt32_k(GemmArgs g)
{
    constexpr int BM = 128, BN = 128, BK = 32, LDR = BK + 4;
    constexpr int WM = 64, WN = 64, TI = 2, TJ = 2;
    constexpr int CA = BM * (BK / 4) / 256, CB = BN * (BK / 4) / 256;      // 4 each
    extern __shared__ __attribute__((aligned(16))) unsigned char smem32[];
    float (*As)[BM][LDR] = (float (*)[BM][LDR])smem32;                       // [2][BM][LDR]
    float (*Bs)[BN][LDR] = (float (*)[BN][LDR])(smem32 + sizeof(float) * 2 * BM * LDR);

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

    f32x4 ra[CA], rb[CB];
    auto load_global = [&](u64 k0) {
#pragma unroll
        for (int i = 0; i < CA; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            const u64 r = m0 + row, k = k0 + kc * 4;
            ra[i] = (r < g.M && k < g.K) ? *(const f32x4*)(A + r * g.lda + k) : (f32x4){0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
            const u64 r = n0 + row, k = k0 + kc * 4;
            rb[i] = (r < g.N && k < g.K) ? *(const f32x4*)(B + r * g.ldb + k) : (f32x4){0, 0, 0, 0};
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CA; ++i) { const int c = tid + 256 * i; *(f32x4*)&As[buf][c >> 3][(c & 7) * 4] = ra[i]; }
#pragma unroll
        for (int i = 0; i < CB; ++i) { const int c = tid + 256 * i; *(f32x4*)&Bs[buf][c >> 3][(c & 7) * 4] = rb[i]; }
    };

    const u64 steps = (g.K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (u64 kt = 0; kt < steps; ++kt) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < steps) load_global((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 8; ++kk) {
            f32x4 fa[TI], fb[TJ];
#pragma unroll
            for (int i = 0; i < TI; ++i) fa[i] = *(const f32x4*)&As[buf][wm * WM + i * 32 + (lane & 31)][kk * 8 + (lane >> 5) * 4];
#pragma unroll
            for (int j = 0; j < TJ; ++j) fb[j] = *(const f32x4*)&Bs[buf][wn * WN + j * 32 + (lane & 31)][kk * 8 + (lane >> 5) * 4];
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < TI; ++i)
#pragma unroll
                    for (int j = 0; j < TJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < steps) store_lds(buf ^ 1);
        __syncthreads();
    }

    float* C = (float*)g.c;
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
// process (all use is ordered on the context's single stream).
struct Workspace { void* ptr{nullptr}; size_t bytes{0}; };
Workspace g_ws[2];

int workspace(int which, size_t bytes, void** out)
{
    Workspace& w = g_ws[which];
    if (w.bytes < bytes) {
        if (w.ptr) { AIXK_HIP(hipDeviceSynchronize()); AIXK_HIP(hipFree(w.ptr)); w.ptr = nullptr; w.bytes = 0; }
        const size_t want = (bytes + (size_t(1) << 20)) & ~((size_t(1) << 20) - 1);
        if (hipMalloc(&w.ptr, want) != hipSuccess) { (void)hipGetLastError(); return fail(AIXK_ENOMEM, "matmul workspace of %zu bytes", want); }
        w.bytes = want;
    }
    *out = w.ptr;
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

} // namespace

namespace aixk {

int matmul_mfma(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out)
{
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    const size_t esz = aixk_dtype_size(out->dtype);
    const uint64_t kq = 16 / esz;                                 // elements per 16-byte chunk
    if (K % kq != 0 || M * N < 64 * 64) return -1;                // odd K / tiny outputs: LDS-tiled kernel
    if (((M + 127) / 128) * ((N + 127) / 128) >= (1ull << 31)) return -1;

    // A as [M,K] and B as [N,K], both with unit stride along K and 16-byte aligned rows
    const char* pa = (const char*)a->data + a->offset * esz;
    uint64_t lda = a->strides[0];
    if (!(a->strides[1] == 1 || K == 1) || lda % kq != 0 || !aligned16(pa)) {
        void* ws;
        AIXK_TRY(workspace(0, M * K * esz, &ws));
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
        AIXK_TRY(workspace(1, N * K * esz, &ws));
        AIXK_TRY(gather_dense(ctx, &bt, ws, N * K));
        pb = (const char*)ws;
        ldb = K;
    }

    GemmArgs g{};
    g.a = pa; g.b = pb; g.c = out->data;
    g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb;
    auto grid_of = [&](uint64_t bm, uint64_t bn) {
        g.tiles_m = (u32)((M + bm - 1) / bm);
        g.tiles_n = (u32)((N + bn - 1) / bn);
        const u32 n = g.tiles_m * g.tiles_n;
        g.swizzle = n % 8u == 0 ? 1u : 0u;
        return n;
    };
    if (out->dtype == AIXK_F32) {
        constexpr size_t lds = 2 * (128 + 128) * 36 * sizeof(float);
        const u32 n = grid_of(128, 128);
        AIXK_TRY(set_lds(gemm_nt32_k, lds));
        hipLaunchKernelGGL(gemm_nt32_k, dim3(n), dim3(256), lds, ctx->stream, g);
        AIXK_HIP(hipGetLastError());
        return AIXK_OK;
    }
    const bool big = ((M + 255) / 256) * ((N + 255) / 256) >= (uint64_t)ctx->cus / 2;
    if (big) {
        constexpr size_t lds = 2 * (256 + 256) * 72 * 2;
        const u32 n = grid_of(256, 256);
        if (out->dtype == AIXK_BF16) { AIXK_TRY(set_lds(gemm_nt16_k<bf16, 256, 256>, lds)); hipLaunchKernelGGL((gemm_nt16_k<bf16, 256, 256>), dim3(n), dim3(256), lds, ctx->stream, g); }
        else { AIXK_TRY(set_lds(gemm_nt16_k<f16, 256, 256>, lds)); hipLaunchKernelGGL((gemm_nt16_k<f16, 256, 256>), dim3(n), dim3(256), lds, ctx->stream, g); }
    } else {
        constexpr size_t lds = 2 * (128 + 128) * 72 * 2;
        const u32 n = grid_of(128, 128);
        if (out->dtype == AIXK_BF16) { AIXK_TRY(set_lds(gemm_nt16_k<bf16, 128, 128>, lds)); hipLaunchKernelGGL((gemm_nt16_k<bf16, 128, 128>), dim3(n), dim3(256), lds, ctx->stream, g); }
        else { AIXK_TRY(set_lds(gemm_nt16_k<f16, 128, 128>, lds)); hipLaunchKernelGGL((gemm_nt16_k<f16, 128, 128>), dim3(n), dim3(256), lds, ctx->stream, g); }
    }
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

} // namespace aixk
