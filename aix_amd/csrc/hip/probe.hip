// probe.hip -- what the matrix pipe of this part delivers when it does nothing but multiply: a loop of independent
// 16-bit MFMAs on register operands, no LDS, no memory traffic.  On MI355X the answer depends on the operand VALUES (the
// part is power-limited: toggling bits in the multipliers and accumulators set the clock), on the instruction
// (v_mfma_f32_16x16x32 rewrites half as many accumulator bits per flop as v_mfma_f32_32x32x16) and on whether a second
// wave per SIMD fills the issue gaps of the first, so a GEMM's fraction of the nominal peak is read against this
// ceiling, measured on the same box in the same run (bench.py prints it beside the GEMM lines).
// No counterpart in the reference (its benchmarks time whole operators: Targets/AIXBenchmarks/Main.cpp:204-248).
#pragma clang fp contract(fast)

#include "common.hpp"

#include <algorithm>
#include <vector>

using namespace aixd;
using namespace aixk;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// SHAPE 0: four waves per workgroup, each 4 x 4 accumulator tiles of v_mfma_f32_32x32x16 (256 accumulator registers);
// SHAPE 1: eight waves per workgroup, each 8 x 4 accumulator tiles of v_mfma_f32_16x16x32 (128 accumulator registers):
// the two register layouts of gemm_nt16_direct_k, before and after it moved to two waves per SIMD.  `rounds` rounds of
// all the wave's accumulator tiles; clocks[0..1] = shader cycles and 100 MHz ticks workgroup 0 spent in the loop.
template <int SHAPE, bool HALF>
__global__ __launch_bounds__(SHAPE ? 512 : 256) void mfma_only_k(const u32x4* __restrict__ src, float* __restrict__ out, int rounds, u64* __restrict__ clocks)
{
    constexpr int NI = SHAPE ? 8 : 4, NJ = 4;
    extern __shared__ unsigned char keep_one_workgroup_per_cu[];
    const int lane = threadIdx.x;
    u32x4 fa[NI], fb[NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i) fa[i] = src[(blockIdx.x % 64 * 12 + i) * 512 + lane];
#pragma unroll
    for (int j = 0; j < NJ; ++j) fb[j] = src[(blockIdx.x % 64 * 12 + 8 + j) * 512 + lane];
    const u64 c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    float sum = 0.0f;
    if constexpr (SHAPE == 0) {
        f32x16 acc[NI][NJ];
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
        for (int r = 0; r < rounds; ++r)
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if constexpr (HALF) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[i]), __builtin_bit_cast(f16x8, fb[j]), acc[i][j], 0, 0, 0);
                    else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[i]), __builtin_bit_cast(bf16x8, fb[j]), acc[i][j], 0, 0, 0);
                }
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) sum += acc[i][j][v];
    } else {
        f32x4 acc[NI][NJ];
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int r = 0; r < rounds; ++r)
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if constexpr (HALF) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fa[i]), __builtin_bit_cast(f16x8, fb[j]), acc[i][j], 0, 0, 0);
                    else acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fa[i]), __builtin_bit_cast(bf16x8, fb[j]), acc[i][j], 0, 0, 0);
                }
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) sum += acc[i][j].x + acc[i][j].y + acc[i][j].z + acc[i][j].w;
    }
    const u64 c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    out[(u64)blockIdx.x * blockDim.x + threadIdx.x] = sum;
    if (threadIdx.x == 0 && blockIdx.x == 0) { clocks[0] = c1 - c0; clocks[1] = w1 - w0; }
}

} // namespace

// One workgroup per compute unit multiplies `gflop_per_launch` GFLOP (rounded to whole rounds) per launch, 200 untimed and
// 7 x 40 timed launches on the context's stream; the median of the seven.  shape: 0 or 1 (see mfma_only_k); dtype:
// AIXK_BF16 or AIXK_F16; operands: `count` 16-bit patterns used round-robin as operand values (one zero: all-zero
// operands).  *tflops: achieved rate; *ghz: shader clock during the loop (cycle counter over the 100 MHz wall clock).
extern "C" int32_t aixk_mfma_only_rate(aixk_ctx* ctx, int32_t shape, int32_t dtype, const uint16_t* operands, uint32_t count, double gflop_per_launch,
                                       float* tflops, float* ghz)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE((shape == 0 || shape == 1) && (dtype == AIXK_BF16 || dtype == AIXK_F16), "mfma_only_rate: shape 0 or 1, bf16 or f16");
    AIXK_REQUIRE(operands && count > 0 && tflops && ghz && gflop_per_launch > 0, "mfma_only_rate: null or empty argument");
    const unsigned cus = (unsigned)ctx->cus, threads = shape ? 512u : 256u;
    const size_t words = (size_t)64 * 12 * 512 * 8;                       // 16-bit values the fragments are cut from
    std::vector<uint16_t> host(words);
    for (size_t i = 0; i < words; ++i) host[i] = operands[i % count];
    void *src = nullptr, *out = nullptr, *clocks = nullptr;
    AIXK_HIP(hipMalloc(&src, words * 2));
    hipError_t e = hipMalloc(&out, (size_t)cus * threads * 4);
    if (e == hipSuccess) e = hipMalloc(&clocks, 16);
    if (e == hipSuccess) e = hipMemcpy(src, host.data(), words * 2, hipMemcpyHostToDevice);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    auto cleanup = [&] { (void)hipFree(src); (void)hipFree(out); (void)hipFree(clocks); if (e0) (void)hipEventDestroy(e0); if (e1) (void)hipEventDestroy(e1); };
    if (e != hipSuccess) { cleanup(); return fail(AIXK_EHIP, "mfma_only_rate: %s", hipGetErrorString(e)); }
    // flops of one round of one wave: 16 tiles of 32 x 32 x 16, or 32 tiles of 16 x 16 x 32
    const double per_round = 2.0 * (shape ? 32.0 * 16 * 16 * 32 : 16.0 * 32 * 32 * 16) * (threads / 64) * cus;
    const int rounds = (int)std::max(1.0, gflop_per_launch * 1e9 / per_round + 0.5);
    constexpr size_t lds = 100 * 1024;                                     // one workgroup per compute unit
    auto launch = [&]() -> hipError_t {
        if (shape == 0 && dtype == AIXK_BF16) hipLaunchKernelGGL((mfma_only_k<0, false>), dim3(cus), dim3(threads), lds, ctx->stream, (const u32x4*)src, (float*)out, rounds, (u64*)clocks);
        else if (shape == 0) hipLaunchKernelGGL((mfma_only_k<0, true>), dim3(cus), dim3(threads), lds, ctx->stream, (const u32x4*)src, (float*)out, rounds, (u64*)clocks);
        else if (dtype == AIXK_BF16) hipLaunchKernelGGL((mfma_only_k<1, false>), dim3(cus), dim3(threads), lds, ctx->stream, (const u32x4*)src, (float*)out, rounds, (u64*)clocks);
        else hipLaunchKernelGGL((mfma_only_k<1, true>), dim3(cus), dim3(threads), lds, ctx->stream, (const u32x4*)src, (float*)out, rounds, (u64*)clocks);
        return hipGetLastError();
    };
    for (auto k : {(const void*)mfma_only_k<0, false>, (const void*)mfma_only_k<0, true>, (const void*)mfma_only_k<1, false>, (const void*)mfma_only_k<1, true>})
        if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    for (int i = 0; i < 200 && e == hipSuccess; ++i) e = launch();        // past the part's power transient (about 10 ms)
    float times[7] = {};
    for (int rep = 0; rep < 7 && e == hipSuccess; ++rep) {
        e = hipEventRecord(e0, ctx->stream);
        for (int i = 0; i < 40 && e == hipSuccess; ++i) e = launch();
        if (e == hipSuccess) e = hipEventRecord(e1, ctx->stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&times[rep], e0, e1);
    }
    u64 c[2] = {0, 1};
    if (e == hipSuccess) e = hipMemcpy(c, clocks, 16, hipMemcpyDeviceToHost);
    cleanup();
    if (e != hipSuccess) return fail(AIXK_EHIP, "mfma_only_rate: %s", hipGetErrorString(e));
    std::sort(times, times + 7);
    *tflops = (float)(per_round * rounds / (times[3] / 40.0 * 1e-3) / 1e12);
    *ghz = (float)((double)c[0] / ((double)c[1] / 100.0) / 1000.0);
    return AIXK_OK;
}
