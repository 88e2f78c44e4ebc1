// matmul.hip -- out[m,n] = a[m,k] . b[k,n] for arbitrary 2-D operand views
// (aixDeviceCPU.cpp:362-389).
//
// Two families:
//   * f32 / f16 / bf16: MFMA kernels with f32 accumulation (matmul_mfma.hip);
//   * f64 and the integer types: the LDS-tiled kernel in this file with an accumulator of the
//     element type (integers wrap as on the CPU); also the fallback for operand layouts the MFMA
//     kernels do not take.
// The result is written row-major from out->data.

#include "common.hpp"

using namespace aixd;
using namespace aixk;

namespace aixk {
// Implemented in matmul_mfma.hip.  Returns AIXK_OK if it launched, -1 if the shape/layout is not
// one it handles (caller falls back), or an error status.
int matmul_mfma(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out);
// The same for a stack of products (a, b, out: the 2-D descriptors of the first matrices; batch: the joint
// collapsed space of the leading dims, operands a, b, out).
int matmul_mfma_batched(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, const Space<3>& batch);
int matmul_mfma_grouped(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint32_t count);
} // namespace aixk

namespace {

template <class T> struct mm_acc { typedef typename traits<T>::W type; };
template <> struct mm_acc<i64> { typedef u64 type; };
template <> struct mm_acc<i32> { typedef u32 type; };
template <> struct mm_acc<i16> { typedef u32 type; };
template <> struct mm_acc<i8>  { typedef u32 type; };
template <> struct mm_acc<u8>  { typedef u32 type; };

template <class T> __device__ __forceinline__ typename mm_acc<T>::type mm_up(T v) { return (typename mm_acc<T>::type)up(v); }
template <class T> __device__ __forceinline__ T mm_down(typename mm_acc<T>::type v)
{
    if constexpr (traits<T>::is_int) return (T)v; else return down<T>(v);
}

constexpr int TM = 64, TN = 64, TK = 16;

struct MatView { u64 off, s0, s1; };

template <class T>
__global__ __launch_bounds__(kBlock) void matmul_tiled_k(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
                                                         MatView va, MatView vb, u64 M, u64 N, u64 K)
{
    typedef typename mm_acc<T>::type A;
    __shared__ A As[TK][TM + 4];
    __shared__ A Bs[TK][TN + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;          // 16 x 16 lanes, 4 x 4 outputs each
    const u64 m0 = (u64)blockIdx.y * TM, n0 = (u64)blockIdx.x * TN;
    A acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (A)0;

    for (u64 k0 = 0; k0 < K; k0 += TK) {
        // A tile: TM x TK, B tile: TK x TN; 1024 elements each, 4 per lane
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int e = threadIdx.x + r * kBlock;
            const int ak = e & (TK - 1), am = e >> 4;                 // k fastest for A
            const u64 gm = m0 + am, gk = k0 + ak;
            As[ak][am] = (gm < M && gk < K) ? mm_up(a[va.off + gm * va.s0 + gk * va.s1]) : (A)0;
            const int bn = e & (TN - 1), bk = e >> 6;                 // n fastest for B
            const u64 gn = n0 + bn, gk2 = k0 + bk;
            Bs[bk][bn] = (gn < N && gk2 < K) ? mm_up(b[vb.off + gk2 * vb.s0 + gn * vb.s1]) : (A)0;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            A ra[4], rb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) ra[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) rb[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += ra[i] * rb[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u64 gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u64 gn = n0 + tx * 4 + j;
            if (gn < N) out[gm * N + gn] = mm_down<T>(acc[i][j]);
        }
    }
}

} // namespace

extern "C" int32_t aixk_matmul(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(b) && valid_tensor(out), "matmul: bad operand descriptor");
    AIXK_REQUIRE(a->rank == 2 && b->rank == 2, "matmul: operands must be 2-D");            // aixCore.hpp:946-955
    AIXK_REQUIRE(a->shape[1] == b->shape[0], "matmul: inner dimensions differ");
    AIXK_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype, "matmul: operands must have the result's element type");
    const uint64_t M = a->shape[0], K = a->shape[1], N = b->shape[1];
    if (M == 0 || N == 0) return AIXK_OK;
    if (K == 0) return aixk_zero(ctx, out->data, M * N * aixk_dtype_size(out->dtype));
    AIXK_REQUIRE(out->data != nullptr, "matmul: null result");
    ctx->gemm_last_route = 0;

    if (out->dtype == AIXK_F32 || out->dtype == AIXK_F16 || out->dtype == AIXK_BF16) {
        const int rc = matmul_mfma(ctx, a, b, out);
        if (rc != -1) return rc;
    }
    const uint64_t gx = (N + TN - 1) / TN, gy = (M + TM - 1) / TM;
    AIXK_REQUIRE(gx < (1ull << 31) && gy < 65536, "matmul: shape too large for the generic kernel");
    const MatView va{a->offset, a->strides[0], a->strides[1]}, vb{b->offset, b->strides[0], b->strides[1]};
    return by_dtype(out->dtype, [&](auto tag) {
        typedef decltype(tag) T;
        hipLaunchKernelGGL((matmul_tiled_k<T>), dim3((unsigned)gx, (unsigned)gy), dim3(kBlock), 0, ctx->stream,
                           (const T*)a->data, (const T*)b->data, (T*)out->data, va, vb, (u64)M, (u64)N, (u64)K);
        AIXK_HIP(hipGetLastError());
        return (int)AIXK_OK;
    });
}

extern "C" int32_t aixk_matmul_route(aixk_ctx* ctx, int32_t* route, int32_t* redone)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(route && redone, "matmul route: null result");
    AIXK_HIP(hipStreamSynchronize(ctx->stream));
    unsigned int flag = 0;
    AIXK_HIP(hipMemcpy(&flag, ctx->counter, sizeof(flag), hipMemcpyDeviceToHost));
    *route = ctx->gemm_last_route;
    *redone = ctx->gemm_last_route == 1 && flag == ctx->gemm_seq;
    return AIXK_OK;
}

// out[..., m, n] = a[..., m, k] . b[..., k, n]: one product per index of the leading dims, which a, b and out share
// (any of them may be a view: permuted, sliced, stride 0).  The results are written densely, row-major over
// (leading dims, m, n), from out->data.
extern "C" int32_t aixk_matmul_grouped(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(count == 0 || (a && b && out), "matmul group: null operand arrays");
    if (count >= 2) {
        bool plain = true;
        for (uint32_t i = 0; i < count && plain; ++i)
            plain = valid_tensor(&a[i]) && valid_tensor(&b[i]) && valid_tensor(&out[i]) && a[i].rank == 2 && b[i].rank == 2 && out[i].rank == 2 &&
                    a[i].shape[1] == b[i].shape[0] && out[i].shape[0] == a[i].shape[0] && out[i].shape[1] == b[i].shape[1] && out[i].data != nullptr &&
                    a[i].shape[0] && b[i].shape[1] && a[i].shape[1];
        if (plain) {
            const int rc = matmul_mfma_grouped(ctx, a, b, out, count);
            if (rc != -1) return rc;
        }
    }
    for (uint32_t i = 0; i < count; ++i) AIXK_TRY(aixk_matmul(ctx, &a[i], &b[i], &out[i]));    // one by one, every check of the single call
    return AIXK_OK;
}

extern "C" int32_t aixk_matmul_batched(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(valid_tensor(a) && valid_tensor(b) && valid_tensor(out), "matmul: bad operand descriptor");
    AIXK_REQUIRE(a->rank >= 2 && a->rank == b->rank && a->rank == out->rank, "matmul: operands and result must have the same rank, at least 2");
    if (a->rank == 2) return aixk_matmul(ctx, a, b, out);
    const int nb = a->rank - 2;
    for (int d = 0; d < nb; ++d)
        AIXK_REQUIRE(a->shape[d] == b->shape[d] && a->shape[d] == out->shape[d], "matmul: leading dimensions differ");
    AIXK_REQUIRE(a->shape[nb + 1] == b->shape[nb], "matmul: inner dimensions differ");
    AIXK_REQUIRE(out->shape[nb] == a->shape[nb] && out->shape[nb + 1] == b->shape[nb + 1], "matmul: result shape does not match the operands");
    AIXK_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype, "matmul: operands must have the result's element type");
    const uint64_t M = a->shape[nb], K = a->shape[nb + 1], N = b->shape[nb + 1];
    uint64_t count = 1;
    for (int d = 0; d < nb; ++d) count *= a->shape[d];
    if (count == 0 || M == 0 || N == 0) return AIXK_OK;
    const size_t esz = aixk_dtype_size(out->dtype);
    AIXK_REQUIRE(out->data != nullptr, "matmul: null result");
    if (K == 0) return aixk_zero(ctx, out->data, count * M * N * esz);

    // the leading dims as one joint iteration space; the result's strides are those of a dense stack
    uint64_t dense[AIXK_MAX_RANK];
    { uint64_t run = M * N; for (int d = nb - 1; d >= 0; --d) { dense[d] = run; run *= a->shape[d]; } }
    const uint64_t* strides[3] = {a->strides, b->strides, dense};
    const uint64_t offsets[3] = {0, 0, 0};
    Space<3> batch;
    AIXK_REQUIRE(collapse<3>(nb, a->shape, strides, offsets, &batch), "matmul: leading dims do not collapse to %d", kMaxDims);

    auto matrix = [](const aixhip_tensor* t, int nb) {
        aixhip_tensor m = *t;
        m.rank = 2;
        m.shape[0] = t->shape[nb]; m.shape[1] = t->shape[nb + 1];
        m.strides[0] = t->strides[nb]; m.strides[1] = t->strides[nb + 1];
        m.size = m.shape[0] * m.shape[1];
        return m;
    };
    aixhip_tensor a2 = matrix(a, nb), b2 = matrix(b, nb), o2 = matrix(out, nb);
    o2.offset = 0; o2.strides[0] = N; o2.strides[1] = 1;
    if (out->dtype == AIXK_F16 || out->dtype == AIXK_BF16) {
        const int rc = matmul_mfma_batched(ctx, &a2, &b2, &o2, batch);
        if (rc != -1) return rc;
    }
    // one launch per product
    uint64_t coord[kMaxDims] = {};
    for (uint64_t i = 0; i < count; ++i) {
        uint64_t oa = a->offset, ob = b->offset;
        for (int d = 0; d < batch.rank; ++d) { oa += coord[d] * batch.stride[0][d]; ob += coord[d] * batch.stride[1][d]; }
        a2.offset = oa; b2.offset = ob;
        o2.data = (char*)out->data + i * M * N * esz;
        AIXK_TRY(aixk_matmul(ctx, &a2, &b2, &o2));
        for (int d = batch.rank - 1; d >= 0; --d) { if (++coord[d] < batch.shape[d]) break; coord[d] = 0; }
    }
    return AIXK_OK;
}
