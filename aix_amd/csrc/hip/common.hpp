// common.hpp -- host-side plumbing shared by the launchers of libaixhip_kernels.so:
// the context, status/error helpers, element-type dispatch, and the layout collapser that
// turns up to three N-d views into the smallest equivalent strided iteration space.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../../include/aixhip_kernels.h"
#include "aix_device.h"

namespace aixk {

constexpr int kMaxDims = AIXK_MAX_RANK;  // rank of a collapsed iteration space the kernels accept: any view the descriptor can hold
constexpr int kBlock = 256;              // threads per workgroup: 4 wavefronts of 64

int fail(int code, const char* fmt, ...);
#define AIXK_HIP(call)                                                                          \
    do {                                                                                        \
        hipError_t e_ = (call);                                                                 \
        if (e_ != hipSuccess)                                                                   \
            return aixk::fail(AIXK_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                              __FILE__, __LINE__);                                              \
    } while (0)
#define AIXK_REQUIRE(cond, ...)                                   \
    do {                                                          \
        if (!(cond)) return aixk::fail(AIXK_EINVAL, __VA_ARGS__); \
    } while (0)
#define AIXK_TRY(expr)                 \
    do {                               \
        int rc_ = (expr);              \
        if (rc_ != AIXK_OK) return rc_; \
    } while (0)

struct RtcModule {
    hipModule_t module{nullptr};
    hipFunction_t fn{nullptr};
};

} // namespace aixk

// The context: one device, one in-order stream.  All launchers enqueue on `stream`.
struct aixk_ctx {
    int device{0};
    hipStream_t stream{nullptr};
    hipDeviceProp_t prop{};
    int cus{256};
    // scratch for multi-block reductions: partial results
    void* scratch{nullptr};
    size_t scratch_bytes{0};
    // this device's address of the static scratch array of reduce.hip (the entry point that allocates nothing)
    void* static_scratch{nullptr};
    // 256 bytes of flags, zeroed at creation.  Word 0: set to `gemm_seq` by a split-plane f32 matmul that met an
    // infinity or a NaN in its operands (the IEEE-faithful kernel then redoes the product); launches are numbered,
    // so the word never has to be cleared.
    unsigned int* counter{nullptr};
    unsigned int gemm_seq{0};
    int gemm_last_route{0};            // what the last aixk_matmul took: 1 the split-plane f32 route (gemm_x3_k), 0 anything else
    // matmul: K-contiguous copies of operands whose layout the kernels cannot consume in place
    // (0: A, 1: B) and the f32 partial results of K splits (2); grown on demand, ordered on `stream`
    // like everything else
    void* gemm_ws[3]{nullptr, nullptr, nullptr};
    size_t gemm_ws_bytes[3]{0, 0, 0};
    // small tables that kernels read from device memory (the operand addresses of a grouped launch): a pinned host ring
    // and its device twin, filled slot by slot and copied on the stream; an event per lap guards the reuse of a slot
    char* table_host{nullptr};
    char* table_dev{nullptr};
    size_t table_bytes{0}, table_used{0};
    hipEvent_t table_lap[2]{nullptr, nullptr};
    int table_half{0};
    // a step being captured into a graph (aixk_capture_begin): its tables live in memory the graph owns, written once
    struct aixk_graph* capturing{nullptr};
    hipStream_t side{nullptr};         // for copies that must happen now while `stream` is capturing
    // runtime-compiled kernels by signature
    std::unordered_map<std::string, aixk_module*> rtc;
    uint64_t rtc_hits{0}, rtc_misses{0};
    // code objects of generated kernels kept on disk (AIXHIP_KERNEL_CACHE_DIR, read when the context is created; empty: off)
    std::string rtc_disk_dir;
    uint64_t rtc_disk_hits{0}, rtc_disk_stores{0};
};

struct aixk_module { aixk::RtcModule m; };
// A captured stretch of the stream.  `tables`: device memory holding the argument tables of its many-blocks launches
// (written when they were captured; the launches read them at every replay), with the pinned memory they were staged in.
struct aixk_graph {
    hipGraph_t graph{nullptr};
    hipGraphExec_t exec{nullptr};
    std::vector<std::pair<void*, void*>> tables;          // (device, pinned host)
    uint64_t nodes{0};
};
struct aixk_event { hipEvent_t ev{nullptr}; };

namespace aixk {

size_t stream_store_min_bytes();                      // runtime.hip: AIXK_STREAM_STORE_MIN_BYTES or its environment override
inline bool streams_out(size_t bytes) { return bytes >= stream_store_min_bytes(); }
int resolve_static_scratch(aixk_ctx* ctx);
// runtime.hip: `bytes` of table space: where the host writes it and where kernels will find it once table_upload() has run
int table_slot(aixk_ctx* ctx, size_t bytes, void** host, const void** dev);
int table_upload(aixk_ctx* ctx, const void* host, const void* dev, size_t bytes);          // reduce.hip; called once per context by aixk_create

inline int set_device(aixk_ctx* ctx)
{
    AIXK_REQUIRE(ctx != nullptr, "null context");
    AIXK_HIP(hipSetDevice(ctx->device));
    return AIXK_OK;
}

// ---- element type dispatch -------------------------------------------------------------------
template <class F> inline int by_dtype(int dtype, F&& f)
{
    using namespace aixd;
    switch (dtype) {
        case AIXK_F64:  return f(double{});
        case AIXK_F32:  return f(float{});
        case AIXK_F16:  return f(f16{});
        case AIXK_BF16: return f(bf16{});
        case AIXK_I64:  return f(i64{});
        case AIXK_I32:  return f(i32{});
        case AIXK_I16:  return f(i16{});
        case AIXK_I8:   return f(i8{});
        case AIXK_U8:   return f(u8{});
        default: return fail(AIXK_EINVAL, "unknown element type %d", dtype);
    }
}

inline bool valid_tensor(const aixhip_tensor* t)
{
    return t && t->rank >= 0 && t->rank <= AIXK_MAX_RANK && t->dtype >= 0 && t->dtype < AIXK_DTYPE_COUNT &&
           (t->size == 0 || t->data != nullptr);
}

inline uint64_t numel(const aixhip_tensor* t)
{
    uint64_t n = 1;
    for (int d = 0; d < t->rank; ++d) n *= t->shape[d];
    return n;
}

// ---- collapsed iteration space ---------------------------------------------------------------
// An iteration space of `rank` dims (outermost first) shared by up to three operands, each with
// its own element offset and per-dim strides.  Kernel-argument POD.
template <int NOPS> struct Space {
    int rank;
    uint64_t shape[kMaxDims];
    uint64_t offset[NOPS];
    uint64_t stride[NOPS][kMaxDims];
};

// Builds the joint collapsed space of NOPS views that all iterate `shape` (rank `rank`):
// drops extent-1 dims and merges neighbours wherever every operand's strides allow
// (stride[d] == stride[d+1] * shape[d+1]).  Returns false if more than kMaxDims dims remain.
template <int NOPS>
inline bool collapse(int rank, const uint64_t* shape, const uint64_t* const strides[NOPS],
                     const uint64_t offsets[NOPS], Space<NOPS>* out)
{
    uint64_t shp[AIXK_MAX_RANK];
    uint64_t str[NOPS][AIXK_MAX_RANK];
    int r = 0;
    for (int d = 0; d < rank; ++d) {
        if (shape[d] == 1) continue;
        shp[r] = shape[d];
        for (int o = 0; o < NOPS; ++o) str[o][r] = strides[o][d];
        ++r;
    }
    // merge from the innermost outwards
    int w = r - 1;                     // write cursor (we build in place, right to left)
    for (int d = r - 2; d >= 0; --d) {
        bool mergeable = true;
        for (int o = 0; o < NOPS; ++o)
            if (str[o][d] != str[o][w] * shp[w]) { mergeable = false; break; }
        if (mergeable) {
            shp[w] *= shp[d];
        } else {
            --w;
            shp[w] = shp[d];
            for (int o = 0; o < NOPS; ++o) str[o][w] = str[o][d];
        }
    }
    int first = (r == 0) ? 0 : w;
    int nr = (r == 0) ? 0 : r - first;
    if (nr > kMaxDims) return false;
    out->rank = nr;
    for (int d = 0; d < kMaxDims; ++d) {
        out->shape[d] = d < nr ? shp[first + d] : 1;
        for (int o = 0; o < NOPS; ++o) out->stride[o][d] = d < nr ? str[o][first + d] : 0;
    }
    for (int o = 0; o < NOPS; ++o) out->offset[o] = offsets[o];
    return true;
}

// Element position of flat logical index i under operand `op` of a collapsed space.
template <int NOPS, class IDX>
__device__ __forceinline__ uint64_t locate(const Space<NOPS>& sp, int op, IDX i)
{
    uint64_t p = sp.offset[op];
    for (int d = sp.rank - 1; d >= 0; --d) {
        const IDX ext = (IDX)sp.shape[d];
        const IDX q = i / ext;
        p += (uint64_t)(i - q * ext) * sp.stride[op][d];
        i = q;
    }
    return p;
}

inline bool collapse1(const aixhip_tensor* t, Space<1>* sp)
{
    const uint64_t* st[1] = {t->strides};
    const uint64_t off[1] = {t->offset};
    return collapse<1>(t->rank, t->shape, st, off, sp);
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

inline void row_major_strides(int rank, const uint64_t* shape, uint64_t* out)
{
    uint64_t run = 1;
    for (int d = rank - 1; d >= 0; --d) { out[d] = run; run *= shape[d]; }
}

// Largest element position (exclusive bound) a view can touch; used for 32-bit index checks.
inline uint64_t view_extent(const aixhip_tensor* t)
{
    uint64_t last = t->offset;
    for (int d = 0; d < t->rank; ++d)
        if (t->shape[d] > 0) last += (t->shape[d] - 1) * t->strides[d];
    return last + 1;
}

inline unsigned grid_for(uint64_t work_items, unsigned per_block, unsigned max_blocks)
{
    uint64_t b = (work_items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > max_blocks) b = max_blocks;
    return (unsigned)b;
}

} // namespace aixk
