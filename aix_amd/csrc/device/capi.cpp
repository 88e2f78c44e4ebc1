// capi.cpp -- include/aixhip.h on top of aix::hip::DeviceHIP: descriptor conversion and the
// exception -> status mapping.  No logic of its own.

#include "../../../include/aixhip.h"
#include "device_hip.hpp"

#include <cstdio>
#include <cstring>
#include <new>
#include <stdexcept>

using aix::DataType;
using aix::DeviceTensorParams;
using aix::hip::DeviceHIP;

struct aixhip_device {
    DeviceHIP impl;
    explicit aixhip_device(size_t index) : impl(index) {}
};

namespace {

thread_local char g_error[1024] = "";

void remember(const char* what) { std::snprintf(g_error, sizeof(g_error), "%s", what); }

template <class F> int32_t guarded(F&& f)
{
    try { f(); return AIXHIP_OK; }
    catch (const std::invalid_argument& e) { remember(e.what()); return AIXHIP_EINVAL; }
    catch (const std::bad_alloc&) { remember("out of host memory"); return AIXHIP_ERUNTIME; }
    catch (const std::exception& e) { remember(e.what()); return AIXHIP_ERUNTIME; }
    catch (...) { remember("unknown error"); return AIXHIP_ERUNTIME; }
}

DeviceTensorParams P(const aixhip_tensor* t)
{
    if (!t) throw std::invalid_argument("null tensor descriptor");
    if (t->rank < 0 || t->rank > AIXK_MAX_RANK) throw std::invalid_argument("tensor rank out of range");
    if (t->dtype < 0 || t->dtype >= AIXK_DTYPE_COUNT) throw std::invalid_argument("unknown data type");
    DeviceTensorParams p;
    p.data = t->data;
    p.dtype = static_cast<DataType>(t->dtype);
    p.offset = t->offset;
    p.size = t->size;
    p.shape.assign(t->shape, t->shape + t->rank);
    p.strides.assign(t->strides, t->strides + t->rank);
    bool dense = true;
    size_t run = 1;
    for (int d = t->rank - 1; d >= 0; --d) { if (t->strides[d] != run) dense = false; run *= t->shape[d]; }
    p.isContiguous = dense;                // as TensorValue computes it (aixCore.hpp:1472-1480)
    return p;
}

DataType DT(int dtype)
{
    if (dtype < 0 || dtype >= AIXK_DTYPE_COUNT) throw std::invalid_argument("unknown data type");
    return static_cast<DataType>(dtype);
}

DeviceHIP& D(aixhip_device* dev)
{
    if (!dev) throw std::invalid_argument("null device");
    return dev->impl;
}

} // namespace

namespace aix::hip {
DeviceHIP* fromHandle(::aixhip_device* handle) { return &D(handle); }
}

extern "C" {

const char* aixhip_last_error(void) { return g_error; }

int32_t aixhip_device_create(int device_index, aixhip_device** out)
{
    return guarded([&] {
        if (!out) throw std::invalid_argument("null out pointer");
        if (device_index < 0) throw std::invalid_argument("negative device index");
        *out = new aixhip_device((size_t)device_index);
    });
}

int32_t aixhip_device_destroy(aixhip_device* dev) { return guarded([&] { delete dev; }); }
int32_t aixhip_type(const aixhip_device* dev) { return dev ? (int32_t)dev->impl.type() : -1; }
const char* aixhip_name(const aixhip_device* dev) { (void)dev; return "HIP"; }
size_t aixhip_data_type_size(int dtype) { return (dtype >= 0 && dtype < AIXK_DTYPE_COUNT) ? aix::Device::dataTypeSize(static_cast<DataType>(dtype)) : 0; }

int32_t aixhip_allocate(aixhip_device* dev, size_t bytes, void** out)
{ return guarded([&] { if (!out) throw std::invalid_argument("null out pointer"); *out = D(dev).allocate(bytes); }); }
int32_t aixhip_allocate_typed(aixhip_device* dev, size_t count, int dtype, void** out)
{ return guarded([&] { if (!out) throw std::invalid_argument("null out pointer"); *out = D(dev).allocate(count, DT(dtype)); }); }
int32_t aixhip_deallocate(aixhip_device* dev, void* memory) { return guarded([&] { D(dev).deallocate(memory); }); }

#define AIXHIP_BINARY(cname, method)                                                                                              \
    int32_t cname(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* a2, const aixhip_tensor* result)              \
    { return guarded([&] { D(dev).method(P(a1), P(a2), P(result)); }); }
#define AIXHIP_UNARY(cname, method)                                                                                               \
    int32_t cname(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result)                                        \
    { return guarded([&] { D(dev).method(P(a), P(result)); }); }

AIXHIP_BINARY(aixhip_add, add)
AIXHIP_BINARY(aixhip_sub, sub)
AIXHIP_BINARY(aixhip_mul, mul)
AIXHIP_BINARY(aixhip_div, div)
AIXHIP_BINARY(aixhip_pow, pow)
AIXHIP_BINARY(aixhip_matmul, matmul)
AIXHIP_UNARY(aixhip_unary, unary)
AIXHIP_UNARY(aixhip_sum, sum)
AIXHIP_UNARY(aixhip_sqrt, sqrt)
AIXHIP_UNARY(aixhip_sin, sin)
AIXHIP_UNARY(aixhip_cos, cos)
AIXHIP_UNARY(aixhip_tanh, tanh)
AIXHIP_UNARY(aixhip_log, log)
AIXHIP_UNARY(aixhip_exp, exp)
AIXHIP_UNARY(aixhip_max, max)
AIXHIP_UNARY(aixhip_argmax, argmax)
AIXHIP_UNARY(aixhip_argmax_indices, argmaxIndices)
AIXHIP_UNARY(aixhip_contiguous, contiguous)
AIXHIP_UNARY(aixhip_reduce_to, reduceTo)
AIXHIP_UNARY(aixhip_max_to, maxTo)

int32_t aixhip_fill(aixhip_device* dev, const void* scalar, int scalar_dtype, const aixhip_tensor* result)
{ return guarded([&] { if (!scalar) throw std::invalid_argument("null scalar"); D(dev).fill(scalar, DT(scalar_dtype), P(result)); }); }
int32_t aixhip_fill_min(aixhip_device* dev, const aixhip_tensor* result) { return guarded([&] { D(dev).fillMin(P(result)); }); }
int32_t aixhip_transpose(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result, size_t dim0, size_t dim1)
{ return guarded([&] { D(dev).transpose(P(a), P(result), dim0, dim1); }); }
int32_t aixhip_copy(aixhip_device* dev, const void* src, int src_dtype, void* dst, int dst_dtype, size_t size)
{ return guarded([&] { D(dev).copy(src, DT(src_dtype), dst, DT(dst_dtype), size); }); }
int32_t aixhip_copy_immediate(aixhip_device* dev, const void* src, int src_dtype, void* dst, int dst_dtype, size_t size)
{ return guarded([&] { D(dev).copyImmediate(src, DT(src_dtype), dst, DT(dst_dtype), size); }); }
int32_t aixhip_argmax_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, size_t dim)
{ return guarded([&] { D(dev).argmaxTo(P(src), P(dst), dim); }); }
int32_t aixhip_argmax_indices_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, size_t dim)
{ return guarded([&] { D(dev).argmaxIndicesTo(P(src), P(dst), dim); }); }
int32_t aixhip_slice_set(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, size_t dim, size_t start, size_t end, size_t step)
{ return guarded([&] { D(dev).sliceSet(P(src), P(dst), dim, start, end, step); }); }
int32_t aixhip_tril(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal)
{ return guarded([&] { D(dev).tril(P(src), P(dst), (ssize_t)diagonal); }); }
int32_t aixhip_triu(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal)
{ return guarded([&] { D(dev).triu(P(src), P(dst), (ssize_t)diagonal); }); }
int32_t aixhip_index_select(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, const aixhip_tensor* indices, size_t dim)
{ return guarded([&] { D(dev).indexSelect(P(src), P(dst), P(indices), dim); }); }
int32_t aixhip_index_add(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, const aixhip_tensor* indices, size_t dim)
{ return guarded([&] { D(dev).indexAdd(P(src), P(dst), P(indices), dim); }); }

int32_t aixhip_empty_cache(aixhip_device* dev) { return guarded([&] { D(dev).emptyCache(); }); }
int32_t aixhip_synchronize(aixhip_device* dev) { return guarded([&] { D(dev).synchronize(); }); }
int32_t aixhip_flush(aixhip_device* dev) { return guarded([&] { D(dev).flush(); }); }
int32_t aixhip_copy_to_host(aixhip_device* dev, void* dst_host, const void* src_device, size_t bytes)
{ return guarded([&] { D(dev).copyToHost(dst_host, src_device, bytes); }); }
int32_t aixhip_copy_from_host(aixhip_device* dev, void* dst_device, const void* src_host, size_t bytes)
{ return guarded([&] { D(dev).copyFromHost(dst_device, src_host, bytes); }); }

int32_t aixhip_get_fuse_config(aixhip_device* dev, aixhip_fuse_config* out)
{
    return guarded([&] {
        if (!out) throw std::invalid_argument("null out pointer");
        const auto& c = D(dev).fuseConfig();
        *out = aixhip_fuse_config{c.elementwiseFusion, c.multiOutputKernels, c.absorbFills, c.diagnostics,
                                  c.flushThreshold, c.maxBufferSlots, c.supportsStridedFusion, !c.deferIdleFills};
    });
}

int32_t aixhip_set_fuse_config(aixhip_device* dev, const aixhip_fuse_config* cfg)
{
    return guarded([&] {
        if (!cfg) throw std::invalid_argument("null config");
        aixhip::fuse::FuseConfig c;
        c.elementwiseFusion = cfg->elementwise_fusion != 0;
        c.multiOutputKernels = cfg->multi_output_kernels != 0;
        c.absorbFills = cfg->absorb_fills != 0;
        c.diagnostics = cfg->diagnostics != 0;
        c.flushThreshold = cfg->flush_threshold ? cfg->flush_threshold : 1;
        c.maxBufferSlots = cfg->max_buffer_slots;
        c.supportsStridedFusion = cfg->supports_strided_fusion != 0;
        c.deferIdleFills = cfg->eager_idle_fills == 0;
        D(dev).setFuseConfig(c);
    });
}

int32_t aixhip_last_flush_diagnostics(aixhip_device* dev, aixhip_flush_diagnostics* out)
{
    return guarded([&] {
        if (!out) throw std::invalid_argument("null out pointer");
        const auto& d = D(dev).lastFlushDiagnostics();
        std::memset(out, 0, sizeof(*out));
        out->ops_recorded = d.opsRecorded; out->fusible_subgraphs = d.fusibleSubgraphs; out->fused_ops = d.fusedOps;
        out->fallback_ops = d.fallbackOps; out->dispatches_saved = d.dispatchesSaved; out->fills_absorbed = d.fillsAbsorbed;
        out->kernel_cache_hits = d.kernelCacheHits; out->kernel_cache_misses = d.kernelCacheMisses;
        std::snprintf(out->subgraph_summary, sizeof(out->subgraph_summary), "%s", d.subgraphSummary.c_str());
        std::snprintf(out->fallback_summary, sizeof(out->fallback_summary), "%s", d.fallbackSummary.c_str());
    });
}

int32_t aixhip_capture_begin(aixhip_device* dev) { return guarded([&] { D(dev).beginCapture(); }); }
int32_t aixhip_capture_end(aixhip_device* dev, aixhip_graph** out)
{
    return guarded([&] {
        if (!out) throw std::invalid_argument("aixhip_capture_end: null out pointer");
        *out = reinterpret_cast<aixhip_graph*>(D(dev).endCapture());
    });
}
int32_t aixhip_capture_abort(aixhip_device* dev) { return guarded([&] { D(dev).abortCapture(); }); }
int32_t aixhip_graph_replay(aixhip_device* dev, aixhip_graph* graph) { return guarded([&] { D(dev).replay(reinterpret_cast<DeviceHIP::StepGraph*>(graph)); }); }
int32_t aixhip_graph_destroy(aixhip_device* dev, aixhip_graph* graph) { return guarded([&] { D(dev).destroyGraph(reinterpret_cast<DeviceHIP::StepGraph*>(graph)); }); }
int32_t aixhip_set_cache_limit(aixhip_device* dev, uint64_t bytes) { return guarded([&] { D(dev).setCacheLimit((size_t)bytes); }); }
int32_t aixhip_batched_launch_stats(aixhip_device* dev, uint64_t* launches, uint64_t* kernels)
{
    return guarded([&] {
        const auto s = D(dev).batchedLaunchStats();
        if (launches) *launches = s.first;
        if (kernels) *kernels = s.second;
    });
}

int32_t aixhip_fuse_kernel_cache_stats(aixhip_device* dev, uint64_t* hits, uint64_t* misses)
{
    return guarded([&] {
        const auto s = D(dev).fuseKernelCacheStats();
        if (hits) *hits = s.first;
        if (misses) *misses = s.second;
    });
}

aixk_ctx* aixhip_kernel_context(aixhip_device* dev) { return dev ? dev->impl.kernelContext() : nullptr; }

int32_t aixhip_memory_stats(aixhip_device* dev, uint64_t* live_bytes, uint64_t* cached_bytes)
{
    return guarded([&] {
        if (live_bytes) *live_bytes = D(dev).allocatedBytes();
        if (cached_bytes) *cached_bytes = D(dev).cachedBytes();
    });
}

} // extern "C"
