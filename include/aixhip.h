/*
 * aixhip.h -- C ABI of the MI355X device backend: one entry point per method of the AIX device
 * plug-in interface, aix::Device (Targets/AIXLib/aixDevice.hpp:30-84).
 *
 * libaixhip.so implements these on top of the C++ class aix::hip::DeviceHIP (which C++ users of
 * AIX plug in directly, exactly as they plug in the reference GPU device, README.MD:166-188).
 * The C ABI exists for every other binding (ctypes, cgo, JNI, ...): plain pointers, sizes and the
 * POD descriptor `aixhip_tensor`, which is the image of aix::DeviceTensorParams
 * (Targets/AIXLib/aixCore.hpp:189-198).  Each declaration cites the virtual it stands for.
 *
 * Semantics are those of a lazy GPU device (Targets/AIXLib/aixDeviceMetal.cpp): calls may return
 * before the work ran; program order is preserved; results are defined after
 * aixhip_synchronize().  Elementwise operators and fills are recorded and fused into runtime
 * compiled kernels.  Results must live in memory from aixhip_allocate on the same device; inputs
 * may also be host memory.
 *
 * Status codes: 0 ok; AIXHIP_EINVAL where the reference throws std::invalid_argument;
 * AIXHIP_ERUNTIME where it throws std::runtime_error (allocation failure, GPU error).
 * aixhip_last_error() gives the message of the last failure on the calling thread.
 * A device is used from one thread at a time (as aix::Device implementations are).
 */
#ifndef AIXHIP_H
#define AIXHIP_H

#include "aixhip_kernels.h"   /* aixhip_tensor, aixk_dtype, aixk_ctx */

#ifdef __cplusplus
extern "C" {
#endif

#define AIXHIP_OK        0
#define AIXHIP_EINVAL    1
#define AIXHIP_ERUNTIME  2

typedef struct aixhip_device aixhip_device;

const char* aixhip_last_error(void);

/* createDevice(type, index): Targets/AIXLib/aixDevices.cpp:24-43.  Fails (AIXHIP_ERUNTIME) if no GPU is visible. */
int32_t aixhip_device_create(int device_index, aixhip_device** out);
int32_t aixhip_device_destroy(aixhip_device* dev);
/* Device::type / Device::name: aixDevice.hpp:35-36.  type is 2 (the value after kGPU_METAL), name "HIP". */
int32_t     aixhip_type(const aixhip_device* dev);
const char* aixhip_name(const aixhip_device* dev);
/* Device::dataTypeSize: aixDevice.hpp:38 */
size_t aixhip_data_type_size(int dtype);

/* Device::allocate(size) / allocate(size, dtype) / deallocate: aixDevice.hpp:40-42 */
int32_t aixhip_allocate(aixhip_device* dev, size_t bytes, void** out);
int32_t aixhip_allocate_typed(aixhip_device* dev, size_t count, int dtype, void** out);
int32_t aixhip_deallocate(aixhip_device* dev, void* memory);

/* Device::add / sub / mul / div / unary(negate): aixDevice.hpp:44-48 */
int32_t aixhip_add(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* a2, const aixhip_tensor* result);
int32_t aixhip_sub(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* a2, const aixhip_tensor* result);
int32_t aixhip_mul(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* a2, const aixhip_tensor* result);
int32_t aixhip_div(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* a2, const aixhip_tensor* result);
int32_t aixhip_unary(aixhip_device* dev, const aixhip_tensor* a1, const aixhip_tensor* result);

/* Device::fill / fillMin / sum: aixDevice.hpp:50-52 (scalar is host memory of scalar_dtype) */
int32_t aixhip_fill(aixhip_device* dev, const void* scalar, int scalar_dtype, const aixhip_tensor* result);
int32_t aixhip_fill_min(aixhip_device* dev, const aixhip_tensor* result);
int32_t aixhip_sum(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);

/* Device::sqrt / sin / cos / tanh / log / exp / pow: aixDevice.hpp:53-59 */
int32_t aixhip_sqrt(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_sin(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_cos(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_tanh(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_log(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_exp(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_pow(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* exp, const aixhip_tensor* result);

/* Device::max / argmax / argmaxIndices / matmul / transpose: aixDevice.hpp:60-64 */
int32_t aixhip_max(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_argmax(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
int32_t aixhip_argmax_indices(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result);
/* matmul: 2-D operands as in the reference; operands and result of the same rank above 2 are a stack of
 * products over their shared leading dims (an extension, see aixk_matmul_batched). */
int32_t aixhip_matmul(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* result);
int32_t aixhip_transpose(aixhip_device* dev, const aixhip_tensor* a, const aixhip_tensor* result, size_t dim0, size_t dim1);

/* Device::copy / copyImmediate / contiguous: aixDevice.hpp:66-68 */
int32_t aixhip_copy(aixhip_device* dev, const void* src, int src_dtype, void* dst, int dst_dtype, size_t size);
int32_t aixhip_copy_immediate(aixhip_device* dev, const void* src, int src_dtype, void* dst, int dst_dtype, size_t size);
int32_t aixhip_contiguous(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst);

/* Device::reduceTo / maxTo / argmaxTo / argmaxIndicesTo: aixDevice.hpp:69-72 */
int32_t aixhip_reduce_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst);
int32_t aixhip_max_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst);
int32_t aixhip_argmax_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, size_t dim);
int32_t aixhip_argmax_indices_to(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, size_t dim);

/* Device::sliceSet / tril / triu / indexSelect / indexAdd: aixDevice.hpp:73-80 */
int32_t aixhip_slice_set(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst,
                         size_t dim, size_t start, size_t end, size_t step);
int32_t aixhip_tril(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal);
int32_t aixhip_triu(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal);
int32_t aixhip_index_select(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst,
                            const aixhip_tensor* indices, size_t dim);
int32_t aixhip_index_add(aixhip_device* dev, const aixhip_tensor* src, const aixhip_tensor* dst,
                         const aixhip_tensor* indices, size_t dim);

/* Device::emptyCache / synchronize: aixDevice.hpp:82-83 */
int32_t aixhip_empty_cache(aixhip_device* dev);
int32_t aixhip_synchronize(aixhip_device* dev);

/* ---- beyond aix::Device: what the reference exposes on its GPU device class for tests and tools ---- */
/* Plan and enqueue what has been recorded, without waiting. */
int32_t aixhip_flush(aixhip_device* dev);
/* Explicit transfers (the host may also dereference device pointers where the BAR mapping allows). */
int32_t aixhip_copy_to_host(aixhip_device* dev, void* dst_host, const void* src_device, size_t bytes);
int32_t aixhip_copy_from_host(aixhip_device* dev, void* dst_device, const void* src_host, size_t bytes);

/* FuseConfig (Targets/AIXLib/aixFuse.hpp:90-99). */
typedef struct aixhip_fuse_config {
    int32_t  elementwise_fusion;
    int32_t  multi_output_kernels;
    int32_t  absorb_fills;
    int32_t  diagnostics;
    uint64_t flush_threshold;
    uint64_t max_buffer_slots;
    int32_t  supports_strided_fusion;
    int32_t  eager_idle_fills;        /* 1: a fill nothing in its window uses runs at once; 0 (default): it waits for its
                                         first user or the next synchronize / flush and is usually absorbed there */
} aixhip_fuse_config;
int32_t aixhip_get_fuse_config(aixhip_device* dev, aixhip_fuse_config* out);
int32_t aixhip_set_fuse_config(aixhip_device* dev, const aixhip_fuse_config* cfg);

/* FlushDiagnostics of the last flush (aixFuse.hpp:144-156); filled only if diagnostics is on. */
typedef struct aixhip_flush_diagnostics {
    uint64_t ops_recorded, fusible_subgraphs, fused_ops, fallback_ops, dispatches_saved, fills_absorbed;
    uint64_t kernel_cache_hits, kernel_cache_misses;
    char     subgraph_summary[256];
    char     fallback_summary[128];
} aixhip_flush_diagnostics;
int32_t aixhip_last_flush_diagnostics(aixhip_device* dev, aixhip_flush_diagnostics* out);
/* DeviceMetal::fuseKernelCacheStats (Targets/AIXTests/DeviceTests.cpp:1774-1807). */
int32_t aixhip_fuse_kernel_cache_stats(aixhip_device* dev, uint64_t* hits, uint64_t* misses);
/* Launches that carried several generated kernels of one signature at once (Adam's update of parameter after parameter
 * as one launch), and how many kernels they carried, since the device was created.  No counterpart in the reference. */
int32_t aixhip_batched_launch_stats(aixhip_device* dev, uint64_t* launches, uint64_t* kernels);
/* The kernel-layer context of this device (stream, events) for timing with aixk_event_*. */
aixk_ctx* aixhip_kernel_context(aixhip_device* dev);
/* A stretch of the device's work as a HIP graph (no counterpart in the reference, whose GPU device amortises dispatch by
 * batching into command buffers, aixDeviceMetal.cpp:1344-1389): what is issued between capture_begin and capture_end is
 * recorded, not run, and aixhip_graph_replay enqueues all of it again -- the same kernels on the same addresses with the
 * same immediates -- with one call, for steps that repeat exactly (a forward + backward pass, updates in place).  Inside
 * a capture: no synchronize, no transfer to or from host memory, nothing compiled or grown for the first time (run the
 * step once before capturing it): status 2.  Blocks that captured work uses stay with the graph: freed, they are not
 * handed out again until the last graph is destroyed; live tensors are used in place by every replay. */
typedef struct aixhip_graph aixhip_graph;
int32_t aixhip_capture_begin(aixhip_device* dev);
int32_t aixhip_capture_end(aixhip_device* dev, aixhip_graph** out);
/* Gives an open capture up -- after an error inside it, say: nothing of it runs, its results are undefined, the device is
 * usable again.  Without an open capture: nothing. */
int32_t aixhip_capture_abort(aixhip_device* dev);
int32_t aixhip_graph_replay(aixhip_device* dev, aixhip_graph* graph);
int32_t aixhip_graph_destroy(aixhip_device* dev, aixhip_graph* graph);
int32_t aixhip_memory_stats(aixhip_device* dev, uint64_t* live_bytes, uint64_t* cached_bytes);
/* The pool of idle blocks is cut back to `bytes` at every synchronize (the reference's GPU device trims its buffer cache
 * to its working-set limit at every commit, aixDeviceMetal.cpp:33, 1369-1373).  Default 0.7 of the card's memory;
 * environment override AIXHIP_CACHE_LIMIT_BYTES. */
int32_t aixhip_set_cache_limit(aixhip_device* dev, uint64_t bytes);

#ifdef __cplusplus
}
#endif
#endif
