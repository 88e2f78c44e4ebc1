/*
 * aixhip_kernels.h -- the thin C ABI between host C++ and the gfx950 kernels.
 *
 * libaixhip_kernels.so (built by hipcc from aix_amd/csrc/hip) exports exactly these
 * symbols.  It is the only code in the project that includes HIP headers.  The host-side
 * device class (DeviceHIP, libaixhip.so) is plain C++20 and talks to the GPU only through
 * this file: plain pointers, sizes and POD descriptors, no C++ types, no torch types.
 *
 * Every launcher is EAGER and ASYNCHRONOUS: it validates its operands on the host, enqueues
 * its kernels on the context's single in-order stream and returns.  Nothing blocks except
 * aixk_sync, aixk_copy_out and aixk_event_elapsed_ms.  Status: 0 = ok, AIXK_EINVAL = contract
 * violation (the reference throws std::invalid_argument there), AIXK_ENOMEM = allocation
 * failure (std::runtime_error in the reference), AIXK_EHIP = a HIP call failed.
 * aixk_last_error() returns the message for the last non-zero status on the calling thread.
 *
 * Operand semantics follow the reference CPU device (Targets/AIXLib/aixDeviceCPU.cpp):
 * results are written contiguously from result->data (result offset/strides ignored) unless
 * stated otherwise; inputs are arbitrary views (offset + strides, stride 0 = broadcast).
 * All tensor memory must be device memory obtained from aixk_alloc on the same context.
 */
#ifndef AIXHIP_KERNELS_H
#define AIXHIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AIXK_MAX_RANK 16

#define AIXK_OK      0
#define AIXK_EINVAL  1
#define AIXK_ENOMEM  2
#define AIXK_EHIP    3

/* Results of at least this many bytes are written with non-temporal (streaming) stores; smaller ones stay in cache
 * for the kernel that reads them next.  The environment variable AIXHIP_STREAM_STORE_MIN_BYTES overrides it. */
#define AIXK_STREAM_STORE_MIN_BYTES (32ull << 20)

/* Element types, numbered as aix::DataType (Targets/AIXLib/aixCore.hpp:44-55). */
enum aixk_dtype {
    AIXK_F64 = 0, AIXK_F32 = 1, AIXK_F16 = 2, AIXK_BF16 = 3,
    AIXK_I64 = 4, AIXK_I32 = 5, AIXK_I16 = 6, AIXK_I8 = 7, AIXK_U8 = 8,
    AIXK_DTYPE_COUNT = 9
};

/* POD image of aix::DeviceTensorParams (Targets/AIXLib/aixCore.hpp:189-198).
 * offset / size / shape / strides count elements. */
typedef struct aixhip_tensor {
    void*    data;
    int32_t  dtype;
    int32_t  rank;
    uint64_t offset;
    uint64_t size;
    uint64_t shape[AIXK_MAX_RANK];
    uint64_t strides[AIXK_MAX_RANK];
} aixhip_tensor;

typedef struct aixk_ctx aixk_ctx;        /* one GPU, one in-order stream, scratch, JIT cache */
typedef struct aixk_module aixk_module;  /* a runtime-compiled fused kernel */
typedef struct aixk_event aixk_event;

typedef struct aixk_device_info {
    char     name[128];
    char     arch[64];
    int32_t  compute_units;
    int32_t  clock_khz;
    int32_t  large_bar;          /* 1 if device memory is host-addressable */
    int32_t  wavefront;
    uint64_t total_mem;
    uint64_t lds_per_block;
} aixk_device_info;

const char* aixk_last_error(void);
size_t      aixk_dtype_size(int dtype);                 /* aix::Device::dataTypeSize, aixDeviceCPU.cpp:685-700 */

/* ---- context, memory, ordering (aixDevice.hpp:40-42, 82-83) ------------- */
int32_t aixk_create(int device_index, aixk_ctx** out);
int32_t aixk_destroy(aixk_ctx* ctx);
int32_t aixk_info(aixk_ctx* ctx, aixk_device_info* out);
/* kind: 0 = device memory (hipMalloc), 1 = managed memory preferring the device,
 *       2 = pinned host memory.  Sizes are padded to a multiple of 256 bytes. */
int32_t aixk_alloc(aixk_ctx* ctx, size_t bytes, int kind, void** out);
int32_t aixk_free(aixk_ctx* ctx, void* ptr, int kind);             /* caller has synchronised */
int32_t aixk_copy_in(aixk_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);   /* stream-ordered; host buffer reusable on return */
int32_t aixk_copy_out(aixk_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);  /* waits for the stream, then copies */
int32_t aixk_copy_dev(aixk_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);
int32_t aixk_zero(aixk_ctx* ctx, void* dst_dev, size_t bytes);
int32_t aixk_sync(aixk_ctx* ctx);                                  /* Device::synchronize, aixDevice.hpp:83 */

/* ---- elementwise (aixDevice.hpp:44-48, 53-59) --------------------------- */
enum aixk_binary_op { AIXK_ADD = 0, AIXK_SUB = 1, AIXK_MUL = 2, AIXK_DIV = 3, AIXK_POW = 4 };
enum aixk_unary_op  { AIXK_NEG = 0, AIXK_SQRT = 1, AIXK_SIN = 2, AIXK_COS = 3, AIXK_TANH = 4, AIXK_LOG = 5, AIXK_EXP = 6 };
/* out[i] = a[view(i)] op b[view(i)], i < out->size (pow: i < a->size); element type = out->dtype.
 * Replaces Device::add/sub/mul/div/pow (aixDeviceCPU.cpp:28-82, 229-242). */
int32_t aixk_binary(aixk_ctx* ctx, int op, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out);
/* out[i] = f(a[view(i)]), i < a->size.  Replaces Device::unary/sqrt/sin/cos/tanh/log/exp
 * (aixDeviceCPU.cpp:84-94, 154-227). */
int32_t aixk_unary(aixk_ctx* ctx, int op, const aixhip_tensor* a, const aixhip_tensor* out);
/* Device::fill / fillMin (aixDeviceCPU.cpp:119-138): scalar is HOST memory of scalar_dtype. */
int32_t aixk_fill(aixk_ctx* ctx, const void* scalar, int scalar_dtype, const aixhip_tensor* out);
int32_t aixk_fill_min(aixk_ctx* ctx, const aixhip_tensor* out);
/* `count` small fills in one launch (the rank-0 constants of an expression, `tensor op scalar` of
 * aixCore.hpp:2384-2438, are filled one Device::fill each): item k writes `elements` copies of the low `element_size`
 * bytes of `bits` -- the value already in the destination's element type -- from `dst` on.  AIXK_EINVAL for an
 * element size other than 1, 2, 4, 8 or more than 65536 elements in one item. */
typedef struct aixk_fill_item { void* dst; uint64_t bits; uint32_t elements; uint32_t element_size; } aixk_fill_item;
int32_t aixk_fill_many(aixk_ctx* ctx, const aixk_fill_item* items, uint32_t count);
/* Device::copy (aixDeviceCPU.cpp:407-423): flat converting copy of n elements, both device memory. */
int32_t aixk_cast(aixk_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype, uint64_t n);

/* ---- data movement (aixDevice.hpp:64, 68, 73-80) ------------------------ */
int32_t aixk_contiguous(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst);      /* aixDeviceCPU.cpp:425-438 */
int32_t aixk_transpose(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* out, uint64_t dim0, uint64_t dim1); /* :391-405 */
/* dst is addressed through its offset and strides (the reference GPU device's behaviour). */
int32_t aixk_slice_set(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                       uint64_t dim, uint64_t start, uint64_t end, uint64_t step);                /* :468-496 */
/* `count` sliceSet calls in one launch (the parts of a cat(), aixCore.hpp:1348-1402, and the windows the backward pass
 * of slices writes, :2228-2233, arrive as runs of Device::sliceSet calls that do not depend on one another): item k is
 * aixk_slice_set(src, dst, dim, start, end, step) of its fields.  All items have one element size; the caller
 * guarantees that no item reads or overwrites what another one writes.  AIXK_EINVAL for more than
 * AIXK_SLICE_ITEMS_MAX items, an empty item, or an item aixk_slice_set would reject; nothing is launched then.
 * No counterpart in the reference's interface (one Device::sliceSet call per part there). */
#define AIXK_SLICE_ITEMS_MAX 512
typedef struct aixk_slice_item { aixhip_tensor src, dst; uint64_t dim, start, end, step; } aixk_slice_item;
int32_t aixk_slice_set_many(aixk_ctx* ctx, const aixk_slice_item* items, uint32_t count);
/* The same with the destination's initialisation folded in: dst (dense, offset 0) is written exactly once --
 * `init_bits` (a value of its element type in the low bytes) outside the slice, src inside.  It is what
 * fill(v) followed by sliceSet computes (the backward of a slice: zeros of the input's shape, then the
 * gradient set into the slice, aixCore.hpp:1200-1203, 2237-2241) without the separate fill pass over dst. */
int32_t aixk_slice_set_init(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                            uint64_t dim, uint64_t start, uint64_t end, uint64_t step, uint64_t init_bits);
int32_t aixk_tri(aixk_ctx* ctx, int upper, const aixhip_tensor* src, const aixhip_tensor* dst, int64_t diagonal); /* :566-622 */
/* indices: int32, addressed through their own offset and strides. */
int32_t aixk_index_select(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                          const aixhip_tensor* indices, uint64_t dim);                           /* :498-530 */
int32_t aixk_index_add(aixk_ctx* ctx, const aixhip_tensor* src, const aixhip_tensor* dst,
                       const aixhip_tensor* indices, uint64_t dim);                              /* :532-564 */

/* ---- reductions (aixDevice.hpp:52, 60-62, 69-72) ------------------------ */
enum aixk_reduce_kind { AIXK_SUM = 0, AIXK_MAX = 1, AIXK_ARGMAX = 2, AIXK_ARGMAX_ONEHOT = 3 };
/* Whole-tensor reduction into a rank-0 result: Device::sum/max/argmax/argmaxIndices
 * (aixDeviceCPU.cpp:140-152, 244-318).  ARGMAX kinds need an int32 result. */
int32_t aixk_reduce_all(aixk_ctx* ctx, int kind, const aixhip_tensor* a, const aixhip_tensor* out);
/* No counterpart in the reference: aixk_reduce_all for callers that cannot allocate (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  Same arguments; the partial results of the
 * workgroups go to a 64 KiB static device array instead of the context's pooled scratch, and no hipMalloc / hipFree /
 * allocating library call is made.  The launch is cut to the workgroups whose partials fit the array (4096 of 16
 * bytes): on parts of up to 256 compute units that is the launch of aixk_reduce_all and the results are the same bit
 * for bit; on larger parts 16-byte accumulators (f64 / i64 sums, argmax of 8-byte types) run on fewer workgroups, with
 * the same result for everything but float sums, whose partial sums are grouped differently.  Limit: at most 2^31
 * elements per call (AIXK_EINVAL beyond).  All calls on one GPU share the array: calls that overlap on one GPU race. */
int32_t aixk_reduce_all_noalloc(aixk_ctx* ctx, int kind, const aixhip_tensor* a, const aixhip_tensor* out);
/* dst (op)= reduction of src over the dims dst lacks: Device::reduceTo / maxTo
 * (aixDeviceCPU.cpp:440-466).  Accumulates INTO dst (caller pre-initialises). kind = SUM|MAX. */
int32_t aixk_reduce_to(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst);
/* The same with the pre-initialisation folded in: every dst element is taken to hold `init_bits`
 * (a value of dst's element type in the low bytes) and is written exactly once, never read.  It is
 * what fill(0) / fillMin() followed by reduceTo / maxTo computes (aixCore.hpp:632-639, 873-891)
 * without the separate fill pass over dst. */
int32_t aixk_reduce_to_init(aixk_ctx* ctx, int kind, const aixhip_tensor* src, const aixhip_tensor* dst, uint64_t init_bits);
/* The second half of a sum over all elements that a generated kernel began (a product that is only formed to be
 * summed -- the gradient of a scalar constant, aixCore.hpp:2384-2438 -- is summed where it is formed): `partials` holds
 * `count` partial sums in device memory, float for f32 / f16 / bf16 results and double for f64; the one-element dst
 * receives round(init + their sum), init being the value the destination was filled with (its bits in the low bytes of
 * init_bits), as aixk_reduce_to_init lands a sum.  No counterpart in the reference's interface. */
int32_t aixk_sum_partials(aixk_ctx* ctx, const void* partials, uint64_t count, const aixhip_tensor* dst, uint64_t init_bits);
/* `count` calls of aixk_sum_partials in one launch (item k is aixk_sum_partials(ctx, partials, count, dst, init_bits) of its
 * fields) when all destinations have one floating-point element type and there are at most AIXK_PARTIALS_ITEMS_MAX items,
 * otherwise item by item in order.  The caller guarantees that no item reads what another one writes.  No counterpart in
 * the reference's interface. */
#define AIXK_PARTIALS_ITEMS_MAX 1024
typedef struct aixk_partials_item { const void* partials; uint64_t count; aixhip_tensor dst; uint64_t init_bits; } aixk_partials_item;
int32_t aixk_sum_partials_many(aixk_ctx* ctx, const aixk_partials_item* items, uint32_t count);
/* Device::argmaxTo / argmaxIndicesTo (aixDeviceCPU.cpp:275-298, 320-360). onehot=1 scatters ones
 * into the pre-zeroed int32 dst of src's shape; onehot=2 also zeroes dst first (the fill(0) the
 * caller issues before argmaxIndicesTo, aixCore.hpp:927-941, folded in: over a handful of rows the
 * one-hot block is then written densely in a single pass). */
int32_t aixk_argmax_to(aixk_ctx* ctx, int onehot, const aixhip_tensor* src, const aixhip_tensor* dst, uint64_t dim);
/* `count` argmaxIndicesTo calls, each with the zero fill of its destination folded in (item k is
 * aixk_argmax_to(ctx, 2, src, dst, dim) of its fields): the masks that the backward pass of max() asks for head after
 * head (aixCore.hpp:927-941, 2170-2175).  One launch when every item is a dense tensor of one element type reduced along its
 * last dim (rows of at least 32 elements, a multiple of 4 and of 16 bytes) and there are at most AIXK_ARGMAX_ITEMS_MAX
 * items, otherwise item by item in order.  The caller guarantees that no item reads what another one writes.
 * No counterpart in the reference's interface (one Device::argmaxIndicesTo call per tensor there). */
#define AIXK_ARGMAX_ITEMS_MAX 1024
typedef struct aixk_argmax_item { aixhip_tensor src, dst; uint64_t dim; } aixk_argmax_item;
int32_t aixk_argmax_onehot_many(aixk_ctx* ctx, const aixk_argmax_item* items, uint32_t count);

/* `count` reduceTo calls that sum a dense matrix down its columns, each with the fill of its destination folded in
 * (item k is aixk_reduce_to_init(ctx, AIXK_SUM, src, dst, init_bits) of its fields): the gradients of biases and of
 * LayerNorm's parameters, which a backward pass asks for layer after layer (aixCore.hpp:2228-2233 sums a gradient to
 * its parameter's shape) and reads only when it reaches the parameters.  Two launches for all items when every item is a
 * dense f32, f16 or bf16 tensor of at least two rows whose last dim (a multiple of 4 elements) is the destination,
 * there are at most AIXK_COLSUM_ITEMS_MAX items and the partial sums fit the context's scratch memory; otherwise item by
 * item in order.  Sums are accumulated as aixk_reduce_to accumulates them and rounded once.  The caller guarantees
 * that no item reads what another one writes.  No counterpart in the reference's interface (one Device::reduceTo call
 * per tensor there). */
#define AIXK_COLSUM_ITEMS_MAX 1024
typedef struct aixk_colsum_item { aixhip_tensor src, dst; uint64_t init_bits; } aixk_colsum_item;
int32_t aixk_sum_columns_many(aixk_ctx* ctx, const aixk_colsum_item* items, uint32_t count);

/* ---- matmul (aixDevice.hpp:63; aixDeviceCPU.cpp:362-389) ---------------- */
/* out[m,n] = a[m,k] . b[k,n]; a, b arbitrary 2-D views; f32/f16/bf16 run on MFMA with f32
 * accumulation, other types on a generic tiled kernel with an accumulator of the element type
 * (f64 and integers). */
int32_t aixk_matmul(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out);
/* Diagnostic (no counterpart in the reference): how the last aixk_matmul on this context was computed.  Waits for the
 * stream.  *route = 1: an f32 product on the bf16 matrix pipe with every operand split into three bf16 planes, 0:
 * anything else.  *redone = 1: that product met an operand the planes cannot carry (an infinity, a NaN, a nonzero
 * magnitude at or below 2^-100) or an accumulator that overflowed, and was computed again in IEEE f32 arithmetic. */
int32_t aixk_matmul_route(aixk_ctx* ctx, int32_t* route, int32_t* redone);
/* An extension of the above: the reference multiplies 2-D operands only (aixCore.hpp:943-976), so an
 * AIX program issues attention as one matmul per (sequence, head) on sliced views.  Here a, b and out
 * may carry the same leading dims in front of the matrix dims: out[..., m, n] = a[..., m, k] . b[..., k, n],
 * one product per index of the leading dims, what the 2-D entry point computes for each (f32 accumulation,
 * one rounding; the order in which the f32 partial sums are added may differ from the 2-D route's).
 * a and b may be any views (permuted, sliced, stride 0); the results are written densely from
 * out->data.  Stacks of small 16-bit products run as ONE launch; everything else is issued product by
 * product through the 2-D entry point.  Rank 2 is the 2-D entry point. */
int32_t aixk_matmul_batched(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out);
/* `count` separate products -- a[i] . b[i] -> out[i], the descriptors in three arrays -- issued together: what a run of
 * Device::matmul calls on same-shaped operands asks for (aixCore.hpp:943-976 has no batch dimension, so attention over
 * (sequence, head) pairs arrives as such a run).  16-bit products of one shape and operand layout that do not fill the
 * chip one by one run as ONE launch; anything else one by one, with the result of aixk_matmul for every product. */
int32_t aixk_matmul_grouped(aixk_ctx* ctx, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint32_t count);

/* ---- runtime-compiled fused elementwise kernels ------------------------- */
/* Compile `source` (HIP C++, one extern "C" __global__ named `entry`) for gfx950 with hipRTC or
 * return the cached module for `key`.  *was_cached tells which.  Replaces the reference's
 * runtime shader compile + pipeline cache (aixDeviceMetalKernelGen.cpp:712-770). */
int32_t aixk_rtc_get(aixk_ctx* ctx, const char* key, const char* source, const char* entry,
                     aixk_module** out, int32_t* was_cached);
/* Launch with a packed kernel-argument block (aixDeviceMetalKernelGen.cpp:772-857). */
int32_t aixk_rtc_launch(aixk_ctx* ctx, aixk_module* mod, uint32_t grid_x, uint32_t block_x,
                        const void* args, size_t args_bytes);
/* One launch for `count` argument blocks of one kernel body.  The module's entry must have the form
 * `extern "C" __global__ void f(const Args* table, const uint32_t* starts, uint32_t count)`: `table` (host memory here,
 * `table_bytes` of it) holds the `count` argument blocks back to back and, `starts_offset` bytes in, count + 1 uint32 --
 * the first workgroup of every block's share of the grid and, last, the grid size.  The table is copied to device
 * memory in stream order; the host's copy may be reused as soon as the call returns.  AIXK_EINVAL if the table exceeds
 * 256 KiB or the shares are not in ascending order.  No counterpart in the reference, whose Adam updates one parameter
 * per dispatch (aixOptimizer.hpp:112-140). */
int32_t aixk_rtc_launch_many(aixk_ctx* ctx, aixk_module* mod, uint32_t block_x, const void* table, size_t table_bytes,
                             size_t starts_offset, uint32_t count);
/* The device-side header every generated kernel is compiled against (types, conversions, math). */
const char* aixk_rtc_prelude(void);
int32_t aixk_rtc_stats(aixk_ctx* ctx, uint64_t* hits, uint64_t* misses);
/* No counterpart in the reference (its kernel cache lives in memory and every process compiles its generated kernels
 * anew, aixDeviceMetalKernelGen.cpp:716-768): with AIXHIP_KERNEL_CACHE_DIR set when the context is created, the
 * code object of every kernel aixk_rtc_get compiles is also kept in that directory, named by a hash of the device header,
 * the source, the target, the compiler's options and version, and a later context (or process) loads it instead of
 * compiling.  A missing, damaged or unloadable file means a compilation, never an error.  loaded / stored: how many code
 * objects this context took from / wrote to the directory. */
int32_t aixk_rtc_disk_stats(aixk_ctx* ctx, uint64_t* loaded, uint64_t* stored);

/* ---- a stretch of the stream as a HIP graph (no counterpart in the reference, whose GPU device amortises dispatch by
 * batching into command buffers, aixDeviceMetal.cpp:1344-1389) ------------------------------------------------------ */
/* Between aixk_capture_begin and aixk_capture_end nothing that is enqueued on the context runs: it is recorded, and
 * aixk_graph_launch enqueues all of it again with one call, on the same addresses with the same arguments.  Inside a
 * capture: no aixk_sync, no event, no transfer to or from host memory (status AIXK_EHIP from the driver); kernels must
 * have been compiled and workspaces grown by an earlier, uncaptured run of the same work.  The argument tables of
 * launches that carry several calls are written when they are captured and kept with the graph; no memset and no copy
 * node enters a graph through this library except device-to-device copies the caller asks for. */
typedef struct aixk_graph aixk_graph;
int32_t aixk_capture_begin(aixk_ctx* ctx);                       /* waits for the stream first */
int32_t aixk_capture_end(aixk_ctx* ctx, aixk_graph** out);
int32_t aixk_capture_abort(aixk_ctx* ctx);                       /* drops an open capture; harmless without one */
int32_t aixk_graph_launch(aixk_ctx* ctx, aixk_graph* graph);
int32_t aixk_graph_nodes(aixk_graph* graph, uint64_t* nodes);
int32_t aixk_graph_destroy(aixk_ctx* ctx, aixk_graph* graph);    /* waits for the stream first */

/* ---- the matrix pipe alone (no counterpart in the reference; a measurement aid) ---------------------------------- */
/* A loop of independent 16-bit MFMAs on register operands, no LDS and no memory traffic, one workgroup per compute unit:
 * the rate the part sustains when it only multiplies -- on a power-limited part a function of the operand values, of the
 * instruction and of the waves per SIMD -- against which a GEMM's fraction of the nominal peak is read.  shape 0: four
 * waves, 4 x 4 tiles of v_mfma_f32_32x32x16 each; shape 1: eight waves, 8 x 4 tiles of v_mfma_f32_16x16x32 each (the
 * register layout of the 256 x 256 GEMM kernel).  dtype AIXK_BF16 or AIXK_F16; `operands`: `count` 16-bit patterns used
 * round-robin as operand values; about `gflop_per_launch` GFLOP per launch, 200 untimed and 280 timed launches on the
 * context's stream.  *tflops: the median rate; *ghz: the shader clock held during the loop. */
int32_t aixk_mfma_only_rate(aixk_ctx* ctx, int32_t shape, int32_t dtype, const uint16_t* operands, uint32_t count, double gflop_per_launch,
                            float* tflops, float* ghz);

/* ---- timing on the context's stream ------------------------------------- */
int32_t aixk_event_create(aixk_ctx* ctx, aixk_event** out);
int32_t aixk_event_record(aixk_ctx* ctx, aixk_event* ev);
int32_t aixk_event_query(aixk_ctx* ctx, aixk_event* ev, int32_t* done);              /* never waits */
int32_t aixk_event_elapsed_ms(aixk_ctx* ctx, aixk_event* start, aixk_event* stop, float* ms); /* waits for stop */
int32_t aixk_event_destroy(aixk_ctx* ctx, aixk_event* ev);

#ifdef __cplusplus
}
#endif
#endif
