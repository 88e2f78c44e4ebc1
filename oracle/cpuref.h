/*
 * cpuref.h -- CPU oracle for the AIX device operator set.
 *
 * TEST INFRASTRUCTURE ONLY.  This library restates, on the host CPU, what the
 * reference's single-threaded CPU device computes for every operator of the
 * aix::Device interface (Targets/AIXLib/aixDeviceCPU.cpp).  Only the tests,
 * the smoke check and the benchmark's cpu_baseline leg may load it; the
 * product (libaixhip / libaixdevice) never links or calls it.
 *
 * All entry points are plain C, take POD tensor descriptors and return 0 on
 * success, CPUREF_EINVAL where the reference throws std::invalid_argument.
 *
 * Parity pinning status (which check pins which function) is listed at the
 * top of cpuref.cpp.
 */
#ifndef AIX_ORACLE_CPUREF_H
#define AIX_ORACLE_CPUREF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CPUREF_MAX_RANK 16
#define CPUREF_OK       0
#define CPUREF_EINVAL   1

/* Element types, numbered as aix::DataType (Targets/AIXLib/aixCore.hpp:44-55). */
enum cpuref_dtype {
    CPUREF_F64 = 0, CPUREF_F32 = 1, CPUREF_F16 = 2, CPUREF_BF16 = 3,
    CPUREF_I64 = 4, CPUREF_I32 = 5, CPUREF_I16 = 6, CPUREF_I8 = 7, CPUREF_U8 = 8,
    CPUREF_DTYPE_COUNT = 9
};

/* Binary layout identical to aixhip_tensor (include/aixhip.h); mirrors
 * aix::DeviceTensorParams (Targets/AIXLib/aixCore.hpp:189-198).  offset, size,
 * shape and strides count elements, not bytes; stride 0 means broadcast. */
typedef struct cpuref_tensor {
    void*    data;
    int32_t  dtype;
    int32_t  rank;
    uint64_t offset;
    uint64_t size;
    uint64_t shape[CPUREF_MAX_RANK];
    uint64_t strides[CPUREF_MAX_RANK];
} cpuref_tensor;

enum cpuref_binary_op { CPUREF_ADD = 0, CPUREF_SUB = 1, CPUREF_MUL = 2, CPUREF_DIV = 3, CPUREF_POW = 4 };
enum cpuref_unary_op  { CPUREF_NEG = 0, CPUREF_SQRT = 1, CPUREF_SIN = 2, CPUREF_COS = 3,
                        CPUREF_TANH = 4, CPUREF_LOG = 5, CPUREF_EXP = 6 };

size_t cpuref_dtype_size(int dtype);

/* ---- literal restatement of the reference CPU device ------------------- */
int cpuref_binary(int op, const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out);
int cpuref_unary(int op, const cpuref_tensor* a, const cpuref_tensor* out);
int cpuref_fill(const void* scalar, int scalar_dtype, const cpuref_tensor* out);
int cpuref_fill_min(const cpuref_tensor* out);
int cpuref_copy(const void* src, int src_dtype, void* dst, int dst_dtype, uint64_t n);
int cpuref_contiguous(const cpuref_tensor* src, const cpuref_tensor* dst);
int cpuref_transpose(const cpuref_tensor* a, const cpuref_tensor* out, uint64_t dim0, uint64_t dim1);
int cpuref_sum(const cpuref_tensor* a, const cpuref_tensor* out);
int cpuref_max(const cpuref_tensor* a, const cpuref_tensor* out);
int cpuref_argmax(const cpuref_tensor* a, const cpuref_tensor* out);
int cpuref_argmax_indices(const cpuref_tensor* a, const cpuref_tensor* out);
int cpuref_reduce_to(const cpuref_tensor* src, const cpuref_tensor* dst);
int cpuref_max_to(const cpuref_tensor* src, const cpuref_tensor* dst);
int cpuref_argmax_to(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim);
int cpuref_argmax_indices_to(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim);
int cpuref_matmul(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out);
/* honor_dst_offset = 0 follows the CPU device (ignores dst->offset); 1 follows the
 * reference GPU device, which adds it (the only variant the reference tests). */
int cpuref_slice_set(const cpuref_tensor* src, const cpuref_tensor* dst, uint64_t dim,
                     uint64_t start, uint64_t end, uint64_t step, int honor_dst_offset);
int cpuref_tril(const cpuref_tensor* src, const cpuref_tensor* dst, int64_t diagonal);
int cpuref_triu(const cpuref_tensor* src, const cpuref_tensor* dst, int64_t diagonal);
/* strided_indices = 0 reads the index tensor flat as the CPU device does; 1 applies
 * its offset and strides as the reference GPU device does. */
int cpuref_index_select(const cpuref_tensor* src, const cpuref_tensor* dst,
                        const cpuref_tensor* indices, uint64_t dim, int strided_indices);
int cpuref_index_add(const cpuref_tensor* src, const cpuref_tensor* dst,
                     const cpuref_tensor* indices, uint64_t dim, int strided_indices);

/* ---- accuracy oracles (not in the reference; exact-accumulation truth) -- */
/* Sum of all elements accumulated in long double; also returns sum of |x|. */
int cpuref_sum_wide(const cpuref_tensor* a, double* sum_out, double* abs_sum_out);
/* dst64[t(i)] += src[i] accumulated in double; abs64 (may be NULL) gets sum |src|.
 * dst_like gives the destination shape; dst64/abs64 hold dst_like->size doubles. */
int cpuref_reduce_to_wide(const cpuref_tensor* src, const cpuref_tensor* dst_like, double* dst64, double* abs64);
/* C = A.B with every product and the running sum in double; out64 is m*n doubles.
 * abs64 (may be NULL) gets sum_k |a_ik||b_kj|.  Multi-threaded over rows. */
int cpuref_matmul_wide(const cpuref_tensor* a, const cpuref_tensor* b, double* out64, double* abs64, int threads);
/* Same arithmetic, operand order and rounding as cpuref_matmul (accumulator of the
 * element type, k ascending) with rows spread over threads; bit-identical to it. */
int cpuref_matmul_rows(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads);
/* Not in the reference (its matmul is 2-D only, aixCore.hpp:943-976): a, b, out of one rank above 2 with
 * the same leading dims; cpuref_matmul_rows on the matrices of every leading index in turn, results
 * dense from out->data.  Pinned by that function and, for the indexing of the stack, by integer
 * stacks against numpy.matmul (tests/test_oracle_golden.py). */
int cpuref_matmul_stack(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads);
/* Not in the reference either: the same products (rank 2 or stacks) with every result element added exactly
 * (cpuref_matmul_wide) and rounded ONCE to the element type by cpuref_copy's conversion -- what a device that keeps
 * 16-bit products in a wide accumulator computes, where the reference keeps the running sum in the element type
 * (aixDeviceCPU.cpp:362-389).  Pinned through the two functions it is composed of and, for the composition, against
 * float64 numpy products rounded once (tests/test_oracle_wide.py). */
int cpuref_matmul_stack_wide(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out, int threads);

/* ---- helpers for tests --------------------------------------------------- */
/* Distance in units in the last place between two f32 arrays: returns the maximum,
 * writes a histogram of min(distance, nbins-1).  NaN pairs count as distance 0,
 * a NaN against a number counts as nbins-1. */
uint64_t cpuref_ulp_hist_f32(const float* x, const float* y, uint64_t n, uint64_t* hist, int nbins);

#ifdef __cplusplus
}
#endif
#endif
