// ref_shim.cpp -- C entry points around the reference's own aix::DeviceCPU.
//
// TEST INFRASTRUCTURE ONLY.  Built only where the reference tree is present (see
// oracle/Makefile, target `ref`): this file is compiled together with the reference's
// aixDeviceCPU.cpp / aixDevices.cpp *from where they lie*; nothing of the reference is
// copied.  The result, oracle/_ref/libaixref.so, lets the tests compare the restatement
// in cpuref.cpp with the real thing bit for bit, and lets the benchmark time the
// reference CPU path itself.
//
// The entry points take the same POD descriptor as cpuref.h and forward to the virtual
// methods of aix::Device (Targets/AIXLib/aixDevice.hpp:30-84) on a DeviceCPU instance.

#include "cpuref.h"

#include <aix.hpp>

#include <stdexcept>

namespace {

aix::DeviceCPU& dev()
{
    static aix::DeviceCPU d;
    return d;
}

aix::DeviceTensorParams P(const cpuref_tensor* t)
{
    aix::DeviceTensorParams p;
    p.data = t->data;
    p.dtype = static_cast<aix::DataType>(t->dtype);
    p.offset = t->offset;
    p.size = t->size;
    p.shape.assign(t->shape, t->shape + t->rank);
    p.strides.assign(t->strides, t->strides + t->rank);
    // contiguity flag as TensorValue would compute it: row-major strides
    bool c = true; size_t run = 1;
    for (int d = t->rank - 1; d >= 0; --d) { if (t->strides[d] != run) c = false; run *= t->shape[d]; }
    p.isContiguous = c;
    return p;
}

template <class F> int guarded(F&& f)
{
    try { f(); return CPUREF_OK; }
    catch (const std::invalid_argument&) { return CPUREF_EINVAL; }
}

} // namespace

extern "C" {

int aixref_binary(int op, const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* out)
{
    return guarded([&] {
        switch (op) {
            case CPUREF_ADD: dev().add(P(a), P(b), P(out)); break;
            case CPUREF_SUB: dev().sub(P(a), P(b), P(out)); break;
            case CPUREF_MUL: dev().mul(P(a), P(b), P(out)); break;
            case CPUREF_DIV: dev().div(P(a), P(b), P(out)); break;
            case CPUREF_POW: dev().pow(P(a), P(b), P(out)); break;
            default: throw std::invalid_argument("op");
        }
    });
}

int aixref_unary(int op, const cpuref_tensor* a, const cpuref_tensor* out)
{
    return guarded([&] {
        switch (op) {
            case CPUREF_NEG:  dev().unary(P(a), P(out)); break;
            case CPUREF_SQRT: dev().sqrt(P(a), P(out)); break;
            case CPUREF_SIN:  dev().sin(P(a), P(out)); break;
            case CPUREF_COS:  dev().cos(P(a), P(out)); break;
            case CPUREF_TANH: dev().tanh(P(a), P(out)); break;
            case CPUREF_LOG:  dev().log(P(a), P(out)); break;
            case CPUREF_EXP:  dev().exp(P(a), P(out)); break;
            default: throw std::invalid_argument("op");
        }
    });
}

int aixref_fill(const void* scalar, int scalar_dtype, const cpuref_tensor* out)
{ return guarded([&] { dev().fill(scalar, static_cast<aix::DataType>(scalar_dtype), P(out)); }); }
int aixref_fill_min(const cpuref_tensor* out) { return guarded([&] { dev().fillMin(P(out)); }); }
int aixref_copy(const void* src, int sdt, void* dst, int ddt, uint64_t n)
{ return guarded([&] { dev().copy(src, static_cast<aix::DataType>(sdt), dst, static_cast<aix::DataType>(ddt), n); }); }
int aixref_contiguous(const cpuref_tensor* s, const cpuref_tensor* d) { return guarded([&] { dev().contiguous(P(s), P(d)); }); }
int aixref_transpose(const cpuref_tensor* a, const cpuref_tensor* o, uint64_t d0, uint64_t d1)
{ return guarded([&] { dev().transpose(P(a), P(o), d0, d1); }); }
int aixref_sum(const cpuref_tensor* a, const cpuref_tensor* o) { return guarded([&] { dev().sum(P(a), P(o)); }); }
int aixref_max(const cpuref_tensor* a, const cpuref_tensor* o) { return guarded([&] { dev().max(P(a), P(o)); }); }
int aixref_argmax(const cpuref_tensor* a, const cpuref_tensor* o) { return guarded([&] { dev().argmax(P(a), P(o)); }); }
int aixref_argmax_indices(const cpuref_tensor* a, const cpuref_tensor* o) { return guarded([&] { dev().argmaxIndices(P(a), P(o)); }); }
int aixref_reduce_to(const cpuref_tensor* s, const cpuref_tensor* d) { return guarded([&] { dev().reduceTo(P(s), P(d)); }); }
int aixref_max_to(const cpuref_tensor* s, const cpuref_tensor* d) { return guarded([&] { dev().maxTo(P(s), P(d)); }); }
int aixref_argmax_to(const cpuref_tensor* s, const cpuref_tensor* d, uint64_t dim) { return guarded([&] { dev().argmaxTo(P(s), P(d), dim); }); }
int aixref_argmax_indices_to(const cpuref_tensor* s, const cpuref_tensor* d, uint64_t dim) { return guarded([&] { dev().argmaxIndicesTo(P(s), P(d), dim); }); }
int aixref_matmul(const cpuref_tensor* a, const cpuref_tensor* b, const cpuref_tensor* o) { return guarded([&] { dev().matmul(P(a), P(b), P(o)); }); }
int aixref_slice_set(const cpuref_tensor* s, const cpuref_tensor* d, uint64_t dim, uint64_t start, uint64_t end, uint64_t step)
{ return guarded([&] { dev().sliceSet(P(s), P(d), dim, start, end, step); }); }
int aixref_tril(const cpuref_tensor* s, const cpuref_tensor* d, int64_t diag) { return guarded([&] { dev().tril(P(s), P(d), diag); }); }
int aixref_triu(const cpuref_tensor* s, const cpuref_tensor* d, int64_t diag) { return guarded([&] { dev().triu(P(s), P(d), diag); }); }
int aixref_index_select(const cpuref_tensor* s, const cpuref_tensor* d, const cpuref_tensor* i, uint64_t dim)
{ return guarded([&] { dev().indexSelect(P(s), P(d), P(i), dim); }); }
int aixref_index_add(const cpuref_tensor* s, const cpuref_tensor* d, const cpuref_tensor* i, uint64_t dim)
{ return guarded([&] { dev().indexAdd(P(s), P(d), P(i), dim); }); }

} // extern "C"
