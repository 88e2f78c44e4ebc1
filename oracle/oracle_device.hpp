// oracle_device.hpp -- the CPU oracle behind the aix::Device interface.  TEST INFRASTRUCTURE:
// used by tests, the smoke check and the benchmark's CPU-baseline leg to run the same driver code
// (front-end, autograd, optimizer) on the CPU restatement of the reference's DeviceCPU
// (Targets/AIXLib/aixDeviceCPU.cpp) that the GPU backend is compared with.  Never part of the
// product libraries.
//
// Every operator forwards to the cpuref_* function restating it; memory is plain host memory;
// synchronize() is a no-op (the CPU device is eager, aixDeviceCPU.cpp).  matmul runs cpuref's
// order-preserving row-parallel form (bit-identical to the literal loop nest) on `threads` threads.
//
// `wide16`: a second way of adding 16-bit numbers up, for telling a device's arithmetic errors from the reference's own
// rounding.  The reference's CPU device keeps the running sum of a matmul, a reduceTo or a sum in the element type,
// so a bf16 sum is rounded to 8 bits after every addition (aixDeviceCPU.cpp:244-253, 336-389); with wide16 those three
// operators add the same terms exactly (cpuref_matmul_wide, cpuref_reduce_to_wide, cpuref_sum_wide: float64) and round
// ONCE to the element type.  Every other operator, and every rounding between operators, is the literal one.
#pragma once

#include "../aix_amd/csrc/device/aix_compat.hpp"
#include "cpuref.h"

#include <cstdlib>
#include <stdexcept>
#include <vector>

namespace oracle {

class OracleDevice final : public aix::Device {
public:
    explicit OracleDevice(int threads = 1, bool wide16 = false) : m_threads(threads), m_wide16(wide16) {}

    aix::DeviceType type() const override { return aix::DeviceType::kCPU; }
    std::string name() const override { return "CPU-oracle"; }

    void* allocate(size_t size) override { return std::malloc(size ? size : 1); }
    void* allocate(size_t size, aix::DataType dtype) override { return allocate(size * cpuref_dtype_size((int)dtype)); }
    void deallocate(void* memory) override { std::free(memory); }

    using P = aix::DeviceTensorParams;
    void add(const P& a, const P& b, const P& r) override { ok(cpuref_binary(CPUREF_ADD, d(a), d(b), d(r))); ++ops; }
    void sub(const P& a, const P& b, const P& r) override { ok(cpuref_binary(CPUREF_SUB, d(a), d(b), d(r))); ++ops; }
    void mul(const P& a, const P& b, const P& r) override { ok(cpuref_binary(CPUREF_MUL, d(a), d(b), d(r))); ++ops; }
    void div(const P& a, const P& b, const P& r) override { ok(cpuref_binary(CPUREF_DIV, d(a), d(b), d(r))); ++ops; }
    void pow(const P& a, const P& b, const P& r) override { ok(cpuref_binary(CPUREF_POW, d(a), d(b), d(r))); ++ops; }
    void unary(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_NEG, d(a), d(r))); ++ops; }
    void sqrt(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_SQRT, d(a), d(r))); ++ops; }
    void sin(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_SIN, d(a), d(r))); ++ops; }
    void cos(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_COS, d(a), d(r))); ++ops; }
    void tanh(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_TANH, d(a), d(r))); ++ops; }
    void log(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_LOG, d(a), d(r))); ++ops; }
    void exp(const P& a, const P& r) override { ok(cpuref_unary(CPUREF_EXP, d(a), d(r))); ++ops; }
    void fill(const void* scalar, aix::DataType st, const P& r) override { ok(cpuref_fill(scalar, (int)st, d(r))); ++ops; }
    void fillMin(const P& r) override { ok(cpuref_fill_min(d(r))); ++ops; }
    void sum(const P& a, const P& r) override
    {
        ++ops;
        if (!wide(r)) { ok(cpuref_sum(d(a), d(r))); return; }
        double total = 0;
        ok(cpuref_sum_wide(d(a), &total, nullptr));
        ok(cpuref_copy(&total, CPUREF_F64, r.data, (int)r.dtype, 1));
    }
    void max(const P& a, const P& r) override { ok(cpuref_max(d(a), d(r))); ++ops; }
    void argmax(const P& a, const P& r) override { ok(cpuref_argmax(d(a), d(r))); ++ops; }
    void argmaxIndices(const P& a, const P& r) override { ok(cpuref_argmax_indices(d(a), d(r))); ++ops; }
    void matmul(const P& a, const P& b, const P& r) override
    {
        ++ops; ++matmuls;
        if (wide(r)) { ok(cpuref_matmul_stack_wide(d(a), d(b), d(r), m_threads)); return; }
        ok(a.shape.size() > 2 ? cpuref_matmul_stack(d(a), d(b), d(r), m_threads) : cpuref_matmul_rows(d(a), d(b), d(r), m_threads));
    }
    void transpose(const P& a, const P& r, size_t d0, size_t d1) override { ok(cpuref_transpose(d(a), d(r), d0, d1)); ++ops; }
    void copy(const void* s, aix::DataType st, void* t, aix::DataType tt, size_t n) override { ok(cpuref_copy(s, (int)st, t, (int)tt, n)); }
    void copyImmediate(const void* s, aix::DataType st, void* t, aix::DataType tt, size_t n) override { copy(s, st, t, tt, n); }
    void contiguous(const P& s, const P& t) override { ok(cpuref_contiguous(d(s), d(t))); ++ops; }
    void reduceTo(const P& s, const P& t) override
    {
        ++ops;
        if (!wide(t) || s.dtype != t.dtype) { ok(cpuref_reduce_to(d(s), d(t))); return; }
        // what the destination holds (written densely from its base, aixDeviceCPU.cpp:255-273) plus the exact sums, rounded once
        std::vector<double> acc(t.size);
        ok(cpuref_copy(t.data, (int)t.dtype, acc.data(), CPUREF_F64, t.size));
        ok(cpuref_reduce_to_wide(d(s), d(t), acc.data(), nullptr));
        ok(cpuref_copy(acc.data(), CPUREF_F64, t.data, (int)t.dtype, t.size));
    }
    void maxTo(const P& s, const P& t) override { ok(cpuref_max_to(d(s), d(t))); ++ops; }
    void argmaxTo(const P& s, const P& t, size_t dim) override { ok(cpuref_argmax_to(d(s), d(t), dim)); ++ops; }
    void argmaxIndicesTo(const P& s, const P& t, size_t dim) override { ok(cpuref_argmax_indices_to(d(s), d(t), dim)); ++ops; }
    void sliceSet(const P& s, const P& t, size_t dim, size_t start, size_t end, size_t step) override
    { ok(cpuref_slice_set(d(s), d(t), dim, start, end, step, 0)); ++ops; }
    void tril(const P& s, const P& t, ssize_t diag) override { ok(cpuref_tril(d(s), d(t), diag)); ++ops; }
    void triu(const P& s, const P& t, ssize_t diag) override { ok(cpuref_triu(d(s), d(t), diag)); ++ops; }
    void indexSelect(const P& s, const P& t, const P& idx, size_t dim) override { ok(cpuref_index_select(d(s), d(t), d(idx), dim, 0)); ++ops; }
    void indexAdd(const P& s, const P& t, const P& idx, size_t dim) override { ok(cpuref_index_add(d(s), d(t), d(idx), dim, 0)); ++ops; }
    void emptyCache() override {}
    void synchronize() override {}

    uint64_t ops{0}, matmuls{0};      // operator calls seen (diagnostics for tests)

private:
    // a descriptor that lives until the end of the full expression it is used in
    struct Desc { cpuref_tensor t; operator const cpuref_tensor*() const { return &t; } };
    static Desc d(const P& p)
    {
        if (p.shape.size() > CPUREF_MAX_RANK) throw std::invalid_argument("rank above 16");
        Desc r{};
        r.t.data = p.data; r.t.dtype = (int32_t)p.dtype; r.t.rank = (int32_t)p.shape.size();
        r.t.offset = p.offset; r.t.size = p.size;
        for (size_t i = 0; i < p.shape.size(); ++i) { r.t.shape[i] = p.shape[i]; r.t.strides[i] = p.strides[i]; }
        return r;
    }
    static void ok(int rc) { if (rc != CPUREF_OK) throw std::invalid_argument("oracle operator rejected its arguments"); }
    bool wide(const P& r) const { return m_wide16 && (r.dtype == aix::DataType::kFloat16 || r.dtype == aix::DataType::kBFloat16); }
    int m_threads;
    bool m_wide16;
};

} // namespace oracle
