// value.hpp -- a small tensor-value front-end over aix::Device.
//
// This is the CALLER side of the device interface: it decides what a device sees, exactly the way
// the AIX front-end does (Targets/AIXLib/aixCore.hpp) --
//   * every operator allocates a fresh contiguous result from the device (:1414-1427);
//   * operands of different shape become stride-0 broadcast VIEWS, no copy (:599-629, 1616-1638);
//   * `tensor op scalar` materialises the scalar as a rank-0 tensor with fill() and reads it
//     through a broadcast view (:2384-2388);
//   * transpose / reshape of contiguous data / select are views (:979-994);
//   * reductions along dims are fill(0 | lowest) followed by reduceTo / maxTo (:632-639, 873-891);
//   * temporaries release their storage (Device::deallocate) as soon as the expression is done,
//     usually long before the device has run anything.
// It exists so that the benchmark and the training example can drive DeviceHIP (or any other
// aix::Device) with the op stream AIX itself would produce.  It is not a port of AIX's tensor
// classes: no printing, no serialisation, no dtype promotion beyond what the drivers need.
#pragma once

#include "../device/aix_compat.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <numeric>
#include <stdexcept>
#include <vector>

namespace aixfe {

using aix::DataType;
using aix::Device;
using aix::DeviceTensorParams;
using aix::Shape;
using aix::Stride;

inline bool isFloat(DataType dt) { return static_cast<size_t>(dt) <= static_cast<size_t>(DataType::kBFloat16); }

inline size_t numel(const Shape& s) { size_t n = 1; for (auto e : s) n *= e; return n; }

inline Stride denseStrides(const Shape& s)
{
    Stride st(s.size());
    size_t run = 1;
    for (size_t d = s.size(); d-- > 0;) { st[d] = run; run *= s[d]; }
    return st;
}

inline Shape broadcastShapes(const Shape& a, const Shape& b)
{
    const size_t r = std::max(a.size(), b.size());
    Shape out(r);
    for (size_t i = 0; i < r; ++i) {
        const size_t ea = i < r - a.size() ? 1 : a[i - (r - a.size())];
        const size_t eb = i < r - b.size() ? 1 : b[i - (r - b.size())];
        if (ea != eb && ea != 1 && eb != 1) throw std::invalid_argument("shapes cannot be broadcast together");
        out[i] = ea == 1 ? eb : ea;
    }
    return out;
}

class Value {
public:
    Value() = default;

    // Uninitialised contiguous tensor.
    Value(Device* dev, DataType dt, Shape shape) : m_dev(dev)
    {
        m_p.dtype = dt;
        m_p.shape = std::move(shape);
        m_p.strides = denseStrides(m_p.shape);
        m_store = std::make_shared<Storage>(dev, dev->allocate(std::max<size_t>(numel(m_p.shape), 1), dt));
    }

    // Every element = v (one device fill).
    static Value full(Device* dev, DataType dt, const Shape& shape, float v)
    {
        Value t(dev, dt, shape);
        dev->fill(&v, DataType::kFloat32, t.params());
        return t;
    }

    // From host memory of the same element type (Device::copy, host source).
    static Value fromHost(Device* dev, DataType dt, const Shape& shape, const void* host)
    {
        Value t(dev, dt, shape);
        dev->copy(host, dt, t.data(), dt, numel(shape));
        return t;
    }

    bool defined() const { return (bool)m_store; }
    // Gives the memory up; shape, strides and type stay readable (what a backward formula needs of a value nobody reads).
    void releaseStorage() { m_store.reset(); }
    Device* device() const { return m_dev; }
    DataType dtype() const { return m_p.dtype; }
    const Shape& shape() const { return m_p.shape; }
    const Stride& strides() const { return m_p.strides; }
    size_t size() const { return numel(m_p.shape); }
    void* data() const { return m_store ? m_store->ptr : nullptr; }
    size_t offset() const { return m_p.offset; }
    bool isContiguous() const
    {
        size_t run = 1;
        for (size_t d = m_p.shape.size(); d-- > 0;) { if (m_p.strides[d] != run) return false; run *= m_p.shape[d]; }
        return true;
    }

    // What the device sees of this value.  The reference is to a member that this call brings up
    // to date: it stays valid while the value lives and is not reshaped.
    const DeviceTensorParams& params() const
    {
        if (!m_store) throw std::logic_error("aixfe::Value: the value's memory has been released (no backward formula was to read it)");
        m_p.data = data(); m_p.isContiguous = isContiguous(); m_p.size = size();
        return m_p;
    }

    // ---- views ------------------------------------------------------------------------------
    Value broadcastTo(const Shape& target) const
    {
        if (target == m_p.shape) return *this;
        if (target.size() < m_p.shape.size()) throw std::invalid_argument("broadcastTo: rank shrinks");
        Value v = *this;
        v.m_p.shape = target;
        v.m_p.strides.assign(target.size(), 0);
        const size_t lead = target.size() - m_p.shape.size();
        for (size_t i = 0; i < m_p.shape.size(); ++i) {
            if (m_p.shape[i] == target[lead + i]) v.m_p.strides[lead + i] = m_p.strides[i];
            else if (m_p.shape[i] != 1) throw std::invalid_argument("broadcastTo: incompatible shape");
        }
        return v;
    }

    Value transpose(size_t d0, size_t d1) const
    {
        Value v = *this;
        std::swap(v.m_p.shape[d0], v.m_p.shape[d1]);
        std::swap(v.m_p.strides[d0], v.m_p.strides[d1]);
        return v;
    }

    Value reshape(const Shape& s) const
    {
        if (numel(s) != size()) throw std::invalid_argument("reshape: element count differs");
        Value v = isContiguous() ? *this : contiguous();
        v.m_p.shape = s;
        v.m_p.strides = denseStrides(s);
        return v;
    }

    // index `i` along the first dim: a view with an offset (how batched matmuls are issued)
    Value select0(size_t i) const
    {
        Value v = *this;
        v.m_p.offset += i * m_p.strides[0];
        v.m_p.shape.erase(v.m_p.shape.begin());
        v.m_p.strides.erase(v.m_p.strides.begin());
        return v;
    }

    Value contiguous() const
    {
        if (isContiguous() && m_p.offset == 0) return *this;
        Value r(m_dev, m_p.dtype, m_p.shape);
        m_dev->contiguous(params(), r.params());
        return r;
    }

    Value to(DataType dt) const
    {
        if (dt == m_p.dtype) return *this;
        Value src = contiguous();
        Value r(m_dev, dt, m_p.shape);
        m_dev->copy(static_cast<const char*>(src.data()) + src.m_p.offset * Device::dataTypeSize(m_p.dtype), m_p.dtype, r.data(), dt, size());
        return r;
    }

    // ---- elementwise ------------------------------------------------------------------------
    using BinaryFn = void (Device::*)(const DeviceTensorParams&, const DeviceTensorParams&, const DeviceTensorParams&);
    using UnaryFn = void (Device::*)(const DeviceTensorParams&, const DeviceTensorParams&);

    Value binary(BinaryFn fn, const Value& other) const
    {
        if (other.m_p.dtype != m_p.dtype) {
            // operands are first converted to the promoted type (aixCore.hpp:1616-1630); the drivers
            // only ever mix a floating tensor with an integer mask, which promotes to the float type
            const bool lf = isFloat(m_p.dtype), rf = isFloat(other.m_p.dtype);
            if (lf == rf) throw std::invalid_argument("binary: unsupported mix of element types");
            return lf ? binary(fn, other.to(m_p.dtype)) : to(other.m_p.dtype).binary(fn, other);
        }
        if (m_p.shape == other.m_p.shape) {
            Value r(m_dev, m_p.dtype, m_p.shape);
            (m_dev->*fn)(params(), other.params(), r.params());
            return r;
        }
        const Shape bc = broadcastShapes(m_p.shape, other.m_p.shape);
        const Value l = broadcastTo(bc), rr = other.broadcastTo(bc);
        Value r(m_dev, m_p.dtype, bc);
        (m_dev->*fn)(l.params(), rr.params(), r.params());
        return r;
    }

    // tensor op scalar: rank-0 tensor + broadcast view
    Value binaryScalar(BinaryFn fn, float s, bool scalarFirst = false) const
    {
        const Value sc = full(m_dev, m_p.dtype, Shape{}, s).broadcastTo(m_p.shape);
        Value r(m_dev, m_p.dtype, m_p.shape);
        if (scalarFirst) (m_dev->*fn)(sc.params(), params(), r.params());
        else (m_dev->*fn)(params(), sc.params(), r.params());
        return r;
    }

    Value& inPlace(BinaryFn fn, const Value& other)
    {
        const Value rhs = other.m_p.shape == m_p.shape ? other : other.broadcastTo(m_p.shape);
        (m_dev->*fn)(params(), rhs.params(), params());
        return *this;
    }

    Value unary(UnaryFn fn) const
    {
        Value r(m_dev, m_p.dtype, m_p.shape);
        (m_dev->*fn)(params(), r.params());
        return r;
    }

    Value operator+(const Value& o) const { return binary(&Device::add, o); }
    Value operator-(const Value& o) const { return binary(&Device::sub, o); }
    Value operator*(const Value& o) const { return binary(&Device::mul, o); }
    Value operator/(const Value& o) const { return binary(&Device::div, o); }
    Value operator+(float s) const { return binaryScalar(&Device::add, s); }
    Value operator-(float s) const { return binaryScalar(&Device::sub, s); }
    Value operator*(float s) const { return binaryScalar(&Device::mul, s); }
    Value operator/(float s) const { return binaryScalar(&Device::div, s); }
    friend Value operator+(float s, const Value& v) { return v.binaryScalar(&Device::add, s, true); }
    friend Value operator-(float s, const Value& v) { return v.binaryScalar(&Device::sub, s, true); }
    friend Value operator*(float s, const Value& v) { return v.binaryScalar(&Device::mul, s, true); }
    friend Value operator/(float s, const Value& v) { return v.binaryScalar(&Device::div, s, true); }
    Value operator-() const { return unary(&Device::unary); }
    Value& operator+=(const Value& o) { return inPlace(&Device::add, o); }
    Value& operator-=(const Value& o) { return inPlace(&Device::sub, o); }
    Value& operator*=(const Value& o) { return inPlace(&Device::mul, o); }
    Value sqrt() const { return unary(&Device::sqrt); }
    Value exp() const { return unary(&Device::exp); }
    Value log() const { return unary(&Device::log); }
    Value tanh() const { return unary(&Device::tanh); }
    Value sin() const { return unary(&Device::sin); }
    Value cos() const { return unary(&Device::cos); }
    Value pow(float e) const { return binaryScalar(&Device::pow, e); }

    void fill(float v) { m_dev->fill(&v, DataType::kFloat32, params()); }

    // `value op scalar` as the reference's value class does it (aixCore.hpp:715-777): the scalar
    // becomes a FULL-SHAPE filled tensor, then the ordinary binary operator runs.  (The float
    // operators above follow its autograd class instead: rank-0 tensor + broadcast view, :2384-2438.)
    Value withScalar(BinaryFn fn, float s, bool scalarFirst = false) const
    {
        const Value sc = full(m_dev, m_p.dtype, m_p.shape, s);
        return scalarFirst ? sc.binary(fn, *this) : binary(fn, sc);
    }

    // ---- reductions ---------------------------------------------------------------------------
    Value sum() const
    {
        Value r(m_dev, m_p.dtype, Shape{});
        m_dev->sum(params(), r.params());
        return r;
    }

    // Sum down to `target` (right-aligned, 1 = reduced): zero-fill then accumulate.
    Value reduceTo(const Shape& target) const
    {
        if (target == m_p.shape) return *this;
        Value r = full(m_dev, m_p.dtype, target, 0.0f);
        m_dev->reduceTo(params(), r.params());
        return r;
    }

    Value sum(size_t dim, bool keepDim) const
    {
        Shape kept = m_p.shape;
        kept[dim] = 1;
        Value r = reduceTo(kept);
        return keepDim ? r : r.squeeze(dim);
    }

    // L2 norm of an f32 tensor as a measurement: the squares are added up row by row first and the row sums after,
    // so that no single running sum grows over more than a row's or a column of rows' worth of terms.  (A CPU device
    // that adds a whole tensor up in one f32 running sum -- aixDeviceCPU.cpp:244-253 -- is 0.2-0.6 % low on millions of
    // squares of similar size: terms under half a unit in the last place of the sum vanish.)
    float l2Norm() const
    {
        const Value squares = (*this) * (*this);
        const Value total = m_p.shape.size() >= 2 && m_p.shape[0] > 1 ? squares.sum(m_p.shape.size() - 1, false).sum() : squares.sum();
        return std::sqrt(total.item());
    }

    Value max(size_t dim, bool keepDim) const
    {
        Shape kept = m_p.shape;
        kept[dim] = 1;
        Value r(m_dev, m_p.dtype, kept);
        m_dev->fillMin(r.params());
        m_dev->maxTo(params(), r.params());
        return keepDim ? r : r.squeeze(dim);
    }

    Value argmax(size_t dim, bool keepDim) const
    {
        Shape kept = m_p.shape;
        kept[dim] = 1;
        Value r(m_dev, DataType::kInt32, kept);
        m_dev->argmaxTo(params(), r.params(), dim);
        return keepDim ? r : r.squeeze(dim);
    }

    Value mean() const { return sum() / (float)size(); }

    // 1 where the element is the (first) maximum along `dim`, 0 elsewhere, int32 (aixCore.hpp:927-941).
    Value argmaxIndices(size_t dim) const
    {
        Value r = full(m_dev, DataType::kInt32, m_p.shape, 0.0f);
        m_dev->argmaxIndicesTo(params(), r.params(), dim);
        return r;
    }

    // aixCore.hpp:1060-1087
    Value unsqueeze(size_t dim) const
    {
        Value v = *this;
        size_t inserted = 1;
        if (!m_p.shape.empty() && dim < m_p.shape.size()) inserted = m_p.strides[dim] * m_p.shape[dim];
        v.m_p.shape.insert(v.m_p.shape.begin() + (long)dim, 1);
        v.m_p.strides.insert(v.m_p.strides.begin() + (long)dim, inserted);
        return v;
    }

    // A strided window along `dim` (view; aixCore.hpp:1089-1145).
    Value slice(size_t dim, size_t start, size_t end, size_t step = 1) const
    {
        if (dim >= m_p.shape.size() || step < 1 || start >= end || end > m_p.shape[dim]) throw std::invalid_argument("slice: bad range");
        Value v = *this;
        v.m_p.offset += start * m_p.strides[dim];
        v.m_p.strides[dim] *= step;
        v.m_p.shape[dim] = (end - start + step - 1) / step;
        return v;
    }

    // Write `src` into that window of *this (in place; aixCore.hpp:1147-1204 with inPlace = true).
    void sliceSetInPlace(const Value& src, size_t dim, size_t start, size_t end, size_t step = 1) const
    {
        m_dev->sliceSet(src.params(), params(), dim, start, end, step);
    }

    // aixCore.hpp:1348-1402: a fresh tensor, one sliceSet per part.
    static Value cat(const std::vector<Value>& parts, size_t dim)
    {
        if (parts.empty()) throw std::invalid_argument("cat: no tensors");
        Shape shape = parts[0].m_p.shape;
        for (size_t i = 1; i < parts.size(); ++i) shape[dim] += parts[i].m_p.shape[dim];
        Value r(parts[0].m_dev, parts[0].m_p.dtype, shape);
        size_t at = 0;
        for (const auto& p : parts) { r.sliceSetInPlace(p, dim, at, at + p.m_p.shape[dim]); at += p.m_p.shape[dim]; }
        return r;
    }

    // aixCore.hpp:1320-1346
    Value tril(ssize_t diagonal = 0) const
    {
        Value r(m_dev, m_p.dtype, m_p.shape);
        m_dev->tril(params(), r.params(), diagonal);
        return r;
    }

    // Zero-padded copy of `src` into the window of a tensor shaped like *this (aixCore.hpp:1147-1204, not in place).
    Value sliceSet(const Value& src, size_t dim, size_t start, size_t end, size_t step = 1) const
    {
        Value r = full(m_dev, m_p.dtype, m_p.shape, 0.0f);
        m_dev->sliceSet(src.params(), r.params(), dim, start, end, step);
        return r;
    }

    // Rows (dim = 0) or other slabs picked by an int32 index vector (aixCore.hpp:1217-1247).
    Value indexSelect(size_t dim, const Value& indices) const
    {
        Shape shape = m_p.shape;
        shape[dim] = indices.shape().empty() ? 1 : indices.shape()[0];
        Value r(m_dev, m_p.dtype, shape);
        m_dev->indexSelect(params(), r.params(), indices.params(), dim);
        return r;
    }

    // *this[indices] += source, in place (aixCore.hpp:1249-1294 with inPlace = true).
    void indexAddInPlace(size_t dim, const Value& indices, const Value& source) const
    {
        m_dev->indexAdd(source.params(), params(), indices.params(), dim);
    }

    Value pow(const Value& e) const
    {
        Value r(m_dev, m_p.dtype, m_p.shape);
        m_dev->pow(params(), e.params(), r.params());
        return r;
    }

    // First element on the host, after a synchronize(); device memory is host-readable on both
    // backends (plain memory on the CPU, large-BAR mapping on the GPU).
    float item() const
    {
        if (m_p.dtype != DataType::kFloat32) throw std::invalid_argument("item: f32 only");
        m_dev->synchronize();
        float v;
        std::memcpy(&v, static_cast<const char*>(data()) + m_p.offset * sizeof(float), sizeof(float));
        return v;
    }

    Value squeeze(size_t dim) const
    {
        Value v = *this;
        if (dim >= m_p.shape.size() || m_p.shape[dim] != 1) return v;
        v.m_p.shape.erase(v.m_p.shape.begin() + (long)dim);
        v.m_p.strides.erase(v.m_p.strides.begin() + (long)dim);
        return v;
    }

    // 2-D operands as in the reference (aixCore.hpp:943-976).  Beyond it: operands of one rank above 2 with the
    // same leading dims are a stack of products, one per leading index, in a single device call.
    Value matmul(const Value& b) const
    {
        const size_t r = m_p.shape.size();
        if (r < 2 || b.m_p.shape.size() != r || m_p.shape[r - 1] != b.m_p.shape[r - 2] ||
            !std::equal(m_p.shape.begin(), m_p.shape.end() - 2, b.m_p.shape.begin()))
            throw std::invalid_argument("matmul: operands must be 2-D (or stacks with the same leading dims) with matching inner dimension");
        Shape out(m_p.shape.begin(), m_p.shape.end() - 1);
        out.push_back(b.m_p.shape[r - 1]);
        Value res(m_dev, m_p.dtype, out);
        m_dev->matmul(params(), b.params(), res.params());
        return res;
    }

private:
    struct Storage {
        Device* dev;
        void* ptr;
        Storage(Device* d, void* p) : dev(d), ptr(p) {}
        ~Storage() { if (dev && ptr) dev->deallocate(ptr); }
        Storage(const Storage&) = delete;
        Storage& operator=(const Storage&) = delete;
    };

    Device* m_dev{nullptr};
    mutable DeviceTensorParams m_p;        // dtype, offset, shape and strides live here; data / size / isContiguous are set by params()
    std::shared_ptr<Storage> m_store;
};

} // namespace aixfe
