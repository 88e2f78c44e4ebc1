// aix_compat.hpp -- the AIX device-plugin interface as this library sees it.
//
// DeviceHIP is a drop-in implementation of aix::Device.  Two ways to build it:
//
//   * inside an AIX checkout: define AIXHIP_USE_AIX_HEADERS and put Targets/AIXLib on the include
//     path; the real <aix.hpp> then provides aix::Device, aix::DeviceTensorParams, aix::DataType,
//     aix::DeviceType, and DeviceHIP derives from the framework's own base class;
//
//   * standalone (this repository, the GPU box): the declarations below restate exactly that
//     interface -- same namespace, names, enumerator values, member order and virtual signatures
//     (Targets/AIXLib/aixDevice.hpp:30-84, aixCore.hpp:44-55, 189-198, aixDeviceType.hpp:15-19)
//     -- so the very same DeviceHIP source compiles without AIX.  Only declarations coincide with
//     AIX; nothing of its implementation is here.
#pragma once

#ifdef AIXHIP_USE_AIX_HEADERS
#include <aix.hpp>
namespace aix {
// AIX has no enumerator for this backend (aixDeviceType.hpp:15-19); the next free value is used.
inline constexpr DeviceType kDeviceTypeHIP = static_cast<DeviceType>(2);
}
#else

#include <cstddef>
#include <cstdint>
#include <string>
#include <sys/types.h>
#include <vector>

namespace aix {

enum class DeviceType { kCPU, kGPU_METAL, kGPU_HIP };
inline constexpr DeviceType kDeviceTypeHIP = DeviceType::kGPU_HIP;

enum class DataType : size_t {
    kFloat64 = 0, kFloat32 = 1, kFloat16 = 2, kBFloat16 = 3,
    kInt64 = 4, kInt32 = 5, kInt16 = 6, kInt8 = 7, kUInt8 = 8,
};
constexpr size_t DataTypeCount = 9;

using Index  = std::vector<size_t>;
using SIndex = std::vector<ssize_t>;
using Shape  = std::vector<size_t>;
using Stride = std::vector<size_t>;

// What every operator receives for each operand.
struct DeviceTensorParams {
    void*    data{nullptr};
    DataType dtype{DataType::kFloat32};
    bool     isContiguous{true};
    size_t   offset{0};     // first element, in elements from `data`
    Shape    shape{};
    size_t   size{0};       // logical element count
    Stride   strides{};     // in elements; 0 = broadcast
};

// The operator set a backend implements (39 virtuals).
class Device {
public:
    virtual ~Device();

    virtual DeviceType type() const = 0;
    virtual std::string name() const = 0;

    static size_t dataTypeSize(DataType dtype);

    virtual void* allocate(size_t size) = 0;
    virtual void* allocate(size_t size, DataType dtype) = 0;
    virtual void deallocate(void* memory) = 0;

    virtual void add(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) = 0;
    virtual void sub(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) = 0;
    virtual void mul(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) = 0;
    virtual void div(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) = 0;
    virtual void unary(const DeviceTensorParams& a1, const DeviceTensorParams& result) = 0;

    virtual void fill(const void* scalar, DataType scalarDType, const DeviceTensorParams& result) = 0;
    virtual void fillMin(const DeviceTensorParams& result) = 0;
    virtual void sum(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void sqrt(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void sin(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void cos(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void tanh(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void log(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void exp(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void pow(const DeviceTensorParams& a, const DeviceTensorParams& exp, const DeviceTensorParams& result) = 0;
    virtual void max(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void argmax(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void argmaxIndices(const DeviceTensorParams& a, const DeviceTensorParams& result) = 0;
    virtual void matmul(const DeviceTensorParams& a, const DeviceTensorParams& b, const DeviceTensorParams& result) = 0;
    virtual void transpose(const DeviceTensorParams& a, const DeviceTensorParams& result, size_t dim0, size_t dim1) = 0;

    virtual void copy(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size) = 0;
    virtual void copyImmediate(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size) = 0;
    virtual void contiguous(const DeviceTensorParams& src, const DeviceTensorParams& dst) = 0;
    virtual void reduceTo(const DeviceTensorParams& src, const DeviceTensorParams& dst) = 0;
    virtual void maxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst) = 0;
    virtual void argmaxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim) = 0;
    virtual void argmaxIndicesTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim) = 0;
    virtual void sliceSet(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                          size_t dim, size_t start, size_t end, size_t step) = 0;
    virtual void tril(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal) = 0;
    virtual void triu(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal) = 0;
    virtual void indexSelect(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                             const DeviceTensorParams& indices, size_t dim) = 0;
    virtual void indexAdd(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                          const DeviceTensorParams& indices, size_t dim) = 0;

    virtual void emptyCache() = 0;
    virtual void synchronize() = 0;
};

} // namespace aix
#endif
