// device_hip.hpp -- aix::Device for one AMD Instinct MI355X (gfx950).
//
// Implements the same pure-virtual operator interface the reference's GPU device implements
// (Targets/AIXLib/aixDevice.hpp:30-84; behavioural template Targets/AIXLib/aixDeviceMetal.cpp), so
// tensors, autograd, optimizers and examples written against aix::Device run unchanged:
//
//     aix::hip::DeviceHIP device;                 // or aix::hip::createDeviceHIP(0)
//     auto x = aix::tensor(..., { .m_device = &device });
//
// Host C++ only: the GPU is reached exclusively through the C ABI of libaixhip_kernels.so
// (include/aixhip_kernels.h).
//
// Execution model
//   * elementwise operators and fills are RECORDED (fuse.hpp) and run as runtime-compiled fused
//     kernels at the next flush; every other operator flushes and is enqueued at once;
//   * everything runs on one in-order stream; results are defined after synchronize();
//   * allocate() returns device memory that the host can dereference (large-BAR mapping): host
//     writes are fast, host reads are slow and meant for scalars / debugging / small tensors;
//   * deallocate() is deferred until the recorded work that may use the block has been enqueued;
//     blocks are then reused from size buckets;
//   * input operands may be host pointers (they are staged); results must be this device's memory,
//     otherwise std::invalid_argument, as on the reference GPU device (aixDeviceMetal.cpp:305-306).
#pragma once

#include "aix_compat.hpp"
#include "fuse.hpp"

#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

struct aixk_ctx;
struct aixk_module;
struct aixhip_tensor;
struct aixhip_device;

namespace aix::hip {

class DeviceHIP : public aix::Device {
public:
    explicit DeviceHIP(size_t deviceIndex = 0);
    ~DeviceHIP() override;
    DeviceHIP(const DeviceHIP&) = delete;
    DeviceHIP& operator=(const DeviceHIP&) = delete;

    DeviceType type() const override { return aix::kDeviceTypeHIP; }
    std::string name() const override { return "HIP"; }

    void* allocate(size_t size) override;
    void* allocate(size_t size, DataType dtype) override;
    void deallocate(void* memory) override;

    void add(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) override;
    void sub(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) override;
    void mul(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) override;
    void div(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) override;
    void unary(const DeviceTensorParams& a1, const DeviceTensorParams& result) override;

    void fill(const void* scalar, DataType scalarDType, const DeviceTensorParams& result) override;
    void fillMin(const DeviceTensorParams& result) override;
    void sum(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void sqrt(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void sin(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void cos(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void tanh(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void log(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void exp(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void pow(const DeviceTensorParams& a, const DeviceTensorParams& exp, const DeviceTensorParams& result) override;
    void max(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void argmax(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void argmaxIndices(const DeviceTensorParams& a, const DeviceTensorParams& result) override;
    void matmul(const DeviceTensorParams& a, const DeviceTensorParams& b, const DeviceTensorParams& result) override;
    void transpose(const DeviceTensorParams& a, const DeviceTensorParams& result, size_t dim0, size_t dim1) override;

    void copy(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size) override;
    void copyImmediate(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size) override;
    void contiguous(const DeviceTensorParams& src, const DeviceTensorParams& dst) override;
    void reduceTo(const DeviceTensorParams& src, const DeviceTensorParams& dst) override;
    void maxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst) override;
    void argmaxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim) override;
    void argmaxIndicesTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim) override;
    void sliceSet(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                  size_t dim, size_t start, size_t end, size_t step) override;
    void tril(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal) override;
    void triu(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal) override;
    void indexSelect(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                     const DeviceTensorParams& indices, size_t dim) override;
    void indexAdd(const DeviceTensorParams& src, const DeviceTensorParams& dst,
                  const DeviceTensorParams& indices, size_t dim) override;

    void emptyCache() override;
    void synchronize() override;

    // ---- beyond the interface -------------------------------------------------------------------
    // Explicit transfers for hosts that should not read device memory through the BAR mapping.
    void copyToHost(void* dstHost, const void* srcDevice, size_t bytes);     // flushes and waits
    void copyFromHost(void* dstDevice, const void* srcHost, size_t bytes);   // stream ordered
    bool isDeviceMemory(const void* p) const { return findBlock(p) != nullptr; }

    void setFuseConfig(const aixhip::fuse::FuseConfig& cfg);                  // flushes first
    const aixhip::fuse::FuseConfig& fuseConfig() const { return m_engine->config(); }
    const aixhip::fuse::FlushDiagnostics& lastFlushDiagnostics() const { return m_engine->lastFlushDiagnostics(); }
    std::pair<size_t, size_t> fuseKernelCacheStats() const;                  // hits, misses (aixDeviceMetal's test hook)
    std::pair<size_t, size_t> batchedLaunchStats() const;                    // launches that carried several flat kernels, kernels carried
    void flush();                                                            // plan + enqueue, no wait
    aixk_ctx* kernelContext() const { return m_ctx; }
    size_t cachedBytes() const { return m_pooledBytes; }
    // A stretch of the device's work as a HIP graph: a step whose operator stream, addresses and immediates repeat (a
    // forward + backward pass, an update in place) is issued once between beginCapture() and endCapture() -- recorded,
    // not run -- and then enqueued again and again by replay() with one call, without the front-end, the planner or a
    // launch per kernel.  The reference's GPU device amortises dispatch by batching into command buffers
    // (aixDeviceMetal.cpp:1344-1389); this goes one step further and has no counterpart there.
    // Inside a capture: no synchronize(), no host transfer (copyToHost / copyFromHost / host operands), nothing that has
    // to compile or grow a workspace for the first time (run the step once uncaptured before) -- std::runtime_error.
    // Every block the captured work touches belongs to the graph from then on: freed, it is kept aside (never handed out
    // again) until the last graph is destroyed, so a replay cannot write into somebody else's tensor; tensors that are
    // still alive (parameters, gradients, the loss) are simply used in place by every replay.
    struct StepGraph;
    void beginCapture();                  // flushes and waits first
    StepGraph* endCapture();              // flushes what was recorded into the graph; nothing of it has run yet
    void abortCapture();                  // gives an open capture up (after an error inside it, say): nothing of it runs, the device is usable again
    void replay(StepGraph* graph);        // enqueues the captured work (after whatever is pending)
    size_t graphNodes(const StepGraph* graph) const;
    void destroyGraph(StepGraph* graph);
    bool capturing() const { return m_capturing; }

    // The pool of idle blocks is cut back to this many bytes at every synchronize() (aixDeviceMetal.cpp:1369-1373 trims
    // its buffer cache to the working-set limit at every commit).  Default: 0.7 of the card's memory, as there (:33).
    void setCacheLimit(size_t bytes) { m_cacheLimit = bytes; }
    size_t cacheLimit() const { return m_cacheLimit; }
    size_t allocatedBytes() const { return m_liveBytes; }

private:
    struct Block {
        size_t bytes;
        bool touched{false};     // enqueued GPU work has referenced the block since it was allocated
        bool freed{false};       // deallocate() has been called; the block waits in m_limbo
        bool inGraph{false};     // captured work uses the block: once freed it is kept aside, not pooled
        uint32_t waiters{0};     // operands and results of waiting products in the block (one lookup tells most callers "none")
    };
    struct Extras;

    // Live allocations by base address.  Operands normally carry a block's base pointer (views
    // differ by offset), so the lookup is one probe of an open-addressing table; a pointer into the
    // middle of a block, or a host pointer, falls back to a scan.
    class BlockTable {
    public:
        Block* find(const void* base) const;
        Block* findContaining(const void* p) const;
        const void* baseOf(const void* p) const;            // start of the block p lies in; nullptr for host memory
        void insert(void* base, size_t bytes);
        bool erase(void* base, size_t* bytes);
        bool empty() const { return m_count == 0; }
        template <class F> void forEach(F f) const { for (const auto& s : m_slots) if (s.key > 1) f((void*)s.key, s.block); }
    private:
        struct Slot { uintptr_t key{0}; mutable Block block{0}; };   // key 0 = never used, 1 = erased
        size_t slotOf(uintptr_t key) const { return (size_t)(((key >> 6) * 0x9E3779B97F4A7C15ull) >> m_shift); }
        void grow();
        std::vector<Slot> m_slots;
        size_t m_count{0}, m_used{0};
        unsigned m_shift{64};
        uintptr_t m_lo{UINTPTR_MAX}, m_hi{0};                   // every block ever inserted lies in [m_lo, m_hi): host pointers miss at once
    };

    const Block* findBlock(const void* p) const;
    size_t bucketBytes(size_t bytes) const;
    void* allocateBlock(size_t bytes, bool track);
    void releaseLimbo();
    void markTouched(const void* p);
    void requireDevice(const DeviceTensorParams& result, const char* op) const;
    // Makes the view's data device memory: a host operand is staged into a temporary block.
    void onDevice(aixhip::fuse::View& v);
    const void* stageRaw(const void* src, size_t bytes);
    void toPod(const DeviceTensorParams& p, aixhip_tensor* out, const char* op) const;
    void toPod(const aixhip::fuse::View& v, aixhip_tensor* out) const;
    void stagedPod(const DeviceTensorParams& p, aixhip_tensor* out, const char* op);      // toPod + staging of a host operand
    void check(int status) const;
    void recordBinary(aixhip::fuse::OpType t, const DeviceTensorParams& a, const DeviceTensorParams& b,
                      const DeviceTensorParams& r, const char* op);
    void recordUnary(aixhip::fuse::OpType t, const DeviceTensorParams& a, const DeviceTensorParams& r, const char* op);
    bool recordTri(aixhip::fuse::OpType t, const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal);
    bool takeInit(const DeviceTensorParams& src, const DeviceTensorParams& dst, uint64_t* bits);
    void flushFor(const void* a = nullptr, const void* b = nullptr, const void* c = nullptr);
    void flushForOperands(const void* a, const void* b, const void* c, bool always);
    void flushWindow(bool final);
    bool fenceInterior(const void* a, const void* b = nullptr, const void* c = nullptr);   // true: flush again once the operator is recorded
    void emitFused(const aixhip::fuse::FusedSubgraphDescriptor& d);
    void emitSingle(const aixhip::fuse::OpRecord& op);
    void emitRowProgram(const aixhip::fuse::FusedSubgraphDescriptor& d);
    void issueFlatBatch();
    bool recordRowReduction(aixhip::fuse::OpType type, const DeviceTensorParams& src, const DeviceTensorParams& dst, uint64_t init);
    void joinBatch(const aixhip::fuse::FusedSubgraphDescriptor& d, aixk_module* mod, const std::string& entry, uint64_t grid, const std::function<std::string()>& manySource);
    void issuePending(bool marked = false);                                   // the waiting matmul and sliceSet calls, one launch per run (see matmul(), sliceSet())

    aixk_ctx* m_ctx{nullptr};
    std::unique_ptr<aixhip::fuse::FuseEngine> m_engine;
    std::unique_ptr<Extras> m_extras;                          // kernel cache, cooling blocks, scratch vectors
    BlockTable m_blocks;
    std::unordered_map<size_t, std::vector<void*>> m_pool;     // free blocks by bucket size
    std::vector<std::pair<void*, size_t>> m_limbo;             // freed, but recorded work may still use them
    size_t m_liveBytes{0}, m_pooledBytes{0}, m_limboBytes{0}, m_totalBytes{0}, m_cacheLimit{~size_t(0)};
    void trimPool();
    void pool(void* p, size_t bytes);     // an idle block goes back to its bucket, or aside if a graph uses it
    bool m_capturing{false};
    size_t m_graphs{0};
    std::vector<std::pair<void*, size_t>> m_graphReserve;      // idle blocks that captured work uses: not handed out while a graph lives
    int m_cus{256};
};

std::unique_ptr<aix::Device> createDeviceHIP(size_t deviceIndex = 0);   // nullptr if no GPU is visible

// The C++ device behind a handle of the C ABI (include/aixhip.h); throws on a null handle.
DeviceHIP* fromHandle(::aixhip_device* handle);

} // namespace aix::hip
