// device_hip.cpp -- DeviceHIP: host-side logic of the MI355X backend (see device_hip.hpp).

#include "device_hip.hpp"

#include "../../../include/aixhip_kernels.h"
#include "hipgen.hpp"
#include "scalar_convert.hpp"

#include <algorithm>
#include <array>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <dlfcn.h>
#include <deque>
#include <iostream>
#include <limits>
#include <stdexcept>
#include <unordered_set>

namespace aix {

#ifndef AIXHIP_USE_AIX_HEADERS
// In an AIX build these two come from the framework's own library (aixDeviceCPU.cpp:26, 685-700).
Device::~Device() = default;

size_t Device::dataTypeSize(DataType dtype)
{
    static const size_t bytes[DataTypeCount] = {8, 4, 2, 2, 8, 4, 2, 1, 1};
    return bytes[static_cast<size_t>(dtype)];
}
#endif

namespace hip {

using aixhip::fuse::FuseCallbacks;
using aixhip::fuse::FuseConfig;
using aixhip::fuse::FuseEngine;
using aixhip::fuse::FusedSubgraphDescriptor;
using aixhip::fuse::OpRecord;
using aixhip::fuse::OpType;
using aixhip::fuse::View;
namespace gen = aixhip::gen;

namespace {

// Freed blocks wait here until the GPU has passed the point at which they were released: the host
// may write into a reused block directly, which is not ordered with the stream.
struct Cooling {
    aixk_event* event;
    std::vector<std::pair<void*, size_t>> blocks;
};

size_t viewEnd(const View& p)
{
    size_t last = p.offset;
    for (size_t d = 0; d < p.rank; ++d) {
        if (p.shape[d] == 0) return p.offset;
        last += (p.shape[d] - 1) * p.strides[d];
    }
    return last + 1;
}

size_t viewEnd(const aixhip_tensor& p)
{
    size_t last = p.offset;
    for (int d = 0; d < p.rank; ++d) {
        if (p.shape[d] == 0) return p.offset;
        last += (p.shape[d] - 1) * p.strides[d];
    }
    return last + 1;
}

int binaryCode(OpType t)
{
    switch (t) {
        case OpType::Add: return AIXK_ADD; case OpType::Sub: return AIXK_SUB; case OpType::Mul: return AIXK_MUL;
        case OpType::Div: return AIXK_DIV; case OpType::Pow: return AIXK_POW; default: return -1;
    }
}

int unaryCode(OpType t)
{
    switch (t) {
        case OpType::Negate: return AIXK_NEG; case OpType::Sqrt: return AIXK_SQRT; case OpType::Sin: return AIXK_SIN;
        case OpType::Cos: return AIXK_COS; case OpType::Tanh: return AIXK_TANH; case OpType::Log: return AIXK_LOG;
        case OpType::Exp: return AIXK_EXP; default: return -1;
    }
}

} // namespace

// AIXHIP_TRACE=1: one line on stderr per kernel or operator the device enqueues (what ran, in which order, how large).
static const bool kTrace = [] { const char* e = std::getenv("AIXHIP_TRACE"); return e && e[0] == '1'; }();
#define AIXHIP_TRACE(...) do { if (kTrace) { std::fprintf(stderr, "[aixhip] " __VA_ARGS__); std::fputc('\n', stderr); } } while (0)

// AIXHIP_ROCTX=1: a roctx range around every Device call, every flush of the planner's window and every send-off of the
// calls that wait, named after the operator, so that a profiler's marker trace (rocprofv3 --marker-trace) cuts a step by
// operator.  The marker library is looked up at run time and only then; without the variable a Marker is one branch.
namespace {
struct Roctx {
    int (*push)(const char*){nullptr};
    int (*pop)(){nullptr};
    Roctx()
    {
        const char* e = std::getenv("AIXHIP_ROCTX");
        if (!e || e[0] != '1') return;
        for (const char* name : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so"}) {
            if (void* lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL)) {
                push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
                pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
                if (push && pop) return;
                push = nullptr; pop = nullptr;
            }
        }
        std::fprintf(stderr, "[aixhip] AIXHIP_ROCTX=1 but no roctx library could be loaded: no markers\n");
    }
};
const Roctx& roctx() { static const Roctx r; return r; }
struct Marker {
    explicit Marker(const char* name) : on(roctx().push != nullptr) { if (on) roctx().push(name); }
    ~Marker() { if (on) roctx().pop(); }
    Marker(const Marker&) = delete;
    Marker& operator=(const Marker&) = delete;
    bool on;
};
} // namespace

struct DeviceHIP::Extras {
    std::unordered_set<const void*> graphBlocks;               // bases of the blocks that captured work uses
    std::deque<Cooling> cooling;
    unsigned flushesSinceEvent{0};
    std::unordered_map<std::string, aixk_module*> kernels;     // signature -> compiled kernel
    uint64_t hits{0}, misses{0};
    // working storage of emitFused, kept from kernel to kernel
    std::string key;
    std::vector<uint64_t> args;
    gen::Space space;
    // Consecutive flat kernels of one signature that do not depend on one another (Adam's update of parameter after
    // parameter, aixOptimizer.hpp:112-140; the per-parameter casts of a mixed-precision step) leave as ONE launch: their
    // argument blocks travel in a table, each with a share of the grid (AIXHIP_BATCH_FLAT_KERNELS=0 switches it off).
    struct FlatBatch {
        std::string key;
        aixk_module* single{nullptr};
        aixk_module* many{nullptr};
        size_t words{0};                    // uint64 words per argument block
        std::vector<uint64_t> table;
        std::vector<uint32_t> starts;       // first workgroup of each block's share; the total last
        aixhip::fuse::PointerSet reads, writes;
        uint32_t count() const { return starts.empty() ? 0 : (uint32_t)starts.size() - 1; }
        void clear() { table.clear(); starts.clear(); reads.clear(); writes.clear(); single = many = nullptr; words = 0; }
    } batch;
    std::vector<aixk_fill_item> smallFills;   // consecutive fills of small live buffers (the rank-0 constants of an expression): one launch
    bool batchFlatKernels = [] { const char* e = std::getenv("AIXHIP_BATCH_FLAT_KERNELS"); return !(e && e[0] == '0'); }();
    uint64_t batchedLaunches{0}, batchedKernels{0};
    // row reductions are recorded and fused with the operators around them (AIXHIP_FUSE_ROW_REDUCTIONS=0 switches it off)
    bool fuseRowReductions = [] { const char* e = std::getenv("AIXHIP_FUSE_ROW_REDUCTIONS"); return !(e && e[0] == '0'); }();
    // matmul calls waiting to be issued together (see DeviceHIP::matmul): per group descriptors in three parallel arrays
    // and what the group reads and writes (block starts); `leaves` marks the groups that the call being looked at must
    // come after (see meetsRead / meetsWrite)
    struct Group { std::vector<aixhip_tensor> a, b, out; aixhip::fuse::PointerSet reads, writes; bool leaves{false}; };
    std::array<Group, 8> groups;
    size_t grouped{0};                  // products waiting in all groups
    // sliceSet and argmaxIndicesTo calls waiting to leave as one launch each (see DeviceHIP::sliceSet, argmaxIndicesTo)
    std::vector<aixk_slice_item> slices;
    std::vector<aixk_argmax_item> onehots;
    // reduceTo calls that sum a matrix down its columns (see DeviceHIP::reduceTo): f32, f16 and bf16 wait apart
    std::array<std::vector<aixk_colsum_item>, 3> colsums;
    // second halves of sums over everything (see DeviceHIP::emitFused): one element type at a time
    std::vector<aixk_partials_item> partialSums;
    // what the waiting calls other than products read and write (block starts), so that a new call knows in one lookup
    // whether it may wait beside them; per destination of waiting sliceSet calls, how it was described and the windows
    // written so far
    aixhip::fuse::PointerSet waitReads, waitWrites;
    struct SliceWindows { aixhip_tensor dst; uint64_t dim; std::vector<std::pair<uint64_t, uint64_t>> ranges; };
    std::unordered_map<const void*, SliceWindows> sliceDsts;
    bool anyPending() const { if (grouped || !slices.empty() || !onehots.empty() || !partialSums.empty()) return true; for (const auto& c : colsums) if (!c.empty()) return true; return false; }
    bool anyUses() const { return grouped + waitReads.size() + waitWrites.size() != 0; }
    // A call is about to read p / to write p: does it have to come after something that waits?  The groups of products it
    // has to come after are marked, and only they leave with the other kinds of waiting calls (issuePending(true)): a
    // weight gradient of a backward pass goes on waiting for the other layers' while the small products of attention
    // come and go.  Whoever gets `true` sends the waiting calls off, so that no mark outlives the question.
    const BlockTable* blocks{nullptr};
    // a waiting product may use p: its block counts them (a pointer the table does not know is looked for in every group)
    bool productsMayUse(const void* p) const
    {
        if (!grouped) return false;
        const Block* b = blocks->find(p);
        return !b || b->waiters;
    }
    bool meetsRead(const void* p)
    {
        if (!p) return false;
        bool hit = waitWrites.size() && waitWrites.contains(p);
        if (productsMayUse(p)) for (auto& g : groups) if (!g.out.empty() && g.writes.contains(p)) hit = g.leaves = true;
        return hit;
    }
    bool meetsWrite(const void* p)
    {
        if (!p) return false;
        bool hit = (waitWrites.size() && waitWrites.contains(p)) || (waitReads.size() && waitReads.contains(p));
        if (productsMayUse(p)) for (auto& g : groups) if (!g.out.empty() && (g.writes.contains(p) || g.reads.contains(p))) hit = g.leaves = true;
        return hit;
    }
    // a call that reads r0, r1 and writes w neither uses what waits nor is used by it (every operand is looked at: all
    // groups in its way are marked)
    bool apartFromWaiting(const void* r0, const void* r1, const void* w)
    {
        bool hit = meetsRead(r0);
        hit = meetsRead(r1) || hit;
        hit = meetsWrite(w) || hit;
        return !hit;
    }
    // p is an operand or the result of a call that waits
    bool waitingUses(const void* p) const
    {
        if (!p || !anyUses()) return false;
        if ((waitWrites.size() && waitWrites.contains(p)) || (waitReads.size() && waitReads.contains(p))) return true;
        if (productsMayUse(p)) for (const auto& g : groups) if (!g.out.empty() && (g.writes.contains(p) || g.reads.contains(p))) return true;
        return false;
    }
    void noteWaiting(const void* r0, const void* r1, const void* w)
    {
        if (r0) waitReads.insert(r0);
        if (r1) waitReads.insert(r1);
        waitWrites.insert(w);
    }
    // results of at least this many bytes are written with non-temporal stores (the kernel layer's rule, same override)
    size_t streamStoreMinBytes = [] {
        const char* e = std::getenv("AIXHIP_STREAM_STORE_MIN_BYTES");
        return e && *e ? (size_t)std::strtoull(e, nullptr, 10) : (size_t)AIXK_STREAM_STORE_MIN_BYTES;
    }();
};

// ---- block table -------------------------------------------------------------------------------
DeviceHIP::Block* DeviceHIP::BlockTable::find(const void* base) const
{
    if (m_slots.empty()) return nullptr;
    const uintptr_t key = (uintptr_t)base;
    const size_t mask = m_slots.size() - 1;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i].key == key) return &m_slots[i].block;
        if (m_slots[i].key == 0) return nullptr;
    }
}

const void* DeviceHIP::BlockTable::baseOf(const void* p) const
{
    if (find(p)) return p;
    const uintptr_t a = (uintptr_t)p;
    if (a < m_lo || a >= m_hi) return nullptr;
    for (const auto& s : m_slots) if (s.key > 1 && a >= s.key && a < s.key + s.block.bytes) return (const void*)s.key;
    return nullptr;
}

DeviceHIP::Block* DeviceHIP::BlockTable::findContaining(const void* p) const
{
    const uintptr_t a = (uintptr_t)p;
    if (a < m_lo || a >= m_hi) return nullptr;
    for (const auto& s : m_slots) if (s.key > 1 && a >= s.key && a < s.key + s.block.bytes) return &s.block;
    return nullptr;
}

void DeviceHIP::BlockTable::grow()
{
    std::vector<Slot> old;
    old.swap(m_slots);
    size_t capacity = 256;
    while (capacity < m_count * 4) capacity <<= 1;
    m_slots.assign(capacity, Slot{});
    m_shift = 64;
    for (size_t c = capacity; c > 1; c >>= 1) --m_shift;
    m_used = m_count;
    const size_t mask = capacity - 1;
    for (const auto& s : old) {
        if (s.key <= 1) continue;
        size_t i = slotOf(s.key);
        while (m_slots[i].key != 0) i = (i + 1) & mask;
        m_slots[i] = s;
    }
}

void DeviceHIP::BlockTable::insert(void* base, size_t bytes)
{
    const uintptr_t key = (uintptr_t)base;
    if (key < m_lo) m_lo = key;
    if (key + bytes > m_hi) m_hi = key + bytes;
    if ((m_used + 1) * 2 > m_slots.size()) grow();
    const size_t mask = m_slots.size() - 1;
    size_t grave = SIZE_MAX;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i].key == key) { m_slots[i].block = Block{bytes}; return; }
        if (m_slots[i].key == 1 && grave == SIZE_MAX) grave = i;
        if (m_slots[i].key == 0) {
            if (grave != SIZE_MAX) i = grave; else ++m_used;
            m_slots[i].key = key;
            m_slots[i].block = Block{bytes};
            ++m_count;
            return;
        }
    }
}

bool DeviceHIP::BlockTable::erase(void* base, size_t* bytes)
{
    if (m_slots.empty()) return false;
    const uintptr_t key = (uintptr_t)base;
    const size_t mask = m_slots.size() - 1;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i].key == 0) return false;
        if (m_slots[i].key != key) continue;
        *bytes = m_slots[i].block.bytes;
        // no gravestone: the entries behind it in the probe sequence move up (linear probing allows that), so chains stay
        // as short as the table's load makes them however many blocks come and go
        size_t hole = i;
        for (size_t j = (i + 1) & mask; m_slots[j].key != 0; j = (j + 1) & mask) {
            const size_t home = slotOf(m_slots[j].key);
            // j's entry may move to the hole if its home is not strictly inside (hole, j] (cyclically)
            const bool between = hole <= j ? (home > hole && home <= j) : (home > hole || home <= j);
            if (!between) { m_slots[hole] = m_slots[j]; hole = j; }
        }
        m_slots[hole] = Slot{};
        --m_count;
        --m_used;
        return true;
    }
}

// ---- construction ------------------------------------------------------------------------------
DeviceHIP::DeviceHIP(size_t deviceIndex)
{
    const int rc = aixk_create((int)deviceIndex, &m_ctx);
    if (rc != AIXK_OK) throw std::runtime_error(std::string("DeviceHIP: ") + aixk_last_error());
    aixk_device_info info{};
    if (aixk_info(m_ctx, &info) == AIXK_OK && info.compute_units > 0) m_cus = info.compute_units;
    m_totalBytes = info.total_mem;
    m_cacheLimit = (size_t)((double)info.total_mem * 0.7);
    if (const char* env = std::getenv("AIXHIP_CACHE_LIMIT_BYTES")) m_cacheLimit = (size_t)std::strtoull(env, nullptr, 10);
    if (aixk_info(m_ctx, &info) == AIXK_OK && !info.large_bar)
        std::cerr << "DeviceHIP: device memory is not host-addressable on this system; tensors must be moved with "
                     "copy()/copyToHost() and never dereferenced on the host." << std::endl;
    FuseConfig cfg;
    cfg.maxBufferSlots = 40;                                 // (pointer arguments are cheap here; 24 cut GeLU's backward formula, 11 loads and 6 stores, in two)
    if (const char* e = std::getenv("AIXHIP_MAX_BUFFER_SLOTS"); e && *e) cfg.maxBufferSlots = std::max<size_t>(4, std::min<size_t>(60, std::strtoull(e, nullptr, 10)));
    cfg.supportsStridedFusion = true;
    m_extras = std::make_unique<Extras>();
    m_extras->blocks = &m_blocks;
    setFuseConfig(cfg);
}

DeviceHIP::~DeviceHIP()
{
    try {
        if (m_engine && m_engine->pendingOps() > 0)
            std::cerr << "DeviceHIP: destroyed with recorded work that was never synchronised." << std::endl;   // aixDeviceMetal.cpp:146-149
        if (m_ctx && m_extras && m_extras->anyPending()) issuePending();           // matmul calls still waiting for company
        if (m_engine) m_engine.reset();
        if (m_ctx) {
            if (m_capturing) { m_capturing = false; aixk_capture_abort(m_ctx); }
            aixk_sync(m_ctx);
            auto& ex = *m_extras;
            for (auto& c : ex.cooling) { aixk_event_destroy(m_ctx, c.event); for (auto& b : c.blocks) aixk_free(m_ctx, b.first, 0); }
            for (auto& b : m_limbo) aixk_free(m_ctx, b.first, 0);
            for (auto& kv : m_pool) for (void* p : kv.second) aixk_free(m_ctx, p, 0);
            for (auto& b : m_graphReserve) aixk_free(m_ctx, b.first, 0);
            m_blocks.forEach([this](void* base, const Block& b) { if (!b.freed) aixk_free(m_ctx, base, 0); });
            aixk_destroy(m_ctx);
        }
    } catch (...) {
    }
}

std::unique_ptr<aix::Device> createDeviceHIP(size_t deviceIndex)
{
    try { return std::make_unique<DeviceHIP>(deviceIndex); }
    catch (const std::exception&) { return nullptr; }             // as createDevice() does for an absent GPU (aixDevices.cpp:28-33)
}

void DeviceHIP::setFuseConfig(const FuseConfig& cfg)
{
    if (m_engine) flush();
    FuseCallbacks cb;
    cb.emitFused = [this](const FusedSubgraphDescriptor& d) { emitFused(d); };
    cb.emitSingle = [this](const OpRecord& op) { emitSingle(op); };
    cb.finishFlush = [this] { issueFlatBatch(); };
    cb.getKernelCacheStats = [this] { return fuseKernelCacheStats(); };
    cb.blockBase = [this](const void* p) { return m_blocks.baseOf(p); };
    FuseConfig own = cfg;
    own.loneCastsAsKernels = m_extras->batchFlatKernels;    // so that runs of them leave as one launch (issueFlatBatch)
    own.groupEqualKernels = m_extras->batchFlatKernels;     // and so that such runs form where the program interleaves kinds
    if (const char* e = std::getenv("AIXHIP_FLUSH_THRESHOLD"); e && *e) own.flushThreshold = std::max<size_t>(1, std::strtoull(e, nullptr, 10));
    m_engine = std::make_unique<FuseEngine>(own, std::move(cb));
    m_blocks.forEach([this](void* base, const Block& b) { if (!b.freed) m_engine->retainBuffer(base); });
}

std::pair<size_t, size_t> DeviceHIP::batchedLaunchStats() const
{
    return {(size_t)m_extras->batchedLaunches, (size_t)m_extras->batchedKernels};
}

std::pair<size_t, size_t> DeviceHIP::fuseKernelCacheStats() const
{
    return {(size_t)m_extras->hits, (size_t)m_extras->misses};
}

void DeviceHIP::check(int status) const
{
    if (status == AIXK_OK) return;
    const std::string msg = std::string("DeviceHIP: ") + aixk_last_error();
    if (status == AIXK_EINVAL) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

// ---- memory ------------------------------------------------------------------------------------
const DeviceHIP::Block* DeviceHIP::findBlock(const void* p) const
{
    if (!p || m_blocks.empty()) return nullptr;
    if (const Block* exact = m_blocks.find(p)) return exact;
    return m_blocks.findContaining(p);
}

// 256-byte steps up to 4 KiB, then eight steps per power of two: at most 12.5 % slack, few buckets.
size_t DeviceHIP::bucketBytes(size_t bytes) const
{
    if (bytes < 256) return 256;
    if (bytes <= 4096) return (bytes + 255) & ~(size_t)255;
    size_t top = 1;
    while ((top << 1) <= bytes) top <<= 1;
    const size_t step = top >> 3;
    return (bytes + step - 1) & ~(step - 1);
}

void* DeviceHIP::allocateBlock(size_t bytes, bool track)
{
    auto& ex = *m_extras;
    // blocks whose release point the GPU has passed become reusable
    while (!ex.cooling.empty()) {
        int32_t done = 0;
        if (aixk_event_query(m_ctx, ex.cooling.front().event, &done) != AIXK_OK || !done) break;
        for (auto& b : ex.cooling.front().blocks) pool(b.first, b.second);
        aixk_event_destroy(m_ctx, ex.cooling.front().event);
        ex.cooling.pop_front();
    }
    const size_t bucket = bucketBytes(bytes);
    void* p = nullptr;
    auto it = m_pool.find(bucket);
    if (it != m_pool.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        m_pooledBytes -= bucket;
    } else if (aixk_alloc(m_ctx, bucket, 0, &p) != AIXK_OK) {
        // out of memory: finish everything, give cached blocks back, try once more (aixDeviceMetal.cpp:1455-1471)
        synchronize();
        emptyCache();
        if (aixk_alloc(m_ctx, bucket, 0, &p) != AIXK_OK)
            throw std::runtime_error(std::string("DeviceHIP: GPU memory allocation has failed for size: ") + std::to_string(bytes) + " bytes. " + aixk_last_error());
    }
    if (track) {
        m_blocks.insert(p, bucket);
        m_liveBytes += bucket;
        m_engine->retainBuffer(p);
    }
    return p;
}

void* DeviceHIP::allocate(size_t size) { return allocateBlock(size, true); }

void* DeviceHIP::allocate(size_t size, DataType dtype) { return allocateBlock(size * dataTypeSize(dtype), true); }

void DeviceHIP::deallocate(void* memory)
{
    if (!memory) return;
    Block* block = m_blocks.find(memory);
    if (!block || block->freed) throw std::invalid_argument("DeviceHIP::deallocate() - Found different type of memory to free.");   // aixDeviceMetal.cpp:253-254
    block->freed = true;                                    // stays in the table until the block leaves m_limbo: work recorded on it may still mark it
    const size_t bytes = block->bytes;
    m_engine->releaseBuffer(memory);
    m_limbo.emplace_back(memory, bytes);
    m_limboBytes += bytes;
    m_liveBytes -= bytes;
    if (m_limboBytes > (size_t(8) << 30)) { issuePending(); flushWindow(false); }   // recorded and waiting work pins too much freed memory
}

void DeviceHIP::markTouched(const void* p)
{
    if (!p || m_blocks.empty()) return;
    Block* b = m_blocks.find(p);
    if (!b) b = m_blocks.findContaining(p);
    if (!b) return;
    b->touched = true;
    if (m_capturing && !b->inGraph) {                       // captured work uses the block: it belongs to the graph (see pool())
        b->inGraph = true;
        m_extras->graphBlocks.insert(m_blocks.find(p) ? p : m_blocks.baseOf(p));
    }
}

// Called once the recorded work that might touch freed blocks has been enqueued.
//
// A freed block that no enqueued work has referenced since it was allocated -- a temporary whose
// value stayed in registers of a fused kernel, an absorbed fill -- is idle and goes straight back
// to the pool.  The others wait for the GPU to pass an event.  An event costs a marker packet
// between two kernels (a few microseconds of idle GPU), so it is not recorded after every flush:
// such blocks wait until 16 flushes have passed or until they amount to a thousandth of the card
// (288 MiB of 288 GiB; at least 32 MiB) and an eighth of what the device holds otherwise,
// whichever comes first.
void DeviceHIP::releaseLimbo()
{
    if (m_limbo.empty()) return;
    auto& ex = *m_extras;
    size_t kept = 0, held = 0;
    for (size_t k = 0; k < m_limbo.size(); ++k) {
        const auto entry = m_limbo[k];
        const Block* b = m_blocks.find(entry.first);        // staging blocks are not in the table: always used
        if (ex.waitingUses(entry.first)) {                  // a call that has not been enqueued yet uses it: it stays
            m_limbo[kept++] = entry;
            ++held;
        } else if (b && !b->touched) {
            size_t bytes = 0;
            m_blocks.erase(entry.first, &bytes);
            pool(entry.first, entry.second);
            m_limboBytes -= entry.second;
        } else {
            m_limbo[kept++] = entry;
        }
    }
    m_limbo.resize(kept);
    if (m_limbo.empty()) return;

    const size_t enough = std::max<size_t>({size_t(32) << 20, m_totalBytes >> 10, (m_liveBytes + m_pooledBytes) / 8});
    if (!m_capturing && ++ex.flushesSinceEvent < 16 && m_limboBytes < enough) return;      // (inside a capture no event is needed: see below)
    ex.flushesSinceEvent = 0;
    std::vector<std::pair<void*, size_t>> stay, leave;
    if (held) {
        for (const auto& entry : m_limbo) (ex.waitingUses(entry.first) ? stay : leave).push_back(entry);
        if (leave.empty()) return;
    } else {
        leave.swap(m_limbo);
    }
    size_t stayBytes = 0;
    for (const auto& entry : stay) stayBytes += entry.second;
    for (const auto& entry : leave) { size_t bytes = 0; m_blocks.erase(entry.first, &bytes); }
    Cooling c{};
    if (m_capturing) {
        // nothing runs while the stream records, and what is recorded runs in stream order: a freed block may be used
        // again by work captured later (the host does not write into blocks while it captures)
        for (auto& b : leave) pool(b.first, b.second);
    } else if (aixk_event_create(m_ctx, &c.event) == AIXK_OK && aixk_event_record(m_ctx, c.event) == AIXK_OK) {
        c.blocks.swap(leave);
        ex.cooling.push_back(std::move(c));
    } else {
        aixk_sync(m_ctx);
        for (auto& b : leave) pool(b.first, b.second);
    }
    m_limbo.swap(stay);
    m_limboBytes = stayBytes;
}

void DeviceHIP::emptyCache()
{
    const Marker marker_("emptyCache");
    for (auto& kv : m_pool) for (void* p : kv.second) aixk_free(m_ctx, p, 0);
    m_pool.clear();
    m_pooledBytes = 0;
}

void DeviceHIP::flush() { flushWindow(true); }

// final: nothing recorded stays behind.  Otherwise fills that nothing recorded so far uses may wait (FuseEngine::flush).
void DeviceHIP::flushWindow(bool final)
{
    const Marker marker_("flush");
    // Calls that wait (small products, sliceSet, one-hot masks, column sums) stay waiting across a flush: they depend on nothing
    // recorded (their callers saw to that), and a kernel that leaves now and uses what they write, or writes what they
    // use, sends them off first (emitFused, emitSingle).
    if (final) issuePending();
    try { m_engine->flush(final); }
    catch (...) { m_extras->batch.clear(); m_extras->smallFills.clear(); throw; }
    if (final) issuePending();                              // (one-hot operators replayed on their own wait as well: emitSingle)
    releaseLimbo();
}

void DeviceHIP::flushFor(const void* a, const void* b, const void* c) { flushForOperands(a, b, c, false); }

// An operator is about to be enqueued at once on these operands -- the last one named is the one it writes (or the only
// one, which it may write), the others are read.  Recorded operators go first only if one of them writes what it reads
// or uses what it writes (`always`: whatever they touch), and so do the calls that wait; all others may as well run after
// it, which keeps the window -- and the kernels fused from it -- whole.
void DeviceHIP::flushForOperands(const void* a, const void* b, const void* c, bool always)
{
    AIXHIP_TRACE("-- operator outside the planner (%zu recorded)", m_engine->pendingOps());
    const void* named[3] = {a, b, c};
    const void* bases[3] = {nullptr, nullptr, nullptr};
    const int last = c ? 2 : b ? 1 : 0;
    bool dependent = always;
    for (int k = 0; k < 3; ++k) {
        const void* p = named[k];
        if (!p) continue;
        const void* base = m_blocks.baseOf(p);              // an operand may point into the middle of a block
        if (base && base != p) { bases[k] = base; dependent = true; }
        if (!dependent) dependent = k == last ? m_engine->pendingTouches(p) : m_engine->pendingWrites(p);
    }
    markTouched(a);                                         // the caller is about to enqueue work on them
    markTouched(b);
    markTouched(c);
    auto& ex = *m_extras;
    auto meets = [&] {                                      // (every operand is asked about: all the groups in the way are marked)
        bool any = false;
        if (!ex.anyUses()) return any;
        for (int k = 0; k < 3; ++k) {
            if (k == last) { any = ex.meetsWrite(named[k]) || any; any = ex.meetsWrite(bases[k]) || any; }
            else           { any = ex.meetsRead(named[k]) || any;  any = ex.meetsRead(bases[k]) || any; }
        }
        return any;
    };
    if (meets()) issuePending(true);
    if (!dependent) return;
    for (int k = 0; k < 3; ++k) {
        if (named[k]) m_engine->recordExternalRead(named[k]);
        if (bases[k]) m_engine->recordExternalRead(bases[k]);
    }
    flushWindow(false);
    if (meets()) issuePending(true);                        // (a one-hot replayed on its own has just begun to wait)
}

// The planner orders recorded operators by the addresses of their buffers.  An operand that points into the middle of
// a block (pointer arithmetic by a caller of the C ABI; the front-end names a block's start and an offset) would escape
// that: operators with such an operand are recorded into a window of their own.
bool DeviceHIP::fenceInterior(const void* a, const void* b, const void* c)
{
    bool any = false;
    for (const void* p : {a, b, c}) if (p && !m_blocks.find(p) && m_blocks.baseOf(p)) any = true;
    if (any) flushForOperands(a, b, c, true);
    return any;
}

void DeviceHIP::synchronize()
{
    const Marker marker_("synchronize");
    if (m_capturing) throw std::runtime_error("DeviceHIP::synchronize: nothing runs while a capture is open (endCapture() first)");
    flush();
    check(aixk_sync(m_ctx));
    auto& ex = *m_extras;
    for (auto& c : ex.cooling) {
        for (auto& b : c.blocks) pool(b.first, b.second);
        aixk_event_destroy(m_ctx, c.event);
    }
    ex.cooling.clear();
    // everything recorded has been enqueued and has finished: blocks freed since the last event are idle too
    for (auto& b : m_limbo) { size_t bytes = 0; m_blocks.erase(b.first, &bytes); pool(b.first, b.second); }
    m_limbo.clear();
    m_limboBytes = 0;
    ex.flushesSinceEvent = 0;
    trimPool();
}

// An idle block goes back to its bucket -- unless a graph's kernels use it: then only work captured into a graph may
// have it again (inside a capture, where everything is ordered on the stream), and once the capture is closed it is kept
// aside for as long as a graph lives.
void DeviceHIP::pool(void* p, size_t bytes)
{
    if (!m_capturing && m_graphs && m_extras->graphBlocks.count(p)) { m_graphReserve.emplace_back(p, bytes); return; }
    m_pool[bytes].push_back(p);
    m_pooledBytes += bytes;
}

void DeviceHIP::beginCapture()
{
    if (m_capturing) throw std::runtime_error("DeviceHIP::beginCapture: a capture is already open");
    synchronize();                                          // everything pending runs, every freed block is idle and pooled
    check(aixk_capture_begin(m_ctx));
    m_capturing = true;
}

DeviceHIP::StepGraph* DeviceHIP::endCapture()
{
    if (!m_capturing) throw std::runtime_error("DeviceHIP::endCapture: no capture is open");
    aixk_graph* g = nullptr;
    try {
        flushWindow(true);                                  // what is still recorded or waiting belongs to the graph
        releaseLimbo();
    } catch (...) { m_capturing = false; aixk_capture_abort(m_ctx); throw; }
    m_capturing = false;
    check(aixk_capture_end(m_ctx, &g));
    ++m_graphs;
    // blocks the captured work uses and that are idle now: aside (they were free to go round inside the capture)
    auto& used = m_extras->graphBlocks;
    for (auto& kv : m_pool) {
        auto& stack = kv.second;
        size_t kept = 0;
        for (size_t k = 0; k < stack.size(); ++k) {
            if (used.count(stack[k])) { m_graphReserve.emplace_back(stack[k], kv.first); m_pooledBytes -= kv.first; }
            else stack[kept++] = stack[k];
        }
        stack.resize(kept);
    }
    // (blocks still in limbo are set aside when their turn to be pooled comes: pool())
    return reinterpret_cast<StepGraph*>(g);
}

// An open capture given up: what is still recorded or waits is flushed into the graph like at endCapture() -- nothing runs --
// and the graph is thrown away.  The results of the abandoned stretch are undefined.
void DeviceHIP::abortCapture()
{
    if (!m_capturing) return;
    StepGraph* g = nullptr;
    try { g = endCapture(); } catch (...) { g = nullptr; }   // (a failing flush has ended the capture itself)
    if (g) destroyGraph(g);
}

void DeviceHIP::replay(StepGraph* graph)
{
    if (m_capturing) throw std::runtime_error("DeviceHIP::replay: a capture is open");
    if (!graph) throw std::invalid_argument("DeviceHIP::replay: null graph");
    flushWindow(true);                                      // pending work first: the graph's kernels may read its results
    check(aixk_graph_launch(m_ctx, reinterpret_cast<aixk_graph*>(graph)));
}

size_t DeviceHIP::graphNodes(const StepGraph* graph) const
{
    uint64_t n = 0;
    if (graph) aixk_graph_nodes(reinterpret_cast<aixk_graph*>(const_cast<StepGraph*>(graph)), &n);
    return (size_t)n;
}

void DeviceHIP::destroyGraph(StepGraph* graph)
{
    if (!graph) return;
    aixk_graph_destroy(m_ctx, reinterpret_cast<aixk_graph*>(graph));      // waits for the stream
    if (m_graphs && --m_graphs == 0) {
        // no graph is left that could write into them: the blocks set aside are ordinary idle blocks again
        for (auto& b : m_graphReserve) { m_pool[b.second].push_back(b.first); m_pooledBytes += b.second; }
        m_graphReserve.clear();
        m_extras->graphBlocks.clear();
        m_blocks.forEach([](void*, Block& b) { b.inGraph = false; });
    }
}

// Idle blocks beyond the cache limit go back to the driver (aixDeviceMetal.cpp:1369-1373, aixDeviceMetalCache.hpp:97-124:
// the least recently used first).  Called with the GPU idle.  Every bucket is a stack whose top is handed out first, so
// its bottom is its coldest block; buckets are taken in the order of the bytes they hold, the fullest first.
void DeviceHIP::trimPool()
{
    while (m_pooledBytes > m_cacheLimit) {
        std::vector<void*>* fullest = nullptr;
        size_t bucket = 0, most = 0;
        for (auto& kv : m_pool)
            if (kv.first * kv.second.size() > most) { most = kv.first * kv.second.size(); fullest = &kv.second; bucket = kv.first; }
        if (!fullest) break;
        // enough of its cold end to get under the limit, or all of it
        const size_t over = m_pooledBytes - m_cacheLimit;
        const size_t count = std::min(fullest->size(), (over + bucket - 1) / bucket);
        for (size_t k = 0; k < count; ++k) aixk_free(m_ctx, (*fullest)[k], 0);
        fullest->erase(fullest->begin(), fullest->begin() + (std::ptrdiff_t)count);
        m_pooledBytes -= count * bucket;
    }
}

void DeviceHIP::copyToHost(void* dstHost, const void* srcDevice, size_t bytes)
{
    const Marker marker_("copyToHost");
    flushFor(srcDevice);
    check(aixk_copy_out(m_ctx, dstHost, srcDevice, bytes));
}

void DeviceHIP::copyFromHost(void* dstDevice, const void* srcHost, size_t bytes)
{
    const Marker marker_("copyFromHost");
    if (!findBlock(dstDevice)) throw std::invalid_argument("DeviceHIP::copyFromHost() result must have GPU memory.");
    flushFor(dstDevice);
    check(aixk_copy_in(m_ctx, dstDevice, srcHost, bytes));
}

// ---- operand handling --------------------------------------------------------------------------
void DeviceHIP::requireDevice(const DeviceTensorParams& result, const char* op) const
{
    if (result.size > 0 && !findBlock(result.data))
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() result must have GPU memory.");      // aixDeviceMetal.cpp:305-306
}

const void* DeviceHIP::stageRaw(const void* src, size_t bytes)
{
    void* tmp = allocateBlock(bytes, false);
    check(aixk_copy_in(m_ctx, tmp, src, bytes));
    m_limbo.emplace_back(tmp, bucketBytes(bytes));          // recycled after the work that reads it is enqueued
    m_limboBytes += bucketBytes(bytes);
    return tmp;
}

void DeviceHIP::onDevice(View& v)
{
    if (!v.data || v.size == 0 || findBlock(v.data)) return;
    // a host tensor handed straight to the device (DeviceTests.cpp:209-215)
    v.data = const_cast<void*>(stageRaw(v.data, viewEnd(v) * dataTypeSize(v.dtype)));
}

void DeviceHIP::toPod(const DeviceTensorParams& p, aixhip_tensor* out, const char* op) const
{
    if (p.shape.size() > AIXK_MAX_RANK)
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() supports at most 16 dimensions.");    // aixDeviceMetal.cpp:671-672
    std::memset(out, 0, sizeof(*out));
    out->data = p.data;
    out->dtype = (int32_t)p.dtype;
    out->rank = (int32_t)p.shape.size();
    out->offset = p.offset;
    out->size = p.size;
    for (size_t d = 0; d < p.shape.size(); ++d) { out->shape[d] = p.shape[d]; out->strides[d] = d < p.strides.size() ? p.strides[d] : 0; }
}

void DeviceHIP::toPod(const View& v, aixhip_tensor* out) const
{
    std::memset(out, 0, sizeof(*out));
    out->data = v.data;
    out->dtype = (int32_t)v.dtype;
    out->rank = (int32_t)v.rank;
    out->offset = v.offset;
    out->size = v.size;
    for (size_t d = 0; d < v.rank; ++d) { out->shape[d] = v.shape[d]; out->strides[d] = v.strides[d]; }
}

void DeviceHIP::stagedPod(const DeviceTensorParams& p, aixhip_tensor* out, const char* op)
{
    toPod(p, out, op);
    if (!out->data || out->size == 0 || findBlock(out->data)) return;
    out->data = const_cast<void*>(stageRaw(out->data, viewEnd(*out) * dataTypeSize(p.dtype)));
}

// ---- recorded (fusable) operators --------------------------------------------------------------
void DeviceHIP::recordBinary(OpType t, const DeviceTensorParams& a, const DeviceTensorParams& b, const DeviceTensorParams& r, const char* op)
{
    const Marker marker_(op);
    requireDevice(r, op);
    if (a.dtype != r.dtype || b.dtype != r.dtype)
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() operands must have the result's data type.");
    if (a.shape.size() > AIXK_MAX_RANK || b.shape.size() > AIXK_MAX_RANK || r.shape.size() > AIXK_MAX_RANK)
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() supports at most 16 dimensions.");
    View va(a), vb(b), out(r);
    out.makeDense();                                        // results are written densely from the base pointer
    onDevice(va);
    onDevice(vb);
    if (va.rank > (uint32_t)gen::kMaxDims || vb.rank > (uint32_t)gen::kMaxDims) {
        // generated kernels index at most 8 collapsed dimensions; views of higher rank (which may not collapse
        // that far) run on the precompiled operator, which takes all 16
        flushFor(va.data, vb.data, out.data);
        aixhip_tensor pa, pb, po;
        toPod(va, &pa); toPod(vb, &pb); toPod(out, &po);
        check(aixk_binary(m_ctx, binaryCode(t), &pa, &pb, &po));
        return;
    }
    const bool fenced = fenceInterior(va.data, vb.data, out.data);
    m_engine->record(t, va, vb, out);
    if (fenced) flushForOperands(out.data, nullptr, nullptr, true);                         // (names the result: somebody may read it through the block's start)
}

void DeviceHIP::recordUnary(OpType t, const DeviceTensorParams& a, const DeviceTensorParams& r, const char* op)
{
    const Marker marker_(op);
    requireDevice(r, op);
    if (a.dtype != r.dtype)
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() operand must have the result's data type.");
    if (a.shape.size() > AIXK_MAX_RANK || r.shape.size() > AIXK_MAX_RANK)
        throw std::invalid_argument(std::string("DeviceHIP::") + op + "() supports at most 16 dimensions.");
    View va(a), out(r);
    out.size = a.size;                                      // unary loops run over the operand (aixDeviceCPU.cpp:90)
    if (!out.sameShape(va)) { out.rank = va.rank; std::memcpy(out.shape, va.shape, va.rank * sizeof(size_t)); }
    out.makeDense();
    onDevice(va);
    if (va.rank > (uint32_t)gen::kMaxDims) {
        flushFor(va.data, out.data);
        aixhip_tensor pa, po;
        toPod(va, &pa); toPod(out, &po);
        check(aixk_unary(m_ctx, unaryCode(t), &pa, &po));
        return;
    }
    const bool fenced = fenceInterior(va.data, out.data);
    m_engine->record(t, va, out);
    if (fenced) flushForOperands(out.data, nullptr, nullptr, true);
}

void DeviceHIP::add(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) { recordBinary(OpType::Add, a1, a2, result, "add"); }
void DeviceHIP::sub(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) { recordBinary(OpType::Sub, a1, a2, result, "sub"); }
void DeviceHIP::mul(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) { recordBinary(OpType::Mul, a1, a2, result, "mul"); }
void DeviceHIP::div(const DeviceTensorParams& a1, const DeviceTensorParams& a2, const DeviceTensorParams& result) { recordBinary(OpType::Div, a1, a2, result, "div"); }
void DeviceHIP::pow(const DeviceTensorParams& a, const DeviceTensorParams& e, const DeviceTensorParams& result) { recordBinary(OpType::Pow, a, e, result, "pow"); }
void DeviceHIP::unary(const DeviceTensorParams& a1, const DeviceTensorParams& result) { recordUnary(OpType::Negate, a1, result, "unary"); }
void DeviceHIP::sqrt(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Sqrt, a, result, "sqrt"); }
void DeviceHIP::sin(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Sin, a, result, "sin"); }
void DeviceHIP::cos(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Cos, a, result, "cos"); }
void DeviceHIP::tanh(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Tanh, a, result, "tanh"); }
void DeviceHIP::log(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Log, a, result, "log"); }
void DeviceHIP::exp(const DeviceTensorParams& a, const DeviceTensorParams& result) { recordUnary(OpType::Exp, a, result, "exp"); }

void DeviceHIP::fill(const void* scalar, DataType scalarDType, const DeviceTensorParams& result)
{
    const Marker marker_("fill");
    requireDevice(result, "fill");
    View out(result);
    out.makeDense();
    const bool fenced = fenceInterior(out.data);
    m_engine->recordFill(scalar, scalarDType, out);
    if (fenced) flushForOperands(out.data, nullptr, nullptr, true);
}

void DeviceHIP::fillMin(const DeviceTensorParams& result)
{
    const Marker marker_("fillMin");
    requireDevice(result, "fillMin");
    View out(result);
    out.makeDense();
    const bool fenced = fenceInterior(out.data);
    m_engine->recordFillMin(out);
    if (fenced) flushForOperands(out.data, nullptr, nullptr, true);
}

// ---- planner callbacks -------------------------------------------------------------------------
void DeviceHIP::emitSingle(const OpRecord& op)
{
    const bool smallFill = (op.type == OpType::Fill || op.type == OpType::FillMin) && op.output.dense && op.output.size <= 65536 && m_extras->batchFlatKernels;
    if (!smallFill || m_extras->batch.count()) issueFlatBatch();            // (a fill joins the fills before it)
    if (op.type == OpType::ArgmaxIndicesTo) {
        // a recorded one-hot that found no company: the stand-alone operator with the zero fill folded in; several in a
        // row wait for each other and leave in one launch (see argmaxIndicesTo())
        auto& ex = *m_extras;
        AIXHIP_TRACE("single %s  %zu elements", aixhip::fuse::opName(op.type), op.output.size);
        const bool apart = ex.apartFromWaiting(op.input0.data, nullptr, op.output.data);
        if (ex.onehots.size() >= AIXK_ARGMAX_ITEMS_MAX || !ex.batchFlatKernels || !apart) issuePending(true);
        aixk_argmax_item item{};
        toPod(op.input0, &item.src); toPod(op.output, &item.dst);
        item.dim = op.input0.rank - 1;
        ex.onehots.push_back(item);
        ex.noteWaiting(op.input0.data, nullptr, op.output.data);
        markTouched(op.input0.data); markTouched(op.output.data);
        if (!ex.batchFlatKernels) issuePending();
        return;
    }
    {
        auto& ex = *m_extras;                               // what waits and is used here, or uses the result's buffer, goes first
        if (ex.anyUses() && !ex.apartFromWaiting(op.input0.data, op.hasInput1 ? op.input1.data : nullptr, op.output.data)) issuePending(true);
    }
    AIXHIP_TRACE("single %s  %zu elements", aixhip::fuse::opName(op.type), op.output.size);
    if ((op.type == OpType::Fill || op.type == OpType::FillMin) && op.output.dense && op.output.size <= 65536 && m_extras->batchFlatKernels) {
        // small fills that follow one another leave together (issueFlatBatch sends them off ahead of whatever comes next)
        aixk_fill_item item{};
        uint8_t bytes[8] = {};
        const size_t esz = op.type == OpType::Fill ? aixhip::fuse::convertScalarInto(op.scalarData.data(), op.scalarDType, op.output.dtype, bytes)
                                                   : aixhip::fuse::lowestScalarInto(op.output.dtype, bytes);
        std::memcpy(&item.bits, bytes, esz);
        item.dst = (char*)op.output.data + op.output.offset * esz;
        item.elements = (uint32_t)op.output.size;
        item.element_size = (uint32_t)esz;
        markTouched(op.output.data);
        for (const auto& f : m_extras->smallFills)
            if (f.dst == item.dst) { issueFlatBatch(); break; }             // a second fill of the same buffer comes after the first
        m_extras->smallFills.push_back(item);
        return;
    }
    aixhip_tensor a, b, o;
    markTouched(op.output.data);
    markTouched(op.input0.data);
    if (op.hasInput1) markTouched(op.input1.data);
    toPod(op.output, &o);
    if (op.type == OpType::Cast) {
        check(aixk_cast(m_ctx, (const char*)op.input0.data + op.input0.offset * dataTypeSize(op.input0.dtype), (int)op.input0.dtype,
                        (char*)op.output.data + op.output.offset * dataTypeSize(op.output.dtype), (int)op.output.dtype, op.output.size));
        return;
    }
    if (op.type == OpType::Fill) { check(aixk_fill(m_ctx, op.scalarData.data(), (int)op.scalarDType, &o)); return; }
    if (op.type == OpType::FillMin) { check(aixk_fill_min(m_ctx, &o)); return; }
    toPod(op.input0, &a);
    if (aixhip::fuse::isRowReduce(op.type)) {               // a recorded row reduction that found no company: the stand-alone kernel
        uint64_t init = 0;
        std::memcpy(&init, op.scalarData.data(), dataTypeSize(op.output.dtype));
        check(aixk_reduce_to_init(m_ctx, op.type == OpType::ReduceTo ? AIXK_SUM : AIXK_MAX, &a, &o, init));
        return;
    }
    if (op.type == OpType::Tril || op.type == OpType::Triu) { check(aixk_tri(m_ctx, op.type == OpType::Triu ? 1 : 0, &a, &o, op.triDiagonal)); return; }
    if (const int code = binaryCode(op.type); code >= 0) {
        toPod(op.input1, &b);
        check(aixk_binary(m_ctx, code, &a, &b, &o));
        return;
    }
    if (const int code = unaryCode(op.type); code >= 0) { check(aixk_unary(m_ctx, code, &a, &o)); return; }
    throw std::runtime_error(std::string("DeviceHIP: operator cannot be replayed: ") + aixhip::fuse::opName(op.type));
}

void DeviceHIP::emitFused(const FusedSubgraphDescriptor& d)
{
    {
        // calls that wait stay waiting unless this kernel reads what they write or writes what they use
        auto& ex = *m_extras;
        bool meets = false;
        if (ex.anyUses()) {
            for (const auto& v : d.inputBuffers) meets = ex.meetsRead(v.data) || meets;
            for (const auto& v : d.outputBuffers) meets = ex.meetsWrite(v.data) || meets;
        }
        if (meets) issuePending(true);
    }
    constexpr size_t kMaxOperands = 64;
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size();
    const size_t esz = dataTypeSize(d.dtype);
    const size_t VEC = 16 / esz;
    const uint64_t n = d.elementCount;
    if (n == 0 || NO == 0) return;
    const size_t rank = d.shape.size();
    if (NI + 1 > kMaxOperands || NO > kMaxOperands || rank > aixhip::fuse::kMaxRank)
        throw std::invalid_argument("DeviceHIP: fused kernel with too many operands or dimensions.");
    if (d.rowLength) { emitRowProgram(d); return; }

    // Joint iteration space over the fused shape: dense views get the dense strides of that shape
    // (their own shape may be a different factorisation of the same count), strided views keep
    // theirs; one extra dense operand stands for the outputs so dims merge only where they may.
    size_t dense[aixhip::fuse::kMaxRank];
    { size_t run = 1; for (size_t dd = rank; dd-- > 0;) { dense[dd] = run; run *= d.shape[dd]; } }
    const size_t* strides[kMaxOperands];
    for (size_t k = 0; k < NI; ++k) {
        const auto& v = d.inputBuffers[k];
        if (v.dense) strides[k] = dense;
        else if (v.sameShape(d.shape)) strides[k] = v.strides;
        else throw std::runtime_error("DeviceHIP: fused kernel received a strided view of a foreign shape");
    }
    strides[NI] = dense;
    // collapse: drop extent-1 dims, merge neighbours where every operand allows it
    uint64_t shp[aixhip::fuse::kMaxRank];
    uint64_t str[kMaxOperands][aixhip::fuse::kMaxRank];
    size_t cr = 0;
    for (size_t dd = 0; dd < rank; ++dd) {
        if (d.shape[dd] == 1) continue;
        bool merged = false;
        if (cr > 0) {
            bool ok = true;
            for (size_t k = 0; k <= NI; ++k) if (str[k][cr - 1] != strides[k][dd] * d.shape[dd]) ok = false;
            if (ok) {
                shp[cr - 1] *= d.shape[dd];
                for (size_t k = 0; k <= NI; ++k) str[k][cr - 1] = strides[k][dd];
                merged = true;
            }
        }
        if (!merged) {
            shp[cr] = d.shape[dd];
            for (size_t k = 0; k <= NI; ++k) str[k][cr] = strides[k][dd];
            ++cr;
        }
    }
    if (cr > (size_t)gen::kMaxDims) throw std::invalid_argument("DeviceHIP: fused view does not collapse to 8 dimensions.");

    auto aligned = [](const void* p) { return ((uintptr_t)p & 15u) == 0; };
    const void* inPtr[kMaxOperands];
    void* outPtr[kMaxOperands];
    bool outsAligned = true;
    for (size_t k = 0; k < NO; ++k) { outPtr[k] = d.outputBuffers[k].data; if (!aligned(outPtr[k])) outsAligned = false; }
    for (size_t k = 0; k < NO; ++k) markTouched(d.outputBuffers[k].data);
    for (size_t k = 0; k < NI; ++k) markTouched(d.inputBuffers[k].data);

    gen::Shape shape = gen::Shape::Gather;
    uint32_t bmask = 0;
    uint64_t chunks = 0;
    if (cr <= 1) {
        bool ok = outsAligned;
        for (size_t k = 0; k < NI && ok; ++k) {
            const uint64_t s = cr ? str[k][0] : 0;
            const char* base = (const char*)d.inputBuffers[k].data + d.inputBuffers[k].offset * dataTypeSize(d.inputBuffers[k].dtype);
            if (cr == 1 && s == 0) { if (k < 32) bmask |= 1u << k; else ok = false; }
            else if (cr == 1 && s != 1) ok = false;
            else if (!aligned(base)) ok = false;
        }
        if (ok) shape = gen::Shape::Flat;
        else bmask = 0;
    } else {
        bool ok = outsAligned && shp[cr - 1] % VEC == 0;
        for (size_t k = 0; k < NI && ok; ++k) {
            const uint64_t s = str[k][cr - 1];
            if (s > 1) ok = false;
            if (s == 1) {
                const char* base = (const char*)d.inputBuffers[k].data + d.inputBuffers[k].offset * dataTypeSize(d.inputBuffers[k].dtype);
                if (!aligned(base)) ok = false;
                for (size_t dd = 0; dd + 1 < cr; ++dd) if (str[k][dd] % VEC) ok = false;
            }
        }
        if (ok) { shape = gen::Shape::Rows; chunks = shp[cr - 1] / VEC; }
    }

    auto& ex = *m_extras;
    gen::Space& space = ex.space;
    if (shape == gen::Shape::Flat) {
        for (size_t k = 0; k < NI; ++k) inPtr[k] = (const char*)d.inputBuffers[k].data + d.inputBuffers[k].offset * dataTypeSize(d.inputBuffers[k].dtype);
    } else {
        space.rank = (uint32_t)cr;
        for (int dd = 0; dd < gen::kMaxDims; ++dd) space.shape[dd] = dd < (int)cr ? shp[dd] : 1;
        space.offset.resize(NI);
        space.stride.resize(NI);
        for (size_t k = 0; k < NI; ++k) {
            inPtr[k] = d.inputBuffers[k].data;
            space.offset[k] = d.inputBuffers[k].offset;
            for (int dd = 0; dd < gen::kMaxDims; ++dd) space.stride[k][dd] = dd < (int)cr ? str[k][dd] : 0;
        }
    }

    bool noAlias = true;                                     // in-place updates: an output that is also an input
    for (const auto& ob : d.outputBuffers) for (const auto& ib : d.inputBuffers) if (ob.data == ib.data) noAlias = false;
    size_t storedBytes = 0;                                  // large results leave through non-temporal stores
    for (const auto& ob : d.outputBuffers) if (ob.size > 1 || n == 1) storedBytes += n * dataTypeSize(ob.dtype);      // (a sum over everything stores next to nothing)
    const bool streamOut = storedBytes >= ex.streamStoreMinBytes;
    gen::signatureInto(ex.key, d, shape, bmask, noAlias, streamOut);
    aixk_module* mod = nullptr;
    auto it = ex.kernels.find(ex.key);
    if (it != ex.kernels.end()) { mod = it->second; ++ex.hits; }
    else {
        int32_t cached = 0;
        const std::string src = gen::source(d, shape, bmask, noAlias, streamOut);
        check(aixk_rtc_get(m_ctx, ex.key.c_str(), src.c_str(), gen::entryName(d, shape).c_str(), &mod, &cached));
        ex.kernels.emplace(ex.key, mod);
        ++ex.misses;
    }

    uint64_t items, perBlock, cap;
    if (shape == gen::Shape::Flat) { items = n / VEC + 1; perBlock = gen::kBlock; cap = 1u << 22; }
    else if (shape == gen::Shape::Rows) { items = n / VEC; perBlock = gen::kBlock; cap = (uint64_t)m_cus * 64; }
    else { items = n; perBlock = gen::kBlock; cap = (uint64_t)m_cus * 64; }
    uint64_t grid = (items + perBlock - 1) / perBlock;
    grid = std::max<uint64_t>(1, std::min(grid, cap));

    // Sums over everything (FuseEngine::recordWholeSum): the kernel leaves one partial sum per workgroup in scratch
    // memory -- its "output" pointer -- and aixk_sum_partials lands their sum in the destination afterwards.
    struct Whole { size_t output; void* scratch; uint64_t init; };
    Whole wholes[8];
    size_t nWholes = 0;
    for (const auto& op : d.ops) {
        if (!op.whole || op.outputIndex == SIZE_MAX) continue;
        if (nWholes == 8) throw std::logic_error("DeviceHIP: more sums over everything in one kernel than the planner allows");
        const size_t wide = d.dtype == DataType::kFloat64 ? 8 : 4;
        issueFlatBatch();                                        // (an allocation that runs out of memory waits for the GPU and drops the pool: nothing enqueued may lag behind)
        void* scratch = allocateBlock(grid * wide, false);
        m_limbo.emplace_back(scratch, bucketBytes(grid * wide));     // recycled once the work enqueued below has passed
        m_limboBytes += bucketBytes(grid * wide);
        uint64_t init = 0;
        std::memcpy(&init, d.scalarData.data() + op.scalarIndex1 * esz, esz);
        wholes[nWholes++] = Whole{op.outputIndex, scratch, init};
        outPtr[op.outputIndex] = scratch;
    }
    gen::packArgsInto(ex.args, d, shape, inPtr, outPtr, n, shape == gen::Shape::Flat ? nullptr : &space, chunks);

    AIXHIP_TRACE("%s  %llu elements, %zu in %zu out", gen::entryName(d, shape).c_str(), (unsigned long long)n, NI, NO);
    if (ex.batchFlatKernels && nWholes == 0) {
        joinBatch(d, mod, gen::entryName(d, shape), grid, [&] { return gen::source(d, shape, bmask, noAlias, streamOut, true); });
        return;
    }
    issueFlatBatch();
    check(aixk_rtc_launch(m_ctx, mod, (uint32_t)grid, gen::kBlock, ex.args.data(), ex.args.size() * sizeof(uint64_t)));
    for (size_t k = 0; k < nWholes; ++k) {
        aixhip_tensor dst;
        toPod(d.outputBuffers[wholes[k].output], &dst);
        if (!ex.batchFlatKernels) { check(aixk_sum_partials(m_ctx, wholes[k].scratch, grid, &dst, wholes[k].init)); continue; }
        // the second half waits like a small product: the scalar gradients of a backward pass are read when it reaches
        // its leaves, and leave together then (the partial sums' block stays in limbo until they have: releaseLimbo)
        const bool apart = ex.apartFromWaiting(wholes[k].scratch, nullptr, dst.data);
        if (ex.partialSums.size() >= AIXK_PARTIALS_ITEMS_MAX || (!ex.partialSums.empty() && ex.partialSums[0].dst.dtype != dst.dtype) || !apart)
            issuePending(true);
        ex.partialSums.push_back(aixk_partials_item{wholes[k].scratch, grid, dst, wholes[k].init});
        ex.noteWaiting(wholes[k].scratch, nullptr, dst.data);
        markTouched(dst.data);
    }
}

// The kernel whose signature is in Extras::key and whose argument block is in Extras::args joins the kernels waiting to
// leave together -- same kernel, reads nothing they write, writes nothing they read or write -- or sends them off and
// starts the next run.  manySource gives the text of the kernel's many-blocks form when that has to be compiled.
void DeviceHIP::joinBatch(const FusedSubgraphDescriptor& d, aixk_module* mod, const std::string& entry, uint64_t grid, const std::function<std::string()>& manySource)
{
    auto& ex = *m_extras;
    auto& B = ex.batch;
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size();
    bool joins = B.count() != 0 && B.key == ex.key && B.count() < 256 && (uint64_t)B.starts.back() + grid < (1u << 30) &&
                 (B.table.size() + ex.args.size()) * sizeof(uint64_t) < (200u << 10);
    if (joins) {
        for (size_t k = 0; k < NI && joins; ++k) if (B.writes.contains(d.inputBuffers[k].data)) joins = false;
        for (size_t k = 0; k < NO && joins; ++k)
            if (B.writes.contains(d.outputBuffers[k].data) || B.reads.contains(d.outputBuffers[k].data)) joins = false;
    }
    if (!joins) issueFlatBatch();
    if (B.count() == 0) { B.key = ex.key; B.single = mod; B.words = ex.args.size(); B.starts.push_back(0); }
    else if (!B.many) {
        ex.key += "|many";
        auto many = ex.kernels.find(ex.key);
        if (many != ex.kernels.end()) { B.many = many->second; ++ex.hits; }
        else {
            int32_t cached = 0;
            const std::string src = manySource();
            check(aixk_rtc_get(m_ctx, ex.key.c_str(), src.c_str(), (entry + "_many").c_str(), &B.many, &cached));
            ex.kernels.emplace(ex.key, B.many);
            ++ex.misses;
        }
    }
    B.table.insert(B.table.end(), ex.args.begin(), ex.args.end());
    B.starts.push_back(B.starts.back() + (uint32_t)grid);
    for (size_t k = 0; k < NI; ++k) B.reads.insert(d.inputBuffers[k].data);
    for (size_t k = 0; k < NO; ++k) B.writes.insert(d.outputBuffers[k].data);
}

// The flat kernels that wait in the batch (emitFused) leave: alone as an ordinary launch, several as one launch of the
// kernel's many-blocks form.  Everything else that enqueues work during a flush calls this first.
void DeviceHIP::issueFlatBatch()
{
    if (!m_extras->smallFills.empty()) {
        auto& fills = m_extras->smallFills;
        struct Clear { std::vector<aixk_fill_item>& f; ~Clear() { f.clear(); } } clearFills{fills};
        check(aixk_fill_many(m_ctx, fills.data(), (uint32_t)fills.size()));
    }
    auto& B = m_extras->batch;
    const uint32_t count = B.count();
    if (count == 0) return;
    struct Clear { Extras::FlatBatch& b; ~Clear() { b.clear(); } } clear{B};
    if (count == 1) {
        check(aixk_rtc_launch(m_ctx, B.single, B.starts[1], gen::kBlock, B.table.data(), B.words * sizeof(uint64_t)));
        return;
    }
    const size_t startsOffset = B.table.size() * sizeof(uint64_t);
    B.table.resize(B.table.size() + (B.starts.size() * sizeof(uint32_t) + 7) / 8);
    std::memcpy((char*)B.table.data() + startsOffset, B.starts.data(), B.starts.size() * sizeof(uint32_t));
    check(aixk_rtc_launch_many(m_ctx, B.many, gen::kBlock, B.table.data(), B.table.size() * sizeof(uint64_t), startsOffset, count));
    ++m_extras->batchedLaunches;
    m_extras->batchedKernels += count;
}

// A fused kernel that holds row reductions: a wave or a workgroup per row (hipgen.hpp: row programs).
void DeviceHIP::emitRowProgram(const FusedSubgraphDescriptor& d)
{
    auto& ex = *m_extras;
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size();
    gen::RowGeometry geo;
    if (!gen::rowGeometry(d, &geo)) throw std::logic_error("DeviceHIP: a row program the generator cannot lay out");
    const void* inPtr[64];
    void* outPtr[64];
    size_t storedBytes = 0;
    for (size_t k = 0; k < NI; ++k) {
        markTouched(d.inputBuffers[k].data);
        inPtr[k] = (const char*)d.inputBuffers[k].data + d.inputBuffers[k].offset * dataTypeSize(d.inputBuffers[k].dtype);
    }
    for (size_t k = 0; k < NO; ++k) {
        markTouched(d.outputBuffers[k].data);
        outPtr[k] = (char*)d.outputBuffers[k].data + d.outputBuffers[k].offset * dataTypeSize(d.outputBuffers[k].dtype);
        storedBytes += d.outputBuffers[k].size * dataTypeSize(d.outputBuffers[k].dtype);
    }
    const bool streamOut = storedBytes >= ex.streamStoreMinBytes;
    gen::rowSignatureInto(ex.key, d, geo, streamOut);
    aixk_module* mod = nullptr;
    auto it = ex.kernels.find(ex.key);
    if (it != ex.kernels.end()) { mod = it->second; ++ex.hits; }
    else {
        int32_t cached = 0;
        const std::string src = gen::rowSource(d, geo, streamOut);
        check(aixk_rtc_get(m_ctx, ex.key.c_str(), src.c_str(), gen::rowEntryName(d, geo).c_str(), &mod, &cached));
        ex.kernels.emplace(ex.key, mod);
        ++ex.misses;
    }
    gen::packRowArgsInto(ex.args, d, inPtr, outPtr);
    AIXHIP_TRACE("%s  rows of %zu, %zu elements, %zu in %zu out", gen::rowEntryName(d, geo).c_str(), d.rowLength, d.elementCount, NI, NO);
    const uint64_t rows = d.elementCount / d.rowLength;
    const uint64_t rowsPerBlock = geo.lanes == 64 ? gen::kBlock / 64 : 1;
    uint64_t grid = (rows + rowsPerBlock - 1) / rowsPerBlock;
    grid = std::max<uint64_t>(1, std::min<uint64_t>(grid, (uint64_t)m_cus * 64));
    if (ex.batchFlatKernels) {
        joinBatch(d, mod, gen::rowEntryName(d, geo), grid, [&] { return gen::rowSource(d, geo, streamOut, true); });
        return;
    }
    issueFlatBatch();
    check(aixk_rtc_launch(m_ctx, mod, (uint32_t)grid, gen::kBlock, ex.args.data(), ex.args.size() * sizeof(uint64_t)));
}

// ---- operators that run at once ------------------------------------------------------------------
void DeviceHIP::sum(const DeviceTensorParams& a, const DeviceTensorParams& result)
{
    const Marker marker_("sum");
    AIXHIP_TRACE("sum");
    requireDevice(result, "sum");
    flushFor(a.data, result.data);
    aixhip_tensor pa, pr; stagedPod(a, &pa, "sum"); toPod(result, &pr, "sum");
    check(aixk_reduce_all(m_ctx, AIXK_SUM, &pa, &pr));
}

void DeviceHIP::max(const DeviceTensorParams& a, const DeviceTensorParams& result)
{
    const Marker marker_("max");
    AIXHIP_TRACE("max");
    requireDevice(result, "max");
    flushFor(a.data, result.data);
    aixhip_tensor pa, pr; stagedPod(a, &pa, "max"); toPod(result, &pr, "max");
    check(aixk_reduce_all(m_ctx, AIXK_MAX, &pa, &pr));
}

void DeviceHIP::argmax(const DeviceTensorParams& a, const DeviceTensorParams& result)
{
    const Marker marker_("argmax");
    if (result.dtype != DataType::kInt32) throw std::invalid_argument("DeviceHIP::argmax supports only int32 data type for its result.");
    requireDevice(result, "argmax");
    flushFor(a.data, result.data);
    aixhip_tensor pa, pr; stagedPod(a, &pa, "argmax"); toPod(result, &pr, "argmax");
    check(aixk_reduce_all(m_ctx, AIXK_ARGMAX, &pa, &pr));
}

void DeviceHIP::argmaxIndices(const DeviceTensorParams& a, const DeviceTensorParams& result)
{
    const Marker marker_("argmaxIndices");
    if (result.dtype != DataType::kInt32) throw std::invalid_argument("DeviceHIP::argmaxIndices supports only int32 data type for its result.");
    requireDevice(result, "argmaxIndices");
    flushFor(a.data, result.data);
    aixhip_tensor pa, pr; stagedPod(a, &pa, "argmaxIndices"); toPod(result, &pr, "argmaxIndices");
    check(aixk_reduce_all(m_ctx, AIXK_ARGMAX_ONEHOT, &pa, &pr));
}

// The interface has no batch dimension (aixCore.hpp:943-976), so attention over (sequence, head) pairs, or any batch of
// small products, arrives as a run of matmul calls of one shape.  One launch per call leaves the chip mostly idle (a
// [512, 512] x [512, 512] bf16 product: 4.4 us for 0.3 us of arithmetic), so such calls are not issued at once: a small
// 16-bit product whose operands lie in device memory joins the group of pending products if it has their shape and
// operand layout and depends on none of them, and the group is issued as ONE launch when anything else happens -- an
// operator of another kind is enqueued, recorded operators are planned, the window is flushed or synchronised.  The
// reference batches its dispatches for the same reason (aixDeviceMetal.cpp:1344-1389).
void DeviceHIP::matmul(const DeviceTensorParams& a, const DeviceTensorParams& b, const DeviceTensorParams& result)
{
    const Marker marker_("matmul");
    requireDevice(result, "matmul");
    AIXHIP_TRACE("matmul rank %zu, %zu x %zu elements", a.shape.size(), a.size, b.size);
    auto& ex = *m_extras;
    const bool sixteen = result.dtype == DataType::kFloat16 || result.dtype == DataType::kBFloat16;
    if (sixteen && a.shape.size() == 2 && b.shape.size() == 2 && result.shape.size() == 2 && a.dtype == result.dtype && b.dtype == result.dtype &&
        a.size && b.size && findBlock(a.data) && findBlock(b.data)) {
        const size_t M = a.shape[0], K = a.shape[1], N = b.shape[1];
        const bool small = K % 8 == 0 && M * N >= 64 * 64 && ((M + 63) / 64) * ((N + 63) / 64) < (size_t)m_cus * 3;
        if (small && b.shape[0] == K && result.shape[0] == M && result.shape[1] == N) {
            // recorded operators that produce an operand, or that still use the result's buffer, go first (and so does
            // every pending product); any other recorded operator may as well run after the product
            if (m_engine->pendingWrites(a.data) || m_engine->pendingWrites(b.data) || m_engine->pendingTouches(result.data)) {
                m_engine->recordExternalRead(a.data);
                m_engine->recordExternalRead(b.data);
                m_engine->recordExternalRead(result.data);      // a fill of the result that nobody has read yet must not be set aside and land behind the product
                flushWindow(false);
            }
            aixhip_tensor pa, pb, pr; toPod(a, &pa, "matmul"); toPod(b, &pb, "matmul"); toPod(result, &pr, "matmul");
            // it may read no waiting result and overwrite nothing that waits: all waiting calls are then independent of
            // each other, whatever group they wait in, and the groups may be issued in any order
            if (!ex.apartFromWaiting(pa.data, pb.data, pr.data)) issuePending(true);
            // the group of its shape and operand layout (forward and backward products of attention alternate between
            // two or three of them), or the emptiest slot
            Extras::Group* into = nullptr;
            for (auto& g : ex.groups) {
                if (g.out.empty()) { if (!into) into = &g; continue; }
                const aixhip_tensor &ga = g.a[0], &gb = g.b[0];
                if (g.out[0].dtype == pr.dtype && ga.shape[0] == M && ga.shape[1] == K && gb.shape[1] == N && ga.strides[0] == pa.strides[0] &&
                    ga.strides[1] == pa.strides[1] && gb.strides[0] == pb.strides[0] && gb.strides[1] == pb.strides[1] && g.out.size() < 4096) { into = &g; break; }
            }
            if (!into) { issuePending(); into = &ex.groups[0]; }
            into->a.push_back(pa); into->b.push_back(pb); into->out.push_back(pr);
            into->reads.insert(pa.data); into->reads.insert(pb.data); into->writes.insert(pr.data);
            for (const void* p : {(const void*)pa.data, (const void*)pb.data, (const void*)pr.data}) if (Block* blk = m_blocks.find(p)) ++blk->waiters;
            ++ex.grouped;
            markTouched(a.data); markTouched(b.data); markTouched(result.data);
            return;
        }
    }
    flushFor(a.data, b.data, result.data);
    aixhip_tensor pa, pb, pr; stagedPod(a, &pa, "matmul"); stagedPod(b, &pb, "matmul"); toPod(result, &pr, "matmul");
    // operands with leading dims in front of the matrix dims: a stack of products (beyond the reference, whose
    // matmul is 2-D only, aixCore.hpp:943-976)
    auto run = [&] { return a.shape.size() > 2 ? aixk_matmul_batched(m_ctx, &pa, &pb, &pr) : aixk_matmul(m_ctx, &pa, &pb, &pr); };
    int status = run();
    if (status == AIXK_ENOMEM) {
        // the kernel layer's own workspaces (gathered operands, K-split partials) are outside the pool: give the
        // cached blocks back to the driver and try once more, as allocateBlock() does for the pool's own requests
        synchronize();
        emptyCache();
        status = run();
    }
    check(status);
}

// With `marked`, only those groups of products leave that the caller has just found in its way (Extras::meetsRead,
// meetsWrite); every waiting call is independent of every other, so the rest may go on waiting.
void DeviceHIP::issuePending(bool marked)
{
    const Marker marker_("calls that waited leave");
    auto& ex = *m_extras;
    if (ex.anyPending()) {
        size_t products = 0, sums = 0;
        for (const auto& g : ex.groups) if (!marked || g.leaves) products += g.out.size();
        for (const auto& c : ex.colsums) sums += c.size();
        AIXHIP_TRACE("-- what waited leaves: %zu sliceSet, %zu argmaxIndicesTo, %zu reduceTo, %zu sums of partials, %zu matmul", ex.slices.size(), ex.onehots.size(), sums,
                     ex.partialSums.size(), products);
        (void)products; (void)sums;
    }
    // A list that fails does not take the others with it: every call here was accepted earlier and returned normally, so
    // all of them are sent off, and the first failure is reported afterwards (from whichever operator, flush or
    // synchronize caused the send-off: errors of calls that wait are reported late).
    int first = AIXK_OK;
    std::string firstError;
    size_t dropped = 0;
    auto sent = [&](int status, size_t calls) {
        if (status == AIXK_OK) return;
        dropped += calls;
        if (first == AIXK_OK) { first = status; firstError = aixk_last_error(); }
    };
    if (!ex.slices.empty()) {
        sent(ex.slices.size() == 1 ? aixk_slice_set(m_ctx, &ex.slices[0].src, &ex.slices[0].dst, ex.slices[0].dim, ex.slices[0].start, ex.slices[0].end, ex.slices[0].step)
                                   : aixk_slice_set_many(m_ctx, ex.slices.data(), (uint32_t)ex.slices.size()), ex.slices.size());
        if (ex.slices.size() > 1) { ++ex.batchedLaunches; ex.batchedKernels += ex.slices.size(); }
        ex.slices.clear();
    }
    if (!ex.onehots.empty()) {
        sent(ex.onehots.size() == 1 ? aixk_argmax_to(m_ctx, 2, &ex.onehots[0].src, &ex.onehots[0].dst, ex.onehots[0].dim)
                                    : aixk_argmax_onehot_many(m_ctx, ex.onehots.data(), (uint32_t)ex.onehots.size()), ex.onehots.size());
        if (ex.onehots.size() > 1) { ++ex.batchedLaunches; ex.batchedKernels += ex.onehots.size(); }
        ex.onehots.clear();
    }
    if (!ex.partialSums.empty()) {
        auto& sums = ex.partialSums;
        sent(sums.size() == 1 ? aixk_sum_partials(m_ctx, sums[0].partials, sums[0].count, &sums[0].dst, sums[0].init_bits)
                              : aixk_sum_partials_many(m_ctx, sums.data(), (uint32_t)sums.size()), sums.size());
        if (sums.size() > 1) { ++ex.batchedLaunches; ex.batchedKernels += sums.size(); }
        sums.clear();
    }
    for (auto& sums : ex.colsums) {
        if (sums.empty()) continue;
        sent(sums.size() == 1 ? aixk_reduce_to_init(m_ctx, AIXK_SUM, &sums[0].src, &sums[0].dst, sums[0].init_bits)
                              : aixk_sum_columns_many(m_ctx, sums.data(), (uint32_t)sums.size()), sums.size());
        if (sums.size() > 1) { ++ex.batchedLaunches; ex.batchedKernels += sums.size(); }
        sums.clear();
    }
    ex.waitReads.clear(); ex.waitWrites.clear(); ex.sliceDsts.clear();
    for (auto& g : ex.groups) {
        const bool leaves = !marked || g.leaves;
        g.leaves = false;
        if (g.out.empty() || !leaves) continue;
        const uint32_t count = (uint32_t)g.out.size();
        sent(count == 1 ? aixk_matmul(m_ctx, &g.a[0], &g.b[0], &g.out[0]) : aixk_matmul_grouped(m_ctx, g.a.data(), g.b.data(), g.out.data(), count), count);
        for (uint32_t i = 0; i < count; ++i)
            for (const void* p : {(const void*)g.a[i].data, (const void*)g.b[i].data, (const void*)g.out[i].data}) if (Block* blk = m_blocks.find(p)) --blk->waiters;
        g.a.clear(); g.b.clear(); g.out.clear(); g.reads.clear(); g.writes.clear();
        ex.grouped -= count;
    }
    if (first == AIXK_OK) return;
    const std::string msg = "DeviceHIP: " + firstError + " (reported when the calls that waited were sent off: " + std::to_string(dropped) +
                            " call(s) accepted earlier did not run, their destinations keep what they held)";
    if (first == AIXK_EINVAL) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

void DeviceHIP::transpose(const DeviceTensorParams& a, const DeviceTensorParams& result, size_t dim0, size_t dim1)
{
    const Marker marker_("transpose");
    AIXHIP_TRACE("transpose");
    requireDevice(result, "transpose");
    flushFor(a.data, result.data);
    aixhip_tensor pa, pr; stagedPod(a, &pa, "transpose"); toPod(result, &pr, "transpose");
    check(aixk_transpose(m_ctx, &pa, &pr, dim0, dim1));
}

void DeviceHIP::copy(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size)
{
    const Marker marker_("copy");
    if (size == 0) return;
    if (!findBlock(dst)) throw std::invalid_argument("DeviceHIP::copy() result must have GPU memory.");        // aixDeviceMetal.cpp:714-715
    // Both ends whole device blocks: the conversion is recorded and fuses into the kernel that produces its
    // operand (converted at the store) or into the one that consumes its result (converted at the load).
    // The planner tells buffers apart by base address, so pointers into the middle of a block run at once.
    {
        const Block* sb = m_blocks.find(src);
        const Block* db = m_blocks.find(dst);
        if (sb && db && !sb->freed && !db->freed && src != dst) {
            View in, out;
            in.data = const_cast<void*>(src); in.dtype = srcDType; in.rank = 1; in.shape[0] = size; in.strides[0] = 1; in.size = size;
            out.data = dst; out.dtype = dstDType; out.rank = 1; out.shape[0] = size; out.strides[0] = 1; out.size = size;
            m_engine->record(OpType::Cast, in, out);
            return;
        }
    }
    flushFor(src, dst);
    const size_t srcBytes = size * dataTypeSize(srcDType);
    if (!findBlock(src)) {
        if (srcDType == dstDType) { check(aixk_copy_in(m_ctx, dst, src, srcBytes)); return; }
        src = stageRaw(src, srcBytes);
    }
    check(aixk_cast(m_ctx, src, (int)srcDType, dst, (int)dstDType, size));
}

void DeviceHIP::copyImmediate(const void* src, DataType srcDType, void* dst, DataType dstDType, size_t size)
{
    const Marker marker_("copyImmediate");
    copy(src, srcDType, dst, dstDType, size);
    synchronize();
}

void DeviceHIP::contiguous(const DeviceTensorParams& src, const DeviceTensorParams& dst)
{
    const Marker marker_("contiguous");
    AIXHIP_TRACE("contiguous");
    requireDevice(dst, "contiguous");
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "contiguous"); toPod(dst, &pd, "contiguous");
    check(aixk_contiguous(m_ctx, &ps, &pd));
}

// The front-end always initialises the destination of reduceTo / maxTo right before the call
// (fill(0) / fillMin(), aixCore.hpp:632-639, 873-891).  While that fill is still waiting in the
// planner's window it is taken out and handed to the reduction kernel as the value every
// destination element "holds", which saves the fill's launch and its pass over dst.
static bool lowestBits(DataType dt, uint64_t* bits)
{
    switch (dt) {
        case DataType::kFloat64:  { const double v = -std::numeric_limits<double>::max(); std::memcpy(bits, &v, 8); return true; }
        case DataType::kFloat32:  { const float v = -std::numeric_limits<float>::max(); std::memcpy(bits, &v, 4); return true; }
        case DataType::kFloat16:  *bits = 0xFBFFu; return true;
        case DataType::kBFloat16: *bits = 0xFF7Fu; return true;
        case DataType::kInt64:    { const int64_t v = std::numeric_limits<int64_t>::min(); std::memcpy(bits, &v, 8); return true; }
        case DataType::kInt32:    { const int32_t v = std::numeric_limits<int32_t>::min(); std::memcpy(bits, &v, 4); return true; }
        case DataType::kInt16:    { const int16_t v = std::numeric_limits<int16_t>::min(); std::memcpy(bits, &v, 2); return true; }
        case DataType::kInt8:     { const int8_t v = std::numeric_limits<int8_t>::min(); std::memcpy(bits, &v, 1); return true; }
        case DataType::kUInt8:    *bits = 0; return true;
    }
    return false;
}

bool DeviceHIP::takeInit(const DeviceTensorParams& src, const DeviceTensorParams& dst, uint64_t* bits)
{
    if (src.data == dst.data || src.size == 0) return false;
    aixhip::fuse::OpRecord fill;
    if (!m_engine->takeTrailingFill(dst, &fill)) return false;
    *bits = 0;
    if (fill.type == OpType::FillMin) return lowestBits(dst.dtype, bits);
    const auto v = aixhip::scalar::decode(fill.scalarData.data(), static_cast<int>(fill.scalarDType));
    return aixhip::scalar::encode(v, static_cast<int>(dst.dtype), bits) != 0;
}

// A sum / maximum over the last dimension of a dense floating-point tensor whose destination's initialisation could be
// folded in is not run at once but recorded: the planner fuses it with the elementwise operators around it into one
// kernel that works row by row (max -> sub -> exp -> sum -> div of aixNeuralNetwork.hpp:188-192 reads its operand once;
// mean, variance and normalisation of a LayerNorm likewise).  The fused kernel adds a row up in the stand-alone row
// kernel's order, so fusing changes no bits; rows that kernel does not take (shorter than 32 elements) are not recorded.
// Everything else runs at once as before.
bool DeviceHIP::recordRowReduction(OpType type, const DeviceTensorParams& src, const DeviceTensorParams& dst, uint64_t init)
{
    if (!m_engine->config().elementwiseFusion || !m_extras->fuseRowReductions) return false;
    if (src.dtype != DataType::kFloat32 && src.dtype != DataType::kFloat16 && src.dtype != DataType::kBFloat16 && src.dtype != DataType::kFloat64) return false;
    if (src.shape.empty() || src.shape.size() > AIXK_MAX_RANK || !src.isContiguous || !m_blocks.find(src.data) || !m_blocks.find(dst.data) || src.size == 0) return false;
    const size_t L = src.shape.back(), esz = dataTypeSize(src.dtype), vec = 16 / esz;
    if (L < 32 || L % vec != 0 || src.offset % vec != 0 || src.size % L != 0 || dst.size != src.size / L) return false;
    if (L / vec > 8 * (L >= 2048 ? 256u : 64u)) return false;              // more than 8 vectors per lane: the stand-alone kernel
    // the destination: the source's shape with the last dim 1 or dropped, dense
    if (!dst.isContiguous || dst.offset != 0) return false;
    const size_t lead = src.shape.size() - 1;
    if (dst.shape.size() != lead && !(dst.shape.size() == lead + 1 && dst.shape.back() == 1)) return false;
    for (size_t d = 0; d < lead; ++d) if (dst.shape[d] != src.shape[d]) return false;
    View in(src), out(dst);
    out.makeDense();
    m_engine->recordRowReduce(type, in, out, &init, L);
    return true;
}

void DeviceHIP::reduceTo(const DeviceTensorParams& src, const DeviceTensorParams& dst)
{
    const Marker marker_("reduceTo");
    AIXHIP_TRACE("reduceTo");
    if (src.dtype != dst.dtype) throw std::invalid_argument("DeviceHIP::reduceTo() requires matching source and destination data types.");
    requireDevice(dst, "reduceTo");
    uint64_t init = 0;
    const bool folded = takeInit(src, dst, &init);
    if (folded && recordRowReduction(OpType::ReduceTo, src, dst, init)) return;
    // The sum of ALL elements of a tensor that a recorded operator is about to produce -- the gradient of a scalar
    // constant is the sum of a product formed for nothing else (aixCore.hpp:2384-2438, 2030-2036) -- is recorded too: the
    // planner lets it join the kernel that holds the product in registers, which then adds it up instead of storing it.
    if (folded && dst.size == 1 && src.size > 1 && src.isContiguous && m_extras->fuseRowReductions && m_engine->config().elementwiseFusion &&
        (src.dtype == DataType::kFloat32 || src.dtype == DataType::kFloat16 || src.dtype == DataType::kBFloat16 || src.dtype == DataType::kFloat64) &&
        src.shape.size() <= AIXK_MAX_RANK && dst.shape.size() <= AIXK_MAX_RANK && findBlock(src.data) && findBlock(dst.data) && m_engine->pendingWrites(src.data)) {
        View in(src), out(dst);
        if (in.dense) {
            m_engine->recordWholeSum(in, out, &init);
            return;
        }
    }
    // A dense matrix summed down its columns -- the gradient of a bias or of a LayerNorm parameter, summed to the
    // parameter's shape (aixCore.hpp:2228-2233) and read only when the backward pass reaches the parameter: like small
    // matmul calls it waits, and all that have gathered by then leave in one pair of launches (see matmul(), sliceSet()).
    auto& ex = *m_extras;
    const int slot = src.dtype == DataType::kFloat32 ? 0 : src.dtype == DataType::kFloat16 ? 1 : src.dtype == DataType::kBFloat16 ? 2 : -1;
    if (folded && slot >= 0 && ex.batchFlatKernels && src.isContiguous && dst.isContiguous && src.shape.size() >= 2 && src.shape.size() <= AIXK_MAX_RANK &&
        !dst.shape.empty() && dst.shape.size() <= AIXK_MAX_RANK && dst.size == src.shape.back() && dst.shape.back() == dst.size && dst.size % 4 == 0 &&
        src.size >= 2 * dst.size && src.offset % 4 == 0 && findBlock(src.data) && findBlock(dst.data) && src.data != dst.data) {
        if (m_engine->pendingWrites(src.data) || m_engine->pendingTouches(dst.data)) {          // recorded producers and users go first
            m_engine->recordExternalRead(src.data);
            m_engine->recordExternalRead(dst.data);             // (a fill of the destination still recorded goes first, it does not wait)
            flushWindow(false);
        }
        auto& sums = ex.colsums[slot];
        const bool apart = ex.apartFromWaiting(src.data, nullptr, dst.data);
        if (sums.size() >= AIXK_COLSUM_ITEMS_MAX || !apart) issuePending(true);
        AIXHIP_TRACE("   (waits: %zu columns)", dst.size);
        aixk_colsum_item item{};
        toPod(src, &item.src, "reduceTo"); toPod(dst, &item.dst, "reduceTo");
        item.init_bits = init;
        sums.push_back(item);
        ex.noteWaiting(src.data, nullptr, dst.data);
        markTouched(src.data); markTouched(dst.data);
        return;
    }
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "reduceTo"); toPod(dst, &pd, "reduceTo");
    check(folded ? aixk_reduce_to_init(m_ctx, AIXK_SUM, &ps, &pd, init) : aixk_reduce_to(m_ctx, AIXK_SUM, &ps, &pd));
}

void DeviceHIP::maxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst)
{
    const Marker marker_("maxTo");
    AIXHIP_TRACE("maxTo");
    if (src.dtype != dst.dtype) throw std::invalid_argument("DeviceHIP::maxTo() requires matching source and destination data types.");
    requireDevice(dst, "maxTo");
    uint64_t init = 0;
    const bool folded = takeInit(src, dst, &init);
    if (folded && recordRowReduction(OpType::MaxTo, src, dst, init)) return;
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "maxTo"); toPod(dst, &pd, "maxTo");
    check(folded ? aixk_reduce_to_init(m_ctx, AIXK_MAX, &ps, &pd, init) : aixk_reduce_to(m_ctx, AIXK_MAX, &ps, &pd));
}

void DeviceHIP::argmaxTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim)
{
    const Marker marker_("argmaxTo");
    AIXHIP_TRACE("argmaxTo");
    if (dst.dtype != DataType::kInt32) throw std::invalid_argument("DeviceHIP::argmaxTo supports only int32 data type for its result.");
    requireDevice(dst, "argmaxTo");
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "argmaxTo"); toPod(dst, &pd, "argmaxTo");
    check(aixk_argmax_to(m_ctx, 0, &ps, &pd, dim));
}

// The mask of max()'s backward pass (aixCore.hpp:2170-2175) is asked for head after head: like small matmul calls, a
// call whose zero fill was folded in and whose operands lie in device memory waits for company and leaves with it in one
// launch (see matmul(), sliceSet()).
void DeviceHIP::argmaxIndicesTo(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim)
{
    const Marker marker_("argmaxIndicesTo");
    AIXHIP_TRACE("argmaxIndicesTo");
    if (dst.dtype != DataType::kInt32) throw std::invalid_argument("DeviceHIP::argmaxIndicesTo supports only int32 data type for its result.");
    requireDevice(dst, "argmaxIndicesTo");
    // the caller zero-fills the destination right before the call (aixCore.hpp:927-941): a fill still waiting in
    // the window is folded into the operator
    uint64_t init = 0;
    const bool folded = takeInit(src, dst, &init);
    auto& ex = *m_extras;
    // Rows that a row program takes (as recordRowReduction has them): recorded, so that the multiplication with the mask
    // that always follows (max()'s backward) finds the ones and zeros in registers
    if (folded && init == 0 && ex.fuseRowReductions && m_engine->config().elementwiseFusion && m_engine->config().supportsStridedFusion &&
        (src.dtype == DataType::kFloat32 || src.dtype == DataType::kFloat16 || src.dtype == DataType::kBFloat16) && src.size && dst.size == src.size &&
        findBlock(src.data) && findBlock(dst.data) && src.data != dst.data && src.isContiguous && dst.isContiguous && dst.offset == 0 && src.shape == dst.shape &&
        !src.shape.empty() && dim + 1 == src.shape.size() && src.shape.size() <= AIXK_MAX_RANK) {
        const size_t L = src.shape.back(), vec = 16 / dataTypeSize(src.dtype);
        if (L >= 32 && L % vec == 0 && src.offset % vec == 0 && L / vec <= 8 * (L >= 2048 ? 256u : 64u) && L < (size_t(1) << 31)) {
            View in(src), out(dst);
            out.makeDense();
            m_engine->recordRowOnehot(in, out, L);
            return;
        }
    }
    if (folded && init == 0 && ex.batchFlatKernels && src.size && src.size < (size_t(1) << 31) && dst.size == src.size && findBlock(src.data) && findBlock(dst.data) &&
        src.data != dst.data && src.isContiguous && dst.isContiguous && dst.offset == 0 && src.shape == dst.shape && !src.shape.empty() &&
        dim + 1 == src.shape.size() && src.shape.size() <= AIXK_MAX_RANK) {
        if (m_engine->pendingWrites(src.data) || m_engine->pendingTouches(dst.data)) {          // recorded producers and users go first
            m_engine->recordExternalRead(src.data);
            m_engine->recordExternalRead(dst.data);             // (a fill of the destination still recorded goes first, it does not wait)
            flushWindow(false);
        }
        const bool apart = ex.apartFromWaiting(src.data, nullptr, dst.data);
        if (ex.onehots.size() >= AIXK_ARGMAX_ITEMS_MAX || !apart) issuePending(true);
        aixk_argmax_item item{};
        toPod(src, &item.src, "argmaxIndicesTo"); toPod(dst, &item.dst, "argmaxIndicesTo");
        item.dim = dim;
        ex.onehots.push_back(item);
        ex.noteWaiting(src.data, nullptr, dst.data);
        markTouched(src.data); markTouched(dst.data);
        return;
    }
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "argmaxIndicesTo"); toPod(dst, &pd, "argmaxIndicesTo");
    if (folded && init != 0) {                                       // not the zero fill: put it back as a pass of its own
        const int32_t value = (int32_t)init;
        check(aixk_fill(m_ctx, &value, AIXK_I32, &pd));
    }
    check(aixk_argmax_to(m_ctx, folded && init == 0 ? 2 : 1, &ps, &pd, dim));
}

// A cat() is one sliceSet per part into a fresh tensor (aixCore.hpp:1348-1402), the seed of a tensor whose slices were
// used is one per slice (:2228-2233): runs of calls that copy a few KB each and do not depend on one another.  Like
// small matmul calls they are not issued at once: a call whose operands lie in device memory waits, and the run leaves
// as ONE launch when anything else happens.  A call joins the run if it reads nothing a waiting call (sliceSet or
// matmul) writes and writes nothing a waiting call reads or writes -- two windows of one destination count as apart
// when the destination is described the same way both times and the windows are ranges of one dim (step 1) that do not
// overlap; otherwise what waits is issued first.
void DeviceHIP::sliceSet(const DeviceTensorParams& src, const DeviceTensorParams& dst, size_t dim, size_t start, size_t end, size_t step)
{
    const Marker marker_("sliceSet");
    AIXHIP_TRACE("sliceSet");
    if (src.dtype != dst.dtype) throw std::invalid_argument("DeviceHIP::sliceSet() requires matching source and destination data types.");
    requireDevice(dst, "sliceSet");
    // the backward of a slice fills the destination (zeros of the input's shape) right before the call:
    // a fill still waiting in the window becomes the value written outside the slice, in the same pass
    uint64_t init = 0;
    const bool folded = takeInit(src, dst, &init);
    auto& ex = *m_extras;
    if (!folded && ex.batchFlatKernels && src.size && findBlock(src.data) && findBlock(dst.data) && src.data != dst.data &&
        src.shape.size() <= AIXK_MAX_RANK && dst.shape.size() <= AIXK_MAX_RANK && dim < dst.shape.size() && step >= 1 && end > start) {
        aixk_slice_item item{};
        toPod(src, &item.src, "sliceSet"); toPod(dst, &item.dst, "sliceSet");
        item.dim = dim; item.start = start; item.end = end; item.step = step;
        // what aixk_slice_set checks, so that a bad call is reported here and now by the path below
        const uint64_t count = (end - start + step - 1) / step;
        uint64_t window = count, whole = 1;
        for (size_t d = 0; d < dst.shape.size(); ++d) if (d != dim) window *= dst.shape[d];
        for (size_t d = 0; d < src.shape.size(); ++d) whole *= src.shape[d];
        if (window == src.size && whole == src.size && start + (count - 1) * step < dst.shape[dim]) {
            if (m_engine->pendingWrites(src.data) || m_engine->pendingTouches(dst.data)) {      // recorded producers and users go first
                m_engine->recordExternalRead(src.data);
                m_engine->recordExternalRead(dst.data);         // (a fill of the destination that could not be folded in goes first, it does not wait)
                flushWindow(false);
            }
            bool independent = ex.slices.size() < AIXK_SLICE_ITEMS_MAX &&
                               (ex.slices.empty() || dataTypeSize(static_cast<DataType>(ex.slices[0].src.dtype)) == dataTypeSize(src.dtype));
            // (products that wait: the copy comes after those that write its source or use its destination)
            bool apartFromProducts = true;
            if (ex.productsMayUse(src.data) || ex.productsMayUse(dst.data)) {
                for (auto& g : ex.groups) {
                    if (g.out.empty() || !(g.writes.contains(src.data) || g.writes.contains(dst.data) || g.reads.contains(dst.data))) continue;
                    g.leaves = true;
                    apartFromProducts = false;
                }
            }
            auto windows = ex.sliceDsts.find(dst.data);
            if (!apartFromProducts) {
                independent = false;
            } else if (independent && windows != ex.sliceDsts.end()) {
                // another window of a destination that waits: apart if nothing that waits reads the destination, it is
                // described the same way, and the ranges do not meet
                const auto& w = windows->second;
                independent = !ex.waitWrites.contains(src.data) && !ex.waitReads.contains(dst.data) && w.dim == dim && step == 1 && w.dst.rank == item.dst.rank &&
                              w.dst.offset == item.dst.offset && !std::memcmp(w.dst.shape, item.dst.shape, sizeof(item.dst.shape)) &&
                              !std::memcmp(w.dst.strides, item.dst.strides, sizeof(item.dst.strides));
                for (size_t i = 0; independent && i < w.ranges.size(); ++i) independent = w.ranges[i].second <= start || end <= w.ranges[i].first;
            } else if (independent) {
                independent = ex.apartFromWaiting(src.data, nullptr, dst.data);
            }
            if (!independent) issuePending(true);
            if (step == 1) {
                auto& w = ex.sliceDsts[dst.data];
                if (w.ranges.empty()) { w.dst = item.dst; w.dim = dim; }
                w.ranges.emplace_back(start, end);
            }
            ex.noteWaiting(src.data, nullptr, dst.data);
            ex.slices.push_back(item);
            markTouched(src.data); markTouched(dst.data);
            return;
        }
    }
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "sliceSet"); toPod(dst, &pd, "sliceSet");
    check(folded ? aixk_slice_set_init(m_ctx, &ps, &pd, dim, start, end, step, init) : aixk_slice_set(m_ctx, &ps, &pd, dim, start, end, step));
}

void DeviceHIP::tril(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal)
{
    const Marker marker_("tril");
    if (src.dtype != dst.dtype) throw std::invalid_argument("DeviceHIP::tril() requires matching source and destination data types.");   // aixDeviceMetal.cpp:1160-1161
    requireDevice(dst, "tril");
    if (recordTri(OpType::Tril, src, dst, diagonal)) return;
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "tril"); toPod(dst, &pd, "tril");
    check(aixk_tri(m_ctx, 0, &ps, &pd, diagonal));
}

void DeviceHIP::triu(const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal)
{
    const Marker marker_("triu");
    if (src.dtype != dst.dtype) throw std::invalid_argument("DeviceHIP::triu() requires matching source and destination data types.");
    requireDevice(dst, "triu");
    if (recordTri(OpType::Triu, src, dst, diagonal)) return;
    flushFor(src.data, dst.data);
    aixhip_tensor ps, pd; stagedPod(src, &ps, "triu"); toPod(dst, &pd, "triu");
    check(aixk_tri(m_ctx, 1, &ps, &pd, diagonal));
}

// tril / triu join the window as elementwise operators (the scale, the mask and the triangle of attention scores become
// one kernel) when both ends are this device's memory, the destination is a whole dense tensor of the source's shape
// and the views fit the generated kernels; everything else runs at once.
bool DeviceHIP::recordTri(OpType type, const DeviceTensorParams& src, const DeviceTensorParams& dst, ssize_t diagonal)
{
    if (src.shape.size() < 2 || src.shape.size() > (size_t)gen::kMaxDims || src.shape != dst.shape || src.size == 0 || src.size != dst.size) return false;
    if (!dst.isContiguous || dst.offset != 0 || !m_blocks.find(src.data) || !m_blocks.find(dst.data)) return false;   // (blocks by their start)
    size_t count = 1;
    for (auto e : src.shape) count *= e;
    if (count != src.size) return false;
    View in(src), out(dst);
    out.makeDense();
    m_engine->recordTri(type, in, out, (int64_t)diagonal);
    return true;
}

void DeviceHIP::indexSelect(const DeviceTensorParams& src, const DeviceTensorParams& dst, const DeviceTensorParams& indices, size_t dim)
{
    const Marker marker_("indexSelect");
    AIXHIP_TRACE("indexSelect");
    requireDevice(dst, "indexSelect");
    flushFor(src.data, indices.data, dst.data);
    aixhip_tensor ps, pd, pi; stagedPod(src, &ps, "indexSelect"); toPod(dst, &pd, "indexSelect"); stagedPod(indices, &pi, "indexSelect");
    check(aixk_index_select(m_ctx, &ps, &pd, &pi, dim));
}

void DeviceHIP::indexAdd(const DeviceTensorParams& src, const DeviceTensorParams& dst, const DeviceTensorParams& indices, size_t dim)
{
    const Marker marker_("indexAdd");
    AIXHIP_TRACE("indexAdd");
    requireDevice(dst, "indexAdd");
    flushFor(src.data, indices.data, dst.data);
    aixhip_tensor ps, pd, pi; stagedPod(src, &ps, "indexAdd"); toPod(dst, &pd, "indexAdd"); stagedPod(indices, &pi, "indexAdd");
    check(aixk_index_add(m_ctx, &ps, &pd, &pi, dim));
}

} // namespace hip
} // namespace aix
