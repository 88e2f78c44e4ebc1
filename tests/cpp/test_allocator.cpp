// test_allocator.cpp -- DeviceHIP's memory bookkeeping (block table, size buckets, limbo, event-gated cooling, cache
// trimming, out-of-memory retry) on the stub kernel layer (stub_kernels.cpp): host only, meant to run under
// AddressSanitizer / UndefinedBehaviorSanitizer (make asan) and ThreadSanitizer (make tsan), the counterpart of the
// reference's sanitizer configurations (CMakeLists.txt:25, 47-53).
// Deferred-free semantics follow aixDeviceMetal.cpp:251-259, 1352-1377; out-of-memory retry :1455-1471.
#include "device/device_hip.hpp"
#include "aixhip_kernels.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <set>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

extern "C" {
void stub_set_budget(aixk_ctx*, size_t);
void stub_set_event_delay(aixk_ctx*, int);
size_t stub_held(aixk_ctx*);
uint64_t stub_launches(aixk_ctx*);
uint64_t stub_allocs(aixk_ctx*);
uint64_t stub_frees(aixk_ctx*);
uint64_t stub_syncs(aixk_ctx*);
long long stub_held_everywhere(void);
void stub_fail_next_matmuls(int);
const char* stub_log(aixk_ctx*);
void stub_log_clear(aixk_ctx*);
}

using aix::DataType;
using aix::DeviceTensorParams;
using aix::hip::DeviceHIP;

static int g_failed = 0;
#define CHECK(cond)                                                                   \
    do {                                                                              \
        if (!(cond)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_failed; } \
    } while (0)

template <class E, class F> static bool throws(F&& f)
{
    try { f(); } catch (const E&) { return true; } catch (...) { return false; }
    return false;
}

static DeviceTensorParams matrix(void* p, size_t rows, size_t cols)
{
    DeviceTensorParams t;
    t.data = p; t.dtype = DataType::kFloat32; t.shape = {rows, cols}; t.size = rows * cols; t.strides = {cols, 1};
    return t;
}

// an eagerly enqueued operator that references the three blocks: from then on they count as used by the GPU
static void touch(DeviceHIP& dev, void* a, void* b, void* r) { dev.matmul(matrix(a, 4, 4), matrix(b, 4, 4), matrix(r, 4, 4)); }

static void test_buckets_and_errors()
{
    DeviceHIP dev;
    std::set<void*> seen;
    for (size_t bytes : {size_t(1), size_t(255), size_t(256), size_t(257), size_t(4096), size_t(4097), size_t(100000), size_t(1) << 20}) {
        void* p = dev.allocate(bytes);
        CHECK(p != nullptr && ((uintptr_t)p & 255) == 0);
        CHECK(seen.insert(p).second);
        CHECK(dev.isDeviceMemory(p) && dev.isDeviceMemory((char*)p + bytes - 1));
    }
    CHECK(dev.allocatedBytes() >= 256 * 3 + 4096 + 4097 + 100000 + (size_t(1) << 20));
    CHECK(dev.allocatedBytes() <= (size_t)((256 * 3 + 512 + 4096 + 4097 + 100000 + (size_t(1) << 20)) * 1.125 + 512));     // <= 12.5 % slack
    int onStack = 0;
    CHECK(!dev.isDeviceMemory(&onStack) && !dev.isDeviceMemory(nullptr));
    CHECK(throws<std::invalid_argument>([&] { dev.deallocate(&onStack); }));          // foreign pointer (aixDeviceMetal.cpp:253-254)
    void* first = *seen.begin();
    dev.deallocate(first);
    CHECK(throws<std::invalid_argument>([&] { dev.deallocate(first); }));             // double free
    dev.deallocate(nullptr);                                                          // harmless
    CHECK(dev.allocate(16, DataType::kFloat64) != nullptr);
    // a result that is not this device's memory is refused (aixDeviceMetal.cpp:305-306)
    float host[16] = {};
    void* a = dev.allocate(64);
    CHECK(throws<std::invalid_argument>([&] { dev.matmul(matrix(a, 4, 4), matrix(a, 4, 4), matrix(host, 4, 4)); }));
}

static void test_untouched_temporaries_recycle_at_the_flush()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    void* t = dev.allocate(1000);
    dev.deallocate(t);
    CHECK(dev.cachedBytes() == 0);                     // in limbo until the recorded window is enqueued
    dev.flush();
    CHECK(dev.cachedBytes() == 1024);
    const uint64_t before = stub_allocs(ctx);
    void* again = dev.allocate(900);                   // same bucket
    CHECK(again == t && stub_allocs(ctx) == before && dev.cachedBytes() == 0);
    dev.deallocate(again);
}

static void test_used_blocks_wait_for_the_gpu()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    stub_set_event_delay(ctx, 3);                      // the "GPU" passes an event only at the fourth query
    void* a = dev.allocate(64); void* b = dev.allocate(64); void* r = dev.allocate(64);
    touch(dev, a, b, r);
    dev.deallocate(r);
    for (int i = 0; i < 16; ++i) dev.flush();          // an event is recorded after 16 flushes
    CHECK(dev.cachedBytes() == 0);
    std::set<void*> fresh;
    for (int i = 0; i < 3; ++i) {                      // three queries: still cooling, r must not be handed out
        void* p = dev.allocate(64);
        CHECK(p != r);
        fresh.insert(p);
    }
    void* p = dev.allocate(64);                        // fourth query: done, the block is back
    CHECK(p == r);
    for (void* q : fresh) dev.deallocate(q);
    dev.deallocate(p);
    dev.synchronize();                                 // everything idle: all of it pooled
    CHECK(dev.cachedBytes() == 4 * 256 && dev.allocatedBytes() == 2 * 256);
    dev.emptyCache();
    CHECK(dev.cachedBytes() == 0 && stub_held(ctx) == 2 * 256);
    dev.deallocate(a); dev.deallocate(b);
}

static void test_out_of_memory_retry()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    void* big = dev.allocate(size_t(1) << 20);
    dev.deallocate(big);
    dev.synchronize();
    CHECK(dev.cachedBytes() == (size_t(1) << 20));
    stub_set_budget(ctx, (size_t(1) << 20) + 4096);    // room for the cached block and little else
    const uint64_t syncs = stub_syncs(ctx);
    void* other = dev.allocate(size_t(1) << 19);       // another bucket: the driver refuses, the cache is dropped, the retry succeeds
    CHECK(other != nullptr && dev.cachedBytes() == 0 && stub_syncs(ctx) > syncs);
    CHECK(throws<std::runtime_error>([&] { dev.allocate(size_t(1) << 21); }));       // beyond the budget even with an empty cache
    CHECK(dev.allocatedBytes() == (size_t(1) << 19));
    // the kernel layer's own workspace failing inside matmul: synchronize, drop the cache, retry once
    void* a = dev.allocate(64);
    void* pooled = dev.allocate(8192);
    dev.deallocate(pooled);
    dev.synchronize();
    CHECK(dev.cachedBytes() == 8192);
    stub_fail_next_matmuls(1);
    touch(dev, a, a, a);
    CHECK(dev.cachedBytes() == 0);
    stub_fail_next_matmuls(2);
    CHECK(throws<std::runtime_error>([&] { touch(dev, a, a, a); }));
    dev.deallocate(other); dev.deallocate(a);
}

// Random allocate / free / use / flush / synchronize / emptyCache traffic with the invariants checked throughout.
static void stress(unsigned seed, int rounds)
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    std::mt19937 rng(seed);
    stub_set_event_delay(ctx, (int)(rng() % 4));
    std::vector<std::pair<void*, size_t>> live;
    std::set<void*> liveSet;
    for (int i = 0; i < rounds; ++i) {
        const unsigned what = rng() % 100;
        if (what < 45 || live.empty()) {
            const size_t bytes = what % 3 == 0 ? 1 + rng() % 300 : (what % 3 == 1 ? 1 + rng() % 70000 : 1 + rng() % 3000000);
            void* p = dev.allocate(bytes);
            CHECK(((uintptr_t)p & 255) == 0);
            CHECK(liveSet.insert(p).second);                           // never a block that is still alive
            static_cast<volatile char*>(p)[0] = 1;                     // the whole extent is ours to write
            static_cast<volatile char*>(p)[bytes - 1] = 1;
            live.emplace_back(p, bytes);
        } else if (what < 80) {
            const size_t k = rng() % live.size();
            dev.deallocate(live[k].first);
            liveSet.erase(live[k].first);
            live[k] = live.back();
            live.pop_back();
        } else if (what < 90 && live.size() >= 3) {
            touch(dev, live[rng() % live.size()].first, live[rng() % live.size()].first, live[rng() % live.size()].first);
        } else if (what < 96) {
            dev.flush();
        } else if (what < 99) {
            dev.synchronize();
        } else {
            dev.emptyCache();
        }
        if (i % 64 == 0) {
            size_t sum = 0;
            for (auto& b : live) { CHECK(dev.isDeviceMemory(b.first)); CHECK(dev.isDeviceMemory((char*)b.first + b.second / 2)); sum += b.second; }
            CHECK(dev.allocatedBytes() >= sum && dev.allocatedBytes() <= sum * 9 / 8 + 256 * live.size());
            CHECK(stub_held(ctx) >= dev.allocatedBytes() + dev.cachedBytes());
        }
    }
    for (auto& b : live) dev.deallocate(b.first);
    dev.synchronize();
    CHECK(dev.allocatedBytes() == 0 && stub_held(ctx) == dev.cachedBytes());
    dev.emptyCache();
    CHECK(stub_held(ctx) == 0 && stub_allocs(ctx) == stub_frees(ctx));
}

// The host side of what the device does between the interface and the kernels -- recorded row reductions and row
// programs, fills that wait for their first user, runs of equal flat kernels and small fills sent off together,
// operands that point into the middle of a block -- driven with random traffic on the stub layer: what runs (under the
// sanitizers) is the planner, the generator, the batch tables and the waiting lists; the kernels only count.
static DeviceTensorParams tensor(void* p, std::vector<size_t> shape, DataType dt = DataType::kFloat32, std::vector<size_t> strides = {}, size_t offset = 0)
{
    DeviceTensorParams t;
    t.data = p; t.dtype = dt; t.shape = shape; t.offset = offset;
    size_t n = 1;
    for (auto e : shape) n *= e;
    t.size = n;
    if (strides.empty()) { strides.resize(shape.size()); size_t run = 1; for (size_t d = shape.size(); d-- > 0;) { strides[d] = run; run *= shape[d]; } }
    bool dense = true; size_t run = 1;
    for (size_t d = shape.size(); d-- > 0;) { if (strides[d] != run) dense = false; run *= shape[d]; }
    t.strides = strides; t.isContiguous = dense;
    return t;
}

static void planner_traffic(unsigned seed, int rounds)
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    std::mt19937 rng(seed);
    const size_t rows = 24, len = 256, n = rows * len;
    std::vector<void*> full, cols;
    auto fresh_full = [&] { void* p = dev.allocate(n * 4); full.push_back(p); return p; };
    auto fresh_col = [&] { void* p = dev.allocate(rows * 4); cols.push_back(p); return p; };
    for (int i = 0; i < 3; ++i) fresh_full();
    fresh_col();
    const float zero = 0.0f, two = 2.0f;
    for (int i = 0; i < rounds; ++i) {
        const unsigned what = rng() % 100;
        void* x = full[rng() % full.size()];
        if (what < 25) {                                               // elementwise, full op full
            void* y = full[rng() % full.size()];
            dev.add(tensor(x, {rows, len}), tensor(y, {rows, len}), tensor(fresh_full(), {rows, len}));
        } else if (what < 33) {                                        // full op (one value per row)
            void* c = cols[rng() % cols.size()];
            dev.sub(tensor(x, {rows, len}), tensor(c, {rows, len}, DataType::kFloat32, {1, 0}), tensor(fresh_full(), {rows, len}));
        } else if (what < 38) {                                        // a product that is only formed to be summed, and a triangle of a sum
            void* prod = dev.allocate(n * 4);
            dev.mul(tensor(x, {rows, len}), tensor(full[0], {rows, len}), tensor(prod, {rows, len}));
            void* s = fresh_col();
            dev.fill(&zero, DataType::kFloat32, tensor(s, {}));
            dev.reduceTo(tensor(prod, {rows, len}), tensor(s, {}));
            if (what & 1) dev.tril(tensor(prod, {rows, len}), tensor(fresh_full(), {rows, len}), 0);
            dev.deallocate(prod);
        } else if (what < 45) {                                        // row maximum / row sum with the fill in front
            void* c = fresh_col();
            if (what & 1) { dev.fillMin(tensor(c, {rows, 1})); dev.maxTo(tensor(x, {rows, len}), tensor(c, {rows, 1})); }
            else { dev.fill(&zero, DataType::kFloat32, tensor(c, {rows, 1})); dev.reduceTo(tensor(x, {rows, len}), tensor(c, {rows, 1})); }
        } else if (what < 55) {                                        // a fill that may wait; sometimes of a block that dies at once
            void* p = fresh_full();
            dev.fill(&two, DataType::kFloat32, tensor(p, {rows, len}));
            if (what & 1) { dev.deallocate(p); full.pop_back(); }
        } else if (what < 62) {                                        // small fills in a row (rank-0 constants)
            for (int k = 0; k < 3; ++k) { void* c = fresh_col(); dev.fill(&two, DataType::kFloat32, tensor(c, {})); }
        } else if (what < 70) {                                        // runs of equal flat kernels: y_k = -x_k
            for (int k = 0; k < 4; ++k) dev.unary(tensor(full[rng() % full.size()], {n}), tensor(fresh_full(), {n}));
        } else if (what < 76) {                                        // an operand inside a block
            dev.unary(tensor((char*)x + 64 * 4, {len}), tensor(fresh_full(), {len}));
        } else if (what < 78) {                                        // an operator that runs at once
            dev.transpose(tensor(x, {rows, len}), tensor(fresh_full(), {len, rows}), 0, 1);
        } else if (what < 79) {                                        // column sums that wait; one source dies while its sum still waits
            void* t = dev.allocate(n * 4);
            dev.unary(tensor(x, {rows, len}), tensor(t, {rows, len}));
            for (void* src : {t, x}) {
                void* c = fresh_full();                                // (the sum is the block's first row)
                dev.fill(&zero, DataType::kFloat32, tensor(c, {len}));
                dev.reduceTo(tensor(src, {rows, len}), tensor(c, {len}));
            }
            dev.deallocate(t);
        } else if (what < 82) {                                        // a cat: row blocks of a fresh tensor, the sources may die at once
            void* whole = fresh_full();
            for (size_t k = 0; k < 4; ++k) {
                void* part = dev.allocate(n);                          // [rows / 4, len] of f32
                dev.unary(tensor(x, {rows / 4, len}), tensor(part, {rows / 4, len}));
                dev.sliceSet(tensor(part, {rows / 4, len}), tensor(whole, {rows, len}), 0, k * (rows / 4), (k + 1) * (rows / 4), 1);
                dev.deallocate(part);
            }
            if (what & 1) dev.sliceSet(tensor(x, {rows / 4, len}), tensor(whole, {rows, len}), 0, 3, 3 + rows / 4, 1);      // overlaps two of them
        } else if (what < 84) {                                        // masks of max()'s backward, then a matmul that waits beside them
            for (int k = 0; k < 3; ++k) {
                void* mask = fresh_full();
                dev.fill(&zero, DataType::kFloat32, tensor(mask, {rows, len}, DataType::kInt32));
                dev.argmaxIndicesTo(tensor(full[rng() % (full.size() - 1)], {rows, len}), tensor(mask, {rows, len}, DataType::kInt32), 1);
            }
            void* h = dev.allocate(n * 4);
            full.push_back(h);
            dev.matmul(tensor(x, {64, 64}, DataType::kBFloat16), tensor(full[0], {64, 64}, DataType::kBFloat16), tensor(h, {64, 64}, DataType::kBFloat16));
        } else if (what < 92 && full.size() > 4) {                     // temporaries die
            const size_t k = 3 + rng() % (full.size() - 3);
            dev.deallocate(full[k]); full[k] = full.back(); full.pop_back();
            if (cols.size() > 2) { dev.deallocate(cols.back()); cols.pop_back(); }
        } else if (what < 97) {
            dev.flush();
        } else {
            dev.synchronize();
        }
    }
    dev.synchronize();
    CHECK(stub_launches(ctx) > 0);
    for (void* p : full) dev.deallocate(p);
    for (void* p : cols) dev.deallocate(p);
    dev.synchronize();
    CHECK(dev.allocatedBytes() == 0);
}

// A small 16-bit product is not enqueued when it is called: it waits for others of its shape.  Flushes that have nothing
// to do with it leave it waiting, and a block it uses stays out of the pool until the product has been enqueued and the
// GPU has passed it, however long ago the caller freed the block.
static void test_blocks_of_calls_that_wait_are_not_handed_out()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    auto half = [](void* p) { DeviceTensorParams t = matrix(p, 64, 64); t.dtype = DataType::kBFloat16; return t; };
    void* a = dev.allocate(8192); void* b = dev.allocate(8192); void* r = dev.allocate(8192);
    void* x = dev.allocate(64); void* y = dev.allocate(64); void* z = dev.allocate(64);
    const uint64_t before = stub_launches(ctx);
    dev.matmul(half(a), half(b), half(r));
    CHECK(stub_launches(ctx) == before);                // waits
    dev.deallocate(a);                                  // the caller is done with an operand
    std::set<void*> fresh;
    for (int i = 0; i < 40; ++i) {                      // other work comes and goes; its flushes record events
        touch(dev, x, y, z);
        void* p = dev.allocate(8192);
        CHECK(p != a && p != b && p != r);
        fresh.insert(p);
    }
    CHECK(stub_launches(ctx) == before + 40);           // the product is still waiting
    touch(dev, r, y, z);                                // its result is read: now it goes, ahead of the reader
    CHECK(stub_launches(ctx) == before + 42);
    dev.synchronize();
    CHECK(dev.cachedBytes() == 8192);                   // and only now is the operand's block back in the pool
    void* again = dev.allocate(8192);
    CHECK(again == a);
    for (void* p : fresh) dev.deallocate(p);
    for (void* p : {again, b, r, x, y, z}) dev.deallocate(p);
}

// Groups of waiting products leave one by one: a reader of one group's result sends that group off and leaves the
// others waiting (the weight gradients of a backward pass go on collecting while the small products of attention come
// and go); a writer of an operand sends off the groups that read it; flush(true) sends off what is left.
static void test_groups_of_products_leave_apart()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    auto half = [](void* p, size_t rows, size_t cols) { DeviceTensorParams t = matrix(p, rows, cols); t.dtype = DataType::kBFloat16; return t; };
    std::vector<void*> all;
    auto block = [&](size_t bytes) { void* p = dev.allocate(bytes); all.push_back(p); return p; };
    void* x = block(64); void* y = block(64);
    // three "weight gradients" [128,64] x [64,128] and, in between, "attention" products [64,64] x [64,64] whose results
    // are read at once
    void* wa[3]; void* wb[3]; void* wr[3];
    uint64_t expected = stub_launches(ctx);
    for (int i = 0; i < 3; ++i) {
        wa[i] = block(128 * 64 * 2); wb[i] = block(64 * 128 * 2); wr[i] = block(128 * 128 * 2);
        dev.matmul(half(wa[i], 128, 64), half(wb[i], 64, 128), half(wr[i], 128, 128));
        CHECK(stub_launches(ctx) == expected);                      // waits
        void* a = block(8192); void* b = block(8192); void* r = block(8192); void* o = block(8192);
        dev.matmul(half(a, 64, 64), half(b, 64, 64), half(r, 64, 64));
        CHECK(stub_launches(ctx) == expected);                      // waits in a group of its own
        dev.transpose(half(r, 64, 64), half(o, 64, 64), 0, 1);      // its result is read: that group leaves, the other stays
        expected += 2;
        CHECK(stub_launches(ctx) == expected);
        dev.transpose(half(wa[i], 128, 64), half(o, 64, 128), 0, 1);    // reading what a waiting product reads disturbs nothing
        expected += 1;
        CHECK(stub_launches(ctx) == expected);
    }
    stub_log_clear(ctx);
    dev.transpose(half(x, 4, 4), half(wb[1], 4, 4), 0, 1);          // an operand of a waiting product is overwritten: the three go first
    expected += 4;
    CHECK(stub_launches(ctx) == expected);
    const std::string log = stub_log(ctx);
    CHECK(log == "aixk_matmul;aixk_matmul;aixk_matmul;aixk_transpose;");
    // two groups wait; the reader of one result leaves the other group waiting, flush(true) sends it off
    void* a = block(8192); void* b = block(8192); void* r = block(8192);
    dev.matmul(half(wa[0], 128, 64), half(wb[0], 64, 128), half(wr[0], 128, 128));
    dev.matmul(half(a, 64, 64), half(b, 64, 64), half(r, 64, 64));
    CHECK(stub_launches(ctx) == expected);
    dev.transpose(half(wr[0], 128, 128), half(wr[2], 128, 128), 0, 1);
    expected += 2;
    CHECK(stub_launches(ctx) == expected);
    dev.flush();
    expected += 1;
    CHECK(stub_launches(ctx) == expected);
    // a product that reads a waiting result sends only that result's group off and then waits itself
    dev.matmul(half(wa[0], 128, 64), half(wb[0], 64, 128), half(wr[0], 128, 128));
    dev.matmul(half(a, 64, 64), half(b, 64, 64), half(r, 64, 64));
    dev.matmul(half(r, 64, 64), half(b, 64, 64), half(a, 64, 64));
    expected += 1;
    CHECK(stub_launches(ctx) == expected);
    dev.synchronize();
    expected += 2;
    CHECK(stub_launches(ctx) == expected);
    (void)y;
    for (void* p : all) dev.deallocate(p);
    dev.synchronize();
    CHECK(dev.allocatedBytes() == 0);
}

// A fill that nothing has read yet is normally set aside at a flush and waits for its first user.  A call that waits
// (a small product, a sliceSet) and is about to overwrite the fill's buffer is such a user: the fill leaves before the call,
// never behind it -- behind it, it would wipe the call's result, and a recorded reader would take the fill's constant.
static void test_fills_do_not_land_behind_calls_that_wait()
{
    auto half = [](void* p, size_t rows = 64) { DeviceTensorParams t = matrix(p, rows, 64); t.dtype = DataType::kBFloat16; return t; };
    auto at = [](const std::string& log, const char* what, size_t from = 0) { return log.find(what, from); };
    const float zero = 0.0f;
    {   // fill(r); matmul(a, b, r); exp(r) -> o
        DeviceHIP dev;
        aixk_ctx* ctx = dev.kernelContext();
        void* a = dev.allocate(8192); void* b = dev.allocate(8192); void* r = dev.allocate(8192); void* o = dev.allocate(8192);
        stub_log_clear(ctx);
        dev.fill(&zero, DataType::kFloat32, half(r));
        dev.matmul(half(a), half(b), half(r));
        dev.exp(half(r), half(o));
        dev.synchronize();
        const std::string log = stub_log(ctx);
        const size_t product = at(log, "aixk_matmul"), reader = std::min(at(log, "Exp"), at(log, "aixk_unary"));
        const size_t fill = std::min(at(log, "aixk_fill"), at(log, "Fill"));
        CHECK(product != std::string::npos && reader != std::string::npos);
        CHECK(fill == std::string::npos || fill < product);                  // (a fill that is dropped as dead would do as well)
        CHECK(product < reader);
        CHECK(at(log, "aixk_fill", product) == std::string::npos && at(log, "Fill", product) == std::string::npos);
        if (g_failed) std::printf("launch order: %s\n", log.c_str());
        for (void* p : {a, b, r, o}) dev.deallocate(p);
    }
    {   // a fill through another view of the destination cannot be folded into sliceSet: it goes first all the same
        DeviceHIP dev;
        aixk_ctx* ctx = dev.kernelContext();
        void* s = dev.allocate(2048); void* r = dev.allocate(8192); void* o = dev.allocate(8192);
        stub_log_clear(ctx);
        dev.fill(&zero, DataType::kFloat32, half(r, 32));
        dev.sliceSet(half(s, 16), half(r), 0, 0, 16, 1);
        dev.exp(half(r), half(o));
        dev.synchronize();
        const std::string log = stub_log(ctx);
        const size_t window = at(log, "aixk_slice_set"), reader = std::min(at(log, "Exp"), at(log, "aixk_unary"));
        const size_t fill = std::min(at(log, "aixk_fill"), at(log, "Fill"));
        CHECK(window != std::string::npos && reader != std::string::npos && fill != std::string::npos);
        CHECK(fill < window && window < reader);
        CHECK(at(log, "aixk_fill", window) == std::string::npos && at(log, "Fill", window) == std::string::npos);
        if (g_failed) std::printf("launch order: %s\n", log.c_str());
        for (void* p : {s, r, o}) dev.deallocate(p);
    }
}

// The pool of idle blocks is cut back to the cache limit at every synchronize(): the fullest bucket first, its coldest
// blocks first (aixDeviceMetal.cpp:1369-1373, aixDeviceMetalCache.hpp:97-124).  Live blocks and blocks the GPU may still
// use are never given back.
static void test_the_pool_is_trimmed_to_the_cache_limit()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    CHECK(dev.cacheLimit() == (size_t)((double)(1ull << 30) * 0.7));      // the stub's card has 1 GiB
    std::vector<void*> big, small;
    for (int i = 0; i < 8; ++i) big.push_back(dev.allocate(1 << 20));
    for (int i = 0; i < 4; ++i) small.push_back(dev.allocate(4096));
    void* live = dev.allocate(1 << 20);
    touch(dev, big[0], big[1], live);                   // some of them have been used by the GPU
    for (void* p : big) dev.deallocate(p);
    for (void* p : small) dev.deallocate(p);
    dev.synchronize();
    CHECK(dev.cachedBytes() == 8 * (size_t(1) << 20) + 4 * 4096);         // under the default limit: all of it is kept
    const uint64_t frees = stub_frees(ctx);
    dev.setCacheLimit(3 * (size_t(1) << 20));
    dev.synchronize();
    CHECK(dev.cachedBytes() <= 3 * (size_t(1) << 20));
    CHECK(dev.cachedBytes() == 2 * (size_t(1) << 20) + 4 * 4096);         // six of the fullest bucket went, the small ones stay
    CHECK(stub_frees(ctx) == frees + 6);
    CHECK(dev.allocatedBytes() == (size_t(1) << 20) && dev.isDeviceMemory(live));
    // the two that stayed are the ones that came back to the pool last (the two the GPU had used: they waited for it, the
    // others were idle at the flush): the top of the stack.  They are handed out again, nothing new is asked for.
    const uint64_t allocs = stub_allocs(ctx);
    void* a = dev.allocate(1 << 20); void* b = dev.allocate(1 << 20);
    CHECK(stub_allocs(ctx) == allocs);
    CHECK((a == big[1] && b == big[0]) || (a == big[0] && b == big[1]));
    dev.setCacheLimit(0);                               // nothing idle is kept
    dev.deallocate(a); dev.deallocate(b); dev.deallocate(live);
    dev.synchronize();
    CHECK(dev.cachedBytes() == 0 && dev.allocatedBytes() == 0 && stub_held(ctx) == 0);
}

// A captured step: blocks that the captured work uses may go round inside the capture (everything there is ordered on the
// stream), but once the capture is closed they are never handed out again while a graph lives -- a replay writes into
// them -- and come back to the pool when the last graph is destroyed.  Nothing runs inside a capture, so synchronize()
// refuses; a replay enqueues the captured launches again, in their order.
static void test_blocks_of_a_captured_step_stay_with_the_graph()
{
    DeviceHIP dev;
    aixk_ctx* ctx = dev.kernelContext();
    void* a = dev.allocate(64); void* b = dev.allocate(64); void* out = dev.allocate(64);
    touch(dev, a, b, out);
    dev.synchronize();
    stub_log_clear(ctx);
    dev.beginCapture();
    CHECK(dev.capturing());
    CHECK(throws<std::runtime_error>([&] { dev.synchronize(); }));
    void* t1 = dev.allocate(5000);
    touch(dev, a, b, t1);                               // captured work writes t1
    dev.deallocate(t1);
    dev.flush();
    void* t2 = dev.allocate(5000);                      // inside the capture the freed block comes round again
    CHECK(t2 == t1);
    touch(dev, t2, b, out);
    dev.deallocate(t2);
    void* idle = dev.allocate(7000);                    // never used by captured work: an ordinary block
    dev.deallocate(idle);
    DeviceHIP::StepGraph* graph = dev.endCapture();
    CHECK(!dev.capturing() && graph != nullptr && dev.graphNodes(graph) == 2);
    const std::string captured = stub_log(ctx);
    const uint64_t allocs = stub_allocs(ctx);
    void* other = dev.allocate(5000);                   // the graph's temporary is not handed out: a fresh block
    CHECK(other != t1 && stub_allocs(ctx) == allocs + 1);
    void* again = dev.allocate(7000);                   // the untouched one is
    CHECK(again == idle && stub_allocs(ctx) == allocs + 1);
    stub_log_clear(ctx);
    dev.replay(graph);
    dev.replay(graph);
    CHECK(std::string(stub_log(ctx)) == captured + captured);
    dev.synchronize();
    // a live block that captured work uses, freed while the graph lives: set aside as well
    dev.deallocate(out);
    dev.synchronize();
    void* fresh = dev.allocate(64);
    CHECK(fresh != out);
    dev.deallocate(other); dev.deallocate(again); dev.deallocate(fresh);
    dev.destroyGraph(graph);
    dev.synchronize();
    void* back = dev.allocate(5000);                    // with the last graph gone its blocks are ordinary idle blocks again
    CHECK(back == t1 || back == other);
    std::set<void*> small;
    for (int i = 0; i < 4; ++i) small.insert(dev.allocate(64));
    CHECK(small.count(out) == 1);
    for (void* p : small) dev.deallocate(p);
    for (void* p : {a, b, back}) dev.deallocate(p);
    dev.synchronize();
    CHECK(dev.allocatedBytes() == 0);
}

static void test_destruction_returns_everything()
{
    const long long before = stub_held_everywhere();
    {
        DeviceHIP dev;
        stub_set_event_delay(dev.kernelContext(), 1000);
        void* a = dev.allocate(5000); void* b = dev.allocate(70000); void* c = dev.allocate(300);
        touch(dev, a, b, c);
        dev.deallocate(b);                              // in limbo
        for (int i = 0; i < 16; ++i) dev.flush();       // now cooling behind an event that never completes
        void* d = dev.allocate(70000);
        dev.deallocate(d);                              // in limbo, never flushed
        (void)a; (void)c;                               // still alive when the device goes away
    }
    CHECK(stub_held_everywhere() == before);
}

int main(int argc, char** argv)
{
    const bool threads = argc > 1 && std::string(argv[1]) == "threads";
    test_buckets_and_errors();
    test_untouched_temporaries_recycle_at_the_flush();
    test_used_blocks_wait_for_the_gpu();
    test_out_of_memory_retry();
    test_blocks_of_calls_that_wait_are_not_handed_out();
    test_groups_of_products_leave_apart();
    test_fills_do_not_land_behind_calls_that_wait();
    test_the_pool_is_trimmed_to_the_cache_limit();
    test_blocks_of_a_captured_step_stay_with_the_graph();
    test_destruction_returns_everything();
    for (unsigned seed = 1; seed <= 4; ++seed) stress(seed, 20000);
    for (unsigned seed = 21; seed <= 24; ++seed) planner_traffic(seed, 3000);
    if (threads) {
        // one device per thread is the contract (no locks inside a device): two devices side by side must share nothing
        std::thread t1(stress, 11u, 20000), t2(stress, 12u, 20000);
        t1.join(); t2.join();
        std::thread t3(planner_traffic, 31u, 2000), t4(planner_traffic, 32u, 2000);
        t3.join(); t4.join();
    }
    CHECK(stub_held_everywhere() == 0);
    if (g_failed) { std::printf("%d allocator checks FAILED\n", g_failed); return 1; }
    std::printf("all allocator checks passed\n");
    return 0;
}
