// test_planner.cpp -- the fusion planner and the HIP source generator, without a GPU.
//
// Pattern of the reference's planner tests (Targets/AIXTests/DeviceTests.cpp:235-289,
// 1810-1879): drive the engine with fake callbacks that capture what it emits, and check the
// descriptors.  Additionally every generated kernel source is compiled with hipRTC for gfx950
// (cross-compilation needs no GPU), so a generator bug fails here, not on the GPU box.
//
// Prints one line per check and exits non-zero if any failed.

#include "device/fuse.hpp"
#include "device/hipgen.hpp"

#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

using namespace aixhip::fuse;
namespace gen = aixhip::gen;
using aix::DataType;
using aix::DeviceTensorParams;

namespace aix {
Device::~Device() = default;
size_t Device::dataTypeSize(DataType dtype)
{
    static const size_t bytes[DataTypeCount] = {8, 4, 2, 2, 8, 4, 2, 1, 1};
    return bytes[static_cast<size_t>(dtype)];
}
} // namespace aix

static int g_failed = 0;
static std::string g_prelude;

#define CHECK(cond)                                                                    \
    do {                                                                               \
        if (!(cond)) { std::printf("FAIL %s:%d  %s\n", __FILE__, __LINE__, #cond); ++g_failed; } \
    } while (0)

static DeviceTensorParams T(uintptr_t id, aix::Shape shape, DataType dt = DataType::kFloat32, aix::Stride strides = {}, size_t offset = 0)
{
    DeviceTensorParams p;
    p.data = reinterpret_cast<void*>(id * 0x10000);
    p.dtype = dt;
    p.shape = shape;
    p.offset = offset;
    size_t n = 1;
    for (auto e : shape) n *= e;
    p.size = n;
    if (strides.empty()) { strides.resize(shape.size()); size_t run = 1; for (size_t d = shape.size(); d-- > 0;) { strides[d] = run; run *= shape[d]; } }
    p.strides = strides;
    bool dense = true; size_t run = 1;
    for (size_t d = shape.size(); d-- > 0;) { if (strides[d] != run) dense = false; run *= shape[d]; }
    p.isContiguous = dense;
    return p;
}

struct Capture {
    std::vector<FusedSubgraphDescriptor> fused;
    std::vector<OpRecord> singles;
    std::vector<std::string> order;           // "F<k>" or "S:<Op>"
    int finishes = 0;
    FuseCallbacks callbacks()
    {
        FuseCallbacks cb;
        cb.emitFused = [this](const FusedSubgraphDescriptor& d) { order.push_back("F" + std::to_string(fused.size())); fused.push_back(d); };
        cb.emitSingle = [this](const OpRecord& op) { order.push_back(std::string("S:") + opName(op.type)); singles.push_back(op); };
        cb.finishFlush = [this] { ++finishes; };
        return cb;
    }
};

static FuseConfig config(bool fusion = true)
{
    FuseConfig c;
    c.maxBufferSlots = 24;
    c.diagnostics = true;
    c.elementwiseFusion = fusion;
    return c;
}

// Compiles one generated kernel for gfx950; returns true on success.
static bool compiles(const FusedSubgraphDescriptor& d, gen::Shape shape)
{
    const std::string src = gen::source(d, shape);
    hiprtcProgram prog;
    const char* names[] = {"aix_device.h"};
    const char* texts[] = {g_prelude.c_str()};
    if (hiprtcCreateProgram(&prog, src.c_str(), "t.hip", 1, texts, names) != HIPRTC_SUCCESS) return false;
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off"};
    const hiprtcResult r = hiprtcCompileProgram(prog, 4, opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0; hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, 0); if (n) hiprtcGetProgramLog(prog, &log[0]);
        std::printf("---- hipRTC log ----\n%s\n---- source ----\n%s\n", log.c_str(), src.c_str());
    }
    hiprtcDestroyProgram(&prog);
    return r == HIPRTC_SUCCESS;
}

static float scalarAt(const FusedSubgraphDescriptor& d, size_t k) { float v; std::memcpy(&v, d.scalarData.data() + 4 * k, 4); return v; }

// tanh(a*b + c) / (1 + exp(-a)) - 0.5*c with every temporary released before the flush.
static void recordChain(FuseEngine& e, float one, float half, bool releaseTemps, const aix::Shape& shape = {4096, 4096})
{
    auto a = T(1, shape), b = T(2, shape), c = T(3, shape), y = T(20, shape);
    auto t = [&](uintptr_t k) { return T(10 + k, shape); };
    for (uintptr_t id : {1, 2, 3, 20, 11, 12, 13, 14, 15, 16, 17, 18, 30, 31}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Mul, a, b, t(1));
    e.record(OpType::Add, t(1), c, t(2));
    e.record(OpType::Tanh, t(2), t(3));
    e.record(OpType::Negate, a, t(4));
    e.record(OpType::Exp, t(4), t(5));
    auto s1 = T(30, {}), s2 = T(31, {});
    e.recordFill(&one, DataType::kFloat32, s1);
    aix::Stride zeros(shape.size(), 0);
    auto s1b = T(30, shape, DataType::kFloat32, zeros), s2b = T(31, shape, DataType::kFloat32, zeros);
    e.record(OpType::Add, s1b, t(5), t(6));
    e.record(OpType::Div, t(3), t(6), t(7));
    e.recordFill(&half, DataType::kFloat32, s2);
    e.record(OpType::Mul, s2b, c, t(8));
    e.record(OpType::Sub, t(7), t(8), y);
    if (releaseTemps)
        for (uintptr_t id : {11, 12, 13, 14, 15, 16, 17, 18, 30, 31}) e.releaseBuffer(reinterpret_cast<void*>(id * 0x10000));
}

static void testChainBecomesOneDenseKernel()
{
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    recordChain(e, 1.0f, 0.5f, true);
    CHECK(e.pendingOps() == 11);
    e.flush();
    CHECK(cap.finishes == 1);
    CHECK(cap.singles.empty());
    CHECK(cap.fused.size() == 1);
    if (cap.fused.size() != 1) return;
    const auto& d = cap.fused[0];
    CHECK(d.ops.size() == 9);                      // the two fills became immediates
    CHECK(d.inputBuffers.size() == 3);             // a, b, c: each loaded once
    CHECK(d.outputBuffers.size() == 1);            // only y reaches memory
    CHECK(d.scalarData.size() == 8);
    CHECK(scalarAt(d, 0) == 1.0f && scalarAt(d, 1) == 0.5f);
    CHECK(d.allContiguous);                        // contiguity is judged on materialised buffers only
    CHECK(d.elementCount == 4096u * 4096u);
    CHECK(d.dtype == DataType::kFloat32);
    const auto& diag = e.lastFlushDiagnostics();
    CHECK(diag.opsRecorded == 11 && diag.fusibleSubgraphs == 1 && diag.fusedOps == 9 && diag.fallbackOps == 0);
    CHECK(diag.fillsAbsorbed == 2 && diag.dispatchesSaved == 8);
    CHECK(compiles(d, gen::Shape::Flat));
    CHECK(compiles(d, gen::Shape::Rows));
    CHECK(compiles(d, gen::Shape::Gather));
    // immediates' values are arguments: another value, same kernel identity (DeviceTests.cpp:1774-1807)
    Capture cap2;
    FuseEngine e2(config(), cap2.callbacks());
    recordChain(e2, 1.0f, 0.25f, true);
    e2.flush();
    CHECK(cap2.fused.size() == 1);
    if (cap2.fused.size() == 1) {
        CHECK(gen::signature(cap2.fused[0], gen::Shape::Flat) == gen::signature(d, gen::Shape::Flat));
        CHECK(scalarAt(cap2.fused[0], 1) == 0.25f);
        CHECK(gen::signature(d, gen::Shape::Flat) != gen::signature(d, gen::Shape::Gather));
    }
}

static void testOperandOrderDoesNotSplitTheKernel()
{
    // C++ leaves the evaluation order of a - b open: record the right operand's subtree first.
    // t8 = 0.5*c starts its own group, the rest grows another; the final sub joins them.
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    aix::Shape shape{512, 512};
    auto a = T(1, shape), b = T(2, shape), c = T(3, shape), y = T(20, shape);
    auto t = [&](uintptr_t k) { return T(10 + k, shape); };
    for (uintptr_t id : {1, 2, 3, 20, 11, 12, 13, 14, 15, 16, 17, 18, 30, 31}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    const float one = 1.0f, half = 0.5f;
    aix::Stride zeros(2, 0);
    e.recordFill(&half, DataType::kFloat32, T(31, {}));
    e.record(OpType::Mul, T(31, shape, DataType::kFloat32, zeros), c, t(8));
    e.recordFill(&one, DataType::kFloat32, T(30, {}));
    e.record(OpType::Negate, a, t(4));
    e.record(OpType::Exp, t(4), t(5));
    e.record(OpType::Add, T(30, shape, DataType::kFloat32, zeros), t(5), t(6));
    e.record(OpType::Mul, a, b, t(1));
    e.record(OpType::Add, t(1), c, t(2));
    e.record(OpType::Tanh, t(2), t(3));
    e.record(OpType::Div, t(3), t(6), t(7));
    e.record(OpType::Sub, t(7), t(8), y);
    for (uintptr_t id : {11, 12, 13, 14, 15, 16, 17, 18, 30, 31}) e.releaseBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.flush();
    CHECK(cap.singles.empty());
    CHECK(cap.fused.size() == 1);
    if (cap.fused.size() != 1) return;
    CHECK(cap.fused[0].ops.size() == 9 && cap.fused[0].inputBuffers.size() == 3 && cap.fused[0].outputBuffers.size() == 1);
    CHECK(cap.fused[0].ops[0].type == OpType::Mul && cap.fused[0].ops.back().type == OpType::Sub);     // program order kept
    CHECK(compiles(cap.fused[0], gen::Shape::Flat));
}

static void testLiveTemporariesAreStoredAndFillsRun()
{
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    recordChain(e, 1.0f, 0.5f, false, {64, 64});
    e.flush();
    CHECK(cap.fused.size() == 1);
    if (cap.fused.size() != 1) return;
    CHECK(cap.fused[0].outputBuffers.size() == 9);             // t1..t8 and y
    CHECK(cap.singles.size() == 2);                            // the two scalar tensors are alive: their fills run
    for (const auto& s : cap.singles) CHECK(s.type == OpType::Fill);
    CHECK(compiles(cap.fused[0], gen::Shape::Flat));
}

static void testFusionDisabledReplaysInOrder()
{
    Capture cap;
    FuseEngine e(config(false), cap.callbacks());
    recordChain(e, 1.0f, 0.5f, true, {8, 8});
    e.flush();
    CHECK(cap.fused.empty());
    CHECK(cap.singles.size() == 11);
    const OpType want[] = {OpType::Mul, OpType::Add, OpType::Tanh, OpType::Negate, OpType::Exp, OpType::Fill, OpType::Add,
                           OpType::Div, OpType::Fill, OpType::Mul, OpType::Sub};
    for (size_t k = 0; k < cap.singles.size() && k < 11; ++k) CHECK(cap.singles[k].type == want[k]);
}

static void testInPlaceUpdatesKeepProgramOrder()
{
    // x = a + b; x += c; x *= x; y = x - a      (in-place: result aliases operand 0, DeviceTests.cpp:1882-1910)
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    aix::Shape s{1000};
    auto a = T(1, s), b = T(2, s), c = T(3, s), x = T(4, s), y = T(5, s);
    for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Add, a, b, x);
    e.record(OpType::Add, x, c, x);
    e.record(OpType::Mul, x, x, x);
    e.record(OpType::Sub, x, a, y);
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() != 1) return;
    const auto& d = cap.fused[0];
    CHECK(d.ops.size() == 4);
    CHECK(d.inputBuffers.size() == 3);
    CHECK(d.outputBuffers.size() == 2);                        // final x and y; earlier values of x never stored
    size_t stores = 0;
    for (const auto& op : d.ops) if (op.outputIndex != SIZE_MAX) ++stores;
    CHECK(stores == 2);
    CHECK(d.ops[2].outputIndex != SIZE_MAX && d.ops[0].outputIndex == SIZE_MAX && d.ops[1].outputIndex == SIZE_MAX);
    CHECK(d.ops[2].inputIndex0 == 3 + 1 && d.ops[2].inputIndex1 == 3 + 1);      // x*x reads the register value of op 1
    CHECK(compiles(d, gen::Shape::Flat));
}

static void testDifferentViewOfAProducedBufferSplitsKernels()
{
    // t = a * b   [64, 32];   u = t^T (stride-swapped view) + c   [32, 64]
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto a = T(1, {64, 32}), b = T(2, {64, 32}), t = T(3, {64, 32}), c = T(4, {32, 64}), u = T(5, {32, 64});
    auto tT = T(3, {32, 64}, DataType::kFloat32, {1, 32});
    for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Mul, a, b, t);
    e.record(OpType::Add, tT, c, u);
    e.releaseBuffer(t.data);                                   // temporary, but the second op loads it
    e.flush();
    CHECK(cap.fused.empty());                                  // two kernels of one op each run as plain operators
    CHECK(cap.singles.size() == 2);
    if (cap.singles.size() == 2) { CHECK(cap.singles[0].type == OpType::Mul); CHECK(cap.singles[1].type == OpType::Add); }
}

static void testWriteAfterReadClosesTheReader()
{
    // u = a + b; v = u * u; then a is overwritten: a = c - c.  The kernel reading the old a must run first.
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    aix::Shape s{256};
    auto a = T(1, s), b = T(2, s), c = T(3, s), u = T(4, s), v = T(5, s);
    for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Add, a, b, u);
    e.record(OpType::Mul, u, u, v);
    e.record(OpType::Sub, c, c, a);
    e.record(OpType::Negate, a, b);
    e.flush();
    CHECK(cap.order.size() == 2);
    CHECK(cap.fused.size() == 2);
    if (cap.fused.size() != 2) return;
    CHECK(cap.fused[0].ops.size() == 2 && cap.fused[0].ops[0].type == OpType::Add);
    CHECK(cap.fused[1].ops.size() == 2 && cap.fused[1].ops[0].type == OpType::Sub);
    CHECK(compiles(cap.fused[1], gen::Shape::Flat));
}

static void testRowBroadcastStaysInOneKernel()
{
    // h = x + bias (bias broadcast along rows), r = tanh(h): what Linear + activation records
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto x = T(1, {128, 256}), bias = T(2, {128, 256}, DataType::kFloat32, {0, 1}), h = T(3, {128, 256}), r = T(4, {128, 256});
    for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Add, x, bias, h);
    e.record(OpType::Tanh, h, r);
    e.releaseBuffer(h.data);
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() != 1) return;
    CHECK(!cap.fused[0].allContiguous);
    CHECK(cap.fused[0].outputBuffers.size() == 1);
    CHECK(compiles(cap.fused[0], gen::Shape::Rows));
    CHECK(compiles(cap.fused[0], gen::Shape::Gather));
}

static void testDeadCodeIsDropped()
{
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto a = T(1, {10}), b = T(2, {10}), t = T(3, {10}), u = T(4, {10});
    for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.record(OpType::Mul, a, b, t);
    e.record(OpType::Exp, t, u);
    e.releaseBuffer(t.data);
    e.releaseBuffer(u.data);
    e.flush();
    CHECK(cap.order.empty());
}

static void testThresholdFlushAndExternalRead()
{
    Capture cap;
    FuseConfig c = config();
    c.flushThreshold = 4;
    FuseEngine e(c, cap.callbacks());
    auto a = T(1, {10}), t = T(2, {10});
    e.retainBuffer(a.data);
    e.record(OpType::Exp, a, t);            // t never retained: only an external read keeps it
    e.record(OpType::Exp, t, t);
    e.record(OpType::Exp, t, t);
    CHECK(cap.finishes == 0);
    e.recordExternalRead(t.data);
    e.record(OpType::Exp, t, t);            // fourth op: planning runs by itself
    CHECK(cap.finishes == 1);
    CHECK(cap.fused.size() == 1);
    if (cap.fused.size() == 1) CHECK(cap.fused[0].outputBuffers.size() == 1 && cap.fused[0].ops.size() == 4);
}

static void testFillMinAndIntegerScalars()
{
    // m = max-style init: fillMin(t); u = t + a  (int32): the immediate is INT_MIN; a float fill into an int8 tensor saturates
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto a = T(1, {100}, DataType::kInt32), t = T(2, {100}, DataType::kInt32), u = T(3, {100}, DataType::kInt32);
    for (uintptr_t id : {1, 2, 3}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.recordFillMin(t);
    e.record(OpType::Add, t, a, u);
    e.releaseBuffer(t.data);
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() == 1) {
        int32_t v; std::memcpy(&v, cap.fused[0].scalarData.data(), 4);
        CHECK(v == INT32_MIN);
        CHECK(compiles(cap.fused[0], gen::Shape::Flat));
    }
    const float big = 300.0f;
    auto bytes = convertScalar(&big, DataType::kFloat32, DataType::kInt8);
    CHECK(bytes.size() == 1 && (int8_t)bytes[0] == 127);
    const float nan = __builtin_nanf("");
    bytes = convertScalar(&nan, DataType::kFloat32, DataType::kInt32);
    int32_t z; std::memcpy(&z, bytes.data(), 4);
    CHECK(z == 0);
    const float pi = 3.14f;
    bytes = convertScalar(&pi, DataType::kFloat32, DataType::kFloat16);
    uint16_t h; std::memcpy(&h, bytes.data(), 2);
    CHECK(h == 0x4248);                                        // Float16Tests.cpp:25-31
}

static void testEveryTypeAndOperatorCompiles()
{
    const OpType unary[] = {OpType::Negate, OpType::Sqrt, OpType::Sin, OpType::Cos, OpType::Tanh, OpType::Log, OpType::Exp};
    const OpType binary[] = {OpType::Add, OpType::Sub, OpType::Mul, OpType::Div, OpType::Pow};
    for (size_t dt = 0; dt < aix::DataTypeCount; ++dt) {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        const DataType t = static_cast<DataType>(dt);
        auto a = T(1, {50}, t), b = T(2, {50}, t);
        e.retainBuffer(a.data); e.retainBuffer(b.data);
        uintptr_t next = 3;
        DeviceTensorParams cur = a;
        for (OpType op : binary) { auto o = T(next++, {50}, t); e.record(op, cur, b, o); cur = o; }
        for (OpType op : unary) { auto o = T(next++, {50}, t); e.record(op, cur, o); cur = o; }
        e.retainBuffer(cur.data);
        e.flush();
        CHECK(cap.fused.size() == 1);
        if (cap.fused.size() == 1) { CHECK(cap.fused[0].ops.size() == 12); CHECK(compiles(cap.fused[0], gen::Shape::Flat)); }
    }
}

static void testPointerSetGrowsAndForgets()
{
    PointerSet set;
    CHECK(!set.contains(reinterpret_cast<void*>(0x1000)));
    const size_t n = 50000;
    for (size_t i = 1; i <= n; ++i) set.insert(reinterpret_cast<void*>(i * 0x100));
    CHECK(set.size() == n);
    bool all = true;
    for (size_t i = 1; i <= n; ++i) if (!set.contains(reinterpret_cast<void*>(i * 0x100))) all = false;
    CHECK(all);
    CHECK(!set.contains(reinterpret_cast<void*>((n + 1) * 0x100)) && !set.contains(reinterpret_cast<void*>(0x80)));
    set.insert(reinterpret_cast<void*>(0x100));                      // twice: still one member
    CHECK(set.size() == n);
    for (size_t i = 1; i <= n; i += 2) set.erase(reinterpret_cast<void*>(i * 0x100));
    CHECK(set.size() == n / 2);
    bool odd_gone = true, even_there = true;
    for (size_t i = 1; i <= n; ++i) {
        const bool in = set.contains(reinterpret_cast<void*>(i * 0x100));
        if (i % 2 == 1 && in) odd_gone = false;
        if (i % 2 == 0 && !in) even_there = false;
    }
    CHECK(odd_gone && even_there);
    // allocate / free churn over the same addresses: graves are reused, lookups stay exact
    for (int round = 0; round < 200; ++round)
        for (size_t i = 1; i <= 300; i += 2) {
            void* p = reinterpret_cast<void*>(i * 0x100);
            set.insert(p);
            if (!set.contains(p)) { CHECK(false); return; }
            set.erase(p);
        }
    CHECK(set.size() == n / 2);
}

static void testViewLimitsAndRoundTrip()
{
    auto p = T(5, {3, 1, 4}, DataType::kInt16, {4, 99, 1}, 7);           // an extent-1 dimension may carry any stride
    View v(p);
    CHECK(v.rank == 3 && v.dense && v.offset == 7 && v.size == 12 && v.dtype == DataType::kInt16);
    const auto q = v.params();
    CHECK(q.data == p.data && q.shape == p.shape && q.strides == p.strides && q.offset == 7 && q.size == 12);
    View w(T(5, {3, 4}, DataType::kInt16, {1, 3}));
    CHECK(!w.dense);
    w.makeDense();
    CHECK(w.dense && w.offset == 0 && w.strides[0] == 4 && w.strides[1] == 1);
    bool threw = false;
    try { View too(T(6, aix::Shape(17, 1))); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw);
    View copy = v;                                                        // copies carry only the meaningful extents
    CHECK(copy.sameShape(v) && copy.strides[1] == 99 && copy.sameShape(aix::Shape{3, 1, 4}) && !copy.sameShape(aix::Shape{3, 4}));
}

static void testEngineStorageIsReusedAcrossWindows()
{
    // many windows through one engine: the descriptor handed out is the engine's own and is refilled,
    // results do not depend on what earlier windows left behind
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    for (int round = 0; round < 50; ++round) {
        const aix::Shape shape{64, (size_t)(8 + round)};
        recordChain(e, 1.0f, 0.5f, true, shape);
        if (round % 3 == 0) {                                            // a second, unrelated kernel in the same window
            auto x = T(40, {10}), y = T(41, {10}), z = T(42, {10});
            for (uintptr_t id : {40, 41, 42}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
            e.record(OpType::Add, x, y, z);
            e.record(OpType::Exp, z, z);
        }
        e.flush();
    }
    CHECK(cap.fused.size() == 50 + 17);
    bool ok = true;
    size_t chains = 0;
    for (const auto& d : cap.fused) {
        if (d.ops.size() == 9) { ++chains; if (d.inputBuffers.size() != 3 || d.outputBuffers.size() != 1 || d.scalarData.size() != 8) ok = false; }
        else if (d.ops.size() != 2 || d.inputBuffers.size() != 2 || d.outputBuffers.size() != 1 || d.elementCount != 10) ok = false;
    }
    CHECK(ok && chains == 50);
}

static void testTrailingFillIsHandedOver()
{
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto a = T(1, {8, 8}), d = T(2, {8}), other = T(3, {8});
    for (uintptr_t id : {1, 2, 3}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    const float zero = 0.0f, seven = 7.0f;
    e.recordFill(&seven, DataType::kFloat32, other);
    e.recordFill(&zero, DataType::kFloat32, d);
    OpRecord fill;
    CHECK(e.takeTrailingFill(d, &fill));                                  // newest operator on d is a fill of all of d
    CHECK(fill.type == OpType::Fill && fill.output.data == d.data && e.pendingOps() == 1);
    float got; std::memcpy(&got, fill.scalarData.data(), 4);
    CHECK(got == 0.0f);
    CHECK(!e.takeTrailingFill(d, &fill));                                 // nothing left for d
    e.recordFill(&zero, DataType::kFloat32, d);
    e.record(OpType::Add, d, other, a.data == nullptr ? d : T(4, {8}));   // somebody reads d after the fill
    CHECK(!e.takeTrailingFill(d, &fill));
    e.flush();
}

static void testCastsFuseAtTheirLoadOrStoreEnd()
{
    const aix::Shape shape{128, 96};
    const size_t n = 128 * 96;
    // (a * b) converted to bf16: the conversion joins the kernel that holds the product in a register
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto a = T(1, shape), b = T(2, shape), t = T(3, shape);
        auto flat = T(3, {n}), out = T(4, {n}, DataType::kBFloat16);
        for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        e.record(OpType::Mul, a, b, t);
        e.record(OpType::Cast, flat, out);
        e.releaseBuffer(reinterpret_cast<void*>(3 * 0x10000));
        e.flush();
        CHECK(cap.singles.empty() && cap.fused.size() == 1);
        if (cap.fused.size() == 1) {
            const auto& d = cap.fused[0];
            CHECK(d.dtype == DataType::kFloat32 && d.ops.size() == 2 && d.inputBuffers.size() == 2 && d.outputBuffers.size() == 1);
            CHECK(d.outputBuffers[0].dtype == DataType::kBFloat16 && d.outputBuffers[0].data == out.data);
            CHECK(compiles(d, gen::Shape::Flat) && compiles(d, gen::Shape::Rows) && compiles(d, gen::Shape::Gather));
            CHECK(gen::signature(d, gen::Shape::Flat).find("|y0:bf16") != std::string::npos);
        }
    }
    // an int32 mask converted to f32 and multiplied: the conversion happens at the load of the kernel that multiplies
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto mask = T(1, {n}, DataType::kInt32), asFloat = T(2, {n}), asFloat2d = T(2, shape), g = T(3, shape), y = T(4, shape);
        for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        e.record(OpType::Cast, mask, asFloat);
        e.record(OpType::Mul, asFloat2d, g, y);
        e.releaseBuffer(reinterpret_cast<void*>(2 * 0x10000));
        e.flush();
        CHECK(cap.singles.empty() && cap.fused.size() == 1);
        if (cap.fused.size() == 1) {
            const auto& d = cap.fused[0];
            CHECK(d.dtype == DataType::kFloat32 && d.ops.size() == 2 && d.outputBuffers.size() == 1);
            CHECK(d.inputBuffers.size() == 2 && d.inputBuffers[0].dtype == DataType::kInt32 && d.inputBuffers[1].dtype == DataType::kFloat32);
            CHECK(compiles(d, gen::Shape::Flat) && compiles(d, gen::Shape::Rows) && compiles(d, gen::Shape::Gather));
        }
    }
    // the converted value read again in its new type: a second kernel, after the first; a fill is never an
    // immediate of a cast (its rounding to the fill's own type would be lost)
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto a = T(1, {n}), h = T(2, {n}, DataType::kFloat16), h2 = T(3, {n}, DataType::kFloat16), c = T(5, {n}, DataType::kFloat16), cf = T(6, {n});
        for (uintptr_t id : {1, 2, 3, 5, 6}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        const float tenth = 0.1f;
        e.record(OpType::Exp, a, a);                 // in place, f32
        e.record(OpType::Cast, a, h);                // joins as the last step of that kernel
        e.record(OpType::Add, h, h, h2);             // f16: must load h from memory
        e.recordFill(&tenth, DataType::kFloat32, c); // f16 tensor filled with 0.1
        e.record(OpType::Cast, c, cf);               // f16 -> f32: needs the rounded value
        e.flush();
        CHECK(cap.order.size() == 4 && cap.order[0] == "F0");
        CHECK(cap.fused.size() == 1 && cap.singles.size() == 3);
        if (cap.fused.size() == 1) {
            CHECK(cap.fused[0].dtype == DataType::kFloat32 && cap.fused[0].ops.size() == 2 && cap.fused[0].outputBuffers.size() == 2);
            CHECK(cap.fused[0].outputBuffers[1].dtype == DataType::kFloat16);
        }
        if (cap.singles.size() == 3) {                    // a lone operator runs as the plain operator
            CHECK(cap.singles[0].type == OpType::Fill && cap.singles[1].type == OpType::Add && cap.singles[2].type == OpType::Cast);
            CHECK(cap.singles[1].input0.data == h.data && cap.singles[2].input0.dtype == DataType::kFloat16);
        }
    }
    // every pair of element types, at the load and at the store
    const DataType all[] = {DataType::kFloat64, DataType::kFloat32, DataType::kFloat16, DataType::kBFloat16, DataType::kInt64,
                            DataType::kInt32, DataType::kInt16, DataType::kInt8, DataType::kUInt8};
    int built = 0;
    for (DataType from : all)
        for (DataType to : all) {
            if (from == to) continue;
            Capture cap;
            FuseEngine e(config(), cap.callbacks());
            auto x = T(1, {n}, from), xt = T(2, {n}, to), y = T(3, {n}, to), back = T(4, {n}, from);
            for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
            e.record(OpType::Cast, x, xt);           // load end
            e.record(OpType::Add, xt, xt, y);
            e.record(OpType::Cast, y, back);         // store end
            e.releaseBuffer(reinterpret_cast<void*>(2 * 0x10000));
            e.flush();
            if (cap.fused.size() != 1 || !cap.singles.empty()) { CHECK(false); continue; }
            const auto& d = cap.fused[0];
            if (!(d.dtype == to && d.ops.size() == 3 && d.outputBuffers.size() == 2)) { CHECK(false); continue; }
            if (!compiles(d, gen::Shape::Flat) || !compiles(d, gen::Shape::Gather)) { CHECK(false); continue; }
            ++built;
        }
    CHECK(built == 72);
}

static void testDenseSidesAdoptTheStridedSidesShape()
{
    const size_t r = 48, c = 32, n = r * c;
    auto flat = [&](uintptr_t id) { return T(id, {n}); };
    auto mat = [&](uintptr_t id) { return T(id, {r, c}); };
    auto rowOf = [&](uintptr_t id) { return T(id, {r, c}, DataType::kFloat32, {0, 1}); };     // a [c] vector broadcast over rows
    auto colOf = [&](uintptr_t id) { return T(id, {c, r}, DataType::kFloat32, {0, 1}); };     // another shape with the same count
    // a dense group opened on a flat view takes on the shape of an operator that brings a broadcast view,
    // and a [rows, cols] result read back flat is the same register value
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        e.record(OpType::Exp, flat(1), flat(2));                 // dense, shape [n]
        e.record(OpType::Mul, mat(2), rowOf(3), mat(4));         // reads the flat result as [r, c]; broadcast operand
        e.record(OpType::Negate, flat(4), flat(5));              // a dense operator rides on the adopted shape
        e.releaseBuffer(reinterpret_cast<void*>(2 * 0x10000));
        e.releaseBuffer(reinterpret_cast<void*>(4 * 0x10000));
        e.flush();
        CHECK(cap.singles.empty() && cap.fused.size() == 1);
        if (cap.fused.size() == 1) {
            const auto& d = cap.fused[0];
            CHECK(d.ops.size() == 3 && d.inputBuffers.size() == 2 && d.outputBuffers.size() == 1 && !d.allContiguous);
            CHECK(d.shape == (aix::Shape{r, c}));
            CHECK(compiles(d, gen::Shape::Rows) && compiles(d, gen::Shape::Gather));
        }
    }
    // two sides that both bring strided views of different shapes cannot share an iteration space
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        for (uintptr_t id : {1, 2, 3, 4, 5, 6}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        e.record(OpType::Add, mat(1), rowOf(2), mat(3));         // bound to [r, c]
        e.record(OpType::Mul, T(3, {c, r}), colOf(4), T(5, {c, r}));   // the dense result viewed as [c, r], with a [c, r] broadcast
        e.flush();
        CHECK(cap.order.size() == 2);                            // two launches, in program order
        size_t launches = cap.fused.size() + cap.singles.size();
        CHECK(launches == 2);
    }
}

static void testTrilJoinsItsNeighbours()
{
    // attention scores: tril(s) * scale + mask (mask broadcast over the stack): one kernel; the triangle's extents and
    // diagonal travel as run-time integers, so another diagonal or stack size reuses the compiled kernel
    for (int upper = 0; upper < 2; ++upper) {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        const aix::Shape shape{3, 4, 64, 64};
        auto s = T(1, shape, DataType::kBFloat16), t = T(2, shape, DataType::kBFloat16), scaled = T(3, shape, DataType::kBFloat16), out = T(4, shape, DataType::kBFloat16);
        auto mask = T(5, shape, DataType::kBFloat16, {0, 0, 64, 1});
        auto scale0 = T(6, {}, DataType::kBFloat16);
        auto scale = T(6, shape, DataType::kBFloat16, {0, 0, 0, 0});
        for (uintptr_t id : {1, 2, 3, 4, 5, 6}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        const float eighth = 0.125f;
        e.recordTri(upper ? OpType::Triu : OpType::Tril, View(s), View(t), -2);
        e.recordFill(&eighth, DataType::kFloat32, View(scale0));
        e.record(OpType::Mul, View(t), View(scale), View(scaled));
        e.record(OpType::Add, View(scaled), View(mask), View(out));
        for (uintptr_t id : {2, 3, 6}) e.releaseBuffer(reinterpret_cast<void*>(id * 0x10000));
        e.flush();
        CHECK(cap.fused.size() == 1 && cap.singles.empty());
        if (cap.fused.size() != 1) continue;
        const auto& d = cap.fused[0];
        CHECK(d.ops.size() == 3 && d.ops[0].type == (upper ? OpType::Triu : OpType::Tril) && d.ops[0].paramIndex == 0);
        CHECK(d.opParams.size() == 3 && d.opParams[0] == 64 && d.opParams[1] == 64 && (int64_t)d.opParams[2] == -2);
        CHECK(d.outputBuffers.size() == 1 && d.inputBuffers.size() == 2);
        CHECK(compiles(d, gen::Shape::Rows));
        CHECK(compiles(d, gen::Shape::Gather));
        const std::string sig = gen::signature(d, gen::Shape::Rows, 0, true);
        CHECK(sig.find(upper ? "Triu(" : "Tril(") != std::string::npos && sig.find("-2") == std::string::npos);
        const auto args = gen::packArgs(d, gen::Shape::Flat, {nullptr, nullptr}, {nullptr}, 3 * 4 * 64 * 64, nullptr, 0);
        CHECK(args.size() == 2 + 1 + 1 + 3 + 1);                  // inputs, output, the scale, (rows, cols, diagonal), n
    }
    // alone in its window it runs as the plain operator
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto a = T(1, {8, 8}), b = T(2, {8, 8});
    for (uintptr_t id : {1, 2}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.recordTri(OpType::Tril, View(a), View(b), 1);
    e.flush();
    CHECK(cap.fused.empty() && cap.singles.size() == 1 && cap.singles[0].type == OpType::Tril && cap.singles[0].triDiagonal == 1);
    // a flat chain of dense tensors: the flat launch shape compiles with the index-dependent operator too
    Capture flat;
    FuseEngine f(config(), flat.callbacks());
    auto x = T(1, {16, 32, 32}), y = T(2, {16, 32, 32}), z = T(3, {16, 32, 32});
    for (uintptr_t id : {1, 2, 3}) f.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    f.record(OpType::Exp, View(x), View(y));
    f.recordTri(OpType::Triu, View(y), View(z), 0);
    f.releaseBuffer(y.data);
    f.flush();
    CHECK(flat.fused.size() == 1 && flat.singles.empty());
    if (flat.fused.size() == 1) { CHECK(flat.fused[0].allContiguous); CHECK(compiles(flat.fused[0], gen::Shape::Flat)); }
}

// Compiles one generated row program for gfx950.
static bool compilesRow(const FusedSubgraphDescriptor& d)
{
    gen::RowGeometry geo;
    if (!gen::rowGeometry(d, &geo)) { std::printf("no row geometry\n"); return false; }
    const std::string src = gen::rowSource(d, geo, false);
    if (std::getenv("AIX_PRINT_ROW_SOURCES")) std::printf("%s\n", src.c_str());
    hiprtcProgram prog;
    const char* names[] = {"aix_device.h"};
    const char* texts[] = {g_prelude.c_str()};
    if (hiprtcCreateProgram(&prog, src.c_str(), "r.hip", 1, texts, names) != HIPRTC_SUCCESS) return false;
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off"};
    const hiprtcResult r = hiprtcCompileProgram(prog, 4, opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0; hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, 0); if (n) hiprtcGetProgramLog(prog, &log[0]);
        std::printf("---- hipRTC log ----\n%s\n---- source ----\n%s\n", log.c_str(), src.c_str());
    }
    hiprtcDestroyProgram(&prog);
    return r == HIPRTC_SUCCESS;
}

static void recordSoftmax(FuseEngine& e, DataType dt, size_t rows, size_t L, uintptr_t base = 0)
{
    // (x - x.max(-1, true)).exp() / that.sum(-1, true)   (aixNeuralNetwork.hpp:188-192)
    auto id = [&](uintptr_t k) { return base + k; };
    auto x = T(id(1), {rows, L}, dt), m = T(id(2), {rows, 1}, dt), d = T(id(3), {rows, L}, dt), ex = T(id(4), {rows, L}, dt);
    auto s = T(id(5), {rows, 1}, dt), y = T(id(6), {rows, L}, dt);
    auto mB = T(id(2), {rows, L}, dt, {1, 0}), sB = T(id(5), {rows, L}, dt, {1, 0});
    for (uintptr_t k = 1; k <= 6; ++k) e.retainBuffer(reinterpret_cast<void*>(id(k) * 0x10000));
    uint8_t lowest[8] = {}, zero[8] = {};
    lowestScalarInto(dt, lowest);
    e.recordRowReduce(OpType::MaxTo, View(x), View(m), lowest, L);
    e.record(OpType::Sub, View(x), View(mB), View(d));
    e.record(OpType::Exp, View(d), View(ex));
    e.recordRowReduce(OpType::ReduceTo, View(ex), View(s), zero, L);
    e.record(OpType::Div, View(ex), View(sB), View(y));
    for (uintptr_t k : {2, 3, 4, 5}) e.releaseBuffer(reinterpret_cast<void*>(id(k) * 0x10000));
}

static void testSoftmaxBecomesOneRowProgram()
{
    for (DataType dt : {DataType::kFloat32, DataType::kBFloat16, DataType::kFloat16, DataType::kFloat64}) {
        for (size_t L : {64, 1024, 4096}) {
            Capture cap;
            FuseEngine e(config(), cap.callbacks());
            recordSoftmax(e, dt, 512, L);
            e.flush();
            CHECK(cap.fused.size() == 1 && cap.singles.empty());
            if (cap.fused.size() != 1) continue;
            const auto& d = cap.fused[0];
            CHECK(d.rowLength == L && d.elementCount == 512 * L && d.dtype == dt);
            CHECK(d.ops.size() == 5 && d.inputBuffers.size() == 1 && d.outputBuffers.size() == 1);
            CHECK(d.ops[0].type == OpType::MaxTo && d.ops[0].perRow && d.ops[0].outputIndex == SIZE_MAX && d.ops[0].scalarIndex1 != SIZE_MAX);
            CHECK(d.ops[1].type == OpType::Sub && !d.ops[1].perRow && d.ops[1].inputIndex1 == 1 + 0);       // the maximum from registers
            CHECK(d.ops[3].type == OpType::ReduceTo && d.ops[3].perRow);
            CHECK(d.ops[4].type == OpType::Div && d.ops[4].outputIndex == 0);
            gen::RowGeometry geo;
            CHECK(gen::rowGeometry(d, &geo) && geo.lanes == (L >= 2048 ? 256 : 64));
            CHECK(compilesRow(d));
            std::vector<uint64_t> args;
            const void* in[1] = {nullptr}; void* out[1] = {nullptr};
            gen::packRowArgsInto(args, d, in, out);
            CHECK(args.size() == 1 + 1 + d.scalarData.size() / aix::Device::dataTypeSize(dt) + 1 + 2);      // in, out, immediates, the input's period, rows, length
        }
    }
    // the per-row results stay visible when somebody still holds them: they are stored by the same kernel
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto x = T(1, {128, 256}), m = T(2, {128, 1}), y = T(3, {128, 256});
        auto mB = T(2, {128, 256}, DataType::kFloat32, {1, 0});
        for (uintptr_t k : {1, 2, 3}) e.retainBuffer(reinterpret_cast<void*>(k * 0x10000));
        uint8_t lowest[8]; lowestScalarInto(DataType::kFloat32, lowest);
        e.recordRowReduce(OpType::MaxTo, View(x), View(m), lowest, 256);
        e.record(OpType::Sub, View(x), View(mB), View(y));
        e.flush();
        CHECK(cap.fused.size() == 1 && cap.singles.empty());
        if (cap.fused.size() == 1) {
            CHECK(cap.fused[0].outputBuffers.size() == 2 && cap.fused[0].ops[0].outputIndex != SIZE_MAX);
            CHECK(compilesRow(cap.fused[0]));
        }
    }
    // a reduction with no elementwise company runs as the stand-alone operator, its initial value travelling along
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto x = T(1, {128, 256}), m = T(2, {128, 1});
        for (uintptr_t k : {1, 2}) e.retainBuffer(reinterpret_cast<void*>(k * 0x10000));
        const float seven = 7.0f;
        e.recordRowReduce(OpType::ReduceTo, View(x), View(m), &seven, 256);
        e.flush();
        CHECK(cap.fused.empty() && cap.singles.size() == 1 && cap.singles[0].type == OpType::ReduceTo && cap.singles[0].rowLength == 256);
        float got; std::memcpy(&got, cap.singles[0].scalarData.data(), 4);
        CHECK(got == 7.0f);
    }
    // with fusion off every record replays alone and in order
    {
        Capture cap;
        FuseEngine e(config(false), cap.callbacks());
        recordSoftmax(e, DataType::kFloat32, 64, 128);
        e.flush();
        CHECK(cap.fused.empty() && cap.singles.size() == 5);
        CHECK(cap.order == (std::vector<std::string>{"S:MaxTo", "S:Sub", "S:Exp", "S:ReduceTo", "S:Div"}));
    }
    // two softmaxes of different row lengths in one window: two kernels
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        recordSoftmax(e, DataType::kFloat32, 64, 128);
        recordSoftmax(e, DataType::kFloat32, 32, 256, 100);
        e.flush();
        CHECK(cap.fused.size() == 2 && cap.singles.empty());
        if (cap.fused.size() == 2) CHECK(cap.fused[0].rowLength == 128 && cap.fused[1].rowLength == 256);
    }
}

static void testLayerNormPiecesShareOneRowProgram()
{
    // mean = sum(x)/L; d = x - mean; var = sum(d*d)/L; y = d / sqrt(var + eps) * gamma + beta
    const size_t rows = 256, L = 768;
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto full = [&](uintptr_t k) { return T(k, {rows, L}); };
    auto col = [&](uintptr_t k) { return T(k, {rows, 1}); };
    auto colB = [&](uintptr_t k) { return T(k, {rows, L}, DataType::kFloat32, {1, 0}); };
    auto rowB = [&](uintptr_t k) { return T(k, {rows, L}, DataType::kFloat32, {0, 1}); };
    auto scalarB = [&](uintptr_t k) { return T(k, {rows, 1}, DataType::kFloat32, {0, 0}); };
    for (uintptr_t k = 1; k <= 20; ++k) e.retainBuffer(reinterpret_cast<void*>(k * 0x10000));
    const float zero = 0.0f, len = (float)L, eps = 1e-5f;
    e.recordRowReduce(OpType::ReduceTo, View(full(1)), View(col(2)), &zero, L);
    e.recordFill(&len, DataType::kFloat32, View(T(3, {})));
    e.record(OpType::Div, View(col(2)), View(scalarB(3)), View(col(4)));          // mean, one value per row
    e.record(OpType::Sub, View(full(1)), View(colB(4)), View(full(5)));
    e.record(OpType::Mul, View(full(5)), View(full(5)), View(full(6)));
    e.recordRowReduce(OpType::ReduceTo, View(full(6)), View(col(7)), &zero, L);
    e.record(OpType::Div, View(col(7)), View(scalarB(3)), View(col(8)));          // variance
    e.recordFill(&eps, DataType::kFloat32, View(T(9, {})));
    e.record(OpType::Add, View(col(8)), View(scalarB(9)), View(col(10)));
    e.record(OpType::Sqrt, View(col(10)), View(col(11)));
    e.record(OpType::Div, View(full(5)), View(colB(11)), View(full(12)));
    e.record(OpType::Mul, View(full(12)), View(rowB(13)), View(full(14)));        // gamma: one row for every row
    e.record(OpType::Add, View(full(14)), View(rowB(15)), View(full(16)));
    for (uintptr_t k : {2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 14}) e.releaseBuffer(reinterpret_cast<void*>(k * 0x10000));
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() != 1) { for (auto& o : cap.order) std::printf("  %s\n", o.c_str()); return; }
    const auto& d = cap.fused[0];
    CHECK(d.rowLength == L && d.inputBuffers.size() == 3 && d.outputBuffers.size() == 1 && d.ops.size() == 11);
    size_t perRow = 0;
    for (const auto& o : d.ops) perRow += o.perRow;
    CHECK(perRow == 6);                                                           // two sums, mean, variance, + eps, sqrt
    CHECK(compilesRow(d));
}

static void testIdleFillsWaitForTheirFirstUser()
{
    // zeroGrad() ... a long time later ... grad = grad + g: the fill is held back by the flushes in between and ends up
    // as an immediate of the accumulation; nothing is launched for it
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto grad = T(1, {512, 64}), g = T(2, {512, 64}), other = T(3, {512, 64}), sink = T(4, {512, 64});
        for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        const float zero = 0.0f;
        e.recordFill(&zero, DataType::kFloat32, View(grad));
        e.record(OpType::Exp, View(other), View(sink));
        e.flush(false);
        CHECK(cap.singles.size() == 1 && cap.singles[0].type == OpType::Exp && cap.fused.empty() && e.waitingFills() == 1);
        e.flush(false);                                             // an empty window changes nothing
        CHECK(e.waitingFills() == 1 && cap.singles.size() == 1);
        CHECK(e.pendingOps() == 0);
        e.record(OpType::Add, View(grad), View(g), View(grad));
        CHECK(e.waitingFills() == 0 && e.pendingOps() == 2);        // the fill rejoined the window ahead of its user
        e.flush(false);
        CHECK(cap.fused.size() == 1 && cap.singles.size() == 1);
        if (cap.fused.size() == 1) {
            const auto& d = cap.fused[0];
            CHECK(d.ops.size() == 1 && d.inputBuffers.size() == 1 && d.inputBuffers[0].data == g.data && d.ops[0].scalarIndex0 != SIZE_MAX);
            CHECK(scalarAt(d, d.ops[0].scalarIndex0) == 0.0f);
        }
    }
    // a final flush runs what waits; a released buffer takes its fill along; a fill somebody in the window uses, a fill of
    // part of a buffer and a fill of memory the device did not hand out never wait
    {
        Capture cap;
        FuseEngine e(config(), cap.callbacks());
        auto a = T(1, {100}), b = T(2, {100}), c = T(3, {100}), part = T(4, {50}, DataType::kFloat32, {}, 8), foreign = T(9, {100});
        for (uintptr_t id : {1, 2, 3, 4}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        const float one = 1.0f;
        e.recordFill(&one, DataType::kFloat32, View(a));
        e.recordFill(&one, DataType::kFloat32, View(b));
        e.recordFillMin(View(c));
        e.recordFill(&one, DataType::kFloat32, View(part));
        e.recordFill(&one, DataType::kFloat32, View(foreign));
        e.flush(false);
        CHECK(e.waitingFills() == 3 && cap.singles.size() == 1);    // `part` ran; nobody can read `foreign`: dropped
        if (std::getenv("AIX_TEST_VERBOSE")) { std::printf("waiting %zu singles %zu fused %zu\n", e.waitingFills(), cap.singles.size(), cap.fused.size()); for (auto& o : cap.order) std::printf("  %s\n", o.c_str()); }
        e.releaseBuffer(b.data);
        CHECK(e.waitingFills() == 2);
        e.flush();
        CHECK(e.waitingFills() == 0 && cap.singles.size() == 3);
        CHECK(cap.singles[1].type == OpType::Fill && cap.singles[1].output.data == a.data && cap.singles[2].type == OpType::FillMin);
    }
    // reading the buffer outside the planner, asking whether work on it is pending, or folding the fill into an eager
    // operator brings it back; so does an operand that points into the middle of the filled block (the device fences such
    // operands with flushes of its own: the planner orders operators by buffer address)
    {
        Capture cap;
        auto cb = cap.callbacks();
        cb.blockBase = [](const void* p) { return reinterpret_cast<const void*>(reinterpret_cast<uintptr_t>(p) & ~uintptr_t(0xFFFF)); };
        FuseEngine e(config(), cb);
        auto a = T(1, {100}), b = T(2, {100}), c = T(3, {100}), d = T(4, {100}), out = T(5, {50});
        for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
        const float two = 2.0f;
        for (auto* t : {&a, &b, &c, &d}) e.recordFill(&two, DataType::kFloat32, View(*t));
        e.flush(false);
        CHECK(e.waitingFills() == 4 && cap.singles.empty());
        e.recordExternalRead(a.data);
        CHECK(e.waitingFills() == 3 && e.pendingOps() == 1);
        CHECK(e.pendingWrites(b.data) && e.waitingFills() == 2 && e.pendingOps() == 2);
        OpRecord fill;
        CHECK(e.takeTrailingFill(View(c), &fill) && fill.type == OpType::Fill && e.waitingFills() == 1 && e.pendingOps() == 2);
        auto inside = T(4, {50});
        inside.data = reinterpret_cast<char*>(inside.data) + 200;   // elements [50, 100) of d by pointer
        e.record(OpType::Negate, View(inside), View(out));
        CHECK(e.waitingFills() == 0 && e.pendingOps() == 4);
        e.flush(false);
        CHECK(e.waitingFills() == 0);                               // a fill that has waited runs with the window it rejoined
        size_t fills = 0;
        for (const auto& op : cap.singles) fills += op.type == OpType::Fill;
        CHECK(fills == 3 && cap.singles.size() == 4);               // a, b, d and the negate (c's fill was handed over)
    }
    // switched off: every fill runs in its own window
    {
        Capture cap;
        FuseConfig c = config();
        c.deferIdleFills = false;
        FuseEngine e(c, cap.callbacks());
        auto a = T(1, {100});
        e.retainBuffer(a.data);
        const float one = 1.0f;
        e.recordFill(&one, DataType::kFloat32, View(a));
        e.flush(false);
        CHECK(e.waitingFills() == 0 && cap.singles.size() == 1);
    }
}

static void testLoneCastsAsKernelsAndTheManyBlocksForm()
{
    // the per-parameter casts of a mixed-precision step: each a one-operator kernel of one signature, so that the device
    // can send them off together; the many-blocks form of a flat kernel compiles
    Capture cap;
    FuseConfig c = config();
    c.loneCastsAsKernels = true;
    FuseEngine e(c, cap.callbacks());
    for (uintptr_t k = 0; k < 3; ++k) {
        auto src = T(1 + 2 * k, {100 + 28 * k}), dst = T(2 + 2 * k, {100 + 28 * k}, DataType::kBFloat16);
        e.retainBuffer(src.data); e.retainBuffer(dst.data);
        e.record(OpType::Cast, View(src), View(dst));
    }
    e.flush();
    CHECK(cap.fused.size() == 3 && cap.singles.empty());
    if (cap.fused.size() != 3) return;
    const std::string sig = gen::signature(cap.fused[0], gen::Shape::Flat, 0, true);
    CHECK(sig == gen::signature(cap.fused[1], gen::Shape::Flat, 0, true) && sig == gen::signature(cap.fused[2], gen::Shape::Flat, 0, true));
    CHECK(compiles(cap.fused[0], gen::Shape::Flat));
    const auto& d = cap.fused[0];
    const std::string src = gen::source(d, gen::Shape::Flat, 0, true, false, true);
    if (std::getenv("AIX_PRINT_MANY_SOURCE")) std::printf("%s\n", src.c_str());
    CHECK(src.find(gen::entryName(d, gen::Shape::Flat) + "_many(const Args* table, const u32* starts, u32 count)") != std::string::npos);
    hiprtcProgram prog;
    const char* names[] = {"aix_device.h"};
    const char* texts[] = {g_prelude.c_str()};
    CHECK(hiprtcCreateProgram(&prog, src.c_str(), "m.hip", 1, texts, names) == HIPRTC_SUCCESS);
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off"};
    const hiprtcResult r = hiprtcCompileProgram(prog, 4, opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0; hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, 0); if (n) hiprtcGetProgramLog(prog, &log[0]);
        std::printf("---- hipRTC log ----\n%s\n---- source ----\n%s\n", log.c_str(), src.c_str());
    }
    CHECK(r == HIPRTC_SUCCESS);
    hiprtcDestroyProgram(&prog);
    // the other launch shapes and a row program have the form too (one operator applied head by head)
    auto compilesText = [&](const std::string& text, const std::string& entry) {
        if (text.find(entry + "_many(const Args* table, const u32* starts, u32 count)") == std::string::npos) return false;
        hiprtcProgram p3;
        if (hiprtcCreateProgram(&p3, text.c_str(), "m3.hip", 1, texts, names) != HIPRTC_SUCCESS) return false;
        const hiprtcResult r3 = hiprtcCompileProgram(p3, 4, opts);
        if (r3 != HIPRTC_SUCCESS) {
            size_t n = 0; hiprtcGetProgramLogSize(p3, &n);
            std::string log(n, 0); if (n) hiprtcGetProgramLog(p3, &log[0]);
            std::printf("---- hipRTC log ----\n%s\n---- source ----\n%s\n", log.c_str(), text.c_str());
        }
        hiprtcDestroyProgram(&p3);
        return r3 == HIPRTC_SUCCESS;
    };
    CHECK(compilesText(gen::source(d, gen::Shape::Rows, 0, true, false, true), gen::entryName(d, gen::Shape::Rows)));
    CHECK(compilesText(gen::source(d, gen::Shape::Gather, 0, true, false, true), gen::entryName(d, gen::Shape::Gather)));
    {
        Capture rows;
        FuseEngine g(config(), rows.callbacks());
        recordSoftmax(g, DataType::kBFloat16, 8, 512);
        g.flush();
        CHECK(rows.fused.size() == 1);
        gen::RowGeometry geo;
        if (rows.fused.size() == 1 && gen::rowGeometry(rows.fused[0], &geo))
            CHECK(compilesText(gen::rowSource(rows.fused[0], geo, false, true), gen::rowEntryName(rows.fused[0], geo)));
        else CHECK(false);
    }
    // the chain of the benchmark in its many-blocks form
    Capture chain;
    FuseEngine f(config(), chain.callbacks());
    recordChain(f, 1.0f, 0.5f, true);
    f.flush();
    CHECK(chain.fused.size() == 1);
    if (chain.fused.size() == 1) {
        const std::string many = gen::source(chain.fused[0], gen::Shape::Flat, 0, true, false, true);
        hiprtcProgram p2;
        CHECK(hiprtcCreateProgram(&p2, many.c_str(), "m2.hip", 1, texts, names) == HIPRTC_SUCCESS);
        CHECK(hiprtcCompileProgram(p2, 4, opts) == HIPRTC_SUCCESS);
        hiprtcDestroyProgram(&p2);
    }
}

static void testRowProgramTakesInAPlainKernel()
{
    // max()'s backward inside a softmax gradient: m = rowmax(x) ... c = cast(mask: int32 -> f32), y = c * m (m broadcast
    // along the row).  The cast starts a kernel of its own (nothing defines or loads its operand); when the product needs
    // both the cast's value and the row program's per-row value, the two kernels become one: the mask is converted at
    // the row program's load, there is no pass that writes a converted copy.
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    const size_t rows = 16, L = 512;
    auto x = T(1, {rows, L}), m = T(2, {rows, 1}), mask = T(3, {rows, L}, DataType::kInt32), c = T(4, {rows, L}), y = T(5, {rows, L});
    auto mB = T(2, {rows, L}, DataType::kFloat32, {1, 0});
    for (uintptr_t id : {1, 2, 3, 4, 5}) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    uint8_t lowest[8] = {};
    lowestScalarInto(DataType::kFloat32, lowest);
    e.recordRowReduce(OpType::MaxTo, View(x), View(m), lowest, L);
    e.record(OpType::Cast, View(mask), View(c));
    e.record(OpType::Mul, View(c), View(mB), View(y));
    e.releaseBuffer(reinterpret_cast<void*>(uintptr_t(4) * 0x10000));
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() != 1) return;
    const auto& d = cap.fused[0];
    CHECK(d.rowLength == L && d.ops.size() == 3 && d.inputBuffers.size() == 2);
    bool sawMask = false;
    for (const auto& in : d.inputBuffers) if (in.dtype == DataType::kInt32) sawMask = true;
    CHECK(sawMask);
    CHECK(d.outputBuffers.size() == 2);                         // m and y; the converted mask is never stored
    CHECK(compilesRow(d));
    // attention's forward pass in one kernel: tril(s) * scale + mask, then the softmax of the rows -- the triangle's rows
    // are the program's rows, the [seq, seq] mask under [heads, seq, seq] scores is a block of rows that comes round again
    Capture cap2;
    FuseEngine f(config(), cap2.callbacks());
    const size_t heads = 3, seq = 64;
    auto sc = T(11, {heads, seq, seq}), t1 = T(12, {heads, seq, seq}), t2 = T(13, {heads, seq, seq}), t3 = T(14, {heads, seq, seq});
    auto half = T(15, {}), halfB = T(15, {heads, seq, seq}, DataType::kFloat32, {0, 0, 0});
    auto msk = T(16, {seq, seq}), mskB = T(16, {heads, seq, seq}, DataType::kFloat32, {0, seq, 1});
    auto mx = T(17, {heads, seq, 1}), mxB = T(17, {heads, seq, seq}, DataType::kFloat32, {seq, 1, 0}), out = T(18, {heads, seq, seq});
    for (uintptr_t id = 11; id <= 18; ++id) f.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    const float h = 0.5f;
    f.recordFill(&h, DataType::kFloat32, View(half));
    f.recordTri(OpType::Tril, View(sc), View(t1), 0);
    f.record(OpType::Mul, View(t1), View(halfB), View(t2));
    f.record(OpType::Add, View(t2), View(mskB), View(t3));
    f.recordRowReduce(OpType::MaxTo, View(t3), View(mx), lowest, seq);
    f.record(OpType::Sub, View(t3), View(mxB), View(out));
    for (uintptr_t id : {12, 13, 14, 15, 17}) f.releaseBuffer(reinterpret_cast<void*>(id * 0x10000));
    f.flush();
    CHECK(cap2.fused.size() == 1 && cap2.singles.empty());
    if (cap2.fused.size() == 1) {
        const auto& k = cap2.fused[0];
        CHECK(k.rowLength == seq && k.ops.size() == 5 && k.ops[0].type == OpType::Tril && k.inputBuffers.size() == 2 && k.outputBuffers.size() == 1);
        CHECK(k.opParams.size() == 3 && k.opParams[0] == seq && k.opParams[1] == seq);
        CHECK(rowOperandPeriod(k.inputBuffers[1], heads * seq, seq) == seq || rowOperandPeriod(k.inputBuffers[0], heads * seq, seq) == seq);
        CHECK(compilesRow(k));
        std::vector<uint64_t> args;
        const void* in[2] = {nullptr, nullptr}; void* o1[1] = {nullptr};
        gen::packRowArgsInto(args, k, in, o1);
        CHECK(args.size() == 2 + 1 + k.scalarData.size() / 4 + 2 + 3 + 2);             // in, out, the immediates, two periods, the triangle, rows, length
    }
    // a triangle of matrices whose rows are not the program's rows stays a kernel of its own
    Capture cap3;
    FuseEngine g(config(), cap3.callbacks());
    auto wide = T(21, {4, 8, 128}), wtri = T(22, {4, 8, 128}), wm = T(23, {4 * 8 * 2, 1}), wflat = T(22, {4 * 8 * 2, 64});
    for (uintptr_t id : {21, 22, 23}) g.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    g.recordTri(OpType::Triu, View(wide), View(wtri), 0);
    g.recordRowReduce(OpType::MaxTo, View(wflat), View(wm), lowest, 64);                 // rows of 64 over matrices of 128 columns
    g.flush();
    CHECK(cap3.fused.size() + cap3.singles.size() == 2);
}

static void testSumOfEverythingJoinsItsProducer()
{
    // the gradient of a scalar constant: p = g * x is formed only to be summed; the kernel goes on around the sum
    // (q = p + x here) and never stores p.  All three launch shapes compile; with no producer in the window the sum is a
    // single operator; a row program does not take it.
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    auto g = T(1, {64, 96}), x = T(2, {64, 96}), p = T(3, {64, 96}), s = T(4, {}), q = T(5, {64, 96}), s2 = T(6, {});
    for (uintptr_t id = 1; id <= 6; ++id) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    const float zero = 0.0f, seven = 7.0f;
    e.record(OpType::Mul, View(g), View(x), View(p));
    e.recordWholeSum(View(p), View(s), &zero);
    e.record(OpType::Add, View(p), View(x), View(q));
    e.recordWholeSum(View(q), View(s2), &seven);
    e.releaseBuffer(reinterpret_cast<void*>(uintptr_t(3) * 0x10000));
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() == 1) {
        const auto& d = cap.fused[0];
        CHECK(d.ops.size() == 4 && d.inputBuffers.size() == 2 && d.outputBuffers.size() == 3);        // s, q, s2: p stays in registers
        CHECK(d.ops[1].type == OpType::ReduceTo && d.ops[1].whole && d.ops[1].outputIndex != SIZE_MAX && d.ops[1].scalarIndex1 != SIZE_MAX);
        CHECK(d.ops[3].whole && d.outputBuffers[d.ops[3].outputIndex].data == s2.data);
        CHECK(d.rowLength == 0);
        CHECK(compiles(d, gen::Shape::Flat) && compiles(d, gen::Shape::Rows) && compiles(d, gen::Shape::Gather));
        const std::string src = gen::source(d, gen::Shape::Flat, 0, true);
        CHECK(src.find("acc" + std::to_string(d.ops[1].outputIndex) + " += up(") != std::string::npos && src.find("row_sum<256>") != std::string::npos);
        CHECK(gen::signature(d, gen::Shape::Flat, 0, true).find("ReduceTo!(") != std::string::npos);
    }
    // nothing in the window produces the operand: a single operator, as before
    Capture alone;
    FuseEngine f(config(), alone.callbacks());
    for (uintptr_t id : {1, 4}) f.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    f.recordWholeSum(View(g), View(s), &zero);
    f.flush();
    CHECK(alone.fused.empty() && alone.singles.size() == 1 && alone.singles[0].type == OpType::ReduceTo && alone.singles[0].whole);
    // a row program keeps its rows: the sum of everything closes it and runs as a single operator
    Capture rows;
    FuseEngine h(config(), rows.callbacks());
    for (uintptr_t id = 1; id <= 30; ++id) h.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    recordSoftmax(h, DataType::kFloat32, 16, 256, 20);
    auto y = T(26, {16, 256}), sy = T(27, {});
    h.recordWholeSum(View(y), View(sy), &zero);
    h.flush();
    CHECK(rows.fused.size() == 1 && rows.singles.size() == 1 && rows.fused[0].rowLength == 256);
    for (const auto& op : rows.fused[0].ops) CHECK(!op.whole);
}

static void testOnehotOfRowMaximaLivesInARowProgram()
{
    // max()'s backward inside a softmax gradient: mask = one-hot of the row maxima of x (int32), c = cast(mask) to the
    // seed's type, y = c * m with m a per-row value of the same program.  One row program; the int32 mask is dead after
    // the window and never stored.  Alone in its window the one-hot is a single operator; alive, it is stored as int32.
    Capture cap;
    FuseEngine e(config(), cap.callbacks());
    const size_t rows = 16, L = 512;
    auto g = T(1, {rows, L}, DataType::kBFloat16), m = T(2, {rows, 1}, DataType::kBFloat16), x = T(3, {rows, L}, DataType::kBFloat16);
    auto mask = T(4, {rows, L}, DataType::kInt32), c = T(5, {rows, L}, DataType::kBFloat16), y = T(6, {rows, L}, DataType::kBFloat16);
    auto mB = T(2, {rows, L}, DataType::kBFloat16, {1, 0});
    for (uintptr_t id = 1; id <= 6; ++id) e.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    uint8_t zero[8] = {};
    e.recordRowReduce(OpType::ReduceTo, View(g), View(m), zero, L);
    e.recordRowOnehot(View(x), View(mask), L);
    e.record(OpType::Cast, View(mask), View(c));
    e.record(OpType::Mul, View(c), View(mB), View(y));
    for (uintptr_t id : {4, 5}) e.releaseBuffer(reinterpret_cast<void*>(id * 0x10000));
    e.flush();
    CHECK(cap.fused.size() == 1 && cap.singles.empty());
    if (cap.fused.size() == 1) {
        const auto& d = cap.fused[0];
        CHECK(d.rowLength == L && d.ops.size() == 4 && d.inputBuffers.size() == 2 && d.outputBuffers.size() == 2);      // g, x -> m, y
        CHECK(d.ops[1].type == OpType::ArgmaxIndicesTo && d.ops[1].outputIndex == SIZE_MAX && d.ops[2].type == OpType::Cast && d.ops[2].inputIndex0 == 2 + 1);
        for (const auto& out : d.outputBuffers) CHECK(out.dtype == DataType::kBFloat16);
        CHECK(compilesRow(d));
    }
    // the mask alive after the window: stored by the program, converted to int32
    Capture kept;
    FuseEngine f(config(), kept.callbacks());
    for (uintptr_t id = 1; id <= 6; ++id) f.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    f.recordRowOnehot(View(x), View(mask), L);
    f.record(OpType::Cast, View(mask), View(c));
    f.record(OpType::Mul, View(c), View(g), View(y));
    f.flush();
    CHECK(kept.fused.size() == 1);
    if (kept.fused.size() == 1) {
        bool storesMask = false;
        for (const auto& out : kept.fused[0].outputBuffers) if (out.data == mask.data && out.dtype == DataType::kInt32) storesMask = true;
        CHECK(storesMask && kept.fused[0].rowLength == L);
        CHECK(compilesRow(kept.fused[0]));
    }
    // alone: the plain operator; read by anything but a cast to the program's type: from memory
    Capture alone;
    FuseEngine h(config(), alone.callbacks());
    for (uintptr_t id = 1; id <= 8; ++id) h.retainBuffer(reinterpret_cast<void*>(id * 0x10000));
    h.recordRowOnehot(View(x), View(mask), L);
    h.flush();
    CHECK(alone.fused.empty() && alone.singles.size() == 1 && alone.singles[0].type == OpType::ArgmaxIndicesTo);
    auto asF32 = T(7, {rows, L}, DataType::kFloat32);
    h.recordRowOnehot(View(x), View(mask), L);
    h.record(OpType::Cast, View(mask), View(asF32));            // to f32, not the program's bf16
    h.flush();
    CHECK(alone.singles.size() >= 2);
    bool maskWritten = false;
    for (const auto& s1 : alone.singles) if (s1.type == OpType::ArgmaxIndicesTo) maskWritten = true;
    CHECK(maskWritten);
}

static void testEqualKernelsLeaveSideBySide()
{
    // head after head: b = a * t (t a transposed view: no operand of a row program, so the product is a kernel of its
    // own), then y = b - max(b) row by row, then c = -y * t.  The planner closes a kernel when the next one reads its
    // result, so in its list the products alternate with the row programs; with groupEqualKernels the four products
    // leave side by side, and a kernel that depends on another never overtakes it, also through a buffer written twice.
    struct Step { std::vector<const void*> reads, writes; };
    auto run = [&](bool group) {
        Capture cap;
        FuseConfig c = config();
        c.groupEqualKernels = group;
        FuseEngine e(c, cap.callbacks());
        uint8_t lowest[8] = {};
        lowestScalarInto(DataType::kFloat32, lowest);
        auto P = [](uintptr_t id) { return reinterpret_cast<void*>(id * 0x10000); };
        for (uintptr_t k = 0; k < 4; ++k) {
            const uintptr_t id = 10 * (k + 1);
            auto a = T(id + 1, {8, 256}), b = T(id + 3, {8, 256}), m = T(id + 4, {8, 1}), y = T(id + 5, {8, 256});
            auto u = T(id + 6, {8, 256}), c2 = T(id + 7, {8, 256});
            auto t = T(id + 2, {8, 256}, DataType::kFloat32, {1, 8});
            auto mB = T(id + 4, {8, 256}, DataType::kFloat32, {1, 0});
            for (uintptr_t j = 1; j <= 7; ++j) e.retainBuffer(P(id + j));
            e.record(OpType::Mul, View(a), View(t), View(b));
            e.recordRowReduce(OpType::MaxTo, View(b), View(m), lowest, 256);
            e.record(OpType::Sub, View(b), View(mB), View(y));
            e.releaseBuffer(P(id + 4));
            e.record(OpType::Negate, View(y), View(u));
            e.record(OpType::Mul, View(u), View(t), View(c2));
            e.releaseBuffer(P(id + 6));
        }
        // one buffer written by two kernels in turn: z = p * q is read by a row reduction, then z = r * s
        auto p0 = T(81, {8, 256}), r0 = T(83, {8, 256}), z = T(90, {8, 256}), mz = T(91, {8, 1});
        auto q0 = T(82, {8, 256}, DataType::kFloat32, {1, 8}), s0 = T(84, {8, 256}, DataType::kFloat32, {1, 8});
        for (uintptr_t id : {81, 82, 83, 84, 90, 91}) e.retainBuffer(P(id));
        e.record(OpType::Mul, View(p0), View(q0), View(z));
        e.recordRowReduce(OpType::MaxTo, View(z), View(mz), lowest, 256);
        e.record(OpType::Mul, View(r0), View(s0), View(z));
        e.flush();
        if (std::getenv("AIX_TEST_VERBOSE")) for (auto& o : cap.order) std::printf("  %s %s\n", group ? "grouped" : "plain  ", o.c_str());
        // what left, in the order it left: reads and writes of every kernel and single operator
        std::vector<Step> steps;
        size_t single = 0;
        for (const auto& o : cap.order) {
            Step st;
            if (o[0] == 'F') {
                const auto& d = cap.fused[std::stoul(o.substr(1))];
                for (const auto& in : d.inputBuffers) st.reads.push_back(in.data);
                for (const auto& out : d.outputBuffers) st.writes.push_back(out.data);
            } else {
                const auto& op = cap.singles[single++];
                st.reads.push_back(op.input0.data);
                if (op.hasInput1) st.reads.push_back(op.input1.data);
                st.writes.push_back(op.output.data);
            }
            steps.push_back(st);
        }
        return steps;
    };
    const auto plain = run(false), grouped = run(true);
    CHECK(plain.size() == grouped.size() && plain.size() >= 11);
    auto buf = [](uintptr_t id) { return reinterpret_cast<const void*>(id * 0x10000); };
    auto has = [](const std::vector<const void*>& v, const void* p) { return std::find(v.begin(), v.end(), p) != v.end(); };
    auto writer = [&](const std::vector<Step>& s, const void* p, size_t nth) { for (size_t k = 0; k < s.size(); ++k) if (has(s[k].writes, p) && nth-- == 0) return k; return (size_t)SIZE_MAX; };
    auto reader = [&](const std::vector<Step>& s, const void* p) { for (size_t k = 0; k < s.size(); ++k) if (has(s[k].reads, p)) return k; return (size_t)SIZE_MAX; };
    // the same work either way: every buffer is written equally often
    for (uintptr_t id : {13, 15, 17, 23, 25, 27, 33, 35, 37, 43, 45, 47, 90, 91}) {
        size_t n1 = 0, n2 = 0;
        for (const auto& st : plain) n1 += has(st.writes, buf(id));
        for (const auto& st : grouped) n2 += has(st.writes, buf(id));
        CHECK(n1 == n2 && n1 >= 1);
    }
    // plain: something between the products of two heads; grouped: the four products are consecutive
    CHECK(writer(plain, buf(23), 0) > writer(plain, buf(13), 0) + 1);
    size_t first = SIZE_MAX, last = 0;
    for (uintptr_t k = 1; k <= 4; ++k) { const size_t w = writer(grouped, buf(10 * k + 3), 0); first = std::min(first, w); last = std::max(last, w); }
    CHECK(first != SIZE_MAX && last - first == 3);
    // in both orders: a product before the kernel that reads it, y before its reader, the two writers of z around its reader
    for (const auto* s : {&plain, &grouped}) {
        for (uintptr_t k = 1; k <= 4; ++k) {
            CHECK(writer(*s, buf(10 * k + 3), 0) < reader(*s, buf(10 * k + 3)));
            CHECK(writer(*s, buf(10 * k + 7), 0) != SIZE_MAX);
        }
        const size_t w1 = writer(*s, buf(90), 0), rd = reader(*s, buf(90)), w2 = writer(*s, buf(90), 1);
        CHECK(w1 < rd && rd < w2 && w2 != SIZE_MAX);
        CHECK(has((*s)[w1].reads, buf(81)) && has((*s)[w2].reads, buf(83)));
    }
}

int main(int argc, char** argv)
{
    if (argc < 2) { std::printf("usage: test_planner <path to aix_device.h>\n"); return 2; }
    std::ifstream f(argv[1]);
    std::stringstream ss; ss << f.rdbuf();
    g_prelude = ss.str();
    if (g_prelude.empty()) { std::printf("cannot read %s\n", argv[1]); return 2; }

    testChainBecomesOneDenseKernel();
    testOperandOrderDoesNotSplitTheKernel();
    testLiveTemporariesAreStoredAndFillsRun();
    testFusionDisabledReplaysInOrder();
    testInPlaceUpdatesKeepProgramOrder();
    testDifferentViewOfAProducedBufferSplitsKernels();
    testWriteAfterReadClosesTheReader();
    testRowBroadcastStaysInOneKernel();
    testDeadCodeIsDropped();
    testThresholdFlushAndExternalRead();
    testFillMinAndIntegerScalars();
    testEveryTypeAndOperatorCompiles();
    testPointerSetGrowsAndForgets();
    testViewLimitsAndRoundTrip();
    testEngineStorageIsReusedAcrossWindows();
    testTrailingFillIsHandedOver();
    testCastsFuseAtTheirLoadOrStoreEnd();
    testDenseSidesAdoptTheStridedSidesShape();
    testTrilJoinsItsNeighbours();
    testSoftmaxBecomesOneRowProgram();
    testLayerNormPiecesShareOneRowProgram();
    testIdleFillsWaitForTheirFirstUser();
    testLoneCastsAsKernelsAndTheManyBlocksForm();
    testRowProgramTakesInAPlainKernel();
    testSumOfEverythingJoinsItsProducer();
    testOnehotOfRowMaximaLivesInARowProgram();
    testEqualKernelsLeaveSideBySide();
    std::printf(g_failed ? "%d checks FAILED\n" : "all planner checks passed\n", g_failed);
    return g_failed ? 1 : 0;
}
