// fuse.hpp -- the lazy elementwise planner behind DeviceHIP.
//
// Same role and the same public surface as the reference's device-agnostic fusion engine
// (Targets/AIXLib/aixFuse.hpp:29-217): a device records elementwise operators and fills instead of
// running them; flush() turns the recorded window into fused multi-output kernels plus ordered
// single operators and hands them to the device through callbacks.  The planning algorithm itself
// is different (see fuse.cpp): a single pass in program order that grows several open groups at
// once under explicit read/write hazard rules, treats every fill as a lazily materialised scalar,
// and classifies contiguity over the buffers that are really loaded or stored -- so an expression
// such as  tanh(a*b + c) / (1 + exp(-a)) - 0.5*c  becomes ONE dense kernel with three 16-byte
// loads, one 16-byte store and two immediates per lane group.
#pragma once

#include "aix_compat.hpp"

#include <algorithm>
#include <array>
#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <unordered_map>
#include <vector>

namespace aixhip::fuse {

using aix::DataType;
using aix::DeviceTensorParams;

// Operator codes; the elementwise ones are the recordable set (aixFuse.hpp:29-88).
enum class OpType {
    Add, Sub, Mul, Div, Negate, Sqrt, Sin, Cos, Tanh, Log, Exp, Pow, Fill, FillMin, Cast,
    Sum, Max, Argmax, ArgmaxIndices, Matmul, Transpose, Copy, Contiguous, ReduceTo, MaxTo,
    ArgmaxTo, ArgmaxIndicesTo, SliceSet, Tril, Triu, IndexSelect, IndexAdd,
};

bool isElementwiseOp(OpType t);
// ReduceTo / MaxTo recorded as row reductions (FuseEngine::recordRowReduce): sum / maximum over the last, dense dimension
inline bool isRowReduce(OpType t) { return t == OpType::ReduceTo || t == OpType::MaxTo; }
const char* opName(OpType t);

struct FuseConfig {
    bool   elementwiseFusion     = true;
    bool   multiOutputKernels    = true;   // let independent ops that share an input join one kernel
    bool   absorbFills           = true;   // fills feed consumers as immediates and run only if needed
    bool   diagnostics           = false;
    size_t flushThreshold        = 200;    // recorded ops that trigger planning
    size_t maxBufferSlots        = 0;      // pointer arguments one fused kernel may take (must be > 0)
    bool   supportsStridedFusion = true;   // may fused kernels read broadcast / strided views
    bool   loneCastsAsKernels    = false;  // a cast with no company is emitted as a one-operator kernel (emitFused), not as a single
    bool   deferIdleFills        = true;   // a fill nothing else in its window touches waits for its first user (see flush())
    bool   groupEqualKernels     = false;  // kernels leave level by level and kind by kind instead of in the planner's order (see flush())
};

// An operand as the planner keeps it: the fields of aix::DeviceTensorParams with the extents and
// strides held in place, so that recording an operator allocates nothing.  `dense` says that the
// view walks its elements in memory order without gaps (extent-1 dimensions may carry any stride).
constexpr size_t kMaxRank = 16;

struct View {
    void*    data{nullptr};
    DataType dtype{DataType::kFloat32};
    bool     dense{true};
    uint32_t rank{0};
    size_t   offset{0};
    size_t   size{0};
    size_t   shape[kMaxRank];              // [0, rank) are meaningful
    size_t   strides[kMaxRank];

    View() {}
    View(const DeviceTensorParams& p);     // std::invalid_argument beyond kMaxRank dimensions
    View(const View& o) { assign(o); }
    View& operator=(const View& o) { if (this != &o) assign(o); return *this; }

    bool sameShape(const View& o) const { return rank == o.rank && std::memcmp(shape, o.shape, rank * sizeof(size_t)) == 0; }
    bool sameShape(const aix::Shape& s) const;
    void makeDense();                      // offset 0 and the dense strides of `shape`
    aix::Shape shapeVector() const { return aix::Shape(shape, shape + rank); }
    DeviceTensorParams params() const;

private:
    void assign(const View& o)
    {
        data = o.data; dtype = o.dtype; dense = o.dense; rank = o.rank; offset = o.offset; size = o.size;
        std::memcpy(shape, o.shape, rank * sizeof(size_t));
        std::memcpy(strides, o.strides, rank * sizeof(size_t));
    }
};

struct OpRecord {
    OpType type{OpType::Add};
    View input0;
    View input1;
    View output;
    std::array<uint8_t, 8> scalarData{};   // Fill: the scalar in scalarDType
    DataType scalarDType = DataType::kFloat32;
    bool hasInput1 = false;
    // Tril / Triu recorded as elementwise operators: the extents of the last two dims and the diagonal
    uint64_t triRows{0}, triCols{0};
    int64_t triDiagonal{0};
    // ReduceTo / MaxTo recorded as a row reduction: elements per row of input0 (its last dimension); scalarData then holds
    // the value the destination was initialised with, in the destination's element type (the folded fill)
    size_t rowLength{0};
    // ReduceTo recorded as the sum of ALL elements of input0 into a one-element output (rowLength 0); scalarData as above
    bool whole{false};
    // Fill / FillMin: the fill has waited outside the window and was brought back because somebody names its buffer: it
    // runs with the window it is in now
    bool hasWaited{false};
};

// How a view takes part in a kernel that works row by row on [rows, length] data (a "row program"): element for element,
// one value per row repeated along the row, a dense block of one or more whole rows that every so many rows see again
// (one row for all rows: gamma of a LayerNorm; the [seq, seq] mask under [batch, heads, seq, seq] scores), one value per
// row (operand of a per-row operator), one element seen from everywhere (a scalar tensor, broadcast), or not at all.
enum class RowOperand { Dense, PerRowBroadcast, RowVector, PerRow, Single, None };
RowOperand rowOperandKind(const View& v, size_t rows, size_t length);
// RowVector operands: how many rows the block holds that every row sees as (row % period); 0 for the other kinds.
size_t rowOperandPeriod(const View& v, size_t rows, size_t length);

// One fused kernel: ops in execution order.  An operand index below inputBuffers.size() names an
// external buffer, an index at or above it names the result of ops[index - inputBuffers.size()];
// SIZE_MAX means "not a tensor" (then the scalar index applies).  scalarData holds the immediates
// already converted to `dtype`.
struct FusedSubgraphDescriptor {
    struct Op {
        OpType type;
        size_t inputIndex0  = SIZE_MAX;
        size_t inputIndex1  = SIZE_MAX;
        size_t outputIndex  = SIZE_MAX;    // into outputBuffers; SIZE_MAX = value stays in registers
        size_t scalarIndex0 = SIZE_MAX;
        size_t scalarIndex1 = SIZE_MAX;
        size_t paramIndex   = SIZE_MAX;    // Tril / Triu: its (rows, cols, diagonal) triple in opParams
        bool   perRow       = false;       // row programs: the operator yields one value per row (a reduction, or arithmetic on such values)
        bool   whole        = false;       // ReduceTo: the sum of the operand over ALL elements of the kernel (plus the immediate scalarIndex1) into
                                           // the one-element output; the kernel hands over one partial sum per workgroup, its caller adds them up
    };
    std::vector<Op> ops;
    std::vector<uint64_t> opParams;        // run-time integers of index-dependent operators, three per Tril / Triu
    std::vector<View> inputBuffers;
    std::vector<View> outputBuffers;
    std::vector<uint8_t> scalarData;
    DataType dtype{DataType::kFloat32};
    bool     allContiguous{true};          // every loaded / stored view is dense
    size_t   elementCount{0};
    aix::Shape shape;                      // iteration shape (outputs are dense over it)
    // Row program: the kernel handles rows of `rowLength` elements (elementCount / rowLength of them) and may hold
    // ReduceTo / MaxTo operators -- sum / maximum over a row, combined with the immediate scalarIndex1 the destination was
    // initialised with -- whose per-row results later operators of the same kernel use.  0: a plain elementwise kernel.
    size_t   rowLength{0};
};
// The descriptor handed to emitFused is reused from kernel to kernel: a callback that wants to keep
// it copies it.

struct FlushDiagnostics {
    size_t opsRecorded = 0;
    size_t fusibleSubgraphs = 0;
    size_t fusedOps = 0;
    size_t fallbackOps = 0;
    size_t dispatchesSaved = 0;
    size_t fillsAbsorbed = 0;
    size_t kernelCacheHits = 0;
    size_t kernelCacheMisses = 0;
    std::string subgraphSummary;
    std::string fallbackSummary;
};

struct FuseCallbacks {
    std::function<void(const FusedSubgraphDescriptor&)> emitFused;
    std::function<void(const OpRecord&)> emitSingle;
    std::function<void()> finishFlush;
    std::function<std::pair<size_t, size_t>()> getKernelCacheStats = [] { return std::pair<size_t, size_t>{0, 0}; };
    // The start of the allocation an operand pointer lies in (operands may point into the middle of a block); an
    // engine without it takes every pointer for a block of its own.
    std::function<const void*(const void*)> blockBase;
};

// Converts a scalar between element types with the device's conversion rules (saturating
// float -> integer, NaN -> 0, 16-bit floats by way of float; aixDeviceCPU.cpp:96-117).
std::vector<uint8_t> convertScalar(const void* scalar, DataType from, DataType to);
std::vector<uint8_t> lowestScalar(DataType dtype);
// The same without the vector: writes at most 8 bytes to `out` and returns how many.
size_t convertScalarInto(const void* scalar, DataType from, DataType to, uint8_t* out);
size_t lowestScalarInto(DataType dtype, uint8_t* out);

// A set of buffer addresses that neither allocates per insertion nor chases pointers on lookup
// (open addressing; allocate() / deallocate() of every temporary pass through it).
class PointerSet {
public:
    bool contains(const void* p) const;
    void insert(const void* p);
    void erase(const void* p);
    void clear() { if (m_used) { std::fill(m_slots.begin(), m_slots.end(), (uintptr_t)0); m_count = m_used = 0; } }
    size_t size() const { return m_count; }

private:
    size_t slotOf(uintptr_t key) const { return (size_t)(((key >> 6) * 0x9E3779B97F4A7C15ull) >> m_shift); }
    void grow();
    std::vector<uintptr_t> m_slots;        // 0 = never used, 1 = erased
    size_t m_count{0}, m_used{0};
    unsigned m_shift{64};
};

class Planner;

class FuseEngine {
public:
    FuseEngine(const FuseConfig& config, FuseCallbacks callbacks);
    ~FuseEngine();

    void record(OpType type, const View& input0, const View& output);
    void record(OpType type, const View& input0, const View& input1, const View& output);
    void recordFill(const void* scalar, DataType scalarDType, const View& output);
    void recordFillMin(const View& output);
    // tril / triu of `input` (its last two dims) as an elementwise operator: the kept part passes through, the rest is 0
    void recordTri(OpType type, const View& input, const View& output, int64_t diagonal);
    // ReduceTo / MaxTo over the last dimension (`rowLength` elements, dense) of `input` into the dense `output`, whose
    // pending initialisation the caller has taken out of the window: `init` is that value in output's element type.
    void recordRowReduce(OpType type, const View& input, const View& output, const void* init, size_t rowLength);
    // The sum of all elements of the dense `input` into the one-element `output`, whose pending initialisation the caller
    // has taken out of the window (`init`, in output's element type).  It joins the kernel that holds its operand in
    // registers -- the product that is only formed to be summed is then never stored -- and is replayed as a plain
    // reduction when there is no such kernel.
    void recordWholeSum(const View& input, const View& output, const void* init);
    // argmaxIndicesTo along the last, dense dimension (`rowLength` elements) of `input` into the dense int32 `output` of
    // the same shape, whose zero fill the caller has taken out of the window: 1 at the first maximum of every row, 0
    // elsewhere.  Inside a row program the ones and zeros are values of the program's type that a cast to that type
    // takes as they are (max()'s backward multiplies the seed with them: the int32 tensor need never exist).
    void recordRowOnehot(const View& input, const View& output, size_t rowLength);
    // Plans and emits the window.  A fill (fill / fillMin of a whole dense buffer that allocate() handed out) that no
    // other operator of the window touches, and that nobody outside is about to read, is not emitted unless `final`:
    // it waits, outside the window, until an operator naming its buffer is recorded (it then rejoins the window ahead
    // of that operator and is usually absorbed as an immediate), until the buffer is read outside the planner
    // (recordExternalRead, takeTrailingFill, pendingWrites / pendingTouches), or until a final flush; a buffer released
    // in between takes its fill along.  zeroGrad() followed, a whole forward and backward pass later, by the first
    // accumulation into the gradient is the case this is for (aixCore.hpp zeroGrad, accumulateGrad).
    void flush(bool final = true);
    size_t waitingFills() const { return m_waiting.size(); }

    const FuseConfig& config() const { return m_config; }
    const FlushDiagnostics& lastFlushDiagnostics() const;
    size_t pendingOps() const { return m_pending.size(); }

    // If the newest pending operator touching output.data is a fill / fillMin of exactly this dense
    // tensor, remove it from the window and hand it over (the caller folds it into the operator
    // it is about to run eagerly); false and no change otherwise.
    bool takeTrailingFill(const View& output, OpRecord* fill);
    bool pendingWrites(const void* buffer);        // a recorded operator of the window writes the buffer
    bool pendingTouches(const void* buffer);       // ... reads or writes it
    void recordExternalRead(const void* buffer);   // the buffer is about to be read outside the planner
    void retainBuffer(void* buffer);               // allocate(): results written here must reach memory
    void releaseBuffer(void* buffer);              // deallocate(): nobody will read it after the window
    void invalidateBuffer(void* buffer);

private:
    void maybeFlush();
    void wake(const void* operand);                // the waiting fills of the operand's buffer rejoin the window
    void setAsideIdleFills();

    FuseConfig m_config;
    FuseCallbacks m_callbacks;
    OpRecord& append(OpType type);
    std::vector<OpRecord> m_pending;       // capacity is kept from window to window
    std::vector<OpRecord> m_window;
    // pendingWrites() / pendingTouches(): per buffer, how many of m_pending[0, m_counted) write / read it
    std::unordered_map<const void*, std::pair<uint32_t, uint32_t>> m_pendingUse;
    size_t m_counted{0};
    void countPending();
    PointerSet m_live;
    std::vector<const void*> m_externalReads;
    std::vector<OpRecord> m_waiting;       // fills set aside by flush(false), oldest first
    PointerSet m_waitingBuffers;
    std::unique_ptr<Planner> m_planner;    // its working storage is kept from window to window
    FusedSubgraphDescriptor m_descriptor;
    // flush(): the order kernels leave in (level, kind, place in the planner's list) and, per buffer, one more than the
    // highest level of a kernel that wrote / read it so far
    struct Order { uint32_t level; uint64_t kind; size_t at; };
    std::vector<Order> m_order;
    std::unordered_map<const void*, std::pair<uint32_t, uint32_t>> m_touched;
    std::optional<FlushDiagnostics> m_diagnostics;
    bool m_flushing{false};
};

} // namespace aixhip::fuse
