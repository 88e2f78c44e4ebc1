// fuse.cpp -- planning a window of recorded elementwise operators into fused kernels.
//
// One pass over the window in program order.  State while walking:
//
//   * open GROUPS: each will become one kernel.  A group knows the views it loads from memory and
//     the views it defines (value kept in registers, perhaps also stored).  Invariant: no open
//     group reads from memory what another open group writes, so open groups can be emitted in
//     any order relative to each other; a group is CLOSED (appended to the emit list) the moment
//     a later operator would break that.
//   * pending FILLS: a fill is not run when recorded.  Readers inside the window take its value as
//     an immediate; the fill kernel itself runs only if something needs the buffer in memory (an
//     operator that cannot take the immediate, or the buffer still being alive at the end).
//
// An operator joins the group that defines one of its operands (same view => same element, the
// value is already in a register), or an open group that loads one of the same views (shared
// read), else it opens a new group.  Joining is refused -- the offending group is closed first --
// whenever the same storage would be seen through two different views inside one kernel.
//
// Which results are stored is decided last, when every reader is known: a result reaches memory
// only if its buffer is still alive after the window, or if a later operator loads it.
//
// Behavioural parity with the reference planner (Targets/AIXLib/aixFuse.cpp) is at the level its
// tests pin: same callbacks, program-order semantics, fills absorbed into immediates, dead
// temporaries never stored, scalar VALUES not part of a kernel's identity.

#include "fuse.hpp"

#include "scalar_convert.hpp"

#include <algorithm>
#include <array>
#include <cassert>
#include <cstring>
#include <limits>
#include <sstream>
#include <stdexcept>

namespace aixhip::fuse {

bool isElementwiseOp(OpType t)
{
    switch (t) {
        case OpType::Add: case OpType::Sub: case OpType::Mul: case OpType::Div: case OpType::Negate:
        case OpType::Sqrt: case OpType::Sin: case OpType::Cos: case OpType::Tanh: case OpType::Log:
        case OpType::Exp: case OpType::Pow: case OpType::Fill: case OpType::FillMin: case OpType::Cast:
        case OpType::Tril: case OpType::Triu:                 // when recorded (FuseEngine::recordTri)
            return true;
        default:
            return false;
    }
}

const char* opName(OpType t)
{
    static const char* names[] = {"Add", "Sub", "Mul", "Div", "Negate", "Sqrt", "Sin", "Cos", "Tanh", "Log", "Exp", "Pow",
                                  "Fill", "FillMin", "Cast", "Sum", "Max", "Argmax", "ArgmaxIndices", "Matmul", "Transpose",
                                  "Copy", "Contiguous", "ReduceTo", "MaxTo", "ArgmaxTo", "ArgmaxIndicesTo", "SliceSet",
                                  "Tril", "Triu", "IndexSelect", "IndexAdd"};
    return names[static_cast<size_t>(t)];
}

size_t convertScalarInto(const void* scalar, DataType from, DataType to, uint8_t* out)
{
    const auto v = scalar::decode(scalar, static_cast<int>(from));
    return scalar::encode(v, static_cast<int>(to), out);
}

size_t lowestScalarInto(DataType dtype, uint8_t* out)
{
    auto put = [&](auto v) { std::memcpy(out, &v, sizeof(v)); return sizeof(v); };
    switch (dtype) {
        case DataType::kFloat64:  return put(std::numeric_limits<double>::lowest());
        case DataType::kFloat32:  return put(std::numeric_limits<float>::lowest());
        case DataType::kFloat16:  return put((uint16_t)0xFBFF);          // aixFloat16.hpp:173-178
        case DataType::kBFloat16: return put((uint16_t)0xFF7F);          // aixFloat16.hpp:767-772
        case DataType::kInt64:    return put(std::numeric_limits<int64_t>::lowest());
        case DataType::kInt32:    return put(std::numeric_limits<int32_t>::lowest());
        case DataType::kInt16:    return put(std::numeric_limits<int16_t>::lowest());
        case DataType::kInt8:     return put(std::numeric_limits<int8_t>::lowest());
        case DataType::kUInt8:    return put((uint8_t)0);
    }
    return 0;
}

std::vector<uint8_t> convertScalar(const void* scalar, DataType from, DataType to)
{
    uint8_t bytes[8] = {};
    const size_t n = convertScalarInto(scalar, from, to, bytes);
    return std::vector<uint8_t>(bytes, bytes + n);
}

std::vector<uint8_t> lowestScalar(DataType dtype)
{
    uint8_t bytes[8] = {};
    const size_t n = lowestScalarInto(dtype, bytes);
    return std::vector<uint8_t>(bytes, bytes + n);
}

// ---- View --------------------------------------------------------------------------------------
namespace {

bool denseLayout(const size_t* shape, const size_t* strides, size_t rank)
{
    size_t run = 1;
    for (size_t d = rank; d-- > 0;) {
        if (shape[d] != 1 && strides[d] != run) return false;
        run *= shape[d];
    }
    return true;
}

} // namespace

View::View(const DeviceTensorParams& p)
    : data(p.data), dtype(p.dtype), rank((uint32_t)p.shape.size()), offset(p.offset), size(p.size)
{
    if (p.shape.size() > kMaxRank) throw std::invalid_argument("aixhip: tensors of more than 16 dimensions are not supported.");
    for (size_t d = 0; d < rank; ++d) { shape[d] = p.shape[d]; strides[d] = d < p.strides.size() ? p.strides[d] : 0; }
    dense = denseLayout(shape, strides, rank);
}

bool View::sameShape(const aix::Shape& s) const
{
    if (s.size() != rank) return false;
    for (size_t d = 0; d < rank; ++d) if (s[d] != shape[d]) return false;
    return true;
}

void View::makeDense()
{
    offset = 0;
    size_t run = 1;
    for (size_t d = rank; d-- > 0;) { strides[d] = run; run *= shape[d]; }
    dense = true;
}

DeviceTensorParams View::params() const
{
    DeviceTensorParams p;
    p.data = data; p.dtype = dtype; p.isContiguous = dense; p.offset = offset; p.size = size;
    p.shape.assign(shape, shape + rank);
    p.strides.assign(strides, strides + rank);
    return p;
}

// ---- PointerSet --------------------------------------------------------------------------------
bool PointerSet::contains(const void* p) const
{
    if (m_slots.empty()) return false;
    const uintptr_t key = (uintptr_t)p;
    const size_t mask = m_slots.size() - 1;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i] == key) return true;
        if (m_slots[i] == 0) return false;
    }
}

void PointerSet::grow()
{
    std::vector<uintptr_t> old;
    old.swap(m_slots);
    size_t capacity = 64;
    while (capacity < m_count * 4) capacity <<= 1;
    m_slots.assign(capacity, 0);
    m_shift = 64;
    for (size_t c = capacity; c > 1; c >>= 1) --m_shift;
    m_used = m_count;
    const size_t mask = capacity - 1;
    for (uintptr_t key : old) {
        if (key <= 1) continue;
        size_t i = slotOf(key);
        while (m_slots[i] != 0) i = (i + 1) & mask;
        m_slots[i] = key;
    }
}

void PointerSet::insert(const void* p)
{
    const uintptr_t key = (uintptr_t)p;
    if (key <= 1) return;
    if ((m_used + 1) * 2 > m_slots.size()) grow();
    const size_t mask = m_slots.size() - 1;
    size_t grave = SIZE_MAX;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i] == key) return;
        if (m_slots[i] == 1 && grave == SIZE_MAX) grave = i;
        if (m_slots[i] == 0) {
            if (grave != SIZE_MAX) m_slots[grave] = key;
            else { m_slots[i] = key; ++m_used; }
            ++m_count;
            return;
        }
    }
}

void PointerSet::erase(const void* p)
{
    if (m_slots.empty()) return;
    const uintptr_t key = (uintptr_t)p;
    if (key <= 1) return;
    const size_t mask = m_slots.size() - 1;
    for (size_t i = slotOf(key);; i = (i + 1) & mask) {
        if (m_slots[i] == key) { m_slots[i] = 1; --m_count; return; }
        if (m_slots[i] == 0) return;
    }
}

// The trailing run of dimensions of `v` that make up one row of `length` elements, or -1: rows are the last dimensions
// whose extents multiply to `length`.
static int rowSplit(const View& v, size_t length)
{
    size_t run = 1;
    int d = (int)v.rank;
    while (d > 0 && run < length) { --d; run *= v.shape[d]; }
    return run == length ? d : -1;
}

RowOperand rowOperandKind(const View& v, size_t rows, size_t length)
{
    if (!v.data || rows == 0 || length == 0) return RowOperand::None;
    const size_t vec = 16 / aix::Device::dataTypeSize(v.dtype);
    bool still = v.size > 1;                                                   // one element seen everywhere: a scalar tensor, broadcast
    for (uint32_t d = 0; d < v.rank; ++d) if (v.shape[d] > 1 && v.strides[d] != 0) still = false;
    if (v.size == rows * length) {
        if (v.dense) return v.offset % vec == 0 ? RowOperand::Dense : RowOperand::None;
        const int split = rowSplit(v, length);
        if (split < 0) return RowOperand::None;
        // strides of the row dims and of the leading dims: all zero, or those of a dense tensor
        auto zeros = [&](int from, int to) { for (int d = from; d < to; ++d) if (v.shape[d] > 1 && v.strides[d] != 0) return false; return true; };
        auto dense = [&](int from, int to) { size_t run = 1; for (int d = to - 1; d >= from; --d) { if (v.shape[d] > 1 && v.strides[d] != run) return false; run *= v.shape[d]; } return true; };
        if (zeros(split, (int)v.rank) && dense(0, split)) return RowOperand::PerRowBroadcast;            // one value per row, repeated along it
        if (still) return RowOperand::Single;
        // a dense block of whole rows that comes round again and again: one row for all rows, or the [seq, seq] mask of
        // attention under [batch, heads, seq, seq] scores (the dims in front of the block have stride 0)
        int from = (int)v.rank;
        { size_t run = 1; while (from > 0 && (v.shape[from - 1] == 1 || v.strides[from - 1] == run)) { --from; run *= v.shape[from]; } }
        if (from > split) return RowOperand::None;
        while (from < split && !zeros(0, from)) ++from;            // (extent-1 dims may sit on either side)
        if (zeros(0, from) && dense(from, (int)v.rank)) return v.offset % vec == 0 ? RowOperand::RowVector : RowOperand::None;
        return RowOperand::None;
    }
    if (v.size == rows && v.dense) return RowOperand::PerRow;
    if (v.size == rows && still) return RowOperand::Single;
    return RowOperand::None;
}

size_t rowOperandPeriod(const View& v, size_t rows, size_t length)
{
    if (rowOperandKind(v, rows, length) != RowOperand::RowVector) return 0;
    // the dims with a stride: everything behind the zero-stride dims in front
    size_t block = 1;
    int d = 0;
    while (d < (int)v.rank && (v.shape[d] == 1 || v.strides[d] == 0)) ++d;
    for (; d < (int)v.rank; ++d) block *= v.shape[d];
    return block / length ? block / length : 1;
}

namespace {

bool isTriOp(OpType t) { return t == OpType::Tril || t == OpType::Triu; }

bool sameView(const View& a, const View& b)
{
    return a.data == b.data && a.dtype == b.dtype && a.offset == b.offset && a.rank == b.rank &&
           std::memcmp(a.shape, b.shape, a.rank * sizeof(size_t)) == 0 &&
           std::memcmp(a.strides, b.strides, a.rank * sizeof(size_t)) == 0;
}

bool isDense(const View& p) { return p.dense; }

// The same elements in the same flat order: identical views, or two dense views of one buffer that
// start at the same element and have the same count (a [rows, cols] result read back as [rows * cols]).
bool sameElements(const View& a, const View& b)
{
    if (sameView(a, b)) return true;
    return a.dense && b.dense && a.data == b.data && a.dtype == b.dtype && a.offset == b.offset && a.size == b.size;
}

// One past the last element position the view touches.
size_t viewEnd(const View& p)
{
    size_t last = p.offset;
    for (size_t d = 0; d < p.rank; ++d) {
        if (p.shape[d] == 0) return p.offset;
        last += (p.shape[d] - 1) * p.strides[d];
    }
    return last + 1;
}

struct Operand {
    enum Kind { kNone, kMemory, kValue, kScalar } kind{kNone};
    size_t index{SIZE_MAX};          // kValue: defining op (window index); kScalar: fill op (window index)
};

// A view inside the window: operand `slot` (0, 1 = inputs, 2 = output) of operator `op`.
struct ViewRef {
    uint32_t op;
    uint32_t slot;
};

struct Group {
    DataType dtype{DataType::kFloat32};
    size_t count{0};
    const View* shape{nullptr};                                // the view whose shape is the iteration space
    bool dense{true};                                          // every loaded view so far is dense
    std::vector<size_t> ops;                                   // window indices, program order
    std::vector<size_t> defs;                                  // per defined view: the latest operator defining it
    std::vector<ViewRef> loads;                                // distinct views loaded from memory
    bool open{true};
    bool absorbed{false};                                      // merged into another group
    bool hasScalar{false};
    size_t rowLen{0};                                          // > 0: a row program over rows of this many elements (it holds a row reduction)
    bool hasTri{false};                                        // holds a tril / triu (their flat index arithmetic is not available row by row)

    size_t rows() const { return rowLen ? count / rowLen : 0; }

    void reset()
    {
        dtype = DataType::kFloat32; count = 0; shape = nullptr; dense = true;
        ops.clear(); defs.clear(); loads.clear();
        open = true; absorbed = false; hasScalar = false; rowLen = 0; hasTri = false;
    }
};

struct Emit {
    bool fused{false};
    size_t index{0};                 // group index or window index
};

struct PendingFill {
    const void* buffer;
    size_t op;                       // window index
    size_t size;                     // elements filled from the base pointer
};

} // namespace

class Planner {
public:
    // A buffer outlives the window if somebody still holds it or if it is about to be read outside the planner.
    struct Liveness {
        const PointerSet* held{nullptr};
        const std::vector<const void*>* external{nullptr};
        bool count(const void* p) const
        {
            if (held->contains(p)) return true;
            for (const void* e : *external) if (e == p) return true;
            return false;
        }
    };

    explicit Planner(const FuseConfig& cfg) : m_cfg(cfg) {}

    void run(const std::vector<OpRecord>& ops, Liveness live)
    {
        m_ops = &ops;
        m_live = live;
        m_operands.assign(ops.size(), {});
        m_perRow.assign(ops.size(), 0);
        m_groupOf.assign(ops.size(), SIZE_MAX);
        m_groupCount = 0;
        m_touchIndex.clear();
        m_touchUsed = 0;
        m_emits.clear();
        m_fills.clear();
        m_fillsAbsorbed = 0;

        for (size_t i = 0; i < ops.size(); ++i) {
            const auto& op = ops[i];
            if (op.type == OpType::Fill || op.type == OpType::FillMin) placeFill(i);
            else if (isElementwiseOp(op.type) && m_cfg.elementwiseFusion) placeOp(i);
            else if (isRowReduce(op.type) && op.rowLength && m_cfg.elementwiseFusion && m_cfg.supportsStridedFusion) placeReduce(i);
            else if (op.whole && m_cfg.elementwiseFusion) placeWhole(i);
            else if (op.type == OpType::ArgmaxIndicesTo && op.rowLength && m_cfg.elementwiseFusion && m_cfg.supportsStridedFusion) placeOnehot(i);
            else placeSingle(i);
        }
        for (size_t g = 0; g < m_groupCount; ++g) closeGroup(g);
        // fills nobody could absorb completely: run them if the buffer outlives the window
        m_rest.clear();
        for (const auto& pf : m_fills) if (m_live.count(pf.buffer)) m_rest.push_back(pf.op);
        std::sort(m_rest.begin(), m_rest.end());
        for (size_t op : m_rest) m_emits.push_back({false, op});
        m_fills.clear();
        decideStores();
    }

    const std::vector<Emit>& emits() const { return m_emits; }
    const Group& group(size_t g) const { return m_groups[g]; }
    size_t fillsAbsorbed() const { return m_fillsAbsorbed; }

    // A group of one operator without immediates runs as a plain single operator.
    bool emitsAsSingle(const Group& g) const { return g.ops.size() == 1 && (!g.hasScalar || isRowReduce(at(g.ops[0]).type)); }

    void describe(const Group& g, FusedSubgraphDescriptor& d)
    {
        const auto& ops = *m_ops;
        d.ops.clear(); d.inputBuffers.clear(); d.outputBuffers.clear(); d.scalarData.clear(); d.opParams.clear();
        d.dtype = g.dtype;
        d.elementCount = g.count;
        d.shape.assign(g.shape->shape, g.shape->shape + g.shape->rank);
        d.allContiguous = true;
        d.rowLength = g.rowLen;
        m_position.resize(ops.size());                        // window index -> position in d.ops (this group's ops only)
        m_scalarSlots.clear();                                // fill op -> scalar index
        auto inputSlot = [&](const View& v) {
            for (size_t k = 0; k < d.inputBuffers.size(); ++k) if (sameView(d.inputBuffers[k], v)) return k;
            d.inputBuffers.push_back(v);
            if (!isDense(v)) d.allContiguous = false;
            return d.inputBuffers.size() - 1;
        };
        // external inputs first, so that value indices (inputs.size() + position) are stable
        for (size_t w : g.ops) {
            const auto& op = ops[w];
            if (m_operands[w][0].kind == Operand::kMemory) inputSlot(op.input0);
            if (m_operands[w][1].kind == Operand::kMemory) inputSlot(op.input1);
        }
        const size_t nIn = d.inputBuffers.size();
        const size_t esz = aix::Device::dataTypeSize(g.dtype);
        auto scalarIndex = [&](size_t fillOp) {
            for (const auto& known : m_scalarSlots) if (known.first == fillOp) return known.second;
            const auto& f = ops[fillOp];
            uint8_t bytes[8] = {};
            const size_t n = f.type == OpType::FillMin ? lowestScalarInto(g.dtype, bytes)
                                                       : convertScalarInto(f.scalarData.data(), f.scalarDType, g.dtype, bytes);
            const size_t slot = d.scalarData.size() / esz;
            d.scalarData.insert(d.scalarData.end(), bytes, bytes + n);
            m_scalarSlots.emplace_back(fillOp, slot);
            return slot;
        };
        for (size_t w : g.ops) {
            const auto& op = ops[w];
            FusedSubgraphDescriptor::Op o;
            o.type = op.type;
            const View* in[2] = {&op.input0, &op.input1};
            size_t* idx[2] = {&o.inputIndex0, &o.inputIndex1};
            size_t* sc[2] = {&o.scalarIndex0, &o.scalarIndex1};
            for (int k = 0; k < 2; ++k) {
                const auto& operand = m_operands[w][k];
                if (operand.kind == Operand::kMemory) *idx[k] = inputSlot(*in[k]);
                else if (operand.kind == Operand::kValue) {
                    if (m_groupOf[operand.index] != m_groupOf[w] || operand.index >= w)
                        throw std::logic_error("fusion planner: a register operand is not defined earlier in the same kernel");
                    *idx[k] = nIn + m_position[operand.index];
                }
                else if (operand.kind == Operand::kScalar) *sc[k] = scalarIndex(operand.index);
            }
            o.perRow = m_perRow[w] != 0;
            o.whole = op.whole;
            if (isRowReduce(op.type)) {
                // the value the destination was initialised with (already in the group's element type) as an immediate
                o.scalarIndex1 = d.scalarData.size() / esz;
                d.scalarData.insert(d.scalarData.end(), op.scalarData.data(), op.scalarData.data() + esz);
            }
            if (op.type == OpType::Tril || op.type == OpType::Triu) {
                o.paramIndex = d.opParams.size() / 3;
                d.opParams.push_back(op.triRows); d.opParams.push_back(op.triCols); d.opParams.push_back((uint64_t)op.triDiagonal);
            }
            if (m_store[w]) {
                o.outputIndex = d.outputBuffers.size();
                d.outputBuffers.push_back(op.output);
                if (!isDense(op.output)) d.allContiguous = false;
            }
            m_position[w] = d.ops.size();
            d.ops.push_back(o);
        }
    }

private:
    const OpRecord& at(size_t i) const { return (*m_ops)[i]; }
    const View& view(ViewRef r) const
    {
        const auto& op = at(r.op);
        return r.slot == 0 ? op.input0 : r.slot == 1 ? op.input1 : op.output;
    }
    const View& defView(size_t definingOp) const { return at(definingOp).output; }

    PendingFill* findFill(const void* buffer)
    {
        for (auto& pf : m_fills) if (pf.buffer == buffer) return &pf;
        return nullptr;
    }
    void eraseFill(const void* buffer)
    {
        for (size_t k = 0; k < m_fills.size(); ++k)
            if (m_fills[k].buffer == buffer) { m_fills[k] = m_fills.back(); m_fills.pop_back(); return; }
    }

    // ---- which open groups touch a buffer --------------------------------------------------------------
    // Every question an operator asks of the open groups starts from one of its buffers (who defines it, who loads it,
    // who has to close before it is overwritten), so the groups are kept per buffer: a window with hundreds of open
    // kernels -- the same short formula applied to tensor after tensor -- costs an operator no more than a small one.
    std::vector<uint32_t>& touchList(const void* buffer)
    {
        auto it = m_touchIndex.find(buffer);
        if (it != m_touchIndex.end()) return m_touchLists[it->second];
        if (m_touchUsed == m_touchLists.size()) m_touchLists.emplace_back();
        m_touchLists[m_touchUsed].clear();
        m_touchIndex.emplace(buffer, (uint32_t)m_touchUsed);
        return m_touchLists[m_touchUsed++];
    }
    void addTouch(size_t g, const void* buffer)
    {
        if (!buffer) return;
        auto& list = touchList(buffer);
        for (uint32_t known : list) if (known == g) return;
        list.insert(std::upper_bound(list.begin(), list.end(), (uint32_t)g), (uint32_t)g);     // ascending, as the groups were made
    }
    void dropTouches(size_t g)
    {
        auto drop = [&](const void* buffer) {
            auto it = m_touchIndex.find(buffer);
            if (it == m_touchIndex.end()) return;
            auto& list = m_touchLists[it->second];
            for (size_t k = 0; k < list.size(); ++k) if (list[k] == g) { list.erase(list.begin() + (long)k); break; }
        };
        for (const ViewRef& r : m_groups[g].loads) drop(view(r).data);
        for (size_t def : m_groups[g].defs) drop(defView(def).data);
    }
    // The open groups that touch `buffer` (and `other`, if given), ascending, copied into `out` so that the caller may
    // close and merge groups while it walks them.
    void touching(const void* buffer, const void* other, std::vector<uint32_t>& out)
    {
        out.clear();
        for (const void* p : {buffer, other}) {
            if (!p) continue;
            auto it = m_touchIndex.find(p);
            if (it == m_touchIndex.end()) continue;
            const auto& list = m_touchLists[it->second];
            if (out.empty()) out.assign(list.begin(), list.end());
            else { for (uint32_t g : list) if (std::find(out.begin(), out.end(), g) == out.end()) out.push_back(g); std::sort(out.begin(), out.end()); }
        }
    }

    size_t newGroup()
    {
        if (m_groupCount == m_groups.size()) m_groups.emplace_back();
        m_groups[m_groupCount].reset();
        return m_groupCount++;
    }

    // ---- fills --------------------------------------------------------------------------------
    void placeFill(size_t i)
    {
        const auto& out = at(i).output;
        if (!m_cfg.absorbFills || !m_cfg.elementwiseFusion) { placeSingle(i); return; }
        // groups that see the buffer's previous content must run before anything overwrites it
        closeGroupsTouching(out.data, SIZE_MAX, nullptr);
        PendingFill* known = findFill(out.data);
        if (known && known->size > out.size) { materialise(out.data); known = nullptr; }   // older, larger fill survives underneath
        if (known) { known->op = i; known->size = out.size; }
        else m_fills.push_back(PendingFill{out.data, i, out.size});                        // written flat from the base pointer
    }

    void materialise(const void* buffer)
    {
        const PendingFill* pf = findFill(buffer);
        if (!pf) return;
        m_emits.push_back({false, pf->op});
        eraseFill(buffer);
    }

    // ---- operators that cannot be fused ----------------------------------------------------------
    void placeSingle(size_t i)
    {
        const auto& op = at(i);
        for (const View* in : {&op.input0, &op.input1}) {
            if (!in->data) continue;
            materialise(in->data);
            closeWriters(in->data);
        }
        if (op.output.data) {
            closeGroupsTouching(op.output.data, SIZE_MAX, nullptr);
            if (op.type == OpType::Fill || op.type == OpType::FillMin) eraseFill(op.output.data);
            else materialise(op.output.data);
        }
        if (op.input0.data) m_operands[i][0].kind = Operand::kMemory;
        if (op.hasInput1 && op.input1.data) m_operands[i][1].kind = Operand::kMemory;
        m_emits.push_back({false, i});
    }

    // ---- fusable operators ---------------------------------------------------------------------
    void placeOp(size_t i)
    {
        const auto& op = at(i);
        const bool binary = op.hasInput1;
        const View* in[2] = {&op.input0, binary ? &op.input1 : nullptr};
        // A cast changes the element type between its operand and its result.  Kernels compute in ONE
        // type and convert at their loads and stores, so a cast is fused at one of its two ends: it
        // joins the kernel that holds its operand in a register as a last step (the value is stored
        // converted; nothing in that kernel may use it further), or it starts / joins a kernel of
        // its result type whose load of the operand converts.
        const bool isCast = op.type == OpType::Cast;

        if (!m_cfg.supportsStridedFusion) {
            const bool dense = isDense(op.output) && (!in[0]->data || isDense(*in[0])) && (!in[1] || !in[1]->data || isDense(*in[1]));
            if (!dense) { placeSingle(i); return; }
        }

        // Resolve operands until nothing more has to be closed (closing a group turns its values
        // into memory loads, which can in turn change the picture).
        size_t target = SIZE_MAX;
        Operand resolved[2];
        for (;;) {                                   // every 'continue' below has closed a group
            bool closedSomething = false;
            target = SIZE_MAX;
            for (int k = 0; k < 2; ++k) {
                resolved[k] = Operand{};
                if (!in[k] || !in[k]->data) continue;
                // an unmaterialised fill covering everything the view can touch -> immediate
                // (not for a cast: the immediate would skip the rounding to the fill's own type)
                if (const PendingFill* f = findFill(in[k]->data)) {
                    if (!isCast && in[k]->dtype == at(f->op).output.dtype && viewEnd(*in[k]) <= f->size) {
                        resolved[k] = Operand{Operand::kScalar, f->op};
                        continue;
                    }
                    materialise(in[k]->data);
                }
                resolved[k].kind = Operand::kMemory;
                touching(in[k]->data, nullptr, m_candA);
                for (size_t gi = 0; gi < m_candA.size(); ++gi) {
                    const size_t g = m_candA[gi];
                    if (!m_groups[g].open) continue;
                    const size_t def = findDef(m_groups[g], in[k]->data);
                    if (def == SIZE_MAX) continue;
                    // (the ones and zeros of a row program's one-hot operator are values of the program's type: only a cast to
                    // that type may take them, and takes them as they are)
                    const bool usable = at(def).type == OpType::ArgmaxIndicesTo
                                            ? isCast && op.output.dtype == m_groups[g].dtype && op.output.size == m_groups[g].count && sameElements(defView(def), *in[k]) &&
                                                  rowOperandKind(op.output, m_groups[g].rows(), m_groups[g].rowLen) == RowOperand::Dense
                                            : valueUsable(m_groups[g], def, *in[k], op) && compatible(m_groups[g], op, in[k]->dtype);
                    if (usable && (target == SIZE_MAX || target == g)) {
                        resolved[k] = Operand{Operand::kValue, def};
                        target = g;
                    } else if (usable && mergeable(m_groups[target], m_groups[g])) {
                        // both operands come from open groups: open groups are independent of each
                        // other, so the two become one kernel
                        resolved[k] = Operand{Operand::kValue, def};
                        mergeInto(target, g);
                    } else {
                        closeGroup(g);
                        closedSomething = true;
                    }
                }
            }
            if (closedSomething) continue;

            // no producer inside the window: share loads with an open group of the same shape
            if (target == SIZE_MAX && m_cfg.multiOutputKernels) {
                touching(resolved[0].kind == Operand::kMemory && in[0] ? in[0]->data : nullptr, resolved[1].kind == Operand::kMemory && in[1] ? in[1]->data : nullptr, m_candA);
                for (size_t gi = 0; gi < m_candA.size() && target == SIZE_MAX; ++gi) {
                    const size_t g = m_candA[gi];
                    if (!m_groups[g].open || !compatible(m_groups[g], op, op.output.dtype)) continue;
                    for (int k = 0; k < 2; ++k)
                        if (resolved[k].kind == Operand::kMemory && loads(m_groups[g], *in[k])) target = g;
                }
            }

            // hazards on the output buffer
            if (closeGroupsTouching(op.output.data, target, &op.output)) continue;
            if (target != SIZE_MAX && slotsAfterJoin(m_groups[target], op, resolved) > m_cfg.maxBufferSlots) {
                closeGroup(target);
                continue;
            }
            // a row program takes its memory operands row by row: whole rows, one value per row, or one row for all
            if (target != SIZE_MAX && m_groups[target].rowLen && !rowOperandsFit(m_groups[target], op, resolved)) {
                closeGroup(target);
                continue;
            }
            break;
        }

        // a fill that this operator overwrites completely never has to run
        if (const PendingFill* f = findFill(op.output.data)) {
            if (isDense(op.output) && op.output.offset == 0 && op.output.size >= f->size) eraseFill(op.output.data);
            else materialise(op.output.data);
        }

        if (target == SIZE_MAX) {
            target = newGroup();
            Group& fresh = m_groups[target];
            fresh.dtype = op.output.dtype;
            fresh.count = op.output.size;
            fresh.shape = &op.output;
        }
        Group& g = m_groups[target];
        adoptShape(g, op);
        for (int k = 0; k < 2; ++k) {
            m_operands[i][k] = resolved[k];
            if (resolved[k].kind == Operand::kMemory) {
                if (!loads(g, *in[k])) g.loads.push_back(ViewRef{(uint32_t)i, (uint32_t)k});
                addTouch(target, in[k]->data);
                if (!isDense(*in[k])) g.dense = false;
            } else if (resolved[k].kind == Operand::kScalar) {
                g.hasScalar = true;
                ++m_fillsAbsorbed;
            }
        }
        bool redefined = false;
        for (auto& def : g.defs) if (sameView(defView(def), op.output)) { def = i; redefined = true; }
        if (!redefined) g.defs.push_back(i);
        addTouch(target, op.output.data);
        g.ops.push_back(i);
        m_groupOf[i] = target;
        if (op.type == OpType::Tril || op.type == OpType::Triu) g.hasTri = true;
        m_perRow[i] = g.rowLen && op.output.size == g.rows() && op.output.size != g.count;
    }

    // ---- row reductions ------------------------------------------------------------------------------
    // sum / maximum over the rows of a dense [rows, length] operand.  It joins the open kernel that holds the operand in
    // registers, or one that loads it, if that kernel can work row by row (rowsFit); later operators of the kernel may
    // use the per-row result -- repeated along the row, or in arithmetic on per-row values -- without a pass over memory
    // in between: max -> sub -> exp -> sum -> div of a softmax is one kernel, one read of the operand.
    void placeReduce(size_t i)
    {
        const auto& op = at(i);
        const View& in = op.input0;
        const size_t L = op.rowLength;
        size_t target = SIZE_MAX;
        Operand resolved{};
        for (;;) {
            bool closedSomething = false;
            target = SIZE_MAX;
            resolved = Operand{};
            if (findFill(in.data)) materialise(in.data);
            resolved.kind = Operand::kMemory;
            touching(in.data, nullptr, m_candA);
            for (size_t gi = 0; gi < m_candA.size(); ++gi) {
                const size_t g = m_candA[gi];
                if (!m_groups[g].open) continue;
                const size_t def = findDef(m_groups[g], in.data);
                if (def == SIZE_MAX) continue;
                const Group& grp = m_groups[g];
                const bool usable = target == SIZE_MAX && !m_perRow[def] && sameElements(defView(def), in) &&     // (a cast at a kernel's load included: the group has the cast's result type)
                                    grp.dtype == in.dtype && grp.count == in.size && rowsFit(grp, L);
                if (usable) { resolved = Operand{Operand::kValue, def}; target = g; }
                else { closeGroup(g); closedSomething = true; }
            }
            if (closedSomething) continue;
            if (target == SIZE_MAX && m_cfg.multiOutputKernels) {
                touching(in.data, nullptr, m_candA);
                for (size_t gi = 0; gi < m_candA.size() && target == SIZE_MAX; ++gi) {
                    const size_t g = m_candA[gi];
                    const Group& grp = m_groups[g];
                    if (grp.open && grp.dtype == in.dtype && grp.count == in.size && rowsFit(grp, L) && loads(grp, in)) target = g;
                }
            }
            if (closeGroupsTouching(op.output.data, target, &op.output)) continue;
            if (target != SIZE_MAX) {
                const Group& grp = m_groups[target];
                size_t slots = grp.loads.size() + grp.defs.size() + 1;
                if (resolved.kind == Operand::kMemory && !loads(grp, in)) ++slots;
                if (slots > m_cfg.maxBufferSlots) { closeGroup(target); continue; }
            }
            break;
        }
        if (findFill(op.output.data)) eraseFill(op.output.data);     // the reduction defines every element of its destination
        if (target == SIZE_MAX) {
            target = newGroup();
            Group& fresh = m_groups[target];
            fresh.dtype = in.dtype;
            fresh.count = in.size;
            fresh.shape = &op.input0;
        }
        Group& g = m_groups[target];
        g.rowLen = L;
        m_operands[i][0] = resolved;
        if (resolved.kind == Operand::kMemory && !loads(g, in)) g.loads.push_back(ViewRef{(uint32_t)i, 0});
        if (resolved.kind == Operand::kMemory) addTouch(target, in.data);
        g.defs.push_back(i);
        addTouch(target, op.output.data);
        g.ops.push_back(i);
        m_groupOf[i] = target;
        m_perRow[i] = 1;
    }

    // ---- the place of every row's first maximum, as ones and zeros ------------------------------------
    // Joins the row program that holds its operand in registers or loads it, else starts one.
    void placeOnehot(size_t i)
    {
        const auto& op = at(i);
        const View& in = op.input0;
        const size_t L = op.rowLength;
        size_t target = SIZE_MAX;
        Operand resolved{};
        for (;;) {
            bool closedSomething = false;
            target = SIZE_MAX;
            resolved = Operand{};
            if (findFill(in.data)) materialise(in.data);
            resolved.kind = Operand::kMemory;
            touching(in.data, nullptr, m_candA);
            for (size_t gi = 0; gi < m_candA.size(); ++gi) {
                const size_t g = m_candA[gi];
                if (!m_groups[g].open) continue;
                const size_t def = findDef(m_groups[g], in.data);
                if (def == SIZE_MAX) continue;
                const Group& grp = m_groups[g];
                const bool usable = target == SIZE_MAX && !m_perRow[def] && !at(def).whole && at(def).type != OpType::ArgmaxIndicesTo && sameElements(defView(def), in) &&
                                    grp.dtype == in.dtype && grp.count == in.size && rowsFit(grp, L);
                if (usable) { resolved = Operand{Operand::kValue, def}; target = g; }
                else { closeGroup(g); closedSomething = true; }
            }
            if (closedSomething) continue;
            if (target == SIZE_MAX && m_cfg.multiOutputKernels) {
                touching(in.data, nullptr, m_candA);
                for (size_t gi = 0; gi < m_candA.size() && target == SIZE_MAX; ++gi) {
                    const size_t g = m_candA[gi];
                    const Group& grp = m_groups[g];
                    if (grp.open && grp.dtype == in.dtype && grp.count == in.size && rowsFit(grp, L) && loads(grp, in)) target = g;
                }
            }
            if (closeGroupsTouching(op.output.data, target, &op.output)) continue;
            if (target != SIZE_MAX) {
                const Group& grp = m_groups[target];
                size_t slots = grp.loads.size() + grp.defs.size() + 1;
                if (resolved.kind == Operand::kMemory && !loads(grp, in)) ++slots;
                if (slots > m_cfg.maxBufferSlots) { closeGroup(target); continue; }
            }
            break;
        }
        if (findFill(op.output.data)) eraseFill(op.output.data);     // every element of the destination is defined
        if (target == SIZE_MAX) {
            target = newGroup();
            Group& fresh = m_groups[target];
            fresh.dtype = in.dtype;
            fresh.count = in.size;
            fresh.shape = &op.input0;
        }
        Group& g = m_groups[target];
        g.rowLen = L;
        m_operands[i][0] = resolved;
        if (resolved.kind == Operand::kMemory && !loads(g, in)) g.loads.push_back(ViewRef{(uint32_t)i, 0});
        if (resolved.kind == Operand::kMemory) addTouch(target, in.data);
        g.defs.push_back(i);
        addTouch(target, op.output.data);
        g.ops.push_back(i);
        m_groupOf[i] = target;
    }

    // ---- the sum of everything ------------------------------------------------------------------
    // Joins the plain kernel that holds its operand in registers (every element once, whatever the launch shape), else
    // it is a single operator.  Nothing in the kernel can use its result, and no row program takes it (its one-element
    // destination is no row operand), so the kernel goes on growing around it.
    void placeWhole(size_t i)
    {
        const auto& op = at(i);
        const View& in = op.input0;
        for (;;) {
            size_t target = SIZE_MAX, def = SIZE_MAX;
            bool closedSomething = false;
            if (findFill(in.data)) { placeSingle(i); return; }
            touching(in.data, nullptr, m_candA);
            for (size_t gi = 0; gi < m_candA.size(); ++gi) {
                const size_t g = m_candA[gi];
                if (!m_groups[g].open) continue;
                const size_t d = findDef(m_groups[g], in.data);
                if (d == SIZE_MAX) continue;
                const Group& grp = m_groups[g];
                size_t wholes = 0;
                for (size_t w : grp.ops) wholes += at(w).whole;
                const bool usable = target == SIZE_MAX && !grp.rowLen && !m_perRow[d] && !at(d).whole && sameElements(defView(d), in) &&
                                    grp.dtype == in.dtype && grp.count == in.size && wholes < 8 &&
                                    grp.loads.size() + grp.defs.size() + 2 <= m_cfg.maxBufferSlots;
                if (usable) { target = g; def = d; }
                else { closeGroup(g); closedSomething = true; }
            }
            if (closedSomething) continue;
            if (target == SIZE_MAX) { placeSingle(i); return; }
            if (closeGroupsTouching(op.output.data, SIZE_MAX, nullptr)) continue;      // (may have closed the target: look again)
            if (findFill(op.output.data)) eraseFill(op.output.data);                   // the sum defines its destination
            Group& g = m_groups[target];
            m_operands[i][0] = Operand{Operand::kValue, def};
            g.defs.push_back(i);
            addTouch(target, op.output.data);
            g.ops.push_back(i);
            g.hasScalar = true;                                                        // (the destination's initial value)
            m_groupOf[i] = target;
            return;
        }
    }

    // Can the group work on rows of `length` elements?  It does already, or everything it loads and stores fits rows.
    bool rowsFit(const Group& g, size_t length) const
    {
        if (g.rowLen) return g.rowLen == length;
        if (length == 0 || g.count % length != 0) return false;
        if (g.hasTri) for (size_t op : g.ops) if (isTriOp(at(op).type) && at(op).triCols != length) return false;
        const size_t rows = g.count / length;
        for (const ViewRef& r : g.loads) {
            const RowOperand k = rowOperandKind(view(r), rows, length);
            if (k != RowOperand::Dense && k != RowOperand::PerRowBroadcast && k != RowOperand::RowVector && k != RowOperand::Single) return false;
        }
        for (size_t def : g.defs) if (rowOperandKind(defView(def), rows, length) != RowOperand::Dense) return false;
        return true;
    }

    // The memory operands and the result of `op` as a member of row program `g`.
    bool rowOperandsFit(const Group& g, const OpRecord& op, const Operand* resolved) const
    {
        const size_t rows = g.rows();
        const bool per = op.output.size == rows && op.output.size != g.count;
        if (isTriOp(op.type) && (per || op.triCols != g.rowLen)) return false;        // a matrix row must be a row of the program
        if (rowOperandKind(op.output, rows, g.rowLen) != (per ? RowOperand::PerRow : RowOperand::Dense)) return false;
        const View* in[2] = {&op.input0, op.hasInput1 ? &op.input1 : nullptr};
        for (int k = 0; k < 2; ++k) {
            if (!in[k] || !in[k]->data || resolved[k].kind != Operand::kMemory) continue;
            const RowOperand kind = rowOperandKind(*in[k], rows, g.rowLen);
            if (kind == RowOperand::Single) continue;
            if (per ? kind != RowOperand::PerRow : (kind != RowOperand::Dense && kind != RowOperand::PerRowBroadcast && kind != RowOperand::RowVector)) return false;
        }
        return true;
    }

    // May `op` take the value that operator `def` of group `g` defines, seeing it through view `v`?
    bool valueUsable(const Group& g, size_t def, const View& v, const OpRecord& op) const
    {
        if (!m_perRow[def]) return sameElements(defView(def), v);
        // a per-row value: to an operator on per-row values it is the same elements; to an operator on whole rows it is the
        // destination seen with the row dimension(s) broadcast
        if (op.output.size == g.rows() && op.output.size != g.count) return sameElements(defView(def), v);
        const View& d = defView(def);
        return op.output.size == g.count && v.data == d.data && v.dtype == d.dtype && v.offset == d.offset &&
               rowOperandKind(v, g.rows(), g.rowLen) == RowOperand::PerRowBroadcast;
    }

    // The latest operator of the group that defines a view of `buffer`, SIZE_MAX if none does.
    size_t findDef(const Group& g, const void* buffer) const
    {
        for (size_t def : g.defs) if (defView(def).data == buffer) return def;
        return SIZE_MAX;
    }

    bool loads(const Group& g, const View& v) const
    {
        for (const ViewRef& r : g.loads) if (sameView(view(r), v)) return true;
        return false;
    }

    // `type` is the element type the operator would compute in inside the group: its result type, or for
    // a cast that takes a register value the operand's type.
    // Strided views are bound to the shape they were made for; dense views (and every result) only need
    // the element count, since the flat index is all that matters for them.  So with different shapes the
    // two can still share a kernel if one side is all dense: a dense operator rides on the group's shape,
    // a dense group adopts the shape of an operator that brings strided views (see adoptShape()).
    static bool denseOperands(const OpRecord& op)
    {
        return isDense(op.output) && (!op.input0.data || isDense(op.input0)) && (!op.hasInput1 || !op.input1.data || isDense(op.input1));
    }

    bool compatible(const Group& g, const OpRecord& op, DataType type) const
    {
        if (g.rowLen) {
            // a row program takes operators on whole rows and operators on per-row values; what their memory operands
            // look like is checked once the operands are resolved (rowOperandsFit)
            if (g.dtype != type) return false;
            if (isTriOp(op.type)) return op.output.size == g.count && op.triCols == g.rowLen;
            return op.output.size == g.count || op.output.size == g.rows();
        }
        if (g.dtype != type || g.count != op.output.size) return false;
        if (g.shape->sameShape(op.output)) return true;
        return g.dense || denseOperands(op);
    }

    static void adoptShape(Group& g, const OpRecord& op)
    {
        if (!g.shape->sameShape(op.output) && !denseOperands(op)) g.shape = &op.output;      // g.dense held, or compatible() had refused
    }

    bool mergeable(const Group& a, const Group& b) const
    {
        if (a.rowLen || b.rowLen) {
            // a row program takes in a kernel of plain elementwise operators (or another program over rows of the same
            // length) if everything that one loads and stores fits the rows: the conversion of a mask that a row
            // program multiplies with then happens at the program's load instead of in a pass of its own
            const size_t length = a.rowLen ? a.rowLen : b.rowLen;
            if (a.dtype != b.dtype || a.count != b.count || !rowsFit(a, length) || !rowsFit(b, length)) return false;
            size_t slots = a.loads.size();
            for (const ViewRef& r : b.loads) if (!loads(a, view(r))) ++slots;
            return slots + a.defs.size() + b.defs.size() + 1 <= m_cfg.maxBufferSlots;
        }
        if (a.dtype != b.dtype || a.count != b.count) return false;
        if (!a.shape->sameShape(*b.shape) && !a.dense && !b.dense) return false;
        size_t count = a.loads.size();
        for (const ViewRef& r : b.loads) if (!loads(a, view(r))) ++count;
        return count + a.defs.size() + b.defs.size() + 1 <= m_cfg.maxBufferSlots;
    }

    // Folds open group `from` into open group `into` (no hazards can exist between open groups).
    void mergeInto(size_t into, size_t from)
    {
        Group& a = m_groups[into];
        Group& b = m_groups[from];
        m_merged.resize(a.ops.size() + b.ops.size());
        std::merge(a.ops.begin(), a.ops.end(), b.ops.begin(), b.ops.end(), m_merged.begin());     // program order
        a.ops.assign(m_merged.begin(), m_merged.end());
        dropTouches(from);
        for (size_t def : b.defs) { a.defs.push_back(def); addTouch(into, defView(def).data); }
        for (const ViewRef& r : b.loads) { if (!loads(a, view(r))) a.loads.push_back(r); addTouch(into, view(r).data); }
        if (!a.shape->sameShape(*b.shape) && !b.dense) a.shape = b.shape;        // a is all dense then: it adopts the shape b's strided views need
        a.dense = a.dense && b.dense;
        a.hasScalar = a.hasScalar || b.hasScalar;
        a.hasTri = a.hasTri || b.hasTri;
        if (!a.rowLen) a.rowLen = b.rowLen;
        for (size_t w : b.ops) m_groupOf[w] = into;
        b.ops.clear(); b.defs.clear(); b.loads.clear();
        b.open = false;                                     // absorbed: never emitted on its own
        b.absorbed = true;
    }

    size_t slotsAfterJoin(const Group& g, const OpRecord& op, const Operand* resolved) const
    {
        size_t slots = g.loads.size() + g.defs.size() + 1;     // every def may have to be stored
        const View* in[2] = {&op.input0, &op.input1};
        for (int k = 0; k < 2; ++k) {
            if (resolved[k].kind != Operand::kMemory) continue;
            if (!loads(g, *in[k])) ++slots;
        }
        return slots;
    }

    // Closes every open group that loads or defines `buffer`, except that the group `keep` may go
    // on if it only ever sees the buffer through exactly the view `same` (in-place elementwise
    // update).  Returns true if it closed anything.
    bool closeGroupsTouching(const void* buffer, size_t keep, const View* same)
    {
        bool closed = false;
        if (!buffer) return false;
        touching(buffer, nullptr, m_candB);
        for (size_t gi = 0; gi < m_candB.size(); ++gi) {
            const size_t g = m_candB[gi];
            Group& grp = m_groups[g];
            if (!grp.open) continue;
            bool touches = false, conflicting = false;
            for (const ViewRef& r : grp.loads) {
                const View& v = view(r);
                if (v.data == buffer) { touches = true; if (!same || !sameView(v, *same)) conflicting = true; }
            }
            for (size_t def : grp.defs) {
                const View& v = defView(def);
                if (v.data == buffer) { touches = true; if (!same || !sameView(v, *same)) conflicting = true; }
            }
            if (!touches) continue;
            if (g == keep && !conflicting) continue;
            closeGroup(g);
            closed = true;
        }
        return closed;
    }

    void closeWriters(const void* buffer)
    {
        touching(buffer, nullptr, m_candB);
        for (size_t gi = 0; gi < m_candB.size(); ++gi)
            if (m_groups[m_candB[gi]].open && findDef(m_groups[m_candB[gi]], buffer) != SIZE_MAX) closeGroup(m_candB[gi]);
    }

    void closeGroup(size_t g)
    {
        if (!m_groups[g].open) return;
        m_groups[g].open = false;
        dropTouches(g);
        m_emits.push_back({true, g});
    }

    // A result is stored iff its buffer outlives the window or a later operator loads it from
    // memory before anything redefines the buffer.  Inside one group only the last definition of a
    // view is stored.
    void decideStores()
    {
        const size_t n = m_ops->size();
        m_store.assign(n, 0);
        for (size_t g = 0; g < m_groupCount; ++g)
            for (size_t def : m_groups[g].defs)
                if (m_live.count(defView(def).data)) m_store[def] = 1;
        m_lastWriter.clear();                                   // buffer -> the latest operator so far that writes it
        for (size_t j = 0; j < n; ++j) {
            const View* in[2] = {&at(j).input0, &at(j).input1};
            for (int k = 0; k < 2; ++k) {
                if (m_operands[j][k].kind != Operand::kMemory || !in[k]->data) continue;
                const auto it = m_lastWriter.find(in[k]->data);
                if (it == m_lastWriter.end()) continue;
                const size_t w = it->second;
                if (m_groupOf[w] != SIZE_MAX) {
                    // the value that must be in memory is the group's last definition of that view
                    for (size_t def : m_groups[m_groupOf[w]].defs)
                        if (sameView(defView(def), at(w).output)) m_store[def] = 1;
                }
            }
            if (at(j).output.data) m_lastWriter[at(j).output.data] = j;
        }
    }

    const FuseConfig& m_cfg;
    const std::vector<OpRecord>* m_ops{nullptr};
    Liveness m_live;
    std::vector<std::array<Operand, 2>> m_operands;
    std::vector<size_t> m_groupOf;
    std::vector<uint8_t> m_perRow;           // the operator yields one value per row of its (row program) group
    std::vector<Group> m_groups;             // [0, m_groupCount) belong to the current window
    size_t m_groupCount{0};
    std::unordered_map<const void*, uint32_t> m_touchIndex;      // buffer -> its list in m_touchLists
    std::vector<std::vector<uint32_t>> m_touchLists;             // (kept from window to window: [0, m_touchUsed) are in use)
    size_t m_touchUsed{0};
    std::vector<uint32_t> m_candA, m_candB;                      // working copies for the loops over touching groups
    std::unordered_map<const void*, size_t> m_lastWriter;        // decideStores()
    std::vector<Emit> m_emits;
    std::vector<PendingFill> m_fills;
    std::vector<uint8_t> m_store;
    std::vector<size_t> m_rest, m_merged, m_position;
    std::vector<std::pair<size_t, size_t>> m_scalarSlots;
    size_t m_fillsAbsorbed{0};
};

// ---- FuseEngine --------------------------------------------------------------------------------
FuseEngine::FuseEngine(const FuseConfig& config, FuseCallbacks callbacks) : m_config(config), m_callbacks(std::move(callbacks))
{
    if (m_config.maxBufferSlots == 0) throw std::invalid_argument("FuseEngine requires FuseConfig::maxBufferSlots > 0.");
    if (!m_callbacks.emitFused || !m_callbacks.emitSingle || !m_callbacks.finishFlush)
        throw std::invalid_argument("FuseEngine requires emitFused, emitSingle and finishFlush callbacks.");
    if (!m_callbacks.getKernelCacheStats) m_callbacks.getKernelCacheStats = [] { return std::pair<size_t, size_t>{0, 0}; };
    m_planner = std::make_unique<Planner>(m_config);
}

FuseEngine::~FuseEngine() = default;

void FuseEngine::maybeFlush()
{
    if (m_pending.size() >= m_config.flushThreshold) flush(false);
}

void FuseEngine::wake(const void* operand)
{
    if (!operand || m_waiting.empty()) return;
    const void* base = m_callbacks.blockBase ? m_callbacks.blockBase(operand) : operand;
    if (!base || !m_waitingBuffers.contains(base)) return;
    size_t kept = 0;
    for (size_t k = 0; k < m_waiting.size(); ++k) {
        if (m_waiting[k].output.data == base) { m_pending.push_back(m_waiting[k]); m_pending.back().hasWaited = true; }
        else { if (kept != k) m_waiting[kept] = m_waiting[k]; ++kept; }
    }
    m_waiting.resize(kept);
    m_waitingBuffers.erase(base);
}

// Moves the window's idle fills (see flush()) from m_window to m_waiting.
void FuseEngine::setAsideIdleFills()
{
    auto isFill = [](const OpRecord& op) { return op.type == OpType::Fill || op.type == OpType::FillMin; };
    size_t kept = 0;
    bool moved = false;
    for (size_t i = 0; i < m_window.size(); ++i) {
        const OpRecord& op = m_window[i];
        bool idle = isFill(op) && !op.hasWaited && op.output.dense && op.output.offset == 0 && m_live.contains(op.output.data) &&
                    !m_waitingBuffers.contains(op.output.data);
        if (idle) for (const void* r : m_externalReads) if (r == op.output.data) { idle = false; break; }
        if (idle) {
            const void* buf = op.output.data;
            for (size_t j = 0; j < m_window.size() && idle; ++j) {
                if (j == i) continue;
                const OpRecord& o = m_window[j];
                if (o.output.data == buf || o.input0.data == buf || (o.hasInput1 && o.input1.data == buf)) idle = false;
            }
            // (the records already moved sit at [0, kept) or were set aside: one set aside touched another buffer, or this
            // fill's buffer would be in m_waitingBuffers)
        }
        if (idle) { m_waiting.push_back(op); m_waitingBuffers.insert(op.output.data); moved = true; continue; }
        if (kept != i) m_window[kept] = m_window[i];
        ++kept;
    }
    if (moved) m_window.resize(kept);
}

OpRecord& FuseEngine::append(OpType type)
{
    m_pending.emplace_back();
    OpRecord& r = m_pending.back();
    r.type = type;
    return r;
}

void FuseEngine::record(OpType type, const View& input0, const View& output)
{
    wake(input0.data); wake(output.data);
    OpRecord& r = append(type);
    r.input0 = input0; r.output = output;
    maybeFlush();
}

void FuseEngine::record(OpType type, const View& input0, const View& input1, const View& output)
{
    wake(input0.data); wake(input1.data); wake(output.data);
    OpRecord& r = append(type);
    r.input0 = input0; r.input1 = input1; r.output = output; r.hasInput1 = true;
    maybeFlush();
}

void FuseEngine::recordFill(const void* scalar, DataType scalarDType, const View& output)
{
    wake(output.data);
    OpRecord& r = append(OpType::Fill);
    r.output = output; r.scalarDType = scalarDType;
    std::memcpy(r.scalarData.data(), scalar, aix::Device::dataTypeSize(scalarDType));
    maybeFlush();
}

void FuseEngine::recordTri(OpType type, const View& input, const View& output, int64_t diagonal)
{
    if ((type != OpType::Tril && type != OpType::Triu) || input.rank < 2) throw std::invalid_argument("recordTri: tril / triu of a tensor of rank 2 or more");
    wake(input.data); wake(output.data);
    OpRecord& r = append(type);
    r.input0 = input; r.output = output;
    r.triRows = input.shape[input.rank - 2]; r.triCols = input.shape[input.rank - 1]; r.triDiagonal = diagonal;
    maybeFlush();
}

void FuseEngine::recordRowReduce(OpType type, const View& input, const View& output, const void* init, size_t rowLength)
{
    if (!isRowReduce(type) || rowLength == 0 || input.size % rowLength != 0 || output.size != input.size / rowLength || input.dtype != output.dtype)
        throw std::invalid_argument("recordRowReduce: a sum / maximum over the rows of a [rows, length] operand into one value per row");
    wake(input.data); wake(output.data);
    OpRecord& r = append(type);
    r.input0 = input; r.output = output; r.rowLength = rowLength;
    r.scalarDType = output.dtype;
    std::memcpy(r.scalarData.data(), init, aix::Device::dataTypeSize(output.dtype));
    maybeFlush();
}

void FuseEngine::recordRowOnehot(const View& input, const View& output, size_t rowLength)
{
    if (rowLength == 0 || input.size % rowLength != 0 || output.size != input.size || output.dtype != DataType::kInt32 || !input.dense || !output.dense)
        throw std::invalid_argument("recordRowOnehot: rows of a dense operand into a dense int32 result of its shape");
    wake(input.data); wake(output.data);
    OpRecord& r = append(OpType::ArgmaxIndicesTo);
    r.input0 = input; r.output = output; r.rowLength = rowLength;
    maybeFlush();
}

void FuseEngine::recordWholeSum(const View& input, const View& output, const void* init)
{
    if (output.size != 1 || input.dtype != output.dtype || !input.dense)
        throw std::invalid_argument("recordWholeSum: the sum of a dense operand into one element of its type");
    wake(input.data); wake(output.data);
    OpRecord& r = append(OpType::ReduceTo);
    r.input0 = input; r.output = output; r.rowLength = 0; r.whole = true;
    r.scalarDType = output.dtype;
    std::memcpy(r.scalarData.data(), init, aix::Device::dataTypeSize(output.dtype));
    maybeFlush();
}

void FuseEngine::recordFillMin(const View& output)
{
    wake(output.data);
    OpRecord& r = append(OpType::FillMin);
    r.output = output;
    maybeFlush();
}

const FlushDiagnostics& FuseEngine::lastFlushDiagnostics() const
{
    static const FlushDiagnostics empty{};
    return m_diagnostics ? *m_diagnostics : empty;
}

void FuseEngine::flush(bool final)
{
    if (m_flushing) return;                  // callbacks may call back into the device
    if (final && !m_waiting.empty()) {       // every waiting fill runs now; nothing recorded since touches their buffers
        m_pending.insert(m_pending.begin(), m_waiting.begin(), m_waiting.end());
        for (const OpRecord& op : m_waiting) m_waitingBuffers.erase(op.output.data);
        m_waiting.clear();
    }
    if (m_pending.empty()) {                 // nothing recorded: the previous flush's diagnostics stay readable
        m_externalReads.clear();
        m_callbacks.finishFlush();
        return;
    }
    m_flushing = true;
    struct Reset { bool& f; ~Reset() { f = false; } } reset{m_flushing};

    if (m_config.diagnostics) { m_diagnostics.emplace(); m_diagnostics->opsRecorded = m_pending.size(); }

    m_window.clear();
    m_window.swap(m_pending);                // operators recorded by callbacks belong to the next window
    m_pendingUse.clear();
    m_counted = 0;
    if (!final && m_config.deferIdleFills && m_config.elementwiseFusion && m_config.absorbFills) setAsideIdleFills();
    const std::vector<OpRecord>& window = m_window;
    // buffers about to be read outside the planner count as alive for this window
    const Planner::Liveness live{&m_live, &m_externalReads};

    size_t fusedKernels = 0, fusedOps = 0, singles = 0;
    std::string groupsText;
    Planner& plan = *m_planner;
    plan.run(window, live);
    // The planner's list is one valid order; any order that keeps two kernels apart only where one touches what the other
    // writes is as good.  Kernels are sent off level by level -- a kernel's level is one more than the highest level of
    // an earlier kernel it depends on -- and kind by kind within a level, so that the same operator applied to tensor
    // after tensor (one attention head after the other) comes out as a run of equal kernels even when the program
    // interleaves it with others; the device sends such runs off as one launch.  Reads and writes are taken per
    // operator (every input, every output of every operator of a kernel): more than a kernel really loads and stores,
    // which can only add dependences.
    m_order.clear();
    m_touched.clear();
    if (!(m_config.groupEqualKernels && m_config.elementwiseFusion)) {
        for (size_t k = 0; k < plan.emits().size(); ++k) m_order.push_back({0, 0, k});
    } else {
        const auto& emits = plan.emits();
        auto each = [&](const Emit& e, auto&& fn) {
            if (!e.fused) { fn(window[e.index]); return; }
            for (size_t op : plan.group(e.index).ops) fn(window[op]);
        };
        for (size_t k = 0; k < emits.size(); ++k) {
            uint32_t level = 0;
            uint64_t kind = emits[k].fused ? 0xcbf29ce484222325ull : 0x84222325cbf29ce4ull;
            each(emits[k], [&](const OpRecord& op) {
                kind = (kind ^ (uint64_t)op.type ^ ((uint64_t)op.output.dtype << 8) ^ ((uint64_t)op.rowLength << 16)) * 0x100000001b3ull;
                const bool fill = op.type == OpType::Fill || op.type == OpType::FillMin;
                for (const void* r : {fill ? nullptr : op.input0.data, op.hasInput1 ? op.input1.data : nullptr}) {
                    if (!r) continue;
                    auto it = m_touched.find(r);
                    if (it != m_touched.end()) level = std::max(level, it->second.first);
                }
                auto it = m_touched.find(op.output.data);
                if (it != m_touched.end()) level = std::max({level, it->second.first, it->second.second});
            });
            each(emits[k], [&](const OpRecord& op) {
                const bool fill = op.type == OpType::Fill || op.type == OpType::FillMin;
                for (const void* r : {fill ? nullptr : op.input0.data, op.hasInput1 ? op.input1.data : nullptr})
                    if (r) { auto& t = m_touched[r]; t.second = std::max(t.second, level + 1); }
                auto& t = m_touched[op.output.data];
                t.first = std::max(t.first, level + 1);
            });
            m_order.push_back({level, kind, k});
        }
        std::sort(m_order.begin(), m_order.end(), [](const Order& a, const Order& b) {
            return a.level != b.level ? a.level < b.level : a.kind != b.kind ? a.kind < b.kind : a.at < b.at;
        });
    }
    for (const Order& o : m_order) {
        const auto& e = plan.emits()[o.at];
        if (!e.fused) { m_callbacks.emitSingle(window[e.index]); ++singles; continue; }
        const auto& g = plan.group(e.index);
        const bool castKernel = m_config.loneCastsAsKernels && g.ops.size() == 1 && window[g.ops[0]].type == OpType::Cast;
        if (plan.emitsAsSingle(g) && !castKernel) { m_callbacks.emitSingle(window[g.ops[0]]); ++singles; continue; }
        plan.describe(g, m_descriptor);
        if (m_descriptor.outputBuffers.empty()) continue;          // nothing of it is ever read: dead code
        m_callbacks.emitFused(m_descriptor);
        if (m_config.diagnostics) {
            if (fusedKernels) groupsText += ", ";
            groupsText += std::to_string(m_descriptor.ops.size()) + " ops";
        }
        ++fusedKernels;
        fusedOps += m_descriptor.ops.size();
    }
    m_callbacks.finishFlush();

    if (m_config.diagnostics) {
        auto& d = *m_diagnostics;
        d.fusibleSubgraphs = fusedKernels;
        d.fusedOps = fusedOps;
        d.fallbackOps = singles;
        d.dispatchesSaved = fusedOps - fusedKernels;
        d.fillsAbsorbed = plan.fillsAbsorbed();
        d.subgraphSummary = std::to_string(fusedKernels) + " subgraphs" + (fusedKernels ? " (" + groupsText + ")" : "");
        d.fallbackSummary = std::to_string(singles) + " individual ops";
        auto [hits, misses] = m_callbacks.getKernelCacheStats();
        d.kernelCacheHits = hits;
        d.kernelCacheMisses = misses;
    }
    m_externalReads.clear();
}

bool FuseEngine::takeTrailingFill(const View& output, OpRecord* fill)
{
    if (m_flushing || !output.data) return false;
    wake(output.data);
    for (size_t k = m_pending.size(); k-- > 0;) {
        const OpRecord& op = m_pending[k];
        const bool reads = op.type != OpType::Fill && op.type != OpType::FillMin &&
                           (op.input0.data == output.data || (op.hasInput1 && op.input1.data == output.data));
        if (reads) return false;
        if (op.output.data != output.data) continue;
        if ((op.type != OpType::Fill && op.type != OpType::FillMin) || op.output.dtype != output.dtype ||
            op.output.offset != output.offset || op.output.size != output.size || !output.dense || !op.output.dense)
            return false;
        *fill = op;
        if (k < m_counted) {                                    // (a fill: it only writes)
            auto it = m_pendingUse.find(op.output.data);
            if (it != m_pendingUse.end() && it->second.first) --it->second.first;
            --m_counted;
        }
        m_pending.erase(m_pending.begin() + (long)k);
        return true;
    }
    return false;
}

// How often the recorded operators write / read each buffer, brought up to date when somebody asks (operators are
// appended far more often than anybody asks).
void FuseEngine::countPending()
{
    for (; m_counted < m_pending.size(); ++m_counted) {
        const OpRecord& op = m_pending[m_counted];
        if (op.output.data) ++m_pendingUse[op.output.data].first;
        if (op.input0.data) ++m_pendingUse[op.input0.data].second;
        if (op.hasInput1 && op.input1.data) ++m_pendingUse[op.input1.data].second;
    }
}

bool FuseEngine::pendingWrites(const void* buffer)
{
    if (!buffer) return false;
    wake(buffer);
    countPending();
    const auto it = m_pendingUse.find(buffer);
    return it != m_pendingUse.end() && it->second.first != 0;
}

bool FuseEngine::pendingTouches(const void* buffer)
{
    if (!buffer) return false;
    wake(buffer);
    countPending();
    const auto it = m_pendingUse.find(buffer);
    return it != m_pendingUse.end() && (it->second.first != 0 || it->second.second != 0);
}

void FuseEngine::recordExternalRead(const void* buffer)
{
    if (!buffer) return;
    wake(buffer);
    for (const void* known : m_externalReads) if (known == buffer) return;
    m_externalReads.push_back(buffer);
}

void FuseEngine::retainBuffer(void* buffer) { if (buffer) m_live.insert(buffer); }

void FuseEngine::releaseBuffer(void* buffer)
{
    if (!buffer) return;
    m_live.erase(buffer);
    if (!m_waiting.empty() && m_waitingBuffers.contains(buffer)) {          // nobody will ever read what the fill would write
        size_t kept = 0;
        for (size_t k = 0; k < m_waiting.size(); ++k)
            if (m_waiting[k].output.data != buffer) { if (kept != k) m_waiting[kept] = m_waiting[k]; ++kept; }
        m_waiting.resize(kept);
        m_waitingBuffers.erase(buffer);
    }
    for (size_t k = 0; k < m_externalReads.size(); ++k)
        if (m_externalReads[k] == buffer) { m_externalReads[k] = m_externalReads.back(); m_externalReads.pop_back(); break; }
}

void FuseEngine::invalidateBuffer(void*) {}

} // namespace aixhip::fuse
