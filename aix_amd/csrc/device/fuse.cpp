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

std::vector<uint8_t> convertScalar(const void* scalar, DataType from, DataType to)
{
    std::vector<uint8_t> out(8, 0);
    const auto v = scalar::decode(scalar, static_cast<int>(from));
    out.resize(scalar::encode(v, static_cast<int>(to), out.data()));
    return out;
}

std::vector<uint8_t> lowestScalar(DataType dtype)
{
    std::vector<uint8_t> out(8, 0);
    auto put = [&](auto v) { std::memcpy(out.data(), &v, sizeof(v)); out.resize(sizeof(v)); };
    switch (dtype) {
        case DataType::kFloat64:  put(std::numeric_limits<double>::lowest()); break;
        case DataType::kFloat32:  put(std::numeric_limits<float>::lowest()); break;
        case DataType::kFloat16:  put((uint16_t)0xFBFF); break;          // aixFloat16.hpp:173-178
        case DataType::kBFloat16: put((uint16_t)0xFF7F); break;          // aixFloat16.hpp:767-772
        case DataType::kInt64:    put(std::numeric_limits<int64_t>::lowest()); break;
        case DataType::kInt32:    put(std::numeric_limits<int32_t>::lowest()); break;
        case DataType::kInt16:    put(std::numeric_limits<int16_t>::lowest()); break;
        case DataType::kInt8:     put(std::numeric_limits<int8_t>::lowest()); break;
        case DataType::kUInt8:    put((uint8_t)0); break;
    }
    return out;
}

namespace {

bool sameView(const DeviceTensorParams& a, const DeviceTensorParams& b)
{
    return a.data == b.data && a.dtype == b.dtype && a.offset == b.offset && a.shape == b.shape && a.strides == b.strides;
}

bool isDense(const DeviceTensorParams& p)
{
    size_t run = 1;
    for (size_t d = p.shape.size(); d-- > 0;) {
        if (p.shape[d] != 1 && p.strides[d] != run) return false;
        run *= p.shape[d];
    }
    return true;
}

// One past the last element position the view touches.
size_t viewEnd(const DeviceTensorParams& p)
{
    size_t last = p.offset;
    for (size_t d = 0; d < p.shape.size(); ++d) {
        if (p.shape[d] == 0) return p.offset;
        last += (p.shape[d] - 1) * p.strides[d];
    }
    return last + 1;
}

struct Operand {
    enum Kind { kNone, kMemory, kValue, kScalar } kind{kNone};
    size_t index{SIZE_MAX};          // kValue: defining op (window index); kScalar: fill op (window index)
};

struct Group {
    DataType dtype{DataType::kFloat32};
    size_t count{0};
    aix::Shape shape;
    bool dense{true};                                          // every loaded view so far is dense
    std::vector<size_t> ops;                                   // window indices, program order
    std::vector<std::pair<DeviceTensorParams, size_t>> defs;   // view -> latest defining op
    std::vector<DeviceTensorParams> loads;                     // distinct views loaded from memory
    bool open{true};
    bool absorbed{false};                                      // merged into another group
    bool hasScalar{false};
};

struct Emit {
    bool fused{false};
    size_t index{0};                 // group index or window index
};

struct PendingFill {
    size_t op;                       // window index
    size_t size;                     // elements filled from the base pointer
};

class Planner {
public:
    // A buffer outlives the window if somebody still holds it or if it is about to be read outside the planner.
    struct Liveness {
        const std::unordered_set<const void*>& held;
        const std::unordered_set<const void*>& external;
        size_t count(const void* p) const { return held.count(p) || external.count(p) ? 1 : 0; }
    };

    Planner(const std::vector<OpRecord>& ops, const FuseConfig& cfg, Liveness live)
        : m_ops(ops), m_cfg(cfg), m_live(live), m_operands(ops.size()), m_groupOf(ops.size(), SIZE_MAX) {}

    void run()
    {
        for (size_t i = 0; i < m_ops.size(); ++i) {
            const auto& op = m_ops[i];
            if (op.type == OpType::Fill || op.type == OpType::FillMin) placeFill(i);
            else if (isElementwiseOp(op.type) && op.type != OpType::Cast && m_cfg.elementwiseFusion) placeOp(i);
            else placeSingle(i);
        }
        for (size_t g = 0; g < m_groups.size(); ++g) closeGroup(g);
        // fills nobody could absorb completely: run them if the buffer outlives the window
        std::vector<size_t> rest;
        for (auto& [buf, pf] : m_fills) if (m_live.count(buf)) rest.push_back(pf.op);
        std::sort(rest.begin(), rest.end());
        for (size_t op : rest) m_emits.push_back({false, op});
        m_fills.clear();
        decideStores();
    }

    const std::vector<Emit>& emits() const { return m_emits; }
    const std::vector<Group>& groups() const { return m_groups; }
    size_t fillsAbsorbed() const { return m_fillsAbsorbed; }

    // A group of one operator without immediates runs as a plain single operator.
    bool emitsAsSingle(const Group& g) const { return g.ops.size() == 1 && !g.hasScalar; }

    FusedSubgraphDescriptor describe(const Group& g) const
    {
        FusedSubgraphDescriptor d;
        d.dtype = g.dtype;
        d.elementCount = g.count;
        d.shape = g.shape;
        d.allContiguous = true;
        std::unordered_map<size_t, size_t> position;          // window index -> position in d.ops
        std::unordered_map<size_t, size_t> scalarSlot;        // fill op -> scalar index
        auto inputSlot = [&](const DeviceTensorParams& v) {
            for (size_t k = 0; k < d.inputBuffers.size(); ++k) if (sameView(d.inputBuffers[k], v)) return k;
            d.inputBuffers.push_back(v);
            if (!isDense(v)) d.allContiguous = false;
            return d.inputBuffers.size() - 1;
        };
        // external inputs first, so that value indices (inputs.size() + position) are stable
        for (size_t w : g.ops) {
            const auto& op = m_ops[w];
            if (m_operands[w][0].kind == Operand::kMemory) inputSlot(op.input0);
            if (m_operands[w][1].kind == Operand::kMemory) inputSlot(op.input1);
        }
        const size_t nIn = d.inputBuffers.size();
        const size_t esz = aix::Device::dataTypeSize(g.dtype);
        auto scalarIndex = [&](size_t fillOp) {
            auto it = scalarSlot.find(fillOp);
            if (it != scalarSlot.end()) return it->second;
            const auto& f = m_ops[fillOp];
            auto bytes = f.type == OpType::FillMin ? lowestScalar(g.dtype)
                                                   : convertScalar(f.scalarData.data(), f.scalarDType, g.dtype);
            const size_t slot = d.scalarData.size() / esz;
            d.scalarData.insert(d.scalarData.end(), bytes.begin(), bytes.end());
            scalarSlot[fillOp] = slot;
            return slot;
        };
        for (size_t w : g.ops) {
            const auto& op = m_ops[w];
            FusedSubgraphDescriptor::Op o;
            o.type = op.type;
            const DeviceTensorParams* in[2] = {&op.input0, &op.input1};
            size_t* idx[2] = {&o.inputIndex0, &o.inputIndex1};
            size_t* sc[2] = {&o.scalarIndex0, &o.scalarIndex1};
            for (int k = 0; k < 2; ++k) {
                const auto& operand = m_operands[w][k];
                if (operand.kind == Operand::kMemory) *idx[k] = inputSlot(*in[k]);
                else if (operand.kind == Operand::kValue) *idx[k] = nIn + position.at(operand.index);
                else if (operand.kind == Operand::kScalar) *sc[k] = scalarIndex(operand.index);
            }
            if (m_store[w]) {
                o.outputIndex = d.outputBuffers.size();
                d.outputBuffers.push_back(op.output);
                if (!isDense(op.output)) d.allContiguous = false;
            }
            position[w] = d.ops.size();
            d.ops.push_back(o);
        }
        return d;
    }

private:
    // ---- fills --------------------------------------------------------------------------------
    void placeFill(size_t i)
    {
        const auto& out = m_ops[i].output;
        if (!m_cfg.absorbFills || !m_cfg.elementwiseFusion) { placeSingle(i); return; }
        // groups that see the buffer's previous content must run before anything overwrites it
        closeGroupsTouching(out.data, SIZE_MAX, nullptr);
        auto it = m_fills.find(out.data);
        if (it != m_fills.end() && it->second.size > out.size) materialise(out.data);   // older, larger fill survives underneath
        m_fills[out.data] = PendingFill{i, out.size};                                   // written flat from the base pointer
    }

    void materialise(const void* buffer)
    {
        auto it = m_fills.find(buffer);
        if (it == m_fills.end()) return;
        m_emits.push_back({false, it->second.op});
        m_fills.erase(it);
    }

    // ---- operators that cannot be fused ----------------------------------------------------------
    void placeSingle(size_t i)
    {
        const auto& op = m_ops[i];
        for (const DeviceTensorParams* in : {&op.input0, &op.input1}) {
            if (!in->data) continue;
            materialise(in->data);
            closeWriters(in->data);
        }
        if (op.output.data) {
            closeGroupsTouching(op.output.data, SIZE_MAX, nullptr);
            if (op.type == OpType::Fill || op.type == OpType::FillMin) m_fills.erase(op.output.data);
            else materialise(op.output.data);
        }
        if (op.input0.data) m_operands[i][0].kind = Operand::kMemory;
        if (op.hasInput1 && op.input1.data) m_operands[i][1].kind = Operand::kMemory;
        m_emits.push_back({false, i});
    }

    // ---- fusable operators ---------------------------------------------------------------------
    void placeOp(size_t i)
    {
        const auto& op = m_ops[i];
        const bool binary = op.hasInput1;
        const DeviceTensorParams* in[2] = {&op.input0, binary ? &op.input1 : nullptr};

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
                auto f = m_fills.find(in[k]->data);
                if (f != m_fills.end()) {
                    if (in[k]->dtype == m_ops[f->second.op].output.dtype && viewEnd(*in[k]) <= f->second.size) {
                        resolved[k] = Operand{Operand::kScalar, f->second.op};
                        continue;
                    }
                    materialise(in[k]->data);
                }
                resolved[k].kind = Operand::kMemory;
                for (size_t g = 0; g < m_groups.size(); ++g) {
                    if (!m_groups[g].open) continue;
                    const auto* def = findDef(m_groups[g], in[k]->data);
                    if (!def) continue;
                    const bool usable = sameView(def->first, *in[k]) && compatible(m_groups[g], op);
                    if (usable && (target == SIZE_MAX || target == g)) {
                        resolved[k] = Operand{Operand::kValue, def->second};
                        target = g;
                    } else if (usable && mergeable(m_groups[target], m_groups[g])) {
                        // both operands come from open groups: open groups are independent of each
                        // other, so the two become one kernel
                        resolved[k] = Operand{Operand::kValue, def->second};
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
                for (size_t g = 0; g < m_groups.size() && target == SIZE_MAX; ++g) {
                    if (!m_groups[g].open || !compatible(m_groups[g], op)) continue;
                    for (int k = 0; k < 2; ++k)
                        if (resolved[k].kind == Operand::kMemory)
                            for (const auto& v : m_groups[g].loads)
                                if (sameView(v, *in[k])) target = g;
                }
            }

            // hazards on the output buffer
            if (closeGroupsTouching(op.output.data, target, &op.output)) continue;
            if (target != SIZE_MAX && slotsAfterJoin(m_groups[target], op, resolved) > m_cfg.maxBufferSlots) {
                closeGroup(target);
                continue;
            }
            break;
        }

        // a fill that this operator overwrites completely never has to run
        auto f = m_fills.find(op.output.data);
        if (f != m_fills.end()) {
            if (isDense(op.output) && op.output.offset == 0 && op.output.size >= f->second.size) m_fills.erase(f);
            else materialise(op.output.data);
        }

        if (target == SIZE_MAX) {
            Group g;
            g.dtype = op.output.dtype;
            g.count = op.output.size;
            g.shape = op.output.shape;
            m_groups.push_back(std::move(g));
            target = m_groups.size() - 1;
        }
        Group& g = m_groups[target];
        for (int k = 0; k < 2; ++k) {
            m_operands[i][k] = resolved[k];
            if (resolved[k].kind == Operand::kMemory) {
                bool known = false;
                for (const auto& v : g.loads) if (sameView(v, *in[k])) known = true;
                if (!known) g.loads.push_back(*in[k]);
                if (!isDense(*in[k])) g.dense = false;
            } else if (resolved[k].kind == Operand::kScalar) {
                g.hasScalar = true;
                ++m_fillsAbsorbed;
            }
        }
        bool redefined = false;
        for (auto& def : g.defs) if (sameView(def.first, op.output)) { def.second = i; redefined = true; }
        if (!redefined) g.defs.emplace_back(op.output, i);
        g.ops.push_back(i);
        m_groupOf[i] = target;
    }

    static const std::pair<DeviceTensorParams, size_t>* findDef(const Group& g, const void* buffer)
    {
        for (const auto& def : g.defs) if (def.first.data == buffer) return &def;
        return nullptr;
    }

    // Same element type and iteration space: identical shape, or equal element counts when both
    // sides only touch dense views (then the flat index is all that matters).
    bool compatible(const Group& g, const OpRecord& op) const
    {
        if (g.dtype != op.output.dtype || g.count != op.output.size) return false;
        if (g.shape == op.output.shape) return true;
        const bool opDense = isDense(op.output) && (!op.input0.data || isDense(op.input0)) &&
                             (!op.hasInput1 || !op.input1.data || isDense(op.input1));
        return g.dense && opDense;
    }

    bool mergeable(const Group& a, const Group& b) const
    {
        if (a.dtype != b.dtype || a.count != b.count) return false;
        if (!(a.shape == b.shape) && !(a.dense && b.dense)) return false;
        size_t loads = a.loads.size();
        for (const auto& v : b.loads) {
            bool known = false;
            for (const auto& w : a.loads) if (sameView(v, w)) known = true;
            if (!known) ++loads;
        }
        return loads + a.defs.size() + b.defs.size() + 1 <= m_cfg.maxBufferSlots;
    }

    // Folds open group `from` into open group `into` (no hazards can exist between open groups).
    void mergeInto(size_t into, size_t from)
    {
        Group& a = m_groups[into];
        Group& b = m_groups[from];
        std::vector<size_t> ops(a.ops.size() + b.ops.size());
        std::merge(a.ops.begin(), a.ops.end(), b.ops.begin(), b.ops.end(), ops.begin());     // program order
        a.ops.swap(ops);
        for (auto& d : b.defs) a.defs.push_back(d);
        for (const auto& v : b.loads) {
            bool known = false;
            for (const auto& w : a.loads) if (sameView(v, w)) known = true;
            if (!known) a.loads.push_back(v);
        }
        a.dense = a.dense && b.dense;
        a.hasScalar = a.hasScalar || b.hasScalar;
        for (size_t w : b.ops) m_groupOf[w] = into;
        b.ops.clear(); b.defs.clear(); b.loads.clear();
        b.open = false;                                     // absorbed: never emitted on its own
        b.absorbed = true;
    }

    size_t slotsAfterJoin(const Group& g, const OpRecord& op, const Operand* resolved) const
    {
        size_t slots = g.loads.size() + g.defs.size() + 1;     // every def may have to be stored
        const DeviceTensorParams* in[2] = {&op.input0, &op.input1};
        for (int k = 0; k < 2; ++k) {
            if (resolved[k].kind != Operand::kMemory) continue;
            bool known = false;
            for (const auto& v : g.loads) if (sameView(v, *in[k])) known = true;
            if (!known) ++slots;
        }
        return slots;
    }

    // Closes every open group that loads or defines `buffer`, except that the group `keep` may go
    // on if it only ever sees the buffer through exactly the view `same` (in-place elementwise
    // update).  Returns true if it closed anything.
    bool closeGroupsTouching(const void* buffer, size_t keep, const DeviceTensorParams* same)
    {
        bool closed = false;
        if (!buffer) return false;
        for (size_t g = 0; g < m_groups.size(); ++g) {
            Group& grp = m_groups[g];
            if (!grp.open) continue;
            bool touches = false, conflicting = false;
            for (const auto& v : grp.loads) if (v.data == buffer) { touches = true; if (!same || !sameView(v, *same)) conflicting = true; }
            for (const auto& d : grp.defs) if (d.first.data == buffer) { touches = true; if (!same || !sameView(d.first, *same)) conflicting = true; }
            if (!touches) continue;
            if (g == keep && !conflicting) continue;
            closeGroup(g);
            closed = true;
        }
        return closed;
    }

    void closeWriters(const void* buffer)
    {
        for (size_t g = 0; g < m_groups.size(); ++g)
            if (m_groups[g].open && findDef(m_groups[g], buffer)) closeGroup(g);
    }

    void closeGroup(size_t g)
    {
        if (!m_groups[g].open) return;
        m_groups[g].open = false;
        m_emits.push_back({true, g});
    }

    // A result is stored iff its buffer outlives the window or a later operator loads it from
    // memory before anything redefines the buffer.  Inside one group only the last definition of a
    // view is stored.
    void decideStores()
    {
        m_store.assign(m_ops.size(), false);
        for (size_t g = 0; g < m_groups.size(); ++g)
            for (const auto& def : m_groups[g].defs)
                if (m_live.count(def.first.data)) m_store[def.second] = true;
        for (size_t j = 0; j < m_ops.size(); ++j) {
            const DeviceTensorParams* in[2] = {&m_ops[j].input0, &m_ops[j].input1};
            for (int k = 0; k < 2; ++k) {
                if (m_operands[j][k].kind != Operand::kMemory || !in[k]->data) continue;
                for (size_t w = j; w-- > 0;) {
                    if (m_ops[w].output.data != in[k]->data) continue;
                    if (m_groupOf[w] != SIZE_MAX) {
                        // the value that must be in memory is the group's last definition of that view
                        for (const auto& def : m_groups[m_groupOf[w]].defs)
                            if (sameView(def.first, m_ops[w].output)) m_store[def.second] = true;
                    }
                    break;
                }
            }
        }
    }

    const std::vector<OpRecord>& m_ops;
    const FuseConfig& m_cfg;
    const Liveness m_live;
    std::vector<std::array<Operand, 2>> m_operands;
    std::vector<size_t> m_groupOf;
    std::vector<Group> m_groups;
    std::vector<Emit> m_emits;
    std::unordered_map<const void*, PendingFill> m_fills;
    std::vector<bool> m_store;
    size_t m_fillsAbsorbed{0};
};

} // namespace

// ---- FuseEngine --------------------------------------------------------------------------------
FuseEngine::FuseEngine(const FuseConfig& config, FuseCallbacks callbacks) : m_config(config), m_callbacks(std::move(callbacks))
{
    if (m_config.maxBufferSlots == 0) throw std::invalid_argument("FuseEngine requires FuseConfig::maxBufferSlots > 0.");
    if (!m_callbacks.emitFused || !m_callbacks.emitSingle || !m_callbacks.finishFlush)
        throw std::invalid_argument("FuseEngine requires emitFused, emitSingle and finishFlush callbacks.");
    if (!m_callbacks.getKernelCacheStats) m_callbacks.getKernelCacheStats = [] { return std::pair<size_t, size_t>{0, 0}; };
}

void FuseEngine::maybeFlush()
{
    if (m_pending.size() >= m_config.flushThreshold) flush();
}

void FuseEngine::record(OpType type, const DeviceTensorParams& input0, const DeviceTensorParams& output)
{
    OpRecord r;
    r.type = type; r.input0 = input0; r.output = output;
    m_pending.push_back(std::move(r));
    maybeFlush();
}

void FuseEngine::record(OpType type, const DeviceTensorParams& input0, const DeviceTensorParams& input1, const DeviceTensorParams& output)
{
    OpRecord r;
    r.type = type; r.input0 = input0; r.input1 = input1; r.output = output; r.hasInput1 = true;
    m_pending.push_back(std::move(r));
    maybeFlush();
}

void FuseEngine::recordFill(const void* scalar, DataType scalarDType, const DeviceTensorParams& output)
{
    OpRecord r;
    r.type = OpType::Fill; r.output = output; r.scalarDType = scalarDType;
    const size_t n = aix::Device::dataTypeSize(scalarDType);
    r.scalarData.assign(static_cast<const uint8_t*>(scalar), static_cast<const uint8_t*>(scalar) + n);
    m_pending.push_back(std::move(r));
    maybeFlush();
}

void FuseEngine::recordFillMin(const DeviceTensorParams& output)
{
    OpRecord r;
    r.type = OpType::FillMin; r.output = output;
    m_pending.push_back(std::move(r));
    maybeFlush();
}

const FlushDiagnostics& FuseEngine::lastFlushDiagnostics() const
{
    static const FlushDiagnostics empty{};
    return m_diagnostics ? *m_diagnostics : empty;
}

void FuseEngine::flush()
{
    if (m_flushing) return;                  // callbacks may call back into the device
    if (m_pending.empty()) {                 // nothing recorded: the previous flush's diagnostics stay readable
        m_externalReads.clear();
        m_callbacks.finishFlush();
        return;
    }
    m_flushing = true;
    struct Reset { bool& f; ~Reset() { f = false; } } reset{m_flushing};

    if (m_config.diagnostics) { m_diagnostics.emplace(); m_diagnostics->opsRecorded = m_pending.size(); }

    std::vector<OpRecord> window;
    window.swap(m_pending);
    // buffers about to be read outside the planner count as alive for this window
    const Planner::Liveness live{m_live, m_externalReads};

    size_t fusedKernels = 0, fusedOps = 0, singles = 0, absorbed = 0;
    std::ostringstream groupsText;
    if (!window.empty()) {
        Planner plan(window, m_config, live);
        plan.run();
        for (const auto& e : plan.emits()) {
            if (!e.fused) { m_callbacks.emitSingle(window[e.index]); ++singles; continue; }
            const auto& g = plan.groups()[e.index];
            if (plan.emitsAsSingle(g)) { m_callbacks.emitSingle(window[g.ops[0]]); ++singles; continue; }
            auto desc = plan.describe(g);
            if (desc.outputBuffers.empty()) continue;          // nothing of it is ever read: dead code
            m_callbacks.emitFused(desc);
            if (fusedKernels) groupsText << ", ";
            groupsText << desc.ops.size() << " ops";
            ++fusedKernels;
            fusedOps += desc.ops.size();
        }
        absorbed = plan.fillsAbsorbed();
    }
    m_callbacks.finishFlush();

    if (m_config.diagnostics) {
        auto& d = *m_diagnostics;
        d.fusibleSubgraphs = fusedKernels;
        d.fusedOps = fusedOps;
        d.fallbackOps = singles;
        d.dispatchesSaved = fusedOps - fusedKernels;
        d.fillsAbsorbed = absorbed;
        d.subgraphSummary = std::to_string(fusedKernels) + " subgraphs" + (fusedKernels ? " (" + groupsText.str() + ")" : "");
        d.fallbackSummary = std::to_string(singles) + " individual ops";
        auto [hits, misses] = m_callbacks.getKernelCacheStats();
        d.kernelCacheHits = hits;
        d.kernelCacheMisses = misses;
    }
    m_externalReads.clear();
}

bool FuseEngine::takeTrailingFill(const DeviceTensorParams& output, OpRecord* fill)
{
    if (m_flushing || !output.data) return false;
    for (size_t k = m_pending.size(); k-- > 0;) {
        const OpRecord& op = m_pending[k];
        const bool reads = op.type != OpType::Fill && op.type != OpType::FillMin &&
                           (op.input0.data == output.data || (op.hasInput1 && op.input1.data == output.data));
        if (reads) return false;
        if (op.output.data != output.data) continue;
        if ((op.type != OpType::Fill && op.type != OpType::FillMin) || op.output.dtype != output.dtype ||
            op.output.offset != output.offset || op.output.size != output.size || !output.isContiguous || !op.output.isContiguous)
            return false;
        *fill = op;
        m_pending.erase(m_pending.begin() + (long)k);
        return true;
    }
    return false;
}

void FuseEngine::recordExternalRead(const void* buffer) { if (buffer) m_externalReads.insert(buffer); }
void FuseEngine::retainBuffer(void* buffer) { if (buffer) m_live.insert(buffer); }
void FuseEngine::releaseBuffer(void* buffer) { if (buffer) { m_live.erase(buffer); m_externalReads.erase(buffer); } }
void FuseEngine::invalidateBuffer(void*) {}

} // namespace aixhip::fuse
