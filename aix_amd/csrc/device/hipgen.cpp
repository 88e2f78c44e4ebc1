// hipgen.cpp -- HIP source generation for fused elementwise kernels (see hipgen.hpp).

#include "hipgen.hpp"

#include <array>
#include <cstring>
#include <sstream>
#include <stdexcept>
#include <vector>

namespace aixhip::gen {

using fuse::FusedSubgraphDescriptor;
using fuse::OpType;

static std::string entryNameWith(const fuse::FusedSubgraphDescriptor& d, const char* tag)
{
    static const char* const types[] = {"f64", "f32", "f16", "bf16", "i64", "i32", "i16", "i8", "u8"};
    std::string name = std::string("aix_fused_") + types[static_cast<size_t>(d.dtype)] + "_" + tag + "_";
    for (const auto& op : d.ops) {
        const char* n = fuse::opName(op.type);
        if (name.size() + std::strlen(n) > 116) { name += "_etc"; break; }
        name += n;
    }
    return name;
}

std::string entryName(const fuse::FusedSubgraphDescriptor& d, Shape shape)
{
    return entryNameWith(d, shape == Shape::Flat ? "flat" : shape == Shape::Rows ? "rows" : "gather");
}

std::string rowEntryName(const fuse::FusedSubgraphDescriptor& d, const RowGeometry& g)
{
    return entryNameWith(d, g.lanes == 64 ? "row64" : "row256");
}

namespace {

const char* typeName(aix::DataType t)
{
    switch (t) {
        case aix::DataType::kFloat64:  return "double";
        case aix::DataType::kFloat32:  return "float";
        case aix::DataType::kFloat16:  return "f16";
        case aix::DataType::kBFloat16: return "bf16";
        case aix::DataType::kInt64:    return "i64";
        case aix::DataType::kInt32:    return "i32";
        case aix::DataType::kInt16:    return "i16";
        case aix::DataType::kInt8:     return "i8";
        case aix::DataType::kUInt8:    return "u8";
    }
    return "float";
}

const char* shortType(aix::DataType t)
{
    static const char* n[] = {"f64", "f32", "f16", "bf16", "i64", "i32", "i16", "i8", "u8"};
    return n[static_cast<size_t>(t)];
}

const char* wordName(size_t bytes) { return bytes == 1 ? "u8" : bytes == 2 ? "u16" : bytes == 4 ? "u32" : "u64"; }

const char* fnName(OpType t)
{
    switch (t) {
        case OpType::Add: return "e_add";   case OpType::Sub: return "e_sub";   case OpType::Mul: return "e_mul";
        case OpType::Div: return "e_div";   case OpType::Pow: return "e_pow";   case OpType::Negate: return "e_neg";
        case OpType::Sqrt: return "e_sqrt"; case OpType::Sin: return "e_sin";   case OpType::Cos: return "e_cos";
        case OpType::Tanh: return "e_tanh"; case OpType::Log: return "e_log";   case OpType::Exp: return "e_exp";
        default: throw std::invalid_argument(std::string("operator cannot be fused: ") + fuse::opName(t));
    }
}

bool isBinary(OpType t) { return t == OpType::Add || t == OpType::Sub || t == OpType::Mul || t == OpType::Div || t == OpType::Pow; }

size_t scalarCount(const FusedSubgraphDescriptor& d)
{
    return d.scalarData.size() / aix::Device::dataTypeSize(d.dtype);
}

bool isTri(OpType t) { return t == OpType::Tril || t == OpType::Triu; }

size_t triCount(const FusedSubgraphDescriptor& d)
{
    size_t n = 0;
    for (const auto& op : d.ops) if (isTri(op.type)) ++n;
    return n;
}

std::string operandText(const FusedSubgraphDescriptor& d, size_t tensorIndex, size_t scalarIndex)
{
    if (tensorIndex != SIZE_MAX) {
        if (tensorIndex < d.inputBuffers.size()) return "x[" + std::to_string(tensorIndex) + "]";
        return "v" + std::to_string(tensorIndex - d.inputBuffers.size());
    }
    if (scalarIndex != SIZE_MAX) return "s[" + std::to_string(scalarIndex) + "]";
    throw std::invalid_argument("fused operator without an operand");
}

// The per-element SSA body shared by the vector loop and the tails.  Every value has the kernel's
// one element type T: loads convert to it and stores convert from it, so a cast is the identity here.
void emitBody(std::ostringstream& o, const FusedSubgraphDescriptor& d)
{
    // kernels with a tril / triu also get the element's flat logical index and the operators' (rows, cols, diagonal)
    if (triCount(d)) o << "__device__ __forceinline__ void aix_body(const T* x, const T* s, T* out, int e, const TriPos* tpos, const u64* tp)\n{\n";
    else o << "__device__ __forceinline__ void aix_body(const T* x, const T* s, T* out)\n{\n";
    for (size_t k = 0; k < d.ops.size(); ++k) {
        const auto& op = d.ops[k];
        if (op.type == OpType::Cast || op.whole) o << "    const T v" << k << " = " << operandText(d, op.inputIndex0, op.scalarIndex0) << ";\n";   // (a sum of everything: the loops add this value up)
        else if (isTri(op.type))
            o << "    const T v" << k << " = tri_keeps(tpos[" << op.paramIndex << "], e, tp[" << 3 * op.paramIndex << "], tp[" << 3 * op.paramIndex + 1 << "], (i64)tp["
              << 3 * op.paramIndex + 2 << "], " << (op.type == OpType::Triu ? 1 : 0) << ") ? " << operandText(d, op.inputIndex0, op.scalarIndex0) << " : zero<T>();\n";
        else {
            o << "    const T v" << k << " = " << fnName(op.type) << "(" << operandText(d, op.inputIndex0, op.scalarIndex0);
            if (isBinary(op.type)) o << ", " << operandText(d, op.inputIndex1, op.scalarIndex1);
            o << ");\n";
        }
        if (op.outputIndex != SIZE_MAX) o << "    out[" << op.outputIndex << "] = v" << k << ";\n";
    }
    o << "}\n\n";
}

} // namespace

namespace {

void appendNumber(std::string& out, uint64_t v, unsigned base = 10)
{
    char digits[24];
    int n = 0;
    do { const unsigned r = (unsigned)(v % base); digits[n++] = (char)(r < 10 ? '0' + r : 'a' + (r - 10)); v /= base; } while (v);
    while (n) out.push_back(digits[--n]);
}

void appendOperand(std::string& out, const FusedSubgraphDescriptor& d, size_t tensorIndex, size_t scalarIndex)
{
    if (tensorIndex != SIZE_MAX) {
        if (tensorIndex < d.inputBuffers.size()) { out += "x["; appendNumber(out, tensorIndex); out += ']'; }
        else { out += 'v'; appendNumber(out, tensorIndex - d.inputBuffers.size()); }
        return;
    }
    if (scalarIndex == SIZE_MAX) throw std::invalid_argument("fused operator without an operand");
    out += "s["; appendNumber(out, scalarIndex); out += ']';
}

} // namespace

void signatureInto(std::string& s, const FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask, bool noAlias, bool streamOut)
{
    s.clear();
    s += shortType(d.dtype);
    s += shape == Shape::Flat ? "|flat" : shape == Shape::Rows ? "|rows" : "|gather";
    if (streamOut && shape != Shape::Gather) s += "|nt";
    if (shape == Shape::Flat) { s += noAlias ? 'r' : 'a'; appendNumber(s, broadcastMask, 16); }
    s += "|i"; appendNumber(s, d.inputBuffers.size());
    s += 'o';  appendNumber(s, d.outputBuffers.size());
    s += 's';  appendNumber(s, scalarCount(d));
    // buffers of another element type than the kernel's (fused casts): part of the identity
    for (size_t k = 0; k < d.inputBuffers.size(); ++k)
        if (d.inputBuffers[k].dtype != d.dtype) { s += "|x"; appendNumber(s, k); s += ':'; s += shortType(d.inputBuffers[k].dtype); }
    for (size_t k = 0; k < d.outputBuffers.size(); ++k)
        if (d.outputBuffers[k].dtype != d.dtype) { s += "|y"; appendNumber(s, k); s += ':'; s += shortType(d.outputBuffers[k].dtype); }
    for (const auto& op : d.ops) {
        s += '|'; s += fuse::opName(op.type); if (op.whole) s += '!'; s += '(';
        appendOperand(s, d, op.inputIndex0, op.scalarIndex0);
        if (isBinary(op.type)) { s += ','; appendOperand(s, d, op.inputIndex1, op.scalarIndex1); }
        s += ')';
        if (op.outputIndex != SIZE_MAX) { s += ">o"; appendNumber(s, op.outputIndex); }
    }
}

std::string signature(const FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask, bool noAlias, bool streamOut)
{
    std::string s;
    signatureInto(s, d, shape, broadcastMask, noAlias, streamOut);
    return s;
}

std::string source(const FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask, bool noAlias, bool streamOut, bool many)
{
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size(), NS = scalarCount(d), NT = triCount(d);
    if (NO == 0) throw std::invalid_argument("fused kernel without outputs");
    if (d.opParams.size() != 3 * NT) throw std::invalid_argument("fused kernel: tril / triu without its parameters");
    const size_t esz = aix::Device::dataTypeSize(d.dtype);
    const size_t AI = NI ? NI : 1, AS = NS ? NS : 1;
    std::ostringstream o;
    o << "#include \"aix_device.h\"\nusing namespace aixd;\n"
      << "// " << signature(d, shape, broadcastMask, noAlias, streamOut) << "\n"
      << "#define AIX_NT " << (streamOut ? "true" : "false") << "\n"
      << "typedef " << typeName(d.dtype) << " T;\n"
      << "typedef " << wordName(esz) << " word_t;\n"
      << "#define VEC (vec16<T>::n)\n#define NI " << NI << "\n#define NO " << NO << "\n#define NS " << NS << "\n";
    // Buffers carry their own element type (a fused cast makes it differ from T): loads convert to T,
    // stores convert from it.  Same type: the bits pass through untouched.
    for (size_t k = 0; k < NI; ++k) o << "typedef " << typeName(d.inputBuffers[k].dtype) << " I" << k << ";\n";
    for (size_t k = 0; k < NO; ++k) o << "typedef " << typeName(d.outputBuffers[k].dtype) << " O" << k << ";\n";
    o << "\n";
    // outputs that are sums over everything: the loops add their value up per lane instead of storing it, the workgroup's
    // total goes to slot BID of the buffer the output pointer names (partial sums in the wide type, one per workgroup)
    std::vector<char> whole(NO, 0);
    bool anyWhole = false;
    for (const auto& op : d.ops) if (op.whole && op.outputIndex != SIZE_MAX) { whole[op.outputIndex] = 1; anyWhole = true; }
    if (anyWhole) o << "typedef traits<T>::W W;\n";
    auto wholeInit = [&](std::ostringstream& os) { for (size_t k = 0; k < NO; ++k) if (whole[k]) os << "    W acc" << k << " = (W)0;\n"; };
    auto wholeAdd = [&](std::ostringstream& os, const char* indent) { for (size_t k = 0; k < NO; ++k) if (whole[k]) os << indent << "acc" << k << " += up(y[" << k << "]);\n"; };
    auto wholeLand = [&](std::ostringstream& os) {
        if (!anyWhole) return;
        os << "    __shared__ W red[4];\n";
        for (size_t k = 0; k < NO; ++k)
            if (whole[k]) os << "    { const W t = row_sum<256>(acc" << k << ", red); if (threadIdx.x == 0) global_ptr<W>((u64)a.out[" << k << "])[BID] = t; }\n";
    };
    auto in_same = [&](size_t k) { return d.inputBuffers[k].dtype == d.dtype; };
    auto out_same = [&](size_t k) { return d.outputBuffers[k].dtype == d.dtype; };
    auto to_t = [&](size_t k, const std::string& e) { return in_same(k) ? e : "convert<I" + std::to_string(k) + ", T>(" + e + ")"; };
    auto from_t = [&](size_t k, const std::string& e) { return out_same(k) ? e : "convert<T, O" + std::to_string(k) + ">(" + e + ")"; };
    emitBody(o, d);

    o << "struct Args {\n    const void* in[" << AI << "];\n    void* out[" << NO << "];\n    u64 sc[" << AS << "];\n";
    if (NT) o << "    u64 tp[" << 3 * NT << "];\n";
    o << "    u64 n;\n";
    if (shape != Shape::Flat) o << "    u64 chunks;\n    u64 rank;\n    u64 shape[" << kMaxDims << "];\n    u64 off[" << AI << "];\n    u64 str[" << AI << "][" << kMaxDims << "];\n";
    o << "};\n\n";

    if (many) {
        // one launch for several argument blocks: the workgroup finds the block whose share of the grid it is in
        o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << entryName(d, shape) << "_many(const Args* table, const u32* starts, u32 count)\n{\n"
          << "    u32 lo = 0, hi = count;\n"
          << "    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (starts[mid] <= blockIdx.x) lo = mid; else hi = mid; }\n"
          << "    const Args a = table[lo];\n"
          << "    const u32 BID = blockIdx.x - starts[lo], GDIM = starts[lo + 1] - starts[lo];\n";
    } else {
        o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << entryName(d, shape) << "(Args a)\n{\n"
          << "    const u32 BID = blockIdx.x, GDIM = gridDim.x;\n    (void)BID; (void)GDIM;\n";
    }
    o << "    T s[" << AS << "];\n";
    for (size_t k = 0; k < NS; ++k) o << "    s[" << k << "] = __builtin_bit_cast(T, (word_t)a.sc[" << k << "]);\n";
    if (NS == 0) o << "    s[0] = zero<T>();\n";
    for (size_t k = 0; k < NI; ++k) o << "    const I" << k << "* in" << k << " = global_ptr<const I" << k << ">((u64)a.in[" << k << "]);\n";
    for (size_t k = 0; k < NO; ++k) o << "    O" << k << "* out" << k << " = global_ptr<O" << k << ">((u64)a.out[" << k << "]);\n";

    if (shape == Shape::Flat) {
        // One vector of VEC elements per operand per lane (16 bytes of T) and as many workgroups as
        // there are vectors: the hardware overlaps the groups' load and compute phases far better than
        // a long per-lane loop does (measured: 87 % of HBM peak for a 3-load / 1-store tanh+exp+div body).
        const char* rs = noAlias ? " __restrict__" : "";
        auto bc = [&](size_t k) { return ((broadcastMask >> k) & 1u) != 0; };
        for (size_t k = 0; k < NI; ++k) {
            if (bc(k)) o << "    const T b" << k << " = " << to_t(k, "in" + std::to_string(k) + "[0]") << ";\n";
            else o << "    const vec<I" << k << ", VEC>*" << rs << " p" << k << " = (const vec<I" << k << ", VEC>*)in" << k << ";\n";
        }
        for (size_t k = 0; k < NO; ++k) o << "    vec<O" << k << ", VEC>*" << rs << " q" << k << " = (vec<O" << k << ", VEC>*)out" << k << ";\n";
        wholeInit(o);
        o << "    const u64 nvec = a.n / VEC;\n"
          << "    for (u64 v = (u64)BID * " << kBlock << " + threadIdx.x; v < nvec; v += (u64)GDIM * " << kBlock << ") {\n";
        for (size_t k = 0; k < NI; ++k) if (!bc(k)) o << "        const vec<I" << k << ", VEC> r" << k << " = p" << k << "[v];\n";
        for (size_t k = 0; k < NO; ++k) o << "        vec<O" << k << ", VEC> w" << k << ";\n";
        if (NT) { o << "        TriPos tpos[" << NT << "];\n"; for (size_t j = 0; j < NT; ++j) o << "        tpos[" << j << "] = tri_origin(v * VEC, a.tp[" << 3 * j << "], a.tp[" << 3 * j + 1 << "]);\n"; }
        o << "#pragma unroll\n        for (int e = 0; e < VEC; ++e) {\n            T x[" << AI << "], y[" << NO << "];\n";
        for (size_t k = 0; k < NI; ++k) {
            if (bc(k)) o << "            x[" << k << "] = b" << k << ";\n";
            else o << "            x[" << k << "] = " << to_t(k, "r" + std::to_string(k) + ".v[e]") << ";\n";
        }
        if (NI == 0) o << "            x[0] = zero<T>();\n";
        o << "            aix_body(x, s, y" << (NT ? ", e, tpos, a.tp" : "") << ");\n";
        for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "            w" << k << ".v[e] = " << from_t(k, "y[" + std::to_string(k) + "]") << ";\n";
        wholeAdd(o, "            ");
        o << "        }\n";
        for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "        store_sel<AIX_NT>(q" << k << " + v, w" << k << ");\n";
        o << "    }\n"
          << "    const u64 done = nvec * VEC;\n"
          << "    if (BID == 0 && done + threadIdx.x < a.n) {\n        const u64 i = done + threadIdx.x;\n        T x[" << AI << "], y[" << NO << "];\n";
        if (NT) { o << "        TriPos tpos[" << NT << "];\n"; for (size_t j = 0; j < NT; ++j) o << "        tpos[" << j << "] = tri_origin(i, a.tp[" << 3 * j << "], a.tp[" << 3 * j + 1 << "]);\n"; }
        for (size_t k = 0; k < NI; ++k) {
            if (bc(k)) o << "        x[" << k << "] = b" << k << ";\n";
            else o << "        x[" << k << "] = " << to_t(k, "in" + std::to_string(k) + "[i]") << ";\n";
        }
        if (NI == 0) o << "        x[0] = zero<T>();\n";
        o << "        aix_body(x, s, y" << (NT ? ", 0, tpos, a.tp" : "") << ");\n";
        for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "        out" << k << "[i] = " << from_t(k, "y[" + std::to_string(k) + "]") << ";\n";
        wholeAdd(o, "        ");
        o << "    }\n";
        wholeLand(o);
        o << "}\n";
        return o.str();
    }

    if (shape == Shape::Rows) {
        wholeInit(o);
        o << "    const int inner = (int)a.rank - 1;\n"
          << "    const u64 total = a.n / VEC;\n"
          << "    for (u64 c = (u64)BID * " << kBlock << " + threadIdx.x; c < total; c += (u64)GDIM * " << kBlock << ") {\n"
          << "        u64 row = c / a.chunks;\n        const u64 col = (c - row * a.chunks) * VEC;\n"
          << "        u64 p[" << AI << "];\n";
        for (size_t k = 0; k < NI; ++k) o << "        p[" << k << "] = a.off[" << k << "];\n";
        o << "        for (int d = inner - 1; d >= 0; --d) {\n            const u64 q = row / a.shape[d], r = row - q * a.shape[d];\n";
        for (size_t k = 0; k < NI; ++k) o << "            p[" << k << "] += r * a.str[" << k << "][d];\n";
        o << "            row = q;\n        }\n";
        // all loads first and without branches (row_vec_ptr / row_vec_fix in the device header say why)
        for (size_t k = 0; k < NI; ++k)
            o << "        vec<I" << k << ", VEC> r" << k << " = *row_vec_ptr<I" << k << ", VEC>(in" << k << " + p[" << k << "], col, a.str[" << k << "][inner] == 0);\n";
        for (size_t k = 0; k < NI; ++k)
            o << "        r" << k << " = row_vec_fix<I" << k << ", VEC>(r" << k << ", in" << k << " + p[" << k << "], a.str[" << k << "][inner] == 0);\n";
        for (size_t k = 0; k < NO; ++k) o << "        vec<O" << k << ", VEC> w" << k << ";\n";
        if (NT) { o << "        TriPos tpos[" << NT << "];\n"; for (size_t j = 0; j < NT; ++j) o << "        tpos[" << j << "] = tri_origin(c * VEC, a.tp[" << 3 * j << "], a.tp[" << 3 * j + 1 << "]);\n"; }
        o << "#pragma unroll\n        for (int e = 0; e < VEC; ++e) {\n            T x[" << AI << "], y[" << NO << "];\n";
        for (size_t k = 0; k < NI; ++k) o << "            x[" << k << "] = " << to_t(k, "r" + std::to_string(k) + ".v[e]") << ";\n";
        if (NI == 0) o << "            x[0] = zero<T>();\n";
        o << "            aix_body(x, s, y" << (NT ? ", e, tpos, a.tp" : "") << ");\n";
        for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "            w" << k << ".v[e] = " << from_t(k, "y[" + std::to_string(k) + "]") << ";\n";
        wholeAdd(o, "            ");
        o << "        }\n";
        for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "        store_sel<AIX_NT>((vec<O" << k << ", VEC>*)(out" << k << " + c * VEC), w" << k << ");\n";
        o << "    }\n";
        wholeLand(o);
        o << "}\n";
        return o.str();
    }

    // gather
    wholeInit(o);
    o << "    for (u64 i = (u64)BID * " << kBlock << " + threadIdx.x; i < a.n; i += (u64)GDIM * " << kBlock << ") {\n"
      << "        u64 rest = i;\n        u64 p[" << AI << "];\n";
    if (NT) { o << "        TriPos tpos[" << NT << "];\n"; for (size_t j = 0; j < NT; ++j) o << "        tpos[" << j << "] = tri_origin(i, a.tp[" << 3 * j << "], a.tp[" << 3 * j + 1 << "]);\n"; }
    for (size_t k = 0; k < NI; ++k) o << "        p[" << k << "] = a.off[" << k << "];\n";
    o << "        for (int d = (int)a.rank - 1; d >= 0; --d) {\n            const u64 q = rest / a.shape[d], r = rest - q * a.shape[d];\n";
    for (size_t k = 0; k < NI; ++k) o << "            p[" << k << "] += r * a.str[" << k << "][d];\n";
    o << "            rest = q;\n        }\n        T x[" << AI << "], y[" << NO << "];\n";
    for (size_t k = 0; k < NI; ++k) o << "        x[" << k << "] = " << to_t(k, "in" + std::to_string(k) + "[p[" + std::to_string(k) + "]]") << ";\n";
    if (NI == 0) o << "        x[0] = zero<T>();\n";
    o << "        aix_body(x, s, y" << (NT ? ", 0, tpos, a.tp" : "") << ");\n";
    for (size_t k = 0; k < NO; ++k) if (!whole[k]) o << "        out" << k << "[i] = " << from_t(k, "y[" + std::to_string(k) + "]") << ";\n";
    wholeAdd(o, "        ");
    o << "    }\n";
    wholeLand(o);
    o << "}\n";
    return o.str();
}

// ---- row programs ------------------------------------------------------------------------------------------------------
bool rowGeometry(const FusedSubgraphDescriptor& d, RowGeometry* g)
{
    if (!d.rowLength || d.elementCount % d.rowLength) return false;
    const size_t vec = 16 / aix::Device::dataTypeSize(d.dtype);
    if (d.rowLength % vec) return false;
    g->lanes = d.rowLength >= 2048 ? 256 : 64;                     // the stand-alone reduction's choice (reduce.hip), for identical sums
    const size_t nvec = d.rowLength / vec;
    g->vectors = (int)((nvec + (size_t)g->lanes - 1) / (size_t)g->lanes);
    return g->vectors >= 1 && g->vectors <= 8;
}

namespace {

char kindLetter(fuse::RowOperand k)
{
    switch (k) {
        case fuse::RowOperand::Dense: return 'd';
        case fuse::RowOperand::PerRowBroadcast: return 'b';
        case fuse::RowOperand::RowVector: return 'r';
        case fuse::RowOperand::PerRow: return 'p';
        case fuse::RowOperand::Single: return 's';
        default: return '?';
    }
}

fuse::RowOperand inputKind(const FusedSubgraphDescriptor& d, size_t k)
{
    const fuse::RowOperand kind = fuse::rowOperandKind(d.inputBuffers[k], d.elementCount / d.rowLength, d.rowLength);
    if (kind == fuse::RowOperand::None) throw std::invalid_argument("row program: an operand that is neither rows, nor one value per row, nor one row");
    return kind;
}

} // namespace

void rowSignatureInto(std::string& s, const FusedSubgraphDescriptor& d, const RowGeometry& g, bool streamOut)
{
    s.clear();
    s += shortType(d.dtype);
    s += "|row"; appendNumber(s, (uint64_t)g.lanes); s += 'x'; appendNumber(s, (uint64_t)g.vectors);
    if (streamOut) s += "|nt";
    s += "|i"; appendNumber(s, d.inputBuffers.size());
    s += 'o';  appendNumber(s, d.outputBuffers.size());
    s += 's';  appendNumber(s, scalarCount(d));
    s += '|';
    for (size_t k = 0; k < d.inputBuffers.size(); ++k) s += kindLetter(inputKind(d, k));
    for (size_t k = 0; k < d.inputBuffers.size(); ++k)
        if (d.inputBuffers[k].dtype != d.dtype) { s += "|x"; appendNumber(s, k); s += ':'; s += shortType(d.inputBuffers[k].dtype); }
    for (size_t k = 0; k < d.outputBuffers.size(); ++k)
        if (d.outputBuffers[k].dtype != d.dtype) { s += "|y"; appendNumber(s, k); s += ':'; s += shortType(d.outputBuffers[k].dtype); }
    for (const auto& op : d.ops) {
        s += '|'; s += fuse::opName(op.type); if (op.perRow) s += '\''; s += '(';
        appendOperand(s, d, op.inputIndex0, op.scalarIndex0);
        if (isBinary(op.type) || fuse::isRowReduce(op.type)) { s += ','; appendOperand(s, d, op.inputIndex1, op.scalarIndex1); }
        s += ')';
        if (op.outputIndex != SIZE_MAX) { s += ">o"; appendNumber(s, op.outputIndex); }
    }
}

std::string rowSource(const FusedSubgraphDescriptor& d, const RowGeometry& g, bool streamOut, bool many)
{
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size(), NS = scalarCount(d);
    if (NO == 0) throw std::invalid_argument("fused kernel without outputs");
    const size_t NT = triCount(d);
    if (d.opParams.size() != 3 * NT) throw std::invalid_argument("fused kernel: tril / triu without its parameters");
    const size_t esz = aix::Device::dataTypeSize(d.dtype);
    const size_t AI = NI ? NI : 1, AS = NS ? NS : 1;
    std::vector<fuse::RowOperand> kinds(NI);
    for (size_t k = 0; k < NI; ++k) kinds[k] = inputKind(d, k);
    std::string sig;
    rowSignatureInto(sig, d, g, streamOut);
    std::ostringstream o;
    o << "#include \"aix_device.h\"\nusing namespace aixd;\n// " << sig << "\n"
      << "#define AIX_NT " << (streamOut ? "true" : "false") << "\n"
      << "typedef " << typeName(d.dtype) << " T;\ntypedef traits<T>::W W;\ntypedef " << wordName(esz) << " word_t;\n"
      << "#define VEC (vec16<T>::n)\n#define NV " << g.vectors << "\n#define G " << g.lanes << "\n";
    for (size_t k = 0; k < NI; ++k) o << "typedef " << typeName(d.inputBuffers[k].dtype) << " I" << k << ";\n";
    for (size_t k = 0; k < NO; ++k) o << "typedef " << typeName(d.outputBuffers[k].dtype) << " O" << k << ";\n";
    auto to_t = [&](size_t k, const std::string& e) { return d.inputBuffers[k].dtype == d.dtype ? e : "convert<I" + std::to_string(k) + ", T>(" + e + ")"; };
    auto from_t = [&](size_t k, const std::string& e) { return d.outputBuffers[k].dtype == d.dtype ? e : "convert<T, O" + std::to_string(k) + ">(" + e + ")"; };
    o << "struct Args {\n    const void* in[" << AI << "];\n    void* out[" << NO << "];\n    u64 sc[" << AS << "];\n    u64 per[" << AI << "];\n";
    if (NT) o << "    u64 tp[" << 3 * NT << "];\n";
    o << "    u64 rows;\n    u64 len;\n};\n\n";
    if (many) {
        o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << rowEntryName(d, g) << "_many(const Args* table, const u32* starts, u32 count)\n{\n"
          << "    u32 lo = 0, hi = count;\n"
          << "    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (starts[mid] <= blockIdx.x) lo = mid; else hi = mid; }\n"
          << "    const Args a = table[lo];\n"
          << "    const u32 BID = blockIdx.x - starts[lo], GDIM = starts[lo + 1] - starts[lo];\n";
    } else {
        o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << rowEntryName(d, g) << "(Args a)\n{\n"
          << "    const u32 BID = blockIdx.x, GDIM = gridDim.x;\n";
    }
    bool anyOnehot = false;
    for (const auto& op : d.ops) if (op.type == OpType::ArgmaxIndicesTo) anyOnehot = true;
    if (anyOnehot) o << "    __shared__ u32 redi[8];\n    (void)redi;\n";
    o << "    __shared__ W red[4];\n    (void)red;\n"
      << "    T s[" << AS << "];\n";
    for (size_t k = 0; k < NS; ++k) o << "    s[" << k << "] = __builtin_bit_cast(T, (word_t)a.sc[" << k << "]);\n";
    if (NS == 0) o << "    s[0] = zero<T>();\n";
    for (size_t k = 0; k < NI; ++k) o << "    const I" << k << "* in" << k << " = global_ptr<const I" << k << ">((u64)a.in[" << k << "]);\n";
    for (size_t k = 0; k < NO; ++k) o << "    O" << k << "* out" << k << " = global_ptr<O" << k << ">((u64)a.out[" << k << "]);\n";
    o << "    const u32 lane = threadIdx.x % G;\n"
      << "    const u64 nvec = a.len / VEC;\n"
      << "    const W lowestW = (W)(-__builtin_huge_val());\n    (void)lowestW;\n";
    if (g.lanes == 64) o << "    for (u64 row = (u64)BID * " << kBlock / 64 << " + threadIdx.x / 64; row < a.rows; row += (u64)GDIM * " << kBlock / 64 << ") {\n";
    else o << "    for (u64 row = BID; row < a.rows; row += GDIM) {\n";
    // operands: whole rows (their own or the one shared row) as vectors, per-row values as scalars
    for (size_t k = 0; k < NI; ++k) {
        if (kinds[k] == fuse::RowOperand::Dense || kinds[k] == fuse::RowOperand::RowVector) {
            // (a block of rows that comes round again: row % period, period 1 for the one row all rows share)
            const std::string base = kinds[k] == fuse::RowOperand::Dense ? " + row * a.len" : " + (row % a.per[" + std::to_string(k) + "]) * a.len";
            o << "        T x" << k << "[NV][VEC];\n#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n"
              << "            const u64 v = lane + (u64)j * G;\n"
              << "            vec<I" << k << ", VEC> r;\n#pragma unroll\n            for (int e = 0; e < VEC; ++e) r.v[e] = zero<I" << k << ">();\n"
              << "            if (v < nvec) r = ((const vec<I" << k << ", VEC>*)(in" << k << base << "))[v];\n"
              << "#pragma unroll\n            for (int e = 0; e < VEC; ++e) x" << k << "[j][e] = " << to_t(k, "r.v[e]") << ";\n        }\n";
        } else if (kinds[k] == fuse::RowOperand::Single) {
            o << "        const T q" << k << " = " << to_t(k, "in" + std::to_string(k) + "[0]") << ";\n";
        } else {
            o << "        const T q" << k << " = " << to_t(k, "in" + std::to_string(k) + "[row]") << ";\n";
        }
    }
    auto fullOperand = [&](size_t tensorIndex, size_t scalarIndex) -> std::string {
        if (tensorIndex != SIZE_MAX) {
            if (tensorIndex < NI) {
                if (kinds[tensorIndex] == fuse::RowOperand::PerRowBroadcast || kinds[tensorIndex] == fuse::RowOperand::Single) return "q" + std::to_string(tensorIndex);
                if (kinds[tensorIndex] == fuse::RowOperand::PerRow) throw std::invalid_argument("row program: a per-row operand of an operator on whole rows");
                return "x" + std::to_string(tensorIndex) + "[j][e]";
            }
            const size_t m = tensorIndex - NI;
            return d.ops[m].perRow ? "p" + std::to_string(m) : "v" + std::to_string(m) + "[j][e]";
        }
        if (scalarIndex != SIZE_MAX) return "s[" + std::to_string(scalarIndex) + "]";
        throw std::invalid_argument("fused operator without an operand");
    };
    auto rowOperand = [&](size_t tensorIndex, size_t scalarIndex) -> std::string {
        if (tensorIndex != SIZE_MAX) {
            if (tensorIndex < NI) {
                if (kinds[tensorIndex] != fuse::RowOperand::PerRow && kinds[tensorIndex] != fuse::RowOperand::Single) throw std::invalid_argument("row program: a row operand of an operator on per-row values");
                return "q" + std::to_string(tensorIndex);
            }
            const size_t m = tensorIndex - NI;
            if (!d.ops[m].perRow) throw std::invalid_argument("row program: a row value used by an operator on per-row values");
            return "p" + std::to_string(m);
        }
        if (scalarIndex != SIZE_MAX) return "s[" + std::to_string(scalarIndex) + "]";
        throw std::invalid_argument("fused operator without an operand");
    };
    for (size_t k = 0; k < d.ops.size(); ++k) {
        const auto& op = d.ops[k];
        if (fuse::isRowReduce(op.type)) {
            const bool sum = op.type == OpType::ReduceTo;
            const std::string init = "s[" + std::to_string(op.scalarIndex1) + "]";
            o << "        W a" << k << " = " << (sum ? "(W)0" : "lowestW") << ";\n#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n"
              << "            if (lane + (u64)j * G < nvec) {\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) { const W w = up(" << fullOperand(op.inputIndex0, op.scalarIndex0) << "); ";
            if (sum) o << "a" << k << " += w; }\n"; else o << "if (w > a" << k << ") a" << k << " = w; }\n";
            o << "            }\n        }\n"
              << "        a" << k << " = " << (sum ? "row_sum" : "row_max") << "<G>(a" << k << ", red);\n";
            // combined with the value the destination was initialised with, as the stand-alone kernels land their results
            if (sum) o << "        const T p" << k << " = down<T>(up(" << init << ") + a" << k << ");\n";
            else o << "        const T p" << k << " = a" << k << " > up(" << init << ") ? down<T>(a" << k << ") : " << init << ";\n";
            if (op.outputIndex != SIZE_MAX) o << "        if (lane == 0) out" << op.outputIndex << "[row] = " << from_t(op.outputIndex, "p" + std::to_string(k)) << ";\n";
            continue;
        }
        if (op.perRow) {
            o << "        const T p" << k << " = ";
            if (op.type == OpType::Cast) o << rowOperand(op.inputIndex0, op.scalarIndex0);
            else {
                o << fnName(op.type) << "(" << rowOperand(op.inputIndex0, op.scalarIndex0);
                if (isBinary(op.type)) o << ", " << rowOperand(op.inputIndex1, op.scalarIndex1);
                o << ")";
            }
            o << ";\n";
            if (op.outputIndex != SIZE_MAX) o << "        if (lane == 0) out" << op.outputIndex << "[row] = " << from_t(op.outputIndex, "p" + std::to_string(k)) << ";\n";
            continue;
        }
        if (op.type == OpType::ArgmaxIndicesTo) {
            // 1 at the row's first maximum, 0 elsewhere (values of T; a store converts them).  Every lane scans its own
            // elements by growing column, so a strict '>' keeps the first of equal values; NaNs are no candidates, but a
            // NaN in column 0 wins outright (it stands in as +infinity at the smallest column), as the stand-alone operator has it.
            const std::string x = fullOperand(op.inputIndex0, op.scalarIndex0);
            o << "        T v" << k << "[NV][VEC];\n        {\n            W bv = lowestW; u32 bi = 0xffffffffu; bool ok = false;\n"
              << "#pragma unroll\n            for (int j = 0; j < NV; ++j) {\n                if (lane + (u64)j * G < nvec) {\n#pragma unroll\n                    for (int e = 0; e < VEC; ++e) {\n"
              << "                        W w = up(" << x << ");\n                        const u32 c = (u32)((lane + (u64)j * G) * VEC + e);\n"
              << "                        if (c == 0 && w != w) w = (W)__builtin_huge_val();\n"
              << "                        if (w == w && (!ok || w > bv)) { bv = w; bi = c; ok = true; }\n"
              << "                    }\n                }\n            }\n"
              << "            const u32 win = row_first_max<G>(bv, bi, ok, red, " << "redi);\n"
              << "            const T one = down<T>((W)1);\n"
              << "#pragma unroll\n            for (int j = 0; j < NV; ++j) {\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) v" << k << "[j][e] = (u32)((lane + (u64)j * G) * VEC + e) == win ? one : zero<T>();\n            }\n        }\n";
            if (op.outputIndex != SIZE_MAX) {
                const size_t qo = op.outputIndex;
                o << "#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n            const u64 v = lane + (u64)j * G;\n            if (v < nvec) {\n"
                  << "                vec<O" << qo << ", VEC> w;\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) w.v[e] = " << from_t(qo, "v" + std::to_string(k) + "[j][e]") << ";\n"
                  << "                store_sel<AIX_NT>((vec<O" << qo << ", VEC>*)(out" << qo << " + row * a.len) + v, w);\n            }\n        }\n";
            }
            continue;
        }
        if (isTri(op.type)) {
            // the row of the program is a row of the matrix: its number within the matrix, the element's column, the diagonal
            const size_t q = 3 * op.paramIndex;
            o << "        T v" << k << "[NV][VEC];\n        {\n            const i64 r = (i64)(row % a.tp[" << q << "]) + (i64)a.tp[" << q + 2 << "];\n"
              << "#pragma unroll\n            for (int j = 0; j < NV; ++j) {\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) {\n"
              << "                    const i64 c = (i64)((lane + (u64)j * G) * VEC + e);\n"
              << "                    v" << k << "[j][e] = (" << (op.type == OpType::Triu ? "c >= r" : "c <= r") << ") ? " << fullOperand(op.inputIndex0, op.scalarIndex0) << " : zero<T>();\n"
              << "                }\n            }\n        }\n";
            if (op.outputIndex != SIZE_MAX) {
                const size_t qo = op.outputIndex;
                o << "#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n            const u64 v = lane + (u64)j * G;\n            if (v < nvec) {\n"
                  << "                vec<O" << qo << ", VEC> w;\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) w.v[e] = " << from_t(qo, "v" + std::to_string(k) + "[j][e]") << ";\n"
                  << "                store_sel<AIX_NT>((vec<O" << qo << ", VEC>*)(out" << qo << " + row * a.len) + v, w);\n            }\n        }\n";
            }
            continue;
        }
        o << "        T v" << k << "[NV][VEC];\n#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n#pragma unroll\n            for (int e = 0; e < VEC; ++e) v" << k << "[j][e] = ";
        if (op.type == OpType::Cast) o << fullOperand(op.inputIndex0, op.scalarIndex0);
        else {
            o << fnName(op.type) << "(" << fullOperand(op.inputIndex0, op.scalarIndex0);
            if (isBinary(op.type)) o << ", " << fullOperand(op.inputIndex1, op.scalarIndex1);
            o << ")";
        }
        o << ";\n        }\n";
        if (op.outputIndex != SIZE_MAX) {
            const size_t q = op.outputIndex;
            o << "#pragma unroll\n        for (int j = 0; j < NV; ++j) {\n            const u64 v = lane + (u64)j * G;\n            if (v < nvec) {\n"
              << "                vec<O" << q << ", VEC> w;\n#pragma unroll\n                for (int e = 0; e < VEC; ++e) w.v[e] = " << from_t(q, "v" + std::to_string(k) + "[j][e]") << ";\n"
              << "                store_sel<AIX_NT>((vec<O" << q << ", VEC>*)(out" << q << " + row * a.len) + v, w);\n            }\n        }\n";
        }
    }
    o << "    }\n}\n";
    return o.str();
}

void packRowArgsInto(std::vector<uint64_t>& a, const FusedSubgraphDescriptor& d, const void* const* inputs, void* const* outputs)
{
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size(), NS = scalarCount(d);
    const size_t AI = NI ? NI : 1, AS = NS ? NS : 1;
    const size_t esz = aix::Device::dataTypeSize(d.dtype);
    a.clear();
    for (size_t k = 0; k < AI; ++k) a.push_back(k < NI ? (uint64_t)(uintptr_t)inputs[k] : 0);
    for (size_t k = 0; k < NO; ++k) a.push_back((uint64_t)(uintptr_t)outputs[k]);
    for (size_t k = 0; k < AS; ++k) {
        uint64_t bits = 0;
        if (k < NS) std::memcpy(&bits, d.scalarData.data() + k * esz, esz);
        a.push_back(bits);
    }
    const size_t rows = d.elementCount / d.rowLength;
    for (size_t k = 0; k < AI; ++k) {
        const size_t period = k < NI ? fuse::rowOperandPeriod(d.inputBuffers[k], rows, d.rowLength) : 0;
        a.push_back(period ? period : 1);
    }
    for (uint64_t v : d.opParams) a.push_back(v);
    a.push_back(rows);
    a.push_back(d.rowLength);
}

void packArgsInto(std::vector<uint64_t>& a, const FusedSubgraphDescriptor& d, Shape shape, const void* const* inputs,
                  void* const* outputs, uint64_t n, const Space* space, uint64_t chunksPerRow)
{
    const size_t NI = d.inputBuffers.size(), NO = d.outputBuffers.size(), NS = scalarCount(d);
    const size_t AI = NI ? NI : 1, AS = NS ? NS : 1;
    const size_t esz = aix::Device::dataTypeSize(d.dtype);
    a.clear();
    for (size_t k = 0; k < AI; ++k) a.push_back(k < NI ? (uint64_t)(uintptr_t)inputs[k] : 0);
    for (size_t k = 0; k < NO; ++k) a.push_back((uint64_t)(uintptr_t)outputs[k]);
    for (size_t k = 0; k < AS; ++k) {
        uint64_t bits = 0;
        if (k < NS) std::memcpy(&bits, d.scalarData.data() + k * esz, esz);     // little endian: low bytes
        a.push_back(bits);
    }
    for (uint64_t v : d.opParams) a.push_back(v);
    a.push_back(n);
    if (shape == Shape::Flat) return;
    if (!space) throw std::invalid_argument("strided fused kernel without an iteration space");
    a.push_back(chunksPerRow);
    a.push_back(space->rank);
    for (int dd = 0; dd < kMaxDims; ++dd) a.push_back(space->shape[dd]);
    for (size_t k = 0; k < AI; ++k) a.push_back(k < NI ? space->offset[k] : 0);
    for (size_t k = 0; k < AI; ++k)
        for (int dd = 0; dd < kMaxDims; ++dd) a.push_back(k < NI ? space->stride[k][dd] : 0);
}

std::vector<uint64_t> packArgs(const FusedSubgraphDescriptor& d, Shape shape, const std::vector<const void*>& inputs,
                               const std::vector<void*>& outputs, uint64_t n, const Space* space, uint64_t chunksPerRow)
{
    std::vector<uint64_t> a;
    packArgsInto(a, d, shape, inputs.data(), outputs.data(), n, space, chunksPerRow);
    return a;
}

} // namespace aixhip::gen
