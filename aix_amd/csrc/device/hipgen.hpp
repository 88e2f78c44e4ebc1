// hipgen.hpp -- turns a fused-subgraph descriptor into HIP C++ source for hipRTC.
//
// Replaces the reference's runtime Metal-source generator
// (Targets/AIXLib/aixDeviceMetalKernelGen.cpp:464-710): same input (a FusedSubgraphDescriptor),
// same idea (one SSA statement per operator, external inputs loaded once, immediates as kernel
// arguments so their VALUES never force a recompile), but the emitted text is HIP for gfx950
// built on the per-element operators of aix_device.h, in one of three launch shapes:
//   flat    every view dense and 16-byte aligned: 16-byte loads/stores, several in flight;
//   rows    the innermost dim is dense-or-broadcast for every view: one 16-byte chunk per lane;
//   gather  any strided view: one element per lane.
#pragma once

#include "fuse.hpp"

#include <array>
#include <string>
#include <vector>

namespace aixhip::gen {

enum class Shape { Flat, Rows, Gather };

// Identity of a generated kernel: element type, launch shape, operator wiring.  Immediates'
// values, pointers, sizes and strides are arguments and not part of it.
// For the flat shape two more facts are compiled in: which inputs are a single broadcast element
// (bit k of broadcastMask), and whether no output aliases an input (the pointers may then be
// declared __restrict__).  streamOut (flat and rows shapes): the results leave through non-temporal stores -- large results
// that nothing reads back from cache.
std::string signature(const fuse::FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask = 0, bool noAlias = true, bool streamOut = false);
// The same text written into `out` (cleared first; its capacity is reused from call to call).
void signatureInto(std::string& out, const fuse::FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask, bool noAlias, bool streamOut = false);

// Source of `extern "C" __global__ void <entryName>(Args)`.  many: of
// `<entryName>_many(const Args* table, const u32* starts, u32 count)` instead -- the same body for `count` argument
// blocks in one launch, workgroups [starts[k], starts[k + 1]) working on table[k] (Adam's update of every parameter,
// the per-parameter casts of a mixed-precision step, one operator applied head by head).
std::string source(const fuse::FusedSubgraphDescriptor& d, Shape shape, uint32_t broadcastMask = 0, bool noAlias = true, bool streamOut = false,
                   bool many = false);

// ---- row programs (descriptor.rowLength > 0) ------------------------------------------------------------------------
// A kernel that works row by row on [rows, rowLength] data: a wave (rows shorter than 2048 elements) or a workgroup per
// row, the row's vectors in registers, sums / maxima over the row by shuffles (and LDS across the four waves) in the
// order of the stand-alone reduction kernels, so that fused and unfused results are the same bits.
struct RowGeometry {
    int lanes{64};          // lanes per row: 64 or 256
    int vectors{1};         // 16-byte vectors per lane and row (compile-time; the tail of a row is masked)
};
// false: the descriptor cannot run as a row program (row too long, not a whole number of vectors)
bool rowGeometry(const fuse::FusedSubgraphDescriptor& d, RowGeometry* g);
void rowSignatureInto(std::string& out, const fuse::FusedSubgraphDescriptor& d, const RowGeometry& g, bool streamOut);
std::string rowSource(const fuse::FusedSubgraphDescriptor& d, const RowGeometry& g, bool streamOut, bool many = false);     // (many: as for source())
// Args of a row program: in[], out[], immediates, per input the period of its block of rows (1 where it has none), the
// (rows, cols, diagonal) of every tril / triu, rows, rowLength
void packRowArgsInto(std::vector<uint64_t>& a, const fuse::FusedSubgraphDescriptor& d, const void* const* inputs, void* const* outputs);

// The kernel's symbol: "aix_fused_<type>_<launch shape>_<operators in order>" (what a profiler's trace shows), at most
// 120 characters.
std::string entryName(const fuse::FusedSubgraphDescriptor& d, Shape shape);
std::string rowEntryName(const fuse::FusedSubgraphDescriptor& d, const RowGeometry& g);

constexpr int kMaxDims = 8;
constexpr int kBlock = 256;

// The iteration space handed to rows / gather kernels.
struct Space {
    uint32_t rank{0};
    uint64_t shape[kMaxDims]{};
    std::vector<uint64_t> offset;                 // per buffer (inputs then outputs)
    std::vector<std::array<uint64_t, kMaxDims>> stride;
};

// Kernel-argument block in the exact layout of the generated `struct Args`.
std::vector<uint64_t> packArgs(const fuse::FusedSubgraphDescriptor& d, Shape shape, const std::vector<const void*>& inputs,
                               const std::vector<void*>& outputs, uint64_t n, const Space* space,
                               uint64_t chunksPerRow);
// The same into `a` (cleared first); inputs / outputs hold one pointer per descriptor buffer.
void packArgsInto(std::vector<uint64_t>& a, const fuse::FusedSubgraphDescriptor& d, Shape shape, const void* const* inputs,
                  void* const* outputs, uint64_t n, const Space* space, uint64_t chunksPerRow);

} // namespace aixhip::gen
