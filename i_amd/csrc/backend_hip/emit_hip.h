// Generic HIP lowering: any kernel of an exec plan that has no hand-written
// counterpart is printed as a gfx950 `extern "C" __global__` function.
//
// The loop nest and scalar semantics come from the statement IR (ic::Module),
// exactly what the C backend prints; what is added here is the mapping to the
// GPU: independent loops on the kernel's outer spine become the work-item
// index space (tile loops -> workgroups, element loops -> lanes, flattened into
// one grid-stride index), reduction loops stay sequential inside a work-item
// (with their accumulators in registers) or, in the second form of a nest, are
// spread over the lanes of a wavefront (WaveLoop below),
// and intermediates that fusion folded below a parallel loop become
// work-item-private storage (registers / scratch when their size is static,
// a per-work-item slice of a device buffer otherwise).
#pragma once
#include <string>
#include <vector>

#include "../compiler/ir.h"

namespace ihipc {

struct PrivateBuffer {
  size_t writeable = 0;   // index into the kernel's writeables
  bool is_static = false;
  size_t static_size = 0; // elements, when static
};

// Every generated kernel is one loop nest: split_nests() below cuts a kernel whose body is a sequence of nests
// (a column sum followed by the division that consumes it) into one kernel per nest before anything is printed,
// the vectors they share being ordinary intermediates of the plan and the stream order the dependency between them.
//
// A nest whose parallel loops enclose reduction loops (a row sum: `for i { s[i] = 0; for j { s[i] += x[i][j] } }`)
// is also printed in a second form, <name>_w, in which one wavefront stands where a work-item stood: the
// reduction loops are dealt out over its 64 lanes (lane l takes iterations l, l + 64, ...), every lane
// accumulates its share in a register, the shares are combined with a butterfly of lane exchanges, and everything
// outside those loops is computed by all 64 lanes alike (same values, same stores).  Consecutive iterations of
// the reduction loop are then read by consecutive lanes.  The launcher picks the form by the extents of the run.
//
// A nest that does nothing but accumulate (sums, products, maxima, minima) under its outermost sequential loop
// has a third form, <name>_g (and <name>_gw, the wavefront form of the same), for runs whose parallel loops alone
// cannot fill the chip (a sum to a single element, a column sum of a few thousand columns): the iterations of
// that loop are dealt out over `parts` groups of work-items, part p taking a contiguous share of them; every
// part accumulates into a copy of its own of each accumulated buffer (a temporary that the launcher fills with
// the reduction's identity first), and a second kernel, ilang_combine, folds the copies into the buffer in part
// order.  (GridForm below.)
struct WaveLoop {
  size_t loop = 0;    // a loop of the parallel body: its accumulators are lane shares, combined after it
  size_t spread = 0;  // the loop whose iterations are dealt out over the lanes: `loop`, or one nested perfectly in it
  std::vector<std::pair<size_t, ic::Op>> accumulators;  // (writeable, its reduction); empty: an elementwise loop
};
// The form with a reduction loop in parts over groups of work-items.
struct GridAccumulator {
  size_t writeable = 0;   // index into the kernel's writeables
  ic::Op op = ic::Op::Add;
  bool init_here = false; // the nest initialises the buffer itself: the combined parts replace its contents
};
struct GridForm {
  bool available = false;
  size_t loop = 0;                      // the loop whose iterations are dealt out over the parts
  ic::Extent<ic::Param> extent;         // its extent
  std::vector<GridAccumulator> accumulators;
  bool wave = false;                    // <name>_gw exists too
  bool loop_is_spread = false;          // ... and in it the same loop also runs over the lanes
  bool held_accumulators = false;       // every accumulated element lives in a register across the loop: the parts only
                                        // store into their copies, which therefore need not start as the identity
};
struct GenericPhase {
  std::string name;                       // f<k>
  std::vector<size_t> parallel_loops;     // loop ids, outermost first (empty: one work-item)
  std::vector<ic::Extent<ic::Param>> parallel_extents;
  std::vector<PrivateBuffer> privates;    // only buffers that no other phase touches
  // the wavefront-per-iteration form (<name>_w), when the nest has one
  std::vector<WaveLoop> wave_loops;
  ic::Extent<ic::Param> wave_extent;      // extent of the first loop spread over the lanes that reduces
  bool wave_contiguous = false;           // consecutive iterations of those loops read consecutive elements
  static constexpr unsigned kWaveThreads = 256;  // work-items per workgroup of that form (4 wavefronts)
  GridForm grid;
};

struct GenericKernel {
  std::string name;                       // f<k>; empty when not emitted
  size_t n_reads = 0, n_writes = 0;
  std::vector<GenericPhase> phases;       // exactly one: the kernel's loop nest
  bool is_private(size_t writeable) const {
    for (const GenericPhase& ph : phases)
      for (const PrivateBuffer& pb : ph.privates)
        if (pb.writeable == writeable) return true;
    return false;
  }
};

struct GenericModule {
  std::string source;                // full HIP translation unit ("" when no kernel needs it)
  size_t rank = 1;                   // R of the View structs in the kernel argument block
  std::vector<GenericKernel> kernels;  // one entry per plan kernel; name empty when not emitted
};

// The plan with every kernel whose body is a sequence of loop nests cut into one kernel per nest (each with the
// buffers its own nest touches, in the order of the original's lists; initialisations of scalars stay with the
// nest that accumulates into them).  origin[k'] is the kernel of `plan` that kernel k' of the result came from.
// The C that the reference emits keeps such a kernel whole (it runs on one core either way); on the GPU every
// nest wants a grid of its own.
ic::ExecPlan split_nests(const ic::ExecPlan& plan, std::vector<size_t>* origin);

// Names of the helper kernels that every module with a GridForm carries: filling a temporary with a reduction's
// identity; folding the parts' copies into the accumulated buffer, with a work-item per element (many elements) or a
// wavefront per element whose lanes run over the parts (few elements, many parts).
constexpr const char* kFillKernel = "ilang_fill";
constexpr const char* kCombineKernel = "ilang_combine";
constexpr const char* kCombineWaveKernel = "ilang_combine_w";

// `emit[k]` selects the kernels to print.  `plan` is one that split_nests has produced.
GenericModule emit_generic_hip(const ic::ExecPlan& plan, const ic::Module& module, const std::vector<bool>& emit);

}  // namespace ihipc
