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

// A kernel whose body is a sequence of loop nests (e.g. a row maximum followed by the subtraction that
// consumes it) has one phase per top-level nest.  By default the phases run inside one launch of one workgroup,
// separated by workgroup barriers (GenericKernel::cooperative).  With ILANG_HIP_PHASES=1 every phase is a launch
// of its own with its own work-item space, the stream order being the grid-wide dependency between them; that
// form is confined to the CPU emulation of the runtime.
//
// A nest whose parallel loops enclose reduction loops (a row sum: `for i { s[i] = 0; for j { s[i] += x[i][j] } }`)
// is also printed in a second form, <name>_w, in which one wavefront stands where a work-item stood: the
// reduction loops are dealt out over its 64 lanes (lane l takes iterations l, l + 64, ...), every lane
// accumulates its share in a register, the shares are combined with a butterfly of lane exchanges, and everything
// outside those loops is computed by all 64 lanes alike (same values, same stores).  Consecutive iterations of
// the reduction loop are then read by consecutive lanes.  The launcher picks the form by the extents of the run.
struct WaveLoop {
  size_t loop = 0;    // a loop of the parallel body: its accumulators are lane shares, combined after it
  size_t spread = 0;  // the loop whose iterations are dealt out over the lanes: `loop`, or one nested perfectly in it
  std::vector<std::pair<size_t, ic::Op>> accumulators;  // (writeable, its reduction); empty: an elementwise loop
};
struct GenericPhase {
  std::string name;                       // f<k> for a single-phase kernel, f<k>_p<i> otherwise
  std::vector<size_t> parallel_loops;     // loop ids, outermost first (empty: one work-item)
  std::vector<ic::Extent<ic::Param>> parallel_extents;
  std::vector<PrivateBuffer> privates;    // only buffers that no other phase touches
  // the wavefront-per-iteration form (<name>_w), when the nest has one
  std::vector<WaveLoop> wave_loops;
  ic::Extent<ic::Param> wave_extent;      // extent of the first loop spread over the lanes that reduces
  bool wave_contiguous = false;           // consecutive iterations of those loops read consecutive elements
  static constexpr unsigned kWaveThreads = 256;  // work-items per workgroup of that form (4 wavefronts)
};

struct GenericKernel {
  std::string name;                       // f<k>; empty when not emitted
  size_t n_reads = 0, n_writes = 0;
  std::vector<GenericPhase> phases;
  // A kernel whose body is a sequence of loop nests, some of them parallel: ONE launch of one workgroup of
  // kCooperativeThreads work-items, every nest spread over them, workgroup barriers between the nests (the phases
  // then describe the nests of that one launch, not launches of their own).
  bool cooperative = false;
  static constexpr unsigned kCooperativeThreads = 1024;
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

// `emit[k]` selects the kernels to print.
GenericModule emit_generic_hip(const ic::ExecPlan& plan, const ic::Module& module, const std::vector<bool>& emit);

}  // namespace ihipc
