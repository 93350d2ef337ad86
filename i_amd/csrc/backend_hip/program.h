// A compiled 𝚒 program for the gfx950 backend: the lowered component, the
// per-kernel choice between a hand-written kernel and a generated one, the
// generated code object, and the executor that walks the exec plan
// (alloc intermediates -> dispatch kernels in order -> free), the device-side
// counterpart of the `exec` function the reference's C backend emits
// (ilang-python/annotated-flashattn.c:312-422).
#pragma once
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../compiler/ir.h"
#include "../runtime/kernel_launch.h"
#include "emit_hip.h"
#include "recognize.h"

namespace ihipc {

enum class DType { F32 = 0, BF16 = 1 };

struct DeviceTensor {
  void* data = nullptr;
  std::vector<size_t> shape;
  DType dtype = DType::F32;
};

struct Program {
  ic::Lowered low;
  ic::Module module;
  std::vector<Recognized> recognized;  // per plan kernel
  // Groups of (input, dimension) pairs that one index symbol ties together, directly or through intermediate
  // results: their extents must agree, or some kernel would index an operand out of bounds.
  std::vector<std::vector<std::pair<size_t, size_t>>> same_extent;
  // Whether the program can be run on its leading index in slices (row_slices_of); sliced[i]: input i is cut along
  // its first dimension with the outputs, the other inputs are needed whole by every slice.
  bool row_sliceable = false;
  std::vector<char> row_sliced;
  // The generated form of the plan: every kernel cut into one kernel per loop nest (split_nests), the statement IR
  // of those, and for each kernel of low.plan the kernels of nest_plan that stand for it, in order.
  ic::ExecPlan nest_plan;
  std::vector<std::vector<size_t>> nests_of;
  GenericModule generic;               // source for every kernel of nest_plan (hand-written ones keep a generated twin)
  std::vector<char> image;             // built lazily unless some kernel can only run generated
  bool image_built = false;
  std::mutex mu;
  std::map<int, hipModule_t> modules;  // per device
  // what set_option / set_clock_probe have stored (kernel choices that the caller takes from the launchers, and where
  // the attention kernels count their clocks); guarded by mu, copied by every execute() when it starts
  ihip::KernelOptions options;
  // what the last execute() dispatched: one line per kernel, "f<k>: <kernel name> (tile ...)"; guarded by mu
  std::string last_report;

  ~Program();
};

// Lower, recognise, emit; builds the generated code object right away when a
// kernel has no hand-written form.  Throws ic::CompileError / returns error text.
std::string compile_program(const ic::Component& component, Program** out);

// Human-readable backend source: the kernel plan followed by the generated HIP.
std::string program_code(const ic::Component& component);

size_t output_count(const Program& p);
std::vector<size_t> output_ranks(const Program& p);
// "" on success
std::string output_shapes(const Program& p, const std::vector<std::vector<size_t>>& input_shapes,
                          std::vector<std::vector<size_t>>* shapes);
size_t input_count(const Program& p);
size_t input_rank(const Program& p, size_t input);
// Whether every output's first dimension is an index that the program only ever maps over: one that stands for the
// first dimension of some inputs (`sliced`, one flag per input) and for no other dimension of any input, that no
// expression sums (or otherwise reduces) over, and that no expression uses twice under different names.  Rows
// r0 .. r1 of the outputs are then what the program computes from rows r0 .. r1 of the sliced inputs and all of
// the others, so a caller may run it slice by slice (the host entry points do, to have the kernels of one slice
// run while the next is on its way to the device).
bool row_sliceable(const Program& p, std::vector<char>* sliced);

// Caller-provided device memory for a program's temporaries (intermediates of multi-kernel plans, dtype
// staging, transposed operands, per-work-item slices of generated kernels).  `used` counts what one
// execution took; limit == 0 means "only add up" (a sizing pass).
struct Workspace {
  void* base = nullptr;
  size_t limit = 0;
  size_t used = 0;
  // temporaries that a launch can do without (the parts of a split loop) are not taken from the workspace at all:
  // for operands whose mandatory temporaries fit it only without them
  bool refuse_optional = false;
};

// Enqueue the program on `stream`.  All tensors live in device memory.
// Temporary buffers are stream-ordered allocations, so the call does not wait
// for the GPU; with a workspace they are carved out of it instead and the
// call allocates and frees no device memory.  Returns "" on success.
std::string execute(Program& p, const std::vector<DeviceTensor>& inputs, const std::vector<DeviceTensor>& outputs,
                    hipStream_t stream, Workspace* workspace = nullptr);

// Program options by name (ihip::set_kernel_option lists them); returns "" or the failure text.
std::string set_option(Program& p, const std::string& name, int value);
// Device memory for two 64-bit counters (or nullptr: off) to which the program's bf16 direct-to-LDS attention kernels
// add the time their workgroups were resident, on the shader clock and on the constant 100 MHz clock.
std::string set_clock_probe(Program& p, void* ticks);
// The kernels the last execute() of this program dispatched, one per line.
std::string last_report(Program& p);
// One more line for that report (the host entry points note a call that ran in slices).
void append_to_report(Program& p, const std::string& line);

// What execute() with a workspace would take from it for these operands, in bytes.  Launches nothing.
std::string workspace_bytes(Program& p, const std::vector<DeviceTensor>& inputs, const std::vector<DeviceTensor>& outputs,
                            size_t* bytes, bool refuse_optional = false);

// Frees the blocks of device memory that execute() keeps per stream for temporaries (those not in use by a call at
// this moment); returns the bytes released.
size_t release_stream_blocks();

}  // namespace ihipc
