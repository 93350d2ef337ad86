// The 𝚒 runtime C ABI (include/i.h): component handles and combinators.
// Reference behaviour: core/src/lib.rs:61-121, 289-351.
#include "../../../include/i.h"

#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <map>
#include <memory>
#include <condition_variable>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../../include/i_hip.h"
#include "../backend_hip/program.h"
#include "../runtime/hip_rt.h"
#include "../runtime/host_copy.h"
#include "../runtime/static_scratch.h"
#include "error.h"
#include "handles.h"

struct i_program {
  ihipc::Program* inner = nullptr;
  ~i_program() { delete inner; }
};

namespace {

i_component* wrap(ic::Component c) { return new i_component{std::make_shared<const ic::Component>(std::move(c))}; }

i_component* combine(const i_component* left, const i_component* right, ic::Component::Kind kind) {
  if (!left) {
    icore::set_error("null left component");
    return nullptr;
  }
  if (!right) {
    icore::set_error("null right component");
    return nullptr;
  }
  ic::Component c;
  c.kind = kind;
  c.a = left->inner;  // component trees are immutable, so sharing is a clone
  c.b = right->inner;
  return wrap(std::move(c));
}

// Strict UTF-8 check, matching CStr::to_str in the reference's read_str.
bool valid_utf8(const char* s) {
  const unsigned char* p = reinterpret_cast<const unsigned char*>(s);
  while (*p) {
    int n = *p < 0x80 ? 0 : (*p >> 5) == 0x6 ? 1 : (*p >> 4) == 0xE ? 2 : (*p >> 3) == 0x1E ? 3 : -1;
    if (n < 0) return false;
    if (n == 1 && *p < 0xC2) return false;
    ++p;
    for (int i = 0; i < n; ++i, ++p)
      if ((*p & 0xC0) != 0x80) return false;
  }
  return true;
}

int fail(const std::string& message) {
  icore::set_error(message);
  return -1;
}

// Shapes of the host operands, cut to the ranks the program reads.
std::vector<std::vector<size_t>> host_shapes(const ihipc::Program& p, const i_tensor* inputs, size_t input_count) {
  std::vector<std::vector<size_t>> out;
  for (size_t i = 0; i < input_count; ++i)
    out.emplace_back(inputs[i].shape ? std::vector<size_t>(inputs[i].shape, inputs[i].shape + inputs[i].rank) : std::vector<size_t>());
  return out;
}

// Device memory for the operands of host calls: one block per device that the library keeps from call to call
// (a host call returns after the GPU has finished, so the block is free again), as large as the largest call needed,
// at most ILANG_HIP_STAGING_MB (default 1024; 0: every operand is allocated, copied and freed on its own).  Calls
// whose operands fit 8 MiB go through a page-locked host mirror of the block as well: the inputs are gathered
// there and cross in one asynchronous copy, the outputs come back in one, instead of a blocking copy from pageable
// memory per operand.  Larger operands cross in page-locked chunks that several host threads fill and empty while
// the chunk before is in flight (runtime/host_copy.h).  A call that finds the block in use by another thread, or
// needs more, allocates as before.
struct Staging {
  void* base = nullptr;
  size_t capacity = 0;
  void* pinned = nullptr;  // a page-locked host mirror of the first kPinnedBytes of the block (small calls)
  std::mutex busy;
};
constexpr size_t kPinnedBytes = size_t(8) << 20;

struct StagingTable {
  std::mutex mu;
  std::map<int, std::unique_ptr<Staging>> blocks;
};
StagingTable& staging_table() {
  static StagingTable* table = new StagingTable();
  return *table;
}
Staging* staging_of_current_device() {
  StagingTable& t = staging_table();
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(t.mu);
  auto& block = t.blocks[device];
  if (!block) block = std::make_unique<Staging>();
  return block.get();
}

// Frees the blocks that no call is using at this moment; returns the bytes released (device and page-locked).
size_t release_staging_blocks() {
  size_t released = 0;
  StagingTable& t = staging_table();
  std::lock_guard<std::mutex> lock(t.mu);
  for (auto& [device, block] : t.blocks) {
    std::unique_lock<std::mutex> idle(block->busy, std::try_to_lock);
    if (!idle.owns_lock()) continue;
    if (block->base) {
      ihip::dev_free(block->base);
      released += block->capacity;
    }
    if (block->pinned) {
      (void)hipHostFree(block->pinned);
      released += kPinnedBytes;
    }
    block->base = block->pinned = nullptr;
    block->capacity = 0;
  }
  return released;
}

size_t staging_limit() {
  static const size_t limit = [] {
    const char* mb = std::getenv("ILANG_HIP_STAGING_MB");
    return (mb ? (size_t)std::max(0, std::atoi(mb)) : size_t(1024)) << 20;
  }();
  return limit;
}

// The two streams beside the call's own that a call in slices uses: `which` 0 carries the uploads, 1 the downloads
// (one each per device, created on first use and kept; not synchronised with the default stream, on which the
// kernels run); nullptr when there is none to be had.
hipStream_t side_stream_of_current_device(int which) {
  static std::mutex mu;
  static std::map<int, hipStream_t>* streams = new std::map<int, hipStream_t>();
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  auto it = streams->find(2 * device + which);
  if (it != streams->end()) return it->second;
  hipStream_t made = nullptr;
  if (hipStreamCreateWithFlags(&made, hipStreamNonBlocking) != hipSuccess) {
    (void)hipGetLastError();
    made = nullptr;
  }
  (*streams)[2 * device + which] = made;
  return made;
}

// A call in slices (large operands of a program that only maps over its leading index, ihipc::row_sliceable): the
// inputs that every slice needs whole are uploaded first; then, slice after slice, the rows of the other inputs go
// up on the upload stream and the program is enqueued on `stream` behind them for just those rows, so the kernels
// of one slice run while the next is on the link; a second host thread brings the rows of the outputs down on the
// download stream as soon as their slice has run, beside the uploads of the slices after it (the link carries both
// directions at once).  Returns false when the call is not taken in slices (nothing has been enqueued then); true
// with the outputs in host memory, or with *err set.
constexpr size_t kSlicedCallBytes = size_t(64) << 20;  // what crosses the link in slices, at least
constexpr size_t kSliceBytes = size_t(32) << 20;       // ... and per slice, about
bool run_host_in_slices(ihipc::Program& p, const i_tensor* inputs, const std::vector<ihipc::DeviceTensor>& in,
                        const std::vector<ihipc::DeviceTensor>& out, const std::vector<float*>& out_ptrs, hipStream_t stream,
                        std::string* err) {
  std::vector<char> sliced;
  if (!ihipc::row_sliceable(p, &sliced) || sliced.size() != in.size() || out.empty() || out[0].shape.empty()) return false;
  const size_t rows = out[0].shape[0];
  auto row_bytes = [](const ihipc::DeviceTensor& t) {
    size_t n = 4;
    for (size_t d = 1; d < t.shape.size(); ++d) n *= t.shape[d];
    return n;
  };
  size_t moving = 0, whole = 0;
  for (size_t i = 0; i < in.size(); ++i) {
    if (sliced[i] && (in[i].shape.empty() || in[i].shape[0] != rows)) return false;
    (sliced[i] ? moving : whole) += row_bytes(in[i]) * (in[i].shape.empty() ? 1 : in[i].shape[0]);
  }
  for (size_t o = 0; o < out.size(); ++o) {
    if (out[o].shape.empty() || out[o].shape[0] != rows || !out_ptrs[o]) return false;
    moving += row_bytes(out[o]) * rows;
  }
  if (rows < 2 || moving < kSlicedCallBytes || moving < whole) return false;
  const size_t wanted = std::min<size_t>(std::min<size_t>(8, rows), std::max<size_t>(2, moving / kSliceBytes));
  const size_t each = (rows + wanted - 1) / wanted, slices = (rows + each - 1) / each;
  hipStream_t up = side_stream_of_current_device(0), down = side_stream_of_current_device(1);
  int device = 0;
  if (!up || !down || hipGetDevice(&device) != hipSuccess) return false;
  std::vector<hipEvent_t> landed(slices, nullptr), done(slices, nullptr);
  auto destroy_events = [&] {
    for (hipEvent_t e : landed)
      if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : done)
      if (e) (void)hipEventDestroy(e);
  };
  for (size_t s = 0; s < slices; ++s)
    if (hipEventCreateWithFlags(&landed[s], hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&done[s], hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      destroy_events();
      return false;
    }
  // the downloads: slice s once the main thread says that it has been enqueued (or that nothing more will be)
  std::mutex mu;
  std::condition_variable changed;
  size_t enqueued = 0;
  bool stop = false;
  std::string down_err;
  auto bring_down_slices = [&] {
    (void)hipSetDevice(device);
    for (size_t s = 0; s < slices; ++s) {
      {
        std::unique_lock<std::mutex> lock(mu);
        changed.wait(lock, [&] { return enqueued > s || stop; });
        if (enqueued <= s) return;
      }
      if (hipStreamWaitEvent(down, done[s], 0) != hipSuccess) {
        down_err = "hipStreamWaitEvent failed";
        return;
      }
      const size_t r0 = s * each, r1 = std::min(rows, r0 + each);
      for (size_t o = 0; o < out.size(); ++o) {
        const size_t at = r0 * row_bytes(out[o]), bytes = (r1 - r0) * row_bytes(out[o]);
        if (ihip::Err e = ihip::download_pipelined(reinterpret_cast<char*>(out_ptrs[o]) + at, static_cast<const char*>(out[o].data) + at, bytes, down);
            !e.empty()) {
          down_err = e;
          return;
        }
      }
    }
  };
  auto bring_down = [&] {
    try {
      bring_down_slices();
    } catch (const std::exception& e) {  // (nothing may leave a thread's function)
      down_err = e.what();
    }
  };
  std::thread helper;
  try {
    helper = std::thread(bring_down);
  } catch (const std::exception&) {
    destroy_events();
    return false;
  }
  auto finish = [&](const std::string& what, bool all_enqueued) {
    {
      std::lock_guard<std::mutex> lock(mu);
      stop = !all_enqueued;
      if (all_enqueued) enqueued = slices;
    }
    changed.notify_all();
    helper.join();
    *err = !what.empty() ? what : down_err;
    if (!err->empty()) {
      (void)hipStreamSynchronize(up);
      (void)hipStreamSynchronize(down);
      (void)ihip::sync(stream);
    }
    destroy_events();
    return true;
  };
  // (the device copies may still be read by the kernels of the call before this one on `stream`: the kept block
  // is handed from call to call only after a wait for `stream`, so nothing is in flight there)
  for (size_t i = 0; i < in.size(); ++i)
    if (!sliced[i]) {
      const size_t bytes = row_bytes(in[i]) * (in[i].shape.empty() ? 1 : in[i].shape[0]);
      if (ihip::Err e = ihip::upload_pipelined(in[i].data, inputs[i].data, bytes, up); !e.empty()) return finish(e, false);
    }
  for (size_t s = 0; s < slices; ++s) {
    const size_t r0 = s * each, r1 = std::min(rows, r0 + each);
    std::vector<ihipc::DeviceTensor> in_s(in), out_s(out);
    for (size_t i = 0; i < in.size(); ++i) {
      if (!sliced[i]) continue;
      const size_t at = r0 * row_bytes(in[i]), bytes = (r1 - r0) * row_bytes(in[i]);
      in_s[i].data = static_cast<char*>(in[i].data) + at;
      in_s[i].shape[0] = r1 - r0;
      if (ihip::Err e = ihip::upload_pipelined(in_s[i].data, static_cast<const char*>(static_cast<const void*>(inputs[i].data)) + at, bytes, up);
          !e.empty())
        return finish(e, false);
    }
    for (size_t o = 0; o < out.size(); ++o) {
      out_s[o].data = static_cast<char*>(out[o].data) + r0 * row_bytes(out[o]);
      out_s[o].shape[0] = r1 - r0;
    }
    if (hipEventRecord(landed[s], up) != hipSuccess || hipStreamWaitEvent(stream, landed[s], 0) != hipSuccess)
      return finish("hipStreamWaitEvent failed", false);
    std::string e;
    try {
      e = ihipc::execute(p, in_s, out_s, stream);
    } catch (const std::exception& ex) {
      e = ex.what();
    }
    if (e.empty() && hipEventRecord(done[s], stream) != hipSuccess) e = "hipEventRecord failed";
    if (!e.empty()) return finish(e, false);
    {
      std::lock_guard<std::mutex> lock(mu);
      enqueued = s + 1;
    }
    changed.notify_all();
  }
  ihipc::append_to_report(p, "host: operands in " + std::to_string(slices) + " slices of " + std::to_string(each) +
                                 " rows, the kernels above are those of the last slice\n");
  return finish({}, true);
}

// Host entry: upload f32 operands, run, download, wait.  Mirrors the
// blocking behaviour of the reference's exec (core/src/lib.rs:200-225).
std::string run_host(ihipc::Program& p, const i_tensor* inputs, size_t input_count, const std::vector<float*>& out_ptrs) {
  const auto in_shapes = host_shapes(p, inputs, input_count);
  std::vector<std::vector<size_t>> out_shapes;
  if (std::string e = ihipc::output_shapes(p, in_shapes, &out_shapes); !e.empty()) return e;
  std::vector<void*> owned;
  hipStream_t stream = nullptr;
  bool staged = false;
  auto cleanup = [&] {
    if (staged) (void)ihip::sync(stream);  // (an early return: nothing may still be using the kept block)
    for (void* ptr : owned) ihip::dev_free(ptr);
  };
  // the operands' device copies: carved from the kept block when it is free and large enough (or can be made so)
  auto bytes_of = [](const std::vector<size_t>& shape) {
    size_t n = 4;
    for (size_t d : shape) n *= d;
    return (std::max<size_t>(n, 4) + 255) / 256 * 256;
  };
  size_t wanted = 0;
  for (size_t i = 0; i < input_count; ++i) wanted += bytes_of(in_shapes[i]);
  for (const auto& shape : out_shapes) wanted += bytes_of(shape);
  std::unique_lock<std::mutex> staging_lock;
  char* carve = nullptr;
  char *mirror = nullptr, *block_base = nullptr;  // mirror != nullptr: host data passes through the page-locked mirror
  if (wanted <= staging_limit()) {
    if (Staging* block = staging_of_current_device()) {
      staging_lock = std::unique_lock<std::mutex>(block->busy, std::try_to_lock);
      if (staging_lock.owns_lock()) {
        if (block->capacity < wanted) {
          ihip::dev_free(block->base);
          block->base = nullptr;
          block->capacity = 0;
          if (ihip::dev_alloc(&block->base, wanted).empty()) block->capacity = wanted;
        }
        if (block->capacity >= wanted) {
          carve = static_cast<char*>(block->base);
          staged = true;
          if (wanted <= kPinnedBytes) {
            if (!block->pinned && hipHostMalloc(&block->pinned, kPinnedBytes, hipHostMallocDefault) != hipSuccess) {
              block->pinned = nullptr;
              (void)hipGetLastError();
            }
            mirror = static_cast<char*>(block->pinned);
          }
          block_base = carve;
        }
      }
    }
  }
  auto device_copy = [&](void** ptr, const std::vector<size_t>& shape) -> ihip::Err {
    if (carve) {
      *ptr = carve;
      carve += bytes_of(shape);
      return {};
    }
    size_t n = 1;
    for (size_t d : shape) n *= d;
    if (ihip::Err e = ihip::dev_alloc(ptr, n * 4); !e.empty()) return e;
    owned.push_back(*ptr);
    return {};
  };
  std::vector<ihipc::DeviceTensor> in, out;
  for (size_t i = 0; i < input_count; ++i) {
    size_t n = 1;
    for (size_t d : in_shapes[i]) n *= d;
    ihipc::DeviceTensor t;
    t.shape = in_shapes[i];
    if (n && !inputs[i].data) {
      cleanup();
      return "input " + std::to_string(i) + " has no data";
    }
    if (ihip::Err e = device_copy(&t.data, in_shapes[i]); !e.empty()) {
      cleanup();
      return e;
    }
    if (mirror && n) std::memcpy(mirror + (static_cast<char*>(t.data) - block_base), inputs[i].data, n * 4);
    in.push_back(std::move(t));
  }
  const size_t input_bytes = carve ? (size_t)(carve - block_base) : 0;  // (the inputs lie first in the block)
  if (mirror && input_bytes) {
    if (ihip::Err e = ihip::h2d(block_base, mirror, input_bytes, stream); !e.empty()) {
      cleanup();
      return e;
    }
  }
  for (size_t o = 0; o < out_shapes.size(); ++o) {
    size_t n = 1;
    for (size_t d : out_shapes[o]) n *= d;
    ihipc::DeviceTensor t;
    t.shape = out_shapes[o];
    if (ihip::Err e = device_copy(&t.data, out_shapes[o]); !e.empty()) {
      cleanup();
      return e;
    }
    out.push_back(std::move(t));
  }
  std::string err;
  // large operands: in slices when the program allows it, else one after the other and then the program
  const bool in_slices = !mirror && run_host_in_slices(p, inputs, in, out, out_ptrs, stream, &err);  // (outputs included)
  if (!in_slices) {
    for (size_t i = 0; !mirror && err.empty() && i < input_count; ++i) {
      size_t n = 1;
      for (size_t d : in_shapes[i]) n *= d;
      err = ihip::upload_pipelined(in[i].data, inputs[i].data, n * 4, stream);
    }
    try {
      if (err.empty()) err = ihipc::execute(p, in, out, stream);
    } catch (const std::exception& e) {
      err = e.what();
    }
  }
  for (size_t o = 0; !in_slices && err.empty() && o < out.size(); ++o) {
    size_t n = 1;
    for (size_t d : out_shapes[o]) n *= d;
    if (n && !out_ptrs[o]) err = "output " + std::to_string(o) + " has no data";
    else if (!mirror) err = ihip::download_pipelined(out_ptrs[o], out[o].data, n * 4, stream);
  }
  if (mirror && err.empty() && carve - block_base > (ptrdiff_t)input_bytes)
    err = ihip::d2h(mirror + input_bytes, block_base + input_bytes, (size_t)(carve - block_base) - input_bytes, stream);
  const ihip::Err sync_err = ihip::sync(stream);
  if (err.empty()) err = sync_err;
  for (size_t o = 0; mirror && err.empty() && o < out.size(); ++o) {
    size_t n = 1;
    for (size_t d : out_shapes[o]) n *= d;
    if (n) std::memcpy(out_ptrs[o], mirror + (static_cast<char*>(out[o].data) - block_base), n * 4);
  }
  cleanup();
  return err;
}

// Argument checks shared by the device entry points; fills `in` / `out` and returns true, or sets the error.
bool device_call_ok(const i_program* program, const i_device_tensor* inputs, size_t input_count,
                    const i_device_tensor* outputs, size_t output_count, std::vector<ihipc::DeviceTensor>* in,
                    std::vector<ihipc::DeviceTensor>* out) {
  if (!program) return fail("null program"), false;
  if (input_count > 0 && !inputs) return fail("null inputs"), false;
  if (output_count != ihipc::output_count(*program->inner)) return fail("wrong output count"), false;
  if (output_count > 0 && !outputs) return fail("null outputs"), false;
  auto convert = [](const i_device_tensor* t, size_t n, std::vector<ihipc::DeviceTensor>* dst) -> bool {
    for (size_t i = 0; i < n; ++i) {
      if (t[i].dtype != I_DTYPE_F32 && t[i].dtype != I_DTYPE_BF16) return false;
      ihipc::DeviceTensor d;
      d.data = t[i].data;
      d.dtype = t[i].dtype == I_DTYPE_BF16 ? ihipc::DType::BF16 : ihipc::DType::F32;
      if (t[i].rank > 0 && !t[i].shape) return false;
      d.shape.assign(t[i].shape, t[i].shape + t[i].rank);
      dst->push_back(std::move(d));
    }
    return true;
  };
  if (!convert(inputs, input_count, in) || !convert(outputs, output_count, out))
    return fail("bad device tensor (dtype or shape)"), false;
  return true;
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

i_component* i_parse(const char* src) {
  if (!src || !valid_utf8(src)) {
    icore::set_error("null source");
    return nullptr;
  }
  try {
    ic::Component c;
    c.kind = ic::Component::Leaf;
    c.expr = ic::parse_expr(src);
    return wrap(std::move(c));
  } catch (const ic::CompileError& e) {
    icore::set_error(e.debug_string());
  } catch (const std::exception& e) {
    icore::set_error(e.what());
  }
  return nullptr;
}

i_component* i_identity(void) { return wrap(ic::Component{}); }

i_component* i_chain(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Chain); }
i_component* i_compose(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Compose); }
i_component* i_fanout(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Fanout); }
i_component* i_pair(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Pair); }

i_component* i_swap(const i_component* component) {
  if (!component) {
    icore::set_error("null component");
    return nullptr;
  }
  ic::Component c;
  c.kind = ic::Component::Swap;
  c.a = component->inner;
  return wrap(std::move(c));
}

char* i_code(const i_component* component) {
  if (!component) {
    icore::set_error("null component");
    return nullptr;
  }
  try {
    const std::string text = ihipc::program_code(*component->inner);
    if (text.find('\0') != std::string::npos) {
      icore::set_error("source contains interior NUL");
      return nullptr;
    }
    char* out = static_cast<char*>(std::malloc(text.size() + 1));
    if (!out) {
      icore::set_error("out of memory");
      return nullptr;
    }
    std::memcpy(out, text.c_str(), text.size() + 1);
    return out;
  } catch (const ic::CompileError& e) {
    icore::set_error(e.debug_string());
  } catch (const std::exception& e) {
    icore::set_error(e.what());
  }
  return nullptr;
}

i_program* i_compile(const i_component* component) {
  if (!component) {
    icore::set_error("null component");
    return nullptr;
  }
  try {
    ihipc::Program* inner = nullptr;
    const std::string err = ihipc::compile_program(*component->inner, &inner);
    if (!err.empty()) {
      icore::set_error(err);
      return nullptr;
    }
    auto* program = new i_program;
    program->inner = inner;
    return program;
  } catch (const ic::CompileError& e) {
    icore::set_error(e.debug_string());
  } catch (const std::exception& e) {
    icore::set_error(e.what());
  }
  return nullptr;
}

size_t i_output_count(const i_program* program) {
  if (!program) {
    icore::set_error("null program");
    return 0;
  }
  return ihipc::output_count(*program->inner);
}

int i_output_ranks(const i_program* program, size_t* ranks) {
  if (!program) return fail("null program");
  if (!ranks) return fail("null ranks");
  const auto r = ihipc::output_ranks(*program->inner);
  for (size_t i = 0; i < r.size(); ++i) ranks[i] = r[i];
  return 0;
}

int i_output_shapes(const i_program* program, const i_tensor* inputs, size_t input_count, size_t** shapes) {
  if (!program) return fail("null program");
  if (input_count > 0 && !inputs) return fail("null inputs");
  if (!shapes) return fail("null shapes");
  std::vector<std::vector<size_t>> out;
  const std::string err = ihipc::output_shapes(*program->inner, host_shapes(*program->inner, inputs, input_count), &out);
  if (!err.empty()) return fail(err);
  for (size_t o = 0; o < out.size(); ++o)
    for (size_t d = 0; d < out[o].size(); ++d) shapes[o][d] = out[o][d];
  return 0;
}

int i_exec_into(const i_program* program, const i_tensor* inputs, size_t input_count, i_tensor_mut* outputs,
                size_t output_count) {
  if (!program) return fail("null program");
  if (input_count > 0 && !inputs) return fail("null inputs");
  if (output_count != ihipc::output_count(*program->inner)) return fail("wrong output count");
  if (output_count > 0 && !outputs) return fail("null outputs");
  // An output whose extents the caller states is checked against what the program writes: a smaller buffer would be
  // overrun on the host.  (The reference takes the caller's word, core/src/lib.rs:200-225; a tensor without a shape
  // array is taken on trust here too.)
  {
    std::vector<std::vector<size_t>> written;
    if (std::string e = ihipc::output_shapes(*program->inner, host_shapes(*program->inner, inputs, input_count), &written); !e.empty())
      return fail(e);
    for (size_t o = 0; o < output_count && o < written.size(); ++o) {
      if (!outputs[o].shape) continue;
      bool same = outputs[o].rank == written[o].size();
      for (size_t d = 0; same && d < written[o].size(); ++d) same = outputs[o].shape[d] == written[o][d];
      if (!same) {
        auto text = [](const size_t* dims, size_t rank) {
          std::string t = "[";
          for (size_t d = 0; d < rank; ++d) t += (d ? ", " : "") + std::to_string(dims[d]);
          return t + "]";
        };
        return fail("output " + std::to_string(o) + " has shape " + text(outputs[o].shape, outputs[o].rank) + ", the program writes " +
                    text(written[o].data(), written[o].size()));
      }
    }
  }
  std::vector<float*> out_ptrs;
  for (size_t o = 0; o < output_count; ++o) out_ptrs.push_back(outputs[o].data);
  const std::string err = run_host(*program->inner, inputs, input_count, out_ptrs);
  return err.empty() ? 0 : fail(err);
}

i_outputs i_exec(const i_program* program, const i_tensor* inputs, size_t input_count) {
  i_outputs none{nullptr, 0};
  if (!program) {
    icore::set_error("null program");
    return none;
  }
  if (input_count > 0 && !inputs) {
    icore::set_error("null inputs");
    return none;
  }
  ihipc::Program& p = *program->inner;
  std::vector<std::vector<size_t>> shapes;
  if (std::string err = ihipc::output_shapes(p, host_shapes(p, inputs, input_count), &shapes); !err.empty()) {
    icore::set_error(err);
    return none;
  }
  const size_t count = shapes.size();
  auto* tensors = static_cast<i_owned_tensor*>(std::calloc(count ? count : 1, sizeof(i_owned_tensor)));
  std::vector<float*> out_ptrs;
  bool ok = tensors != nullptr;
  for (size_t o = 0; ok && o < count; ++o) {
    size_t len = 1;
    for (size_t d : shapes[o]) len *= d;
    tensors[o].rank = shapes[o].size();
    tensors[o].len = len;
    tensors[o].data = static_cast<float*>(std::calloc(len ? len : 1, sizeof(float)));  // zero-filled, as the reference
    tensors[o].shape = static_cast<size_t*>(std::calloc(shapes[o].size() ? shapes[o].size() : 1, sizeof(size_t)));
    ok = tensors[o].data && tensors[o].shape;
    if (ok) std::copy(shapes[o].begin(), shapes[o].end(), tensors[o].shape);
    out_ptrs.push_back(tensors[o].data);
  }
  i_outputs result{tensors, count};
  std::string err = ok ? run_host(p, inputs, input_count, out_ptrs) : std::string("out of memory");
  if (!err.empty()) {
    i_outputs_free(result);
    icore::set_error(err);
    return none;
  }
  return result;
}

int i_exec_into_device(const i_program* program, const i_device_tensor* inputs, size_t input_count,
                       const i_device_tensor* outputs, size_t output_count, void* stream) {
  std::vector<ihipc::DeviceTensor> in, out;
  if (!device_call_ok(program, inputs, input_count, outputs, output_count, &in, &out)) return -1;
  try {
    const std::string err = ihipc::execute(*program->inner, in, out, static_cast<hipStream_t>(stream));
    return err.empty() ? 0 : fail(err);
  } catch (const std::exception& e) {
    return fail(e.what());
  }
}

int i_exec_into_device_noalloc(const i_program* program, const i_device_tensor* inputs, size_t input_count,
                               const i_device_tensor* outputs, size_t output_count, void* stream) {
  std::vector<ihipc::DeviceTensor> in, out;
  if (!device_call_ok(program, inputs, input_count, outputs, output_count, &in, &out)) return -1;
  try {
    // set-up, once per device: the address of this device's copy of the static workspace
    void* base = nullptr;
    if (ihip::Err e = ihip::static_scratch(&base); !e.empty()) return fail(e);
    // size the temporaries first, so that a program that does not fit is refused before anything is enqueued
    // (with the temporaries of split loops first; when that is too much, without them: the loops then run whole)
    size_t need = 0;
    bool refuse_optional = false;
    if (std::string e = ihipc::workspace_bytes(*program->inner, in, out, &need); !e.empty()) return fail(e);
    if (need > ihip::kStaticScratchBytes) {
      refuse_optional = true;
      if (std::string e = ihipc::workspace_bytes(*program->inner, in, out, &need, true); !e.empty()) return fail(e);
    }
    if (need > ihip::kStaticScratchBytes)
      return fail("program needs " + std::to_string(need) + " bytes of temporaries for these operands, the static workspace holds " +
                  std::to_string(ihip::kStaticScratchBytes) + " (use i_exec_into_device)");
    ihipc::Workspace ws{base, ihip::kStaticScratchBytes, 0, refuse_optional};
    const std::string err = ihipc::execute(*program->inner, in, out, static_cast<hipStream_t>(stream), &ws);
    return err.empty() ? 0 : fail(err);
  } catch (const std::exception& e) {
    return fail(e.what());
  }
}

size_t i_hip_release_cached_memory(void) {
  size_t released = ihipc::release_stream_blocks();
  released += release_staging_blocks();
  released += ihip::release_copy_chunks();
  released += ihip::trim_temp_pool();
  return released;
}

int i_hip_program_option(i_program* program, const char* name, int value) {
  if (!program) return fail("null program");
  if (!name) return fail("null option name");
  const std::string err = ihipc::set_option(*program->inner, name, value);
  return err.empty() ? 0 : fail(err);
}

int i_hip_program_clock_probe(i_program* program, void* ticks) {
  if (!program) return fail("null program");
  const std::string err = ihipc::set_clock_probe(*program->inner, ticks);
  return err.empty() ? 0 : fail(err);
}

int i_hip_program_row_slices(const i_program* program, unsigned char* sliced, size_t capacity) {
  if (!program) {
    icore::set_error("null program");
    return -1;
  }
  std::vector<char> flags;
  if (!ihipc::row_sliceable(*program->inner, &flags)) return 0;
  if (sliced && capacity < flags.size()) {
    icore::set_error("the program has " + std::to_string(flags.size()) + " inputs");
    return -1;
  }
  for (size_t i = 0; sliced && i < flags.size(); ++i) sliced[i] = flags[i] ? 1 : 0;
  return (int)flags.size();
}

char* i_hip_program_report(const i_program* program) {
  if (!program) {
    icore::set_error("null program");
    return nullptr;
  }
  const std::string text = ihipc::last_report(*program->inner);
  char* out = static_cast<char*>(std::malloc(text.size() + 1));
  if (!out) {
    icore::set_error("out of memory");
    return nullptr;
  }
  std::memcpy(out, text.c_str(), text.size() + 1);
  return out;
}

void i_component_free(i_component* component) { delete component; }

void i_program_free(i_program* program) { delete program; }

void i_outputs_free(i_outputs outputs) {
  if (!outputs.tensors) return;
  for (size_t i = 0; i < outputs.count; ++i) {
    std::free(outputs.tensors[i].data);
    std::free(outputs.tensors[i].shape);
  }
  std::free(outputs.tensors);
}

void i_string_free(char* s) { std::free(s); }

const char* i_error(void) { return icore::last_error(); }

}  // extern "C"
#pragma GCC visibility pop
