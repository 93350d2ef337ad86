#include "program.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <sstream>

#include "../runtime/hip_rt.h"
#include "../runtime/kernel_launch.h"
#include "hipcc.h"

namespace ihipc {
using namespace ic;
namespace {

size_t product(const std::vector<size_t>& v) {
  size_t n = 1;
  for (size_t x : v) n *= x;
  return n;
}

const PlanBuffer& plan_buffer(const ExecPlan& plan, BufferRef r) {
  return r.kind == BufferRef::Input ? plan.inputs.at(r.id) : r.kind == BufferRef::Intermediate ? plan.intermediates.at(r.id) : plan.outputs.at(r.id);
}

std::string ref_name(BufferRef r) {
  return (r.kind == BufferRef::Input ? "in" : r.kind == BufferRef::Intermediate ? "s" : "out") + std::to_string(r.id);
}

// The temporaries of the calls on one stream of one device share a block that the library keeps: kernels on a
// stream run one after the other, so a call may overwrite what the call before it on the same stream left there,
// and after the first call of a program no call allocates or frees anything (a stream-ordered allocation and its
// release cost the host 20 to 45 us a call here, several times the rest of the executor).  A call carves its
// temporaries off the block; what does not fit is allocated as before, and at its end the call replaces the block
// by one large enough for all it needed, up to ILANG_HIP_ARENA_MB (default 256; 0: no such block) per stream,
// held until the process ends, for the first 16 streams that run programs.  A stream under capture and a second
// call in flight on the same stream from another thread take the allocating path (and so does every call under
// ILANG_HIP_ARENA_MB=0, which tools that guard allocations one by one use).
struct Arena {
  void* base = nullptr;
  size_t capacity = 0;
  size_t last_use = 0;  // (guarded by the table's mutex)
  std::mutex busy;  // held by the call that carves from it
};

// At most 16 (device, stream) pairs keep a block.  A stream beyond that takes the place of the pair that has gone
// unused the longest (an application with a stream per request: its short-lived streams pass through, the
// long-lived ones keep their blocks); an entry is never destroyed, so a call that holds one is never left without.
struct ArenaTable {
  std::mutex mu;
  std::map<std::pair<int, hipStream_t>, std::unique_ptr<Arena>> arenas;
  size_t clock = 0;
};
ArenaTable& arena_table() {
  static ArenaTable* table = new ArenaTable();
  return *table;
}

Arena* arena_of(hipStream_t stream) {
  ArenaTable& t = arena_table();
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(t.mu);
  auto found = t.arenas.find({device, stream});
  if (found == t.arenas.end()) {
    if (t.arenas.size() < 16) {
      found = t.arenas.emplace(std::make_pair(device, stream), std::make_unique<Arena>()).first;
    } else {
      auto oldest = t.arenas.end();
      for (auto it = t.arenas.begin(); it != t.arenas.end(); ++it)
        if (it->first.first == device && (oldest == t.arenas.end() || it->second->last_use < oldest->second->last_use)) oldest = it;
      if (oldest == t.arenas.end()) return nullptr;
      std::unique_lock<std::mutex> idle(oldest->second->busy, std::try_to_lock);
      if (!idle.owns_lock()) return nullptr;  // (in use right now: this call allocates)
      // what the old stream's last call left in the block may still be running: the block goes back stream-ordered
      // on that stream when the stream still exists, else at once
      if (oldest->second->base && hipFreeAsync(oldest->second->base, oldest->first.second) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(oldest->second->base);
      }
      oldest->second->base = nullptr;
      oldest->second->capacity = 0;
      idle.unlock();
      std::unique_ptr<Arena> moved = std::move(oldest->second);
      t.arenas.erase(oldest);
      found = t.arenas.emplace(std::make_pair(device, stream), std::move(moved)).first;
    }
  }
  found->second->last_use = ++t.clock;
  return found->second.get();
}

size_t arena_limit() {
  static const size_t limit = [] {
    const char* mb = std::getenv("ILANG_HIP_ARENA_MB");
    return (mb ? (size_t)std::max(0, std::atoi(mb)) : size_t(256)) << 20;
  }();
  return limit;
}

// Everything the executor needs to know about one invocation.
struct Run {
  Program& p;
  const ExecPlan& plan;
  const std::vector<DeviceTensor>& inputs;
  const std::vector<DeviceTensor>& outputs;
  hipStream_t stream;
  std::vector<void*> temps;                  // stream-ordered allocations to release
  std::vector<void*> intermediates;          // device pointers (f32), null when not needed
  std::map<size_t, void*> input_f32;         // bf16 inputs widened for f32 kernels
  std::map<size_t, void*> output_f32;        // f32 staging for bf16 outputs
  Workspace* workspace = nullptr;            // when set, temporaries are carved out of it and nothing is allocated
  std::vector<std::string> notes;            // one line per dispatched kernel: what ran, on which tile
  Arena* arena = nullptr;                    // when set (and locked by this call), temporaries come off it while they fit
  size_t arena_used = 0, arena_needed = 0;
  bool capturing = false;                    // the stream is being captured into a graph
  ihip::KernelOptions knobs;                 // the program's options as they were when the call started

  size_t dim(DimRef<size_t> d) const { return inputs[d.buffer].shape[d.dim]; }
  size_t extent(const Extent<size_t>& e) const {
    const size_t n = dim(e.source);
    switch (e.kind.kind) {
      case ExtentKind::Semantic: return n;
      case ExtentKind::Base: {
        const size_t f = product(e.kind.factors);
        return f <= 1 ? n : (n + f - 1) / f;
      }
      case ExtentKind::Split: return e.kind.factor;
    }
    return n;
  }
  std::vector<size_t> shape_of(BufferRef r) const {
    std::vector<size_t> out;
    for (const auto& d : plan_buffer(plan, r).shape) out.push_back(dim(d));
    return out;
  }
  std::vector<size_t> layout_of(BufferRef r) const {
    std::vector<size_t> out;
    for (const auto& e : plan_buffer(plan, r).layout) out.push_back(extent(e));
    return out;
  }
  DType dtype_of(BufferRef r) const {
    if (r.kind == BufferRef::Input) return inputs[r.id].dtype;
    if (r.kind == BufferRef::Output) return outputs[r.id].dtype;
    return DType::F32;
  }
  void* raw_ptr(BufferRef r) const {
    if (r.kind == BufferRef::Input) return inputs[r.id].data;
    if (r.kind == BufferRef::Output) return outputs[r.id].data;
    return intermediates[r.id];
  }

  ihip::Err alloc(void** ptr, size_t bytes) {
    if (bytes == 0) bytes = 4;
    if (workspace) {
      // bump allocation in 256-byte steps; the sizing pass has no limit and only adds up
      const size_t step = (bytes + 255) / 256 * 256;
      if (workspace->limit && step > workspace->limit - workspace->used) return "workspace exhausted";
      *ptr = static_cast<char*>(workspace->base) + workspace->used;
      workspace->used += step;
      return {};
    }
    if (arena) {
      const size_t step = (bytes + 255) / 256 * 256;
      arena_needed += step;
      if (step <= arena->capacity - arena_used) {
        *ptr = static_cast<char*>(arena->base) + arena_used;
        arena_used += step;
        return {};
      }
    }
    // (a stream under capture: the plain stream-ordered allocation, which a graph records as a node of its own)
    if (ihip::Err e = capturing ? ihip::check(hipMallocAsync(ptr, bytes, stream), "hipMallocAsync") : ihip::temp_alloc(ptr, bytes, stream);
        !e.empty())
      return e;
    temps.push_back(*ptr);
    return {};
  }

  // A temporary that a launch can do without (the parts of a split loop): with a workspace, which is small and whose
  // sizing pass only adds up, at most 20 MiB are taken for one, so that most of what fits unsplit still fits.
  bool alloc_optional(void** ptr, size_t bytes) {
    if (workspace && (workspace->refuse_optional || bytes > (size_t(20) << 20))) return false;
    return alloc(ptr, bytes).empty();
  }

  // Device pointer to f32 data of a buffer some f32 kernel reads.
  ihip::Err read_f32(BufferRef r, void** ptr) {
    if (dtype_of(r) == DType::F32) {
      *ptr = r.kind == BufferRef::Output && output_f32.count(r.id) ? output_f32[r.id] : raw_ptr(r);
      return {};
    }
    if (r.kind == BufferRef::Output) {  // a bf16 output that a later kernel reads back: use its f32 staging
      *ptr = output_f32.at(r.id);
      return {};
    }
    auto it = input_f32.find(r.id);
    if (it == input_f32.end()) {
      const size_t n = product(inputs[r.id].shape);
      void* tmp = nullptr;
      if (ihip::Err e = alloc(&tmp, n * 4); !e.empty()) return e;
      if (ihip::Err e = ihip::launch_convert(inputs[r.id].data, tmp, ihip::BF16, ihip::F32, n, stream); !e.empty()) return e;
      it = input_f32.emplace(r.id, tmp).first;
    }
    *ptr = it->second;
    return {};
  }
  // Device pointer an f32-producing kernel writes to.
  ihip::Err write_f32(BufferRef r, void** ptr) {
    if (r.kind != BufferRef::Output || outputs[r.id].dtype == DType::F32) {
      *ptr = raw_ptr(r);
      return {};
    }
    auto it = output_f32.find(r.id);
    if (it == output_f32.end()) {
      void* tmp = nullptr;
      if (ihip::Err e = alloc(&tmp, product(shape_of(r)) * 4); !e.empty()) return e;
      it = output_f32.emplace(r.id, tmp).first;
    }
    *ptr = it->second;
    return {};
  }
};

// ---------------------------------------------------------------- hand-written kernels
// Head sizes beyond the fused attention kernels (d or dv above 256, above 128 for f32 operands or d != dv; the
// reference's demo uses 2048,
// ilang-python/flash-attn.py:31-36) run as three hand-written kernels with the score matrix in memory:
// S = Q K^T (MFMA GEMM), P = softmax(scale * S) row by row in place, O = P V (MFMA GEMM).  What the GEMM kernels
// need of the extents decides whether that is possible; the score matrix may take up to 16 GiB.
bool attention_in_parts_usable(DType t, size_t bh, size_t nq, size_t nk, size_t d, size_t dv) {
  if (bh == 0 || nq == 0 || nk == 0 || d == 0 || dv == 0) return false;
  if (bh > 65535 || (bh * nq) > 0x7fffffffull || nk > 0xffffffffull) return false;
  if (bh * nq * nk > (size_t(4) << 30)) return false;  // f32 elements: 16 GiB
  if (t == DType::F32) return ihip::gemm_nt_f32_supported(d) && ihip::gemm_nt_f32_supported(nk);
  return ihip::gemm_nt_bf16_supported(d) && ihip::gemm_nt_bf16_supported(nk);
}

// A product runs on the matrix-instruction kernels whatever its contracted extent k: when k is no multiple of what
// they need (8 in bf16, 4 in f32), or f32 operands are not 16-byte aligned, both operands are first copied into
// temporaries whose rows are padded with zeros (padded_operands below); the padding adds nothing to the sums.
size_t product_k_quantum(DType t) { return t == DType::BF16 ? 8 : 4; }
bool product_extent_usable(DType t, size_t k) {
  const size_t q = product_k_quantum(t), kp = (k + q - 1) / q * q;
  return t == DType::BF16 ? ihip::gemm_nt_bf16_supported(kp) : ihip::gemm_nt_f32_supported(kp);
}

// Returns true when kernel k can run on its hand-written form with these operands.
// The arithmetic of a product: bf16 operands on the bf16 kernels; an f32 operand (say the probabilities of the naive
// attention, an f32 intermediate, against bf16 values) makes it an f32 product, the other operand widened first.
DType product_dtype(const Run& run, const Recognized& r) {
  return run.dtype_of(r.a.buffer) == DType::BF16 && run.dtype_of(r.b.buffer) == DType::BF16 ? DType::BF16 : DType::F32;
}

// The arithmetic of an attention: bf16 when Q, K and V all are; with an f32 operand among them the f32 kernels run
// and the bf16 operands are widened first (as for a product).
DType attention_dtype(const Run& run, const Recognized& r) {
  return run.dtype_of(r.a.buffer) == DType::BF16 && run.dtype_of(r.b.buffer) == DType::BF16 &&
                 run.dtype_of(r.c.buffer) == DType::BF16
             ? DType::BF16
             : DType::F32;
}

bool hand_usable(const Run& run, const Recognized& r) {
  // option generated.only = 1 runs every kernel in its generated form (used to test that path)
  if (run.knobs.generated_only) return false;
  auto rows_cols = [&](const Operand& o) { return run.shape_of(o.buffer); };
  switch (r.kind) {
    case Recognized::None: return false;
    case Recognized::Attention: {
      const DType t = attention_dtype(run, r);
      const auto q = rows_cols(r.a), v = rows_cols(r.c);
      if (q.size() < 2 || v.size() < 2) return false;
      if (ihip::attention_supported(t == DType::BF16 ? ihip::BF16 : ihip::F32, q.back(), v.back(), run.knobs)) return true;
      const auto k = rows_cols(r.b);
      if (k.size() < 2) return false;
      size_t bh = 1;
      for (size_t d = 0; d + 2 < q.size(); ++d) bh *= q[d];
      return attention_in_parts_usable(t, bh, q[q.size() - 2], k[k.size() - 2], q.back(), v.back());
    }
    case Recognized::GemmNT:
    case Recognized::GemmNN: {
      const auto a = rows_cols(r.a);
      if (a.size() < 2) return false;
      return product_extent_usable(product_dtype(run, r), a.back());
    }
    case Recognized::RowSoftmax:
    case Recognized::RowMaxShift:
    case Recognized::RowNormalize:
    case Recognized::RowExp: return true;
  }
  return false;
}

std::set<size_t> hand_intermediates(const Recognized& r) {
  std::set<size_t> out;
  auto add = [&](BufferRef b) {
    if (b.kind == BufferRef::Intermediate) out.insert(b.id);
  };
  add(r.out);
  add(r.a.buffer);
  if (r.kind == Recognized::Attention || r.kind == Recognized::GemmNT || r.kind == Recognized::GemmNN) add(r.b.buffer);
  if (r.kind == Recognized::Attention) {
    add(r.c.buffer);
    if (r.has_scale) add(r.scale.buffer);
  }
  return out;
}

// "attn_... (tile 256 x 64)", with the schedule's request spelled out when no kernel has that tile
std::string describe_launch(const ihip::LaunchNote& note, const Recognized& r) {
  std::string text = note.kernel;
  if (note.tile_i || note.tile_j) {
    text += " (tile " + std::to_string(note.tile_i) + " x " + std::to_string(note.tile_j);
    if ((r.tile_i || r.tile_j) && (r.tile_i != note.tile_i || r.tile_j != note.tile_j))
      text += "; the schedule asks for " + std::to_string(r.tile_i) + " x " + std::to_string(r.tile_j) +
              ", which no hand-written kernel has for these operands";
    text += ")";
  }
  return text;
}

// A product of bf16 operands whose result is a bf16 program output: the GEMM kernels write it themselves.
bool bf16_result_in_place(const Run& run, const Recognized& r) {
  return product_dtype(run, r) == DType::BF16 && r.out.kind == BufferRef::Output && run.outputs[r.out.id].dtype == DType::BF16;
}

// An f32 product through the executor: with few output tiles under a long k loop, the loop in parts over
// workgroups, the partial products in a temporary (no room for it: the unsplit kernel).
ihip::Err launch_product_f32(Run& run, const void* a, const void* b, void* c, size_t bh, size_t m, size_t n, size_t k,
                             ihip::LaunchNote* note) {
  void* partial = nullptr;
  unsigned splits = ihip::gemm_nt_f32_split_k(bh, m, n, k, run.knobs);
  if (splits > 1 && ((m * n) % 4 != 0 || !run.alloc_optional(&partial, bh * splits * m * n * 4))) splits = 1;
  return ihip::launch_gemm_nt_f32(static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(c), bh, m, n, k,
                                  run.stream, note, static_cast<float*>(partial), splits, run.knobs);
}

// Q, K and V in the arithmetic type of the attention: as they are, or read as f32 (bf16 ones widened into temporaries).
ihip::Err attention_operands(Run& run, const Recognized& r, bool bf16, const void** q, const void** k, const void** v) {
  if (bf16) {
    *q = run.raw_ptr(r.a.buffer);
    *k = run.raw_ptr(r.b.buffer);
    *v = run.raw_ptr(r.c.buffer);
    return {};
  }
  void *pq = nullptr, *pk = nullptr, *pv = nullptr;
  if (ihip::Err e = run.read_f32(r.a.buffer, &pq); !e.empty()) return e;
  if (ihip::Err e = run.read_f32(r.b.buffer, &pk); !e.empty()) return e;
  if (ihip::Err e = run.read_f32(r.c.buffer, &pv); !e.empty()) return e;
  *q = pq;
  *k = pk;
  *v = pv;
  return {};
}

// An operand that a kernel moving 16 bytes per lane cannot read where it lies (a view that starts off a 16-byte
// boundary): copied, element by element, into a temporary that it can.
ihip::Err aligned_copy(Run& run, const void** ptr, size_t bytes, size_t elem_bytes) {
  if (reinterpret_cast<uintptr_t>(*ptr) % 16 == 0 || bytes == 0) return {};
  void* tmp = nullptr;
  if (ihip::Err e = run.alloc(&tmp, bytes); !e.empty()) return e;
  if (ihip::Err e = ihip::launch_pad_rows(*ptr, tmp, 1, bytes / elem_bytes, bytes / elem_bytes, elem_bytes, run.stream); !e.empty()) return e;
  *ptr = tmp;
  return {};
}

ihip::Err attention_in_parts(Run& run, const Recognized& r, bool bf16, size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                             const float* scale_ptr, ihip::LaunchNote* note) {
  void* out = nullptr;
  if (ihip::Err e = run.write_f32(r.out, &out); !e.empty()) return e;
  void* scores = nullptr;  // [bh, nq, nk] f32: S, then P in place
  if (ihip::Err e = run.alloc(&scores, bh * nq * nk * 4); !e.empty()) return e;
  float* s = static_cast<float*>(scores);
  const void *q = nullptr, *k = nullptr, *v = nullptr;
  if (ihip::Err e = attention_operands(run, r, bf16, &q, &k, &v); !e.empty()) return e;
  ihip::LaunchNote first, middle, last;
  // (operands the kernels cannot read where they lie, for their alignment: aligned copies)
  if (ihip::Err e = aligned_copy(run, &q, bh * nq * d * (bf16 ? 2 : 4), bf16 ? 2 : 4); !e.empty()) return e;
  if (ihip::Err e = aligned_copy(run, &k, bh * nk * d * (bf16 ? 2 : 4), bf16 ? 2 : 4); !e.empty()) return e;
  if (ihip::Err e = aligned_copy(run, &v, bh * nk * dv * (bf16 ? 2 : 4), bf16 ? 2 : 4); !e.empty()) return e;
  if (ihip::Err e = bf16 ? ihip::launch_gemm_nt_bf16(q, k, s, bh, nq, nk, d, run.stream, 0, 0, &first, ihip::F32, run.knobs)
                         : ihip::launch_gemm_nt_f32(static_cast<const float*>(q), static_cast<const float*>(k), s, bh, nq, nk,
                                                    d, run.stream, &first, nullptr, 1, run.knobs);
      !e.empty())
    return e;
  if (ihip::Err e = ihip::launch_row_softmax(s, s, bh * nq, nk, run.stream, 4, &middle, scale_ptr, 1.0f); !e.empty()) return e;
  if (bf16) {
    void* pb = nullptr;  // the probabilities rounded to bf16, as the fused kernels round them
    if (ihip::Err e = run.alloc(&pb, bh * nq * nk * 2); !e.empty()) return e;
    if (ihip::Err e = ihip::launch_convert(s, pb, ihip::F32, ihip::BF16, bh * nq * nk, run.stream); !e.empty()) return e;
    if (ihip::gemm_nn_bf16_supported(bh, nq, dv, nk, run.knobs)) {
      if (ihip::Err e = ihip::launch_gemm_nn_bf16(pb, v, static_cast<float*>(out), bh, nq, dv, nk, run.stream, 0, 0, &last, ihip::F32,
                                                  nullptr, 1, run.knobs);
          !e.empty())
        return e;
    } else {
      void* vt = nullptr;
      if (ihip::Err e = run.alloc(&vt, bh * dv * nk * 2); !e.empty()) return e;
      if (ihip::Err e = ihip::launch_transpose(v, vt, bh, nk, dv, 2, run.stream); !e.empty()) return e;
      if (ihip::Err e = ihip::launch_gemm_nt_bf16(pb, vt, static_cast<float*>(out), bh, nq, dv, nk, run.stream, 0, 0, &last, ihip::F32,
                                                  run.knobs);
          !e.empty())
        return e;
    }
  } else {
    void* vt = nullptr;
    if (ihip::Err e = run.alloc(&vt, bh * dv * nk * 4); !e.empty()) return e;
    if (ihip::Err e = ihip::launch_transpose(v, vt, bh, nk, dv, 4, run.stream); !e.empty()) return e;
    if (ihip::Err e = launch_product_f32(run, s, vt, out, bh, nq, dv, nk, &last); !e.empty()) return e;
  }
  if (note) *note = ihip::LaunchNote{"attention in three kernels (head size beyond the fused kernels): " + first.kernel + ", " + middle.kernel + ", " + last.kernel, 0, 0};
  return {};
}

// The two operands of an NT product ([rows_a, k] and [rows_b, k], dense) as the matrix-instruction kernels can
// read them: untouched when k is a multiple of their quantum and both are 16-byte aligned, otherwise
// copied into stream-ordered temporaries with every row padded with zeros up to the next multiple; *k becomes the
// padded extent.
ihip::Err padded_operands(Run& run, DType t, const void** a, size_t rows_a, const void** b, size_t rows_b, size_t* k) {
  const size_t q = product_k_quantum(t), kp = (*k + q - 1) / q * q, elem = t == DType::BF16 ? 2 : 4;
  const bool misaligned = reinterpret_cast<uintptr_t>(*a) % 16 != 0 || reinterpret_cast<uintptr_t>(*b) % 16 != 0;
  if (kp == *k && !misaligned) return {};
  void *ta = nullptr, *tb = nullptr;
  if (ihip::Err e = run.alloc(&ta, std::max<size_t>(rows_a * kp * elem, 16)); !e.empty()) return e;
  if (ihip::Err e = run.alloc(&tb, std::max<size_t>(rows_b * kp * elem, 16)); !e.empty()) return e;
  if (ihip::Err e = ihip::launch_pad_rows(*a, ta, rows_a, *k, kp, elem, run.stream); !e.empty()) return e;
  if (ihip::Err e = ihip::launch_pad_rows(*b, tb, rows_b, *k, kp, elem, run.stream); !e.empty()) return e;
  *a = ta;
  *b = tb;
  *k = kp;
  return {};
}

// The operands of a product in its arithmetic type: as they are, or widened to f32 where the other one is f32.
ihip::Err product_operands(Run& run, const Recognized& r, DType t, const void** a, const void** b) {
  if (t == DType::BF16) {
    *a = run.raw_ptr(r.a.buffer);
    *b = run.raw_ptr(r.b.buffer);
    return {};
  }
  void *pa = nullptr, *pb = nullptr;
  if (ihip::Err e = run.read_f32(r.a.buffer, &pa); !e.empty()) return e;
  if (ihip::Err e = run.read_f32(r.b.buffer, &pb); !e.empty()) return e;
  *a = pa;
  *b = pb;
  return {};
}

ihip::Err launch_hand_noted(Run& run, const Recognized& r, ihip::LaunchNote* note) {
  switch (r.kind) {
    case Recognized::Attention: {
      const auto q = run.shape_of(r.a.buffer), k = run.shape_of(r.b.buffer), v = run.shape_of(r.c.buffer);
      const size_t nb = r.batch_rank;
      size_t bh = 1;
      for (size_t d = 0; d < nb; ++d) bh *= q[d];
      const size_t nq = q[nb], dq = q[nb + 1], nk = k[nb], dv = v[nb + 1];
      // repeated indexes constrain shapes; a mismatch would send the kernel out of bounds
      for (size_t d = 0; d < nb; ++d)
        if (k[d] != q[d] || v[d] != q[d]) return "attention operands disagree on a batch extent";
      if (k[nb + 1] != dq || v[nb] != nk) return "attention operands disagree on a contracted extent";
      const bool bf16 = attention_dtype(run, r) == DType::BF16;
      const float* scale_ptr = nullptr;
      if (r.has_scale) {
        void* sp = nullptr;
        if (ihip::Err e = run.read_f32(r.scale.buffer, &sp); !e.empty()) return e;
        scale_ptr = static_cast<const float*>(sp);
      }
      if (!ihip::attention_supported(bf16 ? ihip::BF16 : ihip::F32, dq, dv, run.knobs))
        return attention_in_parts(run, r, bf16, bh, nq, nk, dq, dv, scale_ptr, note);
      void* out = nullptr;
      ihip::DType out_dt = ihip::F32;
      if (bf16 && r.out.kind == BufferRef::Output && run.outputs[r.out.id].dtype == DType::BF16) {
        out = run.raw_ptr(r.out);
        out_dt = ihip::BF16;
      } else if (ihip::Err e = run.write_f32(r.out, &out); !e.empty()) {
        return e;
      }
      // an output view that the bf16 kernels cannot store to where it lies (they store 8 or 16 bytes per lane): the
      // result goes to an aligned temporary and is copied out, element by element, after the launch
      void* out_view = nullptr;
      const size_t out_elem = out_dt == ihip::BF16 ? 2 : 4;
      if (bf16 && reinterpret_cast<uintptr_t>(out) % (out_dt == ihip::BF16 ? 8 : 16) != 0) {
        out_view = out;
        if (ihip::Err e = run.alloc(&out, bh * nq * dv * out_elem); !e.empty()) return e;
      }
      ihip::AttentionOptions options{r.tile_i, r.tile_j, run.knobs};
      // few workgroups under a long key loop (a single head, a few long sequences): the keys of a head in parts
      // over workgroups, each part's result in a temporary (no room for it: the unsplit kernel)
      if (const unsigned splits = ihip::attention_kv_splits(bf16 ? ihip::BF16 : ihip::F32, bh, nq, nk, dq, dv, options); splits > 1) {
        void* partial = nullptr;  // the parts' results, then their row sums' logarithms
        const size_t rows = bh * splits * nq;
        if (run.alloc_optional(&partial, rows * dv * 4 + rows * 4)) {
          options.kv_splits = splits;
          options.partial_o = static_cast<float*>(partial);
          options.partial_lse = static_cast<float*>(partial) + rows * dv;
        }
      }
      const void *pq = nullptr, *pk = nullptr, *pv = nullptr;
      if (ihip::Err e = attention_operands(run, r, bf16, &pq, &pk, &pv); !e.empty()) return e;
      if (bf16) {  // (f32 operands off a 16-byte boundary take the register-staged f32 kernel, which reads element by element)
        if (ihip::Err e = aligned_copy(run, &pq, bh * nq * dq * 2, 2); !e.empty()) return e;
        if (ihip::Err e = aligned_copy(run, &pk, bh * nk * dq * 2, 2); !e.empty()) return e;
        if (ihip::Err e = aligned_copy(run, &pv, bh * nk * dv * 2, 2); !e.empty()) return e;
      }
      if (ihip::Err e = ihip::launch_attention(pq, pk, pv, out, bf16 ? ihip::BF16 : ihip::F32, out_dt, bh, nq, nk, dq, dv, scale_ptr,
                                               1.0f, run.stream, options, note);
          !e.empty() || !out_view)
        return e;
      return ihip::launch_pad_rows(out, out_view, 1, bh * nq * dv, bh * nq * dv, out_elem, run.stream);
    }
    case Recognized::GemmNT: {
      const auto a = run.shape_of(r.a.buffer), b = run.shape_of(r.b.buffer);
      const size_t nb = r.batch_rank;
      size_t bh = 1;
      for (size_t d = 0; d < nb; ++d) {
        if (b[d] != a[d]) return "gemm operands disagree on a batch extent";
        bh *= a[d];
      }
      if (b[nb + 1] != a[nb + 1]) return "gemm operands disagree on the contracted extent";
      void* out = nullptr;
      ihip::DType out_dt = ihip::F32;
      if (bf16_result_in_place(run, r)) {  // the kernel rounds its f32 sums to the bf16 output itself
        out = run.raw_ptr(r.out);
        out_dt = ihip::BF16;
      } else if (ihip::Err e = run.write_f32(r.out, &out); !e.empty()) {
        return e;
      }
      const DType t = product_dtype(run, r);
      const void *pa = nullptr, *pb = nullptr;
      if (ihip::Err e = product_operands(run, r, t, &pa, &pb); !e.empty()) return e;
      size_t k = a[nb + 1];
      if (ihip::Err e = padded_operands(run, t, &pa, bh * a[nb], &pb, bh * b[nb], &k); !e.empty()) return e;
      if (t == DType::F32) return launch_product_f32(run, pa, pb, out, bh, a[nb], b[nb], k, note);
      // few output tiles under a long k loop: the loop is split over workgroups, partial products in a temporary
      // (unless the schedule names one of the kernels' own tiles: then that kernel runs as asked)
      const bool tile_asked = (r.tile_i == 128 && r.tile_j == 128) || (r.tile_i == 256 && r.tile_j == 256);
      if (const unsigned splits = tile_asked && run.knobs.gemm_k_parts < 2 ? 1u : ihip::gemm_nt_bf16_split_k(bh, a[nb], b[nb], k, run.knobs);
          splits > 1 && (a[nb] * b[nb]) % 4 == 0) {
        void* partial = nullptr;
        if (run.alloc_optional(&partial, bh * splits * a[nb] * b[nb] * 4))  // (no room for it: the unsplit kernel)
          return ihip::launch_gemm_nt_bf16_split_k(pa, pb, out, static_cast<float*>(partial), splits, bh, a[nb], b[nb], k, run.stream,
                                                   note, out_dt);
      }
      return ihip::launch_gemm_nt_bf16(pa, pb, out, bh, a[nb], b[nb], k, run.stream, r.tile_i, r.tile_j, note, out_dt, run.knobs);
    }
    case Recognized::GemmNN: {
      // b [B.., K, J]: the direct bf16 kernels read it in place; otherwise it is transposed into a stream-ordered
      // temporary [B.., J, K] and the NT kernel runs
      const auto a = run.shape_of(r.a.buffer), b = run.shape_of(r.b.buffer);
      const size_t nb = r.batch_rank;
      size_t bh = 1;
      for (size_t d = 0; d < nb; ++d) {
        if (b[d] != a[d]) return "gemm operands disagree on a batch extent";
        bh *= a[d];
      }
      const size_t m = a[nb], k = a[nb + 1], n = b[nb + 1];
      if (b[nb] != k) return "gemm operands disagree on the contracted extent";
      const bool f32 = product_dtype(run, r) == DType::F32;
      void* out = nullptr;
      ihip::DType out_dt = ihip::F32;
      if (bf16_result_in_place(run, r)) {
        out = run.raw_ptr(r.out);
        out_dt = ihip::BF16;
      } else if (ihip::Err e = run.write_f32(r.out, &out); !e.empty()) {
        return e;
      }
      const void *pa = nullptr, *pb_rows = nullptr;
      if (ihip::Err e = product_operands(run, r, f32 ? DType::F32 : DType::BF16, &pa, &pb_rows); !e.empty()) return e;
      if (!f32 && ihip::gemm_nn_bf16_supported(bh, m, n, k, run.knobs) && reinterpret_cast<uintptr_t>(pa) % 16 == 0 &&
          reinterpret_cast<uintptr_t>(pb_rows) % 16 == 0) {  // the direct kernels read a row-major right operand themselves
        const bool tile_asked = (r.tile_i == 128 && r.tile_j == 128) || (r.tile_i == 256 && r.tile_j == 256);
        unsigned splits = tile_asked && run.knobs.gemm_k_parts < 2 ? 1u : ihip::gemm_nt_bf16_split_k(bh, m, n, k, run.knobs);
        void* partial = nullptr;
        if (splits > 1 && ((m * n) % 4 != 0 || !run.alloc_optional(&partial, bh * splits * m * n * 4))) splits = 1;
        return ihip::launch_gemm_nn_bf16(pa, pb_rows, out, bh, m, n, k, run.stream, r.tile_i, r.tile_j, note, out_dt,
                                         static_cast<float*>(partial), splits, run.knobs);
      }
      const size_t elem = f32 ? 4 : 2;
      void* bt = nullptr;
      if (ihip::Err e = run.alloc(&bt, bh * n * k * elem); !e.empty()) return e;
      if (ihip::Err e = ihip::launch_transpose(pb_rows, bt, bh, k, n, elem, run.stream); !e.empty()) return e;
      const void* pb = bt;
      size_t kp = k;
      if (ihip::Err e = padded_operands(run, f32 ? DType::F32 : DType::BF16, &pa, bh * m, &pb, bh * n, &kp); !e.empty()) return e;
      if (f32) return launch_product_f32(run, pa, pb, out, bh, m, n, kp, note);
      return ihip::launch_gemm_nt_bf16(pa, pb, out, bh, m, n, kp, run.stream, r.tile_i, r.tile_j, note, out_dt, run.knobs);
    }
    case Recognized::RowSoftmax:
    case Recognized::RowMaxShift:
    case Recognized::RowNormalize:
    case Recognized::RowExp: {
      const auto x = run.shape_of(r.a.buffer);
      size_t rows = 1;
      for (size_t d = 0; d + 1 < x.size(); ++d) rows *= x[d];
      void *in = nullptr, *out = nullptr;
      if (ihip::Err e = run.read_f32(r.a.buffer, &in); !e.empty()) return e;
      if (ihip::Err e = run.write_f32(r.out, &out); !e.empty()) return e;
      const int mode = r.kind == Recognized::RowSoftmax ? 0 : r.kind == Recognized::RowMaxShift ? 1 : r.kind == Recognized::RowNormalize ? 2 : 3;
      // a few very long rows: every row in parts over workgroups, the parts' (max, sum) pairs in a small temporary
      unsigned parts = ihip::row_softmax_parts(rows, x.back(), mode);
      void* stats = nullptr;
      if (parts > 1 && !run.alloc(&stats, rows * parts * 8).empty()) parts = 1;
      return ihip::launch_row_softmax(static_cast<const float*>(in), static_cast<float*>(out), rows, x.back(), run.stream, mode, note,
                                      nullptr, 1.0f, static_cast<float*>(stats), parts);
    }
    default: return "no hand-written kernel";
  }
}

ihip::Err launch_hand(Run& run, const Recognized& r) {
  ihip::LaunchNote note;
  const ihip::Err err = launch_hand_noted(run, r, &note);
  if (err.empty()) run.notes.push_back(note.kernel.empty() ? "nothing to do (empty operands)" : describe_launch(note, r));
  return err;
}

// ---------------------------------------------------------------- generated kernels
ihip::Err ensure_image(Program& p) {
  std::lock_guard<std::mutex> lock(p.mu);
  if (p.image_built) return {};
  if (p.generic.source.empty()) return "program has no generated kernels";
  if (std::string e = hipcc_build(p.generic.source, &p.image); !e.empty()) return e;
  p.image_built = true;
  return {};
}

ihip::Err generic_function(Program& p, const std::string& name, hipFunction_t* fn) {
  if (ihip::Err e = ensure_image(p); !e.empty()) return e;
  std::lock_guard<std::mutex> lock(p.mu);
  int dev = 0;
  if (ihip::Err e = ihip::check(hipGetDevice(&dev), "hipGetDevice"); !e.empty()) return e;
  auto it = p.modules.find(dev);
  if (it == p.modules.end()) {
    hipModule_t mod = nullptr;
    if (ihip::Err e = ihip::load_module(p.image.data(), &mod); !e.empty()) return e;
    it = p.modules.emplace(dev, mod).first;
  }
  return ihip::module_function(it->second, name.c_str(), fn);
}

// Into how many parts to deal out the outermost sequential loop of a generated nest (1: the nest as it is).
// `total` counts the iterations of its parallel loops, `reduced` those of the loop in question, `wave` says which of
// the two forms (a work-item or a wavefront per iteration) would run.  Parts pay when the parallel loops alone leave
// most of the chip idle: enough of them for 16 wavefronts per compute unit, each part with at least 16 iterations of
// a loop that a work-item runs by itself, 4 rounds of the 64 lanes when the loop in parts is the one over the lanes,
// one iteration when the lanes run over a loop inside it; at most 4096, from 16 on a multiple of 8 and from 256 on
// of 32 (the copies of buffers of 64 elements and more are then folded in two passes).
size_t generated_parts(const ihip::KernelOptions& knobs, const GridForm& grid, bool wave, size_t total, size_t reduced) {
  if (!grid.available || (wave && !grid.wave) || knobs.generated_parts == 1 || total == 0) return 1;
  const size_t least = !wave ? 16 : grid.loop_is_spread ? 256 : 1;
  size_t parts;
  if (knobs.generated_parts > 1) {
    parts = (size_t)knobs.generated_parts;
  } else {
    const size_t target = wave ? 4096 : 262144;  // wavefronts / work-items that fill the chip
    if (total * 2 > target) return 1;
    parts = std::min<size_t>(target / total, reduced / least);
  }
  // (at most 4096 parts; 2048 of wavefronts when left to this rule: the pass over the parts of a sum to one element
  // is one wavefront's work and grows with their number, 4096^2 to one element 29.7 us in 4096 parts, 23.8 in 2048)
  parts = std::min<size_t>(std::min<size_t>(parts, wave && knobs.generated_parts <= 1 ? 2048 : 4096), std::max<size_t>(reduced, 1));
  if (parts >= 256) parts = parts / 32 * 32;
  else if (parts >= 16) parts = parts / 8 * 8;
  return parts < 2 ? 1 : parts;
}

ihip::Err launch_generic(Run& run, size_t k, const Step& dispatch) {
  Program& p = run.p;
  const GenericKernel& gk = p.generic.kernels[k];
  if (gk.name.empty() || gk.phases.size() != 1) return "kernel " + std::to_string(k) + " has no generated form";
  const GenericPhase& ph = gk.phases[0];
  const size_t R = p.generic.rank;
  const size_t view_bytes = 8 + 16 * R;
  const size_t nr = std::max<size_t>(gk.n_reads, 1), nw = std::max<size_t>(gk.n_writes, 1);
  std::vector<unsigned char> args((nr + nw) * view_bytes, 0);
  if (args.size() + 8 * nw + 8 > 4000) return "kernel " + std::to_string(k) + " takes too many buffers for one launch";

  auto fill = [&](size_t slot, void* data, BufferRef r) {
    unsigned char* v = args.data() + slot * view_bytes;
    std::memcpy(v, &data, 8);
    const auto shape = run.shape_of(r), layout = run.layout_of(r);
    for (size_t d = 0; d < shape.size() && d < R; ++d) std::memcpy(v + 8 + 8 * d, &shape[d], 8);
    for (size_t d = 0; d < layout.size() && d < R; ++d) std::memcpy(v + 8 + 8 * R + 8 * d, &layout[d], 8);
  };
  for (size_t i = 0; i < dispatch.reads.size(); ++i) {
    void* ptr = nullptr;
    if (ihip::Err e = run.read_f32(dispatch.reads[i], &ptr); !e.empty()) return e;
    fill(i, ptr, dispatch.reads[i]);
  }
  std::vector<void*> write_ptrs(dispatch.writes.size(), nullptr);
  for (size_t i = 0; i < dispatch.writes.size(); ++i) {
    if (!gk.is_private(i))
      if (ihip::Err e = run.write_f32(dispatch.writes[i], &write_ptrs[i]); !e.empty()) return e;
    fill(nr + i, write_ptrs[i], dispatch.writes[i]);
  }
  auto extent_of = [&](const Extent<Param>& e) {
    const BufferRef src = e.source.buffer.writeable ? dispatch.writes.at(e.source.buffer.ind) : dispatch.reads.at(e.source.buffer.ind);
    return run.extent(Extent<size_t>{plan_buffer(run.plan, src).shape.at(e.source.dim), e.kind});
  };
  run.notes.push_back("generated kernel " + gk.name);
  size_t total = 1;
  for (const auto& e : ph.parallel_extents) total *= extent_of(e);
  if (total == 0) return {};
  // The wavefront-per-iteration form (reduction loops spread over 64 lanes), when the nest has one: taken when
  // the reduction is long enough to occupy the lanes and either consecutive lanes read consecutive elements
  // or there are too few iterations to fill the chip with one work-item each.  Option generated.wave = 0 | 1 overrides.
  bool wave = false;
  if (!ph.wave_loops.empty()) {
    const size_t reduced = extent_of(ph.wave_extent);
    // (a nest with a form in parts fills the chip with work-items, whose lanes read along the parallel index)
    wave = reduced >= 128 && (ph.wave_contiguous || (total < 65536 && !ph.grid.available));
    if (run.knobs.generated_wave >= 0) wave = run.knobs.generated_wave == 1;
  }
  bool dynamic_private = false;  // (per-work-item slices of a device buffer are sized for the plain form's grid)
  for (const PrivateBuffer& pb : ph.privates) dynamic_private = dynamic_private || !pb.is_static;
  const size_t parts = dynamic_private ? 1 : generated_parts(run.knobs, ph.grid, wave, total, ph.grid.available ? extent_of(ph.grid.extent) : 0);
  hipFunction_t fn;
  if (parts > 1) {
    // every part accumulates into a copy of its own of each accumulated buffer (filled with the reduction's
    // identity first); ilang_combine folds the copies into the buffer afterwards
    std::vector<size_t> counts;
    size_t floats = 0;
    for (const GridAccumulator& acc : ph.grid.accumulators) {
      counts.push_back(std::max<size_t>(1, product(run.layout_of(dispatch.writes.at(acc.writeable)))));
      floats += counts.back() * parts;
    }
    // How the copies fold.  A buffer of fewer than 64 elements: one pass, a wavefront per element with its lanes
    // over the parts.  Larger ones: a work-item per element, and from 16 parts on in two passes (the copies, read as
    // [parts / w][w * count], fold into w = 8 or 32 copies first), which puts w times as many work-items on the
    // first pass.
    const size_t width = parts >= 256 && parts % 32 == 0 ? 32 : parts >= 16 && parts % 8 == 0 ? 8 : 0;
    size_t most = 0;
    for (size_t c : counts)
      if (c >= 64) most = std::max(most, c);
    const bool two_passes = width != 0 && most != 0;
    if (two_passes) floats += width * most;
    void* partial = nullptr;
    if (run.alloc_optional(&partial, floats * 4)) {
      std::vector<unsigned char> gargs(args);
      gargs.resize(args.size() + 8 * nw + 8, 0);
      float* at = static_cast<float*>(partial);
      struct FillArgs { float* data; size_t count; float value; };
      struct CombineArgs { const float* partial; float* data; size_t parts; size_t count; int op; int keep; };
      hipFunction_t fill_fn, combine_fn, combine_wave_fn;
      if (ihip::Err e = generic_function(p, kFillKernel, &fill_fn); !e.empty()) return e;
      if (ihip::Err e = generic_function(p, kCombineKernel, &combine_fn); !e.empty()) return e;
      if (ihip::Err e = generic_function(p, kCombineWaveKernel, &combine_wave_fn); !e.empty()) return e;
      std::vector<std::pair<CombineArgs, bool>> combines;  // (arguments, a wavefront per element)
      float* const folded = static_cast<float*>(partial) + (floats - (two_passes ? width * most : 0));
      for (size_t a = 0; a < ph.grid.accumulators.size(); ++a) {
        const GridAccumulator& acc = ph.grid.accumulators[a];
        std::memcpy(gargs.data() + args.size() + 8 * acc.writeable, &at, 8);
        const float identity = acc.op == Op::Mul ? 1.0f : acc.op == Op::Max ? -INFINITY : acc.op == Op::Min ? INFINITY : 0.0f;
        // (the parts store every element of their copies themselves when the accumulators live in registers and the
        // buffer has no padding that no work-item owns)
        const bool dense = product(run.shape_of(dispatch.writes.at(acc.writeable))) == counts[a];
        if (!(ph.grid.held_accumulators && dense)) {
          FillArgs fa{at, counts[a] * parts, identity};
          const size_t fgrid = std::min<size_t>((fa.count + 255) / 256, 4096);
          if (ihip::Err e = ihip::launch(fill_fn, (unsigned)fgrid, 1, 1, 256, &fa, sizeof(fa), run.stream); !e.empty()) return e;
        }
        const int op = acc.op == Op::Add ? 0 : acc.op == Op::Mul ? 1 : acc.op == Op::Max ? 2 : 3;
        float* const dst = static_cast<float*>(write_ptrs.at(acc.writeable));
        if (counts[a] < 64) {
          combines.push_back({{at, dst, parts, counts[a], op, acc.init_here ? 0 : 1}, true});
        } else if (two_passes) {
          combines.push_back({{at, folded, parts / width, width * counts[a], op, 0}, false});
          combines.push_back({{folded, dst, width, counts[a], op, acc.init_here ? 0 : 1}, false});
        } else {
          combines.push_back({{at, dst, parts, counts[a], op, acc.init_here ? 0 : 1}, false});
        }
        at += counts[a] * parts;
      }
      std::memcpy(gargs.data() + args.size() + 8 * nw, &parts, 8);
      const std::string name = ph.name + (wave ? "_gw" : "_g");
      if (ihip::Err e = generic_function(p, name, &fn); !e.empty()) return e;
      run.notes.back() += ", as " + name + ": the outermost sequential loop in " + std::to_string(parts) + " parts over " +
                          (wave ? "wavefronts" : "work-items") + ", combined by " + kCombineKernel;
      const size_t units = total * parts;
      const unsigned per_group = wave ? GenericPhase::kWaveThreads / 64 : 64;
      const size_t groups = std::min<size_t>((units + per_group - 1) / per_group, size_t(1) << 20);
      if (ihip::Err e = ihip::launch(fn, (unsigned)groups, 1, 1, wave ? GenericPhase::kWaveThreads : 64, gargs.data(), gargs.size(), run.stream);
          !e.empty())
        return e;
      for (const auto& [ca, by_wave] : combines) {
        const size_t cgrid = std::min<size_t>(by_wave ? (ca.count + 3) / 4 : (ca.count + 255) / 256, 4096);
        if (ihip::Err e = ihip::launch(by_wave ? combine_wave_fn : combine_fn, (unsigned)cgrid, 1, 1, 256, &ca, sizeof(ca), run.stream);
            !e.empty())
          return e;
      }
      return {};
    }
  }
  if (wave) {
    const size_t waves = std::min<size_t>(total, size_t(1) << 16);
    const unsigned per_group = GenericPhase::kWaveThreads / 64;
    for (const PrivateBuffer& pb : ph.privates) fill(nr + pb.writeable, nullptr, dispatch.writes[pb.writeable]);
    if (ihip::Err err = generic_function(p, ph.name + "_w", &fn); !err.empty()) return err;
    run.notes.back() += ", as " + ph.name + "_w: one wavefront per iteration of the parallel loops";
    return ihip::launch(fn, (unsigned)((waves + per_group - 1) / per_group), 1, 1, GenericPhase::kWaveThreads, args.data(), args.size(),
                        run.stream);
  }
  size_t threads = ph.parallel_loops.empty() ? 1 : total;
  // dynamic private buffers cost memory per work-item slot: cap the slots
  size_t slot_elems = 0;
  for (const PrivateBuffer& pb : ph.privates)
    if (!pb.is_static) slot_elems += std::max<size_t>(1, product(run.layout_of(dispatch.writes[pb.writeable])));
  size_t max_threads = size_t(1) << 20;
  if (slot_elems) max_threads = std::max<size_t>(64, std::min(max_threads, (size_t(1) << 28) / (slot_elems * 4)));
  threads = std::min(threads, max_threads);
  const unsigned grid = (unsigned)((threads + 63) / 64);
  const size_t slots = (size_t)grid * 64;
  for (const PrivateBuffer& pb : ph.privates) {
    void* ptr = nullptr;
    if (!pb.is_static) {
      const size_t n = std::max<size_t>(1, product(run.layout_of(dispatch.writes[pb.writeable])));
      if (ihip::Err e = run.alloc(&ptr, n * slots * 4); !e.empty()) return e;
    }
    fill(nr + pb.writeable, ptr, dispatch.writes[pb.writeable]);
  }
  if (ihip::Err e = generic_function(p, ph.name, &fn); !e.empty()) return e;
  return ihip::launch(fn, grid, 1, 1, 64, args.data(), args.size(), run.stream);
}

const Step* find_dispatch(const ExecPlan& plan, size_t k) {
  for (const Step& s : plan.exec)
    if (s.kind == Step::Dispatch && s.id == k) return &s;
  return nullptr;
}

// Which dimensions of which program inputs every index symbol of every expression stands for.  An operand of a
// node is a program input or another node's result; a result dimension stands for whatever its output symbol
// stands for, so the groups carry through chains of expressions.
std::vector<std::vector<std::pair<size_t, size_t>>> tied_extents(const Graph<Node>& graph) {
  using Dims = std::set<std::pair<size_t, size_t>>;
  std::vector<std::vector<Dims>> result_dims(graph.nodes.size());
  std::vector<char> state(graph.nodes.size(), 0);  // 0 not visited, 1 in progress, 2 done
  std::set<std::vector<std::pair<size_t, size_t>>> groups;
  std::function<void(size_t)> visit = [&](size_t n) {
    if (state[n] != 0) return;  // done, or a cycle (which lowering has rejected)
    state[n] = 1;
    const GNode<Node>& g = graph.nodes[n];
    const Node& node = g.inner;
    std::vector<Dims> of_symbol(node.rank);
    for (size_t o = 0; o < node.inputs.size() && o < g.inputs.size(); ++o) {
      const Source& src = g.inputs[o];
      if (!src.is_input && src.id < graph.nodes.size()) visit(src.id);
      for (size_t pos = 0; pos < node.inputs[o].size(); ++pos) {
        const size_t symbol = node.inputs[o][pos];
        if (symbol >= of_symbol.size()) continue;
        if (src.is_input) of_symbol[symbol].insert({src.id, pos});
        else if (src.id < graph.nodes.size() && pos < result_dims[src.id].size())
          of_symbol[symbol].insert(result_dims[src.id][pos].begin(), result_dims[src.id][pos].end());
      }
    }
    for (const Dims& d : of_symbol)
      if (d.size() > 1) groups.insert(std::vector<std::pair<size_t, size_t>>(d.begin(), d.end()));
    for (size_t symbol : node.output) result_dims[n].push_back(symbol < of_symbol.size() ? of_symbol[symbol] : Dims{});
    state[n] = 2;
  };
  for (size_t n = 0; n < graph.nodes.size(); ++n) visit(n);
  return {groups.begin(), groups.end()};
}

// See row_sliceable() in the header.  The dimension sets are those of tied_extents above, kept per symbol of every
// node: a symbol stands for the (input, dimension) pairs of the operand dimensions it indexes, and a result
// dimension for those of its output symbol.
bool row_slices_of(const Graph<Node>& graph, std::vector<char>* sliced) {
  using Dims = std::set<std::pair<size_t, size_t>>;
  std::vector<std::vector<Dims>> result_dims(graph.nodes.size()), symbol_dims(graph.nodes.size());
  std::vector<char> state(graph.nodes.size(), 0);
  std::function<void(size_t)> visit = [&](size_t n) {
    if (state[n] != 0) return;
    state[n] = 1;
    const GNode<Node>& g = graph.nodes[n];
    const Node& node = g.inner;
    std::vector<Dims>& of_symbol = symbol_dims[n];
    of_symbol.assign(node.rank, {});
    for (size_t o = 0; o < node.inputs.size() && o < g.inputs.size(); ++o) {
      const Source& src = g.inputs[o];
      if (!src.is_input && src.id < graph.nodes.size()) visit(src.id);
      for (size_t pos = 0; pos < node.inputs[o].size(); ++pos) {
        const size_t symbol = node.inputs[o][pos];
        if (symbol >= of_symbol.size()) continue;
        if (src.is_input) of_symbol[symbol].insert({src.id, pos});
        else if (src.id < graph.nodes.size() && pos < result_dims[src.id].size())
          of_symbol[symbol].insert(result_dims[src.id][pos].begin(), result_dims[src.id][pos].end());
      }
    }
    for (size_t symbol : node.output) result_dims[n].push_back(symbol < of_symbol.size() ? of_symbol[symbol] : Dims{});
    state[n] = 2;
  };
  for (size_t n = 0; n < graph.nodes.size(); ++n) visit(n);
  // the leading index: the same for every output, and first dimensions of inputs only
  Dims leading;
  if (graph.outputs.empty()) return false;
  for (size_t o = 0; o < graph.outputs.size(); ++o) {
    const Source& out = graph.outputs[o];
    if (out.is_input || out.id >= graph.nodes.size() || result_dims[out.id].empty()) return false;
    if (o == 0) leading = result_dims[out.id][0];
    else if (result_dims[out.id][0] != leading) return false;
  }
  if (leading.empty()) return false;
  for (const auto& [input, pos] : leading)
    if (pos != 0 || input >= graph.inputs) return false;
  auto tied = [&](const Dims& d) {
    for (const auto& pair : d)
      if (leading.count(pair)) return true;
    return false;
  };
  // no expression reduces over it, none has it under two names
  for (size_t n = 0; n < graph.nodes.size(); ++n) {
    const Node& node = graph.nodes[n].inner;
    size_t names = 0;
    for (size_t symbol = 0; symbol < symbol_dims[n].size(); ++symbol) {
      if (!tied(symbol_dims[n][symbol])) continue;
      ++names;
      if (std::find(node.output.begin(), node.output.end(), symbol) == node.output.end()) return false;
    }
    if (names > 1) return false;
  }
  sliced->assign(graph.inputs, 0);
  for (const auto& pair : leading) (*sliced)[pair.first] = 1;
  return true;
}

}  // namespace

Program::~Program() {
  for (auto& kv : modules) ihip::unload_module(kv.second);
}

std::string compile_program(const Component& component, Program** out) {
  auto p = std::make_unique<Program>();
  p->low = lower_component(component);
  p->module = lower_exec_plan_to_module(p->low.plan);
  p->recognized = recognize_kernels(p->low);
  p->same_extent = tied_extents(p->low.graph);
  p->row_sliceable = row_slices_of(p->low.graph, &p->row_sliced);
  if (p->recognized.size() != p->low.plan.kernels.size()) lower_error("kernel recognition lost track of the kernel list");
  // the generated form: one kernel per loop nest
  std::vector<size_t> origin;
  p->nest_plan = split_nests(p->low.plan, &origin);
  p->nests_of.assign(p->low.plan.kernels.size(), {});
  for (size_t n = 0; n < origin.size(); ++n) p->nests_of.at(origin[n]).push_back(n);
  p->generic = emit_generic_hip(p->nest_plan, lower_exec_plan_to_module(p->nest_plan), std::vector<bool>(p->nest_plan.kernels.size(), true));
  bool needs_generated = false;
  for (const Recognized& r : p->recognized) needs_generated |= r.kind == Recognized::None;
  if (needs_generated)
    if (ihip::Err e = ensure_image(*p); !e.empty()) return e;
  *out = p.release();
  return {};
}

std::string program_code(const Component& component) {
  const Lowered low = lower_component(component);
  const Module module = lower_exec_plan_to_module(low.plan);
  const auto rec = recognize_kernels(low);
  std::vector<size_t> origin;
  const ExecPlan nest_plan = split_nests(low.plan, &origin);
  const GenericModule gen = emit_generic_hip(nest_plan, lower_exec_plan_to_module(nest_plan), std::vector<bool>(nest_plan.kernels.size(), true));
  (void)module;
  std::ostringstream os;
  os << "// 𝚒 gfx950 backend plan: " << low.plan.inputs.size() << " input(s), " << low.plan.intermediates.size()
     << " intermediate(s), " << low.plan.outputs.size() << " output(s), " << low.plan.kernels.size() << " kernel(s)\n";
  for (size_t k = 0; k < low.plan.kernels.size(); ++k) {
    const Step* d = find_dispatch(low.plan, k);
    os << "// f" << k << ": " << rec[k].describe();
    if (rec[k].kind != Recognized::None) {
      os << " [";
      os << ref_name(rec[k].a.buffer);
      if (rec[k].kind == Recognized::Attention || rec[k].kind == Recognized::GemmNT || rec[k].kind == Recognized::GemmNN)
        os << ", " << ref_name(rec[k].b.buffer);
      if (rec[k].kind == Recognized::Attention) os << ", " << ref_name(rec[k].c.buffer);
      if (rec[k].has_scale) os << ", scale " << ref_name(rec[k].scale.buffer);
      os << " -> " << ref_name(rec[k].out) << "]; generated form below runs when operands are outside its limits";
    }
    if (rec[k].kind == Recognized::Attention || rec[k].kind == Recognized::GemmNT || rec[k].kind == Recognized::GemmNN) {
      // which of the schedule's tiles exist as kernels is a property of the kernel set, known here; which one
      // runs also depends on the operands (head size, dtype, problem size) and is reported after a run
      const size_t ti = rec[k].tile_i, tj = rec[k].tile_j;
      const bool attn = rec[k].kind == Recognized::Attention;
      const bool known = attn ? (((ti == 64 || ti == 128 || ti == 256) && (tj == 32 || tj == 64)) || (ti == 512 && tj == 32))
                              : ((ti == 128 && tj == 128) || (ti == 256 && tj == 256) ||
                                 (ti + tj == 448 && (ti == 192 || ti == 256) && rec[k].kind == Recognized::GemmNT));
      os << "\n//     " << (known ? "the schedule tile selects the kernel with that workgroup tile where the operands allow it"
                                   : "no hand-written kernel has this tile: the launcher picks one by problem size")
         << (attn ? " (attention tiles: 64 / 128 / 256 query rows x 32 / 64 keys, 512 x 32 at d = 64)"
                  : " (GEMM tiles: 128 x 128, 256 x 256; 192 x 256 and 256 x 192 for a K-contiguous right operand)")
         << "; i_hip_program_report names the kernel that ran";
    }
    os << "\n//     reads";
    for (BufferRef r : d->reads) os << " " << ref_name(r);
    os << "; writes";
    for (BufferRef r : d->writes) os << " " << ref_name(r);
    // the generated form: one kernel per loop nest of the kernel (their names are those of the source below)
    size_t nests = 0;
    for (size_t n = 0; n < origin.size(); ++n) nests += origin[n] == k;
    for (size_t n = 0; n < origin.size(); ++n) {
      if (origin[n] != k || gen.kernels[n].phases.empty()) continue;
      const GenericPhase& ph = gen.kernels[n].phases[0];
      const Step* nd = find_dispatch(nest_plan, n);
      os << "\n//     ";
      if (nests > 1) os << "loop nest as kernel " << ph.name << ", ";
      else os << "generated as " << ph.name << ", ";
      os << "work-items:";
      if (ph.parallel_loops.empty()) os << " 1 (no independent outer loop)";
      for (size_t id : ph.parallel_loops) os << " i" << id;
      if (!ph.privates.empty()) {
        os << "; work-item-private:";
        for (const auto& pb : ph.privates)
          os << " " << ref_name(nd->writes[pb.writeable]) << (pb.is_static ? "[" + std::to_string(pb.static_size) + "]" : "[dynamic]");
      }
      if (!ph.wave_loops.empty()) {
        os << "\n//     " << ph.name << "_w, one wavefront per work-item of the above (long reductions): over its lanes";
        for (const WaveLoop& wl : ph.wave_loops) os << " i" << wl.loop;
      }
      if (ph.grid.available)
        os << "\n//     " << ph.name << "_g" << (ph.grid.wave ? " / " + ph.name + "_gw" : "") << ", loop i" << ph.grid.loop
           << " in parts over groups of work-items (grids that the parallel loops alone leave mostly idle), the parts combined by "
           << kCombineKernel;
    }
    os << "\n";
  }
  os << "\n" << gen.source;
  return os.str();
}

bool row_sliceable(const Program& p, std::vector<char>* sliced) {
  if (p.row_sliceable && sliced) *sliced = p.row_sliced;
  return p.row_sliceable;
}

size_t output_count(const Program& p) { return p.low.plan.count; }
std::vector<size_t> output_ranks(const Program& p) { return p.low.plan.ranks; }
size_t input_count(const Program& p) { return p.low.plan.inputs.size(); }
size_t input_rank(const Program& p, size_t input) { return p.low.plan.inputs.at(input).shape.size(); }

std::string output_shapes(const Program& p, const std::vector<std::vector<size_t>>& input_shapes,
                          std::vector<std::vector<size_t>>* shapes) {
  shapes->clear();
  for (const auto& shape : p.low.plan.shapes) {
    std::vector<size_t> out;
    for (const auto& d : shape) {
      if (d.buffer >= input_shapes.size()) return "program needs input " + std::to_string(d.buffer) + " to size its outputs";
      if (d.dim >= input_shapes[d.buffer].size())
        return "input " + std::to_string(d.buffer) + " has rank " + std::to_string(input_shapes[d.buffer].size()) +
               ", program reads dimension " + std::to_string(d.dim);
      out.push_back(input_shapes[d.buffer][d.dim]);
    }
    shapes->push_back(std::move(out));
  }
  return {};
}

std::string execute(Program& p, const std::vector<DeviceTensor>& inputs, const std::vector<DeviceTensor>& outputs,
                    hipStream_t stream, Workspace* workspace) {
  const ExecPlan& plan = p.low.plan;
  if (inputs.size() < plan.inputs.size())
    return "program takes " + std::to_string(plan.inputs.size()) + " inputs, got " + std::to_string(inputs.size());
  for (size_t i = 0; i < plan.inputs.size(); ++i) {
    if (inputs[i].shape.size() != plan.inputs[i].shape.size())
      return "input " + std::to_string(i) + " has rank " + std::to_string(inputs[i].shape.size()) + ", program expects rank " +
             std::to_string(plan.inputs[i].shape.size());
    if (!inputs[i].data && product(inputs[i].shape) != 0) return "input " + std::to_string(i) + " has no data";
  }
  // operands that share an index must agree on its extent: a kernel takes each loop bound from one of them
  for (const auto& group : p.same_extent) {
    const auto& first = group.front();
    for (const auto& other : group)
      if (inputs.at(other.first).shape.at(other.second) != inputs.at(first.first).shape.at(first.second))
        return "inputs " + std::to_string(first.first) + " and " + std::to_string(other.first) +
               " disagree on an index they share: dimension " + std::to_string(first.second) + " of input " +
               std::to_string(first.first) + " is " + std::to_string(inputs[first.first].shape[first.second]) +
               ", dimension " + std::to_string(other.second) + " of input " + std::to_string(other.first) + " is " +
               std::to_string(inputs[other.first].shape[other.second]);
  }
  if (outputs.size() != plan.count) return "wrong output count";
  Run run{p, plan, inputs, outputs, stream, {}, std::vector<void*>(plan.intermediates.size(), nullptr), {}, {}, workspace};
  {
    std::lock_guard<std::mutex> lock(p.mu);
    run.knobs = p.options;
  }
  for (size_t o = 0; o < outputs.size(); ++o) {
    const auto want = run.shape_of({BufferRef::Output, o});
    if (!outputs[o].shape.empty() && outputs[o].shape != want) return "output " + std::to_string(o) + " has the wrong shape";
    if (!outputs[o].data && product(want) != 0) return "output " + std::to_string(o) + " has no data";
  }

  // which kernels run hand-written, and which intermediates must exist
  std::vector<bool> hand(plan.kernels.size(), false);
  std::set<size_t> needed;
  for (size_t k = 0; k < plan.kernels.size(); ++k) {
    const Step* d = find_dispatch(plan, k);
    if (!d) return "kernel " + std::to_string(k) + " is never dispatched";
    hand[k] = hand_usable(run, p.recognized[k]);
    if (hand[k]) {
      for (size_t id : hand_intermediates(p.recognized[k])) needed.insert(id);
    } else {
      for (size_t nest : p.nests_of[k]) {
        const Step* nd = find_dispatch(p.nest_plan, nest);
        if (!nd) return "kernel " + std::to_string(k) + ": a loop nest of it is never dispatched";
        for (BufferRef r : nd->reads)
          if (r.kind == BufferRef::Intermediate) needed.insert(r.id);
        for (size_t i = 0; i < nd->writes.size(); ++i)
          if (nd->writes[i].kind == BufferRef::Intermediate && !p.generic.kernels[nest].is_private(i)) needed.insert(nd->writes[i].id);
      }
    }
  }

  std::unique_lock<std::mutex> arena_lock;
  if (!workspace) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
      (void)hipGetLastError();
    } else if (capture != hipStreamCaptureStatusNone) {
      run.capturing = true;
    } else if (arena_limit() > 0) {
      if (Arena* arena = arena_of(stream)) {
        arena_lock = std::unique_lock<std::mutex>(arena->busy, std::try_to_lock);
        if (arena_lock.owns_lock()) run.arena = arena;
      }
    }
  }
  auto finish = [&](ihip::Err e) {
    for (auto it = run.temps.rbegin(); it != run.temps.rend(); ++it) (void)hipFreeAsync(*it, stream);
    if (run.arena && run.arena_needed > run.arena->capacity && run.arena_needed <= arena_limit()) {
      // the next call on this stream finds room for everything this one needed
      const size_t bytes = (run.arena_needed + (size_t(1) << 20) - 1) >> 20 << 20;
      void* bigger = nullptr;
      if (ihip::temp_alloc(&bigger, bytes, stream).empty()) {
        if (run.arena->base) (void)hipFreeAsync(run.arena->base, stream);
        run.arena->base = bigger;
        run.arena->capacity = bytes;
      }
    }
    return e;
  };
  for (const Step& step : plan.exec) {
    if (step.kind == Step::Alloc) {
      if (!needed.count(step.id)) continue;
      const size_t n = product(run.layout_of({BufferRef::Intermediate, step.id}));
      if (ihip::Err e = run.alloc(&run.intermediates[step.id], n * 4); !e.empty()) return finish(e);
    } else if (step.kind == Step::Dispatch) {
      ihip::Err e;
      if (hand[step.id]) {
        e = launch_hand(run, p.recognized[step.id]);
      } else {
        // the generated form: the kernel's loop nests one after the other, each a kernel of its own (one line of the report)
        std::string lines;
        for (size_t nest : p.nests_of[step.id]) {
          if (e = launch_generic(run, nest, *find_dispatch(p.nest_plan, nest)); !e.empty()) break;
          lines += (lines.empty() ? "" : "; ") + run.notes.back();
          run.notes.pop_back();
        }
        if (e.empty()) run.notes.push_back(p.nests_of[step.id].size() > 1 ? std::to_string(p.nests_of[step.id].size()) + " loop nests, a kernel each: " + lines : lines);
      }
      if (!e.empty()) return finish("kernel f" + std::to_string(step.id) + ": " + e);
    }
  }
  {
    std::string report;
    size_t n = 0;
    for (const Step& step : plan.exec)
      if (step.kind == Step::Dispatch && n < run.notes.size()) report += "f" + std::to_string(step.id) + ": " + run.notes[n++] + "\n";
    std::lock_guard<std::mutex> lock(p.mu);
    p.last_report = std::move(report);
  }
  // bf16 outputs that were produced through f32 staging
  for (const auto& [o, tmp] : run.output_f32) {
    const size_t n = product(run.shape_of({BufferRef::Output, o}));
    if (ihip::Err e = ihip::launch_convert(tmp, outputs[o].data, ihip::F32, ihip::BF16, n, stream); !e.empty()) return finish(e);
  }
  return finish({});
}

std::string set_option(Program& p, const std::string& name, int value) {
  std::lock_guard<std::mutex> lock(p.mu);
  return ihip::set_kernel_option(p.options, name, value);
}

std::string set_clock_probe(Program& p, void* ticks) {
  if (reinterpret_cast<uintptr_t>(ticks) % 8 != 0) return "clock probe: the counters must be 8-byte aligned";
  std::lock_guard<std::mutex> lock(p.mu);
  p.options.clock_ticks = static_cast<unsigned long long*>(ticks);
  return {};
}

void append_to_report(Program& p, const std::string& line) {
  std::lock_guard<std::mutex> lock(p.mu);
  p.last_report += line;
}

std::string last_report(Program& p) {
  std::lock_guard<std::mutex> lock(p.mu);
  return p.last_report;
}

size_t release_stream_blocks() {
  ArenaTable& t = arena_table();
  std::lock_guard<std::mutex> lock(t.mu);
  size_t released = 0;
  for (auto& [key, arena] : t.arenas) {
    std::unique_lock<std::mutex> idle(arena->busy, std::try_to_lock);
    if (!idle.owns_lock() || !arena->base) continue;
    (void)hipFree(arena->base);  // (waits for what still runs on the device)
    released += arena->capacity;
    arena->base = nullptr;
    arena->capacity = 0;
  }
  return released;
}

std::string workspace_bytes(Program& p, const std::vector<DeviceTensor>& inputs, const std::vector<DeviceTensor>& outputs,
                            size_t* bytes, bool refuse_optional) {
  ihip::DryRun nothing_is_launched;
  Workspace sizing;
  sizing.refuse_optional = refuse_optional;
  sizing.base = reinterpret_cast<void*>(uintptr_t(256));  // never dereferenced: only has to be non-null
  const std::string err = execute(p, inputs, outputs, nullptr, &sizing);
  *bytes = sizing.used;
  return err;
}

}  // namespace ihipc
