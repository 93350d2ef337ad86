#include "emit_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <sstream>

namespace ihipc {
using namespace ic;
namespace {

// ------------------------------------------------------------------ expression printer
std::string scalar_text(float v) {
  if (std::isnan(v)) return "NAN";
  if (std::isinf(v)) return v > 0 ? "INFINITY" : "(-INFINITY)";
  char buf[64];
  snprintf(buf, sizeof buf, "%.9g", (double)v);
  std::string s = buf;
  if (s.find('.') == std::string::npos && s.find('e') == std::string::npos && s.find("inf") == std::string::npos) s += ".0";
  return s + "f";
}

std::string expr_text(const MExpr& e);

std::string fold_call(const char* fn, const std::vector<MExprPtr>& args) {
  std::string acc = expr_text(*args[0]);
  for (size_t i = 1; i < args.size(); ++i) acc = std::string(fn) + "(" + acc + ", " + expr_text(*args[i]) + ")";
  return acc;
}
std::string fold_infix(const char* sym, const std::vector<MExprPtr>& args, bool as_float) {
  std::string acc = "(" + expr_text(*args[0]) + ")";
  for (size_t i = 1; i < args.size(); ++i) acc = "(" + acc + " " + sym + " (" + expr_text(*args[i]) + "))";
  return as_float ? "((float)" + acc + ")" : acc;
}

// scalar semantics of the C backend (compiler/src/backends/c/expr.rs:127-148)
std::string op_text(Op op, const std::vector<MExprPtr>& args) {
  switch (op) {
    case Op::Add: return fold_infix("+", args, false);
    case Op::Mul: return fold_infix("*", args, false);
    case Op::Div: return fold_infix("/", args, false);
    case Op::Sub: return fold_infix("-", args, false);
    case Op::Max: return fold_call("fmaxf", args);
    case Op::Min: return fold_call("fminf", args);
    case Op::Pow: return fold_call("powf", args);
    case Op::Log: return "logf(" + expr_text(*args[0]) + ")";
    case Op::Gt: return fold_infix(">", args, true);
    case Op::Ge: return fold_infix(">=", args, true);
    case Op::Lt: return fold_infix("<", args, true);
    case Op::Le: return fold_infix("<=", args, true);
    case Op::Eq: return fold_infix("==", args, true);
    case Op::Ne: return fold_infix("!=", args, true);
    case Op::And: return fold_infix("&&", args, true);
    case Op::Or: return fold_infix("||", args, true);
    case Op::Xor: {
      std::string acc = expr_text(*args[0]);
      for (size_t i = 1; i < args.size(); ++i)
        acc = "((float)(((" + acc + ") != 0.0f) != ((" + expr_text(*args[i]) + ") != 0.0f)))";
      return acc;
    }
    case Op::Not: return "((float)!(" + expr_text(*args[0]) + "))";
  }
  return "0.0f";
}

// Every element access of a generated kernel is checked against the element count of its buffer ("cap_r<b>" /
// "cap_w<b>", computed once per kernel from the view's layout): a load outside reads 0, a store outside is
// dropped.  The loop nests and index expressions come from the schedule's lowering, and a schedule whose lowering
// is not sound for the given extents (the reference accepts such schedules and reads or writes past its malloc'd
// buffers) must not become a GPU memory fault.  ILANG_HIP_UNCHECKED=1 prints plain accesses (the CPU emulation
// uses it so that its guard pages keep finding such lowerings).
thread_local bool g_checked_accesses = true;

// Elements of writeables that a serial loop keeps in a register (see held_elements): writeable index -> the local
// variable that stands for every access to that buffer while the loop is being printed.
thread_local std::map<size_t, std::string> g_held;

// `base[idx]` with base = readonlys[b].data or writeables[b].data: fills the capacity variable's name
bool buffer_access(const MExpr& e, std::string* cap, bool* writeable = nullptr, size_t* ind = nullptr) {
  if (e.kind != MExpr::Index) return false;
  const MExpr& base = *e.args[0];
  if (base.kind != MExpr::Field || base.field != MField::Data) return false;
  const MExpr* view = base.args[0].get();
  while (view->kind == MExpr::Cast) view = view->args[0].get();
  if (view->kind != MExpr::Index || view->args[0]->kind != MExpr::Ident || view->args[1]->kind != MExpr::Usize) return false;
  const std::string& array = view->args[0]->ident;
  if (array != "readonlys" && array != "writeables") return false;
  *cap = (array == "readonlys" ? "cap_r" : "cap_w") + std::to_string(view->args[1]->usize);
  if (writeable) *writeable = array == "writeables";
  if (ind) *ind = view->args[1]->usize;
  return true;
}
// the local variable that stands for this access, if its buffer is held in a register at this point
const std::string* held_local(const MExpr& e) {
  std::string cap;
  bool writeable = false;
  size_t ind = 0;
  if (!buffer_access(e, &cap, &writeable, &ind) || !writeable) return nullptr;
  auto it = g_held.find(ind);
  return it == g_held.end() ? nullptr : &it->second;
}

std::string expr_text(const MExpr& e) {
  auto b = [&](const char* sym) { return "(" + expr_text(*e.args[0]) + " " + sym + " " + expr_text(*e.args[1]) + ")"; };
  if (const std::string* local = held_local(e)) return *local;
  if (std::string cap; g_checked_accesses && buffer_access(e, &cap)) {
    const std::string idx = expr_text(*e.args[1]);
    return "((" + idx + ") < " + cap + " ? " + expr_text(*e.args[0]) + "[" + idx + "] : 0.0f)";
  }
  switch (e.kind) {
    case MExpr::Usize: return "(size_t)" + std::to_string(e.usize);
    case MExpr::Scalar: return scalar_text(e.scalar);
    case MExpr::Ident: return e.ident;
    case MExpr::Index: return expr_text(*e.args[0]) + "[" + expr_text(*e.args[1]) + "]";
    case MExpr::Field: {
      const char* f = e.field == MField::Data ? "data" : e.field == MField::Shape ? "shape" : e.field == MField::Layout ? "layout" : "rank";
      return expr_text(*e.args[0]) + "." + f;
    }
    case MExpr::Cast: return expr_text(*e.args[0]);
    case MExpr::OpCall: return op_text(e.op, e.args);
    case MExpr::Add: return b("+");
    case MExpr::Sub: return b("-");
    case MExpr::Mul: return b("*");
    case MExpr::Div: return b("/");
    case MExpr::Rem: return b("%");
    case MExpr::Lt: return b("<");
    case MExpr::Eq: return b("==");
    case MExpr::And: return b("&&");
  }
  return "0";
}

// ------------------------------------------------------------------ parallelism analysis
using PAct = Action<Param>;

bool iter_uses(const Iter& it, size_t loop) {
  if (it.raw) return it.loop == loop;
  return std::find(it.loops.begin(), it.loops.end(), loop) != it.loops.end();
}
bool access_uses(const Access<Param>& a, size_t loop) {
  for (const Iter& it : a.index)
    if (iter_uses(it, loop)) return true;
  return false;
}

struct Uses {
  std::vector<const Access<Param>*> all;     // every access
  std::set<Param> written;
};
void collect_scalar(const ScalarExpr<Param>& e, Uses& u) {
  if (e.kind == ScalarExpr<Param>::Acc) u.all.push_back(&e.access);
  for (const auto& a : e.args) collect_scalar(a, u);
}
void collect(const Block<Param>& block, Uses& u);
void collect_one(const PAct& a, Uses& u) {
  switch (a.kind) {
    case PAct::Loop: collect(a.body, u); break;
    case PAct::Init:
      u.all.push_back(&a.write);
      u.written.insert(a.write.buffer);
      break;
    case PAct::Compute:
    case PAct::Snapshot:
      u.all.push_back(&a.write);
      u.written.insert(a.write.buffer);
      for (const auto& r : a.reads) u.all.push_back(&r);
      break;
    case PAct::Scale:
      u.all.push_back(&a.write);
      u.written.insert(a.write.buffer);
      collect_scalar(a.factor, u);
      break;
  }
}
void collect(const Block<Param>& block, Uses& u) {
  for (const PAct& a : block) collect_one(a, u);
}

bool same_iter(const Iter& a, const Iter& b) {
  return a.raw == b.raw && (a.raw ? a.loop == b.loop : a.loops == b.loops && a.factors == b.factors);
}
bool same_access(const Access<Param>& a, const Access<Param>& b) {
  if (!(a.buffer == b.buffer) || a.index.size() != b.index.size()) return false;
  for (size_t d = 0; d < a.index.size(); ++d)
    if (!same_iter(a.index[d], b.index[d])) return false;
  return true;
}
void loop_ids(const Block<Param>& block, std::set<size_t>& ids) {
  for (const PAct& a : block)
    if (a.kind == PAct::Loop) {
      ids.insert(a.id);
      loop_ids(a.body, ids);
    }
}

// Elements held in registers.  Inside a loop L, a written buffer all of whose accesses (reads and writes, L's
// nested loops included) name one and the same element, with an index that neither L nor a loop nested in L
// takes part in, is an accumulator of L: the element is loaded into a local variable before L, every access
// inside L becomes that variable, and it is stored back after L.  (As printed by the C backend the element
// makes a round trip through memory in every iteration, which serialises the loop on the latency of that trip.)
// Buffers of one kernel never overlap: a kernel's readonlys and writeables are disjoint sets of distinct buffers.
// Result: loop id -> writeable indexes.
void held_elements(const Block<Param>& block, std::map<size_t, std::vector<size_t>>& out) {
  for (const PAct& loop : block) {
    if (loop.kind != PAct::Loop) continue;
    Uses u;
    collect(loop.body, u);
    std::set<size_t> inner{loop.id};
    loop_ids(loop.body, inner);
    for (const Param& w : u.written) {
      const Access<Param>* first = nullptr;
      bool ok = w.writeable;
      for (const auto* a : u.all) {
        if (!(a->buffer == w)) continue;
        if (!first) first = a;
        ok = ok && same_access(*first, *a);
      }
      for (size_t id : inner) ok = ok && first && !access_uses(*first, id);
      if (ok) out[loop.id].push_back(w.ind);
    }
    held_elements(loop.body, out);
  }
}

// Buffers that only this kernel touches (fused temporaries) may be privatised.
std::set<size_t> exclusive_intermediates(const ExecPlan& plan, size_t kernel) {
  std::map<size_t, std::set<size_t>> users;
  for (const Step& s : plan.exec)
    if (s.kind == Step::Dispatch) {
      for (BufferRef r : s.reads)
        if (r.kind == BufferRef::Intermediate) users[r.id].insert(s.id);
      for (BufferRef r : s.writes)
        if (r.kind == BufferRef::Intermediate) users[r.id].insert(s.id);
    }
  std::set<size_t> out;
  for (const auto& [id, ks] : users)
    if (ks.size() == 1 && *ks.begin() == kernel) out.insert(id);
  return out;
}

// Parallel loops and private buffers of one phase.  `body` is the phase's statement list (the spine is followed
// while it is a single loop); buffers in `shared` are touched by other phases and must stay in memory.
void analyze(const ExecPlan& plan, size_t k, const Block<Param>& body, const std::set<Param>& shared, GenericPhase& info) {
  const Step* dispatch = nullptr;
  for (const Step& s : plan.exec)
    if (s.kind == Step::Dispatch && s.id == k) dispatch = &s;
  const std::set<size_t> exclusive = exclusive_intermediates(plan, k);

  const Block<Param>* block = &body;
  std::set<Param> privatized;
  while (block->size() == 1 && (*block)[0].kind == PAct::Loop) {
    const PAct& loop = (*block)[0];
    Uses u;
    collect(loop.body, u);
    bool ok = true;
    std::set<Param> want_private;
    for (const Param& w : u.written) {
      bool all_use = true, none_use = true;
      for (const auto* a : u.all)
        if (a->buffer == w) {
          const bool uses = access_uses(*a, loop.id);
          all_use &= uses;
          none_use &= !uses;
        }
      if (all_use) continue;  // distinct iterations touch distinct elements
      const bool can_privatize = none_use && !shared.count(w) && w.writeable && dispatch && w.ind < dispatch->writes.size() &&
                                 dispatch->writes[w.ind].kind == BufferRef::Intermediate &&
                                 exclusive.count(dispatch->writes[w.ind].id);
      if (can_privatize) want_private.insert(w);
      else ok = false;
    }
    if (ok) {
      info.parallel_loops.push_back(loop.id);
      info.parallel_extents.push_back(loop.extent);
      privatized.insert(want_private.begin(), want_private.end());
    }
    block = &loop.body;
  }
  if (info.parallel_loops.empty()) return;
  for (const Param& w : privatized) {
    PrivateBuffer pb;
    pb.writeable = w.ind;
    const PlanBuffer& buf = plan.intermediates[dispatch->writes[w.ind].id];
    pb.is_static = true;
    pb.static_size = 1;
    for (const auto& e : buf.layout) {
      if (e.kind.kind == ExtentKind::Split) pb.static_size *= e.kind.factor;
      else pb.is_static = false;
    }
    if (pb.is_static && pb.static_size > 4096) pb.is_static = false;
    info.privates.push_back(pb);
  }
}

void collect_initialized(const Block<Param>& block, std::set<Param>& out) {
  for (const PAct& a : block) {
    if (a.kind == PAct::Loop) collect_initialized(a.body, out);
    else if (a.kind == PAct::Init) out.insert(a.write.buffer);
  }
}

// The wavefront-per-iteration form of a phase (GenericPhase::wave_loops), or nothing when the nest does not
// qualify.  `body` is the phase's statement list, `initialized` the buffers with an Init anywhere in the kernel
// (a Compute into one of them is `dst = op(dst, reads...)`), `held` the result of held_elements.
// Conditions, with B the body of the innermost parallel loop (every loop above B on the spine is parallel):
//   * statements of B outside loops store values that all 64 lanes compute alike and that do not depend on
//     the stored element itself: Init, Snapshot, a Compute that is no reduction;
//   * every loop L of B is spread over the lanes; inside L there are only Computes, each one either
//     - a reduction (+, *, max, min) into an element that L holds in a register (an accumulator: lane shares,
//       then a butterfly), read by nothing else inside L, or
//     - a store into a work-item-private buffer (every lane has its own copy), or
//     - a store whose element depends on L's iteration, into a buffer of which L touches that element only;
//     what such stores write is used nowhere else in B (lanes would read what other lanes wrote);
//   * some loop has an accumulator, and no private buffer of the phase lives in device memory.
void wave_plan(const Block<Param>& body, const std::set<Param>& initialized, const std::map<size_t, std::vector<size_t>>& held,
               GenericPhase& phase) {
  const Block<Param>* block = &body;
  size_t spine = 0;
  while (block->size() == 1 && (*block)[0].kind == PAct::Loop) {
    ++spine;
    block = &(*block)[0].body;
  }
  if (spine != phase.parallel_loops.size()) return;
  for (const PrivateBuffer& pb : phase.privates)
    if (!pb.is_static) return;
  auto is_private = [&](const Param& w) {
    if (!w.writeable) return false;
    for (const PrivateBuffer& pb : phase.privates)
      if (pb.writeable == w.ind) return true;
    return false;
  };
  std::vector<WaveLoop> loops;
  bool any_accumulator = false, contiguous = true;
  for (size_t n = 0; n < block->size(); ++n) {
    const PAct& st = (*block)[n];
    if (st.kind == PAct::Scale) return;
    if (st.kind == PAct::Compute && initialized.count(st.write.buffer)) return;
    if (st.kind != PAct::Loop) continue;
    WaveLoop wl;
    wl.loop = st.id;
    const auto held_here = held.find(st.id);
    std::set<Param> lane_written;  // written inside the loop, accumulators aside
    std::vector<const PAct*> computes;
    std::vector<const Block<Param>*> todo{&st.body};
    while (!todo.empty()) {
      const Block<Param>* b = todo.back();
      todo.pop_back();
      for (const PAct& a : *b) {
        if (a.kind == PAct::Loop) todo.push_back(&a.body);
        else if (a.kind == PAct::Compute) computes.push_back(&a);
        else return;
      }
    }
    // Which loop goes over the lanes: of the loops nested perfectly from `st` down, the innermost one that
    // drives the last index of everything it reads (consecutive lanes then read consecutive elements), a loop
    // over a split factor below 64 aside (it could not occupy the lanes); `st` itself when there is none.
    const PAct* spread = &st;
    bool spread_contiguous = false;
    {
      std::vector<const PAct*> chain{&st};
      while (chain.back()->body.size() == 1 && chain.back()->body[0].kind == PAct::Loop) chain.push_back(&chain.back()->body[0]);
      for (size_t c = chain.size(); c-- > 0 && !spread_contiguous;) {
        const PAct& cand = *chain[c];
        if (cand.extent.kind.kind == ExtentKind::Split && cand.extent.kind.factor < 64) continue;
        bool reads_any = false, last = true;
        for (const PAct* cp : computes)
          for (const auto& r : cp->reads)
            if (access_uses(r, cand.id)) {
              reads_any = true;
              last = last && iter_uses(r.index.back(), cand.id);
            }
        if (reads_any && last) {
          spread = &cand;
          spread_contiguous = true;
        }
      }
    }
    wl.spread = spread->id;
    contiguous = contiguous && spread_contiguous;
    Uses inside;
    collect(st.body, inside);
    for (const PAct* c : computes) {
      const Param w = c->write.buffer;
      const bool held_by_loop = held_here != held.end() && w.writeable &&
                                std::find(held_here->second.begin(), held_here->second.end(), w.ind) != held_here->second.end();
      if (initialized.count(w)) {
        const bool known = c->op == Op::Add || c->op == Op::Mul || c->op == Op::Max || c->op == Op::Min;
        if (!held_by_loop || !known) return;
        bool seen = false;
        for (const auto& acc : wl.accumulators) {
          if (acc.first != w.ind) continue;
          if (acc.second != c->op) return;
          seen = true;
        }
        if (!seen) wl.accumulators.push_back({w.ind, c->op});
        continue;
      }
      if (!is_private(w)) {
        if (!access_uses(c->write, spread->id)) return;
        for (const auto* a : inside.all)
          if (a->buffer == w && !same_access(*a, c->write)) return;
      }
      lane_written.insert(w);
    }
    for (const PAct* c : computes)
      for (const auto& r : c->reads)
        for (const auto& acc : wl.accumulators)
          if (r.buffer.writeable && r.buffer.ind == acc.first) return;
    // nothing else in B touches what the lanes stored
    for (size_t m = 0; m < block->size(); ++m) {
      if (m == n) continue;
      Uses other;
      collect_one((*block)[m], other);
      for (const auto* a : other.all)
        if (lane_written.count(a->buffer)) return;
    }
    if (!wl.accumulators.empty() && !any_accumulator) {
      any_accumulator = true;
      phase.wave_extent = spread->extent;
    }
    loops.push_back(std::move(wl));
  }
  if (!any_accumulator) return;
  phase.wave_loops = std::move(loops);
  phase.wave_contiguous = contiguous;
}

// Top-level statements of a kernel grouped into phases: every loop is a phase of its own, a run of
// other statements (initialisations of scalars) is one phase.  Returns [first, last) index ranges.
std::vector<std::pair<size_t, size_t>> phase_ranges(const Block<Param>& body) {
  std::vector<std::pair<size_t, size_t>> out;
  size_t i = 0;
  while (i < body.size()) {
    if (body[i].kind == PAct::Loop) {
      out.push_back({i, i + 1});
      ++i;
    } else {
      size_t j = i;
      while (j < body.size() && body[j].kind != PAct::Loop) ++j;
      out.push_back({i, j});
      i = j;
    }
  }
  if (out.empty()) out.push_back({0, 0});
  return out;
}

// ------------------------------------------------------------------ statement printer
// the first access to writeables[ind] in an expression / a statement list
const MExpr* find_writeable_access(const MExpr& e, size_t ind) {
  std::string cap;
  bool writeable = false;
  size_t at = 0;
  if (buffer_access(e, &cap, &writeable, &at) && writeable && at == ind) return &e;
  for (const MExprPtr& a : e.args)
    if (a)
      if (const MExpr* r = find_writeable_access(*a, ind)) return r;
  return nullptr;
}
const MExpr* find_writeable_access(const std::vector<MStmt>& stmts, size_t ind) {
  for (const MStmt& s : stmts) {
    if (s.dst)
      if (const MExpr* r = find_writeable_access(*s.dst, ind)) return r;
    if (s.value && s.kind == MStmt::Set)
      if (const MExpr* r = find_writeable_access(*s.value, ind)) return r;
    if (const MExpr* r = find_writeable_access(s.body, ind)) return r;
  }
  return nullptr;
}

struct Printer {
  std::ostringstream os;
  std::set<std::string> parallel;  // iterator names handled by the work-item decomposition
  const std::map<size_t, std::vector<size_t>>* held = nullptr;  // loop id -> elements to hold in registers (held_elements)
  const std::vector<WaveLoop>* wave = nullptr;  // the wavefront-per-iteration form: loops spread over the lanes
  int serial_depth = 0;                         // loops being printed as loops around the current statement
  static const char* identity_text(Op op) {
    return op == Op::Mul ? "1.0f" : op == Op::Max ? "(-INFINITY)" : op == Op::Min ? "INFINITY" : "0.0f";
  }
  static std::string reduce_text(Op op, const std::string& a, const std::string& b) {
    if (op == Op::Max) return "fmaxf(" + a + ", " + b + ")";
    if (op == Op::Min) return "fminf(" + a + ", " + b + ")";
    return "(" + a + (op == Op::Mul ? " * " : " + ") + b + ")";
  }
  // In the wavefront form all 64 lanes execute the statements outside the spread loops alike; the marker after
  // each of them is a scheduling fence on the device (the lanes of a wavefront run in lockstep there) and a
  // barrier among the 64 threads that stand for the lanes in a CPU emulation.
  void uniform_statement_done(int depth) {
    if (wave && serial_depth == 0) line(depth, "ILANG_WAVE_SYNC();");
  }
  static bool innermost(const std::vector<MStmt>& body) {
    for (const MStmt& s : body)
      if (s.kind == MStmt::Loop || !innermost(s.body)) return false;
    return true;
  }
  void line(int depth, const std::string& s) { os << std::string(2 * depth, ' ') << s << "\n"; }
  void block(const std::vector<MStmt>& stmts, int depth) {
    for (const MStmt& s : stmts) stmt(s, depth);
  }
  void stmt(const MStmt& s, int depth) {
    switch (s.kind) {
      case MStmt::Set: {
        std::string cap;
        if (const std::string* local = held_local(*s.dst)) {
          line(depth, *local + " = " + expr_text(*s.value) + ";");
        } else if (g_checked_accesses && buffer_access(*s.dst, &cap)) {
          const std::string idx = expr_text(*s.dst->args[1]);
          line(depth, "if ((" + idx + ") < " + cap + ") " + expr_text(*s.dst->args[0]) + "[" + idx + "] = " + expr_text(*s.value) + ";");
        } else {
          line(depth, expr_text(*s.dst) + " = " + expr_text(*s.value) + ";");
        }
        uniform_statement_done(depth);
        break;
      }
      case MStmt::Loop:
        if (parallel.count(s.ident)) {
          block(s.body, depth);
        } else {
          // elements this loop accumulates into: loaded before it, kept in a local inside, stored after it
          struct Held { size_t ind; const MExpr* at; std::string local; bool shared; Op op; };
          std::vector<Held> mine;
          const size_t loop_id = (size_t)std::stoul(s.ident.substr(1));
          const WaveLoop* lanes = nullptr;  // this loop is spread over the lanes of the wavefront
          if (wave)
            for (const WaveLoop& wl : *wave)
              if (wl.loop == loop_id) lanes = &wl;
          if (held) {
            auto it = held->find(loop_id);
            if (it != held->end())
              for (size_t ind : it->second)
                if (!g_held.count(ind))
                  if (const MExpr* at = find_writeable_access(s.body, ind)) {
                    Held h{ind, at, "h" + std::to_string(ind) + "_" + s.ident, false, Op::Add};
                    if (lanes)
                      for (const auto& acc : lanes->accumulators)
                        if (acc.first == ind) {
                          h.shared = true;
                          h.op = acc.second;
                        }
                    mine.push_back(h);
                  }
          }
          const int d = mine.empty() ? depth : depth + 1;
          if (!mine.empty()) line(depth, "{");
          for (const Held& h : mine) {
            if (h.shared) {
              // the element as it is before the loop, and this lane's share of what the loop adds to it
              line(d, "const float before_" + h.local + " = " + expr_text(*h.at) + ";");
              line(d, "float " + h.local + " = " + identity_text(h.op) + ";");
            } else {
              line(d, "float " + h.local + " = " + expr_text(*h.at) + ";");
            }
          }
          for (const Held& h : mine) g_held[h.ind] = h.local;
          bool spread = false;  // this loop's iterations are dealt out over the lanes
          if (wave)
            for (const WaveLoop& wl : *wave) spread |= wl.spread == loop_id;
          // an innermost loop that only accumulates into registers: unrolled, so that the loads of several
          // iterations are in flight at once (measured on row sums: 2.1 -> 3.8 TB/s in the wavefront form, 0.6 -> 1.0
          // with a work-item per row)
          if ((spread || !mine.empty()) && innermost(s.body)) line(d, "#pragma unroll 4");
          if (spread)
            line(d, "for (size_t " + s.ident + " = lane; " + s.ident + " < " + expr_text(*s.value) + "; " + s.ident + " += 64) {");
          else
            line(d, "for (size_t " + s.ident + " = 0; " + s.ident + " < " + expr_text(*s.value) + "; ++" + s.ident + ") {");
          ++serial_depth;
          block(s.body, d + 1);
          --serial_depth;
          line(d, "}");
          for (const Held& h : mine) g_held.erase(h.ind);
          for (const Held& h : mine) {
            std::string value = h.local;
            if (h.shared) {
              line(d, "for (int lane_xor = 32; lane_xor > 0; lane_xor >>= 1) " + h.local + " = " +
                          reduce_text(h.op, h.local, "__shfl_xor(" + h.local + ", lane_xor)") + ";");
              value = reduce_text(h.op, "before_" + h.local, h.local);
            }
            std::string cap;  // the checked form applies as for any other store
            const std::string idx = expr_text(*h.at->args[1]);
            if (g_checked_accesses && buffer_access(*h.at, &cap))
              line(d, "if ((" + idx + ") < " + cap + ") " + expr_text(*h.at->args[0]) + "[" + idx + "] = " + value + ";");
            else
              line(d, expr_text(*h.at->args[0]) + "[" + idx + "] = " + value + ";");
          }
          if (!mine.empty()) line(depth, "}");
          uniform_statement_done(depth);
        }
        break;
      case MStmt::If:
        line(depth, "if (" + expr_text(*s.value) + ") {");
        block(s.body, depth + 1);
        line(depth, "}");
        break;
      case MStmt::Return: break;
      default: lower_error("statement kind is not valid inside a kernel");
    }
  }
};

const MStmt* find_loop(const std::vector<MStmt>& stmts, const std::string& iter) {
  for (const MStmt& s : stmts) {
    if (s.kind == MStmt::Loop && s.ident == iter) return &s;
    if (s.kind == MStmt::Loop || s.kind == MStmt::If)
      if (const MStmt* r = find_loop(s.body, iter)) return r;
  }
  return nullptr;
}

}  // namespace

GenericModule emit_generic_hip(const ExecPlan& plan, const Module& module, const std::vector<bool>& emit) {
  const char* unchecked = std::getenv("ILANG_HIP_UNCHECKED");
  g_checked_accesses = !(unchecked && unchecked[0] == '1');
  g_held.clear();  // (an error thrown while a loop was being printed must not leave its substitutions behind)
  GenericModule out;
  out.kernels.resize(plan.kernels.size());
  size_t rank = 1;
  for (const auto& b : plan.inputs) rank = std::max({rank, b.shape.size(), b.layout.size()});
  for (const auto& b : plan.intermediates) rank = std::max({rank, b.shape.size(), b.layout.size()});
  for (const auto& b : plan.outputs) rank = std::max({rank, b.shape.size(), b.layout.size()});
  out.rank = rank;

  std::ostringstream src;
  bool any = false;
  src << "// generated by the i gfx950 backend\n#include <hip/hip_runtime.h>\n#include <math.h>\n#include <stddef.h>\n\n";
  src << "#ifndef ILANG_WAVE_SYNC\n#define ILANG_WAVE_SYNC() __builtin_amdgcn_wave_barrier()\n#endif\n\n";
  src << "struct View { float* data; size_t shape[" << rank << "]; size_t layout[" << rank << "]; };\n\n";
  for (size_t k = 0; k < plan.kernels.size(); ++k) {
    if (!emit[k]) continue;
    any = true;
    GenericKernel& info = out.kernels[k];
    info.name = "f" + std::to_string(k);
    info.n_reads = plan.kernels[k].reads.size();
    info.n_writes = plan.kernels[k].writes.size();
    const Block<Param>& body = plan.kernels[k].body;
    const MFn& fn = module.kernels[k];
    std::map<size_t, std::vector<size_t>> held;
    held_elements(body, held);
    // one statement of the module per action of the plan kernel (a trailing return aside)
    size_t fn_stmts = fn.body.size();
    while (fn_stmts > 0 && fn.body[fn_stmts - 1].kind == MStmt::Return) --fn_stmts;
    // A body that is a sequence of top-level statements is split into phases (one per loop nest).  Default: the
    // phases share one launch of one workgroup with barriers between them, provided some nest has parallel loops
    // (otherwise the kernel stays a single work-item).  ILANG_HIP_PHASES=1: one launch per phase (CPU emulation only).
    const char* want_phases = std::getenv("ILANG_HIP_PHASES");
    const bool separate_launches = want_phases && want_phases[0] == '1';
    auto ranges = phase_ranges(body);
    if (fn_stmts != body.size()) ranges = {{0, body.size()}};  // no statement-by-statement correspondence: one phase
    auto analyze_all = [&](const std::vector<std::pair<size_t, size_t>>& rs, std::vector<Block<Param>>& bodies,
                           std::vector<GenericPhase>& phases) {
      // buffers touched by more than one phase stay in memory
      std::map<Param, size_t> touched;
      bodies.clear();
      phases.clear();
      for (const auto& [first, last] : rs) {
        bodies.emplace_back(body.begin() + first, body.begin() + last);
        Uses u;
        collect(bodies.back(), u);
        std::set<Param> seen;
        for (const auto* a : u.all) seen.insert(a->buffer);
        for (const Param& b : seen) ++touched[b];
      }
      std::set<Param> shared;
      for (const auto& [b, n] : touched)
        if (n > 1) shared.insert(b);
      for (size_t ph = 0; ph < rs.size(); ++ph) {
        GenericPhase phase;
        phase.name = rs.size() == 1 || !separate_launches ? info.name : info.name + "_p" + std::to_string(ph);
        analyze(plan, k, bodies[ph], shared, phase);
        phases.push_back(std::move(phase));
      }
    };
    std::vector<Block<Param>> bodies;
    std::vector<GenericPhase> phases;
    analyze_all(ranges, bodies, phases);
    bool cooperative = false;
    if (ranges.size() > 1 && !separate_launches) {
      for (const GenericPhase& ph : phases) cooperative |= !ph.parallel_loops.empty();
      if (!cooperative) {  // nothing to spread over work-items: the whole body as one phase, one work-item
        ranges = {{0, body.size()}};
        analyze_all(ranges, bodies, phases);
      }
    }
    info.cooperative = cooperative;

    const size_t nr = std::max<size_t>(info.n_reads, 1), nw = std::max<size_t>(info.n_writes, 1);
    src << "struct Args_" << info.name << " { View readonlys[" << nr << "]; View writeables[" << nw << "]; };\n";
    const Step* dispatch = nullptr;
    for (const Step& st : plan.exec)
      if (st.kind == Step::Dispatch && st.id == k) dispatch = &st;
    // element counts of the kernel's views, for the checked accesses: the product of the layout extents (a
    // work-item-private slice or array has the same layout as the buffer it stands for)
    auto emit_capacities = [&](const std::string& pad) {
      if (!g_checked_accesses) return;
      auto rank_of = [&](BufferRef r) {
        return (r.kind == BufferRef::Input ? plan.inputs.at(r.id) : r.kind == BufferRef::Intermediate ? plan.intermediates.at(r.id)
                                                                                                     : plan.outputs.at(r.id)).layout.size();
      };
      for (size_t b = 0; dispatch && b < dispatch->reads.size(); ++b) {
        src << pad << "const size_t cap_r" << b << " = (size_t)1";
        for (size_t d = 0; d < rank_of(dispatch->reads[b]); ++d) src << " * readonlys[" << b << "].layout[" << d << "]";
        src << ";\n";
      }
      for (size_t b = 0; dispatch && b < dispatch->writes.size(); ++b) {
        src << pad << "const size_t cap_w" << b << " = (size_t)1";
        for (size_t d = 0; d < rank_of(dispatch->writes[b]); ++d) src << " * writeables[" << b << "].layout[" << d << "]";
        src << ";\n";
      }
    };
    // work-item-private buffers of one phase: a local array, or this work-item's slice of a device buffer
    auto emit_privates = [&](const GenericPhase& phase, const std::string& pad) {
      for (const PrivateBuffer& pb : phase.privates) {
        if (pb.is_static) {
          src << pad << "float priv" << pb.writeable << "[" << pb.static_size << "];\n";
          src << pad << "writeables[" << pb.writeable << "].data = priv" << pb.writeable << ";\n";
        } else {
          const size_t prank = plan.intermediates[dispatch->writes[pb.writeable].id].layout.size();
          src << pad << "{ size_t n = 1; for (int d = 0; d < " << prank << "; ++d) n *= writeables[" << pb.writeable
              << "].layout[d]; writeables[" << pb.writeable << "].data += wi_first * n; }\n";
        }
      }
    };
    // the statements of one phase spread over the work-items (wi_first, wi_stride); `depth` is the indentation
    auto emit_spread = [&](const GenericPhase& phase, const std::vector<MStmt>& stmts, int depth, bool wave = false) {
      const std::string pad(2 * depth, ' ');
      Printer pr;
      pr.held = &held;
      if (wave) pr.wave = &phase.wave_loops;
      std::vector<std::string> iters;
      for (size_t id : phase.parallel_loops) iters.push_back("i" + std::to_string(id));
      for (const std::string& it : iters) {
        const MStmt* loop = find_loop(stmts, it);
        if (!loop) lower_error("parallel loop " + it + " not found in kernel body");
        src << pad << "const size_t n_" << it << " = " << expr_text(*loop->value) << ";\n";
        pr.parallel.insert(it);
      }
      src << pad << "size_t wi_total = 1;\n";
      for (const std::string& it : iters) src << pad << "wi_total *= n_" << it << ";\n";
      src << pad << "for (size_t wi = wi_first; wi < wi_total; wi += wi_stride) {\n";
      src << pad << "  size_t wi_rest = wi;\n";
      for (size_t t = iters.size(); t-- > 0;) {
        src << pad << "  const size_t " << iters[t] << " = wi_rest % n_" << iters[t] << ";";
        src << " wi_rest /= n_" << iters[t] << ";\n";
      }
      pr.block(stmts, depth + 1);
      src << pr.os.str();
      src << pad << "}\n";
    };
    auto phase_stmts = [&](size_t ph) {
      return std::vector<MStmt>(fn.body.begin() + (fn_stmts == body.size() ? ranges[ph].first : 0),
                                fn.body.begin() + (fn_stmts == body.size() ? ranges[ph].second : fn_stmts));
    };
    if (cooperative) {
      src << "extern \"C\" __global__ void __launch_bounds__(" << GenericKernel::kCooperativeThreads << ") " << info.name
          << "(Args_" << info.name << " args) {\n";
      src << "  const View* readonlys = args.readonlys;\n";
      src << "  View writeables[" << nw << "];\n";
      src << "  for (int b = 0; b < " << nw << "; ++b) writeables[b] = args.writeables[b];\n";
      src << "  // one workgroup: every loop nest below is spread over its work-items, a barrier orders the nests\n";
      src << "  const size_t wi_first = threadIdx.x;\n";
      src << "  const size_t wi_stride = blockDim.x;\n";
      emit_capacities("  ");
      for (size_t ph = 0; ph < ranges.size(); ++ph) {
        if (ph > 0) src << "  __syncthreads();\n";
        src << "  {\n";
        emit_privates(phases[ph], "    ");
        if (phases[ph].parallel_loops.empty()) {
          src << "    if (wi_first == 0) {\n";
          Printer pr;
      pr.held = &held;
          pr.block(phase_stmts(ph), 3);
          src << pr.os.str();
          src << "    }\n";
        } else {
          emit_spread(phases[ph], phase_stmts(ph), 2);
        }
        src << "  }\n";
      }
      src << "}\n\n";
      for (auto& ph : phases) info.phases.push_back(std::move(ph));
      continue;
    }
    std::set<Param> initialized;
    collect_initialized(body, initialized);
    for (size_t ph = 0; ph < ranges.size(); ++ph) {
      GenericPhase& phase = phases[ph];
      wave_plan(bodies[ph], initialized, held, phase);
      const std::vector<MStmt> stmts = phase_stmts(ph);
      // wave: one wavefront per iteration of the parallel loops (<name>_w) instead of one work-item
      for (const bool wave : {false, true}) {
        if (wave && phase.wave_loops.empty()) continue;
        src << "extern \"C\" __global__ void __launch_bounds__(" << (wave ? GenericPhase::kWaveThreads : 64u) << ") " << phase.name
            << (wave ? "_w" : "") << "(Args_" << info.name << " args) {\n";
        src << "  const View* readonlys = args.readonlys;\n";
        src << "  View writeables[" << nw << "];\n";
        src << "  for (int b = 0; b < " << nw << "; ++b) writeables[b] = args.writeables[b];\n";
        if (wave) {
          src << "  const size_t lane = threadIdx.x % 64;\n";
          src << "  const size_t wi_first = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / 64;\n";
          src << "  const size_t wi_stride = ((size_t)gridDim.x * blockDim.x) / 64;\n";
        } else {
          src << "  const size_t wi_first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;\n";
          src << "  const size_t wi_stride = (size_t)gridDim.x * blockDim.x;\n";
        }
        emit_capacities("  ");
        emit_privates(phase, "  ");
        if (phase.parallel_loops.empty()) {
          src << "  if (wi_first != 0) return;\n";
          Printer pr;
          pr.held = &held;
          if (wave) pr.wave = &phase.wave_loops;
          pr.block(stmts, 1);
          src << pr.os.str();
        } else {
          emit_spread(phase, stmts, 1, wave);
        }
        src << "}\n\n";
      }
      info.phases.push_back(std::move(phase));
    }
  }
  if (any) out.source = src.str();
  return out;
}

}  // namespace ihipc
