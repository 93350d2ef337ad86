#include "emit_hip.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
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
// Loops in `parallel` are the work-item index space: their iterators are fixed inside a work-item, so an index that
// one of them takes part in still names one element (a column sum with the row loop outside the column loop keeps
// each work-item's column total in a register across the rows).  A parallel loop with a tail guard below the
// loop in question is no such loop: the guard sits inside, and a load hoisted above it would run for the tail's
// work-items too.
// Result: loop id -> writeable indexes.
void held_elements(const Block<Param>& block, const std::set<size_t>& parallel, std::map<size_t, std::vector<size_t>>& out) {
  for (const PAct& loop : block) {
    if (loop.kind != PAct::Loop) continue;
    if (parallel.count(loop.id)) {
      held_elements(loop.body, parallel, out);
      continue;
    }
    Uses u;
    collect(loop.body, u);
    std::set<size_t> inner{loop.id};
    loop_ids(loop.body, inner);
    {
      std::set<size_t> guarded;
      std::vector<const Block<Param>*> todo{&loop.body};
      while (!todo.empty()) {
        const Block<Param>* b = todo.back();
        todo.pop_back();
        for (const PAct& a : *b)
          if (a.kind == PAct::Loop) {
            if (a.guard) guarded.insert(a.id);
            todo.push_back(&a.body);
          }
      }
      for (size_t id : parallel)
        if (!guarded.count(id)) inner.erase(id);
    }
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
    held_elements(loop.body, parallel, out);
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
  const GridForm* grid = nullptr;               // the form with a loop in parts: `part` of `parts` takes its share of grid->loop
  int serial_depth = 0;                         // loops being printed as loops around the current statement
  // In the form with a loop in parts every part accumulates into copies of the accumulated buffers that the
  // launcher has filled with the reduction's identity: the nest's own initialisations of those buffers are dropped.
  bool dropped_initialisation(const MStmt& s) const {
    if (!grid || s.kind != MStmt::Set || !s.value || s.value->kind != MExpr::Scalar) return false;
    std::string cap;
    bool writeable = false;
    size_t ind = 0;
    if (!buffer_access(*s.dst, &cap, &writeable, &ind) || !writeable) return false;
    for (const GridAccumulator& acc : grid->accumulators)
      if (acc.writeable == ind) return true;
    return false;
  }
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
  // no loop below that is printed as a loop (the parallel ones are the work-item's coordinates)
  bool innermost(const std::vector<MStmt>& body) const {
    for (const MStmt& s : body)
      if ((s.kind == MStmt::Loop && !parallel.count(s.ident)) || !innermost(s.body)) return false;
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
        if (dropped_initialisation(s)) break;
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
            // (in the form with a loop in parts an accumulated element starts as the reduction's identity: what its
            // copy holds is not read, so the copies need no filling when every accumulator is held this way)
            const GridAccumulator* fresh = nullptr;
            if (grid && grid->held_accumulators)
              for (const GridAccumulator& acc : grid->accumulators)
                if (acc.writeable == h.ind) fresh = &acc;
            if (h.shared) {
              // the element as it is before the loop, and this lane's share of what the loop adds to it
              line(d, "const float before_" + h.local + " = " + (fresh ? std::string(identity_text(fresh->op)) : expr_text(*h.at)) + ";");
              line(d, "float " + h.local + " = " + identity_text(h.op) + ";");
            } else {
              line(d, "float " + h.local + " = " + (fresh ? std::string(identity_text(fresh->op)) : expr_text(*h.at)) + ";");
            }
          }
          for (const Held& h : mine) g_held[h.ind] = h.local;
          bool spread = false;  // this loop's iterations are dealt out over the lanes
          if (wave)
            for (const WaveLoop& wl : *wave) spread |= wl.spread == loop_id;
          // an innermost loop that only accumulates into registers: unrolled, so that the loads of several
          // iterations are in flight at once (measured on row sums: 2.1 -> 3.8 TB/s in the wavefront form, 0.6 -> 1.0
          // with a work-item per row)
          // part p takes a run of consecutive iterations of this loop (consecutive rows stay within a page)
          const bool in_parts = grid && grid->loop == loop_id;
          if (in_parts) {
            line(d, "const size_t share_" + s.ident + " = (" + expr_text(*s.value) + " + parts - 1) / parts;");
            line(d, "const size_t end_" + s.ident + " = (part + 1) * share_" + s.ident + " < " + expr_text(*s.value) + " ? (part + 1) * share_" +
                        s.ident + " : " + expr_text(*s.value) + ";");
          }
          if ((spread || !mine.empty()) && innermost(s.body)) line(d, "#pragma unroll 8");
          if (spread && in_parts)
            line(d, "for (size_t " + s.ident + " = part * share_" + s.ident + " + lane; " + s.ident + " < end_" + s.ident + "; " + s.ident + " += 64) {");
          else if (spread)
            line(d, "for (size_t " + s.ident + " = lane; " + s.ident + " < " + expr_text(*s.value) + "; " + s.ident + " += 64) {");
          else if (in_parts)
            line(d, "for (size_t " + s.ident + " = part * share_" + s.ident + "; " + s.ident + " < end_" + s.ident + "; ++" + s.ident + ") {");
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

// ------------------------------------------------------------------ one kernel per loop nest
void visit_scalar_params(ScalarExpr<Param>& e, const std::function<void(Param&)>& f) {
  if (e.kind == ScalarExpr<Param>::Acc) f(e.access.buffer);
  for (auto& a : e.args) visit_scalar_params(a, f);
}
// every reference to a kernel parameter in a block: accesses, and the buffers whose extents bound the loops
void visit_params(Block<Param>& block, const std::function<void(Param&)>& f) {
  for (PAct& a : block) {
    switch (a.kind) {
      case PAct::Loop:
        f(a.extent.source.buffer);
        visit_params(a.body, f);
        break;
      case PAct::Init: f(a.write.buffer); break;
      case PAct::Compute:
      case PAct::Snapshot:
        f(a.write.buffer);
        for (auto& r : a.reads) f(r.buffer);
        break;
      case PAct::Scale:
        f(a.write.buffer);
        visit_scalar_params(a.factor, f);
        break;
    }
  }
}

// The form of a nest with its outermost sequential loop in parts (GridForm), or nothing when the nest does not
// qualify.  Walking down from the top of the body, through the parallel loops, the first sequential loop G is the
// one in parts; on the way there may only be initialisations.  Under G there are only loops, initialisations
// (checked for the first iteration of the loops they sit in) and Computes, and every Compute either stores into a
// work-item-private buffer or accumulates (+, *, max, min) into a buffer that nothing under G reads: then part p
// may run iterations p, p + parts, ... of G on a copy of each accumulated buffer that starts as the reduction's
// identity, and the copies fold into the buffer afterwards, element by element, in part order.
void grid_plan(const Block<Param>& body, const std::set<Param>& accumulating, const std::map<size_t, std::vector<size_t>>& held,
               GenericPhase& phase) {
  auto is_parallel = [&](size_t id) { return std::find(phase.parallel_loops.begin(), phase.parallel_loops.end(), id) != phase.parallel_loops.end(); };
  auto is_private = [&](const Param& w) {
    if (!w.writeable) return false;
    for (const PrivateBuffer& pb : phase.privates)
      if (pb.writeable == w.ind) return true;
    return false;
  };
  std::set<Param> initialised_here;
  const Block<Param>* block = &body;
  const PAct* g = nullptr;
  while (!g) {
    const PAct* only = nullptr;
    for (const PAct& a : *block) {
      if (a.kind == PAct::Loop) {
        if (only) return;
        only = &a;
      } else if (a.kind == PAct::Init) {
        initialised_here.insert(a.write.buffer);
      } else {
        return;
      }
    }
    if (!only) return;
    if (is_parallel(only->id)) block = &only->body;
    else g = only;
  }
  std::map<Param, Op> ops;
  std::vector<const PAct*> computes;
  std::vector<const Block<Param>*> todo{&g->body};
  while (!todo.empty()) {
    const Block<Param>* b = todo.back();
    todo.pop_back();
    for (const PAct& a : *b) {
      if (a.kind == PAct::Loop) todo.push_back(&a.body);
      else if (a.kind == PAct::Init) initialised_here.insert(a.write.buffer);
      else if (a.kind == PAct::Compute) computes.push_back(&a);
      else return;
    }
  }
  for (const PAct* c : computes) {
    const Param w = c->write.buffer;
    if (is_private(w)) continue;
    const bool known = c->op == Op::Add || c->op == Op::Mul || c->op == Op::Max || c->op == Op::Min;
    if (!w.writeable || !accumulating.count(w) || !known) return;
    auto [it, fresh] = ops.emplace(w, c->op);
    if (!fresh && it->second != c->op) return;
  }
  if (ops.empty()) return;
  for (const PAct* c : computes)
    for (const auto& r : c->reads)
      if (ops.count(r.buffer)) return;
  for (const Param& w : initialised_here)
    if (!ops.count(w)) return;  // (an initialisation of something that is no accumulator of this nest)
  phase.grid.available = true;
  phase.grid.loop = g->id;
  phase.grid.extent = g->extent;
  for (const auto& [w, op] : ops) phase.grid.accumulators.push_back({w.ind, op, initialised_here.count(w) != 0});
  // every accumulator kept in a register across G (and nowhere else under it: held by G itself): the parts then
  // never read their copies, they only store into them
  const auto held_by_g = held.find(g->id);
  phase.grid.held_accumulators = held_by_g != held.end();
  for (const auto& [w, op] : ops)
    phase.grid.held_accumulators = phase.grid.held_accumulators &&
                                   std::find(held_by_g->second.begin(), held_by_g->second.end(), w.ind) != held_by_g->second.end();
  // the wavefront form of the same: when the nest has one and G is its loop over (or around) the lanes
  for (const WaveLoop& wl : phase.wave_loops)
    if (wl.loop == g->id && !wl.accumulators.empty()) {
      phase.grid.wave = true;
      phase.grid.loop_is_spread = wl.spread == g->id;
    }
  if (phase.wave_loops.size() != 1) phase.grid.wave = false;
}

}  // namespace

ExecPlan split_nests(const ExecPlan& plan, std::vector<size_t>* origin) {
  ExecPlan out = plan;
  out.kernels.clear();
  out.exec.clear();
  origin->clear();
  std::vector<std::vector<size_t>> pieces_of(plan.kernels.size());   // new kernel ids per old kernel
  std::vector<std::vector<std::vector<size_t>>> kept_reads, kept_writes;  // per new kernel: positions in the old lists
  for (size_t k = 0; k < plan.kernels.size(); ++k) {
    const Kernel<Param>& kernel = plan.kernels[k];
    std::set<Param> initialised;
    collect_initialized(kernel.body, initialised);
    initialised.insert(kernel.accumulates.begin(), kernel.accumulates.end());
    // a run of statements that are no loops goes with the loop after it when that loop writes what the run
    // initialises (a scalar total and the loop that adds to it), otherwise it is a piece of its own
    std::vector<std::pair<size_t, size_t>> ranges;
    for (const auto& [first, last] : phase_ranges(kernel.body)) {
      bool joined = false;
      if (!ranges.empty() && first < last && kernel.body[first].kind == PAct::Loop) {
        const auto [pf, pl] = ranges.back();
        bool run = pf < pl;
        std::set<Param> set_by_run;
        for (size_t n = pf; n < pl; ++n) {
          run = run && kernel.body[n].kind == PAct::Init;
          set_by_run.insert(kernel.body[n].write.buffer);
        }
        if (run) {
          Uses u;
          collect_one(kernel.body[first], u);
          for (const Param& w : u.written) joined = joined || set_by_run.count(w);
        }
      }
      if (joined) ranges.back().second = last;
      else ranges.push_back({first, last});
    }
    for (const auto& [first, last] : ranges) {
      Kernel<Param> piece;
      piece.body.assign(kernel.body.begin() + first, kernel.body.begin() + last);
      std::set<Param> used;
      visit_params(piece.body, [&](Param& p) { used.insert(p); });
      std::vector<size_t> reads, writes;
      std::map<Param, Param> renamed;
      for (size_t r = 0; r < kernel.reads.size(); ++r)
        if (ranges.size() == 1 || used.count(Param{false, r})) {
          renamed[Param{false, r}] = Param{false, reads.size()};
          reads.push_back(r);
          piece.reads.push_back(kernel.reads[r]);
        }
      for (size_t w = 0; w < kernel.writes.size(); ++w)
        if (ranges.size() == 1 || used.count(Param{true, w})) {
          renamed[Param{true, w}] = Param{true, writes.size()};
          writes.push_back(w);
          piece.writes.push_back(kernel.writes[w]);
        }
      visit_params(piece.body, [&](Param& p) {
        auto it = renamed.find(p);
        if (it == renamed.end()) lower_error("kernel body names a buffer that is not in its lists");
        p = it->second;
      });
      for (const Param& w : initialised)
        if (renamed.count(w)) piece.accumulates.push_back(renamed[w]);
      pieces_of[k].push_back(out.kernels.size());
      origin->push_back(k);
      out.kernels.push_back(std::move(piece));
      kept_reads.push_back({reads});
      kept_writes.push_back({writes});
    }
  }
  for (const Step& step : plan.exec) {
    if (step.kind != Step::Dispatch) {
      out.exec.push_back(step);
      continue;
    }
    for (size_t piece : pieces_of.at(step.id)) {
      Step s;
      s.kind = Step::Dispatch;
      s.id = piece;
      for (size_t r : kept_reads[piece][0]) s.reads.push_back(step.reads.at(r));
      for (size_t w : kept_writes[piece][0]) s.writes.push_back(step.writes.at(w));
      out.exec.push_back(std::move(s));
    }
  }
  return out;
}

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
  bool any = false, any_grid = false;
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
    size_t fn_stmts = fn.body.size();
    while (fn_stmts > 0 && fn.body[fn_stmts - 1].kind == MStmt::Return) --fn_stmts;
    const std::vector<MStmt> stmts(fn.body.begin(), fn.body.begin() + fn_stmts);

    GenericPhase phase;
    phase.name = info.name;
    analyze(plan, k, body, {}, phase);
    std::map<size_t, std::vector<size_t>> held;
    held_elements(body, std::set<size_t>(phase.parallel_loops.begin(), phase.parallel_loops.end()), held);
    std::set<Param> initialized;
    collect_initialized(body, initialized);
    initialized.insert(plan.kernels[k].accumulates.begin(), plan.kernels[k].accumulates.end());
    wave_plan(body, initialized, held, phase);
    grid_plan(body, initialized, held, phase);
    any_grid = any_grid || phase.grid.available;

    const size_t nr = std::max<size_t>(info.n_reads, 1), nw = std::max<size_t>(info.n_writes, 1);
    src << "struct Args_" << info.name << " { View readonlys[" << nr << "]; View writeables[" << nw << "]; };\n";
    if (phase.grid.available)
      src << "struct Args_" << info.name << "_g { View readonlys[" << nr << "]; View writeables[" << nw << "]; float* partial[" << nw
          << "]; size_t parts; };\n";
    const Step* dispatch = nullptr;
    for (const Step& st : plan.exec)
      if (st.kind == Step::Dispatch && st.id == k) dispatch = &st;
    auto rank_of = [&](BufferRef r) {
      return (r.kind == BufferRef::Input ? plan.inputs.at(r.id) : r.kind == BufferRef::Intermediate ? plan.intermediates.at(r.id)
                                                                                                   : plan.outputs.at(r.id)).layout.size();
    };
    // element counts of the kernel's views, for the checked accesses: the product of the layout extents (a
    // work-item-private slice or array has the same layout as the buffer it stands for)
    auto emit_capacities = [&](const std::string& pad) {
      if (!g_checked_accesses) return;
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
    // work-item-private buffers: a local array, or this work-item's slice of a device buffer
    auto emit_privates = [&](const std::string& pad) {
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
    // the nest spread over the work-items (wi_first, wi_stride); in_parts: over (work-item, part) pairs
    auto emit_spread = [&](int depth, bool wave, bool in_parts) {
      const std::string pad(2 * depth, ' ');
      Printer pr;
      pr.held = &held;
      if (wave) pr.wave = &phase.wave_loops;
      if (in_parts) pr.grid = &phase.grid;
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
      // The work-item index is a number in mixed radix (the extents of the parallel loops, the last one fastest; in
      // the form with a loop in parts the part is one more digit in front).  Its digits are taken apart once, for the
      // first index and for the stride, and then advanced digit by digit with carries: no division in the loop.
      std::vector<std::string> digits;  // most significant first
      if (in_parts) {
        src << pad << "const size_t parts = args.parts;\n";
        for (const GridAccumulator& acc : phase.grid.accumulators) {
          src << pad << "const size_t part_cap" << acc.writeable << " = (size_t)1";
          for (size_t d = 0; d < rank_of(dispatch->writes[acc.writeable]); ++d)
            src << " * writeables[" << acc.writeable << "].layout[" << d << "]";
          src << ";\n";
        }
        src << pad << "const size_t n_part = parts;\n";
        digits.push_back("part");
      }
      for (const std::string& it : iters) digits.push_back(it);
      const std::string all = in_parts ? "wi_total * parts" : "wi_total";
      src << pad << "if (" << all << " == 0) return;\n";
      if (!digits.empty()) {
        src << pad << "size_t wi_rest = wi_first < " << all << " ? wi_first : 0, step_rest = wi_stride;\n";
        for (size_t t = digits.size(); t-- > 0;) {
          src << pad << "size_t at_" << digits[t] << " = wi_rest % n_" << digits[t] << "; wi_rest /= n_" << digits[t] << ";\n";
          src << pad << "const size_t step_" << digits[t] << " = step_rest % n_" << digits[t] << "; step_rest /= n_" << digits[t] << ";\n";
        }
      }
      src << pad << "for (size_t wi = wi_first; wi < " << all << "; wi += wi_stride) {\n";
      for (const std::string& dg : digits) src << pad << "  const size_t " << dg << " = at_" << dg << ";\n";
      if (in_parts)  // this part's copy of every accumulated buffer stands where the buffer stood
        for (const GridAccumulator& acc : phase.grid.accumulators)
          src << pad << "  writeables[" << acc.writeable << "].data = args.partial[" << acc.writeable << "] + part * part_cap"
              << acc.writeable << ";\n";
      pr.block(stmts, depth + 1);
      src << pr.os.str();
      if (!digits.empty()) {
        src << pad << "  {\n" << pad << "    size_t carry = 0;\n";
        for (size_t t = digits.size(); t-- > 0;) {
          src << pad << "    at_" << digits[t] << " += step_" << digits[t] << " + carry;\n";
          src << pad << "    carry = at_" << digits[t] << " >= n_" << digits[t] << " ? 1 : 0;\n";
          src << pad << "    if (carry) at_" << digits[t] << " -= n_" << digits[t] << ";\n";
        }
        src << pad << "  }\n";
      }
      src << pad << "}\n";
    };
    // forms: the nest as it is; _w: a wavefront per work-item; _g / _gw: either with the outermost sequential loop in parts
    struct Form { bool wave, in_parts; const char* suffix; };
    for (const Form form : {Form{false, false, ""}, Form{true, false, "_w"}, Form{false, true, "_g"}, Form{true, true, "_gw"}}) {
      if (form.wave && !form.in_parts && phase.wave_loops.empty()) continue;
      if (form.in_parts && (!phase.grid.available || (form.wave && !phase.grid.wave))) continue;
      src << "extern \"C\" __global__ void __launch_bounds__(" << (form.wave ? GenericPhase::kWaveThreads : 64u) << ") " << phase.name
          << form.suffix << "(Args_" << info.name << (form.in_parts ? "_g" : "") << " args) {\n";
      src << "  const View* readonlys = args.readonlys;\n";
      src << "  View writeables[" << nw << "];\n";
      src << "  for (int b = 0; b < " << nw << "; ++b) writeables[b] = args.writeables[b];\n";
      if (form.wave) {
        src << "  const size_t lane = threadIdx.x % 64;\n";
        src << "  const size_t wi_first = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / 64;\n";
        src << "  const size_t wi_stride = ((size_t)gridDim.x * blockDim.x) / 64;\n";
      } else {
        src << "  const size_t wi_first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;\n";
        src << "  const size_t wi_stride = (size_t)gridDim.x * blockDim.x;\n";
      }
      emit_capacities("  ");
      emit_privates("  ");
      if (phase.parallel_loops.empty() && !form.in_parts) {
        src << "  if (wi_first != 0) return;\n";
        Printer pr;
        pr.held = &held;
        if (form.wave) pr.wave = &phase.wave_loops;
        pr.block(stmts, 1);
        src << pr.os.str();
      } else {
        emit_spread(1, form.wave, form.in_parts);
      }
      src << "}\n\n";
    }
    info.phases.push_back(std::move(phase));
  }
  if (any_grid) {
    // the two helpers of the form with a loop in parts: the parts' copies start as the reduction's identity, and
    // fold into the accumulated buffer in part order (op: 0 +, 1 *, 2 max, 3 min; keep: the buffer's own value
    // takes part, i.e. the nest did not initialise it)
    src << "struct Args_" << kFillKernel << " { float* data; size_t count; float value; };\n";
    src << "extern \"C\" __global__ void __launch_bounds__(256) " << kFillKernel << "(Args_" << kFillKernel << " args) {\n";
    src << "  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < args.count; e += (size_t)gridDim.x * blockDim.x)\n";
    src << "    args.data[e] = args.value;\n}\n\n";
    src << "struct Args_" << kCombineKernel << " { const float* partial; float* data; size_t parts; size_t count; int op; int keep; };\n";
    src << "extern \"C\" __global__ void __launch_bounds__(256) " << kCombineKernel << "(Args_" << kCombineKernel << " args) {\n";
    src << "  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < args.count; e += (size_t)gridDim.x * blockDim.x) {\n";
    src << "    float acc = args.partial[e];\n";
    src << "    #pragma unroll 8\n";
    src << "    for (size_t p = 1; p < args.parts; ++p) {\n";
    src << "      const float v = args.partial[p * args.count + e];\n";
    src << "      acc = args.op == 0 ? acc + v : args.op == 1 ? acc * v : args.op == 2 ? fmaxf(acc, v) : fminf(acc, v);\n";
    src << "    }\n";
    src << "    if (args.keep) {\n";
    src << "      const float v = args.data[e];\n";
    src << "      acc = args.op == 0 ? v + acc : args.op == 1 ? v * acc : args.op == 2 ? fmaxf(v, acc) : fminf(v, acc);\n";
    src << "    }\n";
    src << "    args.data[e] = acc;\n";
    src << "  }\n}\n\n";
    // the same for a few elements and many parts: a wavefront per element, its lanes over the parts
    src << "extern \"C\" __global__ void __launch_bounds__(256) " << kCombineWaveKernel << "(Args_" << kCombineKernel << " args) {\n";
    src << "  const size_t lane = threadIdx.x % 64;\n";
    src << "  for (size_t e = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / 64; e < args.count; e += ((size_t)gridDim.x * blockDim.x) / 64) {\n";
    src << "    float acc = args.op == 0 ? 0.0f : args.op == 1 ? 1.0f : args.op == 2 ? (-INFINITY) : INFINITY;\n";
    src << "    #pragma unroll 8\n";
    src << "    for (size_t p = lane; p < args.parts; p += 64) {\n";
    src << "      const float v = args.partial[p * args.count + e];\n";
    src << "      acc = args.op == 0 ? acc + v : args.op == 1 ? acc * v : args.op == 2 ? fmaxf(acc, v) : fminf(acc, v);\n";
    src << "    }\n";
    src << "    for (int lane_xor = 32; lane_xor > 0; lane_xor >>= 1) {\n";
    src << "      const float v = __shfl_xor(acc, lane_xor);\n";
    src << "      acc = args.op == 0 ? acc + v : args.op == 1 ? acc * v : args.op == 2 ? fmaxf(acc, v) : fminf(acc, v);\n";
    src << "    }\n";
    src << "    if (args.keep) {\n";
    src << "      const float v = args.data[e];\n";
    src << "      acc = args.op == 0 ? v + acc : args.op == 1 ? v * acc : args.op == 2 ? fmaxf(v, acc) : fminf(v, acc);\n";
    src << "    }\n";
    src << "    ILANG_WAVE_SYNC();\n";
    src << "    if (lane == 0) args.data[e] = acc;\n";
    src << "  }\n}\n\n";
  }
  if (any) out.source = src.str();
  return out;
}

}  // namespace ihipc
