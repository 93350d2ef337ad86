// ExecPlan -> Module, the statement-level IR both text backends print.  This is
// where the scalar semantics are fixed: reduction identities, unary defaults
// (neg, recip, relu-style max/min against 0, e^x, ln, comparisons against 0),
// `dst = op(dst, reads...)` for buffers that have an Init anywhere in the kernel,
// ceil-div loop bounds, the tail guard `tile*F + inner < dim`, row-major flat
// indexing over layout[], Snapshot as plain assignment and Scale as
// `dst = dst * factor`.  Follows compiler/src/lower/exec_plan_to_module.rs:15-760.
#include <algorithm>
#include <cmath>
#include <map>
#include <set>

#include "ir.h"

namespace ic {
namespace {

MExprPtr mk(MExpr e) { return std::make_shared<const MExpr>(std::move(e)); }
MExprPtr usize(size_t v) { MExpr e; e.kind = MExpr::Usize; e.usize = v; return mk(e); }
MExprPtr scalar(float v) { MExpr e; e.kind = MExpr::Scalar; e.scalar = v; return mk(e); }
MExprPtr ident(const std::string& s) { MExpr e; e.kind = MExpr::Ident; e.ident = s; return mk(e); }
MExprPtr index(MExprPtr base, MExprPtr ix) { MExpr e; e.kind = MExpr::Index; e.args = {base, ix}; return mk(e); }
MExprPtr field(MExprPtr base, MField f) { MExpr e; e.kind = MExpr::Field; e.field = f; e.args = {base}; return mk(e); }
MExprPtr cast(MCast c, MExprPtr v) { MExpr e; e.kind = MExpr::Cast; e.cast = c; e.args = {v}; return mk(e); }
MExprPtr bin(MExpr::Kind k, MExprPtr l, MExprPtr r) { MExpr e; e.kind = k; e.args = {l, r}; return mk(e); }
MExprPtr opcall(Op op, std::vector<MExprPtr> args) { MExpr e; e.kind = MExpr::OpCall; e.op = op; e.args = std::move(args); return mk(e); }

MExprPtr input_dim(DimRef<size_t> d) { return index(field(index(ident("inputs"), usize(d.buffer)), MField::Shape), usize(d.dim)); }
MExprPtr param_expr(Param p) { return index(ident(p.writeable ? "writeables" : "readonlys"), usize(p.ind)); }
MExprPtr param_dim(DimRef<Param> d) { return index(field(param_expr(d.buffer), MField::Shape), usize(d.dim)); }

MExprPtr extent_expr(MExprPtr source, const ExtentKind& kind) {
  switch (kind.kind) {
    case ExtentKind::Semantic: return source;
    case ExtentKind::Base: {
      size_t f = 1;
      for (size_t x : kind.factors) f *= x;
      if (f == 1) return source;
      return bin(MExpr::Div, bin(MExpr::Sub, bin(MExpr::Add, source, usize(f)), usize(1)), usize(f));
    }
    case ExtentKind::Split: return usize(kind.factor);
  }
  return source;
}

// iters are outermost first; iter t is weighted by the product of the factors from t on
MExprPtr reconstruct_index(const std::vector<MExprPtr>& iters, const std::vector<size_t>& factors) {
  if (iters.empty()) return usize(0);
  MExprPtr sum;
  for (size_t t = 0; t < iters.size(); ++t) {
    size_t weight = 1;
    if (!factors.empty() && t < factors.size())
      for (size_t f = t; f < factors.size(); ++f) weight *= factors[f];
    MExprPtr term = (factors.empty() || weight == 1) ? iters[t] : bin(MExpr::Mul, iters[t], usize(weight));
    sum = sum ? bin(MExpr::Add, sum, term) : term;
  }
  return sum;
}

MExprPtr init_value(Op op) {
  switch (op) {
    case Op::Add: case Op::Or: case Op::Xor: return scalar(0.0f);
    case Op::Mul: case Op::And: return scalar(1.0f);
    case Op::Max: return scalar(-INFINITY);
    case Op::Min: return scalar(INFINITY);
    default: lower_error(std::string("op ") + op_name(op) + " has no reduction identity");
  }
}

MExprPtr scalar_op_expr(Op op, std::vector<MExprPtr> args) {
  if (args.size() != 1) return opcall(op, std::move(args));
  MExprPtr arg = args[0];
  switch (op) {
    case Op::Add: case Op::Mul: case Op::And: case Op::Or: case Op::Xor: return arg;
    case Op::Sub: return opcall(op, {scalar(0.0f), arg});
    case Op::Div: return opcall(op, {scalar(1.0f), arg});
    case Op::Max: case Op::Min: return opcall(op, {scalar(0.0f), arg});
    case Op::Gt: case Op::Ge: case Op::Lt: case Op::Le: case Op::Eq: case Op::Ne: return opcall(op, {arg, scalar(0.0f)});
    case Op::Pow: return opcall(op, {scalar(2.71828182845904523536f), arg});
    case Op::Log: case Op::Not: return opcall(op, {arg});
  }
  return arg;
}

struct LoopScope {
  std::string iter;
  DimRef<Param> source;
  ExtentKind kind;
};

struct KernelLowerer {
  std::set<Param> initialized;
  std::map<size_t, LoopScope> loops;
  std::vector<std::pair<DimRef<Param>, DimRef<size_t>>> semantic_dims;

  std::optional<DimRef<size_t>> semantic_dim(DimRef<Param> d) const {
    for (const auto& [p, in] : semantic_dims)
      if (p == d) return in;
    return std::nullopt;
  }
  MExprPtr loop_expr(size_t id) const {
    auto it = loops.find(id);
    if (it == loops.end()) lower_error("loop " + std::to_string(id) + " is not in scope");
    return ident(it->second.iter);
  }
  MExprPtr lower_iter(const Iter& it) const {
    if (it.raw) return loop_expr(it.loop);
    std::vector<MExprPtr> iters;
    for (size_t id : it.loops) iters.push_back(loop_expr(id));
    return reconstruct_index(iters, it.factors);
  }
  MExprPtr flat_index(MExprPtr buffer, const std::vector<Iter>& ix) const {
    if (ix.empty()) return usize(0);
    std::vector<MExprPtr> dims;
    for (const Iter& it : ix) dims.push_back(lower_iter(it));
    MExprPtr sum;
    for (size_t d = 0; d < dims.size(); ++d) {
      MExprPtr stride;
      for (size_t l = d + 1; l < dims.size(); ++l) {
        MExprPtr e = index(field(buffer, MField::Layout), usize(l));
        stride = stride ? bin(MExpr::Mul, stride, e) : e;
      }
      MExprPtr term = stride ? bin(MExpr::Mul, dims[d], stride) : dims[d];
      sum = sum ? bin(MExpr::Add, sum, term) : term;
    }
    return sum;
  }
  MExprPtr element(const Access<Param>& a) const {
    MExprPtr buffer = param_expr(a.buffer);
    return index(field(buffer, MField::Data), flat_index(buffer, a.index));
  }
  MExprPtr scale_expr(const ScalarExpr<Param>& e) const {
    if (e.kind == ScalarExpr<Param>::Acc) return element(e.access);
    std::vector<MExprPtr> args;
    for (const auto& a : e.args) args.push_back(scale_expr(a));
    return scalar_op_expr(e.op, std::move(args));
  }
  // semantic position along the dim a loop tiles, rebuilt from every loop in scope over that dim
  MExprPtr reconstruct_extent_index(DimRef<Param> source) const {
    const auto sem = semantic_dim(source);
    std::vector<const LoopScope*> infos;
    for (const auto& [id, info] : loops) {
      const bool same = sem ? (semantic_dim(info.source) == sem) : (info.source == source);
      if (same) infos.push_back(&info);
    }
    std::stable_sort(infos.begin(), infos.end(), [](const LoopScope* a, const LoopScope* b) { return a->kind.order() < b->kind.order(); });
    std::vector<MExprPtr> iters;
    std::vector<size_t> factors;
    bool base = false;
    for (const LoopScope* i : infos) iters.push_back(ident(i->iter));
    for (const LoopScope* i : infos)
      if (i->kind.kind == ExtentKind::Base) {
        factors = i->kind.factors;
        base = true;
        break;
      }
    if (!base)
      for (const LoopScope* i : infos)
        if (i->kind.kind == ExtentKind::Split) factors.push_back(i->kind.factor);
    const size_t expected = infos.empty() ? 0 : infos.size() - 1;
    if (factors.size() > expected) factors.erase(factors.begin(), factors.end() - expected);
    return reconstruct_index(iters, factors);
  }

  std::vector<MStmt> lower_block(const Block<Param>& block) {
    std::vector<MStmt> out;
    for (const auto& a : block) out.push_back(lower_action(a));
    return out;
  }

  MStmt lower_action(const Action<Param>& a) {
    MStmt s;
    switch (a.kind) {
      case Action<Param>::Loop: {
        const std::string iter = "i" + std::to_string(a.id);
        loops[a.id] = {iter, a.extent.source, a.extent.kind};
        std::vector<MStmt> body = lower_block(a.body);
        if (a.guard) {
          MStmt g;
          g.kind = MStmt::If;
          g.value = bin(MExpr::Lt, reconstruct_extent_index(a.extent.source), param_dim(a.extent.source));
          g.body = std::move(body);
          body = {g};
        }
        loops.erase(a.id);
        s.kind = MStmt::Loop;
        s.ident = iter;
        s.value = extent_expr(param_dim(a.extent.source), a.extent.kind);
        s.body = std::move(body);
        return s;
      }
      case Action<Param>::Init: {
        MStmt init;
        init.kind = MStmt::Set;
        init.dst = element(a.write);
        init.value = init_value(a.op);
        MExprPtr cond;
        for (size_t id : a.zero_checks) {
          auto it = loops.find(id);
          if (it == loops.end()) lower_error("zero check references loop " + std::to_string(id));
          MExprPtr c = bin(MExpr::Eq, ident(it->second.iter), usize(0));
          cond = cond ? bin(MExpr::And, cond, c) : c;
        }
        if (!cond) return init;
        s.kind = MStmt::If;
        s.value = cond;
        s.body = {init};
        return s;
      }
      case Action<Param>::Compute: {
        s.kind = MStmt::Set;
        s.dst = element(a.write);
        std::vector<MExprPtr> args;
        if (initialized.count(a.write.buffer)) args.push_back(s.dst);
        for (const auto& r : a.reads) args.push_back(element(r));
        s.value = scalar_op_expr(a.op, std::move(args));
        return s;
      }
      case Action<Param>::Snapshot:
        s.kind = MStmt::Set;
        s.dst = element(a.write);
        s.value = element(a.reads[0]);
        return s;
      case Action<Param>::Scale:
        s.kind = MStmt::Set;
        s.dst = element(a.write);
        s.value = bin(MExpr::Mul, s.dst, scale_expr(a.factor));
        return s;
    }
    return s;
  }
};

void collect_initialized(const Block<Param>& block, std::set<Param>& out) {
  for (const auto& a : block) {
    if (a.kind == Action<Param>::Loop) collect_initialized(a.body, out);
    else if (a.kind == Action<Param>::Init) out.insert(a.write.buffer);
  }
}

std::string buffer_ident(BufferRef r) {
  return (r.kind == BufferRef::Input ? "in" : r.kind == BufferRef::Intermediate ? "s" : "out") + std::to_string(r.id);
}

}  // namespace

Module lower_exec_plan_to_module(const ExecPlan& plan) {
  Module m;
  auto ret = [](MExprPtr v) { MStmt s; s.kind = MStmt::Return; s.value = v; return s; };
  auto set = [](MExprPtr dst, MExprPtr v) { MStmt s; s.kind = MStmt::Set; s.dst = dst; s.value = v; return s; };

  m.count = {"count", MSignature::Count, {ret(usize(plan.count))}};
  m.ranks = {"ranks", MSignature::Ranks, {}};
  for (size_t o = 0; o < plan.ranks.size(); ++o) m.ranks.body.push_back(set(index(ident("ranks"), usize(o)), usize(plan.ranks[o])));
  m.ranks.body.push_back(ret(nullptr));
  m.shapes = {"shapes", MSignature::Shapes, {}};
  for (size_t o = 0; o < plan.shapes.size(); ++o)
    for (size_t d = 0; d < plan.shapes[o].size(); ++d)
      m.shapes.body.push_back(set(index(index(ident("shapes"), usize(o)), usize(d)), input_dim(plan.shapes[o][d])));
  m.shapes.body.push_back(ret(nullptr));

  m.exec = {"exec", MSignature::Exec, {}};
  for (size_t i = 0; i < plan.inputs.size(); ++i) {
    MStmt s;
    s.kind = MStmt::Let;
    s.ident = "in" + std::to_string(i);
    s.type = MType::View;
    s.value = cast(MCast::View, index(ident("inputs"), usize(i)));
    m.exec.body.push_back(s);
  }
  for (size_t o = 0; o < plan.outputs.size(); ++o) {
    MStmt s;
    s.kind = MStmt::Let;
    s.ident = "out" + std::to_string(o);
    s.type = MType::ViewMut;
    s.value = cast(MCast::ViewMut, index(ident("outputs"), usize(o)));
    m.exec.body.push_back(s);
  }
  for (const Step& step : plan.exec) {
    MStmt s;
    switch (step.kind) {
      case Step::Alloc: {
        const PlanBuffer& buffer = plan.intermediates.at(step.id);
        s.kind = MStmt::Alloc;
        s.ident = "s" + std::to_string(step.id);
        for (const auto& d : buffer.shape) s.shape.push_back(input_dim(d));
        for (const auto& e : buffer.layout) s.layout.push_back(extent_expr(input_dim(e.source), e.kind));
        break;
      }
      case Step::Dispatch:
        s.kind = MStmt::Dispatch;
        s.ident = "f" + std::to_string(step.id);
        for (BufferRef r : step.reads) s.reads.push_back(buffer_ident(r));
        for (BufferRef r : step.writes) s.writes.push_back(buffer_ident(r));
        break;
      case Step::Free:
        s.kind = MStmt::Free;
        s.ident = "s" + std::to_string(step.id);
        break;
    }
    m.exec.body.push_back(std::move(s));
  }
  m.exec.body.push_back(ret(nullptr));

  for (size_t k = 0; k < plan.kernels.size(); ++k) {
    const Step* dispatch = nullptr;
    for (const Step& step : plan.exec)
      if (step.kind == Step::Dispatch && step.id == k) {
        dispatch = &step;
        break;
      }
    if (!dispatch) lower_error("kernel " + std::to_string(k) + " is never dispatched");
    KernelLowerer kl;
    auto buffer_shape = [&](BufferRef r) -> const std::vector<DimRef<size_t>>& {
      const auto& list = r.kind == BufferRef::Input ? plan.inputs : r.kind == BufferRef::Intermediate ? plan.intermediates : plan.outputs;
      if (r.id >= list.size()) lower_error("dispatch references nonexistent buffer");
      return list[r.id].shape;
    };
    for (size_t i = 0; i < dispatch->reads.size(); ++i) {
      const auto& shape = buffer_shape(dispatch->reads[i]);
      for (size_t d = 0; d < shape.size(); ++d) kl.semantic_dims.push_back({{Param{false, i}, d}, shape[d]});
    }
    for (size_t i = 0; i < dispatch->writes.size(); ++i) {
      const auto& shape = buffer_shape(dispatch->writes[i]);
      for (size_t d = 0; d < shape.size(); ++d) kl.semantic_dims.push_back({{Param{true, i}, d}, shape[d]});
    }
    collect_initialized(plan.kernels[k].body, kl.initialized);
    kl.initialized.insert(plan.kernels[k].accumulates.begin(), plan.kernels[k].accumulates.end());
    m.kernels.push_back({"f" + std::to_string(k), MSignature::Kernel, kl.lower_block(plan.kernels[k].body)});
  }
  return m;
}

}  // namespace ic
