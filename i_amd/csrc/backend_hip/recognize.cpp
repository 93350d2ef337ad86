#include "recognize.h"

#include <algorithm>
#include <map>
#include <optional>
#include <set>

namespace ihipc {
using namespace ic;
namespace {

struct Term;
struct Arg {
  bool external = true;
  size_t kp_buffer = 0;   // kernel-program buffer id (external)
  std::vector<int> dims;  // symbols of the operand's dims
  int term = -1;          // interior producer
};
struct Term {
  Op op = Op::Add;
  std::vector<int> out;  // output dim symbols
  std::vector<int> red;  // reduced symbols (sorted)
  std::vector<Arg> args;
};

struct TreeBuilder {
  const StageProgram& sp;
  std::vector<Term> terms;
  int next_symbol = 0;

  int build(size_t stage_id, const std::map<size_t, int>& bound) {
    const auto& gnode = sp.graph.nodes[stage_id];
    const Stage& st = gnode.inner;
    std::map<size_t, int> sym = bound;
    std::set<size_t> indexes;
    for (const SAxis& a : st.axes) indexes.insert(a.index);
    for (size_t ix : st.output.shape) indexes.insert(ix);
    for (const auto& in : st.inputs)
      for (size_t ix : in.shape) indexes.insert(ix);
    for (size_t ix : indexes)
      if (!sym.count(ix)) sym[ix] = next_symbol++;
    Term t;
    t.op = st.op;
    std::set<size_t> out_set(st.output.shape.begin(), st.output.shape.end());
    for (size_t ix : st.output.shape) t.out.push_back(sym[ix]);
    for (size_t ix : indexes)
      if (!out_set.count(ix)) t.red.push_back(sym[ix]);
    std::sort(t.red.begin(), t.red.end());
    for (size_t i = 0; i < st.inputs.size(); ++i) {
      Arg a;
      for (size_t ix : st.inputs[i].shape) a.dims.push_back(sym[ix]);
      const Source src = gnode.inputs[i];
      if (st.inputs[i].site && !src.is_input) {
        const Stage& prod = sp.graph.nodes[src.id].inner;
        std::map<size_t, int> pb;
        for (size_t d = 0; d < prod.output.shape.size(); ++d) pb[prod.output.shape[d]] = a.dims[d];
        a.external = false;
        a.term = build(src.id, pb);
      } else {
        a.external = true;
        a.kp_buffer = src.is_input ? src.id : sp.graph.inputs + src.id;
      }
      t.args.push_back(std::move(a));
    }
    terms.push_back(std::move(t));
    return int(terms.size()) - 1;
  }

  // Structural equality of two subtrees up to a renaming of index symbols.
  // `ren` maps symbols of x to symbols of y; unseen symbols are bound on first use.
  bool unify_sym(int p, int q, std::map<int, int>& ren) const {
    auto it = ren.find(p);
    if (it != ren.end()) return it->second == q;
    ren[p] = q;
    return true;
  }
  bool unify_dims(const std::vector<int>& p, const std::vector<int>& q, std::map<int, int>& ren) const {
    if (p.size() != q.size()) return false;
    for (size_t d = 0; d < p.size(); ++d)
      if (!unify_sym(p[d], q[d], ren)) return false;
    return true;
  }
  bool unify_arg(const Arg& p, const Arg& q, std::map<int, int>& ren) const {
    if (p.external != q.external || !unify_dims(p.dims, q.dims, ren)) return false;
    return p.external ? p.kp_buffer == q.kp_buffer : unify(p.term, q.term, ren);
  }
  bool unify(int x, int y, std::map<int, int>& ren) const {
    const Term &a = terms[x], &b = terms[y];
    if (a.op != b.op || a.red.size() != b.red.size() || a.args.size() != b.args.size()) return false;
    if (!unify_dims(a.out, b.out, ren)) return false;
    for (size_t i = 0; i < a.args.size(); ++i)
      if (!unify_arg(a.args[i], b.args[i], ren)) return false;
    return true;
  }
};

struct Matcher {
  const TreeBuilder& tb;
  const std::vector<BufferRef>& refs;  // kernel-program buffer -> plan ref

  const Term& T(int i) const { return tb.terms[i]; }
  Operand operand(const Arg& a) const { return {refs[a.kp_buffer], a.dims}; }

  // S = sum_D q[B.., I, D] * k[B.., J, D], output dims [B.., I, J]
  // sum_D a[B.., I, D] * b[B.., D, J]  (either operand order)
  bool match_mm(int t, Recognized& r) const {
    const Term& add = T(t);
    if (add.op != Op::Add || add.red.size() != 1 || add.args.size() != 1 || add.args[0].external) return false;
    if (add.out.size() < 2) return false;
    const Term& mul = T(add.args[0].term);
    if (mul.op != Op::Mul || !mul.red.empty() || mul.args.size() != 2) return false;
    if (!mul.args[0].external || !mul.args[1].external) return false;
    const int D = add.red[0];
    const size_t nb = add.out.size() - 2;
    const int I = add.out[nb], J = add.out[nb + 1];
    std::vector<int> left(add.out.begin(), add.out.begin() + nb), right = left;
    left.push_back(I);
    left.push_back(D);
    right.push_back(D);
    right.push_back(J);
    if (mul.args[0].dims == left && mul.args[1].dims == right) {
      r.a = operand(mul.args[0]);
      r.b = operand(mul.args[1]);
    } else if (mul.args[1].dims == left && mul.args[0].dims == right) {
      r.a = operand(mul.args[1]);
      r.b = operand(mul.args[0]);
    } else {
      return false;
    }
    r.batch_rank = nb;
    return true;
  }

  bool match_qk(int t, Recognized& r) const {
    const Term& add = T(t);
    if (add.op != Op::Add || add.red.size() != 1 || add.args.size() != 1 || add.args[0].external) return false;
    if (add.out.size() < 2) return false;
    const Term& mul = T(add.args[0].term);
    if (mul.op != Op::Mul || !mul.red.empty() || mul.args.size() != 2) return false;
    if (!mul.args[0].external || !mul.args[1].external) return false;
    const int D = add.red[0];
    const size_t nb = add.out.size() - 2;
    const int I = add.out[nb], J = add.out[nb + 1];
    std::vector<int> batch(add.out.begin(), add.out.begin() + nb);
    auto expect = [&](const Arg& a, int row) {
      std::vector<int> want = batch;
      want.push_back(row);
      want.push_back(D);
      return a.dims == want;
    };
    if (expect(mul.args[0], I) && expect(mul.args[1], J)) {
      r.a = operand(mul.args[0]);
      r.b = operand(mul.args[1]);
    } else if (expect(mul.args[1], I) && expect(mul.args[0], J)) {
      r.a = operand(mul.args[1]);
      r.b = operand(mul.args[0]);
    } else {
      return false;
    }
    r.batch_rank = nb;
    return true;
  }

  // scores: S, or S * scalar (either operand order)
  bool match_scores(int t, Recognized& r) const {
    const Term& top = T(t);
    if (top.op == Op::Mul && top.red.empty() && top.args.size() == 2) {
      for (int s = 0; s < 2; ++s) {
        const Arg &x = top.args[s], &sc = top.args[1 - s];
        if (!x.external && sc.external && sc.dims.empty() && x.dims == top.out && match_qk(x.term, r)) {
          r.has_scale = true;
          r.scale = operand(sc);
          return true;
        }
      }
      return false;
    }
    return match_qk(t, r);
  }

  // E[R.., J] = exp(X - max_J X); the max runs over a private copy of J and must
  // read the very same X.  `match_x` inspects X.
  template <class F>
  bool match_exp_shift(int t, F&& match_x) const {
    const Term& ex = T(t);
    if (ex.op != Op::Pow || !ex.red.empty() || ex.args.size() != 1 || ex.args[0].external) return false;
    const Term& sub = T(ex.args[0].term);
    if (sub.op != Op::Sub || !sub.red.empty() || sub.args.size() != 2) return false;
    if (sub.out != ex.out || sub.out.empty()) return false;
    const Arg &x = sub.args[0], &m = sub.args[1];
    if (m.external || x.dims != sub.out) return false;
    const Term& mx = T(m.term);
    if (mx.op != Op::Max || mx.red.size() != 1 || mx.args.size() != 1) return false;
    std::vector<int> rows(sub.out.begin(), sub.out.end() - 1);
    if (mx.out != rows || m.dims != rows) return false;
    std::map<int, int> ren;
    for (int r : rows) ren[r] = r;
    ren[sub.out.back()] = mx.red[0];
    if (!tb.unify_arg(x, mx.args[0], ren)) return false;
    return match_x(x);
  }

  // X - max_J X and X / sum_J X over an operand buffer X[R.., J] (the reduction runs over a private copy of J
  // and must read the very same X)
  bool match_row_reduce_then(int t, Op outer, Op inner, Operand& x_out) const {
    const Term& top = T(t);
    if (top.op != outer || !top.red.empty() || top.args.size() != 2 || top.out.empty()) return false;
    const Arg &x = top.args[0], &m = top.args[1];
    if (!x.external || m.external || x.dims != top.out) return false;
    const Term& red = T(m.term);
    if (red.op != inner || red.red.size() != 1 || red.args.size() != 1 || !red.args[0].external) return false;
    std::vector<int> rows(top.out.begin(), top.out.end() - 1);
    if (red.out != rows || m.dims != rows) return false;
    std::map<int, int> ren;
    for (int r : rows) ren[r] = r;
    ren[top.out.back()] = red.red[0];
    if (!tb.unify_arg(x, red.args[0], ren)) return false;
    x_out = operand(x);
    return true;
  }

  // P[R.., J] = E / sum_J E, the sum reading the very same E over a private copy of J
  template <class F>
  bool match_softmax(int t, F&& match_x) const {
    const Term& div = T(t);
    if (div.op != Op::Div || !div.red.empty() || div.args.size() != 2) return false;
    const Arg &e = div.args[0], &l = div.args[1];
    if (e.external || l.external || e.dims != div.out || div.out.empty()) return false;
    std::vector<int> rows(div.out.begin(), div.out.end() - 1);
    const Term& sum = T(l.term);
    if (sum.op != Op::Add || sum.red.size() != 1 || sum.args.size() != 1 || sum.args[0].external) return false;
    if (sum.out != rows || l.dims != rows) return false;
    std::map<int, int> ren;
    for (int r : rows) ren[r] = r;
    ren[div.out.back()] = sum.red[0];
    if (!tb.unify_arg(e, sum.args[0], ren)) return false;
    return match_exp_shift(e.term, match_x);
  }

  Recognized match_root(int root, BufferRef out) const {
    Recognized r;
    r.out = out;
    const Term& top = T(root);

    // GEMM-NT
    if (match_qk(root, r)) {
      r.kind = Recognized::GemmNT;
      return r;
    }
    r = Recognized{};
    r.out = out;
    if (match_mm(root, r)) {
      r.kind = Recognized::GemmNN;
      return r;
    }
    r = Recognized{};
    r.out = out;

    // exp of an operand buffer, elementwise
    if (top.op == Op::Pow && top.red.empty() && top.args.size() == 1 && top.args[0].external && !top.out.empty() &&
        top.args[0].dims == top.out) {
      r.kind = Recognized::RowExp;
      r.a = operand(top.args[0]);
      r.batch_rank = r.a.dims.size() - 1;
      return r;
    }

    // the two halves of the row softmax on their own
    {
      Operand x;
      const bool shift = match_row_reduce_then(root, Op::Sub, Op::Max, x);
      if (shift || match_row_reduce_then(root, Op::Div, Op::Add, x)) {
        r.kind = shift ? Recognized::RowMaxShift : Recognized::RowNormalize;
        r.a = x;
        r.batch_rank = x.dims.size() - 1;
        return r;
      }
    }

    // row softmax over an operand buffer
    {
      Operand x;
      if (match_softmax(root, [&](const Arg& a) {
            if (!a.external) return false;
            x = operand(a);
            return true;
          })) {
        r.kind = Recognized::RowSoftmax;
        r.a = x;
        r.batch_rank = x.dims.size() - 1;
        return r;
      }
    }

    // attention: out[B.., I, E] = sum_J P[B.., I, J] * v[B.., J, E]
    if (top.op == Op::Add && top.red.size() == 1 && top.args.size() == 1 && !top.args[0].external && top.out.size() >= 2) {
      const Term& mul = T(top.args[0].term);
      if (mul.op == Op::Mul && mul.red.empty() && mul.args.size() == 2) {
        for (int s = 0; s < 2; ++s) {
          const Arg &p = mul.args[s], &v = mul.args[1 - s];
          if (p.external || !v.external) continue;
          const size_t nb = top.out.size() - 2;
          const int I = top.out[nb], E = top.out[nb + 1], Jr = top.red[0];
          std::vector<int> batch(top.out.begin(), top.out.begin() + nb);
          std::vector<int> want_p = batch, want_v = batch;
          want_p.push_back(I);
          want_p.push_back(Jr);
          want_v.push_back(Jr);
          want_v.push_back(E);
          if (p.dims != want_p || v.dims != want_v) continue;
          Recognized cand;
          cand.out = out;
          if (!match_softmax(p.term, [&](const Arg& a) { return !a.external && match_scores(a.term, cand); })) continue;
          if (cand.batch_rank != nb) continue;
          // q rows must be the output rows, k rows the reduced axis
          if (cand.a.dims[nb] != I || cand.b.dims[nb] != Jr) continue;
          for (size_t d = 0; d < nb; ++d)
            if (cand.a.dims[d] != batch[d] || cand.b.dims[d] != batch[d]) goto next;
          cand.kind = Recognized::Attention;
          cand.c = operand(v);
          return cand;
        next:;
        }
      }
    }
    return r;
  }
};

}  // namespace

std::string Recognized::describe() const {
  std::string tiles;
  if (tile_i || tile_j) tiles = "; schedule tile " + std::to_string(tile_i) + " x " + std::to_string(tile_j);
  switch (kind) {
    case Attention: return (has_scale ? "hand-written FlashAttention kernel (scaled scores)" : "hand-written FlashAttention kernel") + tiles;
    case GemmNT: return "hand-written MFMA GEMM (transposed right operand)" + tiles;
    case GemmNN: return "hand-written MFMA GEMM (row-major right operand: read in place when bf16 with k % 64 == 0 and n % 8 == 0, transposed on the device first otherwise)" + tiles;
    case RowSoftmax: return "hand-written row-softmax kernel";
    case RowMaxShift: return "hand-written row kernel (x - row max)";
    case RowNormalize: return "hand-written row kernel (x / row sum)";
    case RowExp: return "hand-written row kernel (exp x)";
    default: return "generated HIP kernel";
  }
}

std::vector<Recognized> recognize_kernels(const Lowered& low) {
  const StageProgram& sp = low.stages;
  // kernel-program buffer -> exec-plan reference (same rule as the exec-plan lowering)
  std::vector<BufferRef> refs(low.kernels.buffers.size());
  size_t ni = 0, nm = 0;
  for (size_t i = 0; i < low.kernels.buffers.size(); ++i) {
    if (low.kernels.buffers[i].kind == BufferKind::Input) refs[i] = {BufferRef::Input, ni++};
    else if (low.kernels.buffers[i].kind == BufferKind::Intermediate) refs[i] = {BufferRef::Intermediate, nm++};
  }
  for (size_t o = 0; o < low.kernels.outputs.size(); ++o) refs[low.kernels.outputs[o]] = {BufferRef::Output, o};

  std::vector<Recognized> out;
  for (size_t stage = 0; stage < sp.graph.nodes.size(); ++stage) {
    bool fused = false;
    for (const auto& node : sp.graph.nodes)
      for (size_t i = 0; i < node.inputs.size(); ++i)
        fused |= node.inner.inputs[i].site && node.inputs[i] == Source::node(stage, 0);
    if (fused) continue;
    TreeBuilder tb{sp};
    const int root = tb.build(stage, {});
    Matcher m{tb, refs};
    Recognized rec = m.match_root(root, refs[sp.graph.inputs + stage]);
    if (rec.kind == Recognized::Attention || rec.kind == Recognized::GemmNT || rec.kind == Recognized::GemmNN) {
      // the schedule's tile sizes, read off the root stage: its output is [B.., I, E] (attention, J reduced)
      // or [B.., I, J] (GEMM)
      const Stage& st = sp.graph.nodes[stage].inner;
      auto tile_of = [&](size_t index) -> size_t {
        for (const SAxis& a : st.axes)
          if (!a.pruned && a.index == index && a.kind.kind == ExtentKind::Base) {
            size_t t = 1;
            for (size_t f : a.kind.factors) t *= f;
            return a.kind.factors.empty() ? 0 : t;
          }
        return 0;
      };
      const auto& shape = st.output.shape;
      if (shape.size() >= 2) {
        rec.tile_i = tile_of(shape[shape.size() - 2]);
        if (rec.kind != Recognized::Attention) rec.tile_j = tile_of(shape.back());
        else
          for (const SAxis& a : st.axes)
            if (std::find(shape.begin(), shape.end(), a.index) == shape.end()) rec.tile_j = tile_of(a.index);
      }
    }
    out.push_back(rec);
  }
  return out;
}

}  // namespace ihipc
