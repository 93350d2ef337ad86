// StageProgram -> KernelProgram.
//
// Every stage that no consumer computes in place becomes the root of a kernel.
// Emitting a stage allocates loops for its live axes, recursively emits the
// producers that are staged under it and splices their blocks at the depth of
// the compute site (fusion); blocks whose site lies on a loop supplied by an
// outer consumer are hoisted until a stage owns that loop.  Reductions get an
// Init at their init site with zero-checks on exterior reduction loops; loops
// whose index has no deeper live level carry a tail guard.  A reduction whose
// reduced axis is pruned is an online reduction: it snapshots its running value
// and emits a correction (exp-shift for max, divisor for sum) that travels
// down the dataflow until an additive accumulator applies it as Scale actions.
// Follows compiler/src/lower/stage_to_kernel_program.rs:19-1960.
#include <algorithm>
#include <map>
#include <set>
#include <tuple>

#include "ir.h"

namespace ic {
namespace {

using Act = Action<size_t>;
using Blk = Block<size_t>;
using Acc = Access<size_t>;

struct LoopInfo {
  size_t id = 0;
  size_t index = 0;
  ExtentKind kind;
};
using AxisMap = std::map<size_t, LoopInfo>;
using LocalLoops = std::vector<std::pair<size_t, LoopInfo>>;

struct HoistSite {
  bool before = false;  // before / after the consumer axis
  size_t axis = 0;
};
struct Placement {
  bool local = true;
  size_t depth = 0;
  HoistSite site;
};
struct HoistedBlock {
  HoistSite site;
  Blk block;
};
enum class CorrKind { Divisor = 0, ExpShift = 1 };
enum class CorrState { Pending, Shifted, Ready };
struct Correction {
  size_t old_buffer = 0, new_buffer = 0;
  std::vector<size_t> shape;
  CorrKind kind = CorrKind::Divisor;
  CorrState state = CorrState::Pending;
  std::vector<size_t> update_loops;
};
struct HoistedCorrections {
  HoistSite site;
  std::vector<Correction> corrections;
};
struct Emitted {
  Blk block;
  std::vector<HoistedBlock> hoisted;
  std::vector<HoistedCorrections> hoisted_corrections;
  std::vector<Correction> corrections;
};
struct EmittedKey {
  size_t stage_index;
  Stage stage;
  std::vector<Source> inputs;
  std::vector<HoistedBlock> hoisted;
  std::vector<HoistedCorrections> hoisted_corrections;
  std::vector<Correction> corrections;
};

std::vector<size_t> reconstruction_factors(const std::vector<LoopInfo>& infos) {
  std::vector<size_t> factors;
  bool found = false;
  for (const auto& info : infos)
    if (info.kind.kind == ExtentKind::Base) {
      factors = info.kind.factors;
      found = true;
      break;
    }
  if (!found)
    for (const auto& info : infos)
      if (info.kind.kind == ExtentKind::Split) factors.push_back(info.kind.factor);
  const size_t expected = infos.empty() ? 0 : infos.size() - 1;
  if (factors.size() > expected) factors.erase(factors.begin(), factors.end() - expected);
  return factors;
}

std::vector<SAxisRef> stage_axis_refs_for_index(const Stage& st, size_t index) {
  std::vector<std::pair<std::pair<size_t, size_t>, SAxisRef>> refs;
  for (size_t a = 0; a < st.axes.size(); ++a)
    if (st.axes[a].index == index)
      refs.push_back({st.axes[a].kind.order(), st.axes[a].pruned ? st.axes[a].by : SAxisRef{false, a}});
  if (refs.empty()) lower_error("stage has no axes for correction index " + std::to_string(index));
  std::stable_sort(refs.begin(), refs.end(), [](const auto& x, const auto& y) { return x.first < y.first; });
  std::vector<SAxisRef> out;
  for (const auto& r : refs) out.push_back(r.second);
  return out;
}

Layout semantic_shape_layout(const std::vector<size_t>& shape, const Stage& st) {
  Layout out;
  for (size_t index : shape) {
    LayoutDim d;
    d.semantic = true;
    d.index = index;
    d.axes = stage_axis_refs_for_index(st, index);
    out.push_back(d);
  }
  return out;
}

bool requires_online_reduction(const Stage& st) {
  if (!st.output.site) return false;
  std::set<size_t> out(st.output.shape.begin(), st.output.shape.end());
  for (const SAxis& a : st.axes)
    if (a.pruned && !out.count(a.index)) return true;
  return false;
}

void collect_uses(const Blk& block, std::set<size_t>& accessed, std::set<size_t>& written);
void collect_scalar_uses(const ScalarExpr<size_t>& e, std::set<size_t>& accessed) {
  if (e.kind == ScalarExpr<size_t>::Acc) accessed.insert(e.access.buffer);
  else
    for (const auto& a : e.args) collect_scalar_uses(a, accessed);
}
void collect_uses(const Blk& block, std::set<size_t>& accessed, std::set<size_t>& written) {
  for (const Act& a : block) {
    switch (a.kind) {
      case Act::Loop:
        accessed.insert(a.extent.source.buffer);
        collect_uses(a.body, accessed, written);
        break;
      case Act::Init: written.insert(a.write.buffer); break;
      case Act::Compute:
        written.insert(a.write.buffer);
        for (const Acc& r : a.reads) accessed.insert(r.buffer);
        break;
      case Act::Snapshot:
        written.insert(a.write.buffer);
        accessed.insert(a.reads[0].buffer);
        break;
      case Act::Scale:
        written.insert(a.write.buffer);
        collect_scalar_uses(a.factor, accessed);
        break;
    }
  }
}

std::vector<Correction> dedup(std::vector<Correction> in) {
  std::vector<Correction> out;
  for (auto& c : in) {
    bool dup = false;
    for (const auto& e : out) dup |= e.kind == c.kind && e.old_buffer == c.old_buffer && e.new_buffer == c.new_buffer;
    if (!dup) out.push_back(std::move(c));
  }
  return out;
}

struct Builder {
  const StageProgram& program;
  std::vector<Buffer> buffers;
  std::vector<size_t> input_buffers, stage_buffers;
  std::vector<std::optional<Source>> buffer_sources;
  std::vector<GNode<Kernel<size_t>>> kernel_nodes;

  explicit Builder(const StageProgram& p) : program(p) {
    for (size_t i = 0; i < p.input_shapes.size(); ++i) {
      const size_t id = buffers.size();
      input_buffers.push_back(id);
      buffer_sources.push_back(Source::input(i));
      Buffer b;
      b.kind = BufferKind::Input;
      // input_buffers is complete up to `i` here, and an input's dims only name itself
      for (const ShapeDim& d : p.input_shapes[i]) b.shape.push_back({d.input == i ? id : input_buffers.at(d.input), d.dim});
      for (size_t d = 0; d < p.input_shapes[i].size(); ++d) b.layout.push_back({{id, d}, ExtentKind::semantic()});
      buffers.push_back(std::move(b));
    }
    std::set<size_t> output_stages;
    for (Source s : p.graph.outputs)
      if (!s.is_input && s.output == 0) output_stages.insert(s.id);
    for (size_t n = 0; n < p.graph.nodes.size(); ++n) {
      const size_t id = buffers.size();
      const Stage& st = p.graph.nodes[n].inner;
      stage_buffers.push_back(id);
      buffer_sources.push_back(std::nullopt);
      Buffer b;
      b.kind = output_stages.count(n) ? BufferKind::Output : BufferKind::Intermediate;
      for (const ShapeDim& d : p.node_shapes[n]) b.shape.push_back({input_buffers.at(d.input), d.dim});
      for (const LayoutDim& d : st.output.layout) {
        auto output_dim = [&](size_t index) {
          auto it = std::find(st.output.shape.begin(), st.output.shape.end(), index);
          if (it == st.output.shape.end())
            lower_error("stage " + std::to_string(n) + " output layout index " + std::to_string(index) +
                        " is not present in output shape");
          return DimRef<size_t>{id, size_t(it - st.output.shape.begin())};
        };
        if (d.semantic) {
          b.layout.push_back({output_dim(d.index), ExtentKind::semantic()});
        } else {
          if (d.phys.consumer)
            lower_error("stage " + std::to_string(n) + " output layout consumer axis " + std::to_string(d.phys.axis) +
                        " cannot define buffer layout");
          const SAxis& ax = st.axes.at(d.phys.axis);
          if (ax.pruned) lower_error("stage " + std::to_string(n) + " output layout axis " + std::to_string(d.phys.axis) + " is pruned");
          b.layout.push_back({output_dim(ax.index), ax.kind});
        }
      }
      buffers.push_back(std::move(b));
    }
  }

  size_t source_buffer(Source s) const {
    if (s.is_input) {
      if (s.id >= input_buffers.size()) lower_error("source references nonexistent input " + std::to_string(s.id));
      return input_buffers[s.id];
    }
    if (s.output != 0) lower_error("source references output " + std::to_string(s.output));
    if (s.id >= stage_buffers.size()) lower_error("source references nonexistent stage " + std::to_string(s.id));
    return stage_buffers[s.id];
  }

  size_t add_intermediate_like(size_t source) {
    Buffer b = buffers.at(source);
    b.kind = BufferKind::Intermediate;
    buffer_sources.push_back(std::nullopt);
    buffers.push_back(std::move(b));
    return buffers.size() - 1;
  }

  bool fused_only(size_t stage_index) const {
    for (const auto& node : program.graph.nodes)
      for (size_t i = 0; i < node.inputs.size(); ++i)
        if (node.inner.inputs[i].site && node.inputs[i] == Source::node(stage_index, 0)) return true;
    return false;
  }
};

struct KernelBuilder {
  Builder& b;
  size_t root;
  size_t next_loop = 0;
  std::vector<size_t> reads, writes, accessed;
  std::map<size_t, size_t> stage_aliases;
  std::vector<EmittedKey> emitted_stages;
  std::set<std::tuple<size_t, size_t, size_t, size_t>> applied_corrections;

  KernelBuilder(Builder& builder, size_t root_stage) : b(builder), root(root_stage) {}

  size_t alloc_loop() { return next_loop++; }
  void record_access(size_t buffer) {
    if (std::find(accessed.begin(), accessed.end(), buffer) == accessed.end()) accessed.push_back(buffer);
  }
  void record_write(size_t buffer) {
    if (std::find(writes.begin(), writes.end(), buffer) == writes.end()) writes.push_back(buffer);
    record_access(buffer);
  }

  size_t canonical_stage(size_t index) const {
    for (;;) {
      auto it = stage_aliases.find(index);
      if (it == stage_aliases.end() || it->second == index) return index;
      index = it->second;
    }
  }
  size_t canonical_buffer(size_t buffer) const {
    auto it = std::find(b.stage_buffers.begin(), b.stage_buffers.end(), buffer);
    if (it == b.stage_buffers.end()) return buffer;
    return b.stage_buffers[canonical_stage(size_t(it - b.stage_buffers.begin()))];
  }
  size_t source_buffer(Source s) const { return b.source_buffer(s.is_input ? s : Source::node(canonical_stage(s.id), s.output)); }
  std::vector<Source> canonical_inputs(const std::vector<Source>& inputs) const {
    std::vector<Source> out;
    for (Source s : inputs) out.push_back(s.is_input ? s : Source::node(canonical_stage(s.id), s.output));
    return out;
  }

  static LoopInfo resolve(const AxisMap& axes, const AxisMap& parent, SAxisRef ref) {
    const AxisMap& m = ref.consumer ? parent : axes;
    auto it = m.find(ref.axis);
    if (it == m.end())
      lower_error((ref.consumer ? "consumer axis " : "axis ") + std::to_string(ref.axis) + " is not available");
    return it->second;
  }
  static bool available(const AxisMap& axes, const AxisMap& parent, SAxisRef ref) {
    const AxisMap& m = ref.consumer ? parent : axes;
    return m.count(ref.axis) != 0;
  }

  Iter lower_iter(const LayoutDim& d, const AxisMap& axes, const AxisMap& parent) const {
    Iter it;
    if (!d.semantic) {
      it.raw = true;
      it.loop = resolve(axes, parent, d.phys).id;
      return it;
    }
    std::vector<LoopInfo> infos;
    for (SAxisRef r : d.axes) infos.push_back(resolve(axes, parent, r));
    it.raw = false;
    for (const auto& info : infos) it.loops.push_back(info.id);
    it.factors = reconstruction_factors(infos);
    return it;
  }

  Acc lower_access(size_t buffer, const Layout& layout, const AxisMap& axes, const AxisMap& parent) {
    record_access(buffer);
    Acc a;
    a.buffer = buffer;
    for (const LayoutDim& d : layout) a.index.push_back(lower_iter(d, axes, parent));
    return a;
  }

  // ------------------------------------------------------------ placements
  Placement root_placement(const Stage& st) const {
    for (const SAxis& a : st.axes) {
      if (!a.pruned) return {true, 0, {}};
      if (a.by.consumer) return {false, 0, {true, a.by.axis}};
    }
    return {true, 0, {}};
  }
  Placement axis_placement(const Stage& st, const LocalLoops& local, size_t axis, bool before) const {
    if (axis >= st.axes.size()) lower_error("site references nonexistent axis " + std::to_string(axis));
    const SAxis& a = st.axes[axis];
    if (!a.pruned) {
      for (size_t p = 0; p < local.size(); ++p)
        if (local[p].first == axis) return {true, before ? p : p + 1, {}};
      lower_error("site references nonlocal axis " + std::to_string(axis));
    }
    if (a.by.consumer) return {false, 0, {before, a.by.axis}};
    return axis_placement(st, local, a.by.axis, before);
  }
  Placement site_placement(const Stage& st, const LocalLoops& local, SSite site) const {
    return site.root ? root_placement(st) : axis_placement(st, local, site.axis, false);
  }
  Placement hoist_placement(const Stage& st, const LocalLoops& local, HoistSite site) const {
    return axis_placement(st, local, site.axis, site.before);
  }

  size_t layout_depth(const Layout& layout, const LocalLoops& local) const {
    std::map<size_t, size_t> pos;
    for (size_t p = 0; p < local.size(); ++p) pos[local[p].first] = p;
    size_t depth = 0;
    auto one = [&](SAxisRef r) {
      if (r.consumer) return;
      auto it = pos.find(r.axis);
      if (it == pos.end()) lower_error("axis " + std::to_string(r.axis) + " is not local");
      depth = std::max(depth, it->second + 1);
    };
    for (const LayoutDim& d : layout) {
      if (d.semantic)
        for (SAxisRef r : d.axes) one(r);
      else
        one(d.phys);
    }
    return depth;
  }

  // ------------------------------------------------------------ loops
  DimRef<size_t> semantic_dim_for_axis(size_t stage_index, const Stage& st, size_t index) const {
    // the first operand that mentions the index names the loop bound
    for (size_t i = 0; i < st.inputs.size(); ++i) {
      auto it = std::find(st.inputs[i].shape.begin(), st.inputs[i].shape.end(), index);
      if (it != st.inputs[i].shape.end())
        return {source_buffer(b.program.graph.nodes[stage_index].inputs[i]), size_t(it - st.inputs[i].shape.begin())};
    }
    auto it = std::find(st.output.shape.begin(), st.output.shape.end(), index);
    if (it != st.output.shape.end()) return {b.stage_buffers[stage_index], size_t(it - st.output.shape.begin())};
    lower_error("index " + std::to_string(index) + " has no semantic extent source");
  }
  Extent<size_t> loop_extent(size_t stage_index, const Stage& st, size_t axis, const LoopInfo& info) {
    Extent<size_t> e;
    e.source = semantic_dim_for_axis(stage_index, st, info.index);
    record_access(e.source.buffer);
    if (st.axes[axis].pruned) lower_error("axis " + std::to_string(axis) + " is not live");
    e.kind = st.axes[axis].kind;
    return e;
  }
  // a loop needs the `tile*F + inner < dim` guard when no deeper live level of its index exists
  static bool tail_guard(const Stage& st, const LoopInfo& info) {
    if (info.kind.kind == ExtentKind::Semantic) return false;
    const size_t level = info.kind.split_level();
    for (const SAxis& a : st.axes)
      if (!a.pruned && a.index == info.index && a.kind.split_level() > level) return false;
    return true;
  }

  Blk build_loop_block(size_t stage_index, const Stage& st, const LocalLoops& local, const std::vector<Blk>& actions,
                       const Act& compute, size_t depth) {
    Blk block = actions[depth];
    if (depth == local.size()) {
      block.push_back(compute);
      return block;
    }
    Act loop;
    loop.kind = Act::Loop;
    loop.id = local[depth].second.id;
    loop.extent = loop_extent(stage_index, st, local[depth].first, local[depth].second);
    loop.guard = tail_guard(st, local[depth].second);
    loop.body = build_loop_block(stage_index, st, local, actions, compute, depth + 1);
    block.push_back(std::move(loop));
    return block;
  }

  // ------------------------------------------------------------ init
  void validate_init_depth(const Stage& st, const LocalLoops& local, size_t depth) const {
    std::set<size_t> out(st.output.shape.begin(), st.output.shape.end());
    for (size_t p = 0; p < local.size(); ++p)
      if (out.count(local[p].second.index) && p >= depth)
        lower_error("init site is outside output loop " + std::to_string(local[p].second.index));
  }
  std::vector<size_t> init_zero_checks(const Stage& st, const LocalLoops& local, const AxisMap& axes, size_t depth) const {
    std::set<size_t> out(st.output.shape.begin(), st.output.shape.end());
    std::map<size_t, size_t> pos;
    for (size_t p = 0; p < local.size(); ++p) pos[local[p].first] = p;
    std::vector<size_t> checks;
    for (size_t a = 0; a < st.axes.size(); ++a) {
      auto it = axes.find(a);
      if (it == axes.end()) lower_error("axis " + std::to_string(a) + " is not available");
      if (out.count(st.axes[a].index)) continue;
      const bool exterior = st.axes[a].pruned ? true : (pos.count(a) && pos[a] < depth);
      if (exterior && std::find(checks.begin(), checks.end(), it->second.id) == checks.end()) checks.push_back(it->second.id);
    }
    return checks;
  }

  // ------------------------------------------------------------ online corrections
  std::optional<Correction> online_correction(size_t stage_index, const Stage& st, size_t output_buffer, const AxisMap& axes) {
    if (stage_index == root || !requires_online_reduction(st)) return std::nullopt;
    CorrKind kind;
    if (st.op == Op::Add) kind = CorrKind::Divisor;
    else if (st.op == Op::Max) kind = CorrKind::ExpShift;
    else
      lower_error("stage " + std::to_string(stage_index) +
                  " requires online reduction lowering: fused reduction axis is consumed before completion");
    Correction c;
    c.old_buffer = b.add_intermediate_like(output_buffer);
    c.new_buffer = output_buffer;
    c.shape = st.output.shape;
    c.kind = kind;
    std::set<size_t> out(st.output.shape.begin(), st.output.shape.end());
    for (size_t a = 0; a < st.axes.size(); ++a)
      if (st.axes[a].pruned && !out.count(st.axes[a].index)) {
        auto it = axes.find(a);
        if (it != axes.end()) c.update_loops.push_back(it->second.id);
      }
    return c;
  }

  static bool can_apply(const Stage& st, const std::vector<Correction>& corrections) {
    if (st.op != Op::Add || !st.output.site) return false;
    std::set<size_t> out(st.output.shape.begin(), st.output.shape.end());
    for (const Correction& c : corrections) {
      if (c.state != CorrState::Ready) return false;
      for (size_t index : c.shape)
        if (!out.count(index)) return false;
    }
    return true;
  }

  static Correction propagate_one(const Stage& st, size_t input_index, Correction c) {
    if (c.state == CorrState::Ready) return c;
    if (c.kind == CorrKind::Divisor) {
      if (c.state == CorrState::Pending) {
        if (st.op == Op::Div && input_index > 0) {
          c.state = CorrState::Ready;
          return c;
        }
        lower_error("online reduction correction requires a division use before accumulation");
      }
      lower_error("division correction reached invalid shifted state");
    }
    if (c.state == CorrState::Pending) {
      if (st.op == Op::Sub && input_index > 0) {
        c.state = CorrState::Shifted;
        return c;
      }
      lower_error("online max correction requires a subtraction use before exponentiation");
    }
    if (st.op == Op::Pow) {
      c.state = CorrState::Ready;
      return c;
    }
    lower_error("online max correction requires exponentiation before accumulation");
  }
  static std::vector<Correction> propagate(const Stage& st, size_t input_index, std::vector<Correction> in) {
    if (in.empty()) return in;
    if (st.output.site) lower_error("online reduction correction reached unsupported accumulator");
    std::vector<Correction> out;
    for (auto& c : in) out.push_back(propagate_one(st, input_index, std::move(c)));
    return out;
  }

  Act snapshot_action(const Correction& c, const Stage& st, const AxisMap& axes, const AxisMap& parent) {
    record_write(c.old_buffer);
    const Layout layout = semantic_shape_layout(c.shape, st);
    Act a;
    a.kind = Act::Snapshot;
    a.write = lower_access(c.old_buffer, layout, axes, parent);
    a.reads.push_back(lower_access(c.new_buffer, layout, axes, parent));
    return a;
  }

  Act scale_action(const Correction& c, const Stage& st, const Acc& write, const AxisMap& axes, const AxisMap& parent) {
    const Layout layout = semantic_shape_layout(c.shape, st);
    ScalarExpr<size_t> old_e, new_e;
    old_e.access = lower_access(c.old_buffer, layout, axes, parent);
    new_e.access = lower_access(c.new_buffer, layout, axes, parent);
    Act a;
    a.kind = Act::Scale;
    a.write = write;
    if (c.kind == CorrKind::Divisor) {  // old / new
      a.factor.kind = ScalarExpr<size_t>::Binary;
      a.factor.op = Op::Div;
      a.factor.args = {old_e, new_e};
    } else {  // e ^ (old - new)
      ScalarExpr<size_t> diff;
      diff.kind = ScalarExpr<size_t>::Binary;
      diff.op = Op::Sub;
      diff.args = {old_e, new_e};
      a.factor.kind = ScalarExpr<size_t>::Unary;
      a.factor.op = Op::Pow;
      a.factor.args = {diff};
    }
    return a;
  }

  size_t scale_depth(const Stage& st, const LocalLoops& local, const std::vector<Correction>& corrections) const {
    size_t depth = 0;
    for (const Correction& c : corrections) {
      depth = std::max(depth, layout_depth(semantic_shape_layout(c.shape, st), local));
      for (size_t loop : c.update_loops)
        for (size_t p = 0; p < local.size(); ++p)
          if (local[p].second.id == loop) depth = std::max(depth, p + 1);
    }
    return depth;
  }

  Blk scale_block(const Stage& st, size_t stage_index, size_t output_buffer, AxisMap& axes,
                  const LocalLoops& scale_axes, const std::vector<const Correction*>& corrections, const AxisMap& parent,
                  size_t position) {
    if (position == scale_axes.size()) {
      const Acc write = lower_access(output_buffer, st.output.layout, axes, parent);
      Blk out;
      for (const Correction* c : corrections) out.push_back(scale_action(*c, st, write, axes, parent));
      return out;
    }
    const size_t axis = scale_axes[position].first;
    LoopInfo info = scale_axes[position].second;
    info.id = alloc_loop();
    axes[axis] = info;
    Blk body = scale_block(st, stage_index, output_buffer, axes, scale_axes, corrections, parent, position + 1);
    axes[axis] = scale_axes[position].second;
    Act loop;
    loop.kind = Act::Loop;
    loop.id = info.id;
    loop.extent = loop_extent(stage_index, st, axis, info);
    loop.guard = tail_guard(st, info);
    loop.body = std::move(body);
    return {loop};
  }

  void apply_corrections(const Stage& st, size_t stage_index, size_t output_buffer, const AxisMap& stage_axes,
                         const LocalLoops& local, std::vector<Blk>& actions, std::vector<Correction>& outgoing,
                         std::vector<Correction> incoming, const AxisMap& parent) {
    incoming = dedup(std::move(incoming));
    if (incoming.empty()) return;
    for (const Correction& c : incoming)
      if (c.state != CorrState::Ready) lower_error("online reduction correction reached accumulator before correction use");
    const size_t depth = scale_depth(st, local, incoming);
    std::vector<const Correction*> fresh;
    for (const Correction& c : incoming)
      if (applied_corrections.insert({stage_index, c.old_buffer, c.new_buffer, size_t(c.kind)}).second) fresh.push_back(&c);
    if (!fresh.empty()) {
      std::set<size_t> required;
      auto collect_local = [&](const Layout& layout) {
        for (const LayoutDim& d : layout) {
          if (d.semantic) {
            for (SAxisRef r : d.axes)
              if (!r.consumer) required.insert(r.axis);
          } else if (!d.phys.consumer) {
            required.insert(d.phys.axis);
          }
        }
      };
      collect_local(st.output.layout);
      for (const Correction* c : fresh) collect_local(semantic_shape_layout(c->shape, st));
      LocalLoops scale_axes;
      for (size_t p = 0; p < local.size(); ++p)
        if (p >= depth && required.count(local[p].first)) scale_axes.push_back(local[p]);
      AxisMap axes = stage_axes;
      Blk block = scale_block(st, stage_index, output_buffer, axes, scale_axes, fresh, parent, 0);
      actions[depth].insert(actions[depth].end(), block.begin(), block.end());
    }
    if (stage_index != root) outgoing.insert(outgoing.end(), incoming.begin(), incoming.end());
  }

  void handle_corrections(const Stage& st, size_t stage_index, size_t input_index, size_t output_buffer,
                          const AxisMap& stage_axes, const LocalLoops& local, std::vector<Blk>& actions,
                          std::vector<Correction>& outgoing, std::vector<Correction> incoming, const AxisMap& parent) {
    incoming = dedup(std::move(incoming));
    if (incoming.empty()) return;
    if (can_apply(st, incoming)) {
      apply_corrections(st, stage_index, output_buffer, stage_axes, local, actions, outgoing, std::move(incoming), parent);
    } else {
      auto moved = propagate(st, input_index, std::move(incoming));
      outgoing.insert(outgoing.end(), moved.begin(), moved.end());
    }
  }

  std::vector<Correction> emitted_corrections(size_t stage) const {
    const size_t canonical = canonical_stage(stage);
    for (const EmittedKey& k : emitted_stages)
      if (k.stage_index == canonical) return k.corrections;
    return {};
  }

  // ------------------------------------------------------------ reads
  Acc lower_read(Source source, const StageBuf& input, const Stage& st, const AxisMap& axes, const AxisMap& parent) {
    const size_t buffer = source_buffer(source);
    if (!source.is_input && source.output == 0 && input.site) {
      const Stage& producer = b.program.graph.nodes[source.id].inner;
      bool semantic_out = false;
      for (const LayoutDim& d : producer.output.layout) semantic_out |= d.semantic;
      if (semantic_out) {
        // A protected (full-extent) producer is addressed by its semantic indexes.  The reference looks the
        // producer's own index numbers up among this stage's axes (stage_to_kernel_program.rs:1279), which is only
        // right when both expressions happen to number the shared indexes alike (they do in its demo); when they do
        // not, e.g. (I & >ij~j) >> ij-j~ij with the maximum staged at the root, it addresses the buffer with the
        // wrong index and, on non-square operands, out of bounds.  Here dimension d of the producer's output is
        // this stage's index for dimension d of the operand (the positional match every edge is built on), which
        // is the same thing wherever the reference's result is defined.
        const Layout layout = semantic_shape_layout(input.shape, st);
        bool ok = true;
        for (const LayoutDim& d : layout)
          for (SAxisRef r : d.axes) ok &= available(axes, parent, r);
        if (ok) return lower_access(buffer, layout, axes, parent);
      }
    }
    return lower_access(buffer, input.layout, axes, parent);
  }

  // ------------------------------------------------------------ stage emission
  Emitted emit_stage(size_t stage_index, const AxisMap& parent_axes) {
    const auto& gnode = b.program.graph.nodes[stage_index];
    const Stage& st = gnode.inner;
    const size_t output_buffer = b.stage_buffers[stage_index];

    LocalLoops local;
    AxisMap stage_axes;
    for (size_t a = 0; a < st.axes.size(); ++a) {
      if (!st.axes[a].pruned) {
        LoopInfo info{alloc_loop(), st.axes[a].index, st.axes[a].kind};
        local.push_back({a, info});
        stage_axes[a] = info;
      } else {
        auto it = parent_axes.find(st.axes[a].by.axis);
        if (it == parent_axes.end()) lower_error("consumer axis " + std::to_string(st.axes[a].by.axis) + " is not available");
        stage_axes[a] = it->second;
      }
    }

    if (stage_index != root) {
      const auto key_inputs = canonical_inputs(gnode.inputs);
      for (const EmittedKey& existing : emitted_stages) {
        if (!(existing.stage == st) || existing.inputs != key_inputs) continue;
        bool any_pruned = false;
        for (const SAxis& a : st.axes) any_pruned |= a.pruned;
        if (existing.stage_index != stage_index && any_pruned && !st.output.layout.empty())
          lower_error("shared non-root compute-at placement for stage " + std::to_string(stage_index) + " is not supported");
        stage_aliases[stage_index] = existing.stage_index;
        Emitted e;
        for (const HoistedBlock& h : existing.hoisted) e.hoisted.push_back({h.site, {}});
        e.hoisted_corrections = existing.hoisted_corrections;
        e.corrections = existing.corrections;
        return e;
      }
    }

    std::vector<Blk> actions(local.size() + 1);
    std::vector<HoistedBlock> hoisted;
    const std::optional<Correction> online = online_correction(stage_index, st, output_buffer, stage_axes);

    if (st.output.site) {
      const Placement pl = site_placement(st, local, *st.output.site);
      Act init;
      init.kind = Act::Init;
      init.op = st.op;
      if (pl.local) {
        validate_init_depth(st, local, pl.depth);
        init.write = lower_access(output_buffer, st.output.layout, stage_axes, parent_axes);
        init.zero_checks = init_zero_checks(st, local, stage_axes, pl.depth);
        actions[pl.depth].push_back(std::move(init));
      } else {
        init.write = lower_access(output_buffer, st.output.layout, stage_axes, parent_axes);
        hoisted.push_back({pl.site, {init}});
      }
    }
    if (online) {
      const size_t depth = layout_depth(semantic_shape_layout(online->shape, st), local);
      actions[depth].push_back(snapshot_action(*online, st, stage_axes, parent_axes));
    }

    std::vector<HoistedCorrections> hoisted_corrections;
    std::vector<Correction> corrections;
    for (size_t i = 0; i < st.inputs.size(); ++i) {
      const StageBuf& input = st.inputs[i];
      const Source source = gnode.inputs[i];
      if (input.site) {
        if (source.is_input || source.output != 0)
          lower_error("stage " + std::to_string(stage_index) + " input " + std::to_string(i) +
                      " has compute site without stage producer");
        Emitted fused = emit_stage(source.id, stage_axes);
        // blocks hoisted out of the producer land here if this stage owns the loop, else travel on
        for (HoistedBlock& h : fused.hoisted) {
          const Placement pl = hoist_placement(st, local, h.site);
          if (pl.local) actions[pl.depth].insert(actions[pl.depth].end(), h.block.begin(), h.block.end());
          else hoisted.push_back({pl.site, std::move(h.block)});
        }
        for (HoistedCorrections& h : fused.hoisted_corrections) {
          const Placement pl = hoist_placement(st, local, h.site);
          if (can_apply(st, h.corrections)) {
            apply_corrections(st, stage_index, output_buffer, stage_axes, local, actions, corrections,
                              std::move(h.corrections), parent_axes);
          } else if (pl.local) {
            if (!propagate(st, 0, std::move(h.corrections)).empty())
              lower_error("online correction was hoisted to a non-accumulator stage");
          } else {
            hoisted_corrections.push_back({pl.site, propagate(st, 0, std::move(h.corrections))});
          }
        }
        const Placement pl = site_placement(st, local, *input.site);
        if (pl.local) {
          actions[pl.depth].insert(actions[pl.depth].end(), fused.block.begin(), fused.block.end());
          handle_corrections(st, stage_index, i, output_buffer, stage_axes, local, actions, corrections,
                             std::move(fused.corrections), parent_axes);
        } else if (can_apply(st, fused.corrections)) {
          handle_corrections(st, stage_index, i, output_buffer, stage_axes, local, actions, corrections,
                             std::move(fused.corrections), parent_axes);
          hoisted.push_back({pl.site, std::move(fused.block)});
        } else {
          hoisted.push_back({pl.site, std::move(fused.block)});
          hoisted_corrections.push_back({pl.site, propagate(st, i, std::move(fused.corrections))});
        }
      } else if (!source.is_input && source.output == 0) {
        handle_corrections(st, stage_index, i, output_buffer, stage_axes, local, actions, corrections,
                           emitted_corrections(source.id), parent_axes);
      }
    }
    if (online) corrections.push_back(*online);

    if (stage_index != root) {
      EmittedKey key;
      key.stage_index = stage_index;
      key.stage = st;
      key.inputs = canonical_inputs(gnode.inputs);
      key.hoisted = hoisted;
      key.hoisted_corrections = hoisted_corrections;
      key.corrections = corrections;
      emitted_stages.push_back(std::move(key));
    }

    record_write(output_buffer);

    Act compute;
    compute.kind = Act::Compute;
    compute.op = st.op;
    for (size_t i = 0; i < st.inputs.size(); ++i)
      compute.reads.push_back(lower_read(gnode.inputs[i], st.inputs[i], st, stage_axes, parent_axes));
    compute.write = lower_access(output_buffer, st.output.layout, stage_axes, parent_axes);

    Emitted out;
    out.block = build_loop_block(stage_index, st, local, actions, compute, 0);
    out.hoisted = std::move(hoisted);
    out.hoisted_corrections = std::move(hoisted_corrections);
    out.corrections = std::move(corrections);
    return out;
  }

  Blk emit_root() {
    Emitted e = emit_stage(root, {});
    if (!e.hoisted.empty())
      lower_error("stage " + std::to_string(root) + " left fused actions hoisted to unavailable consumer axis " +
                  std::to_string(e.hoisted[0].site.axis) + (e.hoisted[0].site.before ? " before site" : " after site"));
    if (!e.corrections.empty()) lower_error("online reduction correction reached root without an accumulator");
    return std::move(e.block);
  }

  // parameter lists: writes in first-write order, reads = recorded reads then
  // every accessed-but-never-written buffer, all restricted to what the body uses
  void params(const Blk& body, std::vector<size_t>& out_reads, std::vector<size_t>& out_writes) {
    std::set<size_t> acc_raw, wr_raw, acc, wr;
    collect_uses(body, acc_raw, wr_raw);
    for (size_t x : acc_raw) acc.insert(canonical_buffer(x));
    for (size_t x : wr_raw) wr.insert(canonical_buffer(x));
    out_writes.clear();
    for (size_t x : writes) {
      const size_t c = canonical_buffer(x);
      if (wr.count(c)) out_writes.push_back(c);
    }
    out_reads.clear();
    for (size_t x : reads) {
      const size_t c = canonical_buffer(x);
      if (acc.count(c)) out_reads.push_back(c);
    }
    for (size_t x : accessed) {
      const size_t c = canonical_buffer(x);
      if (!acc.count(c)) continue;
      if (!wr.count(c) && std::find(out_reads.begin(), out_reads.end(), c) == out_reads.end()) out_reads.push_back(c);
    }
  }
};

// structural checks on the result (check/kernel_program.rs:74-283)
void validate_block(const Kernel<size_t>& k, const Blk& block, std::set<size_t>& all_loops, std::set<size_t> scope) {
  auto check_iters = [&](const Acc& a, const char* what) {
    for (const Iter& it : a.index) {
      std::vector<size_t> ids = it.raw ? std::vector<size_t>{it.loop} : it.loops;
      if (!it.raw && it.factors.size() + 1 != ids.size())
        lower_error(std::string(what) + " reconstructed iterator has " + std::to_string(ids.size()) + " loops and " +
                    std::to_string(it.factors.size()) + " factors");
      for (size_t id : ids)
        if (!scope.count(id)) lower_error(std::string(what) + " references loop " + std::to_string(id) + " outside scope");
    }
  };
  auto check_write = [&](const Acc& a, const char* what) {
    check_iters(a, what);
    if (std::find(k.writes.begin(), k.writes.end(), a.buffer) == k.writes.end())
      lower_error(std::string(what) + " writes buffer " + std::to_string(a.buffer) + " outside writeables");
  };
  auto check_read = [&](const Acc& a, const char* what) {
    if (std::find(k.reads.begin(), k.reads.end(), a.buffer) == k.reads.end() &&
        std::find(k.writes.begin(), k.writes.end(), a.buffer) == k.writes.end())
      lower_error(std::string(what) + " references buffer " + std::to_string(a.buffer) + " outside params");
    check_iters(a, what);
  };
  for (const Act& a : block) {
    switch (a.kind) {
      case Act::Loop: {
        if (!all_loops.insert(a.id).second) lower_error("loop id " + std::to_string(a.id) + " is repeated");
        auto child = scope;
        child.insert(a.id);
        validate_block(k, a.body, all_loops, child);
        break;
      }
      case Act::Init:
        check_write(a.write, "init");
        for (size_t id : a.zero_checks)
          if (!scope.count(id)) lower_error("init zero check references loop " + std::to_string(id) + " outside scope");
        break;
      case Act::Compute:
        check_write(a.write, "compute write");
        for (const Acc& r : a.reads) check_read(r, "compute read");
        break;
      case Act::Snapshot:
        check_write(a.write, "snapshot write");
        check_read(a.reads[0], "snapshot read");
        break;
      case Act::Scale: check_write(a.write, "scale write"); break;
    }
  }
}

}  // namespace

KernelProgram lower_stages_to_kernels(const StageProgram& program) {
  if (program.input_shapes.size() != program.graph.inputs)
    lower_error("stage program has " + std::to_string(program.input_shapes.size()) + " input shapes for " +
                std::to_string(program.graph.inputs) + " graph inputs");
  Builder b(program);
  KernelProgram out;
  for (Source s : program.graph.outputs) out.outputs.push_back(b.source_buffer(s));

  for (size_t stage = 0; stage < program.graph.nodes.size(); ++stage) {
    if (b.fused_only(stage)) continue;
    KernelBuilder kb(b, stage);
    Kernel<size_t> kernel;
    kernel.body = kb.emit_root();
    kb.params(kernel.body, kernel.reads, kernel.writes);
    GNode<Kernel<size_t>> node;
    for (size_t buffer : kernel.reads) {
      if (!b.buffer_sources[buffer]) lower_error("kernel read buffer " + std::to_string(buffer) + " has no graph source");
      node.inputs.push_back(*b.buffer_sources[buffer]);
    }
    const size_t kernel_id = b.kernel_nodes.size();
    for (size_t o = 0; o < kernel.writes.size(); ++o) b.buffer_sources[kernel.writes[o]] = Source::node(kernel_id, o);
    node.outputs = kernel.writes.size();
    for (size_t w : kernel.writes)
      if (std::find(kernel.reads.begin(), kernel.reads.end(), w) != kernel.reads.end())
        lower_error("buffer " + std::to_string(w) + " is both read and written");
    std::set<size_t> loops;
    validate_block(kernel, kernel.body, loops, {});
    node.inner = std::move(kernel);
    b.kernel_nodes.push_back(std::move(node));
  }
  for (size_t buffer : out.outputs) {
    if (!b.buffer_sources[buffer]) lower_error("program output buffer " + std::to_string(buffer) + " has no graph source");
    out.graph.outputs.push_back(*b.buffer_sources[buffer]);
  }
  out.graph.inputs = program.graph.inputs;
  out.graph.nodes = std::move(b.kernel_nodes);
  out.buffers = std::move(b.buffers);
  return out;
}

}  // namespace ic
