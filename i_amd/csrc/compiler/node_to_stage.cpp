// Graph<Node> -> StageProgram.
//
// Decides, per graph edge, whether a producer is materialised once (no compute
// site on the consuming operand) or duplicated under its consumer (compute
// site present); in the second case the producer axes that line up with the
// consumer loops above the site are pruned (loop fusion), and the producer's
// output keeps only its un-pruned axes (storage folding) unless a reduction's
// output index sits behind an exterior reduction loop (protected: keeps the
// full semantic extent).  Follows compiler/src/lower/node_to_stage.rs:15-862.
#include <algorithm>
#include <map>
#include <set>

#include "ir.h"

namespace ic {
namespace {

struct AxisSource {
  size_t index;
  ExtentKind kind;
};

ExtentKind extent_kind(const Node& node, AxisLevel a) {
  const auto& factors = node.splits[a.index];
  if (factors.empty()) return ExtentKind::semantic();
  if (a.level == 0) return ExtentKind::base(factors);
  return ExtentKind::split(a.level, factors[a.level - 1]);
}

std::vector<AxisSource> axis_sources(const Node& node) {
  std::vector<AxisSource> out;
  for (AxisLevel a : node.order) out.push_back({a.index, extent_kind(node, a)});
  return out;
}

std::optional<SSite> lower_site(const Node& node, const std::optional<NodeSite>& site) {
  if (!site) return std::nullopt;
  if (site->root) return SSite{true, 0};
  for (size_t i = 0; i < node.order.size(); ++i)
    if (node.order[i] == site->at) return SSite{false, i};
  lower_error("site references loop level outside the order");
}

Stage skeleton(const Node& node) {
  Stage st;
  st.op = node.op;
  for (const auto& src : axis_sources(node)) {
    SAxis a;
    a.index = src.index;
    a.kind = src.kind;
    st.axes.push_back(a);
  }
  st.output.shape = node.output;
  st.output.site = lower_site(node, node.init_site);
  for (size_t i = 0; i < node.inputs.size(); ++i) {
    StageBuf in;
    in.shape = node.inputs[i];
    in.site = lower_site(node, node.compute_sites[i]);
    st.inputs.push_back(in);
  }
  return st;
}

// axes of `index`, outermost first (stable for equal order keys)
std::vector<std::pair<size_t, ExtentKind>> axes_for_index(const Stage& st, size_t index) {
  std::vector<std::pair<size_t, ExtentKind>> out;
  for (size_t a = 0; a < st.axes.size(); ++a)
    if (st.axes[a].index == index) out.push_back({a, st.axes[a].kind});
  std::stable_sort(out.begin(), out.end(), [](const auto& x, const auto& y) { return x.second.order() < y.second.order(); });
  return out;
}

SAxisRef stage_axis_ref(const Stage& st, size_t axis) {
  if (axis >= st.axes.size()) lower_error("axis " + std::to_string(axis) + " does not exist while lowering layout");
  return st.axes[axis].pruned ? st.axes[axis].by : SAxisRef{false, axis};
}

std::vector<size_t> consumer_axis_prefix(const Stage& consumer, size_t input_index) {
  if (input_index >= consumer.inputs.size() || !consumer.inputs[input_index].site) return {};
  const SSite site = *consumer.inputs[input_index].site;
  if (site.root) return {};
  if (site.axis + 1 > consumer.axes.size())
    lower_error("consumer input " + std::to_string(input_index) + " compute site references nonexistent axis " +
                std::to_string(site.axis));
  std::vector<size_t> out;
  for (size_t a = 0; a <= site.axis; ++a) out.push_back(a);
  return out;
}

// producer axis -> consumer axis, through the edge's positional shape match;
// reduced producer axes align with an unclaimed consumer axis of the same
// index number and extent kind when exactly one exists.
std::map<size_t, size_t> edge_axis_alignment(const Stage& producer, const Stage& consumer, size_t input_index) {
  if (input_index >= consumer.inputs.size())
    lower_error("consumer input " + std::to_string(input_index) + " does not exist for pruning");
  const StageBuf& input = consumer.inputs[input_index];
  if (producer.output.shape.size() != input.shape.size())
    lower_error("producer output has " + std::to_string(producer.output.shape.size()) +
                " shape dimensions but consumer input " + std::to_string(input_index) + " has " +
                std::to_string(input.shape.size()) + " shape dimensions");
  std::map<size_t, size_t> alignment;
  std::set<size_t> aligned_consumer;
  for (size_t d = 0; d < input.shape.size(); ++d) {
    const size_t pidx = producer.output.shape[d], cidx = input.shape[d];
    const auto paxes = axes_for_index(producer, pidx);
    const auto caxes = axes_for_index(consumer, cidx);
    if (paxes.size() != caxes.size())
      lower_error("producer index " + std::to_string(pidx) + " has " + std::to_string(paxes.size()) +
                  " axes but consumer index " + std::to_string(cidx) + " has " + std::to_string(caxes.size()) + " axes");
    for (size_t i = 0; i < paxes.size(); ++i) {
      if (paxes[i].second != caxes[i].second)
        lower_error("producer extent kind " + paxes[i].second.debug_string() + " does not match consumer extent kind " +
                    caxes[i].second.debug_string());
      alignment[paxes[i].first] = caxes[i].first;
      aligned_consumer.insert(caxes[i].first);
    }
  }
  std::set<size_t> out_idx(producer.output.shape.begin(), producer.output.shape.end());
  std::vector<std::pair<size_t, SAxis>> reduced;
  for (size_t a = 0; a < producer.axes.size(); ++a)
    if (!producer.axes[a].pruned && !out_idx.count(producer.axes[a].index)) reduced.push_back({a, producer.axes[a]});
  std::stable_sort(reduced.begin(), reduced.end(),
                   [](const auto& x, const auto& y) { return x.second.kind.order() < y.second.kind.order(); });
  for (const auto& [paxis, ax] : reduced) {
    if (alignment.count(paxis)) continue;
    std::vector<size_t> candidates;
    for (const auto& [caxis, ckind] : axes_for_index(consumer, ax.index))
      if (!aligned_consumer.count(caxis) && ckind == ax.kind) candidates.push_back(caxis);
    if (candidates.size() == 1) {
      alignment[paxis] = candidates[0];
      aligned_consumer.insert(candidates[0]);
    } else if (candidates.size() > 1) {
      lower_error("producer reduced axis " + std::to_string(paxis) + " ambiguously aligns with consumer index " +
                  std::to_string(ax.index));
    }
  }
  return alignment;
}

std::string fmt_axis_ids(const std::vector<size_t>& v) {
  std::string s = "[";
  for (size_t i = 0; i < v.size(); ++i) s += (i ? ", AxisId(" : "AxisId(") + std::to_string(v[i]) + ")";
  return s + "]";
}

void prune_producer_for_consumer(Stage& producer, const Stage& consumer, size_t input_index) {
  const auto prefix = consumer_axis_prefix(consumer, input_index);
  const auto alignment = edge_axis_alignment(producer, consumer, input_index);
  std::set<size_t> prefix_set(prefix.begin(), prefix.end());
  std::set<size_t> aligned;
  for (const auto& kv : alignment) aligned.insert(kv.second);
  std::vector<size_t> expected, actual;
  for (size_t a : prefix)
    if (aligned.count(a)) expected.push_back(a);
  std::vector<std::pair<size_t, size_t>> pruned;
  for (size_t pa = 0; pa < producer.axes.size(); ++pa) {
    auto it = alignment.find(pa);
    if (it == alignment.end() || !prefix_set.count(it->second)) continue;
    actual.push_back(it->second);
    if (producer.axes[pa].pruned) lower_error("axis " + std::to_string(pa) + " is already pruned");
    if (producer.axes[pa].kind != consumer.axes[it->second].kind)
      lower_error("producer extent kind " + producer.axes[pa].kind.debug_string() +
                  " does not match consumer extent kind " + consumer.axes[it->second].kind.debug_string());
    pruned.push_back({pa, it->second});
  }
  // fused loops must appear in the same relative order on both sides
  if (actual != expected)
    lower_error("producer axes align with consumer axes " + fmt_axis_ids(actual) + ", expected " + fmt_axis_ids(expected));
  for (const auto& [pa, ca] : pruned) {
    producer.axes[pa].pruned = true;
    producer.axes[pa].by = SAxisRef{true, ca};
  }
}

// A reduction output is protected when one of its indexes has an axis that
// comes after an axis of a non-output index: the element is revisited across
// iterations of that exterior loop, so it cannot be folded away.
bool protected_output(const Stage& st) {
  if (!st.output.site) return false;
  std::set<size_t> shape(st.output.shape.begin(), st.output.shape.end());
  bool saw_exterior = false;
  for (const SAxis& a : st.axes) {
    if (shape.count(a.index)) {
      if (saw_exterior) return true;
    } else {
      saw_exterior = true;
    }
  }
  return false;
}

Layout semantic_layout(const Stage& st, const std::vector<size_t>& multi_index) {
  Layout out;
  for (size_t index : multi_index) {
    LayoutDim d;
    d.semantic = true;
    d.index = index;
    for (const auto& [axis, kind] : axes_for_index(st, index)) d.axes.push_back(stage_axis_ref(st, axis));
    out.push_back(d);
  }
  return out;
}

// One dimension per axis of each index, outermost first.  `excluded` drops the
// consumer's own loops above a compute site (input layouts); with
// `include_consumer` false, axes supplied by the consumer are dropped too: that
// is what folds a fused producer's output down to its un-pruned axes.
Layout physical_layout(const Stage& st, const std::vector<size_t>& multi_index, const std::vector<size_t>& excluded,
                       bool include_consumer) {
  Layout out;
  for (size_t index : multi_index)
    for (const auto& [axis, kind] : axes_for_index(st, index)) {
      if (std::find(excluded.begin(), excluded.end(), axis) != excluded.end()) continue;
      const SAxisRef ref = stage_axis_ref(st, axis);
      if (ref.consumer && !include_consumer) continue;
      LayoutDim d;
      d.phys = ref;
      out.push_back(d);
    }
  return out;
}

void assign_layouts(Stage& st, const Node& node, bool physical_output) {
  if (protected_output(st)) physical_output = false;
  st.output.layout = physical_output ? physical_layout(st, node.output, {}, false) : semantic_layout(st, node.output);
  for (size_t i = 0; i < st.inputs.size(); ++i) {
    if (st.inputs[i].site) st.inputs[i].layout = physical_layout(st, node.inputs[i], consumer_axis_prefix(st, i), true);
    else st.inputs[i].layout = semantic_layout(st, node.inputs[i]);
  }
}

struct Builder {
  const Graph<Node>& graph;
  std::vector<GNode<Stage>> nodes;
  std::vector<ProgramShape> shapes;
  std::vector<size_t> input_ranks;
  std::vector<std::optional<size_t>> materialized;
  struct Dup {
    size_t node;
    Stage stage;
    std::vector<Source> inputs;
    size_t stage_id;
  };
  std::vector<Dup> duplicates;

  explicit Builder(const Graph<Node>& g) : graph(g), input_ranks(g.inputs, 0), materialized(g.nodes.size()) {}

  size_t materialized_stage(size_t node) {
    if (materialized[node]) return *materialized[node];
    Stage st = skeleton(graph.nodes[node].inner);
    assign_layouts(st, graph.nodes[node].inner, false);
    const size_t id = instantiate(node, std::move(st), false);
    materialized[node] = id;
    return id;
  }

  size_t duplicate_stage(size_t node, const Stage& consumer, size_t input_index) {
    Stage st = skeleton(graph.nodes[node].inner);
    prune_producer_for_consumer(st, consumer, input_index);
    assign_layouts(st, graph.nodes[node].inner, true);
    return instantiate(node, std::move(st), true);
  }

  size_t instantiate(size_t node_id, Stage st, bool duplicate) {
    const std::vector<Source> inputs = lower_inputs(node_id, st);
    if (duplicate)
      for (const Dup& d : duplicates)
        if (d.node == node_id && d.stage == st && d.inputs == inputs) return d.stage_id;
    ProgramShape shape = stage_shape(st, inputs);
    const size_t id = nodes.size();
    if (duplicate) duplicates.push_back({node_id, st, inputs, id});
    GNode<Stage> gn;
    gn.inner = std::move(st);
    gn.inputs = inputs;
    gn.outputs = graph.nodes[node_id].outputs;
    nodes.push_back(std::move(gn));
    shapes.push_back(std::move(shape));
    return id;
  }

  std::vector<Source> lower_inputs(size_t node_id, const Stage& st) {
    std::vector<Source> out;
    const auto& gin = graph.nodes[node_id].inputs;
    for (size_t i = 0; i < gin.size(); ++i) {
      const Source s = gin[i];
      if (s.is_input) {
        if (st.inputs[i].site)
          lower_error("node " + std::to_string(node_id) + " input " + std::to_string(i) +
                      " is a graph input with a compute site");
        out.push_back(s);
      } else {
        if (s.output != 0)
          lower_error("node " + std::to_string(node_id) + " input " + std::to_string(i) + " references output " +
                      std::to_string(s.output));
        if (st.inputs[i].site) out.push_back(Source::node(duplicate_stage(s.id, st, i)));
        else out.push_back(Source::node(materialized_stage(s.id)));
      }
    }
    return out;
  }

  ProgramShape source_shape(Source s, size_t rank) {
    if (s.is_input) {
      input_ranks[s.id] = std::max(input_ranks[s.id], rank);
      ProgramShape out;
      for (size_t d = 0; d < rank; ++d) out.push_back({s.id, d});
      return out;
    }
    if (s.id >= shapes.size()) lower_error("stage input references shape of nonexistent stage " + std::to_string(s.id));
    if (shapes[s.id].size() != rank)
      lower_error("stage input expects rank " + std::to_string(rank) + " but source stage " + std::to_string(s.id) +
                  " has rank " + std::to_string(shapes[s.id].size()));
    return shapes[s.id];
  }

  ProgramShape stage_shape(const Stage& st, const std::vector<Source>& inputs) {
    std::map<size_t, ShapeDim> dims;  // first operand that mentions an index names its extent
    for (size_t i = 0; i < st.inputs.size(); ++i) {
      const ProgramShape src = source_shape(inputs[i], st.inputs[i].shape.size());
      for (size_t d = 0; d < st.inputs[i].shape.size(); ++d) dims.emplace(st.inputs[i].shape[d], src[d]);
    }
    ProgramShape out;
    for (size_t index : st.output.shape) {
      auto it = dims.find(index);
      if (it == dims.end()) lower_error("stage output index " + std::to_string(index) + " has no input shape source");
      out.push_back(it->second);
    }
    return out;
  }
};

}  // namespace

StageProgram lower_graph_to_stages(const Graph<Node>& graph) {
  Builder b(graph);
  StageProgram out;
  for (Source s : graph.outputs) out.graph.outputs.push_back(s.is_input ? s : Source::node(b.materialized_stage(s.id), s.output));
  for (size_t i = 0; i < graph.inputs; ++i) {
    ProgramShape shape;
    for (size_t d = 0; d < b.input_ranks[i]; ++d) shape.push_back({i, d});
    out.input_shapes.push_back(shape);
  }
  out.graph.inputs = graph.inputs;
  out.graph.nodes = std::move(b.nodes);
  out.node_shapes = std::move(b.shapes);
  // a stage pruned by its consumer can never be a program output or be read without a compute site
  for (size_t n = 0; n < out.graph.nodes.size(); ++n) {
    bool scoped = false;
    for (const SAxis& a : out.graph.nodes[n].inner.axes) scoped |= a.pruned && a.by.consumer;
    if (!scoped) continue;
    for (Source s : out.graph.outputs)
      if (!s.is_input && s.id == n) lower_error("node " + std::to_string(n) + ": graph output references consumer-scoped stage");
  }
  return out;
}

}  // namespace ic
