// Expr -> Node: canonical index numbering (output axes first, then inputs in
// source order), split lists, loop order, compute sites and the reduction init
// site.  Follows compiler/src/lower/expr_to_node.rs:18-195 and
// compiler/src/check/node.rs:116-205.
#include <algorithm>
#include <map>
#include <set>

#include "ir.h"

namespace ic {
namespace {

std::string fmt_axis(AxisLevel a) { return std::to_string(a.index) + std::string(a.level, '\''); }

// Default init site = the last output loop in the order; Root when the output is a scalar.
std::optional<NodeSite> required_init_site(const Node& node, const std::vector<AxisLevel>& order) {
  std::set<size_t> out(node.output.begin(), node.output.end());
  bool has_reduction = false;
  for (size_t i = 0; i < node.rank; ++i) has_reduction |= !out.count(i);
  if (!has_reduction) return std::nullopt;
  size_t output_levels = 0;
  for (size_t i : node.output) output_levels += node.splits[i].size() + 1;
  if (output_levels == 0) return NodeSite{true, {}};
  size_t seen = 0;
  std::optional<size_t> last;
  for (size_t p = 0; p < order.size(); ++p)
    if (out.count(order[p].index)) {
      last = p;
      ++seen;
    }
  if (seen != output_levels) lower_error("order does not contain every output loop level");
  return NodeSite{false, order[*last]};
}

void validate_init_site(const Node& node, const std::vector<AxisLevel>& order, NodeSite site) {
  std::set<size_t> out(node.output.begin(), node.output.end());
  size_t min_depth = 0;
  for (size_t p = 0; p < order.size(); ++p)
    if (out.count(order[p].index)) min_depth = p + 1;
  size_t depth = 0;
  if (!site.root) {
    auto it = std::find(order.begin(), order.end(), site.at);
    if (it == order.end()) lower_error("init site is outside loop order");
    depth = size_t(it - order.begin()) + 1;
  }
  if (depth < min_depth)
    lower_error("init site must be at or inside " +
                (min_depth == 0 ? std::string("Root") : "At(" + fmt_axis(order[min_depth - 1]) + ")"));
}

void validate_node(const Node& node) {
  std::set<size_t> referenced;
  for (size_t i = 0; i < node.inputs.size(); ++i)
    for (size_t ix : node.inputs[i]) {
      if (ix >= node.rank) lower_error("input " + std::to_string(i) + " references nonexistent index " + std::to_string(ix));
      referenced.insert(ix);
    }
  std::set<size_t> out_seen;
  for (size_t ix : node.output) {
    if (ix >= node.rank) lower_error("output references nonexistent index " + std::to_string(ix));
    if (!out_seen.insert(ix).second) lower_error("output repeats index " + std::to_string(ix));
    referenced.insert(ix);
  }
  for (size_t ix = 0; ix < node.rank; ++ix)
    if (!referenced.count(ix)) lower_error("node index " + std::to_string(ix) + " is not referenced");

  std::set<std::pair<size_t, size_t>> seen;
  size_t expected = 0;
  for (const auto& s : node.splits) expected += s.size() + 1;
  for (AxisLevel a : node.order) {
    if (a.index >= node.rank) lower_error("order references nonexistent index " + std::to_string(a.index));
    if (a.level > node.splits[a.index].size()) lower_error("order references nonexistent loop level " + fmt_axis(a));
    if (!seen.insert({a.index, a.level}).second) lower_error("order repeats loop level " + fmt_axis(a));
  }
  if (node.order.size() != expected)
    lower_error("order must contain " + std::to_string(expected) + " loop levels, found " + std::to_string(node.order.size()));
  const auto required = required_init_site(node, node.order);
  if (!required && node.init_site) lower_error("pointwise node cannot have an init site");
  if (required && !node.init_site) lower_error("reduction node must have an init site");
  if (required && node.init_site) validate_init_site(node, node.order, *node.init_site);
}

}  // namespace

Node lower_expr_to_node(const Expr& expr) {
  std::vector<char> axis_order;
  auto add_axis = [&](char a) {
    if (std::find(axis_order.begin(), axis_order.end(), a) == axis_order.end()) axis_order.push_back(a);
  };
  for (char a : expr.output) add_axis(a);
  for (const auto& in : expr.inputs)
    for (char a : in) add_axis(a);
  std::map<char, size_t> axis_map;
  for (size_t i = 0; i < axis_order.size(); ++i) axis_map[axis_order[i]] = i;
  auto lower_pattern = [&](const std::vector<char>& pattern) {
    std::vector<size_t> out;
    for (char a : pattern) {
      auto it = axis_map.find(a);
      if (it == axis_map.end()) lower_error(std::string("unknown local axis `") + a + "`");
      out.push_back(it->second);
    }
    return out;
  };

  Node node;
  node.op = expr.op;
  node.rank = axis_order.size();
  for (const auto& in : expr.inputs) node.inputs.push_back(lower_pattern(in));
  node.output = lower_pattern(expr.output);
  node.splits.resize(node.rank);
  for (const auto& [axis, factors] : expr.splits) {
    auto it = axis_map.find(axis);
    if (it != axis_map.end()) node.splits[it->second] = factors;
  }
  node.compute_sites.assign(expr.inputs.size(), std::nullopt);

  if (expr.permutation.empty()) {
    for (size_t i = 0; i < node.rank; ++i)
      for (size_t level = 0; level <= node.splits[i].size(); ++level) node.order.push_back({i, level});
    node.init_site = required_init_site(node, node.order);
  } else {
    std::optional<AxisLevel> last;
    std::optional<NodeSite> explicit_init;
    for (const PermAtom& atom : expr.permutation) {
      switch (atom.kind) {
        case PermAtom::Axis: {
          auto it = axis_map.find(atom.axis);
          if (it == axis_map.end()) lower_error(std::string("unknown local axis `") + atom.axis + "`");
          last = AxisLevel{it->second, atom.part};
          node.order.push_back(*last);
          break;
        }
        case PermAtom::Input:
          if (atom.operand >= node.compute_sites.size())
            lower_error("permutation references nonexistent input " + std::to_string(atom.operand));
          node.compute_sites[atom.operand] = last ? NodeSite{false, *last} : NodeSite{true, {}};
          break;
        case PermAtom::Bang: explicit_init = last ? NodeSite{false, *last} : NodeSite{true, {}}; break;
      }
    }
    const auto required = required_init_site(node, node.order);
    if (!required && explicit_init) lower_error("pointwise node cannot have an output init directive");
    if (required && explicit_init) {
      validate_init_site(node, node.order, *explicit_init);
      node.init_site = explicit_init;
    } else {
      node.init_site = required;
    }
  }
  validate_node(node);
  return node;
}

}  // namespace ic
