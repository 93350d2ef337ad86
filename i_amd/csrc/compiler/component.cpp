// Language rules for components (compiler/src/check/component.rs:7-412) and the
// wiring of combinator trees into an ordered dataflow graph
// (compiler/src/lower/component_to_graph.rs:11-210).
#include <algorithm>
#include <map>
#include <set>

#include "ir.h"

namespace ic {
namespace {

[[noreturn]] void expr_error(size_t expr, const std::string& message) {
  // surfaces as LowerError { message: "expr N: ..." } (component_to_graph.rs:223-225)
  lower_error("expr " + std::to_string(expr) + ": " + message);
}

std::string apostrophes(size_t n) { return std::string(n, '\''); }

bool reducible(Op op) {
  return op == Op::Add || op == Op::Mul || op == Op::Max || op == Op::Min || op == Op::And || op == Op::Or || op == Op::Xor;
}

void validate_expr(const Expr& e, size_t ix) {
  auto check_chars = [&](const std::vector<char>& pattern, const std::string& what) {
    for (char axis : pattern)
      if (!(axis >= 'a' && axis <= 'z'))
        expr_error(ix, what + " uses invalid axis `" + axis + "`; axes must be [a-z]");
  };
  for (size_t i = 0; i < e.inputs.size(); ++i) check_chars(e.inputs[i], "input " + std::to_string(i));
  check_chars(e.output, "output");
  {
    std::set<char> seen;
    for (char axis : e.output)
      if (!seen.insert(axis).second) expr_error(ix, std::string("output pattern repeats axis `") + axis + "`");
  }
  std::set<char> in_axes, out_axes(e.output.begin(), e.output.end());
  for (const auto& in : e.inputs) in_axes.insert(in.begin(), in.end());
  const bool is_reduction = in_axes != out_axes;

  if (e.inputs.size() == 1) {
    for (char axis : out_axes)
      if (!in_axes.count(axis)) expr_error(ix, std::string("output axis `") + axis + "` does not appear in the input");
    if (e.op == Op::Not) {
      if (is_reduction) expr_error(ix, "operator `Not` is only valid in unary pointwise form");
    } else if (is_reduction && !reducible(e.op)) {
      expr_error(ix, std::string("operator `") + op_name(e.op) + "` is not reducible");
    }
  } else if (e.inputs.size() == 2) {
    if (e.op == Op::Not) expr_error(ix, "operator `Not` is only valid in unary pointwise form");
    if (is_reduction)
      expr_error(ix, std::string("binary operator `") + op_name(e.op) +
                         "` must be pointwise; output axes must match the union of input axes");
  } else {
    expr_error(ix, std::string("operator `") + op_name(e.op) + "` expects one or two inputs, found " +
                       std::to_string(e.inputs.size()));
  }

  // ---- schedule
  std::set<char> local = in_axes;
  local.insert(out_axes.begin(), out_axes.end());
  std::map<char, size_t> split_parts;
  for (const auto& [axis, factors] : e.splits) {
    if (!(axis >= 'a' && axis <= 'z'))
      expr_error(ix, std::string("split uses invalid axis `") + axis + "`; axes must be [a-z]");
    if (!local.count(axis)) expr_error(ix, std::string("split references unknown local axis `") + axis + "`");
    auto it = split_parts.find(axis);
    if (it != split_parts.end()) {
      if (it->second == factors.size()) expr_error(ix, std::string("duplicate split entry for axis `") + axis + "`");
      expr_error(ix, std::string("contradictory split entries for axis `") + axis + "`");
    }
    split_parts[axis] = factors.size();
  }
  if (e.permutation.empty()) return;

  auto expected_refs = [&](const std::set<char>& axes) {
    std::set<std::pair<char, size_t>> out;
    for (char axis : axes) {
      const size_t max_part = split_parts.count(axis) ? split_parts[axis] : 0;
      for (size_t part = 0; part <= max_part; ++part) out.insert({axis, part});
    }
    return out;
  };
  const auto expected = expected_refs(local);
  const auto output_parts = expected_refs(out_axes);
  std::set<std::pair<char, size_t>> seen;
  std::set<size_t> seen_inputs;
  bool seen_bang = false;
  for (const PermAtom& atom : e.permutation) {
    switch (atom.kind) {
      case PermAtom::Axis: {
        if (!(atom.axis >= 'a' && atom.axis <= 'z'))
          expr_error(ix, std::string("permutation uses invalid axis `") + atom.axis + "`; axes must be [a-z]");
        if (!local.count(atom.axis))
          expr_error(ix, std::string("permutation references unknown local axis `") + atom.axis + "`");
        const size_t max_part = split_parts.count(atom.axis) ? split_parts[atom.axis] : 0;
        if (atom.part > max_part)
          expr_error(ix, std::string("permutation references nonexistent split part `") + atom.axis +
                             apostrophes(atom.part) + "`");
        if (!seen.insert({atom.axis, atom.part}).second)
          expr_error(ix, std::string("permutation repeats axis part `") + atom.axis + apostrophes(atom.part) + "`");
        break;
      }
      case PermAtom::Input:
        if (atom.operand >= e.inputs.size())
          expr_error(ix, "permutation references nonexistent input " + std::to_string(atom.operand));
        if (!seen_inputs.insert(atom.operand).second)
          expr_error(ix, "duplicate compute directive for input " + std::to_string(atom.operand));
        break;
      case PermAtom::Bang:
        if (seen_bang) expr_error(ix, "duplicate output init directive");
        if (local == out_axes) expr_error(ix, "output init directive is only valid for reductions");
        seen_bang = true;
        for (const auto& part : output_parts)
          if (!seen.count(part))
            expr_error(ix, std::string("output init cannot appear before output axis part `") + part.first +
                               apostrophes(part.second) + "`");
        break;
    }
  }
  if (seen.size() != expected.size())
    expr_error(ix, "permutation must list each local axis part exactly once; expected " +
                       std::to_string(expected.size()) + ", found " + std::to_string(seen.size()));
  if (seen != expected)
    for (const auto& part : expected)
      if (!seen.count(part))
        expr_error(ix, std::string("permutation is missing axis part `") + part.first + apostrophes(part.second) + "`");
}

void validate_inner(const Component& c, size_t& next_expr) {
  switch (c.kind) {
    case Component::Identity: return;
    case Component::Leaf: validate_expr(c.expr, next_expr++); return;
    case Component::Swap: validate_inner(*c.a, next_expr); return;
    default:
      validate_inner(*c.a, next_expr);
      validate_inner(*c.b, next_expr);
  }
}

// ---------------------------------------------------------------- wiring
struct Partial {
  size_t inputs = 0;
  std::vector<GNode<Node>> nodes;
  std::vector<Source> outputs;
};

Source remap(Source s, const std::vector<Source>& input_map, size_t node_offset) {
  return s.is_input ? input_map[s.id] : Source::node(node_offset + s.id, s.output);
}
std::vector<Source> input_sources(size_t base, size_t len) {
  std::vector<Source> out;
  for (size_t i = 0; i < len; ++i) out.push_back(Source::input(base + i));
  return out;
}
// Appends `g`'s nodes (inputs rewired through input_map) and returns its rewired outputs.
std::vector<Source> splice(Partial& into, Partial g, const std::vector<Source>& input_map) {
  const size_t offset = into.nodes.size();
  std::vector<Source> outs;
  for (Source s : g.outputs) outs.push_back(remap(s, input_map, offset));
  for (auto& n : g.nodes) {
    for (Source& s : n.inputs) s = remap(s, input_map, offset);
    into.nodes.push_back(std::move(n));
  }
  return outs;
}

Partial to_partial(const Component& c) {
  switch (c.kind) {
    case Component::Identity: {
      Partial p;
      p.inputs = 1;
      p.outputs = {Source::input(0)};
      return p;
    }
    case Component::Leaf: {
      Partial p;
      GNode<Node> n;
      n.inner = lower_expr_to_node(c.expr);
      n.inputs = input_sources(0, c.expr.inputs.size());
      p.inputs = n.inner.inputs.size();
      p.nodes.push_back(std::move(n));
      p.outputs = {Source::node(0, 0)};
      return p;
    }
    case Component::Swap: {
      Partial p = to_partial(*c.a);
      if (p.outputs.size() >= 2) std::swap(p.outputs[0], p.outputs[1]);
      return p;
    }
    default: break;
  }
  Partial left = to_partial(*c.a), right = to_partial(*c.b);
  Partial out;
  switch (c.kind) {
    case Component::Pair: {
      const size_t li = left.inputs, ri = right.inputs;
      auto lo = splice(out, std::move(left), input_sources(0, li));
      auto ro = splice(out, std::move(right), input_sources(li, ri));
      out.inputs = li + ri;
      out.outputs = lo;
      out.outputs.insert(out.outputs.end(), ro.begin(), ro.end());
      return out;
    }
    case Component::Chain: {  // roots of left feed leaves of right, left to right
      const size_t li = left.inputs, ri = right.inputs;
      const size_t paired = std::min(left.outputs.size(), ri);
      auto lo = splice(out, std::move(left), input_sources(0, li));
      std::vector<Source> rmap(lo.begin(), lo.begin() + paired);
      for (size_t i = 0; i < ri - paired; ++i) rmap.push_back(Source::input(li + i));
      auto ro = splice(out, std::move(right), rmap);
      out.inputs = li + ri - paired;
      out.outputs.assign(lo.begin() + paired, lo.end());
      out.outputs.insert(out.outputs.end(), ro.begin(), ro.end());
      return out;
    }
    case Component::Compose: {  // roots of right feed leaves of left
      const size_t li = left.inputs, ri = right.inputs;
      const size_t paired = std::min(li, right.outputs.size());
      auto ro = splice(out, std::move(right), input_sources(0, ri));
      std::vector<Source> lmap(ro.begin(), ro.begin() + paired);
      for (size_t i = 0; i < li - paired; ++i) lmap.push_back(Source::input(ri + i));
      auto lo = splice(out, std::move(left), lmap);
      out.inputs = ri + li - paired;
      out.outputs = lo;
      out.outputs.insert(out.outputs.end(), ro.begin() + paired, ro.end());
      return out;
    }
    case Component::Fanout: {  // both read the same leading inputs
      const size_t li = left.inputs, ri = right.inputs;
      const size_t paired = std::min(li, ri);
      auto lo = splice(out, std::move(left), input_sources(0, li));
      std::vector<Source> rmap = input_sources(0, paired);
      for (size_t i = 0; i < ri - paired; ++i) rmap.push_back(Source::input(li + i));
      auto ro = splice(out, std::move(right), rmap);
      out.inputs = li + ri - paired;
      out.outputs = lo;
      out.outputs.insert(out.outputs.end(), ro.begin(), ro.end());
      return out;
    }
    default: lower_error("unknown combinator");
  }
}

}  // namespace

void validate_component(const Component& component) {
  size_t next = 0;
  validate_inner(component, next);
}

Graph<Node> lower_component_to_graph(const Component& component) {
  validate_component(component);
  Partial p = to_partial(component);
  Graph<Node> g;
  g.inputs = p.inputs;
  g.nodes = std::move(p.nodes);
  g.outputs = std::move(p.outputs);
  // graph invariants (check/graph.rs:26-50): operand counts line up, producers precede consumers
  for (size_t n = 0; n < g.nodes.size(); ++n) {
    const auto& node = g.nodes[n];
    if (node.inputs.size() != node.inner.inputs.size())
      lower_error("node " + std::to_string(n) + ": graph has " + std::to_string(node.inputs.size()) + " inputs for " +
                  std::to_string(node.inner.inputs.size()) + " node inputs");
    for (Source s : node.inputs) {
      if (s.is_input && s.id >= g.inputs)
        lower_error("node " + std::to_string(n) + " input references nonexistent input " + std::to_string(s.id));
      if (!s.is_input && s.id >= n)
        lower_error("node " + std::to_string(n) + " input references non-prior node " + std::to_string(s.id));
    }
  }
  return g;
}

}  // namespace ic
