#include "ir.h"

#include <sstream>

namespace ic {

const char* op_name(Op op) {
  switch (op) {
    case Op::Add: return "Add";
    case Op::Mul: return "Mul";
    case Op::Div: return "Div";
    case Op::Sub: return "Sub";
    case Op::Max: return "Max";
    case Op::Min: return "Min";
    case Op::Pow: return "Pow";
    case Op::Log: return "Log";
    case Op::Gt: return "Gt";
    case Op::Ge: return "Ge";
    case Op::Lt: return "Lt";
    case Op::Le: return "Le";
    case Op::Eq: return "Eq";
    case Op::Ne: return "Ne";
    case Op::And: return "And";
    case Op::Or: return "Or";
    case Op::Xor: return "Xor";
    case Op::Not: return "Not";
  }
  return "?";
}

namespace {
// Rust's {:?} for a string: quotes, backslashes and control characters escaped.
std::string debug_quote(const std::string& s) {
  std::string out = "\"";
  for (char ch : s) {
    switch (ch) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\t': out += "\\t"; break;
      case '\r': out += "\\r"; break;
      default: out += ch;
    }
  }
  return out + "\"";
}
}  // namespace

std::string CompileError::debug_string() const {
  if (kind == "ParseError") return "ParseError { offset: " + std::to_string(offset) + ", message: " + debug_quote(message) + " }";
  return kind + " { message: " + debug_quote(message) + " }";
}

void lower_error(const std::string& message) { throw CompileError("LowerError", message); }

std::string ExtentKind::debug_string() const {
  std::ostringstream os;
  switch (kind) {
    case Semantic: os << "Semantic"; break;
    case Base:
      os << "Base([";
      for (size_t i = 0; i < factors.size(); ++i) os << (i ? ", " : "") << factors[i];
      os << "])";
      break;
    case Split: os << "Split { level: " << level << ", factor: " << factor << " }"; break;
  }
  return os.str();
}

Lowered lower_component(const Component& component) {
  Lowered out;
  out.graph = lower_component_to_graph(component);
  out.stages = lower_graph_to_stages(out.graph);
  out.kernels = lower_stages_to_kernels(out.stages);
  out.plan = lower_kernels_to_exec_plan(out.kernels);
  return out;
}

}  // namespace ic
