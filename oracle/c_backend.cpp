/*
 * C text backend for the CPU oracle: renders the compiler's statement IR
 * (ic::Module) to one C translation unit with the generated-library ABI
 * count / ranks / shapes / exec + f0..fN, the way the reference C backend does
 * (compiler/src/backends/c/mod.rs:9-63, stmt.rs:11-192, expr.rs:12-366,
 * fmt.rs:1-21).
 *
 * TEST INFRASTRUCTURE ONLY.  The shipped library never links or calls this
 * file; it is built into oracle/liboracle_cbackend.so for the test-suite and the
 * benchmark's cpu_baseline leg, which compile the emitted text with
 * `cc -O3 -shared -fPIC -lm` (core/src/lib.rs:400-406) and run it on the host.
 *
 * Pinned by: the emitted text for the demo FlashAttention component equals
 * ilang-python/annotated-flashattn.c after comments and whitespace are
 * stripped (tests/golden/flashattn_emitted.c.norm), the substring expectations
 * of compiler/src/backends/c/mod.rs:107-351 restated in tests/test_c_emitter.py,
 * and NumPy closed forms for every other component the tests compile.
 */
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "../i_amd/csrc/core/handles.h"

using namespace ic;

namespace {

// two spaces before every non-empty line; a trailing newline yields no extra line
std::string indent(const std::string& source) {
  std::vector<std::string> lines;
  size_t start = 0;
  while (start < source.size()) {
    size_t end = source.find('\n', start);
    if (end == std::string::npos) end = source.size();
    lines.push_back(source.substr(start, end - start));
    start = end + 1;
  }
  std::string out;
  for (size_t i = 0; i < lines.size(); ++i) {
    if (i) out += "\n";
    if (!lines[i].empty()) out += "  " + lines[i];
  }
  return out;
}

std::string join(const std::vector<std::string>& items, const std::string& sep) {
  std::string out;
  for (size_t i = 0; i < items.size(); ++i) out += (i ? sep : "") + items[i];
  return out;
}

std::string initializer(const std::string& prefix, const std::vector<std::string>& items) {
  return prefix + "{\n" + indent(join(items, ",\n")) + "\n}";
}

std::string render_scalar(float v) {
  if (std::isnan(v)) return "NAN";
  if (std::isinf(v)) return v > 0 ? "INFINITY" : "(-INFINITY)";
  char buf[64];
  snprintf(buf, sizeof buf, "%.8f", (double)v);
  std::string s = buf;
  while (!s.empty() && s.back() == '0') s.pop_back();
  if (!s.empty() && s.back() == '.') s.pop_back();
  return s.find('.') != std::string::npos ? s + "f" : s + ".0f";
}

enum Oper { OAdd, OSub, OMul, ODiv, ORem, OLt, OGt, OLe, OGe, OEq, ONe, OAnd, OOr, ONone };
const char* symbol(Oper o) {
  static const char* s[] = {"+", "-", "*", "/", "%", "<", ">", "<=", ">=", "==", "!=", "&&", "||"};
  return s[o];
}
int precedence(Oper o) {
  switch (o) {
    case OMul: case ODiv: case ORem: return 70;
    case OAdd: case OSub: return 60;
    case OLt: case OGt: case OLe: case OGe: return 50;
    case OEq: case ONe: return 45;
    case OAnd: return 40;
    case OOr: return 30;
    default: return 100;
  }
}
struct Ctx {
  Oper parent = ONone;
  int side = 0;  // 0 none, 1 left, 2 right
};
struct Rendered {
  std::string source;
  int precedence = 100;
  Oper op = ONone;
};

Rendered render_in(const MExpr& e, Ctx ctx);
std::string render(const MExpr& e) { return render_in(e, {}).source; }

Rendered apply_ctx(Rendered r, Ctx ctx) {
  if (ctx.parent == ONone) return r;
  const int pp = precedence(ctx.parent);
  const bool assoc = (ctx.parent == OAdd && r.op == OAdd) || (ctx.parent == OMul && r.op == OMul) ||
                     (ctx.parent == OAnd && r.op == OAnd) || (ctx.parent == OOr && r.op == OOr);
  if (r.precedence < pp || (r.precedence == pp && ctx.side == 2 && !assoc)) r.source = "(" + r.source + ")";
  return r;
}

void collect_add_terms(const MExpr& e, std::vector<const MExpr*>& terms) {
  if (e.kind == MExpr::Add) {
    collect_add_terms(*e.args[0], terms);
    collect_add_terms(*e.args[1], terms);
  } else {
    terms.push_back(&e);
  }
}

std::string render_index(const std::string& base, const MExpr& ix, bool multiline) {
  if (multiline && ix.kind == MExpr::Add) {
    std::vector<const MExpr*> terms;
    collect_add_terms(ix, terms);
    std::vector<std::string> lines;
    for (size_t i = 0; i < terms.size(); ++i) lines.push_back(render(*terms[i]) + (i + 1 == terms.size() ? "" : " +"));
    return base + "[\n" + indent(join(lines, "\n")) + "\n]";
  }
  return base + "[" + render(ix) + "]";
}

Rendered render_binary(Oper o, const MExpr& l, const MExpr& r) {
  Rendered out;
  out.source = render_in(l, {o, 1}).source + " " + symbol(o) + " " + render_in(r, {o, 2}).source;
  out.precedence = precedence(o);
  out.op = o;
  return out;
}

Rendered render_joined(Oper o, const std::vector<MExprPtr>& args, Ctx ctx) {
  if (args.empty()) return {"0.0f", 100, ONone};
  Rendered out;
  out.source = render_in(*args[0], {o, 1}).source;
  for (size_t i = 1; i < args.size(); ++i) out.source += std::string(" ") + symbol(o) + " " + render_in(*args[i], {o, 2}).source;
  out.precedence = precedence(o);
  out.op = o;
  return apply_ctx(out, ctx);
}

std::string call_fold(const char* fn, const std::vector<MExprPtr>& args) {
  if (args.empty()) return "0.0f";
  std::string acc = render(*args[0]);
  for (size_t i = 1; i < args.size(); ++i) acc = std::string(fn) + "(" + acc + ", " + render(*args[i]) + ")";
  return acc;
}

Rendered render_op(Op op, const std::vector<MExprPtr>& args, Ctx ctx) {
  switch (op) {
    case Op::Add: return render_joined(OAdd, args, ctx);
    case Op::Mul: return render_joined(OMul, args, ctx);
    case Op::Div: return render_joined(ODiv, args, ctx);
    case Op::Sub: return render_joined(OSub, args, ctx);
    case Op::Max: return {call_fold("fmaxf", args), 100, ONone};
    case Op::Min: return {call_fold("fminf", args), 100, ONone};
    case Op::Pow: return {call_fold("powf", args), 100, ONone};
    case Op::Log: return {"logf(" + render(*args[0]) + ")", 100, ONone};
    case Op::Gt: return render_joined(OGt, args, ctx);
    case Op::Ge: return render_joined(OGe, args, ctx);
    case Op::Lt: return render_joined(OLt, args, ctx);
    case Op::Le: return render_joined(OLe, args, ctx);
    case Op::Eq: return render_joined(OEq, args, ctx);
    case Op::Ne: return render_joined(ONe, args, ctx);
    case Op::And: return render_joined(OAnd, args, ctx);
    case Op::Or: return render_joined(OOr, args, ctx);
    case Op::Xor: {
      if (args.empty()) return {"0", 100, ONone};
      std::string acc = render(*args[0]);
      for (size_t i = 1; i < args.size(); ++i) acc = "(((" + acc + ") != 0.0f) != ((" + render(*args[i]) + ") != 0.0f))";
      return {acc, 100, ONone};
    }
    case Op::Not: {
      Rendered v = render_in(*args[0], {});
      Rendered out{"!" + (v.precedence < 80 ? "(" + v.source + ")" : v.source), 80, ONone};
      return apply_ctx(out, ctx);
    }
  }
  return {"", 100, ONone};
}

const char* field_name(MField f) {
  switch (f) {
    case MField::Data: return "data";
    case MField::Shape: return "shape";
    case MField::Layout: return "layout";
    case MField::Rank: return "rank";
  }
  return "";
}

Rendered render_in(const MExpr& e, Ctx ctx) {
  Rendered r;
  switch (e.kind) {
    case MExpr::Usize: r.source = std::to_string(e.usize); break;
    case MExpr::Scalar: r.source = render_scalar(e.scalar); break;
    case MExpr::Ident: r.source = e.ident; break;
    case MExpr::Index: {
      const bool data = e.args[0]->kind == MExpr::Field && e.args[0]->field == MField::Data;
      r.source = render_index(render(*e.args[0]), *e.args[1], data);
      break;
    }
    case MExpr::Field: r.source = render(*e.args[0]) + "." + field_name(e.field); break;
    case MExpr::Cast: {
      const char* fn = e.cast == MCast::View ? "as_view" : e.cast == MCast::ViewMut ? "as_view_mut" : "view_mut_as_view";
      r.source = std::string(fn) + "(&" + render(*e.args[0]) + ")";
      break;
    }
    case MExpr::OpCall: return render_op(e.op, e.args, ctx);
    case MExpr::Add: r = render_binary(OAdd, *e.args[0], *e.args[1]); break;
    case MExpr::Sub: r = render_binary(OSub, *e.args[0], *e.args[1]); break;
    case MExpr::Mul: r = render_binary(OMul, *e.args[0], *e.args[1]); break;
    case MExpr::Div: r = render_binary(ODiv, *e.args[0], *e.args[1]); break;
    case MExpr::Rem: r = render_binary(ORem, *e.args[0], *e.args[1]); break;
    case MExpr::Lt: r = render_binary(OLt, *e.args[0], *e.args[1]); break;
    case MExpr::Eq: r = render_binary(OEq, *e.args[0], *e.args[1]); break;
    case MExpr::And: r = render_binary(OAnd, *e.args[0], *e.args[1]); break;
  }
  return apply_ctx(r, ctx);
}

using Env = std::map<std::string, MType>;

std::string render_block(const std::vector<MStmt>& block, Env& env);

std::string array_decl(const std::string& name, const std::vector<MExprPtr>& values) {
  if (values.empty()) return "const size_t* " + name + " = NULL;";
  std::vector<std::string> items;
  for (const auto& v : values) items.push_back(render(*v));
  return "const size_t " + name + "[] = " + initializer("", items) + ";";
}

std::string render_stmt(const MStmt& s, Env& env) {
  switch (s.kind) {
    case MStmt::Let: {
      env[s.ident] = s.type;
      const char* ty = s.type == MType::View ? "const View" : s.type == MType::ViewMut ? "ViewMut" : s.type == MType::Usize ? "size_t" : "float";
      return std::string(ty) + " " + s.ident + " = " + render(*s.value) + ";";
    }
    case MStmt::Set: return render(*s.dst) + " = " + render(*s.value) + ";";
    case MStmt::Alloc: {
      env[s.ident] = MType::ViewMut;
      const std::string l = s.ident + "_layout", sh = s.ident + "_shape";
      return array_decl(l, s.layout) + "\n" + array_decl(sh, s.shape) + "\nViewMut " + s.ident + " = alloc_view_mut(" +
             std::to_string(s.layout.size()) + ", " + (s.layout.empty() ? "NULL" : l) + ", " + (s.shape.empty() ? "NULL" : sh) + ");";
    }
    case MStmt::Free: return "free(" + s.ident + ".data);";
    case MStmt::Dispatch: {
      std::vector<std::string> reads, writes;
      for (const auto& r : s.reads) reads.push_back(env.count(r) && env[r] == MType::ViewMut ? "view_mut_as_view(&" + r + ")" : r);
      for (const auto& w : s.writes) writes.push_back(w);
      return s.ident + "(\n" + indent(initializer("(const View[])", reads)) + ",\n" + indent(initializer("(ViewMut[])", writes)) + "\n);";
    }
    case MStmt::Loop: {
      Env child = env;
      child[s.ident] = MType::Usize;
      return "for (size_t " + s.ident + " = 0; " + s.ident + " < " + render(*s.value) + "; ++" + s.ident + ") {\n" +
             indent(render_block(s.body, child)) + "\n}";
    }
    case MStmt::If: {
      Env child = env;
      return "if (" + render(*s.value) + ") {\n" + indent(render_block(s.body, child)) + "\n}";
    }
    case MStmt::Return: return s.value ? "return " + render(*s.value) + ";" : "return;";
  }
  return "";
}

std::string render_block(const std::vector<MStmt>& block, Env& env) {
  std::vector<std::string> lines;
  for (const auto& s : block) lines.push_back(render_stmt(s, env));
  return join(lines, "\n");
}

std::string render_function(const MFn& f) {
  std::string sig;
  switch (f.signature) {
    case MSignature::Count: sig = "size_t " + f.ident + "(void)"; break;
    case MSignature::Ranks: sig = "void " + f.ident + "(size_t* ranks)"; break;
    case MSignature::Shapes: sig = "void " + f.ident + "(const Tensor* inputs, size_t** shapes)"; break;
    case MSignature::Exec: sig = "void " + f.ident + "(const Tensor* inputs, TensorMut* outputs)"; break;
    case MSignature::Kernel: sig = "void " + f.ident + "(const View* readonlys, ViewMut* writeables)"; break;
  }
  Env env;
  return sig + " {\n" + indent(render_block(f.body, env)) + "\n}";
}

const char* kPrelude =
    "#include <math.h>\n#include <stddef.h>\n#include <stdint.h>\n#include <stdlib.h>\n\n"
    "typedef struct { const float* data; const size_t* shape; const size_t rank; } Tensor;\n"
    "typedef struct { float* data; const size_t* shape; const size_t rank; } TensorMut;\n"
    "typedef struct { const float* data; const size_t* shape; const size_t* layout; } View;\n"
    "typedef struct { float* data; const size_t* shape; const size_t* layout; } ViewMut;\n\n"
    "static inline ViewMut alloc_view_mut(size_t ndims, const size_t* layout, const size_t* shape) {\n"
    "  size_t n = 1;\n  for (size_t i = 0; i < ndims; ++i) n *= layout[i];\n"
    "  float* data = (float*)malloc(n * sizeof(float));\n"
    "  return (ViewMut){ .data = data, .shape = shape, .layout = layout };\n}\n\n"
    "static inline View as_view(const Tensor* t) {\n"
    "  return (View){ .data = t->data, .shape = t->shape, .layout = t->shape };\n}\n\n"
    "static inline ViewMut as_view_mut(const TensorMut* t) {\n"
    "  return (ViewMut){ .data = t->data, .shape = t->shape, .layout = t->shape };\n}\n\n"
    "static inline View view_mut_as_view(const ViewMut* t) {\n"
    "  return (View){ .data = t->data, .shape = t->shape, .layout = t->layout };\n}\n\n";

std::string render_module(const Module& m) {
  std::vector<std::string> kernels;
  for (const auto& k : m.kernels) kernels.push_back(render_function(k));
  return std::string(kPrelude) + render_function(m.count) + "\n\n" + render_function(m.ranks) + "\n\n" +
         render_function(m.shapes) + "\n\n" + join(kernels, "\n\n") + "\n\n" + render_function(m.exec) + "\n";
}

thread_local std::string g_error;

}  // namespace

extern "C" {

/* C source for a component handle made by libi_core's i_parse / combinators.
 * Returns a malloc'd string (free with free()), or NULL with oracle_c_error(). */
__attribute__((visibility("default"))) char* oracle_emit_c(const i_component* component) {
  try {
    if (!component) throw CompileError("LowerError", "null component");
    const Lowered low = lower_component(*component->inner);
    const std::string text = render_module(lower_exec_plan_to_module(low.plan));
    char* out = (char*)malloc(text.size() + 1);
    memcpy(out, text.c_str(), text.size() + 1);
    return out;
  } catch (const CompileError& e) {
    g_error = e.debug_string();
  } catch (const std::exception& e) {
    g_error = e.what();
  }
  return nullptr;
}

__attribute__((visibility("default"))) const char* oracle_c_error(void) { return g_error.c_str(); }
}
