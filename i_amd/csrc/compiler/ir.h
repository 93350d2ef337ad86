// Intermediate representations of the 𝚒 compiler, one family per lowering level:
//
//   Expr / Component   source-shaped tree          (reference: ir/expr.rs, ir/component.rs)
//   Node, Graph<T>     canonical per-expression form, ordered dataflow graph
//                                                   (ir/node.rs, ir/graph.rs)
//   Stage              physical axes with live / pruned slots, layouts, sites
//                                                   (ir/stage.rs)
//   KernelProgram      buffers + kernels made of Loop / Init / Compute /
//                      Snapshot / Scale actions     (ir/kernel_program.rs)
//   ExecPlan           kernels bound to readonly / writeable parameters and
//                      the alloc / dispatch / free schedule (ir/exec_plan.rs)
//   Module             target-independent statement IR (ir/module.rs)
//
// The data carried is the reference's; the representation is plain C++ value
// types (tagged structs instead of enums-with-payload).
#pragma once
#include <cstddef>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace ic {

// ------------------------------------------------------------------ common
enum class Op { Add, Mul, Div, Sub, Max, Min, Pow, Log, Gt, Ge, Lt, Le, Eq, Ne, And, Or, Xor, Not };
const char* op_name(Op op);  // the variant name, as the reference's {:?} prints it

// A failure of one compiler stage.  `kind` is the reference's error type name
// ("ParseError", "LowerError"), kept so messages print the way its Debug output does.
struct CompileError : std::runtime_error {
  std::string kind;
  std::string message;
  size_t offset = 0;  // ParseError only
  CompileError(std::string kind_, std::string message_, size_t offset_ = 0)
      : std::runtime_error(message_), kind(std::move(kind_)), message(std::move(message_)), offset(offset_) {}
  std::string debug_string() const;  // `LowerError { message: "..." }`
};
[[noreturn]] void lower_error(const std::string& message);

struct ExtentKind {
  enum Kind { Semantic, Base, Split } kind = Semantic;
  std::vector<size_t> factors;  // Base: all split factors of the index
  size_t level = 0, factor = 0; // Split
  static ExtentKind semantic() { return {}; }
  static ExtentKind base(std::vector<size_t> f) { ExtentKind k; k.kind = Base; k.factors = std::move(f); return k; }
  static ExtentKind split(size_t level, size_t factor) { ExtentKind k; k.kind = Split; k.level = level; k.factor = factor; return k; }
  bool operator==(const ExtentKind& o) const {
    return kind == o.kind && factors == o.factors && level == o.level && factor == o.factor;
  }
  bool operator!=(const ExtentKind& o) const { return !(*this == o); }
  size_t split_level() const { return kind == Split ? level : 0; }
  // ordering used when the axes of one index are listed outermost first
  std::pair<size_t, size_t> order() const { return kind == Split ? std::make_pair<size_t, size_t>(1, size_t(level)) : std::make_pair<size_t, size_t>(0, 0); }
  std::string debug_string() const;
};

// ------------------------------------------------------------------ expr / component
struct PermAtom {
  enum Kind { Axis, Input, Bang } kind = Axis;
  char axis = 0;
  size_t part = 0;     // number of apostrophes
  size_t operand = 0;  // Input: 0 = left, 1 = right
};

struct Expr {
  Op op = Op::Add;
  std::vector<std::vector<char>> inputs;
  std::vector<char> output;
  std::vector<std::pair<char, std::vector<size_t>>> splits;
  std::vector<PermAtom> permutation;
};

struct Component;
using ComponentPtr = std::shared_ptr<const Component>;
struct Component {
  enum Kind { Identity, Leaf, Compose, Chain, Fanout, Pair, Swap } kind = Identity;
  Expr expr;          // Leaf
  ComponentPtr a, b;  // combinators (Swap uses a)
};

// ------------------------------------------------------------------ node / graph
struct AxisLevel {
  size_t index = 0, level = 0;
  bool operator==(const AxisLevel& o) const { return index == o.index && level == o.level; }
};
struct NodeSite {
  bool root = true;
  AxisLevel at;
  bool operator==(const NodeSite& o) const { return root == o.root && (root || at == o.at); }
};
struct Node {
  Op op = Op::Add;
  size_t rank = 0;
  std::vector<std::vector<size_t>> inputs;  // index lists
  std::vector<size_t> output;
  std::vector<std::vector<size_t>> splits;  // per index
  std::vector<AxisLevel> order;
  std::vector<std::optional<NodeSite>> compute_sites;
  std::optional<NodeSite> init_site;
};

struct Source {
  bool is_input = true;
  size_t id = 0;      // input id or node id
  size_t output = 0;  // node output (always 0 for expression nodes)
  static Source input(size_t i) { return {true, i, 0}; }
  static Source node(size_t n, size_t o = 0) { return {false, n, o}; }
  bool operator==(const Source& o) const { return is_input == o.is_input && id == o.id && (is_input || output == o.output); }
  bool operator!=(const Source& o) const { return !(*this == o); }
};
template <class T>
struct GNode {
  T inner;
  std::vector<Source> inputs;
  size_t outputs = 1;
};
template <class T>
struct Graph {
  size_t inputs = 0;
  std::vector<GNode<T>> nodes;
  std::vector<Source> outputs;
};

// ------------------------------------------------------------------ stage
struct SAxisRef {
  bool consumer = false;  // false: local axis of the same stage
  size_t axis = 0;
  bool operator==(const SAxisRef& o) const { return consumer == o.consumer && axis == o.axis; }
};
struct SAxis {
  bool pruned = false;
  size_t index = 0;
  ExtentKind kind;
  SAxisRef by;  // pruned only
  bool operator==(const SAxis& o) const {
    return pruned == o.pruned && index == o.index && kind == o.kind && (!pruned || by == o.by);
  }
};
struct LayoutDim {
  bool semantic = false;
  SAxisRef phys;               // physical
  size_t index = 0;            // semantic
  std::vector<SAxisRef> axes;  // semantic, outermost first
  bool operator==(const LayoutDim& o) const {
    return semantic == o.semantic && (semantic ? (index == o.index && axes == o.axes) : phys == o.phys);
  }
};
using Layout = std::vector<LayoutDim>;
struct SSite {
  bool root = true;
  size_t axis = 0;
  bool operator==(const SSite& o) const { return root == o.root && (root || axis == o.axis); }
};
struct StageBuf {  // output (site = init) or input (site = compute)
  std::vector<size_t> shape;
  Layout layout;
  std::optional<SSite> site;
  bool operator==(const StageBuf& o) const { return shape == o.shape && layout == o.layout && site == o.site; }
};
struct Stage {
  Op op = Op::Add;
  std::vector<SAxis> axes;
  StageBuf output;
  std::vector<StageBuf> inputs;
  bool operator==(const Stage& o) const { return op == o.op && axes == o.axes && output == o.output && inputs == o.inputs; }
};
struct ShapeDim {
  size_t input = 0, dim = 0;
};
using ProgramShape = std::vector<ShapeDim>;
struct StageProgram {
  std::vector<ProgramShape> input_shapes, node_shapes;
  Graph<Stage> graph;
};

// ------------------------------------------------------------------ kernel program
template <class B>
struct DimRef {
  B buffer{};
  size_t dim = 0;
  bool operator==(const DimRef& o) const { return buffer == o.buffer && dim == o.dim; }
};
template <class B>
struct Extent {
  DimRef<B> source;
  ExtentKind kind;
};
struct Iter {
  bool raw = true;
  size_t loop = 0;              // raw
  std::vector<size_t> loops;    // reconstructed
  std::vector<size_t> factors;  // reconstructed
};
template <class B>
struct Access {
  B buffer{};
  std::vector<Iter> index;
};
template <class B>
struct ScalarExpr {
  enum Kind { Acc, Unary, Binary } kind = Acc;
  Access<B> access;
  Op op = Op::Add;
  std::vector<ScalarExpr<B>> args;  // 1 (unary) or 2 (binary)
};
template <class B>
struct Action {
  enum Kind { Loop, Init, Compute, Snapshot, Scale } kind = Compute;
  // Loop
  size_t id = 0;
  Extent<B> extent;
  bool guard = false;
  std::vector<Action<B>> body;
  // Init / Compute
  Op op = Op::Add;
  Access<B> write;
  std::vector<size_t> zero_checks;
  std::vector<Access<B>> reads;  // Compute reads; Snapshot: reads[0]
  // Scale
  ScalarExpr<B> factor;
};
template <class B>
using Block = std::vector<Action<B>>;
template <class B>
struct Kernel {
  std::vector<B> reads, writes;
  Block<B> body;
  // Buffers whose Computes accumulate (`dst = op(dst, reads...)`) although this body holds no Init of them: a
  // backend that cuts a kernel's body into several kernels keeps the form of each Compute this way.  Empty in
  // every plan the lowering passes produce.
  std::vector<B> accumulates;
};
enum class BufferKind { Input, Intermediate, Output };
struct Buffer {
  BufferKind kind = BufferKind::Intermediate;
  std::vector<DimRef<size_t>> shape;
  std::vector<Extent<size_t>> layout;
};
struct KernelProgram {
  std::vector<Buffer> buffers;
  std::vector<size_t> outputs;
  Graph<Kernel<size_t>> graph;
};

// ------------------------------------------------------------------ exec plan
struct Param {
  bool writeable = false;
  size_t ind = 0;
  bool operator==(const Param& o) const { return writeable == o.writeable && ind == o.ind; }
  bool operator<(const Param& o) const { return writeable != o.writeable ? !writeable : ind < o.ind; }
};
struct BufferRef {
  enum Kind { Input, Intermediate, Output } kind = Input;
  size_t id = 0;
};
struct PlanBuffer {
  std::vector<DimRef<size_t>> shape;  // dims of program inputs
  std::vector<Extent<size_t>> layout;
};
struct Step {
  enum Kind { Alloc, Dispatch, Free } kind = Alloc;
  size_t id = 0;  // intermediate or kernel
  std::vector<BufferRef> reads, writes;
};
struct ExecPlan {
  std::vector<Kernel<Param>> kernels;
  std::vector<PlanBuffer> inputs, intermediates, outputs;
  size_t count = 0;
  std::vector<size_t> ranks;
  std::vector<std::vector<DimRef<size_t>>> shapes;
  std::vector<Step> exec;
};

// ------------------------------------------------------------------ module
struct MExpr;
using MExprPtr = std::shared_ptr<const MExpr>;
enum class MField { Data, Shape, Layout, Rank };
enum class MCast { View, ViewMut, ReadOnly };
struct MExpr {
  enum Kind { Usize, Scalar, Ident, Index, Field, Cast, OpCall, Add, Sub, Mul, Div, Rem, Lt, Eq, And } kind = Usize;
  size_t usize = 0;
  float scalar = 0.0f;
  std::string ident;
  MField field = MField::Data;
  MCast cast = MCast::View;
  Op op = Op::Add;
  std::vector<MExprPtr> args;  // Index: base, index; Field/Cast: base; binary: lhs, rhs; OpCall: operands
};
enum class MType { Usize, Scalar, Tensor, TensorMut, View, ViewMut };
struct MStmt {
  enum Kind { Let, Set, Alloc, Free, Dispatch, Loop, If, Return } kind = Return;
  std::string ident;  // Let name, Alloc dst, Free name, Dispatch kernel, Loop iter
  MType type = MType::Usize;
  MExprPtr value;     // Let value, Set value, Loop bound, If cond, Return value (may be null)
  MExprPtr dst;       // Set destination (a place: ident / index / field chain)
  std::vector<MExprPtr> shape, layout;    // Alloc
  std::vector<std::string> reads, writes; // Dispatch
  std::vector<MStmt> body;                // Loop, If
};
enum class MSignature { Count, Ranks, Shapes, Exec, Kernel };
struct MFn {
  std::string ident;
  MSignature signature = MSignature::Kernel;
  std::vector<MStmt> body;
};
struct Module {
  MFn count, ranks, shapes, exec;
  std::vector<MFn> kernels;
};

// ------------------------------------------------------------------ passes
Expr parse_expr(const std::string& src);                                  // front/parser.rs
void validate_component(const Component& component);                      // check/component.rs
Node lower_expr_to_node(const Expr& expr);                                // lower/expr_to_node.rs (unchecked form)
Graph<Node> lower_component_to_graph(const Component& component);         // lower/component_to_graph.rs
StageProgram lower_graph_to_stages(const Graph<Node>& graph);             // lower/node_to_stage.rs
KernelProgram lower_stages_to_kernels(const StageProgram& program);       // lower/stage_to_kernel_program.rs
ExecPlan lower_kernels_to_exec_plan(const KernelProgram& program);        // lower/kernel_program_to_exec_plan.rs
Module lower_exec_plan_to_module(const ExecPlan& plan);                   // lower/exec_plan_to_module.rs

// Everything from a component down to the exec plan, keeping the intermediate levels.
struct Lowered {
  Graph<Node> graph;
  StageProgram stages;
  KernelProgram kernels;
  ExecPlan plan;
};
Lowered lower_component(const Component& component);

}  // namespace ic
