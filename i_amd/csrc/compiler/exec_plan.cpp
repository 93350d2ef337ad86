// KernelProgram -> ExecPlan: classify buffers (program inputs, intermediates in
// buffer order, outputs in program-output order), bind every kernel buffer to a
// positional readonly / writeable parameter, resolve all shapes and layouts to
// dimensions of program inputs, and schedule alloc-all, dispatch in kernel
// order, free-all in reverse.  Follows
// compiler/src/lower/kernel_program_to_exec_plan.rs:15-450.
#include <algorithm>
#include <set>

#include "ir.h"

namespace ic {
namespace {

struct PlanBuilder {
  const KernelProgram& program;
  std::vector<std::optional<BufferRef>> refs;

  explicit PlanBuilder(const KernelProgram& p) : program(p), refs(p.buffers.size()) {
    size_t next_input = 0, next_intermediate = 0;
    for (size_t i = 0; i < p.buffers.size(); ++i) {
      if (p.buffers[i].kind == BufferKind::Input) refs[i] = BufferRef{BufferRef::Input, next_input++};
      else if (p.buffers[i].kind == BufferKind::Intermediate) refs[i] = BufferRef{BufferRef::Intermediate, next_intermediate++};
    }
    std::set<size_t> outs;
    for (size_t o = 0; o < p.outputs.size(); ++o) {
      const size_t buffer = p.outputs[o];
      if (buffer >= p.buffers.size())
        lower_error("output " + std::to_string(o) + " references nonexistent buffer " + std::to_string(buffer));
      if (p.buffers[buffer].kind != BufferKind::Output)
        lower_error("output " + std::to_string(o) + " references " +
                    (p.buffers[buffer].kind == BufferKind::Input ? "Input" : "Intermediate") + " buffer " + std::to_string(buffer));
      if (!outs.insert(buffer).second) lower_error("output " + std::to_string(o) + " repeats buffer " + std::to_string(buffer));
      refs[buffer] = BufferRef{BufferRef::Output, o};
    }
    for (size_t i = 0; i < p.buffers.size(); ++i)
      if (p.buffers[i].kind == BufferKind::Output && !outs.count(i))
        lower_error("output buffer " + std::to_string(i) + " is not a program output");
  }

  BufferRef ref(size_t buffer) const {
    if (buffer >= refs.size() || !refs[buffer]) lower_error("buffer " + std::to_string(buffer) + " has no exec ref");
    return *refs[buffer];
  }

  DimRef<size_t> resolve(DimRef<size_t> dim, std::vector<size_t>& stack) const {
    if (dim.buffer >= program.buffers.size()) lower_error("references nonexistent buffer " + std::to_string(dim.buffer));
    const Buffer& buffer = program.buffers[dim.buffer];
    if (dim.dim >= buffer.shape.size())
      lower_error("references nonexistent dim " + std::to_string(dim.dim) + " of buffer " + std::to_string(dim.buffer));
    const BufferRef r = ref(dim.buffer);
    if (r.kind == BufferRef::Input) return {r.id, dim.dim};
    if (std::find(stack.begin(), stack.end(), dim.buffer) != stack.end())
      lower_error("shape dim cycle through buffer " + std::to_string(dim.buffer));
    stack.push_back(dim.buffer);
    const auto out = resolve(buffer.shape[dim.dim], stack);
    stack.pop_back();
    return out;
  }

  PlanBuffer lower_buffer(size_t index) const {
    const Buffer& buffer = program.buffers[index];
    PlanBuffer out;
    for (const auto& d : buffer.shape) {
      std::vector<size_t> stack;
      out.shape.push_back(resolve(d, stack));
    }
    for (const auto& e : buffer.layout) {
      std::vector<size_t> stack;
      out.layout.push_back({resolve(e.source, stack), e.kind});
    }
    if (buffer.shape.empty() && !buffer.layout.empty())
      lower_error("buffer " + std::to_string(index) + " has scalar shape and non-scalar layout");
    return out;
  }

  static Param param(const Kernel<size_t>& k, size_t buffer) {
    auto r = std::find(k.reads.begin(), k.reads.end(), buffer);
    if (r != k.reads.end()) return {false, size_t(r - k.reads.begin())};
    auto w = std::find(k.writes.begin(), k.writes.end(), buffer);
    if (w != k.writes.end()) return {true, size_t(w - k.writes.begin())};
    lower_error("buffer " + std::to_string(buffer) + " is not a kernel parameter");
  }
  static Access<Param> access(const Kernel<size_t>& k, const Access<size_t>& a) { return {param(k, a.buffer), a.index}; }
  static ScalarExpr<Param> scalar(const Kernel<size_t>& k, const ScalarExpr<size_t>& e) {
    ScalarExpr<Param> out;
    out.kind = (ScalarExpr<Param>::Kind)e.kind;
    out.op = e.op;
    if (e.kind == ScalarExpr<size_t>::Acc) out.access = access(k, e.access);
    for (const auto& a : e.args) out.args.push_back(scalar(k, a));
    return out;
  }
  static Block<Param> block(const Kernel<size_t>& k, const Block<size_t>& in) {
    Block<Param> out;
    for (const auto& a : in) {
      Action<Param> o;
      o.kind = (Action<Param>::Kind)a.kind;
      o.id = a.id;
      o.guard = a.guard;
      o.op = a.op;
      o.zero_checks = a.zero_checks;
      switch (a.kind) {
        case Action<size_t>::Loop:
          o.extent = {{param(k, a.extent.source.buffer), a.extent.source.dim}, a.extent.kind};
          o.body = block(k, a.body);
          break;
        case Action<size_t>::Init: o.write = access(k, a.write); break;
        case Action<size_t>::Compute:
        case Action<size_t>::Snapshot:
          o.write = access(k, a.write);
          for (const auto& r : a.reads) o.reads.push_back(access(k, r));
          break;
        case Action<size_t>::Scale:
          o.write = access(k, a.write);
          o.factor = scalar(k, a.factor);
          break;
      }
      out.push_back(std::move(o));
    }
    return out;
  }
};

}  // namespace

ExecPlan lower_kernels_to_exec_plan(const KernelProgram& program) {
  PlanBuilder b(program);
  ExecPlan plan;
  plan.outputs.resize(program.outputs.size());
  for (size_t i = 0; i < program.buffers.size(); ++i) {
    const BufferRef r = b.ref(i);
    PlanBuffer pb = b.lower_buffer(i);
    if (r.kind == BufferRef::Input) plan.inputs.push_back(std::move(pb));
    else if (r.kind == BufferRef::Intermediate) plan.intermediates.push_back(std::move(pb));
    else plan.outputs[r.id] = std::move(pb);
  }
  for (const auto& o : plan.outputs) {
    plan.shapes.push_back(o.shape);
    plan.ranks.push_back(o.shape.size());
  }
  plan.count = plan.shapes.size();
  for (size_t k = 0; k < program.graph.nodes.size(); ++k) {
    const auto& kernel = program.graph.nodes[k].inner;
    Kernel<Param> out;
    for (size_t i = 0; i < kernel.reads.size(); ++i) out.reads.push_back({false, i});
    for (size_t i = 0; i < kernel.writes.size(); ++i) out.writes.push_back({true, i});
    try {
      out.body = PlanBuilder::block(kernel, kernel.body);
    } catch (const CompileError& e) {
      lower_error("kernel " + std::to_string(k) + " " + e.message);
    }
    plan.kernels.push_back(std::move(out));
  }
  const size_t n_inter = plan.intermediates.size();
  for (size_t i = 0; i < n_inter; ++i) plan.exec.push_back({Step::Alloc, i, {}, {}});
  for (size_t k = 0; k < program.graph.nodes.size(); ++k) {
    Step s;
    s.kind = Step::Dispatch;
    s.id = k;
    for (size_t buffer : program.graph.nodes[k].inner.reads) s.reads.push_back(b.ref(buffer));
    for (size_t buffer : program.graph.nodes[k].inner.writes) s.writes.push_back(b.ref(buffer));
    plan.exec.push_back(std::move(s));
  }
  for (size_t i = n_inter; i-- > 0;) plan.exec.push_back({Step::Free, i, {}, {}});
  return plan;
}

}  // namespace ic
