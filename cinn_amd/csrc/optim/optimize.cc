#include "optim/optimize.h"

#include <algorithm>
#include <set>

#include "common/type.h"
#include "ir/ir_mutator.h"

namespace cinn {
namespace optim {

using namespace ir;  // NOLINT

namespace {

// index == base + var with var-free base: returns base, else an undefined Expr
Expr SplitUnitStride(const Expr& index, const std::string& var) {
  if (auto* v = index.As<Var>()) {
    if (v->name == var) return MakeIntImm(index.type(), 0);
    return Expr();
  }
  if (index.node_type() == IrNodeTy::Add) {
    auto* add = static_cast<Binary*>(index.get());
    auto* va  = add->a.As<Var>();
    auto* vb  = add->b.As<Var>();
    if (vb && vb->name == var && !UsesVar(add->a, var)) return add->a;
    if (va && va->name == var && !UsesVar(add->b, var)) return add->b;
  }
  return Expr();
}

class Vectorizer : public IrMutator {
 public:
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    auto* f = e.As<For>();
    if (!f || f->for_type != ForType::Vectorized) return MutateChildren(e);
    Expr vec = TryVectorize(f);
    if (vec.defined()) return vec;
    return MakeFor(f->loop_var, f->min, f->extent, ForType::Unrolled, Mutate(f->body));
  }

 private:
  Expr TryVectorize(const For* f) {
    if (!f->extent.is_constant() || !f->min.is_int_imm(0)) return Expr();
    int lanes = static_cast<int>(f->extent.as_int64());
    if (lanes == 1) return Substitute(f->body, f->loop_var.As<Var>()->name, MakeIntImm(f->loop_var.type(), 0));
    Expr body = f->body;
    if (auto* b = body.As<Block>()) {
      if (b->stmts.size() != 1) return Expr();
      body = b->stmts[0];
    }
    auto* st = body.As<Store>();
    if (!st) return Expr();
    auto* ld = st->value.As<Load>();
    if (!ld) return Expr();
    if (ld->buffer->dtype != st->buffer->dtype) return Expr();
    int bytes = lanes * ld->buffer->dtype.bytes();
    if (bytes > 16 || (bytes & (bytes - 1))) return Expr();
    const std::string& var = f->loop_var.As<Var>()->name;
    Expr sbase = SplitUnitStride(st->index, var);
    Expr lbase = SplitUnitStride(ld->index, var);
    if (!sbase.defined() || !lbase.defined()) return Expr();
    return MakeStore(st->buffer, MakeLoad(ld->buffer, MakeRamp(lbase, 1, lanes)), MakeRamp(sbase, 1, lanes));
  }
};

class GpuLoopBinder : public IrMutator {
 public:
  explicit GpuLoopBinder(GpuAxisInfo* info) : info_(info) {}

  // first pass: largest extent per axis
  void Collect(const Expr& body) {
    Walk(body, [&](const Expr& n) {
      auto* f = n.As<For>();
      if (!f || !f->bind_info.valid()) return;
      CINN_CHECK(f->extent.is_constant()) << "a loop bound to a GPU axis needs a constant extent";
      CINN_CHECK(f->min.is_int_imm(0)) << "a loop bound to a GPU axis must start at 0";
      int ext  = static_cast<int>(f->extent.as_int64());
      int* dim = f->bind_info.for_type == ForType::GPUBlock ? info_->grid : info_->block;
      dim[f->bind_info.offset] = std::max(dim[f->bind_info.offset], ext);
      info_->valid             = true;
    });
  }

  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    auto* f = e.As<For>();
    if (!f || !f->bind_info.valid()) return MutateChildren(e);
    bool is_block    = f->bind_info.for_type == ForType::GPUBlock;
    std::string axis = std::string(is_block ? "blockIdx." : "threadIdx.") + "xyz"[f->bind_info.offset];
    Expr axis_var    = MakeVar(axis, f->loop_var.type());
    Expr body        = Substitute(Mutate(f->body), f->loop_var.As<Var>()->name, axis_var);
    int ext          = static_cast<int>(f->extent.as_int64());
    int launched     = (is_block ? info_->grid : info_->block)[f->bind_info.offset];
    if (ext < launched) return MakeIf(axis_var < Expr(ext), body);
    return body;
  }

 private:
  GpuAxisInfo* info_;
};

// cinn/optim/map_extern_call.cc:25-40
const std::set<std::string>& FloatMathNames() {
  static const std::set<std::string> names = {
      "exp",   "erf",  "sigmoid",  "sqrt",  "log",       "log2",  "log10", "floor", "ceil",  "round", "trunc",
      "cos",   "cosh", "tan",      "sin",   "sinh",      "acos",  "acosh", "asin",  "asinh", "atan",  "atanh",
      "isnan", "tanh", "isfinite", "isinf", "remainder", "rsqrt", "cbrt",  "abs",   "pow",   "mod"};
  return names;
}
const std::set<std::string>& IntMathNames() {
  static const std::set<std::string> names = {"left_shift",  "right_shift", "bitwise_or", "bitwise_and",
                                              "bitwise_xor", "bitwise_not", "pow",        "logical_right_shift",
                                              "clz",         "popc",        "mod"};
  return names;
}

bool IsFloatConstant(const Expr& e, double value) {
  if (auto* f = e.As<FloatImm>()) return f->value == value;
  if (auto* c = e.As<Cast>()) return IsFloatConstant(c->v, value);  // a constant rounded to a 16-bit type
  return false;
}

class ExternCallMapper : public IrMutator {
 public:
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    Expr out   = MutateChildren(e);
    auto* call = out.As<Call>();
    if (!call || call->args.empty()) return out;
    std::string name        = call->name;
    std::vector<Expr> args  = call->args;
    if (name == "pow" && args.size() >= 2 && IsFloatConstant(args[1], 0.5)) {
      name = "sqrt";
      args.erase(args.begin() + 1);
    } else if (name == "pow" && args.size() >= 2 && IsFloatConstant(args[1], -0.5)) {
      name = "rsqrt";
      args.erase(args.begin() + 1);
    }
    if (!FloatMathNames().count(name) && !IntMathNames().count(name)) return out;
    const std::string library_name = "cinn_hip_" + name + "_" + common::TypeSuffix(args.front().type());
    Expr mapped                    = MakeCall(out.type(), library_name, std::move(args), call->call_type);
    mapped.As<Call>()->buffer_args = call->buffer_args;
    return mapped;
  }
};

class SyncThreadsUnguard : public IrMutator {
 public:
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    Expr out = MutateChildren(e);
    auto* br = out.As<IfThenElse>();
    if (!br || br->false_case.defined() || br->condition.node_type() != IrNodeTy::EQ) return out;
    if (!static_cast<Binary*>(br->condition.get())->b.is_int_imm(0)) return out;
    Expr body = br->true_case;
    if (auto* b = body.As<Block>()) {
      if (b->stmts.size() != 1) return out;
      body = b->stmts[0];
    }
    auto* call = body.As<Call>();
    if (call && call->name == "__syncthreads") return body;
    return out;
  }
};

}  // namespace

Expr MapExternCall(const Expr& body, const common::Target& target) {
  if (target.arch != common::Target::Arch::AMDGPU) return body;
  ExternCallMapper m;
  return m.Mutate(body);
}

Expr SyncThreadsDropIfThenElse(const Expr& body) {
  SyncThreadsUnguard m;
  return m.Mutate(body);
}

Expr VectorizeLoops(const Expr& body) {
  Vectorizer v;
  return v.Mutate(body);
}

Expr TransformGpuForloops(const Expr& body, GpuAxisInfo* axis_info) {
  GpuLoopBinder binder(axis_info);
  binder.Collect(body);
  return binder.Mutate(body);
}

void OptimizeFuncGPU(LoweredFunc* func) {
  func->body = MapExternCall(func->body, common::DefaultAMDGPUTarget());
  func->body = VectorizeLoops(func->body);
  func->body = TransformGpuForloops(func->body, &func->axis_info);
  func->body = SyncThreadsDropIfThenElse(func->body);
  CINN_CHECK(func->axis_info.valid) << "kernel " << func->name << " has no loop bound to a GPU axis";
}

}  // namespace optim
}  // namespace cinn
