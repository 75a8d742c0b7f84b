#include "optim/optimize.h"

#include <algorithm>
#include <map>
#include <set>
#include <vector>

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

// ---- temporaries: axes and sizes ----------------------------------------------------------------------------------
struct LoopInfo {
  const For* loop;
  std::string var;
};
struct Access {
  BufferRef buffer;
  Expr index;
  std::vector<LoopInfo> loops;  // enclosing loops, outermost first
};

// every Load / Store of a non-global buffer with the loops around it
void CollectAccesses(const Expr& e, std::vector<LoopInfo>* stack, std::vector<Access>* out) {
  if (!e.defined()) return;
  switch (e.node_type()) {
    case IrNodeTy::IntImm:
    case IrNodeTy::UIntImm:
    case IrNodeTy::FloatImm:
    case IrNodeTy::StringImm:
    case IrNodeTy::Var: return;
    case IrNodeTy::Minus:
    case IrNodeTy::Not: CollectAccesses(static_cast<Unary*>(e.get())->v, stack, out); return;
    case IrNodeTy::Cast: CollectAccesses(e.As<Cast>()->v, stack, out); return;
    case IrNodeTy::Select: {
      auto* op = e.As<Select>();
      CollectAccesses(op->condition, stack, out);
      CollectAccesses(op->true_value, stack, out);
      CollectAccesses(op->false_value, stack, out);
      return;
    }
    case IrNodeTy::Load: {
      auto* op = e.As<Load>();
      if (op->buffer->memory_type != MemoryType::Global) out->push_back({op->buffer, op->index, *stack});
      CollectAccesses(op->index, stack, out);
      return;
    }
    case IrNodeTy::Store: {
      auto* op = e.As<Store>();
      if (op->buffer->memory_type != MemoryType::Global) out->push_back({op->buffer, op->index, *stack});
      CollectAccesses(op->value, stack, out);
      CollectAccesses(op->index, stack, out);
      return;
    }
    case IrNodeTy::Ramp: CollectAccesses(e.As<Ramp>()->base, stack, out); return;
    case IrNodeTy::Call:
      for (auto& a : e.As<Call>()->args) CollectAccesses(a, stack, out);
      return;
    case IrNodeTy::Let: CollectAccesses(e.As<Let>()->body, stack, out); return;
    case IrNodeTy::For: {
      auto* op = e.As<For>();
      stack->push_back({op, op->loop_var.As<Var>()->name});
      CollectAccesses(op->body, stack, out);
      stack->pop_back();
      return;
    }
    case IrNodeTy::IfThenElse: {
      auto* op = e.As<IfThenElse>();
      CollectAccesses(op->condition, stack, out);
      CollectAccesses(op->true_case, stack, out);
      CollectAccesses(op->false_case, stack, out);
      return;
    }
    case IrNodeTy::Block:
      for (auto& st : e.As<Block>()->stmts) CollectAccesses(st, stack, out);
      return;
    default: {
      auto* op = static_cast<Binary*>(e.get());
      CollectAccesses(op->a, stack, out);
      CollectAccesses(op->b, stack, out);
    }
  }
}

// Rewrites the indices of temporaries while walking the loops: `zero[buffer]` holds the loops whose variable is to be
// dropped from that buffer's indices wherever they enclose an access.
class BufferAxisRewriter : public IrMutator {
 public:
  explicit BufferAxisRewriter(std::map<const Buffer*, std::set<const For*>> drop) : drop_(std::move(drop)) {}
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    if (auto* f = e.As<For>()) {
      stack_.push_back(f);
      Expr body = Mutate(f->body);
      stack_.pop_back();
      // a loop that runs once: its variable is its first value, everywhere (the loop stays: it is a scope for the
      // declarations inside it)
      if (f->extent.is_int_imm(1)) body = Substitute(body, f->loop_var.As<Var>()->name, f->min);
      if (body.get() == f->body.get()) return e;
      return MakeFor(f->loop_var, f->min, f->extent, f->for_type, body, f->bind_info);
    }
    if (auto* ld = e.As<Load>()) {
      Expr idx = Rewrite(ld->buffer, Mutate(ld->index));
      return idx.get() == ld->index.get() ? e : MakeLoad(ld->buffer, idx);
    }
    if (auto* st = e.As<Store>()) {
      Expr value = Mutate(st->value);
      Expr idx   = Rewrite(st->buffer, Mutate(st->index));
      if (value.get() == st->value.get() && idx.get() == st->index.get()) return e;
      return MakeStore(st->buffer, value, idx);
    }
    return MutateChildren(e);
  }

 private:
  Expr Rewrite(const BufferRef& buffer, Expr index) {
    auto it = drop_.find(buffer.get());
    if (it == drop_.end()) return index;
    for (const For* f : stack_)
      if (it->second.count(f)) index = Substitute(index, f->loop_var.As<Var>()->name, MakeIntImm(f->loop_var.type(), 0));
    return index;
  }
  std::map<const Buffer*, std::set<const For*>> drop_;
  std::vector<const For*> stack_;
};

// [lo, hi] of an integer index expression given the ranges of the loop variables; false when unknown
bool IndexRange(const Expr& e, const std::map<std::string, std::pair<int64_t, int64_t>>& vars, int64_t* lo, int64_t* hi) {
  if (auto* i = e.As<IntImm>()) {
    *lo = *hi = i->value;
    return true;
  }
  if (auto* u = e.As<UIntImm>()) {
    *lo = *hi = static_cast<int64_t>(u->value);
    return true;
  }
  if (auto* v = e.As<Var>()) {
    auto it = vars.find(v->name);
    if (it == vars.end()) return false;
    *lo = it->second.first, *hi = it->second.second;
    return true;
  }
  if (auto* c = e.As<Cast>()) return c->type.is_integer() && IndexRange(c->v, vars, lo, hi);
  if (auto* r = e.As<Ramp>()) {
    if (!IndexRange(r->base, vars, lo, hi)) return false;
    const int64_t span = static_cast<int64_t>(r->stride) * (r->lanes - 1);
    if (span >= 0) *hi += span; else *lo += span;
    return true;
  }
  switch (e.node_type()) {
    case IrNodeTy::Add:
    case IrNodeTy::Sub:
    case IrNodeTy::Mul:
    case IrNodeTy::Div:
    case IrNodeTy::Mod:
    case IrNodeTy::Min:
    case IrNodeTy::Max: break;
    default: return false;
  }
  auto* b = static_cast<Binary*>(e.get());
  int64_t al, ah, bl, bh;
  if (!IndexRange(b->a, vars, &al, &ah) || !IndexRange(b->b, vars, &bl, &bh)) return false;
  switch (e.node_type()) {
    case IrNodeTy::Add: *lo = al + bl, *hi = ah + bh; return true;
    case IrNodeTy::Sub: *lo = al - bh, *hi = ah - bl; return true;
    case IrNodeTy::Mul: {
      const int64_t c[4] = {al * bl, al * bh, ah * bl, ah * bh};
      *lo = *std::min_element(c, c + 4), *hi = *std::max_element(c, c + 4);
      return true;
    }
    case IrNodeTy::Div:
      if (bl <= 0 || al < 0) return false;  // index arithmetic divides non-negative values by positive ones
      *lo = al / bh, *hi = ah / bl;
      return true;
    case IrNodeTy::Mod:
      if (bl <= 0 || al < 0) return false;
      *lo = 0, *hi = std::min(ah, bh - 1);
      return true;
    case IrNodeTy::Min: *lo = std::min(al, bl), *hi = std::min(ah, bh); return true;
    default: *lo = std::max(al, bl), *hi = std::max(ah, bh); return true;
  }
}

// largest index each temporary is accessed with, or "unknown"
void CollectIndexBounds(const Expr& e, std::map<std::string, std::pair<int64_t, int64_t>>* vars,
                        std::map<const Buffer*, int64_t>* bound, std::set<const Buffer*>* unknown) {
  if (!e.defined()) return;
  auto access = [&](const BufferRef& buffer, const Expr& index) {
    if (buffer->memory_type == MemoryType::Global) return;
    int64_t lo, hi;
    if (!IndexRange(index, *vars, &lo, &hi) || lo < 0) {
      unknown->insert(buffer.get());
      return;
    }
    auto it = bound->find(buffer.get());
    if (it == bound->end() || it->second < hi) (*bound)[buffer.get()] = hi;
  };
  if (auto* f = e.As<For>()) {
    const std::string& name = f->loop_var.As<Var>()->name;
    const bool known        = f->min.is_constant() && f->extent.is_constant() && f->extent.as_int64() >= 1;
    if (known) (*vars)[name] = {f->min.as_int64(), f->min.as_int64() + f->extent.as_int64() - 1};
    CollectIndexBounds(f->body, vars, bound, unknown);
    vars->erase(name);
    return;
  }
  if (auto* ld = e.As<Load>()) access(ld->buffer, ld->index);
  if (auto* st = e.As<Store>()) access(st->buffer, st->index);
  // children
  switch (e.node_type()) {
    case IrNodeTy::IntImm:
    case IrNodeTy::UIntImm:
    case IrNodeTy::FloatImm:
    case IrNodeTy::StringImm:
    case IrNodeTy::Var: return;
    case IrNodeTy::Minus:
    case IrNodeTy::Not: CollectIndexBounds(static_cast<Unary*>(e.get())->v, vars, bound, unknown); return;
    case IrNodeTy::Cast: CollectIndexBounds(e.As<Cast>()->v, vars, bound, unknown); return;
    case IrNodeTy::Select: {
      auto* op = e.As<Select>();
      CollectIndexBounds(op->condition, vars, bound, unknown);
      CollectIndexBounds(op->true_value, vars, bound, unknown);
      CollectIndexBounds(op->false_value, vars, bound, unknown);
      return;
    }
    case IrNodeTy::Load: CollectIndexBounds(e.As<Load>()->index, vars, bound, unknown); return;
    case IrNodeTy::Store:
      CollectIndexBounds(e.As<Store>()->value, vars, bound, unknown);
      CollectIndexBounds(e.As<Store>()->index, vars, bound, unknown);
      return;
    case IrNodeTy::Ramp: CollectIndexBounds(e.As<Ramp>()->base, vars, bound, unknown); return;
    case IrNodeTy::Call:
      for (auto& a : e.As<Call>()->args) CollectIndexBounds(a, vars, bound, unknown);
      for (auto& b : e.As<Call>()->buffer_args) unknown->insert(b.get());  // passed whole to a device function
      return;
    case IrNodeTy::Let: CollectIndexBounds(e.As<Let>()->body, vars, bound, unknown); return;
    case IrNodeTy::IfThenElse: {
      auto* op = e.As<IfThenElse>();
      CollectIndexBounds(op->condition, vars, bound, unknown);
      CollectIndexBounds(op->true_case, vars, bound, unknown);
      CollectIndexBounds(op->false_case, vars, bound, unknown);
      return;
    }
    case IrNodeTy::Block:
      for (auto& st : e.As<Block>()->stmts) CollectIndexBounds(st, vars, bound, unknown);
      return;
    default: {
      auto* op = static_cast<Binary*>(e.get());
      CollectIndexBounds(op->a, vars, bound, unknown);
      CollectIndexBounds(op->b, vars, bound, unknown);
    }
  }
}

// index = c * var + (terms without var), c an integer constant: true and c; false when var enters in any other way
bool AffineCoefficient(const Expr& e, const std::string& var, int64_t* c) {
  if (auto* v = e.As<Var>()) {
    *c = v->name == var ? 1 : 0;
    return true;
  }
  int64_t a, b;
  switch (e.node_type()) {
    case IrNodeTy::Add:
    case IrNodeTy::Sub: {
      auto* op = static_cast<Binary*>(e.get());
      if (!AffineCoefficient(op->a, var, &a) || !AffineCoefficient(op->b, var, &b)) return false;
      *c = e.node_type() == IrNodeTy::Add ? a + b : a - b;
      return true;
    }
    case IrNodeTy::Mul: {
      auto* op = static_cast<Binary*>(e.get());
      if (!AffineCoefficient(op->a, var, &a) || !AffineCoefficient(op->b, var, &b)) return false;
      if (a == 0 && b == 0) {
        *c = 0;
        return true;
      }
      if (b == 0 && op->b.is_constant()) {
        *c = a * op->b.as_int64();
        return true;
      }
      if (a == 0 && op->a.is_constant()) {
        *c = b * op->a.as_int64();
        return true;
      }
      return false;
    }
    default:
      if (UsesVar(e, var)) return false;
      *c = 0;
      return true;
  }
}

}  // namespace

Expr UpdateBufferAxes(const Expr& body) {
  std::vector<LoopInfo> stack;
  std::vector<Access> accesses;
  CollectAccesses(body, &stack, &accesses);
  std::map<const Buffer*, std::vector<const Access*>> by_buffer;
  for (auto& a : accesses) by_buffer[a.buffer.get()].push_back(&a);

  std::map<const Buffer*, std::set<const For*>> drop;
  for (auto& kv : by_buffer) {
    const Buffer* buffer = kv.first;
    auto& uses           = kv.second;
    const bool local     = buffer->memory_type == MemoryType::GPULocal;
    // A launch axis (block; thread too for a thread's own buffer) leaves the indices when every access sits in a loop
    // bound to it and the index moves with that loop's variable by the same constant step in all of them: then two
    // accesses of one thread (block) that met in one element before still do, and no others.
    std::set<const For*> accepted;
    for (int is_thread = 0; is_thread <= (local ? 1 : 0); ++is_thread)
      for (int offset = 0; offset < 3; ++offset) {
        const ForType axis = is_thread ? ForType::GPUThread : ForType::GPUBlock;
        std::vector<const For*> loops;
        bool ok      = true;
        int64_t step = 0;
        for (const Access* use : uses) {
          const For* bound = nullptr;
          int found        = 0;
          for (auto& l : use->loops)
            if (l.loop->bind_info.valid() && l.loop->bind_info.for_type == axis && l.loop->bind_info.offset == offset) bound = l.loop, ++found;
          int64_t c = 0;
          if (found != 1 || !AffineCoefficient(use->index, bound->loop_var.As<Var>()->name, &c) || (!loops.empty() && c != step)) {
            ok = false;
            break;
          }
          step = c;
          loops.push_back(bound);
        }
        if (ok && step != 0) accepted.insert(loops.begin(), loops.end());
      }
    // A serial loop around every access of a thread's own buffer: the buffer holds what one iteration needs when the
    // index is step * var + rest with the same step everywhere and 0 <= rest < |step| (so an element belongs to one
    // iteration only); the iterations then share one slice.  Not for shared buffers: the next iteration's writes
    // would meet other threads' reads of this one where the schedule saw distinct elements and put no barrier.
    if (local) {
      std::vector<const For*> common;
      for (size_t u = 0; u < uses.size(); ++u) {
        std::vector<const For*> loops;
        for (auto& l : uses[u]->loops) loops.push_back(l.loop);
        if (u == 0) {
          common = loops;
          continue;
        }
        size_t n = 0;
        while (n < common.size() && n < loops.size() && common[n] == loops[n]) ++n;
        common.resize(n);
      }
      for (const For* f : common) {
        if (f->bind_info.valid()) continue;
        const std::string& var = f->loop_var.As<Var>()->name;
        bool ok = true;
        int64_t step = 0;
        for (size_t u = 0; u < uses.size() && ok; ++u) {
          int64_t c = 0, lo = 0, hi = 0;
          ok = AffineCoefficient(uses[u]->index, var, &c) && c != 0 && (u == 0 || c == step);
          if (!ok) break;
          step = c;
          std::map<std::string, std::pair<int64_t, int64_t>> range;
          for (auto& l : uses[u]->loops) {
            const bool gone = l.loop == f || accepted.count(l.loop);
            if (gone) {
              range[l.var] = {0, 0};
            } else if (l.loop->min.is_constant() && l.loop->extent.is_constant() && l.loop->extent.as_int64() >= 1) {
              range[l.var] = {l.loop->min.as_int64(), l.loop->min.as_int64() + l.loop->extent.as_int64() - 1};
            }
          }
          ok = IndexRange(uses[u]->index, range, &lo, &hi) && lo >= 0 && hi < (step < 0 ? -step : step);
        }
        if (ok) accepted.insert(f);
      }
    }
    if (!accepted.empty()) drop[buffer] = std::move(accepted);
  }
  BufferAxisRewriter rewriter(std::move(drop));
  return rewriter.Mutate(body);
}

void ResizeBuffersToMaxVarRange(LoweredFunc* func) {
  std::map<std::string, std::pair<int64_t, int64_t>> vars;
  std::map<const Buffer*, int64_t> bound;
  std::set<const Buffer*> unknown;
  CollectIndexBounds(func->body, &vars, &bound, &unknown);
  for (auto& buf : func->temp_bufs) {
    if (unknown.count(buf.get())) continue;
    auto it = bound.find(buf.get());
    if (it == bound.end()) continue;
    if (it->second + 1 < buf->num_elements) buf->num_elements = it->second + 1;
  }
}

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
  func->body = UpdateBufferAxes(func->body);
  ResizeBuffersToMaxVarRange(func);
  func->body = TransformGpuForloops(func->body, &func->axis_info);
  func->body = SyncThreadsDropIfThenElse(func->body);
  CINN_CHECK(func->axis_info.valid) << "kernel " << func->name << " has no loop bound to a GPU axis";
}

}  // namespace optim
}  // namespace cinn
