#include "ir/ir_mutator.h"

namespace cinn {
namespace ir {

Expr IrMutator::Mutate(const Expr& e) {
  if (!e.defined()) return e;
  return MutateChildren(e);
}

Expr IrMutator::MutateChildren(const Expr& e) {
  switch (e.node_type()) {
    case IrNodeTy::IntImm:
    case IrNodeTy::UIntImm:
    case IrNodeTy::FloatImm:
    case IrNodeTy::StringImm:
    case IrNodeTy::Var: return e;
    case IrNodeTy::Minus:
    case IrNodeTy::Not: {
      auto* op = static_cast<Unary*>(e.get());
      Expr v   = Mutate(op->v);
      if (v.get() == op->v.get()) return e;
      return e.node_type() == IrNodeTy::Minus ? MakeMinus(v) : MakeNot(v);
    }
    case IrNodeTy::Cast: {
      auto* op = e.As<Cast>();
      Expr v   = Mutate(op->v);
      if (v.get() == op->v.get()) return e;
      return MakeCast(op->type, v);
    }
    case IrNodeTy::Select: {
      auto* op = e.As<Select>();
      Expr c = Mutate(op->condition), t = Mutate(op->true_value), f = Mutate(op->false_value);
      if (c.get() == op->condition.get() && t.get() == op->true_value.get() && f.get() == op->false_value.get())
        return e;
      return MakeSelect(c, t, f);
    }
    case IrNodeTy::Load: {
      auto* op = e.As<Load>();
      Expr idx = Mutate(op->index);
      if (idx.get() == op->index.get()) return e;
      return MakeLoad(op->buffer, idx);
    }
    case IrNodeTy::Store: {
      auto* op = e.As<Store>();
      Expr v = Mutate(op->value), idx = Mutate(op->index);
      if (v.get() == op->value.get() && idx.get() == op->index.get()) return e;
      return MakeStore(op->buffer, v, idx);
    }
    case IrNodeTy::Ramp: {
      auto* op = e.As<Ramp>();
      Expr b   = Mutate(op->base);
      if (b.get() == op->base.get()) return e;
      return MakeRamp(b, op->stride, op->lanes);
    }
    case IrNodeTy::Call: {
      auto* op     = e.As<Call>();
      bool changed = false;
      std::vector<Expr> args;
      for (auto& a : op->args) {
        Expr n = Mutate(a);
        changed |= n.get() != a.get();
        args.push_back(n);
      }
      if (!changed) return e;
      Expr n = MakeCall(op->type, op->name, args, op->call_type);
      n.As<Call>()->buffer_args = op->buffer_args;
      return n;
    }
    case IrNodeTy::Let: {
      auto* op = e.As<Let>();
      Expr b   = Mutate(op->body);
      if (b.get() == op->body.get()) return e;
      return MakeLet(op->symbol, b);
    }
    case IrNodeTy::For: {
      auto* op = e.As<For>();
      Expr mn = Mutate(op->min), ext = Mutate(op->extent), body = Mutate(op->body);
      if (mn.get() == op->min.get() && ext.get() == op->extent.get() && body.get() == op->body.get()) return e;
      return MakeFor(op->loop_var, mn, ext, op->for_type, body, op->bind_info);
    }
    case IrNodeTy::IfThenElse: {
      auto* op = e.As<IfThenElse>();
      Expr c = Mutate(op->condition), t = Mutate(op->true_case), f = Mutate(op->false_case);
      if (c.get() == op->condition.get() && t.get() == op->true_case.get() && f.get() == op->false_case.get())
        return e;
      return MakeIf(c, t, f);
    }
    case IrNodeTy::Block: {
      auto* op     = e.As<Block>();
      bool changed = false;
      std::vector<Expr> stmts;
      for (auto& s : op->stmts) {
        Expr n = Mutate(s);
        changed |= n.get() != s.get();
        stmts.push_back(n);
      }
      if (!changed) return e;
      return MakeBlock(stmts);
    }
    default: {
      auto* op = static_cast<Binary*>(e.get());
      Expr a = Mutate(op->a), b = Mutate(op->b);
      if (a.get() == op->a.get() && b.get() == op->b.get()) return e;
      return MakeBinary(e.node_type(), a, b);
    }
  }
}

namespace {
class SubstituteMutator : public IrMutator {
 public:
  SubstituteMutator(const std::string& name, const Expr& value) : name_(name), value_(value) {}
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    if (auto* v = e.As<Var>()) {
      if (v->name == name_) return value_.type() == v->type ? value_ : MakeCast(v->type, value_);
      return e;
    }
    return MutateChildren(e);
  }

 private:
  const std::string& name_;
  const Expr& value_;
};

class WalkMutator : public IrMutator {
 public:
  explicit WalkMutator(const std::function<void(const Expr&)>& fn) : fn_(fn) {}
  Expr Mutate(const Expr& e) override {
    if (!e.defined()) return e;
    fn_(e);
    return MutateChildren(e);
  }

 private:
  const std::function<void(const Expr&)>& fn_;
};
}  // namespace

Expr Substitute(const Expr& e, const std::string& name, const Expr& value) {
  SubstituteMutator m(name, value);
  return m.Mutate(e);
}

void Walk(const Expr& e, const std::function<void(const Expr&)>& fn) {
  WalkMutator m(fn);
  m.Mutate(e);
}

bool UsesVar(const Expr& e, const std::string& name) {
  bool found = false;
  Walk(e, [&](const Expr& n) {
    if (auto* v = n.As<Var>())
      if (v->name == name) found = true;
  });
  return found;
}

}  // namespace ir
}  // namespace cinn
