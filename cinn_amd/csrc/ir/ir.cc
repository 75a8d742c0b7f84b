#include "ir/ir.h"

#include <cmath>

#include "ir/ir_printer.h"

namespace cinn {
namespace ir {

Expr::Expr(int v) : p_(std::make_shared<IntImm>(common::Int(32), v)) {}
Expr::Expr(int64_t v) : p_(std::make_shared<IntImm>(common::Int(64), v)) {}
Expr::Expr(float v) : p_(std::make_shared<FloatImm>(common::Float(32), v)) {}
Expr::Expr(double v) : p_(std::make_shared<FloatImm>(common::Float(64), v)) {}
Expr::Expr(bool v) : p_(std::make_shared<UIntImm>(common::Bool(), v ? 1 : 0)) {}

bool Expr::is_constant() const {
  if (!p_) return false;
  return p_->node_type == IrNodeTy::IntImm || p_->node_type == IrNodeTy::UIntImm || p_->node_type == IrNodeTy::FloatImm;
}
int64_t Expr::as_int64() const {
  if (auto* i = As<IntImm>()) return i->value;
  if (auto* u = As<UIntImm>()) return static_cast<int64_t>(u->value);
  CINN_CHECK(false) << "expression is not an integer immediate: " << ToString(*this);
  return 0;
}
bool Expr::is_int_imm(int64_t v) const {
  if (auto* i = As<IntImm>()) return i->value == v;
  if (auto* u = As<UIntImm>()) return static_cast<int64_t>(u->value) == v;
  return false;
}

Load::Load(BufferRef b, Expr idx) : IrNode(kNodeTy, Type()), buffer(std::move(b)), index(std::move(idx)) {
  int lanes = 1;
  if (auto* r = index.As<Ramp>()) lanes = r->lanes;
  type = buffer->dtype.with_lanes(lanes);
}

std::string Argument::name() const {
  if (buffer) return buffer->name;
  return var.As<Var>()->name;
}

Expr MakeIntImm(Type t, int64_t v) {
  if (t.code == Type::Code::UInt) return Expr(std::make_shared<UIntImm>(t, static_cast<uint64_t>(v)));
  return Expr(std::make_shared<IntImm>(t, v));
}
Expr MakeFloatImm(Type t, double v) { return Expr(std::make_shared<FloatImm>(t, v)); }
Expr MakeConst(Type t, double v) {
  if (t.is_floating()) return MakeFloatImm(t, v);
  if (t.is_bool()) return Expr(std::make_shared<UIntImm>(t, v != 0 ? 1 : 0));
  return MakeIntImm(t, static_cast<int64_t>(v));
}
Expr MakeVar(const std::string& name, Type t) { return Expr(std::make_shared<Var>(name, t)); }

namespace {
bool IsCompare(IrNodeTy op) {
  return op == IrNodeTy::EQ || op == IrNodeTy::NE || op == IrNodeTy::LT || op == IrNodeTy::LE || op == IrNodeTy::GT ||
         op == IrNodeTy::GE;
}
bool IsLogical(IrNodeTy op) { return op == IrNodeTy::And || op == IrNodeTy::Or; }

// Python-style floor semantics are NOT applied here: Div/Mod on integers mean C truncation, which is
// what index arithmetic on non-negative values needs.
bool FoldInt(IrNodeTy op, int64_t a, int64_t b, int64_t* out) {
  switch (op) {
    case IrNodeTy::Add: *out = a + b; return true;
    case IrNodeTy::Sub: *out = a - b; return true;
    case IrNodeTy::Mul: *out = a * b; return true;
    case IrNodeTy::Div:
      if (b == 0) return false;
      *out = a / b;
      return true;
    case IrNodeTy::Mod:
      if (b == 0) return false;
      *out = a % b;
      return true;
    case IrNodeTy::Min: *out = a < b ? a : b; return true;
    case IrNodeTy::Max: *out = a > b ? a : b; return true;
    default: return false;
  }
}
}  // namespace

Expr MakeBinary(IrNodeTy op, Expr a, Expr b) {
  CINN_CHECK(a.defined() && b.defined());
  // unify int immediates with the other operand's type (int32 literal next to an int64 / float value)
  if (a.type() != b.type()) {
    if (b.is_constant() && !a.is_constant()) {
      b = MakeCast(a.type(), b);
    } else if (a.is_constant() && !b.is_constant()) {
      a = MakeCast(b.type(), a);
    }
  }
  if (!IsLogical(op)) {
    CINN_CHECK(a.type() == b.type()) << "binary operands differ in type: " << common::Type2Str(a.type()) << " vs "
                                     << common::Type2Str(b.type()) << " in " << ToString(a) << " , " << ToString(b);
  }
  Type rt = (IsCompare(op) || IsLogical(op)) ? common::Bool(a.type().lanes) : a.type();

  // integer folding and identities (index arithmetic)
  if (a.type().is_integer() && !IsCompare(op) && !IsLogical(op)) {
    auto* ia = a.As<IntImm>();
    auto* ib = b.As<IntImm>();
    if (ia && ib) {
      int64_t r;
      if (FoldInt(op, ia->value, ib->value, &r)) return MakeIntImm(a.type(), r);
    }
    if (op == IrNodeTy::Add) {
      if (a.is_int_imm(0)) return b;
      if (b.is_int_imm(0)) return a;
    } else if (op == IrNodeTy::Sub) {
      if (b.is_int_imm(0)) return a;
    } else if (op == IrNodeTy::Mul) {
      if (a.is_int_imm(1)) return b;
      if (b.is_int_imm(1)) return a;
      if (a.is_int_imm(0) || b.is_int_imm(0)) return MakeIntImm(a.type(), 0);
    } else if (op == IrNodeTy::Div) {
      if (b.is_int_imm(1)) return a;
    } else if (op == IrNodeTy::Mod) {
      if (b.is_int_imm(1)) return MakeIntImm(a.type(), 0);
    }
  }
  return Expr(std::make_shared<Binary>(op, rt, std::move(a), std::move(b)));
}

Expr MakeCast(Type t, Expr v) {
  if (v.type() == t) return v;
  if (auto* i = v.As<IntImm>()) {
    if (t.is_floating()) return MakeFloatImm(t, static_cast<double>(i->value));
    if (t.is_bool()) return Expr(std::make_shared<UIntImm>(t, i->value != 0));
    if (t.is_integer()) return MakeIntImm(t, i->value);
  }
  if (auto* f = v.As<FloatImm>()) {
    if (t.is_floating()) {
      double val = f->value;
      if (t.is_float(32)) val = static_cast<double>(static_cast<float>(val));
      return MakeFloatImm(t, val);
    }
  }
  return Expr(std::make_shared<Cast>(t, std::move(v)));
}

Expr MakeSelect(Expr c, Expr t, Expr f) {
  CINN_CHECK(t.type() == f.type()) << "select branches differ in type";
  return Expr(std::make_shared<Select>(std::move(c), std::move(t), std::move(f)));
}
Expr MakeLoad(const BufferRef& b, Expr index) { return Expr(std::make_shared<Load>(b, std::move(index))); }
Expr MakeStore(const BufferRef& b, Expr value, Expr index) {
  CINN_CHECK(value.type().ElementOf() == b->dtype.ElementOf())
      << "store of " << common::Type2Str(value.type()) << " into buffer " << b->name << " of "
      << common::Type2Str(b->dtype);
  return Expr(std::make_shared<Store>(b, std::move(value), std::move(index)));
}
Expr MakeRamp(Expr base, int stride, int lanes) { return Expr(std::make_shared<Ramp>(std::move(base), stride, lanes)); }
Expr MakeCall(Type ret, const std::string& name, std::vector<Expr> args, CallType ct) {
  return Expr(std::make_shared<Call>(ret, name, std::move(args), ct));
}
Expr MakeLet(Expr var, Expr value) { return Expr(std::make_shared<Let>(std::move(var), std::move(value))); }
Expr MakeFor(Expr var, Expr min, Expr extent, ForType ft, Expr body, BindInfo bi) {
  return Expr(std::make_shared<For>(std::move(var), std::move(min), std::move(extent), ft, std::move(body), bi));
}
Expr MakeIf(Expr cond, Expr then_case, Expr else_case) {
  return Expr(std::make_shared<IfThenElse>(std::move(cond), std::move(then_case), std::move(else_case)));
}
Expr MakeBlock(std::vector<Expr> stmts) { return Expr(std::make_shared<Block>(std::move(stmts))); }
Expr MakeMinus(Expr v) {
  Type t = v.type();
  return Expr(std::make_shared<Unary>(IrNodeTy::Minus, t, std::move(v)));
}
Expr MakeNot(Expr v) {
  Type t = common::Bool(v.type().lanes);
  return Expr(std::make_shared<Unary>(IrNodeTy::Not, t, std::move(v)));
}
Expr Min(Expr a, Expr b) { return MakeBinary(IrNodeTy::Min, std::move(a), std::move(b)); }
Expr Max(Expr a, Expr b) { return MakeBinary(IrNodeTy::Max, std::move(a), std::move(b)); }

Expr operator+(Expr a, Expr b) { return MakeBinary(IrNodeTy::Add, std::move(a), std::move(b)); }
Expr operator-(Expr a, Expr b) { return MakeBinary(IrNodeTy::Sub, std::move(a), std::move(b)); }
Expr operator*(Expr a, Expr b) { return MakeBinary(IrNodeTy::Mul, std::move(a), std::move(b)); }
Expr operator/(Expr a, Expr b) { return MakeBinary(IrNodeTy::Div, std::move(a), std::move(b)); }
Expr operator%(Expr a, Expr b) { return MakeBinary(IrNodeTy::Mod, std::move(a), std::move(b)); }
Expr operator<(Expr a, Expr b) { return MakeBinary(IrNodeTy::LT, std::move(a), std::move(b)); }
Expr operator<=(Expr a, Expr b) { return MakeBinary(IrNodeTy::LE, std::move(a), std::move(b)); }
Expr operator>(Expr a, Expr b) { return MakeBinary(IrNodeTy::GT, std::move(a), std::move(b)); }
Expr operator>=(Expr a, Expr b) { return MakeBinary(IrNodeTy::GE, std::move(a), std::move(b)); }
Expr operator==(Expr a, Expr b) { return MakeBinary(IrNodeTy::EQ, std::move(a), std::move(b)); }
Expr operator!=(Expr a, Expr b) { return MakeBinary(IrNodeTy::NE, std::move(a), std::move(b)); }
Expr operator&&(Expr a, Expr b) { return MakeBinary(IrNodeTy::And, std::move(a), std::move(b)); }
Expr operator||(Expr a, Expr b) { return MakeBinary(IrNodeTy::Or, std::move(a), std::move(b)); }

std::string ToString(const Expr& e) {
  IrPrinter printer;
  return printer.Print(e);
}

}  // namespace ir
}  // namespace cinn
