#include "ir/ir_printer.h"

#include <cmath>
#include <iomanip>
#include <limits>

namespace cinn {
namespace ir {

std::string IrPrinter::Print(const Expr& e) {
  os_.str("");
  if (!e.defined()) return "<null>";
  if (IsStmt(e)) {
    PrintStmt(e);
  } else {
    Visit(e);
  }
  return os_.str();
}

bool IrPrinter::IsStmt(const Expr& e) {
  switch (e.node_type()) {
    case IrNodeTy::Store:
    case IrNodeTy::Let:
    case IrNodeTy::For:
    case IrNodeTy::IfThenElse:
    case IrNodeTy::Block: return true;
    default: return false;
  }
}

void IrPrinter::Indent() {
  for (int i = 0; i < indent_; ++i) os_ << "  ";
}

void IrPrinter::PrintStmt(const Expr& e) {
  if (auto* b = e.As<Block>()) {
    for (auto& s : b->stmts) PrintStmt(s);
    return;
  }
  Indent();
  Visit(e);
  switch (e.node_type()) {
    case IrNodeTy::For:
    case IrNodeTy::IfThenElse: os_ << "\n"; break;
    default: os_ << ";\n";
  }
}

void IrPrinter::PrintBody(const Expr& body) {
  os_ << "{\n";
  ++indent_;
  PrintStmt(body);
  --indent_;
  Indent();
  os_ << "}";
}

void IrPrinter::Visit(const Expr& e) {
  CINN_CHECK(e.defined()) << "printing an undefined expression";
  switch (e.node_type()) {
    case IrNodeTy::IntImm:
    case IrNodeTy::UIntImm:
    case IrNodeTy::FloatImm:
    case IrNodeTy::StringImm: VisitImm(e); break;
    case IrNodeTy::Var: VisitVar(static_cast<const Var*>(e.get())); break;
    case IrNodeTy::Minus:
    case IrNodeTy::Not: VisitUnary(static_cast<const Unary*>(e.get())); break;
    case IrNodeTy::Cast: VisitCast(static_cast<const Cast*>(e.get())); break;
    case IrNodeTy::Select: VisitSelect(static_cast<const Select*>(e.get())); break;
    case IrNodeTy::Load: VisitLoad(static_cast<const Load*>(e.get())); break;
    case IrNodeTy::Store: VisitStore(static_cast<const Store*>(e.get())); break;
    case IrNodeTy::Ramp: VisitRamp(static_cast<const Ramp*>(e.get())); break;
    case IrNodeTy::Call: VisitCall(static_cast<const Call*>(e.get())); break;
    case IrNodeTy::Let: VisitLet(static_cast<const Let*>(e.get())); break;
    case IrNodeTy::For: VisitFor(static_cast<const For*>(e.get())); break;
    case IrNodeTy::IfThenElse: VisitIf(static_cast<const IfThenElse*>(e.get())); break;
    case IrNodeTy::Block: VisitBlock(static_cast<const Block*>(e.get())); break;
    default: VisitBinary(static_cast<const Binary*>(e.get()));
  }
}

void IrPrinter::VisitImm(const Expr& e) {
  if (auto* i = e.As<IntImm>()) {
    if (i->type.bits == 64) {
      os_ << i->value << "ll";
    } else if (i->type.bits == 32) {
      if (i->value == std::numeric_limits<int32_t>::min()) {
        os_ << "(-2147483647 - 1)";
      } else {
        os_ << i->value;
      }
    } else {
      os_ << "(" << common::TypeCName(i->type) << ")" << i->value;
    }
  } else if (auto* u = e.As<UIntImm>()) {
    if (u->type.is_bool()) {
      os_ << (u->value ? "true" : "false");
    } else if (u->type.bits == 64) {
      os_ << u->value << "ull";
    } else if (u->type.bits == 32) {
      os_ << u->value << "u";
    } else {
      os_ << "(" << common::TypeCName(u->type) << ")" << u->value;
    }
  } else if (auto* f = e.As<FloatImm>()) {
    double v = f->value;
    std::ostringstream s;
    auto print_special = [&](const char* suffix) -> bool {
      if (std::isnan(v)) {
        s << "__builtin_nan" << suffix << "(\"\")";
        return true;
      }
      if (std::isinf(v)) {
        s << (v < 0 ? "-" : "") << "__builtin_inf" << suffix << "()";
        return true;
      }
      return false;
    };
    if (f->type.is_float(64)) {
      if (!print_special("")) {
        s << std::setprecision(std::numeric_limits<double>::max_digits10) << v;
        std::string str = s.str();
        if (str.find('.') == std::string::npos && str.find('e') == std::string::npos) s << ".0";
      }
      os_ << s.str();
    } else {
      if (!print_special("f")) {
        s << std::setprecision(std::numeric_limits<float>::max_digits10) << static_cast<float>(v);
        std::string str = s.str();
        if (str.find('.') == std::string::npos && str.find('e') == std::string::npos) s << ".0";
        s << "f";
      }
      if (f->type.is_float(32)) {
        os_ << s.str();
      } else {
        os_ << "(" << common::TypeCName(f->type) << ")" << s.str();
      }
    }
  } else if (auto* st = e.As<StringImm>()) {
    os_ << "\"" << st->value << "\"";
  }
}

void IrPrinter::VisitVar(const Var* op) { os_ << op->name; }

void IrPrinter::VisitBinary(const Binary* op) {
  const char* sym = nullptr;
  switch (op->node_type) {
    case IrNodeTy::Add: sym = "+"; break;
    case IrNodeTy::Sub: sym = "-"; break;
    case IrNodeTy::Mul: sym = "*"; break;
    case IrNodeTy::Div: sym = "/"; break;
    case IrNodeTy::Mod: sym = "%"; break;
    case IrNodeTy::EQ: sym = "=="; break;
    case IrNodeTy::NE: sym = "!="; break;
    case IrNodeTy::LT: sym = "<"; break;
    case IrNodeTy::LE: sym = "<="; break;
    case IrNodeTy::GT: sym = ">"; break;
    case IrNodeTy::GE: sym = ">="; break;
    case IrNodeTy::And: sym = "&&"; break;
    case IrNodeTy::Or: sym = "||"; break;
    case IrNodeTy::Min:
      os_ << "min(";
      Visit(op->a);
      os_ << ", ";
      Visit(op->b);
      os_ << ")";
      return;
    case IrNodeTy::Max:
      os_ << "max(";
      Visit(op->a);
      os_ << ", ";
      Visit(op->b);
      os_ << ")";
      return;
    default: CINN_CHECK(false) << "not a binary node";
  }
  os_ << "(";
  Visit(op->a);
  os_ << " " << sym << " ";
  Visit(op->b);
  os_ << ")";
}

void IrPrinter::VisitUnary(const Unary* op) {
  os_ << (op->node_type == IrNodeTy::Minus ? "(-" : "(!");
  Visit(op->v);
  os_ << ")";
}

void IrPrinter::VisitCast(const Cast* op) {
  os_ << "((" << common::TypeCName(op->type) << ")(";
  Visit(op->v);
  os_ << "))";
}

void IrPrinter::VisitSelect(const Select* op) {
  os_ << "((";
  Visit(op->condition);
  os_ << ") ? ";
  Visit(op->true_value);
  os_ << " : ";
  Visit(op->false_value);
  os_ << ")";
}

void IrPrinter::VisitLoad(const Load* op) {
  os_ << op->buffer->name << "[";
  Visit(op->index);
  os_ << "]";
}

void IrPrinter::VisitStore(const Store* op) {
  os_ << op->buffer->name << "[";
  Visit(op->index);
  os_ << "] = ";
  Visit(op->value);
}

void IrPrinter::VisitRamp(const Ramp* op) {
  os_ << "ramp(";
  Visit(op->base);
  os_ << ", " << op->stride << ", " << op->lanes << ")";
}

void IrPrinter::VisitCall(const Call* op) {
  os_ << op->name << "(";
  bool first = true;
  for (auto& b : op->buffer_args) {
    if (!first) os_ << ", ";
    os_ << b->name;
    first = false;
  }
  for (auto& a : op->args) {
    if (!first) os_ << ", ";
    Visit(a);
    first = false;
  }
  os_ << ")";
}

void IrPrinter::VisitLet(const Let* op) {
  os_ << common::TypeCName(op->type) << " ";
  Visit(op->symbol);
  if (op->body.defined()) {
    os_ << " = ";
    Visit(op->body);
  }
}

void IrPrinter::VisitFor(const For* op) {
  if (op->bind_info.valid()) {
    os_ << "/* bound to " << (op->bind_info.for_type == ForType::GPUBlock ? "blockIdx." : "threadIdx.")
        << "xyz"[op->bind_info.offset] << " */ ";
  }
  os_ << "for (" << common::TypeCName(op->loop_var.type()) << " ";
  Visit(op->loop_var);
  os_ << " = ";
  Visit(op->min);
  os_ << "; ";
  Visit(op->loop_var);
  os_ << " < ";
  Visit(op->min + op->extent);
  os_ << "; ";
  Visit(op->loop_var);
  os_ << " += 1) ";
  PrintBody(op->body);
}

void IrPrinter::VisitIf(const IfThenElse* op) {
  os_ << "if (";
  Visit(op->condition);
  os_ << ") ";
  PrintBody(op->true_case);
  if (op->false_case.defined()) {
    os_ << " else ";
    PrintBody(op->false_case);
  }
}

void IrPrinter::VisitBlock(const Block* op) {
  // reached only for a Block nested as an expression operand, which the IR never builds
  for (auto& s : op->stmts) PrintStmt(s);
}

}  // namespace ir
}  // namespace cinn
