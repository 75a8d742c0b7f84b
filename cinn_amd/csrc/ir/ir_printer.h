// C-syntax printer for the IR.  It is the base of the HIP device code generator and also the
// debugging dump (ir::ToString).  Immediates follow the reference's spelling rules
// (cinn/ir/ir_printer.cc:44-100): fp32 with max_digits10 and an `f` suffix, 16-bit floats as a cast
// of an fp32 literal, int64 with an `ll` suffix.
#pragma once
#include <sstream>
#include <string>

#include "ir/ir.h"

namespace cinn {
namespace ir {

class IrPrinter {
 public:
  virtual ~IrPrinter() = default;
  std::string Print(const Expr& e);

 protected:
  virtual void Visit(const Expr& e);
  virtual void VisitImm(const Expr& e);
  virtual void VisitVar(const Var* op);
  virtual void VisitBinary(const Binary* op);
  virtual void VisitUnary(const Unary* op);
  virtual void VisitCast(const Cast* op);
  virtual void VisitSelect(const Select* op);
  virtual void VisitLoad(const Load* op);
  virtual void VisitStore(const Store* op);
  virtual void VisitRamp(const Ramp* op);
  virtual void VisitCall(const Call* op);
  virtual void VisitLet(const Let* op);
  virtual void VisitFor(const For* op);
  virtual void VisitIf(const IfThenElse* op);
  virtual void VisitBlock(const Block* op);

  // statements are printed one per line with the current indent; a Block does not add braces itself
  void PrintStmt(const Expr& e);
  void PrintBody(const Expr& body);  // "{ ... }" around a statement or block
  void Indent();
  static bool IsStmt(const Expr& e);

  std::ostringstream os_;
  int indent_{0};
};

}  // namespace ir
}  // namespace cinn
