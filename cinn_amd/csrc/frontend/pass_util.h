// Helper shared by the program passes: emits instructions with inferred output shapes and types.
#pragma once
#include <string>
#include <utility>
#include <vector>

#include "frontend/syntax.h"
#include "hlir/op.h"

namespace cinn {
namespace frontend {

// Builds instructions with inferred output shapes; new variables are named <prefix><n>.
class Emitter {
 public:
  Emitter(std::vector<Instruction>* out, std::string prefix) : out_(out), prefix_(std::move(prefix)) {}

  std::vector<Variable> Emit(const std::string& type, const std::vector<Variable>& inputs,
                             const utils::AttributeMap& attrs) {
    const auto& op = hlir::framework::OpRegistry::Global().Get(type);
    Instruction instr(type);
    instr->inputs = inputs;
    instr->attrs  = attrs;
    std::vector<utils::ShapeType> shapes;
    std::vector<common::Type> types;
    for (auto& in : inputs) {
      shapes.push_back(in->shape);
      types.push_back(in->type);
    }
    auto out_shapes = op.infer_shape(shapes, attrs);
    auto out_types  = op.infer_dtype(types, attrs);
    for (size_t i = 0; i < out_shapes.size(); ++i) {
      Variable v(prefix_ + std::to_string(counter_++));
      v->shape = out_shapes[i];
      v->type  = out_types[i];
      instr->outputs.push_back(v);
    }
    out_->push_back(instr);
    return instr->outputs;
  }
  Variable Emit1(const std::string& type, const std::vector<Variable>& inputs, const utils::AttributeMap& attrs) {
    return Emit(type, inputs, attrs).front();
  }
  // same, but the result is the existing variable `result` (keeps its id for the consumers that follow)
  void EmitInto(const Variable& result, const std::string& type, const std::vector<Variable>& inputs,
                const utils::AttributeMap& attrs) {
    Instruction instr(type);
    instr->inputs  = inputs;
    instr->attrs   = attrs;
    instr->outputs = {result};
    out_->push_back(instr);
  }

 private:
  std::vector<Instruction>* out_;
  std::string prefix_;
  int counter_{0};
};

}  // namespace frontend
}  // namespace cinn
