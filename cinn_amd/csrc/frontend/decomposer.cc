#include "frontend/decomposer.h"

#include <algorithm>

#include "frontend/net_builder.h"
#include "hlir/op.h"

namespace cinn {
namespace frontend {

namespace {

// A NetBuilder whose temporaries get ids that cannot collide with the user's.
class SubBuilder : public NetBuilder {
 public:
  explicit SubBuilder(int serial) : NetBuilder("decomposer"), prefix_("dcp" + std::to_string(serial) + "_") {}
  std::vector<Instruction> TakeInstructions(const Variable& result, const Variable& origin) {
    Program p = Build();
    std::vector<Instruction> out;
    for (auto& ins : p.instructions()) {
      for (auto& o : ins->outputs) {
        if (o == result) {
          // map the result back to the variable the original instruction defined
          o->id = origin->id;
        } else if (o->id.rfind(prefix_, 0) != 0) {
          o->id = prefix_ + o->id;
        }
      }
      out.push_back(ins);
    }
    return out;
  }

 private:
  std::string prefix_;
};

void DecomposeSoftmax(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  auto x      = instr->inputs[0];
  auto output = instr->outputs[0];
  SubBuilder b(serial);
  auto axes = hlir::framework::GetAttr<std::vector<int>>(instr->attrs, "axes", {-1});
  CINN_CHECK(!axes.empty());
  int rank = static_cast<int>(x->shape.size());
  for (auto& a : axes)
    if (a < 0) a += rank;
  std::vector<int> b_axes;
  for (int i = 0; i < rank; ++i)
    if (std::find(axes.begin(), axes.end(), i) == axes.end()) b_axes.push_back(i);
  bool rank_one_fix = b_axes.empty();
  auto mode         = hlir::framework::GetAttr<std::string>(instr->attrs, "mode", "fast");

  auto bcast = [&](const Variable& reduced) {
    if (rank_one_fix) {
      // every axis is reduced: the single result is replicated everywhere
      return b.BroadcastTo(reduced, x->shape, std::vector<int>(reduced->shape.size(), rank - 1));
    }
    return b.BroadcastTo(reduced, x->shape, b_axes);
  };
  Variable result;
  if (mode == "fast") {
    auto x_sum = bcast(b.ReduceSum(b.Exp(x), axes));
    result     = b.Divide(b.Exp(x), x_sum);
  } else {
    auto x_max = bcast(b.ReduceMax(x, axes));
    auto x_exp = b.Exp(b.Subtract(x, x_max));
    auto x_sum = bcast(b.ReduceSum(x_exp, axes));
    result     = b.Divide(b.Exp(b.Subtract(x, x_max)), x_sum);
  }
  auto ins = b.TakeInstructions(result, output);
  out->insert(out->end(), ins.begin(), ins.end());
}

void DecomposeBatchNorm(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  auto x = instr->inputs[0], scale = instr->inputs[1], bias = instr->inputs[2], mean = instr->inputs[3],
       variance = instr->inputs[4];
  auto output   = instr->outputs[0];
  float epsilon = hlir::framework::GetAttr<float>(instr->attrs, "epsilon", 1e-5f);
  auto layout   = hlir::framework::GetAttr<std::string>(instr->attrs, "data_layout", "NCHW");
  CINN_CHECK(layout == "NCHW" || layout == "NHWC") << "batch_norm: unknown data_layout " << layout;
  CINN_CHECK_EQ(x->shape.size(), 4u) << "Input's dimension of BatchNorm op is not 4! Please check.";
  std::vector<int> c_axis = {layout == "NCHW" ? 1 : 3};
  SubBuilder b(serial);
  const std::string type_str = common::Type2Str(x->type);
  auto bc = [&](const Variable& v) { return b.BroadcastTo(v, x->shape, c_axis); };
  // (x - mean) * scale / sqrt(variance + eps) + bias, left to right
  auto eps    = b.FillConstant(variance->shape, epsilon, "bn_epsilon", type_str);
  auto denom  = b.Sqrt(b.Add(variance, eps));
  auto result = b.Add(b.Divide(b.Multiply(b.Subtract(x, bc(mean)), bc(scale)), bc(denom)), bc(bias));
  auto ins    = b.TakeInstructions(result, output);
  out->insert(out->end(), ins.begin(), ins.end());
}

}  // namespace

Program ApplyDecomposer(const Program& program) {
  std::vector<Instruction> out;
  int serial = 0;
  for (auto& ins : program.instructions()) {
    if (ins->op_type == "softmax") {
      DecomposeSoftmax(ins, serial++, &out);
    } else if (ins->op_type == "batch_norm") {
      DecomposeBatchNorm(ins, serial++, &out);
    } else {
      out.push_back(ins);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

}  // namespace frontend
}  // namespace cinn
