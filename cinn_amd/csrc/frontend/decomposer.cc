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
    return TakeInstructions(std::vector<std::pair<Variable, Variable>>{{result, origin}});
  }
  // results[i].first is mapped back to results[i].second, the variable the original instruction defined
  std::vector<Instruction> TakeInstructions(const std::vector<std::pair<Variable, Variable>>& results) {
    Program p = Build();
    std::vector<Instruction> out;
    for (auto& ins : p.instructions()) {
      for (auto& o : ins->outputs) {
        bool mapped = false;
        for (auto& r : results) {
          if (o == r.first) {
            o->id  = r.second->id;
            mapped = true;
          }
        }
        if (!mapped && o->id.rfind(prefix_, 0) != 0) o->id = prefix_ + o->id;
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

// The training form and the gradient (cinn/frontend/decomposer/batch_norm.cc:22-262): statistics over n, h, w as
// E(x) and E(x^2) - E(x)^2, y = (x - mean) * rsqrt(variance + eps) * scale + bias, moving averages
// moving * momentum + saved * (1 - momentum); 16-bit x / dy are computed in fp32 and y / x_grad cast back, the
// per-channel tensors stay fp32 (the reference's AutoCast pass, cinn/frontend/pass/auto_cast.cc:120-190).
struct BatchNormParts {
  SubBuilder* b;
  std::vector<int> x_shape, reduce_dim, c_axis;
  float element_count;
  BatchNormParts(SubBuilder* builder, const std::vector<int>& shape, const std::string& layout) : b(builder), x_shape(shape) {
    CINN_CHECK_EQ(shape.size(), 4u) << "Only 4-D input tensor is supported, but get " << shape.size() << "-D input tensor.";
    CINN_CHECK(layout == "NCHW" || layout == "NHWC") << layout << " setting is not support!";
    if (layout == "NCHW") {
      c_axis = {1}, reduce_dim = {0, 2, 3};
      element_count = static_cast<float>(shape[0] * shape[2] * shape[3]);
    } else {
      c_axis = {3}, reduce_dim = {0, 1, 2};
      element_count = static_cast<float>(shape[0] * shape[1] * shape[2]);
    }
  }
  Variable Reduce(const Variable& v) { return b->ReduceSum(v, reduce_dim); }
  Variable To4d(const Variable& v) { return b->BroadcastTo(v, x_shape, c_axis); }
  Variable Constant(const Variable& like, float value, const char* name) {
    return b->FillConstant(like->shape, value, name, common::Type2Str(like->type));
  }
  Variable Mean(const Variable& x) {
    auto sum = Reduce(x);
    return b->Divide(sum, Constant(sum, element_count, "element_count"));
  }
  Variable Variance(const Variable& x, const Variable& mean) {
    auto sq_sum  = Reduce(b->Multiply(x, b->Identity(x)));
    auto sq_mean = b->Divide(sq_sum, Constant(sq_sum, element_count, "element_count"));
    return b->Subtract(sq_mean, b->Multiply(mean, b->Identity(mean)));
  }
  Variable StdVarianceInv(const Variable& variance, float epsilon) {
    return b->Rsqrt(b->Add(variance, Constant(variance, epsilon, "epsilon")));
  }
  Variable Moving(const Variable& moving, const Variable& saved, float momentum) {
    return b->Add(b->Multiply(moving, Constant(moving, momentum, "factor_0")),
                  b->Multiply(saved, Constant(saved, 1.0f - momentum, "factor_1")));
  }
};

bool Is16Bit(const common::Type& t) { return t.is_float16() || t.is_bfloat16(); }

void DecomposeBatchNormTrain(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  CINN_CHECK_EQ(instr->inputs.size(), 5u) << "batch_norm_train takes x, scale, bias, moving_mean, moving_variance";
  CINN_CHECK_EQ(instr->outputs.size(), 5u);
  auto x = instr->inputs[0], scale = instr->inputs[1], bias = instr->inputs[2], moving_mean = instr->inputs[3],
       moving_variance = instr->inputs[4];
  float epsilon  = hlir::framework::GetAttr<float>(instr->attrs, "epsilon", 1e-5f);
  float momentum = hlir::framework::GetAttr<float>(instr->attrs, "momentum", 0.9f);
  auto layout    = hlir::framework::GetAttr<std::string>(instr->attrs, "data_layout", "NCHW");
  SubBuilder b(serial);
  BatchNormParts h(&b, x->shape, layout);
  const bool narrow = Is16Bit(x->type);
  Variable xf       = narrow ? b.Cast(x, "float32") : x;
  auto mean         = h.Mean(xf);
  auto variance     = h.Variance(xf, mean);
  // the 4-D form of rsqrt(variance + eps), as the reference builds it
  auto variance_4d  = h.To4d(variance);
  auto inv_std_4d   = b.Rsqrt(b.Add(variance_4d, h.Constant(variance_4d, epsilon, "epsilon")));
  auto normalized   = b.Multiply(b.Subtract(xf, h.To4d(mean)), inv_std_4d);
  auto y            = b.Add(b.Multiply(normalized, h.To4d(scale)), h.To4d(bias));
  if (narrow) y = b.Cast(y, common::Type2Str(x->type));
  auto new_mean     = h.Moving(moving_mean, mean, momentum);
  auto new_variance = h.Moving(moving_variance, variance, momentum);
  auto ins = b.TakeInstructions({{y, instr->outputs[0]},
                                 {mean, instr->outputs[1]},
                                 {variance, instr->outputs[2]},
                                 {new_mean, instr->outputs[3]},
                                 {new_variance, instr->outputs[4]}});
  out->insert(out->end(), ins.begin(), ins.end());
}

void DecomposeBatchNormGrad(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  CINN_CHECK_EQ(instr->inputs.size(), 5u) << "batch_norm_grad takes dy, x, scale, save_mean, save_variance";
  CINN_CHECK_EQ(instr->outputs.size(), 3u);
  auto y_grad = instr->inputs[0], x = instr->inputs[1], scale = instr->inputs[2], save_mean = instr->inputs[3],
       save_variance = instr->inputs[4];
  float epsilon = hlir::framework::GetAttr<float>(instr->attrs, "epsilon", 1e-5f);
  auto layout   = hlir::framework::GetAttr<std::string>(instr->attrs, "data_layout", "NCHW");
  SubBuilder b(serial);
  BatchNormParts h(&b, x->shape, layout);
  const bool narrow = Is16Bit(x->type);
  Variable xf  = narrow ? b.Cast(x, "float32") : x;
  Variable dyf = Is16Bit(y_grad->type) ? b.Cast(y_grad, "float32") : y_grad;
  // bias_grad = sum(dy); scale_grad = sum(dy * (x - mean)) * rsqrt(variance + eps)
  auto x_mean_diff = b.Subtract(xf, h.To4d(save_mean));
  auto bias_grad   = h.Reduce(dyf);
  auto dy_xmd_sum  = h.Reduce(b.Multiply(dyf, x_mean_diff));
  auto scale_grad  = b.Multiply(dy_xmd_sum, h.StdVarianceInv(save_variance, epsilon));
  // x_grad = scale * rsqrt(variance + eps) / nhw * (nhw * dy - sum(dy) - (x - mean) * sum(dy * (x - mean)) / (variance + eps))
  auto scaled_inv_std = b.Multiply(scale, h.StdVarianceInv(save_variance, epsilon));
  auto tmp0 = h.To4d(b.Divide(scaled_inv_std, h.Constant(scaled_inv_std, h.element_count, "element_count_1d")));
  auto tmp1 = b.Multiply(dyf, h.Constant(dyf, h.element_count, "element_count_4d"));
  auto tmp2 = h.To4d(bias_grad);
  auto x_mean_diff2 = b.Subtract(xf, h.To4d(save_mean));
  auto tmp3_0 = b.Multiply(x_mean_diff2, h.To4d(dy_xmd_sum));
  auto tmp3   = b.Divide(tmp3_0, h.To4d(b.Add(save_variance, h.Constant(save_variance, epsilon, "epsilon"))));
  auto x_grad = b.Multiply(tmp0, b.Subtract(b.Subtract(tmp1, tmp2), tmp3));
  if (narrow) x_grad = b.Cast(x_grad, common::Type2Str(x->type));
  auto ins = b.TakeInstructions({{x_grad, instr->outputs[0]}, {scale_grad, instr->outputs[1]}, {bias_grad, instr->outputs[2]}});
  out->insert(out->end(), ins.begin(), ins.end());
}

// relu_grad(dout, out) = select(out > 0, dout, 0) (cinn/frontend/decomposer/activation.cc:40-55)
void DecomposeReluGrad(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  CINN_CHECK_EQ(instr->inputs.size(), 2u) << " 2 input tensors for " << instr->op_type;
  auto dout = instr->inputs[0], y = instr->inputs[1];
  SubBuilder b(serial);
  auto zero = b.FillConstant(y->shape, 0.0f, "zero", common::Type2Str(y->type));
  auto res  = b.Select(b.GreaterThan(y, zero), dout, zero);
  auto ins  = b.TakeInstructions(res, instr->outputs[0]);
  out->insert(out->end(), ins.begin(), ins.end());
}

// elementwise_add_grad(dout, x, y; axis) -> dx, dy: dout itself where the shapes agree, else its sum over the
// broadcast dimensions (kept for dx, reshaped to y's shape for dy) - cinn/frontend/decomposer/broadcast.cc:22-159
void DecomposeElementwiseAddGrad(const Instruction& instr, int serial, std::vector<Instruction>* out) {
  CINN_CHECK_EQ(instr->inputs.size(), 3u) << " 3 input tensors for " << instr->op_type;
  CINN_CHECK_EQ(instr->outputs.size(), 2u) << "2 output tensors for " << instr->op_type;
  auto dout = instr->inputs[0];
  auto dx = instr->outputs[0], dy = instr->outputs[1];
  int axis = hlir::framework::GetAttr<int>(instr->attrs, "axis", -1);
  CINN_CHECK(!(axis < 0 && dx->shape.size() < dy->shape.size()))
      << "Please make sure x'rank greater than or equal to y'rank when axis = -1";
  if (axis < 0) axis = static_cast<int>(dx->shape.size()) - static_cast<int>(dy->shape.size());
  SubBuilder b(serial);
  Variable dx_t, dy_t;
  if (dx->shape == dout->shape) {
    dx_t = b.Identity(dout);
  } else {
    std::vector<int> dims;
    for (size_t i = 0; i < dout->shape.size(); ++i)
      if (dx->shape[i] == 1 && dout->shape[i] != 1) dims.push_back(static_cast<int>(i));
    dx_t = b.ReduceSum(dout, dims, true);
  }
  if (dy->shape == dout->shape) {
    dy_t = b.Identity(dout);
  } else {
    std::vector<int> dims;
    const int y_rank = static_cast<int>(dy->shape.size());
    for (int i = 0; i < static_cast<int>(dout->shape.size()); ++i) {
      if (i < axis || i >= axis + y_rank) {
        dims.push_back(i);
      } else if (dy->shape[i - axis] == 1 && dout->shape[i] != 1) {
        dims.push_back(i);
      }
    }
    dy_t = b.Reshape(b.ReduceSum(dout, dims, true), dy->shape);
  }
  auto ins = b.TakeInstructions({{dx_t, dx}, {dy_t, dy}});
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
    } else if (ins->op_type == "relu_grad") {
      DecomposeReluGrad(ins, serial++, &out);
    } else if (ins->op_type == "elementwise_add_grad") {
      DecomposeElementwiseAddGrad(ins, serial++, &out);
    } else if (ins->op_type == "batch_norm_train") {
      DecomposeBatchNormTrain(ins, serial++, &out);
    } else if (ins->op_type == "batch_norm_grad") {
      DecomposeBatchNormGrad(ins, serial++, &out);
    } else {
      out.push_back(ins);
    }
  }
  return Program(std::move(out), program.GetInputs(), program.name());
}

}  // namespace frontend
}  // namespace cinn
