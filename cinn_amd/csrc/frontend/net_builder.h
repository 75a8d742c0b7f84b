// NetBuilder: the graph-construction API.  Method names, argument order and defaults follow
// cinn/frontend/net_builder.h:125-1143 for the operators the gfx950 backend lowers.  Every method
// appends one instruction (CustomInstr) after inferring output shapes and types from the operator
// registry; binary operators whose operands differ in shape get an explicit broadcast_to in front,
// using the alignment rule of pe::GetBroadcastShape (cinn/hlir/pe/broadcast.cc:34-150).
#pragma once
#include <string>
#include <vector>

#include "frontend/syntax.h"

namespace cinn {
namespace frontend {

class NetBuilder {
 public:
  using AttributeMap = utils::AttributeMap;
  explicit NetBuilder(const std::string& name);
  virtual ~NetBuilder() = default;

  Program Build(bool in_reverse = false);
  const std::string& name() const { return name_; }
  size_t size() const { return instrs_.size(); }

  Placeholder CreateInput(const common::Type& type, const utils::ShapeType& shape, const std::string& id_hint = "");
  const std::vector<Variable>& CustomInstr(const std::string& type, const std::vector<Variable>& inputs,
                                           const AttributeMap& attrs);

  // ---- element-wise -----------------------------------------------------------------------------
#define CINN_NETBUILDER_UNARY_FOREACH(m)                                                                         \
  m(Sqrt, sqrt) m(Tanh, tanh) m(Relu, relu) m(Gelu, gelu) m(Sigmoid, sigmoid) m(Identity, identity) m(Exp, exp)  \
      m(Erf, erf) m(Rsqrt, rsqrt) m(Log, log) m(Log2, log2) m(Log10, log10) m(Floor, floor) m(Ceil, ceil)        \
          m(Round, round) m(Trunc, trunc) m(Sin, sin) m(Cos, cos) m(Tan, tan) m(Sinh, sinh) m(Cosh, cosh)        \
              m(Asin, asin) m(Acos, acos) m(Atan, atan) m(Asinh, asinh) m(Acosh, acosh) m(Atanh, atanh)          \
                  m(IsNan, isnan) m(IsFinite, isfinite) m(IsInf, isinf) m(LogicalNot, logical_not)               \
                      m(BitwiseNot, bitwise_not) m(Negative, negative) m(Sign, sign) m(Abs, abs) m(Cbrt, cbrt)   \
                          m(Clz, clz) m(Popc, popc) m(Reciprocal, reciprocal)
#define CINN_NETBUILDER_UNARY_DECL(fn, op) Variable fn(const Variable& x);
  CINN_NETBUILDER_UNARY_FOREACH(CINN_NETBUILDER_UNARY_DECL)
#undef CINN_NETBUILDER_UNARY_DECL

#define CINN_NETBUILDER_BINARY_FOREACH(m)                                                                       \
  m(Add, elementwise_add) m(ElementwiseAdd, elementwise_add) m(Subtract, subtract) m(Divide, divide)            \
      m(Multiply, elementwise_mul) m(ElementwiseMul, elementwise_mul) m(FloorDivide, floor_divide) m(Mod, mod)  \
          m(Remainder, remainder) m(Max, max) m(Min, min) m(Pow, pow) m(LogicalAnd, logical_and)                \
              m(LogicalOr, logical_or) m(LogicalXor, logical_xor) m(BitwiseAnd, bitwise_and)                    \
                  m(BitwiseOr, bitwise_or) m(BitwiseXor, bitwise_xor) m(LeftShift, left_shift)                  \
                      m(RightShift, right_shift) m(Equal, equal) m(NotEqual, not_equal)                         \
                          m(GreaterThan, greater_than) m(LessThan, less_than) m(GreaterEqual, greater_equal)    \
                              m(LessEqual, less_equal) m(LogicalRightShift, logical_right_shift)
#define CINN_NETBUILDER_BINARY_DECL(fn, op) Variable fn(const Variable& lhs, const Variable& rhs, int axis = -1);
  CINN_NETBUILDER_BINARY_FOREACH(CINN_NETBUILDER_BINARY_DECL)
#undef CINN_NETBUILDER_BINARY_DECL

  Variable Select(const Variable& condition, const Variable& true_value, const Variable& false_value);
  Variable Scale(const Variable& x, float scale = 1.0f, float bias = 0.0f, bool bias_after_scale = true);
  Variable Sum(const std::vector<Variable>& inputs);
  Variable Relu6(const Variable& x, float threshold = 6.0f);
  Variable Cast(const Variable& x, const std::string& dtype);
  Variable FillConstant(const utils::ShapeType& shape, float value, const std::string& name,
                        const std::string& dtype, bool force_cpu = false);

  // ---- reductions -------------------------------------------------------------------------------
  Variable ReduceSum(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable ReduceProd(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable ReduceMax(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable ReduceMin(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable ReduceAll(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable ReduceAny(const Variable& x, const utils::ShapeType& dim = {}, bool keep_dim = false);
  Variable Argmax(const Variable& x, const int& axis = 0, const bool& keep_dim = false);
  Variable Argmin(const Variable& x, const int& axis = 0, const bool& keep_dim = false);
  // cinn/frontend/net_builder.h:1028-1046: {indices, positions} resp. the sorted values, both of the operand's shape
  std::vector<Variable> ArgSort(const Variable& operand, const int& axis, const bool& is_ascend = true);
  Variable Sort(const Variable& operand, const int& axis, const bool& is_ascend = true);
  // {values, int64 indices} of the k largest entries along `axis`, as the reference's decomposer composes them
  // (cinn/frontend/decomposer/top_k.cc:22-47: descending sort / argsort, slice, cast); like there, `largest` is
  // accepted and not consulted
  std::vector<Variable> TopK(const Variable& x, int k, int axis, bool largest);

  // ---- shape manipulation -----------------------------------------------------------------------
  Variable BroadcastTo(const Variable& x, const utils::ShapeType& out_shape);
  Variable BroadcastTo(const Variable& x, const utils::ShapeType& out_shape, const utils::ShapeType& broadcast_axes);
  Variable Reshape(const Variable& x, const utils::ShapeType& shape);
  Variable Transpose(const Variable& x, const utils::ShapeType& axis);
  Variable Concat(const std::vector<Variable>& xs, int axis = 0);
  Variable Slice(const Variable& x, const utils::ShapeType& axes, const utils::ShapeType& starts,
                 const utils::ShapeType& ends, const utils::ShapeType& infer_flags = {},
                 const utils::ShapeType& strides = {}, const utils::ShapeType& decrease_axis = {});
  Variable Squeeze(const Variable& x, const utils::ShapeType& axes = {});
  Variable ExpandDims(const Variable& x, const utils::ShapeType& axes);

  // ---- neural-network ops -----------------------------------------------------------------------
  Variable Softmax(const Variable& x, const utils::ShapeType& axes = {-1}, const std::string& mode = "fast",
                   const std::string& data_format = "AnyLayout");
  Variable Matmul(const Variable& x, const Variable& y, bool trans_x = false, bool trans_y = false, float alpha = 1.0f);
  Variable Mul(const Variable& x, const Variable& y, int x_num_col_dims = 1, int y_num_col_dims = 1,
               bool is_infer = false);
  Variable Conv2d(const Variable& x, const Variable& w, const std::vector<int>& strides = {1, 1},
                  const std::vector<int>& paddings = {0, 0}, const std::vector<int>& dilations = {1, 1},
                  int groups = 1, const std::string& data_format = "NCHW",
                  const std::string& padding_algorithm = "EXPLICIT");
  // conv_type "forward" (x, w), "backward_data" (w, dy -> dx of output_shape) or "backward_filter" (x, dy -> dw of
  // output_shape), cinn/frontend/net_builder.h (Conv)
  Variable Conv(const Variable& lhs, const Variable& rhs, const std::vector<int>& strides = {1, 1},
                const std::vector<int>& paddings = {0, 0}, const std::vector<int>& dilations = {1, 1}, int groups = 1,
                const std::string& conv_type = "forward", const std::string& data_format = "NCHW",
                const std::string& padding_algorithm = "EXPLICIT", const std::vector<int>& output_shape = {});
  std::vector<Variable> BatchNorm(const Variable& x, const Variable& scale, const Variable& bias,
                                  const Variable& mean, const Variable& variance, float epsilon = 1e-5f,
                                  float momentum = 0.9f, const std::string& data_layout = "NCHW", bool is_test = true);
  // cinn/frontend/net_builder.cc:419-432
  Variable ReluGrad(const Variable& dout, const Variable& out);
  std::vector<Variable> ElementwiseAddGrad(const Variable& dout, const Variable& x, const Variable& y, int axis = -1);
  std::vector<Variable> BatchNormGrad(const Variable& dy, const Variable& x, const Variable& scale,
                                      const Variable& save_mean, const Variable& save_variance, float epsilon = 1e-5f,
                                      const std::string& data_layout = "NCHW");
  Variable Pool2d(const Variable& x, const std::string& pooling_type, const std::vector<int>& ksize,
                  const std::vector<int>& strides = {1, 1}, const std::vector<int>& paddings = {0, 0},
                  bool ceil_mode = false, bool exclusive = true, bool global_pooling = false,
                  const std::string& data_format = "NCHW", bool adaptive = false,
                  const std::string& padding_algorithm = "EXPLICIT");
  Variable Pool2dGrad(const Variable& x, const Variable& y, const Variable& dy, const std::string& pooling_type,
                      const std::vector<int>& ksize, const std::vector<int>& strides = {1, 1},
                      const std::vector<int>& paddings = {0, 0}, bool ceil_mode = false, bool exclusive = true,
                      bool global_pooling = false, const std::string& data_format = "NCHW", bool adaptive = false,
                      const std::string& padding_algorithm = "EXPLICIT");

 protected:
  Variable UnaryOp(const std::string& op_type, const Variable& x);
  Variable BinaryOp(const std::string& op_type, const Variable& lhs, const Variable& rhs, int axis = -1);
  Variable Reduce(const std::string& op_type, const Variable& x, const utils::ShapeType& dim, bool keep_dim);

 private:
  std::string NewVarId(const std::string& hint = "var");
  std::string name_;
  std::vector<Instruction> instrs_;
  std::vector<Variable> inputs_;
  int var_counter_{0};
};

// Paddle layer_norm expressed in NetBuilder primitives, the composition of the Paddle op mapper
// (cinn/frontend/op_mappers/paddle/layer_norm.cc:83-140).  Returns {y, mean, variance}; scale and
// bias may be undefined Variables.
std::vector<Variable> PaddleLayerNorm(NetBuilder* builder, Variable x, Variable scale, Variable bias,
                                      float epsilon = 1e-5f, int begin_norm_axis = 1);

}  // namespace frontend
}  // namespace cinn
