#include "frontend/net_builder.h"

#include <algorithm>
#include <numeric>

#include "hlir/op.h"

namespace cinn {
namespace frontend {

using hlir::framework::OpRegistry;
using utils::ShapeType;

NetBuilder::NetBuilder(const std::string& name) : name_(name) {}

std::string NetBuilder::NewVarId(const std::string& hint) { return hint + "_" + std::to_string(var_counter_++); }

Program NetBuilder::Build(bool in_reverse) {
  std::vector<Instruction> instrs = instrs_;
  if (in_reverse) std::reverse(instrs.begin(), instrs.end());
  return Program(std::move(instrs), inputs_, name_);
}

Placeholder NetBuilder::CreateInput(const common::Type& type, const ShapeType& shape, const std::string& id_hint) {
  CINN_CHECK(!shape.empty()) << "an input needs a non-empty shape";
  for (int d : shape) CINN_CHECK_GT(d, 0) << "input dimensions must be positive";
  std::string id = id_hint.empty() ? NewVarId("placeholder") : id_hint;
  for (auto& in : inputs_) CINN_CHECK(in->id != id) << "duplicate input name " << id;
  Variable v(id);
  v->shape = shape;
  v->type  = type;
  inputs_.push_back(v);
  return v;
}

const std::vector<Variable>& NetBuilder::CustomInstr(const std::string& type, const std::vector<Variable>& inputs,
                                                     const AttributeMap& attrs) {
  const auto& op = OpRegistry::Global().Get(type);
  if (op.num_inputs >= 0)
    CINN_CHECK_EQ(static_cast<int>(inputs.size()), op.num_inputs) << "operator " << type << ": wrong number of inputs";
  Instruction instr(type);
  instr->inputs = inputs;
  instr->attrs  = attrs;
  std::vector<ShapeType> in_shapes;
  std::vector<common::Type> in_types;
  for (auto& in : inputs) {
    CINN_CHECK(in.defined()) << "operator " << type << " got an undefined input";
    in_shapes.push_back(in->shape);
    in_types.push_back(in->type);
  }
  auto out_shapes = op.infer_shape(in_shapes, attrs);
  auto out_types  = op.infer_dtype(in_types, attrs);
  CINN_CHECK_EQ(out_shapes.size(), out_types.size());
  for (size_t i = 0; i < out_shapes.size(); ++i) {
    Variable out(NewVarId("var"));
    out->shape = out_shapes[i];
    out->type  = out_types[i];
    for (int d : out->shape) CINN_CHECK_GT(d, 0) << "operator " << type << " produces an empty tensor";
    instr->outputs.push_back(out);
  }
  instrs_.push_back(instr);
  return instrs_.back()->outputs;
}

Variable NetBuilder::UnaryOp(const std::string& op_type, const Variable& x) { return CustomInstr(op_type, {x}, {}).front(); }

namespace {
// Output shape and, per operand, the output axis each operand dimension maps to.
void AlignBinaryShapes(const ShapeType& a, const ShapeType& b, int axis, ShapeType* out, ShapeType* axes_a,
                       ShapeType* axes_b) {
  ShapeType sa = a, sb = b;
  CINN_CHECK_GE(axis, -1) << "wrong broadcast axis " << axis;
  if (axis >= 0) {
    // the shorter operand starts at `axis` of the longer one: pad it with ones on the right
    ShapeType& shorter = sa.size() >= sb.size() ? sb : sa;
    size_t longer_rank = std::max(sa.size(), sb.size());
    CINN_CHECK_LE(static_cast<size_t>(axis) + shorter.size(), longer_rank) << "wrong broadcast axis " << axis;
    size_t pad = longer_rank - shorter.size() - axis;
    shorter.insert(shorter.end(), pad, 1);
  }
  size_t rank = std::max(sa.size(), sb.size());
  out->assign(rank, 1);
  axes_a->clear();
  axes_b->clear();
  for (size_t i = 0; i < sa.size(); ++i) axes_a->push_back(static_cast<int>(rank - sa.size() + i));
  for (size_t i = 0; i < sb.size(); ++i) axes_b->push_back(static_cast<int>(rank - sb.size() + i));
  for (size_t i = 0; i < rank; ++i) {
    int da = i >= rank - sa.size() ? sa[i - (rank - sa.size())] : 1;
    int db = i >= rank - sb.size() ? sb[i - (rank - sb.size())] : 1;
    CINN_CHECK(da == db || da == 1 || db == 1) << "incompatible broadcast dims " << da << " and " << db;
    (*out)[i] = std::max(da, db);
  }
  // drop the padding ones again: axes must list one entry per ORIGINAL operand dimension
  axes_a->resize(a.size());
  axes_b->resize(b.size());
}
}  // namespace

Variable NetBuilder::BinaryOp(const std::string& op_type, const Variable& lhs, const Variable& rhs, int axis) {
  CINN_CHECK(lhs->type == rhs->type) << "The inputs type of op " << op_type << " should be equal!";
  Variable a = lhs, b = rhs;
  if (a->shape != b->shape) {
    ShapeType out, axes_a, axes_b;
    AlignBinaryShapes(a->shape, b->shape, axis, &out, &axes_a, &axes_b);
    if (a->shape != out) a = BroadcastTo(a, out, axes_a);
    if (b->shape != out) b = BroadcastTo(b, out, axes_b);
  }
  return CustomInstr(op_type, {a, b}, {{"axis", axis}}).front();
}

Variable NetBuilder::Reduce(const std::string& op_type, const Variable& x, const ShapeType& dim, bool keep_dim) {
  // a single-element tensor reduces to itself (cinn/frontend/net_builder.cc:107-128)
  int64_t product = hlir::framework::ShapeNumel(x->shape);
  if (product == 1) {
    if (keep_dim) return Identity(x);
    CINN_CHECK_GE(x->shape.size(), dim.size()) << "The inputs rank should be greater than or equal to axes.";
    int new_rank = x->shape.size() == dim.size() ? 1 : static_cast<int>(x->shape.size() - dim.size());
    if (dim.empty()) new_rank = 1;
    return Reshape(x, ShapeType(new_rank, 1));
  }
  ShapeType reduce_dim(dim);
  for (auto& d : reduce_dim)
    if (d < 0) d += static_cast<int>(x->shape.size());
  return CustomInstr(op_type, {x}, {{"dim", reduce_dim}, {"keep_dim", keep_dim}}).front();
}

#define CINN_NETBUILDER_UNARY_DEF(fn, op) \
  Variable NetBuilder::fn(const Variable& x) { return UnaryOp(#op, x); }
CINN_NETBUILDER_UNARY_FOREACH(CINN_NETBUILDER_UNARY_DEF)
#undef CINN_NETBUILDER_UNARY_DEF

#define CINN_NETBUILDER_BINARY_DEF(fn, op) \
  Variable NetBuilder::fn(const Variable& lhs, const Variable& rhs, int axis) { return BinaryOp(#op, lhs, rhs, axis); }
CINN_NETBUILDER_BINARY_FOREACH(CINN_NETBUILDER_BINARY_DEF)
#undef CINN_NETBUILDER_BINARY_DEF

Variable NetBuilder::Select(const Variable& condition, const Variable& true_value, const Variable& false_value) {
  return CustomInstr("select", {condition, true_value, false_value}, {}).front();
}
Variable NetBuilder::Scale(const Variable& x, float scale, float bias, bool bias_after_scale) {
  return CustomInstr("scale", {x}, {{"scale", scale}, {"bias", bias}, {"bias_after_scale", bias_after_scale}}).front();
}
Variable NetBuilder::Sum(const std::vector<Variable>& inputs) { return CustomInstr("sum", inputs, {}).front(); }
Variable NetBuilder::Relu6(const Variable& x, float threshold) {
  return CustomInstr("relu6", {x}, {{"threshold", threshold}}).front();
}
Variable NetBuilder::Cast(const Variable& x, const std::string& dtype) {
  if (common::Type2Str(x->type) == dtype) return Identity(x);
  return CustomInstr("cast", {x}, {{"dtype", dtype}}).front();
}
Variable NetBuilder::FillConstant(const ShapeType& shape, float value, const std::string& name, const std::string& dtype,
                                  bool force_cpu) {
  auto out = CustomInstr("fill_constant", {},
                         {{"shape", shape}, {"value", static_cast<double>(value)}, {"dtype", dtype}, {"force_cpu", force_cpu}})
                 .front();
  (void)name;
  return out;
}

Variable NetBuilder::ReduceSum(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_sum", x, dim, keep_dim); }
Variable NetBuilder::ReduceProd(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_prod", x, dim, keep_dim); }
Variable NetBuilder::ReduceMax(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_max", x, dim, keep_dim); }
Variable NetBuilder::ReduceMin(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_min", x, dim, keep_dim); }
Variable NetBuilder::ReduceAll(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_all", x, dim, keep_dim); }
Variable NetBuilder::ReduceAny(const Variable& x, const ShapeType& dim, bool keep_dim) { return Reduce("reduce_any", x, dim, keep_dim); }
Variable NetBuilder::Argmax(const Variable& x, const int& axis, const bool& keep_dim) {
  return CustomInstr("argmax", {x}, {{"axis", axis}, {"keep_dim", keep_dim}}).front();
}
Variable NetBuilder::Argmin(const Variable& x, const int& axis, const bool& keep_dim) {
  return CustomInstr("argmin", {x}, {{"axis", axis}, {"keep_dim", keep_dim}}).front();
}

std::vector<Variable> NetBuilder::ArgSort(const Variable& operand, const int& axis, const bool& is_ascend) {
  return CustomInstr("argsort", {operand}, {{"axis", axis}, {"is_ascend", is_ascend}});
}
Variable NetBuilder::Sort(const Variable& operand, const int& axis, const bool& is_ascend) {
  return CustomInstr("sort", {operand}, {{"axis", axis}, {"is_ascend", is_ascend}}).front();
}

std::vector<Variable> NetBuilder::TopK(const Variable& x, int k, int axis, bool largest) {
  (void)largest;
  CINN_CHECK_GT(k, 0) << "The attribute k must be greater than 0.";
  if (axis < 0) axis += static_cast<int>(x->shape.size());
  CINN_CHECK(axis >= 0 && axis < static_cast<int>(x->shape.size())) << "top_k: axis out of range";
  CINN_CHECK_LE(k, x->shape[axis]) << "top_k: k exceeds the extent of the axis";
  Variable values  = Slice(Sort(x, axis, false), {axis}, {0}, {k});
  Variable indices = Cast(Slice(ArgSort(x, axis, false).at(0), {axis}, {0}, {k}), "int64");
  return {values, indices};
}

Variable NetBuilder::BroadcastTo(const Variable& x, const ShapeType& out_shape) {
  // numpy alignment: the operand's dimensions map onto the trailing output dimensions
  auto x_rank = x->shape.size();
  CINN_CHECK_LE(x_rank, out_shape.size()) << "broadcast_to cannot reduce the rank";
  ShapeType axes;
  if (x_rank == 1) {
    // a vector maps to the FIRST output dimension of its length, a single element to dimension 0
    // (cinn/frontend/net_builder.cc:304-323)
    int found = x->shape[0] == 1 ? 0 : -1;
    for (int i = 0; found < 0 && i < static_cast<int>(out_shape.size()); ++i) {
      if (out_shape[i] == x->shape[0]) found = i;
    }
    CINN_CHECK_GE(found, 0) << "When we broadcast a 1-dimension shape, the number should be contained in the out_shape";
    axes = {found};
  } else {
    for (size_t i = 0; i < x_rank; ++i) {
      size_t o = out_shape.size() - x_rank + i;
      CINN_CHECK(out_shape[o] == x->shape[i] || x->shape[i] == 1) << "cannot broadcast dimension " << i;
      axes.push_back(static_cast<int>(o));
    }
  }
  return BroadcastTo(x, out_shape, axes);
}
Variable NetBuilder::BroadcastTo(const Variable& x, const ShapeType& out_shape, const ShapeType& broadcast_axes) {
  return CustomInstr("broadcast_to", {x}, {{"out_shape", out_shape}, {"broadcast_axes", broadcast_axes}}).front();
}
Variable NetBuilder::Reshape(const Variable& x, const ShapeType& shape) {
  return CustomInstr("reshape", {x}, {{"shape", shape}}).front();
}
Variable NetBuilder::Transpose(const Variable& x, const ShapeType& axis) {
  return CustomInstr("transpose", {x}, {{"axis", axis}}).front();
}
Variable NetBuilder::Concat(const std::vector<Variable>& xs, int axis) {
  CINN_CHECK(!xs.empty()) << "concat needs at least one input";
  if (xs.size() == 1) return Identity(xs[0]);
  return CustomInstr("concat", xs, {{"axis", axis}}).front();
}
Variable NetBuilder::Slice(const Variable& x, const ShapeType& axes, const ShapeType& starts, const ShapeType& ends,
                           const ShapeType& infer_flags, const ShapeType& strides, const ShapeType& decrease_axis) {
  auto out = CustomInstr("slice", {x},
                         {{"axes", axes}, {"starts", starts}, {"ends", ends}, {"infer_flags", infer_flags},
                          {"strides", strides}, {"decrease_axis", decrease_axis}})
                 .front();
  if (!decrease_axis.empty()) {
    ShapeType shape;
    for (int i = 0; i < static_cast<int>(out->shape.size()); ++i) {
      bool drop = std::find(decrease_axis.begin(), decrease_axis.end(), i) != decrease_axis.end() && out->shape[i] == 1;
      if (!drop) shape.push_back(out->shape[i]);
    }
    if (shape.empty()) shape.push_back(1);
    return Reshape(out, shape);
  }
  return out;
}
Variable NetBuilder::Squeeze(const Variable& x, const ShapeType& axes) {
  ShapeType shape;
  int rank = static_cast<int>(x->shape.size());
  for (int i = 0; i < rank; ++i) {
    bool listed = axes.empty();
    for (int a : axes) listed |= ((a < 0 ? a + rank : a) == i);
    if (!(listed && x->shape[i] == 1)) shape.push_back(x->shape[i]);
  }
  if (shape.empty()) shape.push_back(1);
  return Reshape(x, shape);
}
Variable NetBuilder::ReluGrad(const Variable& dout, const Variable& out) {
  return CustomInstr("relu_grad", {dout, out}, {}).front();
}
std::vector<Variable> NetBuilder::ElementwiseAddGrad(const Variable& dout, const Variable& x, const Variable& y, int axis) {
  return CustomInstr("elementwise_add_grad", {dout, x, y}, {{"axis", axis}});
}
Variable NetBuilder::ExpandDims(const Variable& x, const ShapeType& axes) {
  ShapeType shape = x->shape;
  for (int a : axes) {
    int pos = a < 0 ? a + static_cast<int>(shape.size()) + 1 : a;
    CINN_CHECK(pos >= 0 && pos <= static_cast<int>(shape.size())) << "expand_dims axis out of range";
    shape.insert(shape.begin() + pos, 1);
  }
  return Reshape(x, shape);
}

Variable NetBuilder::Softmax(const Variable& x, const ShapeType& axes, const std::string& mode,
                             const std::string& data_format) {
  return CustomInstr("softmax", {x}, {{"axes", axes}, {"mode", mode}, {"data_format", data_format}}).front();
}
Variable NetBuilder::Matmul(const Variable& x, const Variable& y, bool trans_x, bool trans_y, float alpha) {
  return CustomInstr("matmul", {x, y}, {{"trans_a", trans_x}, {"trans_b", trans_y}, {"alpha", alpha}}).front();
}
Variable NetBuilder::Mul(const Variable& x, const Variable& y, int x_num_col_dims, int y_num_col_dims, bool is_infer) {
  return CustomInstr("mul", {x, y},
                     {{"x_num_col_dims", x_num_col_dims}, {"y_num_col_dims", y_num_col_dims}, {"is_infer", is_infer}})
      .front();
}
Variable NetBuilder::Conv2d(const Variable& x, const Variable& w, const std::vector<int>& strides,
                            const std::vector<int>& paddings, const std::vector<int>& dilations, int groups,
                            const std::string& data_format, const std::string& padding_algorithm) {
  return Conv(x, w, strides, paddings, dilations, groups, "forward", data_format, padding_algorithm, {});
}
// cinn/frontend/net_builder.cc:465-486: forward takes (x, w); backward_data (w, dy) and gives dx of `output_shape`;
// backward_filter (x, dy) and gives dw of `output_shape`
Variable NetBuilder::Conv(const Variable& lhs, const Variable& rhs, const std::vector<int>& strides,
                          const std::vector<int>& paddings, const std::vector<int>& dilations, int groups,
                          const std::string& conv_type, const std::string& data_format,
                          const std::string& padding_algorithm, const std::vector<int>& output_shape) {
  return CustomInstr("conv2d", {lhs, rhs},
                     {{"stride", strides},
                      {"padding", paddings},
                      {"dilation", dilations},
                      {"groups", groups},
                      {"conv_type", conv_type},
                      {"data_format", data_format},
                      {"padding_algorithm", padding_algorithm},
                      {"output_shape", output_shape}})
      .front();
}
std::vector<Variable> NetBuilder::BatchNorm(const Variable& x, const Variable& scale, const Variable& bias,
                                            const Variable& mean, const Variable& variance, float epsilon,
                                            float momentum, const std::string& data_layout, bool is_test) {
  // cinn/frontend/net_builder.cc:760-773: one output when is_test, else y, saved mean / variance, moving mean / variance
  return CustomInstr(is_test ? "batch_norm" : "batch_norm_train", {x, scale, bias, mean, variance},
                     {{"epsilon", epsilon}, {"momentum", momentum}, {"data_layout", data_layout}});
}
// outputs x_grad, scale_grad, bias_grad (cinn/frontend/net_builder.cc:776-786)
std::vector<Variable> NetBuilder::BatchNormGrad(const Variable& dy, const Variable& x, const Variable& scale,
                                                const Variable& save_mean, const Variable& save_variance,
                                                float epsilon, const std::string& data_layout) {
  return CustomInstr("batch_norm_grad", {dy, x, scale, save_mean, save_variance},
                     {{"epsilon", epsilon}, {"data_layout", data_layout}});
}

namespace {
utils::AttributeMap Pool2dAttrs(const Variable& x, const std::string& pooling_type, const std::vector<int>& ksize,
                         const std::vector<int>& strides, const std::vector<int>& paddings, bool ceil_mode,
                         bool exclusive, bool global_pooling, const std::string& data_format, bool adaptive,
                         const std::string& padding_algorithm) {
  // attribute normalisation of cinn/frontend/net_builder.cc:538-684
  CINN_CHECK_EQ(x->shape.size(), 4u) << "Input's dim must be 4";
  std::string pool_type;
  std::transform(pooling_type.begin(), pooling_type.end(), std::back_inserter(pool_type),
                 [](unsigned char c) { return std::tolower(c); });
  CINN_CHECK(pool_type == "avg" || pool_type == "max") << "Pool_type must be avg or max, but got: " << pool_type;
  std::vector<int> k(ksize);
  if (k.size() == 1) k.push_back(k[0]);
  CINN_CHECK_EQ(k.size(), 2u) << "Kernel_size length must be 1 or 2";
  std::vector<int> s(strides);
  if (s.size() == 1) s.push_back(s[0]);
  CINN_CHECK_EQ(s.size(), 2u) << "Stride length must be 1 or 2";
  CINN_CHECK(s[0] > 0 && s[1] > 0) << "the stride of pool2d should be greater than 0";
  std::string layout = data_format == "AnyLayout" ? "NCHW" : data_format;
  CINN_CHECK(layout == "NCHW" || layout == "NHWC") << "Data_format must be AnyLayout/NCHW/NHWC";
  CINN_CHECK(padding_algorithm == "EXPLICIT" || padding_algorithm == "SAME" || padding_algorithm == "VALID")
      << "Padding_algorithm must be EXPLICIT/SAME/VALID";
  if (pool_type == "avg" && !global_pooling && adaptive && k[0] == 1 && k[1] == 1) {
    adaptive       = false;
    global_pooling = true;
  }
  int hi = layout == "NCHW" ? 2 : 1, wi = hi + 1;
  std::vector<int> p(paddings);
  if (p.size() == 2) p.insert(p.end(), paddings.begin(), paddings.end());
  CINN_CHECK_EQ(p.size(), 4u) << "Padding size must be 2 or 4";
  if (padding_algorithm == "VALID") {
    p = {0, 0, 0, 0};
  } else if (padding_algorithm == "SAME") {
    int oh = (x->shape[hi] + s[0] - 1) / s[0], ow = (x->shape[wi] + s[1] - 1) / s[1];
    int ph = std::max((oh - 1) * s[0] + k[0] - x->shape[hi], 0);
    int pw = std::max((ow - 1) * s[1] + k[1] - x->shape[wi], 0);
    p      = {ph / 2, pw / 2, ph - ph / 2, pw - pw / 2};
  }
  if (global_pooling || adaptive) p = {0, 0, 0, 0};
  if (global_pooling) k = {x->shape[hi], x->shape[wi]};
  return utils::AttributeMap{{"pool_type", pool_type},
                      {"kernel_size", k},
                      {"stride_size", s},
                      {"padding_size", p},
                      {"ceil_mode", ceil_mode},
                      {"exclusive", exclusive},
                      {"global_pooling", global_pooling},
                      {"data_format", layout},
                      {"adaptive", adaptive},
                      {"padding_algorithm", padding_algorithm}};
}
}  // namespace

Variable NetBuilder::Pool2d(const Variable& x, const std::string& pooling_type, const std::vector<int>& ksize,
                            const std::vector<int>& strides, const std::vector<int>& paddings, bool ceil_mode,
                            bool exclusive, bool global_pooling, const std::string& data_format, bool adaptive,
                            const std::string& padding_algorithm) {
  return CustomInstr("pool2d", {x},
                     Pool2dAttrs(x, pooling_type, ksize, strides, paddings, ceil_mode, exclusive, global_pooling,
                                 data_format, adaptive, padding_algorithm))
      .front();
}
// cinn/frontend/net_builder.cc:686-755: the same attribute normalisation as pool2d, inputs x, y = pool2d(x), dy
Variable NetBuilder::Pool2dGrad(const Variable& x, const Variable& y, const Variable& dy, const std::string& pooling_type,
                                const std::vector<int>& ksize, const std::vector<int>& strides,
                                const std::vector<int>& paddings, bool ceil_mode, bool exclusive, bool global_pooling,
                                const std::string& data_format, bool adaptive, const std::string& padding_algorithm) {
  return CustomInstr("pool2d_grad", {x, y, dy},
                     Pool2dAttrs(x, pooling_type, ksize, strides, paddings, ceil_mode, exclusive, global_pooling,
                                 data_format, adaptive, padding_algorithm))
      .front();
}

std::vector<Variable> PaddleLayerNorm(NetBuilder* builder, Variable x, Variable scale, Variable bias, float epsilon,
                                      int begin_norm_axis) {
  const auto x_shape = x->shape;
  const int x_ndim   = static_cast<int>(x_shape.size());
  CINN_CHECK(begin_norm_axis > 0 && begin_norm_axis <= x_ndim) << "begin_norm_axis out of range";
  int left = 1, right = 1;
  for (int i = 0; i < begin_norm_axis; ++i) left *= x_shape[i];
  for (int i = begin_norm_axis; i < x_ndim; ++i) right *= x_shape[i];

  const auto x_type = x->type;
  if (x_type.is_float16() || x_type.is_bfloat16()) x = builder->Cast(x, "float32");
  const std::string type_str = common::Type2Str(x->type);

  ShapeType shape{left, right};
  auto x_reshape = builder->Reshape(x, shape);
  auto x_reduce  = builder->ReduceSum(x_reshape, {1});
  auto ele_num   = builder->FillConstant({left}, static_cast<float>(right), "layer_norm_ele_num", type_str);
  auto x_mean    = builder->Divide(x_reduce, ele_num);

  // variance as E[x^2] - E[x]^2, clamped at zero
  auto x2        = builder->Multiply(x_reshape, builder->Identity(x_reshape));
  auto x2_reduce = builder->ReduceSum(x2, {1});
  auto x2_mean   = builder->Divide(x2_reduce, ele_num);
  auto x_mean2   = builder->Multiply(x_mean, builder->Identity(x_mean));
  auto zero      = builder->FillConstant({left}, 0.f, "layer_norm_zero", type_str);
  auto x_var     = builder->Max(builder->Subtract(x2_mean, x_mean2), zero);

  auto x_mean_broadcast = builder->BroadcastTo(x_mean, shape, {0});
  auto y_sub            = builder->Subtract(x_reshape, x_mean_broadcast);
  auto epsilon_var      = builder->FillConstant({left}, epsilon, "layer_norm_epsilon", type_str);
  auto x_var_eps        = builder->Add(x_var, epsilon_var);
  auto x_var_sqrt       = builder->Sqrt(x_var_eps);
  auto y_out            = builder->Divide(y_sub, builder->BroadcastTo(x_var_sqrt, shape, {0}));

  if (scale.defined()) {
    if (scale->type.is_float16() || scale->type.is_bfloat16()) scale = builder->Cast(scale, "float32");
    y_out = builder->Multiply(y_out, builder->BroadcastTo(scale, shape, {1}));
  }
  if (bias.defined()) {
    if (bias->type.is_float16() || bias->type.is_bfloat16()) bias = builder->Cast(bias, "float32");
    y_out = builder->Add(y_out, builder->BroadcastTo(bias, shape, {1}));
  }
  y_out = builder->Reshape(y_out, x_shape);
  if (x_type.is_float16()) {
    y_out = builder->Cast(y_out, "float16");
  } else if (x_type.is_bfloat16()) {
    y_out = builder->Cast(y_out, "bfloat16");
  }
  return {y_out, x_mean, x_var};
}

}  // namespace frontend
}  // namespace cinn
