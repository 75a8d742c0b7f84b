#include <algorithm>
#include <cmath>
#include <numeric>

#include "hlir/op.h"

namespace cinn {
namespace hlir {
namespace framework {

using common::Type;
using ir::Expr;

int64_t ShapeNumel(const ShapeType& s) {
  int64_t n = 1;
  for (int d : s) n *= d;
  return n;
}

std::string ExternFuncName(const std::string& fn, const Type& type) {
  return "cinn_hip_" + fn + "_" + common::TypeSuffix(type);
}

OpRegistry& OpRegistry::Global() {
  static OpRegistry r;
  return r;
}
const Operator* OpRegistry::Find(const std::string& name) const {
  for (auto& op : ops_)
    if (op->name == name) return op.get();
  return nullptr;
}
const Operator& OpRegistry::Get(const std::string& name) const {
  auto* op = Find(name);
  CINN_CHECK(op) << "operator '" << name << "' is not registered";
  return *op;
}
Operator& OpRegistry::Register(const std::string& name) {
  CINN_CHECK(!Find(name)) << "operator '" << name << "' registered twice";
  ops_.emplace_back(new Operator);
  ops_.back()->name = name;
  return *ops_.back();
}
std::vector<std::string> OpRegistry::ListAllNames() const {
  std::vector<std::string> names;
  for (auto& op : ops_) names.push_back(op->name);
  return names;
}

namespace {

std::vector<ShapeType> SameShapeAsFirst(const std::vector<ShapeType>& in, const AttributeMap&) { return {in[0]}; }
std::vector<Type> SameTypeAsFirst(const std::vector<Type>& in, const AttributeMap&) { return {in[0]}; }
std::vector<Type> BoolType(const std::vector<Type>&, const AttributeMap&) { return {common::Bool()}; }

// A call of a math function by its target-independent name; optim::MapExternCall picks the device library's function
// for the type of the first argument when the group's kernel is built (cinn/optim/map_extern_call.cc:45-115).
Expr CallExtern(const std::string& fn, const Type& t, std::vector<Expr> args, const Type& ret) {
  CINN_CHECK(!args.empty() && args.front().type() == t) << fn << ": the first argument selects the library function";
  return ir::MakeCall(ret, fn, std::move(args));
}

void RegisterUnaryMath(OpRegistry* r, const std::string& op_name, const std::string& fn) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kElementWise;
  op.infer_shape = SameShapeAsFirst;
  op.infer_dtype = SameTypeAsFirst;
  op.compute     = [fn](const std::vector<Expr>& in, const AttributeMap&, const Type& out) {
    CINN_CHECK(in[0].type().is_floating()) << fn << " needs a floating-point operand";
    return CallExtern(fn, in[0].type(), {in[0]}, out);
  };
}

void RegisterUnaryPredicate(OpRegistry* r, const std::string& op_name, const std::string& fn) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kElementWise;
  op.infer_shape = SameShapeAsFirst;
  op.infer_dtype = BoolType;
  op.compute     = [fn](const std::vector<Expr>& in, const AttributeMap&, const Type& out) {
    if (!in[0].type().is_floating()) return ir::MakeConst(out, fn == "isfinite" ? 1 : 0);
    return CallExtern(fn, in[0].type(), {in[0]}, out);
  };
}

using BinaryEmitter = std::function<Expr(const Expr&, const Expr&, const Type&)>;
void RegisterBinary(OpRegistry* r, const std::string& op_name, BinaryEmitter emit, bool compare = false) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kElementWise;
  op.num_inputs  = 2;
  op.infer_shape = [op_name](const std::vector<ShapeType>& in, const AttributeMap&) {
    CINN_CHECK(in[0] == in[1]) << op_name << ": operands must have the same shape after broadcasting";
    return std::vector<ShapeType>{in[0]};
  };
  op.infer_dtype = compare ? BoolType : SameTypeAsFirst;
  op.compute     = [emit](const std::vector<Expr>& in, const AttributeMap&, const Type& out) {
    return emit(in[0], in[1], out);
  };
}

void RegisterReduce(OpRegistry* r, const std::string& op_name, const std::string& kind) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kReduction;
  op.reduce_kind = kind;
  op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& attrs) {
    auto dim      = GetAttr<std::vector<int>>(attrs, "dim", {});
    bool keep_dim = GetAttr<bool>(attrs, "keep_dim", false);
    int rank      = static_cast<int>(in[0].size());
    std::vector<bool> reduced(rank, dim.empty());
    for (int d : dim) {
      if (d < 0) d += rank;
      CINN_CHECK(d >= 0 && d < rank) << "reduce dim out of range";
      reduced[d] = true;
    }
    ShapeType out;
    for (int i = 0; i < rank; ++i) {
      if (!reduced[i]) {
        out.push_back(in[0][i]);
      } else if (keep_dim) {
        out.push_back(1);
      }
    }
    if (out.empty()) out.push_back(1);
    return std::vector<ShapeType>{out};
  };
  op.infer_dtype = SameTypeAsFirst;
}

// reduce_run_<kind>: the input, viewed as [a, parts, r / parts, c], reduced over its third axis; the result
// [a, parts, c] is declared with the shape `out_shape` (same element count) and the type `dtype` (the input's when
// empty).  Internal op: the reduction splitting pass writes reductions over non-trailing axes as chains of these
// (the reference splits such reductions in cinn/hlir/pass/reduce_split_pass.cc).
void RegisterReduceRun(OpRegistry* r, const std::string& op_name, const std::string& kind) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kReduction;
  op.reduce_kind = kind;
  op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& attrs) {
    const int64_t a = GetAttr<int>(attrs, "a", 1), rr = GetAttr<int>(attrs, "r", 1), c = GetAttr<int>(attrs, "c", 1);
    const int64_t parts = GetAttr<int>(attrs, "parts", 1);
    int64_t numel = 1;
    for (int d : in[0]) numel *= d;
    CINN_CHECK_EQ(a * rr * c, numel) << "reduce_run: a * r * c must be the element count of the input";
    CINN_CHECK(parts >= 1 && rr % parts == 0) << "reduce_run: parts must divide r";
    ShapeType out = GetAttr<std::vector<int>>(attrs, "out_shape", {});
    int64_t out_numel = 1;
    for (int d : out) out_numel *= d;
    CINN_CHECK_EQ(out_numel, a * parts * c) << "reduce_run: out_shape does not hold a * parts * c elements";
    return std::vector<ShapeType>{out};
  };
  op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap& attrs) {
    std::string dtype = GetAttr<std::string>(attrs, "dtype", "");
    return std::vector<Type>{dtype.empty() ? in[0] : common::Str2Type(dtype)};
  };
}

void RegisterArgReduce(OpRegistry* r, const std::string& op_name, const std::string& kind) {
  auto& op       = r->Register(op_name);
  op.pattern     = OpPatternKind::kReduction;
  op.reduce_kind = kind;
  // output shape rule of cinn/hlir/op/contrib/argmax.cc:64-79
  op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& attrs) {
    int axis      = GetAttr<int>(attrs, "axis", 0);
    bool keep_dim = GetAttr<bool>(attrs, "keep_dim", false);
    int rank      = static_cast<int>(in[0].size());
    if (axis < 0) axis += rank;
    CINN_CHECK(axis >= 0 && axis < rank) << "arg-reduce axis out of range";
    ShapeType out;
    for (int i = 0; i < rank; ++i) {
      if (i == axis) {
        if (keep_dim) out.push_back(1);
      } else {
        out.push_back(in[0][i]);
      }
    }
    if (out.empty()) out.push_back(1);
    return std::vector<ShapeType>{out};
  };
  // the result is int32 (argmax.cc:210-213)
  op.infer_dtype = [](const std::vector<Type>&, const AttributeMap&) { return std::vector<Type>{common::Int(32)}; };
}

int ConvOutDim(int in, int pad, int dilation, int k, int stride) {
  // cinn/hlir/pe/nn.cc:235-241
  return (in - ((k - 1) * dilation + 1) + 2 * pad) / stride + 1;
}

}  // namespace

OpRegistry::OpRegistry() {
  OpRegistry* r = this;

  // ---- unary math --------------------------------------------------------------------------------
  for (const char* fn : {"sqrt", "tanh", "sigmoid", "exp", "erf", "rsqrt", "log", "log2", "log10", "floor", "ceil",
                         "round", "trunc", "sin", "cos", "tan", "sinh", "cosh", "asin", "acos", "atan", "asinh",
                         "acosh", "atanh", "cbrt"}) {
    RegisterUnaryMath(r, fn, fn);
  }
  RegisterUnaryPredicate(r, "isnan", "isnan");
  RegisterUnaryPredicate(r, "isinf", "isinf");
  RegisterUnaryPredicate(r, "isfinite", "isfinite");

  auto unary = [&](const std::string& name,
                   std::function<Expr(const Expr&, const AttributeMap&, const Type&)> emit) -> Operator& {
    auto& op       = r->Register(name);
    op.pattern     = OpPatternKind::kElementWise;
    op.infer_shape = SameShapeAsFirst;
    op.infer_dtype = SameTypeAsFirst;
    op.compute     = [emit](const std::vector<Expr>& in, const AttributeMap& attrs, const Type& out) {
      return emit(in[0], attrs, out);
    };
    return op;
  };
  // relu(x) = max(x, 0)   (cinn/hlir/pe/nn.cc:61-64 over lang::Relu)
  unary("relu", [](const Expr& x, const AttributeMap&, const Type& t) { return ir::Max(x, ir::MakeConst(t, 0)); });
  // relu6(x) = min(max(x, 0), threshold)
  unary("relu6", [](const Expr& x, const AttributeMap& a, const Type& t) {
    return ir::Min(ir::Max(x, ir::MakeConst(t, 0)), ir::MakeConst(t, GetAttr<float>(a, "threshold", 6.0f)));
  });
  unary("identity", [](const Expr& x, const AttributeMap&, const Type&) { return x; });
  unary("negative", [](const Expr& x, const AttributeMap&, const Type&) { return ir::MakeMinus(x); });
  unary("reciprocal", [](const Expr& x, const AttributeMap&, const Type& t) { return ir::MakeConst(t, 1) / x; });
  unary("abs", [](const Expr& x, const AttributeMap&, const Type& t) {
    if (t.is_floating()) return CallExtern("abs", t, {x}, t);
    return ir::MakeSelect(x < ir::MakeConst(t, 0), ir::MakeMinus(x), x);
  });
  unary("sign", [](const Expr& x, const AttributeMap&, const Type& t) {
    Expr zero = ir::MakeConst(t, 0);
    return ir::MakeSelect(x > zero, ir::MakeConst(t, 1), ir::MakeSelect(x < zero, ir::MakeConst(t, -1), zero));
  });
  // gelu(x) = x * (0.5 + 0.5 * erf(x * sqrt(0.5)))   (cinn/frontend/decomposer/activation.cc:52-67)
  unary("gelu", [](const Expr& x, const AttributeMap&, const Type& t) {
    Expr half = ir::MakeConst(t, 0.5);
    Expr erf  = CallExtern("erf", t, {x * ir::MakeConst(t, std::sqrt(0.5))}, t);
    return x * (half + half * erf);
  });
  unary("logical_not", [](const Expr& x, const AttributeMap&, const Type&) { return ir::MakeNot(x); }).infer_dtype =
      BoolType;
  unary("bitwise_not", [](const Expr& x, const AttributeMap&, const Type& t) {
    return CallExtern("bitwise_not", t, {x}, t);
  });
  unary("clz", [](const Expr& x, const AttributeMap&, const Type& t) { return CallExtern("clz", t, {x}, t); });
  unary("popc", [](const Expr& x, const AttributeMap&, const Type& t) { return CallExtern("popc", t, {x}, t); });
  // scale: x * scale + bias, or (x + bias) * scale   (cinn/hlir/op/elementwise.cc StrategyForScale)
  unary("scale", [](const Expr& x, const AttributeMap& a, const Type& t) {
    Expr scale = ir::MakeConst(t, GetAttr<float>(a, "scale", 1.0f));
    Expr bias  = ir::MakeConst(t, GetAttr<float>(a, "bias", 0.0f));
    if (GetAttr<bool>(a, "bias_after_scale", true)) return x * scale + bias;
    return (x + bias) * scale;
  });
  {
    auto& op       = unary("cast", [](const Expr& x, const AttributeMap&, const Type& t) { return ir::MakeCast(t, x); });
    op.infer_dtype = [](const std::vector<Type>&, const AttributeMap& a) {
      return std::vector<Type>{common::Str2Type(GetAttr<std::string>(a, "dtype", "float32"))};
    };
  }

  // ---- binary ------------------------------------------------------------------------------------
  RegisterBinary(r, "elementwise_add", [](const Expr& a, const Expr& b, const Type&) { return a + b; });
  RegisterBinary(r, "subtract", [](const Expr& a, const Expr& b, const Type&) { return a - b; });
  RegisterBinary(r, "elementwise_mul", [](const Expr& a, const Expr& b, const Type&) { return a * b; });
  RegisterBinary(r, "divide", [](const Expr& a, const Expr& b, const Type&) { return a / b; });
  RegisterBinary(r, "floor_divide", [](const Expr& a, const Expr& b, const Type& t) {
    if (t.is_floating()) return CallExtern("floor", t, {a / b}, t);
    // floor division of integers: truncate, then step down when the signs differ and there is a remainder
    Expr q = a / b;
    Expr m = a % b;
    Expr zero = ir::MakeConst(t, 0);
    return ir::MakeSelect((m != zero) && ((m < zero) != (b < zero)), q - ir::MakeConst(t, 1), q);
  });
  auto mod_emit = [](const Expr& a, const Expr& b, const Type& t) { return CallExtern("mod", t, {a, b}, t); };
  RegisterBinary(r, "mod", mod_emit);
  RegisterBinary(r, "remainder", mod_emit);
  RegisterBinary(r, "max", [](const Expr& a, const Expr& b, const Type&) { return ir::Max(a, b); });
  RegisterBinary(r, "min", [](const Expr& a, const Expr& b, const Type&) { return ir::Min(a, b); });
  RegisterBinary(r, "pow", [](const Expr& a, const Expr& b, const Type& t) { return CallExtern("pow", t, {a, b}, t); });
  RegisterBinary(r, "logical_and", [](const Expr& a, const Expr& b, const Type&) { return a && b; });
  RegisterBinary(r, "logical_or", [](const Expr& a, const Expr& b, const Type&) { return a || b; });
  RegisterBinary(r, "logical_xor", [](const Expr& a, const Expr& b, const Type&) { return a != b; });
  for (const char* fn : {"bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift", "logical_right_shift"}) {
    std::string f = fn;
    RegisterBinary(r, f, [f](const Expr& a, const Expr& b, const Type& t) { return CallExtern(f, t, {a, b}, t); });
  }
  RegisterBinary(r, "equal", [](const Expr& a, const Expr& b, const Type&) { return a == b; }, true);
  RegisterBinary(r, "not_equal", [](const Expr& a, const Expr& b, const Type&) { return a != b; }, true);
  RegisterBinary(r, "greater_than", [](const Expr& a, const Expr& b, const Type&) { return a > b; }, true);
  RegisterBinary(r, "less_than", [](const Expr& a, const Expr& b, const Type&) { return a < b; }, true);
  RegisterBinary(r, "greater_equal", [](const Expr& a, const Expr& b, const Type&) { return a >= b; }, true);
  RegisterBinary(r, "less_equal", [](const Expr& a, const Expr& b, const Type&) { return a <= b; }, true);

  {
    auto& op       = r->Register("select");
    op.pattern     = OpPatternKind::kElementWise;
    op.num_inputs  = 3;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      CINN_CHECK(in[0] == in[1] && in[1] == in[2]) << "select: operands must have the same shape";
      return std::vector<ShapeType>{in[1]};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) { return std::vector<Type>{in[1]}; };
    op.compute     = [](const std::vector<Expr>& in, const AttributeMap&, const Type&) {
      return ir::MakeSelect(in[0], in[1], in[2]);
    };
  }
  {
    // sum of N equally shaped operands, added left to right
    auto& op       = r->Register("sum");
    op.pattern     = OpPatternKind::kElementWise;
    op.num_inputs  = -1;
    op.infer_shape = SameShapeAsFirst;
    op.infer_dtype = SameTypeAsFirst;
    op.compute     = [](const std::vector<Expr>& in, const AttributeMap&, const Type&) {
      Expr acc = in[0];
      for (size_t i = 1; i < in.size(); ++i) acc = acc + in[i];
      return acc;
    };
  }
  {
    auto& op       = r->Register("fill_constant");
    op.pattern     = OpPatternKind::kElementWise;
    op.num_inputs  = 0;
    op.infer_shape = [](const std::vector<ShapeType>&, const AttributeMap& a) {
      return std::vector<ShapeType>{GetAttr<std::vector<int>>(a, "shape", {1})};
    };
    op.infer_dtype = [](const std::vector<Type>&, const AttributeMap& a) {
      return std::vector<Type>{common::Str2Type(GetAttr<std::string>(a, "dtype", "float32"))};
    };
    op.compute = [](const std::vector<Expr>&, const AttributeMap& a, const Type& t) {
      return ir::MakeConst(t, GetAttr<double>(a, "value", 0.0));
    };
  }

  // ---- index-transforming ops (the lowering maps indices; no scalar compute) -----------------------
  {
    auto& op       = r->Register("broadcast_to");
    op.pattern     = OpPatternKind::kBroadcast;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto out  = GetAttr<std::vector<int>>(a, "out_shape", {});
      auto axes = GetAttr<std::vector<int>>(a, "broadcast_axes", {});
      CINN_CHECK(!out.empty()) << "broadcast_to needs out_shape";
      CINN_CHECK_EQ(axes.size(), in[0].size()) << "broadcast_to: one axis per input dimension";
      for (size_t i = 0; i < axes.size(); ++i) {
        int ax = axes[i] < 0 ? axes[i] + static_cast<int>(out.size()) : axes[i];
        CINN_CHECK(ax >= 0 && ax < static_cast<int>(out.size())) << "broadcast axis out of range";
        CINN_CHECK(in[0][i] == 1 || in[0][i] == out[ax])
            << "broadcast_to: input dim " << in[0][i] << " does not match output dim " << out[ax];
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    auto& op       = r->Register("reshape");
    op.pattern     = OpPatternKind::kInjective;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto shape    = GetAttr<std::vector<int>>(a, "shape", {});
      int64_t numel = ShapeNumel(in[0]);
      int64_t known = 1;
      int infer_at  = -1;
      for (size_t i = 0; i < shape.size(); ++i) {
        if (shape[i] == -1) {
          CINN_CHECK_EQ(infer_at, -1) << "reshape: only one -1 allowed";
          infer_at = static_cast<int>(i);
        } else if (shape[i] == 0) {
          CINN_CHECK_LT(i, in[0].size());
          shape[i] = in[0][i];
          known *= shape[i];
        } else {
          known *= shape[i];
        }
      }
      if (infer_at >= 0) shape[infer_at] = static_cast<int>(numel / known);
      CINN_CHECK_EQ(ShapeNumel(shape), numel) << "reshape changes the number of elements";
      return std::vector<ShapeType>{shape};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    auto& op       = r->Register("transpose");
    op.pattern     = OpPatternKind::kInjective;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto axis = GetAttr<std::vector<int>>(a, "axis", {});
      CINN_CHECK_EQ(axis.size(), in[0].size()) << "transpose: axis must be a permutation of the input dims";
      ShapeType out;
      for (int ax : axis) {
        if (ax < 0) ax += static_cast<int>(in[0].size());
        out.push_back(in[0][ax]);
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    auto& op       = r->Register("slice");
    op.pattern     = OpPatternKind::kInjective;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto axes    = GetAttr<std::vector<int>>(a, "axes", {});
      auto starts  = GetAttr<std::vector<int>>(a, "starts", {});
      auto ends    = GetAttr<std::vector<int>>(a, "ends", {});
      auto strides = GetAttr<std::vector<int>>(a, "strides", {});
      ShapeType out = in[0];
      for (size_t i = 0; i < axes.size(); ++i) {
        int ax  = axes[i] < 0 ? axes[i] + static_cast<int>(in[0].size()) : axes[i];
        int dim = in[0][ax];
        int st  = i < strides.size() ? strides[i] : 1;
        CINN_CHECK_GT(st, 0) << "slice: only positive strides are supported";
        int s = starts[i] < 0 ? starts[i] + dim : starts[i];
        int e = ends[i] < 0 ? ends[i] + dim : ends[i];
        s     = std::min(std::max(s, 0), dim);
        e     = std::min(std::max(e, 0), dim);
        out[ax] = std::max(0, (e - s + st - 1) / st);
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    auto& op       = r->Register("concat");
    op.pattern     = OpPatternKind::kInjective;
    op.num_inputs  = -1;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      int axis = GetAttr<int>(a, "axis", 0);
      if (axis < 0) axis += static_cast<int>(in[0].size());
      ShapeType out = in[0];
      for (size_t i = 1; i < in.size(); ++i) out[axis] += in[i][axis];
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }

  // ---- reductions --------------------------------------------------------------------------------
  RegisterReduce(r, "reduce_sum", "sum");
  RegisterReduce(r, "reduce_prod", "prod");
  RegisterReduce(r, "reduce_max", "max");
  RegisterReduce(r, "reduce_min", "min");
  RegisterReduce(r, "reduce_all", "all");
  RegisterReduce(r, "reduce_any", "any");
  for (const char* kind : {"sum", "prod", "max", "min", "all", "any"})
    RegisterReduceRun(r, std::string("reduce_run_") + kind, kind);
  RegisterArgReduce(r, "argmax", "argmax");
  RegisterArgReduce(r, "argmin", "argmin");

  // ---- ops that the Decomposer rewrites into primitives before the graph is built -----------------
  {
    auto& op       = r->Register("softmax");
    op.pattern     = OpPatternKind::kNonFusible;
    op.infer_shape = SameShapeAsFirst;
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // inference form: inputs x, scale, bias, mean, variance -> y
    auto& op       = r->Register("batch_norm");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 5;
    op.infer_shape = SameShapeAsFirst;
    op.infer_dtype = SameTypeAsFirst;
  }

  {
    // relu_grad(dout, out) -> dx
    auto& op       = r->Register("relu_grad");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 2;
    op.infer_shape = SameShapeAsFirst;
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // elementwise_add_grad(dout, x, y) -> dx, dy with the shapes of x and y
    auto& op       = r->Register("elementwise_add_grad");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 3;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      return std::vector<ShapeType>{in[1], in[2]};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) { return std::vector<Type>{in[1], in[2]}; };
  }
  {
    // training form: x, scale, bias, moving_mean, moving_variance -> y, saved_mean, saved_variance, moving_mean,
    // moving_variance (cinn/hlir/op/nn.cc batch_norm_train)
    auto& op       = r->Register("batch_norm_train");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 5;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      return std::vector<ShapeType>{in[0], in[1], in[1], in[1], in[1]};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) {
      return std::vector<Type>{in[0], in[1], in[1], in[1], in[1]};
    };
  }
  {
    // dy, x, scale, save_mean, save_variance -> x_grad, scale_grad, bias_grad (cinn/hlir/op/nn.cc batch_norm_grad)
    auto& op       = r->Register("batch_norm_grad");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 5;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      CINN_CHECK(in[0] == in[1]) << "batch_norm_grad: dy and x differ in shape";
      return std::vector<ShapeType>{in[1], in[2], in[2]};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) {
      return std::vector<Type>{in[1], in[2], in[2]};
    };
  }

  // ---- library-backed ops ------------------------------------------------------------------------
  {
    // row-major matmul with numpy batch broadcasting; output shape as NetBuilder::GetMatmulOutputShape
    auto& op       = r->Register("matmul");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 2;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      bool tx = GetAttr<bool>(a, "trans_a", false), ty = GetAttr<bool>(a, "trans_b", false);
      ShapeType x = in[0], y = in[1];
      CINN_CHECK(!x.empty() && !y.empty());
      bool x1d = x.size() == 1, y1d = y.size() == 1;
      if (x1d) x = tx ? ShapeType{x[0], 1} : ShapeType{1, x[0]};
      if (y1d) y = ty ? ShapeType{1, y[0]} : ShapeType{y[0], 1};
      int xr = static_cast<int>(x.size()), yr = static_cast<int>(y.size());
      int m = tx ? x[xr - 1] : x[xr - 2], kx = tx ? x[xr - 2] : x[xr - 1];
      int ky = ty ? y[yr - 1] : y[yr - 2], n = ty ? y[yr - 2] : y[yr - 1];
      CINN_CHECK_EQ(kx, ky) << "matmul: inner dimensions differ";
      ShapeType batch;
      int br = std::max(xr, yr) - 2;
      for (int i = 0; i < br; ++i) {
        int xi = i - (br - (xr - 2)), yi = i - (br - (yr - 2));
        int xd = xi >= 0 ? x[xi] : 1, yd = yi >= 0 ? y[yi] : 1;
        CINN_CHECK(xd == yd || xd == 1 || yd == 1) << "matmul: batch dims do not broadcast";
        batch.push_back(std::max(xd, yd));
      }
      ShapeType out = batch;
      if (!x1d) out.push_back(m);
      if (!y1d) out.push_back(n);
      if (out.empty()) out.push_back(1);
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // mul (fc): x flattened at x_num_col_dims times y flattened at y_num_col_dims.  y is [K, N]; with is_infer it
    // is the transposed weight [N, K] and the output takes y's leading dims (GetMulNewShapes,
    // cinn/hlir/pe/transform.cc:186-250; InferShapeForMul, cinn/hlir/op/transform.cc:592-621)
    auto& op       = r->Register("mul");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 2;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      int xn = GetAttr<int>(a, "x_num_col_dims", 1), yn = GetAttr<int>(a, "y_num_col_dims", 1);
      bool is_infer = GetAttr<bool>(a, "is_infer", false);
      CINN_CHECK(in[0].size() >= 2 && in[1].size() >= 2) << "mul: operands need at least two dimensions";
      if (xn < 0) xn += static_cast<int>(in[0].size());
      if (yn < 0) yn += static_cast<int>(in[1].size());
      CINN_CHECK(xn > 0 && xn < static_cast<int>(in[0].size())) << "mul: x_num_col_dims out of range";
      CINN_CHECK(yn > 0 && yn < static_cast<int>(in[1].size())) << "mul: y_num_col_dims out of range";
      ShapeType out(in[0].begin(), in[0].begin() + xn);
      int64_t kx = 1, y_lead = 1, y_trail = 1;
      for (size_t i = xn; i < in[0].size(); ++i) kx *= in[0][i];
      for (int i = 0; i < yn; ++i) y_lead *= in[1][i];
      for (size_t i = yn; i < in[1].size(); ++i) y_trail *= in[1][i];
      if (is_infer) {
        out.insert(out.end(), in[1].begin(), in[1].begin() + yn);
        CINN_CHECK_EQ(kx, y_trail) << "mul (is_infer): the K dimensions of x and the transposed y differ";
      } else {
        out.insert(out.end(), in[1].begin() + yn, in[1].end());
        CINN_CHECK_EQ(kx, y_lead) << "mul: flattened inner dimensions differ";
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    auto& op       = r->Register("conv2d");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 2;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto stride   = GetAttr<std::vector<int>>(a, "stride", {1, 1});
      auto padding  = GetAttr<std::vector<int>>(a, "padding", {0, 0});
      auto dilation = GetAttr<std::vector<int>>(a, "dilation", {1, 1});
      auto layout   = GetAttr<std::string>(a, "data_format", "NCHW");
      CINN_CHECK(in[0].size() == 4 && in[1].size() == 4) << "conv2d: 4-D input and filter expected";
      CINN_CHECK(layout == "NCHW" || layout == "NHWC") << "conv2d: unknown data_format " << layout;
      ShapeType out(4);
      // the gradients (InferShapeForConv2d, cinn/hlir/op/nn.cc:529-552): backward_data takes (w, dy) and gives dx with
      // the spatial extents of `output_shape`; backward_filter takes (x, dy) and gives dw with those of `output_shape`
      auto conv_type = GetAttr<std::string>(a, "conv_type", "forward");
      CINN_CHECK(conv_type == "forward" || conv_type == "backward_data" || conv_type == "backward_filter")
          << "The conv type should be one of {forward, backward_data, backward_filter}.";
      if (conv_type != "forward") {
        auto wanted = GetAttr<std::vector<int>>(a, "output_shape", {});
        CINN_CHECK_EQ(wanted.size(), 4u) << "conv2d " << conv_type << ": output_shape must have rank 4";
        int groups = GetAttr<int>(a, "groups", 1);
        int c = layout == "NCHW" ? 1 : 3, h = layout == "NCHW" ? 2 : 1, w = h + 1;
        if (conv_type == "backward_data") {
          out[0] = in[1][0];
          out[c] = in[0][c] * groups;
        } else {
          out[0] = in[1][c];
          out[c] = in[0][c] / groups;
        }
        out[h] = wanted[h];
        out[w] = wanted[w];
        return std::vector<ShapeType>{out};
      }
      // "input_layout" = "NCHW" on a channels-last convolution: the input (and the [O][I][KH][KW] filter) are still
      // NCHW, only the output is NHWC (the convolution of a network's image input)
      bool nchw_input = GetAttr<std::string>(a, "input_layout", layout) == "NCHW";
      if (layout == "NCHW") {
        out[0] = in[0][0];
        out[1] = in[1][0];
        out[2] = ConvOutDim(in[0][2], padding[0], dilation[0], in[1][2], stride[0]);
        out[3] = ConvOutDim(in[0][3], padding[1], dilation[1], in[1][3], stride[1]);
      } else if (nchw_input) {
        out[0] = in[0][0];
        out[1] = ConvOutDim(in[0][2], padding[0], dilation[0], in[1][2], stride[0]);
        out[2] = ConvOutDim(in[0][3], padding[1], dilation[1], in[1][3], stride[1]);
        out[3] = in[1][0];
      } else {
        // channels-last filters are [O][KH][KW][I] (InferShapeForConv2d reads h / w at 1 / 2, cinn/hlir/op/nn.cc:510-527)
        out[0] = in[0][0];
        out[1] = ConvOutDim(in[0][1], padding[0], dilation[0], in[1][1], stride[0]);
        out[2] = ConvOutDim(in[0][2], padding[1], dilation[1], in[1][2], stride[1]);
        out[3] = in[1][0];
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // conv2d followed by a per-channel affine, an optional residual addition and an optional relu, produced by
    // the conv+bn+relu graph rewrite; inputs x, w, scale, shift[, residual]
    auto& op       = r->Register("hip_conv2d_bn_relu");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = -1;
    const auto* cv = r->Find("conv2d");
    auto conv_shape = cv->infer_shape;
    op.infer_shape = [conv_shape](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto out = conv_shape({in[0], in[1]}, a);
      if (GetAttr<bool>(a, "max_pool", false)) {
        // the 3x3 / stride 2 / padding 1 max pooling folded into an image convolution (channels-last output)
        out[0][1] = (out[0][1] + 2 - 3) / 2 + 1;
        out[0][2] = (out[0][2] + 2 - 3) / 2 + 1;
      }
      return out;
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // two 1x1 channels-last convolutions in a row, each with hip_conv2d_bn_relu's epilogue, produced by the
    // FuseConvChain rewrite; inputs x, w1, scale1, shift1, [residual,] w2, scale2, shift2; outputs e (the first
    // convolution's result) and y
    auto& op       = r->Register("hip_conv2d_bn_relu_chain");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = -1;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      CINN_CHECK(in.size() == 7u || in.size() == 8u) << "hip_conv2d_bn_relu_chain takes 7 or 8 operands";
      const size_t w2 = in.size() == 8u ? 5 : 4;
      CINN_CHECK(in[0].size() == 4u && in[1].size() == 4u && in[w2].size() == 4u) << "hip_conv2d_bn_relu_chain: 4-D operands expected";
      CINN_CHECK(in[1][1] == 1 && in[1][2] == 1 && in[w2][1] == 1 && in[w2][2] == 1 && in[1][3] == in[0][3] && in[w2][3] == in[1][0])
          << "hip_conv2d_bn_relu_chain: [O][1][1][I] filters whose channel counts follow one another expected";
      ShapeType e = {in[0][0], in[0][1], in[0][2], in[1][0]};
      ShapeType y = {in[0][0], in[0][1], in[0][2], in[w2][0]};
      return std::vector<ShapeType>{e, y};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) { return std::vector<Type>{in[0], in[0]}; };
  }
  {
    // a 1x1 channels-last convolution over the channels of two inputs that share the output's pixel grid (the second
    // one sampled at `second_stride`), produced by the FuseShortcutProjection rewrite; inputs x, x2, w
    // [O][1][1][C1 + C2], shift [O]
    auto& op       = r->Register("hip_conv2d_pointwise_pair");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 4;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      CINN_CHECK_EQ(in.size(), 4u) << "hip_conv2d_pointwise_pair takes x, x2, w and shift";
      CINN_CHECK(in[0].size() == 4u && in[1].size() == 4u && in[2].size() == 4u && in[3].size() == 1u)
          << "hip_conv2d_pointwise_pair: 4-D tensors and a 1-D shift expected";
      auto stride = GetAttr<std::vector<int>>(a, "second_stride", {1, 1});
      CINN_CHECK(stride.size() == 2u && stride[0] > 0 && stride[1] > 0) << "hip_conv2d_pointwise_pair: second_stride takes two positive values";
      CINN_CHECK(in[2][1] == 1 && in[2][2] == 1 && in[2][3] == in[0][3] + in[1][3] && in[3][0] == in[2][0] && in[1][0] == in[0][0])
          << "hip_conv2d_pointwise_pair: a [O][1][1][C1 + C2] filter, an [O] shift and inputs of one batch size expected";
      CINN_CHECK((in[0][1] - 1) * stride[0] < in[1][1] && (in[0][2] - 1) * stride[1] < in[1][2])
          << "hip_conv2d_pointwise_pair: the output grid at the second input's stride leaves that input";
      return std::vector<ShapeType>{{in[0][0], in[0][1], in[0][2], in[2][0]}};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // hip_conv2d_bn_relu_chain whose first layer reads a second input of the same pixel grid instead of adding a
    // residual (FuseShortcutProjection); inputs x, x2, w1 [M][1][1][C1 + C2], shift1, w2, scale2, shift2; outputs e, y
    auto& op       = r->Register("hip_conv2d_pair_chain");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 7;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      CINN_CHECK_EQ(in.size(), 7u) << "hip_conv2d_pair_chain takes x, x2, w1, shift1, w2, scale2, shift2";
      CINN_CHECK(in[0].size() == 4u && in[1].size() == 4u && in[2].size() == 4u && in[4].size() == 4u) << "hip_conv2d_pair_chain: 4-D operands expected";
      CINN_CHECK(in[1][0] == in[0][0] && in[1][1] == in[0][1] && in[1][2] == in[0][2]) << "hip_conv2d_pair_chain: both inputs cover the same pixels";
      CINN_CHECK(in[2][1] == 1 && in[2][2] == 1 && in[4][1] == 1 && in[4][2] == 1 && in[2][3] == in[0][3] + in[1][3] && in[4][3] == in[2][0])
          << "hip_conv2d_pair_chain: [M][1][1][C1 + C2] and [O][1][1][M] filters expected";
      ShapeType e = {in[0][0], in[0][1], in[0][2], in[2][0]};
      ShapeType y = {in[0][0], in[0][1], in[0][2], in[4][0]};
      return std::vector<ShapeType>{e, y};
    };
    op.infer_dtype = [](const std::vector<Type>& in, const AttributeMap&) { return std::vector<Type>{in[0], in[0]}; };
  }
  {
    // cinn/hlir/op/contrib/sort.cc:307-350: both keep the operand's shape; argsort has two int32 outputs (indices,
    // positions), sort one of the operand's type
    auto check_axis = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      CINN_CHECK_EQ(in.size(), 1u) << "sort / argsort take one operand";
      int axis = GetAttr<int>(a, "axis", 0);
      if (axis < 0) axis += static_cast<int>(in[0].size());
      CINN_CHECK(axis >= 0 && axis < static_cast<int>(in[0].size())) << "sort / argsort: axis " << axis << " out of range";
    };
    auto& arg       = r->Register("argsort");
    arg.pattern     = OpPatternKind::kNonFusible;
    arg.infer_shape = [check_axis](const std::vector<ShapeType>& in, const AttributeMap& a) {
      check_axis(in, a);
      return std::vector<ShapeType>{in[0], in[0]};
    };
    arg.infer_dtype = [](const std::vector<Type>&, const AttributeMap&) { return std::vector<Type>{common::Int(32), common::Int(32)}; };
    auto& srt       = r->Register("sort");
    srt.pattern     = OpPatternKind::kNonFusible;
    srt.infer_shape = [check_axis](const std::vector<ShapeType>& in, const AttributeMap& a) {
      check_axis(in, a);
      return std::vector<ShapeType>{in[0]};
    };
    srt.infer_dtype = SameTypeAsFirst;
  }
  {
    // pooling output size and attribute meaning as cinn/hlir/pe/nn.cc:956-1109 (PoolImpl)
    auto& op       = r->Register("pool2d");
    op.pattern     = OpPatternKind::kNonFusible;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap& a) {
      auto ksize     = GetAttr<std::vector<int>>(a, "kernel_size", {1, 1});
      auto stride    = GetAttr<std::vector<int>>(a, "stride_size", {1, 1});
      auto padding   = GetAttr<std::vector<int>>(a, "padding_size", {0, 0, 0, 0});
      bool ceil_mode = GetAttr<bool>(a, "ceil_mode", false);
      bool global    = GetAttr<bool>(a, "global_pooling", false);
      bool adaptive  = GetAttr<bool>(a, "adaptive", false);
      auto layout    = GetAttr<std::string>(a, "data_format", "NCHW");
      CINN_CHECK_EQ(in[0].size(), 4u) << "pool2d: 4-D input expected";
      int hi = layout == "NCHW" ? 2 : 1, wi = hi + 1;
      if (padding.size() == 2) padding = {padding[0], padding[1], padding[0], padding[1]};
      ShapeType out = in[0];
      if (global) {
        out[hi] = out[wi] = 1;
      } else if (adaptive) {
        out[hi] = ksize[0];
        out[wi] = ksize[1];
      } else {
        auto od = [&](int n, int k, int p0, int p1, int s) {
          int num = n - k + p0 + p1;
          return (ceil_mode ? (num + s - 1) / s : num / s) + 1;
        };
        out[hi] = od(in[0][hi], ksize[0], padding[0], padding[2], stride[0]);
        out[wi] = od(in[0][wi], ksize[1], padding[1], padding[3], stride[1]);
      }
      return std::vector<ShapeType>{out};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
  {
    // inputs x, y = pool2d(x), dy; the gradient has x's shape (cinn/hlir/op/nn.cc pool2d_grad)
    auto& op       = r->Register("pool2d_grad");
    op.pattern     = OpPatternKind::kNonFusible;
    op.num_inputs  = 3;
    op.infer_shape = [](const std::vector<ShapeType>& in, const AttributeMap&) {
      CINN_CHECK(in[0].size() == 4 && in[1].size() == 4 && in[2].size() == 4) << "pool2d_grad: x, y and dy must be 4-D";
      int64_t ny = 1, ndy = 1;
      for (int d : in[1]) ny *= d;
      for (int d : in[2]) ndy *= d;
      CINN_CHECK(ndy >= ny) << "pool2d_grad: dy holds fewer elements than y";
      return std::vector<ShapeType>{in[0]};
    };
    op.infer_dtype = SameTypeAsFirst;
  }
}

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
