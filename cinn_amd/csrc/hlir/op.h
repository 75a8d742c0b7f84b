// Operator registry of the high-level graph: for every op name its fusion pattern, shape / dtype
// inference and - for element-wise ops - the scalar compute emitter.  It condenses what the reference
// spreads over cinn/hlir/op/*.cc (CINN_REGISTER_OP with infershape / inferdtype / OpPattern and a
// CINNStrategy) and cinn/hlir/pe/*.cc (the compute definitions), keeping the arithmetic of the
// compute definitions; the GPU schedule side lives in hlir/lowering.cc.
#pragma once
#include <functional>
#include <string>
#include <vector>

#include "frontend/syntax.h"
#include "ir/ir.h"

namespace cinn {
namespace hlir {
namespace framework {

using utils::AttributeMap;
using utils::ShapeType;

// same numbering as cinn/hlir/framework/op.h OpPatternKind
enum class OpPatternKind : int {
  kElementWise = 0,
  kBroadcast   = 1,
  kInjective   = 2,
  kReduction   = 3,
  kOutFusible  = 4,
  kNonFusible  = 8
};

struct Operator {
  std::string name;
  OpPatternKind pattern{OpPatternKind::kNonFusible};
  int num_inputs{1};  // -1: variadic
  int num_outputs{1};
  std::function<std::vector<ShapeType>(const std::vector<ShapeType>&, const AttributeMap&)> infer_shape;
  std::function<std::vector<common::Type>(const std::vector<common::Type>&, const AttributeMap&)> infer_dtype;
  // kElementWise: inputs are scalars at the same position of equally shaped operands
  std::function<ir::Expr(const std::vector<ir::Expr>&, const AttributeMap&, const common::Type&)> compute;
  // kReduction: "sum" "prod" "max" "min" "all" "any" "argmax" "argmin"
  std::string reduce_kind;
};

class OpRegistry {
 public:
  static OpRegistry& Global();
  const Operator* Find(const std::string& name) const;
  const Operator& Get(const std::string& name) const;
  Operator& Register(const std::string& name);
  std::vector<std::string> ListAllNames() const;

 private:
  OpRegistry();
  std::vector<std::unique_ptr<Operator>> ops_;
};

template <typename T>
T GetAttr(const AttributeMap& attrs, const std::string& key, const T& dflt) {
  auto it = attrs.find(key);
  if (it == attrs.end()) return dflt;
  if (std::holds_alternative<T>(it->second)) return std::get<T>(it->second);
  // tolerate int <-> float <-> double <-> bool spellings coming from bindings
  if constexpr (std::is_arithmetic_v<T>) {
    if (auto* p = std::get_if<int>(&it->second)) return static_cast<T>(*p);
    if (auto* p = std::get_if<float>(&it->second)) return static_cast<T>(*p);
    if (auto* p = std::get_if<double>(&it->second)) return static_cast<T>(*p);
    if (auto* p = std::get_if<bool>(&it->second)) return static_cast<T>(*p);
  }
  CINN_CHECK(false) << "attribute '" << key << "' has an unexpected type";
  return dflt;
}

// name of a device-library function: cinn_hip_<fn>_<type suffix>; the counterpart of the
// cinn_nvgpu_ naming of cinn/hlir/op/op_util.cc:110-167
std::string ExternFuncName(const std::string& fn, const common::Type& type);

int64_t ShapeNumel(const ShapeType& s);

}  // namespace framework
}  // namespace hlir
}  // namespace cinn
