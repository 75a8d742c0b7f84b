#include "common/type.h"

namespace cinn {
namespace common {

std::string Type2Str(const Type& t) {
  if (t.is_bool()) return "bool";
  switch (t.code) {
    case Type::Code::Int: return "int" + std::to_string(t.bits);
    case Type::Code::UInt: return "uint" + std::to_string(t.bits);
    case Type::Code::Float: return "float" + std::to_string(t.bits);
    case Type::Code::BFloat: return "bfloat16";
    case Type::Code::Handle: return "void*";
    case Type::Code::String: return "string";
    default: return "unk";
  }
}

Type Str2Type(const std::string& s) {
  if (s == "bool") return Bool();
  if (s == "bfloat16") return BFloat16();
  if (s == "float16") return Float16();
  if (s == "float32" || s == "float") return Float(32);
  if (s == "float64" || s == "double") return Float(64);
  if (s == "int8") return Int(8);
  if (s == "int16") return Int(16);
  if (s == "int32" || s == "int") return Int(32);
  if (s == "int64") return Int(64);
  if (s == "uint8") return UInt(8);
  if (s == "uint16") return UInt(16);
  if (s == "uint32") return UInt(32);
  if (s == "uint64") return UInt(64);
  CINN_CHECK(false) << "unknown type string '" << s << "'";
  return Type();
}

std::string TypeSuffix(const Type& t) {
  if (t.is_bool()) return "bool";
  if (t.is_bfloat16()) return "bf16";
  if (t.code == Type::Code::Float) return "fp" + std::to_string(t.bits);
  if (t.code == Type::Code::Int) return "int" + std::to_string(t.bits);
  if (t.code == Type::Code::UInt) return "uint" + std::to_string(t.bits);
  CINN_CHECK(false) << "no device-library suffix for type " << Type2Str(t);
  return "";
}

std::string TypeCName(const Type& t) {
  if (t.is_bool()) return "bool";
  if (t.is_bfloat16()) return "bfloat16";
  if (t.code == Type::Code::Float) {
    if (t.bits == 16) return "float16";
    if (t.bits == 32) return "float";
    if (t.bits == 64) return "double";
  }
  if (t.code == Type::Code::Int) return "int" + std::to_string(t.bits) + "_t";
  if (t.code == Type::Code::UInt) return "uint" + std::to_string(t.bits) + "_t";
  if (t.code == Type::Code::Handle) return "void*";
  CINN_CHECK(false) << "no C name for type " << Type2Str(t);
  return "";
}

}  // namespace common
}  // namespace cinn
