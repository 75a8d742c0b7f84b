// Scalar / vector element types of the IR.  The (code, bits) pair uses the same numbering as the
// runtime tag cinn_type_t (cinn/runtime/cinn_runtime.h:51-93) so a Type maps 1:1 onto the ABI;
// the API mirrors cinn/common/type.h (Float(32), Int(32), Bool(), Type2Str / Str2Type names).
#pragma once
#include <cstdint>
#include <string>

#include "common/check.h"

namespace cinn {
namespace common {

struct Type {
  enum class Code : int { Unk = -1, Int = 0, UInt = 1, Float = 2, Handle = 3, BFloat = 4, String = 5 };
  Code code{Code::Unk};
  int bits{0};
  int lanes{1};

  Type() = default;
  Type(Code c, int b, int l = 1) : code(c), bits(b), lanes(l) {}

  bool valid() const { return code != Code::Unk; }
  bool is_bool() const { return code == Code::UInt && bits == 1; }
  bool is_int(int b = -1) const { return code == Code::Int && (b < 0 || b == bits); }
  bool is_uint(int b = -1) const { return code == Code::UInt && (b < 0 || b == bits); }
  bool is_float(int b = -1) const { return code == Code::Float && (b < 0 || b == bits); }
  bool is_float16() const { return code == Code::Float && bits == 16; }
  bool is_bfloat16() const { return code == Code::BFloat; }
  bool is_floating() const { return code == Code::Float || code == Code::BFloat; }
  bool is_integer() const { return (code == Code::Int || code == Code::UInt) && !is_bool(); }
  bool is_handle() const { return code == Code::Handle; }
  bool is_string() const { return code == Code::String; }
  int bytes() const { return is_bool() ? 1 : (bits + 7) / 8; }
  Type ElementOf() const { return Type(code, bits, 1); }
  Type with_lanes(int l) const { return Type(code, bits, l); }
  bool operator==(const Type& o) const { return code == o.code && bits == o.bits && lanes == o.lanes; }
  bool operator!=(const Type& o) const { return !(*this == o); }
};

inline Type Int(int bits, int lanes = 1) { return Type(Type::Code::Int, bits, lanes); }
inline Type UInt(int bits, int lanes = 1) { return Type(Type::Code::UInt, bits, lanes); }
inline Type Float(int bits, int lanes = 1) { return Type(Type::Code::Float, bits, lanes); }
inline Type BFloat16(int lanes = 1) { return Type(Type::Code::BFloat, 16, lanes); }
inline Type Float16(int lanes = 1) { return Float(16, lanes); }
inline Type Bool(int lanes = 1) { return Type(Type::Code::UInt, 1, lanes); }
inline Type Handle() { return Type(Type::Code::Handle, 64); }
inline Type String() { return Type(Type::Code::String, 64); }

// "float32", "int64", "bool", "bfloat16", ... (cinn/common/type.cc Type2Str / Str2Type spellings)
std::string Type2Str(const Type& t);
Type Str2Type(const std::string& s);
// suffix used in device-library function names: fp32 fp64 fp16 bf16 int32 int64 int8 int16 uint8 bool
std::string TypeSuffix(const Type& t);
// C spelling in generated HIP source
std::string TypeCName(const Type& t);

}  // namespace common
}  // namespace cinn
