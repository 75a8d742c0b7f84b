// The loop-level IR the gfx950 device codegen consumes.  It mirrors the subset of CINN IR that
// reaches a device code generator (node kinds of cinn/ir/ir_base.h:54-118 after schedule blocks and
// Reduce nodes are gone; ForType / BindInfo of cinn/ir/ir.h:613-656; MemoryType of
// cinn/ir/ir_base.h:453-466; _LoweredFunc_ with cuda_axis_info of cinn/ir/lowered_func.h:84-198).
// Indices are flat: every buffer is addressed by one linear element offset.
#pragma once
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "common/check.h"
#include "common/target.h"
#include "common/type.h"

namespace cinn {
namespace ir {

using common::Type;

enum class IrNodeTy {
  IntImm,
  UIntImm,
  FloatImm,
  StringImm,
  Var,
  Add,
  Sub,
  Mul,
  Div,
  Mod,
  Min,
  Max,
  EQ,
  NE,
  LT,
  LE,
  GT,
  GE,
  And,
  Or,
  Minus,
  Not,
  Cast,
  Select,
  Load,
  Store,
  Ramp,
  Call,
  Let,
  For,
  IfThenElse,
  Block,
};

struct IrNode {
  IrNodeTy node_type;
  Type type;
  IrNode(IrNodeTy t, Type ty) : node_type(t), type(ty) {}
  virtual ~IrNode() = default;
};

class Expr {
 public:
  Expr() = default;
  explicit Expr(std::shared_ptr<IrNode> p) : p_(std::move(p)) {}
  Expr(int v);      // NOLINT: int32 immediate
  Expr(int64_t v);  // NOLINT
  Expr(float v);    // NOLINT
  Expr(double v);   // NOLINT
  Expr(bool v);     // NOLINT

  bool defined() const { return p_ != nullptr; }
  IrNode* get() const { return p_.get(); }
  IrNode* operator->() const { return p_.get(); }
  IrNodeTy node_type() const { return p_->node_type; }
  const Type& type() const { return p_->type; }
  template <typename T>
  T* As() const {
    return (p_ && p_->node_type == T::kNodeTy) ? static_cast<T*>(p_.get()) : nullptr;
  }
  bool is_constant() const;
  // value of an Int/UInt immediate; check-fails on anything else
  int64_t as_int64() const;
  bool is_int_imm(int64_t v) const;

 private:
  std::shared_ptr<IrNode> p_;
};

struct IntImm : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::IntImm;
  int64_t value;
  IntImm(Type t, int64_t v) : IrNode(kNodeTy, t), value(v) {}
};
struct UIntImm : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::UIntImm;
  uint64_t value;
  UIntImm(Type t, uint64_t v) : IrNode(kNodeTy, t), value(v) {}
};
struct FloatImm : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::FloatImm;
  double value;
  FloatImm(Type t, double v) : IrNode(kNodeTy, t), value(v) {}
};
struct StringImm : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::StringImm;
  std::string value;
  explicit StringImm(std::string v) : IrNode(kNodeTy, common::String()), value(std::move(v)) {}
};
struct Var : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Var;
  std::string name;
  Var(std::string n, Type t) : IrNode(kNodeTy, t), name(std::move(n)) {}
};

// Add .. Or share one layout; node_type tells them apart.
struct Binary : IrNode {
  Expr a, b;
  Binary(IrNodeTy ty, Type t, Expr x, Expr y) : IrNode(ty, t), a(std::move(x)), b(std::move(y)) {}
};
struct Unary : IrNode {  // Minus, Not
  Expr v;
  Unary(IrNodeTy ty, Type t, Expr x) : IrNode(ty, t), v(std::move(x)) {}
};
struct Cast : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Cast;
  Expr v;
  Cast(Type t, Expr x) : IrNode(kNodeTy, t), v(std::move(x)) {}
};
struct Select : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Select;
  Expr condition, true_value, false_value;
  Select(Expr c, Expr t, Expr f) : IrNode(kNodeTy, t.type()), condition(std::move(c)), true_value(t), false_value(std::move(f)) {}
};

enum class MemoryType { Global, GPUShared, GPULocal };

struct Buffer {
  std::string name;
  Type dtype;
  MemoryType memory_type{MemoryType::Global};
  int64_t num_elements{0};
  // global output that is written once and not re-read by this kernel: vector stores to it carry the
  // non-temporal hint so that they do not displace the data still being read
  bool streaming_store{false};
  bool streaming_load{false};  // read once by the kernel: vector loads bypass the cache allocation policy
  Buffer(std::string n, Type t, MemoryType m, int64_t size) : name(std::move(n)), dtype(t), memory_type(m), num_elements(size) {}
};
using BufferRef = std::shared_ptr<Buffer>;
inline BufferRef MakeBuffer(const std::string& name, Type t, MemoryType m, int64_t size) {
  return std::make_shared<Buffer>(name, t, m, size);
}

// base + i * stride for i in [0, lanes): the index of a vector access
struct Ramp : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Ramp;
  Expr base;
  int stride;
  int lanes;
  Ramp(Expr b, int s, int l) : IrNode(kNodeTy, b.type().with_lanes(l)), base(std::move(b)), stride(s), lanes(l) {}
};
struct Load : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Load;
  BufferRef buffer;
  Expr index;  // scalar offset or Ramp
  Load(BufferRef b, Expr idx);
};
struct Store : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Store;
  BufferRef buffer;
  Expr value;
  Expr index;
  Store(BufferRef b, Expr v, Expr idx) : IrNode(kNodeTy, Type()), buffer(std::move(b)), value(std::move(v)), index(std::move(idx)) {}
};

enum class CallType { Extern, Intrinsic };
struct Call : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Call;
  std::string name;
  std::vector<Expr> args;
  // buffers passed by name (device codegen prints the tensor identifier, as the reference does for
  // tensor arguments of extern calls, cinn/backends/codegen_cuda_dev.cc:275-316)
  std::vector<BufferRef> buffer_args;
  CallType call_type;
  Call(Type ret, std::string n, std::vector<Expr> a, CallType ct = CallType::Extern)
      : IrNode(kNodeTy, ret), name(std::move(n)), args(std::move(a)), call_type(ct) {}
};
struct Let : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Let;
  Expr symbol;  // Var
  Expr body;    // may be undefined: declaration only
  Let(Expr s, Expr b) : IrNode(kNodeTy, s.type()), symbol(std::move(s)), body(std::move(b)) {}
};

// bit flags as in cinn/ir/ir.h:613-622
enum class ForType : int { Serial = 0, Parallel = 1, Vectorized = 1 << 1, Unrolled = 1 << 2, GPUThread = 1 << 3, GPUBlock = 1 << 4 };
struct BindInfo {
  ForType for_type{ForType::Serial};
  int offset{-1};  // 0/1/2 = x/y/z
  bool valid() const { return offset >= 0 && (for_type == ForType::GPUThread || for_type == ForType::GPUBlock); }
};
struct For : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::For;
  Expr loop_var;
  Expr min, extent;
  ForType for_type;
  BindInfo bind_info;
  Expr body;
  For(Expr v, Expr mn, Expr ext, ForType ft, Expr b, BindInfo bi = BindInfo())
      : IrNode(kNodeTy, Type()), loop_var(std::move(v)), min(std::move(mn)), extent(std::move(ext)), for_type(ft), bind_info(bi), body(std::move(b)) {}
};
struct IfThenElse : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::IfThenElse;
  Expr condition, true_case, false_case;
  IfThenElse(Expr c, Expr t, Expr f) : IrNode(kNodeTy, Type()), condition(std::move(c)), true_case(std::move(t)), false_case(std::move(f)) {}
};
struct Block : IrNode {
  static constexpr IrNodeTy kNodeTy = IrNodeTy::Block;
  std::vector<Expr> stmts;
  explicit Block(std::vector<Expr> s) : IrNode(kNodeTy, Type()), stmts(std::move(s)) {}
};

// ---- constructors with light constant folding -------------------------------------------------
Expr MakeIntImm(Type t, int64_t v);
Expr MakeFloatImm(Type t, double v);
Expr MakeConst(Type t, double v);  // immediate of type t (int / uint / bool / float kinds)
Expr MakeVar(const std::string& name, Type t);
Expr MakeBinary(IrNodeTy op, Expr a, Expr b);
Expr MakeCast(Type t, Expr v);
Expr MakeSelect(Expr c, Expr t, Expr f);
Expr MakeLoad(const BufferRef& b, Expr index);
Expr MakeStore(const BufferRef& b, Expr value, Expr index);
Expr MakeRamp(Expr base, int stride, int lanes);
Expr MakeCall(Type ret, const std::string& name, std::vector<Expr> args, CallType ct = CallType::Extern);
Expr MakeLet(Expr var, Expr value);
Expr MakeFor(Expr var, Expr min, Expr extent, ForType ft, Expr body, BindInfo bi = BindInfo());
Expr MakeIf(Expr cond, Expr then_case, Expr else_case = Expr());
Expr MakeBlock(std::vector<Expr> stmts);
Expr MakeMinus(Expr v);
Expr MakeNot(Expr v);
Expr Min(Expr a, Expr b);
Expr Max(Expr a, Expr b);

Expr operator+(Expr a, Expr b);
Expr operator-(Expr a, Expr b);
Expr operator*(Expr a, Expr b);
Expr operator/(Expr a, Expr b);
Expr operator%(Expr a, Expr b);
Expr operator<(Expr a, Expr b);
Expr operator<=(Expr a, Expr b);
Expr operator>(Expr a, Expr b);
Expr operator>=(Expr a, Expr b);
Expr operator==(Expr a, Expr b);
Expr operator!=(Expr a, Expr b);
Expr operator&&(Expr a, Expr b);
Expr operator||(Expr a, Expr b);

// ---- functions and modules ----------------------------------------------------------------------
struct Argument {
  enum class IO { kInput, kOutput };
  BufferRef buffer;  // buffer argument, or
  Expr var;          // scalar argument
  IO io{IO::kInput};
  bool is_buffer() const { return buffer != nullptr; }
  std::string name() const;
};

// launch dimensions of a kernel, the counterpart of CudaAxisInfo (cinn/ir/lowered_func.h:84-113)
struct GpuAxisInfo {
  int grid[3]{1, 1, 1};
  int block[3]{1, 1, 1};
  bool valid{false};
  int block_threads() const { return block[0] * block[1] * block[2]; }
};

struct LoweredFunc {
  std::string name;
  std::vector<Argument> args;
  std::vector<BufferRef> temp_bufs;  // GPUShared / GPULocal allocations of the body
  Expr body;
  GpuAxisInfo axis_info;
  bool is_device{true};  // false: host function (body is one Call to a runtime intrinsic)
};
using LoweredFuncRef = std::shared_ptr<LoweredFunc>;

struct Module {
  std::string name;
  common::Target target;
  std::vector<LoweredFuncRef> functions;
};

// debugging dump in a C-like syntax
std::string ToString(const Expr& e);

}  // namespace ir
}  // namespace cinn
