// Host-side half of a compiled module without an LLVM JIT.
//
// The reference lowers every host function to LLVM IR and JITs it (CodeGenCUDA_Host,
// cinn/backends/codegen_cuda_host.cc:35-168; ExecutionEngine, cinn/backends/llvm/execution_engine.cc);
// the result is a plain `void fn(void* args, int32_t num_args, void* stream)` pointer
// (lower_func_ptr_g).  Here a host function - whose body is one call of a runtime intrinsic with
// constant arguments - is "compiled" into a closure that holds the resolved intrinsic and the baked
// argument values, and is exposed through one of a fixed pool of pre-instantiated C trampolines so
// callers still get a real lower_func_ptr_g.
#pragma once
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "cinn_hip_runtime.h"
#include "ir/ir.h"

namespace cinn {
namespace backends {

// one constant or pass-through argument of a host-side intrinsic call
struct BakedArg {
  enum class Kind { kArgs, kNumArgs, kStream, kInt, kFloat, kBool, kHandle };
  Kind kind{Kind::kInt};
  int64_t i{0};
  double f{0};
  void* p{nullptr};
};

// adaptor that calls one extern "C" intrinsic from a baked argument list; the counterpart of a
// registered extern-function prototype (cinn/backends/extern_func_jit_register.h:40-91,
// REGISTER_EXTERN_FUNC_HELPER in cinn/runtime/cuda/cuda_intrinsics.cc:404-733)
using ApiInvoker = void (*)(const std::vector<BakedArg>& baked, void* args, int32_t num_args, void* stream);

class ExternApiRegistry {
 public:
  static ExternApiRegistry& Global();
  void Register(const std::string& name, ApiInvoker invoker, size_t num_call_args);
  // nullptr when the name is unknown
  ApiInvoker Find(const std::string& name, size_t* num_call_args = nullptr) const;
  std::vector<std::string> Names() const;

 private:
  ExternApiRegistry();
  struct Entry {
    ApiInvoker invoker;
    size_t num_call_args;
  };
  std::map<std::string, Entry> table_;
};

// Pool of trampolines.  Acquire() binds a closure to a free slot and returns the slot's function
// pointer; Release() frees it.  kSlots functions are pre-compiled; when all of them are taken, further stubs are a few
// bytes of machine code each in an executable page (x86-64: load the closure's address into the fourth argument
// register and jump to a common dispatcher), so the number of live compiled functions is bounded by memory only.
class HostStubPool {
 public:
  static constexpr int kSlots = 4096;
  using Closure = std::function<void(void*, int32_t, void*)>;
  static HostStubPool& Global();
  lower_func_ptr_g Acquire(Closure closure);
  void Release(lower_func_ptr_g fn);
  int in_use() const;
  int thunks_in_use() const;  // stubs beyond the pre-compiled slots
};

// Resolves the symbols a host function refers to (kernel handles by name) and builds its closure.
// `kernel_symbols` maps "<kernel>_ptr_"-style names to hipFunction_t handles, as RuntimeSymbols does
// in the reference (cinn/backends/compiler.cc:133-140).
HostStubPool::Closure LowerHostFunction(const ir::LoweredFunc& func, const std::map<std::string, void*>& kernel_symbols);

}  // namespace backends
}  // namespace cinn
