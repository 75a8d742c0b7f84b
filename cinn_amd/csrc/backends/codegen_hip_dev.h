// HIP C++ source generator for gfx950 kernels.  It fills the role of CodeGenCUDA_Dev
// (cinn/backends/codegen_cuda_dev.cc:32-388 over cinn/backends/codegen_c.cc) for the AMDGPU target:
// every device LoweredFunc of a module becomes one `extern "C" __global__` kernel with
// __launch_bounds__ taken from its launch dimensions; buffer arguments print as
// `const T* __restrict__` / `T* __restrict__`; GPUShared / GPULocal temporaries become `__shared__`
// and register arrays; vector copies become cinn_hip_copy_vec<T, N> calls of the device library.
#pragma once
#include <string>

#include "ir/ir.h"
#include "ir/ir_printer.h"

namespace cinn {
namespace backends {

class CodeGenHIP_Dev : public ir::IrPrinter {
 public:
  explicit CodeGenHIP_Dev(const common::Target& target);

  // Source text for all device functions of the module.  `for_hiprtc` selects in-memory-header mode:
  // the text starts with `#include "cinn_hip_runtime_source.h"` which the hiprtc wrapper resolves to
  // the embedded device library.
  std::string Compile(const ir::Module& module, bool for_hiprtc = true);
  std::string CompileFunc(const ir::LoweredFunc& func);

  static const std::string& GetSourceHeader();

 protected:
  void VisitVar(const ir::Var* op) override;
  void VisitBinary(const ir::Binary* op) override;
  void VisitLoad(const ir::Load* op) override;
  void VisitStore(const ir::Store* op) override;
  void VisitFor(const ir::For* op) override;
  void VisitCall(const ir::Call* op) override;

 private:
  void PrintFunctionDeclaration(const ir::LoweredFunc& func);
  void PrintTempBuffers(const ir::LoweredFunc& func);
  common::Target target_;
};

}  // namespace backends
}  // namespace cinn
