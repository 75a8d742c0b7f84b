// Split of a module into its device half and its host half, the role of SplitCudaAndHostModule
// (cinn/backends/codegen_cuda_util.h:49-135): every device function `fn` keeps its body under the
// name `fn_kernel`, and a host function `fn(kernel_args, kernel_args_num, kernel_stream)` is created
// whose body is the single call
//   cinn_call_hip_kernel(fn_kernel_ptr_, kernel_args, kernel_args_num, gx, gy, gz, bx, by, bz, kernel_stream)
// with the launch dimensions of fn's GpuAxisInfo baked in.  Functions that are already host
// functions (library calls) go to the host module unchanged.
#pragma once
#include <utility>

#include "ir/ir.h"

namespace cinn {
namespace backends {

// returns (host module, device module)
std::pair<ir::Module, ir::Module> SplitHostAndDeviceModule(const ir::Module& module);

// name of the kernel generated for host function `fn`, and of the symbol holding its handle
inline std::string KernelNameOf(const std::string& fn) { return fn + "_kernel"; }
inline std::string KernelPtrSymbolOf(const std::string& kernel) { return kernel + "_ptr_"; }

}  // namespace backends
}  // namespace cinn
