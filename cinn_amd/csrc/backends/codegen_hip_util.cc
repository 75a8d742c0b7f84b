#include "backends/codegen_hip_util.h"

namespace cinn {
namespace backends {

std::pair<ir::Module, ir::Module> SplitHostAndDeviceModule(const ir::Module& module) {
  ir::Module host, device;
  host.name     = module.name + "_host";
  device.name   = module.name + "_gpu_device";
  host.target   = module.target;
  device.target = module.target;
  for (auto& f : module.functions) {
    if (!f->is_device) {
      host.functions.push_back(f);
      continue;
    }
    CINN_CHECK(f->axis_info.valid) << "device function " << f->name << " has no launch dimensions";
    auto kernel  = std::make_shared<ir::LoweredFunc>(*f);
    kernel->name = KernelNameOf(f->name);
    device.functions.push_back(kernel);

    auto stub       = std::make_shared<ir::LoweredFunc>();
    stub->name      = f->name;
    stub->is_device = false;
    stub->args      = f->args;
    ir::Expr kernel_ptr = ir::MakeVar(KernelPtrSymbolOf(kernel->name), common::Handle());
    std::vector<ir::Expr> args = {kernel_ptr, ir::MakeVar("kernel_args", common::Handle()),
                                  ir::MakeVar("kernel_args_num", common::Int(32))};
    for (int g : f->axis_info.grid) args.push_back(ir::Expr(g));
    for (int b : f->axis_info.block) args.push_back(ir::Expr(b));
    args.push_back(ir::MakeVar("kernel_stream", common::Handle()));
    stub->body = ir::MakeCall(common::Type(), "cinn_call_hip_kernel", args, ir::CallType::Extern);
    host.functions.push_back(stub);
  }
  return {host, device};
}

}  // namespace backends
}  // namespace cinn
