#include "backends/compiler.h"

#include <cstdlib>
#include <fstream>
#include <mutex>

#include "backends/codegen_hip_dev.h"
#include "backends/codegen_hip_util.h"
#include "backends/host_stub.h"

namespace cinn {
namespace backends {

void SaveSourceCode(const std::string& source) {
  const char* path = getenv("FLAGS_cinn_source_code_save_path");
  if (!path || !*path) return;
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  std::ofstream of(path, std::ios_base::app);
  if (of.is_open()) of << source << std::endl;
}

Compiler::~Compiler() {
  for (auto& kv : functions_) HostStubPool::Global().Release(kv.second);
  for (auto m : modules_) cinn_hip_module_destroy(m);
}

std::string Compiler::GetSourceCode(const ir::Module& module) {
  auto parts = SplitHostAndDeviceModule(module);
  CodeGenHIP_Dev codegen(target_);
  return codegen.Compile(parts.second);
}

void Compiler::Build(const ir::Module& module, const std::string& code) {
  CINN_CHECK(target_.arch == common::Target::Arch::AMDGPU) << "this Compiler only builds for the AMDGPU target";
  auto parts   = SplitHostAndDeviceModule(module);
  auto& host   = parts.first;
  auto& device = parts.second;

  std::map<std::string, void*> symbols;
  if (!device.functions.empty()) {
    CodeGenHIP_Dev codegen(target_);
    source_code_ = code.empty() ? codegen.Compile(device) : code;
    SaveSourceCode(source_code_);

    char* image       = nullptr;
    size_t image_size = 0;
    char* log         = nullptr;
    int status        = cinn_hip_rtc_compile(source_code_.c_str(), 1, getenv("FLAGS_cinn_hiprtc_options"), &image, &image_size, &log);
    std::string log_text = log ? log : "";
    cinn_hip_free_host(log);
    CINN_CHECK_EQ(status, 0) << "hiprtc failed to compile module " << module.name << ":\n"
                             << log_text << "\n---- source ----\n"
                             << source_code_;
    code_object_size_ = image_size;

    int device_count = 0;
    cinn_hip_device_count(&device_count);
    if (device_count > 0) {
      cinn_hip_module_t m = nullptr;
      status              = cinn_hip_module_create(image, image_size, &m);
      CINN_CHECK_EQ(status, 0) << "cannot create a code-object handle";
      modules_.push_back(m);
      for (auto& f : device.functions) {
        void* fn = nullptr;
        status   = cinn_hip_module_get_function(m, f->name.c_str(), &fn);
        CINN_CHECK_EQ(status, 0) << "kernel " << f->name << " not found in the code object: "
                                 << cinn_hip_error_string(status);
        symbols[KernelPtrSymbolOf(f->name)] = fn;
      }
    }
    cinn_hip_free_host(image);
  }

  for (auto& f : host.functions) {
    HostStubPool::Closure closure;
    bool needs_kernel = false;
    if (auto* call = f->body.As<ir::Call>()) needs_kernel = call->name == "cinn_call_hip_kernel";
    if (needs_kernel && symbols.empty()) {
      std::string name = f->name;
      closure          = [name](void*, int32_t, void*) {
        fprintf(stderr, "kernel %s was compiled without a visible GPU and cannot be launched\n", name.c_str());
        abort();
      };
    } else {
      closure = LowerHostFunction(*f, symbols);
    }
    CINN_CHECK(!functions_.count(f->name)) << "function " << f->name << " built twice";
    functions_[f->name] = HostStubPool::Global().Acquire(std::move(closure));
  }
}

void* Compiler::Lookup(const std::string& fn_name) {
  auto it = functions_.find(fn_name);
  if (it == functions_.end()) return nullptr;
  return reinterpret_cast<void*>(it->second);
}

}  // namespace backends
}  // namespace cinn
