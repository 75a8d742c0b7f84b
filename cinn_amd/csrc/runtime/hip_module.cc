// Code-object handle.  Role of runtime::cuda::CUDAModule (cinn/runtime/cuda/cuda_module.cc:35-149):
// the image is kept in host memory and loaded with hipModuleLoadData on the first function lookup,
// under a mutex; functions are looked up by kernel name; the module is unloaded on destroy.
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <string>

#include "cinn_hip_runtime.h"

struct cinn_hip_module {
  std::string image;
  hipModule_t module{nullptr};
  std::mutex mu;
  std::map<std::string, hipFunction_t> functions;
};

extern "C" {

int cinn_hip_module_create(const void* code, size_t code_size, cinn_hip_module_t* out) {
  if (!code || !code_size || !out) return -1;
  auto* m = new cinn_hip_module;
  m->image.assign(static_cast<const char*>(code), code_size);
  *out = m;
  return 0;
}

int cinn_hip_module_get_function(cinn_hip_module_t m, const char* name, void** kernel_fn) {
  if (!m || !name || !kernel_fn) return -1;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->functions.find(name);
  if (it != m->functions.end()) {
    *kernel_fn = it->second;
    return 0;
  }
  if (!m->module) {
    hipError_t st = hipModuleLoadData(&m->module, m->image.data());
    if (st != hipSuccess) {
      (void)hipGetLastError();  // reported through the status, not left behind as the thread's sticky error
      return static_cast<int>(st);
    }
  }
  hipFunction_t fn = nullptr;
  hipError_t st    = hipModuleGetFunction(&fn, m->module, name);
  if (st != hipSuccess) {
    (void)hipGetLastError();
    return static_cast<int>(st);
  }
  m->functions[name] = fn;
  *kernel_fn         = fn;
  return 0;
}

int cinn_hip_module_destroy(cinn_hip_module_t m) {
  if (!m) return 0;
  hipError_t st = hipSuccess;
  if (m->module) st = hipModuleUnload(m->module);
  delete m;
  return static_cast<int>(st);
}

}  // extern "C"
