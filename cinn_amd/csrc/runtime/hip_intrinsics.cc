// Host-side runtime intrinsics that generated host stubs call: kernel launch and memcpy (memset: kernels/fill.hip).
#include <hip/hip_runtime_api.h>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace {
constexpr int kMaxInlineArgs = 64;
}

extern "C" {

void cinn_call_hip_kernel(void* kernel_fn, void* v_args, int num_args, int grid_x, int grid_y, int grid_z,
                          int block_x, int block_y, int block_z, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(kernel_fn != nullptr, "cinn_call_hip_kernel: null kernel function");
  CINN_RT_CHECK(num_args >= 0 && (num_args == 0 || v_args != nullptr), "cinn_call_hip_kernel: bad argument list");
  CINN_RT_CHECK(grid_x > 0 && grid_y > 0 && grid_z > 0 && block_x > 0 && block_y > 0 && block_z > 0,
                "cinn_call_hip_kernel: launch dimensions must be positive, got grid {%d,%d,%d} block {%d,%d,%d}",
                grid_x, grid_y, grid_z, block_x, block_y, block_z);
  CINN_RT_CHECK(static_cast<long long>(block_x) * block_y * block_z <= 1024,
                "cinn_call_hip_kernel: %lld threads per block exceeds 1024",
                static_cast<long long>(block_x) * block_y * block_z);
  // argument slots: a buffer is passed as the address of its device pointer, a scalar as the
  // address of its value inside the pod (cinn/runtime/cuda/cuda_util.cc:95-104)
  void* inline_args[kMaxInlineArgs];
  void** kernel_args = inline_args;
  if (num_args > kMaxInlineArgs) kernel_args = new void*[num_args];
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  for (int i = 0; i < num_args; ++i) {
    if (args[i].type_code_ == CINN_POD_BUFFER_P) {
      auto* buf = static_cast<cinn_buffer_t*>(args[i].value_.v_handle);
      CINN_RT_CHECK(buf != nullptr, "cinn_call_hip_kernel: argument %d is a null buffer", i);
      kernel_args[i] = &buf->memory;
    } else {
      kernel_args[i] = &args[i].value_;
    }
  }
  CINN_HIP_CALL(hipModuleLaunchKernel(static_cast<hipFunction_t>(kernel_fn), grid_x, grid_y, grid_z, block_x, block_y,
                                      block_z, 0, static_cast<hipStream_t>(stream), kernel_args, nullptr));
  if (kernel_args != inline_args) delete[] kernel_args;
}

void cinn_call_cuda_kernel(void* kernel_fn, void* v_args, int num_args, int grid_x, int grid_y, int grid_z,
                           int block_x, int block_y, int block_z, void* stream) {
  cinn_call_hip_kernel(kernel_fn, v_args, num_args, grid_x, grid_y, grid_z, block_x, block_y, block_z, stream);
}

void cinn_call_cuda_memcpy(void* v_args, int num_args, size_t count, void* stream) {
  CINN_RT_CHECK(num_args == 2, "cinn_call_cuda_memcpy takes an input and an output buffer, got %d arguments", num_args);
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  auto* in   = static_cast<cinn_buffer_t*>(args[0].value_.v_handle);
  auto* out  = static_cast<cinn_buffer_t*>(args[1].value_.v_handle);
  CINN_HIP_CALL(hipMemcpyAsync(out->memory, in->memory, count, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
