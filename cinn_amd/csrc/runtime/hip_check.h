// Abort-on-error wrappers for the runtime intrinsics, the counterpart of CUDA_CALL /
// CUDA_DRIVER_CALL / NVRTC_CALL (cinn/backends/cuda_util.h:30-88): a failed HIP call inside a
// `cinn_call_*` intrinsic prints the call, the HIP error string and the location, then aborts.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>

#define CINN_HIP_CALL(expr)                                                                                   \
  do {                                                                                                        \
    hipError_t cinn_hip_status__ = (expr);                                                                    \
    if (cinn_hip_status__ != hipSuccess) {                                                                    \
      fprintf(stderr, "%s:%d: HIP call `%s` failed: %s\n", __FILE__, __LINE__, #expr,                         \
              hipGetErrorString(cinn_hip_status__));                                                          \
      abort();                                                                                                \
    }                                                                                                         \
  } while (0)

#define CINN_RT_CHECK(cond, ...)                                                  \
  do {                                                                            \
    if (!(cond)) {                                                                \
      fprintf(stderr, "%s:%d: check `%s` failed: ", __FILE__, __LINE__, #cond);   \
      fprintf(stderr, __VA_ARGS__);                                               \
      fprintf(stderr, "\n");                                                      \
      abort();                                                                    \
    }                                                                             \
  } while (0)

// A kernel launched with hipLaunchKernelGGL reports failure through the thread's sticky "last error", which an earlier,
// unrelated HIP call (the application's own, or a status-returning cinn_hip_* call that failed) may have left set.
// Every cinn_call_* intrinsic starts by clearing it, so that the check after its launches sees its own errors only.
#define CINN_HIP_CLEAR_STALE_ERROR() (void)hipGetLastError()
