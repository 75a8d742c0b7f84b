// TEMPORARY: replaced by kernels/*.hip
#include <cstdio>
#include <cstdlib>
#include "cinn_hip_runtime.h"
extern "C" {
void cinn_call_cublas(void*, int, bool, bool, bool, float, float, int, int, int, int, int, int, int, int, void*) { fprintf(stderr, "cinn_call_cublas: not built\n"); abort(); }
void cinn_call_batched_cublas(void*, int, int, bool, bool, bool, float, float, int, int, int, int, int, int, int, int, void*) { abort(); }
void cinn_call_cudnn_conv2d_forward(void*, int, int, float, float, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, void*) { abort(); }
void cinn_call_hip_conv2d_bn_relu(void*, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, void*) { abort(); }
void cinn_call_cudnn_pool2d_forward(void*, int, int, int, float, float, int, int, int, int, int, int, int, int, int, int, int, int, int, int, void*) { abort(); }
void cinn_call_cudnn_softmax_forward(void*, int, int, int, float, float, int, int, int, int, int, int, int, int, void*) { abort(); }
}
