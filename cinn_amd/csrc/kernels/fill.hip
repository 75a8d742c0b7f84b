// cinn_call_cuda_memset as a kernel.  The reference calls cudaMemsetAsync (cinn/runtime/cuda/cuda_util.cc:439-449);
// here the bytes are written by a small fill kernel, because a memset node recorded into a captured graph
// (Program::ExecuteGraph records whatever its instructions launch) has replayed with wrong results on this platform,
// while a kernel node replays like any other launch.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// Bytes [0, head) and [head + 16 * vecs, count) are written one per thread by the first and last blocks' worth of
// threads, the 16-byte aligned body as one vector per thread (grid-stride).
__global__ void __launch_bounds__(256)
fill_bytes_kernel(unsigned char* dst, unsigned char value, size_t count, size_t head, size_t vecs) {
  const size_t tid    = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  const unsigned word = 0x01010101u * value;
  const u32x4 v       = {word, word, word, word};
  u32x4* body         = reinterpret_cast<u32x4*>(dst + head);
  for (size_t i = tid; i < vecs; i += stride) body[i] = v;
  const size_t tail_begin = head + 16 * vecs;
  if (tid < head) dst[tid] = value;
  if (tid < count - tail_begin) dst[tail_begin + tid] = value;  // fewer than 16 bytes
}

}  // namespace

extern "C" void cinn_call_cuda_memset(void* v_args, int num_args, int value, size_t count, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 1, "cinn_call_cuda_memset takes one output buffer, got %d arguments", num_args);
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  CINN_RT_CHECK(args[0].type_code_ == CINN_POD_BUFFER_P, "cinn_call_cuda_memset: the argument is not a buffer");
  auto* out = static_cast<cinn_buffer_t*>(args[0].value_.v_handle);
  CINN_RT_CHECK(out && out->memory, "cinn_call_cuda_memset: null buffer");
  CINN_RT_CHECK(count <= out->memory_size || out->memory_size == 0,
                "cinn_call_cuda_memset: %zu bytes do not fit the buffer of %zu", count, (size_t)out->memory_size);
  if (count == 0) return;
  auto* dst         = static_cast<unsigned char*>(out->memory);
  const size_t misal = reinterpret_cast<uintptr_t>(dst) & 15;
  size_t head        = misal ? 16 - misal : 0;
  if (head > count) head = count;
  const size_t vecs   = (count - head) / 16;
  size_t blocks       = (vecs + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 2048) blocks = 2048;  // 8 blocks per CU; the body loop strides
  hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), dst,
                     static_cast<unsigned char>(value), count, head, vecs);
  CINN_HIP_CALL(hipGetLastError());
}
