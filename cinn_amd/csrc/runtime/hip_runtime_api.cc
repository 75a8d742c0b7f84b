// Device memory, streams, events, target query and ABI helpers of the C-ABI runtime.
#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

static_assert(sizeof(cinn_type_t) == 12, "cinn_type_t must stay 12 bytes");
static_assert(sizeof(cinn_buffer_t) == 120, "cinn_buffer_t must stay 120 bytes");
static_assert(offsetof(cinn_buffer_t, memory) == 16, "cinn_buffer_t::memory offset");
static_assert(offsetof(cinn_buffer_t, type) == 32, "cinn_buffer_t::type offset");
static_assert(offsetof(cinn_buffer_t, dimensions) == 44, "cinn_buffer_t::dimensions offset");
static_assert(offsetof(cinn_buffer_t, dims) == 48, "cinn_buffer_t::dims offset");
static_assert(offsetof(cinn_buffer_t, memory_size) == 88, "cinn_buffer_t::memory_size offset");
static_assert(sizeof(cinn_pod_value_t) == 16, "cinn_pod_value_t must stay 16 bytes");
static_assert(offsetof(cinn_pod_value_t, value_) == 8, "cinn_pod_value_t::value_ offset");

namespace {
// status of a HIP call for a status-returning entry point: the error is reported through the return value, so the
// thread's sticky "last error" is cleared - it must not surface later in an unrelated launch check
int Status(hipError_t st) {
  if (st != hipSuccess) (void)hipGetLastError();
  return static_cast<int>(st);
}
}  // namespace

extern "C" {

void cinn_hip_buffer_init(cinn_buffer_t* buf, void* device_ptr, int32_t type_code, int32_t bits, const int32_t* dims,
                          int32_t ndims) {
  memset(buf, 0, sizeof(*buf));
  buf->device            = cinn_unk_device;
  buf->memory            = static_cast<uint8_t*>(device_ptr);
  buf->flag              = cinn_buffer_on_device;
  buf->type.code         = type_code;
  buf->type.bits         = static_cast<uint8_t>(bits);
  // the reference's cinn_float32_t() & co. leave lanes at 0 (cinn/runtime/cinn_runtime.cc passes
  // num_asterisks in the lanes slot); buffers made by its Tensor class therefore carry lanes == 0
  buf->type.lanes        = 0;
  buf->type.num_asterisks = 0;
  buf->dimensions        = ndims > CINN_BUFFER_MAX_DIMS ? CINN_BUFFER_MAX_DIMS : ndims;
  uint64_t n             = 1;
  for (int i = 0; i < buf->dimensions; ++i) {
    buf->dims[i] = dims[i];
    n *= static_cast<uint64_t>(dims[i]);
  }
  buf->lazy        = 1;
  buf->memory_size = n * ((bits + 7) / 8);
}

void cinn_hip_pod_from_buffer(cinn_pod_value_t* out, cinn_buffer_t* buf) {
  out->type_code_      = CINN_POD_BUFFER_P;
  out->value_.v_handle = buf;
}
void cinn_hip_pod_from_int32(cinn_pod_value_t* out, int32_t v) {
  out->type_code_     = CINN_POD_INT32;
  out->value_.v_int64 = v;
}
void cinn_hip_pod_from_float(cinn_pod_value_t* out, float v) {
  out->type_code_       = CINN_POD_FLOAT;
  out->value_.v_float64 = v;
}

int cinn_hip_device_count(int* count) {
  *count = 0;
  hipError_t st = hipGetDeviceCount(count);
  if (st != hipSuccess) {
    *count = 0;
    (void)hipGetLastError();
  }
  return static_cast<int>(st);
}

int cinn_hip_malloc(void** dptr, size_t bytes) { return Status(hipMalloc(dptr, bytes ? bytes : 1)); }
int cinn_hip_free(void* dptr) { return Status(hipFree(dptr)); }
int cinn_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (stream) return Status(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
  return Status(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
}
int cinn_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
  if (stream) {
    hipError_t st = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
    if (st != hipSuccess) return static_cast<int>(st);
    return Status(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  }
  return Status(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}
int cinn_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
  return Status(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
}
int cinn_hip_memset(void* dst, int value, size_t bytes, void* stream) {
  return Status(hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(stream)));
}
int cinn_hip_device_synchronize(void) { return Status(hipDeviceSynchronize()); }
int cinn_hip_stream_create(void** stream) {
  hipStream_t s = nullptr;
  hipError_t st = hipStreamCreate(&s);  // default priority only
  *stream       = s;
  return static_cast<int>(st);
}
int cinn_hip_stream_destroy(void* stream) {
  (void)cinn_hip_scratch_release_stream(stream);  // its scratch is retired with it, so a recycled handle starts empty
  return Status(hipStreamDestroy(static_cast<hipStream_t>(stream)));
}
int cinn_hip_stream_synchronize(void* stream) {
  return Status(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}
int cinn_hip_event_create(void** event) {
  hipEvent_t e  = nullptr;
  hipError_t st = hipEventCreate(&e);
  *event        = e;
  return static_cast<int>(st);
}
int cinn_hip_event_destroy(void* event) { return Status(hipEventDestroy(static_cast<hipEvent_t>(event))); }
int cinn_hip_event_record(void* event, void* stream) {
  return Status(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}
int cinn_hip_event_synchronize(void* event) { return Status(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int cinn_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  return Status(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}
const char* cinn_hip_error_string(int status) { return hipGetErrorString(static_cast<hipError_t>(status)); }
void cinn_hip_free_host(void* p) { free(p); }

int cinn_hip_get_target_info(cinn_hip_target_info* info) {
  // MI355X (gfx950) datasheet values; overwritten from the live device below when there is one
  memset(info, 0, sizeof(*info));
  info->wavefront_size                  = 64;
  info->max_threads_per_block           = 1024;
  info->multi_processor_count           = 256;
  info->max_threads_per_multi_processor = 2048;
  info->max_blocks_per_multi_processor  = 32;
  info->lds_bytes_per_block             = 64 * 1024;
  info->lds_bytes_per_multi_processor   = 160 * 1024;
  info->num_xcd                         = 8;
  info->from_device                     = 0;
  strncpy(info->arch, "gfx950", sizeof(info->arch) - 1);

  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return 0;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
  info->from_device                     = 1;
  info->wavefront_size                  = prop.warpSize;
  info->max_threads_per_block           = prop.maxThreadsPerBlock;
  info->multi_processor_count           = prop.multiProcessorCount;
  info->max_threads_per_multi_processor = prop.maxThreadsPerMultiProcessor;
  if (prop.maxBlocksPerMultiProcessor > 0) info->max_blocks_per_multi_processor = prop.maxBlocksPerMultiProcessor;
  info->lds_bytes_per_block = static_cast<int>(prop.sharedMemPerBlock);
  if (prop.maxSharedMemoryPerMultiProcessor > 0)
    info->lds_bytes_per_multi_processor = static_cast<int>(prop.maxSharedMemoryPerMultiProcessor);
  // gcnArchName looks like "gfx950:sramecc+:xnack-"
  const char* colon = strchr(prop.gcnArchName, ':');
  size_t n          = colon ? static_cast<size_t>(colon - prop.gcnArchName) : strlen(prop.gcnArchName);
  if (n >= sizeof(info->arch)) n = sizeof(info->arch) - 1;
  memcpy(info->arch, prop.gcnArchName, n);
  info->arch[n] = 0;
  return 0;
}

}  // extern "C"
