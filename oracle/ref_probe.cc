// Checker built against the REFERENCE's own runtime sources (cinn/runtime/cinn_runtime.{h,cc},
// cinn/common/float16.h, cinn/common/bfloat16.h), compiled where they lie; see oracle/Makefile.
// It exports what the parity tests need from the real reference: the ABI struct layouts, the
// cinn_pod_value_t accessors and the host fp16 / bf16 conversions.  Test infrastructure only.
#include <cstddef>
#include <cstring>

#include "cinn/runtime/cinn_runtime.h"

extern "C" {

// layout table: {sizeof(cinn_type_t), sizeof(cinn_buffer_t), offsets of memory, type, dimensions, dims,
// memory_size, sizeof(cinn_pod_value_t)}
void ref_abi_layout(long* out) {
  out[0] = sizeof(cinn_type_t);
  out[1] = sizeof(cinn_buffer_t);
  out[2] = offsetof(cinn_buffer_t, memory);
  out[3] = offsetof(cinn_buffer_t, type);
  out[4] = offsetof(cinn_buffer_t, dimensions);
  out[5] = offsetof(cinn_buffer_t, dims);
  out[6] = offsetof(cinn_buffer_t, memory_size);
  out[7] = sizeof(cinn_pod_value_t);
  out[8] = offsetof(cinn_buffer_t, flag);
  out[9] = offsetof(cinn_buffer_t, align);
}

// cinn_type_code<T>() values in the order of the table in cinn_runtime.h
void ref_pod_type_codes(int* out) {
  out[0]  = cinn_type_code<int32_t>();
  out[1]  = cinn_type_code<int64_t>();
  out[2]  = cinn_type_code<float>();
  out[3]  = cinn_type_code<double>();
  out[4]  = cinn_type_code<void*>();
  out[5]  = cinn_type_code<char*>();
  out[6]  = cinn_type_code<char const*>();
  out[7]  = cinn_type_code<cinn_buffer_t*>();
  out[8]  = cinn_type_code<int8_t>();
  out[9]  = cinn_type_code<bool>();
  out[10] = cinn_type_code<cinn::common::float16>();
  out[11] = cinn_type_code<int16_t>();
  out[12] = cinn_type_code<uint8_t>();
  out[13] = cinn_type_code<uint16_t>();
  out[14] = cinn_type_code<uint32_t>();
  out[15] = cinn_type_code<uint64_t>();
  out[16] = cinn_type_code<cinn::common::bfloat16>();
}

// reads a pod array / buffer that was filled by the library under test, through the reference's accessors
void* ref_read_pod_buffer_memory(void* pod_array, int index) {
  cinn_pod_value_t* args = static_cast<cinn_pod_value_t*>(pod_array);
  cinn_buffer_t* buf     = cinn_pod_value_to_buffer_p(&args[index]);
  return buf->memory;
}
int ref_read_pod_type_code(void* pod_array, int index) {
  return static_cast<cinn_pod_value_t*>(pod_array)[index].type_code();
}
void ref_read_buffer(void* buffer, long* out) {
  cinn_buffer_t* buf = static_cast<cinn_buffer_t*>(buffer);
  out[0]             = static_cast<long>(buf->type.code);
  out[1]             = buf->type.bits;
  out[2]             = buf->type.lanes;
  out[3]             = buf->dimensions;
  out[4]             = static_cast<long>(buf->num_elements());
  out[5]             = static_cast<long>(buf->memory_size);
  out[6]             = buf->on_device() ? 1 : 0;
  for (int i = 0; i < buf->dimensions && i < 8; ++i) out[7 + i] = buf->dims[i];
}
int ref_type_of(int which, long* out) {
  cinn_type_t t;
  switch (which) {
    case 0: t = cinn_float32_t(); break;
    case 1: t = cinn_float16_t(); break;
    case 2: t = cinn_bfloat16_t(); break;
    case 3: t = cinn_int32_t(); break;
    case 4: t = cinn_bool_t(); break;
    case 5: t = cinn_float64_t(); break;
    case 6: t = cinn_int64_t(); break;
    default: return 1;
  }
  out[0] = static_cast<long>(t.code);
  out[1] = t.bits;
  out[2] = t.lanes;
  return 0;
}

// host conversions of the reference's 16-bit float structs
void ref_float_to_half(const float* in, unsigned short* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = cinn::common::float16(in[i]).x;
}
void ref_half_to_float(const unsigned short* in, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = static_cast<float>(cinn::common::raw_uint16_to_float16(in[i]));
}
void ref_float_to_bfloat16(const float* in, unsigned short* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = cinn::common::bfloat16(in[i]).x;
}
void ref_bfloat16_to_float(const unsigned short* in, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = static_cast<float>(cinn::common::raw_uint16_to_bfloat16(in[i]));
}
// the fp16 host test kernel of cinn/common/float16_bfloat16_host_test.cc:27-36: (x+1+y)*(x+1-y) in half
void ref_half_test_kernel(const unsigned short* x, const unsigned short* y, unsigned short* out, long n) {
  using cinn::common::float16;
  for (long i = 0; i < n; ++i) {
    float16 x_i = cinn::common::raw_uint16_to_float16(x[i]), y_i = cinn::common::raw_uint16_to_float16(y[i]);
    x_i += float16(1);
    out[i] = ((x_i + y_i) * (x_i - y_i)).x;
  }
}
}
