/*
 * C-ABI of the MI355X (gfx950) runtime for the CINN GPU backend.
 *
 * Everything a JIT'd / trampolined host stub of a compiled CINN program calls on the GPU path is
 * declared here with plain pointers and sizes.  Each entry point names the reference interface it
 * replaces (paths are relative to the CINN source tree).
 *
 * Error convention (same as the reference's CUDA_CALL / CUDA_DRIVER_CALL / CHECK macros,
 * cinn/backends/cuda_util.h:30-88): the `cinn_call_*` intrinsics return void and abort() the process
 * with a message on stderr when a HIP call fails or an argument is invalid.  The `cinn_hip_*`
 * management entry points return 0 on success and a non-zero HIP / hiprtc status otherwise and
 * never abort, so a binding can turn them into exceptions.
 *
 * Threading: entry points may be called from any thread; module loading and the kernel cache are
 * guarded by a mutex, launches are not serialised (HIP streams order them).
 */
#ifndef CINN_HIP_RUNTIME_H_
#define CINN_HIP_RUNTIME_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------------
 * ABI structs.  Layout-identical to cinn/runtime/cinn_runtime.h:51-93 (cinn_type_t), :186-292
 * (cinn_buffer_t, 120 bytes: memory@16, type@32, dimensions@44, dims@48, memory_size@88) and
 * :390-461 (cinn_value_t / cinn_pod_value_t, 16 bytes) as compiled by a C++11 compiler on x86-64.
 * ---------------------------------------------------------------------------------------------- */

typedef enum cinn_type_code_t {
  cinn_type_unk    = -1,
  cinn_type_int    = 0,
  cinn_type_uint   = 1,
  cinn_type_float  = 2,
  cinn_type_handle = 3,
  cinn_type_bfloat = 4
} cinn_type_code_t;

typedef struct cinn_type_t {
  int32_t code; /* a cinn_type_code_t, stored in 4 bytes */
  uint8_t bits;
  uint16_t lanes;
  uint8_t num_asterisks;
} cinn_type_t;

typedef int cinn_dimension_t;

typedef enum cinn_device_kind_t {
  cinn_unk_device    = -1,
  cinn_x86_device    = 0,
  cinn_opencl_device = 1,
  cinn_arm_device    = 2
} cinn_device_kind_t;

typedef enum cinn_buffer_kind_t { cinn_buffer_on_host = 0, cinn_buffer_on_device = 1 << 1 } cinn_buffer_kind_t;

#define CINN_BUFFER_MAX_DIMS 8

typedef struct cinn_buffer_t {
  int32_t device; /* a cinn_device_kind_t */
  const void* device_interface;
  uint8_t* memory; /* device pointer on the GPU path */
  uint64_t flag;
  cinn_type_t type;
  int32_t dimensions;
  cinn_dimension_t dims[CINN_BUFFER_MAX_DIMS];
  char lazy;
  uint64_t memory_size;
  uint16_t align;
  void* external_malloc; /* std::function<int(void*, cinn_buffer_t*)>* in the reference; opaque here */
  void* external_free;
} cinn_buffer_t;

typedef union cinn_value_t {
  int64_t v_int64;
  double v_float64;
  void* v_handle;
  char* v_str;
} cinn_value_t;

typedef struct cinn_pod_value_t {
  int type_code_; /* values of cinn_type_code<T>() below */
  cinn_value_t value_;
} cinn_pod_value_t;

/* cinn_type_code<T>() table, cinn/runtime/cinn_runtime.h:469-491 */
enum {
  CINN_POD_INT32 = 0,
  CINN_POD_INT64 = 1,
  CINN_POD_FLOAT = 2,
  CINN_POD_DOUBLE = 3,
  CINN_POD_VOID_P = 4,
  CINN_POD_CHAR_P = 5,
  CINN_POD_CONST_CHAR_P = 6,
  CINN_POD_BUFFER_P = 7,
  CINN_POD_INT8 = 8,
  CINN_POD_BOOL = 9,
  CINN_POD_FLOAT16 = 10,
  CINN_POD_INT16 = 11,
  CINN_POD_UINT8 = 12,
  CINN_POD_UINT16 = 13,
  CINN_POD_UINT32 = 14,
  CINN_POD_UINT64 = 15,
  CINN_POD_BFLOAT16 = 16
};

/* Host-stub type every compiled fused group is exposed as (cinn_runtime.h:498-499). */
typedef void (*lower_func_ptr_g)(void* pod_args, int32_t num_args, void* stream);

/* Helpers to fill ABI structs from a binding (cinn_runtime.cc buffer_p_to_cinn_pod_value etc.). */
void cinn_hip_buffer_init(cinn_buffer_t* buf, void* device_ptr, int32_t type_code, int32_t bits, const int32_t* dims,
                          int32_t ndims);
void cinn_hip_pod_from_buffer(cinn_pod_value_t* out, cinn_buffer_t* buf);
void cinn_hip_pod_from_int32(cinn_pod_value_t* out, int32_t v);
void cinn_hip_pod_from_float(cinn_pod_value_t* out, float v);

/* ------------------------------------------------------------------------------------------------
 * Runtime intrinsics called by host stubs.
 * ---------------------------------------------------------------------------------------------- */

/* Launch a kernel of a loaded code object.  Replaces cinn_call_cuda_kernel
 * (cinn/runtime/cuda/cuda_util.h:75-84, cuda_util.cc:78-119): `kernel_fn` is a hipFunction_t,
 * `v_args` is cinn_pod_value_t[num_args]; a buffer argument is passed as its device pointer, a
 * scalar by the address of its value; dynamic LDS is always 0.  `stream` is a hipStream_t
 * (NULL = the null stream). */
void cinn_call_hip_kernel(void* kernel_fn, void* v_args, int num_args, int grid_x, int grid_y, int grid_z,
                          int block_x, int block_y, int block_z, void* stream);
/* Same function under the name upstream host stubs already reference. */
void cinn_call_cuda_kernel(void* kernel_fn, void* v_args, int num_args, int grid_x, int grid_y, int grid_z,
                           int block_x, int block_y, int block_z, void* stream);

/* Row-major C = alpha * op(A) * op(B) + beta * C (optionally C^T when trans_o) on MFMA matrix
 * cores.  Replaces cinn_call_cublas (cuda_util.h:86-101, cuda_util.cc:121-310).  v_args = {A, B, C}
 * buffers; a1..a4 / b1..b4 are the operand shapes left-padded to 4-D; leading dims broadcast per
 * the reference rules.  Element type is taken from A's cinn_type_t (fp32, fp16, bf16, fp64);
 * 16-bit inputs accumulate in fp32. */
void cinn_call_cublas(void* v_args, int num_args, bool trans_a, bool trans_b, bool trans_o, float alpha, float beta,
                      int a1, int a2, int a3, int a4, int b1, int b2, int b3, int b4, void* stream);

/* Replaces cinn_call_batched_cublas (cuda_util.h:103-120, cuda_util.cc:312-437): v_args holds one
 * shared operand, then (num_args-1)/2 other operands, then as many outputs; opside selects which
 * side the shared operand is on (0 = left). */
void cinn_call_batched_cublas(void* v_args, int num_args, int opside, bool trans_a, bool trans_b, bool trans_o,
                              float alpha, float beta, int a1, int a2, int a3, int a4, int b1, int b2, int b3, int b4,
                              void* stream);

/* y = alpha * conv2d(x, w) + beta * y, cross-correlation, zero padding, as an implicit GEMM on
 * MFMA.  Replaces cinn_call_cudnn_conv2d_forward (cuda_util.cc:603-720).  format: 0 = NCHW,
 * 1 = NHWC with [O][KH][KW][I] filters (cudnnTensorFormat_t values), 2 = NHWC output from an NCHW
 * input and [O][I][KH][KW] filter (for inputs with few channels).  Extents are passed in
 * n, c, h, w order whatever the format.  Groups need format 0.  v_args = {x, w, y}. */
void cinn_call_cudnn_conv2d_forward(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                    int input_c, int input_h, int input_w, int filter_n, int filter_c, int filter_h,
                                    int filter_w, int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h,
                                    int dilation_w, int groups, int output_n, int output_c, int output_h,
                                    int output_w, void* stream);

/* Extension with no counterpart in the reference: the same convolution with a per-output-channel
 * affine (y = conv * scale[c] + shift[c]), an optional residual addition and an optional ReLU
 * applied in the kernel epilogue on the fp32 accumulators, so an inference batch_norm (+ shortcut
 * + relu) that follows a convolution costs no extra pass over HBM.
 * v_args = {x, w, scale, shift, y} or {x, w, scale, shift, residual, y}; scale / shift are fp32
 * [output_c]; residual has y's shape, type and layout and needs format 1 or 2.
 * relu: bit 0 = ReLU; bit 1 = a 3x3 / stride 2 / padding 1 max pooling follows the ReLU inside the kernel: y is then
 * the pooled tensor [n][(output_h - 1) / 2 + 1][(output_w - 1) / 2 + 1][output_c] while output_h / output_w stay the
 * convolution's own extents.  Bit 1 needs bit 0, format 2, no residual and the 7x7 / stride 2 / padding 3 convolution
 * of a 3-channel image in a 16-bit type (anything else aborts with a message); the graph rewrite sets it only then. */
void cinn_call_hip_conv2d_bn_relu(void* v_args, int num_args, int format, int relu, int input_n, int input_c,
                                  int input_h, int input_w, int filter_n, int filter_c, int filter_h, int filter_w,
                                  int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                                  int groups, int output_n, int output_c, int output_h, int output_w, void* stream);

/* Extension with no counterpart in the reference (there every convolution is one cudnnConvolutionForward,
 * cinn/runtime/cuda/cuda_util.cc:603-720): two 1x1, stride 1, unpadded channels-last convolutions in a row, each with the
 * epilogue of cinn_call_hip_conv2d_bn_relu, where the first one's result is wanted as well -
 *   e = act1(conv(x, w1) * scale1 + shift1 [+ residual])   [n][h][w][middle_c]
 *   y = act2(conv(e, w2) * scale2 + shift2)                [n][h][w][output_c]
 * v_args = {x, w1, scale1, shift1, [residual,] w2, scale2, shift2, e, y}; x is [n][h][w][input_c], w1
 * [middle_c][1][1][input_c], w2 [output_c][1][1][middle_c], scales / shifts fp32.  relu: bit 0 = ReLU in act1, bit 1 = in
 * act2.  For 16-bit types and the channel counts 64 -> 256 -> 64 | 128 (n h w a multiple of 16) one kernel computes
 * both and e is never read back; any other shape runs the two convolutions one after the other,
 * with the same results as two cinn_call_hip_conv2d_bn_relu calls.  The graph rewrite that emits this call
 * (FuseConvChain) only does so for shapes of the first kind. */
void cinn_call_hip_conv2d_bn_relu_chain(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w,
                                        int input_c, int middle_c, int output_c, void* stream);

/* Extension with no counterpart in the reference (there a projection shortcut is one cudnnConvolutionForward and the
 * layer that adds it another, cinn/runtime/cuda/cuda_util.cc:603-720): one 1x1 convolution over the channels of two
 * channels-last inputs that share the output's pixel grid,
 *   y[n][oy][ox][:] = act(w[:, :input_c] x[n][oy][ox][:] + w[:, input_c:] x2[n][oy second_stride_h][ox second_stride_w][:] + shift)
 * v_args = {x, x2, w, shift, y}; x is [n][h][w][input_c], x2 [n][second_h][second_w][second_c], w
 * [output_c][1][1][input_c + second_c] (each row: the weights of x's channels, then those of x2's), shift fp32 [output_c],
 * y [n][h][w][output_c]; x, x2, w and y share one 16-bit floating-point type.  relu: bit 0 = ReLU.  This is a bottleneck
 * block's last 1x1 layer and its strided 1x1 projection shortcut in one launch, once their batch-norm scales are
 * multiplied into the filters (the FuseShortcutProjection rewrite does that); the K loop of the implicit-GEMM kernel
 * walks x's channels and then x2's.  Shapes the kernel does not take (channel counts that are not multiples of 64, too
 * few output tiles: ConvPairShape in kernels/conv_chain.h) abort with a message - there is no two-launch form of this
 * call; the rewrite emits it for qualifying shapes only. */
void cinn_call_hip_conv2d_pointwise_pair(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w,
                                         int input_c, int second_h, int second_w, int second_c, int second_stride_h,
                                         int second_stride_w, int output_c, void* stream);

/* Extension with no counterpart in the reference: cinn_call_hip_conv2d_bn_relu_chain whose first layer reads a second
 * input of the same pixel grid instead of adding a residual -
 *   e = act1([w1[:, :input_c] x + w1[:, input_c:] x2] + shift1)   [n][h][w][middle_c]
 *   y = act2(conv(e, w2) * scale2 + shift2)                       [n][h][w][output_c]
 * v_args = {x, x2, w1, shift1, w2, scale2, shift2, e, y}; x is [n][h][w][input_c], x2 [n][h][w][second_c], w1
 * [middle_c][1][1][input_c + second_c], w2 [output_c][1][1][middle_c], shifts and scale fp32; 16-bit types.  relu: bit 0
 * = ReLU in act1, bit 1 = in act2.  This is the first bottleneck block of a stage whose projection shortcut has
 * stride 1: expansion and projection as one product (their batch-norm scales multiplied into w1's halves by the
 * FuseShortcutProjection rewrite), then the next block's reduction.  For 64 + 64 -> 256 -> 64 channels (n h w a multiple of
 * 16) one kernel computes both; other shapes run cinn_call_hip_conv2d_pointwise_pair and then the second layer. */
void cinn_call_hip_conv2d_pair_chain(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w, int input_c,
                                     int second_c, int middle_c, int output_c, void* stream);

/* cinn_call_cudnn_conv2d_forward for callers that cannot allocate.  No counterpart in the reference: it exists for
 * code that runs under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same arguments and
 * results as the call above for format 1 and 2 with groups == 1 (always on the general channels-last MFMA kernel);
 * it calls no hipMalloc / hipFree and no allocating library routine.  What the kernels need beyond x, w and y (a page
 * of zeros, the fp32 partial sums of a split reduction) lives in a static device array of
 * cinn_hip_conv2d_forward_noalloc_scratch_limit() = 16 MiB (+ 256 bytes) that every GPU the library runs on holds
 * until the process ends.  Returns 0 on success; 1 for an unsupported format, type, group count or shape; 2 when the
 * shape's partial sums exceed the limit (nothing is launched in either case; the reason is printed to stderr).
 * All calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads) race.
 * cinn_hip_conv2d_forward_noalloc_init looks the array's device address up for the current device ahead of time
 * (otherwise the first call on a device does). */
int cinn_call_hip_conv2d_forward_noalloc(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                         int input_c, int input_h, int input_w, int filter_n, int filter_c, int filter_h,
                                         int filter_w, int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h,
                                         int dilation_w, int groups, int output_n, int output_c, int output_h,
                                         int output_w, void* stream);
int cinn_hip_conv2d_forward_noalloc_init(void);
size_t cinn_hip_conv2d_forward_noalloc_scratch_limit(void);

/* Replaces cinn_call_cudnn_pool2d_forward (cuda_util.cc:969-1041).  mode: 0 = max,
 * 1 = avg counting padding, 2 = avg excluding padding, 3 = max (deterministic) — the
 * cudnnPoolingMode_t values.  v_args = {x, y}. */
void cinn_call_cudnn_pool2d_forward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                    int input_n, int input_c, int input_h, int input_w, int kernel_h, int kernel_w,
                                    int pad_h, int pad_w, int stride_h, int stride_w, int output_n, int output_c,
                                    int output_h, int output_w, void* stream);

/* Replaces cinn_call_cudnn_softmax_forward (cuda_util.cc:1121-1167), which always runs
 * CUDNN_SOFTMAX_LOG: y = alpha * log_softmax(x) + beta * y over C (mode 1, per position) or over
 * C*H*W (mode 0, per instance).  v_args = {x, y}. */
void cinn_call_cudnn_softmax_forward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                     int input_n, int input_c, int input_h, int input_w, int output_n, int output_c,
                                     int output_h, int output_w, void* stream);

/* argsort / sort along one axis.  The reference has no library call for them: its `argsort` and `sort` operators
 * (cinn/hlir/op/contrib/sort.cc:50-139) are generated loops over the device functions cinn_nvgpu_lt_num_* /
 * cinn_nvgpu_gt_num_* and cinn_nvgpu_next_smallest_int32 (cinn_cuda_runtime_source.cuh:645-715), whose second step
 * mutates one shared buffer from every thread.  This call gives the result that algorithm defines when run in order -
 * the stable order by (count of smaller elements, index); descending: count of larger elements - without shared
 * state.  The tensor is [outer][size][inner], sorted along `size`.  outputs: bit 0 = int32 indices, bit 1 = int32
 * positions (the count of smaller / larger elements of every element, the reference's second `argsort` output before
 * its second step consumes it), bit 2 = sorted values (the input's type); v_args = {x, then the requested outputs in
 * that order}.  fp16 / bf16 / fp32 / fp64 / int32 / int64; at most 16384 (8-byte types: 10922) elements along the
 * sorted axis. */
void cinn_call_hip_argsort(void* v_args, int num_args, int outer, int size, int inner, int is_ascend, int outputs,
                           void* stream);

/* Gradients of the three calls above, with the reference's argument lists.  Gather-form kernels (one thread or block
 * per gradient element, fp32 accumulation), formats 0 = NCHW / [F][C][KH][KW] and 1 = NHWC / [F][KH][KW][C]; every result
 * is out = alpha * gradient + beta * out.
 * cinn_call_cudnn_conv2d_backward_data (cuda_util.cc:722-843): v_args = {w, dy, dx}.
 * cinn_call_cudnn_conv2d_backward_filter (cuda_util.cc:845-967): v_args = {x, dy, dw}. */
void cinn_call_cudnn_conv2d_backward_data(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                          int input_c, int input_h, int input_w, int filter_n, int filter_c,
                                          int filter_h, int filter_w, int pad_h, int pad_w, int stride_h, int stride_w,
                                          int dilation_h, int dilation_w, int groups, int output_n, int output_c,
                                          int output_h, int output_w, void* stream);
void cinn_call_cudnn_conv2d_backward_filter(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                            int input_c, int input_h, int input_w, int filter_n, int filter_c,
                                            int filter_h, int filter_w, int pad_h, int pad_w, int stride_h,
                                            int stride_w, int dilation_h, int dilation_w, int groups, int output_n,
                                            int output_c, int output_h, int output_w, void* stream);

/* Replaces cinn_call_cudnn_pool2d_backward (cuda_util.cc:1043-1119).  v_args = {x, y, dy, dx}; modes as in the
 * forward call.  Max pooling sends a window's gradient to its first maximum (rows, then columns; x == y decides). */
void cinn_call_cudnn_pool2d_backward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                     int input_n, int input_c, int input_h, int input_w, int kernel_h, int kernel_w,
                                     int pad_h, int pad_w, int stride_h, int stride_w, int output_n, int output_c,
                                     int output_h, int output_w, void* stream);

/* Replaces cinn_call_cudnn_softmax_backward (cuda_util.cc:1169-1217), which always runs CUDNN_SOFTMAX_LOG:
 * dx = alpha * (dy - exp(y) * sum(dy)) + beta * dx over C (mode 1) or C*H*W (mode 0).  v_args = {y, dy, dx}. */
void cinn_call_cudnn_softmax_backward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                      int input_n, int input_c, int input_h, int input_w, int output_n, int output_c,
                                      int output_h, int output_w, void* stream);

/* Replace cinn_call_cuda_memset / cinn_call_cuda_memcpy (cuda_util.cc:439-462). */
void cinn_call_cuda_memset(void* v_args, int num_args, int value, size_t count, void* stream);
void cinn_call_cuda_memcpy(void* v_args, int num_args, size_t count, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Run-time compilation and code-object loading.
 * ---------------------------------------------------------------------------------------------- */

/* HIP source -> gfx950 code object through hiprtc.  Replaces nvrtc::Compiler::operator()
 * (cinn/backends/nvrtc/nvrtc_util.cc:40-152).  The device library is prepended as an in-memory
 * header when `with_device_lib` is non-zero.  On success *code / *code_size describe a malloc'd
 * image the caller frees with cinn_hip_free_host; on failure the compile log is left in
 * *log (malloc'd, may be NULL) and a non-zero status is returned. */
int cinn_hip_rtc_compile(const char* source, int with_device_lib, const char* extra_options, char** code,
                         size_t* code_size, char** log);
void cinn_hip_free_host(void* p);
/* The device library source text (wave64 reductions, math table, 128-bit access helpers) that
 * replaces cinn/runtime/cuda/cinn_cuda_runtime_source.cuh. */
const char* cinn_hip_device_lib_source(void);

/* Code-object handle.  Replaces runtime::cuda::CUDAModule (cinn/runtime/cuda/cuda_module.cc:35-149):
 * the image is loaded lazily with hipModuleLoadData on first cinn_hip_module_get_function. */
typedef struct cinn_hip_module* cinn_hip_module_t;
int cinn_hip_module_create(const void* code, size_t code_size, cinn_hip_module_t* out);
int cinn_hip_module_get_function(cinn_hip_module_t m, const char* name, void** kernel_fn);
int cinn_hip_module_destroy(cinn_hip_module_t m);

/* ------------------------------------------------------------------------------------------------
 * Device memory, streams, events.  Replace CudaMemoryMng (cinn/hlir/framework/memory.cc:43-64)
 * and the cudaMemcpy / cudaDeviceSynchronize calls of frontend/computation.cc:186-215 and
 * hlir/framework/graph_compiler.cc:212-222.
 * ---------------------------------------------------------------------------------------------- */
int cinn_hip_device_count(int* count);
int cinn_hip_malloc(void** dptr, size_t bytes);
int cinn_hip_free(void* dptr);
int cinn_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream);
int cinn_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream);
int cinn_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int cinn_hip_memset(void* dst, int value, size_t bytes, void* stream);
int cinn_hip_device_synchronize(void);
int cinn_hip_stream_create(void** stream);
int cinn_hip_stream_destroy(void* stream);
int cinn_hip_stream_synchronize(void* stream);
int cinn_hip_event_create(void** event);
int cinn_hip_event_destroy(void* event);
int cinn_hip_event_record(void* event, void* stream);
int cinn_hip_event_synchronize(void* event);
int cinn_hip_event_elapsed_ms(void* start, void* stop, float* ms);
const char* cinn_hip_error_string(int status);

/* Library-owned device scratch (partial sums of split reductions in the convolution / GEMM kernels, transposed copies
 * of GEMM operands).  The reference has no such buffer of its own: cuBLAS / cuDNN keep theirs inside their handles
 * (cinn/runtime/cuda/cuda_util.cc:45-76 CublasHandle, 465-514 CudnnHandle with its workspace).  One buffer per stream
 * and purpose, grown on demand by the cinn_call_* that needs it; an outgrown buffer is retired, not freed, because a
 * captured graph may still hold its address, and no call waits for the device.  While a stream is being captured
 * nothing can be allocated: reserve first (one eager run of the same calls does it, or this call; 0 = leave as is).
 * The call also creates the device's 256-byte page of zeros that convolution kernels read masked-out chunks from.
 * cinn_hip_scratch_release_retired frees the retired buffers; only a caller that knows that no instantiated graph
 * refers to them may call it. */
int cinn_hip_scratch_reserve(void* stream, size_t split_k_bytes, size_t transpose_bytes);
int cinn_hip_scratch_info(void* stream, size_t* split_k_capacity, size_t* transpose_capacity, size_t* retired_bytes);
int cinn_hip_scratch_release_retired(void);
/* Lifetime rule: scratch is keyed by (current device, stream handle, kind) and outlives the stream.  Call this before
 * hipStreamDestroy: the stream's buffers join the retired ones (a graph captured on the stream may still hold their
 * addresses) and a later stream that happens to get the same handle value starts empty. */
int cinn_hip_scratch_release_stream(void* stream);

/* Kernel choice of cinn_call_cudnn_conv2d_forward / cinn_call_hip_conv2d_bn_relu for 3x3, stride 1, padding 1
 * convolutions on channels-last 16-bit tensors: 0 = never the kernel that keeps the input patch resident in LDS,
 * 1 = where it is expected to win (default; FLAGS_cinn_hip_conv_patch sets the initial value), 2 = wherever the shape
 * qualifies.  Returns the previous mode; any other argument only reads it.  No counterpart in the reference (cuDNN picks
 * its algorithm inside cudnnConvolutionForward, cinn/runtime/cuda/cuda_util.cc:560-640); a tuning and test switch.
 * The setting is one atomic integer of the process: a convolution call that runs concurrently with a change uses the
 * old or the new value as a whole, never a mixture. */
int cinn_hip_conv_patch_mode(int mode);
/* Block size of that kernel for more than 64 input channels: 4 or 2 tiles of 16 pixel slots per computing wavefront
 * (256 or 128 slots per block); 0 = chosen per shape (2 when 4 would give fewer than 192 blocks and 2 gives more).
 * Returns the previous setting; another value only reads it.  Initial value from FLAGS_cinn_hip_conv_patch_tiles.
 * Atomic like the mode above. */
int cinn_hip_conv_patch_tiles(int tiles);
/* The same kernel family for exactly 64 input channels: 1 = the form that walks the pixels in its outer loop with the
 * whole filter in registers, so that a tile's results are stored while the next is multiplied (default), 0 = the form
 * that walks the filter taps in its outer loop and stores at the end.  Both give the same bits.  Returns the previous
 * setting; another value only reads it.  Initial value from FLAGS_cinn_hip_conv_patch_stream.  Atomic like the mode. */
int cinn_hip_conv_patch_stream(int on);
/* cinn_call_hip_conv2d_bn_relu_chain: 1 = one kernel where the shape qualifies (default; initial value from
 * FLAGS_cinn_hip_conv_chain), 0 = always the two convolutions one after the other.  Returns the previous setting;
 * another value only reads it.  Atomic like the mode. */
int cinn_hip_conv_chain_mode(int mode);
/* Device descriptor consumed by schedules.  Replaces common::Target's cudaDeviceGetAttribute
 * queries (cinn/common/target.cc:55-84, 177-221).  Filled from the live device when one is
 * present, otherwise with the MI355X datasheet values (256 CUs, wave64, 160 KiB LDS per CU). */
typedef struct cinn_hip_target_info {
  int wavefront_size;
  int max_threads_per_block;
  int multi_processor_count;
  int max_threads_per_multi_processor;
  int max_blocks_per_multi_processor;
  int lds_bytes_per_block;
  int lds_bytes_per_multi_processor;
  int num_xcd;
  int from_device; /* 1 when read from a live GPU */
  char arch[32];
} cinn_hip_target_info;
int cinn_hip_get_target_info(cinn_hip_target_info* info);

#ifdef __cplusplus
}
#endif
#endif /* CINN_HIP_RUNTIME_H_ */
