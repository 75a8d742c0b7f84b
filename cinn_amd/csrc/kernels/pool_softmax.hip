// Pooling and log-softmax kernels behind cinn_call_cudnn_pool2d_forward / cinn_call_cudnn_softmax_forward.
// Both are HBM-bound gather / reduce kernels with little reuse: one thread per output element for pooling
// (consecutive threads on consecutive output columns, so input rows are read with unit stride inside a
// window row), one block per softmax group.
//
// Pooling follows pe::PoolImpl (cinn/hlir/pe/nn.cc:956-1109): max pads with the lowest value of the type;
// avg divides every element by the divisor BEFORE adding (divisor = window positions inside the input for
// the exclusive mode, kh*kw otherwise), window rows then columns in ascending order.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <climits>
#include <cstdint>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace {

struct PoolParams {
  int n, c, ih, iw, oh, ow, kh, kw, ph, pw, sh, sw;
  int mode;  // 0 / 3 max, 1 avg counting padding, 2 avg excluding padding
  float alpha, beta;
};

template <typename T>
__global__ void __launch_bounds__(256) pool2d_nchw_kernel(const T* __restrict__ in, T* __restrict__ out, PoolParams p) {
  const int64_t total = (int64_t)p.n * p.c * p.oh * p.ow;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int x   = (int)(idx % p.ow);
  const int y   = (int)((idx / p.ow) % p.oh);
  const int64_t plane = idx / ((int64_t)p.ow * p.oh);
  const T* src  = in + plane * p.ih * p.iw;
  const int ys = y * p.sh - p.ph, xs = x * p.sw - p.pw;
  float result;
  if (p.mode == 0 || p.mode == 3) {
    float m = -3.402823466e+38f;
    for (int ry = 0; ry < p.kh; ++ry) {
      const int yy = ys + ry;
      if (yy < 0 || yy >= p.ih) continue;
      for (int rx = 0; rx < p.kw; ++rx) {
        const int xx = xs + rx;
        if (xx < 0 || xx >= p.iw) continue;
        const float v = (float)src[yy * p.iw + xx];
        m             = v > m ? v : m;
      }
    }
    result = m;
  } else {
    float factor = (float)(p.kh * p.kw);
    if (p.mode == 2) {
      const int y0 = ys > 0 ? ys : 0, x0 = xs > 0 ? xs : 0;
      const int y1 = ys + p.kh < p.ih ? ys + p.kh : p.ih, x1 = xs + p.kw < p.iw ? xs + p.kw : p.iw;
      const int count = (y1 - y0) * (x1 - x0);
      factor          = (float)(count > 1 ? count : 1);
    }
    float acc = 0.0f;
    for (int ry = 0; ry < p.kh; ++ry) {
      const int yy = ys + ry;
      for (int rx = 0; rx < p.kw; ++rx) {
        const int xx = xs + rx;
        float v      = 0.0f;
        if (yy >= 0 && yy < p.ih && xx >= 0 && xx < p.iw) v = (float)src[yy * p.iw + xx];
        acc += v / factor;
      }
    }
    result = acc;
  }
  float v = p.alpha * result;
  if (p.beta != 0.0f) v += p.beta * (float)out[idx];
  out[idx] = (T)v;
}


// fp64 tensors, either layout: one thread per output element, the arithmetic of the kernel above in double
__global__ void __launch_bounds__(256) pool2d_f64_kernel(const double* __restrict__ in, double* __restrict__ out, PoolParams p,
                                                         int nhwc) {
  const int64_t total = (int64_t)p.n * p.c * p.oh * p.ow;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int x, y, c;
  int64_t n;
  if (nhwc) {
    c = (int)(idx % p.c);
    x = (int)((idx / p.c) % p.ow);
    y = (int)((idx / ((int64_t)p.c * p.ow)) % p.oh);
    n = idx / ((int64_t)p.c * p.ow * p.oh);
  } else {
    x = (int)(idx % p.ow);
    y = (int)((idx / p.ow) % p.oh);
    c = (int)((idx / ((int64_t)p.ow * p.oh)) % p.c);
    n = idx / ((int64_t)p.ow * p.oh * p.c);
  }
  auto at = [&](int yy, int xx) -> double {
    return nhwc ? in[((n * p.ih + yy) * p.iw + xx) * p.c + c] : in[((n * p.c + c) * p.ih + yy) * p.iw + xx];
  };
  const int ys = y * p.sh - p.ph, xs = x * p.sw - p.pw;
  double result;
  if (p.mode == 0 || p.mode == 3) {
    double m = -1.7976931348623157e+308;
    for (int ry = 0; ry < p.kh; ++ry) {
      const int yy = ys + ry;
      if (yy < 0 || yy >= p.ih) continue;
      for (int rx = 0; rx < p.kw; ++rx) {
        const int xx = xs + rx;
        if (xx < 0 || xx >= p.iw) continue;
        const double v = at(yy, xx);
        m              = v > m ? v : m;
      }
    }
    result = m;
  } else {
    double factor = (double)(p.kh * p.kw);
    if (p.mode == 2) {
      const int y0 = ys > 0 ? ys : 0, x0 = xs > 0 ? xs : 0;
      const int y1 = ys + p.kh < p.ih ? ys + p.kh : p.ih, x1 = xs + p.kw < p.iw ? xs + p.kw : p.iw;
      const int count = (y1 - y0) * (x1 - x0);
      factor          = (double)(count > 1 ? count : 1);
    }
    double acc = 0.0;
    for (int ry = 0; ry < p.kh; ++ry) {
      const int yy = ys + ry;
      for (int rx = 0; rx < p.kw; ++rx) {
        const int xx = xs + rx;
        double v     = 0.0;
        if (yy >= 0 && yy < p.ih && xx >= 0 && xx < p.iw) v = at(yy, xx);
        acc += v / factor;
      }
    }
    result = acc;
  }
  double v = (double)p.alpha * result;
  if (p.beta != 0.0f) v += (double)p.beta * out[idx];
  out[idx] = v;
}

// Channels-last pooling: one thread per output pixel and group of V consecutive channels (V elements = 16 bytes
// when the channel count allows), so that every access is one contiguous vector and consecutive lanes read
// consecutive vectors.  Arithmetic and order of operations are those of the NCHW kernel.
// Blocks are dispatched round-robin to the 8 XCDs, each with an L2 of its own; the grid (a multiple of 8 blocks) is
// renumbered so that an XCD works on one contiguous eighth of the output, and overlapping windows of neighbouring
// output rows find their shared input rows in that XCD's L2 instead of fetching them once per XCD.
template <typename T, int V>
__global__ void __launch_bounds__(256) pool2d_nhwc_kernel(const T* __restrict__ in, T* __restrict__ out, PoolParams p) {
  const int groups    = p.c / V;
  const int64_t total = (int64_t)p.n * p.oh * p.ow * groups;
  const unsigned block = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int64_t idx   = (int64_t)block * 256 + threadIdx.x;
  if (idx >= total) return;
  const int g         = (int)(idx % groups);
  const int64_t pixel = idx / groups;
  const int x         = (int)(pixel % p.ow);
  const int y         = (int)((pixel / p.ow) % p.oh);
  const int64_t n     = pixel / ((int64_t)p.ow * p.oh);
  const T* src        = in + n * p.ih * p.iw * p.c + g * V;
  const int ys = y * p.sh - p.ph, xs = x * p.sw - p.pw;
  const bool is_max = p.mode == 0 || p.mode == 3;
  float acc[V];
  float factor = (float)(p.kh * p.kw);
  if (p.mode == 2) {
    const int y0 = ys > 0 ? ys : 0, x0 = xs > 0 ? xs : 0;
    const int y1 = ys + p.kh < p.ih ? ys + p.kh : p.ih, x1 = xs + p.kw < p.iw ? xs + p.kw : p.iw;
    const int count = (y1 - y0) * (x1 - x0);
    factor          = (float)(count > 1 ? count : 1);
  }
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = is_max ? -3.402823466e+38f : 0.0f;
  for (int ry = 0; ry < p.kh; ++ry) {
    const int yy = ys + ry;
    if (yy < 0 || yy >= p.ih) continue;
    for (int rx = 0; rx < p.kw; ++rx) {
      const int xx = xs + rx;
      if (xx < 0 || xx >= p.iw) continue;
      T v[V];
      __builtin_memcpy(v, src + ((int64_t)yy * p.iw + xx) * p.c, V * sizeof(T));
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float f = (float)v[e];
        if (is_max)
          acc[e] = f > acc[e] ? f : acc[e];
        else
          acc[e] += f / factor;
      }
    }
  }
  T* dst = out + pixel * p.c + g * V;
  T res[V];
  if (p.beta != 0.0f) __builtin_memcpy(res, dst, V * sizeof(T));
#pragma unroll
  for (int e = 0; e < V; ++e) {
    float r = p.alpha * acc[e];
    if (p.beta != 0.0f) r += p.beta * (float)res[e];
    res[e] = (T)r;
  }
  __builtin_memcpy(dst, res, V * sizeof(T));
}


// Max pooling of fp16 channels-last tensors with a small window (3x3 stride 2 after the first convolution of an image
// network): the generic kernel above spends ~800 instructions per thread - 64-bit index divisions, a float conversion
// and a compare / select pair per element and tap - and is bound by them, not by memory (25 us for 64 MB at batch 32).
// Here the indices are 32-bit, the window is unrolled with clamped, unconditional loads (all in flight together), taps
// outside the image are replaced by -inf, and the maximum is taken on packed halves.  The maximum of halves is exact,
// so results equal the generic kernel's (which compares the same values as floats) except that max(+0, -0) may carry
// either sign.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
template <int KH, int KW>
__global__ void __launch_bounds__(256) maxpool_nhwc_f16_kernel(const _Float16* __restrict__ in, _Float16* __restrict__ out,
                                                               PoolParams p) {
  const unsigned groups = (unsigned)p.c >> 3;
  const unsigned total  = (unsigned)p.n * p.oh * p.ow * groups;
  const unsigned block  = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);  // an XCD works on one eighth
  const unsigned idx    = block * 256u + threadIdx.x;
  if (idx >= total) return;
  const unsigned pixel = idx / groups, g = idx - pixel * groups;
  const unsigned t = pixel / (unsigned)p.ow, x = pixel - t * p.ow;
  const unsigned n = t / (unsigned)p.oh, y = t - n * p.oh;
  const _Float16* src = in + (int64_t)n * p.ih * p.iw * p.c + g * 8;
  const int ys = (int)y * p.sh - p.ph, xs = (int)x * p.sw - p.pw;
  const _Float16 ninf = -__builtin_huge_valf();
  half8 v[KH][KW];
#pragma unroll
  for (int ry = 0; ry < KH; ++ry) {
    const int yy = ys + ry, yc = yy < 0 ? 0 : (yy < p.ih ? yy : p.ih - 1);
#pragma unroll
    for (int rx = 0; rx < KW; ++rx) {
      const int xx = xs + rx, xc = xx < 0 ? 0 : (xx < p.iw ? xx : p.iw - 1);
      v[ry][rx]    = *reinterpret_cast<const half8*>(src + (unsigned)((yc * p.iw + xc) * p.c));
    }
  }
  half8 acc;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = ninf;
#pragma unroll
  for (int ry = 0; ry < KH; ++ry)
#pragma unroll
    for (int rx = 0; rx < KW; ++rx) {
      const bool ok = (unsigned)(ys + ry) < (unsigned)p.ih && (unsigned)(xs + rx) < (unsigned)p.iw;
      half8 tap     = v[ry][rx];
#pragma unroll
      for (int e = 0; e < 8; ++e) tap[e] = ok ? tap[e] : ninf;
      acc = __builtin_elementwise_max(acc, tap);
    }
  *reinterpret_cast<half8*>(out + (int64_t)pixel * p.c + g * 8) = acc;
}

// Channels-last pooling whose window is the whole image (global average / max pooling): the generic kernel would give
// each thread the entire image of its channels to walk through.  Here a block of 256 threads takes one image and 64
// channels: 8 channel groups of 8 x 32 pixel slices, partial results combined through LDS.  The average still divides
// every element before adding; only the order of the additions differs from the generic kernel.
template <typename T, int V>
__global__ void __launch_bounds__(256) global_pool_nhwc_kernel(const T* __restrict__ in, T* __restrict__ out, PoolParams p) {
  constexpr int GROUPS = 8;   // channel groups per block
  constexpr int SLICES = 32;  // pixel slices
  __shared__ float partial[SLICES][GROUPS * V + 1];
  const int groups_per_image = (p.c / V + GROUPS - 1) / GROUPS;
  const int n     = blockIdx.x / groups_per_image;
  const int g     = (blockIdx.x % groups_per_image) * GROUPS + (threadIdx.x % GROUPS);
  const int slice = threadIdx.x / GROUPS;
  const bool is_max = p.mode == 0 || p.mode == 3;
  const int pixels  = p.ih * p.iw;
  const float factor = (float)pixels;
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = is_max ? -3.402823466e+38f : 0.0f;
  if (g * V < p.c) {
    const T* src = in + (int64_t)n * pixels * p.c + g * V;
    for (int px = slice; px < pixels; px += SLICES) {
      T v[V];
      __builtin_memcpy(v, src + (int64_t)px * p.c, V * sizeof(T));
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float f = (float)v[e];
        if (is_max)
          acc[e] = f > acc[e] ? f : acc[e];
        else
          acc[e] += f / factor;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) partial[slice][(threadIdx.x % GROUPS) * V + e] = acc[e];
  __syncthreads();
  // thread t < GROUPS * V finishes channel t of the block
  if (threadIdx.x < GROUPS * V) {
    const int c = (blockIdx.x % groups_per_image) * GROUPS * V + threadIdx.x;
    if (c < p.c) {
      float r = is_max ? -3.402823466e+38f : 0.0f;
      for (int s2 = 0; s2 < SLICES; ++s2) {
        const float f = partial[s2][threadIdx.x];
        r             = is_max ? (f > r ? f : r) : r + f;
      }
      T* dst = out + (int64_t)n * p.c + c;
      r      = p.alpha * r;
      if (p.beta != 0.0f) r += p.beta * (float)*dst;
      *dst = (T)r;
    }
  }
}

template <typename T>
void LaunchPoolNhwc(const void* x, void* y, const PoolParams& p, hipStream_t s) {
  constexpr int V = 16 / sizeof(T);
  const bool global = p.oh == 1 && p.ow == 1 && p.kh == p.ih && p.kw == p.iw && p.ph == 0 && p.pw == 0;
  if (global && p.c % V == 0 && p.ih * p.iw >= 16) {
    const int groups_per_image = (p.c / V + 7) / 8;
    hipLaunchKernelGGL((global_pool_nhwc_kernel<T, V>), dim3((unsigned)(p.n * groups_per_image)), dim3(256), 0, s,
                       static_cast<const T*>(x), static_cast<T*>(y), p);
    return;
  }
  if (sizeof(T) == 2 && p.c % 8 == 0) {
    // fp16 max pooling with a 3x3 window and no alpha / beta: the packed-half kernel
    const int64_t total = (int64_t)p.n * p.oh * p.ow * (p.c / 8);
    const bool is_f16   = std::is_same<T, _Float16>::value;
    if (is_f16 && (p.mode == 0 || p.mode == 3) && p.kh == 3 && p.kw == 3 && p.alpha == 1.0f && p.beta == 0.0f &&
        total < (1ll << 31) && (int64_t)p.ih * p.iw * p.c < (1ll << 31)) {
      hipLaunchKernelGGL((maxpool_nhwc_f16_kernel<3, 3>), dim3((unsigned)(((total + 255) / 256 + 7) / 8 * 8)), dim3(256), 0, s,
                         static_cast<const _Float16*>(x), static_cast<_Float16*>(y), p);
      return;
    }
  }
  if (p.c % V == 0) {
    const int64_t total = (int64_t)p.n * p.oh * p.ow * (p.c / V);
    hipLaunchKernelGGL((pool2d_nhwc_kernel<T, V>), dim3((unsigned)(((total + 255) / 256 + 7) / 8 * 8)), dim3(256), 0, s,
                       static_cast<const T*>(x), static_cast<T*>(y), p);
  } else {
    const int64_t total = (int64_t)p.n * p.oh * p.ow * p.c;
    hipLaunchKernelGGL((pool2d_nhwc_kernel<T, 1>), dim3((unsigned)(((total + 255) / 256 + 7) / 8 * 8)), dim3(256), 0, s,
                       static_cast<const T*>(x), static_cast<T*>(y), p);
  }
}

// block-wide reduction helper over 256 threads
template <typename OP>
__device__ __forceinline__ float BlockReduce(float v, float* scratch, OP op) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return op(op(scratch[0], scratch[1]), op(scratch[2], scratch[3]));
}

// y = alpha * log_softmax(x) + beta * y over `len` elements at stride `stride`, one block per group.
// group g = (outer, inner): base = outer * len * stride_outer_unit + inner
template <typename T>
__global__ void __launch_bounds__(256) log_softmax_kernel(const T* __restrict__ in, T* __restrict__ out, int len, int inner,
                                                          float alpha, float beta) {
  __shared__ float scratch[4];
  const int64_t g     = blockIdx.x;
  const int64_t outer = g / inner, in_idx = g % inner;
  const int64_t base  = outer * len * inner + in_idx;
  float m = -3.402823466e+38f;
  for (int i = threadIdx.x; i < len; i += 256) {
    float v = (float)in[base + (int64_t)i * inner];
    m       = v > m ? v : m;
  }
  m = BlockReduce(m, scratch, [](float a, float b) { return a > b ? a : b; });
  float s = 0.0f;
  for (int i = threadIdx.x; i < len; i += 256) s += expf((float)in[base + (int64_t)i * inner] - m);
  s = BlockReduce(s, scratch, [](float a, float b) { return a + b; });
  const float lse = m + logf(s);
  for (int i = threadIdx.x; i < len; i += 256) {
    const int64_t at = base + (int64_t)i * inner;
    float v          = alpha * ((float)in[at] - lse);
    if (beta != 0.0f) v += beta * (float)out[at];
    out[at] = (T)v;
  }
}

cinn_buffer_t* BufferArg(void* v_args, int index) {
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  CINN_RT_CHECK(args[index].type_code_ == CINN_POD_BUFFER_P, "argument %d is not a buffer", index);
  return static_cast<cinn_buffer_t*>(args[index].value_.v_handle);
}

enum class Elem { kF32, kF16, kBF16, kF64 };
Elem ElemOf(const cinn_buffer_t* b) {
  const int bytes = b->type.bits / CHAR_BIT;
  if (b->type.code == cinn_type_float && bytes == 8) return Elem::kF64;
  if (b->type.code == cinn_type_float && bytes == 4) return Elem::kF32;
  if (b->type.code == cinn_type_float && bytes == 2) return Elem::kF16;
  if (b->type.code == cinn_type_bfloat) return Elem::kBF16;
  fprintf(stderr, "unsupported data type code %d bits %d\n", b->type.code, b->type.bits);
  abort();
}

}  // namespace

extern "C" {

void cinn_call_cudnn_pool2d_forward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                    int input_n, int input_c, int input_h, int input_w, int kernel_h, int kernel_w,
                                    int pad_h, int pad_w, int stride_h, int stride_w, int output_n, int output_c,
                                    int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 2, "cinn_call_cudnn_pool2d_forward takes x and y, got %d arguments", num_args);
  CINN_RT_CHECK(format == 0 || format == 1, "pool2d: unknown tensor format %d", format);
  CINN_RT_CHECK(mode >= 0 && mode <= 3, "pool2d: unknown pooling mode %d", mode);
  CINN_RT_CHECK(output_n == input_n && output_c == input_c, "pool2d: batch / channel mismatch");
  CINN_RT_CHECK(kernel_h > 0 && kernel_w > 0 && stride_h > 0 && stride_w > 0 && output_h > 0 && output_w > 0,
                "pool2d: kernel, stride and output sizes must be positive");
  // the last window must start inside the padded input
  CINN_RT_CHECK((output_h - 1) * stride_h - pad_h < input_h && (output_w - 1) * stride_w - pad_w < input_w,
                "pool2d: output %dx%d does not fit input %dx%d", output_h, output_w, input_h, input_w);
  cinn_buffer_t* x = BufferArg(v_args, 0);
  cinn_buffer_t* y = BufferArg(v_args, 1);
  PoolParams p{input_n, input_c, input_h, input_w, output_h, output_w, kernel_h, kernel_w, pad_h, pad_w, stride_h,
               stride_w, mode,    alpha,   beta};
  const int64_t total = (int64_t)input_n * input_c * output_h * output_w;
  CINN_RT_CHECK((int64_t)input_c * input_h * input_w * input_n < INT_MAX && total < INT_MAX, "pool2d: tensor too large");
  dim3 grid((unsigned)((total + 255) / 256));
  auto s = static_cast<hipStream_t>(stream);
  if (ElemOf(x) == Elem::kF64) {
    hipLaunchKernelGGL(pool2d_f64_kernel, grid, dim3(256), 0, s, reinterpret_cast<const double*>(x->memory),
                       reinterpret_cast<double*>(y->memory), p, format);
    CINN_HIP_CALL(hipGetLastError());
    return;
  }
  if (format == 1) {
    switch (ElemOf(x)) {
      case Elem::kF64: break;  // taken above
      case Elem::kF32: LaunchPoolNhwc<float>(x->memory, y->memory, p, s); break;
      case Elem::kF16: LaunchPoolNhwc<_Float16>(x->memory, y->memory, p, s); break;
      case Elem::kBF16: LaunchPoolNhwc<__bf16>(x->memory, y->memory, p, s); break;
    }
    CINN_HIP_CALL(hipGetLastError());
    return;
  }
  switch (ElemOf(x)) {
    case Elem::kF64: break;  // taken above
    case Elem::kF32:
      hipLaunchKernelGGL(pool2d_nchw_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(x->memory),
                         reinterpret_cast<float*>(y->memory), p);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(pool2d_nchw_kernel<_Float16>, grid, dim3(256), 0, s, reinterpret_cast<const _Float16*>(x->memory),
                         reinterpret_cast<_Float16*>(y->memory), p);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(pool2d_nchw_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(x->memory),
                         reinterpret_cast<__bf16*>(y->memory), p);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

void cinn_call_cudnn_softmax_forward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                     int input_n, int input_c, int input_h, int input_w, int output_n, int output_c,
                                     int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 2, "cinn_call_cudnn_softmax_forward takes x and y, got %d arguments", num_args);
  CINN_RT_CHECK(format == 0, "softmax: only NCHW (format 0) is implemented, got format %d", format);
  CINN_RT_CHECK(mode == 0 || mode == 1, "softmax: unknown mode %d", mode);
  CINN_RT_CHECK(input_n == output_n && input_c == output_c && input_h == output_h && input_w == output_w,
                "softmax: input and output shapes differ");
  cinn_buffer_t* x = BufferArg(v_args, 0);
  cinn_buffer_t* y = BufferArg(v_args, 1);
  // mode 1 (per position): groups = n * h * w, length c, stride h*w; mode 0 (per instance): groups = n
  const int len   = mode == 1 ? input_c : input_c * input_h * input_w;
  const int inner = mode == 1 ? input_h * input_w : 1;
  const int64_t groups = (int64_t)input_n * inner;
  CINN_RT_CHECK(groups > 0 && groups < INT_MAX && len > 0, "softmax: bad extents");
  dim3 grid((unsigned)groups);
  auto s = static_cast<hipStream_t>(stream);
  switch (ElemOf(x)) {
    case Elem::kF64: CINN_RT_CHECK(false, "softmax: fp64 tensors are not implemented"); break;
    case Elem::kF32:
      hipLaunchKernelGGL(log_softmax_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(x->memory),
                         reinterpret_cast<float*>(y->memory), len, inner, alpha, beta);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(log_softmax_kernel<_Float16>, grid, dim3(256), 0, s, reinterpret_cast<const _Float16*>(x->memory),
                         reinterpret_cast<_Float16*>(y->memory), len, inner, alpha, beta);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(log_softmax_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(x->memory),
                         reinterpret_cast<__bf16*>(y->memory), len, inner, alpha, beta);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

}  // extern "C"
