// Backward intrinsics of the vendor-library call sites: cinn_call_cudnn_conv2d_backward_data /
// cinn_call_cudnn_conv2d_backward_filter (cinn/runtime/cuda/cuda_util.cc:722-967), cinn_call_cudnn_pool2d_backward
// (1043-1119) and cinn_call_cudnn_softmax_backward (1169-1217).  Same argument lists and tensor formats
// (0 = NCHW with [F][C][KH][KW] filters, 1 = NHWC with [F][KH][KW][C] filters), results
// out = alpha * gradient + beta * out, fp32 accumulation for fp32 / fp16 / bf16 tensors, fp64 for fp64 tensors.
//
// These are the straightforward gather forms - one thread (or, for the filter gradient, one block) per gradient
// element, summing its contributions in a fixed order - not tiled MFMA kernels: the inference path never calls them.
//   dx[n,c,iy,ix] = sum over f of the group, ky, kx with iy = oy * stride - pad + ky * dilation (same in x):
//                   dy[n,f,oy,ox] * w[f,c',ky,kx]
//   dw[f,c',ky,kx] = sum over n, oy, ox: x[n,c,oy * stride - pad + ky * dilation, ...] * dy[n,f,oy,ox]
//   max pooling: the gradient of a window goes to its first maximum in (ky, kx) order (x == y decides, as the
//                library compares the forward output with the input); average pooling divides by kh * kw (mode 1)
//                or by the number of window positions inside the input (mode 2)
//   log-softmax (the only algorithm the reference requests): dx = dy - exp(y) * sum(dy) over the softmax axis
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace {

cinn_buffer_t* Arg(void* v_args, int index) {
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
  fprintf(stderr, "backward intrinsic: unsupported data type code %d bits %d\n", b->type.code, b->type.bits);
  abort();
}

// the type sums are kept in
template <typename T>
struct AccOf {
  typedef float type;
};
template <>
struct AccOf<double> {
  typedef double type;
};
__device__ __forceinline__ float Fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double Fma(double a, double b, double c) { return __builtin_fma(a, b, c); }

struct ConvDims {
  int n, c, ih, iw;      // input
  int f, fc, kh, kw;     // filter: f output channels, fc = c / groups input channels each
  int oh, ow;
  int ph, pw, sh, sw, dh, dw, groups;
  int nhwc;
  float alpha, beta;
};

// element offsets in either format
__device__ __forceinline__ int64_t TensorAt(int nhwc, int C, int H, int W, int n, int c, int h, int w) {
  return nhwc ? (((int64_t)n * H + h) * W + w) * C + c : (((int64_t)n * C + c) * H + h) * W + w;
}
__device__ __forceinline__ int64_t FilterAt(int nhwc, int FC, int KH, int KW, int f, int c, int ky, int kx) {
  return nhwc ? (((int64_t)f * KH + ky) * KW + kx) * FC + c : (((int64_t)f * FC + c) * KH + ky) * KW + kx;
}

template <typename T>
__global__ void __launch_bounds__(256)
conv_backward_data_kernel(const T* __restrict__ w, const T* __restrict__ dy, T* __restrict__ dx, ConvDims p) {
  const int64_t total = (int64_t)p.n * p.c * p.ih * p.iw;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  // idx enumerates dx in its own memory order, so that consecutive threads write consecutive elements
  int n, c, iy, ix;
  if (p.nhwc) {
    c  = (int)(idx % p.c);
    ix = (int)((idx / p.c) % p.iw);
    iy = (int)((idx / ((int64_t)p.c * p.iw)) % p.ih);
    n  = (int)(idx / ((int64_t)p.c * p.iw * p.ih));
  } else {
    ix = (int)(idx % p.iw);
    iy = (int)((idx / p.iw) % p.ih);
    c  = (int)((idx / ((int64_t)p.iw * p.ih)) % p.c);
    n  = (int)(idx / ((int64_t)p.iw * p.ih * p.c));
  }
  const int g = c / p.fc, cl = c - g * p.fc;
  const int fg = p.f / p.groups;
  typedef typename AccOf<T>::type Acc;
  Acc acc = 0;
  for (int fl = 0; fl < fg; ++fl) {
    const int f = g * fg + fl;
    for (int ky = 0; ky < p.kh; ++ky) {
      const int ty = iy + p.ph - ky * p.dh;
      if (ty < 0 || ty % p.sh != 0) continue;
      const int oy = ty / p.sh;
      if (oy >= p.oh) continue;
      for (int kx = 0; kx < p.kw; ++kx) {
        const int tx = ix + p.pw - kx * p.dw;
        if (tx < 0 || tx % p.sw != 0) continue;
        const int ox = tx / p.sw;
        if (ox >= p.ow) continue;
        acc = Fma((Acc)dy[TensorAt(p.nhwc, p.f, p.oh, p.ow, n, f, oy, ox)],
                  (Acc)w[FilterAt(p.nhwc, p.fc, p.kh, p.kw, f, cl, ky, kx)], acc);
      }
    }
  }
  Acc v = (Acc)p.alpha * acc;
  if (p.beta != 0.0f) v += (Acc)p.beta * (Acc)dx[idx];
  dx[idx] = (T)v;
}

// one block per filter-gradient element: the 256 threads stride over (n, oy, ox), partial sums meet in LDS
template <typename T>
__global__ void __launch_bounds__(256)
conv_backward_filter_kernel(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ dw, ConvDims p) {
  typedef typename AccOf<T>::type Acc;
  __shared__ Acc partial[256];
  const int64_t e = blockIdx.x;  // dw in its own memory order
  int f, cl, ky, kx;
  if (p.nhwc) {
    cl = (int)(e % p.fc);
    kx = (int)((e / p.fc) % p.kw);
    ky = (int)((e / ((int64_t)p.fc * p.kw)) % p.kh);
    f  = (int)(e / ((int64_t)p.fc * p.kw * p.kh));
  } else {
    kx = (int)(e % p.kw);
    ky = (int)((e / p.kw) % p.kh);
    cl = (int)((e / ((int64_t)p.kw * p.kh)) % p.fc);
    f  = (int)(e / ((int64_t)p.kw * p.kh * p.fc));
  }
  const int fg = p.f / p.groups;
  const int c  = (f / fg) * p.fc + cl;
  const int64_t positions = (int64_t)p.n * p.oh * p.ow;
  Acc acc = 0;
  for (int64_t q = threadIdx.x; q < positions; q += 256) {
    const int ox = (int)(q % p.ow);
    const int oy = (int)((q / p.ow) % p.oh);
    const int n  = (int)(q / ((int64_t)p.ow * p.oh));
    const int iy = oy * p.sh - p.ph + ky * p.dh, ix = ox * p.sw - p.pw + kx * p.dw;
    if (iy < 0 || iy >= p.ih || ix < 0 || ix >= p.iw) continue;
    acc = Fma((Acc)x[TensorAt(p.nhwc, p.c, p.ih, p.iw, n, c, iy, ix)],
              (Acc)dy[TensorAt(p.nhwc, p.f, p.oh, p.ow, n, f, oy, ox)], acc);
  }
  partial[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) partial[threadIdx.x] += partial[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    Acc v = (Acc)p.alpha * partial[0];
    if (p.beta != 0.0f) v += (Acc)p.beta * (Acc)dw[e];
    dw[e] = (T)v;
  }
}

struct PoolDims {
  int n, c, ih, iw, oh, ow, kh, kw, ph, pw, sh, sw;
  int mode, nhwc;
  float alpha, beta;
};

template <typename T>
__global__ void __launch_bounds__(256)
pool_backward_kernel(const T* __restrict__ x, const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx,
                     PoolDims p) {
  const int64_t total = (int64_t)p.n * p.c * p.ih * p.iw;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int n, c, iy, ix;
  if (p.nhwc) {
    c  = (int)(idx % p.c);
    ix = (int)((idx / p.c) % p.iw);
    iy = (int)((idx / ((int64_t)p.c * p.iw)) % p.ih);
    n  = (int)(idx / ((int64_t)p.c * p.iw * p.ih));
  } else {
    ix = (int)(idx % p.iw);
    iy = (int)((idx / p.iw) % p.ih);
    c  = (int)((idx / ((int64_t)p.iw * p.ih)) % p.c);
    n  = (int)(idx / ((int64_t)p.iw * p.ih * p.c));
  }
  typedef typename AccOf<T>::type Acc;
  const bool is_max = p.mode == 0 || p.mode == 3;
  const Acc mine    = (Acc)x[idx];
  Acc acc = 0;
  // windows (oy, ox) that contain (iy, ix): oy * sh - ph <= iy < oy * sh - ph + kh
  for (int oy = 0; oy < p.oh; ++oy) {
    const int ys = oy * p.sh - p.ph;
    if (iy < ys || iy >= ys + p.kh) continue;
    for (int ox = 0; ox < p.ow; ++ox) {
      const int xs = ox * p.sw - p.pw;
      if (ix < xs || ix >= xs + p.kw) continue;
      const int64_t o = TensorAt(p.nhwc, p.c, p.oh, p.ow, n, c, oy, ox);
      const Acc g     = (Acc)dy[o];
      if (is_max) {
        const Acc m = (Acc)y[o];
        if (mine != m) continue;
        // the first element of the window (rows, then columns) that equals the maximum takes the gradient
        bool first = true;
        for (int ry = 0; ry < p.kh && first; ++ry) {
          const int yy = ys + ry;
          if (yy < 0 || yy >= p.ih) continue;
          for (int rx = 0; rx < p.kw; ++rx) {
            const int xx = xs + rx;
            if (xx < 0 || xx >= p.iw) continue;
            if (yy == iy && xx == ix) { ry = p.kh; break; }
            if ((Acc)x[TensorAt(p.nhwc, p.c, p.ih, p.iw, n, c, yy, xx)] == m) { first = false; break; }
          }
        }
        if (first) acc += g;
      } else {
        Acc factor = (Acc)(p.kh * p.kw);
        if (p.mode == 2) {
          const int y0 = ys > 0 ? ys : 0, x0 = xs > 0 ? xs : 0;
          const int y1 = ys + p.kh < p.ih ? ys + p.kh : p.ih, x1 = xs + p.kw < p.iw ? xs + p.kw : p.iw;
          const int count = (y1 - y0) * (x1 - x0);
          factor          = (Acc)(count > 1 ? count : 1);
        }
        acc += g / factor;
      }
    }
  }
  Acc v = (Acc)p.alpha * acc;
  if (p.beta != 0.0f) v += (Acc)p.beta * (Acc)dx[idx];
  dx[idx] = (T)v;
}

// one block per softmax group: `len` elements `inner` apart
template <typename T>
__global__ void __launch_bounds__(256)
log_softmax_backward_kernel(const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int len, int inner,
                            float alpha, float beta) {
  __shared__ float partial[256];
  const int64_t group = blockIdx.x;
  const int64_t base  = (group / inner) * (int64_t)len * inner + group % inner;
  float s = 0.0f;
  for (int i = threadIdx.x; i < len; i += 256) s += (float)dy[base + (int64_t)i * inner];
  partial[threadIdx.x] = s;
  __syncthreads();
  for (int k = 128; k > 0; k >>= 1) {
    if ((int)threadIdx.x < k) partial[threadIdx.x] += partial[threadIdx.x + k];
    __syncthreads();
  }
  const float sum = partial[0];
  for (int i = threadIdx.x; i < len; i += 256) {
    const int64_t o = base + (int64_t)i * inner;
    float v         = alpha * ((float)dy[o] - __expf((float)y[o]) * sum);
    if (beta != 0.0f) v += beta * (float)dx[o];
    dx[o] = (T)v;
  }
}

ConvDims MakeConvDims(const char* what, int format, float alpha, float beta, int in, int ic, int ih, int iw, int fn, int fc,
                      int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, int groups, int on, int oc, int oh,
                      int ow) {
  CINN_RT_CHECK(format == 0 || format == 1, "%s: unknown tensor format %d", what, format);
  CINN_RT_CHECK(groups >= 1 && ic % groups == 0 && fn % groups == 0, "%s: bad group count %d", what, groups);
  CINN_RT_CHECK(fc == ic / groups, "%s: filter has %d input channels, expected %d", what, fc, ic / groups);
  CINN_RT_CHECK(on == in && oc == fn, "%s: output gradient is [%d,%d,..], expected [%d,%d,..]", what, on, oc, in, fn);
  CINN_RT_CHECK(sh > 0 && sw > 0 && dh > 0 && dw > 0, "%s: strides and dilations must be positive", what);
  const int want_oh = (ih - ((fh - 1) * dh + 1) + 2 * ph) / sh + 1;
  const int want_ow = (iw - ((fw - 1) * dw + 1) + 2 * pw) / sw + 1;
  CINN_RT_CHECK(oh == want_oh && ow == want_ow, "%s: output is %dx%d, the shapes give %dx%d", what, oh, ow, want_oh, want_ow);
  CINN_RT_CHECK((int64_t)in * ic * ih * iw < INT_MAX && (int64_t)on * oc * oh * ow < INT_MAX, "%s: tensor too large", what);
  ConvDims p;
  p.n = in, p.c = ic, p.ih = ih, p.iw = iw;
  p.f = fn, p.fc = fc, p.kh = fh, p.kw = fw;
  p.oh = oh, p.ow = ow;
  p.ph = ph, p.pw = pw, p.sh = sh, p.sw = sw, p.dh = dh, p.dw = dw, p.groups = groups;
  p.nhwc  = format == 1;
  p.alpha = alpha, p.beta = beta;
  return p;
}

}  // namespace

extern "C" {

void cinn_call_cudnn_conv2d_backward_data(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                          int input_c, int input_h, int input_w, int filter_n, int filter_c,
                                          int filter_h, int filter_w, int pad_h, int pad_w, int stride_h, int stride_w,
                                          int dilation_h, int dilation_w, int groups, int output_n, int output_c,
                                          int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 3, "cinn_call_cudnn_conv2d_backward_data takes w, dy and dx, got %d arguments", num_args);
  const ConvDims p = MakeConvDims("conv2d_backward_data", format, alpha, beta, input_n, input_c, input_h, input_w, filter_n,
                                  filter_c, filter_h, filter_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w,
                                  groups, output_n, output_c, output_h, output_w);
  cinn_buffer_t* w  = Arg(v_args, 0);
  cinn_buffer_t* dy = Arg(v_args, 1);
  cinn_buffer_t* dx = Arg(v_args, 2);
  const int64_t total = (int64_t)p.n * p.c * p.ih * p.iw;
  dim3 grid((unsigned)((total + 255) / 256));
  auto s = static_cast<hipStream_t>(stream);
  switch (ElemOf(dx)) {
    case Elem::kF64:
      hipLaunchKernelGGL(conv_backward_data_kernel<double>, grid, dim3(256), 0, s, reinterpret_cast<const double*>(w->memory), reinterpret_cast<const double*>(dy->memory), reinterpret_cast<double*>(dx->memory), p);
      break;
    case Elem::kF32:
      hipLaunchKernelGGL(conv_backward_data_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(w->memory),
                         reinterpret_cast<const float*>(dy->memory), reinterpret_cast<float*>(dx->memory), p);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(conv_backward_data_kernel<_Float16>, grid, dim3(256), 0, s,
                         reinterpret_cast<const _Float16*>(w->memory), reinterpret_cast<const _Float16*>(dy->memory),
                         reinterpret_cast<_Float16*>(dx->memory), p);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(conv_backward_data_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(w->memory),
                         reinterpret_cast<const __bf16*>(dy->memory), reinterpret_cast<__bf16*>(dx->memory), p);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

void cinn_call_cudnn_conv2d_backward_filter(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                            int input_c, int input_h, int input_w, int filter_n, int filter_c,
                                            int filter_h, int filter_w, int pad_h, int pad_w, int stride_h,
                                            int stride_w, int dilation_h, int dilation_w, int groups, int output_n,
                                            int output_c, int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 3, "cinn_call_cudnn_conv2d_backward_filter takes x, dy and dw, got %d arguments", num_args);
  const ConvDims p = MakeConvDims("conv2d_backward_filter", format, alpha, beta, input_n, input_c, input_h, input_w,
                                  filter_n, filter_c, filter_h, filter_w, pad_h, pad_w, stride_h, stride_w, dilation_h,
                                  dilation_w, groups, output_n, output_c, output_h, output_w);
  cinn_buffer_t* x  = Arg(v_args, 0);
  cinn_buffer_t* dy = Arg(v_args, 1);
  cinn_buffer_t* dw = Arg(v_args, 2);
  const int64_t total = (int64_t)p.f * p.fc * p.kh * p.kw;
  CINN_RT_CHECK(total < INT_MAX, "conv2d_backward_filter: filter too large");
  dim3 grid((unsigned)total);
  auto s = static_cast<hipStream_t>(stream);
  switch (ElemOf(dw)) {
    case Elem::kF64:
      hipLaunchKernelGGL(conv_backward_filter_kernel<double>, grid, dim3(256), 0, s, reinterpret_cast<const double*>(x->memory), reinterpret_cast<const double*>(dy->memory), reinterpret_cast<double*>(dw->memory), p);
      break;
    case Elem::kF32:
      hipLaunchKernelGGL(conv_backward_filter_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(x->memory),
                         reinterpret_cast<const float*>(dy->memory), reinterpret_cast<float*>(dw->memory), p);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(conv_backward_filter_kernel<_Float16>, grid, dim3(256), 0, s,
                         reinterpret_cast<const _Float16*>(x->memory), reinterpret_cast<const _Float16*>(dy->memory),
                         reinterpret_cast<_Float16*>(dw->memory), p);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(conv_backward_filter_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(x->memory),
                         reinterpret_cast<const __bf16*>(dy->memory), reinterpret_cast<__bf16*>(dw->memory), p);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

void cinn_call_cudnn_pool2d_backward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                     int input_n, int input_c, int input_h, int input_w, int kernel_h, int kernel_w,
                                     int pad_h, int pad_w, int stride_h, int stride_w, int output_n, int output_c,
                                     int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 4, "cinn_call_cudnn_pool2d_backward takes x, y, dy and dx, got %d arguments", num_args);
  CINN_RT_CHECK(format == 0 || format == 1, "pool2d_backward: unknown tensor format %d", format);
  CINN_RT_CHECK(mode >= 0 && mode <= 3, "pool2d_backward: unknown pooling mode %d", mode);
  CINN_RT_CHECK(output_n == input_n && output_c == input_c, "pool2d_backward: batch / channel mismatch");
  CINN_RT_CHECK(kernel_h > 0 && kernel_w > 0 && stride_h > 0 && stride_w > 0 && output_h > 0 && output_w > 0,
                "pool2d_backward: bad window");
  CINN_RT_CHECK((int64_t)input_n * input_c * input_h * input_w < INT_MAX, "pool2d_backward: tensor too large");
  PoolDims p;
  p.n = input_n, p.c = input_c, p.ih = input_h, p.iw = input_w, p.oh = output_h, p.ow = output_w;
  p.kh = kernel_h, p.kw = kernel_w, p.ph = pad_h, p.pw = pad_w, p.sh = stride_h, p.sw = stride_w;
  p.mode = mode, p.nhwc = format == 1;
  p.alpha = alpha, p.beta = beta;
  cinn_buffer_t* x  = Arg(v_args, 0);
  cinn_buffer_t* y  = Arg(v_args, 1);
  cinn_buffer_t* dy = Arg(v_args, 2);
  cinn_buffer_t* dx = Arg(v_args, 3);
  const int64_t total = (int64_t)p.n * p.c * p.ih * p.iw;
  dim3 grid((unsigned)((total + 255) / 256));
  auto s = static_cast<hipStream_t>(stream);
  switch (ElemOf(dx)) {
    case Elem::kF64:
      hipLaunchKernelGGL(pool_backward_kernel<double>, grid, dim3(256), 0, s, reinterpret_cast<const double*>(x->memory), reinterpret_cast<const double*>(y->memory), reinterpret_cast<const double*>(dy->memory),
                         reinterpret_cast<double*>(dx->memory), p);
      break;
    case Elem::kF32:
      hipLaunchKernelGGL(pool_backward_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(x->memory),
                         reinterpret_cast<const float*>(y->memory), reinterpret_cast<const float*>(dy->memory),
                         reinterpret_cast<float*>(dx->memory), p);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(pool_backward_kernel<_Float16>, grid, dim3(256), 0, s, reinterpret_cast<const _Float16*>(x->memory),
                         reinterpret_cast<const _Float16*>(y->memory), reinterpret_cast<const _Float16*>(dy->memory),
                         reinterpret_cast<_Float16*>(dx->memory), p);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(pool_backward_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(x->memory),
                         reinterpret_cast<const __bf16*>(y->memory), reinterpret_cast<const __bf16*>(dy->memory),
                         reinterpret_cast<__bf16*>(dx->memory), p);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

void cinn_call_cudnn_softmax_backward(void* v_args, int num_args, int mode, int format, float alpha, float beta,
                                      int input_n, int input_c, int input_h, int input_w, int output_n, int output_c,
                                      int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 3, "cinn_call_cudnn_softmax_backward takes y, dy and dx, got %d arguments", num_args);
  CINN_RT_CHECK(format == 0, "softmax_backward: only NCHW (format 0) is implemented, got format %d", format);
  CINN_RT_CHECK(mode == 0 || mode == 1, "softmax_backward: unknown mode %d", mode);
  CINN_RT_CHECK(input_n == output_n && input_c == output_c && input_h == output_h && input_w == output_w,
                "softmax_backward: input and output shapes differ");
  cinn_buffer_t* y  = Arg(v_args, 0);
  cinn_buffer_t* dy = Arg(v_args, 1);
  cinn_buffer_t* dx = Arg(v_args, 2);
  const int len   = mode == 1 ? input_c : input_c * input_h * input_w;
  const int inner = mode == 1 ? input_h * input_w : 1;
  const int64_t groups = (int64_t)input_n * inner;
  CINN_RT_CHECK(groups > 0 && groups < INT_MAX && len > 0, "softmax_backward: bad extents");
  dim3 grid((unsigned)groups);
  auto s = static_cast<hipStream_t>(stream);
  switch (ElemOf(dx)) {
    case Elem::kF64: CINN_RT_CHECK(false, "softmax_backward: fp64 tensors are not implemented"); break;
    case Elem::kF32:
      hipLaunchKernelGGL(log_softmax_backward_kernel<float>, grid, dim3(256), 0, s, reinterpret_cast<const float*>(y->memory),
                         reinterpret_cast<const float*>(dy->memory), reinterpret_cast<float*>(dx->memory), len, inner, alpha, beta);
      break;
    case Elem::kF16:
      hipLaunchKernelGGL(log_softmax_backward_kernel<_Float16>, grid, dim3(256), 0, s,
                         reinterpret_cast<const _Float16*>(y->memory), reinterpret_cast<const _Float16*>(dy->memory),
                         reinterpret_cast<_Float16*>(dx->memory), len, inner, alpha, beta);
      break;
    case Elem::kBF16:
      hipLaunchKernelGGL(log_softmax_backward_kernel<__bf16>, grid, dim3(256), 0, s, reinterpret_cast<const __bf16*>(y->memory),
                         reinterpret_cast<const __bf16*>(dy->memory), reinterpret_cast<__bf16*>(dx->memory), len, inner, alpha, beta);
      break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

}  // extern "C"
