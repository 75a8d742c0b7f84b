// Depthwise convolution on channels-last tensors (groups == input channels == output channels): one filter per channel,
// so there is no matrix product - every output is kh * kw multiply-adds and the kernel is bound by HBM.
// Reference semantics: conv2d with groups (cinn/hlir/pe/nn.cc:220-313 for the dense loop nest, cuda_util.cc:603-720
// for the cuDNN call with a group count); accumulation in fp32 in tap order (dy, dx), zero padding.
//
// One thread per output pixel and 16 bytes of channels: consecutive lanes take consecutive channel vectors of a pixel,
// then the next pixel, so every access is a contiguous vector.  The filter arrives as [C][KH][KW] (the channels-last
// filter form [OC][KH][KW][IC / groups] with one input channel per group) and is staged in LDS transposed to
// [tap][C], so that a lane's weights of a tap are one 16-byte LDS read.  A block stages the filter once and then
// walks through kItemsPerThread pixel-vectors per thread.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

#include "conv_nhwc.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

constexpr int kThreads        = 256;
constexpr int kItemsPerThread = 2;
constexpr int kMaxFilterBytes = 64 * 1024;

struct DwParams {
  int n, h, w, c;
  int kh, kw, oh, ow;
  int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
  float alpha, residual_scale;
  int relu;
};

// KS > 0: a KS x KS filter known at compile time - the vectors of all taps are requested before the first is used
// (taps outside the image read the pixel's own image origin and are skipped in the arithmetic), so a thread has KS * KS
// loads in flight instead of one behind each bounds check.  KS == 0: any filter, taps visited one by one.
template <typename T, int V, int KS>
__global__ void __launch_bounds__(kThreads)
depthwise_nhwc_kernel(const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, const float* __restrict__ scale,
                      const float* __restrict__ shift, const T* __restrict__ residual, const T* __restrict__ zeros,
                      DwParams p) {
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  T* wl          = reinterpret_cast<T*>(lds_raw);  // [tap][c]
  const int taps = p.kh * p.kw;
  // [c][tap] in memory: 16 bytes at a time, scattered to [tap][c]
  for (int v = threadIdx.x; v * V < p.c * taps; v += kThreads) {
    T wv[V];
    __builtin_memcpy(wv, w + v * V, V * sizeof(T));
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const int i = v * V + e;
      const int c = i / taps, t = i - c * taps;
      wl[t * p.c + c] = wv[e];
    }
  }
  __syncthreads();
  // the tensors have fewer than 2^31 elements (checked by the caller): 32-bit index arithmetic
  const unsigned groups = p.c / V;
  const unsigned total  = (unsigned)p.n * p.oh * p.ow * groups;
#pragma unroll 1
  for (int it = 0; it < kItemsPerThread; ++it) {
    const unsigned idx = (blockIdx.x * kItemsPerThread + it) * kThreads + threadIdx.x;
    if (idx >= total) break;
    const unsigned pixel = idx / groups;
    const int g          = (int)(idx - pixel * groups);
    const unsigned row   = pixel / p.ow;  // n * oh + oy
    const int ox         = (int)(pixel - row * p.ow);
    const unsigned n     = row / p.oh;
    const int oy         = (int)(row - n * p.oh);
    const T* src         = x + (size_t)n * p.h * p.w * p.c + g * V;
    const int iy0 = oy * p.stride_h - p.pad_h, ix0 = ox * p.stride_w - p.pad_w;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.0f;
    if (KS > 0) {
      constexpr int TAPS = KS * KS > 0 ? KS * KS : 1;
      constexpr int KSD  = KS > 0 ? KS : 1;
      T xv[TAPS][V];
      // a tap outside the image reads zeros (as the padded input would hold); the tap's offset from the window's
      // corner is the same for every lane
      const T* corner = src + (iy0 * p.w + ix0) * p.c;
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const int dy = (t / KSD) * p.dil_h, dx = (t % KSD) * p.dil_w;
        const bool ok = (unsigned)(iy0 + dy) < (unsigned)p.h && (unsigned)(ix0 + dx) < (unsigned)p.w;
        __builtin_memcpy(xv[t], ok ? corner + (dy * p.w + dx) * p.c : zeros, V * sizeof(T));
      }
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        T wv[V];
        __builtin_memcpy(wv, wl + t * p.c + g * V, V * sizeof(T));
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = __builtin_fmaf((float)xv[t][e], (float)wv[e], acc[e]);
      }
    } else {
      for (int dy = 0; dy < p.kh; ++dy) {
        const int iy = iy0 + dy * p.dil_h;
        if (iy < 0 || iy >= p.h) continue;
        for (int dx = 0; dx < p.kw; ++dx) {
          const int ix = ix0 + dx * p.dil_w;
          if (ix < 0 || ix >= p.w) continue;
          T xv[V], wv[V];
          __builtin_memcpy(xv, src + (iy * p.w + ix) * p.c, V * sizeof(T));
          __builtin_memcpy(wv, wl + (dy * p.kw + dx) * p.c + g * V, V * sizeof(T));
#pragma unroll
          for (int e = 0; e < V; ++e) acc[e] = __builtin_fmaf((float)xv[e], (float)wv[e], acc[e]);
        }
      }
    }
    const size_t off = (size_t)pixel * p.c + g * V;
    T out[V], rv[V];
    if (residual) __builtin_memcpy(rv, residual + off, V * sizeof(T));
    float sc[V], sh[V];
#pragma unroll
    for (int e = 0; e < V; ++e) sc[e] = p.alpha, sh[e] = 0.0f;
    if (scale) __builtin_memcpy(sc, scale + g * V, V * sizeof(float));
    if (shift) __builtin_memcpy(sh, shift + g * V, V * sizeof(float));
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float v = __builtin_fmaf(acc[e], sc[e], sh[e]);
      if (residual) v = __builtin_fmaf(p.residual_scale, (float)rv[e], v);
      if (p.relu) v = v > 0.0f ? v : 0.0f;
      out[e] = (T)v;
    }
    __builtin_memcpy(y + off, out, V * sizeof(T));
  }
}

template <typename T>
void Launch(const ConvNhwcArgs& a, hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  DwParams p;
  p.n = a.n, p.h = a.h, p.w = a.w_in, p.c = a.c;
  p.kh = a.kh, p.kw = a.kw, p.oh = a.oh, p.ow = a.ow;
  p.pad_h = a.pad_h, p.pad_w = a.pad_w, p.stride_h = a.stride_h, p.stride_w = a.stride_w;
  p.dil_h = a.dil_h, p.dil_w = a.dil_w;
  p.alpha = a.alpha, p.residual_scale = a.residual_scale, p.relu = a.relu ? 1 : 0;
  const int64_t total  = (int64_t)a.n * a.oh * a.ow * (a.c / V);
  const int64_t blocks = (total + kThreads * kItemsPerThread - 1) / (kThreads * kItemsPerThread);
  const size_t lds     = (size_t)a.kh * a.kw * a.c * sizeof(T);
  auto kernel = depthwise_nhwc_kernel<T, V, 0>;
  if (a.kh == 3 && a.kw == 3) kernel = depthwise_nhwc_kernel<T, V, 3>;
  if (a.kh == 5 && a.kw == 5) kernel = depthwise_nhwc_kernel<T, V, 5>;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), lds, stream, static_cast<const T*>(a.x),
                     static_cast<const T*>(a.w), static_cast<T*>(a.y), a.scale, a.shift,
                     static_cast<const T*>(a.residual), static_cast<const T*>(ConvZeroPage()), p);
  CINN_HIP_CALL(hipGetLastError());
}

}  // namespace

bool DepthwiseNhwcSupported(const ConvNhwcArgs& a, int groups) {
  if (a.nchw_input || groups != a.c || a.oc != a.c) return false;
  const int bytes = a.type.bits / CHAR_BIT;
  const bool fp   = (a.type.code == cinn_type_float && (bytes == 4 || bytes == 2)) || (a.type.code == cinn_type_bfloat && bytes == 2);
  if (!fp) return false;
  const int v = 16 / bytes;
  if (a.c % v != 0) return false;
  if ((int64_t)a.kh * a.kw * a.c * bytes > kMaxFilterBytes) return false;
  if ((int64_t)a.n * a.oh * a.ow * (a.c / v) / (kThreads * kItemsPerThread) >= INT_MAX) return false;
  return reinterpret_cast<uintptr_t>(a.x) % 16 == 0 && reinterpret_cast<uintptr_t>(a.y) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.residual) % 16 == 0;
}

void RunDepthwiseNhwc(const ConvNhwcArgs& a, hipStream_t stream) {
  const int bytes = a.type.bits / CHAR_BIT;
  if (bytes == 4) {
    Launch<float>(a, stream);
  } else if (a.type.code == cinn_type_bfloat) {
    Launch<__bf16>(a, stream);
  } else {
    Launch<_Float16>(a, stream);
  }
}

}  // namespace cinn_hip_kernels
