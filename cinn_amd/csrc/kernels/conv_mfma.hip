// Hand-written CDNA4 (gfx950) convolution behind cinn_call_cudnn_conv2d_forward and its fused
// batch_norm / relu variant: NCHW cross-correlation with zero padding as an implicit GEMM on MFMA,
//
//   out[n, f, y, x] = sum_{c, ry, rx} in[n, c, y*s + ry*d - p, x*s + rx*d - p] * w[f, c, ry, rx]
//
// GEMM view per group: M = output channels, N = n * oh * ow output pixels (flattened over the batch so that
// small images still fill a tile), K = (c / groups) * kh * kw.  The weight matrix is [M][K] as stored.  The
// im2col matrix is never materialised: every thread owns one output pixel of the tile and decodes k into
// (c, ry, rx) with two multiply-shift divisions by host-computed magic numbers, so a gathered element costs
// a few integer instructions, two range checks and one load - and the entry point touches no device memory
// beyond its operands (nothing to allocate or upload on the first call of a shape, safe under stream capture).
//
// Block tile 128 (channels) x 128 (pixels), 256 threads = 4 wavefronts in a 2x2 grid, each 64x64 = 2x2 MFMA
// tiles of 32x32.
//   fp32          : K step 16, v_mfma_f32_32x32x2f32; LDS tiles [k][row] read with conflict-free ds_read_b32.
//   fp16 / bf16   : K step 32, v_mfma_f32_32x32x16_{f16,bf16} (fp32 accumulation); LDS tiles [row][k] with
//                   64-byte rows whose 16-byte chunks are XOR-swizzled for conflict-free ds_read_b128.
// The epilogue applies alpha / beta, or the per-channel affine (+ relu) of an inference batch_norm.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

#include "cinn_hip_runtime.h"
#include "kernels/conv_nhwc.h"
#include "runtime/hip_check.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct ConvParams {
  int n, c, ih, iw;        // input
  int f, kh, kw;           // filter: f output channels, c / groups input channels each
  int oh, ow;              // output
  int ph, pw, sh, sw;      // padding, stride
  int dh, dw;              // dilation
  // exact division of 0 <= k < 2^31 by kh * kw and by kw: q = (k * magic) >> shift with a 64-bit product
  unsigned magic_taps, shift_taps, magic_kw, shift_kw;
  int groups;
  int k_total;             // (c / groups) * kh * kw
  int pixels;              // n * oh * ow
  float alpha, beta;
  int epilogue;            // 0: alpha / beta, 1: affine, 2: affine + relu
};

constexpr int kTileM   = 128;
constexpr int kTileN   = 128;
constexpr int kThreads = 256;

template <typename T>
struct ConvTraits;
template <>
struct ConvTraits<float> {
  static constexpr int kStep = 16;
  static constexpr bool kHalf = false;
};
template <>
struct ConvTraits<_Float16> {
  static constexpr int kStep = 32;
  static constexpr bool kHalf = true;
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct ConvTraits<__bf16> {
  static constexpr int kStep = 32;
  static constexpr bool kHalf = true;
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// 16-bit tiles: rows of 32 elements = 64 bytes = 4 chunks; chunk position = chunk ^ ((row >> 1) & 3)
__device__ __forceinline__ int HalfTileOffset(int row, int chunk) { return row * 64 + ((chunk ^ ((row >> 1) & 3)) << 4); }

template <typename T>
__global__ void __launch_bounds__(kThreads)
conv2d_igemm_kernel(const T* __restrict__ in, const T* __restrict__ w, T* __restrict__ out,
                    const float* __restrict__ scale, const float* __restrict__ shift, ConvParams p) {
  constexpr int BK = ConvTraits<T>::kStep;
  // fp32: A[BK][128 + 4] and B[BK][128 + 4] floats; 16-bit: A[128][32] and B[128][32] halves (8 KiB each)
  __shared__ __attribute__((aligned(16))) char lds_a[ConvTraits<T>::kHalf ? kTileM * 64 : BK * (kTileM + 4) * 4];
  __shared__ __attribute__((aligned(16))) char lds_b[ConvTraits<T>::kHalf ? kTileN * 64 : BK * (kTileN + 4) * 4];

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int group = blockIdx.z;
  const int fg    = p.f / p.groups;  // output channels per group
  const int cg    = p.c / p.groups;  // input channels per group
  const int f0    = blockIdx.y * kTileM;  // within the group
  const int p0    = blockIdx.x * kTileN;
  const int ohw   = p.oh * p.ow;
  const int K     = p.k_total;

  // the output pixel this thread gathers for
  const int my_pix   = p0 + (tid & 127);
  const bool pix_ok  = my_pix < p.pixels;
  int pn = 0, py = 0, px = 0;
  if (pix_ok) {
    pn      = my_pix / ohw;
    int rem = my_pix - pn * ohw;
    py      = rem / p.ow;
    px      = rem - py * p.ow;
  }
  const int iy0 = py * p.sh - p.ph;
  const int ix0 = px * p.sw - p.pw;
  const T* in_pix = in + ((int64_t)pn * p.c + (int64_t)group * cg) * p.ih * p.iw + (int64_t)iy0 * p.iw + ix0;
  const T* w_grp  = w + (int64_t)group * fg * K;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto gather = [&](int k) -> T {
    if (!pix_ok || k >= K) return (T)0.0f;
    const int c   = (int)(((unsigned long long)(unsigned)k * p.magic_taps) >> p.shift_taps);
    const int tap = k - c * (p.kh * p.kw);
    const int ry  = (int)(((unsigned long long)(unsigned)tap * p.magic_kw) >> p.shift_kw);
    const int dy = ry * p.dh, dx = (tap - ry * p.kw) * p.dw;
    int iy = iy0 + dy, ix = ix0 + dx;
    if (iy < 0 || iy >= p.ih || ix < 0 || ix >= p.iw) return (T)0.0f;
    return in_pix[(c * p.ih + dy) * p.iw + dx];
  };

  for (int k0 = 0; k0 < K; k0 += BK) {
    if constexpr (!ConvTraits<T>::kHalf) {
      float(*As)[kTileM + 4] = reinterpret_cast<float(*)[kTileM + 4]>(lds_a);
      float(*Bs)[kTileN + 4] = reinterpret_cast<float(*)[kTileN + 4]>(lds_b);
      float ra[8], rb[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int e = tid + 256 * i;
        int k = e & 15, f = e >> 4;
        ra[i] = (f0 + f < fg && k0 + k < K) ? (float)w_grp[(int64_t)(f0 + f) * K + k0 + k] : 0.0f;
        rb[i] = (float)gather(k0 + (tid >> 7) + 2 * i);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int e = tid + 256 * i;
        As[e & 15][e >> 4]               = ra[i];
        Bs[(tid >> 7) + 2 * i][tid & 127] = rb[i];
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        const int k = kk + (lane >> 5);
        float af[2], bf[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          af[t] = As[k][wm * 64 + t * 32 + (lane & 31)];
          bf[t] = Bs[k][wn * 64 + t * 32 + (lane & 31)];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
      __syncthreads();
    } else {
      typedef typename ConvTraits<T>::vec8 vec8;
      const bool vec_ok = (K & 7) == 0;  // rows of w start 16-byte aligned
      vec8 ra[2], rb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        int q = tid + 256 * i;  // weight chunk: row q / 4, chunk q % 4
        int f = q >> 2, c = q & 3;
        int k = k0 + c * 8;
        if (f0 + f < fg && vec_ok && k + 8 <= K) {
          ra[i] = *reinterpret_cast<const vec8*>(w_grp + (int64_t)(f0 + f) * K + k);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) ra[i][e] = (f0 + f < fg && k + e < K) ? w_grp[(int64_t)(f0 + f) * K + k + e] : (T)0.0f;
        }
        int kg = (tid >> 7) + 2 * i;  // gathered chunk: pixel tid % 128, k group kg
#pragma unroll
        for (int e = 0; e < 8; ++e) rb[i][e] = gather(k0 + kg * 8 + e);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        int q = tid + 256 * i;
        *reinterpret_cast<vec8*>(lds_a + HalfTileOffset(q >> 2, q & 3))               = ra[i];
        *reinterpret_cast<vec8*>(lds_b + HalfTileOffset(tid & 127, (tid >> 7) + 2 * i)) = rb[i];
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        vec8 af[2], bf[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          af[t] = *reinterpret_cast<const vec8*>(lds_a + HalfTileOffset(wm * 64 + t * 32 + (lane & 31), kk * 2 + (lane >> 5)));
          bf[t] = *reinterpret_cast<const vec8*>(lds_b + HalfTileOffset(wn * 64 + t * 32 + (lane & 31), kk * 2 + (lane >> 5)));
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = ConvTraits<T>::mfma(af[i], bf[j], acc[i][j]);
      }
      __syncthreads();
    }
  }

  // epilogue: element r of lane l is channel 8*(r/4) + 4*(l/32) + r%4, pixel l%32 of its 32x32 tile
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int pix = p0 + wn * 64 + j * 32 + (lane & 31);
    if (pix >= p.pixels) continue;
    const int n   = pix / ohw;
    const int rem = pix - n * ohw;
    T* out_pix    = out + ((int64_t)n * p.f + (int64_t)group * fg) * ohw + rem;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int f = f0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (f >= fg) continue;
        T* dst  = out_pix + (int64_t)f * ohw;
        float v = acc[i][j][r];
        if (p.epilogue == 0) {
          v *= p.alpha;
          if (p.beta != 0.0f) v += p.beta * (float)*dst;
        } else {
          v = v * scale[group * fg + f] + shift[group * fg + f];
          if (p.epilogue == 2) v = v > 0.0f ? v : 0.0f;
        }
        *dst = (T)v;
      }
    }
  }
}

// q = (n * magic) >> shift == n / d for 0 <= n < 2^31 (Granlund-Montgomery with a 64-bit product)
void MagicFor(int d, unsigned* magic, unsigned* shift) {
  int l = 0;
  while ((1ll << l) < d) ++l;
  *shift = 31 + l;
  *magic = (unsigned)(((1ull << *shift) / (unsigned)d) + 1);
  if (d == 1) {  // 2^31 + 1 would round n = 2^31 - 1 up; d == 1 needs no rounding at all
    *shift = 0;
    *magic = 1;
  }
}

// fp64 tensors (no matrix-core path is wired for them): one thread per output element, products added in
// (channel, filter row, filter column) order.  nhwc: x [N][H][W][C], w [F][KH][KW][C/groups], y [N][OH][OW][F].
struct DirectConvDims {
  int n, c, ih, iw, f, fc, kh, kw, oh, ow, ph, pw, sh, sw, dh, dw, groups, nhwc;
  double alpha, beta;
};
__global__ void __launch_bounds__(256)
conv2d_f64_kernel(const double* __restrict__ x, const double* __restrict__ w, double* __restrict__ y, DirectConvDims p) {
  const int64_t total = (int64_t)p.n * p.f * p.oh * p.ow;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int n, f, oy, ox;
  if (p.nhwc) {
    f  = (int)(idx % p.f);
    ox = (int)((idx / p.f) % p.ow);
    oy = (int)((idx / ((int64_t)p.f * p.ow)) % p.oh);
    n  = (int)(idx / ((int64_t)p.f * p.ow * p.oh));
  } else {
    ox = (int)(idx % p.ow);
    oy = (int)((idx / p.ow) % p.oh);
    f  = (int)((idx / ((int64_t)p.ow * p.oh)) % p.f);
    n  = (int)(idx / ((int64_t)p.ow * p.oh * p.f));
  }
  const int c0 = (f / (p.f / p.groups)) * p.fc;
  double acc   = 0.0;
  for (int cl = 0; cl < p.fc; ++cl) {
    const int c = c0 + cl;
    for (int ky = 0; ky < p.kh; ++ky) {
      const int iy = oy * p.sh - p.ph + ky * p.dh;
      if (iy < 0 || iy >= p.ih) continue;
      for (int kx = 0; kx < p.kw; ++kx) {
        const int ix = ox * p.sw - p.pw + kx * p.dw;
        if (ix < 0 || ix >= p.iw) continue;
        const int64_t xi = p.nhwc ? (((int64_t)n * p.ih + iy) * p.iw + ix) * p.c + c
                                  : (((int64_t)n * p.c + c) * p.ih + iy) * p.iw + ix;
        const int64_t wi = p.nhwc ? (((int64_t)f * p.kh + ky) * p.kw + kx) * p.fc + cl
                                  : (((int64_t)f * p.fc + cl) * p.kh + ky) * p.kw + kx;
        acc = __builtin_fma(x[xi], w[wi], acc);
      }
    }
  }
  double v = p.alpha * acc;
  if (p.beta != 0.0) v += p.beta * y[idx];
  y[idx] = v;
}

cinn_buffer_t* BufferArg(void* v_args, int index) {
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  CINN_RT_CHECK(args[index].type_code_ == CINN_POD_BUFFER_P, "conv2d: argument %d is not a buffer", index);
  return static_cast<cinn_buffer_t*>(args[index].value_.v_handle);
}

void RunConv(cinn_buffer_t* x, cinn_buffer_t* w, cinn_buffer_t* y, const float* scale, const float* shift,
             cinn_buffer_t* residual, int epilogue, int format, float alpha, float beta, int in, int ic, int ih, int iw, int fn, int fc, int fh, int fw, int ph,
             int pw, int sh, int sw, int dh, int dw, int groups, int on, int oc, int oh, int ow, hipStream_t stream) {
  CINN_RT_CHECK(format >= 0 && format <= 2, "conv2d: unknown tensor format %d", format);
  CINN_RT_CHECK(groups >= 1 && ic % groups == 0 && fn % groups == 0, "conv2d: bad group count %d", groups);
  CINN_RT_CHECK(fc == ic / groups, "conv2d: filter has %d input channels, expected %d", fc, ic / groups);
  CINN_RT_CHECK(on == in && oc == fn, "conv2d: output is [%d,%d,..], expected [%d,%d,..]", on, oc, in, fn);
  CINN_RT_CHECK(sh > 0 && sw > 0 && dh > 0 && dw > 0, "conv2d: strides and dilations must be positive");
  const int want_oh = (ih - ((fh - 1) * dh + 1) + 2 * ph) / sh + 1;
  const int want_ow = (iw - ((fw - 1) * dw + 1) + 2 * pw) / sw + 1;
  CINN_RT_CHECK(oh == want_oh && ow == want_ow, "conv2d: output is %dx%d, the shapes give %dx%d", oh, ow, want_oh, want_ow);
  CINN_RT_CHECK((int64_t)in * ic * ih * iw < INT_MAX && (int64_t)on * oc * oh * ow < INT_MAX, "conv2d: tensor too large");
  CINN_RT_CHECK(fh * dh < 32768 && fw * dw < 32768, "conv2d: filter extent too large");
  if (x->type.code == cinn_type_float && x->type.bits == 64) {
    CINN_RT_CHECK(format != 2 && epilogue == 0, "conv2d: fp64 tensors take the plain convolution in NCHW or NHWC only");
    DirectConvDims d{in, ic, ih, iw, fn, fc, fh, fw, oh, ow, ph, pw, sh, sw, dh, dw, groups, format == 1, alpha, beta};
    const int64_t total = (int64_t)on * oc * oh * ow;
    hipLaunchKernelGGL(conv2d_f64_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const double*>(x->memory), reinterpret_cast<const double*>(w->memory),
                       reinterpret_cast<double*>(y->memory), d);
    CINN_HIP_CALL(hipGetLastError());
    return;
  }
  if (format != 0) {
    // channels-last output; format 2 reads an NCHW input and [OC][IC][KH][KW] weights
    cinn_hip_kernels::ConvNhwcArgs a;
    a.x = x->memory, a.w = w->memory, a.y = y->memory;
    a.scale = scale, a.shift = shift;
    a.residual       = residual ? residual->memory : (epilogue == 0 && beta != 0.0f ? y->memory : nullptr);
    a.alpha          = epilogue == 0 ? alpha : 1.0f;
    a.residual_scale = residual ? 1.0f : beta;
    a.relu           = epilogue >= 2;
    a.pool_after     = epilogue == 3;
    a.nchw_input     = format == 2;
    a.n = in, a.h = ih, a.w_in = iw, a.c = ic;
    a.oc = fn, a.kh = fh, a.kw = fw, a.oh = oh, a.ow = ow;
    a.pad_h = ph, a.pad_w = pw, a.stride_h = sh, a.stride_w = sw, a.dil_h = dh, a.dil_w = dw;
    a.type = x->type;
    if (groups != 1) {
      CINN_RT_CHECK(cinn_hip_kernels::DepthwiseNhwcSupported(a, groups),
                    "conv2d: of grouped convolutions the channels-last kernels take depthwise ones only (groups %d, channels %d -> %d)",
                    groups, ic, fn);
      cinn_hip_kernels::RunDepthwiseNhwc(a, stream);
      return;
    }
    CINN_RT_CHECK(cinn_hip_kernels::ConvNhwcSupported(a), "conv2d: channels-last needs the channel count (%d) to be a multiple of 16 bytes", ic);
    cinn_hip_kernels::RunConvNhwc(a, stream);
    return;
  }
  CINN_RT_CHECK(residual == nullptr, "conv2d: a residual input needs the channels-last format");
  CINN_RT_CHECK(epilogue != 3, "conv2d: a fused max pooling needs the channels-last format");

  ConvParams p;
  p.n = in, p.c = ic, p.ih = ih, p.iw = iw;
  p.f = fn, p.kh = fh, p.kw = fw;
  p.oh = oh, p.ow = ow;
  p.ph = ph, p.pw = pw, p.sh = sh, p.sw = sw;
  p.groups   = groups;
  p.k_total  = fc * fh * fw;
  p.pixels   = in * oh * ow;
  p.alpha    = alpha;
  p.beta     = beta;
  p.epilogue = epilogue;
  p.dh = dh, p.dw = dw;
  MagicFor(fh * fw, &p.magic_taps, &p.shift_taps);
  MagicFor(fw, &p.magic_kw, &p.shift_kw);

  dim3 grid((p.pixels + kTileN - 1) / kTileN, (fn / groups + kTileM - 1) / kTileM, groups);
  CINN_RT_CHECK(grid.y <= 65535 && grid.z <= 65535, "conv2d: grid too large");
  const int bytes = x->type.bits / CHAR_BIT;
  if (x->type.code == cinn_type_float && bytes == 4) {
    hipLaunchKernelGGL(conv2d_igemm_kernel<float>, grid, dim3(kThreads), 0, stream, reinterpret_cast<const float*>(x->memory),
                       reinterpret_cast<const float*>(w->memory), reinterpret_cast<float*>(y->memory), scale, shift, p);
  } else if (x->type.code == cinn_type_float && bytes == 2) {
    hipLaunchKernelGGL(conv2d_igemm_kernel<_Float16>, grid, dim3(kThreads), 0, stream,
                       reinterpret_cast<const _Float16*>(x->memory), reinterpret_cast<const _Float16*>(w->memory),
                       reinterpret_cast<_Float16*>(y->memory), scale, shift, p);
  } else if (x->type.code == cinn_type_bfloat) {
    hipLaunchKernelGGL(conv2d_igemm_kernel<__bf16>, grid, dim3(kThreads), 0, stream,
                       reinterpret_cast<const __bf16*>(x->memory), reinterpret_cast<const __bf16*>(w->memory),
                       reinterpret_cast<__bf16*>(y->memory), scale, shift, p);
  } else {
    fprintf(stderr, "conv2d: unsupported data type code %d bits %d\n", x->type.code, x->type.bits);
    abort();
  }
  CINN_HIP_CALL(hipGetLastError());
}

}  // namespace

extern "C" {

void cinn_call_cudnn_conv2d_forward(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                    int input_c, int input_h, int input_w, int filter_n, int filter_c, int filter_h,
                                    int filter_w, int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h,
                                    int dilation_w, int groups, int output_n, int output_c, int output_h,
                                    int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 3, "cinn_call_cudnn_conv2d_forward takes x, w and y, got %d arguments", num_args);
  RunConv(BufferArg(v_args, 0), BufferArg(v_args, 1), BufferArg(v_args, 2), nullptr, nullptr, nullptr, 0, format, alpha, beta,
          input_n, input_c, input_h, input_w, filter_n, filter_c, filter_h, filter_w, pad_h, pad_w, stride_h, stride_w,
          dilation_h, dilation_w, groups, output_n, output_c, output_h, output_w, static_cast<hipStream_t>(stream));
}

void cinn_call_hip_conv2d_bn_relu(void* v_args, int num_args, int format, int relu, int input_n, int input_c,
                                  int input_h, int input_w, int filter_n, int filter_c, int filter_h, int filter_w,
                                  int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                                  int groups, int output_n, int output_c, int output_h, int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 5 || num_args == 6,
                "cinn_call_hip_conv2d_bn_relu takes x, w, scale, shift, [residual] and y, got %d arguments", num_args);
  cinn_buffer_t* scale = BufferArg(v_args, 2);
  cinn_buffer_t* shift = BufferArg(v_args, 3);
  CINN_RT_CHECK(scale->type.code == cinn_type_float && scale->type.bits == 32 && shift->type.bits == 32,
                "cinn_call_hip_conv2d_bn_relu: scale / shift must be fp32");
  RunConv(BufferArg(v_args, 0), BufferArg(v_args, 1), BufferArg(v_args, num_args - 1),
          reinterpret_cast<const float*>(scale->memory), reinterpret_cast<const float*>(shift->memory),
          num_args == 6 ? BufferArg(v_args, 4) : nullptr, (relu & 2) ? 3 : ((relu & 1) ? 2 : 1), format, 1.0f, 0.0f, input_n, input_c, input_h,
          input_w, filter_n, filter_c, filter_h, filter_w, pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w,
          groups, output_n, output_c, output_h, output_w, static_cast<hipStream_t>(stream));
}

void cinn_call_hip_conv2d_bn_relu_chain(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w,
                                        int input_c, int middle_c, int output_c, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 9 || num_args == 10,
                "cinn_call_hip_conv2d_bn_relu_chain takes x, w1, scale1, shift1, [residual], w2, scale2, shift2, e and y, "
                "got %d arguments", num_args);
  const int r = num_args == 10 ? 1 : 0;  // a residual shifts what follows it
  cinn_buffer_t* x  = BufferArg(v_args, 0);
  cinn_buffer_t* w1 = BufferArg(v_args, 1);
  cinn_buffer_t* s1 = BufferArg(v_args, 2);
  cinn_buffer_t* t1 = BufferArg(v_args, 3);
  cinn_buffer_t* res = r ? BufferArg(v_args, 4) : nullptr;
  cinn_buffer_t* w2 = BufferArg(v_args, 4 + r);
  cinn_buffer_t* s2 = BufferArg(v_args, 5 + r);
  cinn_buffer_t* t2 = BufferArg(v_args, 6 + r);
  cinn_buffer_t* e  = BufferArg(v_args, 7 + r);
  cinn_buffer_t* y  = BufferArg(v_args, 8 + r);
  for (cinn_buffer_t* f : {s1, t1, s2, t2})
    CINN_RT_CHECK(f->type.code == cinn_type_float && f->type.bits == 32, "cinn_call_hip_conv2d_bn_relu_chain: scale / shift must be fp32");
  CINN_RT_CHECK(input_n > 0 && input_h > 0 && input_w > 0 && input_c > 0 && middle_c > 0 && output_c > 0,
                "cinn_call_hip_conv2d_bn_relu_chain: extents must be positive");
  hipStream_t st = static_cast<hipStream_t>(stream);
  cinn_hip_kernels::ConvChainArgs a;
  a.x = x->memory, a.w1 = w1->memory, a.scale1 = reinterpret_cast<const float*>(s1->memory);
  a.shift1 = reinterpret_cast<const float*>(t1->memory), a.residual = res ? res->memory : nullptr, a.relu1 = (relu & 1) != 0;
  a.e = e->memory, a.w2 = w2->memory, a.scale2 = reinterpret_cast<const float*>(s2->memory);
  a.shift2 = reinterpret_cast<const float*>(t2->memory), a.relu2 = (relu & 2) != 0, a.y = y->memory;
  a.m = (int64_t)input_n * input_h * input_w, a.k1 = input_c, a.n1 = middle_c, a.n2 = output_c, a.type = x->type;
  const bool same_type = w1->type.code == x->type.code && w1->type.bits == x->type.bits && w2->type.code == x->type.code &&
                         w2->type.bits == x->type.bits && e->type.bits == x->type.bits && y->type.bits == x->type.bits;
  if (same_type && cinn_hip_kernels::TryConvChain(a, st)) return;
  // any other shape or type: the two convolutions one after the other
  RunConv(x, w1, e, a.scale1, a.shift1, res, a.relu1 ? 2 : 1, 1, 1.0f, 0.0f, input_n, input_c, input_h, input_w, middle_c, input_c,
          1, 1, 0, 0, 1, 1, 1, 1, 1, input_n, middle_c, input_h, input_w, st);
  RunConv(e, w2, y, a.scale2, a.shift2, nullptr, a.relu2 ? 2 : 1, 1, 1.0f, 0.0f, input_n, middle_c, input_h, input_w, output_c,
          middle_c, 1, 1, 0, 0, 1, 1, 1, 1, 1, input_n, output_c, input_h, input_w, st);
}

void cinn_call_hip_conv2d_pair_chain(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w, int input_c,
                                     int second_c, int middle_c, int output_c, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 9, "cinn_call_hip_conv2d_pair_chain takes x, x2, w1, shift1, w2, scale2, shift2, e and y, got %d arguments",
                num_args);
  cinn_buffer_t* x  = BufferArg(v_args, 0);
  cinn_buffer_t* x2 = BufferArg(v_args, 1);
  cinn_buffer_t* w1 = BufferArg(v_args, 2);
  cinn_buffer_t* t1 = BufferArg(v_args, 3);
  cinn_buffer_t* w2 = BufferArg(v_args, 4);
  cinn_buffer_t* s2 = BufferArg(v_args, 5);
  cinn_buffer_t* t2 = BufferArg(v_args, 6);
  cinn_buffer_t* e  = BufferArg(v_args, 7);
  cinn_buffer_t* y  = BufferArg(v_args, 8);
  for (cinn_buffer_t* f : {t1, s2, t2})
    CINN_RT_CHECK(f->type.code == cinn_type_float && f->type.bits == 32, "cinn_call_hip_conv2d_pair_chain: scale / shift must be fp32");
  const bool is_16 = x->type.bits == 16 && (x->type.code == cinn_type_float || x->type.code == cinn_type_bfloat);
  for (cinn_buffer_t* b : {x2, w1, w2, e, y})
    CINN_RT_CHECK(is_16 && b->type.code == x->type.code && b->type.bits == x->type.bits,
                  "cinn_call_hip_conv2d_pair_chain: x, x2, w1, w2, e and y must share one 16-bit floating-point type");
  CINN_RT_CHECK(input_n > 0 && input_h > 0 && input_w > 0 && input_c > 0 && second_c > 0 && middle_c > 0 && output_c > 0,
                "cinn_call_hip_conv2d_pair_chain: extents must be positive");
  hipStream_t st = static_cast<hipStream_t>(stream);
  cinn_hip_kernels::ConvChainArgs a;
  a.x = x->memory, a.w1 = w1->memory, a.scale1 = nullptr;
  a.shift1 = reinterpret_cast<const float*>(t1->memory), a.residual = nullptr, a.relu1 = (relu & 1) != 0;
  a.e = e->memory, a.w2 = w2->memory, a.scale2 = reinterpret_cast<const float*>(s2->memory);
  a.shift2 = reinterpret_cast<const float*>(t2->memory), a.relu2 = (relu & 2) != 0, a.y = y->memory;
  a.m = (int64_t)input_n * input_h * input_w, a.k1 = input_c, a.n1 = middle_c, a.n2 = output_c, a.type = x->type;
  a.x2 = x2->memory, a.k1b = second_c;
  if (cinn_hip_kernels::TryConvChain(a, st)) return;
  // any other shape: the first layer over both inputs (which has shape limits of its own), then the second layer
  cinn_pod_value_t first[5];
  cinn_buffer_t* first_bufs[5] = {x, x2, w1, t1, e};
  for (int i = 0; i < 5; ++i) {
    first[i].type_code_      = CINN_POD_BUFFER_P;
    first[i].value_.v_handle = first_bufs[i];
  }
  cinn_call_hip_conv2d_pointwise_pair(first, 5, relu & 1, input_n, input_h, input_w, input_c, input_h, input_w, second_c, 1, 1, middle_c,
                                      stream);
  RunConv(e, w2, y, a.scale2, a.shift2, nullptr, a.relu2 ? 2 : 1, 1, 1.0f, 0.0f, input_n, middle_c, input_h, input_w, output_c,
          middle_c, 1, 1, 0, 0, 1, 1, 1, 1, 1, input_n, output_c, input_h, input_w, st);
}

void cinn_call_hip_conv2d_pointwise_pair(void* v_args, int num_args, int relu, int input_n, int input_h, int input_w,
                                         int input_c, int second_h, int second_w, int second_c, int second_stride_h,
                                         int second_stride_w, int output_c, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 5, "cinn_call_hip_conv2d_pointwise_pair takes x, x2, w, shift and y, got %d arguments", num_args);
  cinn_buffer_t* x     = BufferArg(v_args, 0);
  cinn_buffer_t* x2    = BufferArg(v_args, 1);
  cinn_buffer_t* w     = BufferArg(v_args, 2);
  cinn_buffer_t* shift = BufferArg(v_args, 3);
  cinn_buffer_t* y     = BufferArg(v_args, 4);
  CINN_RT_CHECK(shift->type.code == cinn_type_float && shift->type.bits == 32, "cinn_call_hip_conv2d_pointwise_pair: shift must be fp32");
  const bool is_16 = x->type.bits == 16 && (x->type.code == cinn_type_float || x->type.code == cinn_type_bfloat);
  for (cinn_buffer_t* b : {x2, w, y})
    CINN_RT_CHECK(is_16 && b->type.code == x->type.code && b->type.bits == x->type.bits,
                  "cinn_call_hip_conv2d_pointwise_pair: x, x2, w and y must share one 16-bit floating-point type");
  CINN_RT_CHECK(input_n > 0 && input_h > 0 && input_w > 0 && input_c > 0 && second_h > 0 && second_w > 0 && second_c > 0 &&
                    second_stride_h > 0 && second_stride_w > 0 && output_c > 0,
                "cinn_call_hip_conv2d_pointwise_pair: extents and strides must be positive");
  CINN_RT_CHECK((input_h - 1) * second_stride_h < second_h && (input_w - 1) * second_stride_w < second_w,
                "cinn_call_hip_conv2d_pointwise_pair: a %dx%d grid at stride %dx%d does not fit the second input's %dx%d pixels",
                input_h, input_w, second_stride_h, second_stride_w, second_h, second_w);
  const int64_t m = (int64_t)input_n * input_h * input_w;
  CINN_RT_CHECK(cinn_hip_kernels::ConvPairShape(m, input_c, second_c, output_c),
                "cinn_call_hip_conv2d_pointwise_pair: no kernel for %lld pixels, %d + %d -> %d channels (ConvPairShape)",
                (long long)m, input_c, second_c, output_c);
  cinn_hip_kernels::ConvNhwcArgs a;
  a.x = x->memory, a.w = w->memory, a.y = y->memory;
  a.scale = nullptr, a.shift = reinterpret_cast<const float*>(shift->memory);
  a.residual = nullptr, a.alpha = 1.0f, a.residual_scale = 0.0f;
  a.relu = (relu & 1) != 0, a.nchw_input = false;
  a.n = input_n, a.h = input_h, a.w_in = input_w, a.c = input_c;
  a.oc = output_c, a.kh = 1, a.kw = 1, a.oh = input_h, a.ow = input_w;
  a.pad_h = a.pad_w = 0, a.stride_h = a.stride_w = a.dil_h = a.dil_w = 1;
  a.type = x->type;
  a.x2 = x2->memory, a.h2 = second_h, a.w2 = second_w, a.c2 = second_c;
  a.stride2_h = second_stride_h, a.stride2_w = second_stride_w;
  cinn_hip_kernels::RunConvNhwc(a, static_cast<hipStream_t>(stream));
}

}  // extern "C"
