// First convolution of a network on the MFMA units: NCHW input with a handful of channels (an image), [O][I][KH][KW]
// filter, channels-last output with the fused epilogue of the other convolution kernels.
//
// With 3 input channels there is nothing contiguous along the reduction index to load, and gathering the im2col
// operand element by element from global memory costs one load instruction per tap.  Here a block stages what it
// needs in LDS with coalesced loads and builds MFMA fragments from there:
//   * the filter, once per block, as the GEMM operand [64 output channels][segments of 8 taps]: a segment is 8
//     neighbouring dx of one (c, dy) row, zero-padded past KW, so a fragment is one ds_read_b128;
//   * per output tile of 8 x 16 pixels of one image, the input patch [C][PH][PW] that the tile's windows cover
//     (zero outside the image).  The 8 taps of a segment are 8 consecutive patch elements for every pixel, so the
//     pixel-operand fragment of a lane is 16 consecutive bytes of LDS (read as dwords when the stride keeps them
//     4-byte aligned, else as halves);
//   * a block walks through several tiles, so the filter staging is amortised.
// Each of the 4 wavefronts owns 32 pixels (two tile rows) x 64 channels = two 32x32 accumulators.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdlib>

#include <mutex>

#include "kernels/conv_nhwc.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kTileH    = 8;
constexpr int kTileW    = 16;
constexpr int kOcBlock  = 64;
constexpr int kStagePitch = kOcBlock / 2 + 8;  // floats; the staging tile holds 32 channels at a time
constexpr int kMaxSegments = 32;
constexpr int kRowsPerWave = 16;  // patch rows (c, pr) a wavefront loads per tile: c * patch_h <= 64, patch_w <= 64

struct StemParams {
  int n, c, h, w;
  int oc, kh, kw;
  int oh, ow;
  int pad_h, pad_w, stride_h, stride_w;
  int segs_per_row;  // ceil(kw / 8)
  int segments;      // c * kh * segs_per_row
  int segments_pad;  // rounded up to what one MFMA K slice consumes
  int patch_h, patch_w;  // patch_w even
  int filter_pitch;      // bytes per output channel of the staged filter (an odd number of 16-byte units)
  int filter_bytes, patch_bytes;
  int tiles_h, tiles_w, tiles, tiles_per_block;
  int relu;
  float alpha, residual_scale;
};

template <typename T>
struct Mfma16;
template <>
struct Mfma16<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 run(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 run(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// K loop of one tile: 16-bit types, two segments (16 taps) per MFMA.  STEPS > 0: the trip count is known at compile
// time and the loop is unrolled, so that the LDS reads of all steps can be in flight together.
template <typename T, int STEPS>
struct TileMma {
  static __device__ __forceinline__ void Run(const char* filter, const T* patch, const int* seg_offset, const int* seg_mask,
                                             int pixel_offset, bool dword_aligned, int lane, const StemParams& p,
                                             f32x16 (&acc)[2]) {
  typedef typename Mfma16<T>::vec8 vec8;
  const int kg    = lane >> 5;
  const int steps = STEPS > 0 ? STEPS : p.segments_pad / 2;
#pragma unroll
  for (int kk = 0; kk < steps; ++kk) {
    const int seg  = 2 * kk + kg;
    const T* src   = patch + seg_offset[seg] + pixel_offset;
    const int mask = seg_mask[seg];
    T a[8];
    if (dword_aligned) {
      uint32_t d[4];
      const uint32_t* s32 = reinterpret_cast<const uint32_t*>(src);
#pragma unroll
      for (int i = 0; i < 4; ++i) d[i] = s32[i];
      __builtin_memcpy(a, d, 16);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = src[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (!((mask >> e) & 1)) a[e] = (T)0.0f;
    vec8 af;
    __builtin_memcpy(&af, a, 16);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      vec8 bf = *reinterpret_cast<const vec8*>(filter + (j * 32 + (lane & 31)) * p.filter_pitch + seg * 16);
      acc[j]  = Mfma16<T>::run(af, bf, acc[j]);
    }
  }
  }
};

// fp32: one segment (8 taps) per step, lanes 0-31 take taps 0..3 and lanes 32-63 taps 4..7; v_mfma_f32_32x32x2_f32
// number e of the step multiplies tap e of each half
template <int STEPS>
struct TileMma<float, STEPS> {
  static __device__ __forceinline__ void Run(const char* filter, const float* patch, const int* seg_offset,
                                             const int* seg_mask, int pixel_offset, bool, int lane, const StemParams& p,
                                             f32x16 (&acc)[2]) {
  const int kg    = lane >> 5;
  const int steps = STEPS > 0 ? STEPS : p.segments_pad;
#pragma unroll
  for (int seg = 0; seg < steps; ++seg) {
    const float* src = patch + seg_offset[seg] + pixel_offset + 4 * kg;
    const int mask   = seg_mask[seg] >> (4 * kg);
    float a[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) a[e] = ((mask >> e) & 1) ? src[e] : 0.0f;
    f32x4 b[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
      b[j] = *reinterpret_cast<const f32x4*>(filter + (j * 32 + (lane & 31)) * p.filter_pitch + seg * 32 + kg * 16);
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[j][e], acc[j], 0, 0, 0);
  }
  }
};

template <typename T, int STEPS>
__global__ void __launch_bounds__(256)
conv_stem_kernel(const T* __restrict__ x, const T* __restrict__ w, T* y, const float* __restrict__ scale,
                 const float* __restrict__ shift, const T* residual, StemParams p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ int seg_offset[kMaxSegments];  // patch offset of tap 0 of a segment, for the pixel at the tile origin
  __shared__ int seg_mask[kMaxSegments];    // which of its 8 taps exist
  __shared__ int row_base[4 * kRowsPerWave];  // patch row (c, pr) -> element offset of channel c in an image
  __shared__ int row_pr[4 * kRowsPerWave];    // patch row -> pr
  char* filter = lds;
  T* patch     = reinterpret_cast<T*>(lds + p.filter_bytes);
  float* stage = reinterpret_cast<float*>(lds + p.filter_bytes + p.patch_bytes);

  const int tid     = threadIdx.x;
  const int lane    = tid & 63;
  const int wave    = tid >> 6;
  const int oc_base = blockIdx.y * kOcBlock;

  // ---- segment table and filter, once per block ---------------------------------------------------------------
  for (int seg = tid; seg < p.segments_pad; seg += 256) {
    int off = 0, mask = 0;
    if (seg < p.segments) {
      const int row = seg / p.segs_per_row;  // (c, dy)
      const int sx  = seg - row * p.segs_per_row;
      const int c   = row / p.kh;
      const int dy  = row - c * p.kh;
      off           = (c * p.patch_h + dy) * p.patch_w + sx * 8;
      for (int e = 0; e < 8; ++e) mask |= (sx * 8 + e < p.kw ? 1 : 0) << e;
    }
    seg_offset[seg] = off;
    seg_mask[seg]   = mask;
  }
  const int patch_rows = p.c * p.patch_h;
  for (int r = tid; r < patch_rows; r += 256) {
    const int c = r / p.patch_h;
    row_base[r] = c * p.h * p.w;
    row_pr[r]   = r - c * p.patch_h;
  }
  // filter: (output channel, segment) pairs round-robin over the threads; all global loads first, then the LDS stores
  {
    constexpr int kPairs = kOcBlock * kMaxSegments / 256;
    T taps[kPairs][8];
#pragma unroll
    for (int it = 0; it < kPairs; ++it) {
      const int q   = tid + 256 * it;
      const int ocl = q / p.segments_pad;
      const int seg = q - ocl * p.segments_pad;
      const int oc  = oc_base + ocl;
      const int row = seg / p.segs_per_row;  // c * kh + dy
      const int sx  = seg - row * p.segs_per_row;
      const bool ok = q < kOcBlock * p.segments_pad && seg < p.segments && oc < p.oc;
      const T* src  = w + ((int64_t)oc * p.c * p.kh + row) * p.kw + sx * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) taps[it][e] = (ok && sx * 8 + e < p.kw) ? src[e] : (T)0.0f;
    }
#pragma unroll
    for (int it = 0; it < kPairs; ++it) {
      const int q = tid + 256 * it;
      if (q < kOcBlock * p.segments_pad) {
        const int ocl = q / p.segments_pad;
        const int seg = q - ocl * p.segments_pad;
        __builtin_memcpy(filter + ocl * p.filter_pitch + seg * 8 * sizeof(T), taps[it], 8 * sizeof(T));
      }
    }
  }

  // pixel of this lane inside a tile: wavefront w owns tile rows 2w and 2w+1
  const int tr           = 2 * wave + ((lane & 31) >> 4);
  const int tc           = lane & 15;
  const int pixel_offset = tr * p.stride_h * p.patch_w + tc * p.stride_w;
  const bool dword_aligned = sizeof(T) == 2 && (p.stride_w & 1) == 0;

  // epilogue mapping: per 32-channel half, 4 channel groups of 8 per pixel
  const int cg = tid & 3;
  float sc[2][8], sh[2][8];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      int oc   = oc_base + j * 32 + cg * 8 + e;
      oc       = oc < p.oc ? oc : p.oc - 1;
      sc[j][e] = scale ? scale[oc] : p.alpha;
      sh[j][e] = shift ? shift[oc] : 0.0f;
    }
  const bool full = (p.oc & 7) == 0;

  // Patch rows (c, pr) go round-robin to the wavefronts, lanes along the row.  All loads of a thread are issued before
  // anything waits for them, and the patch of the next tile is fetched into registers while the current one is being
  // multiplied.
  T regs[kRowsPerWave];
  auto fetch_patch = [&](int t) {
    const int n   = t / (p.tiles_h * p.tiles_w);
    const int rem = t - n * (p.tiles_h * p.tiles_w);
    const int th  = rem / p.tiles_w;
    const int ih0 = th * kTileH * p.stride_h - p.pad_h;
    const int iw  = (rem - th * p.tiles_w) * kTileW * p.stride_w - p.pad_w + lane;
    const T* image    = x + (int64_t)n * p.c * p.h * p.w;
    const bool col_ok = t < p.tiles && lane < p.patch_w && (unsigned)iw < (unsigned)p.w;
#pragma unroll
    for (int k = 0; k < kRowsPerWave; ++k) {
      const int r = wave + 4 * k;
      T v         = (T)0.0f;
      if (r < patch_rows) {
        const int ih = ih0 + row_pr[r];
        if (col_ok && (unsigned)ih < (unsigned)p.h) v = image[row_base[r] + ih * p.w + iw];
      }
      regs[k] = v;
    }
  };

  __syncthreads();  // row tables
  fetch_patch(blockIdx.x);
  for (int t = blockIdx.x; t < p.tiles; t += gridDim.x) {
    const int n   = t / (p.tiles_h * p.tiles_w);
    const int rem = t - n * (p.tiles_h * p.tiles_w);
    const int th  = rem / p.tiles_w;
    const int oh0 = th * kTileH;
    const int ow0 = (rem - th * p.tiles_w) * kTileW;

#pragma unroll
    for (int k = 0; k < kRowsPerWave; ++k) {
      const int r = wave + 4 * k;
      if (r < patch_rows && lane < p.patch_w) patch[r * p.patch_w + lane] = regs[k];
    }
    // patch (and, the first time, the filter) complete; every wavefront has finished the previous tile's stores,
    // so the staging tile is free again
    __syncthreads();
    fetch_patch(t + gridDim.x);  // nothing is read past the last tile

    f32x16 acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
    TileMma<T, STEPS>::Run(filter, patch, seg_offset, seg_mask, pixel_offset, dword_aligned, lane, p, acc);

    // the two 32-channel halves go through the staging tile one after the other (half the LDS, one more block per CU)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (j > 0) __syncthreads();  // first half has been read
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wave * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        stage[row * kStagePitch + (lane & 31)] = acc[j][r];
      }
      __syncthreads();  // staged; after the MFMAs nobody reads the patch any more
      const int oc0 = oc_base + j * 32 + cg * 8;
      if (oc0 >= p.oc) continue;
      for (int pixel = tid >> 2; pixel < kTileH * kTileW; pixel += 64) {
        const int oh = oh0 + (pixel >> 4), ow = ow0 + (pixel & 15);
        if (oh >= p.oh || ow >= p.ow) continue;
        float v[8];
        *reinterpret_cast<f32x4*>(&v[0]) = *reinterpret_cast<const f32x4*>(&stage[pixel * kStagePitch + cg * 8]);
        *reinterpret_cast<f32x4*>(&v[4]) = *reinterpret_cast<const f32x4*>(&stage[pixel * kStagePitch + cg * 8 + 4]);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(v[e], sc[j][e], sh[j][e]);
        const int64_t off = (((int64_t)n * p.oh + oh) * p.ow + ow) * p.oc + oc0;
        if (full) {
          T out[8];
          if (residual) {
            T rv[8];
            __builtin_memcpy(rv, residual + off, 8 * sizeof(T));
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(p.residual_scale, (float)rv[e], v[e]);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) out[e] = (T)(p.relu ? fmaxf(v[e], 0.0f) : v[e]);
          __builtin_memcpy(y + off, out, 8 * sizeof(T));
        } else {
          for (int e = 0; e < 8 && oc0 + e < p.oc; ++e) {
            float r = v[e];
            if (residual) r += p.residual_scale * (float)residual[off + e];
            y[off + e] = (T)(p.relu ? fmaxf(r, 0.0f) : r);
          }
        }
      }
    }
  }
}

bool FillParams(const ConvNhwcArgs& a, StemParams* out) {
  StemParams p;
  p.n = a.n, p.c = a.c, p.h = a.h, p.w = a.w_in;
  p.oc = a.oc, p.kh = a.kh, p.kw = a.kw, p.oh = a.oh, p.ow = a.ow;
  p.pad_h = a.pad_h, p.pad_w = a.pad_w, p.stride_h = a.stride_h, p.stride_w = a.stride_w;
  const int elem     = a.type.bits / CHAR_BIT;
  p.segs_per_row     = (a.kw + 7) / 8;
  p.segments         = a.c * a.kh * p.segs_per_row;
  p.segments_pad     = elem == 2 ? (p.segments + 1) / 2 * 2 : p.segments;
  if (p.segments_pad > kMaxSegments) return false;
  if (a.c * ((kTileH - 1) * a.stride_h + a.kh) > 4 * kRowsPerWave) return false;
  if ((kTileW - 1) * a.stride_w + p.segs_per_row * 8 + 1 > 64) return false;
  p.patch_h          = (kTileH - 1) * a.stride_h + a.kh;
  p.patch_w          = ((kTileW - 1) * a.stride_w + p.segs_per_row * 8 + 1) / 2 * 2;
  int units          = p.segments_pad * 8 * elem / 16;
  if (units % 2 == 0) units += 1;  // odd pitch in 16-byte units: 16 consecutive rows fall into distinct bank groups
  p.filter_pitch     = units * 16;
  p.filter_bytes     = kOcBlock * p.filter_pitch;
  p.patch_bytes      = (a.c * p.patch_h * p.patch_w * elem + 15) / 16 * 16;
  p.tiles_h          = (a.oh + kTileH - 1) / kTileH;
  p.tiles_w          = (a.ow + kTileW - 1) / kTileW;
  p.tiles            = a.n * p.tiles_h * p.tiles_w;
  p.tiles_per_block  = 0;  // unused: blocks stride over the tiles
  p.relu             = a.relu ? 1 : 0;
  p.alpha            = a.alpha;
  p.residual_scale   = a.residual_scale;
  *out               = p;
  return true;
}

int LdsBytes(const StemParams& p) { return p.filter_bytes + p.patch_bytes + kTileH * kTileW * kStagePitch * 4; }

template <typename T, int STEPS>
void Launch(const ConvNhwcArgs& a, const StemParams& p, hipStream_t stream) {
  auto kernel     = conv_stem_kernel<T, STEPS>;
  const int bytes = LdsBytes(p);
  {
    static std::mutex mu;  // per instantiation: the attribute only ever grows
    static int configured = 0;
    std::lock_guard<std::mutex> lock(mu);
    if (bytes > configured) {
      CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
      configured = bytes;
    }
  }
  // a few blocks per CU stride over the tiles: the filter staging is amortised and the tail is short
  int per_cu = (160 * 1024) / bytes;
  if (per_cu > 4) per_cu = 4;
  const int resident = 256 * per_cu;  // as many blocks as fit at once: one round, no tail of a second one
  dim3 grid(p.tiles < resident ? p.tiles : resident, (p.oc + kOcBlock - 1) / kOcBlock);
  hipLaunchKernelGGL(kernel, grid, dim3(256), bytes, stream, static_cast<const T*>(a.x), static_cast<const T*>(a.w),
                     static_cast<T*>(a.y), a.scale, a.shift, static_cast<const T*>(a.residual), p);
  CINN_HIP_CALL(hipGetLastError());
}

}  // namespace

bool ConvStemSupported(const ConvNhwcArgs& a) {
  if (!a.nchw_input || a.dil_h != 1 || a.dil_w != 1) return false;
  if (getenv("FLAGS_cinn_hip_conv_stem_gather")) return false;  // keep the element-gather loader selectable
  StemParams p;
  if (!FillParams(a, &p)) return false;
  if (LdsBytes(p) > 96 * 1024) return false;
  return (int64_t)a.n * a.c * a.h * a.w_in < INT_MAX;
}

void RunConvStem(const ConvNhwcArgs& a, hipStream_t stream) {
  StemParams p;
  CINN_RT_CHECK(FillParams(a, &p), "conv2d (NCHW-input): filter too large for the staged kernel");
  // the 7x7 filter over 3 channels (21 segments) has its own unrolled instance
  const bool rgb7 = p.segments == 21;
  if (a.type.code == cinn_type_bfloat) {
    rgb7 ? Launch<__bf16, 11>(a, p, stream) : Launch<__bf16, 0>(a, p, stream);
  } else if (a.type.bits == 16) {
    rgb7 ? Launch<_Float16, 11>(a, p, stream) : Launch<_Float16, 0>(a, p, stream);
  } else {
    rgb7 ? Launch<float, 21>(a, p, stream) : Launch<float, 0>(a, p, stream);
  }
}

}  // namespace cinn_hip_kernels
