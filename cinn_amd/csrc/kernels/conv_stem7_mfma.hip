// The first convolution of an image network in its usual form - 7x7, stride 2, padding 3 over a 3-channel NCHW image,
// 16-bit types - with channels-last output and the fused epilogue of the other convolution kernels.
//
// conv_stem_kernel (conv_stem_mfma.hip) handles any small-channel NCHW convolution but spends its time around the
// MFMAs: 2-byte global loads and LDS stores for the patch, four barriers and an fp32 staging pass per 128-pixel tile
// (46 us for 9 GFLOP and 51 MB at batch 32).  This kernel is built like conv3x3_c64_patch_kernel:
//   * a block is persistent and walks over tiles of 448 output pixels (rows of one image); wavefronts 0..3 compute,
//     wavefronts 4..7 fetch the next tile's input rows - whole 16-byte vectors of the NCHW rows - into the other of two
//     patch buffers while the current tile is multiplied: one barrier per tile;
//   * the patch is [3 channels][input rows][8 + W + 8 columns] with the zero halo stored; the reduction index is
//     (channel, dy) x 8 column slots: slot 0 is the column left of the window (zero filter weight; cleared in the
//     fragment so that a NaN there cannot leak), slots 1..7 the filter's columns, so a window starts at the even
//     column 2 ox - 4 and a fragment is four aligned dwords.  21 such segments, padded to 24 = 6 MFMA slices;
//   * a computing wavefront holds 7 x 4 accumulators of v_mfma_f32_16x16x32 (112 pixels x 64 channels) and computes
//     the transposed tile, so that the epilogue runs in registers and, after an exchange between lanes (DPP row shifts
//     by 8), every store instruction writes 8 pixels x 128 contiguous bytes;
//   * the filter is staged once per block as [64 channels][192], rows swizzled as in conv3x3_c64_patch_kernel.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdlib>

#include "kernels/conv_nhwc.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma16;
template <>
struct Mfma16<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x4 mma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

constexpr int kTMW       = 7;                  // 16-pixel tiles per computing wavefront
constexpr int kWaves     = 4;                  // computing wavefronts (as many fetching ones)
constexpr int kCapacity  = kWaves * kTMW * 16; // pixels per tile
constexpr int kSegments  = 21;                 // (channel, dy)
constexpr int kSlices    = 6;                  // MFMA slices of 4 segments
constexpr int kFilterRow = kSlices * 4 * 16;   // bytes of a filter row: 24 segments of 8 halves
constexpr int kFilterBytes = 64 * kFilterRow;
constexpr int kTableBytes  = 2 * 64 * 4;       // scale and shift of the block's 64 channels
constexpr int kMaxVectors  = 6;                // 16-byte vectors a fetching thread holds per tile
constexpr int kLdsLimit    = 160 * 1024;

struct Stem7Params {
  const uint16_t* x;  // [N][3][H][W]
  const uint16_t* w;  // [OC][3][7][7]
  uint16_t* y;        // [N][OH][OW][OC]
  const float* scale;
  const float* shift;
  const uint16_t* residual;
  float alpha, residual_scale;
  int relu;
  int n, h, w_in, oc, oh, ow;
  int rows;        // output rows per tile
  int strips;      // tiles per image
  int tiles;       // n * strips
  int patch_rows;  // input rows per channel held for a tile: 2 (rows - 1) + 7
  int pitch;       // bytes between patch rows: 64 modulo 256, at least 2 (W + 16)
  int patch_bytes;
  unsigned ow_magic, ow_shift;    // n / OW
  unsigned vec_magic, vec_shift;  // n / (W / 8)
};

__device__ __forceinline__ int FilterKey(int r) { return ((r >> 1) & 1) * 2 + ((r >> 3) & 1) * 4 + ((r >> 2) & 1); }

template <bool SHR>
__device__ __forceinline__ unsigned RowShift8(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, SHR ? 0x118 : 0x108, 0xf, 0xf, true);
}

// Block barrier that orders LDS accesses only.  __syncthreads() also waits until every global store of the wavefront
// has completed (its release covers global memory); here that would stall the computing wavefronts at every tile until
// the tile's 57 KB of results have left, instead of letting them drain under the next tile's MFMAs.
__device__ __forceinline__ void BarrierLds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <typename T>
__global__ void __launch_bounds__(128 * kWaves) conv_stem7_kernel(Stem7Params p) {
  typedef typename Mfma16<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* const filter = lds;
  float* const table = reinterpret_cast<float*>(lds + kFilterBytes);  // [scale | shift][64]
  char* const patch0 = lds + kFilterBytes + kTableBytes;
  const int tid      = threadIdx.x;
  const int lane     = tid & 63;
  const int wave     = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0       = blockIdx.y * 64;
  const int row_vecs = p.w_in >> 3;  // 16-byte vectors per image row

  // ---- once per block: both patch buffers zero (the halo columns stay so), the filter slice in fragment order
  for (int v = tid; v < (2 * p.patch_bytes) >> 4; v += 128 * kWaves) *reinterpret_cast<u32x4*>(patch0 + v * 16) = u32x4{0u, 0u, 0u, 0u};
  for (int q = tid; q < 64 * 4 * kSlices; q += 128 * kWaves) {
    const int row = q / (4 * kSlices), seg = q - row * (4 * kSlices);
    uint16_t taps[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (seg < kSegments) {
      const uint16_t* src = p.w + ((int64_t)(n0 + row) * kSegments + seg) * 7;  // [oc][c][dy][7]
#pragma unroll
      for (int e = 0; e < 7; ++e) taps[e + 1] = src[e];
    }
    const int slot = (seg & ~7) | ((seg & 7) ^ FilterKey(row));
    __builtin_memcpy(filter + row * kFilterRow + slot * 16, taps, 16);
  }
  if (tid < 64) {
    table[tid]      = p.scale ? p.scale[n0 + tid] : p.alpha;
    table[64 + tid] = p.shift ? p.shift[n0 + tid] : 0.0f;
  }
  __syncthreads();

  if (wave >= kWaves) {
    // ---- fetching wavefronts: vector v of a tile = 8 columns of one (channel, patch row)
    const int ft      = tid - 64 * kWaves;
    const int vectors = 3 * p.patch_rows * row_vecs;
    int k = 0;
    for (int t = blockIdx.x; t < p.tiles; t += gridDim.x, ++k) {
      const int img   = t / p.strips;
      const int iy0   = (t - img * p.strips) * p.rows * 2 - 3;
      const uint16_t* image = p.x + (int64_t)img * 3 * p.h * p.w_in;
      char* const buf = patch0 + (k & 1) * p.patch_bytes;
      u32x4 regs[kMaxVectors];
      int dst[kMaxVectors];
#pragma unroll
      for (int e = 0; e < kMaxVectors; ++e) {
        const int v = ft + 64 * kWaves * e;
        dst[e]      = -1;
        regs[e]     = u32x4{0u, 0u, 0u, 0u};
        if (v < vectors) {
          const int prow = (int)(((uint64_t)(unsigned)v * p.vec_magic) >> p.vec_shift);  // channel * patch_rows + pr
          const int col  = v - prow * row_vecs;
          const int c    = prow / p.patch_rows;
          const int iy   = iy0 + prow - c * p.patch_rows;
          dst[e]         = prow * p.pitch + 16 + col * 16;  // image column 0 sits at patch column 8
          if ((unsigned)iy < (unsigned)p.h)
            regs[e] = *reinterpret_cast<const u32x4*>(image + ((int64_t)c * p.h + iy) * p.w_in + col * 8);
        }
      }
#pragma unroll
      for (int e = 0; e < kMaxVectors; ++e)
        if (dst[e] >= 0) *reinterpret_cast<u32x4*>(buf + dst[e]) = regs[e];
      BarrierLds();  // tile k is in its buffer; the other buffer's tile (k - 1) has been multiplied
    }
    return;
  }

  // ---- computing wavefronts
  const int kgc  = ((lane >> 4) & 1) * 2 + (lane >> 5);  // k chunk of this lane group: 0, 2, 1, 3
  const int pix0 = wave * (kTMW * 16) + (lane & 15);
  // byte offset of the window's first column (2 ox - 4, patch column 2 ox + 4) in the patch row of the window's first
  // input row (2 ly), per tile; pixels beyond the tile read offset 0, their results are not stored
  int a_pix[kTMW];
#pragma unroll
  for (int i = 0; i < kTMW; ++i) {
    const int pix = pix0 + 16 * i;
    const int ly  = (int)(((uint64_t)(unsigned)pix * p.ow_magic) >> p.ow_shift);
    const int ox  = pix - ly * p.ow;
    a_pix[i]      = ly < p.rows ? 2 * ly * p.pitch + (2 * ox + 4) * 2 : 0;
  }
  // segment 4 s + kgc = (channel, dy) of slice s; the padding segments 21..23 read segment 0 and are cleared
  int seg_off[kSlices];
#pragma unroll
  for (int s = 0; s < kSlices; ++s) {
    int seg    = 4 * s + kgc;
    seg        = seg < kSegments ? seg : 0;
    const int c = seg / 7;
    seg_off[s] = (c * p.patch_rows + seg - 7 * c) * p.pitch;
  }
  const bool pad_lane = 4 * (kSlices - 1) + kgc >= kSegments;  // in the last slice
  // filter fragment of tile j: row 32 (j / 2) + 8 g' + 4 (j % 2) + r' (q = lane & 15 = 4 g' + r'); slices of equal
  // parity differ by whole 128-byte groups
  const char* b_base[2][4];
  {
    const int q = lane & 15;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 32 * (j >> 1) + 8 * (q >> 2) + 4 * (j & 1) + (q & 3);
#pragma unroll
      for (int sp = 0; sp < 2; ++sp) b_base[sp][j] = filter + row * kFilterRow + (((4 * sp + kgc) ^ FilterKey(row)) << 4);
    }
  }
  const int g   = lane >> 4;
  const int px  = lane & 15;
  const int oc0 = n0 + 8 * g;
  T* const Y         = reinterpret_cast<T*>(p.y);
  const T* const R   = reinterpret_cast<const T*>(p.residual);
  const int st_chunk = g + 4 * (px >> 3);  // 16-byte chunk of a pixel's 64 channels that this lane stores

  int k = 0;
  for (int t = blockIdx.x; t < p.tiles; t += gridDim.x, ++k) {
    const int img  = t / p.strips;
    const int oy0  = (t - img * p.strips) * p.rows;
    const int npix = min(p.rows, p.oh - oy0) * p.ow;
    const char* const buf = patch0 + (k & 1) * p.patch_bytes;
    BarrierLds();  // tile k is in its buffer

    f32x4 acc[kTMW][4];
#pragma unroll
    for (int i = 0; i < kTMW; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // 42 rows of 4 MFMAs: row 7 s + i multiplies the pixel fragment of tile i, slice s, with the slice's four filter
    // fragments.  Pixel fragments are requested three rows ahead into one register set per tile, the next slice's
    // filter fragments during rows 0 and 1 of a slice; scheduling barriers pin that order.
    // the raw dwords of a fragment are requested early and patched when the row that uses them starts: slot 0 (the
    // column left of the window) is cleared, and so are the padding segments of the last slice
    const char* a_tile[kTMW];
#pragma unroll
    for (int i = 0; i < kTMW; ++i) a_tile[i] = buf + a_pix[i];
    auto read_a = [&](int s, int i) -> u32x4 {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(a_tile[i] + seg_off[s]);
      u32x4 d;
#pragma unroll
      for (int e = 0; e < 4; ++e) d[e] = src[e];
      return d;
    };
    auto patched = [&](int s, u32x4 d) -> vec8 {
      d[0] &= 0xffff0000u;
      if (s == kSlices - 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) d[e] = pad_lane ? 0u : d[e];
      }
      return __builtin_bit_cast(vec8, d);
    };
    auto read_b = [&](int s, int j) -> vec8 { return *reinterpret_cast<const vec8*>(b_base[s & 1][j] + (s >> 1) * 128); };
    u32x4 ar[kTMW];
    vec8 bf[2][4];
#pragma unroll
    for (int r = 0; r < 3; ++r) ar[r] = read_a(0, r);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[0][j] = read_b(0, j);
#define CINN_SB __builtin_amdgcn_sched_barrier(0)
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
#pragma unroll
      for (int i = 0; i < kTMW; ++i) {
        CINN_SB;
        const vec8 af = patched(s, ar[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          CINN_SB;
          acc[i][j] = Mfma16<T>::mma(bf[s & 1][j], af, acc[i][j]);
          CINN_SB;
          const int rr = kTMW * s + i + 3;
          if (j == 0 && rr < kTMW * kSlices) ar[rr % kTMW] = read_a(rr / kTMW, rr % kTMW);
          if ((j == 1 || j == 2) && i < 2 && s + 1 < kSlices) bf[(s + 1) & 1][i * 2 + j - 1] = read_b(s + 1, i * 2 + j - 1);
        }
      }
    }
    CINN_SB;
#undef CINN_SB

    // epilogue in registers, as in conv3x3_c64_patch_kernel
    const int64_t out_row0 = ((int64_t)img * p.oh + oy0) * p.ow;
    float sc[2][8], sh[2][8];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sc[s][e] = table[8 * g + 32 * s + e];
        sh[s][e] = table[64 + 8 * g + 32 * s + e];
      }
#pragma unroll
    for (int i = 0; i < kTMW; ++i) {
      const int pix = pix0 + 16 * i;
      vec8 res[2] = {};
      if (R && pix < npix) {
        const int64_t o = (out_row0 + pix) * p.oc + oc0;
        res[0] = *reinterpret_cast<const vec8*>(R + o);
        res[1] = *reinterpret_cast<const vec8*>(R + o + 32);
      }
      u32x4 out[2];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        vec8 o8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float v = __builtin_fmaf(acc[i][2 * s + (e >> 2)][e & 3], sc[s][e], sh[s][e]);
          if (R) v = __builtin_fmaf(p.residual_scale, (float)res[s][e], v);
          asm volatile("" : "+v"(v));  // keeps the fused multiply-add and the conversion apart (one rounding each)
          if (p.relu) v = v > 0.0f ? v : 0.0f;
          o8[e] = (T)v;
        }
        out[s] = __builtin_bit_cast(u32x4, o8);
      }
      u32x4 first, second;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned from_below = RowShift8<true>(out[1][d]);   // second half of lane px - 8
        const unsigned from_above = RowShift8<false>(out[0][d]);  // first half of lane px + 8
        first[d]  = px < 8 ? out[0][d] : from_below;
        second[d] = px < 8 ? from_above : out[1][d];
      }
      const int p_first  = pix - px + (px & 7);
      const int p_second = p_first + 8;
      if (p_first < npix) *reinterpret_cast<u32x4*>(Y + (out_row0 + p_first) * p.oc + n0 + 8 * st_chunk) = first;
      if (p_second < npix) *reinterpret_cast<u32x4*>(Y + (out_row0 + p_second) * p.oc + n0 + 8 * st_chunk) = second;
    }
  }
}

// q = (n * magic) >> shift == n / d for 0 <= n < 2^31
void MagicFor(int d, unsigned* magic, unsigned* shift) {
  int l = 0;
  while ((1ll << l) < d) ++l;
  *shift = 31 + l;
  *magic = (unsigned)(((1ull << *shift) / (unsigned)d) + 1);
  if (d == 1) {
    *shift = 0;
    *magic = 1;
  }
}

bool FillParams(const ConvNhwcArgs& a, Stem7Params* out) {
  const bool is_f16  = a.type.code == cinn_type_float && a.type.bits == 16;
  const bool is_bf16 = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if ((!is_f16 && !is_bf16) || !a.nchw_input) return false;
  if (a.c != 3 || a.kh != 7 || a.kw != 7 || a.stride_h != 2 || a.stride_w != 2 || a.pad_h != 3 || a.pad_w != 3 ||
      a.dil_h != 1 || a.dil_w != 1)
    return false;
  if (a.oc % 64 != 0 || a.w_in % 8 != 0 || a.ow > kCapacity) return false;
  if (a.oh != (a.h + 6 - 7) / 2 + 1 || a.ow != (a.w_in + 6 - 7) / 2 + 1) return false;
  if ((int64_t)a.n * 3 * a.h * a.w_in >= INT_MAX || (int64_t)a.n * a.oh * a.ow * a.oc >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.y) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(a.residual) % 16 != 0)
    return false;
  Stem7Params p;
  int rows = kCapacity / a.ow;
  rows     = rows < a.oh ? rows : a.oh;
  p.strips = (a.oh + rows - 1) / rows;
  rows     = (a.oh + p.strips - 1) / p.strips;
  if ((int64_t)a.oh * a.ow * 5 < (int64_t)p.strips * kCapacity * 4) return false;  // mostly empty tiles
  p.rows       = rows;
  p.tiles      = a.n * p.strips;
  p.patch_rows = 2 * (rows - 1) + 7;
  p.pitch      = ((a.w_in + 16) * 2 + 255 - 64) / 256 * 256 + 64;
  p.patch_bytes = 3 * p.patch_rows * p.pitch;
  if (kFilterBytes + kTableBytes + 2 * p.patch_bytes > kLdsLimit) return false;
  if (3 * p.patch_rows * (a.w_in / 8) > kMaxVectors * 64 * kWaves) return false;
  p.x = static_cast<const uint16_t*>(a.x), p.w = static_cast<const uint16_t*>(a.w), p.y = static_cast<uint16_t*>(a.y);
  p.scale = a.scale, p.shift = a.shift, p.residual = static_cast<const uint16_t*>(a.residual);
  p.alpha = a.alpha, p.residual_scale = a.residual_scale, p.relu = a.relu ? 1 : 0;
  p.n = a.n, p.h = a.h, p.w_in = a.w_in, p.oc = a.oc, p.oh = a.oh, p.ow = a.ow;
  MagicFor(a.ow, &p.ow_magic, &p.ow_shift);
  MagicFor(a.w_in / 8, &p.vec_magic, &p.vec_shift);
  *out = p;
  return true;
}

template <typename T>
void Launch(const Stem7Params& p, hipStream_t stream) {
  auto kernel = conv_stem7_kernel<T>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  // persistent blocks: one per CU (its eight wavefronts use the register file of a CU's four SIMDs two by two)
  const int per_group = 256 / (p.oc / 64) > 0 ? 256 / (p.oc / 64) : 1;
  dim3 grid(p.tiles < per_group ? p.tiles : per_group, p.oc / 64);
  hipLaunchKernelGGL(kernel, grid, dim3(128 * kWaves), kFilterBytes + kTableBytes + 2 * p.patch_bytes, stream, p);
}

}  // namespace

bool TryConvStem7(const ConvNhwcArgs& a, hipStream_t stream) {
  static const bool enabled = !(getenv("FLAGS_cinn_hip_conv_stem7") && atoi(getenv("FLAGS_cinn_hip_conv_stem7")) == 0);
  if (!enabled) return false;
  Stem7Params p;
  if (!FillParams(a, &p)) return false;
  if (a.type.code == cinn_type_bfloat) {
    Launch<__bf16>(p, stream);
  } else {
    Launch<_Float16>(p, stream);
  }
  CINN_HIP_CALL(hipGetLastError());
  return true;
}

}  // namespace cinn_hip_kernels
