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
// POOL: the 3x3, stride 2, padding 1 max pooling that follows such a convolution (after batch norm and relu) runs in
// the same kernel, so that the full-resolution tensor (51 MB at batch 32) never reaches memory.  A tile is then five
// convolution rows (one per computing wavefront, five of them; three wavefronts fetch), which give two pooled rows; the
// rows are staged in LDS as 16-bit values after the epilogue, and all eight wavefronts take the maxima.  (Four
// computing wavefronts with nine tiles of 16 pixels each were tried: the 144 accumulators leave too few registers,
// 58 us against 38.)  One row in
// four is computed twice (by the tile above as well).  Values are non-negative after the relu, so taps outside the
// image count as zeros.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdlib>

#include "kernels/conv_nhwc.h"
#include "kernels/mfma_tile.h"
#include "kernels/stem_pool.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

using namespace tile;

constexpr int kTMW       = 7;                  // 16-pixel tiles per computing wavefront
constexpr int kWaves     = 4;                  // computing wavefronts (as many fetching ones)
constexpr int kCapacity  = kWaves * kTMW * 16; // pixels per tile
constexpr int kSegments  = 21;                 // (channel, dy)
constexpr int kSlices    = 6;                  // MFMA slices of 4 segments
constexpr int kFilterRow = kSlices * 4 * 16;   // bytes of a filter row: 24 segments of 8 halves
constexpr int kFilterBytes = 64 * kFilterRow;
constexpr int kTableBytes  = 2 * 64 * 4;       // scale and shift of the block's 64 channels
constexpr int kLdsLimit    = 160 * 1024;
constexpr int kStagePitch  = 144;              // bytes between staged pixels (POOL): 64 channels + 16

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
  int pool_h, pool_w;             // POOL: extents of the pooled output (y is [N][pool_h][pool_w][OC])
};

// element-wise maximum of eight 16-bit values (exact in either type)
__device__ __forceinline__ f16x8 Max8(f16x8 a, f16x8 b) { return __builtin_elementwise_max(a, b); }
__device__ __forceinline__ bf16x8 Max8(bf16x8 a, bf16x8 b) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (float)a[e] > (float)b[e] ? a[e] : b[e];
  return r;
}

template <typename T, bool POOL>
__global__ void __launch_bounds__(512) conv_stem7_kernel(Stem7Params p) {
  constexpr int CW   = POOL ? 5 : kWaves;  // computing wavefronts (POOL: one per convolution row of a tile)
  constexpr int TM   = kTMW;               // 16-pixel tiles per computing wavefront
  constexpr int FT   = 512 - 64 * CW;      // fetching threads
  constexpr int MAXV = POOL ? 7 : 6;       // 16-byte vectors a fetching thread holds per tile
  typedef typename Mfma16<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* const filter = lds;
  float* const table = reinterpret_cast<float*>(lds + kFilterBytes);  // [scale | shift][64]
  char* const patch0 = lds + kFilterBytes + kTableBytes;
  char* const stage  = patch0 + 2 * p.patch_bytes;  // POOL: [5 rows][OW] pixels of kStagePitch bytes
  const int tid      = threadIdx.x;
  const int lane     = tid & 63;
  const int wave     = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0       = blockIdx.y * 64;
  const int row_vecs = p.w_in >> 3;  // 16-byte vectors per image row

  // ---- once per block: both patch buffers zero (the halo columns stay so), the filter slice in fragment order
  for (int v = tid; v < (2 * p.patch_bytes) >> 4; v += 512) *reinterpret_cast<u32x4*>(patch0 + v * 16) = u32x4{0u, 0u, 0u, 0u};
  for (int q = tid; q < 64 * 4 * kSlices; q += 512) {
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

  // tile t: image t / strips, strip t % strips; its first input row
  auto first_input_row = [&](int strip) { return POOL ? 8 * strip - 5 : strip * p.rows * 2 - 3; };
  // POOL: maxima of the staged tile - 2 pooled rows x pool_w pixels x 8 channel groups over all 512 threads
  auto pool_tile = [&](int img, int strip) {
    T* const Yp = reinterpret_cast<T*>(p.y);
    const int items = 2 * p.pool_w * 8;
    for (int it = tid; it < items; it += 512) {
      const int grp  = it & 7, q = it >> 3;
      const int prow = q >= p.pool_w ? 1 : 0, px = q - prow * p.pool_w;
      const int py   = 2 * strip + prow;
      if (py >= p.pool_h) continue;
      vec8 best = {};
#pragma unroll
      for (int dy = 0; dy < 3; ++dy)
#pragma unroll
        for (int dx = 0; dx < 3; ++dx) {
          const int cx = 2 * px - 1 + dx;
          vec8 v = {};
          if ((unsigned)cx < (unsigned)p.ow)
            v = *reinterpret_cast<const vec8*>(stage + ((2 * prow + dy) * p.ow + cx) * kStagePitch + grp * 16);
          best = Max8(best, v);
        }
      *reinterpret_cast<vec8*>(Yp + (((int64_t)img * p.pool_h + py) * p.pool_w + px) * p.oc + n0 + grp * 8) = best;
    }
  };

  if (wave >= CW) {
    // ---- fetching wavefronts: vector v of a tile = 8 columns of one (channel, patch row)
    const int ft      = tid - 64 * CW;
    const int vectors = 3 * p.patch_rows * row_vecs;
    auto fetch = [&](int t, int k) {
      const int img   = t / p.strips;
      const int iy0   = first_input_row(t - img * p.strips);
      const uint16_t* image = p.x + (int64_t)img * 3 * p.h * p.w_in;
      char* const buf = patch0 + (k & 1) * p.patch_bytes;
      u32x4 regs[MAXV];
      int dst[MAXV];
#pragma unroll
      for (int e = 0; e < MAXV; ++e) {
        const int v = ft + FT * e;
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
      for (int e = 0; e < MAXV; ++e)
        if (dst[e] >= 0) *reinterpret_cast<u32x4*>(buf + dst[e]) = regs[e];
    };
    int k = 0;
    if (POOL) {
      // tile k + 1 is fetched while tile k is multiplied; then these wavefronts help with tile k's maxima
      if ((int)blockIdx.x < p.tiles) fetch(blockIdx.x, 0);
      for (int t = blockIdx.x; t < p.tiles; t += gridDim.x, ++k) {
        BarrierLds();  // tile k is in its buffer; the staged tile k - 1 has been pooled
        if (t + (int)gridDim.x < p.tiles) fetch(t + gridDim.x, k + 1);
        BarrierLds();  // tile k's convolution rows are staged
        pool_tile(t / p.strips, t % p.strips);
      }
    } else {
      for (int t = blockIdx.x; t < p.tiles; t += gridDim.x, ++k) {
        fetch(t, k);
        BarrierLds();  // tile k is in its buffer; the other buffer's tile (k - 1) has been multiplied
      }
    }
    return;
  }

  // ---- computing wavefronts
  const int kgc  = ((lane >> 4) & 1) * 2 + (lane >> 5);  // k chunk of this lane group: 0, 2, 1, 3
  // byte offset of the window's first column (2 ox - 4, patch column 2 ox + 4) in the patch row of the window's first
  // input row (2 ly), per tile; pixels beyond the tile read offset 0, their results are not stored
  const int pix0 = wave * (TM * 16) + (lane & 15);
  int a_pix[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (POOL) {  // wavefront w multiplies convolution row w of the tile
      const int ox = 16 * i + (lane & 15);
      a_pix[i]     = ox < p.ow ? 2 * wave * p.pitch + (2 * ox + 4) * 2 : 0;
    } else {
      const int pix = pix0 + 16 * i;
      const int ly  = (int)(((uint64_t)(unsigned)pix * p.ow_magic) >> p.ow_shift);
      const int ox  = pix - ly * p.ow;
      a_pix[i]      = ly < p.rows ? 2 * ly * p.pitch + (2 * ox + 4) * 2 : 0;
    }
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

    f32x4 acc[TM][4];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // 6 TM rows of 4 MFMAs: row TM s + i multiplies the pixel fragment of tile i, slice s, with the slice's four filter
    // fragments.  Pixel fragments are requested three rows ahead into a ring of four register sets, the next slice's
    // filter fragments during rows 0 and 1 of a slice; scheduling barriers pin that order.
    // The raw dwords of a fragment are requested early and patched when the row that uses them starts: slot 0 (the
    // column left of the window) is cleared, and so are the padding segments of the last slice.
    auto read_a = [&](int s, int i) -> u32x4 {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(buf + (a_pix[i] + seg_off[s]));
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
    u32x4 ar[4];
    vec8 bf[2][4];
#pragma unroll
    for (int r = 0; r < 3; ++r) ar[r] = read_a(0, r);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[0][j] = read_b(0, j);
#define CINN_SB __builtin_amdgcn_sched_barrier(0)
#pragma unroll
    for (int s = 0; s < kSlices; ++s) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        CINN_SB;
        const vec8 af = patched(s, ar[(TM * s + i) % 4]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          CINN_SB;
          acc[i][j] = Mfma16<T>::mma(bf[s & 1][j], af, acc[i][j]);
          CINN_SB;
          const int rr = TM * s + i + 3;
          if (j == 0 && rr < TM * kSlices) ar[rr % 4] = read_a(rr / TM, rr % TM);
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
    if (POOL) {
      // this wavefront's convolution row, after scale, shift and relu, into the staging tile (zeros for a row outside
      // the image); then the maxima
      const int strip  = t - img * p.strips;
      const bool valid = (unsigned)(4 * strip - 1 + wave) < (unsigned)p.oh;  // this wavefront's row exists
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int ox = 16 * i + px;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            // relu as a max (a NaN becomes 0, as with v > 0 ? v : 0), zero for a row outside the image; the empty asm
            // keeps the fused multiply-add and the conversion apart (one rounding each)
            v[e] = __builtin_fmaxf(__builtin_fmaf(acc[i][2 * s + (e >> 2)][e & 3], sc[s][e], sh[s][e]), 0.0f);
            v[e] = valid ? v[e] : 0.0f;
            asm volatile("" : "+v"(v[e]));
          }
          const u32x4 o8 = {PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3]), PackPair<T>(v[4], v[5]), PackPair<T>(v[6], v[7])};
          if (ox < p.ow) *reinterpret_cast<u32x4*>(stage + (wave * p.ow + ox) * kStagePitch + (g + 4 * s) * 16) = o8;
        }
      }
      BarrierLds();  // the five rows are staged
      pool_tile(img, strip);
      continue;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
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
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = __builtin_fmaf(acc[i][2 * s + (e >> 2)][e & 3], sc[s][e], sh[s][e]);
          if (R) v[e] = __builtin_fmaf(p.residual_scale, (float)res[s][e], v[e]);
          const float m = __builtin_fmaxf(v[e], 0.0f);
          v[e]          = p.relu ? m : v[e];
          asm volatile("" : "+v"(v[e]));  // keeps the fused multiply-add and the conversion apart (one rounding each)
        }
        out[s] = u32x4{PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3]), PackPair<T>(v[4], v[5]), PackPair<T>(v[6], v[7])};
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

bool FillParams(const ConvNhwcArgs& a, Stem7Params* out) {
  const bool is_f16  = a.type.code == cinn_type_float && a.type.bits == 16;
  const bool is_bf16 = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if ((!is_f16 && !is_bf16) || !a.nchw_input) return false;
  if (a.c != 3 || a.kh != 7 || a.kw != 7 || a.stride_h != 2 || a.stride_w != 2 || a.pad_h != 3 || a.pad_w != 3 ||
      a.dil_h != 1 || a.dil_w != 1)
    return false;
  if (a.oc % 64 != 0 || a.w_in % 8 != 0 || a.ow > kCapacity) return false;
  if (a.pool_after && (!a.relu || a.residual || a.ow > kTMW * 16)) return false;
  if (a.oh != (a.h + 6 - 7) / 2 + 1 || a.ow != (a.w_in + 6 - 7) / 2 + 1) return false;
  if ((int64_t)a.n * 3 * a.h * a.w_in >= INT_MAX || (int64_t)a.n * a.oh * a.ow * a.oc >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.y) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(a.residual) % 16 != 0)
    return false;
  Stem7Params p;
  p.pool_h = p.pool_w = 0;
  int rows;
  if (a.pool_after) {
    // 3x3, stride 2, padding 1 pooling: a tile is 5 convolution rows -> 2 pooled rows
    p.pool_h = (a.oh + 2 - 3) / 2 + 1;
    p.pool_w = (a.ow + 2 - 3) / 2 + 1;
    rows     = 5;
    p.strips = (p.pool_h + 1) / 2;
  } else {
    rows     = kCapacity / a.ow;
    rows     = rows < a.oh ? rows : a.oh;
    p.strips = (a.oh + rows - 1) / rows;
    rows     = (a.oh + p.strips - 1) / p.strips;
    if ((int64_t)a.oh * a.ow * 5 < (int64_t)p.strips * kCapacity * 4) return false;  // mostly empty tiles
  }
  p.rows       = rows;
  p.tiles      = a.n * p.strips;
  p.patch_rows = 2 * (rows - 1) + 7;
  p.pitch      = ((a.w_in + 16) * 2 + 255 - 64) / 256 * 256 + 64;
  p.patch_bytes = 3 * p.patch_rows * p.pitch;
  const int stage_bytes = a.pool_after ? 5 * a.ow * kStagePitch : 0;
  if (kFilterBytes + kTableBytes + 2 * p.patch_bytes + stage_bytes > kLdsLimit) return false;
  if (3 * p.patch_rows * (a.w_in / 8) > (a.pool_after ? 7 * 192 : 6 * 256)) return false;
  p.x = static_cast<const uint16_t*>(a.x), p.w = static_cast<const uint16_t*>(a.w), p.y = static_cast<uint16_t*>(a.y);
  p.scale = a.scale, p.shift = a.shift, p.residual = static_cast<const uint16_t*>(a.residual);
  p.alpha = a.alpha, p.residual_scale = a.residual_scale, p.relu = a.relu ? 1 : 0;
  p.n = a.n, p.h = a.h, p.w_in = a.w_in, p.oc = a.oc, p.oh = a.oh, p.ow = a.ow;
  MagicFor(a.ow, &p.ow_magic, &p.ow_shift);
  MagicFor(a.w_in / 8, &p.vec_magic, &p.vec_shift);
  *out = p;
  return true;
}

template <typename T, bool POOL>
void Launch(const Stem7Params& p, hipStream_t stream) {
  auto kernel = conv_stem7_kernel<T, POOL>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  // persistent blocks: one per CU (its eight wavefronts use the register file of a CU's four SIMDs two by two)
  const int per_group = 256 / (p.oc / 64) > 0 ? 256 / (p.oc / 64) : 1;
  dim3 grid(p.tiles < per_group ? p.tiles : per_group, p.oc / 64);
  const int stage_bytes = POOL ? 5 * p.ow * kStagePitch : 0;
  hipLaunchKernelGGL(kernel, grid, dim3(512), kFilterBytes + kTableBytes + 2 * p.patch_bytes + stage_bytes, stream, p);
}

}  // namespace

namespace {
bool Stem7Enabled() {
  static const bool enabled = !(getenv("FLAGS_cinn_hip_conv_stem7") && atoi(getenv("FLAGS_cinn_hip_conv_stem7")) == 0);
  return enabled;
}
}  // namespace

bool StemPoolFusableShape(int n, int c, int h, int w, int oc, int kh, int kw, int stride_h, int stride_w, int pad_h,
                          int pad_w, int dil_h, int dil_w, int type_code, int type_bits) {
  if (!Stem7Enabled() || stride_h < 1 || stride_w < 1) return false;
  ConvNhwcArgs a{};
  a.nchw_input = true, a.relu = true, a.pool_after = true;
  a.n = n, a.c = c, a.h = h, a.w_in = w, a.oc = oc, a.kh = kh, a.kw = kw;
  a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w, a.dil_h = dil_h, a.dil_w = dil_w;
  a.oh = (h + 2 * pad_h - ((kh - 1) * dil_h + 1)) / stride_h + 1;
  a.ow = (w + 2 * pad_w - ((kw - 1) * dil_w + 1)) / stride_w + 1;
  a.type.code  = static_cast<cinn_type_code_t>(type_code);
  a.type.bits  = static_cast<uint8_t>(type_bits);
  a.type.lanes = 1;
  Stem7Params p;
  return FillParams(a, &p);
}

bool TryConvStem7(const ConvNhwcArgs& a, hipStream_t stream) {
  if (!Stem7Enabled()) return false;
  Stem7Params p;
  if (!FillParams(a, &p)) return false;
  if (a.type.code == cinn_type_bfloat) {
    a.pool_after ? Launch<__bf16, true>(p, stream) : Launch<__bf16, false>(p, stream);
  } else {
    a.pool_after ? Launch<_Float16, true>(p, stream) : Launch<_Float16, false>(p, stream);
  }
  CINN_HIP_CALL(hipGetLastError());
  return true;
}

}  // namespace cinn_hip_kernels
