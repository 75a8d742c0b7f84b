// Channels-last implicit-GEMM convolution for CDNA4 (gfx950) on the MFMA units.
//
//   y[pixel][oc] = epilogue( sum_k  im2col(x)[pixel][k] * w[oc][k] )        pixel = (n, oh, ow), k = (dy, dx, c)
//
// With NHWC activations and [OC][KH][KW][IC] weights both GEMM operands have the reduction index contiguous in
// memory, so every lane moves 16-byte chunks: a chunk of the im2col operand is 8 (fp16 / bf16) or 4 (fp32)
// consecutive channels of one input pixel, present or - outside the image - zero.  Nothing is gathered element
// by element and no im2col buffer exists.
//
//   * block tile BM pixels x BN output channels: 64x64 by default (short-K, small-grid layers are bound by load
//     latency, which the number of resident blocks hides; 128x128 and 128x64 are selectable), 256 threads = 4
//     wavefronts in a 2x2 grid, K step of 128 bytes per row; grids below one block per CU split K over blockIdx.y;
//   * operand tiles in LDS as [row][128 bytes], 16-byte chunks XOR-swizzled (conflict-free ds_read_b128 of MFMA
//     fragments), double buffered with the next step's global loads in flight during the MFMAs;
//   * v_mfma_f32_32x32x16_{f16,bf16} or v_mfma_f32_32x32x2_f32, fp32 accumulation;
//   * epilogue staged through LDS so that each lane writes 16 contiguous bytes of one pixel: per-channel affine
//     (folded batch norm), residual addition and relu are applied there on the fp32 accumulators;
//   * a second loader reads an NCHW input with few channels directly, k = (c, dy, dx) with dx padded to a chunk,
//     so that the image never has to be transposed or channel-padded in memory; shapes whose filter and input
//     patch fit LDS (the network's first convolution) go to the staged kernel of conv_stem_mfma.hip instead.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>
#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

#include "kernels/conv_nhwc.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = 128;  // one tile row per K step

struct Params {
  int n, h, w, c;
  int oc, kh, kw;
  int oh, ow;
  int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
  int k_total;  // reduction length as the kernel walks it
  int kwp;      // NCHW-input loader: KW rounded up to one chunk
  int pixels;   // n * oh * ow
  int relu;
  float alpha, residual_scale;
  // exact division of values below 2^31 by oh*ow, ow, c and kw: q = (n * magic) >> shift (64-bit product)
  unsigned magic_plane, shift_plane, magic_ow, shift_ow, magic_c, shift_c, magic_kw, shift_kw;
  int steps_per_split;  // K steps each blockIdx.y handles; with more than one split the kernel writes raw fp32 partial
                        // sums to the workspace and SplitReduceKernel applies the epilogue
  int splits;
  // Tail split (splits == 1): the first full_tiles tiles (a multiple of the CU count) are one block each; every tile
  // after them is tail_splits blocks of tail_steps K steps, which write fp32 partial sums [tile - full_tiles][part]
  // [BM][BN] to the workspace for TailReduceKernel.  tail_splits == 1: no tile is split.
  int full_tiles, tail_splits, tail_steps;
};

__device__ __forceinline__ int FastDiv(int n, unsigned magic, unsigned shift) {
  return (int)(((unsigned long long)(unsigned)n * magic) >> shift);
}

// byte offset of 16-byte chunk `chunk` (0..7) of row `row` inside an operand tile
__device__ __forceinline__ int TileOffset(int row, int chunk) {
  int key = (row ^ (row >> 3)) & 7;
  return row * kRowBytes + ((chunk ^ key) << 4);
}

// ---- one K step of MFMAs on a wave tile ---------------------------------------------------------------------
template <typename T, int TM, int TN>
struct WaveMma;

template <int TM, int TN>
struct WaveMma<float, TM, TN> {
  static __device__ __forceinline__ void Step(const char* a_tile, const char* b_tile, int a_row, int b_row, int lane,
                                              f32x16 (&acc)[TM][TN]) {
    const int half = lane >> 5;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      // lanes 0-31 take chunk 2q, lanes 32-63 chunk 2q+1: the two k values of v_mfma_f32_32x32x2_f32 are element e
      // of each, which permutes k identically for both operands
      f32x4 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const f32x4*>(a_tile + TileOffset(a_row + 32 * i, 2 * q + half));
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const f32x4*>(b_tile + TileOffset(b_row + 32 * j, 2 * q + half));
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
    }
  }
};

template <typename T>
struct Half16;
template <>
struct Half16<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Half16<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

template <typename T, int TM, int TN>
struct WaveMma {
  typedef typename Half16<T>::vec8 vec8;
  static __device__ __forceinline__ void Step(const char* a_tile, const char* b_tile, int a_row, int b_row, int lane,
                                              f32x16 (&acc)[TM][TN]) {
    const int half = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      vec8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const vec8*>(a_tile + TileOffset(a_row + 32 * i, 2 * kk + half));
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const vec8*>(b_tile + TileOffset(b_row + 32 * j, 2 * kk + half));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Half16<T>::mfma(a[i], b[j], acc[i][j]);
    }
  }
};

// ---- the kernel -----------------------------------------------------------------------------------------------
// FAST (channels-last loader, C a multiple of one K step, both operands below 2 GiB): a K step lies inside one filter
// tap, so the tap and its channel offset are block-uniform and advance on the scalar unit; chunks are fetched with raw
// buffer loads whose range check returns zeros for a chunk outside the image (its offset is replaced by one beyond the
// tensor) - no page of zeros, no 64-bit address arithmetic, no select per address half.  The fp32 MFMAs run on the same
// lanes as the other vector instructions (64 more of those per K step cost the fp32 kernel 17-22 %), so every vector
// instruction the loader does not execute is matrix time: 63 -> 14 per K step.
template <typename T, int BM, int BN, int WM, int WN, bool NCHW_IN, int PF, bool FAST>
__global__ void
__launch_bounds__(64 * WM * WN, (sizeof(T) == 4 && BM == 64 && BN == 64 && !NCHW_IN) ? 4 : 1)  // fp32 64x64: four blocks per CU
conv_nhwc_mfma_kernel(const T* __restrict__ x, const T* __restrict__ w, T* y, const float* __restrict__ scale,
                      const float* __restrict__ shift, const T* residual, float* __restrict__ workspace,
                      const void* __restrict__ zero_page, Params p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int E      = 16 / sizeof(T);  // elements per chunk
  constexpr int BK     = 8 * E;           // elements per K step
  constexpr int A_TILE = BM * kRowBytes;
  constexpr int STAGE  = (BM + BN) * kRowBytes;
  constexpr int THREADS = 64 * WM * WN;  // WM x WN wavefronts, each a (BM / WM) x (BN / WN) tile
  constexpr int RP     = THREADS / 8;    // tile rows one pass of the loaders covers (8 chunks per row)
  constexpr int RA     = BM / RP;        // chunks of the pixel operand per thread and step
  constexpr int RB     = BN / RP;
  constexpr int TM     = BM / (32 * WM);  // 32x32 MFMA tiles per wavefront
  constexpr int TN     = BN / (32 * WN);
  constexpr int SLD    = BN + 8;  // row pitch (floats) of the epilogue staging tile
  static_assert(RA >= 1 && RB >= 1 && TM >= 1 && TN >= 1, "tile too small for the wavefront grid");

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm   = wave / WN;
  const int wn   = wave % WN;

  // Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own L2: hand every XCD a contiguous band
  // of tiles, channel tiles fastest, so that blocks sharing a pixel panel share an L2.
  const int tiles_n = (p.oc + BN - 1) / BN;
  const int tiles   = ((p.pixels + BM - 1) / BM) * tiles_n;
  int bid           = blockIdx.x;
  int tail_part     = -1;  // >= 0: this block computes part tail_part of a split tile
  if (p.tail_splits > 1 && bid >= p.full_tiles) {
    const int c = bid - p.full_tiles;
    bid         = p.full_tiles + c / p.tail_splits;
    tail_part   = c - (bid - p.full_tiles) * p.tail_splits;
  } else {
    const int whole = p.tail_splits > 1 ? p.full_tiles : tiles;
    const int q = whole >> 3, r = whole & 7, xcd = bid & 7;
    bid = xcd * q + (xcd < r ? xcd : r) + (bid >> 3);
  }
  const int tile_id = bid;
  const int m0 = (bid / tiles_n) * BM;
  const int n0 = (bid % tiles_n) * BN;

  const int cc = tid & 7;   // chunk column this thread loads
  const int lr = tid >> 3;  // first tile row this thread loads

  // The residual operand of the epilogue is requested now, 8 channels of each output row this thread will store:
  // a layer with a short reduction (1x1 convolutions over 64 channels) would otherwise wait for it after the MFMAs,
  // a second memory latency on top of the operands' (ResNet-50's 64 -> 256 layers at batch 32: 25-31 -> 19-24 us).
  constexpr int EPI_CPR  = BN / 8;
  constexpr int EPI_ROWS = THREADS / EPI_CPR;
  constexpr int EPI_RPT  = BM / EPI_ROWS;  // output rows per thread
  struct alignas(16) Res8 { T v[8]; };
  // (not in the fp32 64x64 instance: its blocks are bound by the matrix pipe with four wavefronts per SIMD to cover a
  // late read, and its register budget goes to the grouped sums below)
  constexpr bool EARLY_RES = !(sizeof(T) == 4 && BM == 64 && BN == 64 && !NCHW_IN);
  Res8 res_pre[EARLY_RES ? EPI_RPT : 1];
  const bool prefetch_res = EARLY_RES &&
      residual != nullptr && p.splits == 1 && tail_part < 0 && (p.oc & 7) == 0 && n0 + (tid % EPI_CPR) * 8 < p.oc;
  if (prefetch_res) {
#pragma unroll
    for (int i = 0; i < EPI_RPT; ++i) {
      const int m = m0 + tid / EPI_CPR + i * EPI_ROWS;
      if (m < p.pixels)
        res_pre[i] = *reinterpret_cast<const Res8*>(residual + (int64_t)m * p.oc + n0 + (tid % EPI_CPR) * 8);
    }
  }

  // per-row state of the pixel operand
  // base: element offset of the image (NCHW loader) or of the window origin (ih0, iw0) of the row, which may lie
  // before the tensor (channels-last loader: a chunk is at base + tap offset)
  int base[RA], ih0[RA], iw0[RA];
#pragma unroll
  for (int i = 0; i < RA; ++i) {
    int m = m0 + lr + RP * i;
    if (m < p.pixels) {
      int n   = FastDiv(m, p.magic_plane, p.shift_plane);
      int rem = m - n * (p.oh * p.ow);
      int oh  = FastDiv(rem, p.magic_ow, p.shift_ow);
      int ow  = rem - oh * p.ow;
      ih0[i]  = oh * p.stride_h - p.pad_h;
      iw0[i]  = ow * p.stride_w - p.pad_w;
      base[i] = NCHW_IN ? n * p.h * p.w * p.c : ((n * p.h + ih0[i]) * p.w + iw0[i]) * p.c;
    } else {
      base[i] = 0;
      ih0[i]  = INT_MIN / 2;  // fails every bounds test
      iw0[i]  = 0;
    }
  }
  // position of this thread's chunk in the reduction: channel offset and filter tap (channels-last loader)
  const int total_steps = (p.k_total + BK - 1) / BK;
  const int my_steps    = tail_part >= 0 ? p.tail_steps : p.steps_per_split;
  const int step0       = (tail_part >= 0 ? tail_part : (int)blockIdx.y) * my_steps;
  const int step1       = step0 + my_steps < total_steps ? step0 + my_steps : total_steps;
  int ck = 0, dy = 0, dx = 0;
  static_assert(!(FAST && NCHW_IN), "the uniform-tap loader reads channels-last images");
  if (FAST) {
    // block-uniform: ck is the channel offset of the step's first chunk
    int kc  = step0 * BK;
    int tap = FastDiv(kc, p.magic_c, p.shift_c);
    ck      = kc - tap * p.c;
    dy      = FastDiv(tap, p.magic_kw, p.shift_kw);
    dx      = tap - dy * p.kw;
  } else if (!NCHW_IN) {
    int kc  = step0 * BK + cc * E;
    int tap = FastDiv(kc, p.magic_c, p.shift_c);
    ck      = kc - tap * p.c;
    dy      = FastDiv(tap, p.magic_kw, p.shift_kw);
    dx      = tap - dy * p.kw;
  }
  // rows of the filter operand this thread loads
  int wrow[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    int oc  = n0 + lr + RP * i;
    wrow[i] = oc < p.oc ? oc * p.k_total : -1;  // checked on the host: oc * k_total < 2^31
  }

  // uniform-tap loader: byte offsets of this thread's chunk of each row at tap (0, 0), channel 0 (a window origin may
  // lie before the tensor: the 32-bit sum with the tap's offset is what has to be in range), and the two buffers
  unsigned a_off[RA], b_off[RB];
  __amdgpu_buffer_rsrc_t x_rsrc, w_rsrc;
  if constexpr (FAST) {
#pragma unroll
    for (int i = 0; i < RA; ++i) a_off[i] = (unsigned)(base[i] + cc * E) * (unsigned)sizeof(T);
#pragma unroll
    for (int i = 0; i < RB; ++i)  // a filter row beyond OC stays out of range whatever is added (operands < 2 GiB)
      b_off[i] = wrow[i] >= 0 ? (unsigned)(wrow[i] + cc * E) * (unsigned)sizeof(T) : 0x80000000u;
    x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x), 0, p.n * p.h * p.w * p.c * (int)sizeof(T), 0x00020000);
    w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(w), 0, p.oc * p.k_total * (int)sizeof(T), 0x00020000);
  }

  // Register slots for the K steps in flight: the loads of step s + PF are issued while step s is computed, so a
  // block keeps PF steps of global-memory latency covered by itself (slot of step t: t % PF).
  u32x4 ra_slots[PF][RA], rb_slots[PF][RB];
  // Loads are unconditional: a chunk that lies outside the image, beyond K or beyond this block's K range is read from
  // a page of zeros instead.  Straight-line code lets the compiler count exactly how many loads may still be in flight
  // when a slot is consumed (s_waitcnt vmcnt(N)); a branch per chunk would make it wait for all of them.
  const T* zeros = static_cast<const T*>(zero_page);
  auto load_step = [&](int step, u32x4 (&ra)[RA], u32x4 (&rb)[RB]) {
    const bool live = step < step1;
    if constexpr (FAST) {
      // steps beyond this block's range fetch something in range or zeros; nothing multiplies what they bring
      const int dyo = dy * p.dil_h, dxo = dx * p.dil_w;
      const unsigned tap_bytes = (unsigned)((dyo * p.w + dxo) * p.c + ck) * (unsigned)sizeof(T);
#pragma unroll
      for (int i = 0; i < RA; ++i) {
        const bool ok = (unsigned)(ih0[i] + dyo) < (unsigned)p.h && (unsigned)(iw0[i] + dxo) < (unsigned)p.w;
        ra[i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, ok ? a_off[i] + tap_bytes : 0x80000000u, 0, 0);
      }
      const unsigned kb_bytes = (unsigned)(step * BK) * (unsigned)sizeof(T);
#pragma unroll
      for (int i = 0; i < RB; ++i) rb[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, b_off[i] + kb_bytes, 0, 0);
      ck += BK;
      if (ck == p.c) {
        ck = 0;
        if (++dx == p.kw) {
          dx = 0;
          ++dy;
        }
      }
    } else if (!NCHW_IN) {
      const bool tap_ok = live && dy < p.kh;
      const int dyo = dy * p.dil_h, dxo = dx * p.dil_w;
      const int tap_offset = (dyo * p.w + dxo) * p.c + ck;  // the same for every row of this thread
#pragma unroll
      for (int i = 0; i < RA; ++i) {
        bool ok      = tap_ok && (unsigned)(ih0[i] + dyo) < (unsigned)p.h && (unsigned)(iw0[i] + dxo) < (unsigned)p.w;
        const T* src = ok ? x + (base[i] + tap_offset) : zeros;
        ra[i]        = *reinterpret_cast<const u32x4*>(src);
      }
      const int kb     = step * BK + cc * E;
      const bool kb_ok = live && kb < p.k_total;
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        bool ok      = kb_ok && wrow[i] >= 0;
        const T* src = ok ? w + (wrow[i] + kb) : zeros;
        rb[i]        = *reinterpret_cast<const u32x4*>(src);
      }
      // advance to the next step
      ck += BK;
      while (ck >= p.c) {
        ck -= p.c;
        if (++dx == p.kw) {
          dx = 0;
          ++dy;
        }
      }
    } else {
      // k = (c, dy, dx) with dx padded to a chunk: one chunk is E neighbouring taps of one input row
      const int chunks_per_row = p.kwp / E;
      const int q              = step * 8 + cc;
      const int row_id         = q / chunks_per_row;
      const int dx0            = (q - row_id * chunks_per_row) * E;
      const int c              = row_id / p.kh;
      const int ky             = row_id - c * p.kh;
      const bool c_ok          = live && c < p.c;
#pragma unroll
      for (int i = 0; i < RA; ++i) {
        T tmp[E];
        int ih       = ih0[i] + ky * p.dil_h;
        bool row_ok  = c_ok && (unsigned)ih < (unsigned)p.h;
        const T* src = x + base[i] + (c * p.h + ih) * p.w;
#pragma unroll
        for (int e = 0; e < E; ++e) {
          int iw  = iw0[i] + (dx0 + e) * p.dil_w;
          bool ok = row_ok && dx0 + e < p.kw && (unsigned)iw < (unsigned)p.w;
          tmp[e]  = ok ? src[iw] : (T)0.0f;
        }
        __builtin_memcpy(&ra[i], tmp, 16);
      }
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        T tmp[E];
        int oc       = n0 + lr + RP * i;
        bool row_ok  = c_ok && oc < p.oc;
        const T* src = w + ((int64_t)(oc * p.c + c) * p.kh + ky) * p.kw;
#pragma unroll
        for (int e = 0; e < E; ++e) tmp[e] = (row_ok && dx0 + e < p.kw) ? src[dx0 + e] : (T)0.0f;
        __builtin_memcpy(&rb[i], tmp, 16);
      }
    }
  };
  auto store_step = [&](char* stage, const u32x4 (&ra)[RA], const u32x4 (&rb)[RB]) {
#pragma unroll
    for (int i = 0; i < RA; ++i) *reinterpret_cast<u32x4*>(stage + TileOffset(lr + RP * i, cc)) = ra[i];
#pragma unroll
    for (int i = 0; i < RB; ++i) *reinterpret_cast<u32x4*>(stage + A_TILE + TileOffset(lr + RP * i, cc)) = rb[i];
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  // A launch with a tail split: a whole tile adds its products up in the same groups of tail_steps K steps as the
  // parts of a split tile, group sums added in ascending order like TailReduceKernel adds the parts, so that a pixel's
  // result does not depend on which kind of tile it fell into (equal images at two batch positions give equal bits).
  constexpr bool GROUPED = std::is_same<T, float>::value && BM == 64 && BN == 64 && !NCHW_IN;
  f32x16 total[GROUPED ? TM : 1][GROUPED ? TN : 1];
  int until_group_end = INT_MAX;
  if constexpr (GROUPED) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) total[i][j][r] = 0.0f;
    if (p.tail_splits > 1 && tail_part < 0) until_group_end = p.tail_steps;
  }
  auto end_of_step = [&]() {
    if constexpr (GROUPED) {
      if (--until_group_end == 0) {
        // a real branch, taken once per group: as selects the compiler reads every accumulator after every K step
        asm volatile("; end of a group of K steps");
        until_group_end = p.tail_steps;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            total[i][j] += acc[i][j];
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
          }
      }
    }
  };

  static_assert(PF % 2 == 0, "the LDS stage of a step must be a compile-time function of its slot");
  const int steps = step1 - step0;
#pragma unroll
  for (int i = 0; i < PF; ++i)
    if (i == 0 || i < steps) load_step(step0 + i, ra_slots[i], rb_slots[i]);
  store_step(lds, ra_slots[0], rb_slots[0]);
  if (PF < steps) load_step(step0 + PF, ra_slots[0], rb_slots[0]);
  __syncthreads();
  const int a_row = wm * (BM / WM) + (lane & 31);
  const int b_row = wn * (BN / WN) + (lane & 31);
  int s = 0;
  // whole groups of PF steps: branch-free, every sub-step refills the slot it has just emptied
  for (; s + PF <= steps; s += PF) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      char* cur = lds + (i & 1) * STAGE;  // s is a multiple of PF, PF is even
      WaveMma<T, TM, TN>::Step(cur, cur + A_TILE, a_row, b_row, lane, acc);
      store_step(lds + ((i + 1) & 1) * STAGE, ra_slots[(i + 1) % PF], rb_slots[(i + 1) % PF]);
      load_step(step0 + s + i + 1 + PF, ra_slots[(i + 1) % PF], rb_slots[(i + 1) % PF]);
      end_of_step();
      __syncthreads();
    }
  }
  // the last steps < PF; their data is already in the slots
#pragma unroll
  for (int i = 0; i < PF - 1; ++i) {
    if (s + i < steps) {
      char* cur = lds + (i & 1) * STAGE;
      WaveMma<T, TM, TN>::Step(cur, cur + A_TILE, a_row, b_row, lane, acc);
      store_step(lds + ((i + 1) & 1) * STAGE, ra_slots[(i + 1) % PF], rb_slots[(i + 1) % PF]);
      end_of_step();
      __syncthreads();
    }
  }
  if constexpr (GROUPED) {
    if (p.tail_splits > 1 && tail_part < 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = total[i][j] + acc[i][j];  // the last group, like the last part
    }
  }

  // ---- epilogue: accumulators -> LDS (fp32) -> 8 channels of one pixel per lane ----------------------------------
  // When the whole fp32 tile does not fit the LDS of the two stages it is staged one wavefront row at a time.
  constexpr bool ONE_PASS = BM * SLD * 4 <= 2 * STAGE;
  constexpr int PASSES    = ONE_PASS ? 1 : WM;
  constexpr int PROWS     = BM / PASSES;      // tile rows staged per pass
  constexpr int CPR       = BN / 8;           // 8-channel groups per tile row
  constexpr int ROWS      = THREADS / CPR;    // rows the block stores per sweep
  float* st               = reinterpret_cast<float*>(lds);
  const int cg            = tid % CPR;
  const int oc0           = n0 + cg * 8;
  const bool active       = oc0 < p.oc;
  const bool full         = (p.oc & 7) == 0;  // then every group is whole and 16-byte aligned
  float sc[8], sh[8];
  if (active && p.splits == 1 && tail_part < 0) {
    if (full && scale && shift) {
      __builtin_memcpy(sc, scale + oc0, 32);
      __builtin_memcpy(sh, shift + oc0, 32);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        int oc = oc0 + e < p.oc ? oc0 + e : p.oc - 1;
        sc[e]  = scale ? scale[oc] : p.alpha;
        sh[e]  = shift ? shift[oc] : 0.0f;
      }
    }
  }
  float* ws = workspace + (int64_t)blockIdx.y * p.pixels * p.oc;  // split-K: fp32 partial sums [split][pixel][oc]
  // tail split: this block's [BM][BN] slice
  float* tail_ws = workspace + ((int64_t)(tile_id - p.full_tiles) * p.tail_splits + tail_part) * (BM * BN);
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    if (pass > 0) __syncthreads();  // the previous pass has been read
    if (ONE_PASS || wm == pass) {
      const int row_base = ONE_PASS ? wm * (BM / WM) : 0;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            int row = row_base + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            int col = wn * (BN / WN) + j * 32 + (lane & 31);
            st[row * SLD + col] = acc[i][j][r];
          }
    }
    __syncthreads();
    if (!active) continue;
    static_assert(PROWS % ROWS == 0 && CPR == EPI_CPR && ROWS == EPI_ROWS, "rows per thread are whole");
#pragma unroll
    for (int it = 0; it < PROWS / ROWS; ++it) {
      const int row = tid / CPR + it * ROWS;
      const int m   = m0 + pass * PROWS + row;
      if (m >= p.pixels) break;
      float v[8];
      *reinterpret_cast<f32x4*>(&v[0]) = *reinterpret_cast<const f32x4*>(&st[row * SLD + cg * 8]);
      *reinterpret_cast<f32x4*>(&v[4]) = *reinterpret_cast<const f32x4*>(&st[row * SLD + cg * 8 + 4]);
      if (tail_part >= 0) {
        float* dst = tail_ws + (pass * PROWS + row) * BN + cg * 8;
        *reinterpret_cast<f32x4*>(dst)     = *reinterpret_cast<const f32x4*>(&v[0]);
        *reinterpret_cast<f32x4*>(dst + 4) = *reinterpret_cast<const f32x4*>(&v[4]);
        continue;
      }
      const int64_t off = (int64_t)m * p.oc + oc0;
      if (p.splits > 1) {
        if (full) {
          *reinterpret_cast<f32x4*>(ws + off)     = *reinterpret_cast<const f32x4*>(&v[0]);
          *reinterpret_cast<f32x4*>(ws + off + 4) = *reinterpret_cast<const f32x4*>(&v[4]);
        } else {
          for (int e = 0; e < 8 && oc0 + e < p.oc; ++e) ws[off + e] = v[e];
        }
        continue;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(v[e], sc[e], sh[e]);
      if (full) {
        T out[8];
        if (residual) {
          // requested at the start of the kernel, or read here
          const Res8 rv = EARLY_RES ? res_pre[EARLY_RES ? pass * (PROWS / ROWS) + it : 0] : *reinterpret_cast<const Res8*>(residual + off);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(p.residual_scale, (float)rv.v[e], v[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (T)(p.relu ? fmaxf(v[e], 0.0f) : v[e]);
        __builtin_memcpy(y + off, out, 8 * sizeof(T));
      } else {
        for (int e = 0; e < 8 && oc0 + e < p.oc; ++e) {
          float t = v[e];
          if (residual) t = __builtin_fmaf(p.residual_scale, (float)residual[off + e], t);
          y[off + e] = (T)(p.relu ? fmaxf(t, 0.0f) : t);
        }
      }
    }
  }
}

// Sums the partial results of a split-K convolution and applies the epilogue: one thread per output element group of
// 4 channels (oc % 4 == 0) or per element.
template <typename T, int V>
__global__ void __launch_bounds__(256)
SplitReduceKernel(const float* __restrict__ workspace, T* y, const float* __restrict__ scale, const float* __restrict__ shift,
                  const T* residual, Params p) {
  const int64_t total = (int64_t)p.pixels * p.oc / V;
  const int64_t idx   = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t off = idx * V;
  const int oc0     = (int)(off % p.oc);
  float v[V];
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = 0.0f;
  for (int sp = 0; sp < p.splits; ++sp) {
    float part[V];
    __builtin_memcpy(part, workspace + (int64_t)sp * p.pixels * p.oc + off, V * sizeof(float));
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] += part[e];
  }
  T rv[V], out[V];
  if (residual) __builtin_memcpy(rv, residual + off, V * sizeof(T));
#pragma unroll
  for (int e = 0; e < V; ++e) {
    float t = v[e] * (scale ? scale[oc0 + e] : p.alpha) + (shift ? shift[oc0 + e] : 0.0f);
    if (residual) t += p.residual_scale * (float)rv[e];
    out[e] = (T)(p.relu ? fmaxf(t, 0.0f) : t);
  }
  __builtin_memcpy(y + off, out, V * sizeof(T));
}

// Sums the parts of the split tiles behind the first full_tiles tiles and applies the epilogue: one thread per 4
// channels of one pixel of one split tile.
template <typename T, int BM, int BN>
__global__ void __launch_bounds__(256)
TailReduceKernel(const float* __restrict__ workspace, T* y, const float* __restrict__ scale, const float* __restrict__ shift,
                 const T* residual, Params p) {
  constexpr int PER_TILE = BM * BN / 4;
  const int idx     = blockIdx.x * 256 + threadIdx.x;
  const int tile    = idx / PER_TILE;  // among the split tiles
  const int e       = idx - tile * PER_TILE;
  const int row     = e / (BN / 4);
  const int col     = (e - row * (BN / 4)) * 4;
  const int tiles_n = (p.oc + BN - 1) / BN;
  const int t       = p.full_tiles + tile;
  const int m       = (t / tiles_n) * BM + row;
  const int oc0     = (t % tiles_n) * BN + col;
  if (m >= p.pixels || oc0 >= p.oc) return;
  f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
  const float* src = workspace + (int64_t)tile * p.tail_splits * (BM * BN) + row * BN + col;
  for (int part = 0; part < p.tail_splits; ++part) v += *reinterpret_cast<const f32x4*>(src + (int64_t)part * (BM * BN));
  const int64_t off = (int64_t)m * p.oc + oc0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (oc0 + k >= p.oc) break;
    float r = __builtin_fmaf(v[k], scale ? scale[oc0 + k] : p.alpha, shift ? shift[oc0 + k] : 0.0f);
    if (residual) r = __builtin_fmaf(p.residual_scale, (float)residual[off + k], r);
    y[off + k] = (T)(p.relu ? fmaxf(r, 0.0f) : r);
  }
}

// ---- host side ------------------------------------------------------------------------------------------------
struct TileChoice {
  int bm, bn, waves;
};

// two operand stages; the epilogue stages the fp32 tile in the same memory, whole if it fits, else one wavefront row
// (bm / wm rows) at a time
int LdsBytes(int bm, int bn, int wm) {
  int stages  = 2 * (bm + bn) * kRowBytes;
  int whole   = bm * (bn + 8) * 4;
  if (whole <= stages) return stages;
  int staging = (bm / wm) * (bn + 8) * 4;
  return stages > staging ? stages : staging;
}

// Block tile.  Measured over the ResNet-50 layer shapes at batch 32, the 64x64 tile is the fastest or within a few per
// cent of the fastest everywhere: the kernel prefetches one K step ahead, so what hides the load latency is the number
// of blocks resident on a CU, and the small tile (32 KiB of LDS) allows five.  The larger tiles stay selectable for
// experiments (FLAGS_cinn_hip_conv_tile = 0: 128x128, 1: 128x64, 2: 64x64).
TileChoice ChooseTile(int pixels, int oc) {
  static const int forced = [] {
    const char* e = getenv("FLAGS_cinn_hip_conv_tile");
    return e ? atoi(e) : -1;
  }();
  const TileChoice options[4] = {{128, 128, 4}, {128, 64, 4}, {64, 64, 4}, {128, 128, 8}};
  if (forced >= 0 && forced < 4) return options[forced];
  (void)pixels;
  (void)oc;
  return options[2];
}

// K splits: layers whose tile grid cannot fill the 256 CUs spend their time waiting for one block's serial chain of
// loads; splitting the reduction puts several blocks of the same tile on different CUs
int ChooseSplits(int tiles, int steps, bool fp32, size_t bytes_per_split, size_t cap) {
  static const int forced = [] {
    const char* e = getenv("FLAGS_cinn_hip_conv_splits");
    return e ? atoi(e) : 0;
  }();
  if (forced > 0) return forced < steps ? forced : steps;
  static const bool balance = [] {  // FLAGS_cinn_hip_conv_split_balance=0: the powers of two below for fp32 as well
    const char* e = getenv("FLAGS_cinn_hip_conv_split_balance");
    return !(e && e[0] == '0');
  }();
  if (fp32 && balance && tiles < 256) {
    // fp32 blocks are bound by the matrix pipe, which the blocks of a CU share: the launch takes as long as the CU
    // with the most parts, ceil(tiles * s / 256) / s of a whole tile - 200 tiles: four ways 1.0, five ways 0.8.  Every
    // part keeps at least 8 K steps; 0.02 per part stands for the partial sums it writes and the reduction reads.
    int best = 1;
    double best_cost = 1.0;
    for (int s = 2; s <= 8 && steps / s >= 8; ++s) {
      if (cap != 0 && (size_t)s * bytes_per_split > cap) break;
      const double cost = (double)((tiles * s + 255) / 256) / s + 0.02 * s;
      if (cost < best_cost - 1e-9) best_cost = cost, best = s;
    }
    return best;
  }
  // only grids that leave CUs without a single block are split, and every part keeps at least 8 K steps
  int splits = 1;
  if (tiles >= 256) return 1;
  while (tiles * splits < 640 && steps / (splits * 2) >= 8 && splits < 8) splits *= 2;
  return splits;
}

// Where a launch takes its scratch from: the library's per-stream arena (the default), or a caller-fixed region that
// must be large enough (the entry point that allocates nothing).
struct ScratchSource {
  float* fixed_partials{nullptr};   // null: the arena
  size_t fixed_partials_bytes{0};
  const void* zero_page{nullptr};   // null: the arena's page
  bool status_only{false};          // failed runtime calls are reported and returned instead of aborting
};

// split count and K steps per split of one launch
// cap: bytes the partial sums may take (0: no limit; the entry point that allocates nothing has a fixed region)
void PlanSplits(Params* p, int bm, int bn, int elem_bytes, size_t cap = 0) {
  const int bk    = 128 / elem_bytes;
  const int tiles = ((p->pixels + bm - 1) / bm) * ((p->oc + bn - 1) / bn);
  const int steps = (p->k_total + bk - 1) / bk;
  p->splits          = ChooseSplits(tiles, steps, elem_bytes == 4, (size_t)p->pixels * p->oc * sizeof(float), cap);
  p->steps_per_split = (steps + p->splits - 1) / p->splits;
  p->splits          = (steps + p->steps_per_split - 1) / p->steps_per_split;
  p->full_tiles      = tiles;
  p->tail_splits     = 1;
  p->tail_steps      = steps;
}

// Tail split of an fp32 launch.  Its blocks are bound by the matrix pipe, a CU holds four of them and runs them at a
// quarter of the speed each, so a launch takes as long as the CU with the most tiles: 784 tiles on 256 CUs take the
// time of 4 per CU although the average is 3.06.  The tiles beyond the last multiple of the CU count are therefore
// cut along K into parts small enough to spread evenly, and their partial sums go through the workspace (a fraction
// of what a split of the whole grid moves).  Returns the bytes of workspace needed, 0 when no tile is split.
// FLAGS_cinn_hip_conv_tail_split=0 switches it off.
size_t PlanTailSplit(Params* p, int bm, int bn, int elem_bytes) {
  static const bool enabled = [] {
    const char* e = getenv("FLAGS_cinn_hip_conv_tail_split");
    return !(e && e[0] == '0');
  }();
  constexpr int kCus = 256;
  const int bk    = 128 / elem_bytes;
  const int tiles = ((p->pixels + bm - 1) / bm) * ((p->oc + bn - 1) / bn);
  const int steps = (p->k_total + bk - 1) / bk;
  if (!enabled || p->splits != 1 || tiles < kCus) return 0;
  const int full = tiles / kCus * kCus, rest = tiles - full;
  if (rest == 0) return 0;
  // time of the remainder in units of one tile on a CU of its own: ceil(rest * parts / CUs) / parts
  double best = 1.0;
  int best_parts = 1;
  for (int parts = 2; parts <= 16; parts *= 2) {
    const int part_steps = (steps + parts - 1) / parts;
    if (part_steps < 2) break;
    const int real_parts = (steps + part_steps - 1) / part_steps;
    if ((size_t)rest * real_parts * bm * bn * sizeof(float) > ((size_t)24 << 20)) break;
    const double t = (double)((rest * real_parts + kCus - 1) / kCus) / real_parts;
    if (t < best - 1e-9) best = t, best_parts = real_parts;
  }
  // Worth a second launch (4-6 us) only when it saves more than that: a tile on a CU of its own takes about half a
  // microsecond per K step (16 MFMAs of 64 clocks), so the remainder gets (1 - best) * steps / 2 us shorter.
  if (best_parts == 1 || (1.0 - best) * steps < 20.0) return 0;
  p->full_tiles  = full;
  p->tail_steps  = (steps + best_parts - 1) / best_parts;
  p->tail_splits = (steps + p->tail_steps - 1) / p->tail_steps;
  return (size_t)rest * p->tail_splits * bm * bn * sizeof(float);
}

// Raises the dynamic LDS limit of one kernel instantiation, once per instantiation and process (a failed attempt is
// tried again by the next call).  cinn_hip_conv2d_forward_noalloc_init walks every instantiation ahead of time, so
// that a first call under capture does nothing but launch (this runtime accepts the attribute call during a capture;
// what it refuses there is allocating or clearing memory).
template <typename T, int BM, int BN, int WM, int WN, bool NCHW_IN, int PF = 2, bool FAST = false>
hipError_t Configure() {
  static std::atomic<bool> done{false};
  if (done.load(std::memory_order_acquire)) return hipSuccess;
  const hipError_t status = hipFuncSetAttribute(
      reinterpret_cast<const void*>(conv_nhwc_mfma_kernel<T, BM, BN, WM, WN, NCHW_IN, PF, FAST>),
      hipFuncAttributeMaxDynamicSharedMemorySize, LdsBytes(BM, BN, WM));
  if (status == hipSuccess) done.store(true, std::memory_order_release);
  return status;
}

// A failed runtime call: the allocating entry points abort with the message (the reference's CUDA_CALL), the entry
// point that allocates nothing reports and returns a status.
int LaunchFailed(const ScratchSource& src, hipError_t err, const char* what) {
  if (!src.status_only) CINN_RT_CHECK(false, "conv2d (channels-last): %s: %s", what, hipGetErrorString(err));
  fprintf(stderr, "cinn_call_hip_conv2d_forward_noalloc: %s: %s\n", what, hipGetErrorString(err));
  return 1;
}

template <typename T, int BM, int BN, int WM, int WN, bool NCHW_IN, int PF = 2, bool FAST = false>
int Launch(const ConvNhwcArgs& a, const Params& p_in, hipStream_t stream, const ScratchSource& src) {
  // PF: K steps in flight per block
  auto kernel      = conv_nhwc_mfma_kernel<T, BM, BN, WM, WN, NCHW_IN, PF, FAST>;
  const int bytes  = LdsBytes(BM, BN, WM);
  if (hipError_t err = Configure<T, BM, BN, WM, WN, NCHW_IN, PF, FAST>(); err != hipSuccess)
    return LaunchFailed(src, err, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
  Params p = p_in;
  PlanSplits(&p, BM, BN, sizeof(T), src.fixed_partials ? src.fixed_partials_bytes : 0);
  const int tiles  = ((p.pixels + BM - 1) / BM) * ((p.oc + BN - 1) / BN);
  float* workspace = nullptr;
  int blocks       = tiles;
  if constexpr (std::is_same<T, float>::value && BM == 64 && BN == 64 && !NCHW_IN) {
    if (const size_t need = PlanTailSplit(&p, BM, BN, sizeof(T)); need > 0) {
      if (src.fixed_partials && need > src.fixed_partials_bytes) {
        p.full_tiles = tiles, p.tail_splits = 1;  // the fixed scratch is too small: every tile stays whole
      } else {
        workspace = src.fixed_partials ? src.fixed_partials : static_cast<float*>(Scratch(ScratchKind::kSplitK, need, stream));
        blocks    = p.full_tiles + (tiles - p.full_tiles) * p.tail_splits;
      }
    }
  }
  // fp32 partial sums [split][pixel][oc]
  if (p.splits > 1) {
    const size_t need = (size_t)p.splits * p.pixels * p.oc * sizeof(float);
    if (src.fixed_partials) {
      if (need > src.fixed_partials_bytes) return LaunchFailed(src, hipErrorOutOfMemory, "partial sums do not fit the fixed scratch");
      workspace = src.fixed_partials;
    } else {
      workspace = static_cast<float*>(Scratch(ScratchKind::kSplitK, need, stream));
    }
  }
  hipLaunchKernelGGL(kernel, dim3(blocks, p.splits), dim3(64 * WM * WN), bytes, stream, static_cast<const T*>(a.x),
                     static_cast<const T*>(a.w), static_cast<T*>(a.y), a.scale, a.shift, static_cast<const T*>(a.residual),
                     workspace, FAST ? nullptr : (src.zero_page ? src.zero_page : ZeroPage()), p);  // FAST reads no page of zeros
  if (hipError_t err = hipGetLastError(); err != hipSuccess) return LaunchFailed(src, err, "kernel launch");
  if (p.tail_splits > 1) {
    const int threads = (tiles - p.full_tiles) * (BM * BN / 4);
    hipLaunchKernelGGL((TailReduceKernel<T, BM, BN>), dim3((unsigned)(threads / 256)), dim3(256), 0, stream, workspace,
                       static_cast<T*>(a.y), a.scale, a.shift, static_cast<const T*>(a.residual), p);
    if (hipError_t err = hipGetLastError(); err != hipSuccess) return LaunchFailed(src, err, "launch of the tail reduction");
  }
  if (p.splits > 1) {
    if (p.oc % 4 == 0) {
      const int64_t total = (int64_t)p.pixels * p.oc / 4;
      hipLaunchKernelGGL((SplitReduceKernel<T, 4>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, workspace,
                         static_cast<T*>(a.y), a.scale, a.shift, static_cast<const T*>(a.residual), p);
    } else {
      const int64_t total = (int64_t)p.pixels * p.oc;
      hipLaunchKernelGGL((SplitReduceKernel<T, 1>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, workspace,
                         static_cast<T*>(a.y), a.scale, a.shift, static_cast<const T*>(a.residual), p);
    }
    if (hipError_t err = hipGetLastError(); err != hipSuccess) return LaunchFailed(src, err, "launch of the split reduction");
  }
  return 0;
}

// block tile and wavefront grid of a launch: {BM, BN, WM, WN}
struct TileShape {
  int bm, bn, wm, wn;
};
TileShape TileFor(const ConvNhwcArgs& a, const Params& p) {
  TileChoice t = ChooseTile(p.pixels, p.oc);
  if (a.nchw_input) return t.bm == 128 ? TileShape{128, 64, 2, 2} : TileShape{64, 64, 2, 2};
  if (t.bm == 128 && t.bn == 128 && t.waves == 8) return {128, 128, 2, 4};
  if (t.bm == 128 && t.bn == 128) return {128, 128, 2, 2};
  if (t.bm == 128) return {128, 64, 2, 2};
  return {64, 64, 2, 2};
}

// The uniform-tap loader takes channels-last layers whose channel count is a multiple of one K step (128 bytes) and
// whose operands stay below 2 GiB (32-bit byte offsets; an offset with the top bit set is its "out of range").
// FLAGS_cinn_hip_conv_uniform_tap=0 keeps every layer on the per-lane loader.
template <typename T>
bool UniformTap(const ConvNhwcArgs& a, const Params& p) {
  static const bool enabled = [] {
    const char* e = getenv("FLAGS_cinn_hip_conv_uniform_tap");
    return !(e && e[0] == '0');
  }();
  constexpr int64_t kLimit = ((int64_t)1 << 31) - 4096;  // the steps requested beyond the last stay below 2^32
  const int bk = kRowBytes / (int)sizeof(T);
  return enabled && !a.nchw_input && a.c % bk == 0 && (int64_t)a.n * a.h * a.w_in * a.c * (int64_t)sizeof(T) < kLimit &&
         (int64_t)a.oc * p.k_total * (int64_t)sizeof(T) < kLimit;
}

template <typename T>
int Dispatch(const ConvNhwcArgs& a, const Params& p, hipStream_t stream, const ScratchSource& src = ScratchSource()) {
  const TileShape t = TileFor(a, p);
  if (a.nchw_input) {
    if (t.bm == 128) return Launch<T, 128, 64, 2, 2, true>(a, p, stream, src);
    return Launch<T, 64, 64, 2, 2, true>(a, p, stream, src);
  }
  if (UniformTap<T>(a, p)) {
    if (t.bm == 128 && t.bn == 128 && t.wn == 4) return Launch<T, 128, 128, 2, 4, false, 2, true>(a, p, stream, src);
    if (t.bm == 128 && t.bn == 128) return Launch<T, 128, 128, 2, 2, false, 2, true>(a, p, stream, src);
    if (t.bm == 128) return Launch<T, 128, 64, 2, 2, false, 2, true>(a, p, stream, src);
    return Launch<T, 64, 64, 2, 2, false, 2, true>(a, p, stream, src);
  }
  if (t.bm == 128 && t.bn == 128 && t.wn == 4) return Launch<T, 128, 128, 2, 4, false>(a, p, stream, src);
  if (t.bm == 128 && t.bn == 128) return Launch<T, 128, 128, 2, 2, false>(a, p, stream, src);
  if (t.bm == 128) return Launch<T, 128, 64, 2, 2, false>(a, p, stream, src);
  return Launch<T, 64, 64, 2, 2, false>(a, p, stream, src);
}

// every instantiation Dispatch<T> can reach
template <typename T>
hipError_t ConfigureAll() {
  const hipError_t all[10] = {Configure<T, 128, 64, 2, 2, true>(),
                              Configure<T, 64, 64, 2, 2, true>(),
                              Configure<T, 128, 128, 2, 4, false>(),
                              Configure<T, 128, 128, 2, 2, false>(),
                              Configure<T, 128, 64, 2, 2, false>(),
                              Configure<T, 64, 64, 2, 2, false>(),
                              Configure<T, 128, 128, 2, 4, false, 2, true>(),
                              Configure<T, 128, 128, 2, 2, false, 2, true>(),
                              Configure<T, 128, 64, 2, 2, false, 2, true>(),
                              Configure<T, 64, 64, 2, 2, false, 2, true>()};
  for (hipError_t e : all)
    if (e != hipSuccess) return e;
  return hipSuccess;
}

int ChunkElems(const cinn_type_t& t) { return 16 / (t.bits / CHAR_BIT); }

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

// kernel parameters of one convolution (shapes, magic numbers of the index divisions)
Params MakeParams(const ConvNhwcArgs& a) {
  Params p;
  p.n = a.n, p.h = a.h, p.w = a.w_in, p.c = a.c;
  p.oc = a.oc, p.kh = a.kh, p.kw = a.kw;
  p.oh = a.oh, p.ow = a.ow;
  p.pad_h = a.pad_h, p.pad_w = a.pad_w, p.stride_h = a.stride_h, p.stride_w = a.stride_w;
  p.dil_h = a.dil_h, p.dil_w = a.dil_w;
  const int e = ChunkElems(a.type);
  p.kwp       = (a.kw + e - 1) / e * e;
  p.k_total   = a.nchw_input ? a.c * a.kh * p.kwp : a.kh * a.kw * a.c;
  p.pixels    = a.n * a.oh * a.ow;
  p.relu      = a.relu ? 1 : 0;
  p.alpha     = a.alpha;
  p.residual_scale = a.residual_scale;
  MagicFor(a.oh * a.ow, &p.magic_plane, &p.shift_plane);
  MagicFor(a.ow, &p.magic_ow, &p.shift_ow);
  MagicFor(a.c, &p.magic_c, &p.shift_c);
  MagicFor(a.kw, &p.magic_kw, &p.shift_kw);
  CINN_RT_CHECK((int64_t)a.oc * p.k_total < INT_MAX, "conv2d (channels-last): filter too large for 32-bit offsets");
  return p;
}

}  // namespace

bool ConvNhwcSupported(const ConvNhwcArgs& a) {
  const bool is_float = a.type.code == cinn_type_float && (a.type.bits == 32 || a.type.bits == 16);
  const bool is_bf16  = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if (!is_float && !is_bf16) return false;
  if (a.nchw_input) return true;
  return a.c % ChunkElems(a.type) == 0;
}

void RunConvNhwc(const ConvNhwcArgs& a, hipStream_t stream) {
  CINN_RT_CHECK(ConvNhwcSupported(a), "conv2d (channels-last): unsupported type or channel count %d", a.c);
  CINN_RT_CHECK((int64_t)a.n * a.h * a.w_in * a.c < INT_MAX && (int64_t)a.n * a.oh * a.ow * a.oc < INT_MAX,
                "conv2d (channels-last): tensor too large for 32-bit offsets");
  if (a.x2 != nullptr) {
    CINN_RT_CHECK(TryPointwiseConvAsGemm(a, stream),
                  "conv2d (channels-last): no kernel takes a second input for this shape (%d pixels, %d + %d -> %d channels)",
                  a.n * a.oh * a.ow, a.kh * a.kw * a.c, a.c2, a.oc);
    return;
  }
  if (TryConvStem7(a, stream)) return;
  CINN_RT_CHECK(!a.pool_after, "conv2d: only the 7x7 / stride 2 image convolution in a 16-bit type takes a fused max pooling");
  if (ConvStemSupported(a)) {
    RunConvStem(a, stream);
    return;
  }
  if (TryConvPatch(a, stream)) return;
  if (TryPointwiseConvAsGemm(a, stream)) return;
  const Params p = MakeParams(a);
  if (a.type.code == cinn_type_bfloat) {
    Dispatch<__bf16>(a, p, stream);
  } else if (a.type.bits == 16) {
    Dispatch<_Float16>(a, p, stream);
  } else {
    Dispatch<float>(a, p, stream);
  }
}

}  // namespace cinn_hip_kernels

// ---- the entry point that allocates nothing -------------------------------------------------------------------
// cinn_call_hip_conv2d_forward_noalloc: cinn_call_cudnn_conv2d_forward for callers that cannot call hipMalloc (code
// under graph capture, tight serving loops).  Its scratch - the page of zeros that masked-out chunks are read from and
// the fp32 partial sums of a split reduction - lives in this file-scope device array instead of the library's arena.
// Every GPU the library runs on holds its own copy, at its own address, until the process ends; the host-side name
// `scratch` is only a handle for hipGetSymbolAddress, never a device address.
namespace {

constexpr size_t kNoAllocZeroBytes     = 256;                 // never written by any kernel: stays zero
constexpr size_t kNoAllocPartialsBytes = (size_t)16 << 20;    // split-K partial sums, rewritten by every call
static __device__ __align__(256) unsigned char scratch[kNoAllocZeroBytes + kNoAllocPartialsBytes];

constexpr int kNoAllocMaxDevices = 64;
std::mutex g_noalloc_mu;
unsigned char* g_noalloc_ptr[kNoAllocMaxDevices];  // device address of `scratch` on each device, once looked up

// device address of this device's copy of `scratch`; 0 = ok
int NoAllocScratch(unsigned char** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kNoAllocMaxDevices) {
    fprintf(stderr, "cinn_call_hip_conv2d_forward_noalloc: no current device (or more than %d devices)\n", kNoAllocMaxDevices);
    return 1;
  }
  std::lock_guard<std::mutex> lock(g_noalloc_mu);
  if (!g_noalloc_ptr[device]) {
    void* ptr      = nullptr;
    hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr) {
      fprintf(stderr, "cinn_call_hip_conv2d_forward_noalloc: hipGetSymbolAddress(scratch) failed on device %d: %s\n", device,
              hipGetErrorString(err));
      return 1;
    }
    g_noalloc_ptr[device] = static_cast<unsigned char*>(ptr);
  }
  *out = g_noalloc_ptr[device];
  return 0;
}

}  // namespace

extern "C" {

size_t cinn_hip_conv2d_forward_noalloc_scratch_limit(void) { return kNoAllocPartialsBytes; }

int cinn_hip_conv2d_forward_noalloc_init(void) {
  using namespace cinn_hip_kernels;
  unsigned char* base = nullptr;
  if (NoAllocScratch(&base) != 0) return 1;
  // the LDS limit of every kernel the entry point can launch, so that a call under capture only launches
  for (hipError_t e : {ConfigureAll<float>(), ConfigureAll<_Float16>(), ConfigureAll<__bf16>()}) {
    if (e != hipSuccess) {
      fprintf(stderr, "cinn_hip_conv2d_forward_noalloc_init: hipFuncSetAttribute failed: %s\n", hipGetErrorString(e));
      return 1;
    }
  }
  return 0;
}

int cinn_call_hip_conv2d_forward_noalloc(void* v_args, int num_args, int format, float alpha, float beta, int input_n,
                                         int input_c, int input_h, int input_w, int filter_n, int filter_c, int filter_h,
                                         int filter_w, int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h,
                                         int dilation_w, int groups, int output_n, int output_c, int output_h,
                                         int output_w, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  using namespace cinn_hip_kernels;
  const char* const me = "cinn_call_hip_conv2d_forward_noalloc";
#define CINN_NOALLOC_REJECT(code, ...)  \
  do {                                  \
    fprintf(stderr, "%s: ", me);        \
    fprintf(stderr, __VA_ARGS__);       \
    fprintf(stderr, "\n");              \
    return code;                        \
  } while (0)
  if (num_args != 3 || !v_args) CINN_NOALLOC_REJECT(1, "takes x, w and y, got %d arguments", num_args);
  auto* pods = static_cast<cinn_pod_value_t*>(v_args);
  cinn_buffer_t* bufs[3];
  for (int i = 0; i < 3; ++i) {
    if (pods[i].type_code_ != CINN_POD_BUFFER_P || !pods[i].value_.v_handle) CINN_NOALLOC_REJECT(1, "argument %d is not a buffer", i);
    bufs[i] = static_cast<cinn_buffer_t*>(pods[i].value_.v_handle);
    if (!bufs[i]->memory) CINN_NOALLOC_REJECT(1, "argument %d has no device memory", i);
  }
  if (format != 1 && format != 2)
    CINN_NOALLOC_REJECT(1, "format %d: only channels-last outputs (1, or 2 with an NCHW input) run without allocation", format);
  if (groups != 1) CINN_NOALLOC_REJECT(1, "groups = %d: only ungrouped convolutions", groups);
  if (filter_c != input_c || output_n != input_n || output_c != filter_n)
    CINN_NOALLOC_REJECT(1, "inconsistent extents (filter channels %d vs %d, output [%d,%d] vs [%d,%d])", filter_c, input_c,
                        output_n, output_c, input_n, filter_n);
  if (stride_h <= 0 || stride_w <= 0 || dilation_h <= 0 || dilation_w <= 0)
    CINN_NOALLOC_REJECT(1, "strides and dilations must be positive");
  const int want_oh = (input_h - ((filter_h - 1) * dilation_h + 1) + 2 * pad_h) / stride_h + 1;
  const int want_ow = (input_w - ((filter_w - 1) * dilation_w + 1) + 2 * pad_w) / stride_w + 1;
  if (output_h != want_oh || output_w != want_ow || want_oh <= 0 || want_ow <= 0)
    CINN_NOALLOC_REJECT(1, "output is %dx%d, the shapes give %dx%d", output_h, output_w, want_oh, want_ow);
  if ((int64_t)input_n * input_c * input_h * input_w >= INT_MAX || (int64_t)output_n * output_c * output_h * output_w >= INT_MAX ||
      (int64_t)filter_n * filter_c * filter_h * filter_w * 8 >= INT_MAX)
    CINN_NOALLOC_REJECT(1, "tensor too large for 32-bit offsets");
  ConvNhwcArgs a;
  a.x = bufs[0]->memory, a.w = bufs[1]->memory, a.y = bufs[2]->memory;
  a.scale = a.shift = nullptr;
  a.residual        = beta != 0.0f ? bufs[2]->memory : nullptr;
  a.alpha           = alpha;
  a.residual_scale  = beta;
  a.relu            = false;
  a.nchw_input      = format == 2;
  a.n = input_n, a.h = input_h, a.w_in = input_w, a.c = input_c;
  a.oc = filter_n, a.kh = filter_h, a.kw = filter_w, a.oh = output_h, a.ow = output_w;
  a.pad_h = pad_h, a.pad_w = pad_w, a.stride_h = stride_h, a.stride_w = stride_w, a.dil_h = dilation_h, a.dil_w = dilation_w;
  a.type = bufs[0]->type;
  if (!ConvNhwcSupported(a))
    CINN_NOALLOC_REJECT(1, "unsupported element type (code %d, %d bits) or %d input channels are not whole 16-byte chunks",
                        a.type.code, a.type.bits, input_c);
  // the size check comes before any launch: the partial sums of the split this shape gets must fit
  Params p          = MakeParams(a);
  const TileShape t = TileFor(a, p);
  PlanSplits(&p, t.bm, t.bn, a.type.bits / CHAR_BIT, kNoAllocPartialsBytes);
  const size_t need = p.splits > 1 ? (size_t)p.splits * p.pixels * p.oc * sizeof(float) : 0;
  if (need > kNoAllocPartialsBytes)
    CINN_NOALLOC_REJECT(2, "this shape splits its reduction %d ways and needs %zu bytes of partial sums; the static scratch holds %zu",
                        p.splits, need, kNoAllocPartialsBytes);
#undef CINN_NOALLOC_REJECT
  unsigned char* base = nullptr;
  if (NoAllocScratch(&base) != 0) return 1;
  ScratchSource src;
  src.zero_page            = base;
  src.fixed_partials       = reinterpret_cast<float*>(base + kNoAllocZeroBytes);
  src.fixed_partials_bytes = kNoAllocPartialsBytes;
  src.status_only          = true;
  const Params fresh = MakeParams(a);  // Launch plans the split itself, identically
  if (a.type.code == cinn_type_bfloat) return Dispatch<__bf16>(a, fresh, static_cast<hipStream_t>(stream), src);
  if (a.type.bits == 16) return Dispatch<_Float16>(a, fresh, static_cast<hipStream_t>(stream), src);
  return Dispatch<float>(a, fresh, static_cast<hipStream_t>(stream), src);
}

}  // extern "C"
