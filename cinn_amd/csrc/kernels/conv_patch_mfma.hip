// 3x3, stride 1, padding 1 convolutions over 64 input channels on channels-last 16-bit tensors, with the input patch
// of a block resident in LDS.
//
// The implicit-GEMM kernels fetch the im2col operand of a tile tap by tap: every input pixel travels from L2 to LDS
// nine times, and with 64 output channels per block that traffic (42-45 bytes per clock and CU is what the
// direct-to-LDS path delivers) bounds the K loop.  Here a block owns a band of output rows of ONE image and keeps the
// input rows that band needs in LDS for the whole kernel, loaded once; a filter tap is then nothing but a constant
// added to the LDS address, and only the filter (9 stages of 64 x 64) streams through a ring while the K loop runs.
//   * Patch layout: [rows + 2][W + 2] positions with the zero halo stored (lanes that would fetch a pixel outside the
//     image fetch from a page of zeros instead), so the K loop needs no masks.  A position holds its 64 channels in
//     128 bytes and is 160 bytes apart from the next: with that pitch the sixteen lanes LDS serves together on a
//     16-byte fragment read (eight consecutive positions, two neighbouring chunks) fall into sixteen different bank
//     groups whatever the tap's shift, without an address swizzle - the tap's shift and the slice of the K step are
//     immediate offsets of the read instruction, the loop contains no address arithmetic at all.  (With one VALU
//     instruction per MFMA in the loop - selects for masked lanes, swizzled addresses - a computing wavefront, which is
//     alone on its SIMD, reached 52 % of the MFMA rate; instruction issue, not LDS or MFMA throughput, was the bound.)
//     A direct-to-LDS load writes 64 consecutive 16-byte slots: ten slots per position, the last two dummies.
//   * Wavefront roles as in gemm16_dma_kernel<.., FEED>: wavefronts 0..3 only compute, 4..7 only issue direct-to-LDS
//     loads (three filter stages, the patch, then a filter stage per K step), wait for them and meet the others at
//     one barrier per K step (one filter tap).
//   * A computing wavefront holds 7 x 4 accumulators of v_mfma_f32_16x16x32: 112 pixels x 64 output channels, the
//     block 448 pixels.  The MFMA computes the transposed tile (filter fragment as the first operand): a lane then
//     owns, for one pixel, the output channels 8 g + 4 (j % 2) + r (+ 32 for tiles j = 2, 3), because tile j's filter
//     fragment is built from the rows 32 (j / 2) + 8 g' + 4 (j % 2) + r'.  The epilogue (scale, shift, residual,
//     relu) runs in registers; lanes of a row of 16 then exchange halves (DPP row shifts by 8) so that a store
//     instruction writes 8 pixels x 128 contiguous bytes.  No LDS staging, no barrier after the K loop.
//   * Filter stage rows are swizzled with a key made of bits 1, 3 and 2 of the row, which keeps those permuted
//     fragment reads conflict free.
//
// More than 64 input channels (conv3x3_patch_chunks_kernel): the K loop walks the channels 64 at a time and, inside a
// chunk, the nine taps.  The patch of a chunk is what the single-chunk kernel keeps; two such buffers alternate, and
// the feeding wavefronts fetch the next chunk's patch a few loads per K step while the current one is multiplied.  A
// K step is still one filter stage of 64 x 64 (chunk c, tap t: the columns t C + 64 c .. + 63 of a filter row), the
// ring slot is the tap modulo 3 whatever the chunk, and switching buffers is one add per pixel tile and chunk.  The
// input then travels L2 -> LDS once instead of nine times, which is what bounds the implicit-GEMM tiles on the 14 x 14
// and 28 x 28 layers (their blocks are few and small, so the filter is re-fetched per 128 pixels there as well).
#include <hip/hip_runtime.h>

#include <atomic>
#include <climits>
#include <cstdint>
#include <cstdlib>

#include "kernels/conv_nhwc.h"
#include "kernels/mfma_tile.h"
#include "runtime/hip_check.h"

namespace cinn_hip_kernels {
namespace {

using namespace tile;

constexpr int kTMW      = 7;            // 16-pixel tiles per computing wavefront
constexpr int kWaves    = 4;            // computing wavefronts (as many feeding ones)
constexpr int kCapacity = kWaves * kTMW * 16;  // pixels per block
constexpr int kPitch    = 160;          // bytes between patch positions
constexpr int kNS       = 3;            // filter stages in the ring
constexpr int kBTile    = 64 * 128;     // bytes of a filter stage: 64 rows (output channels) of 64 halves
constexpr int kTaps     = 9;
constexpr int kLdsLimit = 160 * 1024;

struct PatchParams {
  const uint16_t* x;
  const uint16_t* w;
  uint16_t* y;
  const float* scale;
  const float* shift;
  const uint16_t* residual;
  const void* zero_page;  // 256 bytes of zeros in device memory
  float alpha, residual_scale;
  int relu;
  int n, h, w_in, oc;
  int c;            // input channels (a multiple of 64)
  int stack;        // chunked kernel: images per block, stacked with one row of zeros between them (1: bands of one image)
  int rows;         // output rows per band (stacked images: their rows and the separating rows)
  int bands;        // bands per image
  int patch_loads;  // 1 KiB loads that cover the (rows + 2) (W + 2) positions of 10 slots
  int first_loads;  // streaming kernel: the first so many of them cover the rows that the band's first 64 pixels read
  unsigned long long* probe;  // measurement hook (cinn_hip_conv_patch_set_probe): 16 words per block, or null
  unsigned w_magic, w_shift;    // n / W == (n * w_magic) >> w_shift (chunked kernel: W rounded up to a multiple of 8)
  unsigned pw_magic, pw_shift;  // the same for W + 2
};

// vmcnt(n): at most n of the wavefront's loads still in flight (they complete in issue order); lgkmcnt / expcnt open
#define CINN_VMCNT(n) ((((n) & 15) | (((n) >> 4) << 14)) | 0x0F70)

// The folded scale and shift of a lane's output channels (8 g .. 8 g + 7 and 32 + 8 g .. + 7 of the block's 64; alpha
// and 0 without a table), fetched before the K loop so that the epilogue does not start with a trip to memory.  The
// empty asm pins the loads there: the compiler would otherwise sink them to their first use.
struct LaneScaleShift {
  float sc[2][8], sh[2][8];
};
__device__ __forceinline__ void LoadScaleShift(const PatchParams& p, int n0, int lane, LaneScaleShift* out) {
  const int oc0 = n0 + 8 * (lane >> 4);
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      out->sc[s][e] = p.scale ? p.scale[oc0 + 32 * s + e] : p.alpha;
      out->sh[s][e] = p.shift ? p.shift[oc0 + 32 * s + e] : 0.0f;
    }
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) asm volatile("" : "+v"(out->sc[s][e]), "+v"(out->sh[s][e]));
}

// Epilogue in registers (scale, shift, residual, relu), then whole 128-byte lines to global memory.  acc[i][j]: tile i
// of 16 pixel slots (this lane: slot pix0 + 16 i of the band), transposed result tile j.  Slots are the band's pixels
// in order (PADDED false: npix of them are real), or image rows padded to wp slots, a multiple of 8 (PADDED true: slot
// q is column q % wp of the band's row q / wp; p.w_magic / p.w_shift divide by wp).
template <typename T, int TMW, bool PADDED>
__device__ __forceinline__ void PatchEpilogue(const PatchParams& p, const f32x4 (&acc)[TMW][4], const LaneScaleShift& ss,
                                              int img, int y0, int n0, int rows, int wp, int pix0, int lane) {
  typedef typename Mfma16<T>::vec8 vec8;
  const int W    = p.w_in;
  const int npix = rows * W;
  // the band's pixel in slot q (counted from the first pixel of the band's first image row), or -1
  auto pixel_of = [&](int q) -> int {
    if (!PADDED) return q < npix ? q : -1;
    const int ly = (int)(((uint64_t)(unsigned)q * p.w_magic) >> p.w_shift);
    const int lx = q - ly * wp;
    if (ly >= rows || lx >= W) return -1;
    if (p.stack == 1) return ly * W + lx;
    // stacked images: row ly of the band is row ly % (H + 1) of image ly / (H + 1); row H is the separator
    const int k = ly / (p.h + 1), iy = ly - k * (p.h + 1);
    return iy < p.h ? (k * p.h + iy) * W + lx : -1;
  };
  // lane = (slot lane & 15 of each tile; channels 8 g .. 8 g + 7 and 32 + 8 g .. + 7)
  const int g   = lane >> 4;
  const int px  = lane & 15;
  const int oc0 = n0 + 8 * g;
  const int64_t out_row0 = ((int64_t)img * p.h + y0) * W;
  T* const Y       = reinterpret_cast<T*>(p.y);
  const T* const R = reinterpret_cast<const T*>(p.residual);
  const int st_chunk = g + 4 * (px >> 3);  // 16-byte chunk of a pixel's 64 channels that this lane stores
#pragma unroll
  for (int i = 0; i < TMW; ++i) {
    const int slot = pix0 + 16 * i;
    vec8 res[2] = {};
    if (R) {
      const int pix = pixel_of(slot);
      if (pix >= 0) {
        const int64_t o = (out_row0 + pix) * p.oc + oc0;
        res[0] = *reinterpret_cast<const vec8*>(R + o);
        res[1] = *reinterpret_cast<const vec8*>(R + o + 32);
      }
    }
    u32x4 out[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // explicit fused multiply-adds rounded to fp32 and an empty asm before the conversion: the same arithmetic,
        // in the same order, as the epilogues of the other convolution kernels; the relu is a max (a NaN becomes 0,
        // as with v > 0 ? v : 0) under a select on the flag, the conversion takes two values at a time
        v[e] = __builtin_fmaf(acc[i][2 * s + (e >> 2)][e & 3], ss.sc[s][e], ss.sh[s][e]);
        if (R) v[e] = __builtin_fmaf(p.residual_scale, (float)res[s][e], v[e]);
        const float m = __builtin_fmaxf(v[e], 0.0f);
        v[e]          = p.relu ? m : v[e];
        asm volatile("" : "+v"(v[e]));
      }
      out[s] = u32x4{PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3]), PackPair<T>(v[4], v[5]), PackPair<T>(v[6], v[7])};
    }
    // first store: slots 0..7 of the tile as whole 128-byte lines (lanes px < 8: their own channels 8 g ..; lanes
    // px >= 8: the channels 32 + 8 g .. of slot px - 8); second store: slots 8..15 (lanes px >= 8: their own channels
    // 32 + 8 g ..; lanes px < 8: the channels 8 g .. of slot px + 8)
    u32x4 first, second;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const unsigned from_below = RowShift8<true>(out[1][d]);   // second half of lane px - 8
      const unsigned from_above = RowShift8<false>(out[0][d]);  // first half of lane px + 8
      first[d]  = px < 8 ? out[0][d] : from_below;
      second[d] = px < 8 ? from_above : out[1][d];
    }
    const int p_first  = pixel_of(slot - px + (px & 7));
    const int p_second = pixel_of(slot - px + (px & 7) + 8);
    if (p_first >= 0) *reinterpret_cast<u32x4*>(Y + (out_row0 + p_first) * p.oc + n0 + 8 * st_chunk) = first;
    if (p_second >= 0) *reinterpret_cast<u32x4*>(Y + (out_row0 + p_second) * p.oc + n0 + 8 * st_chunk) = second;
  }
}

template <typename T>
__global__ void __launch_bounds__(128 * kWaves) conv3x3_c64_patch_kernel(PatchParams p) {
  constexpr int L = 64 / 8 / kWaves;  // 1 KiB filter loads per feeding wavefront and stage
  typedef typename Mfma16<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char* const ring  = lds;                  // kNS filter stages
  char* const patch = lds + kNS * kBTile;   // positions of kPitch bytes
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds);

  const int tid     = threadIdx.x;
  const int lane    = tid & 63;
  const int wave    = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int band    = blockIdx.x % p.bands;
  const int img     = blockIdx.x / p.bands;
  const int n0      = blockIdx.y * 64;
  const int W       = p.w_in;
  const int PW      = W + 2;
  const int y0      = band * p.rows;
  const int rows    = min(p.rows, p.h - y0);
  const int npix    = rows * W;
  const int npos    = (p.rows + 2) * PW;  // positions the patch has room for
  constexpr int ktot = kTaps * 64;        // filter row length

  // The patch: load q fills the slots 64 q .. 64 q + 63; slot s = chunk s % 10 of position s / 10.  All eight
  // wavefronts take part (the computing ones have nothing else to do yet): wavefront w issues the loads w, w + 8, ...
  auto load_patch = [&](int first) {
    const char* const ximg  = reinterpret_cast<const char*>(p.x + (int64_t)img * p.h * W * 64);
    const char* const zeros = static_cast<const char*>(p.zero_page);
    for (int q = first; q < p.patch_loads; q += 2 * kWaves) {
      const unsigned slot  = 64u * q + lane;
      const unsigned pos   = (slot * 52429u) >> 19;  // slot / 10 for slot < 2^16
      const unsigned chunk = slot - 10u * pos;
      const int pr         = (int)(((uint64_t)pos * p.pw_magic) >> p.pw_shift);
      const int iy         = y0 - 1 + pr;
      const int ix         = (int)pos - pr * PW - 1;
      const bool inside    = chunk < 8u && (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)W && (int)pos < npos;
      const char* src      = inside ? ximg + ((unsigned)(iy * W + ix) * 128u + chunk * 16u) : zeros + ((lane & 7) << 4);
      AsyncCopy16(src, lds_addr + (unsigned)(patch - lds) + q * 1024);
    }
  };

  if (wave >= kWaves) {
    const int f = wave - kWaves;
    // ---- filter stages: load t covers rows 8 (f L + t) .. + 7 of the stage
    unsigned b_off[L];
#pragma unroll
    for (int t = 0; t < L; ++t) {
      const int row = 8 * (f * L + t) + (lane >> 3);
      b_off[t]      = (unsigned)(row * ktot + (((lane & 7) ^ FilterKey(row)) << 3)) * 2u;
    }
    const char* const wbase = reinterpret_cast<const char*>(p.w + (int64_t)n0 * ktot);
    auto issue_stage = [&](int slot, int kt) {
#pragma unroll
      for (int t = 0; t < L; ++t) AsyncCopy16(wbase + kt * 128 + b_off[t], lds_addr + slot * kBTile + (f * L + t) * 1024);
    };
#pragma unroll
    for (int st = 0; st < kNS; ++st) issue_stage(st, st);
    load_patch(wave);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // everything requested so far has landed
    __syncthreads();
    // per K step: stage kt + 1 has landed (the kNS - 2 requested after it may be in flight); the barrier says that
    // stage kt has been read by everyone; its slot takes stage kt + kNS
#pragma unroll
    for (int kt = 0; kt + 1 < kTaps; ++kt) {
      if (kt > 0 && kt + kNS <= kTaps) {
        __builtin_amdgcn_s_waitcnt(CINN_VMCNT((kNS - 2) * L));
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      __syncthreads();
      if (kt + kNS < kTaps) issue_stage(kt % kNS, kt + kNS);
    }
    return;
  }

  // ---- computing wavefronts
  load_patch(wave);
  const int frag_kg = ((lane >> 4) & 1) * 2 + (lane >> 5);  // k chunks 0, 2, 1, 3 for the lane groups 0..3
  const int pix0    = wave * (kTMW * 16) + (lane & 15);
  // LDS address of this lane's chunk of K slice 0 under tap (0, 0), per tile (slice 1: 64 bytes further; tap (dy, dx):
  // (dy (W + 2) + dx) positions further).  Lanes beyond the band's last pixel read position 0; their results are not
  // stored.
  const char* a_base[kTMW];
#pragma unroll
  for (int i = 0; i < kTMW; ++i) {
    const int pix = pix0 + 16 * i;
    const int ly  = (int)(((uint64_t)(unsigned)pix * p.w_magic) >> p.w_shift);
    const int pos = pix < npix ? ly * PW + (pix - ly * W) : 0;
    a_base[i]     = patch + pos * kPitch + frag_kg * 16;
  }
  // Filter fragment of tile j, slice kk: row 32 (j / 2) + 8 g' + 4 (j % 2) + r' (q = lane & 15 = 4 g' + r')
  const char* b_base[2][4];
  {
    const int q = lane & 15;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 32 * (j >> 1) + 8 * (q >> 2) + 4 * (j & 1) + (q & 3);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) b_base[kk][j] = ring + row * 128 + (((kk * 4 + frag_kg) ^ FilterKey(row)) << 4);
    }
  }
  const int row_pitch = PW * kPitch;

  f32x4 acc[kTMW][4];
#pragma unroll
  for (int i = 0; i < kTMW; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  // A K step (one tap) is 14 rows of 4 MFMAs: row r multiplies the pixel fragment of tile r % 7, slice r / 7, with the
  // four filter fragments of that slice.  Pixel fragments live in one register set per tile and are requested three
  // rows ahead - also across the end of a step: the patch does not change, so the first three of the next step need
  // no barrier.  Filter fragments: slice 1 is requested in rows 0 and 1; the barrier that hands the stage's slot back
  // follows row 9 (both slices are in registers by then), the next stage's slice 0 is requested in rows 11 and 12.
  // All nine steps are unrolled: ring slots and the dx part of a tap's shift are immediate offsets.
  vec8 ar[kTMW];
  vec8 bf[2][4];
  auto read_a = [&](int i, int kk, int dx) -> vec8 { return *reinterpret_cast<const vec8*>(a_base[i] + dx * kPitch + kk * 64); };
  auto read_b = [&](int slot, int kk, int j) -> vec8 { return *reinterpret_cast<const vec8*>(b_base[kk][j] + slot * kBTile); };
  __builtin_amdgcn_s_waitcnt(0x0F70);  // this wavefront's share of the patch has landed
  __syncthreads();                     // the patch and the first filter stages are in LDS
#pragma unroll
  for (int r = 0; r < 3; ++r) ar[r] = read_a(r, 0, 0);
#pragma unroll
  for (int j = 0; j < 4; ++j) bf[0][j] = read_b(0, 0, j);
#define CINN_SB __builtin_amdgcn_sched_barrier(0)
#pragma unroll
  for (int kt = 0; kt < kTaps; ++kt) {
    const bool has_next = kt + 1 < kTaps;
    const int dx        = kt % 3;
    // requests for the next step: its dx, and one row of positions further when this step ends a filter row (the
    // bases move on after the step)
    const int next_dx   = dx == 2 ? 0 : dx + 1;
    const int next_row  = dx == 2 ? row_pitch : 0;
#pragma unroll
    for (int r = 0; r < 2 * kTMW; ++r) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        CINN_SB;
        acc[r % kTMW][j] = Mfma16<T>::mma(bf[r / kTMW][j], ar[r % kTMW], acc[r % kTMW][j]);
        CINN_SB;
        if (j == 0) {
          if (r + 3 < 2 * kTMW) {
            ar[(r + 3) % kTMW] = read_a((r + 3) % kTMW, (r + 3) / kTMW, dx);
          } else if (has_next) {
            ar[r + 3 - 2 * kTMW] =
                *reinterpret_cast<const vec8*>(a_base[r + 3 - 2 * kTMW] + next_row + next_dx * kPitch);
          }
        }
        if ((j == 1 || j == 2) && r < 2) bf[1][r * 2 + j - 1] = read_b(kt % kNS, 1, r * 2 + j - 1);
        if ((j == 1 || j == 2) && r >= 11 && r < 13 && has_next)
          bf[0][(r - 11) * 2 + j - 1] = read_b((kt + 1) % kNS, 0, (r - 11) * 2 + j - 1);
      }
      if (r == 9 && has_next) {
        CINN_SB;
        __syncthreads();
      }
    }
    if (dx == 2 && has_next) {
      CINN_SB;
#pragma unroll
      for (int i = 0; i < kTMW; ++i) a_base[i] += row_pitch;
    }
  }
#undef CINN_SB

  LaneScaleShift ss;
  LoadScaleShift(p, n0, lane, &ss);
  PatchEpilogue<T, kTMW, false>(p, acc, ss, img, y0, n0, rows, W, pix0, lane);
}
// s_waitcnt vmcnt(n) for a count that is a constant only after unrolling (the builtin wants a literal)
__device__ __forceinline__ void WaitLoadsInFlight(int n) {
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(0)); break;
    case 1: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(1)); break;
    case 2: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(2)); break;
    case 3: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(3)); break;
    case 4: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(4)); break;
    case 5: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(5)); break;
    case 6: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(6)); break;
    case 7: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(7)); break;
    case 8: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(8)); break;
    case 9: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(9)); break;
    case 10: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(10)); break;
    case 11: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(11)); break;
    case 12: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(12)); break;
    case 13: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(13)); break;
    case 14: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(14)); break;
    case 15: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(15)); break;
    case 16: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(16)); break;
    case 17: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(17)); break;
    case 18: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(18)); break;
    case 19: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(19)); break;
    case 20: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(20)); break;
    case 21: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(21)); break;
    case 22: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(22)); break;
    case 23: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(23)); break;
    case 24: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(24)); break;
    case 25: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(25)); break;
    case 26: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(26)); break;
    case 27: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(27)); break;
    case 28: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(28)); break;
    case 29: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(29)); break;
    case 30: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(30)); break;
    case 31: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(31)); break;
    case 32: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(32)); break;
    case 33: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(33)); break;
    case 34: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(34)); break;
    case 35: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(35)); break;
    case 36: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(36)); break;
    case 37: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(37)); break;
    case 38: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(38)); break;
    case 39: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(39)); break;
    case 40: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(40)); break;
    default: __builtin_amdgcn_s_waitcnt(CINN_VMCNT(0)); break;
  }
}

// The same layer with the three phases of conv3x3_c64_patch_kernel - fetch the patch, multiply, store - overlapped
// inside a block instead of following each other.  That kernel walks the taps in its outer loop (a filter stage is
// used once, by every pixel), so no pixel is finished before the last tap and all stores come at the end.  Here the
// pixels are the outer loop: the WHOLE filter sits in registers (eight computing wavefronts, wavefront (pg, h) keeps
// the 9 x 64 x 32 filter of the output channels 32 h .. 32 h + 31: 144 registers), a wavefront takes one tile of 16
// pixels through all nine taps (36 MFMAs on two accumulators), converts and stores it, and goes on to the next while
// those stores drain.  Per MFMA it reads LDS half as often as the tap-major loop needs for the same tile shape, two
// wavefronts share a SIMD (one's epilogue and LDS waits are covered by the other's MFMAs) and there are no feeding
// wavefronts and no barrier per K step: the loads are all issued at the start.
//   * LDS: the patch from 0, as in the other kernel; the filter stages of the taps 0..7 (swizzled rows as there) at
//     kStreamFilter; the folded scale / shift of the block's 64 channels in the last KiB.  The ninth stage does not
//     fit beside them; it travels in the two dummy slots that every patch position has behind its 128 bytes (a patch
//     load fills 64 consecutive slots of 16 bytes, ten per position): dummy slot d = 2 position + (0 | 1), d < 512,
//     holds chunk d % 8 of filter row d / 8.  Nothing in LDS is written twice, so no load has to wait for a reader.
//   * Tiles are dealt round-robin, tile 4 s + pg in step s, so the block moves down the band together: step 0 only
//     reads the first rows of the patch (p.first_loads loads, which also cover the ninth stage) and starts when those
//     and the filter have landed.  During step 0 a wavefront moves its filter fragments from LDS into registers, each
//     just ahead of its first MFMA.  Everything else is waited for once, after step 0; then the block runs free.
//     What a block requests (148 KB: 74 KB of patch, 74 KB of filter) leaves L2 at about 44 GB/s per CU when all CUs
//     pull at once (direct-to-LDS loads of a load-only kernel land 8 KiB per CU every 0.18 us whatever they hit), so
//     the first MFMA cannot come before about 3 us into the block and the last row lands about a microsecond later.
//   * All global loads are the untracked direct-to-LDS ones (also scale / shift): the compiler sees LDS reads and
//     global stores only and never waits for the latter.  (A residual operand is read with ordinary loads in the
//     epilogue, which then waits for the stores before it too - correct, slower; 3x3 layers rarely have one.)
// Sums are formed in the same order as in conv3x3_c64_patch_kernel (tap, then the two halves of the channels) and the
// epilogue is the same arithmetic: results are bit-identical.

// Measurement hook: with a buffer set, one wavefront of every block stores the 100 MHz counter and the core clock
// counter at up to eight points (16 words per block).  `chosen` must be wavefront-uniform; every lane stores the same
// words.  The stores count like any other in vmcnt: a wait of that wavefront for its loads then waits for them as
// well, never for less (the stamps come from a wavefront that does not wait during step 0).
__device__ __forceinline__ void PatchStamp(unsigned long long* probe, bool chosen, int slot) {
  if (probe && chosen) {
    unsigned long long* at = probe + 16 * (blockIdx.x + gridDim.x * blockIdx.y) + 2 * slot;
    at[0] = __builtin_amdgcn_s_memrealtime();
    at[1] = __builtin_readcyclecounter();
  }
}

constexpr int kStreamWaves  = 8;
constexpr int kStreamSteps  = 7;                                       // tiles per wavefront
constexpr int kStreamScale  = kLdsLimit - 1024;                        // 64 scales, 64 shifts (fp32)
constexpr int kStreamFilter = kStreamScale - (kTaps - 1) * kBTile;     // eight stages of 8 KiB
constexpr int kStreamLast   = 64 * 8;                                  // dummy slots that hold the ninth stage
constexpr int kStreamLastLoads = (kStreamLast / 2 * 10 + 63) / 64;     // patch loads that cover their positions

template <typename T>
__global__ void __launch_bounds__(64 * kStreamWaves) conv3x3_c64_stream_kernel(PatchParams p) {
  typedef typename Mfma16<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char* const patch = lds;
  char* const filt  = lds + kStreamFilter;
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds);

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pg   = wave & 3;   // tiles pg, pg + 4, ...
  const int half = wave >> 2;  // output channels 32 half .. + 31 of the block's 64
  const int band = blockIdx.x % p.bands;
  const int img  = blockIdx.x / p.bands;
  const int n0   = blockIdx.y * 64;
  const int W    = p.w_in;
  const int PW   = W + 2;
  const int y0   = band * p.rows;
  const int rows = min(p.rows, p.h - y0);
  const int npix = rows * W;
  const int npos = (p.rows + 2) * PW;
  constexpr int ktot = kTaps * 64;
  const char* const zeros = static_cast<const char*>(p.zero_page);
  const char* const wblk  = reinterpret_cast<const char*>(p.w + (int64_t)n0 * ktot);
  PatchStamp(p.probe, wave == 0, 0);

  // ---- every load of the block, those that step 0 needs first
  if (wave == 0) {  // lanes 0..15: four scales each, 16..31: four shifts each
    const char* src = zeros + ((lane & 7) << 4);
    if (lane < 16 && p.scale) src = reinterpret_cast<const char*>(p.scale + n0 + 4 * lane);
    if (lane >= 16 && lane < 32 && p.shift) src = reinterpret_cast<const char*>(p.shift + n0 + 4 * (lane - 16));
    AsyncCopy16(src, lds_addr + kStreamScale);
  }
  {  // filter stages 0..7: this wavefront fetches the rows 8 wave .. + 7 of each
    const int row      = 8 * wave + (lane >> 3);
    const unsigned off = (unsigned)(row * ktot + (((lane & 7) ^ FilterKey(row)) << 3)) * 2u;
#pragma unroll
    for (int t = 0; t + 1 < kTaps; ++t) AsyncCopy16(wblk + off + t * 128, lds_addr + kStreamFilter + t * kBTile + wave * 1024);
  }
  // patch loads q = wave, wave + 8, ... of [lo, hi): load q fills the slots 64 q .. 64 q + 63 (slot s = chunk s % 10 of
  // position s / 10; chunks 8 and 9 are the dummies, of which the first 512 carry the ninth filter stage and the
  // others are not fetched at all: their lanes sit the load out)
  auto load_patch = [&](int lo, int hi) {
    const char* const ximg = reinterpret_cast<const char*>(p.x + (int64_t)img * p.h * W * 64);
    for (int q = lo + ((wave - lo) & 7); q < hi; q += kStreamWaves) {
      const unsigned slot  = 64u * q + lane;
      const unsigned pos   = (slot * 52429u) >> 19;  // slot / 10 for slot < 2^16
      const unsigned chunk = slot - 10u * pos;
      const int pr         = (int)(((uint64_t)pos * p.pw_magic) >> p.pw_shift);
      const int iy         = y0 - 1 + pr;
      const int ix         = (int)pos - pr * PW - 1;
      const bool inside    = chunk < 8u && (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)W && (int)pos < npos;
      const unsigned d     = 2u * pos + (chunk - 8u);  // dummy slot number
      const char* src      = inside ? ximg + ((unsigned)(iy * W + ix) * 128u + chunk * 16u) : zeros + ((lane & 7) << 4);
      if (chunk >= 8u) src = wblk + ((d >> 3) * ktot + (kTaps - 1) * 64 + (d & 7u) * 8u) * 2u;
      if (chunk < 8u || d < (unsigned)kStreamLast) AsyncCopy16(src, lds_addr + q * 1024);
    }
  };
  // The address unit's queue holds less than the block requests and serves the oldest wavefront first: without the
  // barrier, one wavefront's loads for the last rows would queue in front of another's loads for the first.  (One
  // barrier: more of them, a finer order, cost more than the order gains - a round of one load per wavefront with a
  // barrier takes 0.1 to 0.2 us.)
  load_patch(0, p.first_loads);
  __builtin_amdgcn_s_barrier();
  load_patch(p.first_loads, p.patch_loads);
  // how many of this wavefront's patch loads lie below load number x
  auto mine_below = [&](int x) -> int { return x > wave ? (x - wave + kStreamWaves - 1) / kStreamWaves : 0; };

  // ---- addresses
  const int frag_kg = ((lane >> 4) & 1) * 2 + (lane >> 5);  // k chunks 0, 2, 1, 3 for the lane groups 0..3
  const int px      = lane & 15;
  const int g       = lane >> 4;
  // position of this lane's pixel of step s in the patch (tap (0, 0), K slice 0); lanes beyond the band read position 0
  const char* a_pos[kStreamSteps];
#pragma unroll
  for (int s = 0; s < kStreamSteps; ++s) {
    const int pix = 16 * (4 * s + pg) + px;
    const int ly  = (int)(((uint64_t)(unsigned)pix * p.w_magic) >> p.w_shift);
    const int pos = pix < npix ? ly * PW + (pix - ly * W) : 0;
    a_pos[s]      = patch + pos * kPitch + frag_kg * 16;
  }
  const int row_pitch = PW * kPitch;
  // filter fragment of tile j (rows 32 half + 8 g' + 4 j + r', q = lane & 15 = 4 g' + r'), K slice kk: in stage 0, and
  // where the ninth stage has it
  const char* b_base[2][2];
  const char* b_last[2][2];
  {
    const int q = lane & 15;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = 32 * half + 8 * (q >> 2) + 4 * j + (q & 3);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        b_base[kk][j] = filt + row * 128 + (((kk * 4 + frag_kg) ^ FilterKey(row)) << 4);
        const int d   = 8 * row + kk * 4 + frag_kg;
        b_last[kk][j] = patch + (d >> 1) * kPitch + 128 + (d & 1) * 16;
      }
    }
  }
  // this lane's first output element: pixel 16 pg + px of the band, channels n0 + 32 half + 8 g ..
  const int oc0 = n0 + 32 * half + 8 * g;
  T* const Y       = reinterpret_cast<T*>(p.y);
  const T* const R = reinterpret_cast<const T*>(p.residual);
  const int64_t out0 = (((int64_t)img * p.h + y0) * W + 16 * pg + px) * p.oc + oc0;

  // ---- the filter and the rows that step 0 reads have landed (this wavefront's part: at most the patch loads it
  // issued after them are in flight)
  WaitLoadsInFlight(mine_below(p.patch_loads) - mine_below(p.first_loads));
  BarrierLds();
  PatchStamp(p.probe, wave == 0, 1);

  vec8 bf[kTaps][2][2];
  auto read_b = [&](int t, int kk, int j) -> vec8 {
    return *reinterpret_cast<const vec8*>(t + 1 < kTaps ? b_base[kk][j] + t * kBTile : b_last[kk][j]);
  };
  auto read_a = [&](int s, int u) -> vec8 {  // pixel fragment u = 2 tap + kk of step s
    const int tap = u >> 1, kk = u & 1;
    return *reinterpret_cast<const vec8*>(a_pos[s] + (tap / 3) * row_pitch + (tap % 3) * kPitch + kk * 64);
  };
  float sc[8], sh[8];
  // scale, shift, residual, relu, conversion: the arithmetic of PatchEpilogue
  auto finish = [&](const f32x4 (&acc)[2], int s) -> u32x4 {
    vec8 res = {};
    const bool valid = 16 * (4 * s + pg) + px < npix;
    if (R && valid) res = *reinterpret_cast<const vec8*>(R + out0 + (int64_t)s * 64 * p.oc);
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = __builtin_fmaf(acc[e >> 2][e & 3], sc[e], sh[e]);
      if (R) v[e] = __builtin_fmaf(p.residual_scale, (float)res[e], v[e]);
      const float m = __builtin_fmaxf(v[e], 0.0f);
      v[e]          = p.relu ? m : v[e];
      asm volatile("" : "+v"(v[e]));
    }
    return u32x4{PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3]), PackPair<T>(v[4], v[5]), PackPair<T>(v[6], v[7])};
  };
  auto store = [&](u32x4 out, int s) {
    if (16 * (4 * s + pg) + px < npix) *reinterpret_cast<u32x4*>(Y + out0 + (int64_t)s * 64 * p.oc) = out;
  };

#define CINN_SB __builtin_amdgcn_sched_barrier(0)
  constexpr int kFrags = 2 * kTaps;  // pixel fragments per tile
  // Pixel fragments go through a ring of four register sets, requested three MFMA pairs ahead; fragment u of step s
  // has the slot (kFrags s + u) % 4, so the ring runs on across the steps.  In step 0 the filter fragments of pair
  // u + 2 are requested with them.
  vec8 ar[4];
  f32x4 acc[2];
  u32x4 held;
#pragma unroll
  for (int s = 0; s < kStreamSteps; ++s) {
    if (s == 1) {
      // Everything else is waited for once, BEFORE the first store is issued: a wait is for "at most n operations in
      // flight", loads or stores, and with stores among them it would wait for their acknowledgement (most of a
      // microsecond) where it only needs the loads.  (Waits before each of the next steps, for just the rows they
      // add, were measured: 14.5 us per launch against 13.5, for that reason.)
      __builtin_amdgcn_s_waitcnt(CINN_VMCNT(0));  // all of this wavefront's patch loads have landed
      BarrierLds();                               // ... and everyone else's
      PatchStamp(p.probe, wave == 0, 3);
      store(held, 0);
    }
    // the first fragments of a step are requested during the step before, except across that wait
    if (s < 2) {
#pragma unroll
      for (int u = 0; u < 3; ++u) ar[(kFrags * s + u) & 3] = read_a(s, u);
    }
    if (s == 0) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int j = 0; j < 2; ++j) bf[u >> 1][u & 1][j] = read_b(u >> 1, u & 1, j);
    }
    acc[0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    acc[1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < kFrags; ++u) {
      const int m = kFrags * s + u;
      CINN_SB;
      acc[0] = Mfma16<T>::mma(bf[u >> 1][u & 1][0], ar[m & 3], acc[0]);
      CINN_SB;
      if (u + 3 < kFrags) {
        ar[(m + 3) & 3] = read_a(s, u + 3);
      } else if (s >= 1 && s + 1 < kStreamSteps) {
        ar[(m + 3) & 3] = read_a(s + 1, u + 3 - kFrags);
      }
      if (s == 0 && u + 2 < kFrags) {
        bf[(u + 2) >> 1][(u + 2) & 1][0] = read_b((u + 2) >> 1, (u + 2) & 1, 0);
        bf[(u + 2) >> 1][(u + 2) & 1][1] = read_b((u + 2) >> 1, (u + 2) & 1, 1);
      }
      CINN_SB;
      acc[1] = Mfma16<T>::mma(bf[u >> 1][u & 1][1], ar[m & 3], acc[1]);
      CINN_SB;
    }
    if (s == 0) {
      const float* const tab = reinterpret_cast<const float*>(lds + kStreamScale);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = tab[32 * half + 8 * g + e], b = tab[64 + 32 * half + 8 * g + e];
        sc[e] = p.scale ? a : p.alpha;
        sh[e] = p.shift ? b : 0.0f;
      }
      held = finish(acc, 0);
      PatchStamp(p.probe, wave == 0, 2);
    } else {
      store(finish(acc, s), s);
      if (s == 3) PatchStamp(p.probe, wave == 0, 4);
    }
  }
#undef CINN_SB
  PatchStamp(p.probe, wave == 0, 5);
}

template <bool B>
struct BoolTag {
  static constexpr bool value = B;
};

constexpr int kPatchSteps = 4;  // K steps of a chunk after whose barriers the feeding wavefronts fetch patch loads
constexpr int kRing       = kTaps;  // filter stages in the chunked kernel's ring: the slot of a stage is its tap
constexpr int kChunkStagesAhead = 2;  // a stage has landed this many K steps before the step that multiplies with it

// Loads a feeding wavefront of the chunked kernel may still have in flight when it arrives at the barrier that closes
// K step (chunk, tap t): everything it issued after filter stage s + ahead, which must have landed (the computing
// wavefronts read a stage's fragments one step before they multiply with them, so ahead = 2).  After the barrier of a
// step u the wavefront issues pl patch loads (taps below kPatchSteps of a chunk that is not the last) and then the l
// loads of stage u + kRing (while that stage exists, i.e. in chunks that are not the last); stage s + ahead was issued
// after barrier s + ahead - kRing, so the steps from there to s - 1 count.  In the first chunk the steps before step 0
// stand for the stages issued before the loop, in order and without patch loads between them.  At the last barrier
// before the computing wavefronts touch the next chunk's patch (tap 9 - ahead of a chunk that is not the last) that
// patch must have landed as well: only the stages issued after the last patch load may be in flight.  In the last
// chunk a stage beyond its tap 8 does not exist: the count is the one for the last stage that does.
__host__ __device__ __forceinline__ constexpr int ChunkLoadsInFlight(int t, bool first, bool last, int pl, int l,
                                                                     int ahead = kChunkStagesAhead) {
  if (last && t + ahead > kTaps - 1) ahead = kTaps - 1 - t;
  if (ahead <= 0) return 0;
  int n = 0;
  for (int u = t - (kRing - 1 - ahead); u < t; ++u) {
    const bool before = u < 0;  // a step of the previous chunk, or a stage fetched before the loop
    const int tap     = before ? u + kTaps : u;
    if (before && first) {
      n += l;
    } else if (before || !last) {
      n += (tap < kPatchSteps ? pl : 0) + l;
    }
  }
  const int patch_tap = kTaps - ahead;
  if (!last && t == patch_tap) {
    const int after_patch = (patch_tap - (kPatchSteps - 1)) * l;
    n                     = n < after_patch ? n : after_patch;
  }
  return n;
}

// C = 64 * chunks input channels.  TMW: 16-slot tiles per computing wavefront (the block holds 64 TMW pixel slots of
// one band: 4 for 256, or 2 for 128 where larger blocks would be too few); PL: patch loads a feeding wavefront issues
// per K step, so a chunk's patch is at most 4 * kPatchSteps * PL KiB.
// LDS: a ring of nine filter stages (a whole chunk: the slot of a stage is its tap, and a stage is requested eight K
// steps before its use - the filters of a layer are read once per launch and XCD, from memory rather than from L2),
// then two patch buffers of patch_loads KiB each.  At least two chunks.  The loop starts as soon as the first patch
// and the stages 0 and 1 have landed.
//
// A K step (one tap of one chunk) is 2 TMW rows of four MFMAs - 256 clocks with two tiles, less than an LDS read
// takes to return under load - so the filter fragments of a step are read during the step before it, into one of
// three register sets (the tap modulo 3: an immediate whatever the chunk); pixel fragments sit in a ring of four,
// requested three rows ahead.  One barrier closes every step s = 9 c + t but the last:
//   computing wavefronts   have multiplied with every fragment of stage s before it (its slot may be refilled); after
//                          it they read the fragments of stage s + 2 during step s + 1, and in the last rows of
//                          step t = 8 the first pixel fragments of the next chunk's patch;
//   feeding wavefronts     before it: stage s + 2 has landed and, at t = 7, the next chunk's patch (loads complete in
//                          order: ChunkLoadsInFlight counts what was issued later and may still be in flight); after
//                          it: PL patch loads of chunk c + 1 (steps t < kPatchSteps; the buffer was last read in step
//                          9 c - 1, which its barrier has closed), then stage s + 9 into the slot of stage s.
template <typename T, int TMW, int PL>
__global__ void __launch_bounds__(128 * kWaves) conv3x3_patch_chunks_kernel(PatchParams p) {
  constexpr int L     = 64 / 8 / kWaves;     // 1 KiB filter loads per feeding wavefront and stage
  constexpr int NPL   = PL * kPatchSteps;     // patch loads per feeding wavefront and chunk
  constexpr int R     = 2 * TMW;              // MFMA rows (of four) per K step
  constexpr int AHEAD = kChunkStagesAhead;
  static_assert(TMW % 2 == 0 && TMW >= 2, "the ring of four pixel fragments wants an even number of tiles");
  typedef typename Mfma16<T>::vec8 vec8;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char* const ring  = lds;
  char* const patch = lds + kRing * kBTile;
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds);
  const unsigned patch_addr = lds_addr + kRing * kBTile;

  const int tid     = threadIdx.x;
  const int lane    = tid & 63;
  const int wave    = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int band    = blockIdx.x % p.bands;
  const int img     = (blockIdx.x / p.bands) * p.stack;  // the block's (first) image
  const int n0      = blockIdx.y * 64;
  const int W       = p.w_in;
  const int PW      = W + 2;
  const int C       = p.c;
  const int chunks  = C >> 6;
  const int y0      = band * p.rows;
  // a band of one image, or min(stack, images left) whole images with a row of zeros after each but the last
  const int rows    = p.stack == 1 ? min(p.rows, p.h - y0) : min(p.stack, p.n - img) * (p.h + 1) - 1;
  const int WP      = (W + 7) & ~7;           // pixel slots per image row: a 16-lane tile is two halves of one row each
  const int npos    = (p.rows + 2) * PW;
  const int ktot    = kTaps * C;              // filter row length
  const int patch_bytes = p.patch_loads * 1024;

  if (wave >= kWaves) {
    const int f = wave - kWaves;
    // ---- the patch: load q fills the slots 64 q .. 64 q + 63 of a buffer, slot s = chunk s % 10 of position s / 10;
    // this wavefront issues the loads q = f + 4 i.  Source pointers are kept per load and move on by 128 bytes per
    // chunk (lanes that fetch halo or dummy slots stay on the page of zeros).  Loads beyond the last one repeat it: the
    // count per K step stays a constant, which the vmcnt waits rely on.
    const char* src[NPL];
    unsigned step_bytes[NPL];
    unsigned dst[NPL];
    {
      const char* const ximg  = reinterpret_cast<const char*>(p.x + (int64_t)img * p.h * W * C);
      const char* const zeros = static_cast<const char*>(p.zero_page);
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int q          = min(f + kWaves * i, p.patch_loads - 1);
        const unsigned slot  = 64u * q + lane;
        const unsigned pos   = (slot * 52429u) >> 19;  // slot / 10 for slot < 2^16
        const unsigned chunk = slot - 10u * pos;
        const int pr         = (int)(((uint64_t)pos * p.pw_magic) >> p.pw_shift);
        int iy               = y0 - 1 + pr;  // row of the image, or of the stack
        int k                = 0;            // image of the stack
        if (p.stack > 1 && iy >= 0) {
          k  = iy / (p.h + 1);
          iy = iy - k * (p.h + 1);           // H: the row of zeros between two images
        }
        const int ix         = (int)pos - pr * PW - 1;
        const bool inside    = chunk < 8u && (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)W && (int)pos < npos &&
                            img + k < p.n;
        src[i]        = inside ? ximg + ((int64_t)((k * p.h + iy) * W + ix) * C * 2 + chunk * 16u) : zeros + ((lane & 7) << 4);
        step_bytes[i] = inside ? 128u : 0u;
        dst[i]        = (unsigned)q * 1024u;
      }
    }
    auto issue_patch = [&](int first, int count, unsigned buffer) {
#pragma unroll
      for (int i = first; i < first + count; ++i) {
        AsyncCopy16(src[i], buffer + dst[i]);
        src[i] += step_bytes[i];
      }
    };
    // ---- filter stages: load t covers rows 8 (f L + t) .. + 7 of the stage
    unsigned b_off[L];
#pragma unroll
    for (int t = 0; t < L; ++t) {
      const int row = 8 * (f * L + t) + (lane >> 3);
      b_off[t]      = (unsigned)(row * ktot + (((lane & 7) ^ FilterKey(row)) << 3)) * 2u;
    }
    const char* const wbase = reinterpret_cast<const char*>(p.w + (int64_t)n0 * ktot);
    auto issue_stage = [&](int slot, int chunk, int tap) {
      const char* const w0 = wbase + (tap * C + chunk * 64) * 2;
#pragma unroll
      for (int t = 0; t < L; ++t) AsyncCopy16(w0 + b_off[t], lds_addr + slot * kBTile + (f * L + t) * 1024);
    };
    // the first patch and the stages 0 and 1 are all the first K step needs; the other stages land while it runs
    issue_patch(0, NPL, patch_addr);
#pragma unroll
    for (int st = 0; st < kRing; ++st) issue_stage(st, 0, st);
    WaitLoadsInFlight((kRing - AHEAD) * L);
    BarrierLds();
    auto feed_chunk = [&](auto first_tag, auto last_tag, int c) {
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr bool LAST  = decltype(last_tag)::value;
      const unsigned next_buffer = patch_addr + ((c + 1) & 1) * patch_bytes;
#pragma unroll
      for (int t = 0; t + (LAST ? 1 : 0) < kTaps; ++t) {
        WaitLoadsInFlight(ChunkLoadsInFlight(t, FIRST, LAST, PL, L, AHEAD));
        BarrierLds();
        if (!LAST) {
          if (t < kPatchSteps) issue_patch(t * PL, PL, next_buffer);
          issue_stage(t, c + 1, t);
        }
      }
    };
    feed_chunk(BoolTag<true>{}, BoolTag<false>{}, 0);
    for (int c = 1; c + 1 < chunks; ++c) feed_chunk(BoolTag<false>{}, BoolTag<false>{}, c);
    feed_chunk(BoolTag<false>{}, BoolTag<true>{}, chunks - 1);
    return;
  }

  // ---- computing wavefronts
  const int frag_kg = ((lane >> 4) & 1) * 2 + (lane >> 5);  // k chunks 0, 2, 1, 3 for the lane groups 0..3
  const int pix0    = wave * (TMW * 16) + (lane & 15);
  // LDS address of this lane's chunk of K slice 0 under tap (0, 0) in the patch buffer of the current chunk, per tile.
  // The eight lanes LDS serves together hold consecutive slots of one image row, i.e. consecutive positions: with
  // tiles that straddle rows (positions two apart at the seam) a third of the reads of a 14-wide image took two
  // passes, and LDS reads, half an instruction per MFMA here, are what the K loop waits for.  Slots beyond the row's
  // last pixel read that pixel's position again (a broadcast, no conflict); slots beyond the band read position 0.
  const char* a_base[TMW];
#pragma unroll
  for (int i = 0; i < TMW; ++i) {
    const int slot = pix0 + 16 * i;
    const int ly   = (int)(((uint64_t)(unsigned)slot * p.w_magic) >> p.w_shift);
    const int lx   = min(slot - ly * WP, W - 1);
    const int pos  = ly < rows ? ly * PW + lx : 0;
    a_base[i]      = patch + pos * kPitch + frag_kg * 16;
  }
  LaneScaleShift ss;
  LoadScaleShift(p, n0, lane, &ss);
  const char* b_base[2][4];
  {
    const int q = lane & 15;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 32 * (j >> 1) + 8 * (q >> 2) + 4 * (j & 1) + (q & 3);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) b_base[kk][j] = ring + row * 128 + (((kk * 4 + frag_kg) ^ FilterKey(row)) << 4);
    }
  }
  const int row_pitch = PW * kPitch;

  f32x4 acc[TMW][4];
#pragma unroll
  for (int i = 0; i < TMW; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

#define CINN_SB __builtin_amdgcn_sched_barrier(0)
  {
    // Row r of a step multiplies the pixel fragment of tile r % TMW, slice r / TMW (ring entry r % 4) with the four
    // filter fragments of that slice from the set of this tap.  After the first MFMA of a row the pixel fragment three
    // rows on is requested, after its second and third MFMA two filter fragments of the NEXT tap (slice 0 first).
    vec8 ar[4];
    vec8 bf[3][2][4];
    auto read_b = [&](int slot, int kk, int j) -> vec8 { return *reinterpret_cast<const vec8*>(b_base[kk][j] + slot * kBTile); };
    auto row_base = [&](int q) -> const char* { return a_base[q % TMW] + (q / TMW) * 64; };  // row q of a step: tile, slice
    BarrierLds();  // the first patch and the filter stages 0 and 1 are in LDS
#pragma unroll
    for (int r = 0; r < 3; ++r) ar[r] = *reinterpret_cast<const vec8*>(row_base(r));
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[0][kk][j] = read_b(0, kk, j);
    auto multiply_chunk = [&](auto last_tag, int to_next) {
      constexpr bool LAST = decltype(last_tag)::value;
#pragma unroll
      for (int kt = 0; kt < kTaps; ++kt) {
        const bool has_next = !(LAST && kt + 1 == kTaps);
        const int dx        = kt % 3;
        const int next_dx   = dx == 2 ? 0 : dx + 1;
        const int next_off  = kt + 1 == kTaps ? to_next : (dx == 2 ? row_pitch : 0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            CINN_SB;
            acc[r % TMW][j] = Mfma16<T>::mma(bf[kt % 3][r / TMW][j], ar[r % 4], acc[r % TMW][j]);
            CINN_SB;
            if (j == 0) {
              if (r + 3 < R) {
                ar[(r + 3) % 4] = *reinterpret_cast<const vec8*>(row_base(r + 3) + dx * kPitch);
              } else if (has_next) {
                ar[(r + 3) % 4] = *reinterpret_cast<const vec8*>(row_base(r + 3 - R) + next_off + next_dx * kPitch);
              }
            }
            if ((j == 1 || j == 2) && r < 4 && has_next) {
              const int f = r * 2 + j - 1;  // 0..7: slice f / 4, filter tile f % 4
              bf[(kt + 1) % 3][f / 4][f % 4] = read_b((kt + 1) % kRing, f / 4, f % 4);
            }
          }
        }
        if (has_next) {
          CINN_SB;
          BarrierLds();
        }
        if (has_next && (dx == 2)) {
          CINN_SB;
#pragma unroll
          for (int i = 0; i < TMW; ++i) a_base[i] += next_off;
        }
      }
    };
    for (int c = 0; c + 1 < chunks; ++c) multiply_chunk(BoolTag<false>{}, ((c & 1) ? -patch_bytes : patch_bytes) - 2 * row_pitch);
    multiply_chunk(BoolTag<true>{}, 0);
  }
#undef CINN_SB

  PatchEpilogue<T, TMW, true>(p, acc, ss, img, y0, n0, rows, WP, pix0, lane);
}
#undef CINN_VMCNT

struct PatchPlan {
  int rows, bands, patch_loads, lds_bytes;
  int stack{1};  // images per block (chunked kernel, small images)
  int blocks(int n) const { return ((n + stack - 1) / stack) * bands; }  // per group of 64 output channels
};

// rows per band and LDS footprint; false when the patch does not fit or more than a fifth of the blocks' pixel slots
// would stay empty
bool PlanFor(const ConvNhwcArgs& a, PatchPlan* plan) {
  int rows = kCapacity / a.w_in;
  if (rows < 1) return false;
  rows            = rows < a.h ? rows : a.h;
  const int bands = (a.h + rows - 1) / rows;
  rows            = (a.h + bands - 1) / bands;
  if ((int64_t)a.h * a.w_in * 5 < (int64_t)bands * kCapacity * 4) return false;
  const int slots = (rows + 2) * (a.w_in + 2) * 10;
  if (slots >= 65536) return false;  // the kernel divides slot numbers by 10 with a 16-bit reciprocal
  const int patch_loads = (slots + 63) / 64;
  const int bytes       = kNS * kBTile + patch_loads * 1024;
  if (bytes > kLdsLimit) return false;
  *plan = PatchPlan{rows, bands, patch_loads, bytes, 1};
  return true;
}

// The streaming kernel's plan: the same bands; the patch must end below the filter stages, have the 256 positions
// whose dummy slots carry the ninth stage, and the first loads - the rows that the band's first 64 pixels read, and
// those positions - are the ones step 0 waits for.
bool PlanStreamFor(const ConvNhwcArgs& a, PatchPlan* plan, int* first_loads) {
  int rows = kCapacity / a.w_in;
  if (rows < 1) return false;
  rows            = rows < a.h ? rows : a.h;
  const int bands = (a.h + rows - 1) / rows;
  rows            = (a.h + bands - 1) / bands;
  if ((int64_t)a.h * a.w_in * 5 < (int64_t)bands * kCapacity * 4) return false;
  const int slots = (rows + 2) * (a.w_in + 2) * 10;
  if (slots >= 65536) return false;
  const int patch_loads = (slots + 63) / 64;
  if (patch_loads * 1024 > kStreamFilter || patch_loads < kStreamLastLoads) return false;
  const int npix     = rows * a.w_in;
  const int last_row = ((npix < 64 ? npix : 64) - 1) / a.w_in;  // band row of the last pixel of step 0
  const int need     = (last_row + 3) * (a.w_in + 2) * 10;      // slots of the patch rows 0 .. last_row + 2
  int first          = (need + 63) / 64;
  first              = first > kStreamLastLoads ? first : kStreamLastLoads;
  *first_loads       = first < patch_loads ? first : patch_loads;
  *plan = PatchPlan{rows, bands, patch_loads, kLdsLimit, 1};
  return true;
}

// The same for more than 64 channels: bands of at most 64 TMW pixel slots (image rows padded to a multiple of 8
// slots) and two patch buffers; rows are given up until
// the buffers fit.  *per_step: patch loads per feeding wavefront and K step (2 or 3).  False when more than three tenths
// of the pixel slots would stay empty.
template <int TMW>
bool PlanChunksFor(const ConvNhwcArgs& a, PatchPlan* plan, int* per_step) {
  constexpr int capacity = kWaves * TMW * 16;
  const int wp = (a.w_in + 7) & ~7;  // pixel slots per image row
  int rows     = capacity / wp;
  // small images: several whole images per block, stacked with a row of zeros between them (the bottom halo of one
  // and the top halo of the next); that row is computed and not stored
  for (int stack = (rows + 1) / (a.h + 1) < a.n ? (rows + 1) / (a.h + 1) : a.n; stack >= 2; --stack) {
    const int stacked     = stack * (a.h + 1) - 1;
    const int slots       = (stacked + 2) * (a.w_in + 2) * 10;
    const int patch_loads = (slots + 63) / 64;
    const int bytes       = kRing * kBTile + 2 * patch_loads * 1024;
    if (patch_loads > kWaves * kPatchSteps * 3 || bytes > kLdsLimit) continue;
    if ((int64_t)stack * a.h * a.w_in * 10 < (int64_t)capacity * 7) break;
    *plan     = PatchPlan{stacked, 1, patch_loads, bytes, stack};
    *per_step = patch_loads > kWaves * kPatchSteps * 2 ? 3 : 2;
    return true;
  }
  rows = rows < a.h ? rows : a.h;
  for (; rows >= 1; --rows) {
    const int bands       = (a.h + rows - 1) / rows;
    const int even        = (a.h + bands - 1) / bands;
    const int slots       = (even + 2) * (a.w_in + 2) * 10;
    const int patch_loads = (slots + 63) / 64;
    const int bytes       = kRing * kBTile + 2 * patch_loads * 1024;
    if (patch_loads > kWaves * kPatchSteps * 3 || bytes > kLdsLimit) continue;
    if ((int64_t)a.h * a.w_in * 10 < (int64_t)bands * capacity * 7) return false;
    *plan     = PatchPlan{even, bands, patch_loads, bytes, 1};
    *per_step = patch_loads > kWaves * kPatchSteps * 2 ? 3 : 2;  // 32 KiB, else 48 KiB of patch per buffer
    return true;
  }
  return false;
}

template <typename T, int TMW, int PL>
void LaunchChunks(const PatchParams& p, const PatchPlan& plan, hipStream_t stream) {
  auto kernel = conv3x3_patch_chunks_kernel<T, TMW, PL>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  dim3 grid(plan.blocks(p.n), p.oc / 64);
  hipLaunchKernelGGL(kernel, grid, dim3(128 * kWaves), plan.lds_bytes, stream, p);
}

template <typename T>
void Launch(const PatchParams& p, const PatchPlan& plan, hipStream_t stream) {
  auto kernel = conv3x3_c64_patch_kernel<T>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  dim3 grid(p.n * p.bands, p.oc / 64);
  hipLaunchKernelGGL(kernel, grid, dim3(128 * kWaves), plan.lds_bytes, stream, p);
}

template <typename T>
void LaunchStream(const PatchParams& p, const PatchPlan& plan, hipStream_t stream) {
  auto kernel = conv3x3_c64_stream_kernel<T>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  dim3 grid(p.n * p.bands, p.oc / 64);
  hipLaunchKernelGGL(kernel, grid, dim3(64 * kStreamWaves), plan.lds_bytes, stream, p);
}

// 64 input channels: 1 = the streaming kernel (pixels outermost, filter in registers), 0 = the tap-major one; -1: not read
std::atomic<int> g_patch_stream{-1};

int PatchStream() {
  int on = g_patch_stream.load(std::memory_order_relaxed);
  if (on < 0) {
    const char* v = getenv("FLAGS_cinn_hip_conv_patch_stream");
    on            = v && *v ? (atoi(v) != 0) : 1;
    g_patch_stream.store(on, std::memory_order_relaxed);
  }
  return on;
}

std::atomic<unsigned long long*> g_patch_probe{nullptr};

// 0: never, 1: where it is expected to win, 2: wherever the shape qualifies; -1: not read yet
std::atomic<int> g_patch_mode{-1};

int PatchMode() {
  int mode = g_patch_mode.load(std::memory_order_relaxed);
  if (mode < 0) {
    const char* v = getenv("FLAGS_cinn_hip_conv_patch");
    mode          = v && *v ? atoi(v) : 1;
    g_patch_mode.store(mode, std::memory_order_relaxed);
  }
  return mode;
}

// 0: chosen per shape, 2 / 4: 16-slot tiles per computing wavefront of the chunked kernel; -1: not read yet
std::atomic<int> g_patch_tiles{-1};

int PatchTiles() {
  int tiles = g_patch_tiles.load(std::memory_order_relaxed);
  if (tiles < 0) {
    const char* v = getenv("FLAGS_cinn_hip_conv_patch_tiles");
    tiles         = v && *v ? atoi(v) : 0;
    if (tiles != 2 && tiles != 4) tiles = 0;
    g_patch_tiles.store(tiles, std::memory_order_relaxed);
  }
  return tiles;
}

}  // namespace

bool TryConvPatch(const ConvNhwcArgs& a, hipStream_t stream) {
  const int flag = PatchMode();
  if (flag == 0) return false;
  const bool is_f16  = a.type.code == cinn_type_float && a.type.bits == 16;
  const bool is_bf16 = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if ((!is_f16 && !is_bf16) || a.nchw_input) return false;
  if (a.kh != 3 || a.kw != 3 || a.stride_h != 1 || a.stride_w != 1 || a.pad_h != 1 || a.pad_w != 1 || a.dil_h != 1 ||
      a.dil_w != 1 || a.oh != a.h || a.ow != a.w_in)
    return false;
  if (a.c % 64 != 0 || a.c > 2048 || a.oc % 64 != 0) return false;  // one chunk, or two and more
  if ((int64_t)a.n * a.h * a.w_in * a.c >= INT_MAX || (int64_t)a.n * a.h * a.w_in * a.oc >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.w) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(a.y) % 16 != 0 || reinterpret_cast<uintptr_t>(a.residual) % 16 != 0)
    return false;
  const bool chunked = a.c != 64;
  int per_step       = 0;
  int tiles          = 4;  // 16-slot tiles per computing wavefront of the chunked kernel
  int first_loads    = 0;
  bool streaming     = false;
  PatchPlan plan;
  if (chunked) {
    // Blocks of 256 pixel slots; when those leave most of the chip idle (256 -> 256 on 14x14 at batch 32: 128 blocks)
    // and blocks of 128 slots give more, the kernel with the schedule for short K steps takes them.
    // FLAGS_cinn_hip_conv_patch_tiles=2|4 (or cinn_hip_conv_patch_tiles) forces one form.
    const int forced_tiles = PatchTiles();
    const bool fits4 = forced_tiles != 2 && PlanChunksFor<4>(a, &plan, &per_step);
    const int64_t blocks4 = fits4 ? (int64_t)plan.blocks(a.n) * (a.oc / 64) : 0;
    if (forced_tiles == 2 || (forced_tiles == 0 && blocks4 < 192)) {
      PatchPlan plan2;
      int per_step2 = 0;
      if (PlanChunksFor<2>(a, &plan2, &per_step2) && per_step2 == 2 && (int64_t)plan2.blocks(a.n) * (a.oc / 64) > blocks4) {
        plan = plan2, per_step = per_step2, tiles = 2;
      } else if (!fits4) {
        return false;
      }
    } else if (!fits4) {
      return false;
    }
  } else if (PatchStream() && PlanStreamFor(a, &plan, &first_loads)) {
    streaming = true;
  } else if (!PlanFor(a, &plan)) {
    return false;
  }
  // one block per band, image and 64 output channels; below ~100 blocks most of the chip would idle and the
  // implicit-GEMM tiles are the better choice
  if (flag != 2 && (int64_t)plan.blocks(a.n) * (a.oc / 64) < 96) return false;
  // stacked small images (512 -> 512 on 7x7 at batch 32: 128 blocks of two images, 23.1 us inside ResNet-50) lose to the
  // implicit GEMM with its reduction split four ways (16.6 + 4.8 us) until they fill most of the chip
  if (flag != 2 && plan.stack > 1 && (int64_t)plan.blocks(a.n) * (a.oc / 64) < 192) return false;
  PatchParams p;
  p.x = static_cast<const uint16_t*>(a.x), p.w = static_cast<const uint16_t*>(a.w), p.y = static_cast<uint16_t*>(a.y);
  p.scale = a.scale, p.shift = a.shift, p.residual = static_cast<const uint16_t*>(a.residual);
  p.zero_page = ConvZeroPage();
  p.alpha = a.alpha, p.residual_scale = a.residual_scale, p.relu = a.relu ? 1 : 0;
  p.n = a.n, p.h = a.h, p.w_in = a.w_in, p.oc = a.oc, p.c = a.c;
  p.rows = plan.rows, p.bands = plan.bands, p.patch_loads = plan.patch_loads, p.stack = plan.stack;
  p.first_loads = first_loads;
  p.probe       = g_patch_probe.load(std::memory_order_relaxed);
  MagicFor(chunked ? (a.w_in + 7) & ~7 : a.w_in, &p.w_magic, &p.w_shift);
  MagicFor(a.w_in + 2, &p.pw_magic, &p.pw_shift);
  if (chunked && tiles == 2) {
    if (is_bf16) {
      LaunchChunks<__bf16, 2, 2>(p, plan, stream);
    } else {
      LaunchChunks<_Float16, 2, 2>(p, plan, stream);
    }
  } else if (chunked && per_step == 2) {
    if (is_bf16) {
      LaunchChunks<__bf16, 4, 2>(p, plan, stream);
    } else {
      LaunchChunks<_Float16, 4, 2>(p, plan, stream);
    }
  } else if (chunked) {
    if (is_bf16) {
      LaunchChunks<__bf16, 4, 3>(p, plan, stream);
    } else {
      LaunchChunks<_Float16, 4, 3>(p, plan, stream);
    }
  } else if (streaming) {
    if (is_bf16) {
      LaunchStream<__bf16>(p, plan, stream);
    } else {
      LaunchStream<_Float16>(p, plan, stream);
    }
  } else if (is_bf16) {
    Launch<__bf16>(p, plan, stream);
  } else {
    Launch<_Float16>(p, plan, stream);
  }
  CINN_HIP_CALL(hipGetLastError());
  return true;
}

}  // namespace cinn_hip_kernels

extern "C" int cinn_hip_conv_patch_loads_in_flight(int tap, int first_chunk, int last_chunk, int patch_loads_per_step) {
  return cinn_hip_kernels::ChunkLoadsInFlight(tap, first_chunk != 0, last_chunk != 0, patch_loads_per_step, 64 / 8 / cinn_hip_kernels::kWaves);
}

extern "C" int cinn_hip_conv_patch_tiles(int tiles) {
  const int before = cinn_hip_kernels::PatchTiles();
  if (tiles == 0 || tiles == 2 || tiles == 4) cinn_hip_kernels::g_patch_tiles.store(tiles, std::memory_order_relaxed);
  return before;
}

extern "C" void cinn_hip_conv_patch_set_probe(void* buffer) {
  cinn_hip_kernels::g_patch_probe.store(static_cast<unsigned long long*>(buffer), std::memory_order_relaxed);
}

extern "C" int cinn_hip_conv_patch_stream(int on) {
  const int before = cinn_hip_kernels::PatchStream();
  if (on == 0 || on == 1) cinn_hip_kernels::g_patch_stream.store(on, std::memory_order_relaxed);
  return before;
}

extern "C" int cinn_hip_conv_patch_mode(int mode) {
  const int before = cinn_hip_kernels::PatchMode();
  if (mode >= 0 && mode <= 2) cinn_hip_kernels::g_patch_mode.store(mode, std::memory_order_relaxed);
  return before;
}
