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
  int rows;         // output rows per band
  int bands;        // bands per image
  int patch_loads;  // 1 KiB loads that cover the (rows + 2) (W + 2) positions of 10 slots
  unsigned w_magic, w_shift;    // n / W == (n * w_magic) >> w_shift
  unsigned pw_magic, pw_shift;  // the same for W + 2
};

// vmcnt(n): at most n of the wavefront's loads still in flight (they complete in issue order); lgkmcnt / expcnt open
#define CINN_VMCNT(n) ((((n) & 15) | (((n) >> 4) << 14)) | 0x0F70)

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

  // ---- epilogue in registers: lane = (pixel lane & 15 of each tile; channels 8 g .. 8 g + 7 and 32 + 8 g .. + 7)
  const int g   = lane >> 4;
  const int px  = lane & 15;
  const int oc0 = n0 + 8 * g;
  float sc[2][8], sh[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sc[s][e] = p.scale ? p.scale[oc0 + 32 * s + e] : p.alpha;
      sh[s][e] = p.shift ? p.shift[oc0 + 32 * s + e] : 0.0f;
    }
  const int64_t out_row0 = ((int64_t)img * p.h + y0) * W;
  T* const Y       = reinterpret_cast<T*>(p.y);
  const T* const R = reinterpret_cast<const T*>(p.residual);
  const int st_chunk = g + 4 * (px >> 3);  // 16-byte chunk of a pixel's 64 channels that this lane stores
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
        // explicit fused multiply-adds rounded to fp32 and an empty asm before the conversion: the same arithmetic,
        // in the same order, as the epilogues of the other convolution kernels
        float v = __builtin_fmaf(acc[i][2 * s + (e >> 2)][e & 3], sc[s][e], sh[s][e]);
        if (R) v = __builtin_fmaf(p.residual_scale, (float)res[s][e], v);
        asm volatile("" : "+v"(v));
        if (p.relu) v = v > 0.0f ? v : 0.0f;
        o8[e] = (T)v;
      }
      out[s] = __builtin_bit_cast(u32x4, o8);
    }
    // first store: pixels 0..7 of the tile as whole 128-byte lines (lanes px < 8: their own channels 8 g ..; lanes
    // px >= 8: the channels 32 + 8 g .. of pixel px - 8); second store: pixels 8..15 (lanes px >= 8: their own channels
    // 32 + 8 g ..; lanes px < 8: the channels 8 g .. of pixel px + 8)
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
#undef CINN_VMCNT

struct PatchPlan {
  int rows, bands, patch_loads, lds_bytes;
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
  *plan = PatchPlan{rows, bands, patch_loads, bytes};
  return true;
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
  if (a.c != 64 || a.oc % 64 != 0) return false;
  if ((int64_t)a.n * a.h * a.w_in * a.c >= INT_MAX || (int64_t)a.n * a.h * a.w_in * a.oc >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.w) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(a.y) % 16 != 0 || reinterpret_cast<uintptr_t>(a.residual) % 16 != 0)
    return false;
  PatchPlan plan;
  if (!PlanFor(a, &plan)) return false;
  // one block per band, image and 64 output channels; below ~100 blocks most of the chip would idle and the
  // implicit-GEMM tiles are the better choice
  if (flag != 2 && (int64_t)a.n * plan.bands * (a.oc / 64) < 96) return false;
  PatchParams p;
  p.x = static_cast<const uint16_t*>(a.x), p.w = static_cast<const uint16_t*>(a.w), p.y = static_cast<uint16_t*>(a.y);
  p.scale = a.scale, p.shift = a.shift, p.residual = static_cast<const uint16_t*>(a.residual);
  p.zero_page = ConvZeroPage();
  p.alpha = a.alpha, p.residual_scale = a.residual_scale, p.relu = a.relu ? 1 : 0;
  p.n = a.n, p.h = a.h, p.w_in = a.w_in, p.oc = a.oc;
  p.rows = plan.rows, p.bands = plan.bands, p.patch_loads = plan.patch_loads;
  MagicFor(a.w_in, &p.w_magic, &p.w_shift);
  MagicFor(a.w_in + 2, &p.pw_magic, &p.pw_shift);
  if (is_bf16) {
    Launch<__bf16>(p, plan, stream);
  } else {
    Launch<_Float16>(p, plan, stream);
  }
  CINN_HIP_CALL(hipGetLastError());
  return true;
}

}  // namespace cinn_hip_kernels

extern "C" int cinn_hip_conv_patch_mode(int mode) {
  const int before = cinn_hip_kernels::PatchMode();
  if (mode >= 0 && mode <= 2) cinn_hip_kernels::g_patch_mode.store(mode, std::memory_order_relaxed);
  return before;
}
