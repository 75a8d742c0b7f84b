// Two 1x1 convolutions in a row, as one kernel: E = act(X W1^T * s1 + t1 + R),  Y = act(E W2^T * s2 + t2)  on
// channels-last 16-bit tensors seen as matrices of M pixels (X [M][K1], W1 [N1][K1], R and E [M][N1], W2 [N2][N1],
// Y [M][N2]); E is an output too.  This is what the end of one ResNet bottleneck and the start of the next are: the
// expansion 64 -> 256 with the shortcut added, then the reduction 256 -> 64 of the next block.  Run separately, both
// are streams: the first writes E (51 MB at batch 32 on 56 x 56) and the second reads it back to produce a tensor a
// quarter its size.  Here a block takes 16 pixels at a time through both products with E's rows in LDS in between, so
// E is written once and never read, and one launch with its start-up goes away: 28.0-28.4 us against 22.2 + 14.6 us
// inside ResNet-50 at batch 32 (128 MB at 4.6 TB/s).
//
//   * No operand tile is staged and no filter streams: both filters live in registers as MFMA operands for the whole
//     kernel, split by output columns over the block's four wavefronts (wavefront w: the columns w N1 / 4 .. of W1 and
//     w N2 / 4 .. of W2: 32 + 32 registers for 64 -> 256 -> 64).  Blocks are persistent and walk over groups of 16
//     pixels; three of them share a CU and cover each other's barriers and waits.
//   * First product, as in gemm16_shortk_kernel: X's rows are read from global memory straight in fragment layout (16
//     bytes of one row per lane, every wavefront reads the group's rows), v_mfma_f32_16x16x32 computes the transposed
//     tile, so that a lane owns 4 consecutive columns of one pixel; scale and shift are applied and the fp32 values go
//     to an LDS tile [16][N1].  After a barrier all threads walk that tile as whole rows, 8 columns (16 bytes of E)
//     per thread and pass: the shortcut's 16 bytes (requested one group ahead) are added, relu, one rounding to the
//     16-bit type; the 16 bytes go to E in global memory - whole lines per store instruction - and into a second LDS
//     tile [16][N1] of 16-bit values.
//   * Second product: that tile is the pixel operand (one ds_read_b128 per 32 channels; rows 32 bytes over a multiple
//     of 256 apart and the k chunks 0, 2, 1, 3 on the four lane groups, which keeps the sixteen lanes LDS serves
//     together on sixteen bank groups), W2's fragments are the other one; the result's 4 columns per lane turn into
//     whole rows in a third small LDS tile and leave as 16-byte stores.
//   * Sums are formed in the order of the kernels that run the two layers separately (gemm16_shortk_kernel for the
//     first - 32-channel blocks in ascending order on unpermuted k chunks -, gemm16_dma_kernel for the second) and the
//     epilogues are the same arithmetic: the first result is bit-identical to the two-launch form.
//   * K1B > 0: the first product reads K1B more channels of the same pixels from a second tensor X2 [M][K1B] (W1 is then
//     [N1][K1 + K1B]): an expansion and a stride-1 projection shortcut of another tensor as one product, instead of a
//     shortcut tensor of E's size that one kernel writes and this one reads.  No residual in that form.
// Measured and not kept: the same pair one stage later (128 -> 512 -> 128 on 28 x 28: the filters fill half of a CU's
// register file, so one block of eight wavefronts per CU, every barrier and LDS latency exposed) took 27.4-28.2 us
// against 17.5 + 10.5 us for the two launches; a separate wavefront that only loads (rows of X and of the shortcut
// copied straight into LDS two groups ahead, so that the computing wavefronts never wait for a load behind their own
// stores) left that time unchanged and cost the 64-channel form a block per CU (35.5 us).
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

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct ChainParams {
  const uint16_t* x;
  const uint16_t* x2;  // second input of the first product, or null
  const uint16_t* w1;
  const float* scale1;
  const float* shift1;
  const uint16_t* residual;  // may be null
  uint16_t* e;
  const uint16_t* w2;
  const float* scale2;
  const float* shift2;
  uint16_t* y;
  int relu1, relu2;
  int groups;  // M / 16
};

template <typename T, int K1, int N1, int N2, int WAVES, int K1B = 0, bool RES = false>
__global__ void __launch_bounds__(64 * WAVES) conv1x1_chain_kernel(ChainParams p) {
  static_assert(!(RES && K1B > 0), "a second input takes the place of the residual");
  typedef typename Mfma16<T>::vec8 vec8;
  constexpr int THREADS = 64 * WAVES;
  constexpr int KT      = K1 + K1B;            // channels of the first product: X's, then X2's
  constexpr int KB1     = KT / 32;             // 32-channel blocks of the first product
  static_assert(K1 % 32 == 0 && K1B % 32 == 0, "whole 32-channel blocks from either input");
  constexpr int KB2     = N1 / 32;             // ... of the second
  constexpr int J1      = N1 / (16 * WAVES);   // 16-column tiles of E per wavefront
  constexpr int J2      = N2 / (16 * WAVES);   // 16-column tiles of Y per wavefront
  constexpr int kRow32  = (N1 + 4) * 4;        // bytes of a row of the fp32 tile
  constexpr int kRow16  = N1 * 2 + 32;         // bytes of a row of the 16-bit tile
  constexpr int kRowY   = N2 * 2 + 16;
  constexpr int CPR     = N1 / 8;              // 16-byte chunks of E per row
  constexpr int PASSES  = 16 * CPR / THREADS;  // chunks per thread and group
  constexpr int CPY     = N2 / 8;
  static_assert(J1 >= 1 && J2 >= 1 && PASSES >= 1 && THREADS % CPR == 0 && 16 * CPY <= THREADS, "shape");
  __shared__ __attribute__((aligned(16))) char s_f32[16 * kRow32];
  __shared__ __attribute__((aligned(16))) char s_e16[16 * kRow16];
  __shared__ __attribute__((aligned(16))) char s_y16[16 * kRowY];
  __shared__ __attribute__((aligned(16))) float s_sc1[N1], s_sh1[N1], s_sc2[N2], s_sh2[N2];

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  for (int i = tid; i < N1; i += THREADS) {
    s_sc1[i] = p.scale1 ? p.scale1[i] : 1.0f;
    s_sh1[i] = p.shift1 ? p.shift1[i] : 0.0f;
  }
  for (int i = tid; i < N2; i += THREADS) {
    s_sc2[i] = p.scale2 ? p.scale2[i] : 1.0f;
    s_sh2[i] = p.shift2 ? p.shift2[i] : 0.0f;
  }
  const int frow = lane & 15;                                     // row of the fragment this lane holds
  const int g4   = lane >> 4;                                     // lane group
  const int fk1  = g4 * 8;                                        // first product: k chunks 0, 1, 2, 3
  const int fk2  = (((lane >> 4) & 1) * 2 + (lane >> 5)) * 8;     // second: 0, 2, 1, 3
  const int c1   = wave * (N1 / WAVES);                           // this wavefront's first column of E
  const int c2   = wave * (N2 / WAVES);                           // ... of Y
  vec8 wf1[J1][KB1];
  vec8 wf2[J2][KB2];
#pragma unroll
  for (int j = 0; j < J1; ++j)
#pragma unroll
    for (int kb = 0; kb < KB1; ++kb)
      wf1[j][kb] = *reinterpret_cast<const vec8*>(p.w1 + (int64_t)(c1 + 16 * j + frow) * KT + 32 * kb + fk1);
#pragma unroll
  for (int j = 0; j < J2; ++j)
#pragma unroll
    for (int kb = 0; kb < KB2; ++kb)
      wf2[j][kb] = *reinterpret_cast<const vec8*>(p.w2 + (int64_t)(c2 + 16 * j + frow) * N1 + 32 * kb + fk2);
  // the filter fragments are complete before the loop starts (left to the compiler, the waits for them would sit at
  // their first use inside the loop, where they would also wait for the rows just requested)
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
  for (int j = 0; j < J1; ++j)
#pragma unroll
    for (int kb = 0; kb < KB1; ++kb) asm volatile("" : "+v"(wf1[j][kb]));
#pragma unroll
  for (int j = 0; j < J2; ++j)
#pragma unroll
    for (int kb = 0; kb < KB2; ++kb) asm volatile("" : "+v"(wf2[j][kb]));
  __syncthreads();

  int g = blockIdx.x;
  if (g >= p.groups) return;
  // whether there is a residual is a template parameter: with a run-time condition around its loads the compiler
  // cannot count the loads in flight (see the request below)
  const T* const R = RES ? reinterpret_cast<const T*>(p.residual) : nullptr;
  T* const E       = reinterpret_cast<T*>(p.e);
  T* const Y       = reinterpret_cast<T*>(p.y);
  // a thread's chunk of pass i: row i (THREADS / CPR) + tid / CPR of the group, columns 8 (tid % CPR) ..
  const int ch_row = tid / CPR, ch_col = (tid % CPR) * 8;
  auto request = [&](int grp, vec8* xa, vec8* rr) {
    const uint16_t* const x_g = p.x + (int64_t)grp * 16 * K1;
#pragma unroll
    for (int kb = 0; kb < K1 / 32; ++kb) xa[kb] = *reinterpret_cast<const vec8*>(x_g + frow * K1 + 32 * kb + fk1);
    if (K1B > 0) {
      const uint16_t* const x2_g = p.x2 + (int64_t)grp * 16 * K1B;
#pragma unroll
      for (int kb = 0; kb < K1B / 32; ++kb) xa[K1 / 32 + kb] = *reinterpret_cast<const vec8*>(x2_g + frow * K1B + 32 * kb + fk1);
    }
    if (R) {
      const T* const r_g = R + (int64_t)grp * 16 * N1;
#pragma unroll
      for (int i = 0; i < PASSES; ++i)
        rr[i] = *reinterpret_cast<const vec8*>(r_g + (i * (THREADS / CPR) + ch_row) * N1 + ch_col);
    }
  };
  vec8 xa[2][KB1];
  vec8 rr[2][PASSES];
  request(g, xa[0], rr[0]);
  for (;;) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int gn        = g + (int)gridDim.x;
      const bool has_next = gn < p.groups;
      // Requested whether or not there is a next group (then the last group's rows once more, unused): with a request
      // that depends on a condition the compiler cannot count the loads in flight at the first use of this group's
      // rows and waits for all of them - the ones requested a moment ago included, i.e. no group is ever fetched ahead
      request(has_next ? gn : p.groups - 1, xa[u ^ 1], rr[u ^ 1]);
      // ---- first product: this wavefront's J1 tiles of the group's 16 pixels
      f32x4 acc1[J1];
#pragma unroll
      for (int j = 0; j < J1; ++j) acc1[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kb = 0; kb < KB1; ++kb)
#pragma unroll
        for (int j = 0; j < J1; ++j) acc1[j] = Mfma16<T>::mma(wf1[j][kb], xa[u][kb], acc1[j]);
#pragma unroll
      for (int j = 0; j < J1; ++j) {
        const int col  = c1 + 16 * j + 4 * g4;
        const f32x4 sc = *reinterpret_cast<const f32x4*>(&s_sc1[col]);
        const f32x4 sh = *reinterpret_cast<const f32x4*>(&s_sh1[col]);
        f32x4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = __builtin_fmaf(acc1[j][r], sc[r], sh[r]);
        *reinterpret_cast<f32x4*>(s_f32 + frow * kRow32 + col * 4) = v;
      }
      BarrierLds();
      // ---- E as whole rows: shortcut, relu, one rounding; to global memory and into the 16-bit tile
      T* const e_g = E + (int64_t)g * 16 * N1;
#pragma unroll
      for (int i = 0; i < PASSES; ++i) {
        const int row  = i * (THREADS / CPR) + ch_row;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(s_f32 + row * kRow32 + ch_col * 4);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(s_f32 + row * kRow32 + ch_col * 4 + 16);
        float t[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          t[q] = q < 4 ? lo[q] : hi[q - 4];
          if (R) t[q] = __builtin_fmaf(1.0f, (float)rr[u][i][q], t[q]);
          const float m = __builtin_fmaxf(t[q], 0.0f);  // a NaN becomes 0, as with v > 0 ? v : 0
          t[q]          = p.relu1 ? m : t[q];
          asm volatile("" : "+v"(t[q]));
        }
        const u32x4 out = {PackPair<T>(t[0], t[1]), PackPair<T>(t[2], t[3]), PackPair<T>(t[4], t[5]), PackPair<T>(t[6], t[7])};
        *reinterpret_cast<u32x4*>(e_g + row * N1 + ch_col)           = out;
        *reinterpret_cast<u32x4*>(s_e16 + row * kRow16 + ch_col * 2) = out;
      }
      BarrierLds();
      // ---- second product: all N1 channels of the 16 pixels against this wavefront's J2 tiles of W2
      f32x4 acc2[J2];
#pragma unroll
      for (int j = 0; j < J2; ++j) acc2[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kb = 0; kb < KB2; ++kb) {
        const vec8 eb = *reinterpret_cast<const vec8*>(s_e16 + frow * kRow16 + (32 * kb + fk2) * 2);
#pragma unroll
        for (int j = 0; j < J2; ++j) acc2[j] = Mfma16<T>::mma(wf2[j][kb], eb, acc2[j]);
      }
#pragma unroll
      for (int j = 0; j < J2; ++j) {
        const int col  = c2 + 16 * j + 4 * g4;
        const f32x4 sc = *reinterpret_cast<const f32x4*>(&s_sc2[col]);
        const f32x4 sh = *reinterpret_cast<const f32x4*>(&s_sh2[col]);
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v[r]          = __builtin_fmaf(acc2[j][r], sc[r], sh[r]);
          const float m = __builtin_fmaxf(v[r], 0.0f);
          v[r]          = p.relu2 ? m : v[r];
          asm volatile("" : "+v"(v[r]));
        }
        const u32x2 out = {PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3])};
        *reinterpret_cast<u32x2*>(s_y16 + frow * kRowY + col * 2) = out;
      }
      BarrierLds();
      if (tid < 16 * CPY) {
        const int row = tid / CPY, col = (tid % CPY) * 8;
        *reinterpret_cast<u32x4*>(Y + ((int64_t)g * 16 + row) * N2 + col) =
            *reinterpret_cast<const u32x4*>(s_y16 + row * kRowY + col * 2);
      }
      if (!has_next) return;
      g = gn;
    }
  }
}

template <typename T, int K1, int N1, int N2, int WAVES, int BLOCKS_PER_CU, int K1B = 0>
void LaunchChain(const ChainParams& p, hipStream_t stream) {
  const int resident = 256 * BLOCKS_PER_CU;
  dim3 grid(p.groups < resident ? p.groups : resident);
  if (K1B == 0 && p.residual != nullptr) {
    hipLaunchKernelGGL((conv1x1_chain_kernel<T, K1, N1, N2, WAVES, 0, true>), grid, dim3(64 * WAVES), 0, stream, p);
  } else {
    hipLaunchKernelGGL((conv1x1_chain_kernel<T, K1, N1, N2, WAVES, K1B, false>), grid, dim3(64 * WAVES), 0, stream, p);
  }
}

// 1: where the shape qualifies (default), 0: never; -1: not read yet
std::atomic<int> g_chain_mode{-1};

int ChainMode() {
  int mode = g_chain_mode.load(std::memory_order_relaxed);
  if (mode < 0) {
    const char* v = getenv("FLAGS_cinn_hip_conv_chain");
    mode          = v && *v ? (atoi(v) != 0) : 1;
    g_chain_mode.store(mode, std::memory_order_relaxed);
  }
  return mode;
}

}  // namespace

bool ConvChainShape(int64_t m, int k1, int n1, int n2) {
  if (m <= 0 || m % 16 != 0 || m * n1 >= INT_MAX) return false;
  return k1 == 64 && n1 == 256 && (n2 == 64 || n2 == 128);
}

bool ConvChainShape2(int64_t m, int k1, int k1b, int n1, int n2) {
  if (m <= 0 || m % 16 != 0 || m * n1 >= INT_MAX) return false;
  return k1 == 64 && k1b == 64 && n1 == 256 && n2 == 64;
}

bool TryConvChain(const ConvChainArgs& a, hipStream_t stream) {
  if (!ChainMode()) return false;
  const bool is_f16  = a.type.code == cinn_type_float && a.type.bits == 16;
  const bool is_bf16 = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if (!is_f16 && !is_bf16) return false;
  if (a.x2 != nullptr) {
    if (a.residual != nullptr || !ConvChainShape2(a.m, a.k1, a.k1b, a.n1, a.n2)) return false;
  } else if (!ConvChainShape(a.m, a.k1, a.n1, a.n2)) {
    return false;
  }
  const void* ptrs[] = {a.x, a.x2, a.w1, a.residual, a.e, a.w2, a.y};
  for (const void* ptr : ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return false;
  ChainParams p;
  p.x = static_cast<const uint16_t*>(a.x), p.x2 = static_cast<const uint16_t*>(a.x2), p.w1 = static_cast<const uint16_t*>(a.w1);
  p.scale1 = a.scale1, p.shift1 = a.shift1, p.residual = static_cast<const uint16_t*>(a.residual);
  p.e = static_cast<uint16_t*>(a.e), p.w2 = static_cast<const uint16_t*>(a.w2);
  p.scale2 = a.scale2, p.shift2 = a.shift2, p.y = static_cast<uint16_t*>(a.y);
  p.relu1 = a.relu1 ? 1 : 0, p.relu2 = a.relu2 ? 1 : 0;
  p.groups = static_cast<int>(a.m / 16);
#define CINN_CHAIN(K1, N1, N2, WAVES, BPC)                      \
  do {                                                          \
    if (is_bf16) {                                              \
      LaunchChain<__bf16, K1, N1, N2, WAVES, BPC>(p, stream);   \
    } else {                                                    \
      LaunchChain<_Float16, K1, N1, N2, WAVES, BPC>(p, stream); \
    }                                                           \
  } while (0)
  if (a.x2 != nullptr) {
    if (is_bf16) {
      LaunchChain<__bf16, 64, 256, 64, 4, 2, 64>(p, stream);  // twice the filter registers of the first product: two blocks per CU
    } else {
      LaunchChain<_Float16, 64, 256, 64, 4, 2, 64>(p, stream);
    }
  } else if (a.n2 == 64) {
    CINN_CHAIN(64, 256, 64, 4, 3);   // 163 registers: three blocks per CU
  } else {
    CINN_CHAIN(64, 256, 128, 4, 2);  // 200 registers: two
  }
#undef CINN_CHAIN
  CINN_HIP_CALL(hipGetLastError());
  return true;
}

}  // namespace cinn_hip_kernels

extern "C" int cinn_hip_conv_chain_mode(int mode) {
  const int before = cinn_hip_kernels::ChainMode();
  if (mode == 0 || mode == 1) cinn_hip_kernels::g_chain_mode.store(mode, std::memory_order_relaxed);
  return before;
}
