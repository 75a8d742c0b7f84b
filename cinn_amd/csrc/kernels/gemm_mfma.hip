// Hand-written CDNA4 (gfx950) GEMM kernels behind cinn_call_cublas / cinn_call_batched_cublas.
//
//   C[M,N] = alpha * op(A)[M,K] * op(B)[K,N] + beta * C          (row-major, optional batch)
//
// Kernels:
//   * gemm16_dma_kernel   - bf16 / fp16 with A stored [M][K] (the common case) and K % 64 == 0, on
//     v_mfma_f32_16x16x32: 256x256x64 tile, 512 threads, direct global -> LDS loads of whole 128-byte lines into two
//     stages, transposing LDS reads for row-major B; also as 128x128 tiles (two or four stages) and 256x64 tiles, and
//     with the A operand gathered from a channels-last image (implicit-GEMM convolution); see the comment at the kernel.
//   * gemm16_mfma_kernel  - bf16 / fp16 inputs, any operand layout (used for transposed A), fp32 accumulation on v_mfma_f32_32x32x16_{bf16,f16}.
//     256x256 block tile, 64-deep K step, 256 threads = 4 wavefronts in a 2x2 grid, each wavefront owning a
//     128x128 tile (16 MFMA accumulator tiles = 256 accumulator registers).  Both operand tiles live in LDS
//     as [row][k] with k contiguous, 128 bytes per row, double buffered (2 x 64 KiB of the 160 KiB per CU);
//     16-byte chunks are XOR-swizzled so that the ds_read_b128 of MFMA fragments and the transposing stores
//     are conflict free.  Operands whose contiguous axis is not K (row-major B, transposed A) are transposed
//     in registers (8x8 blocks of 16-bit values) on their way into LDS.  Requires M%256 == N%256 == K%64 == 0.
//   * gemm32_mfma_kernel  - fp32 on v_mfma_f32_32x32x2f32, 128x128 tile (64x64 when that is what fills the chip),
//     for M%128 == N%128 == K%32 == 0.
//   * gemm_generic_kernel - any shape / transpose / type (fp16, bf16, fp32, fp64): 64x64 LDS tile, FMA units.
// Shapes the tile kernels do not take (ragged, or too few tiles to fill the chip) run on the bounds-checked MFMA
// kernel of conv_nhwc_mfma.hip as a 1x1 convolution, after transposing copies of the operands that are not
// K-contiguous (transpose2d_kernel); gemm_generic_kernel is left with K % (16 bytes) != 0 and fp64.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include <climits>
#include <cstdint>
#include <map>
#include <mutex>

#include "cinn_hip_runtime.h"
#include "kernels/conv_nhwc.h"
#include "runtime/hip_check.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

template <typename T>
struct Half16;
template <>
struct Half16<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Half16<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// two fp32 values rounded to nearest even into one dword of two T (v_cvt_pk_f16_f32 / v_cvt_pk_bf16_f32)
template <typename T>
__device__ __forceinline__ uint32_t PackPair(float a, float b) {
  typedef T pair_t __attribute__((ext_vector_type(2)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, pair_t));
}

constexpr int kBM      = 256;
constexpr int kBN      = 256;
constexpr int kBK      = 64;
constexpr int kThreads = 256;
// one operand tile: 256 rows x 64 halves = 256 x 128 bytes
constexpr int kTileBytes  = kBM * kBK * 2;
constexpr int kStageBytes = 2 * kTileBytes;  // A tile + B tile

// byte offset of 16-byte chunk `chunk` (0..7) of row `row` inside an operand tile
__device__ __forceinline__ int TileOffset(int row, int chunk) {
  int key = (row ^ (row >> 3)) & 7;
  return row * 128 + ((chunk ^ key) << 4);
}

// 8x8 transpose of 16-bit values held as 8 rows of 4 dwords: out[c] = column c of in
__device__ __forceinline__ void Transpose8x8(const u32x4 (&in)[8], u32x4 (&out)[8]) {
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int d  = c >> 1;  // dword that holds column c
    const bool hi = c & 1;  // upper half of that dword
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
      unsigned a = in[2 * rp][d];
      unsigned b = in[2 * rp + 1][d];
      // low half from row 2rp, high half from row 2rp+1
      out[c][rp] = hi ? __builtin_amdgcn_perm(b, a, 0x07060302u) : __builtin_amdgcn_perm(b, a, 0x05040100u);
    }
  }
}

// Global -> register staging of one 256-row operand tile, two access patterns.
// K_CONTIG: the operand is [rows][K] in memory (K contiguous): thread t copies chunk (t & 7) of rows
//           (t >> 3) + 32 i.  Otherwise the operand is [K][rows] (rows contiguous): thread t owns the 8x8
//           block at k-block (t >> 5), row-block (t & 31) and transposes it.
template <bool K_CONTIG>
struct TileLoader {
  u32x4 regs[8];
  __device__ __forceinline__ void Load(const uint16_t* __restrict__ base, int64_t ld, int row0, int k0, int tid) {
    if (K_CONTIG) {
      const uint16_t* p = base + (int64_t)(row0 + (tid >> 3)) * ld + k0 + (tid & 7) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) regs[i] = *reinterpret_cast<const u32x4*>(p + (int64_t)(32 * i) * ld);
    } else {
      const uint16_t* p = base + (int64_t)(k0 + (tid >> 5) * 8) * ld + row0 + (tid & 31) * 8;
#pragma unroll
      for (int r = 0; r < 8; ++r) regs[r] = *reinterpret_cast<const u32x4*>(p + (int64_t)r * ld);
    }
  }
  __device__ __forceinline__ void Store(char* tile, int tid) {
    if (K_CONTIG) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *reinterpret_cast<u32x4*>(tile + TileOffset((tid >> 3) + 32 * i, tid & 7)) = regs[i];
    } else {
      u32x4 t[8];
      Transpose8x8(regs, t);
#pragma unroll
      for (int c = 0; c < 8; ++c) *reinterpret_cast<u32x4*>(tile + TileOffset((tid & 31) * 8 + c, tid >> 5)) = t[c];
    }
  }
};

// A_KC: A is stored [M][K] (not transposed).  B_KC: B is stored [N][K] (transposed).
template <typename T, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(kThreads)
gemm16_mfma_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C, int M, int N,
                   int K, int64_t lda, int64_t ldb, int64_t ldc, float alpha, float beta, int64_t stride_a,
                   int64_t stride_b, int64_t stride_c) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename Half16<T>::vec8 vec8;

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm   = wave >> 1;  // wavefront row in the 2x2 grid
  const int wn   = wave & 1;

  // XCD-aware tile order: consecutive workgroup ids go to different XCDs (8 of them, each with its own L2), so
  // give every XCD a contiguous band of tiles that share A row panels
  const int tiles_n = N / kBN;
  const int tiles   = (M / kBM) * tiles_n;
  int bid           = blockIdx.x;
  if ((tiles & 7) == 0) bid = (bid & 7) * (tiles >> 3) + (bid >> 3);
  const int m0 = (bid / tiles_n) * kBM;
  const int n0 = (bid % tiles_n) * kBN;

  A += (int64_t)blockIdx.y * stride_a;
  B += (int64_t)blockIdx.y * stride_b;
  C += (int64_t)blockIdx.y * stride_c;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  TileLoader<A_KC> la;
  TileLoader<B_KC> lb;
  const int kt_count = K / kBK;

  la.Load(A, lda, m0, 0, tid);
  lb.Load(B, ldb, n0, 0, tid);
  la.Store(lds, tid);
  lb.Store(lds + kTileBytes, tid);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_kg  = lane >> 5;

  for (int kt = 0; kt < kt_count; ++kt) {
    char* cur = lds + (kt & 1) * kStageBytes;
    char* nxt = lds + ((kt + 1) & 1) * kStageBytes;
    const bool more = kt + 1 < kt_count;
    if (more) {
      la.Load(A, lda, m0, (kt + 1) * kBK, tid);
      lb.Load(B, ldb, n0, (kt + 1) * kBK, tid);
    }
    const char* a_tile = cur;
    const char* b_tile = cur + kTileBytes;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      vec8 af[4], bf[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        af[t] = *reinterpret_cast<const vec8*>(a_tile + TileOffset(wm * 128 + t * 32 + frag_row, kk * 2 + frag_kg));
        bf[t] = *reinterpret_cast<const vec8*>(b_tile + TileOffset(wn * 128 + t * 32 + frag_row, kk * 2 + frag_kg));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Half16<T>::mfma(af[i], bf[j], acc[i][j]);
    }
    if (more) {
      la.Store(nxt, tid);
      lb.Store(nxt + kTileBytes, tid);
    }
    __syncthreads();
  }

  // epilogue: accumulator element r of lane l sits at row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its tile
  T* Ct = reinterpret_cast<T*>(C);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn * 128 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        T* dst  = Ct + (int64_t)row * ldc + col;
        float v = alpha * acc[i][j][r];
        if (beta != 0.0f) v += beta * (float)*dst;
        *dst = (T)v;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// bf16 / fp16 with A stored [M][K]: direct global -> LDS loads (global_load_lds_dwordx4), 8 wavefronts.
// 256x256 block tile, K step 64, 512 threads in a 2 (M) x 4 (N) wavefront grid, each wavefront a 128x64 tile = 8 x 4
// accumulators of v_mfma_f32_16x16x32 (measured on sustained MFMA-only loops with random operands: 2.14 PFLOP/s
// with 16x16x32 against 1.92 with 32x32x16 - the chip is power limited and the narrow shape moves less accumulator
// data per flop), two wavefronts per SIMD.
//   * Every row of an operand tile is one whole 128-byte line.  With a K step of 32 (64-byte rows) the vector L1
//     fetches every line twice from L2, one step apart, and that fill traffic bounds the feed: measured 32 bytes per
//     clock and CU with 64-byte rows against 48-51 with 128-byte rows.
//   * A lane of a load instruction writes its 16 bytes at LDS base + 16 * lane, so the swizzle that makes the fragment
//     reads conflict free is applied on the global side: each lane fetches the chunk that belongs at its LDS slot.
//     A load instruction covers 8 rows x 128 bytes.  Its address is a scalar base (stepped along K with scalar adds)
//     plus a fixed 32-bit offset per lane.
//   * 16-byte LDS reads are served eight lanes of each wavefront half at a time (lanes 8p..8p+7 together with
//     32+8p..32+8p+7; found by counting bank conflicts): the fragment layout gives those sixteen lanes sixteen
//     different 16-byte bank groups (SQ_LDS_BANK_CONFLICT = 0).
//   * B stored [K][N] (the plain row-major matmul) is kept as [k][n] in LDS ([64 k][512 B], a load instruction
//     covers 2 k-rows) and read with ds_read_b64_tr_b16, which hands every lane four consecutive k of one column -
//     no transposition in registers.
//   * NS stages (two of 64 KiB for the 256x256 tile) and one barrier per K step, three MFMA rows (12 MFMAs) before the step's end: by then every
//     fragment of stage s is in registers, so those rows cover the first fragment reads of stage s+1, and stage s's
//     slot is free for the loads of stage s+2, spread over the three rows after the barrier and the first rows of
//     the next step (about the rate at which the vector memory path drains them); they are waited for at the barrier
//     of step s+1.  Of the two wavefronts of a SIMD the older one runs ahead and then waits at the barrier: it issues
//     the loads of both.
//   * A fragments in a ring of four (requested three rows ahead), B fragments in two sets; scheduling barriers pin
//     the order.  The main loop has no branches: the last one to three steps, which have nothing left to request,
//     are peeled.
//   * The result tile goes through LDS (two passes of 128 rows) so that a store instruction covers two whole 512-byte
//     rows of C.
// In core clocks a K step takes about 2330 clocks for 2048 of MFMA at 4096^3 (the rest: the slower wavefront of each
// SIMD waiting for its loads and the barrier, about 190 clocks, and issue gaps); what the kernel delivers beyond that
// is set by the clock the chip sustains under this load (1.7-1.9 GHz measured against the 2.4 GHz of the quoted peak).
// Requires M % BM == N % BN == K % 64 == 0.
// ---------------------------------------------------------------------------------------------------
constexpr int kDmaThreads = 512;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// Direct global -> LDS loads: 16 bytes per lane, written at LDS address m0 + 16 * lane (+ the instruction offset).
// Inline assembly, so that the compiler does not track these loads: tracked, they get a conservative
// s_waitcnt vmcnt(0) before every LDS read.
// The address is split into a wave-uniform base (scalar registers) and a 32-bit byte offset per lane,
// so that stepping along K costs scalar additions only.  IMM is added to both the global address and the LDS address:
// the loads of one operand tile use one m0 (SetLdsBase) and differ in IMM (a multiple of 1 KiB, below 4 KiB).
__device__ __forceinline__ void SetLdsBase(unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(lds_addr_uniform) : "memory");
}
// the same for a load with a full 64-bit address per lane
__device__ __forceinline__ void AsyncCopy16To(const void* src, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr_uniform), "v"(src) : "memory");
}
template <int IMM>
__device__ __forceinline__ void AsyncCopy16At(const void* base_uniform, unsigned lane_offset) {
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" : : "v"(lane_offset), "s"(base_uniform), "n"(IMM) : "memory");
}
__device__ __forceinline__ void AsyncCopy16Slot(const void* base_uniform, unsigned lane_offset, int slot) {
  switch (slot) {
    case 0: AsyncCopy16At<0>(base_uniform, lane_offset); break;
    case 1: AsyncCopy16At<1024>(base_uniform, lane_offset); break;
    case 2: AsyncCopy16At<2048>(base_uniform, lane_offset); break;
    default: AsyncCopy16At<3072>(base_uniform, lane_offset); break;
  }
}

constexpr int kD64BK   = 64;
constexpr int kD64Tile = kBM * kD64BK * 2;  // one operand tile of a stage: 32 KiB

// epilogue operands of gemm16_dma_kernel: v = acc * (scale[col] or alpha) + shift[col] + residual_scale * R, relu
struct DmaEpilogue {
  const float* scale;     // per output column, or null: alpha
  const float* shift;     // per output column, or null
  const void* residual;   // [M][N] like C (may be C itself: the beta term of a GEMM), or null
  float alpha;
  float residual_scale;
  int relu;
  int streaming;          // store the result with non-temporal stores (large outputs nobody re-reads from L2)
  // Split reduction: blockIdx.z = s takes the K steps [s * steps_per_split, (s + 1) * steps_per_split) and writes its
  // raw fp32 sums to partials[s][M][N]; the epilogue is applied by gemm16_split_reduce_kernel.  Null: no split.
  float* partials;
  int steps_per_split;
  // Measurement hook (cinn_hip_gemm_set_probe): when set, thread 0 of every block writes eight 64-bit words at
  // probe + 8 * (linear block index) - the constant 100 MHz clock and the core clock counter at block start, after the
  // first operands have landed, after the K loop and after the last store was issued.  Null in normal use.
  unsigned long long* probe = nullptr;
};

// `first_wave` must be wavefront-uniform (a scalar branch: a lane-dependent one ahead of the direct-to-LDS loads makes
// the compiler move their scalar base addresses into vector registers, which the instruction does not take); every
// lane of that wavefront stores the same words to the same address.
__device__ __forceinline__ void ProbeStamp(unsigned long long* probe, bool first_wave, int slot) {
  if (probe && first_wave) {
    unsigned long long* at = probe + 8 * (blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) + 2 * slot;
    at[0] = __builtin_amdgcn_s_memrealtime();
    at[1] = __builtin_readcyclecounter();
  }
}

// Implicit-GEMM view of a channels-last convolution for gemm16_dma_kernel<.., CONV = true>: row m of A is output pixel
// m = (n, oy, ox), K runs over (dy, dx, c) with c contiguous; a 64-deep K step lies inside one filter tap (the channel
// count is a multiple of 64), so a load instruction still fetches whole 128-byte lines: 64 channels of one input pixel,
// or, outside the image, zeros from `zero_page`.
struct ConvGeom {
  int h, w, c;          // input extents (NHWC)
  int oh_ow, ow;        // output plane
  int kw;               // filter width (dy = tap / kw)
  int stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  const void* zero_page;  // at least 128 bytes of zeros
  // A second channels-last input read through a 1x1 window (no padding) on the same output grid, or null: after the
  // first steps1 K steps (all taps and channels of the first input) the K loop goes on over its c2 channels, pixel
  // (oy stride2_h, ox stride2_w) for output pixel (oy, ox); the filter rows are [first input's K | c2] accordingly.
  const void* x2;
  int h2, w2, c2, stride2_h, stride2_w;
  int steps1;
};

// BM x BN block tile on a WAVES_M x WAVES_N grid of wavefronts: 256x256 on 2x4 (8 wavefronts of 128x64) for large
// problems, 128x128 on 2x2 (4 wavefronts of 64x64, two blocks per CU) when 256x256 tiles would leave CUs idle.
// FEED: the block carries WAVES_M x WAVES_N more wavefronts that only issue the direct-to-LDS loads, wait for them and
// take part in the barriers, while the first WAVES_M x WAVES_N only compute.  A wavefront that issues a load
// instruction stalls until the address unit has taken it (about 16 clocks per KiB and CU), and with one computing
// wavefront per SIMD nobody else is there to issue MFMAs meanwhile: measured on the 128x128 tile (four stages,
// implicit GEMM, K = 4608) a K step took 1102 clocks for 512 of MFMA with the loads issued by the computing
// wavefronts and 531 without any loads.
// PAIR (with CONV): the convolution has a second input (ConvGeom::x2) whose channels continue the K loop.
template <typename T, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool CONV = false, int NS = 2, bool FEED = false,
          bool PAIR = false>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N * (FEED ? 2 : 1))
gemm16_dma_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* C, int M, int N, int K,
                  int64_t lda, int64_t ldb, int64_t ldc, DmaEpilogue epi, int64_t stride_a, int64_t stride_b,
                  int64_t stride_c, int xcd_cols, int sub_rows, int sub_cols, ConvGeom geom) {
  constexpr int NW      = WAVES_M * WAVES_N;                // computing wavefronts
  constexpr int THREADS = 64 * NW * (FEED ? 2 : 1);
  constexpr int TM      = BM / WAVES_M / 16;  // 16x16 accumulator tiles per wavefront along M and N
  constexpr int TN      = BN / WAVES_N / 16;
  constexpr int A_TILE  = BM * kD64BK * 2;    // bytes of one operand tile of a stage
  constexpr int B_TILE  = BN * kD64BK * 2;
  // With two wavefronts per SIMD the older one of each pair (wavefronts 0 .. NW/2-1) wins the MFMA arbitration, runs
  // ahead and then waits at the step's barrier; it issues all the loads (their issue stalls cost it nothing), so the
  // younger one, which the barrier waits for, has no loads to issue or wait for.
  constexpr int LW      = FEED ? NW : ((TM == 8 && !CONV) ? NW / 2 : NW);  // wavefronts that issue loads
  constexpr int LPA     = BM / 8 / LW;                        // loads (of 1 KiB per wavefront) per thread, operand and step
  constexpr int LPB     = BN / 8 / LW;
  static_assert(LPA >= 1 && LPB >= 1 && LPA <= 8 && LPB <= 8 && TM % 4 == 0 && TN == 4, "unsupported tile shape");
  constexpr int STAGE = A_TILE + B_TILE;
  // PAIR: behind the stages, every thread parks its offsets into the second input until the K loop gets there
  // (registers are what the 256x256 tile has none left of)
  constexpr int STASH = PAIR ? THREADS * LPA * 8 : 0;
  static_assert(!PAIR || CONV, "a second input belongs to a convolution");
  static_assert(NS >= 2 && NS * STAGE + STASH <= 160 * 1024, "the stages do not fit LDS");
  __shared__ __attribute__((aligned(1024))) char lds[NS * STAGE + STASH];
  const unsigned lds_addr =
      __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)lds);
  // stage s lives in slot s % NS
  auto sa = [&](int slot) -> char* { return lds + slot * STAGE; };
  auto sb = [&](int slot) -> char* { return lds + slot * STAGE + A_TILE; };
  typedef typename Half16<T>::vec8 vec8;
  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool feeder = FEED && wave >= NW;  // loads only
  const int wm   = (wave % NW) / WAVES_N;
  const int wn   = (wave % NW) % WAVES_N;

  int tile_row, tile_col;
  if (sub_rows > 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    tile_row = (xcd / xcd_cols) * sub_rows + idx / sub_cols;
    tile_col = (xcd % xcd_cols) * sub_cols + idx % sub_cols;
  } else {
    const int tiles_n = (N + BN - 1) / BN;
    tile_row = blockIdx.x / tiles_n;
    tile_col = blockIdx.x % tiles_n;
  }
  const int m0 = tile_row * BM;
  const int n0 = tile_col * BN;
  if (m0 >= M || n0 >= N) return;  // padding of the XCD rectangles (the whole block leaves)
  A += (int64_t)blockIdx.y * stride_a;
  B += (int64_t)blockIdx.y * stride_b;
  C += (int64_t)blockIdx.y * stride_c;
  ProbeStamp(epi.probe, wave == 0, 0);

  // Load q = LPA wave + t of an operand fills LDS bytes [1024 q, 1024 q + 1024) of its tile: 8 rows of a
  // [row][64 halves] tile, or 512 / BN k-rows of a [k][BN halves] tile.
  // GEMM operands: byte offset of the lane's chunk from the tile's first row (A, B stored [N][K]) or from column n0
  // of row 0 (B stored [K][N]), less the instruction offset 1024 t of load t (which the LDS address needs)
  // (an instruction offset is below 4 KiB: loads t and t + 4 differ in m0 instead)
  unsigned a_off[LPA], b_off[LPB];
  const bool loader = FEED ? feeder : (LW == NW || wave < LW);
  const int lwave   = loader ? (FEED ? wave - NW : wave) : 0;
  // The last tile row / column may reach beyond M / N: its lanes fetch the last valid row (or 8-column chunk)
  // instead - what they compute is not stored.  The bases lie kBias bytes below the tile and every lane offset
  // includes kBias, so that an offset less its instruction offset never wraps below zero.
  constexpr int kBias = 4096;
  // this block's K steps: all of them, or the split's share
  const int kt0 = epi.partials ? (int)blockIdx.z * epi.steps_per_split : 0;
  const int64_t b_step = (B_KC ? kD64BK : (int64_t)kD64BK * ldb) * 2;  // bytes per K step
  const char* const a_base = reinterpret_cast<const char*>(A + (int64_t)m0 * lda) - kBias + (int64_t)kt0 * (kD64BK * 2);
  const char* const b_base =
      reinterpret_cast<const char*>(B + (B_KC ? (int64_t)n0 * ldb : (int64_t)n0)) - kBias + kt0 * b_step;
  const int a_last = M - 1 - m0;  // last valid row of this tile (>= 0)
  const int b_last = N - 1 - n0;
  // CONV: a_off is the byte offset of the lane's chunk at the top-left corner of the pixel's window (it may lie before
  // the image: the tap's offset is added modulo 2^32), a_yx that corner's coordinates, 16 bits each
  int a_yx[LPA];
  // CONV: the input the loads are reading (the second one of a pair takes over after geom.steps1 steps), and the
  // lane's offsets and window corners in the second input
  const char* src = reinterpret_cast<const char*>(A);
  int src_h = geom.h, src_w = geom.w, src_c = geom.c;
  int steps_to_switch = PAIR ? geom.steps1 : -1;
  unsigned* const stash = reinterpret_cast<unsigned*>(lds + NS * STAGE) + tid;  // word i of a thread: stash[i THREADS]
#pragma unroll
  for (int t = 0; t < LPA; ++t) {
    const int row = 8 * (lwave * LPA + t) + (lane >> 3);
    const int key = (row & 7) ^ ((row >> 3) & 1);  // chunk swizzle of a [row][64 halves] tile, see the fragment reads
    if (CONV) {
      const int pixel = m0 + row;
      const int n     = pixel / geom.oh_ow;
      const int rem   = pixel - n * geom.oh_ow;
      const int oy    = rem / geom.ow;
      const int ox    = rem - oy * geom.ow;
      const int iy0   = oy * geom.stride_h - geom.pad_h;
      const int ix0   = ox * geom.stride_w - geom.pad_w;
      // a pixel beyond the last one gets a window that starts far above the image: every tap reads zeros
      a_yx[t]         = pixel < M ? (iy0 & 0xffff) | (ix0 << 16) : 0x8000;
      a_off[t]        = ((unsigned)((n * geom.h + iy0) * geom.w + ix0) * (unsigned)geom.c + (((lane & 7) ^ key) << 3)) * 2u;
      if (PAIR) {
        const int iy2 = oy * geom.stride2_h;
        const int ix2 = ox * geom.stride2_w;
        stash[(2 * t) * THREADS]     = pixel < M ? (iy2 & 0xffff) | (ix2 << 16) : 0x8000;
        stash[(2 * t + 1) * THREADS] = ((unsigned)((n * geom.h2 + iy2) * geom.w2 + ix2) * (unsigned)geom.c2 + (((lane & 7) ^ key) << 3)) * 2u;
      }
    } else {
      const int row_c = row < a_last ? row : a_last;
      a_off[t] = (unsigned)(((int64_t)row_c * lda + (((lane & 7) ^ key) << 3)) * 2 + kBias - 1024 * (t & 3));
    }
  }
  // CONV: filter tap and first channel of the K step whose loads are being issued (all loads of one step are issued
  // between two advances)
  int tap_dy = 0, tap_dx = 0, tap_c0 = 0;
  if (CONV && kt0 > 0) {
    const int k0  = kt0 * kD64BK;
    const int tap = k0 / geom.c;
    tap_c0        = k0 - tap * geom.c;
    tap_dy        = tap / geom.kw;
    tap_dx        = tap - tap_dy * geom.kw;
  }
  auto advance_tap = [&]() {
    tap_c0 += kD64BK;
    if (tap_c0 == src_c) {
      tap_c0 = 0;
      if (++tap_dx == geom.kw) {
        tap_dx = 0;
        ++tap_dy;
      }
    }
    if (PAIR && --steps_to_switch == 0) {  // the first input is through: the second one's single tap follows
      src   = static_cast<const char*>(geom.x2);
      src_h = geom.h2, src_w = geom.w2, src_c = geom.c2;
      tap_dy = tap_dx = tap_c0 = 0;
#pragma unroll
      for (int t = 0; t < LPA; ++t) {
        a_yx[t]  = (int)stash[(2 * t) * THREADS];
        a_off[t] = stash[(2 * t + 1) * THREADS];
      }
    }
  };
#pragma unroll
  for (int t = 0; t < LPB; ++t) {
    const int q = lwave * LPB + t;
    if (B_KC) {
      const int row = 8 * q + (lane >> 3);
      const int key = (row & 7) ^ ((row >> 3) & 1);
      const int row_c = row < b_last ? row : b_last;
      b_off[t]      = (unsigned)(((int64_t)row_c * ldb + (((lane & 7) ^ key) << 3)) * 2 + kBias - 1024 * (t & 3));
    } else {
      constexpr int CH = BN / 8;  // 16-byte chunks per k-row
      const int krow   = q * (64 / CH) + lane / CH;
      const int chunk  = (lane % CH) ^ (2 * (krow & 3)) ^ (8 * ((krow >> 4) & 1));
      const int last_c = (b_last + 1) / 8 - 1;  // N % 8 == 0: the last whole chunk of this tile's columns
      const int chunk_c = chunk < last_c ? chunk : last_c;
      b_off[t]         = (unsigned)(((int64_t)krow * ldb + (chunk_c << 3)) * 2 + kBias - 1024 * (t & 3));
    }
  }
  // load t of step kt: first the LPA loads of the A tile, then the LPB loads of the B tile
  auto issue_one = [&](char* a_tile, char* b_tile, int kt, int t) {
    if (t < LPA) {
      if (CONV) {
        const int iy      = (short)(a_yx[t] & 0xffff) + tap_dy * geom.dil_h;
        const int ix      = (a_yx[t] >> 16) + tap_dx * geom.dil_w;
        const bool inside = (unsigned)iy < (unsigned)src_h && (unsigned)ix < (unsigned)src_w;
        // the tap's offset is uniform: ((dy dil_h) w + dx dil_w) c + c0 elements
        const unsigned tap_off =
            ((unsigned)((tap_dy * geom.dil_h) * src_w + tap_dx * geom.dil_w) * (unsigned)src_c + tap_c0) * 2u;
        const char* from = inside ? src + (a_off[t] + tap_off)
                                  : static_cast<const char*>(geom.zero_page) + ((lane & 7) << 4);
        AsyncCopy16To(from, lds_addr + (unsigned)(a_tile - lds) + (lwave * LPA + t) * 1024);
      } else {
        SetLdsBase(lds_addr + (unsigned)(a_tile - lds) + (lwave * LPA + (t & ~3)) * 1024);
        AsyncCopy16Slot(a_base + (int64_t)kt * (kD64BK * 2), a_off[t], t & 3);
      }
    } else {
      SetLdsBase(lds_addr + (unsigned)(b_tile - lds) + (lwave * LPB + ((t - LPA) & ~3)) * 1024);
      AsyncCopy16Slot(b_base + kt * b_step, b_off[t - LPA], (t - LPA) & 3);
    }
  };

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

  // v_mfma_f32_16x16x32: lane l holds, of A, row l % 16 and k = 8 (l / 16) .. + 7 of a 32-deep slice (one 16-byte
  // chunk); of B likewise for column l % 16; of the result, column l % 16 and rows 4 (l / 16) .. + 3.
  // Which 8 of the 32 k a lane group holds is free as long as A and B agree: groups 0..3 take the k chunks 0, 2, 1, 3,
  // so that lanes l and l + 32, which the LDS serves together on a 16-byte read, fetch chunks that differ in bit 0
  // (the row swizzle then puts them in different banks).
  const int frag_row = lane & 15;
  const int frag_kg  = ((lane >> 4) & 1) * 2 + (lane >> 5);
  // [row][64 halves] tiles keep chunk c of row r at chunk position c ^ (r & 7) ^ ((r >> 3) & 1): the eight lanes the
  // LDS serves together from one k group hit eight different 16-byte bank groups, and the key depends on r % 16 only,
  // so one address register per slice serves all of a wavefront's tiles (tile i is an immediate offset of 2 KiB i).
  const int frag_key = (frag_row & 7) ^ (frag_row >> 3);
  int frag_off[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) frag_off[kk] = frag_row * 128 + (((kk * 4 + frag_kg) ^ frag_key) << 4);
  auto read_a = [&](const char* a_tile, int kk, int i) -> vec8 {
    return *reinterpret_cast<const vec8*>(a_tile + frag_off[kk] + (wm * TM + i) * 2048);
  };
  auto read_b = [&](const char* b_tile, int kk, int j) -> vec8 {
    if (B_KC) {
      return *reinterpret_cast<const vec8*>(b_tile + frag_off[kk] + (wn * TN + j) * 2048);
    } else {
      // a transposing read hands lane i of a group of 16 four consecutive k of column i: the group addresses a block
      // of 4 k-rows x 16 columns, every lane four columns of one k-row
      s16x4 part[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int k   = kk * 32 + 8 * frag_kg + 4 * r + ((lane & 15) >> 2);
        const int n   = wn * (TN * 16) + j * 16 + 4 * (lane & 3);
        const int off = k * (BN * 2) + (((n >> 3) ^ (2 * (k & 3)) ^ (8 * ((k >> 4) & 1))) << 4) + (n & 7) * 2;
        part[r] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(b_tile + off));
      }
      s16x8 both = __builtin_shufflevector(part[0], part[1], 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(vec8, both);
    }
  };
#define CINN_SB __builtin_amdgcn_sched_barrier(0)
  // A K step is ROWS = 2 TM rows of TN MFMAs: row r multiplies the A fragment of tile r % TM, slice r / TM (32 deep),
  // with the TN B fragments of that slice.  A fragments live in a ring of four (row r + 3 is requested after the first
  // MFMA of row r), B fragments in two sets (the second slice's are requested early in the first, the next stage's
  // after the barrier).  The barrier follows row ROWS - 4: by then every fragment of the stage is in registers, so
  // the three rows after it (12 MFMAs) run while the first fragments of the next stage are fetched, and the stage's
  // LDS is free for the loads of the stage after next, issued in those same rows.
  constexpr int ROWS = 2 * TM;
  constexpr int BAR  = ROWS - 4;
  // One load per row keeps pace with the 16 clocks per load instruction and CU at which the vector memory path
  // drains: EARLY loads of stage s + 2 in the three rows after the barrier of step s, the others in the first rows
  // of step s + 1.
  // A wavefront tile of 64 rows has short steps (8 rows): all its loads go into the three rows after the barrier.
  // Loader wavefronts that carry their partner's loads too issue two per row.
  constexpr int EPR   = TM == 4 ? 3 : (LW < NW ? 2 : 1);  // loads per row: after the barrier ...
  constexpr int EARLY = 3 * EPR < LPA + LPB ? 3 * EPR : LPA + LPB;
  constexpr int LATE  = LPA + LPB - EARLY;
  // ... and in the first rows of the next step (two per row also when one per row would not get them all out before
  // the barrier that waits for them)
  constexpr int LPR   = (LW < NW || LATE > ROWS - 3) ? 2 : 1;
  static_assert(LATE >= 0 && (LATE + LPR - 1) / LPR <= BAR + 1, "the late loads are issued before the barrier that waits for them");
  // slot of a row's per-row loads that follows MFMA j (-1: none)
#define CINN_LOAD_SLOT(P, j) ((P) == 1 ? ((j) == 3 ? 0 : -1) : (P) == 2 ? ((j) == 1 ? 0 : (j) == 3 ? 1 : -1) : (j) - 1)
  vec8 ring[4];
  vec8 bf[2][TN];

  const int nk_all = K / kD64BK;
  const int nk     = epi.partials ? (nk_all - kt0 < epi.steps_per_split ? nk_all - kt0 : epi.steps_per_split) : nk_all;
  constexpr int L = LPA + LPB;  // loads of a loader wavefront per stage
  // vmcnt(n): at most n of the wavefront's loads still in flight; they complete in the order they were issued
#define CINN_VMCNT(n) ((((n) & 15) | (((n) >> 4) << 14)) | 0x0F70)
  if (FEED) {
    // Feeding wavefronts: every slot is free at the start, so all NS stages go out at once; then, per K step, wait
    // for the next stage (the NS - 2 requested after it may stay in flight), meet the computing wavefronts at the
    // step's barrier - which also tells that the step's own slot has been read - and refill that slot.
    if (feeder) {
#pragma unroll
      for (int st = 0; st < NS; ++st) {
        if (st < nk) {
#pragma unroll
          for (int t = 0; t < L; ++t) issue_one(sa(st), sb(st), st, t);
          if (CONV) advance_tap();
        }
      }
      if (nk >= NS) {
        __builtin_amdgcn_s_waitcnt(CINN_VMCNT((NS - 1) * L));  // stage 0 has landed
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
      __syncthreads();
      int kt = 0;
      for (; kt + NS < nk; ++kt) {  // steps that have a stage to request
        __builtin_amdgcn_s_waitcnt(CINN_VMCNT((NS - 2) * L));  // stage kt + 1 has landed
        __syncthreads();
        switch (kt % NS) {  // slot of stage kt, now read by everyone
          case 0:
#pragma unroll
            for (int t = 0; t < L; ++t) issue_one(sa(0), sb(0), kt + NS, t);
            break;
          case 1:
#pragma unroll
            for (int t = 0; t < L; ++t) issue_one(sa(1 % NS), sb(1 % NS), kt + NS, t);
            break;
          case 2:
#pragma unroll
            for (int t = 0; t < L; ++t) issue_one(sa(2 % NS), sb(2 % NS), kt + NS, t);
            break;
          default:
#pragma unroll
            for (int t = 0; t < L; ++t) issue_one(sa(3 % NS), sb(3 % NS), kt + NS, t);
            break;
        }
        if (CONV) advance_tap();
      }
      for (; kt + 1 < nk; ++kt) {  // the last steps: everything is requested, wait for all of it
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
      }
    }
  } else if (loader) {
#pragma unroll
    for (int st = 0; st < NS - 1; ++st) {
      if (st < nk) {
#pragma unroll
        for (int t = 0; t < L; ++t) issue_one(sa(st), sb(st), st, t);
        if (CONV) advance_tap();
      }
    }
    if (nk > NS - 1) {
#pragma unroll
      for (int t = 0; t < EARLY; ++t) issue_one(sa(NS - 1), sb(NS - 1), NS - 1, t);
      if (CONV && LATE == 0) advance_tap();
      __builtin_amdgcn_s_waitcnt(CINN_VMCNT((NS - 2) * L + EARLY));  // stage 0 has landed, later ones may be in flight
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    }
  }
  if (!feeder) {
  __syncthreads();
  ProbeStamp(epi.probe, wave == 0, 1);
#pragma unroll
  for (int i = 0; i < 3; ++i) ring[i] = read_a(sa(0), 0, i);
#pragma unroll
  for (int j = 0; j < TN; ++j) bf[0][j] = read_b(sb(0), 0, j);
  }

  // Step u of a group of NS (slot of its stage: u).  After its barrier the slot is free for stage s + NS: the first
  // EARLY loads go out in the three rows after the barrier, the others in the first rows of step s + 1 (there: stage
  // s + NS - 1 into slot u - 1).  WAIT: the s_waitcnt before the barrier; in the steady state the NS - 2 stages
  // requested after stage s + 1 may stay in flight.
#define CINN_GEMM_STEP(U, HAS_NEXT, HAS_LATE, HAS_LOAD, DO_LOADS, WAIT)                                       \
  {                                                                                                          \
    const int s         = kt + U;                                                                            \
    const bool has_next = HAS_NEXT;                                                                          \
    const bool has_late = HAS_LATE;                                                                          \
    const bool has_load = HAS_LOAD;                                                                          \
    _Pragma("unroll") for (int r = 0; r < ROWS; ++r) {                                                       \
      _Pragma("unroll") for (int j = 0; j < TN; ++j) {                                                       \
        CINN_SB;                                                                                             \
        acc[r % TM][j] = Half16<T>::mfma16(bf[r / TM][j], ring[r % 4], acc[r % TM][j]);                      \
        CINN_SB;                                                                                             \
        if (j == 0) {                                                                                        \
          if (r + 3 < ROWS) {                                                                                \
            ring[(r + 3) % 4] = read_a(sa(U), (r + 3) / TM, (r + 3) % TM);                                   \
          } else if (has_next) {                                                                             \
            ring[(r + 3) % 4] = read_a(sa((U + 1) % NS), 0, r + 3 - ROWS);                                   \
          }                                                                                                  \
        }                                                                                                    \
        if ((j == 1 || j == 2) && r >= TM / 2 - 2 && r < TM / 2) {                                           \
          bf[1][(r - (TM / 2 - 2)) * 2 + j - 1] = read_b(sb(U), 1, (r - (TM / 2 - 2)) * 2 + j - 1);         \
        }                                                                                                    \
        if ((j == 1 || j == 2) && r >= ROWS - 3 && r < ROWS - 1 && has_next) {                               \
          bf[0][(r - (ROWS - 3)) * 2 + j - 1] = read_b(sb((U + 1) % NS), 0, (r - (ROWS - 3)) * 2 + j - 1);  \
        }                                                                                                    \
        if (DO_LOADS && CINN_LOAD_SLOT(LPR, j) >= 0 && r * LPR + CINN_LOAD_SLOT(LPR, j) < LATE) {            \
          CINN_SB;                                                                                           \
          if (has_late)                                                                                      \
            issue_one(sa((U + NS - 1) % NS), sb((U + NS - 1) % NS), s + NS - 1,                              \
                      EARLY + r * LPR + CINN_LOAD_SLOT(LPR, j));                                             \
          if (CONV && r * LPR + CINN_LOAD_SLOT(LPR, j) == LATE - 1) advance_tap(); /* that stage is requested */ \
        }                                                                                                    \
        if (DO_LOADS && r >= ROWS - 3 && CINN_LOAD_SLOT(EPR, j) >= 0 &&                                      \
            (r - (ROWS - 3)) * EPR + CINN_LOAD_SLOT(EPR, j) < EARLY) {                                       \
          CINN_SB;                                                                                           \
          if (has_load) issue_one(sa(U), sb(U), s + NS, (r - (ROWS - 3)) * EPR + CINN_LOAD_SLOT(EPR, j));    \
          if (CONV && LATE == 0 && (r - (ROWS - 3)) * EPR + CINN_LOAD_SLOT(EPR, j) == EARLY - 1) advance_tap(); \
        }                                                                                                    \
      }                                                                                                      \
      if (r == BAR && has_next) {                                                                            \
        CINN_SB;                                                                                             \
        __builtin_amdgcn_s_waitcnt(WAIT); /* stage s+1 landed (vmcnt), fragments arrived (lgkmcnt(0)) */     \
        __syncthreads();                                                                                     \
      }                                                                                                      \
    }                                                                                                        \
  }
  // groups of NS steps that all have a stage to request: no branches around the loads; then the last steps with
  // the conditions evaluated and every load waited for
  constexpr int kSteadyWait = CINN_VMCNT((NS - 2) * L) & ~0x0F00;
#define CINN_GEMM_LOOP(DO_LOADS)                                                                              \
  {                                                                                                          \
    int kt = 0;                                                                                              \
    for (; kt + 2 * NS - 1 < nk; kt += NS) {                                                                 \
      _Pragma("unroll") for (int u = 0; u < NS; ++u) {                                                       \
        CINN_GEMM_STEP(u, true, true, true, DO_LOADS, kSteadyWait)                                           \
      }                                                                                                      \
    }                                                                                                        \
    for (; kt < nk; kt += NS) {                                                                              \
      _Pragma("unroll") for (int u = 0; u < NS; ++u) {                                                       \
        if (kt + u < nk) CINN_GEMM_STEP(u, s + 1 < nk, s + NS - 1 < nk, s + NS < nk, DO_LOADS, 0x0070)       \
      }                                                                                                      \
    }                                                                                                        \
  }
  if (feeder) {
    // nothing to compute
  } else if (loader) {
    CINN_GEMM_LOOP(true)
  } else {
    CINN_GEMM_LOOP(false)
  }
#undef CINN_GEMM_LOOP
#undef CINN_VMCNT
#undef CINN_LOAD_SLOT
#undef CINN_GEMM_STEP
#undef CINN_SB
  ProbeStamp(epi.probe, wave == 0, 2);

  // Epilogue on the fp32 accumulators: v = fma(residual_scale, R[row][col], fma(acc, scale[col] or alpha, shift[col]))
  // (explicit fused multiply-adds rounded to fp32, and an empty asm between them and the conversion to T: left to the
  // compiler, some accumulators get v_fma_mixlo_f16 - one rounding, straight to fp16 - and others v_fma_f32 plus a
  // conversion - two roundings - and equal inputs then differ in the last bit depending on their row in the tile),
  // optional relu, one rounding to T.  The tile goes through LDS so that every lane moves 16 bytes and a store
  // instruction covers whole rows of the C tile instead of 64 two-byte pieces: as 16-bit values, 64 rows of every
  // wavefront per pass, or - with a residual, which is added before the rounding - as fp32, 32 rows per pass.
  if (epi.partials) {
    // split reduction: the raw sums as fp32 rows (through LDS, 32 rows per wavefront row and pass, so that a lane
    // stores 2 x 16 contiguous bytes)
    constexpr int kRowFloats = BN + 4;
    constexpr int IB         = 2;
    constexpr int PASS_ROWS  = WAVES_M * IB * 16;
    constexpr int CPR8       = BN / 8;
    static_assert(PASS_ROWS * kRowFloats * 4 <= NS * STAGE, "the staged partial sums do not fit the operand stages");
    static_assert(PASS_ROWS * CPR8 % THREADS == 0, "the copy-out loop assumes whole rounds");
    float* stage = reinterpret_cast<float*>(lds);
    float* P     = epi.partials + (int64_t)blockIdx.z * M * N;
#pragma unroll
    for (int pass = 0; pass < TM / IB; ++pass) {
      __syncthreads();
      if (!feeder)
#pragma unroll
      for (int ii = 0; ii < IB; ++ii)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int lrow = wm * (IB * 16) + ii * 16 + (lane & 15);
            const int col  = wn * (TN * 16) + j * 16 + 4 * (lane >> 4);
            *reinterpret_cast<f32x4*>(stage + lrow * kRowFloats + col) = acc[IB * pass + ii][j];
          }
      __syncthreads();
#pragma unroll
      for (int e = 0; e < PASS_ROWS * CPR8 / THREADS; ++e) {
        const int chunk = e * THREADS + tid;
        const int lrow  = chunk / CPR8;
        const int c8    = chunk % CPR8;
        const int row   = m0 + (lrow / (IB * 16)) * (TM * 16) + pass * (IB * 16) + lrow % (IB * 16);
        if (row >= M || n0 + c8 * 8 >= N) continue;
        float* dst = P + (int64_t)row * N + n0 + c8 * 8;
        *reinterpret_cast<f32x4*>(dst)     = *reinterpret_cast<const f32x4*>(stage + lrow * kRowFloats + c8 * 8);
        *reinterpret_cast<f32x4*>(dst + 4) = *reinterpret_cast<const f32x4*>(stage + lrow * kRowFloats + c8 * 8 + 4);
      }
    }
    return;
  }
  T* Ct       = reinterpret_cast<T*>(C);
  const T* Rt = reinterpret_cast<const T*>(epi.residual);
  if (Rt) Rt += (int64_t)blockIdx.y * stride_c;
  float sc[TN][4], sh[TN][4];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int col  = n0 + wn * (TN * 16) + j * 16 + 4 * (lane >> 4) + r;
      col      = col < N ? col : N - 1;
      sc[j][r] = epi.scale ? epi.scale[col] : epi.alpha;
      sh[j][r] = epi.shift ? epi.shift[col] : 0.0f;
    }
  constexpr int CPR = BN / 8;  // 8-column chunks per row
  if (!Rt) {
    constexpr int kRowBytes = (BN + 8) * 2;
    constexpr int IB        = 4;  // 16-row blocks per wavefront and pass: 64 rows
    constexpr int PASS_ROWS = WAVES_M * IB * 16;
    static_assert(PASS_ROWS * kRowBytes <= NS * STAGE, "the staged result does not fit the operand stages");
    static_assert(PASS_ROWS * CPR % THREADS == 0, "the copy-out loop assumes whole rounds");
#pragma unroll
    for (int pass = 0; pass < TM / IB; ++pass) {
      __syncthreads();  // the last stage (or the previous pass) has been read
      // a lane's four consecutive columns of a row leave as one 8-byte LDS write; the relu is a max (a NaN becomes 0,
      // as with v > 0 ? v : 0), chosen by a branch around the pass so that the other form carries no select
      auto stage_pass = [&](auto relu_tag) {
        constexpr bool RELU = decltype(relu_tag)::value;
#pragma unroll
        for (int ii = 0; ii < IB; ++ii)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int lrow = wm * (IB * 16) + ii * 16 + (lane & 15);
            const int col  = wn * (TN * 16) + j * 16 + 4 * (lane >> 4);
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              v[r] = __builtin_fmaf(acc[IB * pass + ii][j][r], sc[j][r], sh[j][r]);
              if (RELU) v[r] = __builtin_fmaxf(v[r], 0.0f);
              asm volatile("" : "+v"(v[r]));  // keeps the fma and the conversion apart, see above
            }
            const u32x2 out = {PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3])};
            *reinterpret_cast<u32x2*>(lds + lrow * kRowBytes + col * 2) = out;
          }
      };
      if (!feeder) {
        if (epi.relu) {
          stage_pass(std::true_type{});
        } else {
          stage_pass(std::false_type{});
        }
      }
      __syncthreads();
#pragma unroll
      for (int e = 0; e < PASS_ROWS * CPR / THREADS; ++e) {
        const int chunk = e * THREADS + tid;
        const int lrow  = chunk / CPR;
        const int c16   = chunk % CPR;
        const int row   = m0 + (lrow / (IB * 16)) * (TM * 16) + pass * (IB * 16) + lrow % (IB * 16);
        const u32x4 v   = *reinterpret_cast<const u32x4*>(lds + lrow * kRowBytes + c16 * 16);
        // streaming stores: results that do not sit dirty in L2 shorten the write-back at the end of the kernel
        // (4096^3 2 %, 8192^3 3.6 % faster); a convolution inside a network keeps its output cached for the next
        // layer instead (ResNet-50 0.4 % slower with streaming stores)
        if (row >= M || n0 + c16 * 8 >= N) continue;
        u32x4* dst = reinterpret_cast<u32x4*>(Ct + (int64_t)row * ldc + n0 + c16 * 8);
        if (epi.streaming) {
          __builtin_nontemporal_store(v, dst);
        } else {
          *dst = v;
        }
      }
    }
    ProbeStamp(epi.probe, wave == 0, 3);
    return;
  }
  constexpr int kRowFloats = BN + 4;
  constexpr int IB         = 2;  // 16-row blocks per wavefront and pass: 32 rows of fp32
  constexpr int PASS_ROWS  = WAVES_M * IB * 16;
  static_assert(PASS_ROWS * kRowFloats * 4 <= NS * STAGE, "the staged result does not fit the operand stages");
  static_assert(PASS_ROWS * CPR % THREADS == 0, "the copy-out loop assumes whole rounds");
  float* stage = reinterpret_cast<float*>(lds);
  // The residual chunks of a pass are requested one pass ahead (those of the first pass before the first barrier), so
  // that their latency runs under the staging of the accumulators instead of after it.
  constexpr int EPT = PASS_ROWS * CPR / THREADS;  // chunks per thread and pass
  vec8 res[2][EPT];
  auto request_residual = [&](int pass, vec8* out) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int chunk = e * THREADS + tid;
      const int lrow  = chunk / CPR;
      const int c8    = chunk % CPR;
      const int row   = m0 + (lrow / (IB * 16)) * (TM * 16) + pass * (IB * 16) + lrow % (IB * 16);
      if (row < M && n0 + c8 * 8 < N) out[e] = *reinterpret_cast<const vec8*>(Rt + (int64_t)row * ldc + n0 + c8 * 8);
    }
  };
  request_residual(0, res[0]);
#pragma unroll
  for (int pass = 0; pass < TM / IB; ++pass) {
    __syncthreads();
    if (!feeder)
#pragma unroll
    for (int ii = 0; ii < IB; ++ii)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
          const int lrow = wm * (IB * 16) + ii * 16 + (lane & 15);
          const int col  = wn * (TN * 16) + j * 16 + 4 * (lane >> 4);
          f32x4 v4;
#pragma unroll
          for (int r = 0; r < 4; ++r) v4[r] = __builtin_fmaf(acc[IB * pass + ii][j][r], sc[j][r], sh[j][r]);
          *reinterpret_cast<f32x4*>(stage + lrow * kRowFloats + col) = v4;
        }
    __syncthreads();
    if (pass + 1 < TM / IB) request_residual(pass + 1, res[(pass + 1) & 1]);
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int chunk = e * THREADS + tid;
      const int lrow  = chunk / CPR;
      const int c8    = chunk % CPR;
      const int row   = m0 + (lrow / (IB * 16)) * (TM * 16) + pass * (IB * 16) + lrow % (IB * 16);
      if (row >= M || n0 + c8 * 8 >= N) continue;
      const int64_t o = (int64_t)row * ldc + n0 + c8 * 8;
      const f32x4 lo  = *reinterpret_cast<const f32x4*>(stage + lrow * kRowFloats + c8 * 8);
      const f32x4 hi  = *reinterpret_cast<const f32x4*>(stage + lrow * kRowFloats + c8 * 8 + 4);
      const vec8& rq  = res[pass & 1][e];
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        v[q] = __builtin_fmaf(epi.residual_scale, (float)rq[q], q < 4 ? lo[q] : hi[q - 4]);
        // the relu as a max under a select on the flag: no compare per value
        const float m = __builtin_fmaxf(v[q], 0.0f);
        v[q]          = epi.relu ? m : v[q];
        asm volatile("" : "+v"(v[q]));
      }
      const u32x4 out = {PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3]), PackPair<T>(v[4], v[5]), PackPair<T>(v[6], v[7])};
      if (epi.streaming) {
        __builtin_nontemporal_store(out, reinterpret_cast<u32x4*>(Ct + o));
      } else {
        *reinterpret_cast<u32x4*>(Ct + o) = out;
      }
    }
  }
  ProbeStamp(epi.probe, wave == 0, 3);
}

// ---------------------------------------------------------------------------------------------------
// Short reductions (K = 64; B stored [N][K], or [K][N] gathered once per block) - 1x1 convolutions over few channels:
// 2 * K flop per output element make these products a stream of C (and of the residual), and a tiled kernel, whose
// block waits for its operands, computes for a moment and then writes its tile, never has enough bytes in flight.
// Here nothing is staged and nobody waits for a neighbour: a wavefront keeps its NT * 16 filter rows in registers as
// MFMA operands for the whole kernel and walks over groups of 16 rows of A, computing the transposed tile
// D[n][m] = sum_k B[n][k] * A[m][k] on v_mfma_f32_16x16x32, so that a lane ends up with 4 consecutive columns of one
// row of C; the tile turns into whole rows in a piece of LDS private to the wavefront (as finished 16-bit values, or
// as fp32 when a residual - read as whole rows, 16 bytes per lane - is still to be added) and leaves as 16-byte stores.
// Both operands are read from global memory straight in fragment layout (16 bytes of one row per lane); the rows and
// the residual of the next group are requested before the current group is computed.  Per-column scale / shift sit
// in LDS.  No block barrier after the start-up.
// Measured on [100352, 64] x [256, 64]^T (51 MB of results, fp16; 19.4 us): the same stores alone, in this kernel's
// pattern of four 256-byte row pieces per instruction, take 9.6 us (5.3 TB/s), a copy of 12.8 MB into 51 MB 13.5 us;
// with the stores removed the kernel takes 12.2 us, with the row loads removed 15.4 us.  Start-up (launch, 16 KB of
// filter fragments per wavefront) is 5 us of that.  Neither the instruction count of the epilogue (219 -> 122 vector
// instructions per group with packed conversions, a max for the relu and scalar group addresses), nor exact waits
// (loads in inline assembly, vmcnt counted by hand), nor 12 or 16 wavefronts per CU changed the time: the loop is
// bound by stores and loads taking turns on the memory side, not by issue.
// ---------------------------------------------------------------------------------------------------
template <typename T, int NT, int KH, bool RES, bool B_KC, bool RELU>
__global__ void __launch_bounds__(256)
gemm16_shortk_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C, int M, int N,
                     int64_t lda, int64_t ldb, int64_t ldc, DmaEpilogue epi, int64_t stride_a, int64_t stride_b,
                     int64_t stride_c, int ny) {
  typedef typename Half16<T>::vec8 vec8;
  constexpr int NW = NT * 16;  // columns per wavefront
  __shared__ __attribute__((aligned(16))) float s_scale[NW];
  __shared__ __attribute__((aligned(16))) float s_shift[NW];
  // staging row in bytes, padded so that the 16 rows of a write spread over the banks: the finished 16-bit tile, or -
  // with a residual, which arrives as whole rows and is added before the rounding - the fp32 tile
  constexpr int kStageRow     = RES ? (NW + 4) * 4 : NW * 2 + 16;
  constexpr int kChunksPerRow = NW / 8;  // 8 columns: 16 bytes of C per lane
  constexpr int kRowsPerStore = 64 / kChunksPerRow;
  __shared__ __attribute__((aligned(16))) char s_stage[4 * 16 * kStageRow];
  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* my_stage = s_stage + wave * 16 * kStageRow;  // private to the wavefront: no block barrier in the loop
  // consecutive block ids go round-robin to the 8 XCDs: the ny column panels of one row range stay on one XCD
  const int lin = blockIdx.x, xcd = lin & 7, idx = lin >> 3;
  const int n0    = (idx % ny) * NW;
  const int slot  = (idx / ny) * 8 + xcd;
  const int slots = gridDim.x / ny;
  A += (int64_t)blockIdx.y * stride_a;
  B += (int64_t)blockIdx.y * stride_b;
  C += (int64_t)blockIdx.y * stride_c;
  const T* Rt = reinterpret_cast<const T*>(epi.residual);
  if (RES) Rt += (int64_t)blockIdx.y * stride_c;
  for (int i = tid; i < NW; i += 256) {
    s_scale[i] = epi.scale ? epi.scale[n0 + i] : epi.alpha;
    s_shift[i] = epi.shift ? epi.shift[n0 + i] : 0.0f;
  }
  const int frow = lane & 15;        // row of the fragment this lane reads
  const int fk   = (lane >> 4) * 8;  // its 8 elements of a 32-deep k block
  vec8 wf[NT][KH];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int kh = 0; kh < KH; ++kh)
      if (B_KC) {
        wf[j][kh] = *reinterpret_cast<const vec8*>(B + (int64_t)(n0 + j * 16 + frow) * ldb + kh * 32 + fk);
      } else {
        // B stored [K][N]: the 8 k values of a fragment are a column, gathered once per block
        uint16_t col[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) col[q] = B[(int64_t)(kh * 32 + fk + q) * ldb + n0 + j * 16 + frow];
        __builtin_memcpy(&wf[j][kh], col, 16);
      }
  // The filter fragments are complete before the loop starts; left to the compiler, the waits for them sit at their
  // first use, inside the loop, where they would also wait for the rows just requested.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) asm volatile("" : "+v"(wf[j][kh]));
  __syncthreads();

  const int groups  = (M + 15) >> 4;
  const int gstride = slots * 4;
  int g             = slot * 4 + wave;
  if (g >= groups) return;
  // A group's first row is the same for the whole wavefront: its address is scalar arithmetic, and what a lane adds
  // (its row inside the group, its columns) is computed once - 32-bit element offsets, 16 rows of a matrix being far
  // below 2^31 elements.  Only the last group of a matrix whose rows are not a multiple of 16 clamps its rows.
  constexpr int kStores = 16 / kRowsPerStore;
  const int a_lane = frow * (int)lda + fk;
  int c_lane[kStores];
#pragma unroll
  for (int i = 0; i < kStores; ++i)
    c_lane[i] = (i * kRowsPerStore + lane / kChunksPerRow) * (int)ldc + n0 + (lane % kChunksPerRow) * 8;
  auto request = [&](int grp, vec8* xa, vec8* rr) {
    const int valid           = M - grp * 16;  // rows of the group inside the matrix
    const uint16_t* const a_g = A + (int64_t)grp * 16 * lda;
    const int a_at            = valid >= 16 ? a_lane : min(frow, valid - 1) * (int)lda + fk;
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) xa[kh] = *reinterpret_cast<const vec8*>(a_g + a_at + kh * 32);
    if (RES) {
      const T* const r_g = Rt + (int64_t)grp * 16 * ldc;
#pragma unroll
      for (int i = 0; i < kStores; ++i) {
        const int at = valid >= 16 ? c_lane[i]
                                   : min(i * kRowsPerStore + lane / kChunksPerRow, valid - 1) * (int)ldc + n0 +
                                         (lane % kChunksPerRow) * 8;
        rr[i] = *reinterpret_cast<const vec8*>(r_g + at);
      }
    }
  };
  // a ring of D groups: the rows (and residual) of the group D - 1 steps ahead are requested while the current one is
  // computed (three steps ahead measured the same as one: 17.6 against 17.0 us for 100352 x 256 x 64)
  constexpr int D = 2;
  static_assert(D == 2, "the loop below requests exactly one group ahead");
  vec8 xa[D][KH];
  vec8 rr[D][RES ? kStores : 1];
  request(g, xa[0], rr[0]);
  for (;;) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int gn        = g + gstride;
      const bool has_next = gn < groups;
      if (has_next) request(gn, xa[(u + 1) % D], rr[(u + 1) % D]);
      f32x4 acc[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kh = 0; kh < KH; ++kh)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j] = Half16<T>::mfma16(wf[j][kh], xa[u][kh], acc[j]);
      // the sums are wanted in ordinary registers: the epilogue's arithmetic cannot read the accumulation registers,
      // and a copy per value is a fifth of this loop's instructions
#pragma unroll
      for (int j = 0; j < NT; ++j) asm volatile("" : "+v"(acc[j]));
      const int valid   = M - g * 16;
      T* const c_g      = reinterpret_cast<T*>(C) + (int64_t)g * 16 * ldc;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const f32x4 sc = *reinterpret_cast<const f32x4*>(&s_scale[j * 16 + 4 * (lane >> 4)]);
        const f32x4 sh = *reinterpret_cast<const f32x4*>(&s_shift[j * 16 + 4 * (lane >> 4)]);
        if (RES) {
          f32x4 v4;
#pragma unroll
          for (int r = 0; r < 4; ++r) v4[r] = __builtin_fmaf(acc[j][r], sc[r], sh[r]);
          *reinterpret_cast<f32x4*>(my_stage + frow * kStageRow + (j * 16 + 4 * (lane >> 4)) * 4) = v4;
        } else {
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            v[r] = __builtin_fmaf(acc[j][r], sc[r], sh[r]);
            if (RELU) v[r] = __builtin_fmaxf(v[r], 0.0f);  // a NaN becomes 0, as with v > 0 ? v : 0
            asm volatile("" : "+v"(v[r]));  // one rounding to T for every element, see gemm16_dma_kernel's epilogue
          }
          u32x2 out = {PackPair<T>(v[0], v[1]), PackPair<T>(v[2], v[3])};
          *reinterpret_cast<u32x2*>(my_stage + frow * kStageRow + (j * 16 + 4 * (lane >> 4)) * 2) = out;
        }
      }
      // the wavefront's own 16 x NW tile comes back as whole rows: 16 bytes of C per lane, full lines per store
      // (8-byte pieces of 32 contiguous bytes per row write at little more than half the rate)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int i = 0; i < kStores; ++i) {
        const int srow = i * kRowsPerStore + lane / kChunksPerRow;
        const int ch   = lane % kChunksPerRow;
        u32x4 v;
        if (RES) {
          const f32x4 lo = *reinterpret_cast<const f32x4*>(my_stage + srow * kStageRow + ch * 32);
          const f32x4 hi = *reinterpret_cast<const f32x4*>(my_stage + srow * kStageRow + ch * 32 + 16);
          float t[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            t[q] = __builtin_fmaf(epi.residual_scale, (float)rr[u][RES ? i : 0][q], q < 4 ? lo[q] : hi[q - 4]);
            if (RELU) t[q] = __builtin_fmaxf(t[q], 0.0f);
            asm volatile("" : "+v"(t[q]));
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = PackPair<T>(t[2 * q], t[2 * q + 1]);
        } else {
          v = *reinterpret_cast<const u32x4*>(my_stage + srow * kStageRow + ch * 16);
        }
        if (srow < valid) {
          u32x4* dst = reinterpret_cast<u32x4*>(c_g + c_lane[i]);
          if (epi.streaming) {
            __builtin_nontemporal_store(v, dst);
          } else {
            *dst = v;
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (!has_next) return;
      g = gn;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// Few rows (M <= 64: a classifier at inference batch sizes, a decoding step): C[M][N] = A[M][K] . B[N][K]^T is bound by
// one pass over B.  The tiled kernels give such a product M-tiles that are mostly padding and a handful of blocks; here
// a block owns 16 output columns of MT row tiles (rows from 16 MT blockIdx.y: the launcher gives every row tile a block
// of its own) and its eight wavefronts split K.  A lane's share of a 16x16x32 fragment is 8
// consecutive k of one row - 16 contiguous bytes in both operands - so fragments come straight from global memory, no
// LDS on the way: every wavefront keeps U k-blocks of loads in flight (two register sets), B is read exactly once
// from memory, A (at most 64 rows) comes out of L2.  The eight partial tiles meet in LDS; wavefront t finishes row
// tile t (scale / shift, residual, relu - the epilogue of gemm16_dma_kernel - then 2-byte stores: the result is small).
template <typename T, int MT>
__global__ void __launch_bounds__(512)
gemm16_skinny_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C, int M, int N,
                     int K, DmaEpilogue epi) {
  typedef typename Half16<T>::vec8 vec8;
  constexpr int NWAVES = 8;
  constexpr int U      = 4;  // k-blocks per register set
  __shared__ __attribute__((aligned(16))) float s_part[NWAVES][MT][64][4];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n0   = blockIdx.x * 16;
  const int m0   = blockIdx.y * (MT * 16);  // first of this block's rows
  const int fr   = lane & 15;               // row of the fragment this lane reads (a row of A, a column of C for B)
  const int fk   = (lane >> 4) * 8;  // its 8 elements of a 32-deep k block
  const int kw   = K / NWAVES;       // this wavefront's share of K, a multiple of 32
  const int nkb  = kw / 32;
  const int bcol = min(n0 + fr, N - 1);
  const uint16_t* bp = B + (int64_t)bcol * K + wave * kw + fk;
  const uint16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) ap[t] = A + (int64_t)min(m0 + t * 16 + fr, M - 1) * K + wave * kw + fk;
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  vec8 bf[2][U], af[2][U][MT];
  auto request = [&](int set, int kb0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kb = min(kb0 + u, nkb - 1);  // beyond the share: the last block again, not multiplied
      bf[set][u]   = *reinterpret_cast<const vec8*>(bp + kb * 32);
#pragma unroll
      for (int t = 0; t < MT; ++t) af[set][u][t] = *reinterpret_cast<const vec8*>(ap[t] + kb * 32);
    }
  };
  auto multiply = [&](int set, int kb0) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (kb0 + u < nkb) {
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = Half16<T>::mfma16(af[set][u][t], bf[set][u], acc[t]);
      }
  };
  request(0, 0);
  for (int kb0 = 0; kb0 < nkb; kb0 += 2 * U) {
    if (kb0 + U < nkb) request(1, kb0 + U);
    multiply(0, kb0);
    if (kb0 + 2 * U < nkb) request(0, kb0 + 2 * U);
    multiply(1, kb0 + U);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4*>(&s_part[wave][t][lane][0]) = acc[t];
  __syncthreads();
  if (wave >= MT) return;
  // wavefront t: row tile t.  Lane = (column n0 + lane % 16, rows 16 t + 4 (lane / 16) .. + 3)
  f32x4 sum = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) sum += *reinterpret_cast<const f32x4*>(&s_part[w][wave][lane][0]);
  const int col = n0 + fr;
  if (col >= N) return;
  const float sc = epi.scale ? epi.scale[col] : epi.alpha;
  const float sh = epi.shift ? epi.shift[col] : 0.0f;
  T* Ct          = reinterpret_cast<T*>(C);
  const T* Rt    = reinterpret_cast<const T*>(epi.residual);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = m0 + wave * 16 + 4 * (lane >> 4) + r;
    if (row >= M) continue;
    float v = __builtin_fmaf(sum[r], sc, sh);
    if (Rt) v = __builtin_fmaf(epi.residual_scale, (float)Rt[(int64_t)row * N + col], v);
    asm volatile("" : "+v"(v));  // one rounding to T, see gemm16_dma_kernel's epilogue
    if (epi.relu) v = v > 0.0f ? v : 0.0f;
    Ct[(int64_t)row * N + col] = (T)v;
  }
}

// ---------------------------------------------------------------------------------------------------
// fp32 on v_mfma_f32_32x32x2f32: 128x128 (or 64x64) tile, K step KS = 32 or 64, 4 wavefronts each a quarter of the tile.
// LDS holds A as [k][m] and B as [k][n] (row stride TILE + 4 floats) so that a fragment read is one conflict-free
// ds_read_b32 per lane; the K step is deep enough (16 MFMAs of 64 clocks per accumulator) to cover the latency of
// the next step's global loads, which travel as 16 bytes per lane and whole 128-byte lines per row.
// ---------------------------------------------------------------------------------------------------
constexpr int kF32Tile = 128;
constexpr int kF32K    = 32;

// KSPLIT == 2 (with the 64x64 tile, whose wavefronts own a single accumulator tile): 8 wavefronts, two per 32x32
// quadrant, each taking every other k pair of a step - a SIMD then holds two independent MFMA chains, which hides
// the latency between dependent MFMAs and of the LDS reads; the two partial tiles are added through LDS at the end.
template <int TILE, bool TRANS_A, bool TRANS_B, int KSPLIT, int KS>
__global__ void __launch_bounds__(256 * KSPLIT)
gemm32_mfma_kernel(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C, int M, int N, int K,
                   int64_t lda, int64_t ldb, int64_t ldc, float alpha, float beta, int64_t stride_a, int64_t stride_b,
                   int64_t stride_c, int xcd_cols, int sub_rows, int sub_cols) {
  // Row pitch of the [k][row] tiles.  An operand whose contiguous axis is the row index is copied with 16-byte
  // accesses (pitch a multiple of 4 floats; + 4 keeps the k rows of a fragment read apart).  One whose contiguous axis
  // is k is scattered, four 4-byte writes per thread: a wavefront's lanes are (k chunk 0..7) x (row 0..7), so the bank
  // of a write is pitch * 4 * chunk + row (mod 32) - with an odd pitch the eight chunks fall into eight different
  // groups of four banks (TILE + 5: 20, 8, 28, 16, 4, 24, 12 away from chunk 0) and the scatter is conflict-free; with
  // TILE + 4 chunks 0, 2, 4, 6 share their banks (SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE 0.33 on 1024^3).
  constexpr int PA = TILE + (TRANS_A ? 4 : 5);
  constexpr int PB = TILE + (TRANS_B ? 5 : 4);
  __shared__ __attribute__((aligned(16))) float As[2][KS][PA];
  __shared__ __attribute__((aligned(16))) float Bs[2][KS][PB];
  constexpr int TT      = TILE / 64;  // 32x32 MFMA tiles per wavefront and dimension
  constexpr int THREADS = 256 * KSPLIT;
  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int kgrp = wave >> 2;  // which k pairs of a step this wavefront takes
  const int wm = (wave >> 1) & 1, wn = wave & 1;
  // consecutive workgroups go round-robin to the 8 XCDs: give each XCD a compact rectangle of tiles (see
  // gemm16_dma_kernel), so that its L2 holds few A and B panels
  int tile_row = blockIdx.y, tile_col = blockIdx.x;
  if (sub_rows > 0) {
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    const int xcd = lin & 7, idx = lin >> 3;
    tile_row = (xcd / xcd_cols) * sub_rows + idx / sub_cols;
    tile_col = (xcd % xcd_cols) * sub_cols + idx % sub_cols;
  }
  const int m0 = tile_row * TILE;
  const int n0 = tile_col * TILE;
  A += (int64_t)blockIdx.z * stride_a;
  B += (int64_t)blockIdx.z * stride_b;
  C += (int64_t)blockIdx.z * stride_c;

  f32x16 acc[TT][TT];
#pragma unroll
  for (int i = 0; i < TT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Each thread stages EL4 groups of 4 floats of either operand per K step, 16 bytes per access.  An operand whose
  // contiguous axis is k is fetched as 8 rows x 128 bytes per wavefront access (whole lines) and scattered into
  // [k][row]; one whose contiguous axis is the row index is copied as it is.
  // The staging registers are a ring of PF steps: the loads of step kt + PF are issued in step kt, so that PF - 1 steps
  // of MFMAs cover their latency (a 64x64 tile's step is short: 8 MFMAs per wavefront).
  constexpr int EL4 = TILE * KS / 4 / THREADS;
  constexpr int PF  = TILE == 64 ? 4 : 2;
  f32x4 ra[PF][EL4], rb[PF][EL4];
  auto load_one = [&](const float* __restrict__ P, int64_t ld, int row0, int k0, bool k_contig, int i) -> f32x4 {
    const int u = tid + THREADS * i;
    if (k_contig) {
      const int r = u / (KS / 4), kc = u % (KS / 4);
      return *reinterpret_cast<const f32x4*>(P + (int64_t)(row0 + r) * ld + k0 + kc * 4);
    }
    const int k = u / (TILE / 4), c = u % (TILE / 4);
    return *reinterpret_cast<const f32x4*>(P + (int64_t)(k0 + k) * ld + row0 + c * 4);
  };
  auto store_one = [&](auto* S, bool k_contig, int i, f32x4 v) {  // S: one buffer of As or Bs, float [KS][pitch]
    const int u = tid + THREADS * i;
    if (k_contig) {
      const int r = u / (KS / 4), kc = u % (KS / 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) S[kc * 4 + j][r] = v[j];
    } else {
      const int k = u / (TILE / 4), c = u % (TILE / 4);
      *reinterpret_cast<f32x4*>(&S[k][c * 4]) = v;
    }
  };
  auto load_tiles = [&](int slot, int k0) {
#pragma unroll
    for (int i = 0; i < EL4; ++i) {
      ra[slot][i] = load_one(A, lda, m0, k0, !TRANS_A, i);
      rb[slot][i] = load_one(B, ldb, n0, k0, TRANS_B, i);
    }
  };
  auto store_tiles = [&](int slot, int buf) {
#pragma unroll
    for (int i = 0; i < EL4; ++i) {
      store_one(As[buf], !TRANS_A, i, ra[slot][i]);
      store_one(Bs[buf], TRANS_B, i, rb[slot][i]);
    }
  };

  const int kt_count = K / KS;
#pragma unroll
  for (int d = 0; d < PF; ++d)
    if (d < kt_count) load_tiles(d, d * KS);
  store_tiles(0, 0);
  __syncthreads();
  // one K step: refill ring slot u (it went into LDS at the end of the previous step), all fragment reads of the step,
  // then its MFMAs, then the next step's registers into the other LDS buffer
#define CINN_GEMM32_STEP(U, REFILL, NEXT)                                                                   \
  {                                                                                                         \
    const int kt  = kt0 + U;                                                                                \
    const int cur = U & 1; /* PF is even */                                                                 \
    if (REFILL) load_tiles(U, (kt + PF) * KS);                                                              \
    constexpr int KP = KS / 2 / KSPLIT;                                                                     \
    float af[KP][TT], bf[KP][TT];                                                                           \
    _Pragma("unroll") for (int kp = 0; kp < KP; ++kp) {                                                     \
      const int k = 2 * (kp * KSPLIT + kgrp) + (lane >> 5);                                                 \
      _Pragma("unroll") for (int t = 0; t < TT; ++t) {                                                      \
        af[kp][t] = As[cur][k][wm * (TILE / 2) + t * 32 + (lane & 31)];                                     \
        bf[kp][t] = Bs[cur][k][wn * (TILE / 2) + t * 32 + (lane & 31)];                                     \
      }                                                                                                     \
    }                                                                                                       \
    _Pragma("unroll") for (int kp = 0; kp < KP; ++kp)                                                       \
      _Pragma("unroll") for (int i = 0; i < TT; ++i)                                                        \
        _Pragma("unroll") for (int j = 0; j < TT; ++j)                                                      \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[kp][i], bf[kp][j], acc[i][j], 0, 0, 0);       \
    if (NEXT) store_tiles((U + 1) % PF, cur ^ 1);                                                           \
    __syncthreads();                                                                                        \
  }
  // groups of PF steps that all have a step to request (no conditions inside), then the last steps
  int kt0 = 0;
  for (; kt0 + 2 * PF <= kt_count; kt0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u) CINN_GEMM32_STEP(u, true, true)
  }
  for (; kt0 < kt_count; kt0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u)
      if (kt0 + u < kt_count) CINN_GEMM32_STEP(u, kt + PF < kt_count, kt + 1 < kt_count)
  }
#undef CINN_GEMM32_STEP
  if (KSPLIT == 2) {
    // the last barrier of the loop has passed: the operand tiles are no longer read
    static_assert(KSPLIT == 1 || TT == 1, "the partial tile exchange assumes one accumulator tile per wavefront");
    float* part = &As[0][0][0] + ((wave & 3) * 16) * 64 + lane;  // [quadrant][element][lane]
    if (kgrp == 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) part[r * 64] = acc[0][0][r];
    }
    __syncthreads();
    if (kgrp == 1) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][0][r] += part[r * 64];
  }
#pragma unroll
  for (int i = 0; i < TT; ++i) {
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      const int col = n0 + wn * (TILE / 2) + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * (TILE / 2) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        float* dst = C + (int64_t)row * ldc + col;
        float v    = alpha * acc[i][j][r];
        if (beta != 0.0f) v += beta * *dst;
        *dst = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// Generic kernel: any M, N, K, transposes and element type; accumulates in ACC (float, or double for fp64).
// 64x64 tile, K step 16, 256 threads each computing a 4x4 micro tile.
// ---------------------------------------------------------------------------------------------------
template <typename T, typename ACC>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int M, int N, int K, int64_t lda,
                    int64_t ldb, int64_t ldc, bool trans_a, bool trans_b, float alpha, float beta, int64_t stride_a,
                    int64_t stride_b, int64_t stride_c) {
  __shared__ ACC As[16][64 + 1];
  __shared__ ACC Bs[16][64 + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  A += (int64_t)blockIdx.z * stride_a;
  B += (int64_t)blockIdx.z * stride_b;
  C += (int64_t)blockIdx.z * stride_c;
  ACC acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (ACC)0;
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = tid + 256 * i;  // 0..1023 = 16 x 64
      int k = e >> 6, r = e & 63;
      ACC av = (ACC)0, bv = (ACC)0;
      if (k0 + k < K) {
        if (m0 + r < M) av = (ACC)(trans_a ? A[(int64_t)(k0 + k) * lda + m0 + r] : A[(int64_t)(m0 + r) * lda + k0 + k]);
        if (n0 + r < N) bv = (ACC)(trans_b ? B[(int64_t)(n0 + r) * ldb + k0 + k] : B[(int64_t)(k0 + k) * ldb + n0 + r]);
      }
      As[k][r] = av;
      Bs[k][r] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      ACC a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = As[k][ty * 4 + i];
        b[i] = Bs[k][tx * 4 + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = m0 + ty * 4 + i;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int col = n0 + tx * 4 + j;
      if (col >= N) continue;
      T* dst = C + (int64_t)row * ldc + col;
      ACC v  = (ACC)alpha * acc[i][j];
      if (beta != 0.0f) v += (ACC)beta * (ACC)*dst;
      *dst = (T)v;
    }
  }
}

// [rows][cols] -> [cols][rows] through a 32x32 LDS tile (odd pitch), blockIdx.z = batch.  Brings an operand whose
// contiguous axis is not K into the K-contiguous form the bounds-checked MFMA path wants.
template <typename T>
__global__ void __launch_bounds__(256)
transpose2d_kernel(const T* __restrict__ in, T* __restrict__ out, int rows, int cols, int64_t in_stride, int64_t out_stride) {
  __shared__ T tile[32][33];
  in += (int64_t)blockIdx.z * in_stride;
  out += (int64_t)blockIdx.z * out_stride;
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  const int tx = threadIdx.x, ty = threadIdx.y;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty + 8 * i, c = c0 + tx;
    if (r < rows && c < cols) tile[ty + 8 * i][tx] = in[(int64_t)r * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + ty + 8 * i, r = r0 + tx;
    if (r < rows && c < cols) out[(int64_t)c * rows + r] = tile[tx][ty + 8 * i];
  }
}

void LaunchTranspose(const void* in, void* out, int rows, int cols, int batch, int64_t in_stride, int elem_bytes,
                     hipStream_t stream) {
  dim3 grid((cols + 31) / 32, (rows + 31) / 32, batch);
  CINN_RT_CHECK(grid.y <= 65535, "gemm: operand with %d rows is too tall for the transposing copy", rows);
  const int64_t out_stride = (int64_t)rows * cols;
  if (elem_bytes == 2) {
    hipLaunchKernelGGL((transpose2d_kernel<uint16_t>), grid, dim3(32, 8), 0, stream, static_cast<const uint16_t*>(in),
                       static_cast<uint16_t*>(out), rows, cols, in_stride, out_stride);
  } else {
    hipLaunchKernelGGL((transpose2d_kernel<uint32_t>), grid, dim3(32, 8), 0, stream, static_cast<const uint32_t*>(in),
                       static_cast<uint32_t*>(out), rows, cols, in_stride, out_stride);
  }
  CINN_HIP_CALL(hipGetLastError());
}

enum class GemmType { kF16, kBF16, kF32, kF64 };

struct GemmProblem {
  GemmType type;
  const void* a;
  const void* b;
  void* c;
  int m, n, k;
  bool trans_a, trans_b;  // op(A) is [m,k]: A stored [k,m] when trans_a; op(B) is [k,n]: B stored [n,k] when trans_b
  float alpha, beta;
  int batch;
  int64_t stride_a, stride_b, stride_c;  // in elements; 0 broadcasts the operand over the batch
  // convolution epilogue (direct-to-LDS kernels only): per-column scale / shift, residual of C's shape, relu
  const float* scale{nullptr};
  const float* shift{nullptr};
  const void* residual{nullptr};
  float residual_scale{0.0f};
  bool relu{false};
  // A is the input of a channels-last convolution (implicit GEMM), not a matrix
  const ConvGeom* conv{nullptr};
  // the result is a layer's activation: leave it in L2 for the next kernel
  bool keep_in_cache{false};
};

template <typename T, bool A_KC, bool B_KC>
void LaunchFast16(const GemmProblem& p, hipStream_t stream) {
  auto kernel = gemm16_mfma_kernel<T, A_KC, B_KC>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      2 * kStageBytes));
    return true;
  }();
  (void)configured;
  int64_t lda = p.trans_a ? p.m : p.k;
  int64_t ldb = p.trans_b ? p.k : p.n;
  dim3 grid((p.m / kBM) * (p.n / kBN), p.batch, 1);
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 2 * kStageBytes, stream, static_cast<const uint16_t*>(p.a),
                     static_cast<const uint16_t*>(p.b), static_cast<uint16_t*>(p.c), p.m, p.n, p.k, lda, ldb,
                     (int64_t)p.n, p.alpha, p.beta, p.stride_a, p.stride_b, p.stride_c);
}

// Sum of the fp32 partial tiles of a split reduction, then the epilogue of gemm16_dma_kernel: 8 columns per thread
// (N % 8 == 0), the same fused multiply-adds and the single rounding to T.
template <typename T>
__global__ void __launch_bounds__(256)
gemm16_split_reduce_kernel(const float* __restrict__ partials, T* C, int64_t total8, int N, int64_t plane, int splits,
                           DmaEpilogue epi) {
  typedef typename Half16<T>::vec8 vec8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total8) return;
  const int64_t off = idx * 8;
  const int col     = (int)(off % N);
  float v[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) v[q] = 0.0f;
  // four partial tiles at a time, all their loads in flight together (a fifth split and beyond repeat the round)
  const T* Rt = reinterpret_cast<const T*>(epi.residual);
  vec8 rq;
  if (Rt) rq = *reinterpret_cast<const vec8*>(Rt + off);
  f32x4 sc[2], sh[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    sc[h] = epi.scale ? *reinterpret_cast<const f32x4*>(epi.scale + col + 4 * h) : f32x4{epi.alpha, epi.alpha, epi.alpha, epi.alpha};
    sh[h] = epi.shift ? *reinterpret_cast<const f32x4*>(epi.shift + col + 4 * h) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  for (int s0 = 0; s0 < splits; s0 += 4) {
    f32x4 part[4][2];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        part[u][h] = s0 + u < splits ? *reinterpret_cast<const f32x4*>(partials + (s0 + u) * plane + off + 4 * h)
                                     : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] += part[u][0][q], v[4 + q] += part[u][1][q];
  }
  vec8 out;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    float t = __builtin_fmaf(v[q], sc[q >> 2][q & 3], sh[q >> 2][q & 3]);
    if (Rt) t = __builtin_fmaf(epi.residual_scale, (float)rq[q], t);
    asm volatile("" : "+v"(t));
    if (epi.relu) t = t > 0.0f ? t : 0.0f;
    out[q] = (T)t;
  }
  *reinterpret_cast<vec8*>(C + off) = out;
}

// split a tiles_m x tiles_n grid over the 8 XCDs as gr x gc rectangles with the smallest half-perimeter; sub_rows
// stays 0 when the grid does not divide
void XcdRectangles(int tiles_m, int tiles_n, int* xcd_cols, int* sub_rows, int* sub_cols) {
  for (int gc = 1; gc <= 8; gc *= 2) {
    const int gr = 8 / gc;
    if (tiles_m % gr != 0 || tiles_n % gc != 0) continue;
    const int r = tiles_m / gr, c = tiles_n / gc;
    if (*sub_rows == 0 || r + c < *sub_rows + *sub_cols) {
      *xcd_cols = gc;
      *sub_rows = r;
      *sub_cols = c;
    }
  }
}

// The same for tile counts that do not divide: rectangles of ceil(tiles_m / gr) x ceil(tiles_n / gc) tiles, the grid
// is 8 * sub_rows * sub_cols blocks and those that fall outside the tile grid return at once.
void XcdRectanglesPadded(int tiles_m, int tiles_n, int* xcd_cols, int* sub_rows, int* sub_cols) {
  for (int gc = 1; gc <= 8; gc *= 2) {
    const int gr = 8 / gc;
    const int r = (tiles_m + gr - 1) / gr, c = (tiles_n + gc - 1) / gc;
    if (*sub_rows == 0 || r + c < *sub_rows + *sub_cols) {
      *xcd_cols = gc;
      *sub_rows = r;
      *sub_cols = c;
    }
  }
}

// device buffer of the time-stamp hook, or null (cinn_hip_gemm_set_probe)
std::atomic<unsigned long long*> g_gemm_probe{nullptr};

template <typename T, bool B_KC, int BM, int BN, int WAVES_M, int WAVES_N, bool CONV = false, int NS = 2, bool FEED = false,
          bool PAIR = false>
void LaunchDma16(const GemmProblem& p, hipStream_t stream, int splits = 1) {
  int64_t ldb = p.trans_b ? p.k : p.n;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  // XCD rectangles for tile grids large enough to have panels to share; a small grid per batch entry is numbered
  // linearly (padded rectangles would leave whole XCDs with nothing but blocks that return at once)
  int xcd_cols = 0, sub_rows = 0, sub_cols = 0;
  if (tiles_m * tiles_n >= 64) XcdRectanglesPadded(tiles_m, tiles_n, &xcd_cols, &sub_rows, &sub_cols);
  dim3 grid(sub_rows > 0 ? 8 * sub_rows * sub_cols : tiles_m * tiles_n, p.batch, splits);
  DmaEpilogue epi;
  epi.probe           = g_gemm_probe.load(std::memory_order_relaxed);
  epi.partials        = nullptr;
  epi.steps_per_split = 0;
  if (splits > 1) {
    CINN_RT_CHECK(p.batch == 1 && p.beta == 0.0f, "a split reduction takes one unbatched product without a beta term");
    epi.partials        = static_cast<float*>(cinn_hip_kernels::Scratch(cinn_hip_kernels::ScratchKind::kSplitK, (size_t)splits * p.m * p.n * sizeof(float), stream));
    epi.steps_per_split = (p.k / kD64BK + splits - 1) / splits;
  }
  epi.scale          = p.scale;
  epi.shift          = p.shift;
  epi.alpha          = p.alpha;
  epi.relu           = p.relu ? 1 : 0;
  epi.residual       = p.residual ? p.residual : (p.beta != 0.0f ? p.c : nullptr);
  epi.residual_scale = p.residual ? p.residual_scale : p.beta;
  // plain GEMMs whose result exceeds half of the L2 capacity (8 x 4 MiB) stream it out
  epi.streaming = !p.keep_in_cache && (int64_t)p.batch * p.m * p.n * 2 >= (16 << 20);
  ConvGeom geom{};
  if (CONV) geom = *p.conv;
  hipLaunchKernelGGL((gemm16_dma_kernel<T, B_KC, BM, BN, WAVES_M, WAVES_N, CONV, NS, FEED, PAIR>), grid,
                     dim3(64 * WAVES_M * WAVES_N * (FEED ? 2 : 1)), 0,
                     stream, static_cast<const uint16_t*>(p.a), static_cast<const uint16_t*>(p.b),
                     static_cast<uint16_t*>(p.c), p.m, p.n, p.k, (int64_t)p.k, ldb, (int64_t)p.n, epi, p.stride_a,
                     p.stride_b, p.stride_c, xcd_cols, sub_rows, sub_cols, geom);
  if (splits > 1) {
    const int64_t total8 = (int64_t)p.m * p.n / 8;
    hipLaunchKernelGGL((gemm16_split_reduce_kernel<T>), dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0, stream,
                       epi.partials, static_cast<T*>(p.c), total8, p.n, (int64_t)p.m * p.n, splits, epi);
  }
}

// gemm16_shortk_kernel: K = 64, either layout of B, N a multiple of the 128 columns of a wavefront, at least 16384 rows.
// FLAGS_cinn_hip_gemm_shortk=0 switches it off.
template <typename T, int NT, int KH>
void LaunchShortK(const GemmProblem& p, hipStream_t stream) {
  const int ny     = p.n / (NT * 16);
  const int groups = (p.m + 15) / 16;
  // two blocks of four wavefronts per CU, spread evenly over the XCDs and the column panels
  int slots = (groups + 3) / 4;
  slots     = slots < 512 / ny ? slots : 512 / ny;
  slots     = (slots + 7) / 8 * 8;
  DmaEpilogue epi;
  epi.scale          = p.scale;
  epi.shift          = p.shift;
  epi.alpha          = p.alpha;
  epi.relu           = p.relu ? 1 : 0;
  epi.residual       = p.residual ? p.residual : (p.beta != 0.0f ? p.c : nullptr);
  epi.residual_scale = p.residual ? p.residual_scale : p.beta;
  epi.streaming      = !p.keep_in_cache && (int64_t)p.batch * p.m * p.n * 2 >= (16 << 20);
  dim3 grid(slots * ny, p.batch, 1);
#define CINN_SHORTK_R(RES, B_KC, RELU)                                                                              \
  hipLaunchKernelGGL((gemm16_shortk_kernel<T, NT, KH, RES, B_KC, RELU>), grid, dim3(256), 0, stream,                  \
                     static_cast<const uint16_t*>(p.a), static_cast<const uint16_t*>(p.b), static_cast<uint16_t*>(p.c), \
                     p.m, p.n, (int64_t)p.k, (int64_t)(B_KC ? p.k : p.n), (int64_t)p.n, epi, p.stride_a, p.stride_b,    \
                     p.stride_c, ny)
#define CINN_SHORTK(RES, B_KC)      \
  do {                              \
    if (epi.relu) {                 \
      CINN_SHORTK_R(RES, B_KC, true);  \
    } else {                        \
      CINN_SHORTK_R(RES, B_KC, false); \
    }                               \
  } while (0)
  if (epi.residual) {
    if (p.trans_b) {
      CINN_SHORTK(true, true);
    } else {
      CINN_SHORTK(true, false);
    }
  } else if (p.trans_b) {
    CINN_SHORTK(false, true);
  } else {
    CINN_SHORTK(false, false);
  }
#undef CINN_SHORTK
#undef CINN_SHORTK_R
}

template <typename T>
bool TryShortK(const GemmProblem& p, hipStream_t stream) {
  static const bool enabled = !(getenv("FLAGS_cinn_hip_gemm_shortk") && atoi(getenv("FLAGS_cinn_hip_gemm_shortk")) == 0);
  if (!enabled || p.conv || p.trans_a) return false;
  // measured against the tiled kernels (fp16): 100352 x 256 x 64 17.0 against 22.7 us; with 64 columns, or a
  // K of 128 or 256, or many small batch entries (the filter fragments are reloaded per block) the tiled kernels win
  if (p.k != 64 || p.n % 128 != 0 || p.n > 8192 || p.m < 16384 || p.batch > 65535) return false;
  // 8-byte accesses to C and the residual, 16-byte accesses to A and B
  if (reinterpret_cast<uintptr_t>(p.a) % 16 != 0 || reinterpret_cast<uintptr_t>(p.b) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(p.c) % 8 != 0 || reinterpret_cast<uintptr_t>(p.residual) % 8 != 0 ||
      p.stride_a % 8 != 0 || p.stride_b % 8 != 0 || p.stride_c % 4 != 0)
    return false;
  LaunchShortK<T, 8, 2>(p, stream);
  return true;
}

// gemm16_skinny_kernel: at most 64 rows, A [M][K] and B stored [N][K] (a const weight after the program pass has
// transposed it), one unbatched product, K a multiple of 256 (eight wavefronts of 32-deep blocks).
// FLAGS_cinn_hip_gemm_skinny=0 switches it off.
template <typename T>
bool TrySkinny(const GemmProblem& p, hipStream_t stream) {
  static const bool enabled = !(getenv("FLAGS_cinn_hip_gemm_skinny") && atoi(getenv("FLAGS_cinn_hip_gemm_skinny")) == 0);
  if (!enabled || p.conv || p.trans_a || !p.trans_b || p.batch != 1) return false;
  if (p.m > 64 || p.k % 256 != 0 || (int64_t)p.n * p.k >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(p.a) % 16 != 0 || reinterpret_cast<uintptr_t>(p.b) % 16 != 0) return false;
  DmaEpilogue epi;
  epi.partials        = nullptr;
  epi.steps_per_split = 0;
  epi.scale           = p.scale;
  epi.shift           = p.shift;
  epi.alpha           = p.alpha;
  epi.relu            = p.relu ? 1 : 0;
  epi.residual        = p.residual ? p.residual : (p.beta != 0.0f ? p.c : nullptr);
  epi.residual_scale  = p.residual ? p.residual_scale : p.beta;
  epi.streaming       = 0;
  int mt = (p.m + 15) / 16;
  dim3 grid((unsigned)((p.n + 15) / 16));
  // Fewer column blocks than CUs: one block per 16 rows as well.  A block's traffic is its 16 columns of B plus the
  // rows of A it multiplies, and with all of A (128 KB at 32 x 2048, against 64 KB of B) the few CUs at work are bound
  // by what one CU can pull in; row blocks read B again, out of L2.  ResNet-50's classifier, 32 x 2048 -> 1000: 126
  // blocks instead of 63, 2.2 us less.  With the chip full, the row tiles stay in one block's registers (B read once).
  // FLAGS_cinn_hip_gemm_skinny_rows: 0 never splits the rows, 2 always.
  static const int rows_flag = getenv("FLAGS_cinn_hip_gemm_skinny_rows") ? atoi(getenv("FLAGS_cinn_hip_gemm_skinny_rows")) : 1;
  if (rows_flag == 2 || (rows_flag == 1 && grid.x < 256)) grid.y = mt, mt = 1;
#define CINN_SKINNY(MT)                                                                                        \
  hipLaunchKernelGGL((gemm16_skinny_kernel<T, MT>), grid, dim3(512), 0, stream, static_cast<const uint16_t*>(p.a), \
                     static_cast<const uint16_t*>(p.b), static_cast<uint16_t*>(p.c), p.m, p.n, p.k, epi)
  switch (mt) {
    case 1: CINN_SKINNY(1); break;
    case 2: CINN_SKINNY(2); break;
    case 3: CINN_SKINNY(3); break;
    default: CINN_SKINNY(4); break;
  }
#undef CINN_SKINNY
  return true;
}

// FLAGS_cinn_hip_gemm_feed=0: the four-stage 128x128 instances issue their loads from the computing wavefronts
bool FeedWavefronts() {
  static const bool on = !(getenv("FLAGS_cinn_hip_gemm_feed") && atoi(getenv("FLAGS_cinn_hip_gemm_feed")) == 0);
  return on;
}

// A stored [M][K], K % 64 == 0, N % 8 == 0 (whole 16-byte chunks per row of C and of a row-major B): 256x256 tiles
// when they fill the chip, else 128x128 tiles when there are enough of those; M and N need not be multiples of the
// tile (the last tile row / column computes some rows / columns that are not stored); false when neither applies
template <typename T>
bool TryDma16(const GemmProblem& p, hipStream_t stream) {
  if (TrySkinny<T>(p, stream)) return true;
  if (p.trans_a || p.k % 64 != 0 || p.n % 8 != 0) return false;
  if (TryShortK<T>(p, stream)) return true;
  // every access moves 16 bytes
  if (reinterpret_cast<uintptr_t>(p.a) % 16 != 0 || reinterpret_cast<uintptr_t>(p.b) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(p.c) % 16 != 0 || reinterpret_cast<uintptr_t>(p.residual) % 16 != 0 ||
      p.stride_a % 8 != 0 || p.stride_b % 8 != 0 || p.stride_c % 8 != 0)
    return false;
  // lanes address a tile with 32-bit byte offsets from its first row: 256 rows of K, or 64 rows of N, 16-bit elements
  if (p.k >= (1 << 22) || p.n >= (1 << 24)) return false;
  const int64_t tiles256 = (int64_t)((p.m + 255) / 256) * ((p.n + 255) / 256) * p.batch;
  const int64_t tiles128 = (int64_t)((p.m + 127) / 128) * ((p.n + 127) / 128) * p.batch;
  static const int forced = getenv("FLAGS_cinn_hip_gemm_tile") ? atoi(getenv("FLAGS_cinn_hip_gemm_tile")) : 0;
  // narrow outputs with B stored [N][K] (convolutions to 64 channels): 256x64 tiles on 4x1 wavefronts, two blocks per CU
  const bool narrow = p.trans_b && p.n % 128 != 0 && p.n % 64 == 0 && forced == 0 && !(p.conv && p.conv->x2) &&
                      (int64_t)((p.m + 255) / 256) * (p.n / 64) * p.batch >= 256;
  // 128x128 tiles keep two stages of 32 KiB and two blocks per CU, or - when there is at most one block per CU
  // anyway - four stages: three K steps of loads in flight instead of one (2048^3: 27.8 -> 21.9 us; with more
  // blocks than CUs two blocks of two stages are faster).  FLAGS_cinn_hip_gemm_stages = 2 / 4 forces one form.
  static const int forced_stages = getenv("FLAGS_cinn_hip_gemm_stages") ? atoi(getenv("FLAGS_cinn_hip_gemm_stages")) : 0;
  const int stages = forced_stages ? forced_stages : (tiles128 <= 256 ? 4 : 2);
  if (narrow) {
    if (forced_stages == 4) {
      if (p.conv) {
        LaunchDma16<T, true, 256, 64, 4, 1, true, 4>(p, stream);
      } else {
        LaunchDma16<T, true, 256, 64, 4, 1, false, 4>(p, stream);
      }
    } else if (p.conv) {
      LaunchDma16<T, true, 256, 64, 4, 1, true>(p, stream);
    } else {
      LaunchDma16<T, true, 256, 64, 4, 1>(p, stream);
    }
    return true;
  }
  // Few tiles and a long reduction over K-contiguous operands (2048 -> 512 1x1 on 7x7 at batch 32: 52 tiles of 128x128,
  // K = 2048): 64x64 tiles, one computing and one feeding wavefront per block, four stages - 14.1 against 21.0 us on the
  // 64x64 tiles of the convolution kernel with split K and its reduce kernel.  (3x3 layers measured slower here.)
  // From K = 1024 with up to 127 such tiles as well (1024 -> 256 1x1 on 14x14 at batch 32, 98 tiles: 9.8 against 12.7 us
  // on the register-staged 64x64 tiles and 10.5 us on 128x128 tiles with four stages).
  const bool few_tiles_long_k = (tiles128 < 96 && p.k >= 2048) || (tiles128 < 128 && p.k >= 1024);
  if (p.trans_b && !p.conv && ((forced == 0 && FeedWavefronts() && few_tiles_long_k && p.batch == 1) || forced == 64)) {
    LaunchDma16<T, true, 64, 64, 1, 1, false, 4, true>(p, stream);
    return true;
  }
  if (p.conv && p.conv->x2 != nullptr) {
    // a convolution with a second input: the same tile choices, no split of K (ConvPairShape repeats the conditions)
    if (!p.trans_b || p.batch != 1) return false;
    if (tiles256 >= 192 && forced != 128) {
      LaunchDma16<T, true, 256, 256, 2, 4, true, 2, false, true>(p, stream);
    } else if (tiles128 >= 192 || (tiles128 >= 128 && p.k >= 4096)) {
      if (stages == 4) {
        LaunchDma16<T, true, 128, 128, 2, 2, true, 4, true, true>(p, stream);
      } else {
        LaunchDma16<T, true, 128, 128, 2, 2, true, 2, false, true>(p, stream);
      }
    } else {
      return false;
    }
    return true;
  }
  if (p.conv) {
    // implicit-GEMM convolution: filters are [OC][K]
    if (!p.trans_b) return false;
    if (tiles256 >= 192 && forced != 128) {
      LaunchDma16<T, true, 256, 256, 2, 4, true>(p, stream);
      return true;
    }
    // Few tiles and a long reduction (512 -> 512 3x3 on 7x7 at batch 32: 52 tiles of 128x128, K = 4608): the
    // reduction is split over blockIdx.z so that about 200 blocks run, each at least 8 K steps long; a second kernel
    // adds the partial sums.
    // FLAGS_cinn_hip_gemm_split_k: 0 switches it off, a value of 2 or more forces that many splits
    static const int split_flag = getenv("FLAGS_cinn_hip_gemm_split_k") ? atoi(getenv("FLAGS_cinn_hip_gemm_split_k")) : 1;
    if (split_flag != 0 && FeedWavefronts() && forced == 0 && tiles128 >= 32 && tiles128 < 96 && p.k >= 2048 && p.batch == 1 &&
        p.n % 8 == 0) {
      int splits = split_flag >= 2 ? split_flag : (int)((208 + tiles128 - 1) / tiles128);
      while (splits > 1 && p.k / kD64BK / splits < 8) --splits;
      if (splits > 1) {
        LaunchDma16<T, true, 128, 128, 2, 2, true, 4, true>(p, stream, splits);
        return true;
      }
    }
    // measured on ResNet-50 at batch 32 (fp16): from 192 tiles of 128x128 (four stages up to 256 tiles) the network
    // is 0.5-1 % faster with these layers here than on the 64x64 tiles of the convolution kernel, with 96 tiles 2 %
    // slower; a long K (52 against 73 us at 196 tiles, K = 4608) pays from 128 tiles
    // with the loads issued by wavefronts of their own, a long reduction pays from 96 tiles (256 -> 256 3x3 on 14x14
    // at batch 32, 98 tiles, K = 2304: 21.0 against 22.4 us)
    if (tiles128 >= 192 || (tiles128 >= 128 && p.k >= 4096) || (tiles128 >= 96 && p.k >= 2048 && FeedWavefronts()) ||
        (forced == 128 && tiles128 > 0)) {
      if (stages == 4 && FeedWavefronts()) {
        LaunchDma16<T, true, 128, 128, 2, 2, true, 4, true>(p, stream);
      } else if (stages == 4) {
        LaunchDma16<T, true, 128, 128, 2, 2, true, 4>(p, stream);
      } else {
        LaunchDma16<T, true, 128, 128, 2, 2, true>(p, stream);
      }
      return true;
    }
    return false;
  }
  // rows and columns a tiling computes beyond M and N: 256x256 tiles are passed over when they would compute a fifth
  // more than 128x128 tiles (a [512,64] result is a quarter of one 256x256 tile)
  const double area256 = (double)((p.m + 255) / 256) * ((p.n + 255) / 256) * 4.0;
  const double area128 = (double)((p.m + 127) / 128) * ((p.n + 127) / 128);
  const bool wasteful256 = area256 > 1.2 * area128 && tiles128 >= 128;
  // two K steps or fewer: a block is all start-up and epilogue, and two co-resident blocks of 128x128 overlap them
  // (128 -> 512 1x1 on 28x28 with its residual at batch 32: 20.4 against 21.3 us)
  const bool short_k = p.k <= 128 && tiles128 >= 128;
  if (tiles256 >= 192 && forced != 128 && !wasteful256 && !(short_k && forced == 0)) {
    if (p.trans_b) {
      LaunchDma16<T, true, 256, 256, 2, 4>(p, stream);
    } else {
      LaunchDma16<T, false, 256, 256, 2, 4>(p, stream);
    }
    return true;
  }
  if ((tiles128 >= 128 && forced != 256) || (forced == 128 && tiles128 > 0)) {
    if (stages == 4 && FeedWavefronts()) {
      if (p.trans_b) {
        LaunchDma16<T, true, 128, 128, 2, 2, false, 4, true>(p, stream);
      } else {
        LaunchDma16<T, false, 128, 128, 2, 2, false, 4, true>(p, stream);
      }
    } else if (stages == 4) {
      if (p.trans_b) {
        LaunchDma16<T, true, 128, 128, 2, 2, false, 4>(p, stream);
      } else {
        LaunchDma16<T, false, 128, 128, 2, 2, false, 4>(p, stream);
      }
    } else if (p.trans_b) {
      LaunchDma16<T, true, 128, 128, 2, 2>(p, stream);
    } else {
      LaunchDma16<T, false, 128, 128, 2, 2>(p, stream);
    }
    return true;
  }
  if (tiles256 >= 64) {
    if (p.trans_b) {
      LaunchDma16<T, true, 256, 256, 2, 4>(p, stream);
    } else {
      LaunchDma16<T, false, 256, 256, 2, 4>(p, stream);
    }
    return true;
  }
  return false;
}

bool UseRegisterStaging() {
  static const bool on = getenv("FLAGS_cinn_hip_gemm_register_staging") && atoi(getenv("FLAGS_cinn_hip_gemm_register_staging")) != 0;
  return on;
}

// 256x256 tiles with register staging: every operand layout (used for A stored [K][M])
template <typename T>
void DispatchFast16(const GemmProblem& p, hipStream_t stream) {
  bool a_kc = !p.trans_a, b_kc = p.trans_b;
  if (a_kc && b_kc) LaunchFast16<T, true, true>(p, stream);
  if (a_kc && !b_kc) LaunchFast16<T, true, false>(p, stream);
  if (!a_kc && b_kc) LaunchFast16<T, false, true>(p, stream);
  if (!a_kc && !b_kc) LaunchFast16<T, false, false>(p, stream);
}

template <typename T, typename ACC>
void LaunchGeneric(const GemmProblem& p, hipStream_t stream) {
  int64_t lda = p.trans_a ? p.m : p.k;
  int64_t ldb = p.trans_b ? p.k : p.n;
  dim3 grid((p.n + 63) / 64, (p.m + 63) / 64, p.batch);
  hipLaunchKernelGGL((gemm_generic_kernel<T, ACC>), grid, dim3(256), 0, stream, static_cast<const T*>(p.a),
                     static_cast<const T*>(p.b), static_cast<T*>(p.c), p.m, p.n, p.k, lda, ldb, (int64_t)p.n, p.trans_a,
                     p.trans_b, p.alpha, p.beta, p.stride_a, p.stride_b, p.stride_c);
}

void LaunchFast32(const GemmProblem& p, hipStream_t stream) {
  int64_t lda = p.trans_a ? p.m : p.k;
  int64_t ldb = p.trans_b ? p.k : p.n;
  // 128x128 tiles unless they leave most of the 256 CUs idle; then 64x64 tiles, four times as many blocks
  const bool small = (int64_t)(p.n / kF32Tile) * (p.m / kF32Tile) * p.batch < 256;
  const int tile   = small ? 64 : kF32Tile;
  dim3 grid(p.n / tile, p.m / tile, p.batch);
  const float* a = static_cast<const float*>(p.a);
  const float* b = static_cast<const float*>(p.b);
  float* c       = static_cast<float*>(p.c);
  int xcd_cols = 0, sub_rows = 0, sub_cols = 0;
  XcdRectangles(p.m / tile, p.n / tile, &xcd_cols, &sub_rows, &sub_cols);
#define CINN_LAUNCH_F32(TA, TB)                                                                                        \
  do {                                                                                                                 \
    if (small) {                                                                                                       \
      hipLaunchKernelGGL((gemm32_mfma_kernel<64, TA, TB, 2, 32>), grid, dim3(512), 0, stream, a, b, c, p.m, p.n, p.k,  \
                         lda, ldb, (int64_t)p.n, p.alpha, p.beta, p.stride_a, p.stride_b, p.stride_c, xcd_cols,       \
                         sub_rows, sub_cols);                                                                          \
    } else {                                                                                                           \
      hipLaunchKernelGGL((gemm32_mfma_kernel<128, TA, TB, 1, 32>), grid, dim3(256), 0, stream, a, b, c, p.m, p.n, p.k, \
                         lda, ldb, (int64_t)p.n, p.alpha, p.beta, p.stride_a, p.stride_b, p.stride_c, xcd_cols,       \
                         sub_rows, sub_cols);                                                                          \
    }                                                                                                                  \
  } while (0)
  if (!p.trans_a && !p.trans_b) CINN_LAUNCH_F32(false, false);
  if (!p.trans_a && p.trans_b) CINN_LAUNCH_F32(false, true);
  if (p.trans_a && !p.trans_b) CINN_LAUNCH_F32(true, false);
  if (p.trans_a && p.trans_b) CINN_LAUNCH_F32(true, true);
#undef CINN_LAUNCH_F32
}

bool ForceGeneric() {
  static const bool force = getenv("FLAGS_cinn_hip_gemm_generic") && atoi(getenv("FLAGS_cinn_hip_gemm_generic")) != 0;
  return force;
}

void RunGemm(const GemmProblem& p, hipStream_t stream) {
  CINN_RT_CHECK(p.m > 0 && p.n > 0 && p.k > 0 && p.batch > 0, "gemm: dimensions must be positive, got m=%d n=%d k=%d batch=%d",
                p.m, p.n, p.k, p.batch);
  CINN_RT_CHECK(p.a && p.b && p.c, "gemm: null operand");
  CINN_RT_CHECK(p.batch <= 65535, "gemm: batch %d exceeds the grid limit", p.batch);
  const bool fast16 = !ForceGeneric() && p.m % kBM == 0 && p.n % kBN == 0 && p.k % kBK == 0;
  const bool aligned16 = reinterpret_cast<uintptr_t>(p.a) % 16 == 0 && reinterpret_cast<uintptr_t>(p.b) % 16 == 0 &&
                         p.stride_a % 4 == 0 && p.stride_b % 4 == 0;
  const bool fast32 = !ForceGeneric() && p.m % kF32Tile == 0 && p.n % kF32Tile == 0 && p.k % kF32K == 0 && aligned16;
  if (!ForceGeneric() && !UseRegisterStaging() && (p.type == GemmType::kBF16 || p.type == GemmType::kF16)) {
    const bool taken = p.type == GemmType::kBF16 ? TryDma16<__bf16>(p, stream) : TryDma16<_Float16>(p, stream);
    if (taken) {
      CINN_HIP_CALL(hipGetLastError());
      return;
    }
  }
  // Shapes the big-tile kernels do not take (ragged, or so few tiles that most CUs would idle) go to the
  // channels-last convolution kernels: a 1x1 convolution over m "pixels" is this GEMM with both operands
  // K-contiguous (A [m,k], B stored [n,k]); those kernels bound-check every tile edge, use 64x64 tiles and split K
  // when the grid is small.  An operand stored the other way round is transposed into scratch first, which costs one
  // pass over that operand.
  const int elem_bytes = p.type == GemmType::kF32 ? 4 : (p.type == GemmType::kF64 ? 8 : 2);
  const bool tile_fit  = p.type == GemmType::kF32 ? fast32 : fast16;
  const int64_t tiles  = p.type == GemmType::kF32 ? (int64_t)(p.m / 64) * (p.n / 64) * p.batch
                                                  : (int64_t)(p.m / kBM) * (p.n / kBN) * p.batch;
  const bool few_tiles = tile_fit && tiles < 64;
  const bool flexible  = !ForceGeneric() && p.type != GemmType::kF64 && p.k % (16 / elem_bytes) == 0 &&
                         reinterpret_cast<uintptr_t>(p.a) % 16 == 0 && reinterpret_cast<uintptr_t>(p.b) % 16 == 0;
  if (flexible && (!tile_fit || few_tiles)) {
    const char* a_base = static_cast<const char*>(p.a);
    const char* b_base = static_cast<const char*>(p.b);
    int64_t stride_a = p.stride_a, stride_b = p.stride_b;
    if (p.trans_a || !p.trans_b) {
      const int batch_a    = p.trans_a ? (p.stride_a == 0 ? 1 : p.batch) : 0;
      const int batch_b    = !p.trans_b ? (p.stride_b == 0 ? 1 : p.batch) : 0;
      const size_t bytes_a = (size_t)batch_a * p.m * p.k * elem_bytes;
      const size_t bytes_b = (size_t)batch_b * p.k * p.n * elem_bytes;
      char* scratch        = static_cast<char*>(cinn_hip_kernels::Scratch(cinn_hip_kernels::ScratchKind::kTranspose, bytes_a + bytes_b, stream));
      if (p.trans_a) {  // stored [k][m]
        LaunchTranspose(p.a, scratch, p.k, p.m, batch_a, p.stride_a, elem_bytes, stream);
        a_base   = scratch;
        stride_a = p.stride_a == 0 ? 0 : (int64_t)p.m * p.k;
      }
      if (!p.trans_b) {  // stored [k][n]
        LaunchTranspose(p.b, scratch + bytes_a, p.k, p.n, batch_b, p.stride_b, elem_bytes, stream);
        b_base   = scratch + bytes_a;
        stride_b = p.stride_b == 0 ? 0 : (int64_t)p.k * p.n;
      }
    }
    for (int b = 0; b < p.batch; ++b) {
      cinn_hip_kernels::ConvNhwcArgs a;
      a.x = a_base + (int64_t)b * stride_a * elem_bytes;
      a.w = b_base + (int64_t)b * stride_b * elem_bytes;
      a.y = static_cast<char*>(p.c) + (int64_t)b * p.stride_c * elem_bytes;
      a.scale = a.shift = nullptr;
      a.residual        = p.beta != 0.0f ? a.y : nullptr;
      a.alpha           = p.alpha;
      a.residual_scale  = p.beta;
      a.relu            = false;
      a.nchw_input      = false;
      a.n = 1, a.h = 1, a.w_in = p.m, a.c = p.k;
      a.oc = p.n, a.kh = 1, a.kw = 1, a.oh = 1, a.ow = p.m;
      a.pad_h = a.pad_w = 0;
      a.stride_h = a.stride_w = a.dil_h = a.dil_w = 1;
      a.type.code  = p.type == GemmType::kBF16 ? cinn_type_bfloat : cinn_type_float;
      a.type.bits  = static_cast<uint8_t>(elem_bytes * CHAR_BIT);
      a.type.lanes = 1;
      cinn_hip_kernels::RunConvNhwc(a, stream);
    }
    return;
  }
  switch (p.type) {
    case GemmType::kBF16:
      if (fast16) {
        DispatchFast16<__bf16>(p, stream);
      } else {
        LaunchGeneric<__bf16, float>(p, stream);
      }
      break;
    case GemmType::kF16:
      if (fast16) {
        DispatchFast16<_Float16>(p, stream);
      } else {
        LaunchGeneric<_Float16, float>(p, stream);
      }
      break;
    case GemmType::kF32:
      if (fast32) {
        LaunchFast32(p, stream);
      } else {
        LaunchGeneric<float, float>(p, stream);
      }
      break;
    case GemmType::kF64: LaunchGeneric<double, double>(p, stream); break;
  }
  CINN_HIP_CALL(hipGetLastError());
}

GemmType TypeOf(const cinn_buffer_t* buf) {
  int bytes = buf->type.bits / CHAR_BIT;
  if (buf->type.code == cinn_type_float && bytes == 2) return GemmType::kF16;
  if (buf->type.code == cinn_type_float && bytes == 4) return GemmType::kF32;
  if (buf->type.code == cinn_type_float && bytes == 8) return GemmType::kF64;
  if (buf->type.code == cinn_type_bfloat) return GemmType::kBF16;
  fprintf(stderr, "unsupported gemm data type: code %d, bits %d\n", buf->type.code, buf->type.bits);
  abort();
}

cinn_buffer_t* BufferArg(void* v_args, int index) {
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  CINN_RT_CHECK(args[index].type_code_ == CINN_POD_BUFFER_P, "gemm: argument %d is not a buffer", index);
  return static_cast<cinn_buffer_t*>(args[index].value_.v_handle);
}

}  // namespace

namespace cinn_hip_kernels {

bool ConvPairShape(int64_t m, int c1, int c2, int oc) {
  if (m <= 0 || m >= INT_MAX || c1 <= 0 || c2 <= 0 || oc <= 0 || c1 % kD64BK != 0 || c2 % kD64BK != 0 || oc % 8 != 0) return false;
  // the tile counts from which TryDma16 sends an implicit GEMM to one of its instances without splitting K
  const int64_t tiles256 = ((m + 255) / 256) * ((oc + 255) / 256);
  const int64_t tiles128 = ((m + 127) / 128) * ((oc + 127) / 128);
  return tiles256 >= 192 || tiles128 >= 192 || (tiles128 >= 128 && c1 + c2 >= 4096);
}

bool TryPointwiseConvAsGemm(const ConvNhwcArgs& a, hipStream_t stream) {
  // FLAGS_cinn_hip_conv_pointwise_gemm: 0 keeps 1x1 layers on the convolution kernel, 2 sends every one the GEMM
  // kernels can take to them, whatever the grid (for measurements)
  static const int mode = getenv("FLAGS_cinn_hip_conv_pointwise_gemm") ? atoi(getenv("FLAGS_cinn_hip_conv_pointwise_gemm")) : 1;
  const bool enabled = mode != 0;
  // a second input has no other implementation: the measurement flags do not apply to it
  const bool pair = a.x2 != nullptr;
  if (!pair && (!enabled || ForceGeneric() || UseRegisterStaging())) return false;
  const bool is_f16  = a.type.code == cinn_type_float && a.type.bits == 16;
  const bool is_bf16 = a.type.code == cinn_type_bfloat && a.type.bits == 16;
  if (!is_f16 && !is_bf16) return false;
  if (a.nchw_input) return false;
  const int64_t pixels = (int64_t)a.n * a.oh * a.ow;
  if (pixels >= INT_MAX) return false;
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.w) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(a.y) % 16 != 0 || reinterpret_cast<uintptr_t>(a.residual) % 16 != 0)
    return false;
  if (reinterpret_cast<uintptr_t>(a.x2) % 16 != 0) return false;
  const bool pointwise = !pair && a.kh == 1 && a.kw == 1 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 0 && a.pad_w == 0 &&
                         a.oh == a.h && a.ow == a.w_in;
  GemmProblem p;
  ConvGeom geom{};
  if (pointwise) {
    // measured inside ResNet-50 at batch 32: the GEMM kernels win from 192 tiles of 128x128 and a K loop of two steps
    // or more; smaller grids are better served by the 64x64 tiles and split K of the convolution kernel
    const bool narrow = a.oc % 128 != 0 && a.oc % 64 == 0 && ((pixels + 255) / 256) * (a.oc / 64) >= 256;
    static const bool shortk_on = !(getenv("FLAGS_cinn_hip_gemm_shortk") && atoi(getenv("FLAGS_cinn_hip_gemm_shortk")) == 0);
    const bool shortk = shortk_on && a.c == 64 && a.oc % 128 == 0 && pixels >= 16384;
    static const int forced_tile = getenv("FLAGS_cinn_hip_gemm_tile") ? atoi(getenv("FLAGS_cinn_hip_gemm_tile")) : 0;
    // few tiles but a long reduction: the single-wavefront 64x64 tiles of the GEMM kernel (see TryDma16)
    const bool long_k = forced_tile == 64 || (forced_tile == 0 && a.oc % 64 == 0 &&
                                              (a.c >= 2048 || (a.c >= 1024 && ((pixels + 127) / 128) * ((a.oc + 127) / 128) < 128)));
    // at most 64 pixels (a matmul with few rows written as a 1x1 layer, its bias as the shift): gemm16_skinny_kernel
    const bool few_rows = forced_tile == 0 && pixels <= 64 && a.c % 256 == 0;
    if (mode != 2 && !shortk && !long_k && !few_rows &&
        (a.c < 128 || (!narrow && ((pixels + 127) / 128) * ((a.oc + 127) / 128) < 192)))
      return false;
    p.k = a.c;
  } else {
    // any filter, stride, padding, dilation: implicit GEMM, K = kh * kw * c with 64-channel steps inside a tap
    static const bool conv_enabled = !(getenv("FLAGS_cinn_hip_conv_implicit_gemm") && atoi(getenv("FLAGS_cinn_hip_conv_implicit_gemm")) == 0);
    if ((!conv_enabled && !pair) || a.c % 64 != 0 || (int64_t)a.n * a.h * a.w_in * a.c >= INT_MAX) return false;
    // window corners are kept as two signed 16-bit coordinates
    if (a.h + a.pad_h >= 32768 || a.w_in + a.pad_w >= 32768) return false;
    geom.h = a.h, geom.w = a.w_in, geom.c = a.c;
    geom.oh_ow = a.oh * a.ow, geom.ow = a.ow, geom.kw = a.kw;
    geom.stride_h = a.stride_h, geom.stride_w = a.stride_w, geom.pad_h = a.pad_h, geom.pad_w = a.pad_w;
    geom.dil_h = a.dil_h, geom.dil_w = a.dil_w;
    geom.zero_page = ConvZeroPage();
    p.conv = &geom;
    p.k    = a.kh * a.kw * a.c;
    if (pair) {
      // the second input's pixel (oy stride2_h, ox stride2_w) must exist for every output pixel
      if (a.c2 <= 0 || a.c2 % 64 != 0 || a.stride2_h <= 0 || a.stride2_w <= 0 || (a.oh - 1) * a.stride2_h >= a.h2 ||
          (a.ow - 1) * a.stride2_w >= a.w2 || a.h2 >= 32768 || a.w2 >= 32768 || (int64_t)a.n * a.h2 * a.w2 * a.c2 >= INT_MAX)
        return false;
      geom.x2 = a.x2;
      geom.h2 = a.h2, geom.w2 = a.w2, geom.c2 = a.c2;
      geom.stride2_h = a.stride2_h, geom.stride2_w = a.stride2_w;
      geom.steps1    = p.k / kD64BK;
      p.k += a.c2;
    }
  }
  p.type    = is_bf16 ? GemmType::kBF16 : GemmType::kF16;
  p.a       = a.x;  // [pixels][c], or the NHWC input of the implicit GEMM
  p.b       = a.w;  // [oc][kh * kw * c]
  p.c       = a.y;
  p.m       = static_cast<int>(pixels);
  p.n       = a.oc;
  p.trans_a = false;
  p.trans_b = true;
  p.alpha   = a.alpha;
  p.beta    = 0.0f;
  p.batch   = 1;
  p.stride_a = p.stride_b = p.stride_c = 0;
  p.scale          = a.scale;
  p.shift          = a.shift;
  p.residual       = a.residual;
  p.residual_scale = a.residual_scale;
  p.relu           = a.relu;
  p.keep_in_cache  = true;
  const bool taken = is_bf16 ? TryDma16<__bf16>(p, stream) : TryDma16<_Float16>(p, stream);
  if (taken) CINN_HIP_CALL(hipGetLastError());
  return taken;
}

}  // namespace cinn_hip_kernels

extern "C" {

// Measurement hook, exported but deliberately absent from the public header (declared in kernels/conv_nhwc.h): every
// later launch of the direct-to-LDS GEMM kernel writes four time-stamp pairs per block to `device_buffer` (8 x 8 bytes
// per block of the launch; the caller sizes it), until it is called again with null.
void cinn_hip_gemm_set_probe(void* device_buffer) {
  g_gemm_probe.store(static_cast<unsigned long long*>(device_buffer), std::memory_order_relaxed);
}

// Shape algebra of cinn_call_cublas (cinn/runtime/cuda/cuda_util.cc:121-310) restated for a row-major kernel:
// the result is [a1', a2', M, N] with M = trans_a ? a4 : a3, K = trans_a ? a3 : a4, N = trans_b ? b3 : b4;
// trans_o stores the transposed product, which is the product of the swapped, re-transposed operands.
// Leading dimensions broadcast: an operand whose leading dims are 1 is shared by every batch.
void cinn_call_cublas(void* v_args, int num_args, bool trans_a, bool trans_b, bool trans_o, float alpha, float beta,
                      int a1, int a2, int a3, int a4, int b1, int b2, int b3, int b4, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  CINN_RT_CHECK(num_args == 3, "cinn_call_cublas takes A, B and C, got %d arguments", num_args);
  cinn_buffer_t* A = BufferArg(v_args, 0);
  cinn_buffer_t* B = BufferArg(v_args, 1);
  cinn_buffer_t* C = BufferArg(v_args, 2);
  const int m = trans_a ? a4 : a3;
  const int k = trans_a ? a3 : a4;
  const int n = trans_b ? b3 : b4;
  CINN_RT_CHECK(k == (trans_b ? b4 : b3), "cinn_call_cublas: inner dimensions differ (%d vs %d)", k, trans_b ? b4 : b3);
  CINN_RT_CHECK((a1 == b1 || a1 == 1 || b1 == 1) && (a2 == b2 || a2 == 1 || b2 == 1),
                "cinn_call_cublas: batch dims [%d,%d] and [%d,%d] do not broadcast", a1, a2, b1, b2);
  const int o1 = a1 > b1 ? a1 : b1, o2 = a2 > b2 ? a2 : b2;

  GemmProblem p;
  p.type  = TypeOf(A);
  p.alpha = alpha;
  p.beta  = beta;
  // The batch goes to the grid.  Both batch dims fold into one when every operand is either batched over both or
  // broadcast over both (one stride per operand describes it); otherwise one launch per leading index o1.
  const int64_t a_mat = (int64_t)a3 * a4, b_mat = (int64_t)b3 * b4, c_mat = (int64_t)m * n;
  const int elem = A->type.bits / CHAR_BIT;
  const bool a_full = a1 == o1 && a2 == o2, a_bcast = a1 == 1 && a2 == 1;
  const bool b_full = b1 == o1 && b2 == o2, b_bcast = b1 == 1 && b2 == 1;
  const bool fold   = o1 > 1 && (a_full || a_bcast) && (b_full || b_bcast) && (int64_t)o1 * o2 <= 65535;
  const int launches = fold ? 1 : o1;
  const int batch    = fold ? o1 * o2 : o2;
  for (int i1 = 0; i1 < launches; ++i1) {
    const char* a_base = reinterpret_cast<const char*>(A->memory) + (a1 == 1 ? 0 : (int64_t)i1 * a2 * a_mat) * elem;
    const char* b_base = reinterpret_cast<const char*>(B->memory) + (b1 == 1 ? 0 : (int64_t)i1 * b2 * b_mat) * elem;
    char* c_base       = reinterpret_cast<char*>(C->memory) + (int64_t)i1 * o2 * c_mat * elem;
    const int64_t sa = fold ? (a_full ? a_mat : 0) : (a2 == 1 ? 0 : a_mat);
    const int64_t sb = fold ? (b_full ? b_mat : 0) : (b2 == 1 ? 0 : b_mat);
    if (!trans_o) {
      p.a = a_base, p.b = b_base, p.c = c_base;
      p.m = m, p.n = n, p.k = k;
      p.trans_a = trans_a, p.trans_b = trans_b;
      p.stride_a = sa, p.stride_b = sb;
    } else {
      // C^T[n, m] = op(B)^T[n, k] * op(A)^T[k, m]
      p.a = b_base, p.b = a_base, p.c = c_base;
      p.m = n, p.n = m, p.k = k;
      p.trans_a = !trans_b, p.trans_b = !trans_a;
      p.stride_a = sb, p.stride_b = sa;
    }
    p.batch    = batch;
    p.stride_c = c_mat;
    RunGemm(p, static_cast<hipStream_t>(stream));
  }
}

// cinn_call_batched_cublas (cuda_util.cc:312-437): v_args = {shared operand, others..., outputs...}; every
// (other_i, output_i) pair is one cinn_call_cublas-shaped problem with the shared operand on side `opside`.
void cinn_call_batched_cublas(void* v_args, int num_args, int opside, bool trans_a, bool trans_b, bool trans_o,
                              float alpha, float beta, int a1, int a2, int a3, int a4, int b1, int b2, int b3, int b4,
                              void* stream) {
  CINN_RT_CHECK(num_args >= 3 && (num_args - 1) % 2 == 0, "cinn_call_batched_cublas: %d arguments", num_args);
  const int pairs = (num_args - 1) / 2;
  auto* args      = static_cast<cinn_pod_value_t*>(v_args);
  for (int i = 0; i < pairs; ++i) {
    cinn_pod_value_t triple[3];
    triple[opside == 0 ? 0 : 1] = args[0];
    triple[opside == 0 ? 1 : 0] = args[1 + i];
    triple[2]                   = args[1 + pairs + i];
    cinn_call_cublas(triple, 3, trans_a, trans_b, trans_o, alpha, beta, a1, a2, a3, a4, b1, b2, b3, b4, stream);
  }
}

}  // extern "C"
