// Device helpers shared by the kernels that keep a convolution's input patch in LDS (conv_patch_mfma.hip,
// conv_stem7_mfma.hip): the 16x16x32 MFMA per element type, the swizzle of filter-stage rows read in permuted order,
// lane exchange for whole-line stores, an LDS-only block barrier, and the host-side reciprocal for index divisions.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace cinn_hip_kernels {
namespace tile {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// two fp32 values rounded to nearest even into one dword of two T (v_cvt_pk_f16_f32 / v_cvt_pk_bf16_f32)
template <typename T>
__device__ __forceinline__ uint32_t PackPair(float a, float b) {
  typedef T pair_t __attribute__((ext_vector_type(2)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, pair_t));
}

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

// Filter rows of a [64 rows][64 halves] stage are read in the order 32 (j / 2) + 8 g' + 4 (j % 2) + r' (tile j,
// q = lane & 15 = 4 g' + r'), which leaves a lane of the transposed MFMA result with 2 x 8 consecutive output channels
// of one pixel.  The 16-byte chunk c of row r sits at chunk slot c ^ FilterKey(r): bits 1 and 3 of the row tell the
// eight rows apart that LDS serves together, so those reads are conflict free.
__device__ __forceinline__ int FilterKey(int r) { return ((r >> 1) & 1) * 2 + ((r >> 3) & 1) * 4 + ((r >> 2) & 1); }

// the value that lane (l & 15) - 8 (SHR) or + 8 of the same row of 16 lanes holds; 0 where that lane does not exist
template <bool SHR>
__device__ __forceinline__ unsigned RowShift8(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, SHR ? 0x118 : 0x108, 0xf, 0xf, true);
}

// Block barrier that orders LDS accesses only.  __syncthreads() also waits until every global store of the wavefront
// has completed (its release covers global memory), which would hold a persistent block at every tile until the
// tile's results have left the CU instead of letting them drain under the next tile's MFMAs.
__device__ __forceinline__ void BarrierLds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// 16 bytes per lane from global memory straight into LDS at lds_addr_uniform + 16 * lane.  Inline assembly, so that
// the compiler does not track the load (tracked, every later LDS read would wait for vmcnt(0)).
__device__ __forceinline__ void AsyncCopy16(const void* src, unsigned lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr_uniform), "v"(src) : "memory");
}

// q = (n * magic) >> shift == n / d for 0 <= n < 2^31 (Granlund-Montgomery with a 64-bit product)
inline void MagicFor(int d, unsigned* magic, unsigned* shift) {
  int l = 0;
  while ((1ll << l) < d) ++l;
  *shift = 31 + l;
  *magic = (unsigned)(((1ull << *shift) / (unsigned)d) + 1);
  if (d == 1) {  // 2^31 + 1 would round n = 2^31 - 1 up; d == 1 needs no rounding at all
    *shift = 0;
    *magic = 1;
  }
}

}  // namespace tile
}  // namespace cinn_hip_kernels
