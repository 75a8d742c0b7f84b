// argsort / sort along one axis: cinn_call_hip_argsort.
//
// What the reference computes (cinn/hlir/op/contrib/sort.cc:50-139 over the intrinsics cinn_host_lt_num_* /
// cinn_host_gt_num_* and cinn_host_next_smallest_int32, cinn/runtime/cpu/host_intrinsics.cc:67-106; the same on the GPU,
// cinn_cuda_runtime_source.cuh:645-715): every element gets the count of elements of its row that are smaller (larger
// when descending) - its *position* - and the index list is then built by taking, slot after slot, the element with
// the smallest position that has not been taken yet, the first such element on ties.  So the result is the order by
// (position, index): a stable sort, ascending or descending, with every NaN at position 0 (no comparison with a NaN
// is true) interleaved by index with the other elements of position 0.
//
// The reference's device code runs that second step from every thread on one shared buffer of positions that each
// call overwrites - it races.  Here an element computes its final slot directly:
//   slot(k) = #{ j : position(j) < position(k) } + #{ j < k : position(j) == position(k) },
// which is the same order and needs no shared mutable state; the index (and for sort the value) is scattered to that
// slot.  Rows without a NaN - the usual case, checked per tile - need one pass only, because position order is value
// order there: slot(k) = #{ x_j < x_k } + #{ j < k : x_j == x_k }.
//
// One block owns a tile of `size` elements along the sorted axis x TI neighbours along the axes after it (consecutive
// in memory, so loads and stores of a tile are whole lines when inner > 1; TI = 1 for the trailing axis).  The keys sit
// in LDS; the scan over a column reads four keys per instruction, the same for every lane of a column (a broadcast).
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

#include "cinn_hip_runtime.h"
#include "runtime/hip_check.h"

namespace {

constexpr int kThreads  = 256;
constexpr int kLdsLimit = 128 * 1024;

struct SortParams {
  const void* x;
  int32_t* index;  // may be null
  int32_t* rank;   // may be null: the position of every element (count of smaller / larger elements of its row)
  void* sorted;    // may be null
  int size, inner, ti;  // ti: neighbouring columns per tile
  int tiles_per_outer;  // ceil(inner / ti)
  int descending;
};

template <typename T>
struct KeyOf {
  typedef float type;
};
template <>
struct KeyOf<double> {
  typedef double type;
};
template <>
struct KeyOf<int32_t> {
  typedef int32_t type;
};
template <>
struct KeyOf<int64_t> {
  typedef int64_t type;
};

template <typename K>
__device__ __forceinline__ bool IsNan(K v) {
  return v != v;
}

// Ahead: a comes strictly before b in value order; AheadOrEqual: or ties with it
template <bool DESC, typename K>
__device__ __forceinline__ bool Ahead(K a, K b) {
  return DESC ? a > b : a < b;
}
template <bool DESC, typename K>
__device__ __forceinline__ bool AheadOrEqual(K a, K b) {
  return DESC ? a >= b : a <= b;
}

// a key that is never strictly ahead of any other: the padding of a column
template <bool DESC, typename K>
__device__ __forceinline__ K LastKey() {
  if (sizeof(K) == 8 && K(0.5) != K(0)) return DESC ? K(-__builtin_huge_val()) : K(__builtin_huge_val());
  if (K(0.5) != K(0)) return DESC ? K(-__builtin_huge_valf()) : K(__builtin_huge_valf());
  if (sizeof(K) == 8) return DESC ? K(LLONG_MIN) : K(LLONG_MAX);
  return DESC ? K(INT_MIN) : K(INT_MAX);
}

template <typename T, bool DESC>
__global__ void __launch_bounds__(kThreads) argsort_tile_kernel(SortParams p) {
  typedef typename KeyOf<T>::type K;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int size = p.size, ti = p.ti;
  const int size4 = (size + 3) & ~3;  // rows of the tile, padded so that four keys of a column are one aligned read
  K* const keys = reinterpret_cast<K*>(lds);                                   // [ti][size4]
  int* const pos = reinterpret_cast<int*>(lds + (size_t)ti * size4 * sizeof(K));  // [ti][size4], NaN tiles only
  const int outer = blockIdx.x / p.tiles_per_outer;
  const int i0    = (blockIdx.x - outer * p.tiles_per_outer) * ti;
  const int cols  = min(ti, p.inner - i0);
  const int64_t base = (int64_t)outer * size * p.inner + i0;
  const T* const X   = static_cast<const T*>(p.x);
  const int items    = size * cols;

  // item q = row k = q / cols, column c = q % cols: consecutive threads on consecutive addresses
  int has_nan = 0;
  for (int q = threadIdx.x; q < items; q += kThreads) {
    const int k = q / cols, c = q - k * cols;
    const K v   = static_cast<K>(X[base + (int64_t)k * p.inner + c]);
    keys[c * size4 + k] = v;
    has_nan |= IsNan(v) ? 1 : 0;
  }
  // the padding is read, four keys at a time, with the keys behind an element: never strictly ahead of anything
  for (int q = threadIdx.x; q < cols * (size4 - size); q += kThreads) {
    const int c = q / (size4 - size), k = size + q - c * (size4 - size);
    keys[c * size4 + k] = LastKey<DESC, K>();
  }
  has_nan = __syncthreads_or(has_nan);

  auto scatter = [&](int k, int c, int slot, int position) {
    const int64_t at = base + (int64_t)slot * p.inner + c;
    if (p.index) p.index[at] = k;
    if (p.sorted) static_cast<T*>(p.sorted)[at] = X[base + (int64_t)k * p.inner + c];
    if (p.rank) p.rank[base + (int64_t)k * p.inner + c] = position;
  };

  if (!has_nan) {
    // here items are (column, row) with the row fastest: the lanes of a wavefront scan the same column.  Keys before
    // the element count when they are ahead of it or equal, keys behind it when they are strictly ahead: two loops of
    // one comparison and one add per key, around the group of four that holds the element itself.
    for (int q = threadIdx.x; q < items; q += kThreads) {
      const int c = q / size, k = q - c * size;
      const K* col = keys + c * size4;
      const K mine = col[k];
      const int kg = k & ~3;
      int slot = 0, ahead = 0;
      for (int j = 0; j < kg; j += 4) {
        K v[4];
        __builtin_memcpy(v, col + j, sizeof(v));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          slot += AheadOrEqual<DESC>(v[u], mine) ? 1 : 0;
          ahead += Ahead<DESC>(v[u], mine) ? 1 : 0;
        }
      }
      {
        K v[4];
        __builtin_memcpy(v, col + kg, sizeof(v));
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool is_ahead = Ahead<DESC>(v[u], mine);
          ahead += is_ahead ? 1 : 0;
          slot += (is_ahead || (kg + u < k && v[u] == mine)) ? 1 : 0;
        }
      }
      int behind = 0;
      for (int j = kg + 4; j < size4; j += 4) {
        K v[4];
        __builtin_memcpy(v, col + j, sizeof(v));
#pragma unroll
        for (int u = 0; u < 4; ++u) behind += Ahead<DESC>(v[u], mine) ? 1 : 0;
      }
      scatter(k, c, slot + behind, ahead + behind);
    }
    return;
  }

  // tiles with a NaN: positions first, then the order by (position, index)
  for (int q = threadIdx.x; q < items; q += kThreads) {
    const int c = q / size, k = q - c * size;
    const K* col = keys + c * size4;
    const K mine = col[k];
    int ahead = 0;
    for (int j = 0; j < size; ++j) ahead += Ahead<DESC>(col[j], mine) ? 1 : 0;
    pos[c * size4 + k] = ahead;
  }
  __syncthreads();
  for (int q = threadIdx.x; q < items; q += kThreads) {
    const int c = q / size, k = q - c * size;
    const int* col = pos + c * size4;
    const int mine = col[k];
    int slot = 0;
    for (int j = 0; j < size; ++j) slot += (col[j] < mine || (col[j] == mine && j < k)) ? 1 : 0;
    scatter(k, c, slot, mine);
  }
}

enum class Elem { kF32, kF64, kF16, kBF16, kI32, kI64, kUnsupported };

Elem ElemOf(const cinn_buffer_t* b) {
  const auto& t = b->type;
  if (t.code == cinn_type_float && t.bits == 32) return Elem::kF32;
  if (t.code == cinn_type_float && t.bits == 64) return Elem::kF64;
  if (t.code == cinn_type_float && t.bits == 16) return Elem::kF16;
  if (t.code == cinn_type_bfloat && t.bits == 16) return Elem::kBF16;
  if (t.code == cinn_type_int && t.bits == 32) return Elem::kI32;
  if (t.code == cinn_type_int && t.bits == 64) return Elem::kI64;
  return Elem::kUnsupported;
}

cinn_buffer_t* BufferArg(void* v_args, int index) {
  auto* args = static_cast<cinn_pod_value_t*>(v_args);
  CINN_RT_CHECK(args[index].type_code_ == CINN_POD_BUFFER_P, "argsort: argument %d is not a buffer", index);
  auto* b = static_cast<cinn_buffer_t*>(args[index].value_.v_handle);
  CINN_RT_CHECK(b && b->memory, "argsort: argument %d has no device memory", index);
  return b;
}

template <typename T, bool DESC>
void LaunchDirection(const SortParams& p, int blocks, size_t lds_bytes, hipStream_t stream) {
  auto kernel = argsort_tile_kernel<T, DESC>;
  static const bool configured = [&] {  // once per instantiation, thread-safe
    CINN_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    return true;
  }();
  (void)configured;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), lds_bytes, stream, p);
}

template <typename T>
void Launch(const SortParams& p, int blocks, size_t lds_bytes, hipStream_t stream) {
  if (p.descending) {
    LaunchDirection<T, true>(p, blocks, lds_bytes, stream);
  } else {
    LaunchDirection<T, false>(p, blocks, lds_bytes, stream);
  }
}

}  // namespace

extern "C" void cinn_call_hip_argsort(void* v_args, int num_args, int outer, int size, int inner, int is_ascend,
                                       int outputs, void* stream) {
  CINN_HIP_CLEAR_STALE_ERROR();
  const int want = ((outputs & 1) ? 1 : 0) + ((outputs & 2) ? 1 : 0) + ((outputs & 4) ? 1 : 0);
  CINN_RT_CHECK(outputs >= 1 && outputs <= 7, "argsort: outputs is a set of bits 1 (indices), 2 (positions), 4 (sorted values), got %d", outputs);
  CINN_RT_CHECK(num_args == 1 + want, "argsort: the input and %d outputs expected, got %d arguments", want, num_args);
  CINN_RT_CHECK(outer >= 0 && size >= 0 && inner >= 0, "argsort: negative extent");
  if ((int64_t)outer * size * inner == 0) return;
  CINN_RT_CHECK((int64_t)outer * size * inner < INT_MAX, "argsort: tensor too large for 32-bit offsets");
  cinn_buffer_t* x = BufferArg(v_args, 0);
  const Elem elem  = ElemOf(x);
  CINN_RT_CHECK(elem != Elem::kUnsupported, "argsort: element type (code %d, %d bits) is not one of fp16 / bf16 / fp32 / fp64 / int32 / int64",
                (int)x->type.code, (int)x->type.bits);
  SortParams p{};
  p.x   = x->memory;
  int a = 1;
  auto int32_output = [&](const char* what) {
    cinn_buffer_t* b = BufferArg(v_args, a++);
    CINN_RT_CHECK(b->type.code == cinn_type_int && b->type.bits == 32, "argsort: the %s output must be int32", what);
    return reinterpret_cast<int32_t*>(b->memory);
  };
  if (outputs & 1) p.index = int32_output("index");
  if (outputs & 2) p.rank = int32_output("position");
  if (outputs & 4) {
    cinn_buffer_t* b = BufferArg(v_args, a++);
    CINN_RT_CHECK(b->type.code == x->type.code && b->type.bits == x->type.bits, "argsort: the sorted output must have the input's type");
    CINN_RT_CHECK(b->memory != x->memory, "argsort: sorting in place is not supported");
    p.sorted = b->memory;
  }
  p.size = size, p.inner = inner, p.descending = is_ascend ? 0 : 1;
  const size_t key_bytes = (elem == Elem::kF64 || elem == Elem::kI64) ? 8 : 4;
  const size_t per_col   = (size_t)((size + 3) & ~3) * (key_bytes + 4);  // keys and, for tiles with a NaN, positions
  CINN_RT_CHECK(per_col <= (size_t)kLdsLimit, "argsort: %d elements along the sorted axis exceed the %zu that one block's LDS holds", size,
                (size_t)kLdsLimit / (key_bytes + 4));
  // neighbouring columns per tile: whole 64-byte pieces of a row when there are that many, bounded by LDS and by the
  // work one block should carry
  int ti = inner < 16 ? inner : 16;
  while (ti > 1 && (per_col * ti > (size_t)kLdsLimit / 2 || (int64_t)size * ti > 8192)) ti /= 2;
  p.ti              = ti;
  p.tiles_per_outer = (inner + ti - 1) / ti;
  const int64_t blocks = (int64_t)outer * p.tiles_per_outer;
  CINN_RT_CHECK(blocks < INT_MAX, "argsort: too many tiles");
  const size_t lds_bytes = per_col * ti;
  auto s = static_cast<hipStream_t>(stream);
  switch (elem) {
    case Elem::kF32: Launch<float>(p, (int)blocks, lds_bytes, s); break;
    case Elem::kF64: Launch<double>(p, (int)blocks, lds_bytes, s); break;
    case Elem::kF16: Launch<_Float16>(p, (int)blocks, lds_bytes, s); break;
    case Elem::kBF16: Launch<__bf16>(p, (int)blocks, lds_bytes, s); break;
    case Elem::kI32: Launch<int32_t>(p, (int)blocks, lds_bytes, s); break;
    case Elem::kI64: Launch<int64_t>(p, (int)blocks, lds_bytes, s); break;
    default: break;
  }
  CINN_HIP_CALL(hipGetLastError());
}
