/*
 * CPU restatement of the reference's compute definitions for the GPU-backend hot path.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker the HIP path is compared against (tests/,
 * __graft_entry__.smoke()) and the timed CPU baseline of bench.py.  Nothing in the product may call it.
 *
 * Every function follows one reference definition (paths relative to the CINN tree) and keeps its
 * operation order: sums run over ascending indices in the storage type unless stated otherwise, no
 * fused multiply-add is used (compile with -ffp-contract=off), matching LLVM's x86 code generation of
 * the host path without fast-math.  OpenMP only splits the outermost independent dimension, so results
 * do not depend on the thread count.
 *
 * 16-bit floats: the reference's host structs round every operation to the 16-bit type.  Functions
 * with the suffix _f16 / _bf16 take and return raw bit patterns; where the reference accumulates in
 * the 16-bit type there are two variants: *_native (every partial sum rounded, the literal host
 * semantics) and the default one that accumulates in fp32 and rounds once (what an fp32-accumulating
 * GPU kernel computes; the parity bar of 1e-2 is checked against this one and the distance of the
 * literal variant is reported by the tests).
 *
 * Pinning (what fixes each function independently of this file): see the table in oracle/README.md.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------------------------------------
 * 16-bit float conversions.
 * float -> half: round to nearest even, as _cvtss_sh(val, 0) and the device __float2half do
 * (cinn/common/float16.h:95-121).  float -> bfloat16: the device path rounds to nearest even
 * (__float2bfloat16), the host struct TRUNCATES (memcpy of the high half, cinn/common/bfloat16.h:68-80);
 * both are provided.
 * ---------------------------------------------------------------------------------------------- */
static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

uint16_t oracle_float_to_half(float f) {
  uint32_t x    = f32_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t abs  = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) { /* inf / nan */
    if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((abs >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (abs >= 0x477ff000u) { /* rounds to or beyond 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (abs < 0x38800000u) { /* subnormal half or zero: value * 2^24 rounded to nearest even integer */
    if (abs < 0x33000000u) return (uint16_t)sign; /* below half of the smallest subnormal (2^-25) -> 0 */
    int exp       = (int)(abs >> 23);              /* biased exponent, 102..112 */
    uint32_t mant = (abs & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift     = 126 - exp;                     /* 14..24 bits to drop */
    uint32_t q    = mant >> shift;
    uint32_t rem  = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  {
    uint32_t mant = abs & 0x7fffffu;
    uint32_t exp  = (abs >> 23) - 112u; /* rebias 127 -> 15 */
    uint32_t q    = (exp << 10) | (mant >> 13);
    uint32_t rem  = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* a carry into the exponent is correct */
    return (uint16_t)(sign | q);
  }
}

/* float -> half rounding TOWARD ZERO.  This is what the reference's host struct does when it is built
 * with the reference's own flags (-mavx -mfma, no -mf16c): the portable branch of
 * cinn/common/float16.h:102-118 drops the low significand bits.  Kept to measure how far the literal host
 * arithmetic is from the round-to-nearest device arithmetic; parity is NOT checked against it. */
uint16_t oracle_float_to_half_trunc(float f) {
  uint32_t x    = f32_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t abs  = x & 0x7fffffffu;
  if (abs >= 0x7f800000u) {
    if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((abs >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (abs > 0x477fe000u) return (uint16_t)(sign | 0x7c00u); /* anything above 65504 becomes inf there */
  if (abs < 0x38800000u) {
    if (abs < 0x33800000u) return (uint16_t)sign; /* below the smallest subnormal 2^-24 */
    int exp       = (int)(abs >> 23);
    uint32_t mant = (abs & 0x7fffffu) | 0x800000u;
    return (uint16_t)(sign | (mant >> (126 - exp)));
  }
  return (uint16_t)(sign | ((((abs >> 23) - 112u) << 10) | ((abs & 0x7fffffu) >> 13)));
}

float oracle_half_to_float(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp  = (h >> 10) & 0x1fu;
  uint32_t mant = h & 0x3ffu;
  if (exp == 0x1fu) return bits_f32(sign | 0x7f800000u | (mant << 13));
  if (exp == 0) {
    if (mant == 0) return bits_f32(sign);
    float v = (float)mant * 5.9604644775390625e-08f; /* 2^-24 */
    return sign ? -v : v;
  }
  return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

uint16_t oracle_float_to_bf16_rne(float f) {
  uint32_t x = f32_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}
uint16_t oracle_float_to_bf16_trunc(float f) { return (uint16_t)(f32_bits(f) >> 16); }
float oracle_bf16_to_float(uint16_t b) { return bits_f32((uint32_t)b << 16); }

void oracle_float_to_half_array(const float* in, uint16_t* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = oracle_float_to_half(in[i]);
}
void oracle_float_to_half_trunc_array(const float* in, uint16_t* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = oracle_float_to_half_trunc(in[i]);
}
void oracle_half_to_float_array(const uint16_t* in, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = oracle_half_to_float(in[i]);
}
void oracle_float_to_bf16_array(const float* in, uint16_t* out, long n, int truncate) {
  for (long i = 0; i < n; ++i) out[i] = truncate ? oracle_float_to_bf16_trunc(in[i]) : oracle_float_to_bf16_rne(in[i]);
}
void oracle_bf16_to_float_array(const uint16_t* in, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = oracle_bf16_to_float(in[i]);
}

/* fp16 helpers: one operation in fp32 followed by one rounding equals the correctly rounded half
 * operation for + - * / and sqrt (fp32 carries more than 2*11+2 significand bits). */
static inline float hround(float v) { return oracle_half_to_float(oracle_float_to_half(v)); }

/* ------------------------------------------------------------------------------------------------
 * Config 1: y = relu(a + b).  pe::Add (cinn/hlir/pe/broadcast.cc:247) then pe::Relu = max(x, 0)
 * (cinn/hlir/pe/nn.cc:61-64).  max follows the C ternary (x > 0 ? x : 0), so relu(NaN) = 0 and
 * relu(-0) = 0.
 * ---------------------------------------------------------------------------------------------- */
void oracle_add_relu_f32(const float* a, const float* b, float* y, long n) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; ++i) {
    float s = a[i] + b[i];
    y[i]    = s > 0.0f ? s : 0.0f;
  }
}

/* ------------------------------------------------------------------------------------------------
 * Softmax over the last axis of [rows, cols].
 * mode 0 ("fast", the default of NetBuilder::Softmax, cinn/frontend/net_builder.h:782-785; also
 * pe::Softmax, cinn/hlir/pe/nn.cc:755-796): exp(x) / sum(exp(x)), no max shift.
 * mode 1 (any other mode of the decomposer, cinn/frontend/decomposer/activation.cc:70-118):
 * exp(x - max) / sum(exp(x - max)).
 * ---------------------------------------------------------------------------------------------- */
void oracle_softmax_f32(const float* x, float* y, long rows, long cols, int mode) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float* yr       = y + r * cols;
    float shift     = 0.0f;
    if (mode != 0) {
      float m = -3.40282e+38f;
      for (long c = 0; c < cols; ++c) m = xr[c] > m ? xr[c] : m;
      shift = m;
    }
    float sum = 0.0f;
    for (long c = 0; c < cols; ++c) sum += expf(mode != 0 ? xr[c] - shift : xr[c]);
    for (long c = 0; c < cols; ++c) yr[c] = expf(mode != 0 ? xr[c] - shift : xr[c]) / sum;
  }
}

/* fp16 softmax.  Every element-wise result is a half (exp and the quotient are rounded to half).
 * native_accumulate != 0: the row sum is accumulated in half, one rounding per addition, ascending
 * index (the literal semantics of cinn_sum_fp16, cinn_cuda_runtime_source.cuh:435, applied serially as
 * on the host); otherwise the halves are summed in fp32 and the sum rounded once. */
void oracle_softmax_f16(const uint16_t* x, uint16_t* y, long rows, long cols, int mode, int native_accumulate) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    const uint16_t* xr = x + r * cols;
    uint16_t* yr       = y + r * cols;
    float shift        = 0.0f;
    if (mode != 0) {
      float m = oracle_half_to_float(0xfbff);
      for (long c = 0; c < cols; ++c) {
        float v = oracle_half_to_float(xr[c]);
        m       = v > m ? v : m;
      }
      shift = m;
    }
    float sum = 0.0f;
    for (long c = 0; c < cols; ++c) {
      float v = oracle_half_to_float(xr[c]);
      if (mode != 0) v = hround(v - shift);
      float e = hround(expf(v));
      sum     = native_accumulate ? hround(sum + e) : sum + e;
    }
    sum = hround(sum);
    for (long c = 0; c < cols; ++c) {
      float v = oracle_half_to_float(xr[c]);
      if (mode != 0) v = hround(v - shift);
      float e = hround(expf(v));
      yr[c]   = oracle_float_to_half(e / sum);
    }
  }
}

/* ------------------------------------------------------------------------------------------------
 * layer_norm over the trailing `cols` elements, the composition of the Paddle op mapper
 * (cinn/frontend/op_mappers/paddle/layer_norm.cc:83-140), all in fp32:
 *   mean = sum(x) / n ; var = max(sum(x*x) / n - mean*mean, 0) ;
 *   y = (x - mean) / sqrt(var + eps) * gamma + beta
 * gamma / beta may be NULL.  mean / var outputs may be NULL.
 * ---------------------------------------------------------------------------------------------- */
static void layer_norm_row(const float* xr, const float* gamma, const float* beta, float* yr, float* mean_out,
                           float* var_out, long cols, float eps) {
  float n  = (float)cols;
  float s1 = 0.0f, s2 = 0.0f;
  for (long c = 0; c < cols; ++c) s1 += xr[c];
  for (long c = 0; c < cols; ++c) s2 += xr[c] * xr[c];
  float mean = s1 / n;
  float var  = s2 / n - mean * mean;
  var        = var > 0.0f ? var : 0.0f;
  float sd   = sqrtf(var + eps);
  for (long c = 0; c < cols; ++c) {
    float v = (xr[c] - mean) / sd;
    if (gamma) v = v * gamma[c];
    if (beta) v = v + beta[c];
    yr[c] = v;
  }
  if (mean_out) *mean_out = mean;
  if (var_out) *var_out = var;
}

void oracle_layer_norm_f32(const float* x, const float* gamma, const float* beta, float* y, float* mean, float* var,
                           long rows, long cols, float eps) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r)
    layer_norm_row(x + r * cols, gamma, beta, y + r * cols, mean ? mean + r : 0, var ? var + r : 0, cols, eps);
}

/* fp16 input: cast to fp32, compute as above, cast the result back (layer_norm.cc:90-93, 126-130);
 * gamma / beta / mean / var stay fp32. */
void oracle_layer_norm_f16(const uint16_t* x, const float* gamma, const float* beta, uint16_t* y, float* mean,
                           float* var, long rows, long cols, float eps) {
#pragma omp parallel
  {
    float* xf = (float*)malloc(sizeof(float) * (size_t)cols);
    float* yf = (float*)malloc(sizeof(float) * (size_t)cols);
#pragma omp for schedule(static)
    for (long r = 0; r < rows; ++r) {
      for (long c = 0; c < cols; ++c) xf[c] = oracle_half_to_float(x[r * cols + c]);
      layer_norm_row(xf, gamma, beta, yf, mean ? mean + r : 0, var ? var + r : 0, cols, eps);
      for (long c = 0; c < cols; ++c) y[r * cols + c] = oracle_float_to_half(yf[c]);
    }
    free(xf);
    free(yf);
  }
}

/* ------------------------------------------------------------------------------------------------
 * int32 reductions over the last axis of [rows, cols].
 * reduce_sum: pe::ReduceSum (cinn/hlir/pe/reduction.cc:205-207), wrap-around int32 arithmetic.
 * argmax: index of the FIRST maximum, int32 (cinn/hlir/op/contrib/argmax.cc:48-93).
 * ---------------------------------------------------------------------------------------------- */
void oracle_reduce_sum_i32(const int32_t* x, int32_t* y, long rows, long cols) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    uint32_t s = 0; /* unsigned: wrap-around without undefined behaviour */
    for (long c = 0; c < cols; ++c) s += (uint32_t)x[r * cols + c];
    y[r] = (int32_t)s;
  }
}
void oracle_argmax_i32(const int32_t* x, int32_t* y, long rows, long cols) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    long best = 0;
    for (long c = 1; c < cols; ++c)
      if (x[r * cols + c] > x[r * cols + best]) best = c;
    y[r] = (int32_t)best;
  }
}
void oracle_argmax_f32(const float* x, int32_t* y, long rows, long cols) {
#pragma omp parallel for schedule(static)
  for (long r = 0; r < rows; ++r) {
    long best = 0;
    for (long c = 1; c < cols; ++c)
      if (x[r * cols + c] > x[r * cols + best]) best = c;
    y[r] = (int32_t)best;
  }
}

/* The literal algorithm of the reference for one row of `size` elements at stride `stride`: argsort in
 * descending order through the rank count cinn_host_gt_num and the destructive scan
 * cinn_host_next_smallest_int32 (cinn/hlir/op/contrib/sort.cc:50-118 with
 * cinn/runtime/cpu/host_intrinsics.cc:67-79, 99-106), then element 0 of the sorted indices
 * (argmax.cc:80-91).  O(size^2); for small inputs, to pin oracle_argmax_* on ties. */
int32_t oracle_argmax_by_argsort_i32(const int32_t* x, long size, long stride) {
  int32_t* rank = (int32_t*)malloc(sizeof(int32_t) * (size_t)size);
  for (long i = 0; i < size; ++i) { /* number of elements greater than x[i] */
    int32_t out = 0;
    for (long j = (size - 1) * stride; j >= 0; j -= stride)
      if (x[j] > x[i * stride]) out++;
    rank[i] = out;
  }
  /* position 0 of the sorted index list = first call of next_smallest over the ranks: the smallest rank,
   * the first one on ties (strict <) */
  long id = -1;
  for (long i = 0; i < size; ++i)
    if (id == -1 || rank[i] < rank[id]) id = i;
  free(rank);
  return (int32_t)id;
}

/* argsort / sort along one axis of [outer][size][inner], the literal three loop nests of the reference
 * (cinn/hlir/op/contrib/sort.cc:50-139; the generated host code is spelled out in sort_test.cc:96-124):
 *   positions[k] = cinn_host_lt_num(x, size, x[k], offset, stride)   (gt_num when descending: the count of larger
 *                  elements; host_intrinsics.cc:99-118 scan from the last element down, which changes nothing)
 *   index[j]     = cinn_host_next_smallest_int32(positions, size, j, offset, stride) for j = 0 .. size - 1 in order:
 *                  the first entry with the smallest value, which the call then overwrites with INT32_MAX
 *                  (host_intrinsics.cc:67-79)
 *   sorted[j]    = x[index[j]]
 * `positions_out` receives the positions as computed by the first nest (the second nest consumes a copy).  Doubles
 * carry fp32 / fp64 / 16-bit values exactly; int64 values beyond 2^53 are not meant for this helper. */
#define ORACLE_ARGSORT(NAME, T)                                                                                         \
  void NAME(const T* x, int32_t* index, int32_t* positions_out, T* sorted, long outer, long size, long inner,           \
            int is_ascend) {                                                                                            \
    int32_t* work = (int32_t*)malloc(sizeof(int32_t) * (size_t)(size > 0 ? size : 1));                                  \
    for (long o = 0; o < outer; ++o)                                                                                    \
      for (long i = 0; i < inner; ++i) {                                                                                \
        const long offset = o * size * inner + i, stride = inner;                                                       \
        for (long k = 0; k < size; ++k) {                                                                               \
          const T num = x[offset + k * stride];                                                                         \
          int32_t out = 0;                                                                                              \
          for (long j = (size - 1) * stride + offset; j >= offset; j -= stride)                                         \
            if (is_ascend ? x[j] < num : x[j] > num) out++;                                                             \
          work[k] = out;                                                                                                \
          if (positions_out) positions_out[offset + k * stride] = out;                                                  \
        }                                                                                                               \
        for (long slot = 0; slot < size; ++slot) {                                                                      \
          long id = -1;                                                                                                 \
          for (long k = 0; k < size; ++k)                                                                               \
            if (id == -1 || work[k] < work[id]) id = k;                                                                 \
          work[id] = 2147483647;                                                                                        \
          if (index) index[offset + slot * stride] = (int32_t)id;                                                       \
          if (sorted) sorted[offset + slot * stride] = x[offset + id * stride];                                         \
        }                                                                                                               \
      }                                                                                                                 \
    free(work);                                                                                                         \
  }
ORACLE_ARGSORT(oracle_argsort_f64, double)
ORACLE_ARGSORT(oracle_argsort_i64, int64_t)
#undef ORACLE_ARGSORT

/* ------------------------------------------------------------------------------------------------
 * Matmul, row-major: C[M,N] = alpha * op(A) * op(B) (+ beta * C), op = optional transpose.
 * pe::Matmul (cinn/hlir/pe/transform.cc:252-310): sum over ascending k, then multiplied by alpha when
 * alpha != 1.  A is [M,K] (or [K,M] when trans_a), B is [K,N] (or [N,K] when trans_b).
 * ---------------------------------------------------------------------------------------------- */
void oracle_matmul_f32(const float* a, const float* b, float* c, long m, long n, long k, int trans_a, int trans_b,
                       float alpha, float beta) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < m; ++i) {
    for (long j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (long p = 0; p < k; ++p) {
        float av = trans_a ? a[p * m + i] : a[i * k + p];
        float bv = trans_b ? b[j * k + p] : b[p * n + j];
        acc += av * bv;
      }
      float v = alpha != 1.0f ? acc * alpha : acc;
      if (beta != 0.0f) v = v + beta * c[i * n + j];
      c[i * n + j] = v;
    }
  }
}

/* Same with float64 accumulation: the mathematically exact side for tolerance checks of large K. */
void oracle_matmul_f32_acc64(const float* a, const float* b, float* c, long m, long n, long k, int trans_a,
                             int trans_b, float alpha) {
#pragma omp parallel for schedule(static)
  for (long i = 0; i < m; ++i) {
    for (long j = 0; j < n; ++j) {
      double acc = 0.0;
      for (long p = 0; p < k; ++p) {
        double av = trans_a ? a[p * m + i] : a[i * k + p];
        double bv = trans_b ? b[j * k + p] : b[p * n + j];
        acc += av * bv;
      }
      c[i * n + j] = (float)(acc * alpha);
    }
  }
}

/* 16-bit inputs (kind 0 = fp16, 1 = bf16), products and sum in fp32 ascending k, one rounding of the
 * result (bf16: round to nearest even).  This is the "fp32 accumulate" contract of the GEMM config;
 * cublasGemmEx(CUDA_R_16BF, COMPUTE_32F) in cinn/runtime/cuda/cublas_util.h:25-115 has the same one. */
void oracle_matmul_16(const uint16_t* a, const uint16_t* b, uint16_t* c, long m, long n, long k, int trans_a,
                      int trans_b, float alpha, int kind) {
#pragma omp parallel
  {
    float* bcol = (float*)malloc(sizeof(float) * (size_t)k);
#pragma omp for schedule(static)
    for (long j = 0; j < n; ++j) {
      for (long p = 0; p < k; ++p) {
        uint16_t raw = trans_b ? b[j * k + p] : b[p * n + j];
        bcol[p]      = kind == 0 ? oracle_half_to_float(raw) : oracle_bf16_to_float(raw);
      }
      for (long i = 0; i < m; ++i) {
        float acc = 0.0f;
        for (long p = 0; p < k; ++p) {
          uint16_t raw = trans_a ? a[p * m + i] : a[i * k + p];
          float av     = kind == 0 ? oracle_half_to_float(raw) : oracle_bf16_to_float(raw);
          acc += av * bcol[p];
        }
        float v      = alpha != 1.0f ? acc * alpha : acc;
        c[i * n + j] = kind == 0 ? oracle_float_to_half(v) : oracle_float_to_bf16_rne(v);
      }
    }
    free(bcol);
  }
}

/* ------------------------------------------------------------------------------------------------
 * conv2d NCHW, cross-correlation with zero padding: pe::Conv2d_NCHW (cinn/hlir/pe/nn.cc:220-313),
 *   out[n,f,y,x] = sum_{rc,ry,rx} pad(in)[n, rc, y*s + ry*d, x*s + rx*d] * w[f, rc, ry, rx]
 * reduce order rc -> ry -> rx, output size (in - ((k-1)*d + 1) + 2*p) / s + 1 (nn.cc:235-241).
 * groups: input channels of group g are [g*ic/groups, (g+1)*ic/groups).
 * ---------------------------------------------------------------------------------------------- */
void oracle_conv2d_nchw_f32(const float* in, const float* w, float* out, long n, long ic, long ih, long iw, long oc,
                            long kh, long kw, long ph, long pw, long sh, long sw, long dh, long dw, long groups) {
  long oh  = (ih - ((kh - 1) * dh + 1) + 2 * ph) / sh + 1;
  long ow  = (iw - ((kw - 1) * dw + 1) + 2 * pw) / sw + 1;
  long icg = ic / groups, ocg = oc / groups;
#pragma omp parallel for collapse(2) schedule(static)
  for (long b = 0; b < n; ++b) {
    for (long f = 0; f < oc; ++f) {
      long g = f / ocg;
      for (long y = 0; y < oh; ++y) {
        for (long x = 0; x < ow; ++x) {
          float acc = 0.0f;
          for (long rc = 0; rc < icg; ++rc) {
            for (long ry = 0; ry < kh; ++ry) {
              long yy = y * sh + ry * dh - ph;
              for (long rx = 0; rx < kw; ++rx) {
                long xx = x * sw + rx * dw - pw;
                float v = 0.0f;
                if (yy >= 0 && yy < ih && xx >= 0 && xx < iw) v = in[((b * ic + g * icg + rc) * ih + yy) * iw + xx];
                acc += v * w[((f * icg + rc) * kh + ry) * kw + rx];
              }
            }
          }
          out[((b * oc + f) * oh + y) * ow + x] = acc;
        }
      }
    }
  }
}

/* fp16 tensors, fp32 accumulation, one rounding of the result (cuDNN's contract for half tensors:
 * compute type fp32, cinn/runtime/cuda/cuda_util.cc get_cudnn_compute_dtype). */
void oracle_conv2d_nchw_f16(const uint16_t* in, const uint16_t* w, uint16_t* out, long n, long ic, long ih, long iw,
                            long oc, long kh, long kw, long ph, long pw, long sh, long sw, long dh, long dw,
                            long groups) {
  long oh  = (ih - ((kh - 1) * dh + 1) + 2 * ph) / sh + 1;
  long ow  = (iw - ((kw - 1) * dw + 1) + 2 * pw) / sw + 1;
  long icg = ic / groups, ocg = oc / groups;
#pragma omp parallel for collapse(2) schedule(static)
  for (long b = 0; b < n; ++b) {
    for (long f = 0; f < oc; ++f) {
      long g = f / ocg;
      for (long y = 0; y < oh; ++y) {
        for (long x = 0; x < ow; ++x) {
          float acc = 0.0f;
          for (long rc = 0; rc < icg; ++rc) {
            for (long ry = 0; ry < kh; ++ry) {
              long yy = y * sh + ry * dh - ph;
              for (long rx = 0; rx < kw; ++rx) {
                long xx = x * sw + rx * dw - pw;
                float v = 0.0f;
                if (yy >= 0 && yy < ih && xx >= 0 && xx < iw)
                  v = oracle_half_to_float(in[((b * ic + g * icg + rc) * ih + yy) * iw + xx]);
                acc += v * oracle_half_to_float(w[((f * icg + rc) * kh + ry) * kw + rx]);
              }
            }
          }
          out[((b * oc + f) * oh + y) * ow + x] = oracle_float_to_half(acc);
        }
      }
    }
  }
}

/* ------------------------------------------------------------------------------------------------
 * Inference batch_norm NCHW + optional relu: pe::BatchNorm_NCHW (cinn/hlir/pe/nn.cc:700-721),
 *   y = (x - mean[c]) * scale[c] / sqrt(var[c] + eps) + bias[c]     evaluated left to right.
 * ---------------------------------------------------------------------------------------------- */
void oracle_batch_norm_relu_nchw_f32(const float* x, const float* scale, const float* bias, const float* mean,
                                     const float* var, float* y, long n, long c, long hw, float eps, int relu) {
#pragma omp parallel for collapse(2) schedule(static)
  for (long b = 0; b < n; ++b) {
    for (long ch = 0; ch < c; ++ch) {
      float sd = sqrtf(var[ch] + eps);
      for (long i = 0; i < hw; ++i) {
        long idx = (b * c + ch) * hw + i;
        float v  = (x[idx] - mean[ch]) * scale[ch] / sd + bias[ch];
        if (relu) v = v > 0.0f ? v : 0.0f;
        y[idx] = v;
      }
    }
  }
}
/* fp16: every operation rounds to half (the tensor dtype of the whole chain is half). */
void oracle_batch_norm_relu_nchw_f16(const uint16_t* x, const uint16_t* scale, const uint16_t* bias,
                                     const uint16_t* mean, const uint16_t* var, uint16_t* y, long n, long c, long hw,
                                     float eps, int relu) {
#pragma omp parallel for collapse(2) schedule(static)
  for (long b = 0; b < n; ++b) {
    for (long ch = 0; ch < c; ++ch) {
      float epsh = hround(eps);
      float sd   = hround(sqrtf(hround(oracle_half_to_float(var[ch]) + epsh)));
      float m = oracle_half_to_float(mean[ch]), s = oracle_half_to_float(scale[ch]), bi = oracle_half_to_float(bias[ch]);
      for (long i = 0; i < hw; ++i) {
        long idx = (b * c + ch) * hw + i;
        float v  = hround(oracle_half_to_float(x[idx]) - m);
        v        = hround(v * s);
        v        = hround(v / sd);
        v        = hround(v + bi);
        if (relu) v = v > 0.0f ? v : 0.0f;
        y[idx] = oracle_float_to_half(v);
      }
    }
  }
}

/* ------------------------------------------------------------------------------------------------
 * pool2d NCHW: pe::PoolImpl (cinn/hlir/pe/nn.cc:956-1109).
 * max: padding takes the lowest value of the type, result = max over the window.
 * avg: zero padding, every element is DIVIDED first and then summed (ry -> rx order);
 *      exclusive: divisor = number of window positions inside the un-padded input (at least 1),
 *      otherwise kh*kw.  Output size (in - k + p_head + p_tail) / s + 1, ceil_mode adds s-1 to p_tail.
 * pad = {top, left, bottom, right}.
 * ---------------------------------------------------------------------------------------------- */
void oracle_pool2d_nchw_f32(const float* in, float* out, long n, long c, long ih, long iw, long kh, long kw, long pt,
                            long pl, long pb, long pr, long sh, long sw, int is_max, int exclusive, int ceil_mode) {
  if (ceil_mode) {
    pb += sh - 1;
    pr += sw - 1;
  }
  long oh = (ih - kh + pt + pb) / sh + 1;
  long ow = (iw - kw + pl + pr) / sw + 1;
#pragma omp parallel for schedule(static)
  for (long bc = 0; bc < n * c; ++bc) {
    const float* src = in + bc * ih * iw;
    float* dst       = out + bc * oh * ow;
    for (long y = 0; y < oh; ++y) {
      for (long x = 0; x < ow; ++x) {
        if (is_max) {
          float m = -3.402823466e+38f; /* lang::min_value(Float(32)) */
          for (long ry = 0; ry < kh; ++ry) {
            for (long rx = 0; rx < kw; ++rx) {
              long yy = y * sh + ry - pt, xx = x * sw + rx - pl;
              float v = (yy >= 0 && yy < ih && xx >= 0 && xx < iw) ? src[yy * iw + xx] : -3.402823466e+38f;
              m       = v > m ? v : m;
            }
          }
          dst[y * ow + x] = m;
        } else {
          float factor = (float)(kh * kw);
          if (exclusive) {
            long ys = y * sh - pt, xs = x * sw - pl;
            long ye = ys + kh < ih ? ys + kh : ih, xe = xs + kw < iw ? xs + kw : iw;
            ys      = ys > 0 ? ys : 0;
            xs      = xs > 0 ? xs : 0;
            long f  = (ye - ys) * (xe - xs);
            factor  = (float)(f > 1 ? f : 1);
          }
          float acc = 0.0f;
          for (long ry = 0; ry < kh; ++ry) {
            for (long rx = 0; rx < kw; ++rx) {
              long yy = y * sh + ry - pt, xx = x * sw + rx - pl;
              float v = (yy >= 0 && yy < ih && xx >= 0 && xx < iw) ? src[yy * iw + xx] : 0.0f;
              acc += v / factor;
            }
          }
          dst[y * ow + x] = acc;
        }
      }
    }
  }
}
