/*
 * zmi_oracle.c -- CPU restatement of the reference's LowOHA int8 matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the zendnn_amd package,
 * libzmi_lowoha.so, the C++ adapter) may link, load or call this file; it is
 * used by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline
 * leg, always as the checker or the timed CPU baseline.
 *
 * It takes the same flat structs as the C ABI (include/zmi_lowoha.h) but with
 * HOST pointers, so one ctypes description drives both sides of a parity test.
 *
 * Each function cites the reference file:line whose arithmetic it follows
 * (paths relative to zendnnl/src/ of the reference tree).  The reference's
 * default backend for this path is AOCL-DLP (github.com/amd/aocl-dlp, pinned
 * at b3db7f5800aca3ba3ce5bdfab10f557c5b896e5a), which is not vendored; its
 * semantics are the ones the reference's own scalar kernel states
 * (operators/matmul/matmul_ref_kernel.cpp), and that is what is restated.
 *
 * Parity status of each function (what pins it, see tests/test_oracle_*.py):
 *   zo_f32_to_bf16_ctor / _rne   exhaustive hi-half table + torch bfloat16
 *   zo_quant_per_token           closed forms (constant row, zero row, NaN/Inf,
 *                                ties-to-even), |q|<=127, max|q|==127
 *   zo_gemm_s32                  int64 brute force, all-ones closed form, the
 *                                reference example's deterministic recipe
 *   zp compensation              integer identity sum((a-zp)w) == sum(aw)-zp*sum(w); with a weight zero-point the
 *                                product of the shifted operands in Python integers (u8 / s8, transposed A)
 *   dequant chain / bias         special cases (unit scales, equal per-channel
 *                                scales == per-tensor), op order from source
 *   post-ops                     libm double evaluation within 2 f32 ulp (mish = x * tanh(softplus(x)) included: double
 *                                evaluation, the limits for large |x|, mish(0) = 0)
 *   per-group scales             closed form (all-ones operands, power-of-two scales: every step exact),
 *                                equal power-of-two group scales == per-token chain bit for bit,
 *                                numpy float32 brute force on small random cases
 *   zo_f32_to_f16                round trip of all 65536 half values, numpy float16 on 4 million random bit patterns and
 *                                on every tie / boundary case (except the documented carry case, which has known answers)
 *   zo_fp16_to_f32, Q8_0 unpack  all 65536 half values against numpy float16; block layout by construction
 *                                of the packed buffer from known rows and scales (numpy), bf16 via torch
 *   zo_s4_to_s8 (W4A8 widening)  every nibble value in both positions (known answers), numpy shift/mask
 *                                restatement on random buffers, both orientations with padded ldb
 *   zo_quant_per_group           per-group constants (closed form), == zo_quant_per_token on the
 *                                [M*G, K/G] view
 *   zo_quant_asym                closed forms (rows k * 2^-e: scale, zero-point and every code known exactly;
 *                                constant and non-finite rows), dequantization within half a step, codes of
 *                                the row minimum / maximum, zero-point against Python fractions
 *   zo_woq_dequant, zo_matmul_woq  nibble order, sign extension, orientation and leading dimension on hand-built bytes;
 *                                both dequantization formulas on operands that keep every step exact (known answers
 *                                that tell the formulas apart); bf16-valued scales (exact f32 product) against torch's
 *                                rounding of the exact double product, per tensor / channel / group; the product
 *                                against numpy float64 (to 2e-6 of the magnitude sum) and exactly on integer operands.
 *                                The reference's own GEMM on the dequantized matrix is AOCL's: its summation order is
 *                                parity unpinned, the comparison of products is to a tolerance.
 *   dynamic u8 (per tensor)      closed forms (values k / 4: scale 0.25, zero-point 100, codes and product known exactly;
 *                                constant and non-finite tensors; the 2.5 * 255 tie), identity weights dequantize to the
 *                                source within half a step; with a bf16 scale buffer the codes are made with the narrowed
 *                                scale and the zero-point with the un-narrowed one (closed form: scale 0.3 -> 0.30078125,
 *                                codes known exactly); the AVX-512 kernels' reciprocal form: parity unpinned on ties
 *   zo_gated_act, zo_moe_reduce  brute force + the reference example's closed form
 *   prepack layout, weight_prepack_size values: parity unpinned (opaque by the
 *     reference's contract; only the round trip matmul(prepack(B)) == matmul(B)
 *     is checkable) -- the oracle has no function for them.
 *   AOCL-DLP's vectorised SWISH / GELU_TANH last-ulp behaviour: parity unpinned
 *     (only a run of AOCL-DLP could pin it; the scalar reference defines the target).
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/build.py).
 * -ffp-contract=off matters: the reference chain is a sequence of separately
 * rounded f32 operations.
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/zmi_lowoha.h"

#define ZO_EXPORT __attribute__((visibility("default")))

/* ---- bf16 ------------------------------------------------------------- */

/* bfloat16_t::bfloat16_t(float), common/bfloat16.cpp:27-51: zero and subnormal
 * inputs give a signed zero, NaN keeps the high half with the quiet bit set,
 * normals round to nearest even.  Used by the matmul store
 * (operators/matmul/matmul_ref_kernel.cpp:207-218) and the gated activation
 * (lowoha_operators/matmul/group_matmul/group_matmul_moe_act.cpp:110-117). */
ZO_EXPORT uint16_t zo_f32_to_bf16_ctor(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t exp = u & 0x7f800000u, man = u & 0x007fffffu;
  if (exp == 0) return (uint16_t)((u >> 16) & 0x8000u);
  if (exp == 0x7f800000u) {
    if (man == 0) return (uint16_t)(u >> 16);
    return (uint16_t)((u >> 16) | 0x40u);
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* bfloat16_t::f32_to_bf16_val, common/bfloat16.cpp:69-79: the plain bit trick,
 * no special cases.  Used by the MoE weighted reduce
 * (group_matmul/group_matmul_moe_postop.cpp:85-88, 262-283). */
ZO_EXPORT uint16_t zo_f32_to_bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* bfloat16_t::bf16_to_f32_val, common/bfloat16.cpp:60-66. */
ZO_EXPORT float zo_bf16_to_f32(uint16_t h) {
  uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

ZO_EXPORT void zo_f32_to_bf16_buf(const float *src, uint16_t *dst, int64_t n, int ctor) {
  for (int64_t i = 0; i < n; ++i)
    dst[i] = ctor ? zo_f32_to_bf16_ctor(src[i]) : zo_f32_to_bf16_rne(src[i]);
}

/* ---- helpers ---------------------------------------------------------- */

static int64_t zo_nelems(const zmi_quant_t *q) {
  int64_t n = 1;
  for (int i = 0; i < q->ndims; ++i) n *= q->dims[i];
  return n;
}

/* read_and_cast<float> of the reference for the dtypes this path uses. */
ZO_EXPORT float zo_fp16_to_f32(uint16_t h);
ZO_EXPORT uint16_t zo_f32_to_f16(float f);

static float zo_read_f32(const void *p, int32_t dt, int64_t i) {
  switch (dt) {
  case ZMI_DT_F32: return ((const float *)p)[i];
  case ZMI_DT_F16: return zo_fp16_to_f32(((const uint16_t *)p)[i]);
  case ZMI_DT_BF16: return zo_bf16_to_f32(((const uint16_t *)p)[i]);
  case ZMI_DT_S32: return (float)((const int32_t *)p)[i];
  case ZMI_DT_S8: return (float)((const int8_t *)p)[i];
  case ZMI_DT_U8: return (float)((const uint8_t *)p)[i];
  default: return 0.0f;
  }
}

static int32_t zo_read_s32(const void *p, int32_t dt, int64_t i) {
  switch (dt) {
  case ZMI_DT_S32: return ((const int32_t *)p)[i];
  case ZMI_DT_S8: return ((const int8_t *)p)[i];
  case ZMI_DT_U8: return ((const uint8_t *)p)[i];
  case ZMI_DT_F32: return (int32_t)((const float *)p)[i];
  default: return 0;
  }
}

/* ---- per-token dynamic quantization ------------------------------------ */

/* dynamic_per_token_quant_{bf16,f32}_s8_ref,
 * lowoha_operators/reorder/reorder_data_type/scalar_impl/dynamic_per_token_ref_kernel.cpp:31-36,70-96:
 * absmax over finite values; scale = max(absmax,1e-10)/127 clamped to >= 1e-10;
 * q = (int8) nearbyint(v / scale) (true division, ties to even, truncating
 * narrow); non-finite -> 0. */
ZO_EXPORT void zo_quant_per_token(const void *src, int32_t src_dt, int64_t M, int64_t K,
                                  int64_t ld_src, int8_t *dst, int64_t ld_dst, float *scales) {
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float absmax = 0.0f;
    for (int64_t j = 0; j < K; ++j) {
      float v = zo_read_f32(src, src_dt, m * ld_src + j);
      if (isfinite(v)) {
        float a = fabsf(v);
        if (a > absmax) absmax = a;
      }
    }
    if (absmax < 1e-10f) absmax = 1e-10f;
    float scale = absmax / 127.0f;
    if (scale < 1e-10f) scale = 1e-10f;
    scales[m] = scale;
    if (!dst) continue;
    for (int64_t j = 0; j < K; ++j) {
      float v = zo_read_f32(src, src_dt, m * ld_src + j);
      if (!isfinite(v)) { dst[m * ld_dst + j] = 0; continue; }
      int32_t q = (int32_t)nearbyintf(v / scale);
      dst[m * ld_dst + j] = (int8_t)q;
    }
  }
}

/* Per-group dynamic quantization, symmetric: the per-token rule applied to each of the G
 * slices of a row (lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/
 * per_group_avx512_f32_fma_kernel.cpp:78-86 for the scale, :276-292 for q = nearbyint(v / scale)
 * with the true division; dispatch by the {M,G} scale dims, lowoha_reorder.cpp:167-171).
 * scales is {M,G} row-major. */
ZO_EXPORT void zo_quant_per_group(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t G,
                                  int64_t ld_src, int8_t *dst, int64_t ld_dst, float *scales) {
  const int64_t gs = K / G;
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t g = 0; g < G; ++g) {
      float absmax = 0.0f;
      for (int64_t j = 0; j < gs; ++j) {
        float v = zo_read_f32(src, src_dt, m * ld_src + g * gs + j);
        if (isfinite(v)) {
          float a = fabsf(v);
          if (a > absmax) absmax = a;
        }
      }
      if (absmax < 1e-10f) absmax = 1e-10f;
      float scale = absmax / 127.0f;
      if (scale < 1e-10f) scale = 1e-10f;
      scales[m * G + g] = scale;
      if (!dst) continue;
      for (int64_t j = 0; j < gs; ++j) {
        float v = zo_read_f32(src, src_dt, m * ld_src + g * gs + j);
        dst[m * ld_dst + g * gs + j] = isfinite(v) ? (int8_t)(int32_t)nearbyintf(v / scale) : 0;
      }
    }
  }
}

/* Dynamic quantization, asymmetric (u8 rows + s32 zero-points), per token (G == 1) or per group:
 * lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/per_token_avx512_f32_fma_kernel.cpp:89-116
 * (compute_asymmetric_scale_zp: min / max over finite values, an empty or non-finite range becomes [0, 0], a range
 * of width 0 becomes [min, min + 1], scale = (max - min) / 255 clamped to >= 1e-10, zp = round(-min / scale) in
 * double, half away from zero, clamped to the s32 range) and :636-680 (q = clamp(nearbyint(v / scale) + zp, 0, 255)
 * with the true division, non-finite elements -> 0 as the scalar tail :672-677 and the file's notes say; the
 * reference's vector loop gets there through VCVTPS2DQ's 0x80000000 plus a wrapping add, which gives 255 instead
 * when zp < 0, and its tail casts quotients beyond s32, which C leaves undefined: here the sum is taken in 64
 * bits, which agrees with both wherever both are defined); the per-group kernels apply the same rule to every slice
 * of a row (per_group_avx512_f32_fma_kernel.cpp:91-115, :694-760).  scales, zps: {M,G} row-major. */
ZO_EXPORT void zo_quant_asym(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t G, int64_t ld_src,
                             uint8_t *dst, int64_t ld_dst, float *scales, int32_t *zps) {
  const int64_t gs = K / G;
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t g = 0; g < G; ++g) {
      float lo = INFINITY, hi = -INFINITY;
      for (int64_t j = 0; j < gs; ++j) {
        float v = zo_read_f32(src, src_dt, m * ld_src + g * gs + j);
        if (isfinite(v)) {
          if (v < lo) lo = v;
          if (v > hi) hi = v;
        }
      }
      if (lo > hi || !isfinite(lo) || !isfinite(hi)) lo = hi = 0.0f;
      if (hi <= lo) hi = lo + 1.0f;
      float scale = (hi - lo) / 255.0f;
      if (scale < 1e-10f) scale = 1e-10f;
      double zd = round((double)(-lo) / (double)scale);
      int32_t zp = zd < -2147483648.0 ? INT32_MIN : zd > 2147483647.0 ? INT32_MAX : (int32_t)zd;
      scales[m * G + g] = scale;
      zps[m * G + g] = zp;
      if (!dst) continue;
      for (int64_t j = 0; j < gs; ++j) {
        float v = zo_read_f32(src, src_dt, m * ld_src + g * gs + j);
        if (!isfinite(v)) { dst[m * ld_dst + g * gs + j] = 0; continue; }
        float t = nearbyintf(v / scale);
        if (t > 4e9f) t = 4e9f;
        if (t < -4e9f) t = -4e9f;
        int64_t q = (int64_t)t + (int64_t)zp;
        dst[m * ld_dst + g * gs + j] = (uint8_t)(q < 0 ? 0 : q > 255 ? 255 : q);
      }
    }
  }
}

/* ---- exact integer GEMM -------------------------------------------------- */

/* Accumulator of compute_quantized_matmul,
 * operators/matmul/matmul_ref_kernel.cpp:1003-1030 (non-grouped branch):
 * acc[m,n] = sum_k a[m,k] * w[k,n] in int32.  The sum is also carried in int64
 * and the function returns the number of elements whose int64 value does not
 * fit int32 (0 for every case the tests use), so "bit-exact s32" is checked
 * against arithmetic that cannot wrap. */
__attribute__((target_clones("default", "avx2", "arch=skylake-avx512")))
static void zo_dot_rows_s8(const int8_t *a, const int8_t *bt, int64_t K, int64_t N,
                           int64_t ldbt, int32_t *out) {
  for (int64_t n = 0; n < N; ++n) {
    const int8_t *b = bt + n * ldbt;
    int32_t s = 0;
    for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
    out[n] = s;
  }
}

__attribute__((target_clones("default", "avx2", "arch=skylake-avx512")))
static void zo_dot_rows_u8(const uint8_t *a, const int8_t *bt, int64_t K, int64_t N,
                           int64_t ldbt, int32_t *out) {
  for (int64_t n = 0; n < N; ++n) {
    const int8_t *b = bt + n * ldbt;
    int32_t s = 0;
    for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)b[k];
    out[n] = s;
  }
}

/* Fast path used for large shapes and for the timed CPU baseline: weights are
 * transposed once to [N,K] so the k loop is contiguous for both operands. */
ZO_EXPORT void zo_transpose_s8(const int8_t *B, int64_t K, int64_t N, int64_t ldb, int8_t *Bt) {
  #pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) Bt[n * K + k] = B[k * ldb + n];
}

ZO_EXPORT void zo_gemm_s32_bt(const void *A, int32_t a_dt, int64_t lda, const int8_t *Bt,
                              int64_t ldbt, int64_t M, int64_t N, int64_t K, int32_t *acc,
                              int64_t ldacc) {
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    if (a_dt == ZMI_DT_U8)
      zo_dot_rows_u8((const uint8_t *)A + m * lda, Bt, K, N, ldbt, acc + m * ldacc);
    else
      zo_dot_rows_s8((const int8_t *)A + m * lda, Bt, K, N, ldbt, acc + m * ldacc);
  }
}

/* General (strided, optionally transposed) form with the int64 overflow check. */
ZO_EXPORT int64_t zo_gemm_s32(const void *A, int32_t a_dt, int32_t transA, int64_t lda,
                              const int8_t *B, int32_t transB, int64_t ldb, int64_t M, int64_t N,
                              int64_t K, int32_t *acc, int64_t ldacc) {
  int64_t overflow = 0;
  #pragma omp parallel for schedule(static) reduction(+ : overflow)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      int64_t s = 0;
      for (int64_t k = 0; k < K; ++k) {
        int64_t ai = transA ? k * lda + m : m * lda + k;
        int64_t bi = transB ? n * ldb + k : k * ldb + n;
        int32_t a = (a_dt == ZMI_DT_U8) ? (int32_t)((const uint8_t *)A)[ai]
                                        : (int32_t)((const int8_t *)A)[ai];
        s += (int64_t)a * (int64_t)B[bi];
      }
      if (s > INT32_MAX || s < INT32_MIN) overflow++;
      acc[m * ldacc + n] = (int32_t)s;
    }
  }
  return overflow;
}

/* compute_zero_point_compensation, src_zp-only branch,
 * operators/matmul/matmul_ref_kernel.cpp:71-91 (same as
 * lowoha_operators/matmul/lru_cache/lowoha_cache.hpp:99-133):
 * comp[n] = 0 - src_zp * sum_k w[k,n]. */
ZO_EXPORT void zo_zp_comp(const int8_t *B, int32_t transB, int64_t ldb, int64_t K, int64_t N,
                          int32_t src_zp, int32_t *comp) {
  for (int64_t n = 0; n < N; ++n) {
    int32_t s = 0;
    for (int64_t k = 0; k < K; ++k) s += B[transB ? n * ldb + k : k * ldb + n];
    comp[n] = 0 - src_zp * s;
  }
}

/* ---- element-wise post-ops ---------------------------------------------- */

/* Constants of operators/matmul/matmul_ref_kernel.hpp:31-33. */
#define ZO_SQRT_2_OVER_PI 0.79788458347320556640625f
#define ZO_SQRT_2_OVER_2 0.707106769084930419921875f
#define ZO_FITTING_CONST 0.044715f

/* operators/matmul/matmul_ref_kernel.cpp:694-761, same expressions and the
 * same float/double promotion as the C++ source. */
static float zo_gelu_tanh(float x) {
  float v = tanhf(ZO_SQRT_2_OVER_PI * x * (1 + ZO_FITTING_CONST * x * x));
  return (float)(0.5 * x * (1.0f + v));
}
static float zo_gelu_erf(float x) {
  float v = x * ZO_SQRT_2_OVER_2;
  return 0.5f * x * (1.0f + erff(v));
}
static float zo_sigmoid(float x) { return (float)(1.0 / (1.0 + expf(-x))); }
static float zo_swish(float x, float scale) {
  float sx = x * scale;
  return (float)(x * (1.0 / (1.0 + expf(-sx))));
}

ZO_EXPORT float zo_eltwise(int32_t po, float x, float alpha, float beta) {
  switch (po) {
  case ZMI_PO_RELU: return x > 0 ? x : 0;
  /* the AOCL wiring passes a fixed default slope, backends/aocl/aocl_postop.cpp:410 */
  case ZMI_PO_LEAKY_RELU: return x > 0 ? x : 0.01f * x;
  case ZMI_PO_GELU_TANH: return zo_gelu_tanh(x);
  case ZMI_PO_GELU_ERF: return zo_gelu_erf(x);
  case ZMI_PO_SIGMOID: return zo_sigmoid(x);
  /* swish scale is the constant 1, backends/aocl/aocl_postop.cpp:421-423 */
  case ZMI_PO_SWISH: return zo_swish(x, 1.0f);
  case ZMI_PO_TANH: return tanhf(x);
  case ZMI_PO_CLIP: { x = x > alpha ? x : alpha; return x > beta ? beta : x; }
  /* elu_fwd .. log_fwd, operators/matmul/matmul_ref_kernel.cpp:694-751 (elu subtracts the double constant 1.0) */
  case ZMI_PO_ELU: return x > 0 ? x : (float)(alpha * (expf(x) - 1.0));
  case ZMI_PO_SQUARE: return x * x;
  case ZMI_PO_ABS: return x > 0 ? x : -x;
  case ZMI_PO_SQRT: return sqrtf(x);
  case ZMI_PO_EXP: return expf(x);
  case ZMI_PO_LOG: return logf(x);
  /* mish_fwd, operators/matmul/matmul_ref_kernel.cpp:755-760 (std:: overloads on float: all float arithmetic) */
  case ZMI_PO_MISH: {
    const float softplus = fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x)));
    return x * tanhf(softplus);
  }
  default: return x;
  }
}

/* ---- full quantized matmul ---------------------------------------------- */

typedef struct zo_matmul_call {
  char layout;
  int32_t transA, transB, M, N, K;
  float alpha;
  const void *src; int32_t lda;
  const void *weight; int32_t ldb;
  const void *bias; float beta;
  void *dst; int32_t ldc;
  const zmi_matmul_params_t *params;
  int32_t *acc_out;   /* optional [M,N]: the raw s32 accumulator (before compensation) */
  float *scale_out;   /* optional [M]: the per-token scales a dynamic_quant call computed */
  int32_t *zp_out;    /* optional [1]: the zero-point a dynamic_quant call to u8 computed */
} zo_matmul_call;

static void zo_store(void *dst, int32_t dt, int64_t i, float val) {
  /* store_output, operators/matmul/matmul_ref_kernel.cpp:154-254 */
  switch (dt) {
  case ZMI_DT_U8:
    val = val < 0.0f ? 0.0f : (val > 255.0f ? 255.0f : val);
    ((uint8_t *)dst)[i] = (uint8_t)nearbyintf(val);
    break;
  case ZMI_DT_S8:
    val = val < -128.0f ? -128.0f : (val > 127.0f ? 127.0f : val);
    ((int8_t *)dst)[i] = (int8_t)nearbyintf(val);
    break;
  case ZMI_DT_S32:
    val = val < (float)INT32_MIN ? (float)INT32_MIN : (val > (float)INT32_MAX ? (float)INT32_MAX : val);
    /* (float)INT32_MAX is 2^31; the reference's cast of it is out of range, so pin it */
    ((int32_t *)dst)[i] = val >= 2147483648.0f ? INT32_MAX : (int32_t)nearbyintf(val);
    break;
  case ZMI_DT_BF16: ((uint16_t *)dst)[i] = zo_f32_to_bf16_ctor(val); break;
  case ZMI_DT_F16: ((uint16_t *)dst)[i] = zo_f32_to_f16(val); break;
  default: ((float *)dst)[i] = val; break;
  }
}

/* ---- GGML Q8_0 packed weights ------------------------------------------------------------ */

/* fp16_to_fp32 of lowoha_operators/matmul/ggml_weight_unpack.cpp:54-65 (llama.cpp's), restated on the bit
 * fields: exact conversion of every half value, subnormals included. */
ZO_EXPORT float zo_fp16_to_f32(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  uint32_t u;
  if (e == 0x1f) u = sign | 0x7f800000u | (m << 13);              /* inf / NaN */
  else if (e != 0) u = sign | ((e + 112u) << 23) | (m << 13);     /* normal: rebias 15 -> 127 */
  else if (m == 0) u = sign;                                      /* zero */
  else {                                                          /* subnormal: m * 2^-24 */
    float f = (float)m * 5.9604644775390625e-08f;
    memcpy(&u, &f, 4);
    u |= sign;
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* float16_t(float), common/float16.cpp:124-205: round to nearest even into half precision.  f32 zeros and
 * subnormals, and magnitudes that round below the smallest half subnormal, give a signed zero; magnitudes from
 * 65520 up give infinity; NaN keeps the top ten mantissa bits and is made quiet.  A half-subnormal result whose
 * rounding carries into the exponent (magnitudes in [2^-14 - 2^-25, 2^-14)) loses the carry, because the
 * reference masks that result with the mantissa field: it stores a signed zero there, and so does this. */
ZO_EXPORT uint16_t zo_f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t e = (u >> 23) & 0xffu, m = u & 0x7fffffu;
  if (e == 0) return sign;
  if (e == 255) return m ? (uint16_t)(sign | 0x7c00u | (m >> 13) | 0x200u) : (uint16_t)(sign | 0x7c00u);
  int32_t he = (int32_t)e - 112;                     /* exponent bias 127 -> 15 */
  if (he >= 31) return (uint16_t)(sign | 0x7c00u);
  if (he <= 0) {
    if (he < -10) return sign;
    const uint32_t full = m | 0x800000u;             /* with the implicit one */
    const int shift = 14 - he;
    const uint32_t half = 1u << (shift - 1);
    uint32_t q = full >> shift;
    if ((full & half) && ((full & (half - 1u)) || (q & 1u))) q += 1u;
    return (uint16_t)(sign | (q & 0x3ffu));
  }
  uint32_t q = m >> 13;
  if ((m & 0x1000u) && ((m & 0xfffu) || (q & 1u))) {
    q += 1u;
    if (q > 0x3ffu) {
      q = 0;
      he += 1;
      if (he >= 31) return (uint16_t)(sign | 0x7c00u);
    }
  }
  return (uint16_t)(sign | ((uint32_t)he << 10) | q);
}

/* fp32_to_bf16 of ggml_weight_unpack.cpp:66-73: NaN quieted, else round to nearest even (no flush). */
static uint16_t zo_ggml_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 64u);
  return (uint16_t)((u + (0x7fffu + ((u >> 16) & 1u))) >> 16);
}

/* ggml_unpack_weight_buffer, Q8_0 branch with bf16 scales (ggml_weight_unpack.cpp:190-236): blocks
 * [N][K/32] of { fp16 d; int8 qs[32] } -> rows[n*K + g*32 + i] = qs[i], scales[g*N + n] = bf16(f32(d)). */
ZO_EXPORT void zo_ggml_q8_0_unpack(const void *blocks, int64_t N, int64_t K, int8_t *rows, uint16_t *scales) {
  const int64_t ng = K / 32;
  const uint8_t *b = (const uint8_t *)blocks;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t g = 0; g < ng; ++g) {
      const uint8_t *blk = b + (n * ng + g) * 34;
      uint16_t d;
      memcpy(&d, blk, 2);
      scales[g * N + n] = zo_ggml_f32_to_bf16(zo_fp16_to_f32(d));
      memcpy(rows + n * K + g * 32, blk + 2, 32);
    }
}

/* cvt_s4_to_s8 with extract_4bit_nibble, lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:33-41, 144-163:
 * element (row, col) of the K x N weight matrix sits at physical index row * ldb + col (col * ldb + row when
 * transposed) of a nibble array, two per byte, even index = low nibble; the nibble is sign-extended from bit 3
 * (-8 .. 7).  The result is a contiguous row-major [K, N] s8 matrix. */
ZO_EXPORT void zo_s4_to_s8(const void *packed, int64_t K, int64_t N, int64_t ldb, int32_t transposed, int8_t *out) {
  const uint8_t *w = (const uint8_t *)packed;
  for (int64_t row = 0; row < K; ++row)
    for (int64_t col = 0; col < N; ++col) {
      const int64_t idx = transposed ? col * ldb + row : row * ldb + col;
      const uint8_t byte = w[idx / 2];
      int32_t v = (idx % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
      if (v & 0x08) v -= 16;
      out[row * N + col] = (int8_t)v;
    }
}

/* matmul_direct for the int8 path.  Pipeline of lowoha_operators/matmul/
 * lowoha_matmul.cpp:278-510: optional dynamic per-token quantization of a
 * bf16/f32 source (matmul/quantization/reorder_quantization.cpp:43-280), then
 * the int8 GEMM and the dequantization chain of
 * operators/matmul/matmul_ref_kernel.cpp:1032-1053:
 *   y = float(acc); y *= alpha (if != 1); y += beta * C (if beta);
 *   y += float(zp_comp[n]); y *= src_scale[per-tensor | m]; y *= wei_scale[n % len];
 *   y += bias[n]; post-ops in order; y = y * dst_scale + dst_zp (quantize_dst);
 *   store with the dtype's rounding.
 * Returns a ZMI_* status. */
ZO_EXPORT int32_t zo_matmul_int8(const zo_matmul_call *c) {
  zmi_matmul_params_t pl = *c->params;   /* working copy: the GGML unpack sets the weight scales */
  const zmi_matmul_params_t *p = &pl;
  const int64_t M = c->M, N = c->N, K = c->K;
  if (p->dt_wei != ZMI_DT_S8 && p->dt_wei != ZMI_DT_S4) return ZMI_UNIMPLEMENTED;
  const void *weight = c->weight;
  int64_t ldb = c->ldb;
  int32_t transB = c->transB;
  int8_t *ggml_rows = NULL;
  uint16_t *ggml_scales = NULL;
  int64_t w4a8_groups = 0;
  if (p->dt_wei == ZMI_DT_S4) {
    /* W4A8: validate_w4a8_inputs, lowoha_operators/matmul/lowoha_matmul_utils.cpp:72-176 (bf16 source with
     * dynamic_quant and s8 compute, bf16 destination, symmetric, {G,N} f32 / bf16 weight scales, K/G a multiple
     * of 4, source scale dims {1,1}, {M,1} or {M,G}); anything else with s4 weights is the weight-only path,
     * which is not restated here.  The weights are widened once to [K,N] s8
     * (w4a8ReorderAndCacheWeightsAocl, backends/aocl/aocl_kernel.cpp:704-793). */
    if (p->dt_src == ZMI_DT_S8) return ZMI_FAILURE;
    if (p->dynamic_quant && (p->dt_src == ZMI_DT_F32 || p->dt_dst == ZMI_DT_F32)) return ZMI_FAILURE;
    if (p->dt_src == ZMI_DT_U8 && (p->src_scale.buff || p->dynamic_quant)) return ZMI_FAILURE;
    if (!(p->dynamic_quant && p->dt_src == ZMI_DT_BF16)) return ZMI_UNIMPLEMENTED;
    if (p->dt_compute != ZMI_DT_S8 || p->dt_dst != ZMI_DT_BF16) return ZMI_FAILURE;
    if (p->wei_zp.buff || p->src_zp.buff || !p->wei_scale.buff) return ZMI_FAILURE;
    if (p->wei_scale.dt != ZMI_DT_F32 && p->wei_scale.dt != ZMI_DT_BF16) return ZMI_FAILURE;
    if (p->wei_scale.ndims != 2) return ZMI_FAILURE;
    const int64_t G = p->wei_scale.dims[0];
    if (G <= 0 || p->wei_scale.dims[1] != N || K % G != 0 || (K / G) % 4 != 0) return ZMI_FAILURE;
    if (p->src_scale.dt != ZMI_DT_F32 && p->src_scale.dt != ZMI_DT_BF16) return ZMI_FAILURE;
    if (p->src_scale.ndims != 2) return ZMI_FAILURE;
    const int64_t sr = p->src_scale.dims[0], sc = p->src_scale.dims[1];
    if (!((sr == 1 && sc == 1) || (sr == M && sc == 1) || (sr == M && sc == G))) return ZMI_FAILURE;
    ggml_rows = (int8_t *)malloc((size_t)N * K);
    zo_s4_to_s8(weight, K, N, ldb, transB, ggml_rows);
    weight = ggml_rows; ldb = N; transB = 0;
    w4a8_groups = G;
  }
  if (p->pack_format_b == 1) {
    /* validate_ggml_packed_inputs + unpack_ggml_weights_and_cache,
     * lowoha_operators/matmul/ggml_weight_unpack.cpp:155-183, 367-420: transB required, the unpacked
     * rows are [N, K], the scales become the bf16 {K/32, N} weight scales */
    if (!transB || K % 32 != 0) return ZMI_FAILURE;
    ggml_rows = (int8_t *)malloc((size_t)N * K);
    ggml_scales = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(K / 32) * N);
    zo_ggml_q8_0_unpack(weight, N, K, ggml_rows, ggml_scales);
    weight = ggml_rows; ldb = K;
    pl.wei_scale.buff = ggml_scales; pl.wei_scale.dt = ZMI_DT_BF16;
    pl.wei_scale.ndims = 2; pl.wei_scale.dims[0] = K / 32; pl.wei_scale.dims[1] = N;
  }

  const void *A = c->src;
  int32_t a_dt = p->dt_src;
  int64_t lda = c->lda;
  int32_t transA = c->transA;
  int8_t *qbuf = NULL;
  float *sbuf = NULL;
  const float *src_scale = NULL;
  int64_t src_scale_n = p->src_scale.buff ? zo_nelems(&p->src_scale) : 0;
  int32_t src_scale_dt = p->src_scale.dt;

  const int dyn = p->dynamic_quant && (a_dt == ZMI_DT_BF16 || a_dt == ZMI_DT_F32) &&
                  (p->dt_compute == ZMI_DT_S8 || p->dt_compute == ZMI_DT_U8);
  int32_t dyn_zp = 0;
  if (dyn && p->dt_compute == ZMI_DT_U8) {
    /* dynamic asymmetric quantization of the source to u8: the GEMM reads ONE source zero-point
     * (operators/matmul/matmul_ref_kernel.cpp:935-939, backends/aocl/aocl_kernel.cpp:971-980), so the granularity that
     * means something is per tensor: src_scale and src_zp of one element each
     * (matmul/quantization/reorder_quantization.cpp:60-75, 208-230: dims and types required, buffers optional).
     * Parameters: compute_scale_zp, lowoha_operators/reorder/lowoha_reorder_utils.cpp:708-765 -- min / max over the
     * finite values ([0, 0] when there is none), max = min + 1 when max <= min, scale = (max - min) / 255,
     * zp = round(-min / scale) in double (half away from zero, clamped to s32) with the scale as computed, and only
     * then scale = max(scale, 1e-10).  Elements: q = clamp(int32(nearbyint(v / scale)) + zp, 0, 255)
     * (reorder_data_type/scalar_impl/scalar_ref_kernels.cpp:36-40); non-finite elements, whose cast the reference
     * leaves undefined, give 0 as in its per-token kernels.  The reference's AVX-512 per-tensor kernels may multiply
     * by a reciprocal instead of dividing: parity of the last count on exact ties is unpinned. */
    if (transA || zo_nelems(&p->src_scale) != 1 || p->src_zp.ndims <= 0 || zo_nelems(&p->src_zp) != 1 ||
        p->src_zp.dt != ZMI_DT_S32)
      return ZMI_UNIMPLEMENTED;
    float lo = 3.402823466e+38f, hi = -3.402823466e+38f;
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) {
        float v = zo_read_f32(A, a_dt, m * lda + k);
        if (isfinite(v)) { if (v < lo) lo = v; if (v > hi) hi = v; }
      }
    if (lo == 3.402823466e+38f && hi == -3.402823466e+38f) lo = hi = 0.0f;
    if (hi <= lo) hi = lo + 1.0f;
    float s = (hi - lo) / 255.0f;
    double zd = round((double)(-lo) / (double)s);
    dyn_zp = zd < -2147483648.0 ? INT32_MIN : zd > 2147483647.0 ? INT32_MAX : (int32_t)zd;
    if (s < 1e-10f) s = 1e-10f;
    /* a bf16 scale buffer: the parameters are stored first (narrowed, lowoha_reorder_utils.cpp:600-628, 810) and the
     * codes are then made by the static reorder on what the buffer reads back as (lowoha_reorder.cpp:186-205) */
    if (p->src_scale.dt == ZMI_DT_BF16) s = zo_bf16_to_f32(zo_f32_to_bf16_rne(s));
    qbuf = (int8_t *)malloc((size_t)M * K);
    sbuf = (float *)malloc(sizeof(float));
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) {
        float v = zo_read_f32(A, a_dt, m * lda + k);
        int64_t q = 0;
        if (isfinite(v)) {
          float t = nearbyintf(v / s);
          if (t > 4e9f) t = 4e9f;
          if (t < -4e9f) t = -4e9f;
          q = (int64_t)t + (int64_t)dyn_zp;
          q = q < 0 ? 0 : q > 255 ? 255 : q;
        }
        ((uint8_t *)qbuf)[m * K + k] = (uint8_t)q;
      }
    sbuf[0] = s;
    if (c->scale_out) c->scale_out[0] = sbuf[0];
    if (c->zp_out) c->zp_out[0] = dyn_zp;
    pl.src_zp.buff = &dyn_zp; pl.src_zp.dt = ZMI_DT_S32;
    A = qbuf; a_dt = ZMI_DT_U8; lda = K;
    src_scale = sbuf; src_scale_n = 1; src_scale_dt = ZMI_DT_F32;
  } else if (dyn) {
    if (transA) return ZMI_UNIMPLEMENTED;
    qbuf = (int8_t *)malloc((size_t)M * K);
    sbuf = (float *)malloc(sizeof(float) * (size_t)M);
    int64_t dn = 1;
    for (int i = 0; i < p->src_scale.ndims; ++i) dn *= p->src_scale.dims[i];
    if (dn > M && dn % M == 0 && K % (dn / M) == 0) {
      free(sbuf);
      sbuf = (float *)malloc(sizeof(float) * (size_t)dn);
      zo_quant_per_group(A, a_dt, M, K, dn / M, lda, qbuf, K, sbuf);
    } else if (dn == M && M > 1) {
      zo_quant_per_token(A, a_dt, M, K, lda, qbuf, K, sbuf);
    } else {
      /* per-tensor dynamic scale: same formula over the whole tensor,
       * lowoha_operators/reorder/lowoha_reorder_utils.cpp:724-761 */
      float absmax = 0.0f;
      for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
          float v = zo_read_f32(A, a_dt, m * lda + k);
          if (isfinite(v) && fabsf(v) > absmax) absmax = fabsf(v);
        }
      if (absmax < 1e-10f) absmax = 1e-10f;
      float s = absmax / 127.0f;
      if (s < 1e-10f) s = 1e-10f;
      for (int64_t m = 0; m < M; ++m) {
        sbuf[m] = s;
        for (int64_t k = 0; k < K; ++k) {
          float v = zo_read_f32(A, a_dt, m * lda + k);
          qbuf[m * K + k] = isfinite(v) ? (int8_t)(int32_t)nearbyintf(v / s) : 0;
        }
      }
      dn = 1;
    }
    if (p->src_scale.dt == ZMI_DT_BF16) {
      /* the computed f32 scales are narrowed into the scale buffer's dtype (write_scale / float_to_bf16 =
       * bfloat16_t::f32_to_bf16_val, lowoha_operators/reorder/lowoha_reorder_utils.cpp:600-628, :835-856) and the
       * GEMM reads the narrowed values back; the rows above were quantized with the f32 scales */
      const int64_t ns = dn == 1 ? M : dn;
      for (int64_t i = 0; i < ns; ++i) sbuf[i] = zo_bf16_to_f32(zo_f32_to_bf16_rne(sbuf[i]));
    }
    if (c->scale_out) memcpy(c->scale_out, sbuf, sizeof(float) * (size_t)dn);
    if (w4a8_groups > 1 && dn <= M) {
      /* broadcast_w4a8_src_scale, backends/aocl/aocl_kernel.cpp:167-236: compact per-tensor / per-token
       * scales are repeated over the G groups, and the per-group GEMM follows */
      float *wide = (float *)malloc(sizeof(float) * (size_t)M * w4a8_groups);
      for (int64_t m = 0; m < M; ++m)
        for (int64_t g = 0; g < w4a8_groups; ++g) wide[m * w4a8_groups + g] = sbuf[dn == 1 ? 0 : m];
      free(sbuf);
      sbuf = wide;
      dn = M * w4a8_groups;
    }
    A = qbuf; a_dt = ZMI_DT_S8; lda = K;
    src_scale = sbuf; src_scale_n = dn; src_scale_dt = ZMI_DT_F32;
  } else if (a_dt != ZMI_DT_S8 && a_dt != ZMI_DT_U8) {
    return ZMI_UNIMPLEMENTED;
  } else {
    src_scale = (const float *)p->src_scale.buff;
  }

  /* Per-group source scales ({M,G}, with {G,N} weight scales): per-group branch of
   * compute_quantized_matmul, operators/matmul/matmul_ref_kernel.cpp:917-1001 --
   *   sum = 0; for g: grp = float(sum_{k in g} a*w) * ss[m*G+g]; grp *= ws[g*N+n]; sum += grp
   * then alpha, beta, bias, post-ops (the source / weight scale multiplications of the
   * plain chain are skipped, :1041-1048).  The validator admits it for symmetric
   * s8 / bf16 / f32 sources and f32 / bf16 destinations only
   * (lowoha_operators/matmul/lowoha_matmul_utils.cpp:253-301). */
  if (src_scale_n > M && src_scale_n % M == 0) {
    const int64_t G = src_scale_n / M;
    const int64_t wn = p->wei_scale.buff ? zo_nelems(&p->wei_scale) : 0;
    if (K % G != 0 || wn != G * N || p->src_zp.buff || a_dt != ZMI_DT_S8 ||
        !(p->dt_dst == ZMI_DT_F32 || p->dt_dst == ZMI_DT_BF16)) {
      free(qbuf); free(sbuf); free(ggml_rows); free(ggml_scales);
      return ZMI_FAILURE;
    }
    const int64_t gs = K / G;
    const int8_t *W = (const int8_t *)weight;
    #pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n = 0; n < N; ++n) {
        float sum = 0.0f;
        for (int64_t g = 0; g < G; ++g) {
          int32_t group_sum = 0;
          for (int64_t k = g * gs; k < (g + 1) * gs; ++k) {
            int32_t a = ((const int8_t *)A)[transA ? k * lda + m : m * lda + k];
            group_sum += a * (int32_t)W[transB ? n * ldb + k : k * ldb + n];
          }
          float grp = (float)group_sum * zo_read_f32(src_scale, src_scale_dt, m * G + g);
          grp *= zo_read_f32(p->wei_scale.buff, p->wei_scale.dt, g * N + n);
          sum += grp;
        }
        float y = sum;
        if (c->alpha != 1.0f) y *= c->alpha;
        if (c->beta != 0.0f) y += zo_read_f32(c->dst, p->dt_dst, m * (int64_t)c->ldc + n) * c->beta;
        if (c->bias) y += zo_read_f32(c->bias, p->dt_bias == ZMI_DT_NONE ? ZMI_DT_F32 : p->dt_bias, n);
        for (int i = 0; i < p->n_postops; ++i) {
          const zmi_post_op_t *po = &p->postops[i];
          if (po->po_type == ZMI_PO_BINARY_ADD || po->po_type == ZMI_PO_BINARY_MUL) {
            int64_t ld = po->leading_dim > 0 ? po->leading_dim : N;
            int rowb = (po->ndims == 2 && po->dims[0] == 1) || po->ndims == 1;
            float t = zo_read_f32(po->buff, po->dtype, rowb ? n : m * ld + n);
            y = po->po_type == ZMI_PO_BINARY_ADD ? y + t : y * t;
          } else {
            y = zo_eltwise(po->po_type, y, po->alpha, po->beta);
          }
        }
        zo_store(c->dst, p->dt_dst, m * (int64_t)c->ldc + n, y);
      }
    }
    free(qbuf); free(sbuf); free(ggml_rows); free(ggml_scales);
    return ZMI_SUCCESS;
  }

  int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)M * N);
  if (!transA && M * N * K > (1 << 22)) {
    int8_t *Bt = (int8_t *)weight;
    int64_t ldbt = ldb;
    int8_t *tmp = NULL;
    if (!transB) {
      tmp = (int8_t *)malloc((size_t)N * K);
      zo_transpose_s8((const int8_t *)weight, K, N, ldb, tmp);
      Bt = tmp; ldbt = K;
    }
    zo_gemm_s32_bt(A, a_dt, lda, Bt, ldbt, M, N, K, acc, N);
    free(tmp);
  } else {
    zo_gemm_s32(A, a_dt, transA, lda, (const int8_t *)weight, transB, ldb, M, N, K, acc, N);
  }
  if (c->acc_out) memcpy(c->acc_out, acc, sizeof(int32_t) * (size_t)M * N);

  int32_t src_zp = p->src_zp.buff ? zo_read_s32(p->src_zp.buff, p->src_zp.dt, 0) : 0;
  int32_t *comp = NULL;
  if (src_zp) {
    comp = (int32_t *)malloc(sizeof(int32_t) * (size_t)N);
    zo_zp_comp((const int8_t *)weight, transB, ldb, K, N, src_zp, comp);
  }
  /* a weight zero-point (per tensor): the 2-D compensation of cache_or_compute_zp_compensation,
   * lowoha_operators/matmul/lru_cache/lowoha_cache.hpp:151-232:
   * comp[m,n] = -src_zp * colsum[n] - wei_zp * rowsum[m] + src_zp * wei_zp * K, rowsum over the source as given
   * (u8 or s8); its column term is `comp` above, the rest is one int32 per row */
  int32_t wei_zp = p->wei_zp.buff ? zo_read_s32(p->wei_zp.buff, p->wei_zp.dt, 0) : 0;
  int32_t *rowc = NULL;
  if (wei_zp) {
    rowc = (int32_t *)malloc(sizeof(int32_t) * (size_t)M);
    for (int64_t m = 0; m < M; ++m) {
      int32_t rs = 0;
      for (int64_t k = 0; k < K; ++k) {
        const int64_t i = transA ? k * lda + m : m * lda + k;
        rs += a_dt == ZMI_DT_U8 ? (int32_t)((const uint8_t *)A)[i] : (int32_t)((const int8_t *)A)[i];
      }
      rowc[m] = -wei_zp * rs + src_zp * wei_zp * (int32_t)K;
    }
  }
  const int per_token = (src_scale_n == M && M > 1);
  const int64_t wei_scale_n = p->wei_scale.buff ? zo_nelems(&p->wei_scale) : 0;
  const float dst_scale = p->dst_scale.buff ? zo_read_f32(p->dst_scale.buff, p->dst_scale.dt, 0) : 1.0f;
  const int has_dst_q = p->dst_scale.buff != NULL || p->dst_zp.buff != NULL;
  const float dst_zp = p->dst_zp.buff ? zo_read_f32(p->dst_zp.buff, p->dst_zp.dt, 0) : 0.0f;

  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float y = (float)acc[m * N + n];
      if (c->alpha != 1.0f) y *= c->alpha;
      if (c->beta != 0.0f) y += zo_read_f32(c->dst, p->dt_dst, m * (int64_t)c->ldc + n) * c->beta;
      if (comp || rowc) y += (float)((comp ? comp[n] : 0) + (rowc ? rowc[m] : 0));
      if (src_scale_n) y *= zo_read_f32(src_scale, src_scale_dt, per_token ? m : 0);
      if (wei_scale_n) y *= zo_read_f32(p->wei_scale.buff, p->wei_scale.dt, n % wei_scale_n);
      if (c->bias) y += zo_read_f32(c->bias, p->dt_bias == ZMI_DT_NONE ? ZMI_DT_F32 : p->dt_bias, n);
      for (int i = 0; i < p->n_postops; ++i) {
        const zmi_post_op_t *po = &p->postops[i];
        if (po->po_type == ZMI_PO_BINARY_ADD || po->po_type == ZMI_PO_BINARY_MUL) {
          /* binary_add_fwd / binary_mul_fwd with scale 1,
           * operators/matmul/matmul_ref_kernel.cpp:753-759; operand is
           * {1,N} (row broadcast) or {M,N} with leading_dim */
          int64_t ld = po->leading_dim > 0 ? po->leading_dim : N;
          int rowb = (po->ndims == 2 && po->dims[0] == 1) || po->ndims == 1;
          float t = zo_read_f32(po->buff, po->dtype, rowb ? n : m * ld + n);
          y = po->po_type == ZMI_PO_BINARY_ADD ? y + t : y * t;
        } else {
          y = zo_eltwise(po->po_type, y, po->alpha, po->beta);
        }
      }
      if (has_dst_q) y = y * dst_scale + dst_zp;
      zo_store(c->dst, p->dt_dst, m * (int64_t)c->ldc + n, y);
    }
  }
  free(acc); free(comp); free(rowc); free(qbuf); free(sbuf); free(ggml_rows); free(ggml_scales);
  return ZMI_SUCCESS;
}

/* ---- weight-only quantization ---------------------------------------------------------- */

/* cvt_int4_to_bf16, lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:43-139: every 4-bit code of the K x N
 * weight matrix (physical nibble index row * ldb + col, or col * ldb + row when transposed; even index = low nibble;
 * s4 codes sign-extended, u4 codes as they are) becomes one bf16 value,
 *   f = float(code); f = (f - zp) * scale, or for u4 codes with a bf16 zero-point f = (f - 8) * scale + zp;
 *   out[row * N + col] = bfloat16_t(f),
 * the scale / zero-point read per tensor (1 element), per column (N elements) or per K group and column
 * (element count / N groups of K / groups rows each: index group * N + col). */
ZO_EXPORT void zo_woq_dequant(const void *packed, int64_t K, int64_t N, int64_t ldb, int32_t transposed, int32_t wei_dt,
                              const void *scales, int64_t scale_n, int32_t scale_dt,
                              const void *zp, int64_t zp_n, int32_t zp_dt, uint16_t *out) {
  const uint8_t *w = (const uint8_t *)packed;
  const int float_domain_u4 = zp_dt == ZMI_DT_BF16 && wei_dt == ZMI_DT_U4;
  int64_t group_size = K;
  if (scale_n > 1 && scale_n != N) {
    const int64_t groups = scale_n / N;
    if (groups > 0) group_size = K / groups;
  }
  for (int64_t row = 0; row < K; ++row)
    for (int64_t col = 0; col < N; ++col) {
      const int64_t idx = transposed ? col * ldb + row : row * ldb + col;
      const uint8_t byte = w[idx / 2];
      int32_t v = (idx % 2 == 0) ? (byte & 0x0F) : (byte >> 4);
      if (wei_dt == ZMI_DT_S4 && (v & 0x08)) v -= 16;
      float f = (float)v;
      const int64_t so = scale_n <= 1 ? 0 : scale_n == N ? col : (row / group_size) * N + col;
      const float scale = scale_n ? zo_read_f32(scales, scale_dt, so) : 1.0f;
      float zpv = 0.0f;
      if (zp_n >= 1) zpv = zo_read_f32(zp, zp_dt, zp_n == 1 ? 0 : zp_n == N ? col : (row / group_size) * N + col);
      if (float_domain_u4) {
        f = (f - 8) * scale;
        f = f + zpv;
      } else {
        f = (f - zpv) * scale;
      }
      out[row * N + col] = zo_f32_to_bf16_ctor(f);
    }
}

/* matmul_direct with a bf16 source, s4 / u4 weights and no dynamic_quant.  Rules: validate_matmul_direct_inputs,
 * lowoha_operators/matmul/lowoha_matmul_utils.cpp:214-328 (constant weights, no source / destination quantization
 * parameters, u4 weights need a bf16 or s8 zero-point, a bf16 source does not store f16).  Arithmetic: the weights
 * become bf16 once (zo_woq_dequant), then the bf16 GEMM with f32 accumulation in k order and the tail of
 * compute_matmul, operators/matmul/matmul_ref_kernel.cpp:877-896: sum *= alpha (if != 1); sum += C * beta (if beta);
 * sum += bias; then the post-ops in order and the store (no destination quantization on this path, :499-502).
 * The reference's own GEMM on the bf16 matrix is AOCL's, whose summation order is not part of its contract: results
 * are compared with this function to a tolerance, not bit for bit. */
ZO_EXPORT int32_t zo_matmul_woq(const zo_matmul_call *c, int32_t is_weights_const) {
  const zmi_matmul_params_t *p = c->params;
  const int64_t M = c->M, N = c->N, K = c->K;
  if (!(p->dt_src == ZMI_DT_BF16 && (p->dt_wei == ZMI_DT_S4 || p->dt_wei == ZMI_DT_U4) && !p->dynamic_quant))
    return ZMI_UNIMPLEMENTED;
  if (!is_weights_const) return ZMI_FAILURE;
  if (p->src_scale.buff || p->dst_scale.buff || p->src_zp.buff || p->dst_zp.buff) return ZMI_FAILURE;
  if (p->dt_wei == ZMI_DT_U4 && (!p->wei_zp.buff || (p->wei_zp.dt != ZMI_DT_BF16 && p->wei_zp.dt != ZMI_DT_S8)))
    return ZMI_FAILURE;
  if (p->dt_dst == ZMI_DT_F16 || !p->wei_scale.buff) return ZMI_FAILURE;
  const int64_t ns = zo_nelems(&p->wei_scale), nz = p->wei_zp.buff ? zo_nelems(&p->wei_zp) : 0;
  if (!(ns == 1 || ns == N || (ns > N && ns % N == 0 && K % (ns / N) == 0))) return ZMI_FAILURE;
  if (nz && !(nz == 1 || nz == N || nz == ns)) return ZMI_FAILURE;
  uint16_t *wb = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)K * N);
  zo_woq_dequant(c->weight, K, N, c->ldb, c->transB, p->dt_wei, p->wei_scale.buff, ns,
                 p->wei_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p->wei_scale.dt, p->wei_zp.buff, nz, p->wei_zp.dt, wb);
  const uint16_t *A = (const uint16_t *)c->src;
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float sum = 0.0f;
      for (int64_t k = 0; k < K; ++k)
        sum += zo_bf16_to_f32(A[c->transA ? k * c->lda + m : m * c->lda + k]) * zo_bf16_to_f32(wb[k * N + n]);
      float y = sum;
      const int64_t o = m * (int64_t)c->ldc + n;
      if (c->alpha != 1.0f) y *= c->alpha;
      if (c->beta != 0.0f) y += zo_read_f32(c->dst, p->dt_dst, o) * c->beta;
      if (c->bias) y += zo_read_f32(c->bias, p->dt_bias == ZMI_DT_NONE ? ZMI_DT_F32 : p->dt_bias, n);
      for (int i = 0; i < p->n_postops; ++i) {
        const zmi_post_op_t *po = &p->postops[i];
        if (po->po_type == ZMI_PO_BINARY_ADD || po->po_type == ZMI_PO_BINARY_MUL) {
          int64_t ld = po->leading_dim > 0 ? po->leading_dim : N;
          int rowb = (po->ndims == 2 && po->dims[0] == 1) || po->ndims == 1;
          float t = zo_read_f32(po->buff, po->dtype, rowb ? n : m * ld + n);
          y = po->po_type == ZMI_PO_BINARY_ADD ? y + t : y * t;
        } else {
          y = zo_eltwise(po->po_type, y, po->alpha, po->beta);
        }
      }
      zo_store(c->dst, p->dt_dst, o, y);
    }
  }
  free(wb);
  return ZMI_SUCCESS;
}

/* ---- gated activation ----------------------------------------------------- */

/* silu_and_mul_row_scalar_{bf16,f32}, gelu_and_mul_*, swiglu_oai_mul_*,
 * lowoha_operators/matmul/group_matmul/group_matmul_moe_act.cpp:88-154:
 * split halves [gate | up], dst[:,0:dim] = act(gate) * up, f32 math,
 * bf16 result through the bfloat16_t constructor. */
static float zo_sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

ZO_EXPORT void zo_gated_act(int32_t act, void *buf, int32_t dt, int64_t M, int64_t N, int64_t ld) {
  const int64_t dim = N / 2;
  #pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < dim; ++n) {
      float g, u, r;
      if (act == ZMI_ACT_SWIGLU_OAI_MUL) {
        g = zo_read_f32(buf, dt, m * ld + 2 * n);
        u = zo_read_f32(buf, dt, m * ld + 2 * n + 1);
        g = fmaxf(-7.0f, fminf(g, 7.0f));
        u = fmaxf(-7.0f, fminf(u, 7.0f));
        float sig = zo_sigmoid_f(g * 1.702f);
        r = (1.0f + u) * g * sig;
      } else {
        g = zo_read_f32(buf, dt, m * ld + n);
        u = zo_read_f32(buf, dt, m * ld + dim + n);
        if (act == ZMI_ACT_SILU_AND_MUL) r = (g * zo_sigmoid_f(g)) * u;
        else r = (g * 0.5f * (1.0f + erff(g * 0.7071067811865476f))) * u;
      }
      if (dt == ZMI_DT_BF16) ((uint16_t *)buf)[m * ld + n] = zo_f32_to_bf16_ctor(r);
      else if (dt == ZMI_DT_F16) ((uint16_t *)buf)[m * ld + n] = zo_f32_to_f16(r);   /* :165-182 */
      else ((float *)buf)[m * ld + n] = r;
    }
  }
}

/* ---- MoE weighted reduce ---------------------------------------------------- */

/* moe_weighted_reduce_avx512_{bf16,f32},
 * lowoha_operators/matmul/group_matmul/group_matmul_moe_postop.cpp:191-286:
 * acc = w0*x0 (one rounding), then acc = fma(wk, xk, acc) for k = 1..topk-1,
 * bf16 store with the plain RNE bit trick.  (The scalar twin at :103-129 starts
 * from 0 and uses mul+add; the two differ by at most one f32 rounding per term.) */
ZO_EXPORT void zo_moe_reduce(const void *const *row_ptrs, const float *w, int32_t skip_weighted,
                             int64_t T, int32_t topk, int64_t D, int32_t dt, void *out, int64_t ldo) {
  #pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; ++t) {
    for (int64_t d = 0; d < D; ++d) {
      float acc = 0.0f;
      for (int k = 0; k < topk; ++k) {
        float wk = skip_weighted ? 1.0f : w[t * topk + k];
        float x = zo_read_f32(row_ptrs[t * topk + k], dt, d);
        acc = (k == 0) ? wk * x : fmaf(wk, x, acc);
      }
      if (dt == ZMI_DT_BF16) ((uint16_t *)out)[t * ldo + d] = zo_f32_to_bf16_rne(acc);
      else if (dt == ZMI_DT_F16) ((uint16_t *)out)[t * ldo + d] = zo_f32_to_f16(acc);   /* store_from_f32, :84-100 */
      else ((float *)out)[t * ldo + d] = acc;
    }
  }
}

/* ---- timed CPU baseline helper ------------------------------------------------ */

/* Threads an OpenMP parallel region of this library runs on (what the timed helper below uses). */
ZO_EXPORT int32_t zo_omp_threads(void) {
  int32_t n = 1;
  #pragma omp parallel
  {
    #pragma omp single
    n = omp_get_num_threads();
  }
  return n;
}

/* One decode-style call on already-quantized operands, the shape of work the
 * reference's CPU path spends its time on (s8 x s8 -> s32 GEMM over
 * pre-transposed weights, then scale * scale and SiLU, bf16 store).  Used only
 * by bench.py's cpu_baseline leg. */
ZO_EXPORT void zo_bench_s8_gemm(const int8_t *A, const int8_t *Bt, const float *sa, const float *sb,
                                int64_t M, int64_t N, int64_t K, int32_t po, uint16_t *dst) {
  #pragma omp parallel
  {
    int32_t *row = (int32_t *)malloc(sizeof(int32_t) * 256);
    #pragma omp for schedule(static) collapse(2)
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n0 = 0; n0 < N; n0 += 256) {
        int64_t nb = N - n0 < 256 ? N - n0 : 256;
        zo_dot_rows_s8(A + m * K, Bt + n0 * K, K, nb, K, row);
        for (int64_t j = 0; j < nb; ++j) {
          float y = (float)row[j];
          y *= sa[m];
          y *= sb[n0 + j];
          y = zo_eltwise(po, y, 0.0f, 0.0f);
          dst[m * N + n0 + j] = zo_f32_to_bf16_ctor(y);
        }
      }
    }
    free(row);
  }
}
