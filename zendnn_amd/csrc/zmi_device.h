// Device-side types shared by the gfx950 kernels and the host dispatch code:
// the packed-weight blob, the epilogue descriptor and the per-expert table.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/zmi_lowoha.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------
// Packed weight blob ("mem_format_b == 'r'").
//
//   [ header 256 B ][ colsum int32[N_pad] ][ tiles ]
//
// tiles is an array [N_pad/32][K_pad/32] of 1 KiB fragments.  Fragment (nb,kb)
// holds weight rows kb*32..+31 of columns nb*32..+31 exactly as one wavefront
// feeds them to v_mfma_i32_32x32x32_i8 as the B operand: lane i owns bytes
// [16i, 16i+16) = B[kb*32 + (i/32)*16 + b][nb*32 + i%32], b = 0..15.  A
// wavefront therefore loads a fragment with one fully coalesced 16-byte-per-lane
// load and needs no LDS staging or shuffles for B.  Fragments of one column
// block are contiguous along K, so every wavefront streams contiguous memory.
// Padding rows / columns are zero.  colsum[n] = sum_k B[k][n] feeds the source
// zero-point compensation in the GEMM epilogue.
// ---------------------------------------------------------------------------
#define ZMI_BLOB_MAGIC 0x31424f4c42494d5aULL  // "ZMIBLOB1"
#define ZMI_BLOB_HEADER_BYTES 256
#define ZMI_KPAD 128
#define ZMI_NPAD 64
// Bytes skipped between consecutive column blocks.  Without it the streams of
// all column blocks at the same K offset sit a power of two apart and land on
// the same L2 / memory channel.
#ifndef ZMI_NB_SKEW
#define ZMI_NB_SKEW 0
#endif

struct ZmiBlobHeader {
  uint64_t magic;
  uint32_t version;
  uint32_t flags;
  int64_t K, N, K_pad, N_pad;
  int64_t colsum_off, tiles_off, total_bytes;
  int32_t src_dtype, sym_group_size;
};

static inline __host__ __device__ int64_t zmi_round_up(int64_t x, int64_t m) {
  return (x + m - 1) / m * m;
}
static inline __host__ __device__ int64_t zmi_blob_kpad(int64_t K) { return zmi_round_up(K, ZMI_KPAD); }
static inline __host__ __device__ int64_t zmi_blob_npad(int64_t N) { return zmi_round_up(N, ZMI_NPAD); }
static inline __host__ __device__ int64_t zmi_blob_colsum_off() { return ZMI_BLOB_HEADER_BYTES; }
static inline __host__ __device__ int64_t zmi_blob_tiles_off(int64_t N) {
  return zmi_round_up(ZMI_BLOB_HEADER_BYTES + zmi_blob_npad(N) * 4, 256);
}
// distance in bytes between the fragment streams of consecutive column blocks
static inline __host__ __device__ int64_t zmi_blob_nb_stride(int64_t K) {
  return zmi_blob_kpad(K) * 32 + ZMI_NB_SKEW;
}
// 4-bit tiles (W4A8 decode shapes): per 32-column block one 2 KiB piece per pair of 64-k chunks
static inline __host__ __device__ int64_t zmi_s4_nb_stride(int64_t K) { return zmi_blob_kpad(K) * 16 + ZMI_NB_SKEW; }
static inline __host__ __device__ int64_t zmi_s4_tiles_bytes(int64_t K, int64_t N) {
  return zmi_s4_nb_stride(K) * (zmi_blob_npad(N) / 32);
}
// 4-bit tiles of the weight-only path (k_woq.hip): [ceil(N/32)][ceil(K/64)] pieces of 1 KiB
static inline __host__ __device__ int64_t zmi_woq_tiles_bytes(int64_t K, int64_t N) {
  return ((N + 31) / 32) * ((K + 63) / 64) * 1024;
}
static inline __host__ __device__ int64_t zmi_blob_bytes(int64_t K, int64_t N) {
  return zmi_blob_tiles_off(N) + zmi_blob_nb_stride(K) * (zmi_blob_npad(N) / 32);
}

// Activations for the large-M kernel use the same fragment order: an array
// [ceil(M/32)][K_pad/32] of 1 KiB fragments, fragment (mb, kb) lane i bytes
// [16i, 16i+16) = A[mb*32 + i%32][kb*32 + (i/32)*16 + b].  Byte offset of A[r][k]:
static inline __host__ __device__ int64_t zmi_afrag_off(int64_t r, int64_t k, int64_t k_pad) {
  return ((r >> 5) * (k_pad >> 5) + (k >> 5)) * 1024 + ((((k >> 4) & 1) << 5) + (r & 31)) * 16 + (k & 15);
}
static inline __host__ __device__ int64_t zmi_afrag_bytes(int64_t M, int64_t K) {
  return zmi_round_up(M, 32) * zmi_blob_kpad(K);
}

// ---------------------------------------------------------------------------
// Epilogue: everything between the s32 accumulator and the stored element.
//   y = float(acc + comp[n])            comp[n] = -src_zp * colsum[n], in s32
//   (alpha != 1 or beta != 0: y = float(acc)*alpha + beta*C + float(comp[n]))
//   y *= src_scale (tensor or row m);  y *= wei_scale[n % len];  y += bias[n]
//   post-ops in order;  y = y * dst_scale + dst_zp;  store as dst dtype.
// ---------------------------------------------------------------------------
#define ZMI_MAX_PO 4

struct ZmiPostOp {
  int32_t type;        // enum zmi_post_op_type
  int32_t dtype;       // binary operand dtype
  const void *buff;    // binary operand
  int32_t ld;          // leading dimension of a {M,N} operand
  int32_t rowb;        // 1: operand is {1,N} and broadcast over rows
  float alpha, beta;   // clip bounds
};

// (ZMI_SS_GROUP_PTR: one scale per row and K group, {M, G} row-major; only the per-group kernel reads it)
enum { ZMI_SS_NONE = 0, ZMI_SS_VALUE = 1, ZMI_SS_TENSOR_PTR = 2, ZMI_SS_TOKEN_PTR = 3, ZMI_SS_GROUP_PTR = 4 };

// Straight-line epilogue variants: alpha == 1, beta == 0, no destination
// quantization, bf16 or f32 destination, at most one element-wise post-op of
// the named type.  Everything else runs the generic interpreter.
enum { ZMI_EK_GENERIC = 0, ZMI_EK_NONE = 1, ZMI_EK_SWISH = 2, ZMI_EK_GELU_TANH = 3, ZMI_EK_RELU = 4 };

struct ZmiEpilogue {
  int32_t src_scale_mode;  // ZMI_SS_*
  int32_t src_scale_dt;
  int32_t wei_scale_mode;  // 0: none; 1: per tensor; 2: per channel (indexed by n); 3: per K group and channel, {G, N}
  int32_t wei_scale_dt;
  int32_t has_zp;
  int32_t bias_dt;
  float alpha, beta;
  int32_t n_po;
  ZmiPostOp po[ZMI_MAX_PO];
  int32_t has_dst_q;
  const void *dst_scale_ptr;
  int32_t dst_scale_dt;
  float dst_scale_val;
  const void *dst_zp_ptr;
  int32_t dst_zp_dt;
  float dst_zp_val;
  int32_t dst_dt;
  int32_t gated_act;      // enum zmi_gated_act; != 0: columns are [gate | up] halves
  int32_t fast_kind;      // ZMI_EK_*: straight-line epilogue variant, 0 = generic interpreter
  int32_t n_groups;       // > 0: per-group source and weight scales over G = n_groups slices of K
};

// One GEMM problem: C[M,N] = epilogue(A[M,K] x blob), with the operands the
// epilogue reads per problem.  The grouped kernels take an array of these in
// device memory, one per expert; the epilogue descriptor is shared.
struct ZmiProblem {
  const void *A;          // u8 / s8, row-major, K contiguous
  int64_t lda;
  const uint8_t *blob;    // packed weights
  void *dst;
  int64_t ldc;
  int32_t M, N, K;
  int32_t a_is_u8;
  const void *src_scale_ptr;   // ZMI_SS_TENSOR_PTR / ZMI_SS_TOKEN_PTR
  const void *wei_scale_ptr;   // null with mode 1: wei_scale_val is used
  const int32_t *src_zp_ptr;   // null: src_zp_val is used
  const void *bias;
  float src_scale_val;         // ZMI_SS_VALUE
  float wei_scale_val;
  int32_t src_zp_val;
  // weight zero-point (per tensor): the kernels see it as one int32 per row that joins the accumulator's
  // compensation, row_comp[m] = -wei_zp * sum_k A[m, k] + src_zp * wei_zp * K (reference: the 2-D compensation of
  // cache_or_compute_zp_compensation, lowoha_operators/matmul/lru_cache/lowoha_cache.hpp:151-232, without its
  // column term, which is the blob's colsum).  Only the kernels that finish elements through zmi_finish_element
  // read it; the API keeps calls with a weight zero-point on those.
  const int32_t *row_comp;     // null: no weight zero-point
  int32_t wei_zp_val;          // host-side planning only (value, or a device pointer and its dtype)
  int32_t wei_zp_dt;
  const void *wei_zp_ptr;
};

#ifdef __HIPCC__
// A pointer that is known to address global memory.  Pointers that reach a kernel
// inside a problem table are generic to the compiler, and accesses through them
// become flat instructions, which share a counter with LDS reads: a wait for an
// LDS read then also waits for every store in flight.
#define ZMI_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ ZMI_GLOBAL T *zmi_global(const void *p) {
  return (ZMI_GLOBAL T *)(uintptr_t)p;
}

// ------------------------------------------------------------------ device math
__device__ __forceinline__ float zmi_bf16_to_f32(uint16_t h) {
  return __uint_as_float(((uint32_t)h) << 16);
}

// Store rounding of the matmul output and the gated activation: normals round
// to nearest even, zero and subnormal inputs give a signed zero, NaN keeps its
// high half with the quiet bit set (reference: bfloat16_t(float),
// zendnnl/src/common/bfloat16.cpp:27-51).
__device__ __forceinline__ uint16_t zmi_f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t e = u & 0x7f800000u;
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  if (e == 0) r = (u >> 16) & 0x8000u;
  if (e == 0x7f800000u) r = (u >> 16) | ((u & 0x007fffffu) ? 0x40u : 0u);
  return (uint16_t)r;
}

// Plain round-to-nearest-even bit trick used by the MoE weighted reduce
// (reference: bfloat16_t::f32_to_bf16_val, zendnnl/src/common/bfloat16.cpp:69-79).
__device__ __forceinline__ uint16_t zmi_f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// half precision <-> f32 (reference: float16_t, common/float16.cpp:77-205).  Widening is exact (the hardware
// conversion).  Narrowing rounds to nearest even like the hardware does, except where the reference's own code does
// something else: f32 subnormals become signed zeros whatever the mode, NaN keeps its top mantissa bits and is made
// quiet, and a half-subnormal result whose rounding carries into the exponent (magnitudes in [2^-14 - 2^-25, 2^-14))
// is stored as a signed zero, because the reference masks it with the mantissa field.  Integer code, so that the
// result does not depend on the wavefront's denormal mode.
__device__ __forceinline__ float zmi_f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ uint16_t zmi_f32_to_f16(float f) {
  const uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const uint32_t e = (u >> 23) & 0xffu, m = u & 0x7fffffu;
  if (e == 0) return (uint16_t)sign;
  if (e == 255) return (uint16_t)(m ? (sign | 0x7c00u | (m >> 13) | 0x200u) : (sign | 0x7c00u));
  int he = (int)e - 112;
  if (he >= 31) return (uint16_t)(sign | 0x7c00u);
  if (he <= 0) {
    if (he < -10) return (uint16_t)sign;
    const uint32_t full = m | 0x800000u;
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

__device__ __forceinline__ float zmi_ld_f32(const void *p, int dt, int64_t i) {
  switch (dt) {
  case ZMI_DT_BF16: return zmi_bf16_to_f32(((const uint16_t *)p)[i]);
  case ZMI_DT_F16: return zmi_f16_to_f32(((const uint16_t *)p)[i]);
  case ZMI_DT_S32: return (float)((const int32_t *)p)[i];
  case ZMI_DT_S8: return (float)((const int8_t *)p)[i];
  case ZMI_DT_U8: return (float)((const uint8_t *)p)[i];
  default: return ((const float *)p)[i];
  }
}

// Per-token quantization of one element: (int8) rint(v / scale) with the division correctly
// rounded, the reference's "true divide" (scalar twin: dynamic_per_token_ref_kernel.cpp:70-96);
// non-finite inputs give 0.  The division is what the quantization kernels spend their time
// on, so it is replaced by v * inv (inv = 1 / scale, correctly rounded, once per row) wherever
// that provably rounds to the same integer: |v * inv - v / scale| <= 127 * 2^-23 < 1.6e-5 and
// the rounded quotient is within 127 * 2^-24 of the true one, so the two can round to
// different integers only when v * inv lies within 3.8e-5 of a half-integer; those elements
// (about one in a thousand) take the division.
__device__ __forceinline__ int8_t zmi_quant_elem(float v, float scale, float inv) {
  const bool finite = (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u;
  const float x = finite ? v : 0.0f;
  const float t = __fmul_rn(x, inv);
  float r = rintf(t);
  if (fabsf(t - r) > 0.4999f) r = rintf(__fdiv_rn(x, scale));
  return (int8_t)(int32_t)r;
}

// exp(x) from the hardware exp2 with a split product x*log2(e) so the argument
// error does not grow with |x|; about 2 ulp over the range the activations use.
__device__ __forceinline__ float zmi_expf(float x) {
  const float l2e_hi = 1.44269502162933349609375f;
  const float l2e_lo = 1.925963033500011e-08f;
  float t = x * l2e_hi;
  float r = __builtin_fmaf(x, l2e_hi, -t) + x * l2e_lo;   // rounding error of t plus the low part
  float e = __builtin_amdgcn_exp2f(t);
  // an overflowed e must stay +inf (inf * negative correction + inf would be NaN), and exp(-inf) is 0
  // (there t = -inf makes the correction term NaN)
  return (e == __builtin_inff() || e == 0.0f) ? e : __builtin_fmaf(e, r * 0.693147182464599609375f, e);
}

__device__ __forceinline__ float zmi_sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + zmi_expf(-x));
}

// Element-wise post-ops (reference definitions:
// zendnnl/src/operators/matmul/matmul_ref_kernel.cpp:694-761).
__device__ __forceinline__ float zmi_eltwise(int type, float x, float alpha, float beta) {
  switch (type) {
  case ZMI_PO_RELU: return x > 0.0f ? x : 0.0f;
  case ZMI_PO_LEAKY_RELU: return x > 0.0f ? x : 0.01f * x;
  case ZMI_PO_GELU_TANH: {
    // reference: v = tanhf(u); 0.5 * x * (1.0f + v), u = sqrt(2/pi) x (1 + 0.044715 x^2).
    // 1 + tanh(u) == 2 sigmoid(2u) is evaluated accurately, then rounded through
    // the float value of tanh (v) exactly as the reference's "1.0f + v" sees it,
    // so the negative tail cancels onto the same 2^-24 grid.
    float u = 0.79788458347320556640625f * x * (1.0f + 0.044715f * x * x);
    float v = 2.0f * zmi_sigmoid(2.0f * u) - 1.0f;
    return (0.5f * x) * (1.0f + v);
  }
  case ZMI_PO_GELU_ERF: return 0.5f * x * (1.0f + erff(x * 0.707106769084930419921875f));
  case ZMI_PO_SIGMOID: return zmi_sigmoid(x);
  case ZMI_PO_SWISH: return x * zmi_sigmoid(x);
  case ZMI_PO_TANH: return tanhf(x);
  case ZMI_PO_CLIP: { x = x > alpha ? x : alpha; return x > beta ? beta : x; }
  // (the remaining element-wise types of the reference's kernel, matmul_ref_kernel.cpp:694-751)
  case ZMI_PO_ELU: return x > 0.0f ? x : alpha * (zmi_expf(x) - 1.0f);
  case ZMI_PO_SQUARE: return x * x;
  case ZMI_PO_ABS: return x > 0.0f ? x : -x;
  case ZMI_PO_SQRT: return __fsqrt_rn(x);
  case ZMI_PO_EXP: return zmi_expf(x);
  case ZMI_PO_LOG: return logf(x);
  // mish_fwd, matmul_ref_kernel.cpp:755-760: x * tanh(softplus(x)), softplus = max(x, 0) + log1p(exp(-|x|))
  case ZMI_PO_MISH: return x * tanhf(fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))));
  default: return x;
  }
}

// Gated activations (reference: group_matmul/group_matmul_moe_act.cpp:88-154).
__device__ __forceinline__ float zmi_gated(int act, float g, float u) {
  if (act == ZMI_ACT_SILU_AND_MUL) return (g * zmi_sigmoid(g)) * u;
  if (act == ZMI_ACT_GELU_AND_MUL) return (g * 0.5f * (1.0f + erff(g * 0.7071067811865476f))) * u;
  // swiglu_oai: clamp to [-7, 7], (1 + u) * g * sigmoid(1.702 g)
  g = fmaxf(-7.0f, fminf(g, 7.0f));
  u = fmaxf(-7.0f, fminf(u, 7.0f));
  return (1.0f + u) * g * zmi_sigmoid(g * 1.702f);
}

// Per-column constants of the epilogue, loaded once per lane.
struct ZmiColCtx {
  float wscale;
  float bias;
  int32_t comp;    // everything added to the MFMA accumulator: u8 shift and zero-point compensation
  int32_t shift;   // the u8 part alone (128 * colsum): accumulator + shift is the true sum of a*w
};

__device__ __forceinline__ ZmiColCtx zmi_col_ctx(const ZmiEpilogue &e, const ZmiProblem &p,
                                                 const int32_t *colsum, int n, int N) {
  ZmiColCtx c;
  c.wscale = 1.0f;
  c.bias = 0.0f;
  c.comp = 0;
  c.shift = 0;
  if (n < N) {
    if (e.wei_scale_mode) {
      c.wscale = p.wei_scale_ptr ? zmi_ld_f32(p.wei_scale_ptr, e.wei_scale_dt, e.wei_scale_mode == 1 ? 0 : n)
                                 : p.wei_scale_val;
    }
    if (p.bias) c.bias = zmi_ld_f32(p.bias, e.bias_dt, n);
    // u8 activations enter the MFMA as (a - 128): add 128 * colsum back, then
    // subtract zp * colsum; both in s32
    int32_t k = p.a_is_u8 ? 128 : 0;
    if (e.has_zp) k -= p.src_zp_ptr ? *p.src_zp_ptr : p.src_zp_val;
    if (k) c.comp = k * colsum[n];
    if (p.a_is_u8) c.shift = 128 * colsum[n];
  }
  return c;
}

// ---- the same constants, requested early and decoded late ------------------------------------
// A kernel that must not wait in its prologue fetches the aligned 32-bit word that holds an
// element (an aligned word never leaves the element's page) and picks the element out of it
// when the epilogue starts.  The request is one instruction whatever the element type is and
// is issued whether or not the array exists (then from `fallback`, any readable word), so
// the requests form a branch-free run of loads that nothing waits on.
__device__ __forceinline__ int zmi_log2_size(int dt) {
  return dt == ZMI_DT_BF16 ? 1 : (dt == ZMI_DT_S8 || dt == ZMI_DT_U8) ? 0 : 2;
}
__device__ __forceinline__ uint32_t zmi_ld_word(const void *p, const void *fallback, int dt, int64_t i) {
  const uintptr_t addr = p ? (uintptr_t)p + ((uintptr_t)i << zmi_log2_size(dt)) : (uintptr_t)fallback;
  return *(ZMI_GLOBAL const uint32_t *)(addr & ~(uintptr_t)3);
}
__device__ __forceinline__ float zmi_word_f32(uint32_t word, const void *p, int dt, int64_t i) {
  const uintptr_t addr = (uintptr_t)p + ((uintptr_t)i << zmi_log2_size(dt));
  const uint32_t raw = word >> ((uint32_t)(addr & 3) * 8);
  switch (dt) {
  case ZMI_DT_BF16: return __uint_as_float(raw << 16);
  case ZMI_DT_S32: return (float)(int32_t)raw;
  case ZMI_DT_S8: return (float)(int8_t)raw;
  case ZMI_DT_U8: return (float)(uint8_t)raw;
  default: return __uint_as_float(raw);
  }
}

struct ZmiColRaw {
  uint32_t wscale, bias;
  int32_t colsum;
};
// n_ok: a column index that exists (the caller clamps); the decode step below knows whether
// the lane's real column does.
__device__ __forceinline__ ZmiColRaw zmi_col_raw(const ZmiEpilogue &e, const ZmiProblem &p, const int32_t *colsum,
                                                 int n_ok) {
  ZmiColRaw r;
  r.wscale = zmi_ld_word(p.wei_scale_ptr, colsum, e.wei_scale_dt, e.wei_scale_mode == 1 ? 0 : n_ok);
  r.bias = zmi_ld_word(p.bias, colsum, e.bias_dt, n_ok);
  r.colsum = *(ZMI_GLOBAL const int32_t *)(uintptr_t)(colsum + n_ok);
  return r;
}
__device__ __forceinline__ int32_t zmi_zp_raw(const ZmiProblem &p, const int32_t *colsum) {
  return *(ZMI_GLOBAL const int32_t *)(uintptr_t)(p.src_zp_ptr ? p.src_zp_ptr : colsum);
}
// Same result as zmi_col_ctx(e, p, colsum, n, N) from the words fetched for column n_ok.
__device__ __forceinline__ ZmiColCtx zmi_col_ctx_raw(const ZmiEpilogue &e, const ZmiProblem &p, const ZmiColRaw &r,
                                                     int32_t zp_raw, int n, int n_ok, int N) {
  ZmiColCtx c;
  c.wscale = 1.0f;
  c.bias = 0.0f;
  c.comp = 0;
  c.shift = 0;
  if (n < N) {
    if (e.wei_scale_mode) {
      c.wscale = p.wei_scale_ptr ? zmi_word_f32(r.wscale, p.wei_scale_ptr, e.wei_scale_dt, e.wei_scale_mode == 1 ? 0 : n_ok)
                                 : p.wei_scale_val;
    }
    if (p.bias) c.bias = zmi_word_f32(r.bias, p.bias, e.bias_dt, n_ok);
    int32_t k = p.a_is_u8 ? 128 : 0;
    if (e.has_zp) k -= p.src_zp_ptr ? zp_raw : p.src_zp_val;
    if (k) c.comp = k * r.colsum;
    if (p.a_is_u8) c.shift = 128 * r.colsum;
  }
  return c;
}
__device__ __forceinline__ uint32_t zmi_row_scale_raw(const ZmiEpilogue &e, const ZmiProblem &p, const void *fallback,
                                                      int m_ok) {
  const bool have = e.src_scale_mode == ZMI_SS_TENSOR_PTR || e.src_scale_mode == ZMI_SS_TOKEN_PTR;
  return zmi_ld_word(have ? p.src_scale_ptr : nullptr, fallback, e.src_scale_dt,
                     e.src_scale_mode == ZMI_SS_TOKEN_PTR ? m_ok : 0);
}
__device__ __forceinline__ float zmi_row_scale_from_raw(const ZmiEpilogue &e, const ZmiProblem &p, uint32_t raw, int m_ok) {
  switch (e.src_scale_mode) {
  case ZMI_SS_VALUE: return p.src_scale_val;
  case ZMI_SS_TENSOR_PTR: return zmi_word_f32(raw, p.src_scale_ptr, e.src_scale_dt, 0);
  case ZMI_SS_TOKEN_PTR: return zmi_word_f32(raw, p.src_scale_ptr, e.src_scale_dt, m_ok);
  default: return 1.0f;
  }
}

__device__ __forceinline__ float zmi_row_scale(const ZmiEpilogue &e, const ZmiProblem &p, int m) {
  switch (e.src_scale_mode) {
  case ZMI_SS_VALUE: return p.src_scale_val;
  case ZMI_SS_TENSOR_PTR: return zmi_ld_f32(p.src_scale_ptr, e.src_scale_dt, 0);
  case ZMI_SS_TOKEN_PTR: return zmi_ld_f32(p.src_scale_ptr, e.src_scale_dt, m);
  default: return 1.0f;
  }
}

// What follows the scaled accumulator: bias, post-ops in order, destination quantization
// (reference: operators/matmul/matmul_ref_kernel.cpp:1049-1053 and the post-op loop after it).
// The per-group kernel enters here with its f32 sum of group terms.
__device__ __forceinline__ float zmi_epilogue_tail(const ZmiEpilogue &e, float y, float bias, int m, int n) {
  y = __fadd_rn(y, bias);
  for (int i = 0; i < e.n_po; ++i) {
    const ZmiPostOp &po = e.po[i];
    if (po.type == ZMI_PO_BINARY_ADD || po.type == ZMI_PO_BINARY_MUL) {
      float t = zmi_ld_f32(po.buff, po.dtype, po.rowb ? (int64_t)n : (int64_t)m * po.ld + n);
      y = po.type == ZMI_PO_BINARY_ADD ? __fadd_rn(y, t) : __fmul_rn(y, t);
    } else {
      y = zmi_eltwise(po.type, y, po.alpha, po.beta);
    }
  }
  if (e.has_dst_q) {
    float ds = e.dst_scale_ptr ? zmi_ld_f32(e.dst_scale_ptr, e.dst_scale_dt, 0) : e.dst_scale_val;
    float dz = e.dst_zp_ptr ? zmi_ld_f32(e.dst_zp_ptr, e.dst_zp_dt, 0) : e.dst_zp_val;
    y = __fadd_rn(__fmul_rn(y, ds), dz);
  }
  return y;
}

// acc -> f32 value before the store conversion (all steps separately rounded,
// in the reference's order).
__device__ __forceinline__ float zmi_epilogue_value(const ZmiEpilogue &e, int32_t acc, const ZmiColCtx &c,
                                                    float rscale, int m, int n, const void *dst,
                                                    int64_t ldc) {
  float y;
  if (e.alpha == 1.0f && e.beta == 0.0f) {
    y = (float)(acc + c.comp);
  } else {
    // the reference scales and accumulates before it adds the compensation
    y = (float)(acc + c.shift);
    if (e.alpha != 1.0f) y = __fmul_rn(y, e.alpha);
    if (e.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(dst, e.dst_dt, (int64_t)m * ldc + n), e.beta));
    if (e.has_zp) y = __fadd_rn(y, (float)(c.comp - c.shift));
  }
  if (e.src_scale_mode) y = __fmul_rn(y, rscale);
  if (e.wei_scale_mode) y = __fmul_rn(y, c.wscale);
  return zmi_epilogue_tail(e, y, c.bias, m, n);
}

// Straight-line form of zmi_epilogue_value + zmi_store for the ZMI_EK_* variants:
// same operations in the same order, no interpretation in the inner loop.
template <int EK>
__device__ __forceinline__ float zmi_fast_value(int32_t acc, const ZmiColCtx &c, float rscale, bool has_rs,
                                                bool has_ws, bool has_bias) {
  float y = (float)(acc + c.comp);
  if (has_rs) y = __fmul_rn(y, rscale);
  if (has_ws) y = __fmul_rn(y, c.wscale);
  if (has_bias) y = __fadd_rn(y, c.bias);
  if (EK == ZMI_EK_SWISH) y = zmi_eltwise(ZMI_PO_SWISH, y, 0.0f, 0.0f);
  if (EK == ZMI_EK_GELU_TANH) y = zmi_eltwise(ZMI_PO_GELU_TANH, y, 0.0f, 0.0f);
  if (EK == ZMI_EK_RELU) y = zmi_eltwise(ZMI_PO_RELU, y, 0.0f, 0.0f);
  return y;
}

template <bool BF16>
__device__ __forceinline__ void zmi_fast_store(void *dst, int64_t i, float y) {
  if (BF16) ((uint16_t *)dst)[i] = zmi_f32_to_bf16(y);
  else ((float *)dst)[i] = y;
}

// ---- bf16-destination forms used by the large-M kernel ---------------------------
// Two f32 values -> packed bf16 with the hardware conversion.  With the
// wavefront's f32 denormal mode set to flush (zmi_set_f32_flush) it is
// bit-identical to zmi_f32_to_bf16 on every input: round to nearest even,
// zero / subnormal -> signed zero, NaN quieted with its payload kept.
typedef __bf16 zmi_bf16x2 __attribute__((ext_vector_type(2)));
typedef float zmi_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t zmi_pack_bf16(float lo, float hi) {
  zmi_f32x2 v = {lo, hi};
  zmi_bf16x2 r = __builtin_convertvector(v, zmi_bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}
// MODE register, bits [5:4]: single-precision denormal mode, 0 = flush inputs and results
__device__ __forceinline__ void zmi_set_f32_flush() { __builtin_amdgcn_s_setreg(1 | (4 << 6) | (1 << 11), 0); }

// Activations evaluated for a bf16 store: plain hardware exp2 / reciprocal, fused
// multiply-adds.  The result differs from the separately rounded f32 form by
// about 1e-6 relative, 1/2000 of half a bf16 unit in the last place.
template <int EK>
__device__ __forceinline__ float zmi_act_bf16(float x) {
  if (EK == ZMI_EK_RELU) return x > 0.0f ? x : 0.0f;
  if (EK == ZMI_EK_SWISH) {
    const float e = __builtin_amdgcn_exp2f(x * -1.44269502162933349609375f);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
  }
  if (EK == ZMI_EK_GELU_TANH) {
    // exp(-2u) = exp2(x * (c0 + c1 x^2)), u = sqrt(2/pi) x (1 + 0.044715 x^2); then the
    // reference's "0.5 x (1.0f + tanhf(u))" with tanh(u) = 2 sigmoid(2u) - 1 rounded to float
    const float c0 = -2.0f * 1.44269502162933349609375f * 0.79788458347320556640625f;
    const float c1 = c0 * 0.044715f;
    const float a = x * __builtin_fmaf(c1, x * x, c0);
    const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a));
    const float v = __builtin_fmaf(2.0f, s, -1.0f);
    return (0.5f * x) * (1.0f + v);
  }
  return x;
}

// A straight-line epilogue kind applied to a finished f32 value that goes to a bf16 store (callers: the kernels
// whose value is already the scaled sum plus bias, with the wavefront in the flush mode above).
__device__ __forceinline__ float zmi_act_bf16_kind(int fast_kind, float y) {
  switch (fast_kind) {
  case ZMI_EK_SWISH: return zmi_act_bf16<ZMI_EK_SWISH>(y);
  case ZMI_EK_GELU_TANH: return zmi_act_bf16<ZMI_EK_GELU_TANH>(y);
  case ZMI_EK_RELU: return zmi_act_bf16<ZMI_EK_RELU>(y);
  default: return y;
  }
}

// Store conversions (reference: store_output,
// zendnnl/src/operators/matmul/matmul_ref_kernel.cpp:154-254).
__device__ __forceinline__ void zmi_store(void *dst, int dt, int64_t i, float y) {
  switch (dt) {
  case ZMI_DT_BF16: ((uint16_t *)dst)[i] = zmi_f32_to_bf16(y); break;
  case ZMI_DT_F16: ((uint16_t *)dst)[i] = zmi_f32_to_f16(y); break;
  case ZMI_DT_S32: {
    float v = fminf(fmaxf(y, -2147483648.0f), 2147483648.0f);
    ((int32_t *)dst)[i] = v >= 2147483648.0f ? 2147483647 : (int32_t)rintf(v);
    break;
  }
  case ZMI_DT_S8: ((int8_t *)dst)[i] = (int8_t)rintf(fminf(fmaxf(y, -128.0f), 127.0f)); break;
  case ZMI_DT_U8: ((uint8_t *)dst)[i] = (uint8_t)rintf(fminf(fmaxf(y, 0.0f), 255.0f)); break;
  default: ((float *)dst)[i] = y; break;
  }
}

// True when the s32 accumulator (plus compensation) is the stored value: s32
// destination, no scales, no bias, no post-ops.  The integer is then written
// as is, which is exact where a float round trip would not be.
__device__ __forceinline__ bool zmi_epilogue_is_raw_s32(const ZmiEpilogue &e, const void *bias) {
  return e.dst_dt == ZMI_DT_S32 && !e.src_scale_mode && !e.wei_scale_mode && !bias && !e.n_po &&
         !e.has_dst_q && e.alpha == 1.0f && e.beta == 0.0f;
}

// One finished output element: accumulator -> epilogue -> store at dst[m * ldc + n].  The
// kernels that produce one element per thread (decode, the K-slice reduction) end here.
__device__ __forceinline__ void zmi_finish_element(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiColCtx &c_in,
                                                   float rs, int32_t s, int m, int n) {
  ZmiColCtx c = c_in;
  if (p.row_comp) c.comp += p.row_comp[m];   // (a weight zero-point: see ZmiProblem)
  const bool has_rs = epi.src_scale_mode != ZMI_SS_NONE, has_ws = epi.wei_scale_mode != 0;
  const bool has_bias = p.bias != nullptr;
  const int64_t o = (int64_t)m * p.ldc + n;
  const bool bf = epi.dst_dt == ZMI_DT_BF16;
  switch (epi.fast_kind) {
  case ZMI_EK_NONE: {
    const float y = zmi_fast_value<ZMI_EK_NONE>(s, c, rs, has_rs, has_ws, has_bias);
    if (bf) zmi_fast_store<true>(p.dst, o, y); else zmi_fast_store<false>(p.dst, o, y);
    break;
  }
  case ZMI_EK_SWISH: {
    const float y = zmi_fast_value<ZMI_EK_SWISH>(s, c, rs, has_rs, has_ws, has_bias);
    if (bf) zmi_fast_store<true>(p.dst, o, y); else zmi_fast_store<false>(p.dst, o, y);
    break;
  }
  case ZMI_EK_GELU_TANH: {
    const float y = zmi_fast_value<ZMI_EK_GELU_TANH>(s, c, rs, has_rs, has_ws, has_bias);
    if (bf) zmi_fast_store<true>(p.dst, o, y); else zmi_fast_store<false>(p.dst, o, y);
    break;
  }
  default:
    if (zmi_epilogue_is_raw_s32(epi, p.bias)) ((int32_t *)p.dst)[o] = s + c.comp;
    else zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_value(epi, s, c, rs, m, n, p.dst, p.ldc));
  }
}
// ---- one element finished with the arithmetic of the MFMA-bound kernel's epilogue (k_ring.hip) ----
// The kernels that take part of a grouped launch beside it end here, so that a result does not depend on which
// kernel computed it: bf16 destinations with a straight-line epilogue use the separately rounded scale chain with
// absent scales as 1 and an absent bias as -0, the hardware exponential / reciprocal forms of the activations and the
// hardware bf16 conversion under the flush-denormals mode; f32 destinations the conditional chain of zmi_fast_value;
// everything else the interpreter.
__device__ __forceinline__ float zmi_ring_chain(int32_t acc, const ZmiColCtx &c, float rs, bool has_bias) {
  return __fadd_rn(__fmul_rn(__fmul_rn((float)(acc + c.comp), rs), c.wscale), has_bias ? c.bias : -0.0f);
}

__device__ __forceinline__ void zmi_finish_element_ring(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiColCtx &c,
                                                        float rs, int32_t s, int m, int n) {
  const bool has_rs = epi.src_scale_mode != ZMI_SS_NONE, has_ws = epi.wei_scale_mode != 0;
  const bool has_bias = p.bias != nullptr;
  const int64_t o = (int64_t)m * p.ldc + n;
  if (epi.fast_kind != ZMI_EK_GENERIC && epi.dst_dt == ZMI_DT_BF16) {
    zmi_set_f32_flush();
    float y = zmi_ring_chain(s, c, rs, has_bias);
    switch (epi.fast_kind) {
    case ZMI_EK_SWISH: y = zmi_act_bf16<ZMI_EK_SWISH>(y); break;
    case ZMI_EK_GELU_TANH: y = zmi_act_bf16<ZMI_EK_GELU_TANH>(y); break;
    case ZMI_EK_RELU: y = zmi_act_bf16<ZMI_EK_RELU>(y); break;
    default: break;
    }
    zmi_global<uint16_t>(p.dst)[o] = (uint16_t)zmi_pack_bf16(y, 0.0f);
    return;
  }
  if (epi.fast_kind != ZMI_EK_GENERIC && epi.dst_dt == ZMI_DT_F32) {
    float y;
    switch (epi.fast_kind) {
    case ZMI_EK_SWISH: y = zmi_fast_value<ZMI_EK_SWISH>(s, c, rs, has_rs, has_ws, has_bias); break;
    case ZMI_EK_GELU_TANH: y = zmi_fast_value<ZMI_EK_GELU_TANH>(s, c, rs, has_rs, has_ws, has_bias); break;
    case ZMI_EK_RELU: y = zmi_fast_value<ZMI_EK_RELU>(s, c, rs, has_rs, has_ws, has_bias); break;
    default: y = zmi_fast_value<ZMI_EK_NONE>(s, c, rs, has_rs, has_ws, has_bias); break;
    }
    zmi_global<float>(p.dst)[o] = y;
    return;
  }
  if (zmi_epilogue_is_raw_s32(epi, p.bias)) ((int32_t *)p.dst)[o] = s + c.comp;
  else zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_value(epi, s, c, rs, m, n, p.dst, p.ldc));
}

// Gated pair (gate column n, up column n + N/2) -> output column n; straight-line epilogues only (no element-wise
// post-op in front of the activation), bf16 or f32 destination.
__device__ __forceinline__ void zmi_finish_gated_ring(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiColCtx &cg,
                                                      const ZmiColCtx &cu, float rs, int32_t sg, int32_t su, int m, int n) {
  const bool has_rs = epi.src_scale_mode != ZMI_SS_NONE, has_ws = epi.wei_scale_mode != 0;
  const bool has_bias = p.bias != nullptr;
  const int64_t o = (int64_t)m * p.ldc + n;
  if (epi.dst_dt == ZMI_DT_BF16) {
    zmi_set_f32_flush();
    const float y0 = zmi_ring_chain(sg, cg, rs, has_bias), y1 = zmi_ring_chain(su, cu, rs, has_bias);
    // gate and up are rounded to bf16 first, as when the activation reads a stored GEMM result
    const uint32_t gu = zmi_pack_bf16(y0, y1);
    const float g = __uint_as_float(gu << 16), u = __uint_as_float(gu & 0xffff0000u);
    const float z = epi.gated_act == ZMI_ACT_SILU_AND_MUL ? zmi_act_bf16<ZMI_EK_SWISH>(g) * u : zmi_gated(epi.gated_act, g, u);
    zmi_global<uint16_t>(p.dst)[o] = (uint16_t)zmi_pack_bf16(z, 0.0f);
  } else {
    const float y0 = zmi_fast_value<ZMI_EK_NONE>(sg, cg, rs, has_rs, has_ws, has_bias);
    const float y1 = zmi_fast_value<ZMI_EK_NONE>(su, cu, rs, has_rs, has_ws, has_bias);
    zmi_global<float>(p.dst)[o] = zmi_gated(epi.gated_act, y0, y1);
  }
}
#endif  // __HIPCC__
