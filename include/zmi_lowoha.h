/*
 * zmi_lowoha.h -- C ABI of the MI355X (gfx950) implementation of ZenDNN's
 * LowOHA quantized-matmul path.
 *
 * One shared library, libzmi_lowoha.so, exports exactly the entry points a
 * binding for this path needs.  Every function takes plain C types: pointers,
 * sizes and the flat structs below.  There are no C++ or torch types in any
 * signature, so the same header serves cgo / JNI / ctypes / a C++ adapter.
 *
 * Pointer domain
 *   Every *data* pointer (src, weight, bias, dst, scale / zero-point buffers,
 *   post-op operands, row_ptrs targets, prepack blobs) must be dereferenceable
 *   by the GPU: hipMalloc, hipMallocManaged or hipHostMalloc memory.  One-element
 *   scale / zero-point buffers may also live in ordinary host memory; the
 *   library detects that and passes the value by kernel argument.
 *   Pointer *tables* (the per-expert arrays of group calls, row_ptrs itself)
 *   are host arrays; the library uploads them.
 *
 * Stream and ordering
 *   All work is enqueued on the calling thread's stream (zmi_set_stream; the
 *   default is the HIP null stream).  Calls return as soon as the work is
 *   enqueued; results are ordered with later work on the same stream.
 *
 * Status codes are the numeric values of the reference's status_t
 * (zendnnl/src/common/error_status.hpp:33-57).
 */
#ifndef ZMI_LOWOHA_H
#define ZMI_LOWOHA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Every entry point is exported; everything else in the library is hidden. */
#define ZMI_API __attribute__((visibility("default")))

/* ---- status_t (common/error_status.hpp:33-57) ------------------------- */
#define ZMI_SUCCESS          1
#define ZMI_FAILURE          0
#define ZMI_UNIMPLEMENTED   (-1)
#define ZMI_ISA_UNSUPPORTED (-21)

/* ---- data_type_t (common/data_types.hpp:44-58), same numeric values ---- */
enum zmi_dtype {
  ZMI_DT_NONE = 0, ZMI_DT_F32 = 1, ZMI_DT_F16 = 2, ZMI_DT_BF16 = 3,
  ZMI_DT_S32 = 4, ZMI_DT_S64 = 5, ZMI_DT_S16 = 6, ZMI_DT_S8 = 7,
  ZMI_DT_S4 = 8, ZMI_DT_U32 = 9, ZMI_DT_U16 = 10, ZMI_DT_U8 = 11,
  ZMI_DT_U4 = 12
};

/* ---- post_op_type_t (operators/common/post_op.hpp:36-57) --------------- */
enum zmi_post_op_type {
  ZMI_PO_NONE = 0, ZMI_PO_ELU = 1, ZMI_PO_RELU = 2, ZMI_PO_LEAKY_RELU = 3,
  ZMI_PO_GELU_TANH = 4, ZMI_PO_GELU_ERF = 5, ZMI_PO_SIGMOID = 6,
  ZMI_PO_SWISH = 7, ZMI_PO_TANH = 8, ZMI_PO_SOFTMAX = 9, ZMI_PO_POOLING = 10,
  ZMI_PO_SQUARE = 11, ZMI_PO_ABS = 12, ZMI_PO_SQRT = 13, ZMI_PO_EXP = 14,
  ZMI_PO_LOG = 15, ZMI_PO_CLIP = 16, ZMI_PO_BINARY_ADD = 17,
  ZMI_PO_BINARY_MUL = 18, ZMI_PO_MISH = 19
};

/* ---- matmul_algo_t (operators/matmul/matmul_config.hpp:37-52) ---------- */
enum zmi_matmul_algo {
  ZMI_ALGO_NONE = -1, ZMI_ALGO_DYNAMIC_DISPATCH = 0,
  ZMI_ALGO_AOCL_DLP_BLOCKED = 1, ZMI_ALGO_ONEDNN_BLOCKED = 2,
  ZMI_ALGO_LIBXSMM_BLOCKED = 3, ZMI_ALGO_AOCL_DLP = 4, ZMI_ALGO_ONEDNN = 5,
  ZMI_ALGO_LIBXSMM = 6, ZMI_ALGO_BATCHED_SGEMM = 7, ZMI_ALGO_AUTO_TUNER = 8,
  ZMI_ALGO_REFERENCE = 9, ZMI_ALGO_NATIVE_GEMM = 10,
  ZMI_ALGO_NATIVE_BRGEMM = 11
};

/* ---- grp_matmul_gated_act_t (group_matmul/group_matmul_direct.hpp:153) - */
enum zmi_gated_act {
  ZMI_ACT_NONE = 0, ZMI_ACT_SILU_AND_MUL = 1, ZMI_ACT_GELU_AND_MUL = 2,
  ZMI_ACT_SWIGLU_OAI_MUL = 3
};

#define ZMI_MAX_DIMS 4

/* matmul_quantization_params_t::matmul_quant_t (matmul/lowoha_common.hpp:77-86).
 * The element count is the product of dims[0..ndims); ndims == 0 means 1. */
typedef struct zmi_quant_t {
  const void *buff;
  int32_t dt;
  int32_t ndims;
  int64_t dims[ZMI_MAX_DIMS];
} zmi_quant_t;

/* matmul_post_op (matmul/lowoha_common.hpp:49-63). */
typedef struct zmi_post_op_t {
  int32_t po_type;      /* enum zmi_post_op_type */
  int32_t dtype;        /* dtype of buff (binary ops) */
  void *buff;
  int32_t ndims;
  int32_t leading_dim;  /* -1 => N */
  int64_t dims[ZMI_MAX_DIMS];
  float alpha;          /* clip: lower bound */
  float beta;           /* clip: upper bound */
} zmi_post_op_t;

/* matmul_batch_params_t (matmul/lowoha_common.hpp:110-127). */
typedef struct zmi_batch_params_t {
  int32_t Batch_A;
  int32_t Batch_B;
  uint64_t batch_stride_src;  /* (uint64_t)-1 => derive from the dimensions */
  uint64_t batch_stride_wei;
  uint64_t batch_stride_dst;
} zmi_batch_params_t;

/* matmul_params (matmul/lowoha_common.hpp:145-227), flattened. */
typedef struct zmi_matmul_params_t {
  int32_t dt_src, dt_wei, dt_dst, dt_bias, dt_compute;  /* matmul_data_types; dt_wei: s8, or s4 for W4A8 (bf16 src, dynamic_quant,
                                                          * s8 compute, bf16 dst: lowoha_matmul_utils.cpp:72-176), or s4 / u4
                                                          * with a bf16 src and no dynamic_quant: weight-only quantization
                                                          * (constant weights, wei_scale of 1, N or groups x N elements, for u4
                                                          * a wei_zp of s8 or bf16 type; bf16 / f32 dst:
                                                          * lowoha_matmul_utils.cpp:214-250, 313-328, aocl_kernel.cpp:43-139) */
  int32_t n_postops;
  const zmi_post_op_t *postops;
  zmi_quant_t src_scale, wei_scale, dst_scale, src_zp, wei_zp, dst_zp;
                              /* wei_zp: one zero-point for the weight tensor (s8 / u8 / s32, host or device), single
                               * problems with s8 / u8 sources (aocl_kernel.cpp:982-985, lru_cache/lowoha_cache.hpp:151-232);
                               * with 4-bit weight-only weights: 1, N or groups x N zero-points (device memory beyond one) */
  char mem_format_a;          /* 'n' */
  char mem_format_b;          /* 'n' plain weights, 'r' blob from zmi_reorder_direct */
  int32_t lowoha_algo;        /* enum zmi_matmul_algo */
  int32_t num_threads;        /* accepted and ignored: the GPU grid replaces OpenMP */
  int32_t dynamic_quant;
  int32_t pack_format_b;      /* 0: plain weights; 1: GGML Q8_0 blocks [N][K/32] x {fp16 d, int8 qs[32]}
                               * (transB and constant weights required; source scales {M, K/32}) */
  uint32_t total_matmul;
  uint32_t active_matmul;
  int32_t weight_cache_type;  /* 0 none, 1/2 keep a packed copy keyed by pointer */
} zmi_matmul_params_t;

/* Sets every field of *p to the reference's constructor defaults
 * (matmul/lowoha_common.hpp:223-226). */
ZMI_API void zmi_matmul_params_init(zmi_matmul_params_t *p);
ZMI_API void zmi_batch_params_init(zmi_batch_params_t *p);

/* matmul_direct (matmul/lowoha_matmul.hpp:104-108; body lowoha_matmul.cpp:278).
 * C = postops(alpha * A * B + beta * C + bias) for u8/s8 (or bf16/f32 with
 * dynamic_quant) activations x s8 weights, s32 accumulation. */
ZMI_API int32_t zmi_matmul_direct(char layout, int32_t transA, int32_t transB,
                          int32_t M, int32_t N, int32_t K, float alpha,
                          const void *src, int32_t lda,
                          const void *weight, int32_t ldb,
                          const void *bias, float beta,
                          void *dst, int32_t ldc, int32_t is_weights_const,
                          const zmi_batch_params_t *batch_params,
                          const zmi_matmul_params_t *params);

/* group_matmul_moe_postop_params (group_matmul/group_matmul_direct.hpp:96-128).
 * row_ptrs is a HOST array of num_tokens*topk device row pointers. */
typedef struct zmi_moe_postop_t {
  int32_t num_tokens;
  int32_t topk;
  void *output;
  int32_t ldc_output;
  const float *topk_weights;  /* device, [num_tokens, topk] */
  int32_t skip_weighted;
  const void **row_ptrs;
} zmi_moe_postop_t;

/* grp_matmul_fused_moe_params (group_matmul/group_matmul_direct.hpp:406-577).
 * Every array has n entries (n == 0 means "vector empty"). */
typedef struct zmi_fused_moe_t {
  int32_t n_down_weight; const void *const *down_weight;
  int32_t n_N_down;      const int32_t *N_down;
  int32_t n_ldb_down;    const int32_t *ldb_down;
  int32_t n_bias_down;   const void *const *bias_down;
  int32_t bias_dt_down;
  int32_t n_down_scale;  const zmi_quant_t *down_scale;
  int32_t n_down_zp;     const zmi_quant_t *down_zp;
  int32_t n_dst_down;    void *const *dst_down;   /* 0 => write Op2 into src[] */
  int32_t n_ldc_down;    const int32_t *ldc_down;
} zmi_fused_moe_t;

/* The std::vector arguments of group_matmul_direct, one (length, pointer)
 * pair per vector so that the reference's size checks can be reproduced
 * (matmul/group_matmul_direct.cpp:812-1063). */
typedef struct zmi_group_args_t {
  int32_t n_layout;  const char *layout;
  int32_t n_transA;  const uint8_t *transA;
  int32_t n_transB;  const uint8_t *transB;
  int32_t n_M;       const int32_t *M;
  int32_t n_N;       const int32_t *N;
  int32_t n_K;       const int32_t *K;
  int32_t n_alpha;   const float *alpha;
  int32_t n_src;     const void *const *src;
  int32_t n_lda;     const int32_t *lda;
  int32_t n_weight;  const void *const *weight;
  int32_t n_ldb;     const int32_t *ldb;
  int32_t n_bias;    const void *const *bias;
  int32_t n_beta;    const float *beta;
  int32_t n_dst;     void *const *dst;
  int32_t n_ldc;     const int32_t *ldc;
  int32_t n_is_weights_const; const uint8_t *is_weights_const;
  int32_t n_params;  const zmi_matmul_params_t *params;
} zmi_group_args_t;

/* group_matmul_direct (matmul/lowoha_matmul.hpp:204-223; body
 * matmul/group_matmul_direct.cpp:747).  gated_act is the value of
 * grp_matmul_gated_act_params::act, or ZMI_ACT_NONE for a null pointer. */
ZMI_API int32_t zmi_group_matmul_direct(const zmi_group_args_t *args,
                                const zmi_moe_postop_t *moe_postop,
                                int32_t gated_act,
                                const zmi_fused_moe_t *fused_moe);

/* prepack_params_t (reorder/prepack/lowoha_prepack.hpp:75-108). */
typedef struct zmi_prepack_params_t {
  int32_t algo;         /* must be ZMI_ALGO_AOCL_DLP_BLOCKED */
  int32_t wei_dtype;
  int32_t src_dtype;
  int64_t K, N, ldb;
  int32_t transposed;
  int32_t sym_group_size;
  size_t cached_size;   /* written by zmi_weight_prepack_size */
} zmi_prepack_params_t;

/* reorder_params_t (reorder/lowoha_reorder_common.hpp:146-204), the fields
 * the prepack and dynamic per-token modes read. */
typedef struct zmi_reorder_params_t {
  int32_t src_dtype, dst_dtype;
  zmi_quant_t scale;        /* dynamic mode: device buffer the scales are WRITTEN to */
  zmi_quant_t zero_point;   /* empty: symmetric (s8 rows); an s32 buffer with the scale's dims: asymmetric (u8 rows), {M,1} or {M,G} */
  int32_t algo;             /* reorder_algo_t: -1 none, 0 DT, 1 native, 2 reference */
  int32_t num_threads;
  int32_t n_src_shape;   int64_t src_shape[ZMI_MAX_DIMS];
  int32_t n_dst_shape;   int64_t dst_shape[ZMI_MAX_DIMS];
  int32_t n_src_strides; int64_t src_strides[ZMI_MAX_DIMS];
  int32_t n_dst_strides; int64_t dst_strides[ZMI_MAX_DIMS];
  int32_t dynamic_quant;
  int32_t is_prepack;
  zmi_prepack_params_t prepack;
} zmi_reorder_params_t;

ZMI_API void zmi_reorder_params_init(zmi_reorder_params_t *p);

/* weight_prepack_size (reorder/prepack/lowoha_prepack.hpp:165; body
 * lowoha_prepack.cpp:285-313): bytes of the packed blob, a multiple of 64,
 * 0 on invalid parameters.  Also stores it in params->prepack.cached_size. */
ZMI_API size_t zmi_weight_prepack_size(zmi_reorder_params_t *params);

/* reorder_direct (reorder/lowoha_reorder.hpp:103; body lowoha_reorder.cpp:43):
 * is_prepack   -> pack [K,N] s8 weights into the MFMA-fragment blob at dst;
 * dynamic_quant-> per-token symmetric bf16/f32 -> s8 with scales written to
 *                 params->scale.buff (dst may be NULL: scales only). */
ZMI_API int32_t zmi_reorder_direct(const void *src, void *dst,
                           zmi_reorder_params_t *params);

/* group_dynamic_quant_params_t (reorder/lowoha_reorder_common.hpp:357-368). */
typedef struct zmi_group_dq_params_t {
  int32_t src_dtype, dst_dtype, scale_dtype;
  int32_t num_threads;
  int32_t num_groups;
} zmi_group_dq_params_t;

/* group_dynamic_quant (reorder/lowoha_reorder.hpp:120-128; body
 * lowoha_reorder.cpp:279).  n matrices; strides are {row, col} pairs in
 * elements, row stride 0 meaning contiguous. */
ZMI_API int32_t zmi_group_dynamic_quant(int32_t n, const void *const *src,
                                const int32_t *M, const int32_t *K,
                                const int64_t *src_row_stride,
                                void *const *dst,
                                const int64_t *dst_row_stride,
                                void *const *scale,
                                const zmi_group_dq_params_t *params);

/* zmi_matmul_direct_noalloc: zmi_matmul_direct for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid it).  It has no counterpart in the reference.  Same arguments,
 * arithmetic and kernels as zmi_matmul_direct, for the decode-shaped call whose
 * source rows are quantized at run time: bf16 / f32 source with dynamic_quant and
 * s8 compute, source scale dims {1} or {M,1} (buff null or a device buffer that
 * receives the scales), prepacked weights (mem_format_b 'r'), no transposes,
 * M <= 128 and K <= 4096; anything else returns unimplemented / failure.  The
 * quantized rows and their scales live in a fixed 514 KiB array inside the
 * library's device image (one copy per GPU, held until the process ends) instead
 * of the calling thread's scratch arena; the call makes no hipMalloc / hipFree.
 * All calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered by the stream.
 * The first call with a given blob reads the blob's header back once. */
ZMI_API int32_t zmi_matmul_direct_noalloc(char layout, int32_t transA, int32_t transB,
                          int32_t M, int32_t N, int32_t K, float alpha,
                          const void *src, int32_t lda,
                          const void *weight, int32_t ldb,
                          const void *bias, float beta,
                          void *dst, int32_t ldc, int32_t is_weights_const,
                          const zmi_batch_params_t *batch_params,
                          const zmi_matmul_params_t *params);

/* ---- Library services with no counterpart in the reference ------------ */

/* Selects the GPU (hipSetDevice) and creates the per-device state.  Optional:
 * the first compute call does it for device 0. */
ZMI_API int32_t zmi_init(int32_t device);
/* hipStream_t used by the calling thread's later calls (NULL = null stream). */
ZMI_API void zmi_set_stream(void *hip_stream);
ZMI_API void *zmi_get_stream(void);
/* Text of the calling thread's most recent failure ("" if none). */
ZMI_API const char *zmi_last_error(void);
/* Name of the kernel variant the calling thread's last compute call used. */
ZMI_API const char *zmi_last_kernel(void);
/* Frees the packed-weight cache kept for mem_format_b == 'n' constant weights
 * (reference: clear_aocl_matmul_weight_caches, backends/aocl/aocl_kernel.cpp:294). */
ZMI_API void zmi_clear_weight_cache(void);
/* Frees the calling thread's scratch arena (reference: clear_fused_moe_scratch,
 * group_matmul/group_matmul_direct.hpp:683). */
ZMI_API void zmi_clear_scratch(void);
/* The library reads its environment switches (ZMI_*, ZENDNNL_*) once per process; this reads them again.  Not while
 * calls of other threads are in flight.  (No counterpart in the reference, whose switches are read per call.) */
ZMI_API void zmi_reload_env(void);
/* Library version string. */
ZMI_API const char *zmi_version(void);

/* Device-side MoE routing glue.  In the reference the framework scatters
 * tokens to experts on the host (docs/operator/low_overhead_operator/
 * lowoha_group_matmul_operator.md:238-259); on a GPU that step must not
 * round-trip through the host, so the library offers it.
 *
 * zmi_moe_route: from topk_ids [T, topk] (s32, device) builds
 *   counts[E]      rows per expert,
 *   offsets[E+1]   exclusive prefix sum of counts,
 *   slot_of[T*topk] position of (t,k) in the expert-sorted row order
 *                  (stable: within an expert rows keep (t,k) order).
 * All outputs are device s32 buffers. */
ZMI_API int32_t zmi_moe_route(const int32_t *topk_ids, int32_t T, int32_t topk,
                      int32_t E, int32_t *counts, int32_t *offsets,
                      int32_t *slot_of);

/* zmi_moe_router_topk: the step in front of zmi_moe_route -- router logits
 * [T, E] (f32 or bf16, device, row stride ldl elements) -> topk_ids [T, topk]
 * (s32) and topk_weights [T, topk] (f32), both device.  The reference has no
 * counterpart (routing is the framework's, same document); its MoE post-op
 * consumes exactly these two arrays (group_matmul_moe_postop.cpp:103-129).
 *   ids:     the topk largest logits of the token in descending order, equal
 *            logits in ascending expert order (the head of a stable descending
 *            sort); -0 == +0, NaN sorts last;
 *   weights: softmax over all E logits in f32, of the selected experts; with
 *            renormalize != 0 divided by the sum of the topk selected weights.
 * Limits: E <= 512, topk <= min(E, 64). */
ZMI_API int32_t zmi_moe_router_topk(const void *logits, int32_t logits_dt, int64_t ldl,
                            int32_t T, int32_t E, int32_t topk, int32_t renormalize,
                            int32_t *topk_ids, float *topk_weights);

/* zmi_moe_fused_device: whole MoE block with routing kept on the device.
 * x [T,H] bf16 -> per-token s8 quantization -> expert-sorted scatter ->
 * Op1 (gate|up, s8 blob) -> act(gate)*up -> bf16 -> per-token s8 ->
 * Op2 (down, s8 blob) -> out[t] = sum_k w[t,k] * y[slot(t,k)] (bf16).
 * Same arithmetic as zmi_group_matmul_direct with fused_moe + moe_postop;
 * only the scatter / row_ptrs construction moves from the caller to the GPU. */
typedef struct zmi_moe_device_t {
  int32_t T, H, I, E, topk;
  const void *x;  int32_t ldx;              /* bf16 [T, ldx] */
  const int32_t *topk_ids;                  /* [T, topk] */
  const float *topk_weights;                /* [T, topk] */
  const void *const *w13_blob;              /* host array [E] of prepack blobs of [H, 2I] = [gate | up] */
  const void *const *w2_blob;               /* host array [E] of prepack blobs [I, H] */
  const float *const *w13_scale;            /* host array [E] of device f32 [2I] */
  const float *const *w2_scale;             /* host array [E] of device f32 [H] */
  int32_t gated_act;
  void *out; int32_t ldo;                   /* bf16 [T, ldo] */
} zmi_moe_device_t;
ZMI_API int32_t zmi_moe_fused_device(const zmi_moe_device_t *d);

/* ---- Measurement aids (no counterpart in the reference; not on the path of any
 * call above).  They measure what this device sustains with nothing in the way,
 * the denominators next to the nominal peaks.
 *
 * zmi_calib_hbm_read: launches a kernel that only reads `bytes` bytes (a multiple
 * of 128 KiB) with the decode kernels' launch shape, `warm` untimed and `launches`
 * timed launches over the n_bufs device buffers in turn (rotate enough of them to
 * exceed the on-die cache).  us_per_launch: between two events on `stream`;
 * span_us: first wavefront's start to last wavefront's end inside one launch.
 *
 * zmi_calib_mfma_i8: one launch of `iters` x 8 v_mfma_i32_32x32x32_i8 per wavefront,
 * 4 wavefronts per workgroup, wgs_per_cu workgroups per compute unit.  operands:
 * 6 KiB of int8 operand fragments in device memory; vary_operands != 0 feeds
 * consecutive instructions different fragments (what random GEMM data does to the
 * multipliers).  tops: 1e12 int8 operations per second (2 per multiply-add);
 * shader_mhz: average shader clock inside the loop. */
ZMI_API int32_t zmi_calib_hbm_read(void *const *bufs, int32_t n_bufs, uint64_t bytes,
                           int32_t warm, int32_t launches, void *stream,
                           float *us_per_launch, float *span_us);
/* The same read with the launch shape given: workgroups of `threads` threads (256, 512, 1024), `requests` requests
 * of 16 bytes per lane (8, 14, 16), bytes / (threads * requests * 16) workgroups.  The best shape's figure is the
 * ceiling a streaming kernel of this size can be held against. */
ZMI_API int32_t zmi_calib_hbm_read_shape(void *const *bufs, int32_t n_bufs, uint64_t bytes,
                           int32_t threads, int32_t requests, int32_t warm, int32_t launches,
                           void *stream, float *us_per_launch, float *span_us);
/* No counterpart in the reference (its planner is internal: matmul/partitioning).  Which large-M kernel a single
 * problem of this shape gets when its destination is bf16, its rows 16-byte aligned and its epilogue one of the
 * straight-line ones: tile_rows 0 = none of them (a decode-shaped kernel takes the call), else the tile height
 * (64 / 128 / 256); k_slices >= 1; persistent 1 = the persistent form (k_pring.hip), 0 = the tiled one (k_ring.hip).
 * Needs no device (256 compute units are assumed without one); honours the ZMI_* overrides. */
ZMI_API int32_t zmi_large_m_plan(int32_t M, int32_t N, int32_t K, int32_t *tile_rows, int32_t *k_slices,
                         int32_t *persistent);
ZMI_API int32_t zmi_calib_mfma_i8(const void *operands, int32_t vary_operands,
                          int32_t wgs_per_cu, int32_t iters, void *stream,
                          float *tops, float *shader_mhz);

#ifdef __cplusplus
}
#endif
#endif /* ZMI_LOWOHA_H */
