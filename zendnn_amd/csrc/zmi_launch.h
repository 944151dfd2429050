// Host-callable launchers of the gfx950 kernels (one per .hip file).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>

#include "zmi_device.h"

// Raises a kernel's limit of dynamic LDS to `bytes` the first time it is needed on the current
// device (the attribute belongs to the device's copy of the kernel); callable from any thread.
inline hipError_t zmi_func_smem_once(const void *func, int bytes) {
  static std::mutex mu;
  static std::map<std::pair<int, const void *>, int> done;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lk(mu);
  int &have = done[std::make_pair(dev, func)];
  if (have >= bytes) return hipSuccess;
  e = hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) have = bytes;
  return e;
}

// Environment switches.  The process reads each of them once, at the first call that asks for any (zmi_reload_env()
// reads them again; with ZMI_ENV_LIVE=1 in the environment at that first call every look goes to the environment,
// which is how the tests flip switches between calls).  zmi_env returns the value, or null when the variable is unset.
enum ZmiEnvVar {
  ZE_DECODE_ROWGROUP_KERNEL,
  ZE_DECODE_SELFQ_MIN_WGS,
  ZE_DECODE_SELFQ_MAX_M,
  ZE_NO_DECODE_SELFQ,
  ZE_DECODE_NO_ROW_PAIRS,
  ZE_DECODE_RPW,
  ZE_NO_GROUP_DECODE,
  ZE_PERGROUP_GENERIC,
  ZE_NO_S4_STREAM,
  ZE_PRING_GRID,
  ZE_NO_GROUP_STREAM,
  ZE_WOQ_BLOCKS,
  ZE_DECODE_MAX_M,
  ZE_NO_DECODE_KERNEL,
  ZE_NO_DECODE_SLICED,
  ZE_GEMM_TOP,
  ZE_RING_SPLITK,
  ZE_PRING,
  ZE_RING_MIN_M,
  ZE_PGRING_MIN_M,
  ZE_NO_FUSED_QUANT,
  ZE_GROUP_TOP,
  ZE_GROUP_STREAM_TOP,
  ZE_GROUP_STREAM_SLICES,
  ZE_GROUP_DECODE,
  ZE_ZENDNNL_LRU_CACHE_CAPACITY,
  ZE_NO_SLICE_ARRIVALS,
  ZE_NO_SIDE_STREAM,
  ZE_FUSED_WAIT_US,
  ZE_ZENDNNL_DIAGNOSTICS_ENABLE,
  ZE_ZENDNNL_MATMUL_WEIGHT_CACHE,
  ZE_NO_UNCACHED_FLAGS,
  ZE_NO_GROUP_RING_SLICES,
  ZE_COUNT
};
const char *zmi_env(ZmiEnvVar v);

// One matrix of a (possibly grouped) per-token quantization launch; row_start is
// the index of its first row in the launch's global row numbering.
struct ZmiQuantMat {
  const void *src;
  int8_t *dst;       // may be null: scales only
  void *scale;
  int64_t ld_src, ld_dst;
  int32_t M, K;
  int32_t row_start;
  int32_t frag_kpad;   // 0: dst rows are K-contiguous with stride ld_dst; > 0: dst is fragment-major with this K_pad
  // optional row gather (8-rows-per-workgroup kernel only): destination row r is quantized from
  // source row gather[r] / gather_div, rows with gather[r] < 0 are skipped
  const int32_t *gather;
  int32_t gather_div;
};

// k_prepack.hip
hipError_t zmi_launch_prepack(const int8_t *B, int64_t K, int64_t N, int64_t ldb, int transposed,
                              int32_t src_dtype, int32_t sym_group_size, uint8_t *blob,
                              hipStream_t stream);

// k_quant.hip
hipError_t zmi_launch_quant_rows(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t ld_src,
                                 int8_t *dst, int64_t ld_dst, int64_t frag_kpad, void *scales, int32_t scale_dt,
                                 hipStream_t stream);
// rows8 != 0: row_start of every matrix is a multiple of 8 and zmi_quant_mat_frag8_ok holds for all of them
hipError_t zmi_launch_quant_group(const ZmiQuantMat *mats_dev, int n_mat, int64_t total_rows,
                                  int32_t src_dt, int32_t scale_dt, int rows8, hipStream_t stream);
bool zmi_quant_mat_frag8_ok(const ZmiQuantMat &m, int32_t src_dt);
hipError_t zmi_launch_quant_gather(const void *x, int32_t x_dt, int64_t ldx, int64_t K, const int32_t *gather,
                                   int32_t gather_div, int64_t n_rows, int8_t *dst, int64_t frag_kpad, float *scales,
                                   hipStream_t stream);
hipError_t zmi_launch_quant_tensor(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t ld_src,
                                   int8_t *dst, int64_t ld_dst, int64_t frag_kpad, float *scales,
                                   unsigned int *amax_scratch, hipStream_t stream);

// k_ring.hip: A in fragment-major order; `top` is the largest tile height (128 or 256)
int zmi_ring_pick_top(int64_t rows, int64_t out_cols);
int zmi_ring_pick_top_group(int64_t rows, int n_prob, int64_t K, int64_t N, bool gated);
// K slices of a one-problem ring launch.  When a problem has fewer tiles than the device
// has CUs, every tile is computed by `slices` workgroups, each over its own range of K;
// they leave int32 partial tiles in `partial`, and a second kernel adds the slices of each
// tile and runs the epilogue.
struct ZmiRingSplit {
  int slices;              // 1: no slicing, the pointer is unused
  int32_t *partial;        // tiles * slices * tile rows * 256 words
  unsigned int *arrivals;  // null, or a zeroed word per tile (zero again after the launch): the slice that arrives last
                           // at its tile's word adds the others' partial tiles to its own and finishes the elements,
                           // and there is no reduction launch
};
struct ZmiRingPlan {
  int top;                 // tile height (with ZMI_RING_PAD when slices > 1)
  int slices;
  int tiles;
  size_t partial_bytes;    // 0 when slices == 1
};
// top_hint: tile height to use when the launch is not sliced (0: zmi_ring_pick_top);
// force_slices: 0 = choose, n = that many slices where the shape allows it.
ZmiRingPlan zmi_ring_plan(int M, int N, int K, int top_hint, int force_slices);
// side (optional): a second stream with two events.  An unsliced launch with 256-row tiles puts the remainder rows'
// tiles (their own kernel: 64- or 128-row tiles) on it, between a fork and a join on `stream`, so that they run on
// the CUs the 256-row tiles leave free instead of behind them.
struct ZmiRingSide {
  hipStream_t stream;
  hipEvent_t fork, join;
};
hipError_t zmi_launch_gemm_ring(const ZmiProblem &p, const ZmiEpilogue &epi, int top, const ZmiRingSplit *split,
                                hipStream_t stream, const ZmiRingSide *side = nullptr);
// k_pring.hip: the persistent form for one problem (A in fragment-major order, bf16 destination, straight-line epilogue)
bool zmi_pring_takes(const ZmiProblem &p, const ZmiEpilogue &epi);
hipError_t zmi_launch_gemm_pring(const ZmiProblem &p, const ZmiEpilogue &epi, hipStream_t stream);
hipError_t zmi_launch_gemm_ring_group(const ZmiProblem *probs_host, const ZmiProblem *probs_dev, int n_prob,
                                      int top, int64_t worst_rows, int worst_cols, int *tab_dev, bool tab_ready,
                                      const ZmiEpilogue &epi, hipStream_t stream, const ZmiRingSplit *split = nullptr);
// tiles of such a launch at tile height `top` (a bound when the row counts live on the device: probs_host null)
int zmi_ring_group_items(const ZmiProblem *probs_host, int n_prob, int top, int64_t worst_rows, int worst_cols, bool gated);

// k_group_decode.hip: the problems of a grouped launch that have 1 .. 16 rows (rows in fragment order), gated or not;
// one workgroup per (problem, 32 output columns), max_out_cols = the widest problem's output columns
bool zmi_group_decode_takes(const ZmiEpilogue &epi, int N);
// Weight-traffic-bound grouped launch on the MFMA-bound kernel's tiles (k_stream.hip)
bool zmi_group_stream_takes(const ZmiEpilogue &epi, int N, int top_flags);
int zmi_cu_count();   // compute units of the current device
// k_util.hip: the per-row compensation of a weight zero-point (see ZmiProblem::row_comp)
hipError_t zmi_launch_row_comp(const void *A, int64_t lda, bool transA, bool is_u8, int M, int K, int32_t wei_zp_val,
                               const void *wei_zp_ptr, int32_t wei_zp_dt, int32_t src_zp_val, const int32_t *src_zp_ptr,
                               int32_t *out, hipStream_t stream);
int zmi_stream_items(const ZmiProblem *probs_host, int n_prob, int top, int64_t worst_rows, int worst_cols, bool gated);
size_t zmi_stream_partial_bytes(int items, int slices, int top);
hipError_t zmi_launch_gemm_stream_group(const ZmiProblem *probs_host, const ZmiProblem *probs_dev, int n_prob, int top,
                                        int64_t worst_rows, int worst_cols, const int *tab_dev, const ZmiRingSplit *split,
                                        const ZmiEpilogue &epi, hipStream_t stream);
// Fills the tile table of a grouped launch (4 + 3 * n_prob ints) from the problems' row counts on the device
hipError_t zmi_launch_ring_table(const ZmiProblem *probs_dev, int n_prob, int top, bool gated, int *tab_dev, hipStream_t stream);
hipError_t zmi_launch_gemm_group_decode(const ZmiProblem *probs_dev, int n_prob, int max_out_cols, const ZmiEpilogue &epi,
                                        hipStream_t stream);

// k_smallm.hip
struct ZmiFusedQuant {
  const void *x;          // bf16 / f32 rows, null: no fused quantization
  int64_t ldx;
  int32_t x_dt;
  int8_t *q;              // s8 rows out (== ZmiProblem::A)
  int64_t ldq;
  float *scales;          // f32 scale per row out (== ZmiProblem::src_scale_ptr)
  void *user_scales;      // optional copy in user_dt
  int32_t user_dt;
  // Hand-off between the quantizing and the streaming workgroups of one launch: one device word per row,
  // set to the launch's `epoch` once the row and its scale are in memory.  The epoch only names the launch
  // (a fresh value per launch from the calling thread); nothing is counted, so a launch that fails or never
  // runs leaves nothing behind that a later launch could trip over.
  unsigned int *flags;    // [>= M]
  unsigned int epoch;
  unsigned int *error;    // host-visible word, set to 1 by a wavefront whose wait ran out
  uint32_t wait_ticks;    // limit of the wait in ticks of the 100 MHz real-time counter; 0: give up at once
  int32_t per_row;        // per-group kernels only: one scale per row (scales[row]) stands for all its groups
  int32_t flags_uncached; // the flags lie in uncached device memory: the wait through the scalar unit may be used
  int32_t n_copies;       // copies of the flag words, 1024 words apart (1: just flags[0 .. M))
};

int zmi_smallm_grid(const ZmiProblem &p);
hipError_t zmi_launch_gemm_smallm_fused(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant &fq,
                                        hipStream_t stream);
hipError_t zmi_launch_gemm_smallm(const ZmiProblem &p, const ZmiEpilogue &epi, hipStream_t stream);

// k_pergroup.hip: per-group symmetric scales ({M,G} source, {G,N} weights), any M; s8 rows with a
// 16-byte aligned leading dimension; group sizes 16, 32 or a multiple of 64
bool zmi_pergroup_group_size_ok(int64_t gs);
struct ZmiFusedQuant;
// fq != null (decode-shaped problems only): the per-group quantization of the M rows is part of the launch
// tiles_s4 != null (widened s4 weights): decode-shaped problems with K >= 1024 stream the 4-bit tiles instead of the blob
hipError_t zmi_launch_gemm_pergroup(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq,
                                    hipStream_t stream, const uint8_t *tiles_s4 = nullptr);
// true when the launch above takes the decode-shaped kernel (up to 16 rows, K = 512 .. 4096 in whole eighths)
bool zmi_pergroup_decode_shape(const ZmiProblem &p, int G);
// true when it would stream 4-bit tiles if it had them
bool zmi_pergroup_s4_shape(const ZmiProblem &p, int G);
// asymmetric form: u8 rows, f32 scales {M,G} and s32 zero-points {M,G} (G == 1: per token); a bf16 copy of the
// scales goes to user_scales when user_dt says so
hipError_t zmi_launch_quant_asym(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, uint8_t *q,
                                 int64_t ldq, float *scales, int32_t *zps, void *user_scales, int32_t user_dt,
                                 hipStream_t stream);
// the same with the s8 rows written in MFMA fragment order (groups of 32, 64 or 128, 16-byte aligned rows)
bool zmi_quant_groups_frag_ok(const void *x, int32_t x_dt, int64_t K, int64_t ldx, int64_t G);
hipError_t zmi_launch_quant_groups_frag(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, int8_t *q,
                                        float *scales, void *user_scales, int32_t user_dt, hipStream_t stream);
// k_pgring.hip: the per-group GEMM at large M (fragment-order rows, MFMA 32x32x32, scales through LDS);
// group sizes 32 (K a multiple of 64), 64 and multiples of 128
bool zmi_pgring_takes(int64_t M, int64_t N, int64_t K, int64_t gs);
int64_t zmi_pgring_ws_cols(int64_t N);
// scales {rows, cols} (f32 / bf16) -> f32 rows of out_cols columns: the weight scales {G, N} with
// out_cols = zmi_pgring_ws_cols(N); bf16 source scales {M, G} with out_cols = G
hipError_t zmi_launch_pgring_scales(const void *src, int32_t dt, int64_t rows, int64_t cols, int64_t out_cols, float *out,
                                    hipStream_t stream);
// p.A: s8 rows in fragment order; ss: {M, G} f32 source scales; ws: the padded f32 weight scales
hipError_t zmi_launch_gemm_pgring(const ZmiProblem &p, const ZmiEpilogue &epi, const float *ss, const float *ws,
                                  hipStream_t stream);
// Dynamic asymmetric quantization of a whole [M, K] bf16 / f32 source to u8 with one scale and one zero-point
// (k_asym.hip).  lohi: 2 * M floats of scratch; scale / zp: one element each, device memory.
hipError_t zmi_launch_quant_asym_tensor(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, uint8_t *q,
                                        int64_t ldq, float *lohi, float *scale, int32_t *zp, void *user_scale,
                                        int32_t user_dt, hipStream_t stream);

// Weight-only quantization (k_woq.hip): bf16 rows x 4-bit weights dequantized to bf16 in registers, f32 accumulation.
struct ZmiWoqProblem {
  const void *A;            // bf16 [M, lda] (or [K, lda] when transA)
  int64_t lda;
  int32_t transA;
  int32_t a_fast;           // rows can be read 16 bytes at a time (no transA, K, lda multiples of 8, 16-byte aligned base)
  const uint32_t *tiles;    // zmi_woq_tiles_bytes(K, N) bytes from zmi_launch_woq_tiles
  void *dst;
  int64_t ldc;
  int32_t M, N, K;
  int32_t is_u4;            // codes 0 .. 15 instead of -8 .. 7
  int32_t has_zp;
  int32_t zp_float_domain;  // u4 codes with a bf16 zero-point: (code - 8) * scale + zp
  const float *sf;          // [n_groups][N] f32 scales and zero-points (zmi_launch_woq_params)
  const float *zf;
  int32_t group_size;       // K / n_groups
  int32_t n_groups;
  const void *bias;
};
// a scale / zero-point tensor as the caller gave it: mode 0 = one value (at ptr, or val when ptr is null), 1 = one
// per column, 2 = one per K group and column, {n_groups, N}
struct ZmiWoqParamSrc {
  const void *ptr;
  int32_t dt, mode;
  float val;
};
hipError_t zmi_launch_woq_params(const ZmiWoqParamSrc &s, const ZmiWoqParamSrc &z, int64_t G, int64_t N, float *sf,
                                 float *zf, hipStream_t stream);
hipError_t zmi_launch_woq_tiles(const void *packed, int64_t K, int64_t N, int64_t ldb, bool transB, uint32_t *out,
                                hipStream_t stream);
// (of the epilogue descriptor only alpha, beta, bias_dt, the post-ops and dst_dt are read)
hipError_t zmi_launch_gemm_woq(const ZmiWoqProblem &p, const ZmiEpilogue &epi, hipStream_t stream);
// column blocks of 32 a workgroup of that launch multiplies with each row fragment (1 or 2)
int zmi_woq_blocks(const ZmiWoqProblem &p);

// 4-bit tiles of a blob of widened s4 weights (zmi_s4_tiles_bytes(K, N) bytes)
hipError_t zmi_launch_s4_tiles(const uint8_t *blob, int64_t K, int64_t N, uint8_t *out, hipStream_t stream);
// per (row, group) dynamic quantization of bf16 / f32 rows: s8 rows (ld ldq), f32 scales {M,G} and an
// optional copy of the scales in the caller's buffer (f32 or bf16)
hipError_t zmi_launch_quant_groups(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, int8_t *q,
                                   int64_t ldq, float *scales, void *user_scales, int32_t user_dt, hipStream_t stream);

// k_decode.hip: single problem, M <= 128, K_pad <= 4096
bool zmi_decode_kernel_fits(const ZmiProblem &p);
// fq != null: the launch also quantizes the M source rows (its grid must be resident at once)
// partial: int32 workspace of zmi_decode16_partial_bytes() for the K-sliced form (K beyond 4096, up to 16 given rows);
// arrivals: one zeroed word per 32-column block (left zeroed) -- with it the last slice of a block finishes the
// elements, without it a second kernel does
hipError_t zmi_launch_gemm_decode(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq,
                                  hipStream_t stream, int32_t *partial = nullptr, unsigned int *arrivals = nullptr);
int zmi_decode16_slices(int M, int64_t K, int64_t lda);
size_t zmi_decode16_partial_bytes(int M, int N, int64_t K);
int zmi_decode_grid(const ZmiProblem &p);
// true when the launch above takes the 16-row kernel (rows fetched by global->LDS loads behind the first weights)
bool zmi_decode_16row_kernel(const ZmiProblem &p, bool fused_quant);
struct ZmiFusedQuant;
// true when a launch with these rows quantizes them inside the workgroups that use them (no hand-off)
bool zmi_decode_selfq_takes(const ZmiProblem &p, const ZmiFusedQuant *fq);

// k_moe.hip
struct ZmiActMat {
  void *buf;
  int64_t ld;
  int32_t M, N;
  int32_t row_start;
};
hipError_t zmi_launch_gated_act(const ZmiActMat *mats_dev, const ZmiActMat *mat0, int n_mat,
                                int64_t total_rows, int max_N, int32_t act, int32_t dt, hipStream_t stream);
hipError_t zmi_launch_moe_combine(const void *const *row_ptrs_dev, const void *rows_base, int64_t row_ld,
                                  const int32_t *slot_of, const float *weights, int skip_weighted,
                                  int T, int topk, int D, int32_t dt, void *out, int64_t ldo,
                                  hipStream_t stream);
// align: every expert's first slot is rounded up to a multiple of it (1: dense numbering).
// src_of (optional, n_slots entries): the flat (token, k) index that fills each slot, -1 for idle slots.
size_t zmi_moe_route_scratch_ints(int64_t n, int E);
hipError_t zmi_launch_moe_router_topk(const void *logits, int logits_dt, int64_t ldl, int T, int E, int topk,
                                      int renormalize, int32_t *topk_ids, float *topk_weights, hipStream_t stream);
hipError_t zmi_launch_moe_route(const int32_t *topk_ids, int T, int topk, int E, int align, int32_t *counts,
                                int32_t *offsets, int32_t *slot_of, int32_t *src_of, int n_slots,
                                int32_t *hist_scratch, hipStream_t stream);
// A1 is fragment-major over the slot numbering, K_pad = zmi_blob_kpad(H)
hipError_t zmi_launch_moe_quant_scatter(const void *x, int64_t ldx, int T, int H, int topk,
                                        const int32_t *slot_of, int8_t *A1, float *s1, hipStream_t stream);
struct ZmiMoeTables {   // device arrays of E entries each
  const void *const *w13_blob;
  const void *const *w2_blob;
  const float *const *w13_scale;
  const float *const *w2_scale;
};
hipError_t zmi_launch_moe_build_problems(ZmiMoeTables tb, int E, int H, int I, const int32_t *counts,
                                         const int32_t *offsets, const int8_t *A1, const float *s1, void *act,
                                         const int8_t *A2, const float *s2, void *Y, ZmiProblem *op1,
                                         ZmiProblem *op2, int top1, int top2, int *tab1, int *tab2,
                                         hipStream_t stream);

// k_util.hip
hipError_t zmi_launch_pad_rows(const void *src, int64_t M, int64_t K, int64_t ld_src, int trans,
                               int8_t *dst, int64_t ld_dst, hipStream_t stream);
// GGML Q8_0 blocks ([N][K/32] x {fp16 d, int8 qs[32]}) -> s8 rows [N, K] and bf16 scales {K/32, N}
hipError_t zmi_launch_ggml_q8_0_unpack(const void *blocks, int64_t N, int64_t K, int8_t *rows, uint16_t *scales,
                                       hipStream_t stream);
// packed s4 codes of a [rows, ld] matrix (two per byte, even index = low nibble) -> s8 [rows, cols]
hipError_t zmi_launch_s4_widen(const void *packed, int64_t rows, int64_t cols, int64_t ld, int8_t *out, hipStream_t stream);
// one f32 / bf16 scale per tensor or per row -> f32 {M, G}
hipError_t zmi_launch_broadcast_scales(const void *src, int32_t dt, int per_tensor, int64_t M, int64_t G, float *out,
                                       hipStream_t stream);
// sc[i] = bf16(sc[i]) for i < n; the first n_user narrowed values also go to a caller's bf16 buffer (may be null)
hipError_t zmi_launch_narrow_scales(float *sc, int64_t n, void *user_bf16, int64_t n_user, hipStream_t stream);
// u8 / s8 rows (or their transpose) -> fragment-major s8; u8 values are shifted by -128
hipError_t zmi_launch_repack_frag(const void *src, int64_t M, int64_t K, int64_t ld_src, int trans, int is_u8,
                                  int8_t *dst, hipStream_t stream);
