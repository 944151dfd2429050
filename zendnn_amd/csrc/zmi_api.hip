// C ABI: matmul_direct, reorder_direct (prepack and dynamic per-token modes),
// weight_prepack_size, group_dynamic_quant.
#include <cmath>
#include <cstring>
#include <vector>

#include "zmi_api.h"
#include "zmi_host.h"

namespace zmi {

bool is_dynamic_quant_config(const zmi_matmul_params_t &p);
// elements the dims of a quantization parameter describe, buffer or not (1 without dims)
static int64_t shape_elems(const zmi_quant_t &q) {
  int64_t n = 1;
  for (int i = 0; i < q.ndims; ++i) n *= q.dims[i];
  return n;
}

// Mirrors validate_matmul_direct_inputs of the reference
// (zendnnl/src/lowoha_operators/matmul/lowoha_matmul_utils.cpp:180-411) for the
// rules that concern the int8 path.  Every failure is status failure.
int32_t validate_matmul(const void *src, const void *weight, const void *dst, int M, int N, int K,
                        int Batch_A, int Batch_B, const zmi_matmul_params_t &p, bool is_weights_const) {
  (void)is_weights_const;
  if (!src || !weight || !dst) { set_error("null src / weight / dst"); return ZMI_FAILURE; }
  if (M <= 0 || N <= 0 || K <= 0) { set_error("M, N, K must be positive"); return ZMI_FAILURE; }
  if (Batch_A <= 0 || Batch_B <= 0) { set_error("batch sizes must be positive"); return ZMI_FAILURE; }
  const bool is_int8 = p.dt_wei == ZMI_DT_S8;
  if ((p.src_scale.buff || p.dst_scale.buff || p.src_zp.buff || p.dst_zp.buff) && !is_int8) {
    set_error("src / dst scales and zero-points are given but the weights are not s8");
    return ZMI_FAILURE;
  }
  if (p.src_scale.buff) {
    const int64_t n = nelems(p.src_scale);
    if (n != 1) {
      const bool src_ok = p.dt_src == ZMI_DT_S8 || p.dt_src == ZMI_DT_BF16 || p.dt_src == ZMI_DT_F32;
      const bool sym = !p.src_zp.buff;
      const bool dst_ok = p.dt_dst == ZMI_DT_F32 || p.dt_dst == ZMI_DT_BF16;
      const bool per_token = n == M;
      const bool per_group = n > M && n % M == 0 && K % (n / M) == 0;
      if (!(src_ok && sym && dst_ok && (per_token || per_group))) {
        set_error("source scales per row or per K-group: the source must be s8 / bf16 / f32 without a zero-point and the destination f32 / bf16");
        return ZMI_FAILURE;
      }
      const int64_t wn = p.wei_scale.buff ? nelems(p.wei_scale) : 0;
      if (per_token && p.pack_format_b != 1 && wn != N) {
        set_error("a source scale per row goes with a weight scale per column (N elements)");
        return ZMI_FAILURE;
      }
      // (GGML-packed weights carry their per-group scales inside the packed buffer: lowoha_matmul_utils.cpp:276-283)
      if (per_group && p.pack_format_b != 1 && wn != (n / M) * N) {
        set_error("a source scale per K-group goes with a weight scale of groups x N elements");
        return ZMI_FAILURE;
      }
    }
  }
  auto per_tensor = [](const zmi_quant_t &q, const char *name) {
    if (q.buff && nelems(q) != 1) { set_error(std::string(name) + " must hold exactly one element (one value for the tensor)"); return false; }
    return true;
  };
  if (!per_tensor(p.src_zp, "source zero-point") || !per_tensor(p.dst_scale, "destination scale") ||
      !per_tensor(p.dst_zp, "destination zero-point"))
    return ZMI_FAILURE;
  const int s = p.dt_src, d = p.dt_dst;
  if (!(s == ZMI_DT_F32 || s == ZMI_DT_BF16 || s == ZMI_DT_U8 || s == ZMI_DT_S8 || s == ZMI_DT_F16)) {
    set_error("unsupported source data type");
    return ZMI_FAILURE;
  }
  if (!(d == ZMI_DT_F32 || d == ZMI_DT_BF16 || d == ZMI_DT_U8 || d == ZMI_DT_S8 || d == ZMI_DT_S32 ||
        d == ZMI_DT_F16)) {
    set_error("unsupported destination data type");
    return ZMI_FAILURE;
  }
  if (s == ZMI_DT_F32 && (d == ZMI_DT_BF16 || d == ZMI_DT_F16)) {
    set_error("f32 source with bf16 / f16 destination");
    return ZMI_FAILURE;
  }
  if ((s == ZMI_DT_BF16 && d == ZMI_DT_F16) || (s == ZMI_DT_F16 && d == ZMI_DT_BF16)) {
    set_error("mixed bf16 / f16 source and destination");
    return ZMI_FAILURE;
  }
  const int bmax = Batch_A > Batch_B ? Batch_A : Batch_B, bmin = Batch_A < Batch_B ? Batch_A : Batch_B;
  if (bmax % bmin != 0) { set_error("batch sizes do not broadcast"); return ZMI_FAILURE; }
  for (int i = 0; i < p.n_postops; ++i) {
    const zmi_post_op_t &po = p.postops[i];
    if (po.po_type == ZMI_PO_CLIP && (!std::isfinite(po.alpha) || !std::isfinite(po.beta))) {
      set_error("clip bounds must be finite");
      return ZMI_FAILURE;
    }
    if (po.po_type == ZMI_PO_MISH) {
      // refused where the reference refuses it (lowoha_matmul_utils.cpp:379-408): source scales per row or per
      // K group on s8 rows (is_sym_quant_config, lowoha_matmul_utils.hpp:184-204), dynamic quantization, W4A8;
      // the static scale chain computes it
      const bool sym_quant = p.dt_src == ZMI_DT_S8 && p.dt_wei == ZMI_DT_S8 && !p.src_zp.buff &&
                             (p.dt_dst == ZMI_DT_F32 || p.dt_dst == ZMI_DT_BF16) && shape_elems(p.src_scale) > 1;
      const bool w4a8 = p.dt_wei == ZMI_DT_S4 && p.dynamic_quant;
      if (sym_quant || is_dynamic_quant_config(p) || w4a8) {
        set_error("mish is not supported with per-row / per-group source scales, dynamic quantization or W4A8");
        return ZMI_FAILURE;
      }
    }
  }
  return ZMI_SUCCESS;
}

bool is_dynamic_quant_config(const zmi_matmul_params_t &p) {
  // reference: is_dynamic_quant_config, matmul/lowoha_matmul_utils.hpp:215-230
  return p.dynamic_quant && p.dt_wei == ZMI_DT_S8 && (p.dt_src == ZMI_DT_BF16 || p.dt_src == ZMI_DT_F32) &&
         (p.dt_compute == ZMI_DT_S8 || p.dt_compute == ZMI_DT_U8);
}

// Translates the quantization parameters and post-ops of one call into the
// kernels' shared epilogue descriptor (*out) and the per-problem operands
// (scale / zero-point / bias fields of *prob).  Returns a ZMI_* status.
int32_t build_epilogue(const zmi_matmul_params_t &p, int M, int N, float alpha, float beta, const void *bias,
                       ZmiEpilogue *out, ZmiProblem *prob, bool allow_wei_zp) {
  ZmiEpilogue e;
  std::memset(&e, 0, sizeof(e));
  e.alpha = alpha;
  e.beta = beta;
  e.dst_dt = p.dt_dst;
  prob->bias = bias;
  prob->src_scale_ptr = nullptr; prob->wei_scale_ptr = nullptr; prob->src_zp_ptr = nullptr;
  prob->src_scale_val = 1.0f; prob->wei_scale_val = 1.0f; prob->src_zp_val = 0;
  e.bias_dt = p.dt_bias == ZMI_DT_NONE ? ZMI_DT_F32 : p.dt_bias;
  if (bias && !(e.bias_dt == ZMI_DT_F32 || e.bias_dt == ZMI_DT_BF16 || e.bias_dt == ZMI_DT_S32 ||
                e.bias_dt == ZMI_DT_S8)) {
    set_error("unsupported bias dtype");
    return ZMI_UNIMPLEMENTED;
  }
  // source scale
  e.src_scale_mode = ZMI_SS_NONE;
  if (p.src_scale.buff) {
    const int64_t n = nelems(p.src_scale);
    e.src_scale_dt = p.src_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p.src_scale.dt;
    if (e.src_scale_dt != ZMI_DT_F32 && e.src_scale_dt != ZMI_DT_BF16) {
      set_error("source scale must be f32 or bf16");
      return ZMI_UNIMPLEMENTED;
    }
    if (n == 1) {
      const void *dp;
      if (!scalar_param_f32(p.src_scale.buff, e.src_scale_dt, &prob->src_scale_val, &dp)) return ZMI_FAILURE;
      prob->src_scale_ptr = dp;
      e.src_scale_mode = dp ? ZMI_SS_TENSOR_PTR : ZMI_SS_VALUE;
    } else if (n == M) {
      prob->src_scale_ptr = p.src_scale.buff;
      e.src_scale_mode = ZMI_SS_TOKEN_PTR;
    } else if (n > M && n % M == 0) {
      // {M, G}: one scale per row and K group (lowoha_matmul_utils.cpp:262-270)
      prob->src_scale_ptr = p.src_scale.buff;
      e.src_scale_mode = ZMI_SS_GROUP_PTR;
      e.n_groups = (int32_t)(n / M);
    } else {
      set_error("source scale must be per-tensor, per-token {M,1} or per-group {M,G}");
      return ZMI_FAILURE;
    }
  }
  // weight scale
  if (p.wei_scale.buff) {
    const int64_t n = nelems(p.wei_scale);
    e.wei_scale_dt = p.wei_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p.wei_scale.dt;
    if (e.wei_scale_dt != ZMI_DT_F32 && e.wei_scale_dt != ZMI_DT_BF16) {
      set_error("weight scale must be f32 or bf16");
      return ZMI_UNIMPLEMENTED;
    }
    if (n == 1) {
      const void *dp;
      if (!scalar_param_f32(p.wei_scale.buff, e.wei_scale_dt, &prob->wei_scale_val, &dp)) return ZMI_FAILURE;
      prob->wei_scale_ptr = dp;
      e.wei_scale_mode = 1;
    } else if (n == N && e.n_groups == 0) {
      prob->wei_scale_ptr = p.wei_scale.buff;
      e.wei_scale_mode = 2;
    } else if (e.n_groups > 0 && n == (int64_t)e.n_groups * N) {
      prob->wei_scale_ptr = p.wei_scale.buff;
      e.wei_scale_mode = 3;
    } else if (e.n_groups > 0) {
      // lowoha_matmul_utils.cpp:292-301
      set_error("source scales per K-group: the weight scale must hold groups x N elements");
      return ZMI_FAILURE;
    } else {
      set_error("per-group weight scales need a per-group source scale ({M,G} with the same G)");
      return ZMI_UNIMPLEMENTED;
    }
  }
  if (e.n_groups > 0 && e.wei_scale_mode != 3) {
    set_error("per-group source scale requires a per-group weight scale of G * N elements");
    return ZMI_FAILURE;
  }
  if (p.wei_zp.buff) {
    // one zero-point for the whole weight tensor, read as an integer whatever its dtype (reference: read_and_cast in
    // aocl_kernel.cpp:982-985); a single matmul_direct problem with s8 / u8 rows only
    if (!allow_wei_zp || e.n_groups > 0) {
      set_error("a weight zero-point is implemented for single problems with s8 / u8 sources and per-tensor or per-channel scales");
      return ZMI_UNIMPLEMENTED;
    }
    if (p.wei_zp.dt != ZMI_DT_S8 && p.wei_zp.dt != ZMI_DT_U8 && p.wei_zp.dt != ZMI_DT_S32) {
      set_error("weight zero-point: s8, u8 or s32");
      return ZMI_FAILURE;
    }
    prob->wei_zp_dt = p.wei_zp.dt;
    if (is_device_pointer(p.wei_zp.buff)) {
      prob->wei_zp_ptr = p.wei_zp.buff;
    } else {
      prob->wei_zp_val = p.wei_zp.dt == ZMI_DT_S8 ? (int32_t)*(const int8_t *)p.wei_zp.buff
                         : p.wei_zp.dt == ZMI_DT_U8 ? (int32_t)*(const uint8_t *)p.wei_zp.buff : *(const int32_t *)p.wei_zp.buff;
    }
  }
  if (p.src_zp.buff) {
    if (!scalar_param_s32(p.src_zp.buff, p.src_zp.dt, &prob->src_zp_val, &prob->src_zp_ptr)) return ZMI_FAILURE;
    e.has_zp = 1;
  }
  if (p.dst_scale.buff || p.dst_zp.buff) {
    e.has_dst_q = 1;
    e.dst_scale_val = 1.0f;
    e.dst_zp_val = 0.0f;
    e.dst_scale_dt = p.dst_scale.dt;
    e.dst_zp_dt = p.dst_zp.dt;
    if (p.dst_scale.buff && !scalar_param_f32(p.dst_scale.buff, p.dst_scale.dt, &e.dst_scale_val, &e.dst_scale_ptr))
      return ZMI_FAILURE;
    if (p.dst_zp.buff && !scalar_param_f32(p.dst_zp.buff, p.dst_zp.dt, &e.dst_zp_val, &e.dst_zp_ptr))
      return ZMI_FAILURE;
    if (!p.dst_zp.buff) e.dst_zp_val = 0.0f;
  }
  // post-ops (normalised like lowoha_matmul.cpp:335-356: leading_dim -1 -> N,
  // reversed clip bounds swapped)
  int n_po = 0;
  for (int i = 0; i < p.n_postops; ++i) {
    const zmi_post_op_t &po = p.postops[i];
    if (po.po_type == ZMI_PO_NONE) continue;
    if (n_po >= ZMI_MAX_PO) { set_error("too many post-ops"); return ZMI_UNIMPLEMENTED; }
    ZmiPostOp &d = e.po[n_po];
    d.type = po.po_type;
    d.alpha = po.alpha;
    d.beta = po.beta;
    switch (po.po_type) {
    case ZMI_PO_RELU: case ZMI_PO_LEAKY_RELU: case ZMI_PO_GELU_TANH: case ZMI_PO_GELU_ERF:
    case ZMI_PO_SIGMOID: case ZMI_PO_SWISH: case ZMI_PO_TANH:
      break;
    // The reference's AOCL wiring drops these types without a word (backends/aocl/aocl_postop.cpp:476-479, the
    // fault its validator already refuses mish for); here they compute what the reference's own kernel defines
    // (operators/matmul/matmul_ref_kernel.cpp:694-751; elu's alpha is the post-op's alpha).
    case ZMI_PO_ELU: case ZMI_PO_SQUARE: case ZMI_PO_ABS: case ZMI_PO_SQRT: case ZMI_PO_EXP: case ZMI_PO_LOG:
      break;
    // (the validator has refused it on the paths where the reference does)
    case ZMI_PO_MISH:
      break;
    case ZMI_PO_CLIP:
      if (d.alpha > d.beta) { float t = d.alpha; d.alpha = d.beta; d.beta = t; }
      break;
    case ZMI_PO_BINARY_ADD: case ZMI_PO_BINARY_MUL: {
      if (!po.buff) { set_error("binary post-op without operand"); return ZMI_FAILURE; }
      d.buff = po.buff;
      d.dtype = po.dtype == ZMI_DT_NONE ? ZMI_DT_F32 : po.dtype;
      if (d.dtype != ZMI_DT_F32 && d.dtype != ZMI_DT_BF16 && d.dtype != ZMI_DT_F16 && d.dtype != ZMI_DT_S32 &&
          d.dtype != ZMI_DT_S8 && d.dtype != ZMI_DT_U8) {
        set_error("binary post-op operand: f32, bf16, f16, s32, s8 or u8");
        return ZMI_UNIMPLEMENTED;
      }
      d.ld = po.leading_dim > 0 ? po.leading_dim : N;
      const bool row = (po.ndims == 2 && po.dims[0] == 1 && po.dims[1] == N) || (po.ndims == 1 && po.dims[0] == N);
      const bool full = po.ndims == 2 && po.dims[0] == M && po.dims[1] == N;
      if (!row && !full) { set_error("binary post-op operand must be {1,N} or {M,N}"); return ZMI_UNIMPLEMENTED; }
      d.rowb = row ? 1 : 0;
      break;
    }
    default:
      // (softmax and pooling are not element-wise)
      set_error("post-op type not implemented on the int8 path");
      return ZMI_UNIMPLEMENTED;
    }
    ++n_po;
  }
  e.n_po = n_po;
  e.fast_kind = ZMI_EK_GENERIC;
  if (alpha == 1.0f && beta == 0.0f && !e.has_dst_q && n_po <= 1 && (p.dt_dst == ZMI_DT_BF16 || p.dt_dst == ZMI_DT_F32)) {
    if (n_po == 0) e.fast_kind = ZMI_EK_NONE;
    else if (e.po[0].type == ZMI_PO_SWISH) e.fast_kind = ZMI_EK_SWISH;
    else if (e.po[0].type == ZMI_PO_GELU_TANH) e.fast_kind = ZMI_EK_GELU_TANH;
    else if (e.po[0].type == ZMI_PO_RELU) e.fast_kind = ZMI_EK_RELU;
  }
  *out = e;
  return ZMI_SUCCESS;
}

// Kernel choice for one problem.  Measured on MI355X with K = 4096 (us per call, bf16 rows
// quantized per token, bf16 out), N = 4096 / 14336:
//   rows   decode kernel   small-M kernel   ring (K-sliced)
//     32     12 / 23         14 / 24          28 / 35
//     64     17 / 34         21 / 35          28 / 36
//    128     23 / 58         36 / 74          34 / 45
// The decode kernel reads every row once per 32-column block (the rows cross L2 N / 32
// times), the ring kernel once per 256 columns but needs three launches when it slices K:
// up to 64 rows, and up to 128 rows while the output is narrow, the decode kernel wins.
static bool wide_output(int M, int N) { return (int64_t)M * N >= 96 * 8192; }

static bool decode_kernel_allowed(int M, int N, int K) {
  // ZMI_DECODE_MAX_M (0 .. 128) caps the rows the decode kernel takes; the tests use it to
  // reach the other kernels with few rows
  int max_m = 128;
  if (const char *env = zmi_env(ZE_DECODE_MAX_M)) max_m = std::atoi(env);
  if (zmi_env(ZE_NO_DECODE_KERNEL)) max_m = 0;
  if (M > max_m || M > 128 || zmi_blob_kpad(K) > 4096) return false;
  return M <= 64 || !wide_output(M, N);
}

// Up to 16 rows with K beyond the decode kernel's 4096: its 16-row form in K slices (partial sums + a small reduction).
// (ZMI_NO_DECODE_SLICED: the small-M kernel instead, as before the sliced form existed.)
static bool decode_sliced_allowed(int M, int N, int K) {
  (void)N;
  int max_m = 16;
  if (const char *env = zmi_env(ZE_DECODE_MAX_M)) max_m = std::min(max_m, std::atoi(env));
  if (zmi_env(ZE_NO_DECODE_KERNEL) || zmi_env(ZE_NO_DECODE_SLICED)) max_m = 0;
  return M <= max_m && zmi_blob_kpad(K) > 4096 && zmi_decode16_slices(M, K, zmi_round_up(K, 16)) >= 2;
}

// Tile height and K slices of a one-problem ring launch.  ZMI_GEMM_TOP (128 / 256) and
// ZMI_RING_SPLITK (1 = never slice, n = n slices) override the choice; the tests use them
// to reach every kernel configuration with small shapes.
ZmiRingPlan plan_ring_gemm(int M, int N, int K) {
  int top_hint = 0, force = 0;
  if (const char *env = zmi_env(ZE_GEMM_TOP)) {
    const int v = std::atoi(env);
    if (v == 128 || v == 256) top_hint = v;
    if (v == 64) top_hint = 64 | 0x10000;   // (ZMI_RING_PAD)
  }
  if (const char *env = zmi_env(ZE_RING_SPLITK)) force = std::atoi(env);
  return zmi_ring_plan(M, N, K, top_hint, force);
}

// Whether a launch may quantize its own rows and hand them over inside the launch.  Not under stream capture: the
// hand-off names the launch by a per-thread number baked into the kernel arguments, and a replayed graph would find
// the flags of its first run already stamped (the quantization is then a launch of its own, which replays correctly).
static bool fused_quant_allowed() {
  if (zmi_env(ZE_NO_FUSED_QUANT)) return false;
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream(), &cs) != hipSuccess) { (void)hipGetLastError(); return true; }
  return cs == hipStreamCaptureStatusNone;
}

// The persistent form of the large-M kernel (k_pring.hip) or the tiled one (k_ring.hip)?  Both last as long as their
// busiest compute unit, so the two are priced in units of one 256 x 256 tile (main loop and epilogue, K = 4096:
// 62 us) and the cheaper one takes the call; the persistent form also takes a tie when M fills its 256-row bands.
//   persistent: the launch's own cell assignment is walked (k_pring.hip: XCDs by column, an XCD's cells split evenly
//   over its compute units, tiles of 1 .. 4 cells that never cross a band) with a tile of 1 / 2 / 3 / 4 cells at
//   0.40 / 0.57 / 0.78 / 1;
//   tiled: 256-row tiles 1 per round of one tile per compute unit; 128-row tiles 0.57 while there is at most one per
//   compute unit and 0.95 per round of two (the second workgroup on a unit hides the first one's epilogue, no more);
//   64-row tiles 0.40 and 0.60.
// The prices are from these measurements on MI355X (K = 4096, whole call in us, tiled / persistent): M x N =
// 2048 x 4096 51.7 / 47.7, 1024 x 4096 39.1 / 35.1, 2048 x 2048 41.6 / 38.4, 512 x 14336 48.0 / 45.3, 768 x 14336
// 68.8 / 62.5, 1300 x 14336 138.7 / 103.5, 1536 x 14336 130.7 / 106.7, 2048 x 14336 138.0 / 126.7, 4096 x 14336
// 266.9 / 243.8, 2048 x 5000 69.4 / 61.0 (persistent cheaper or tie); 1536 x 4096 49.2 / 58.5, 1100 x 4096 42.7 / 53.5,
// 600 x 8192 42.8 / 51.3, 1100 x 14336 78.0 / 87.4, 300 x 14336 41.7 / 42.7 (tiled cheaper, or a tie with a partly
// filled band).  ZMI_PRING = 0 / 1 overrides the choice.
static double pring_price(int M, int N) {
  static const double tile_price[5] = {0.0, 0.40, 0.57, 0.78, 1.0};
  const int np = (int)(zmi_blob_npad(N) / 64), bands = (M + 255) / 256;
  const int cpx = std::max(1, zmi_cu_count() / 8);
  double worst = 0.0;
  for (int x = 0; x < 8; ++x) {
    const int wx = (int)((int64_t)(x + 1) * np / 8) - (int)((int64_t)x * np / 8);
    if (wx <= 0) continue;
    const int64_t cells = (int64_t)wx * bands;
    for (int j = 0; j < cpx; ++j) {
      int u = (int)(cells * j / cpx);
      const int u1 = (int)(cells * (j + 1) / cpx);
      double price = 0.0;
      while (u < u1) {
        const int band_end = (u / wx + 1) * wx;
        const int n = std::min(u1, band_end) - u;
        const int k = (n + 3) / 4;
        const int ni = (n + k - 1) / k;
        price += tile_price[ni];
        u += ni;
      }
      worst = std::max(worst, price);
    }
  }
  return worst;
}

static double ring_price(int M, int N, int top) {
  const int th = top & 0xffff;
  if (th <= 0) return 1e30;
  const int64_t n_cu = zmi_cu_count();
  const int64_t tiles = (int64_t)((M + th - 1) / th) * ((N + 255) / 256);
  if (th == 256) return (double)((tiles + n_cu - 1) / n_cu);
  const double alone = th == 128 ? 0.57 : 0.40, paired = th == 128 ? 0.95 : 0.60;
  if (tiles <= n_cu) return alone;
  return (double)((tiles + 2 * n_cu - 1) / (2 * n_cu)) * paired;
}

// (shape only: what the call's epilogue and alignment allow is zmi_pring_takes)
static bool pring_cheaper(int M, int N, int ring_top) {
  if (const char *env = zmi_env(ZE_PRING)) return std::atoi(env) != 0;
  if (M < 256 || zmi_env(ZE_GEMM_TOP)) return false;   // (a forced tile height asks for the tiled form)
  const double mine = pring_price(M, N), other = ring_price(M, N, ring_top);
  return mine < other - 1e-9 || (mine < other + 1e-9 && M % 256 == 0);
}

static bool pring_wanted(const ZmiProblem &prob, const ZmiEpilogue &epi, int ring_top) {
  return zmi_pring_takes(prob, epi) && pring_cheaper(prob.M, prob.N, ring_top);
}

int32_t run_single_gemm(const ZmiProblem &prob, const ZmiEpilogue &epi, const ZmiRingPlan *plan) {
  if (decode_kernel_allowed(prob.M, prob.N, prob.K)) {
    set_kernel_name(zmi_decode_16row_kernel(prob, false) ? "decode16_dma_rows_mfma16x16x64" : "decode_lds_rows_mfma16x16x64");
    if (!hip_ok(zmi_launch_gemm_decode(prob, epi, nullptr, stream()), "decode GEMM launch")) return ZMI_FAILURE;
  } else if (decode_sliced_allowed(prob.M, prob.N, prob.K) && zmi_decode16_slices(prob.M, prob.K, prob.lda) >= 2) {
    // (the scratch arena was sized for the partial sums by the caller)
    int32_t *partial = (int32_t *)arena().alloc(zmi_decode16_partial_bytes(prob.M, prob.N, prob.K));
    if (!partial) { set_error("no scratch for the K-sliced decode GEMM"); return ZMI_FAILURE; }
    set_kernel_name("decode16_ksliced_dma_rows_mfma16x16x64");
    if (!hip_ok(zmi_launch_gemm_decode(prob, epi, nullptr, stream(), partial, slice_arrivals(zmi_blob_npad(prob.N) / 32)),
                "decode GEMM launch"))
      return ZMI_FAILURE;
  } else if (!use_ring_kernel(prob.M, prob.N, prob.K)) {
    set_kernel_name("smallm_splitk_mfma16x16x64");
    if (!hip_ok(zmi_launch_gemm_smallm(prob, epi, stream()), "small-M GEMM launch")) return ZMI_FAILURE;
  } else {
    // prob.A is fragment-major here (see use_ring_kernel)
    if (!plan) { set_error("ring GEMM without a launch plan"); return ZMI_FAILURE; }
    ZmiRingSplit split = {1, nullptr, nullptr};
    if (plan->slices > 1) {
      // (the scratch arena was sized for the partial tiles by the caller)
      split.slices = plan->slices;
      split.partial = (int32_t *)arena().alloc(plan->partial_bytes);
      if (!split.partial) { set_error("no scratch for the K-sliced GEMM"); return ZMI_FAILURE; }
      // (null: a reduction launch finishes the elements -- also with a weight zero-point, whose per-row term only
      // the reduction's element-finishing code adds)
      split.arrivals = prob.row_comp ? nullptr : slice_arrivals(plan->tiles);
    }
    if (plan->slices == 1 && pring_wanted(prob, epi, plan->top)) {
      set_kernel_name("pring_mfma32x32x32_persistent");
      if (!hip_ok(zmi_launch_gemm_pring(prob, epi, stream()), "persistent MFMA GEMM launch")) return ZMI_FAILURE;
      return ZMI_SUCCESS;
    }
    const int th = plan->top & 0xffff;
    set_kernel_name(plan->slices > 1 ? (th == 64 ? "ring_mfma32x32x32_top64_ksliced" : "ring_mfma32x32x32_top128_ksliced")
                                     : (th == 256 ? "ring_mfma32x32x32_top256"
                                                  : th == 64 ? "ring_mfma32x32x32_top64" : "ring_mfma32x32x32_top128"));
    const ZmiRingSide side = side_stream();
    if (!hip_ok(zmi_launch_gemm_ring(prob, epi, plan->top, &split, stream(), &side), "MFMA GEMM launch")) return ZMI_FAILURE;
  }
  return ZMI_SUCCESS;
}

// Problems with more rows than the small-M kernels take run on the MFMA-bound
// kernel, which reads the activations in fragment-major order.
bool use_ring_kernel(int M, int N, int K) {
  if (decode_kernel_allowed(M, N, K) || decode_sliced_allowed(M, N, K)) return false;
  // ZMI_RING_MIN_M overrides the choice (the tests reach the 64-row tile through it)
  if (const char *env = zmi_env(ZE_RING_MIN_M)) {
    const int min_m = std::atoi(env);
    if (min_m > 0) return M >= min_m;
  }
  // (33 .. 128 rows with K beyond the decode kernel's: the small-M kernel multiplies every weight chunk by up to
  // eight row blocks out of L2 and falls behind the K-sliced tiles: K = 14336, N = 4096: M = 64 48 us against 35,
  // M = 128 93 against 41)
  if (zmi_blob_kpad(K) > 4096) return M > 32;
  return M > 128 || (M > 64 && wide_output(M, N));
}

// rows from which the per-group GEMM takes the MFMA-tiled kernel (ZMI_PGRING_MIN_M overrides; 0 turns it off)
int pgring_min_rows() {
  if (const char *env = zmi_env(ZE_PGRING_MIN_M)) {
    const int v = std::atoi(env);
    return v > 0 ? v : 0x7fffffff;
  }
  return 129;
}

bool a_needs_repack(const void *A, int64_t lda, int K, bool transA) {
  return transA || (K % 16) != 0 || (lda % 16) != 0 || (((uintptr_t)A) % 16) != 0;
}


// W4A8 (bf16 source quantized at run time, packed s4 weights with {G,N} scales, bf16 destination):
// validate_w4a8_inputs, matmul/lowoha_matmul_utils.cpp:72-176, in its order.  Other uses of s4 weights
// (weight-only quantization with bf16 compute) are not part of this library.
int32_t validate_w4a8(const zmi_matmul_params_t &p, int M, int N, int K) {
  if (p.dt_src == ZMI_DT_S8) { set_error("s4 weights with an s8 source: the 4-bit path quantizes a bf16 source itself (set dynamic_quant)"); return ZMI_FAILURE; }
  if (p.dynamic_quant && (p.dt_src == ZMI_DT_F32 || p.dt_dst == ZMI_DT_F32)) { set_error("s4 weights with dynamic_quant: source and destination must both be bf16 (f32 given)"); return ZMI_FAILURE; }
  if (p.dt_src == ZMI_DT_U8 && (p.src_scale.buff || p.dynamic_quant)) { set_error("s4 weights with a u8 source: the 4-bit path is symmetric and starts from bf16"); return ZMI_FAILURE; }
  const bool entry = p.dynamic_quant && p.dt_src == ZMI_DT_BF16;
  if (entry && p.dt_compute != ZMI_DT_S8) { set_error("s4 weights with dynamic_quant: dt_compute must be s8"); return ZMI_FAILURE; }
  if (!entry) { set_error("s4 weights go with a bf16 source: with dynamic_quant and s8 compute (W4A8), or without dynamic_quant (weight-only quantization)"); return ZMI_FAILURE; }
  if (p.dt_dst != ZMI_DT_BF16) { set_error("s4 weights with dynamic_quant: dt_dst must be bf16"); return ZMI_FAILURE; }
  if (p.wei_zp.buff || p.src_zp.buff) { set_error("s4 weights with dynamic_quant: zero-points are not taken (weights and source are symmetric)"); return ZMI_FAILURE; }
  const zmi_quant_t &ws = p.wei_scale;
  if (!ws.buff) { set_error("s4 weights with dynamic_quant: wei_scale.buff is missing"); return ZMI_FAILURE; }
  if (ws.dt != ZMI_DT_F32 && ws.dt != ZMI_DT_BF16) { set_error("s4 weights with dynamic_quant: wei_scale.dt must be f32 or bf16"); return ZMI_FAILURE; }
  if (ws.ndims != 2) { set_error("s4 weights with dynamic_quant: wei_scale must be two-dimensional, {groups, N}"); return ZMI_FAILURE; }
  const int64_t G = ws.dims[0];
  if (G <= 0 || ws.dims[1] != N) { set_error("s4 weights with dynamic_quant: wei_scale dims must be {groups >= 1, N}"); return ZMI_FAILURE; }
  if (K % G != 0) { set_error("s4 weights with dynamic_quant: the weight scale groups do not divide K"); return ZMI_FAILURE; }
  if ((K / G) % 4 != 0) { set_error("s4 weights with dynamic_quant: a scale group must span a multiple of 4 values of K"); return ZMI_FAILURE; }
  const zmi_quant_t &ss = p.src_scale;
  if (ss.dt != ZMI_DT_F32 && ss.dt != ZMI_DT_BF16) { set_error("s4 weights with dynamic_quant: src_scale.dt must be f32 or bf16"); return ZMI_FAILURE; }
  if (ss.ndims != 2) { set_error("s4 weights with dynamic_quant: src_scale must be two-dimensional"); return ZMI_FAILURE; }
  const int64_t r = ss.dims[0], c = ss.dims[1];
  if (!((r == 1 && c == 1) || (r == M && c == 1) || (r == M && c == G))) {
    set_error("s4 weights with dynamic_quant: src_scale dims must be {1,1} (tensor), {M,1} (row) or {M,groups}");
    return ZMI_FAILURE;
  }
  return ZMI_SUCCESS;
}

}  // namespace zmi

using namespace zmi;

extern "C" {

void zmi_matmul_params_init(zmi_matmul_params_t *p) {
  std::memset(p, 0, sizeof(*p));
  p->mem_format_a = 'n';
  p->mem_format_b = 'n';
  p->lowoha_algo = ZMI_ALGO_NONE;
  p->weight_cache_type = 2;
}

void zmi_batch_params_init(zmi_batch_params_t *p) {
  p->Batch_A = 1;
  p->Batch_B = 1;
  p->batch_stride_src = p->batch_stride_wei = p->batch_stride_dst = (uint64_t)-1;
}

void zmi_reorder_params_init(zmi_reorder_params_t *p) {
  std::memset(p, 0, sizeof(*p));
  p->algo = 0;  // reorder_algo_t::DT
  p->prepack.algo = ZMI_ALGO_NONE;
}

// groups of a dynamic call's source scale dims ({M,G} with G > 1), else 0
static int64_t pg_groups_of(const zmi_matmul_params_t &p, int M) {
  int64_t n = 1;
  for (int i = 0; i < p.src_scale.ndims; ++i) n *= p.src_scale.dims[i];
  return n > M && n % M == 0 ? n / M : 0;
}

// One matrix product (Batch_A == Batch_B == 1): everything matmul_direct does for one (src, weight, dst).
static int32_t matmul_single(char layout, int32_t transA, int32_t transB, int32_t M, int32_t N, int32_t K,
                             float alpha, const void *src, int32_t lda, const void *weight, int32_t ldb,
                             const void *bias, float beta, void *dst, int32_t ldc, int32_t is_weights_const,
                             const zmi_matmul_params_t &p) {
  const int Batch_A = 1, Batch_B = 1;
  if (is_woq_config(p))
    return matmul_woq(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc, is_weights_const, p);
  const bool w4a8 = p.dt_wei == ZMI_DT_S4;
  if (w4a8) {
    // (the shape rules of this path keep the kernels inside their buffers: checked whatever the diagnostics switch says)
    if (!src || !weight || !dst || M <= 0 || N <= 0 || K <= 0) { set_error("null pointer or non-positive dimension"); return ZMI_FAILURE; }
    int32_t st = validate_w4a8(p, M, N, K);
    if (st != ZMI_SUCCESS) return st;
    // (the general validator's post-op rule, lowoha_matmul_utils.cpp:379-408, for this path)
    for (int i = 0; i < p.n_postops; ++i)
      if (p.postops[i].po_type == ZMI_PO_MISH) {
        set_error("mish is not supported with per-row / per-group source scales, dynamic quantization or W4A8");
        return ZMI_FAILURE;
      }
    if (p.pack_format_b != 0 || p.mem_format_b == 'r') { set_error("s4 weights are passed as plain packed nibbles (mem_format_b 'n', no pack format)"); return ZMI_FAILURE; }
  } else if (diagnostics_enabled()) {
    int32_t st = validate_matmul(src, weight, dst, M, N, K, Batch_A, Batch_B, p, is_weights_const != 0);
    if (st != ZMI_SUCCESS) return st;
  } else if (!src || !weight || !dst || M <= 0 || N <= 0 || K <= 0) {
    set_error("null pointer or non-positive dimension");
    return ZMI_FAILURE;
  }
  // ---- what this library implements of matmul_direct: the int8 path ----
  if (p.dt_wei != ZMI_DT_S8 && !w4a8) { set_error("weights: s8, s4 (W4A8, or weight-only with a bf16 source) or u4 (weight-only with a bf16 source)"); return ZMI_UNIMPLEMENTED; }
  if (layout != 'r' && layout != 'R') { set_error("only row-major layout is implemented"); return ZMI_UNIMPLEMENTED; }
  const bool ggml = p.pack_format_b == 1;
  if (p.pack_format_b != 0 && !ggml) { set_error("unknown pack_format_b"); return ZMI_FAILURE; }
  if (ggml) {
    // reference: validate_ggml_packed_inputs, matmul/ggml_weight_unpack.cpp:155-183
    if (!is_weights_const) { set_error("GGML packed weights require constant weights"); return ZMI_FAILURE; }
    if (!transB) { set_error("GGML packed weights require transB = true (the packed layout is N x K)"); return ZMI_FAILURE; }
    if (K % 32 != 0) { set_error("GGML packed weights: K must be a multiple of 32"); return ZMI_FAILURE; }
    if (p.mem_format_b == 'r') { set_error("GGML packed weights are unpacked and reordered by the library (mem_format_b must be 'n')"); return ZMI_FAILURE; }
  }
  if (p.mem_format_b == 'r' && p.lowoha_algo != ZMI_ALGO_AOCL_DLP_BLOCKED) {
    // contract of the reference: prepacked weights require the blocked algo
    set_error("mem_format_b == 'r' requires lowoha_algo == aocl_dlp_blocked");
    return ZMI_FAILURE;
  }
  const bool dyn = w4a8 || is_dynamic_quant_config(p);
  if (!dyn && p.dt_src != ZMI_DT_S8 && p.dt_src != ZMI_DT_U8) {
    set_error("source must be u8 / s8, or bf16 / f32 with dynamic_quant and an s8 compute type");
    return ZMI_UNIMPLEMENTED;
  }
  if (dyn && p.dt_compute == ZMI_DT_U8) {
    // Dynamic asymmetric quantization of the source to u8 (matmul/quantization/reorder_quantization.cpp:60-75, 208-230:
    // scale and zero-point dims and types are required, their buffers optional).  The GEMM reads ONE source zero-point
    // (backends/aocl/aocl_kernel.cpp:971-980), so the granularity that means something is per tensor: the source
    // becomes u8 rows with one scale and one zero-point in device memory, and the call goes on as a static u8 call.
    if (w4a8 || pg_groups_of(p, M) || nelems(p.src_scale) != 1 || p.src_zp.ndims <= 0 || nelems(p.src_zp) != 1) {
      set_error("dynamic quantization to u8: one source scale and one source zero-point (dims {1} / {1,1}) are implemented");
      return ZMI_UNIMPLEMENTED;
    }
    if (p.src_zp.dt != ZMI_DT_S32) { set_error("dynamic quantization to u8: src_zp.dt must be s32"); return ZMI_FAILURE; }
    const int32_t sdt = p.src_scale.dt;
    if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("dynamic quantization: src_scale.dt must be f32 or bf16"); return ZMI_FAILURE; }
    if (transA) { set_error("dynamic quantization of a transposed source is not implemented"); return ZMI_UNIMPLEMENTED; }
    if (lda < K) { set_error("leading dimension too small"); return ZMI_FAILURE; }
    if ((p.src_scale.buff && !is_device_pointer(p.src_scale.buff)) || (p.src_zp.buff && !is_device_pointer(p.src_zp.buff))) {
      set_error("dynamic quantization to u8 writes src_scale / src_zp: device memory (or null: the library keeps them)");
      return ZMI_FAILURE;
    }
    if (!ensure_device()) return ZMI_FAILURE;
    // (its own scratch: the static call that follows lays out the thread's arena anew)
    static thread_local Arena rows;
    const size_t qb = Arena::padded((size_t)M * K), lb = Arena::padded(sizeof(float) * 2 * (size_t)M);
    if (!rows.begin(qb + lb + 3 * 256)) return ZMI_FAILURE;
    uint8_t *q = (uint8_t *)rows.alloc(qb);
    float *lohi = (float *)rows.alloc(lb);
    float *s32 = (float *)rows.alloc(4);
    void *s16 = rows.alloc(2);
    int32_t *zp = (int32_t *)rows.alloc(4);
    if (!q || !lohi || !s32 || !s16 || !zp) { set_error("no scratch for the quantized source"); return ZMI_FAILURE; }
    float *scale_f32 = sdt == ZMI_DT_F32 && p.src_scale.buff ? (float *)p.src_scale.buff : s32;
    void *scale_bf16 = sdt == ZMI_DT_BF16 ? (p.src_scale.buff ? (void *)p.src_scale.buff : s16) : nullptr;
    int32_t *zp_out = p.src_zp.buff ? (int32_t *)p.src_zp.buff : zp;
    if (!hip_ok(zmi_launch_quant_asym_tensor(src, p.dt_src, M, K, lda, q, K, lohi, scale_f32, zp_out, scale_bf16, sdt, stream()),
                "asymmetric quantization launch"))
      return ZMI_FAILURE;
    zmi_matmul_params_t ip = p;
    ip.dt_src = ZMI_DT_U8;
    ip.dynamic_quant = 0;
    ip.src_scale.buff = sdt == ZMI_DT_BF16 ? (const void *)scale_bf16 : (const void *)scale_f32;   // (the GEMM reads the narrowed value)
    ip.src_scale.ndims = 1; ip.src_scale.dims[0] = 1;
    ip.src_zp.buff = zp_out;
    ip.src_zp.ndims = 1; ip.src_zp.dims[0] = 1;
    return matmul_single(layout, 0, transB, M, N, K, alpha, q, K, weight, ldb, bias, beta, dst, ldc, is_weights_const, ip);
  }
  if (lda < (transA ? M : K) || ldc < N || ldb < (transB ? K : N)) {
    if (p.mem_format_b != 'r' || lda < (transA ? M : K) || ldc < N) { set_error("leading dimension too small"); return ZMI_FAILURE; }
  }
  int64_t dyn_scale_n = 0;
  if (dyn) {
    dyn_scale_n = 1;
    for (int i = 0; i < p.src_scale.ndims; ++i) dyn_scale_n *= p.src_scale.dims[i];
    if (!(dyn_scale_n == 1 || dyn_scale_n == M || (dyn_scale_n > M && dyn_scale_n % M == 0 && K % (dyn_scale_n / M) == 0))) {
      set_error("dynamic source scale dims must be {1}, {M,1} or {M,G} with K divisible by G");
      return ZMI_FAILURE;
    }
    if (p.src_zp.buff) { set_error("dynamic quantization is symmetric: no source zero-point"); return ZMI_FAILURE; }
    if (transA) { set_error("dynamic quantization of a transposed source is not implemented"); return ZMI_UNIMPLEMENTED; }
  }
  // per-group scales ({M,G} source, {G,N} weights): G slices of K (lowoha_matmul_utils.cpp:262-301)
  int64_t pg_groups = 0;
  if (dyn) {
    if (dyn_scale_n > M) pg_groups = dyn_scale_n / M;
  } else if (p.src_scale.buff) {
    const int64_t n = nelems(p.src_scale);
    if (n > M && n % M == 0) pg_groups = n / M;
  }
  // W4A8 with one source scale per tensor or per row: the source is quantized that way, then the scales are
  // repeated over the weights' G groups and the per-group GEMM follows (broadcast_w4a8_src_scale,
  // matmul/backends/aocl/aocl_kernel.cpp:167-236).  G == 1 is the plain per-channel chain.
  const bool bcast_src = w4a8 && pg_groups == 0 && p.wei_scale.dims[0] > 1;
  if (bcast_src) pg_groups = p.wei_scale.dims[0];
  // (K = 32 is one packed block per column: {M,1} source scales ARE {M, K / 32}; one group of 32)
  if (ggml && K == 32 && pg_groups == 0 && M > 1 && (dyn ? dyn_scale_n : (p.src_scale.buff ? nelems(p.src_scale) : 0)) == M)
    pg_groups = 1;
  if (ggml) {
    // reference: ggml_is_sym_quant (ggml_weight_unpack.cpp:142-153), checked after the source was quantized:
    // s8 (or dynamically quantized) source, symmetric, more than one source scale, f32 / bf16 destination
    const bool src_ok = dyn || p.dt_src == ZMI_DT_S8;
    const int64_t sn = dyn ? dyn_scale_n : (p.src_scale.buff ? nelems(p.src_scale) : 0);
    if (!src_ok || p.src_zp.buff || sn <= 1 || !(p.dt_dst == ZMI_DT_F32 || p.dt_dst == ZMI_DT_BF16)) {
      set_error("GGML packed weights are supported only for symmetric per-group int8 matmul");
      return ZMI_FAILURE;
    }
    if (pg_groups != K / 32) {
      // (the packed scales are one per 32 k: the source scales must be {M, K / 32})
      set_error("GGML packed weights: source scale dims must be {M, K / 32}");
      return pg_groups ? ZMI_FAILURE : ZMI_UNIMPLEMENTED;
    }
  }
  if (pg_groups) {
    if (K % pg_groups != 0) { set_error("per-group source scale: K must be divisible by the number of groups"); return ZMI_FAILURE; }
    if (p.src_zp.buff) { set_error("per-group source scales are symmetric: no source zero-point"); return ZMI_FAILURE; }
    if (p.dt_src == ZMI_DT_U8) { set_error("per-group source scales need an s8 / bf16 / f32 source"); return ZMI_FAILURE; }
    if (p.dt_dst != ZMI_DT_F32 && p.dt_dst != ZMI_DT_BF16) { set_error("per-group source scales need an f32 / bf16 destination"); return ZMI_FAILURE; }
    if (!ggml && (!p.wei_scale.buff || nelems(p.wei_scale) != pg_groups * N)) {
      set_error("per-group source scale requires a per-group weight scale of G * N elements");
      return ZMI_FAILURE;
    }
    if (!zmi_pergroup_group_size_ok(K / pg_groups)) {
      set_error("per-group scales: group sizes of 16, 32 or a multiple of 64 are implemented");
      return ZMI_UNIMPLEMENTED;
    }
  }
  if (!ensure_device()) return ZMI_FAILURE;
  if (dyn && p.src_scale.buff && !is_device_pointer(p.src_scale.buff)) {
    // with dynamic_quant the scale buffer is an OUTPUT that the kernels write
    set_error("dynamic_quant: src_scale.buff receives the computed scales and must be device memory (or null)");
    return ZMI_FAILURE;
  }

  // ---- scratch plan ----
  const bool use_cache = !ggml && p.mem_format_b != 'r' && is_weights_const &&
                         std::min(weight_cache_env(), p.weight_cache_type) > 0;
  const bool pack_in_arena = !ggml && p.mem_format_b != 'r' && !use_cache;
  const size_t widen_bytes = w4a8 && pack_in_arena ? (size_t)K * (size_t)N : 0;
  const int64_t K16 = zmi_round_up(K, 16);
  const bool ring = !pg_groups && use_ring_kernel(M, N, K);
  const int64_t frag_kpad = ring ? zmi_blob_kpad(K) : 0;
  const size_t a_bytes = ring ? (size_t)zmi_afrag_bytes(M, K) : (size_t)M * K16;
  const bool repack_a = !dyn && (ring || a_needs_repack(src, lda, K, transA != 0));
  size_t need = 0;
  if (pack_in_arena) need += Arena::padded((size_t)zmi_blob_bytes(K, N));
  if (widen_bytes) need += Arena::padded(widen_bytes);
  if (bcast_src) need += Arena::padded(sizeof(float) * (size_t)M * (size_t)pg_groups);
  if (dyn) need += Arena::padded(a_bytes) + Arena::padded(sizeof(float) * (size_t)M * (size_t)(pg_groups ? pg_groups : 1)) + 256;
  if (repack_a) need += Arena::padded(a_bytes);
  // a weight zero-point: one compensation word per row, and the kernels that finish their elements through
  // zmi_finish_element (the decode and small-M kernels; the large-M kernel in K slices with its reduction launch)
  const bool wzp = p.wei_zp.buff != nullptr;
  if (wzp && (dyn || pg_groups || ggml || w4a8)) {
    set_error("a weight zero-point is implemented for s8 / u8 sources and per-tensor or per-channel scales");
    return ZMI_UNIMPLEMENTED;
  }
  if (wzp) need += Arena::padded(sizeof(int32_t) * (size_t)M);
  ZmiRingPlan plan = {};
  if (ring) {
    plan = plan_ring_gemm(M, N, K);
    if (wzp && plan.slices < 2) plan = zmi_ring_plan(M, N, K, 0, 2);
    need += Arena::padded(plan.partial_bytes);
  }
  if (!pg_groups && decode_sliced_allowed(M, N, K)) need += Arena::padded(zmi_decode16_partial_bytes(M, N, K));
  // per-group scales at large M: fragment-order rows, f32 weight scales in padded rows, f32 source scales
  const bool pgring = pg_groups && M >= pgring_min_rows() && zmi_pgring_takes(M, N, K, K / pg_groups);
  if (pgring)
    need += Arena::padded((size_t)zmi_afrag_bytes(M, K)) +
            Arena::padded(sizeof(float) * (size_t)pg_groups * (size_t)zmi_pgring_ws_cols(N)) +
            Arena::padded(sizeof(float) * (size_t)M * (size_t)pg_groups);
  if (!arena().begin(need)) return ZMI_FAILURE;

  // ---- weights ----
  const uint8_t *blob;
  const void *ggml_scales = nullptr;
  const uint8_t *tiles_s4 = nullptr;
  if (ggml) {
    blob = packed_ggml_q8_0(weight, K, N, &ggml_scales);
    if (!blob) return ZMI_FAILURE;
  } else if (p.mem_format_b == 'r') {
    if (!blob_matches(weight, K, N)) return ZMI_FAILURE;
    blob = (const uint8_t *)weight;
  } else if (w4a8) {
    void *wide = widen_bytes ? arena().alloc(widen_bytes) : nullptr;
    void *slot = pack_in_arena ? arena().alloc((size_t)zmi_blob_bytes(K, N)) : nullptr;
    blob = packed_s4_weights(weight, K, N, ldb, transB != 0, use_cache, wide, slot, &tiles_s4);
    if (!blob) return ZMI_FAILURE;
  } else {
    void *slot = pack_in_arena ? arena().alloc((size_t)zmi_blob_bytes(K, N)) : nullptr;
    blob = packed_weights(weight, K, N, ldb, transB != 0, p.dt_src, use_cache, slot);
    if (!blob) return ZMI_FAILURE;
  }

  // ---- source ----
  zmi_matmul_params_t ep = p;   // working copy: the caller's struct is never modified
  if (ggml) {
    // the unpack sets the weight scales: bf16, {K / 32, N} (ggml_weight_unpack.cpp:412-420)
    ep.wei_scale.buff = ggml_scales;
    ep.wei_scale.dt = ZMI_DT_BF16;
    ep.wei_scale.ndims = 2; ep.wei_scale.dims[0] = K / 32; ep.wei_scale.dims[1] = N;
  }
  ZmiProblem prob;
  std::memset(&prob, 0, sizeof(prob));
  prob.blob = blob;
  prob.dst = dst;
  prob.ldc = ldc;
  prob.M = M; prob.N = N; prob.K = K;
  ZmiFusedQuant fused;
  std::memset(&fused, 0, sizeof(fused));
  bool use_fused = false;
  int8_t *a_frag = nullptr;   // per-group GEMM at large M: the rows in fragment order, once they exist
  if (dyn) {
    // reference: reorder_quantization_wrapper, matmul/quantization/reorder_quantization.cpp:43-280
    int8_t *q = (int8_t *)arena().alloc(a_bytes);
    float *sc = (float *)arena().alloc(sizeof(float) * (size_t)M * (size_t)(pg_groups && !bcast_src ? pg_groups : 1));
    unsigned int *amax = (unsigned int *)arena().alloc(256);
    // bytes of q between K and K16 stay unwritten: the blob's rows beyond K are zero
    int32_t sdt = p.src_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p.src_scale.dt;
    if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("source scale must be f32 or bf16"); return ZMI_FAILURE; }
    prob.A = q; prob.lda = K16;
    const bool per_token = (dyn_scale_n == M && M > 1) || M == 1;
    // decode shapes: quantization fused into the GEMM launch when its whole grid is resident at once
    const bool decode_kernel = decode_kernel_allowed(M, N, K);
    // (the decode kernel's producers are its first workgroups and wait for nothing, so its grid need not be resident)
    if (pg_groups && !bcast_src) {
      // reference: the per-group dynamic reorder in front of the sym-quant GEMM
      // (matmul/quantization/reorder_quantization.cpp:43-280 with {M,G} scale dims)
      if (zmi_pergroup_decode_shape(prob, (int)pg_groups) && fused_quant_allowed()) {
        // decode shapes: the quantization is part of the GEMM launch (its first M workgroups)
        if (!fused_handoff(&fused)) return ZMI_FAILURE;
        fused.x = src; fused.ldx = lda; fused.x_dt = p.dt_src;
        fused.q = q; fused.ldq = K16; fused.scales = sc;
        fused.user_scales = (void *)p.src_scale.buff; fused.user_dt = sdt;
        use_fused = true;
      } else if (pgring && zmi_quant_groups_frag_ok(src, p.dt_src, K, lda, pg_groups)) {
        // large M: the quantized rows go straight into MFMA fragment order
        a_frag = (int8_t *)arena().alloc((size_t)zmi_afrag_bytes(M, K));
        if (!hip_ok(zmi_launch_quant_groups_frag(src, p.dt_src, M, K, lda, pg_groups, a_frag, sc, (void *)p.src_scale.buff, sdt,
                                                 stream()), "per-group quant launch"))
          return ZMI_FAILURE;
      } else if (!hip_ok(zmi_launch_quant_groups(src, p.dt_src, M, K, lda, pg_groups, q, K16, sc, (void *)p.src_scale.buff,
                                                 sdt, stream()), "per-group quant launch")) {
        return ZMI_FAILURE;
      }
      ep.src_scale.buff = sc;
      ep.src_scale.dt = ZMI_DT_F32;
      ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = pg_groups;
    } else if (bcast_src && per_token && K % 4 == 0 && zmi_pergroup_decode_shape(prob, (int)pg_groups) &&
               fused_quant_allowed()) {
      // W4A8 decode shapes with one scale per row: the per-token quantization is part of the per-group GEMM
      // launch, whose workgroups read the row's scale for every group (no broadcast copy)
      if (!fused_handoff(&fused)) return ZMI_FAILURE;
      fused.x = src; fused.ldx = lda; fused.x_dt = p.dt_src;
      fused.q = q; fused.ldq = K16; fused.scales = sc;
      fused.user_scales = (void *)p.src_scale.buff; fused.user_dt = sdt;
      fused.per_row = 1;
      use_fused = true;
      ep.src_scale.buff = sc;
      ep.src_scale.dt = ZMI_DT_F32;
      ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = pg_groups;
    } else if (per_token && !bcast_src && !ring && M <= 128 && K % 4 == 0 && (decode_kernel || zmi_smallm_grid(prob) <= 512) &&
               !decode_sliced_allowed(M, N, K) && fused_quant_allowed()) {
      // (the K-sliced decode kernel takes quantized rows: with the quantization of 14336-element rows inside the
      // launch its workgroups wait longer than the separate launch costs -- 32 against 22 us)
      if (!fused_handoff(&fused)) return ZMI_FAILURE;
      fused.x = src; fused.ldx = lda; fused.x_dt = p.dt_src;
      fused.q = q; fused.ldq = K16; fused.scales = sc;
      fused.user_scales = (void *)p.src_scale.buff; fused.user_dt = sdt;
      use_fused = true;
      ep.src_scale.buff = sc;
      ep.src_scale.dt = ZMI_DT_F32;
      ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = 1;
    } else if (dyn_scale_n == M && (M > 1 || decode_sliced_allowed(M, N, K))) {
      // (one row in front of the K-sliced decode kernel: the row kernel, one launch, instead of the per-tensor pair)
      void *scale_out = p.src_scale.buff ? (void *)p.src_scale.buff : (void *)sc;
      // (without a caller buffer the scales live in scratch, in the dtype the params name: the reference allocates
      // its own buffer of that dtype, reorder_quantization.cpp:103-117, and its GEMM reads the narrowed values back)
      if (!hip_ok(zmi_launch_quant_rows(src, p.dt_src, M, K, lda, q, K16, frag_kpad, scale_out, sdt, stream()), "quant launch"))
        return ZMI_FAILURE;
      ep.src_scale.buff = scale_out;
      ep.src_scale.dt = sdt;
      ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = 1;
    } else {
      // one scale for the whole tensor; with M == 1 this is the per-token case too
      if (!hip_ok(zmi_launch_quant_tensor(src, p.dt_src, M, K, lda, q, K16, frag_kpad, sc, amax, stream()), "quant launch"))
        return ZMI_FAILURE;
      if (sdt == ZMI_DT_BF16) {
        // a bf16 scale dtype: the GEMM multiplies by the narrowed value, which also goes to the caller's buffer
        if (!hip_ok(zmi_launch_narrow_scales(sc, M, (void *)p.src_scale.buff, 1, stream()), "scale narrowing launch"))
          return ZMI_FAILURE;
      } else if (p.src_scale.buff) {
        if (!hip_ok(hipMemcpyAsync((void *)p.src_scale.buff, sc, sizeof(float), hipMemcpyDeviceToDevice, stream()),
                    "hipMemcpyAsync(scale)"))
          return ZMI_FAILURE;
      }
      ep.src_scale.buff = sc;
      ep.src_scale.dt = ZMI_DT_F32;
      ep.src_scale.ndims = 1; ep.src_scale.dims[0] = 1;
    }
    if (bcast_src && !use_fused) {
      float *wide = (float *)arena().alloc(sizeof(float) * (size_t)M * (size_t)pg_groups);
      if (!hip_ok(zmi_launch_broadcast_scales(ep.src_scale.buff, ep.src_scale.dt, ep.src_scale.ndims == 1, M, pg_groups,
                                              wide, stream()), "scale broadcast launch"))
        return ZMI_FAILURE;
      ep.src_scale.buff = wide;
      ep.src_scale.dt = ZMI_DT_F32;
      ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = pg_groups;
    }
    prob.A = q; prob.lda = K16; prob.a_is_u8 = 0;
    ep.dt_src = ZMI_DT_S8;
    ep.dt_wei = ZMI_DT_S8;   // (the s4 codes were widened)
  } else if (repack_a) {
    int8_t *a2 = (int8_t *)arena().alloc(a_bytes);
    if (ring) {
      if (!hip_ok(zmi_launch_repack_frag(src, M, K, lda, transA != 0, p.dt_src == ZMI_DT_U8, a2, stream()), "repack launch")) return ZMI_FAILURE;
    } else {
      if (!hip_ok(zmi_launch_pad_rows(src, M, K, lda, transA != 0, a2, K16, stream()), "pad launch")) return ZMI_FAILURE;
    }
    prob.A = a2; prob.lda = K16; prob.a_is_u8 = p.dt_src == ZMI_DT_U8;
  } else {
    prob.A = src; prob.lda = lda; prob.a_is_u8 = p.dt_src == ZMI_DT_U8;
  }

  ZmiEpilogue epi;
  int32_t st = build_epilogue(ep, M, N, alpha, beta, bias, &epi, &prob, true);
  if (st != ZMI_SUCCESS) return st;
  if (wzp && (prob.wei_zp_ptr || prob.wei_zp_val != 0)) {
    int32_t *rc = (int32_t *)arena().alloc(sizeof(int32_t) * (size_t)M);
    if (!rc) { set_error("no scratch for the weight zero-point compensation"); return ZMI_FAILURE; }
    if (!hip_ok(zmi_launch_row_comp(src, lda, transA != 0, p.dt_src == ZMI_DT_U8, M, K, prob.wei_zp_val, prob.wei_zp_ptr,
                                    prob.wei_zp_dt, prob.src_zp_val, prob.src_zp_ptr, rc, stream()), "zero-point compensation launch"))
      return ZMI_FAILURE;
    prob.row_comp = rc;
  }
  if (epi.n_groups > 0 && pgring && !use_fused) {
    const int64_t G = epi.n_groups, np = zmi_pgring_ws_cols(N);
    int8_t *af = a_frag ? a_frag : (int8_t *)arena().alloc((size_t)zmi_afrag_bytes(M, K));
    float *wsp = (float *)arena().alloc(sizeof(float) * (size_t)G * (size_t)np);
    const float *ssp = (const float *)prob.src_scale_ptr;
    bool ok = (a_frag || hip_ok(zmi_launch_repack_frag(prob.A, M, K, prob.lda, 0, 0, af, stream()), "repack launch")) &&
              hip_ok(zmi_launch_pgring_scales(prob.wei_scale_ptr, epi.wei_scale_dt, G, N, np, wsp, stream()), "scale launch");
    if (ok && epi.src_scale_dt != ZMI_DT_F32) {
      float *wide = (float *)arena().alloc(sizeof(float) * (size_t)M * (size_t)G);
      ok = hip_ok(zmi_launch_pgring_scales(prob.src_scale_ptr, epi.src_scale_dt, M, G, G, wide, stream()), "scale launch");
      ssp = wide;
    }
    prob.A = af;
    set_kernel_name("pergroup_ring_mfma32x32x32");
    st = ok && hip_ok(zmi_launch_gemm_pgring(prob, epi, ssp, wsp, stream()), "per-group GEMM launch") ? ZMI_SUCCESS : ZMI_FAILURE;
  } else if (epi.n_groups > 0) {
    const bool s4_stream = tiles_s4 && zmi_pergroup_s4_shape(prob, epi.n_groups);
    set_kernel_name(s4_stream ? (use_fused ? (fused.per_row ? "pergroup_decode_s4_mfma16x16x64 (fused per-token quant)" : "pergroup_decode_s4_mfma16x16x64 (fused per-group quant)") : "pergroup_decode_s4_mfma16x16x64")
                    : use_fused ? "pergroup_decode_mfma16x16x64 (fused per-group quant)"
                    : zmi_pergroup_decode_shape(prob, epi.n_groups) ? "pergroup_decode_mfma16x16x64" : "pergroup_mfma16x16x64");
    st = hip_ok(zmi_launch_gemm_pergroup(prob, epi, use_fused ? &fused : nullptr, stream(), tiles_s4), "per-group GEMM launch")
             ? ZMI_SUCCESS : ZMI_FAILURE;
  } else if (use_fused) {
    // a one-row scale in device memory reads like a per-token scale
    if (epi.src_scale_mode == ZMI_SS_TENSOR_PTR) epi.src_scale_mode = ZMI_SS_TOKEN_PTR;
    if (decode_kernel_allowed(prob.M, prob.N, prob.K)) {
      set_kernel_name(zmi_decode_selfq_takes(prob, &fused) ? "decode16x2_selfquant_mfma16x16x64 (per-token quant in the workgroup)"
                      : zmi_decode_16row_kernel(prob, true) && fused.flags_uncached ? "decode16_dma_rows_mfma16x16x64 (fused per-token quant)"
                                                            : "decode_lds_rows_mfma16x16x64 (fused per-token quant)");
      st = hip_ok(zmi_launch_gemm_decode(prob, epi, &fused, stream()), "fused decode GEMM launch") ? ZMI_SUCCESS : ZMI_FAILURE;
    } else {
      set_kernel_name("smallm_splitk_mfma16x16x64 (fused per-token quant)");
      st = hip_ok(zmi_launch_gemm_smallm_fused(prob, epi, fused, stream()), "fused small-M GEMM launch") ? ZMI_SUCCESS : ZMI_FAILURE;
    }
  } else {
    st = run_single_gemm(prob, epi, ring ? &plan : nullptr);
  }
  upload_fence();
  return st;
}

// bytes of one element (s4 weights never reach the batched form)
static size_t dt_bytes(int32_t dt) {
  switch (dt) {
  case ZMI_DT_F32: case ZMI_DT_S32: return 4;
  case ZMI_DT_BF16: case ZMI_DT_F16: case ZMI_DT_S16: return 2;
  case ZMI_DT_S64: return 8;
  default: return 1;
  }
}

// matmul_direct: one product, or the batched form.  Reference for the batched form: bmm_execute,
// matmul/partitioning/bmm/looper/bmm_looper.cpp:192-223 (strides: the caller's in elements, or derived from the
// dimensions when (size_t)-1) and :326-340 (batch b reads src batch b % Batch_A, weight batch b % Batch_B --
// index 0 when that side has one batch -- and writes dst batch b); every batch runs with the same parameters
// except binary post-op operands with a leading batch dimension > 1, which advance by dims[1] * dims[2]
// elements per batch (apply_bmm_postop_offsets, matmul/lowoha_matmul_utils.cpp:36-70).  Here the batches are
// launches on the one stream, in order.
int32_t zmi_matmul_direct(char layout, int32_t transA, int32_t transB, int32_t M, int32_t N, int32_t K,
                          float alpha, const void *src, int32_t lda, const void *weight, int32_t ldb,
                          const void *bias, float beta, void *dst, int32_t ldc, int32_t is_weights_const,
                          const zmi_batch_params_t *batch_params, const zmi_matmul_params_t *params) {
  clear_error();
  note_operand(src); note_operand(weight); note_operand(dst); note_operand(bias);
  if (async_failure_pending()) return ZMI_FAILURE;
  if (!params) { set_error("null params"); return ZMI_FAILURE; }
  const zmi_matmul_params_t &p = *params;
  const int Batch_A = batch_params ? batch_params->Batch_A : 1;
  const int Batch_B = batch_params ? batch_params->Batch_B : 1;
  if (Batch_A == 1 && Batch_B == 1) {
    // (3-D binary operands of one batch read like 2-D ones)
    bool has_3d = false;
    for (int i = 0; i < p.n_postops; ++i) has_3d = has_3d || p.postops[i].ndims == 3;
    if (!has_3d)
      return matmul_single(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc, is_weights_const, p);
  }
  if (diagnostics_enabled() && p.dt_wei != ZMI_DT_S4) {
    int32_t st = validate_matmul(src, weight, dst, M, N, K, Batch_A, Batch_B, p, is_weights_const != 0);
    if (st != ZMI_SUCCESS) return st;
  } else if (!src || !weight || !dst || M <= 0 || N <= 0 || K <= 0 || Batch_A <= 0 || Batch_B <= 0) {
    set_error("null pointer or non-positive dimension");
    return ZMI_FAILURE;
  }
  const int batch_count = Batch_A > Batch_B ? Batch_A : Batch_B;
  if (batch_count > 1) {
    if (p.dt_wei != ZMI_DT_S8) { set_error("batched matmul: only s8 weights are implemented"); return ZMI_UNIMPLEMENTED; }
    if (p.dynamic_quant) {
      // (the reference quantizes the {Batch_A, M, K} source as one 3-D tensor in front of the batches,
      // matmul/quantization/reorder_quantization.cpp:126-137)
      set_error("batched matmul with dynamic_quant is not implemented");
      return ZMI_UNIMPLEMENTED;
    }
    if (p.pack_format_b != 0) { set_error("GGML packed weights do not take a weight batch"); return ZMI_FAILURE; }
    if (p.mem_format_b == 'r' && Batch_B > 1 && batch_params->batch_stride_wei == (uint64_t)-1) {
      set_error("batched prepacked weights need batch_stride_wei (bytes from one packed buffer to the next)");
      return ZMI_FAILURE;
    }
  }
  const uint64_t none = (uint64_t)-1;
  const uint64_t s_src = batch_params && batch_params->batch_stride_src != none ? batch_params->batch_stride_src
                                                                                : (uint64_t)(transA ? K : M) * (uint64_t)lda;
  const uint64_t s_wei = batch_params && batch_params->batch_stride_wei != none ? batch_params->batch_stride_wei
                                                                                : (uint64_t)(transB ? N : K) * (uint64_t)ldb;
  const uint64_t s_dst = batch_params && batch_params->batch_stride_dst != none ? batch_params->batch_stride_dst
                                                                                : (uint64_t)M * (uint64_t)ldc;
  const size_t src_b = s_src * dt_bytes(p.dt_src), wei_b = s_wei * dt_bytes(p.dt_wei), dst_b = s_dst * dt_bytes(p.dt_dst);
  for (int b = 0; b < batch_count; ++b) {
    zmi_matmul_params_t bp = p;
    std::vector<zmi_post_op_t> pos(p.postops, p.postops + (p.postops ? p.n_postops : 0));
    bp.postops = pos.data();
    for (size_t i = 0; i < pos.size(); ++i) {
      zmi_post_op_t &po = pos[i];
      if ((po.po_type != ZMI_PO_BINARY_ADD && po.po_type != ZMI_PO_BINARY_MUL) || !po.buff || po.ndims != 3) continue;
      const int32_t odt = po.dtype == ZMI_DT_NONE ? ZMI_DT_F32 : po.dtype;
      if (po.dims[0] > 1) {
        if (po.dims[0] < batch_count) { set_error("binary post-op operand has fewer batches than the product"); return ZMI_FAILURE; }
        po.buff = (uint8_t *)po.buff + (size_t)b * (size_t)(po.dims[1] * po.dims[2]) * dt_bytes(odt);
      }
      po.ndims = 2; po.dims[0] = po.dims[1]; po.dims[1] = po.dims[2]; po.dims[2] = 0;
    }
    const uint8_t *a = (const uint8_t *)src + (size_t)(Batch_A == 1 ? 0 : b % Batch_A) * src_b;
    const uint8_t *w = (const uint8_t *)weight + (size_t)(Batch_B == 1 ? 0 : b % Batch_B) * wei_b;
    uint8_t *c = (uint8_t *)dst + (size_t)b * dst_b;
    int32_t st = matmul_single(layout, transA, transB, M, N, K, alpha, a, lda, w, ldb, bias, beta, c, ldc, is_weights_const, bp);
    if (st != ZMI_SUCCESS) return st;
  }
  return ZMI_SUCCESS;
}

// ---- prepack ---------------------------------------------------------------------------------

// reference: validate_prepack_params, reorder/prepack/lowoha_prepack.cpp:53-96
static int32_t validate_prepack(const zmi_prepack_params_t &pp) {
  if (pp.K <= 0 || pp.N <= 0) { set_error("prepack: K and N must be positive"); return ZMI_FAILURE; }
  const int64_t min_ld = pp.transposed ? pp.K : pp.N;
  if (pp.ldb < min_ld) { set_error("prepack: ldb too small"); return ZMI_FAILURE; }
  if (pp.algo != ZMI_ALGO_AOCL_DLP_BLOCKED) { set_error("prepack: only aocl_dlp_blocked is supported"); return ZMI_UNIMPLEMENTED; }
  if (pp.wei_dtype != ZMI_DT_S8) { set_error("prepack: only s8 weights are implemented"); return ZMI_UNIMPLEMENTED; }
  return ZMI_SUCCESS;
}

int32_t zmi_large_m_plan(int32_t M, int32_t N, int32_t K, int32_t *tile_rows, int32_t *k_slices, int32_t *persistent) {
  clear_error();
  if (M <= 0 || N <= 0 || K <= 0 || !tile_rows || !k_slices || !persistent) { set_error("large_m_plan: bad arguments"); return ZMI_FAILURE; }
  *tile_rows = 0; *k_slices = 0; *persistent = 0;
  if (!use_ring_kernel(M, N, K)) return ZMI_SUCCESS;   // (the decode-shaped kernels take the call)
  const ZmiRingPlan plan = plan_ring_gemm(M, N, K);
  *tile_rows = plan.top & 0xffff;
  *k_slices = plan.slices;
  *persistent = plan.slices == 1 && N >= 64 && N % 4 == 0 && pring_cheaper(M, N, plan.top) ? 1 : 0;
  if (*persistent) *tile_rows = 256;
  return ZMI_SUCCESS;
}

size_t zmi_weight_prepack_size(zmi_reorder_params_t *params) {
  clear_error();
  if (!params) return 0;
  params->prepack.cached_size = 0;
  if (validate_prepack(params->prepack) != ZMI_SUCCESS) return 0;
  const size_t sz = (size_t)zmi_round_up(zmi_blob_bytes(params->prepack.K, params->prepack.N), 64);
  params->prepack.cached_size = sz;
  return sz;
}

static int32_t reorder_dynamic(const void *src, void *dst, zmi_reorder_params_t &rp) {
  // reference: validate_dynamic_quant_params + the fused per-token dispatch,
  // reorder/lowoha_reorder.cpp:60-204
  if (!src) { set_error("reorder: null src"); return ZMI_FAILURE; }
  if (rp.n_src_shape != 2) { set_error("dynamic quantization: only 2-D [M,K] shapes are implemented"); return ZMI_UNIMPLEMENTED; }
  if (rp.n_dst_shape != rp.n_src_shape || std::memcmp(rp.src_shape, rp.dst_shape, sizeof(int64_t) * rp.n_src_shape) != 0) {
    set_error("reorder: src_shape and dst_shape differ");
    return ZMI_FAILURE;
  }
  const int64_t M = rp.src_shape[0], K = rp.src_shape[1];
  if (M <= 0 || K <= 0) { set_error("reorder: non-positive shape"); return ZMI_FAILURE; }
  if (rp.dst_dtype != ZMI_DT_S8 && rp.dst_dtype != ZMI_DT_U8) {
    set_error("dynamic quantization: the destination must be s8 or u8");
    return ZMI_FAILURE;
  }
  if (!(rp.src_dtype == ZMI_DT_BF16 || rp.src_dtype == ZMI_DT_F32)) {
    set_error("dynamic quantization: only bf16 / f32 sources are implemented");
    return ZMI_UNIMPLEMENTED;
  }
  // a zero-point buffer selects the asymmetric form (reference: validate_dynamic_quant_params,
  // reorder/lowoha_reorder_utils.cpp:549-580: without one the destination must be s8, with one u8, s32 zero-points)
  const bool asym = rp.zero_point.buff != nullptr;
  if (!asym && rp.dst_dtype != ZMI_DT_S8) { set_error("dynamic quantization without a zero-point buffer is symmetric: s8 destination"); return ZMI_FAILURE; }
  if (asym) {
    if (rp.zero_point.ndims == 0) { set_error("asymmetric dynamic quantization: zero_point dims are required"); return ZMI_FAILURE; }
    if (rp.zero_point.dt != ZMI_DT_S32) { set_error("asymmetric dynamic quantization: zero-points are s32"); return ZMI_FAILURE; }
    if (rp.dst_dtype != ZMI_DT_U8) { set_error("asymmetric dynamic quantization: u8 destination"); return ZMI_FAILURE; }
  }
  if (!rp.scale.buff) { set_error("dynamic quantization: scale buffer is required"); return ZMI_FAILURE; }
  const int32_t sdt = rp.scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : rp.scale.dt;
  if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("dynamic quantization: scale must be f32 or bf16"); return ZMI_FAILURE; }
  int64_t ld = K;
  if (rp.n_src_strides == 2) {
    if (rp.src_strides[1] != 1 || rp.src_strides[0] < K) { set_error("dynamic quantization: rows must be contiguous"); return ZMI_UNIMPLEMENTED; }
    ld = rp.src_strides[0];
  } else if (rp.n_src_strides != 0) {
    set_error("reorder: strides do not match the shape");
    return ZMI_FAILURE;
  }
  const int64_t sn = nelems(rp.scale);
  if (!ensure_device()) return ZMI_FAILURE;
  if (asym) {
    // scale and zero-point share granularity and dims (lowoha_reorder_utils.cpp:644-658); per token {M,1} or per
    // group {M,G} along K
    if (rp.zero_point.ndims != rp.scale.ndims ||
        std::memcmp(rp.zero_point.dims, rp.scale.dims, sizeof(rp.scale.dims[0]) * rp.scale.ndims) != 0) {
      set_error("asymmetric dynamic quantization: scale and zero_point dims differ");
      return ZMI_FAILURE;
    }
    if (!(rp.scale.ndims == 2 && rp.scale.dims[0] == M && rp.scale.dims[1] >= 1 && rp.scale.dims[1] != K)) {
      set_error("asymmetric dynamic quantization: {M,1} and {M,G} scale dims are implemented");
      return ZMI_UNIMPLEMENTED;
    }
    const int64_t G = rp.scale.dims[1];
    if (K % G != 0) { set_error("dynamic quantization: per-group scale needs K divisible by the number of groups"); return ZMI_FAILURE; }
    float *sc = (float *)rp.scale.buff;
    void *user = nullptr;
    if (sdt != ZMI_DT_F32) {
      if (!arena().begin(Arena::padded(sizeof(float) * (size_t)(M * G)))) return ZMI_FAILURE;
      sc = (float *)arena().alloc(sizeof(float) * (size_t)(M * G));
      user = (void *)rp.scale.buff;
    }
    if (!hip_ok(zmi_launch_quant_asym(src, rp.src_dtype, M, K, ld, G, (uint8_t *)dst, K, sc, (int32_t *)rp.zero_point.buff, user,
                                      sdt, stream()), "asymmetric quant launch"))
      return ZMI_FAILURE;
    set_kernel_name(G == 1 ? "quant_asym_per_token" : "quant_asym_groups");
    return ZMI_SUCCESS;
  }
  if (rp.scale.ndims == 2 && rp.scale.dims[0] == M && rp.scale.dims[1] == 1) {
    if (!hip_ok(zmi_launch_quant_rows(src, rp.src_dtype, M, K, ld, (int8_t *)dst, K, 0, (void *)rp.scale.buff, sdt, stream()),
                "quant launch"))
      return ZMI_FAILURE;
    set_kernel_name("quant_rows_per_token");
    return ZMI_SUCCESS;
  }
  if (sn == 1) {
    if (sdt != ZMI_DT_F32) { set_error("per-tensor dynamic scale must be f32"); return ZMI_UNIMPLEMENTED; }
    if (!arena().begin(Arena::padded(sizeof(float) * (size_t)M) + 256)) return ZMI_FAILURE;
    float *sc = (float *)arena().alloc(sizeof(float) * (size_t)M);
    unsigned int *amax = (unsigned int *)arena().alloc(256);
    if (!hip_ok(zmi_launch_quant_tensor(src, rp.src_dtype, M, K, ld, (int8_t *)dst, K, 0, sc, amax, stream()), "quant launch"))
      return ZMI_FAILURE;
    if (!hip_ok(hipMemcpyAsync((void *)rp.scale.buff, sc, sizeof(float), hipMemcpyDeviceToDevice, stream()), "hipMemcpyAsync"))
      return ZMI_FAILURE;
    set_kernel_name("quant_tensor");
    return ZMI_SUCCESS;
  }
  // per-group along K: scale dims {M, G}, 1 < G < K, K % G == 0 (reference: is_per_group_col_dims and the
  // fused per-group dispatch, reorder/lowoha_reorder.cpp:167-171; dims rule lowoha_reorder_utils.cpp:180-211)
  if (rp.scale.ndims == 2 && rp.scale.dims[0] == M && rp.scale.dims[1] > 1 && rp.scale.dims[1] != K) {
    const int64_t G = rp.scale.dims[1];
    if (K % G != 0) { set_error("dynamic quantization: per-group scale needs K divisible by the number of groups"); return ZMI_FAILURE; }
    float *sc = (float *)rp.scale.buff;
    void *user = nullptr;
    if (sdt != ZMI_DT_F32) {
      if (!arena().begin(Arena::padded(sizeof(float) * (size_t)(M * G)))) return ZMI_FAILURE;
      sc = (float *)arena().alloc(sizeof(float) * (size_t)(M * G));
      user = (void *)rp.scale.buff;
    }
    if (!hip_ok(zmi_launch_quant_groups(src, rp.src_dtype, M, K, ld, G, (int8_t *)dst, K, sc, user, sdt, stream()),
                "per-group quant launch"))
      return ZMI_FAILURE;
    set_kernel_name("quant_groups");
    return ZMI_SUCCESS;
  }
  set_error("dynamic quantization: scale dims must be {1}, {M,1} or {M,G}");
  return ZMI_UNIMPLEMENTED;
}

int32_t zmi_reorder_direct(const void *src, void *dst, zmi_reorder_params_t *params) {
  clear_error();
  note_operand(src); note_operand(dst);
  if (!params) { set_error("null params"); return ZMI_FAILURE; }
  if (params->is_prepack) {
    // reference: weight_prepack_into, reorder/prepack/lowoha_prepack.cpp:315-373
    int32_t st = validate_prepack(params->prepack);
    if (st != ZMI_SUCCESS) return st;
    if (!src || !dst) { set_error("prepack: null weights or destination"); return ZMI_FAILURE; }
    if (!ensure_device()) return ZMI_FAILURE;
    const zmi_prepack_params_t &pp = params->prepack;
    if (!hip_ok(zmi_launch_prepack((const int8_t *)src, pp.K, pp.N, pp.ldb, pp.transposed, pp.src_dtype,
                                   pp.sym_group_size, (uint8_t *)dst, stream()), "prepack launch"))
      return ZMI_FAILURE;
    set_kernel_name("prepack_mfma_fragments");
    return ZMI_SUCCESS;
  }
  if (params->dynamic_quant) return reorder_dynamic(src, dst, *params);
  set_error("static reorder / dtype conversion modes are not part of this path");
  return ZMI_UNIMPLEMENTED;
}

int32_t zmi_group_dynamic_quant(int32_t n, const void *const *src, const int32_t *M, const int32_t *K,
                                const int64_t *src_row_stride, void *const *dst, const int64_t *dst_row_stride,
                                void *const *scale, const zmi_group_dq_params_t *params) {
  // reference: group_dynamic_quant, reorder/lowoha_reorder.cpp:279-404
  clear_error();
  if (!params || n <= 0 || !src || !M || !K || !dst || !scale) { set_error("group_dynamic_quant: bad arguments"); return ZMI_FAILURE; }
  for (int32_t i = 0; i < n; ++i) { note_operand(src[i]); note_operand(dst[i]); note_operand(scale[i]); }
  if (!(params->src_dtype == ZMI_DT_BF16 || params->src_dtype == ZMI_DT_F32) || params->dst_dtype != ZMI_DT_S8) {
    set_error("group_dynamic_quant: only bf16/f32 -> s8");
    return ZMI_FAILURE;
  }
  const int32_t sdt = params->scale_dtype == ZMI_DT_NONE ? ZMI_DT_F32 : params->scale_dtype;
  if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("group_dynamic_quant: scale must be f32 or bf16"); return ZMI_FAILURE; }
  if (params->num_groups > 1) {
    // per-group: every matrix gets {M[i], num_groups} scales (lowoha_reorder.cpp:318-393); one launch per matrix
    const int64_t G = params->num_groups;
    size_t need = 0;
    for (int i = 0; i < n; ++i) {
      if (M[i] < 0 || K[i] <= 0) { set_error("group_dynamic_quant: bad shape"); return ZMI_FAILURE; }
      if (M[i] == 0) continue;
      if (K[i] % G != 0) { set_error("group_dynamic_quant: per-group requires K % num_groups == 0"); return ZMI_FAILURE; }
      if (!src[i] || !dst[i] || !scale[i]) { set_error("group_dynamic_quant: null buffer for an active matrix"); return ZMI_FAILURE; }
      if (sdt != ZMI_DT_F32) need += Arena::padded(sizeof(float) * (size_t)(M[i] * G));
    }
    if (!ensure_device()) return ZMI_FAILURE;
    if (!arena().begin(need)) return ZMI_FAILURE;
    for (int i = 0; i < n; ++i) {
      if (M[i] == 0) continue;
      const int64_t lds_ = src_row_stride && src_row_stride[i] ? src_row_stride[i] : K[i];
      const int64_t ldd = dst_row_stride && dst_row_stride[i] ? dst_row_stride[i] : K[i];
      if (lds_ < K[i] || ldd < K[i]) { set_error("group_dynamic_quant: row stride smaller than K"); return ZMI_FAILURE; }
      float *sc = (float *)scale[i];
      void *user = nullptr;
      if (sdt != ZMI_DT_F32) { sc = (float *)arena().alloc(sizeof(float) * (size_t)(M[i] * G)); user = scale[i]; }
      if (!hip_ok(zmi_launch_quant_groups(src[i], params->src_dtype, M[i], K[i], lds_, G, (int8_t *)dst[i], ldd, sc, user, sdt,
                                          stream()), "per-group quant launch"))
        return ZMI_FAILURE;
    }
    set_kernel_name("quant_groups");
    return ZMI_SUCCESS;
  }
  std::vector<ZmiQuantMat> mats;
  int64_t rows = 0;
  for (int i = 0; i < n; ++i) {
    if (M[i] < 0 || K[i] <= 0) { set_error("group_dynamic_quant: bad shape"); return ZMI_FAILURE; }
    if (M[i] == 0) continue;
    if (!src[i] || !dst[i] || !scale[i]) { set_error("group_dynamic_quant: null buffer for an active matrix"); return ZMI_FAILURE; }
    ZmiQuantMat m = {};
    m.src = src[i]; m.dst = (int8_t *)dst[i]; m.scale = scale[i];
    m.ld_src = src_row_stride && src_row_stride[i] ? src_row_stride[i] : K[i];
    m.ld_dst = dst_row_stride && dst_row_stride[i] ? dst_row_stride[i] : K[i];
    if (m.ld_src < K[i] || m.ld_dst < K[i]) { set_error("group_dynamic_quant: row stride smaller than K"); return ZMI_FAILURE; }
    m.M = M[i]; m.K = K[i]; m.row_start = (int32_t)rows;
    rows += M[i];
    mats.push_back(m);
  }
  if (mats.empty()) return ZMI_SUCCESS;
  if (!ensure_device()) return ZMI_FAILURE;
  if (!arena().begin(0)) return ZMI_FAILURE;
  const ZmiQuantMat *dev = (const ZmiQuantMat *)upload(mats.data(), mats.size() * sizeof(ZmiQuantMat));
  if (!dev) return ZMI_FAILURE;
  bool ok = hip_ok(zmi_launch_quant_group(dev, (int)mats.size(), rows, params->src_dtype, sdt, 0, stream()), "quant launch");
  upload_fence();
  set_kernel_name("quant_rows_grouped");
  return ok ? ZMI_SUCCESS : ZMI_FAILURE;
}

}  // extern "C"
