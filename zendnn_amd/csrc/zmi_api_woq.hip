// matmul_direct, weight-only quantization: a bf16 source, s4 / u4 weights with scales (and zero-points), no
// dynamic_quant.  Reference: the WOQ branch of matmul_direct's AOCL wiring
// (lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:43-139 cvt_int4_to_bf16, :640-702 the cached bf16 matrix,
// :944-966 the call site) behind the rules of validate_matmul_direct_inputs
// (lowoha_operators/matmul/lowoha_matmul_utils.cpp:214-328).
#include <cstring>

#include "../../include/zmi_lowoha.h"
#include "zmi_api.h"

namespace zmi {

bool is_woq_config(const zmi_matmul_params_t &p) {
  // lowoha_matmul_utils.cpp:215-219
  return p.dt_src == ZMI_DT_BF16 && (p.dt_wei == ZMI_DT_S4 || p.dt_wei == ZMI_DT_U4) && !p.dynamic_quant;
}

int32_t matmul_woq(char layout, int32_t transA, int32_t transB, int32_t M, int32_t N, int32_t K, float alpha,
                   const void *src, int32_t lda, const void *weight, int32_t ldb, const void *bias, float beta, void *dst,
                   int32_t ldc, int32_t is_weights_const, const zmi_matmul_params_t &p) {
  // (these rules keep the kernel inside its buffers: checked whatever the diagnostics switch says)
  if (!src || !weight || !dst || M <= 0 || N <= 0 || K <= 0) { set_error("null pointer or non-positive dimension"); return ZMI_FAILURE; }
  if (!is_weights_const) { set_error("4-bit weights with a bf16 source (weight-only quantization) must be constant: is_weights_const"); return ZMI_FAILURE; }
  if (p.src_scale.buff || p.dst_scale.buff || p.src_zp.buff || p.dst_zp.buff) {
    set_error("weight-only quantization takes no source or destination scales / zero-points");
    return ZMI_FAILURE;
  }
  const bool u4 = p.dt_wei == ZMI_DT_U4;
  if (u4) {
    if (!p.wei_zp.buff) { set_error("u4 weights need wei_zp"); return ZMI_FAILURE; }
    if (p.wei_zp.dt != ZMI_DT_BF16 && p.wei_zp.dt != ZMI_DT_S8) { set_error("u4 weights: wei_zp.dt must be bf16 or s8"); return ZMI_FAILURE; }
  }
  if (p.dt_dst == ZMI_DT_F16) { set_error("a bf16 source does not go with an f16 destination"); return ZMI_FAILURE; }
  if (!p.wei_scale.buff) { set_error("weight-only quantization needs wei_scale"); return ZMI_FAILURE; }
  // ---- what is implemented of it ----
  if (layout != 'r' && layout != 'R') { set_error("only row-major layout is implemented"); return ZMI_UNIMPLEMENTED; }
  if (p.pack_format_b != 0 || p.mem_format_b == 'r') { set_error("4-bit weights are passed as plain packed nibbles (mem_format_b 'n', no pack format)"); return ZMI_FAILURE; }
  if (p.dt_dst != ZMI_DT_BF16 && p.dt_dst != ZMI_DT_F32) { set_error("weight-only quantization: dt_dst bf16 or f32"); return ZMI_UNIMPLEMENTED; }
  const int32_t sdt = p.wei_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p.wei_scale.dt;
  if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("wei_scale.dt must be f32 or bf16"); return ZMI_FAILURE; }
  if (lda < (transA ? M : K) || ldc < N || ldb < (transB ? K : N)) { set_error("leading dimension smaller than the row it strides"); return ZMI_FAILURE; }

  ZmiWoqProblem w;
  std::memset(&w, 0, sizeof(w));
  ZmiWoqParamSrc sc{nullptr, sdt, 0, 1.0f}, zp{nullptr, ZMI_DT_F32, 0, 0.0f};
  // scale granularity: one value, one per column, or {G, N} (cvt_int4_to_bf16's own reading of the element count)
  const int64_t ns = nelems(p.wei_scale);
  w.n_groups = 1;
  if (ns == 1) {
    if (!scalar_param_f32(p.wei_scale.buff, sdt, &sc.val, &sc.ptr)) return ZMI_FAILURE;
  } else if (ns == N) {
    sc.mode = 1;
    sc.ptr = p.wei_scale.buff;
  } else if (ns > N && ns % N == 0 && K % (ns / N) == 0) {
    sc.mode = 2;
    sc.ptr = p.wei_scale.buff;
    w.n_groups = (int32_t)(ns / N);
  } else {
    set_error("wei_scale must hold 1, N or groups x N elements, with groups dividing K");
    return ZMI_FAILURE;
  }
  w.group_size = K / w.n_groups;
  if (w.n_groups > 1 && w.group_size % 8 != 0) {
    set_error("weight-only quantization: a scale group must span a multiple of 8 values of K");
    return ZMI_UNIMPLEMENTED;
  }
  if (p.wei_zp.buff) {
    const int32_t zdt = p.wei_zp.dt;
    if (zdt != ZMI_DT_BF16 && zdt != ZMI_DT_S8 && zdt != ZMI_DT_U8 && zdt != ZMI_DT_S32 && zdt != ZMI_DT_F32) {
      set_error("wei_zp.dt: s8 or bf16 (u8, s32 and f32 are also read)");
      return ZMI_FAILURE;
    }
    const int64_t nz = nelems(p.wei_zp);
    w.has_zp = 1;
    zp.dt = zdt;
    w.zp_float_domain = u4 && zdt == ZMI_DT_BF16;
    if (nz == 1) {
      if (!scalar_param_f32(p.wei_zp.buff, zdt, &zp.val, &zp.ptr)) return ZMI_FAILURE;
    } else if (nz == N) {
      zp.mode = 1;
      zp.ptr = p.wei_zp.buff;
    } else if (sc.mode == 2 && nz == ns) {
      zp.mode = 2;
      zp.ptr = p.wei_zp.buff;
    } else {
      set_error("wei_zp must hold 1, N or as many elements as a per-group wei_scale");
      return ZMI_FAILURE;
    }
  }

  if (!ensure_device()) return ZMI_FAILURE;
  const bool use_cache = std::min(weight_cache_env(), p.weight_cache_type) > 0;
  const size_t tile_bytes = (size_t)zmi_woq_tiles_bytes(K, N);
  const size_t blob_bytes = tile_bytes + 2 * sizeof(float) * (size_t)w.n_groups * (size_t)N;
  if (!arena().begin(use_cache ? 0 : Arena::padded(blob_bytes))) return ZMI_FAILURE;
  void *slot = use_cache ? nullptr : arena().alloc(blob_bytes);
  if (!use_cache && !slot) { set_error("no scratch for the 4-bit weights"); return ZMI_FAILURE; }
  // (a cached weight keeps the scales and zero-points it was first seen with, like the reference's cached bf16 matrix)
  const uint8_t *blob = packed_woq_weights(weight, K, N, ldb, transB != 0, w.n_groups, sc, zp, use_cache, slot);
  if (!blob) return ZMI_FAILURE;
  w.tiles = (const uint32_t *)blob;
  w.sf = (const float *)(blob + tile_bytes);
  w.zf = w.sf + (size_t)w.n_groups * N;

  // alpha, beta, bias and the post-ops go the way of every other call; the quantization parameters are this path's own
  zmi_matmul_params_t ep = p;
  ep.src_scale = ep.wei_scale = ep.dst_scale = ep.src_zp = ep.wei_zp = ep.dst_zp = zmi_quant_t{};
  ZmiEpilogue epi;
  ZmiProblem prob;
  std::memset(&prob, 0, sizeof(prob));
  int32_t st = build_epilogue(ep, M, N, alpha, beta, bias, &epi, &prob);
  if (st != ZMI_SUCCESS) return st;

  w.A = src; w.lda = lda; w.transA = transA ? 1 : 0;
  w.a_fast = !transA && K % 8 == 0 && K >= 64 && lda % 8 == 0 && ((uintptr_t)src & 15) == 0 && (int64_t)M * lda < ((int64_t)1 << 30);
  w.dst = dst; w.ldc = ldc;
  w.M = M; w.N = N; w.K = K;
  w.is_u4 = u4 ? 1 : 0;
  w.bias = bias;
  const bool two = zmi_woq_blocks(w) == 2;
  set_kernel_name(u4 ? (two ? "woq_u4_dequant_mfma32x32x16_bf16 (two column blocks per workgroup)" : "woq_u4_dequant_mfma32x32x16_bf16")
                     : (two ? "woq_s4_dequant_mfma32x32x16_bf16 (two column blocks per workgroup)" : "woq_s4_dequant_mfma32x32x16_bf16"));
  st = hip_ok(zmi_launch_gemm_woq(w, epi, stream()), "weight-only GEMM launch") ? ZMI_SUCCESS : ZMI_FAILURE;
  upload_fence();
  return st;
}

}  // namespace zmi
