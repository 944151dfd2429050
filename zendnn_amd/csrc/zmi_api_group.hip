// C ABI: group_matmul_direct (independent expert GEMMs, gated activation,
// fused MoE Op1 -> act -> Op2, weighted reduce) and the device-side MoE glue.
#include <algorithm>
#include <cstring>
#include <vector>

#include "zmi_api.h"
#include "zmi_host.h"
#include "zmi_ring_table.h"

using namespace zmi;

namespace {

struct SizeCheck {
  size_t num_ops;
  bool relaxed;
  bool bad(size_t s) const { return relaxed ? s < num_ops : s != num_ops; }
};

// op2_k_for_act of the reference (group_matmul_parallel_common.hpp:202): a gated
// activation halves the width of Op1's output.
int op2_k_for_act(int N, int act) { return act != ZMI_ACT_NONE ? N / 2 : N; }

bool all_null(void *const *v, int n, size_t num_ops) {
  const size_t m = std::min((size_t)n, num_ops);
  for (size_t i = 0; i < m; ++i)
    if (v[i]) return false;
  return true;
}

// Always-on guards and the diagnostics validator of the reference
// (matmul/group_matmul_direct.cpp:185-699 and :768-1063), for the rules that do
// not depend on the CPU scheduling.  Every failure is status failure.
int32_t validate_group(const zmi_group_args_t &a, const zmi_moe_postop_t *postop, int gated_act,
                       const zmi_fused_moe_t *fm, size_t *num_ops_out, bool *op1_internal_out,
                       bool *op2_internal_out) {
  if (a.n_M <= 0 || a.n_params <= 0 || a.n_src <= 0) { set_error("group call: M, params and src must each hold at least one entry"); return ZMI_FAILURE; }
  const bool opt_in = a.params[0].active_matmul > 0;
  if (opt_in) {
    const uint32_t am = a.params[0].active_matmul, tm = a.params[0].total_matmul;
    if (am > (uint32_t)a.n_M) { set_error("group call: params[0].active_matmul counts more experts than M has entries"); return ZMI_FAILURE; }
    if (tm > 0 && tm < am) { set_error("group call: params[0].total_matmul is smaller than active_matmul"); return ZMI_FAILURE; }
  }
  const size_t num_ops = opt_in ? (size_t)a.params[0].active_matmul : (size_t)a.n_M;
  *num_ops_out = num_ops;
  const SizeCheck sc{num_ops, opt_in};

  // library-managed outputs: with fused_moe, dst (Op1) and dst_down (Op2) may
  // be empty / all null; a mix of null and non-null entries is an error
  bool op1_internal = false, op2_internal = false;
  if (fm) {
    if (a.n_dst == 0 || all_null(a.dst, a.n_dst, num_ops)) op1_internal = true;
    else {
      for (size_t i = 0; i < std::min((size_t)a.n_dst, num_ops); ++i)
        if (!a.dst[i] && i < (size_t)a.n_M && a.M[i] > 0) { set_error("fused_moe: dst entries of active experts must be all null (library scratch) or all set"); return ZMI_FAILURE; }
    }
    if (fm->n_dst_down == 0 || all_null(fm->dst_down, fm->n_dst_down, num_ops)) op2_internal = true;
    else {
      for (size_t i = 0; i < std::min((size_t)fm->n_dst_down, num_ops); ++i)
        if (!fm->dst_down[i] && i < (size_t)a.n_M && a.M[i] > 0) { set_error("fused_moe: dst_down entries of active experts must be all null (library scratch) or all set"); return ZMI_FAILURE; }
    }
  }
  *op1_internal_out = op1_internal;
  *op2_internal_out = op2_internal;

  if (sc.bad(a.n_N) || sc.bad(a.n_K) || sc.bad(a.n_weight) || sc.bad(a.n_lda) || sc.bad(a.n_ldb) ||
      sc.bad(a.n_layout) || sc.bad(a.n_transA) || sc.bad(a.n_transB) || sc.bad(a.n_alpha) || sc.bad(a.n_beta) ||
      sc.bad(a.n_bias) || sc.bad(a.n_is_weights_const) || sc.bad(a.n_params) ||
      (!op1_internal && (sc.bad(a.n_dst) || sc.bad(a.n_ldc)))) {
    set_error("group call: a per-expert array is shorter than the number of experts");
    return ZMI_FAILURE;
  }
  if (opt_in && a.params[0].total_matmul > a.params[0].active_matmul) {
    const size_t tm = a.params[0].total_matmul;
    if ((size_t)a.n_weight < tm || (size_t)a.n_K < tm || (size_t)a.n_N < tm || (size_t)a.n_ldb < tm ||
        (size_t)a.n_transB < tm || (size_t)a.n_is_weights_const < tm) {
      set_error("group call: weight-side arrays must cover all total_matmul experts");
      return ZMI_FAILURE;
    }
  }
  if (op1_internal) {
    if (a.n_dst != 0 && sc.bad(a.n_dst)) { set_error("fused_moe with library-held Op1 output: dst has entries but not one per expert"); return ZMI_FAILURE; }
    if (a.n_ldc != 0 && sc.bad(a.n_ldc)) { set_error("fused_moe with library-held Op1 output: ldc has entries but not one per expert"); return ZMI_FAILURE; }
  }
  if (op2_internal && fm->n_ldc_down != 0 && sc.bad(fm->n_ldc_down)) { set_error("fused_moe with library-held Op2 output: ldc_down has entries but not one per expert"); return ZMI_FAILURE; }
  if (a.n_src != 1 && sc.bad(a.n_src)) { set_error("group call: src holds neither one entry (chain) nor one per expert"); return ZMI_FAILURE; }
  const bool run_act = gated_act != ZMI_ACT_NONE;
  if (a.n_src == 1) {
    if (postop) { set_error("moe_postop needs one src per expert (not the one-src chain form)"); return ZMI_FAILURE; }
    if (run_act) { set_error("gated_act needs one src per expert (not the one-src chain form)"); return ZMI_FAILURE; }
    if (fm) { set_error("fused_moe needs one src per expert (not the one-src chain form)"); return ZMI_FAILURE; }
  }
  if (fm && fm->n_down_weight == 0) { set_error("fused_moe given without down_weight entries (pass no fused_moe to switch it off)"); return ZMI_FAILURE; }
  if (a.n_src == 1) {
    // sequential chain
    if (!a.src[0]) { set_error("chain form: src[0] is null"); return ZMI_FAILURE; }
    for (size_t i = 0; i < num_ops; ++i) {
      if (!a.weight[i] || !a.dst[i]) { set_error("chain form: a layer has a null weight or dst"); return ZMI_FAILURE; }
      if (a.M[i] <= 0 || a.N[i] <= 0 || a.K[i] <= 0) { set_error("chain form: M, N, K of every layer must be positive"); return ZMI_FAILURE; }
    }
    for (size_t i = 1; i < num_ops; ++i) {
      if (a.M[i] != a.M[0]) { set_error("chain form: every layer must have the first layer's M"); return ZMI_FAILURE; }
      if (a.K[i] != a.N[i - 1]) { set_error("chain form: a layer's K must equal the previous layer's N"); return ZMI_FAILURE; }
    }
    return ZMI_SUCCESS;
  }
  for (size_t i = 0; i < num_ops; ++i) {
    if (a.M[i] < 0 || a.N[i] <= 0 || a.K[i] <= 0) { set_error("group call: N and K must be positive and M non-negative for every expert"); return ZMI_FAILURE; }
    if (a.M[i] > 0) {
      if (!a.src[i] || !a.weight[i]) { set_error("group call: an expert with rows has a null src or weight"); return ZMI_FAILURE; }
      if (!op1_internal && !a.dst[i]) { set_error("group call: an expert with rows has a null dst"); return ZMI_FAILURE; }
    }
  }
  if (run_act) {
    const int dt = a.params[0].dt_dst;
    if (dt != ZMI_DT_F32 && dt != ZMI_DT_BF16 && dt != ZMI_DT_F16) { set_error("gated_act: dt_dst must be f32, bf16 or f16"); return ZMI_FAILURE; }
    for (size_t i = 1; i < num_ops; ++i)
      if (a.params[i].dt_dst != dt) { set_error("gated_act: all experts must share one dt_dst"); return ZMI_FAILURE; }
    for (size_t i = 0; i < num_ops; ++i)
      if (a.N[i] % 2 != 0) { set_error("gated_act: N holds gate and up halves and must be even"); return ZMI_FAILURE; }
    if (!op1_internal && !fm) {
      bool tight = false, wide = false;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        if (a.ldc[i] < a.N[i]) tight = true; else wide = true;
      }
      if (tight && wide) { set_error("gated_act: mixed tight / wide dst layouts"); return ZMI_FAILURE; }
    }
  }
  if (run_act || fm) {
    for (size_t i = 0; i < num_ops; ++i)
      if (a.layout[i] != 'r' && a.layout[i] != 'R') { set_error("gated_act / fused_moe: layout must be 'r' for every expert"); return ZMI_FAILURE; }
  }
  if (fm) {
    if (sc.bad(fm->n_down_weight) || sc.bad(fm->n_N_down) || sc.bad(fm->n_ldb_down) || sc.bad(fm->n_bias_down) ||
        (!op2_internal && (sc.bad(fm->n_dst_down) || sc.bad(fm->n_ldc_down)))) {
      set_error("fused_moe: a per-expert array is shorter than the number of experts");
      return ZMI_FAILURE;
    }
    if (fm->n_down_scale != 0 && (size_t)fm->n_down_scale < num_ops) { set_error("fused_moe: down_scale has entries but fewer than one per expert"); return ZMI_FAILURE; }
    if (fm->n_down_zp != 0 && (size_t)fm->n_down_zp < num_ops) { set_error("fused_moe: down_zp has entries but fewer than one per expert"); return ZMI_FAILURE; }
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.N[i] % 2 != 0) { set_error("fused_moe: N holds gate and up halves and must be even"); return ZMI_FAILURE; }
      if (a.M[i] > 0) {
        if (!fm->down_weight[i]) { set_error("fused_moe: an expert with rows has a null down_weight"); return ZMI_FAILURE; }
        if (!op2_internal && !fm->dst_down[i]) { set_error("fused_moe: an expert with rows has a null dst_down"); return ZMI_FAILURE; }
      }
      if (fm->N_down[i] <= 0) { set_error("fused_moe: N_down <= 0"); return ZMI_FAILURE; }
      const int kd = op2_k_for_act(a.N[i], gated_act);
      const int min_ldb = a.transB[i] ? kd : fm->N_down[i];
      if (fm->ldb_down[i] < min_ldb) { set_error("fused_moe: ldb_down is smaller than a row of down_weight"); return ZMI_FAILURE; }
      if (!op2_internal) {
        if (fm->ldc_down[i] < fm->N_down[i]) { set_error("fused_moe: ldc_down is smaller than N_down"); return ZMI_FAILURE; }
      } else {
        if (a.M[i] > 0 && a.lda[i] < fm->N_down[i]) { set_error("fused_moe with library-held Op2 output: the result goes back into src, whose lda must hold N_down"); return ZMI_FAILURE; }
        if (a.M[i] > 0 && a.params[i].dt_src != a.params[i].dt_dst) { set_error("fused_moe with library-held Op2 output: the result goes back into src, so dt_src must equal dt_dst"); return ZMI_FAILURE; }
      }
      if (fm->bias_down[i] && fm->bias_dt_down == ZMI_DT_NONE) { set_error("fused_moe: bias_down given without bias_dt_down"); return ZMI_FAILURE; }
    }
    if (postop)
      for (size_t i = 1; i < num_ops; ++i)
        if (fm->N_down[i] != fm->N_down[0]) { set_error("fused_moe with moe_postop: all experts must share one N_down"); return ZMI_FAILURE; }
  }
  if (postop) {
    for (size_t i = 1; i < num_ops; ++i) {
      if (a.N[i] != a.N[0]) { set_error("moe_postop: all experts must share one N"); return ZMI_FAILURE; }
      if (a.params[i].dt_dst != a.params[0].dt_dst) { set_error("moe_postop: all experts must share one dt_dst"); return ZMI_FAILURE; }
    }
    // validate_group_matmul_moe_postop (group_matmul/group_matmul_moe_postop.cpp)
    const int D = fm ? fm->N_down[0] : a.N[0];
    const int dt = a.params[0].dt_dst;
    if (!postop->row_ptrs || !postop->output) { set_error("moe_postop: row_ptrs and output must be non-null"); return ZMI_FAILURE; }
    if (postop->num_tokens <= 0 || postop->topk <= 0) { set_error("moe_postop: num_tokens and topk must be positive"); return ZMI_FAILURE; }
    if (postop->ldc_output < D) { set_error("moe_postop: ldc_output < D"); return ZMI_FAILURE; }
    if (dt != ZMI_DT_F32 && dt != ZMI_DT_BF16 && dt != ZMI_DT_F16) { set_error("moe_postop: dst dtype must be f32, bf16 or f16"); return ZMI_FAILURE; }
    if (!postop->skip_weighted && !postop->topk_weights) { set_error("moe_postop: topk_weights required"); return ZMI_FAILURE; }
  }
  return ZMI_SUCCESS;
}

// One epilogue descriptor serves a grouped launch only if every expert asks for
// the same arithmetic.
bool params_uniform(const zmi_group_args_t &a, size_t num_ops) {
  const zmi_matmul_params_t &p0 = a.params[0];
  for (size_t i = 0; i < num_ops; ++i) {
    const zmi_matmul_params_t &p = a.params[i];
    if (p.dt_src != p0.dt_src || p.dt_wei != p0.dt_wei || p.dt_dst != p0.dt_dst || p.dt_bias != p0.dt_bias ||
        p.dt_compute != p0.dt_compute || p.dynamic_quant != p0.dynamic_quant || p.mem_format_b != p0.mem_format_b ||
        p.n_postops != p0.n_postops)
      return false;
    if (a.alpha[i] != a.alpha[0] || a.beta[i] != a.beta[0]) return false;
    if ((a.bias[i] != nullptr) != (a.bias[0] != nullptr) && a.M[i] > 0 && a.M[0] > 0) return false;
    for (int j = 0; j < p.n_postops; ++j) {
      const zmi_post_op_t &x = p.postops[j], &y = p0.postops[j];
      if (x.po_type != y.po_type || x.alpha != y.alpha || x.beta != y.beta) return false;
      if (x.po_type == ZMI_PO_BINARY_ADD || x.po_type == ZMI_PO_BINARY_MUL) return false;
    }
    if ((p.src_zp.buff != nullptr) != (p0.src_zp.buff != nullptr)) return false;
    // (the shared epilogue reads every expert's scales in one dtype)
    if (p.wei_scale.dt != p0.wei_scale.dt || p.src_scale.dt != p0.src_scale.dt) return false;
    if (p.dst_scale.buff || p.dst_zp.buff || p.wei_zp.buff) return false;
    if ((p.wei_scale.buff != nullptr) != (p0.wei_scale.buff != nullptr)) return false;
    if (p.wei_scale.buff && ((nelems(p.wei_scale) == 1) != (nelems(p0.wei_scale) == 1))) return false;
    if (!p.dynamic_quant) {
      if ((p.src_scale.buff != nullptr) != (p0.src_scale.buff != nullptr)) return false;
      if (p.src_scale.buff && ((nelems(p.src_scale) == 1) != (nelems(p0.src_scale) == 1))) return false;
    }
  }
  return true;
}

// When every matrix of a grouped quantization qualifies for the 8-rows-per-workgroup
// kernel, its rows are renumbered so that each matrix starts at a multiple of 8.
int64_t renumber_rows8(std::vector<ZmiQuantMat> &mats, int32_t src_dt, int64_t total_rows, int *rows8) {
  *rows8 = 0;
  for (const ZmiQuantMat &m : mats)
    if (!zmi_quant_mat_frag8_ok(m, src_dt)) return total_rows;
  int64_t r = 0;
  for (ZmiQuantMat &m : mats) { m.row_start = (int32_t)r; r += zmi_round_up(m.M, 8); }
  *rows8 = 1;
  return r;
}

struct Stage {
  std::vector<ZmiProblem> probs;
  ZmiEpilogue epi;
  mutable bool streamed = false;   // set by launch_stage: the weight-traffic-bound kernel took the large experts
  mutable bool ring_sliced = false;  // set by launch_stage: the MFMA-bound kernel's launch went out in K slices
};

int group_top(int64_t rows, int n_prob, int64_t K, int64_t N, bool gated) {
  if (const char *env = zmi_env(ZE_GROUP_TOP)) { int v = std::atoi(env); if (v > 0) return v; }
  return zmi_ring_pick_top_group(rows, n_prob, K, N, gated);
}

// Whether the weight-traffic-bound kernel takes a grouped launch, and how: top = tile height (with ZMI_RING_PAD; 0: the
// MFMA-bound kernel keeps the launch), slices = K slices per tile.  max_rows: rows of the largest expert (for a launch
// whose row counts live on the device: a class derived from the average); tiles: (expected) number of tiles at that height.
// Up to 256 rows an expert is one row block: its weights pass once, and the MFMA work of 256 rows takes about as
// long as its weights need to arrive.  A launch needs two tiles per compute unit to be worth it; a plain (not gated)
// launch of 128-row tiles that would leave workgroup slots empty gets there by K slices (8 experts x 28 .. 36 rows,
// 14336 -> 4096: 128 tiles in 4 slices each).
struct StreamPlan { int top, slices; };
// room for the workspace of a K-sliced grouped launch: such a launch has at most 2 x (compute units) items of 128 rows
// or (compute units) items of 256 rows (64 MiB on 256 compute units), twice that for the slack of a launch sized by
// a bound; a launch that would need more runs unsliced
size_t stream_partial_bound() { return (size_t)zmi_cu_count() * 2 * 256 * 256 * sizeof(int32_t); }
StreamPlan group_stream_plan(int max_rows, const ZmiEpilogue &epi, int N, int K, int64_t tiles) {
  StreamPlan plan = {0, 1};
  if ((max_rows <= 16 || max_rows > 256) && !zmi_env(ZE_GROUP_STREAM_TOP)) return plan;
  const int th = max_rows <= 128 ? 128 : 256;
  const int64_t slots = th == 128 ? 2 * (int64_t)zmi_cu_count() : zmi_cu_count();   // workgroups the device holds at once
  const int nk = (int)(zmi_blob_kpad(K) / 64);
  int slices = 1;
  // (256-row tiles are not sliced: two workgroups on the halves of one tile's K stream at 4.1 TB/s together where the
  // MFMA-bound kernel's deep-ring build reaches the same end sooner: 115 + 35 us against 136 us on config 4's Op2)
  if (epi.gated_act == 0 && th == 128 && tiles > 0 && tiles * 2 <= slots) slices = (int)std::min<int64_t>(4, slots / tiles);
  while (slices > 1 && nk / slices < 16) --slices;
  if (const char *env = zmi_env(ZE_GROUP_STREAM_SLICES)) slices = std::max(1, std::atoi(env));
  if (epi.gated_act != 0) slices = 1;
  int top = 0;
  if (tiles >= slots || slices > 1) top = th | ZMI_RING_PAD;
  if (const char *env = zmi_env(ZE_GROUP_STREAM_TOP)) top = std::atoi(env);   // (0 switches the kernel off)
  if (!top || !zmi_group_stream_takes(epi, N, top)) return plan;
  plan.top = top;
  plan.slices = slices;
  return plan;
}

// K slices for a grouped launch of the MFMA-bound kernel that leaves compute units empty (a down projection of a few
// experts: 2 experts x ~128 rows, 14336 -> 4096, is 32 tiles): 2 .. 4 slices per tile while tiles x slices still fit one
// workgroup per compute unit (the deep-ring build) and a slice keeps 24 stages of 64 k; the slice that arrives last at
// its tile's word adds the partial tiles and finishes the elements (exact: int32).  Beyond one workgroup per compute
// unit slices lose: 8 experts x 113 .. 142 rows, 14336 -> 4096 (192 tiles), two slices each as 384 workgroups of the
// two-per-unit build took 182 us against 139 us for the 192 unsliced ones with the deep ring.  The workspace comes out
// of the room reserved for sliced grouped launches.
ZmiRingSplit ring_group_split(int top, int items, int K, bool gated) {
  ZmiRingSplit rs = {1, nullptr, nullptr};
  const int th = top & 0xffff;
  if (gated || !(top & ZMI_RING_PAD) || th == 256 || items <= 0 || zmi_env(ZE_NO_GROUP_RING_SLICES)) return rs;
  const int64_t slots = zmi_cu_count();
  int slices = (int)std::min<int64_t>(4, slots / items);
  const int nk = (int)(zmi_blob_kpad(K) / 64);
  while (slices > 1 && nk / slices < 24) --slices;
  if (slices < 2) return rs;
  const size_t bytes = (size_t)items * slices * th * 256 * sizeof(int32_t);
  if (bytes > stream_partial_bound()) return rs;
  unsigned int *arr = slice_arrivals(items);
  int32_t *partial = arr ? (int32_t *)arena().alloc(bytes) : nullptr;
  if (!arr || !partial) return rs;
  rs.slices = slices;
  rs.partial = partial;
  rs.arrivals = arr;
  return rs;
}

// Every expert's activations are fragment-major.  Experts with more than 16 rows: one launch of the MFMA-bound
// kernel; experts with 1 .. 16 rows: one launch of the decode-shaped grouped kernel (weight streaming, gated
// activation in its epilogue), reference: the ALGO-3 decode tile, group_matmul/group_matmul_dispatch.cpp:779.
int32_t launch_stage(const Stage &st, const char *what) {
  if (st.probs.empty()) return ZMI_SUCCESS;
  const ZmiProblem *dev = (const ZmiProblem *)upload(st.probs.data(), st.probs.size() * sizeof(ZmiProblem));
  if (!dev) return ZMI_FAILURE;
  const int n = (int)st.probs.size();
  const bool gated = st.epi.gated_act != 0;
  int64_t rows = 0;
  int cols = 0, kmax = 0, small = 0, large = 0, max_rows = 0;
  bool small_ok = true;
  for (const ZmiProblem &q : st.probs) {
    rows += q.M; cols = std::max(cols, (int)q.N); kmax = std::max(kmax, (int)q.K); max_rows = std::max(max_rows, (int)q.M);
    if (q.M > 0 && q.M <= 16) { ++small; small_ok = small_ok && zmi_group_decode_takes(st.epi, q.N); }
    else if (q.M > 16) ++large;
  }
  // The decode-shaped kernel runs as a launch of its own, behind the MFMA-bound one: worth it when the small experts
  // are most of the weight traffic (a decode step: 0.26 against 0.32 ms for 8 experts x 2 .. 6 rows of configuration
  // 4's block); a few small experts among large ones stream under the large ones' MFMA work inside the one launch
  // instead (configuration 5: 0.45 against 0.49 ms).  ZMI_GROUP_DECODE=1 forces the split (tests).
  const bool force_split = zmi_env(ZE_GROUP_DECODE) != nullptr;
  const bool split = small > 0 && small_ok && (small >= large || force_split);
  int top = group_top(rows, n, kmax, cols, gated);
  // experts of at most 256 rows are a stream of their weights: the kernel built for that takes the launch
  int64_t tiles_th = 0;
  for (const ZmiProblem &q : st.probs)
    if (q.M > 16)
      tiles_th += max_rows <= 128 ? zmi_ring_items<128>(q.M, q.N, 128 | ZMI_RING_PAD, gated) : zmi_ring_items<256>(q.M, q.N, 256 | ZMI_RING_PAD, gated);
  const StreamPlan sp = group_stream_plan(max_rows, st.epi, cols, kmax, tiles_th);
  if (sp.top) top = sp.top;
  if (split) top |= ZMI_RING_SKIP_SMALL;
  if (large > 0 || !split) {
    int *tab = (int *)arena().alloc(sizeof(int) * (4 + 3 * (size_t)n));
    if (!tab) { set_error("scratch exhausted (tile table)"); return ZMI_FAILURE; }
    st.streamed = sp.top != 0;
    if (sp.top) {
      ZmiRingSplit rs = {1, nullptr, nullptr};
      if (sp.slices > 1) {
        const int items = zmi_stream_items(st.probs.data(), n, top, 0, 0, gated);
        rs.slices = sp.slices;
        rs.partial = (int32_t *)arena().alloc(zmi_stream_partial_bytes(items, sp.slices, top));
        if (!rs.partial) rs.slices = 1;   // (no room: the unsliced launch is as right)
      }
      if (!hip_ok(zmi_launch_ring_table(dev, n, top, gated, tab, stream()), what)) return ZMI_FAILURE;
      if (!hip_ok(zmi_launch_gemm_stream_group(st.probs.data(), dev, n, top, 0, 0, tab, &rs, st.epi, stream()), what)) return ZMI_FAILURE;
    } else {
      const ZmiRingSplit rs = ring_group_split(top, zmi_ring_group_items(st.probs.data(), n, top, 0, 0, gated), kmax, gated);
      st.ring_sliced = rs.slices > 1;
      if (!hip_ok(zmi_launch_gemm_ring_group(st.probs.data(), dev, n, top, 0, 0, tab, false, st.epi, stream(), &rs), what))
        return ZMI_FAILURE;
    }
  }
  if (split && !hip_ok(zmi_launch_gemm_group_decode(dev, n, gated ? cols / 2 : cols, st.epi, stream()), what)) return ZMI_FAILURE;
  return ZMI_SUCCESS;
}

}  // namespace

extern "C" {

int32_t zmi_group_matmul_direct(const zmi_group_args_t *args, const zmi_moe_postop_t *moe_postop,
                                int32_t gated_act, const zmi_fused_moe_t *fused_moe) {
  clear_error();
  if (!args) { set_error("null args"); return ZMI_FAILURE; }
  const zmi_group_args_t &a = *args;
  for (int32_t i = 0; a.src && i < a.n_src; ++i) note_operand(a.src[i]);
  for (int32_t i = 0; a.weight && i < a.n_weight; ++i) note_operand(a.weight[i]);
  for (int32_t i = 0; a.bias && i < a.n_bias; ++i) note_operand(a.bias[i]);
  for (int32_t i = 0; a.dst && i < a.n_dst; ++i) note_operand(a.dst[i]);
  if (fused_moe) {
    for (int32_t i = 0; fused_moe->down_weight && i < fused_moe->n_down_weight; ++i) note_operand(fused_moe->down_weight[i]);
    for (int32_t i = 0; fused_moe->bias_down && i < fused_moe->n_bias_down; ++i) note_operand(fused_moe->bias_down[i]);
    for (int32_t i = 0; fused_moe->dst_down && i < fused_moe->n_dst_down; ++i) note_operand(fused_moe->dst_down[i]);
  }
  if (moe_postop) { note_operand(moe_postop->output); note_operand(moe_postop->topk_weights); }
  size_t num_ops = 0;
  bool op1_internal = false, op2_internal = false;
  int32_t st = validate_group(a, moe_postop, gated_act, fused_moe, &num_ops, &op1_internal, &op2_internal);
  if (st != ZMI_SUCCESS) return st;
  if (num_ops == 0) return ZMI_SUCCESS;

  // ---- sequential chain: layer i consumes layer i-1's output (group_matmul_direct.cpp:1137-1164)
  if (a.n_src == 1) {
    const void *cur = a.src[0];
    for (size_t i = 0; i < num_ops; ++i) {
      zmi_batch_params_t bp;
      zmi_batch_params_init(&bp);
      zmi_matmul_params_t p = a.params[i];
      st = zmi_matmul_direct(a.layout[i], a.transA[i], a.transB[i], a.M[i], a.N[i], a.K[i], a.alpha[i], cur, a.lda[i],
                             a.weight[i], a.ldb[i], a.bias[i], a.beta[i], a.dst[i], a.ldc[i], a.is_weights_const[i], &bp, &p);
      if (st != ZMI_SUCCESS) return st;
      cur = a.dst[i];
    }
    return ZMI_SUCCESS;
  }

  // ---- experts the grouped kernels do not take: per-group scales ({M,G} source with {G,N} weight scales), GGML
  // Q8_0 packed weights and W4A8 (s4 weights).  The reference runs them through the same per-expert sym-quant
  // GEMM as matmul_direct (group_matmul/group_matmul_dispatch.cpp:472-515, group_matmul_direct.cpp:1222-1260);
  // here a plain grouped call (no fused MoE, no gated activation) runs such experts one by one on the
  // matmul_direct path, then the weighted reduce if there is one. ----
  const bool run_act = gated_act != ZMI_ACT_NONE;
  bool one_by_one = false;
  for (size_t i = 0; i < num_ops; ++i) {
    if (a.M[i] <= 0) continue;
    const zmi_matmul_params_t &pi = a.params[i];
    int64_t sn = 1;
    for (int d = 0; d < pi.src_scale.ndims; ++d) sn *= pi.src_scale.dims[d];
    const bool has_scale_dims = pi.src_scale.ndims > 0 && (pi.src_scale.buff || pi.dynamic_quant);
    if (pi.dt_wei == ZMI_DT_S4 || pi.pack_format_b == 1 || (has_scale_dims && sn > a.M[i] && sn % a.M[i] == 0))
      one_by_one = true;
  }
  if (one_by_one) {
    // A gated activation and the fused block on such experts are the two-pass composition of the reference
    // (run_fused_moe_legacy_two_pass, group_matmul/group_matmul_fused_moe.cpp:906-1078; per-group scales never take
    // its vertically fused form, same file :705-711): Op1 per expert into the caller's wide dst, the activation
    // over all experts in place, Op2 per expert with the parameters setup_op2_dispatch_scratch derives (:761-880).
    if ((fused_moe || run_act) && (op1_internal || op2_internal)) {
      set_error("per-group / GGML-packed / s4 experts: fused_moe needs the caller's dst and dst_down (library-held intermediates are not implemented)");
      return ZMI_UNIMPLEMENTED;
    }
    if (run_act) {
      for (size_t i = 0; i < num_ops; ++i)
        if (a.M[i] > 0 && a.ldc[i] < a.N[i]) {
          set_error("per-group / GGML-packed / s4 experts: gated_act needs a dst that holds all N columns (ldc >= N)");
          return ZMI_UNIMPLEMENTED;
        }
    }
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.M[i] <= 0) continue;
      zmi_batch_params_t bp;
      zmi_batch_params_init(&bp);
      st = zmi_matmul_direct(a.layout[i], a.transA[i], a.transB[i], a.M[i], a.N[i], a.K[i], a.alpha[i], a.src[i], a.lda[i],
                             a.weight[i], a.ldb[i], a.bias[i], a.beta[i], a.dst[i], a.ldc[i], a.is_weights_const[i], &bp,
                             &a.params[i]);
      if (st != ZMI_SUCCESS) return st;
    }
    if (run_act) {
      // reference: group_matmul_moe_act_execute, group_matmul/group_matmul_moe_act.cpp
      if (!ensure_device()) return ZMI_FAILURE;
      std::vector<ZmiActMat> mats;
      int64_t r0 = 0;
      int maxN = 0;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        ZmiActMat m;
        m.buf = a.dst[i]; m.ld = a.ldc[i]; m.M = a.M[i]; m.N = a.N[i]; m.row_start = (int32_t)r0;
        r0 += a.M[i];
        maxN = std::max(maxN, a.N[i]);
        mats.push_back(m);
      }
      if (!mats.empty()) {
        const ZmiActMat *dev = (const ZmiActMat *)upload(mats.data(), mats.size() * sizeof(ZmiActMat));
        if (!dev) return ZMI_FAILURE;
        if (!hip_ok(zmi_launch_gated_act(dev, nullptr, (int)mats.size(), r0, maxN, gated_act, a.params[0].dt_dst, stream()), "gated act launch")) return ZMI_FAILURE;
        upload_fence();
      }
    }
    if (fused_moe) {
      const zmi_fused_moe_t &fm = *fused_moe;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        const zmi_matmul_params_t &p1 = a.params[i];
        const int kd = op2_k_for_act(a.N[i], gated_act);
        zmi_matmul_params_t p2;
        zmi_matmul_params_init(&p2);
        p2.dt_src = p1.dt_dst; p2.dt_wei = p1.dt_wei; p2.dt_dst = p1.dt_dst; p2.dt_bias = fm.bias_dt_down;
        p2.dynamic_quant = p1.dynamic_quant; p2.dt_compute = p1.dt_compute;
        p2.weight_cache_type = p1.weight_cache_type;
        const bool ggml = p1.pack_format_b == 1;
        if (ggml) p2.pack_format_b = 1;   // (both projections of a GGML expert are packed; the scales are inside the blocks)
        else if (fm.n_down_scale) p2.wei_scale = fm.down_scale[i];
        if (fm.n_down_zp) p2.wei_zp = fm.down_zp[i];
        if (p2.dynamic_quant) {
          const bool op1_per_group = p1.src_scale.ndims == 2 && p1.src_scale.dims[1] > 1;
          p2.src_scale.buff = nullptr;
          p2.src_scale.dt = p1.src_scale.dt;
          p2.src_scale.ndims = p1.src_scale.ndims;
          for (int d = 0; d < p1.src_scale.ndims; ++d) p2.src_scale.dims[d] = p1.src_scale.dims[d];
          if (op1_per_group) {
            // Op1's group count does not carry over (K differs): Op2's comes from the down projection's weight scale
            int64_t g2 = 1;
            if (ggml) g2 = kd / 32;
            else if (fm.n_down_scale) {
              const zmi_quant_t &ds = fm.down_scale[i];
              if (ds.ndims == 2 && ds.dims[0] > 1) g2 = ds.dims[0];
              else if (ds.ndims == 3 && ds.dims[1] > 1) g2 = ds.dims[1];
            }
            p2.src_scale.ndims = 2; p2.src_scale.dims[0] = p1.src_scale.dims[0]; p2.src_scale.dims[1] = g2;
          }
          if (p1.src_zp.dt != ZMI_DT_NONE && p1.src_zp.ndims == 2 && p1.src_zp.dims[1] > 1) {
            set_error("fused_moe: per-group source zero-points are not supported on the down projection");
            return ZMI_FAILURE;
          }
        }
        zmi_batch_params_t bp;
        zmi_batch_params_init(&bp);
        st = zmi_matmul_direct(a.layout[i], 0, a.transB[i], a.M[i], fm.N_down[i], kd, 1.0f, a.dst[i], a.ldc[i],
                               fm.down_weight[i], fm.ldb_down[i], fm.bias_down[i], 0.0f, fm.dst_down[i], fm.ldc_down[i],
                               a.is_weights_const[i], &bp, &p2);
        if (st != ZMI_SUCCESS) return st;
      }
    }
    if (moe_postop) goto postop_only;
    return ZMI_SUCCESS;
  }

  // ---- per-expert validation through the single-matmul rules ----
  for (size_t i = 0; i < num_ops; ++i) {
    if (a.M[i] <= 0) continue;
    const void *dsti = op1_internal ? (const void *)a.src[i] : (const void *)a.dst[i];
    if (diagnostics_enabled()) {
      st = validate_matmul(a.src[i], a.weight[i], dsti, a.M[i], a.N[i], a.K[i], 1, 1, a.params[i], a.is_weights_const[i] != 0);
      if (st != ZMI_SUCCESS) return st;
    }
    if (a.params[i].dt_wei != ZMI_DT_S8) { set_error("only s8 weights are implemented"); return ZMI_UNIMPLEMENTED; }
    if (a.layout[i] != 'r' && a.layout[i] != 'R') { set_error("only row-major layout is implemented"); return ZMI_UNIMPLEMENTED; }
    if (a.params[i].pack_format_b != 0) { set_error("GGML-packed weights are not implemented"); return ZMI_UNIMPLEMENTED; }
  }

  if (!params_uniform(a, num_ops)) {
    // experts disagree on dtypes / post-ops: run them one by one
    if (fused_moe || run_act) { set_error("fused_moe / gated_act need uniform per-expert params"); return ZMI_UNIMPLEMENTED; }
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.M[i] <= 0) continue;
      zmi_batch_params_t bp;
      zmi_batch_params_init(&bp);
      st = zmi_matmul_direct(a.layout[i], a.transA[i], a.transB[i], a.M[i], a.N[i], a.K[i], a.alpha[i], a.src[i], a.lda[i],
                             a.weight[i], a.ldb[i], a.bias[i], a.beta[i], a.dst[i], a.ldc[i], a.is_weights_const[i], &bp,
                             &a.params[i]);
      if (st != ZMI_SUCCESS) return st;
    }
    if (moe_postop) goto postop_only;
    return ZMI_SUCCESS;
  }

  {
    const zmi_matmul_params_t &p0 = a.params[0];
    const bool dyn = is_dynamic_quant_config(p0);
    if (!dyn && p0.dt_src != ZMI_DT_S8 && p0.dt_src != ZMI_DT_U8) {
      set_error("source must be u8 / s8, or bf16 / f32 with dynamic_quant and an s8 compute type");
      return ZMI_UNIMPLEMENTED;
    }
    if (dyn && p0.dt_compute == ZMI_DT_U8) { set_error("dynamic u8 quantization is not implemented"); return ZMI_UNIMPLEMENTED; }
    const int dst_es = p0.dt_dst == ZMI_DT_BF16 || p0.dt_dst == ZMI_DT_F16 ? 2 : (p0.dt_dst == ZMI_DT_F32 || p0.dt_dst == ZMI_DT_S32 ? 4 : 1);
    if (fused_moe && !(p0.dt_dst == ZMI_DT_BF16 || p0.dt_dst == ZMI_DT_F32)) { set_error("fused_moe needs a bf16 or f32 dst"); return ZMI_UNIMPLEMENTED; }
    if (fused_moe && !dyn) { set_error("fused_moe is implemented for dynamic_quant int8 only"); return ZMI_UNIMPLEMENTED; }
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.M[i] <= 0) continue;
      if (a.transA[i]) { set_error("transposed sources are not implemented in group calls"); return ZMI_UNIMPLEMENTED; }
      if (dyn) {
        int64_t sn = 1;
        for (int d = 0; d < a.params[i].src_scale.ndims; ++d) sn *= a.params[i].src_scale.dims[d];
        if (!(sn == a.M[i] || sn == 1)) { set_error("dynamic per-group source scales are not implemented"); return ZMI_UNIMPLEMENTED; }
        if (sn == 1 && a.M[i] > 1) { set_error("per-tensor dynamic scales are not implemented in group calls"); return ZMI_UNIMPLEMENTED; }
        if (a.params[i].src_zp.buff) { set_error("dynamic quantization is symmetric"); return ZMI_FAILURE; }
      }
      if (run_act && a.beta[i] != 0.0f) { set_error("gated_act with beta != 0 is not implemented"); return ZMI_UNIMPLEMENTED; }
    }
    if (!ensure_device()) return ZMI_FAILURE;

    // can the gated activation run inside the GEMM epilogue?
    bool fuse_act = run_act && gated_act != ZMI_ACT_SWIGLU_OAI_MUL;
    for (size_t i = 0; i < num_ops && fuse_act; ++i)
      if (a.M[i] > 0 && (a.N[i] / 2) % 32 != 0) fuse_act = false;
    // internal Op1 scratch holds only the activated half when the epilogue produces it; with the
    // stand-alone activation kernel it is as wide as a caller-visible dst ([gate | up], result in
    // the first half)
    const bool tight_internal = op1_internal && fuse_act;

    // ---- scratch plan ----
    size_t need = 0;
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.M[i] <= 0) continue;
      if (dyn) need += Arena::padded((size_t)zmi_afrag_bytes(a.M[i], a.K[i])) + Arena::padded(sizeof(float) * (size_t)a.M[i]);
      else need += Arena::padded((size_t)zmi_afrag_bytes(a.M[i], a.K[i]));
      const bool cache = a.params[i].mem_format_b != 'r' && a.is_weights_const[i] &&
                         std::min(weight_cache_env(), a.params[i].weight_cache_type) > 0;
      if (a.params[i].mem_format_b != 'r' && !cache) need += Arena::padded((size_t)zmi_blob_bytes(a.K[i], a.N[i]));
      if (op1_internal) {
        const int w = tight_internal ? a.N[i] / 2 : a.N[i];
        need += Arena::padded((size_t)a.M[i] * w * dst_es);
      }
      if (fused_moe) {
        const int kd = op2_k_for_act(a.N[i], gated_act);
        need += Arena::padded((size_t)zmi_afrag_bytes(a.M[i], kd)) + Arena::padded(sizeof(float) * (size_t)a.M[i]);
        const bool cache2 = a.is_weights_const[i] && std::min(weight_cache_env(), a.params[i].weight_cache_type) > 0;
        if (!cache2) need += Arena::padded((size_t)zmi_blob_bytes(kd, fused_moe->N_down[i]));
      }
    }
    if (moe_postop) {
      const size_t tbl = sizeof(void *) * (size_t)moe_postop->num_tokens * moe_postop->topk;
      need += Arena::padded(tbl);
    }
    need += 4096 + 2 * Arena::padded(sizeof(int) * (4 + 3 * num_ops));
    // Room for the partial tiles of a K-sliced stage, only where a stage can go out in slices: a plain epilogue and,
    // among the experts of more than 16 rows, at most one 128-row tile per compute unit (the least group_stream_plan and
    // ring_group_split ask for), or a forced slice count.  (A stage that finds no room runs unsliced.)
    {
      const int64_t n_cu = zmi_cu_count();
      const bool forced = zmi_env(ZE_GROUP_STREAM_SLICES) != nullptr;
      int64_t t1 = 0, t2 = 0;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 16) continue;
        const int64_t row_blocks = (a.M[i] + 127) / 128;
        t1 += row_blocks * ((a.N[i] + 255) / 256);
        if (fused_moe) t2 += row_blocks * ((fused_moe->N_down[i] + 255) / 256);
      }
      const int sliced_stages = ((forced || (!fuse_act && t1 <= n_cu)) ? 1 : 0) + ((fused_moe && (forced || t2 <= n_cu)) ? 1 : 0);
      need += (size_t)sliced_stages * Arena::padded(stream_partial_bound());
    }
    if (!arena().begin(need)) return ZMI_FAILURE;

    // ---- stage 1: sources (dynamic per-token quantization of every expert in one launch)
    std::vector<const void *> A1(num_ops, nullptr);
    std::vector<int64_t> lda1(num_ops, 0);
    std::vector<void *> s1(num_ops, nullptr);
    int32_t s1_dt = ZMI_DT_F32;
    if (dyn) {
      // reference: group_reorder_quantization_wrapper, matmul/quantization/reorder_quantization.cpp:307-696
      std::vector<ZmiQuantMat> mats;
      int64_t r0 = 0;
      int rows8 = 0;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        const int64_t kp = zmi_blob_kpad(a.K[i]);
        ZmiQuantMat m = {};
        m.src = a.src[i];
        m.dst = (int8_t *)arena().alloc((size_t)zmi_afrag_bytes(a.M[i], a.K[i]));
        float *sc = (float *)arena().alloc(sizeof(float) * (size_t)a.M[i]);
        m.scale = a.params[i].src_scale.buff ? (void *)a.params[i].src_scale.buff : (void *)sc;
        m.ld_src = a.lda[i]; m.ld_dst = kp; m.M = a.M[i]; m.K = a.K[i]; m.row_start = (int32_t)r0;
        m.frag_kpad = (int32_t)kp;
        r0 += a.M[i];
        mats.push_back(m);
        A1[i] = m.dst; lda1[i] = kp; s1[i] = m.scale;
      }
      // (the dtype the params name, whether the scales go to a caller's buffer or to scratch: the GEMM reads them back)
      s1_dt = p0.src_scale.dt != ZMI_DT_NONE ? p0.src_scale.dt : ZMI_DT_F32;
      if (s1_dt != ZMI_DT_F32 && s1_dt != ZMI_DT_BF16) { set_error("source scale must be f32 or bf16"); return ZMI_FAILURE; }
      r0 = renumber_rows8(mats, p0.dt_src, r0, &rows8);
      const ZmiQuantMat *dev = (const ZmiQuantMat *)upload(mats.data(), mats.size() * sizeof(ZmiQuantMat));
      if (!dev) return ZMI_FAILURE;
      if (!hip_ok(zmi_launch_quant_group(dev, (int)mats.size(), r0, p0.dt_src, s1_dt, rows8, stream()), "grouped quant launch")) return ZMI_FAILURE;
    } else {
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        int8_t *t = (int8_t *)arena().alloc((size_t)zmi_afrag_bytes(a.M[i], a.K[i]));
        if (!hip_ok(zmi_launch_repack_frag(a.src[i], a.M[i], a.K[i], a.lda[i], 0, a.params[i].dt_src == ZMI_DT_U8, t, stream()), "repack launch")) return ZMI_FAILURE;
        A1[i] = t; lda1[i] = zmi_blob_kpad(a.K[i]);
      }
    }

    // ---- stage 2: Op1 ----
    Stage op1;
    std::vector<void *> op1_dst(num_ops, nullptr);
    std::vector<int64_t> op1_ld(num_ops, 0);
    bool have_epi = false;
    for (size_t i = 0; i < num_ops; ++i) {
      if (a.M[i] <= 0) continue;
      const zmi_matmul_params_t &p = a.params[i];
      ZmiProblem pr;
      std::memset(&pr, 0, sizeof(pr));
      if (p.mem_format_b == 'r') {
        if (p.lowoha_algo != ZMI_ALGO_AOCL_DLP_BLOCKED) { set_error("mem_format_b == 'r' requires lowoha_algo == aocl_dlp_blocked"); return ZMI_FAILURE; }
        if (!blob_matches(a.weight[i], a.K[i], a.N[i])) return ZMI_FAILURE;
        pr.blob = (const uint8_t *)a.weight[i];
      } else {
        const bool cache = a.is_weights_const[i] && std::min(weight_cache_env(), p.weight_cache_type) > 0;
        void *slot = cache ? nullptr : arena().alloc((size_t)zmi_blob_bytes(a.K[i], a.N[i]));
        pr.blob = packed_weights(a.weight[i], a.K[i], a.N[i], a.ldb[i], a.transB[i] != 0, p.dt_src, cache, slot);
        if (!pr.blob) return ZMI_FAILURE;
      }
      if (op1_internal) {
        const int w = tight_internal ? a.N[i] / 2 : a.N[i];
        op1_dst[i] = arena().alloc((size_t)a.M[i] * w * dst_es);
        op1_ld[i] = w;
      } else {
        op1_dst[i] = a.dst[i];
        op1_ld[i] = a.ldc[i];
      }
      pr.A = A1[i]; pr.lda = lda1[i]; pr.dst = op1_dst[i]; pr.ldc = op1_ld[i];
      pr.M = a.M[i]; pr.N = a.N[i]; pr.K = a.K[i];
      pr.a_is_u8 = (!dyn && p.dt_src == ZMI_DT_U8) ? 1 : 0;
      zmi_matmul_params_t ep = p;
      if (dyn) {
        ep.dt_src = ZMI_DT_S8;
        ep.src_scale.buff = s1[i]; ep.src_scale.dt = s1_dt; ep.src_scale.ndims = 2;
        ep.src_scale.dims[0] = a.M[i]; ep.src_scale.dims[1] = 1;
      }
      ZmiEpilogue e;
      st = build_epilogue(ep, a.M[i], a.N[i], a.alpha[i], a.beta[i], a.bias[i], &e, &pr);
      if (st != ZMI_SUCCESS) return st;
      // M == 1: a one-row per-token scale is the same thing as a per-tensor device scale
      if (dyn && e.src_scale_mode == ZMI_SS_TENSOR_PTR) e.src_scale_mode = ZMI_SS_TOKEN_PTR;
      if (!have_epi) { op1.epi = e; have_epi = true; }
      else if (e.src_scale_mode != op1.epi.src_scale_mode || e.wei_scale_mode != op1.epi.wei_scale_mode) {
        set_error("experts disagree on scale granularity or host/device placement of one-element scales");
        return ZMI_UNIMPLEMENTED;
      }
      op1.probs.push_back(pr);
    }
    if (!have_epi) {
      upload_fence();
      if (moe_postop) goto postop_only;
      return ZMI_SUCCESS;
    }
    op1.epi.gated_act = fuse_act ? gated_act : ZMI_ACT_NONE;
    st = launch_stage(op1, "Op1 GEMM launch");
    if (st != ZMI_SUCCESS) return st;
    set_kernel_name(op1.streamed ? (fuse_act ? "group: stream_mfma32x32x32 (gated epilogue)" : "group: stream_mfma32x32x32")
                                 : (fuse_act ? "group: ring_mfma32x32x32 (gated epilogue)"
                                             : op1.ring_sliced ? "group: ring_mfma32x32x32 (K slices)" : "group: ring_mfma32x32x32"));

    if (run_act && !fuse_act) {
      // reference: group_matmul_moe_act_execute, group_matmul/group_matmul_moe_act.cpp
      std::vector<ZmiActMat> mats;
      int64_t r0 = 0;
      int maxN = 0;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        ZmiActMat m;
        m.buf = op1_dst[i]; m.ld = op1_ld[i]; m.M = a.M[i]; m.N = a.N[i]; m.row_start = (int32_t)r0;
        r0 += a.M[i];
        maxN = std::max(maxN, a.N[i]);
        mats.push_back(m);
      }
      const ZmiActMat *dev = (const ZmiActMat *)upload(mats.data(), mats.size() * sizeof(ZmiActMat));
      if (!dev) return ZMI_FAILURE;
      if (!hip_ok(zmi_launch_gated_act(dev, nullptr, (int)mats.size(), r0, maxN, gated_act, p0.dt_dst, stream()), "gated act launch")) return ZMI_FAILURE;
    }

    // ---- stage 3: Op2 (down projection), reference: run_fused_moe_legacy_two_pass,
    // group_matmul/group_matmul_fused_moe.cpp:906-1078
    if (fused_moe) {
      const zmi_fused_moe_t &fm = *fused_moe;
      std::vector<ZmiQuantMat> mats;
      std::vector<int8_t *> A2(num_ops, nullptr);
      std::vector<float *> s2(num_ops, nullptr);
      std::vector<int64_t> lda2(num_ops, 0);
      int64_t r0 = 0;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        const int kd = op2_k_for_act(a.N[i], gated_act);
        const int64_t kp = zmi_blob_kpad(kd);
        ZmiQuantMat m = {};
        m.src = op1_dst[i];
        m.dst = (int8_t *)arena().alloc((size_t)zmi_afrag_bytes(a.M[i], kd));
        m.scale = arena().alloc(sizeof(float) * (size_t)a.M[i]);
        m.ld_src = op1_ld[i]; m.ld_dst = kp; m.M = a.M[i]; m.K = kd; m.row_start = (int32_t)r0;
        m.frag_kpad = (int32_t)kp;
        r0 += a.M[i];
        mats.push_back(m);
        A2[i] = m.dst; s2[i] = (float *)m.scale; lda2[i] = kp;
      }
      int rows8 = 0;
      r0 = renumber_rows8(mats, p0.dt_dst, r0, &rows8);
      const ZmiQuantMat *dev = (const ZmiQuantMat *)upload(mats.data(), mats.size() * sizeof(ZmiQuantMat));
      if (!dev) return ZMI_FAILURE;
      // the down projection's source scales take Op1's scale dtype (group_matmul_fused_moe.cpp:816-820): with bf16
      // the scale is narrowed and the GEMM multiplies by the narrowed value
      if (!hip_ok(zmi_launch_quant_group(dev, (int)mats.size(), r0, p0.dt_dst, s1_dt, rows8, stream()), "grouped quant launch (Op2)")) return ZMI_FAILURE;

      Stage op2;
      bool have2 = false;
      for (size_t i = 0; i < num_ops; ++i) {
        if (a.M[i] <= 0) continue;
        const int kd = op2_k_for_act(a.N[i], gated_act);
        ZmiProblem pr;
        std::memset(&pr, 0, sizeof(pr));
        const bool cache = a.is_weights_const[i] && std::min(weight_cache_env(), a.params[i].weight_cache_type) > 0;
        void *slot = cache ? nullptr : arena().alloc((size_t)zmi_blob_bytes(kd, fm.N_down[i]));
        pr.blob = packed_weights(fm.down_weight[i], kd, fm.N_down[i], fm.ldb_down[i], a.transB[i] != 0, ZMI_DT_S8, cache, slot);
        if (!pr.blob) return ZMI_FAILURE;
        pr.A = A2[i]; pr.lda = lda2[i];
        if (op2_internal) { pr.dst = const_cast<void *>(a.src[i]); pr.ldc = a.lda[i]; }
        else { pr.dst = fm.dst_down[i]; pr.ldc = fm.ldc_down[i]; }
        pr.M = a.M[i]; pr.N = fm.N_down[i]; pr.K = kd;
        zmi_matmul_params_t ep;
        zmi_matmul_params_init(&ep);
        ep.dt_src = ZMI_DT_S8; ep.dt_wei = ZMI_DT_S8; ep.dt_dst = p0.dt_dst; ep.dt_bias = fm.bias_dt_down;
        ep.src_scale.buff = s2[i]; ep.src_scale.dt = s1_dt; ep.src_scale.ndims = 2;
        ep.src_scale.dims[0] = a.M[i]; ep.src_scale.dims[1] = 1;
        if (fm.n_down_scale) ep.wei_scale = fm.down_scale[i];
        if (fm.n_down_zp && fm.down_zp[i].buff) { set_error("down_zp is not implemented (symmetric weights only)"); return ZMI_UNIMPLEMENTED; }
        ZmiEpilogue e;
        st = build_epilogue(ep, a.M[i], fm.N_down[i], 1.0f, 0.0f, fm.bias_down[i], &e, &pr);
        if (st != ZMI_SUCCESS) return st;
        if (e.src_scale_mode == ZMI_SS_TENSOR_PTR) e.src_scale_mode = ZMI_SS_TOKEN_PTR;
        if (!have2) { op2.epi = e; have2 = true; }
        else if (e.wei_scale_mode != op2.epi.wei_scale_mode) { set_error("experts disagree on down_scale granularity"); return ZMI_UNIMPLEMENTED; }
        op2.probs.push_back(pr);
      }
      st = launch_stage(op2, "Op2 GEMM launch");
      if (st != ZMI_SUCCESS) return st;
    }
  }

postop_only:
  if (moe_postop) {
    // reference: group_matmul_moe_postop_execute, group_matmul/group_matmul_moe_postop.cpp:506
    if (!ensure_device()) return ZMI_FAILURE;
    const int D = fused_moe ? fused_moe->N_down[0] : a.N[0];
    const int dt = a.params[0].dt_dst;
    if (dt != ZMI_DT_BF16 && dt != ZMI_DT_F32 && dt != ZMI_DT_F16) { set_error("moe_postop: rows of f32, bf16 or f16"); return ZMI_FAILURE; }
    const size_t tbl = sizeof(void *) * (size_t)moe_postop->num_tokens * moe_postop->topk;
    const void *const *rp = (const void *const *)upload(moe_postop->row_ptrs, tbl);
    if (!rp) return ZMI_FAILURE;
    if (!hip_ok(zmi_launch_moe_combine(rp, nullptr, 0, nullptr, moe_postop->topk_weights, moe_postop->skip_weighted,
                                       moe_postop->num_tokens, moe_postop->topk, D, dt, moe_postop->output,
                                       moe_postop->ldc_output, stream()), "moe combine launch"))
      return ZMI_FAILURE;
  }
  upload_fence();
  return ZMI_SUCCESS;
}

int32_t zmi_moe_route(const int32_t *topk_ids, int32_t T, int32_t topk, int32_t E, int32_t *counts,
                      int32_t *offsets, int32_t *slot_of) {
  clear_error();
  if (!topk_ids || !counts || !offsets || !slot_of || T <= 0 || topk <= 0 || E <= 0) { set_error("moe_route: bad arguments"); return ZMI_FAILURE; }
  if (E > 2047) { set_error("moe_route: at most 2047 experts"); return ZMI_UNIMPLEMENTED; }
  if (!ensure_device()) return ZMI_FAILURE;
  const size_t hist_ints = zmi_moe_route_scratch_ints((int64_t)T * topk, E);
  if (!arena().begin(Arena::padded(hist_ints * sizeof(int32_t)))) return ZMI_FAILURE;
  int32_t *hist = hist_ints ? (int32_t *)arena().alloc(hist_ints * sizeof(int32_t)) : nullptr;
  if (!hip_ok(zmi_launch_moe_route(topk_ids, T, topk, E, 1, counts, offsets, slot_of, nullptr, 0, hist, stream()), "moe route launch")) return ZMI_FAILURE;
  set_kernel_name("moe_route");
  return ZMI_SUCCESS;
}

int32_t zmi_moe_router_topk(const void *logits, int32_t logits_dt, int64_t ldl, int32_t T, int32_t E, int32_t topk,
                            int32_t renormalize, int32_t *topk_ids, float *topk_weights) {
  clear_error();
  if (!logits || !topk_ids || !topk_weights || T <= 0 || E <= 0 || topk <= 0 || ldl < E) { set_error("moe_router_topk: bad arguments"); return ZMI_FAILURE; }
  if (topk > E) { set_error("moe_router_topk: topk exceeds the number of experts"); return ZMI_FAILURE; }
  if (logits_dt != ZMI_DT_F32 && logits_dt != ZMI_DT_BF16) { set_error("moe_router_topk: logits must be f32 or bf16"); return ZMI_FAILURE; }
  if (E > 512 || topk > 64) { set_error("moe_router_topk: at most 512 experts and topk <= 64"); return ZMI_UNIMPLEMENTED; }
  if (!ensure_device()) return ZMI_FAILURE;
  if (!hip_ok(zmi_launch_moe_router_topk(logits, logits_dt, ldl, T, E, topk, renormalize, topk_ids, topk_weights, stream()), "moe router launch")) return ZMI_FAILURE;
  set_kernel_name("moe_router_topk");
  return ZMI_SUCCESS;
}

int32_t zmi_moe_fused_device(const zmi_moe_device_t *d) {
  clear_error();
  if (!d || !d->x || !d->topk_ids || !d->topk_weights || !d->w13_blob || !d->w2_blob || !d->w13_scale || !d->w2_scale || !d->out) {
    set_error("moe_fused_device: null argument");
    return ZMI_FAILURE;
  }
  note_operand(d->x); note_operand(d->topk_ids); note_operand(d->topk_weights); note_operand(d->w13_blob);
  note_operand(d->w2_blob); note_operand(d->w13_scale); note_operand(d->w2_scale); note_operand(d->out);
  const int T = d->T, H = d->H, I = d->I, E = d->E, topk = d->topk;
  if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || topk <= 0 || d->ldx < H || d->ldo < H) { set_error("moe_fused_device: bad shape"); return ZMI_FAILURE; }
  if (H % 16 != 0 || I % 32 != 0) { set_error("moe_fused_device: H must be a multiple of 16 and I of 32"); return ZMI_UNIMPLEMENTED; }
  if (d->gated_act != ZMI_ACT_SILU_AND_MUL && d->gated_act != ZMI_ACT_GELU_AND_MUL) { set_error("moe_fused_device: silu_and_mul or gelu_and_mul"); return ZMI_UNIMPLEMENTED; }
  if (E > 2047) { set_error("moe_fused_device: at most 2047 experts"); return ZMI_UNIMPLEMENTED; }
  if (!ensure_device()) return ZMI_FAILURE;
  const int64_t R = (int64_t)T * topk;
  // every expert's rows start on a fragment row (multiple of 32 slots): at most 31 idle slots per expert
  const int64_t Rp = zmi_round_up(R + 31 * (int64_t)E, 32);
  const int64_t kpH = zmi_blob_kpad(H), kpI = zmi_blob_kpad(I);
  size_t need = 0;
  need += Arena::padded(sizeof(int32_t) * E) + Arena::padded(sizeof(int32_t) * (E + 1)) + Arena::padded(sizeof(int32_t) * R);
  need += Arena::padded(sizeof(int32_t) * Rp);
  need += Arena::padded((size_t)Rp * kpH) + Arena::padded(sizeof(float) * Rp);       // A1, s1
  need += Arena::padded((size_t)Rp * I * 2);                                         // act bf16
  need += Arena::padded((size_t)Rp * kpI) + Arena::padded(sizeof(float) * Rp);       // A2, s2
  need += Arena::padded((size_t)Rp * H * 2);                                         // Y bf16
  need += 2 * Arena::padded(sizeof(ZmiProblem) * E) + 4096 + 2 * Arena::padded(sizeof(int) * (4 + 3 * (size_t)E));
  // Op2 in K slices: only where its planners can ask for them (at most one 128-row tile per compute unit, or forced)
  if (zmi_env(ZE_GROUP_STREAM_SLICES) || (R / 128) * (int64_t)((H + 255) / 256) <= (int64_t)zmi_cu_count())
    need += Arena::padded(stream_partial_bound());
  const size_t hist_ints = zmi_moe_route_scratch_ints(R, E);
  need += Arena::padded(hist_ints * sizeof(int32_t));
  if (!arena().begin(need)) return ZMI_FAILURE;
  int32_t *route_hist = hist_ints ? (int32_t *)arena().alloc(hist_ints * sizeof(int32_t)) : nullptr;
  int32_t *counts = (int32_t *)arena().alloc(sizeof(int32_t) * E);
  int32_t *offsets = (int32_t *)arena().alloc(sizeof(int32_t) * (E + 1));
  int32_t *slot_of = (int32_t *)arena().alloc(sizeof(int32_t) * R);
  int32_t *src_of = (int32_t *)arena().alloc(sizeof(int32_t) * Rp);
  int8_t *A1 = (int8_t *)arena().alloc((size_t)Rp * kpH);
  float *s1 = (float *)arena().alloc(sizeof(float) * Rp);
  void *act = arena().alloc((size_t)Rp * I * 2);
  int8_t *A2 = (int8_t *)arena().alloc((size_t)Rp * kpI);
  float *s2 = (float *)arena().alloc(sizeof(float) * Rp);
  void *Y = arena().alloc((size_t)Rp * H * 2);
  int *tile_tab1 = (int *)arena().alloc(sizeof(int) * (4 + 3 * (size_t)E));
  int *tile_tab2 = (int *)arena().alloc(sizeof(int) * (4 + 3 * (size_t)E));
  ZmiProblem *op1 = (ZmiProblem *)arena().alloc(sizeof(ZmiProblem) * E);
  ZmiProblem *op2 = (ZmiProblem *)arena().alloc(sizeof(ZmiProblem) * E);

  // the four per-expert pointer tables travel in one upload
  std::vector<const void *> tbl(4 * (size_t)E);
  for (int e = 0; e < E; ++e) {
    tbl[e] = d->w13_blob[e]; tbl[E + e] = d->w2_blob[e]; tbl[2 * E + e] = d->w13_scale[e]; tbl[3 * E + e] = d->w2_scale[e];
    if (!tbl[e] || !tbl[E + e] || !tbl[2 * E + e] || !tbl[3 * E + e]) { set_error("moe_fused_device: null expert table entry"); return ZMI_FAILURE; }
  }
  for (int e = 0; e < E; ++e) {
    if (!blob_matches(d->w13_blob[e], H, 2 * I) || !blob_matches(d->w2_blob[e], I, H)) return ZMI_FAILURE;
  }
  const void *const *tdev = (const void *const *)upload(tbl.data(), tbl.size() * sizeof(void *));
  if (!tdev) return ZMI_FAILURE;
  ZmiMoeTables tb;
  tb.w13_blob = tdev; tb.w2_blob = tdev + E;
  tb.w13_scale = (const float *const *)(tdev + 2 * E); tb.w2_scale = (const float *const *)(tdev + 3 * E);

  hipStream_t s = stream();
  if (!hip_ok(zmi_launch_moe_route(d->topk_ids, T, topk, E, 32, counts, offsets, slot_of, src_of, (int)Rp, route_hist, s), "moe route launch")) return ZMI_FAILURE;
  // every slot quantizes its token's row itself (8 slots per workgroup, whole 128-byte lines of the
  // fragment layout); rows that do not allow 16-byte loads take the per-token scatter form
  if (hipSuccess != zmi_launch_quant_gather(d->x, ZMI_DT_BF16, d->ldx, H, src_of, topk, Rp, A1, kpH, s1, s)) {
    (void)hipGetLastError();
    if (!hip_ok(zmi_launch_moe_quant_scatter(d->x, d->ldx, T, H, topk, slot_of, A1, s1, s), "quant scatter launch")) return ZMI_FAILURE;
  }
  // row counts live on the device: the grids are sized for the worst case, and the kernel that builds
  // the per-expert problem tables fills the tile tables of both grouped launches as well
  int top1 = group_top(R, E, H, 2 * I, true), top2 = group_top(R, E, I, H, false);
  // (the row counts are not known here: experts with 1 .. 16 rows, if there are any, are the decode-shaped grouped
  // kernel's, whose workgroups leave at once for every other expert; the MFMA-bound kernel's tile table skips them)
  ZmiEpilogue probe;
  std::memset(&probe, 0, sizeof(probe));
  probe.fast_kind = ZMI_EK_NONE;
  // (worth a launch of its own only when small experts are most of the work: see launch_stage; the row counts live
  // on the device, so the average decides)
  const bool decode_step = R <= 16 * (int64_t)E || zmi_env(ZE_GROUP_DECODE) != nullptr;
  const bool small2 = decode_step && zmi_group_decode_takes(probe, H);
  probe.gated_act = d->gated_act;
  const bool small1 = decode_step && zmi_group_decode_takes(probe, 2 * I);
  const int avg_rows = (int)((R + E - 1) / E);
  ZmiEpilogue probe1 = probe;
  probe.gated_act = 0;
  // (an average of up to 96 rows: taken to be at most 128 everywhere; up to 224: at most 256; the expected tile count
  // takes every expert to have rows)
  const int row_class = avg_rows <= 96 ? 128 : (avg_rows <= 224 ? 256 : 0);
  const int64_t blocks = row_class ? std::max<int64_t>(R / row_class, std::min<int64_t>(E, R)) : 0;
  const StreamPlan sp1 = group_stream_plan(row_class, probe1, 2 * I, H, blocks * ((I + 127) / 128));
  const StreamPlan sp2 = group_stream_plan(row_class, probe, H, I, blocks * ((H + 255) / 256));
  const int stream1 = sp1.top, stream2 = sp2.top;
  if (stream1) top1 = stream1;
  if (stream2) top2 = stream2;
  if (small1) top1 |= ZMI_RING_SKIP_SMALL;
  if (small2) top2 |= ZMI_RING_SKIP_SMALL;
  if (!hip_ok(zmi_launch_moe_build_problems(tb, E, H, I, counts, offsets, A1, s1, act, A2, s2, Y, op1, op2, top1, top2, tile_tab1, tile_tab2, s), "problem table launch")) return ZMI_FAILURE;

  ZmiEpilogue e1;
  std::memset(&e1, 0, sizeof(e1));
  e1.src_scale_mode = ZMI_SS_TOKEN_PTR; e1.src_scale_dt = ZMI_DT_F32;
  e1.wei_scale_mode = 2; e1.wei_scale_dt = ZMI_DT_F32;
  e1.bias_dt = ZMI_DT_F32; e1.alpha = 1.0f; e1.beta = 0.0f; e1.dst_dt = ZMI_DT_BF16; e1.fast_kind = ZMI_EK_NONE;
  ZmiEpilogue e2 = e1;
  e1.gated_act = d->gated_act;
  if (stream1) {
    if (!hip_ok(zmi_launch_gemm_stream_group(nullptr, op1, E, top1, R, 2 * I, tile_tab1, nullptr, e1, s), "Op1 GEMM launch")) return ZMI_FAILURE;
  } else if (!hip_ok(zmi_launch_gemm_ring_group(nullptr, op1, E, top1, R, 2 * I, tile_tab1, true, e1, s), "Op1 GEMM launch")) {
    return ZMI_FAILURE;
  }
  if (small1 && !hip_ok(zmi_launch_gemm_group_decode(op1, E, I, e1, s), "Op1 decode-shaped GEMM launch")) return ZMI_FAILURE;
  // idle slots between experts are quantized too (their values are never read back)
  if (!hip_ok(zmi_launch_quant_rows(act, ZMI_DT_BF16, Rp, I, I, A2, kpI, kpI, s2, ZMI_DT_F32, s), "Op2 quant launch")) return ZMI_FAILURE;
  if (stream2) {
    ZmiRingSplit rs = {1, nullptr, nullptr};
    if (sp2.slices > 1) {
      rs.slices = sp2.slices;
      rs.partial = (int32_t *)arena().alloc(zmi_stream_partial_bytes(zmi_stream_items(nullptr, E, top2, R, H, false), sp2.slices, top2));
      if (!rs.partial) rs.slices = 1;
    }
    if (!hip_ok(zmi_launch_gemm_stream_group(nullptr, op2, E, top2, R, H, tile_tab2, &rs, e2, s), "Op2 GEMM launch")) return ZMI_FAILURE;
  } else {
    const ZmiRingSplit rs = ring_group_split(top2, zmi_ring_group_items(nullptr, E, top2, R, H, false), I, false);
    if (!hip_ok(zmi_launch_gemm_ring_group(nullptr, op2, E, top2, R, H, tile_tab2, true, e2, s, &rs), "Op2 GEMM launch"))
      return ZMI_FAILURE;
  }
  if (small2 && !hip_ok(zmi_launch_gemm_group_decode(op2, E, H, e2, s), "Op2 decode-shaped GEMM launch")) return ZMI_FAILURE;
  if (!hip_ok(zmi_launch_moe_combine(nullptr, Y, H, slot_of, d->topk_weights, 0, T, topk, H, ZMI_DT_BF16, d->out, d->ldo, s), "moe combine launch")) return ZMI_FAILURE;
  upload_fence();
  set_kernel_name("moe_fused_device");
  return ZMI_SUCCESS;
}

}  // extern "C"
