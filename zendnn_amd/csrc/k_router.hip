// MoE router for gfx950: softmax over a token's expert logits and its top-k experts, on the device.
//
// The reference leaves routing to the framework: its MoE entry point takes topk weights and row
// pointers the caller built on the host (docs/operator/low_overhead_operator/
// lowoha_group_matmul_operator.md:238-259; weights consumed by
// zendnnl/src/lowoha_operators/matmul/group_matmul/group_matmul_moe_postop.cpp:103-129).  On a GPU the
// logits are device memory and the ids feed zmi_moe_route / zmi_moe_fused_device, so the step between
// them is offered here instead of a round trip through the host.
//
//   * one wavefront per token, 4 tokens per workgroup; lane l holds experts l, l + 64, ... (at most 8);
//   * selection is on the logits themselves (softmax is monotonic, but two different logits can round
//     to one probability): the k largest, equal values in ascending expert order -- the first k entries
//     of a stable descending sort; -0 and +0 compare equal, NaN sorts behind everything;
//   * weights: p_e = exp(x_e - max) / sum_e' exp(x_e' - max), f32 terms, sums in double (wavefront
//     butterfly, the same order on every run); with renormalize the k selected weights are divided by
//     their sum, evaluated as exp(x_e - max) / sum_selected exp(x_e' - max).
#include "zmi_device.h"
#include "zmi_launch.h"

#define RTK_WAVES 4
#define RTK_PER_LANE 8

namespace {

// float -> unsigned key whose unsigned order is the float order; -0 == +0; NaN lowest
__device__ __forceinline__ uint32_t rtk_key(float x) {
  if (x != x) return 0u;
  const uint32_t u = __float_as_uint(x + 0.0f);   // -0 + 0 = +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

}  // namespace

__global__ __launch_bounds__(RTK_WAVES * 64) void zmi_moe_router_topk_kernel(const void *logits, int logits_dt, int64_t ldl,
                                                                             int T, int E, int topk, int renormalize,
                                                                             int32_t *topk_ids, float *topk_weights) {
  const int lane = threadIdx.x % 64;
  const int t = blockIdx.x * RTK_WAVES + threadIdx.x / 64;
  if (t >= T) return;   // (whole wavefronts; nothing below synchronizes across wavefronts)
  float x[RTK_PER_LANE];
  uint32_t key[RTK_PER_LANE];
#pragma unroll
  for (int j = 0; j < RTK_PER_LANE; ++j) {
    const int e = lane + 64 * j;
    float v = -__builtin_inff();
    if (e < E)
      v = logits_dt == ZMI_DT_BF16 ? zmi_bf16_to_f32(((const uint16_t *)logits)[(int64_t)t * ldl + e])
                                   : ((const float *)logits)[(int64_t)t * ldl + e];
    x[j] = v;
    key[j] = e < E ? rtk_key(v) : 0u;
  }
  // ---- softmax denominators ----
  float m = x[0];
#pragma unroll
  for (int j = 1; j < RTK_PER_LANE; ++j) m = fmaxf(m, x[j]);   // (fmaxf skips NaN; a NaN logit reaches the sum below)
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) m = fmaxf(m, __shfl_xor(m, s, 64));
  // (the sums are kept in double so that their rounding stays out of the 1e-6 the weights are held to;
  // the terms are f32)
  double dsum = 0.0;
#pragma unroll
  for (int j = 0; j < RTK_PER_LANE; ++j)
    if (lane + 64 * j < E) dsum += (double)zmi_expf(x[j] - m);
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) dsum += __shfl_xor(dsum, s, 64);
  const float sum = (float)dsum;

  // ---- k rounds of argmax over what is left (key, then lower expert index) ----
  unsigned taken = 0;   // bit j: this lane's j-th expert has been selected
  float e_mine = 0.0f;  // lane kk keeps the kk-th selected expert's exp(x - max) (topk <= 64)
  double e_sel = 0.0;   // their sum, in selection order (the same on every lane)
  for (int kk = 0; kk < topk; ++kk) {
    uint32_t bk = 0u;
    int be = 0x7fffffff;
    float bx = 0.0f;
#pragma unroll
    for (int j = 0; j < RTK_PER_LANE; ++j) {
      const int e = lane + 64 * j;
      const bool live = e < E && !((taken >> j) & 1u);
      // ascending j is ascending e within a lane: strict > keeps the lower index on ties
      if (live && (be == 0x7fffffff || key[j] > bk)) { bk = key[j]; be = e; bx = x[j]; }
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
      const uint32_t ok = (uint32_t)__shfl_xor((int)bk, s, 64);
      const int oe = __shfl_xor(be, s, 64);
      const float ox = __shfl_xor(bx, s, 64);
      const bool other = oe != 0x7fffffff && (be == 0x7fffffff || ok > bk || (ok == bk && oe < be));
      if (other) { bk = ok; be = oe; bx = ox; }
    }
    // every lane now holds the winner
    if (be % 64 == lane) taken |= 1u << (be / 64);
    const float ex = zmi_expf(bx - m);
    e_sel += (double)ex;
    if (lane == 0) topk_ids[(int64_t)t * topk + kk] = be;
    if (lane == kk) e_mine = ex;
  }
  // renormalized: p_i / sum_sel p_j == e_i / sum_sel e_j (one division instead of two)
  if (lane < topk) topk_weights[(int64_t)t * topk + lane] = e_mine / (renormalize ? (float)e_sel : sum);
}

hipError_t zmi_launch_moe_router_topk(const void *logits, int logits_dt, int64_t ldl, int T, int E, int topk,
                                      int renormalize, int32_t *topk_ids, float *topk_weights, hipStream_t stream) {
  if (T <= 0) return hipSuccess;
  if (E <= 0 || E > 64 * RTK_PER_LANE || topk <= 0 || topk > E || topk > 64) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((T + RTK_WAVES - 1) / RTK_WAVES)), block(RTK_WAVES * 64);
  hipLaunchKernelGGL(zmi_moe_router_topk_kernel, grid, block, 0, stream, logits, logits_dt, ldl, T, E, topk, renormalize,
                     topk_ids, topk_weights);
  return hipGetLastError();
}
