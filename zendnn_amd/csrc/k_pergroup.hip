// Per-group symmetric int8 GEMM for gfx950: C[M, N] = tail(sum_g float(acc_g) * ss[m, g] * ws[g, n]).
//
// Call site replaced: the aocl_gemm_s8s8s32o{f32,bf16}_sym_quant call with a group size
// (zendnnl/src/lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:1239-1257, group size set at
// :913-917); semantics restated by the reference's scalar kernel, per-group branch
// (zendnnl/src/operators/matmul/matmul_ref_kernel.cpp:917-1001): K is cut into G groups, every group's
// integer sum is scaled by the source scale of (row, group), then by the weight scale of
// (group, column), and the f32 terms are added in group order.
//
// The order of the f32 additions is part of the result, so K is NOT split across wavefronts:
// one wavefront owns a 16-column block (and 16 * RB rows) and walks K front to back with
// v_mfma_i32_16x16x64_i8, folding the integer accumulator into the f32 sum at every group
// boundary.  Weights are read once per row block straight from the prepacked blob (a
// 16-column half of a 1 KiB fragment is 256 contiguous bytes per 16 k), D chunks of 64 k
// ahead; the scales of the next group are requested one group ahead.  Groups of 16 or 32 k
// share a 64-k chunk: the chunk is multiplied once per group with the other groups' lanes
// of the row operand zeroed.
#include "zmi_device.h"
#include "zmi_launch.h"

#define PG_WAVES 4

template <int RB, int D>
__global__ __launch_bounds__(PG_WAVES * 64) void zmi_gemm_pergroup_kernel(ZmiProblem p, ZmiEpilogue epi, int n_cb,
                                                                          int n_items, int gs) {
  const int lane = threadIdx.x % 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int item = blockIdx.x * PG_WAVES + wave;
  if (item >= n_items) return;
  const int cb = item % n_cb, rbk = item / n_cb;
  const int M = p.M, N = p.N, K = p.K, G = epi.n_groups;
  const int nch = (int)(zmi_blob_kpad(K) / 64);
  const int c16 = lane % 16, g4 = lane / 16;
  const int col = cb * 16 + c16;
  const int row0 = rbk * 16 * RB;
  const uint8_t *bsrc = p.blob + zmi_blob_tiles_off(N) + (int64_t)(cb / 2) * zmi_blob_nb_stride(K) + (g4 / 2) * 1024 +
                        ((g4 % 2) * 32 + (cb % 2) * 16 + c16) * 16;
  const int8_t *A = (const int8_t *)p.A;

  // ---- operand ring: D chunks of 64 k in flight ----
  v4i b[D], a[D][RB];
  auto request = [&](int slot, int c) {
    const bool in = c < nch;                       // (uniform) past the end: nothing is read
    b[slot] = in ? *(const v4i *)(bsrc + (int64_t)c * 2048) : (v4i){0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < RB; ++j) {
      const int row = row0 + j * 16 + c16;
      const int k = c * 64 + g4 * 16;
      a[slot][j] = (in && row < M && k < K) ? *(const v4i *)(A + (int64_t)row * p.lda + k) : (v4i){0, 0, 0, 0};
    }
  };
#pragma unroll
  for (int s = 0; s < D; ++s) request(s, s);

  // ---- scales of the next group to be folded ----
  float wsn, ssn[RB][4];
  auto request_scales = [&](int gi) {
    wsn = col < N ? zmi_ld_f32(p.wei_scale_ptr, epi.wei_scale_dt, (int64_t)gi * N + col) : 0.0f;
#pragma unroll
    for (int j = 0; j < RB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = row0 + j * 16 + g4 * 4 + q;   // accumulator element q of this lane
        ssn[j][q] = row < M ? zmi_ld_f32(p.src_scale_ptr, epi.src_scale_dt, (int64_t)row * G + gi) : 0.0f;
      }
  };
  request_scales(0);

  v4i acc[RB];
  float sum[RB][4];
#pragma unroll
  for (int j = 0; j < RB; ++j) {
    acc[j] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 4; ++q) sum[j][q] = 0.0f;
  }
  // group gi is complete in acc: sum += (float(acc) * ss[m, gi]) * ws[gi, n], each step rounded
  auto fold = [&](int gi) {
    const float wsv = wsn;
    float ssv[RB][4];
#pragma unroll
    for (int j = 0; j < RB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) ssv[j][q] = ssn[j][q];
    if (gi + 1 < G) request_scales(gi + 1);
#pragma unroll
    for (int j = 0; j < RB; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float t = __fmul_rn((float)acc[j][q], ssv[j][q]);
        t = __fmul_rn(t, wsv);
        sum[j][q] = __fadd_rn(sum[j][q], t);
      }
      acc[j] = (v4i){0, 0, 0, 0};
    }
  };

  const int cpg = gs >= 64 ? gs / 64 : 1;   // chunks per group
  const int sub = gs >= 64 ? 1 : 64 / gs;   // groups per chunk
  for (int c0 = 0; c0 < nch; c0 += D) {
#pragma unroll
    for (int s = 0; s < D; ++s) {
      const int c = c0 + s;
      if (c < nch) {
        if (sub == 1) {
#pragma unroll
          for (int j = 0; j < RB; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[s][j], b[s], acc[j], 0, 0, 0);
          if ((c + 1) % cpg == 0) fold(c / cpg);
        } else {
          for (int t = 0; t < sub; ++t) {
            const int gi = c * sub + t;
            if (gi >= G) break;   // (K_pad beyond K)
            const bool mine = (g4 * 16) / gs == t;   // this lane's 16 k belong to group t of the chunk
#pragma unroll
            for (int j = 0; j < RB; ++j) {
              const v4i am = mine ? a[s][j] : (v4i){0, 0, 0, 0};
              acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(am, b[s], acc[j], 0, 0, 0);
            }
            fold(gi);
          }
        }
      }
      request(s, c + D);
    }
  }

  // ---- alpha / beta, then the common tail; acc element q of lane l is row (l / 16) * 4 + q, column l % 16 ----
  if (col >= N) return;
  const float bias = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, col) : 0.0f;
#pragma unroll
  for (int j = 0; j < RB; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = row0 + j * 16 + g4 * 4 + q;
      if (m >= M) continue;
      const int64_t o = (int64_t)m * p.ldc + col;
      float y = sum[j][q];
      if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
      if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, epi.dst_dt, o), epi.beta));
      zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_tail(epi, y, bias, m, col));
    }
}

bool zmi_pergroup_group_size_ok(int64_t gs) { return gs > 0 && (gs % 64 == 0 || gs == 32 || gs == 16); }

hipError_t zmi_launch_gemm_pergroup(const ZmiProblem &p, const ZmiEpilogue &epi, hipStream_t stream) {
  const int G = epi.n_groups;
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || G <= 0 || p.K % G != 0) return hipErrorInvalidValue;
  const int gs = p.K / G;
  if (!zmi_pergroup_group_size_ok(gs)) return hipErrorInvalidValue;
  if (epi.src_scale_mode != ZMI_SS_GROUP_PTR || epi.wei_scale_mode != 3 || !p.src_scale_ptr || !p.wei_scale_ptr)
    return hipErrorInvalidValue;
  if (p.a_is_u8 || epi.has_zp || epi.gated_act) return hipErrorInvalidValue;   // symmetric s8 rows only
  if (p.lda % 16 != 0 || ((uintptr_t)p.A) % 16 != 0 || p.lda < p.K) return hipErrorInvalidValue;   // 16-byte row loads
  const int n_cb = (int)(zmi_blob_npad(p.N) / 16);
  const int rb = p.M <= 16 ? 1 : 4;
  const int n_rb = (p.M + 16 * rb - 1) / (16 * rb);
  const int n_items = n_cb * n_rb;
  const dim3 grid((n_items + PG_WAVES - 1) / PG_WAVES), block(PG_WAVES * 64);
  if (rb == 1) hipLaunchKernelGGL((zmi_gemm_pergroup_kernel<1, 8>), grid, block, 0, stream, p, epi, n_cb, n_items, gs);
  else hipLaunchKernelGGL((zmi_gemm_pergroup_kernel<4, 4>), grid, block, 0, stream, p, epi, n_cb, n_items, gs);
  return hipGetLastError();
}

// ---- per-group dynamic quantization -----------------------------------------------------------
// Reference: the per-group symmetric kernels of the dynamic reorder
// (zendnnl/src/lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/
// per_group_avx512_f32_fma_kernel.cpp:78-86 scale, :276-292 quantization): per (row, group)
// absmax over finite values, scale = max(absmax, 1e-10) / 127 clamped to >= 1e-10,
// q = (int8) nearbyint(v / scale) with the true division, non-finite -> 0; i.e. the per-token
// rule applied to every group of a row.  One workgroup per row, one wavefront per group in turn.
template <bool BF16>
__global__ __launch_bounds__(256) void zmi_quant_groups_kernel(const void *x, int64_t ldx, int K, int G, int8_t *q,
                                                               int64_t ldq, float *scales, void *user_scales,
                                                               int32_t user_dt) {
  const int m = blockIdx.x, lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int gs = K / G;
  for (int g = wave; g < G; g += 4) {
    const int64_t base = (int64_t)m * ldx + (int64_t)g * gs;
    auto ld = [&](int k) { return BF16 ? zmi_bf16_to_f32(((const uint16_t *)x)[base + k]) : ((const float *)x)[base + k]; };
    float amax = 0.0f;
    for (int k = lane; k < gs; k += 64) {
      const float a = fabsf(ld(k));
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if (amax < 1e-10f) amax = 1e-10f;
    float s = __fdiv_rn(amax, 127.0f);
    if (s < 1e-10f) s = 1e-10f;
    const float inv = __fdiv_rn(1.0f, s);
    if (lane == 0) {
      scales[(int64_t)m * G + g] = s;
      if (user_scales) {
        if (user_dt == ZMI_DT_BF16) ((uint16_t *)user_scales)[(int64_t)m * G + g] = zmi_f32_to_bf16_rne(s);
        else ((float *)user_scales)[(int64_t)m * G + g] = s;
      }
    }
    int8_t *dst = q + (int64_t)m * ldq + (int64_t)g * gs;
    for (int k = lane; k < gs; k += 64) dst[k] = zmi_quant_elem(ld(k), s, inv);
  }
}

hipError_t zmi_launch_quant_groups(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, int8_t *q,
                                   int64_t ldq, float *scales, void *user_scales, int32_t user_dt, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  if (G <= 0 || K % G != 0 || (x_dt != ZMI_DT_BF16 && x_dt != ZMI_DT_F32)) return hipErrorInvalidValue;
  if (x_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_groups_kernel<true>, dim3((unsigned)M), dim3(256), 0, stream, x, ldx, (int)K, (int)G, q,
                       ldq, scales, user_scales, user_dt);
  else
    hipLaunchKernelGGL(zmi_quant_groups_kernel<false>, dim3((unsigned)M), dim3(256), 0, stream, x, ldx, (int)K, (int)G, q,
                       ldq, scales, user_scales, user_dt);
  return hipGetLastError();
}
