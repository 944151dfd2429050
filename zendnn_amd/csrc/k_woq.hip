// Weight-only quantization: C[M,N] = epilogue(A[M,K] bf16 x dequant(W[K,N] 4-bit)), f32 accumulation on the bf16 MFMA.
//
// Reference: matmul_direct with a bf16 source, s4 / u4 weights and no dynamic_quant turns every 4-bit code into a bf16
// value once (cvt_int4_to_bf16, lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:43-139:
//   f = float(code); f = (f - zp) * scale, or (f - 8) * scale + zp for u4 codes with a bf16 zero-point;
//   w = bfloat16_t(f)), caches the bf16 matrix and runs a bf16 GEMM with f32 accumulation on it.  Here the weights stay
// 4-bit in memory (a quarter of the bf16 matrix, the bound of a decode-shaped call) and every workgroup makes the
// same bf16 values in registers, with the same three f32 operations and the same rounding, right before the MFMA.
//
// Tiles: [N/32][K/64] pieces of 1 KiB; lane l of a wavefront owns 16 bytes of a piece = 4 dwords, dword t holding the
// 8 codes (k = 64*kc + 16*t + 8*(l/32) + j, j = 0..7 from the low nibble up; n = 32*nb + l%32): the B operand of four
// v_mfma_f32_32x32x16_bf16 in a row, one coalesced 16-byte load per lane.
//
// Kernel: one workgroup per 32 columns (and per 32 * MT rows), its wavefronts take the K chunks in turn (kc = wave,
// wave + W, ...), each keeping 8 chunks of weights in flight; the wavefronts' f32 sums meet in LDS, then alpha / beta /
// bias / post-ops / store per element (compute_matmul, operators/matmul/matmul_ref_kernel.cpp:877-896 and the post-op
// loop after it).
#include <hip/hip_runtime.h>

#include "../../include/zmi_lowoha.h"
#include "zmi_device.h"
#include "zmi_launch.h"

typedef __bf16 woq_bf16x8 __attribute__((ext_vector_type(8)));
typedef float woq_f32x16 __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------------------------------- tiles
__global__ __launch_bounds__(256) void zmi_woq_tiles_kernel(const uint8_t *packed, int64_t K, int64_t N, int64_t ldb,
                                                            int transB, uint32_t *out, int64_t n_dwords) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_dwords) return;
  const int64_t nkc = (K + 63) / 64;
  const int t = (int)(i & 3), lane = (int)((i >> 2) & 63);
  const int64_t piece = i >> 8, kc = piece % nkc, nb = piece / nkc;
  const int64_t n = nb * 32 + (lane & 31), k0 = kc * 64 + t * 16 + (lane >> 5) * 8;
  uint32_t d = 0;
  if (n < N) {
    for (int j = 0; j < 8; ++j) {
      const int64_t k = k0 + j;
      if (k >= K) break;
      const int64_t idx = transB ? n * ldb + k : k * ldb + n;
      const uint32_t byte = packed[idx >> 1];
      d |= ((idx & 1) ? (byte >> 4) : (byte & 15u)) << (4 * j);
    }
  }
  out[i] = d;
}

hipError_t zmi_launch_woq_tiles(const void *packed, int64_t K, int64_t N, int64_t ldb, bool transB, uint32_t *out,
                                hipStream_t stream) {
  const int64_t n_dwords = zmi_woq_tiles_bytes(K, N) / 4;
  hipLaunchKernelGGL(zmi_woq_tiles_kernel, dim3((unsigned)((n_dwords + 255) / 256)), dim3(256), 0, stream,
                     (const uint8_t *)packed, K, N, ldb, transB ? 1 : 0, out, n_dwords);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------- GEMM
// Q: 0 = s4 codes, no zero-point; 1 = s4 codes with a zero-point; 2 = u4 codes, (code - zp) * scale;
//    3 = u4 codes, (code - 8) * scale + zp
template <int Q>
__device__ __forceinline__ woq_bf16x8 woq_dequant(uint32_t d, float s, float z) {
  uint32_t o[4];
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    float f[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int j = 2 * jj + h;
      const int v = Q >= 2 ? (int)((d >> (4 * j)) & 15u) : ((int)(d << (28 - 4 * j)) >> 28);
      float x = (float)v;
      if (Q == 0) x = __fmul_rn(x, s);
      else if (Q == 3) x = __fadd_rn(__fmul_rn(__fsub_rn(x, 8.0f), s), z);
      else x = __fmul_rn(__fsub_rn(x, z), s);
      f[h] = x;
    }
    // (round to nearest even; f32 subnormals count as zero in this mode, as in the reference's bfloat16_t(float))
    o[jj] = zmi_pack_bf16(f[0], f[1]);
  }
  uint4 r = {o[0], o[1], o[2], o[3]};
  return __builtin_bit_cast(woq_bf16x8, r);
}

__device__ __forceinline__ uint4 woq_load_a(const ZmiWoqProblem &p, int row, int k) {
  uint4 r = {0u, 0u, 0u, 0u};
  if (row >= p.M || k >= p.K) return r;
  const uint16_t *a = (const uint16_t *)p.A;
  if (p.a_fast) return *(const uint4 *)(a + (int64_t)row * p.lda + k);
  uint32_t e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int kk = k + j;
    e[j] = kk < p.K ? (uint32_t)a[p.transA ? (int64_t)kk * p.lda + row : (int64_t)row * p.lda + kk] : 0u;
  }
  r.x = e[0] | (e[1] << 16); r.y = e[2] | (e[3] << 16); r.z = e[4] | (e[5] << 16); r.w = e[6] | (e[7] << 16);
  return r;
}

__device__ __forceinline__ float woq_param(const void *ptr, int dt, int mode, float val, int g, int n, int N) {
  if (!ptr) return val;
  return zmi_ld_f32(ptr, dt, mode == 0 ? 0 : mode == 1 ? (int64_t)n : (int64_t)g * N + n);
}

template <int MT> struct WoqWaves { static constexpr int W = MT <= 2 ? 8 : 4; };

template <int MT, int Q>
__global__ __launch_bounds__(WoqWaves<MT>::W * 64) void zmi_gemm_woq_kernel(ZmiWoqProblem p, ZmiEpilogue epi) {
  constexpr int W = WoqWaves<MT>::W, U = 8;
  extern __shared__ float woq_red[];   // [W][MT * 16][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nb = blockIdx.x, m0 = blockIdx.y * 32 * MT;
  const int nc = min(nb * 32 + (lane & 31), p.N - 1), kh = lane >> 5;
  const int nkc = (p.K + 63) / 64;
  const uint4 *wt = (const uint4 *)p.tiles + (int64_t)nb * nkc * 64 + lane;
  const bool fine = p.scale_mode == 2 && (p.group_size & 63) != 0;

  woq_f32x16 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

  uint4 wq[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int kc = wave + u * W;
    wq[u] = kc < nkc ? wt[(int64_t)kc * 64] : uint4{0u, 0u, 0u, 0u};
  }
  zmi_set_f32_flush();
  for (int kc0 = wave; kc0 < nkc; kc0 += U * W) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kc = kc0 + u * W;
      if (kc >= nkc) break;
      // this chunk's rows and parameters are requested ahead of the next chunk of weights for this slot: loads come
      // back in the order they were asked for
      uint4 af[4][MT];
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < MT; ++i) af[t][i] = woq_load_a(p, m0 + 32 * i + (lane & 31), kc * 64 + t * 16 + kh * 8);
      int g = min((kc * 64) / p.group_size, p.n_groups - 1);
      float s = woq_param(p.scale, p.scale_dt, p.scale_mode, p.scale_val, g, nc, p.N);
      float z = Q == 0 ? 0.0f : woq_param(p.zp, p.zp_dt, p.zp_mode, p.zp_val, g, nc, p.N);
      const uint4 w = wq[u];
      const int kn = kc + U * W;
      if (kn < nkc) wq[u] = wt[(int64_t)kn * 64];
      const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (fine) {
          g = min((kc * 64 + t * 16 + kh * 8) / p.group_size, p.n_groups - 1);
          s = woq_param(p.scale, p.scale_dt, p.scale_mode, p.scale_val, g, nc, p.N);
          if (Q != 0) z = woq_param(p.zp, p.zp_dt, p.zp_mode, p.zp_val, g, nc, p.N);
        }
        const woq_bf16x8 b = woq_dequant<Q>(wd[t], s, z);
#pragma unroll
        for (int i = 0; i < MT; ++i)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(woq_bf16x8, af[t][i]), b, acc[i], 0, 0, 0);
      }
    }
  }
  // back to IEEE subnormals for the element-wise tail (the mode the other kernels' tails run in)
  __builtin_amdgcn_s_setreg(1 | (4 << 6) | (1 << 11), 3);

#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) woq_red[((wave * MT + i) * 16 + r) * 64 + lane] = acc[i][r];
  __syncthreads();
  for (int sidx = threadIdx.x; sidx < MT * 16 * 64; sidx += W * 64) {
    const int ln = sidx & 63, r = (sidx >> 6) & 15, i = sidx >> 10;
    const int m = m0 + 32 * i + 8 * (r >> 2) + 4 * (ln >> 5) + (r & 3), n = nb * 32 + (ln & 31);
    if (m >= p.M || n >= p.N) continue;
    float y = woq_red[sidx];
#pragma unroll
    for (int w = 1; w < W; ++w) y = __fadd_rn(y, woq_red[w * MT * 16 * 64 + sidx]);
    const int64_t o = (int64_t)m * p.ldc + n;
    if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
    if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, epi.dst_dt, o), epi.beta));
    // (-0 is the one value whose addition changes nothing, not even the sign of a zero)
    const float b = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, n) : -0.0f;
    zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_tail(epi, y, b, m, n));
  }
}

template <int MT>
static hipError_t woq_launch_q(const ZmiWoqProblem &p, const ZmiEpilogue &epi, int q, hipStream_t stream) {
  constexpr int W = WoqWaves<MT>::W;
  const int smem = W * MT * 16 * 64 * 4;
  const dim3 grid((unsigned)((p.N + 31) / 32), (unsigned)((p.M + 32 * MT - 1) / (32 * MT)));
  const void *f = q == 0 ? (const void *)zmi_gemm_woq_kernel<MT, 0> : q == 1 ? (const void *)zmi_gemm_woq_kernel<MT, 1>
                : q == 2 ? (const void *)zmi_gemm_woq_kernel<MT, 2> : (const void *)zmi_gemm_woq_kernel<MT, 3>;
  hipError_t e = zmi_func_smem_once(f, smem);
  if (e != hipSuccess) return e;
  switch (q) {
  case 0: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 0>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 1: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 1>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 2: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 2>), grid, dim3(W * 64), smem, stream, p, epi); break;
  default: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 3>), grid, dim3(W * 64), smem, stream, p, epi); break;
  }
  return hipGetLastError();
}

hipError_t zmi_launch_gemm_woq(const ZmiWoqProblem &p, const ZmiEpilogue &epi, hipStream_t stream) {
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || !p.A || !p.tiles || !p.dst || p.group_size <= 0 || p.n_groups <= 0 ||
      (p.scale_mode == 2 && (p.group_size % 8 != 0 || (int64_t)p.group_size * p.n_groups != p.K)) ||
      (p.a_fast && (p.transA || p.K % 8 != 0 || p.lda % 8 != 0 || ((uintptr_t)p.A & 15) != 0)) ||
      (p.M + 127) / 128 > 65535)
    return hipErrorInvalidValue;
  const int q = p.is_u4 ? (p.zp_float_domain ? 3 : 2) : (p.has_zp ? 1 : 0);
  if (p.is_u4 && !p.has_zp) return hipErrorInvalidValue;
  if (p.M <= 32) return woq_launch_q<1>(p, epi, q, stream);
  if (p.M <= 64) return woq_launch_q<2>(p, epi, q, stream);
  return woq_launch_q<4>(p, epi, q, stream);
}
