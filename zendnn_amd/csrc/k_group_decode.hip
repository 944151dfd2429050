// Decode-shaped grouped int8 GEMM for gfx950: the experts of a grouped (MoE) launch that have
// at most 16 rows, optionally with the gated activation in the epilogue.
//
// Reference counterpart: the in-house decode microkernel with its fused gate / up epilogue
// (zendnnl/src/lowoha_operators/matmul/group_matmul/custom_kernel/ukernel/int8_microkernel.cpp:196-606;
// gate / up column pairing: custom_kernel/pack.hpp:126-142; selection per expert:
// group_matmul/group_matmul_dispatch.cpp:779).  With a handful of rows an expert's GEMM is a
// stream of its weights; the MFMA-bound kernel (k_ring.hip) would push them through 64-row tiles.
//
//   * one workgroup of 8 wavefronts per (expert, 32 output columns); experts with no rows or with
//     more than 16 (the MFMA-bound kernel's) leave at once;
//   * wavefront w streams the w-th eighth of K of the column block, 16-byte-per-lane loads, up to 16
//     of them in flight, straight from the blob into v_mfma_i32_16x16x64_i8 operands;
//   * gated (columns [gate | up]): the same wavefront streams the matching up block c + N/2 behind the
//     gate block -- every chunk's registers are re-requested for the up block as soon as its MFMAs are
//     issued -- so silu(gate) * up is local to a thread and the two GEMMs' results never leave the chip;
//   * the rows of a grouped launch are in fragment order (zmi_afrag_off): the 16 x 64 operand of a
//     chunk is 4 runs of 256 bytes there, so it is loaded straight from global memory (L2), no LDS;
//   * the per-column / per-row constants are requested behind the weights as raw words;
//   * partial tiles of the 8 wavefronts meet in LDS (integers: any order, bit-exact), one thread
//     finishes one output element with the arithmetic of the MFMA-bound kernel's epilogue, so an
//     expert's result does not depend on which of the two kernels took it.
#include "zmi_device.h"
#include "zmi_launch.h"

#define GD_WAVES 8
#define GD_THREADS (GD_WAVES * 64)

template <bool GATED>
__global__ __launch_bounds__(GD_THREADS, 4) void zmi_gemm_group_decode_kernel(const ZmiProblem *probs, int n_blk_max,
                                                                              ZmiEpilogue epi) {
  __shared__ int32_t red[GD_WAVES * (GATED ? 2 : 1) * 512];
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int e = (int)blockIdx.x / n_blk_max, blk = (int)blockIdx.x % n_blk_max;
  const ZmiProblem p = probs[e];
  const int M = p.M, N = p.N, K = p.K;
  if (M <= 0 || M > 16) return;
  const int half = N / 2;
  const int ncols = GATED ? half : N;          // output columns
  if (blk * 32 >= ncols) return;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nchunks = K_pad / 64;
  const int c_begin = wave * nchunks / GD_WAVES;
  const int c_end = (wave + 1) * nchunks / GD_WAVES;
  const int c16 = lane % 16, g = lane / 16;
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  // weight operand of chunk c, 16-column half h of column block nb: fragments (nb, 2c + g/2), lane (g%2)*32 + h*16 + c16
  const uint8_t *wsrc = tiles + (int64_t)blk * zmi_blob_nb_stride(K) + (g / 2) * 1024 + ((g % 2) * 32 + c16) * 16;
  const int64_t up_off = GATED ? (int64_t)(half / 32) * zmi_blob_nb_stride(K) : 0;
  // row operand of chunk c: rows 0..15 of the first fragment row, fragments 2c + g/2, lane (g%2)*32 + row
  const uint8_t *asrc = (const uint8_t *)p.A + (g / 2) * 1024 + ((g % 2) * 32 + c16) * 16;

  v4i acc[GATED ? 2 : 1][2];
#pragma unroll
  for (int s = 0; s < (GATED ? 2 : 1); ++s) { acc[s][0] = (v4i){0, 0, 0, 0}; acc[s][1] = (v4i){0, 0, 0, 0}; }

  for (int c0 = c_begin; c0 < c_end; c0 += 8) {
    v4i a[8], b[8][2];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      // past the end of the slice: re-read its first chunk (valid memory), the row operand is zeroed below
      const int c = c0 + u < c_end ? c0 + u : c_begin;
      b[u][0] = __builtin_nontemporal_load((const v4i *)(wsrc + (int64_t)c * 2048));
      b[u][1] = __builtin_nontemporal_load((const v4i *)(wsrc + (int64_t)c * 2048 + 256));
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + u < c_end ? c0 + u : c_begin;
      a[u] = *(const v4i *)(asrc + (int64_t)c * 2048);
      if (c0 + u >= c_end) a[u] = (v4i){0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      acc[0][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][0], acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][1], acc[0][1], 0, 0, 0);
      if (GATED) {
        const int c = c0 + u < c_end ? c0 + u : c_begin;
        b[u][0] = __builtin_nontemporal_load((const v4i *)(wsrc + up_off + (int64_t)c * 2048));
        b[u][1] = __builtin_nontemporal_load((const v4i *)(wsrc + up_off + (int64_t)c * 2048 + 256));
      }
    }
    if (GATED) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        acc[1][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][0], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u], b[u][1], acc[1][1], 0, 0, 0);
      }
    }
  }

  // this thread's output element: row tid / 32, output column blk * 32 + tid % 32; constants as raw words
  const int e_row = tid / 32, e_col = tid % 32;
  const int e_n = blk * 32 + e_col;
  const int n_ok = e_n < ncols ? e_n : ncols - 1, m_ok = e_row < M ? e_row : M - 1;
  const ZmiColRaw craw0 = zmi_col_raw(epi, p, colsum, n_ok);
  ZmiColRaw craw1 = craw0;
  if (GATED) craw1 = zmi_col_raw(epi, p, colsum, n_ok + half);
  const int32_t zp_word = zmi_zp_raw(p, colsum);
  const uint32_t rs_word = zmi_row_scale_raw(epi, p, colsum, m_ok);

  // ---- cross-wavefront reduction through LDS ----
  constexpr int SETS = GATED ? 2 : 1;
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int q = 0; q < 4; ++q) red[(wave * SETS + s) * 512 + (h * 4 + q) * 64 + lane] = acc[s][h][q];
  __syncthreads();
  if (e_n >= ncols || e_row >= M) return;
  // acc[s][h][q] of lane l is row (l/16)*4 + q, column h*16 + l%16
  const int off = ((e_col / 16) * 4 + e_row % 4) * 64 + (e_row / 4) * 16 + e_col % 16;
  int32_t sum[SETS];
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
    sum[s] = 0;
#pragma unroll
    for (int w = 0; w < GD_WAVES; ++w) sum[s] += red[(w * SETS + s) * 512 + off];
  }
  const float rs = zmi_row_scale_from_raw(epi, p, rs_word, m_ok);
  if (!GATED) {
    const ZmiColCtx cc = zmi_col_ctx_raw(epi, p, craw0, zp_word, e_n, n_ok, N);
    zmi_finish_element_ring(p, epi, cc, rs, sum[0], e_row, e_n);
    return;
  }
  const ZmiColCtx cg = zmi_col_ctx_raw(epi, p, craw0, zp_word, e_n, n_ok, half);
  const ZmiColCtx cu = zmi_col_ctx_raw(epi, p, craw1, zp_word, e_n + half, n_ok + half, N);
  zmi_finish_gated_ring(p, epi, cg, cu, rs, sum[0], sum[1], e_row, e_n);
}

bool zmi_group_decode_takes(const ZmiEpilogue &epi, int N) {
  const bool gated = epi.gated_act != 0;
  // gated: the up block of output block c is column block c + N/2/32; an element-wise post-op in front of the
  // activation is the MFMA-bound kernel's interpreter's
  if (gated && ((N / 2) % 32 != 0 || epi.fast_kind != ZMI_EK_NONE)) return false;
  if (epi.n_groups > 0) return false;
  return zmi_env(ZE_NO_GROUP_DECODE) == nullptr;
}

hipError_t zmi_launch_gemm_group_decode(const ZmiProblem *probs_dev, int n_prob, int max_out_cols, const ZmiEpilogue &epi,
                                        hipStream_t stream) {
  if (n_prob <= 0 || max_out_cols <= 0) return hipSuccess;
  const int n_blk = (max_out_cols + 31) / 32;
  const dim3 grid((unsigned)((int64_t)n_prob * n_blk)), block(GD_THREADS);
  if (epi.gated_act != 0) hipLaunchKernelGGL(zmi_gemm_group_decode_kernel<true>, grid, block, 0, stream, probs_dev, n_blk, epi);
  else hipLaunchKernelGGL(zmi_gemm_group_decode_kernel<false>, grid, block, 0, stream, probs_dev, n_blk, epi);
  return hipGetLastError();
}
