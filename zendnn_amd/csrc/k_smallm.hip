// Small-M (decode) int8 GEMM for gfx950 (HBM-bound weight streaming), any K:
// C[M<=128, N] = epilogue(A[M,K] x blob).  k_decode.hip takes these shapes when K_pad <= 4096
// (its rows fit LDS); this kernel takes the longer K.
//
// Replaces, for decode shapes, the same aocl_gemm_s8s8s32o*_sym_quant call site
// as the large-M kernel (zendnnl/src/lowoha_operators/matmul/backends/aocl/
// aocl_kernel.cpp:1239-1257) and the reference's in-house decode microkernel
// (matmul/group_matmul/custom_kernel/ukernel/int8_microkernel.cpp:196-606).
//
// The weights (K*N bytes) dominate the traffic and each byte is used once, so
// the kernel is organised around streaming them at full HBM rate:
//   * one workgroup per 32-column block of the blob (contiguous K_pad*32 bytes);
//   * its W wavefronts split K: wavefront w streams one contiguous slice with
//     16-byte-per-lane loads (all 64 lanes hit whole 256-byte segments) and keeps
//     several loads in flight before the first MFMA;
//   * the few activation rows come from L2 straight into the A operand
//     registers; v_mfma_i32_16x16x64_i8 turns each 2 KiB of weights into two
//     16x16 partial tiles per 16 rows;
//   * the W partial tiles are summed through LDS (integer, so the order is
//     immaterial and the result is bit-exact) and the epilogue runs once.
#include "zmi_device.h"
#include "zmi_fused_quant.h"
#include "zmi_launch.h"

// Optional fused per-token quantization (single-problem launches only).  The
// workgroups with the lowest indices quantize one source row each (same
// arithmetic as k_quant.hip) AFTER every wavefront has put its first weight
// loads in flight, publish the rows with a device-scope counter, and every
// workgroup waits for the counter before it reads the s8 rows.  The weight
// stream therefore hides the whole quantization, and the decode call is one launch.
// The wait is bounded; producers never wait for anything, and the host only
// uses this form when the whole grid is resident at once.
template <int MB, int UNROLL>
__global__ __launch_bounds__(1024) void zmi_gemm_smallm_kernel(ZmiProblem p, ZmiEpilogue epi, ZmiFusedQuant fq) {
  extern __shared__ __attribute__((aligned(16))) int32_t red[];   // [W][MB*2*4*64]
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int W = blockDim.x / 64;
  const int blk = blockIdx.x;   // one 32-column block of the blob
  const int M = p.M, N = p.N, K = p.K;
  const int64_t K_pad = zmi_blob_kpad(K);
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());

  // the two 16-column groups h = 0, 1 this workgroup multiplies
  const int wcol[2] = {blk * 32, blk * 32 + 16};
  const int *ocol = wcol;

  // lane role inside a 16x16x64 operand: column / row c16, k group g (16 bytes each)
  const int c16 = lane % 16, g = lane / 16;
  const uint8_t *bsrc[2];
  #pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t nb = wcol[h] / 32;
    const int coff = wcol[h] % 32;
    // fragment (nb, 2c + g/2), lane (g%2)*32 + coff + c16
    bsrc[h] = tiles + nb * zmi_blob_nb_stride(K) + (g / 2) * 1024 + ((g % 2) * 32 + coff + c16) * 16;
  }
  const int8_t *A = (const int8_t *)p.A;
  const uint32_t xor_mask = p.a_is_u8 ? 0x80808080u : 0u;

  v4i acc[MB][2];
  #pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    #pragma unroll
    for (int h = 0; h < 2; ++h) acc[mb][h] = (v4i){0, 0, 0, 0};

  const int nchunks = (int)(K_pad / 64);
  const int c_begin = (int)((int64_t)wave * nchunks / W);
  const int c_end = (int)((int64_t)(wave + 1) * nchunks / W);

  v4i b[UNROLL][2];
  auto load_b = [&](int c) {
    #pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      // past the end of the slice: re-read the slice's first chunk (valid memory), result unused
      const int cc = c + u < c_end ? c + u : c_begin;
      b[u][0] = *(const v4i *)(bsrc[0] + (int64_t)cc * 2048);
      b[u][1] = *(const v4i *)(bsrc[1] + (int64_t)cc * 2048);
    }
  };

  if (fq.x) {
    // producer workgroups quantize their rows before they start streaming (loads
    // return in order per wavefront: behind the weight loads the row would wait
    // for the whole first batch of HBM traffic)
    float *fred = reinterpret_cast<float *>(red);
    for (int row = blockIdx.x; row < M; row += gridDim.x) {
      zmi_fused_quant_row(fq, row, K, fred);
      zmi_fq_publish(fq, row);
    }
  }
  // The first group of weight loads goes out before anything else.  With fused
  // quantization wavefront 0 polls the counter first (a poll issued behind its
  // own weight loads would only return after them) and streams afterwards.
  if (!fq.x || wave != 0) load_b(c_begin);
  if (fq.x) {
    // (one waiting wavefront per workgroup; the others learn the outcome through LDS)
    if (wave == 0) {
      const bool ok = zmi_fq_wait(fq, M);
      if (lane == 0) red[0] = ok ? 1 : 0;
      load_b(c_begin);
    }
    __syncthreads();
    const bool rows_ok = red[0] != 0;
    __syncthreads();                 // (the partial tiles are written there later)
    if (!rows_ok) return;            // the wait ran out: nothing is computed from unpublished rows
    asm volatile("" ::: "memory");   // the row loads below stay below the wait
  }

  for (int c = c_begin; c < c_end; c += UNROLL) {
    if (c != c_begin) load_b(c);
    v4i a[UNROLL][MB];
    #pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int cc = c + u;
      const int k = cc * 64 + g * 16;
      #pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int r = mb * 16 + c16;
        v4i v = {0, 0, 0, 0};
        if (cc < c_end && r < M && k < K) {
          v = *(const v4i *)(A + (int64_t)r * p.lda + k);
          if (xor_mask) { v[0] ^= xor_mask; v[1] ^= xor_mask; v[2] ^= xor_mask; v[3] ^= xor_mask; }
        }
        a[u][mb] = v;
      }
    }
    #pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      #pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        // chunks past the end have zero A operands, so whatever b holds adds nothing
        acc[mb][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u][mb], b[u][0], acc[mb][0], 0, 0, 0);
        acc[mb][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u][mb], b[u][1], acc[mb][1], 0, 0, 0);
      }
  }

  // ---- cross-wavefront reduction through LDS ----
  constexpr int PER_WAVE = MB * 2 * 4 * 64;
  #pragma unroll
  for (int mb = 0; mb < MB; ++mb)
    #pragma unroll
    for (int h = 0; h < 2; ++h)
      #pragma unroll
      for (int j = 0; j < 4; ++j) red[wave * PER_WAVE + ((mb * 2 + h) * 4 + j) * 64 + lane] = acc[mb][h][j];
  __syncthreads();

  const int rows = M < MB * 16 ? M : MB * 16;

  // acc[mb][h][j] of lane l is row mb*16 + (l/16)*4 + j, column h*16 + l%16
  auto fetch = [&](int row, int h, int cidx) -> int32_t {
    const int mb = row / 16, rr = row % 16;
    const int off = ((mb * 2 + h) * 4 + rr % 4) * 64 + (rr / 4) * 16 + cidx;
    int32_t s = 0;
    for (int w = 0; w < W; ++w) s += red[w * PER_WAVE + off];
    return s;
  };

  for (int e = tid; e < rows * 32; e += blockDim.x) {
    const int row = e / 32, col = e % 32;
    const int h = col / 16, cidx = col % 16;
    const int n = ocol[h] + cidx;
    if (n >= N) continue;
    zmi_finish_element(p, epi, zmi_col_ctx(epi, p, colsum, n, N), zmi_row_scale(epi, p, row), fetch(row, h, cidx), row, n);
  }
}

template <int MB, int UNROLL>
static hipError_t launch_small(const ZmiProblem &p, int grid, int W, const ZmiEpilogue &epi, const ZmiFusedQuant &fq,
                               hipStream_t stream) {
  size_t smem = (size_t)W * MB * 2 * 4 * 64 * sizeof(int32_t);
  if (smem < 256) smem = 256;
  {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_smallm_kernel<MB, UNROLL>, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL((zmi_gemm_smallm_kernel<MB, UNROLL>), dim3(grid), dim3(W * 64), smem, stream, p, epi, fq);
  return hipGetLastError();
}

// Picks the number of K-splitting wavefronts: enough workgroups*wavefronts to
// keep about 8 wavefronts on every one of the 256 CUs, bounded by the chunks
// available, by 16 wavefronts per workgroup and by the LDS the reduction needs.
static int pick_waves(int grid, int MB, int64_t K_pad) {
  const int nchunks = (int)(K_pad / 64);
  int W = 4;
  while (W < 16 && (int64_t)grid * W < 2048) W *= 2;
  while (W > 1 && (size_t)W * MB * 2048 > 128 * 1024) W /= 2;
  while (W > 1 && W > nchunks) W /= 2;
  return W;
}

static hipError_t dispatch_small(const ZmiProblem &p, int grid, const ZmiEpilogue &epi, const ZmiFusedQuant &fq,
                                 hipStream_t stream) {
  if (grid <= 0) return hipSuccess;
  if (epi.gated_act != 0) return hipErrorInvalidValue;   // gated GEMMs are grouped launches: the large-M kernel
  const int64_t K_pad = zmi_blob_kpad(p.K);
  const int mb = (p.M + 15) / 16;
  if (mb <= 1) return launch_small<1, 8>(p, grid, pick_waves(grid, 1, K_pad), epi, fq, stream);
  if (mb <= 2) return launch_small<2, 4>(p, grid, pick_waves(grid, 2, K_pad), epi, fq, stream);
  if (mb <= 4) return launch_small<4, 2>(p, grid, pick_waves(grid, 4, K_pad), epi, fq, stream);
  return launch_small<8, 1>(p, grid, pick_waves(grid, 8, K_pad), epi, fq, stream);
}

static int small_blocks(const ZmiProblem &p) { return (int)(zmi_blob_npad(p.N) / 32); }

hipError_t zmi_launch_gemm_smallm(const ZmiProblem &p, const ZmiEpilogue &epi, hipStream_t stream) {
  if (p.M <= 0) return hipSuccess;
  if (p.M > 128) return hipErrorInvalidValue;
  ZmiFusedQuant none = {};
  return dispatch_small(p, small_blocks(p), epi, none, stream);
}

int zmi_smallm_grid(const ZmiProblem &p) { return small_blocks(p); }

// Same, with the per-token quantization of the source rows fused into the launch.
// Only valid when the whole grid is resident at once (zmi_smallm_grid(p) <= 2 * #CUs).
hipError_t zmi_launch_gemm_smallm_fused(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant &fq,
                                        hipStream_t stream) {
  if (p.M <= 0) return hipSuccess;
  if (p.M > 128) return hipErrorInvalidValue;
  return dispatch_small(p, small_blocks(p), epi, fq, stream);
}
