// Large-M int8 GEMM for gfx950 (MFMA-bound): C = epilogue(A[M,K] x blob), A is
// u8 / s8 row-major, the weights are the prepacked fragment blob, accumulation
// is s32 on v_mfma_i32_32x32x32_i8.
//
// Replaces the reference's aocl_gemm_u8s8s32o* / aocl_gemm_s8s8s32o*[_sym_quant]
// call sites (zendnnl/src/lowoha_operators/matmul/backends/aocl/
// aocl_kernel.cpp:1190-1295) and, in grouped form, the per-expert GEMMs of
// group_matmul_run_parallel_dispatch (matmul/group_matmul/
// group_matmul_dispatch.cpp:1096).
//
// Workgroup = 4 wavefronts = BM x 256 output tile (gated: BM x 128 outputs from
// 256 weight columns).  Each wavefront owns all BM rows of a 64-column slice:
//   * B fragments go straight from global memory to VGPRs, 16 B per lane, fully
//     coalesced and unshared between wavefronts, prefetched one K stage ahead;
//   * the A tile (shared by the 4 wavefronts) is staged through LDS, double
//     buffered, row stride padded to 144 B so the 16-byte MFMA operand reads of
//     16 consecutive rows fall in 16 different 16-byte bank groups.
// One barrier per 128-wide K stage.
#include "zmi_device.h"
#include "zmi_launch.h"

#define G_BK 128
#define G_LDS_STRIDE 144
#define G_THREADS 256

template <int BM>
struct GemmSmem {
  int8_t a[2][BM][G_LDS_STRIDE];
};

// Decodes blockIdx.x into (problem, tile row, tile column).  Work items are
// numbered so that the 8 XCDs (which receive consecutive workgroup ids round
// robin) each get a contiguous range, and inside a range tiles sharing weight
// columns and activation rows are neighbours, so every XCD's private L2 sees a
// compact working set.
struct TileCoord {
  int prob;
  int tm, tn;
  bool valid;
};

template <int BM>
__device__ __forceinline__ TileCoord zmi_tile_coord(const ZmiProblem &p0, const ZmiProblem *probs,
                                                    int n_prob, bool gated, int n_items, int m_lo,
                                                    ZmiProblem &out) {
  // a gated tile produces 128 output columns from 256 weight columns
  const int cols_per_tile = gated ? 128 : 256;
  TileCoord tc;
  const int nb = gridDim.x;
  int b = blockIdx.x;
  // XCD-contiguous renumbering (only when the grid divides evenly)
  int id = (nb % 8 == 0) ? (b % 8) * (nb / 8) + b / 8 : b;
  tc.valid = id < n_items;
  tc.prob = 0;
  tc.tm = tc.tn = 0;
  if (!tc.valid) return tc;
  if (!probs) {
    out = p0;
    const int tiles_m = (out.M + BM - 1) / BM;
    const int ncols = gated ? out.N / 2 : out.N;
    const int tiles_n = (ncols + cols_per_tile - 1) / cols_per_tile;
    const int GM = tiles_m < 4 ? tiles_m : 4;
    const int per_group = GM * tiles_n;
    const int group = id / per_group;
    const int first_m = group * GM;
    const int gm = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int r = id % per_group;
    tc.tm = first_m + r % gm;
    tc.tn = r / gm;
    return tc;
  }
  // grouped: items are laid out problem after problem, n-major inside a problem
  int base = 0;
  for (int e = 0; e < n_prob; ++e) {
    const int M = probs[e].M;
    if (M <= m_lo) continue;
    const int tiles_m = (M + BM - 1) / BM;
    const int ncols = gated ? probs[e].N / 2 : probs[e].N;
    const int tiles_n = (ncols + cols_per_tile - 1) / cols_per_tile;
    const int cnt = tiles_m * tiles_n;
    if (id < base + cnt) {
      out = probs[e];
      tc.prob = e;
      const int r = id - base;
      tc.tm = r % tiles_m;
      tc.tn = r / tiles_m;
      return tc;
    }
    base += cnt;
  }
  tc.valid = false;
  return tc;
}

template <int BM>
__global__ __launch_bounds__(G_THREADS) void zmi_gemm_mfma_kernel(ZmiProblem p0, const ZmiProblem *probs,
                                                                  int n_prob, int n_items, int m_lo,
                                                                  ZmiEpilogue epi) {
  constexpr int MI = BM / 32;            // MFMA row tiles per wavefront
  constexpr int A_CHUNKS = BM * 8 / G_THREADS;   // 16-byte chunks of the A stage per thread
  extern __shared__ __attribute__((aligned(16))) int8_t smem_raw[];
  GemmSmem<BM> &sm = *reinterpret_cast<GemmSmem<BM> *>(smem_raw);

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const bool gated = epi.gated_act != 0;
  ZmiProblem p;
  const TileCoord tc = zmi_tile_coord<BM>(p0, probs, n_prob, gated, n_items, m_lo, p);
  if (!tc.valid) return;

  const int M = p.M, N = p.N, K = p.K;
  const int64_t K_pad = zmi_blob_kpad(K), N_pad = zmi_blob_npad(N);
  const int64_t kblocks = K_pad / 32;
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int m0 = tc.tm * BM;

  // column blocks (32 wide) this wavefront multiplies
  int64_t nb0, nb1;
  int n_out0;            // first output column of the wavefront
  bool wave_active;
  if (!gated) {
    n_out0 = tc.tn * 256 + wave * 64;
    nb0 = n_out0 / 32;
    nb1 = nb0 + 1;
    wave_active = n_out0 < N_pad;
  } else {
    // [gate | up] halves: output column c needs weight columns c and c + N/2
    const int half = N / 2;
    n_out0 = tc.tn * 128 + wave * 32;
    nb0 = n_out0 / 32;
    nb1 = nb0 + half / 32;
    wave_active = n_out0 < half;
  }
  const v4i *bp0 = (const v4i *)(tiles + nb0 * kblocks * 1024) + lane;
  const v4i *bp1 = (const v4i *)(tiles + nb1 * kblocks * 1024) + lane;
  if (!wave_active) { bp0 = (const v4i *)tiles + lane; bp1 = bp0; }

  v16i acc[MI][2];
  #pragma unroll
  for (int mi = 0; mi < MI; ++mi)
    #pragma unroll
    for (int ni = 0; ni < 2; ++ni)
      #pragma unroll
      for (int j = 0; j < 16; ++j) acc[mi][ni][j] = 0;

  // A staging: thread t owns chunks c = i*256 + t -> row c/8, 16-byte column c%8
  const int8_t *A = (const int8_t *)p.A;
  const int64_t lda = p.lda;
  const uint32_t xor_mask = p.a_is_u8 ? 0x80808080u : 0u;
  const int a_kc = tid % 8;
  const int8_t *a_src[A_CHUNKS];
  #pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    int row = i * (G_THREADS / 8) + tid / 8;
    int gr = m0 + row;
    if (gr > M - 1) gr = M - 1;
    a_src[i] = A + (int64_t)gr * lda + a_kc * 16;
  }

  const int nk = (int)(K_pad / G_BK);

  auto load_a = [&](int kt, v4i (&r)[A_CHUNKS]) {
    const int k = kt * G_BK + a_kc * 16;
    #pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      v4i v = {0, 0, 0, 0};
      if (k < K) v = *(const v4i *)(a_src[i] + (int64_t)kt * G_BK);
      // u8 -> s8 shift; the blob's padded K rows are zero, so padded A columns need no care
      if (xor_mask) { v[0] ^= xor_mask; v[1] ^= xor_mask; v[2] ^= xor_mask; v[3] ^= xor_mask; }
      r[i] = v;
    }
  };
  auto store_a = [&](int buf, const v4i (&r)[A_CHUNKS]) {
    #pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      int row = i * (G_THREADS / 8) + tid / 8;
      *(v4i *)&sm.a[buf][row][a_kc * 16] = r[i];
    }
  };
  auto load_b = [&](int kt, v4i (&b)[2][4]) {
    #pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      b[0][kb] = bp0[(int64_t)(kt * 4 + kb) * 64];
      b[1][kb] = bp1[(int64_t)(kt * 4 + kb) * 64];
    }
  };
  auto compute = [&](int buf, const v4i (&b)[2][4]) {
    #pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      v4i a[MI];
      #pragma unroll
      for (int mi = 0; mi < MI; ++mi)
        a[mi] = *(const v4i *)&sm.a[buf][mi * 32 + lane % 32][kb * 32 + (lane / 32) * 16];
      #pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        acc[mi][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[mi], b[0][kb], acc[mi][0], 0, 0, 0);
        acc[mi][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[mi], b[1][kb], acc[mi][1], 0, 0, 0);
      }
    }
  };

  v4i areg[A_CHUNKS];
  v4i bA[2][4], bB[2][4];
  load_a(0, areg);
  load_b(0, bA);
  store_a(0, areg);
  __syncthreads();

  for (int kt = 0; kt < nk; kt += 2) {
    // even stage: compute from bA / LDS buffer 0, prefetch stage kt+1 into bB / buffer 1
    const bool has1 = kt + 1 < nk;
    if (has1) { load_a(kt + 1, areg); load_b(kt + 1, bB); }
    if (wave_active) compute(0, bA);
    if (has1) store_a(1, areg);
    __syncthreads();
    if (!has1) break;
    // odd stage
    const bool has2 = kt + 2 < nk;
    if (has2) { load_a(kt + 2, areg); load_b(kt + 2, bA); }
    if (wave_active) compute(1, bB);
    if (has2) store_a(0, areg);
    __syncthreads();
  }

  if (!wave_active) return;

  // ------------------------------------------------------------------ epilogue
  // acc[mi][ni][j] is row m0 + mi*32 + (j/4)*8 + (lane/32)*4 + j%4,
  // column block ni, column lane%32.
  const void *bias = p.bias;
  const int cl = lane % 32;

  if (!gated) {
    ZmiColCtx cc[2];
    int ncol[2];
    #pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      ncol[ni] = n_out0 + ni * 32 + cl;
      cc[ni] = zmi_col_ctx(epi, p, colsum, ncol[ni], N);
    }
    const bool raw = zmi_epilogue_is_raw_s32(epi, bias);
    #pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      #pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int m = m0 + mi * 32 + (j / 4) * 8 + (lane / 32) * 4 + (j % 4);
        if (m >= M) continue;
        const float rs = raw ? 1.0f : zmi_row_scale(epi, p, m);
        #pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
          const int n = ncol[ni];
          if (n >= N) continue;
          const int64_t o = (int64_t)m * p.ldc + n;
          if (raw) {
            ((int32_t *)p.dst)[o] = acc[mi][ni][j] + cc[ni].comp;
          } else {
            float y = zmi_epilogue_value(epi, acc[mi][ni][j], cc[ni], rs, m, n, p.dst, p.ldc);
            zmi_store(p.dst, epi.dst_dt, o, y);
          }
        }
      }
    }
  } else {
    const int half = N / 2;
    const int n = n_out0 + cl;           // output column; gate = n, up = n + half
    ZmiColCtx cg = zmi_col_ctx(epi, p, colsum, n, half);
    ZmiColCtx cu = zmi_col_ctx(epi, p, colsum, n < half ? n + half : N, N);
    #pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      #pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int m = m0 + mi * 32 + (j / 4) * 8 + (lane / 32) * 4 + (j % 4);
        if (m >= M || n >= half) continue;
        const float rs = zmi_row_scale(epi, p, m);
        float g = zmi_epilogue_value(epi, acc[mi][0][j], cg, rs, m, n, p.dst, p.ldc);
        float u = zmi_epilogue_value(epi, acc[mi][1][j], cu, rs, m, n + half, p.dst, p.ldc);
        if (epi.dst_dt == ZMI_DT_BF16) {
          // the unfused path stores the GEMM result as bf16 before the activation reads it
          g = zmi_bf16_to_f32(zmi_f32_to_bf16(g));
          u = zmi_bf16_to_f32(zmi_f32_to_bf16(u));
        }
        const float r = zmi_gated(epi.gated_act, g, u);
        zmi_store(p.dst, epi.dst_dt, (int64_t)m * p.ldc + n, r);
      }
    }
  }
}

template <int BM>
static hipError_t launch_bm(const ZmiProblem &p0, const ZmiProblem *probs, int n_prob, int n_items,
                            int m_lo, const ZmiEpilogue &epi, hipStream_t stream) {
  const size_t smem = sizeof(GemmSmem<BM>);
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)zmi_gemm_mfma_kernel<BM>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  // round the grid up to a multiple of 8 so the XCD renumbering applies
  int grid = (n_items + 7) / 8 * 8;
  hipLaunchKernelGGL(zmi_gemm_mfma_kernel<BM>, dim3(grid), dim3(G_THREADS), smem, stream, p0, probs, n_prob,
                     n_items, m_lo, epi);
  return hipGetLastError();
}

static int items_of(const ZmiProblem &p, int BM, bool gated) {
  const int tiles_m = (p.M + BM - 1) / BM;
  const int ncols = gated ? p.N / 2 : p.N;
  const int per = gated ? 128 : 256;
  return tiles_m * ((ncols + per - 1) / per);
}

hipError_t zmi_launch_gemm_mfma(const ZmiProblem &p, const ZmiEpilogue &epi, int BM, hipStream_t stream) {
  if (p.M <= 0) return hipSuccess;
  const int n_items = items_of(p, BM, epi.gated_act != 0);
  switch (BM) {
  case 64: return launch_bm<64>(p, nullptr, 1, n_items, 0, epi, stream);
  case 256: return launch_bm<256>(p, nullptr, 1, n_items, 0, epi, stream);
  default: return launch_bm<128>(p, nullptr, 1, n_items, 0, epi, stream);
  }
}

// Runs every problem with M > m_lo.  probs_host mirrors probs_dev and sizes the
// grid; when it is null (row counts known only on the device) the grid is
// worst_items and surplus workgroups exit at once.
hipError_t zmi_launch_gemm_mfma_group(const ZmiProblem *probs_host, const ZmiProblem *probs_dev, int n_prob,
                                      int m_lo, int worst_items, const ZmiEpilogue &epi, int BM,
                                      hipStream_t stream) {
  int n_items = worst_items;
  if (probs_host) {
    n_items = 0;
    for (int e = 0; e < n_prob; ++e)
      if (probs_host[e].M > m_lo) n_items += items_of(probs_host[e], BM, epi.gated_act != 0);
  }
  if (n_items <= 0) return hipSuccess;
  ZmiProblem dummy = {};
  switch (BM) {
  case 64: return launch_bm<64>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
  case 256: return launch_bm<256>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
  default: return launch_bm<128>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
  }
}
