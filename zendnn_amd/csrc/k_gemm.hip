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
#include <type_traits>

#include "zmi_device.h"
#include "zmi_launch.h"

#define G_BK 128
#define G_LDS_STRIDE 144
#define G_THREADS 256

template <int BM>
struct GemmSmem {
  int8_t a[2][BM][G_LDS_STRIDE];
};

// Epilogue staging (reuses the A buffers): one 32 x 64 s32 tile per wavefront,
// row pitch 72 words so that the two half-waves of an accumulator store (rows
// 4 apart) fall in different halves of the banks, then BM row scales.
#define G_EPI_LD 72
#define G_EPI_WAVE_WORDS (32 * G_EPI_LD)
template <int BM>
constexpr size_t gemm_smem_bytes() {
  size_t a = sizeof(GemmSmem<BM>);
  size_t e = (size_t)4 * G_EPI_WAVE_WORDS * 4 + (size_t)BM * 4;
  return a > e ? a : e;
}

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
__global__ __launch_bounds__(G_THREADS, (BM > 128 ? 1 : 2)) void zmi_gemm_mfma_kernel(ZmiProblem p0, const ZmiProblem *probs,
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
  const int64_t nb_stride = zmi_blob_nb_stride(K);
  const v4i *bp0 = (const v4i *)(tiles + nb0 * nb_stride) + lane;
  const v4i *bp1 = (const v4i *)(tiles + nb1 * nb_stride) + lane;
  if (!wave_active) { bp0 = (const v4i *)tiles + lane; bp1 = bp0; }

  const int nk = (int)(K_pad / G_BK);

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
    a_src[i] = A + (int64_t)gr * lda;
  }

  // Loads never branch: a chunk that starts at or beyond K re-reads the last
  // valid chunk of the row instead (the blob's rows beyond K are zero, so the
  // values do not matter, only that the address is valid).
  auto load_a = [&](int kt, v4i (&r)[A_CHUNKS]) {
    // rows are readable up to K rounded up to 16 (the host repacks A otherwise)
    const int k_last = ((K + 15) & ~15) - 16;
    int k = kt * G_BK + a_kc * 16;
    if (k > k_last) k = k_last;
    #pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) r[i] = *(const v4i *)(a_src[i] + k);
  };
  // u8 -> s8 shift (a - 128) happens here, after the MFMAs of the stage, so that
  // nothing consumes the loaded registers while the loads are in flight
  auto store_a = [&](int buf, v4i (&r)[A_CHUNKS]) {
    #pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      int row = i * (G_THREADS / 8) + tid / 8;
      v4i v = r[i];
      v[0] ^= xor_mask; v[1] ^= xor_mask; v[2] ^= xor_mask; v[3] ^= xor_mask;
      *(v4i *)&sm.a[buf][row][a_kc * 16] = v;
    }
  };
  // One K stage: 4 k blocks x MI row tiles x 2 column blocks of MFMA.  The A
  // fragments of k block kb+1 are requested from LDS right after the two MFMAs
  // that used the fragments of kb.  The B fragments of the next stage were
  // requested from global memory, ahead of the next A tile, when this stage
  // began (two register sets, bA / bB), so one wait at the end of the stage
  // covers both and a second workgroup on the CU fills the gap.
  v4i bA[2][4], bB[2][4];
  v4i areg[A_CHUNKS];
  auto load_b = [&](int kt, v4i (&b)[2][4]) {
    #pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      b[0][kb] = bp0[(int64_t)(kt * 4 + kb) * 64];
      b[1][kb] = bp1[(int64_t)(kt * 4 + kb) * 64];
    }
  };
  auto run_stage = [&](int buf, const v4i (&b)[2][4]) {
    v4i a[MI];
    #pragma unroll
    for (int mi = 0; mi < MI; ++mi)
      a[mi] = *(const v4i *)&sm.a[buf][mi * 32 + lane % 32][(lane / 32) * 16];
    #pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      #pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        acc[mi][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[mi], b[0][kb], acc[mi][0], 0, 0, 0);
        acc[mi][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[mi], b[1][kb], acc[mi][1], 0, 0, 0);
        if (kb < 3) a[mi] = *(const v4i *)&sm.a[buf][mi * 32 + lane % 32][(kb + 1) * 32 + (lane / 32) * 16];
      }
    }
  };

  load_b(0, bA);
  load_a(0, areg);
  store_a(0, areg);
  __syncthreads();

  // Two stages per trip and no branch inside: the prefetch of the stage after
  // the last one is clamped to the last stage (a redundant but valid load), so
  // the loop body is straight-line code.
  const int last = nk - 1;
  for (int kt = 0; kt + 1 < nk; kt += 2) {
    load_b(kt + 1, bB);
    load_a(kt + 1, areg);
    run_stage(0, bA);
    store_a(1, areg);
    __syncthreads();
    const int nx = kt + 2 < last ? kt + 2 : last;
    load_b(nx, bA);
    load_a(nx, areg);
    run_stage(1, bB);
    store_a(0, areg);
    __syncthreads();
  }
  if (nk & 1) {
    run_stage(0, bA);
    __syncthreads();
  }

  // ------------------------------------------------------------------ epilogue
  // The A buffers are free now.  Each wavefront moves its accumulators, one
  // 32-row MFMA tile at a time, through its own LDS staging tile and reads them
  // back row by row with lane == column: the loop over rows is a real loop (the
  // register-indexed accumulators otherwise force 128 unrolled copies of the
  // epilogue arithmetic), and every store instruction writes 64 consecutive
  // elements of one output row.  The per-row source scales go through LDS too.
  int32_t *stage = reinterpret_cast<int32_t *>(smem_raw) + wave * G_EPI_WAVE_WORDS;
  float *row_scale = reinterpret_cast<float *>(smem_raw) + 4 * G_EPI_WAVE_WORDS;
  for (int r = tid; r < BM; r += G_THREADS) {
    const int m = m0 + r;
    row_scale[r] = m < M ? zmi_row_scale(epi, p, m) : 1.0f;
  }
  __syncthreads();
  if (!wave_active) return;

  const int cl = lane % 32, hi = lane / 32;
  const void *bias = p.bias;
  if (!gated) {
    const int n = n_out0 + lane;
    const ZmiColCtx cc = zmi_col_ctx(epi, p, colsum, n, N);
    const bool raw = zmi_epilogue_is_raw_s32(epi, bias);
    #pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      // acc[mi][ni][j] is row (j/4)*8 + hi*4 + j%4 of the tile, column ni*32 + cl
      #pragma unroll
      for (int ni = 0; ni < 2; ++ni)
        #pragma unroll
        for (int j = 0; j < 16; ++j)
          stage[((j / 4) * 8 + hi * 4 + (j % 4)) * G_EPI_LD + ni * 32 + cl] = acc[mi][ni][j];
      __builtin_amdgcn_wave_barrier();
      const int mbase = m0 + mi * 32;
      const int rows = (M - mbase) < 32 ? (M - mbase) : 32;
      const float *rsc = row_scale + mi * 32;
      if (n < N && rows > 0) {
        const bool has_rs = epi.src_scale_mode != ZMI_SS_NONE, has_ws = epi.wei_scale_mode != 0;
        const bool has_bias = bias != nullptr, bf16 = epi.dst_dt == ZMI_DT_BF16;
        // one straight-line row loop per variant; the variant is uniform for the launch
        auto run = [&](auto ek, auto is_bf16) {
          #pragma unroll 4
          for (int r = 0; r < rows; ++r) {
            const float y = zmi_fast_value<decltype(ek)::value>(stage[r * G_EPI_LD + lane], cc, rsc[r], has_rs,
                                                                has_ws, has_bias);
            zmi_fast_store<decltype(is_bf16)::value>(p.dst, (int64_t)(mbase + r) * p.ldc + n, y);
          }
        };
        using std::integral_constant;
        using T = integral_constant<bool, true>;
        using F = integral_constant<bool, false>;
        switch (epi.fast_kind * 2 + (bf16 ? 1 : 0)) {
        case ZMI_EK_NONE * 2: run(integral_constant<int, ZMI_EK_NONE>{}, F{}); break;
        case ZMI_EK_NONE * 2 + 1: run(integral_constant<int, ZMI_EK_NONE>{}, T{}); break;
        case ZMI_EK_SWISH * 2: run(integral_constant<int, ZMI_EK_SWISH>{}, F{}); break;
        case ZMI_EK_SWISH * 2 + 1: run(integral_constant<int, ZMI_EK_SWISH>{}, T{}); break;
        case ZMI_EK_GELU_TANH * 2: run(integral_constant<int, ZMI_EK_GELU_TANH>{}, F{}); break;
        case ZMI_EK_GELU_TANH * 2 + 1: run(integral_constant<int, ZMI_EK_GELU_TANH>{}, T{}); break;
        case ZMI_EK_RELU * 2: run(integral_constant<int, ZMI_EK_RELU>{}, F{}); break;
        case ZMI_EK_RELU * 2 + 1: run(integral_constant<int, ZMI_EK_RELU>{}, T{}); break;
        default:
          // generic interpreter (any post-op chain, alpha / beta, destination quantization, raw s32)
          #pragma unroll 1
          for (int r = 0; r < rows; ++r) {
            const int m = mbase + r;
            const int32_t a = stage[r * G_EPI_LD + lane];
            const int64_t o = (int64_t)m * p.ldc + n;
            if (raw) {
              ((int32_t *)p.dst)[o] = a + cc.comp;
            } else {
              const float y = zmi_epilogue_value(epi, a, cc, rsc[r], m, n, p.dst, p.ldc);
              zmi_store(p.dst, epi.dst_dt, o, y);
            }
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  } else {
    // gate tile in staging columns 0..31, up tile in 32..63; half-wave hi takes
    // the odd / even rows, lane cl the output column n_out0 + cl
    const int half = N / 2;
    const int n = n_out0 + cl;
    const ZmiColCtx cg = zmi_col_ctx(epi, p, colsum, n, half);
    const ZmiColCtx cu = zmi_col_ctx(epi, p, colsum, n < half ? n + half : N, N);
    #pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      #pragma unroll
      for (int ni = 0; ni < 2; ++ni)
        #pragma unroll
        for (int j = 0; j < 16; ++j)
          stage[((j / 4) * 8 + hi * 4 + (j % 4)) * G_EPI_LD + ni * 32 + cl] = acc[mi][ni][j];
      __builtin_amdgcn_wave_barrier();
      const int mbase = m0 + mi * 32;
      #pragma unroll 2
      for (int rr = 0; rr < 16; ++rr) {
        const int r = rr * 2 + hi;
        const int m = mbase + r;
        if (m >= M || n >= half) continue;
        const float rs = row_scale[mi * 32 + r];
        float g = zmi_epilogue_value(epi, stage[r * G_EPI_LD + cl], cg, rs, m, n, p.dst, p.ldc);
        float u = zmi_epilogue_value(epi, stage[r * G_EPI_LD + 32 + cl], cu, rs, m, n + half, p.dst, p.ldc);
        if (epi.dst_dt == ZMI_DT_BF16) {
          // the unfused path stores the GEMM result as bf16 before the activation reads it
          g = zmi_bf16_to_f32(zmi_f32_to_bf16(g));
          u = zmi_bf16_to_f32(zmi_f32_to_bf16(u));
        }
        zmi_store(p.dst, epi.dst_dt, (int64_t)m * p.ldc + n, zmi_gated(epi.gated_act, g, u));
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <int BM>
static hipError_t launch_bm(const ZmiProblem &p0, const ZmiProblem *probs, int n_prob, int n_items,
                            int m_lo, const ZmiEpilogue &epi, hipStream_t stream) {
  const size_t smem = gemm_smem_bytes<BM>();
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
#ifndef ZMI_GEMM_ONLY_BM128
  case 64: return launch_bm<64>(p, nullptr, 1, n_items, 0, epi, stream);
  case 256: return launch_bm<256>(p, nullptr, 1, n_items, 0, epi, stream);
#endif
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
#ifndef ZMI_GEMM_ONLY_BM128
  case 64: return launch_bm<64>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
  case 256: return launch_bm<256>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
#endif
  default: return launch_bm<128>(dummy, probs_dev, n_prob, n_items, m_lo, epi, stream);
  }
}
