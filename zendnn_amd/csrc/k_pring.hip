// Large-M int8 GEMM for gfx950, persistent form: one workgroup per compute unit walks a
// share of the output that is cut so that every compute unit gets the same number of
// 64-column units, whatever the tile count is.
//
// Replaces the same call sites as k_ring.hip (aocl_gemm_u8s8s32o* / aocl_gemm_s8s8s32o*,
// zendnnl/src/lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:1190-1295) for one
// problem with many rows, a bf16 destination and a straight-line epilogue.
//
// Why: 256 x 256 tiles of a 2048 x 14336 output are 448 tiles on 256 compute units, two
// rounds of which the second is three quarters full.  Here the output is a grid of
// (256-row band, 64-column unit) cells; the XCDs split the columns, the 32 compute units
// of an XCD split its cells evenly in band-major order, and a compute unit covers its run
// of cells with tiles of 256 x (64 * NI) outputs, NI = 4, 3, 2 or 1 (seven cells: one tile
// of 256 x 256 and one of 256 x 192).  The main loop is k_ring.hip's: both operands in MFMA
// fragment order, stages of 64 k moved global -> LDS by global_load_lds_dwordx4 into a ring
// of four, two k blocks per stage with the next block's fragment reads under the current
// block's MFMAs, one workgroup barrier per stage; a wavefront computes 128 x (32 * NI).
#include <cstdlib>
#include <type_traits>

#include "zmi_device.h"
#include "zmi_launch.h"

#define PR_THREADS 256
#define PR_NS 4                            // (five stages, the whole LDS, measured the same)
#define PR_STAGE 32768                     // 16 pairs of 2 KiB: 8 activation fragment rows + up to 8 weight column blocks
#define PR_RING (PR_NS * PR_STAGE)
#define PR_ROWS_OFF (4 * 32 * 132 * 4)     // 256 row scales behind the epilogue's staging (the ring is free by then)
#define PR_SMEM PR_RING

extern __shared__ __attribute__((aligned(16))) char zmi_pring_smem[];

#ifdef PR_TIMING
// measurement build only: per workgroup and tile, the constant-rate clock at five points of the tile
__device__ unsigned long long pr_times[256 * 4 * 8];
#define PR_STAMP(i) do { if (threadIdx.x == 0 && pr_tile_no < 4) pr_times[(blockIdx.x * 4 + pr_tile_no) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#define PR_STAMPC(i) do { if (threadIdx.x == 0 && pr_tile_no < 4) pr_times[(blockIdx.x * 4 + pr_tile_no) * 8 + (i)] = __builtin_amdgcn_s_memtime(); } while (0)
extern "C" __attribute__((visibility("default"))) int zmi_debug_pring_times(unsigned long long *out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(pr_times), sizeof(pr_times));
}
#else
#define PR_STAMP(i)
#define PR_STAMPC(i)
#endif

__device__ __forceinline__ void pr_dma_pair(const void *base, uint32_t voff, uint32_t lds) {
  // two consecutive 1 KiB fragments: LDS address = m0 + offset + lane * 16
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024"
               ::"s"(lds), "v"(voff), "s"(base)
               : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void pr_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void pr_barrier() { asm volatile("s_barrier" ::: "memory"); }

// (the output is written once and not read again by this launch: streaming stores, 1 % on the whole launch)
__device__ __forceinline__ void pr_store(ZMI_GLOBAL uint16_t *o, v2u v) {
  __builtin_nontemporal_store(v, (ZMI_GLOBAL v2u *)o);
}

// One strip of 32 rows x (32 * NI) columns of a wavefront: staged in LDS by the caller, read back LPR lanes per
// row, finished and stored as runs of 4 bf16.  MASK: rows beyond M and column runs beyond N are skipped.
template <int NI, int EK, bool MASK>
__device__ __forceinline__ void pr_strip(const int32_t *stage, const float *rsc, const ZmiColCtx (&cc)[3][4],
                                         int rq, int cq, uint16_t *dst0, int64_t ldc, int rows_left, const bool (&run_ok)[3]) {
  constexpr int LPR = (NI % 2 == 0) ? 16 : 8;
  constexpr int RUNS = NI * 32 / (LPR * 4);
  constexpr int RPI = 64 / LPR, ITS = 32 / RPI, LD = NI * 32 + 4;
  ZMI_GLOBAL uint16_t *o = zmi_global<uint16_t>(dst0);
  const int32_t *sp = stage + rq * LD + cq * 4;
  const float *rp = rsc + rq;
#pragma unroll 2
  for (int it = 0; it < ITS; ++it) {
    v4i a[RUNS];
#pragma unroll
    for (int r = 0; r < RUNS; ++r) a[r] = *(const v4i *)(sp + r * LPR * 4);
    const float rs = *rp;
    if (!MASK || it * RPI + rq < rows_left) {
#pragma unroll
      for (int r = 0; r < RUNS; ++r) {
        float y[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // the reference's separately rounded scale chain (absent scales are 1, an absent bias is -0)
          y[j] = __fadd_rn(__fmul_rn(__fmul_rn((float)(a[r][j] + cc[r][j].comp), rs), cc[r][j].wscale), cc[r][j].bias);
          y[j] = zmi_act_bf16<EK>(y[j]);
        }
        const v2u v = {zmi_pack_bf16(y[0], y[1]), zmi_pack_bf16(y[2], y[3])};
        if (!MASK || run_ok[r]) pr_store(o + r * LPR * 4, v);
      }
    }
    sp += RPI * LD;
    rp += RPI;
    o += RPI * ldc;
  }
}

// One tile: rows band * 256 .. + 255, columns pair0 * 64 .. + NI * 64 - 1.
template <int NI, int EK>
__device__ __forceinline__ void pr_tile(const ZmiProblem &p, const ZmiEpilogue &epi, int band, int pair0, bool first,
                                        int pr_tile_no) {
  (void)pr_tile_no;
  PR_STAMP(0);
  PR_STAMPC(5);
  constexpr int MI = 4, AF = 8, P = AF + 2 * NI, NPM = (P + 3) / 4, NS = PR_NS, STAGE = PR_STAGE;
  char *smem = zmi_pring_smem;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / 2, wn = wave % 2;

  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nk = K_pad / 64;
  const int64_t frow_bytes = (int64_t)K_pad * 32;
  const uint8_t *Afr = (const uint8_t *)p.A;
  const uint8_t *Bfr = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int a_last = (M + 31) / 32 - 1;
  const int b_last = (int)(zmi_blob_npad(N) / 32) - 1;
  const int m0 = band * 256;

  // ---- this wavefront's share of a stage: pairs wave, wave + 4, ... -------------------
  const uint8_t *gbase[NPM];
  uint32_t lds_dst[NPM];
#pragma unroll
  for (int j = 0; j < NPM; ++j) {
    int r = wave + 4 * j;
    if (r >= P) r = P - 1;                 // surplus slot of a short wavefront: never issued
    int64_t frow;
    const uint8_t *base;
    if (r < AF) {
      const int fr = m0 / 32 + r;
      frow = fr < a_last ? fr : a_last;
      base = Afr;
    } else {
      const int fc = pair0 * 2 + (r - AF);
      frow = fc < b_last ? fc : b_last;
      base = Bfr;
    }
    gbase[j] = base + frow * frow_bytes;
    lds_dst[j] = r * 2048;
  }
  const int n_my = (P - wave + 3) / 4;      // pairs this wavefront really loads
  const bool short_wave = n_my < NPM;

  uint32_t voff = lane * 16;
  const uint32_t voff_max = lane * 16 + (nk - 1) * 2048;
  auto issue_all = [&](int slot) {
#pragma unroll
    for (int j = 0; j < NPM; ++j)
      if (j < NPM - 1 || !short_wave) pr_dma_pair(gbase[j], voff, lds_dst[j] + slot * STAGE);
    voff = voff + 2048 < voff_max ? voff + 2048 : voff_max;
  };

  v16i acc[NI][MI];
#pragma unroll
  for (int ni = 0; ni < NI; ++ni)
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0;

  v4i fa[2][MI], fb[2][NI];
  const char *lbase = smem + lane * 16;

  // One phase = MI * NI MFMAs on the fragments of set `cur`, each of the first ones followed by one LDS fragment
  // read into the other set; in the second phase of a stage the global -> LDS pairs of the stage NS - 1 ahead are
  // spread over the phase.
  auto phase = [&](int cur, int rd_slot, int rd_kb, bool do_issue, int is_slot) {
    const char *pr = lbase + rd_slot * STAGE + rd_kb * 1024;
    constexpr int NM = MI * NI;
    constexpr int ISTEP = NM / NPM > 0 ? NM / NPM : 1;
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      const int ni = i / MI, mi = i % MI;
      acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[cur][ni], fa[cur][mi], acc[ni][mi], 0, 0, 0);
      if (i < NI) fb[cur ^ 1][i] = *(const v4i *)(pr + (AF + wn * NI + i) * 2048);
      else if (i < NI + MI) fa[cur ^ 1][i - NI] = *(const v4i *)(pr + (wm * MI + (i - NI)) * 2048);
      if (do_issue && i % ISTEP == 0 && i / ISTEP < NPM) {
        const int j = i / ISTEP;
        if (j < NPM - 1 || !short_wave) pr_dma_pair(gbase[j], voff, lds_dst[j] + is_slot * STAGE);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (NM < NI + MI) {
#pragma unroll
      for (int i = NM; i < NI + MI; ++i) {
        if (i < NI) fb[cur ^ 1][i] = *(const v4i *)(pr + (AF + wn * NI + i) * 2048);
        else fa[cur ^ 1][i - NI] = *(const v4i *)(pr + (wm * MI + (i - NI)) * 2048);
      }
    }
    if (do_issue && NM / ISTEP < NPM) {
#pragma unroll
      for (int j = NM / ISTEP; j < NPM; ++j)
        if (j < NPM - 1 || !short_wave) pr_dma_pair(gbase[j], voff, lds_dst[j] + is_slot * STAGE);
    }
  };

  // ---- epilogue constants, requested ahead of the first stages as raw words nothing touches before the main loop
  // is over: the row scale of row `tid` of the band and this lane's column constants
  constexpr int LPR = (NI % 2 == 0) ? 16 : 8;
  constexpr int RUNS = NI * 32 / (LPR * 4);
  constexpr int LD = NI * 32 + 4;
  float *row_scale = reinterpret_cast<float *>(smem + PR_ROWS_OFF);
  const int rs_row = m0 + tid < M ? m0 + tid : M - 1;
  const int cq = lane % LPR, rq = lane / LPR;
  const int n0w = (pair0 * 2 + wn * NI) * 32;
  int n_run[RUNS];
  ZmiColRaw craw[RUNS][4];
#pragma unroll
  for (int r = 0; r < RUNS; ++r) n_run[r] = n0w + r * LPR * 4 + cq * 4;

  // the ring (and the epilogue's staging in it) of the tile before this one is free, its stores have been counted
  if (!first) {
    pr_wait_vm<0>();
    pr_barrier();
  }
  const uint32_t rs_word = zmi_row_scale_raw(epi, p, colsum, rs_row);
  const int32_t zp_word = zmi_zp_raw(p, colsum);
#pragma unroll
  for (int r = 0; r < RUNS; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) craw[r][j] = zmi_col_raw(epi, p, colsum, n_run[r] + j < N ? n_run[r] + j : N - 1);

  // ---- prologue: NS - 1 stages in flight, the first one landed ---------------------------
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) issue_all(s);
  if (short_wave) pr_wait_vm<(NS - 2) * (NPM - 1) * 2>();
  else pr_wait_vm<(NS - 2) * NPM * 2>();
  pr_barrier();
  PR_STAMP(1);
  {
    const char *pr = lbase;
#pragma unroll
    for (int i = 0; i < NI; ++i) fb[0][i] = *(const v4i *)(pr + (AF + wn * NI + i) * 2048);
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[0][i] = *(const v4i *)(pr + (wm * MI + i) * 2048);
  }

  int slot = 0;
  for (int s = 0; s < nk; ++s) {
    const int slot_next = slot + 1 == NS ? 0 : slot + 1;
    const int slot_prev = slot == 0 ? NS - 1 : slot - 1;
    phase(0, slot, 1, false, 0);
    // stage s + 1 has landed (loads are issued every stage, clamped at the end, so the count is uniform)
    if (short_wave) pr_wait_vm<(NS - 3) * (NPM - 1) * 2>();
    else pr_wait_vm<(NS - 3) * NPM * 2>();
    pr_barrier();
    phase(1, slot_next, 0, true, slot_prev);
    voff = voff + 2048 < voff_max ? voff + 2048 : voff_max;
    slot = slot_next;
  }
  pr_wait_vm<0>();
  pr_barrier();
  PR_STAMP(2);
  PR_STAMPC(6);

  // ------------------------------------------------------------------------ epilogue
  if (tid < 256) row_scale[tid] = m0 + tid < M ? zmi_row_scale_from_raw(epi, p, rs_word, rs_row) : 1.0f;
  ZmiColCtx cc[3][4];
  bool run_ok[3] = {false, false, false};
  const bool has_bias = p.bias != nullptr;
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    run_ok[r] = n_run[r] < N;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n_run[r] + j;
      cc[r][j] = zmi_col_ctx_raw(epi, p, craw[r][j], zp_word, n, n < N ? n : N - 1, N);
      if (!has_bias) cc[r][j].bias = -0.0f;
    }
  }
  __syncthreads();
  int32_t *stage = reinterpret_cast<int32_t *>(smem) + wave * (32 * 132);
  const int hi = lane / 32, cl = lane % 32;
  const bool cols_ok = (pair0 + NI) * 64 <= N;
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    // this wavefront's 32 x (32 * NI) strip -> LDS (row = lane % 32, 4 consecutive columns per store)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4i o = {acc[ni][mi][g * 4], acc[ni][mi][g * 4 + 1], acc[ni][mi][g * 4 + 2], acc[ni][mi][g * 4 + 3]};
        *(v4i *)&stage[cl * LD + ni * 32 + g * 8 + hi * 4] = o;
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int mbase = m0 + wm * 128 + mi * 32;
    const float *rsc = row_scale + wm * 128 + mi * 32;
    uint16_t *d0 = (uint16_t *)p.dst + (int64_t)(mbase + rq) * p.ldc + n_run[0];
    if (cols_ok && mbase + 32 <= M) pr_strip<NI, EK, false>(stage, rsc, cc, rq, cq, d0, p.ldc, 32, run_ok);
    else if (mbase < M) pr_strip<NI, EK, true>(stage, rsc, cc, rq, cq, d0, p.ldc, M - mbase, run_ok);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  }
  PR_STAMP(3);
#ifdef PR_TIMING
  if (threadIdx.x == 0 && pr_tile_no < 4) pr_times[(blockIdx.x * 4 + pr_tile_no) * 8 + 4] = NI;
#endif
}

// Cells of the (band, 64-column unit) grid: XCD x owns the units [x * np / 8, (x + 1) * np / 8) of every band (one
// XCD walks the whole activation matrix and an eighth of the weights, through its own L2); its cells, band-major,
// are split evenly over its compute units, and a compute unit covers its run with tiles of up to four units that
// never cross a band.  Workgroup ids go round robin over the XCDs.
template <int EK>
__global__ __launch_bounds__(PR_THREADS, 1) void zmi_gemm_pring_kernel(ZmiProblem p, ZmiEpilogue epi) {
  const int np = (int)(zmi_blob_npad(p.N) / 64);
  const int bands = (p.M + 255) / 256;
  const int b = blockIdx.x, x = b % 8, j = b / 8, cpx = gridDim.x / 8;
  const int px0 = (int)((int64_t)x * np / 8), px1 = (int)((int64_t)(x + 1) * np / 8);
  const int wx = px1 - px0;
  const int64_t cells = (int64_t)wx * bands;
  int u = (int)(cells * j / cpx);
  const int u1 = (int)(cells * (j + 1) / cpx);
  zmi_set_f32_flush();
  bool first = true;
  int tile_no = 0;
  while (u < u1) {
    const int band = u / wx, pin = u % wx;
    const int band_end = (band + 1) * wx;
    const int n = (u1 < band_end ? u1 : band_end) - u;
    const int k = (n + 3) / 4;
    const int ni = (n + k - 1) / k;
    const int pair0 = px0 + pin;
    switch (ni) {
    case 4: pr_tile<4, EK>(p, epi, band, pair0, first, tile_no); break;
    case 3: pr_tile<3, EK>(p, epi, band, pair0, first, tile_no); break;
    case 2: pr_tile<2, EK>(p, epi, band, pair0, first, tile_no); break;
    default: pr_tile<1, EK>(p, epi, band, pair0, first, tile_no); break;
    }
    first = false;
    ++tile_no;
    u += ni;
  }
}

// One problem with a bf16 destination, a straight-line epilogue, 16-byte aligned rows and N a multiple of 4.
bool zmi_pring_takes(const ZmiProblem &p, const ZmiEpilogue &epi) {
  if (epi.gated_act != 0 || epi.dst_dt != ZMI_DT_BF16 || epi.fast_kind == ZMI_EK_GENERIC || epi.n_groups > 0) return false;
  if (p.row_comp) return false;
  if (((uintptr_t)p.dst) % 16 != 0 || (p.ldc * 2) % 16 != 0 || p.N % 4 != 0) return false;
  return p.M > 0 && p.N >= 64;
}

template <int EK>
static hipError_t pring_launch(const ZmiProblem &p, const ZmiEpilogue &epi, int grid, hipStream_t stream) {
  hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_pring_kernel<EK>, PR_SMEM);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((zmi_gemm_pring_kernel<EK>), dim3(grid), dim3(PR_THREADS), PR_SMEM, stream, p, epi);
  return hipGetLastError();
}

// p.A in fragment-major order (zmi_afrag_off).  One workgroup per compute unit.
hipError_t zmi_launch_gemm_pring(const ZmiProblem &p, const ZmiEpilogue &epi, hipStream_t stream) {
  if (!zmi_pring_takes(p, epi)) return hipErrorInvalidValue;
  int grid = zmi_cu_count() / 8 * 8;
  // (ZMI_PRING_GRID: fewer workgroups, so that small test shapes give every workgroup several tiles)
  if (const char *env = zmi_env(ZE_PRING_GRID)) {
    const int g = std::atoi(env) / 8 * 8;
    if (g >= 8 && g < grid) grid = g;
  }
  if (grid < 8) return hipErrorInvalidValue;
  switch (epi.fast_kind) {
  case ZMI_EK_SWISH: return pring_launch<ZMI_EK_SWISH>(p, epi, grid, stream);
  case ZMI_EK_GELU_TANH: return pring_launch<ZMI_EK_GELU_TANH>(p, epi, grid, stream);
  case ZMI_EK_RELU: return pring_launch<ZMI_EK_RELU>(p, epi, grid, stream);
  default: return pring_launch<ZMI_EK_NONE>(p, epi, grid, stream);
  }
}
