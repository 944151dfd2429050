// Large-M int8 GEMM for gfx950 (MFMA-bound), single and grouped:
//   C = epilogue(A[M,K] x blob), s32 accumulation on v_mfma_i32_32x32x32_i8.
//
// Replaces the reference's aocl_gemm_u8s8s32o* / aocl_gemm_s8s8s32o*[_sym_quant]
// call sites (zendnnl/src/lowoha_operators/matmul/backends/aocl/
// aocl_kernel.cpp:1190-1295) and, in grouped form, the per-expert GEMMs of
// group_matmul_run_parallel_dispatch (matmul/group_matmul/
// group_matmul_dispatch.cpp:1096).
//
// Both operands arrive in MFMA fragment order (1 KiB fragments of 32 rows x 32 k,
// see zmi_device.h): the weights from the prepack, the activations from the
// quantization / repack pass that precedes the GEMM.  A workgroup of 4 wavefronts
// (2 x 2) owns a BM x 256 tile (gated: BM x 128 outputs from 2 x 128 weight
// columns) and walks K in stages of 64:
//   * every stage is BM/32 + 8 contiguous 2 KiB fragment pairs; each wavefront
//     moves its share with global_load_lds_dwordx4 (global memory -> LDS without
//     passing through registers) into a ring of NS stages, NS-1 stages ahead;
//   * a wavefront computes (BM/2) x 128: per 32-wide k block it reads BM/64 + 4
//     fragments from LDS (linear 16 bytes per lane, conflict free) for
//     (BM/64) x 4 MFMAs; the reads of the next k block are interleaved with the
//     MFMAs of the current one, two register sets;
//   * one workgroup barrier per stage, placed between the two k blocks, where it
//     orders "stage s+1 has landed" and "stage s-1 is free" at once.
// The MFMA takes the weight fragment as its first operand, so a lane's 16
// accumulators of a 32 x 32 block are 4 runs of 4 consecutive output columns of
// one output row.  The epilogue moves each 32 x 128 strip through LDS and reads
// it back with 16 lanes per row, so the arithmetic runs in a rolled loop with
// the per-column constants of a lane fixed in registers, and a row is stored as
// 128-byte (bf16) or 256-byte (f32) runs.
#include <type_traits>

#include "zmi_device.h"
#include "zmi_launch.h"
#include "zmi_ring_table.h"

#ifndef ZMI_RING_EPI_UNROLL
#define ZMI_RING_EPI_UNROLL 2
#endif
#define R_THREADS 256
#define R_BN 256
#define R_EPI_LD 132                       // words per staged row (128 + 4: rows 4 banks apart)
#define R_EPI_WAVE_WORDS (32 * R_EPI_LD)

extern __shared__ __attribute__((aligned(16))) char zmi_ring_smem[];

__device__ __forceinline__ void zmi_dma_pair(const void *base, uint32_t voff, uint32_t lds) {
  // two consecutive 1 KiB fragments: LDS address = m0 + offset + lane * 16
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024"
               ::"s"(lds), "v"(voff), "s"(base)
               : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void zmi_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void zmi_wg_barrier() { asm volatile("s_barrier" ::: "memory"); }

// DEEP: the launch has at most one workgroup per CU, so the ring takes the whole LDS
// (more stages in flight) instead of leaving room for a second workgroup.
template <int BM, bool DEEP = false>
struct RingCfg {
  static constexpr int AF = BM / 32;                 // activation fragment rows per tile
  static constexpr int P = AF + 8;                   // 2 KiB pairs per stage
  static constexpr int STAGE = P * 2048;
  static constexpr int NS = BM == 256 ? 4 : (DEEP ? (BM == 128 ? 6 : 7) : 3);
  static constexpr int OCC = (BM == 256 || DEEP) ? 1 : 2;
  static constexpr int NPAIR_MAX = (P + 3) / 4;
  static constexpr int RING = STAGE * NS;
  static constexpr int EPI = 4 * R_EPI_WAVE_WORDS * 4;     // epilogue staging, reuses the ring
  static constexpr int ROWS_OFF = RING > EPI ? RING : EPI;  // BM row scales, live during the main loop
  static constexpr int SMEM = ROWS_OFF + BM * 4;
};

// Interior strips with a bf16 destination: every row and column of the strip is
// valid and 8-byte stores are aligned, so the loop body is straight-line code.
// GATED pairs run 0 (gate) with run 1 (up) through silu(g) * u.
template <int EK, bool GATED>
__device__ __forceinline__ void zmi_ring_strip_bf16(const int32_t *stage, const float *rsc, const ZmiColCtx (&cc)[2][4],
                                                    int r4, int c16, uint16_t *dst0, int64_t ldc, int run1_off) {
  // dst0: element (first row of the strip + r4, first column of run 0)
  ZMI_GLOBAL uint16_t *o = zmi_global<uint16_t>(dst0);
  const int32_t *sp = stage + r4 * R_EPI_LD + c16 * 4;
  const float *rp = rsc + r4;
#pragma unroll ZMI_RING_EPI_UNROLL
  for (int it = 0; it < 8; ++it) {
    const v4i a0 = *(const v4i *)sp;
    const v4i a1 = *(const v4i *)(sp + 64);
    const float rs = *rp;
    float y0[4], y1[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      y0[j] = __fadd_rn(__fmul_rn(__fmul_rn((float)(a0[j] + cc[0][j].comp), rs), cc[0][j].wscale), cc[0][j].bias);
      y1[j] = __fadd_rn(__fmul_rn(__fmul_rn((float)(a1[j] + cc[1][j].comp), rs), cc[1][j].wscale), cc[1][j].bias);
    }
    if (!GATED) {
#pragma unroll
      for (int j = 0; j < 4; ++j) { y0[j] = zmi_act_bf16<EK>(y0[j]); y1[j] = zmi_act_bf16<EK>(y1[j]); }
      const v2u v0 = {zmi_pack_bf16(y0[0], y0[1]), zmi_pack_bf16(y0[2], y0[3])};
      const v2u v1 = {zmi_pack_bf16(y1[0], y1[1]), zmi_pack_bf16(y1[2], y1[3])};
      *(ZMI_GLOBAL v2u *)o = v0;
      *(ZMI_GLOBAL v2u *)(o + run1_off) = v1;
    } else {
      float z[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // gate and up are rounded to bf16 first, as when the activation reads a stored GEMM result
        const uint32_t gu = zmi_pack_bf16(y0[j], y1[j]);
        const float g = __uint_as_float(gu << 16), u = __uint_as_float(gu & 0xffff0000u);
        z[j] = zmi_act_bf16<ZMI_EK_SWISH>(g) * u;
      }
      const v2u v = {zmi_pack_bf16(z[0], z[1]), zmi_pack_bf16(z[2], z[3])};
      *(ZMI_GLOBAL v2u *)o = v;
    }
    sp += 4 * R_EPI_LD;
    rp += 4;
    o += 4 * ldc;
  }
}

template <int BM, bool DEEP>
__global__ __launch_bounds__(R_THREADS, (RingCfg<BM, DEEP>::OCC)) void zmi_gemm_ring_kernel(ZmiProblem p0,
                                                                                   const ZmiProblem *probs,
                                                                                   int n_prob, int n_items,
                                                                                   const int *tile_tab, int bm_idx, int top_flags,
                                                                                   ZmiRingSplit split, ZmiEpilogue epi) {
  using Cfg = RingCfg<BM, DEEP>;
  constexpr int MI = BM / 64, NI = 4;
  constexpr int AF = Cfg::AF, STAGE = Cfg::STAGE, NS = Cfg::NS, NPM = Cfg::NPAIR_MAX;
  char *smem = zmi_ring_smem;

  const int top = top_flags & 0xffff;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / 2, wn = wave % 2;
  const bool gated = epi.gated_act != 0;

  // ---- which tile -------------------------------------------------------------------
  // Workgroup ids go round robin over the 8 XCDs; renumber so that every XCD gets
  // a contiguous range of tiles, and order tiles so that neighbours share weight
  // columns (and, for one problem, a band of activation rows).
  // Grouped launches read the tile table made by zmi_ring_count_kernel: the real tile count
  // (the grid is only a bound when the row counts live on the device) and, per problem,
  // the index of its first tile.
  if (tile_tab) n_items = tile_tab[bm_idx] * split.slices;
  const int b = blockIdx.x;
  const int per_xcd = (n_items + 7) / 8;
  const int item = (b % 8) * per_xcd + b / 8;
  if (b / 8 >= per_xcd || item >= n_items) return;
  // K slices of one tile are neighbours (same XCD: their partial sums meet in one L2)
  const int n_slice = split.slices;
  const int id = item / n_slice, slice = item % n_slice;
  ZmiProblem p;
  int tm, tn, m0;
  {
    const int per = gated ? 128 : 256;
    if (!probs) {
      p = p0;
      int full; bool rem;
      zmi_ring_rows<BM>(p.M, top_flags, full, rem);
      const int tiles_m = full + (rem ? 1 : 0);
      const int ncols = gated ? p.N / 2 : p.N;
      const int tiles_n = (ncols + per - 1) / per;
      const int GM = tiles_m < 8 ? tiles_m : 8;
      const int per_group = GM * tiles_n;
      const int group = id / per_group;
      const int first_m = group * GM;
      const int gm = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
      const int r = id % per_group;
      tm = first_m + r % gm;
      tn = r / gm;
      m0 = tm < full ? tm * top : (p.M / top) * top;
    } else {
      // the problem that owns tile `id`: the last one whose first tile is <= id (64 candidates per step)
      const int *starts = tile_tab + 4 + bm_idx * n_prob;
      int e = -1;
      for (int e0 = 0; e0 < n_prob; e0 += 64) {
        const int ee = e0 + lane;
        const int st = ee < n_prob ? starts[ee] : 0x7fffffff;
        const int c = __popcll(__ballot(st <= id));
        if (c > 0) e = e0 + c - 1;
        if (c < 64) break;
      }
      e = __builtin_amdgcn_readfirstlane(e);
      bool found = e >= 0;
      tm = tn = m0 = 0;
      if (found) {
        const int M = probs[e].M;
        int full; bool rem;
        zmi_ring_rows<BM>(M, top_flags, full, rem);
        const int tiles_m = full + (rem ? 1 : 0);
        const int r = id - starts[e];
        found = tiles_m > 0;
        if (found) {
          tm = r % tiles_m;
          tn = r / tiles_m;
          m0 = tm < full ? tm * top : (M / top) * top;
        }
      }
      if (!found) return;
      p = probs[e];
    }
  }

  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nk_all = K_pad / 64;
  const int k_first = (int)((int64_t)slice * nk_all / n_slice);           // this slice's stages of 64 k
  const int nk = (int)((int64_t)(slice + 1) * nk_all / n_slice) - k_first;
  const int64_t frow_bytes = (int64_t)K_pad * 32;
  const uint8_t *Afr = (const uint8_t *)p.A;
  const uint8_t *Bfr = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int a_last = (M + 31) / 32 - 1;
  const int b_last = (int)(zmi_blob_npad(N) / 32) - 1;
  const int half = N / 2;

  // ---- this wavefront's share of a stage: pairs wave, wave+4, ... ---------------------
  const uint8_t *gbase[NPM];
  uint32_t lds_dst[NPM];
#pragma unroll
  for (int j = 0; j < NPM; ++j) {
    int r = wave + 4 * j;
    if (r >= Cfg::P) r = Cfg::P - 1;       // surplus slot of a short wavefront: never issued
    int64_t frow;
    const uint8_t *base;
    if (r < AF) {
      int fr = m0 / 32 + r;
      frow = fr < a_last ? fr : a_last;
      base = Afr;
    } else {
      const int q = r - AF;
      int fc;
      if (!gated) {
        fc = tn * 8 + q;
      } else {
        // LDS order per wavefront column half: [gate 2w, gate 2w+1, up 2w, up 2w+1]
        const int w = q / 4, qq = q % 4;
        fc = tn * 4 + w * 2 + (qq & 1);
        const int lim = half / 32 - 1;
        if (fc > lim) fc = lim;
        if (qq >= 2) fc += half / 32;
      }
      frow = fc < b_last ? fc : b_last;
      base = Bfr;
    }
    gbase[j] = base + frow * frow_bytes;
    lds_dst[j] = r * 2048;
  }
  const int n_my = (Cfg::P - wave + 3) / 4;      // pairs this wavefront really loads
  const bool short_wave = n_my < NPM;

  uint32_t voff = lane * 16 + k_first * 2048;
  const uint32_t voff_max = lane * 16 + (k_first + nk - 1) * 2048;
  auto issue_all = [&](int slot) {
#pragma unroll
    for (int j = 0; j < NPM; ++j)
      if (j < NPM - 1 || !short_wave) zmi_dma_pair(gbase[j], voff, lds_dst[j] + slot * STAGE);
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

  // One phase = MI*NI MFMAs on the fragments of set `cur`; the first MI+NI of them
  // are each followed by one LDS fragment read into the other set.  In the second
  // phase of a stage the global->LDS pairs of the stage NS-1 ahead are spread over
  // the phase so that no wavefront sits in a queue of loads while its MFMAs wait.
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
        if (j < NPM - 1 || !short_wave) zmi_dma_pair(gbase[j], voff, lds_dst[j] + is_slot * STAGE);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (NM < NI + MI) {
      // fewer MFMAs than fragments (BM == 64): the remaining reads follow
#pragma unroll
      for (int i = NM; i < NI + MI; ++i) {
        if (i < NI) fb[cur ^ 1][i] = *(const v4i *)(pr + (AF + wn * NI + i) * 2048);
        else fa[cur ^ 1][i - NI] = *(const v4i *)(pr + (wm * MI + (i - NI)) * 2048);
      }
    }
    if (do_issue && NM / ISTEP < NPM) {
#pragma unroll
      for (int j = NM / ISTEP; j < NPM; ++j)
        if (j < NPM - 1 || !short_wave) zmi_dma_pair(gbase[j], voff, lds_dst[j] + is_slot * STAGE);
    }
  };

  // ---- epilogue constants: requested here, ahead of the first stages (so that the counted
  // waits of the main loop cover them), as raw words that nothing touches before the main
  // loop is over (a wait here would hold the loop back by a memory round trip per dependent
  // load): the row scale of row `tid` of the tile and this lane's eight column constants
  float *row_scale = reinterpret_cast<float *>(smem + Cfg::ROWS_OFF);
  const int rs_row = m0 + tid < M ? m0 + tid : M - 1;
  const uint32_t rs_word = zmi_row_scale_raw(epi, p, colsum, rs_row);
  const int32_t zp_word = zmi_zp_raw(p, colsum);
  const int hi = lane / 32, cl = lane % 32;
  const int c16 = lane % 16, r4 = lane / 16;
  const void *bias = p.bias;
  const bool has_rs = epi.src_scale_mode != ZMI_SS_NONE, has_ws = epi.wei_scale_mode != 0;
  const bool has_bias = bias != nullptr;
  const int dst_dt = epi.dst_dt;

  // output columns of this lane: two runs of 4
  int n_run[2];
  ZmiColRaw craw[2][4];
  auto col_ok = [&](int n) { return n < N ? n : N - 1; };
  if (!gated) {
    n_run[0] = tn * 256 + wn * 128 + c16 * 4;
    n_run[1] = n_run[0] + 64;
  } else {
    // run 0: gate columns n, run 1: the matching up columns n + N/2; output column n
    n_run[0] = tn * 128 + wn * 64 + c16 * 4;
    n_run[1] = n_run[0] + half;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int j = 0; j < 4; ++j) craw[h][j] = zmi_col_raw(epi, p, colsum, col_ok(n_run[h] + j));
  const int n_lim = gated ? half : N;
  // vector stores need every row start aligned
  const int es = dst_dt == ZMI_DT_BF16 ? 2 : (dst_dt == ZMI_DT_S8 || dst_dt == ZMI_DT_U8 ? 1 : 4);
  const bool vec_ok = (((uintptr_t)p.dst) % 16 == 0) && ((p.ldc * es) % 16 == 0);
  const bool raw = zmi_epilogue_is_raw_s32(epi, bias);

  // ---- prologue: NS-1 stages in flight, the first one landed --------------------------
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) issue_all(s);
  if (short_wave) zmi_wait_vm<(NS - 2) * (NPM - 1) * 2>();
  else zmi_wait_vm<(NS - 2) * NPM * 2>();
  zmi_wg_barrier();
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
    // stage s+1 has landed (loads are issued every stage, clamped at the end, so the count is uniform)
    if (short_wave) zmi_wait_vm<(NS - 3) * (NPM - 1) * 2>();
    else zmi_wait_vm<(NS - 3) * NPM * 2>();
    zmi_wg_barrier();
    phase(1, slot_next, 0, true, slot_prev);
    voff = voff + 2048 < voff_max ? voff + 2048 : voff_max;
    slot = slot_next;
  }
  zmi_wait_vm<0>();
  zmi_wg_barrier();

  // ---- K slices: every slice leaves its int32 partial tile in the workspace, in register
  // order (16 bytes per lane and store: whole cache lines), and is done;
  // zmi_ring_reduce_kernel adds the slices of a tile and runs the epilogue on all CUs.
  // With arrival words the slices write their tiles through to device scope (word stores that bypass the caches,
  // 256 contiguous bytes per instruction), wait for the acknowledgements and count themselves in at the tile's word;
  // the slice that arrives last reads the others' tiles with loads of the same scope into its own accumulators and
  // goes on to the epilogue.  No fence (a release fence at device scope writes back the whole L2) and no second
  // launch: M = 128, K = 4096, N = 14336 in four slices 38.2 -> 36.4 us per call (the last slice's loads are one
  // compute unit's: 384 KiB at its own rate).
  if (BM != 256 && n_slice > 1 && split.arrivals) {
    constexpr int CH = NI * MI * 4;
    auto words = [&](int s) { return (unsigned int *)split.partial + (((int64_t)id * n_slice + s) * 4 + wave) * (CH * 256) + lane; };
    unsigned int *mine = words(slice);
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          __hip_atomic_store(mine + ((ni * MI + mi) * 16 + e) * 64, (unsigned int)acc[ni][mi][e], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    zmi_wait_vm<0>();
    zmi_wg_barrier();
    int *flag = reinterpret_cast<int *>(smem);   // (the ring is free)
    if (tid == 0) {
      const unsigned int before = __hip_atomic_fetch_add(split.arrivals + id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = before == (unsigned int)(n_slice - 1);
      if (last) __hip_atomic_store(split.arrivals + id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *flag = last ? 1 : 0;
    }
    zmi_wg_barrier();
    const bool last = *flag != 0;
    zmi_wg_barrier();   // (everybody has read the word before the epilogue reuses the ring)
    if (!last) return;
    for (int s = 0; s < n_slice; ++s) {
      if (s == slice) continue;
      const unsigned int *theirs = words(s);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            acc[ni][mi][e] += (int32_t)__hip_atomic_load(theirs + ((ni * MI + mi) * 16 + e) * 64, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT);
    }
  } else if (BM != 256 && n_slice > 1) {   // (256-row tiles are chosen only when they cover the CUs)
    constexpr int CH = NI * MI * 4;   // 16-byte chunks per lane
    int32_t *mine = split.partial + (((int64_t)id * n_slice + slice) * 4 + wave) * (CH * 256) + lane * 4;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4i o = {acc[ni][mi][g * 4], acc[ni][mi][g * 4 + 1], acc[ni][mi][g * 4 + 2], acc[ni][mi][g * 4 + 3]};
          *zmi_global<v4i>(mine + ((ni * MI + mi) * 4 + g) * 256) = o;
        }
    return;
  }

  // ------------------------------------------------------------------------ epilogue
  // decode the constants requested in the prologue
  if (tid < BM) row_scale[tid] = m0 + tid < M ? zmi_row_scale_from_raw(epi, p, rs_word, rs_row) : 1.0f;
  ZmiColCtx cc[2][4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (!gated) {
      cc[0][j] = zmi_col_ctx_raw(epi, p, craw[0][j], zp_word, n_run[0] + j, col_ok(n_run[0] + j), N);
      cc[1][j] = zmi_col_ctx_raw(epi, p, craw[1][j], zp_word, n_run[1] + j, col_ok(n_run[1] + j), N);
    } else {
      cc[0][j] = zmi_col_ctx_raw(epi, p, craw[0][j], zp_word, n_run[0] + j, col_ok(n_run[0] + j), half);
      cc[1][j] = zmi_col_ctx_raw(epi, p, craw[1][j], zp_word, n_run[0] + j < half ? n_run[1] + j : N,
                                 col_ok(n_run[1] + j), N);
    }
  }
  __syncthreads();
  int32_t *stage = reinterpret_cast<int32_t *>(smem) + wave * R_EPI_WAVE_WORDS;
  // the bf16 fast forms multiply / add unconditionally: absent scales are 1, an absent bias is -0
  if (dst_dt == ZMI_DT_BF16 && epi.fast_kind != ZMI_EK_GENERIC) {
    zmi_set_f32_flush();
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (!has_bias) cc[h][j].bias = -0.0f;
  }
  // The strips are visited by a static loop (the accumulators are registers: a
  // dynamic index would make the compiler select among all of them); the
  // arithmetic inside a strip is a rolled loop.
  auto do_strip = [&](auto mic) {
    constexpr int mi = decltype(mic)::value;
    // this wavefront's 32 x 128 strip -> LDS (row = lane % 32, 4 consecutive columns per store)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        v4i o = {acc[ni][mi][g * 4], acc[ni][mi][g * 4 + 1], acc[ni][mi][g * 4 + 2], acc[ni][mi][g * 4 + 3]};
        *(v4i *)&stage[cl * R_EPI_LD + ni * 32 + g * 8 + hi * 4] = o;
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();

    const int mbase = m0 + wm * (BM / 2) + mi * 32;
    const float *rsc = row_scale + wm * (BM / 2) + mi * 32;

    auto run = [&](auto ek, auto dtc) {
      constexpr int EK = decltype(ek)::value;
      constexpr int DT = decltype(dtc)::value;    // 0: f32, 1: bf16
#pragma unroll 2
      for (int it = 0; it < 8; ++it) {
        const int r = it * 4 + r4;
        const int m = mbase + r;
        const v4i a0 = *(const v4i *)&stage[r * R_EPI_LD + c16 * 4];
        const v4i a1 = *(const v4i *)&stage[r * R_EPI_LD + 64 + c16 * 4];
        const float rs = rsc[r];
        if (m >= M) continue;
        float y0[4], y1[4];
        if (DT == 1) {
          // bf16 store: the reference's separately rounded scale chain (absent scales are 1, absent bias -0)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            y0[j] = __fadd_rn(__fmul_rn(__fmul_rn((float)(a0[j] + cc[0][j].comp), rs), cc[0][j].wscale), cc[0][j].bias);
            y1[j] = __fadd_rn(__fmul_rn(__fmul_rn((float)(a1[j] + cc[1][j].comp), rs), cc[1][j].wscale), cc[1][j].bias);
            if (!gated) { y0[j] = zmi_act_bf16<EK>(y0[j]); y1[j] = zmi_act_bf16<EK>(y1[j]); }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            y0[j] = zmi_fast_value<EK>(a0[j], cc[0][j], rs, has_rs, has_ws, has_bias);
            y1[j] = zmi_fast_value<EK>(a1[j], cc[1][j], rs, has_rs, has_ws, has_bias);
          }
        }
        if (!gated) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const float *y = h ? y1 : y0;
            const int n = n_run[h];
            if (n >= N) continue;
            const int64_t o = (int64_t)m * p.ldc + n;
            if (vec_ok && n + 3 < N) {
              if (DT == 1) {
                const v2u v = {zmi_pack_bf16(y[0], y[1]), zmi_pack_bf16(y[2], y[3])};
                *zmi_global<v2u>((uint16_t *)p.dst + o) = v;
              } else {
                *zmi_global<v4f>((float *)p.dst + o) = (v4f){y[0], y[1], y[2], y[3]};
              }
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (n + j < N) {
                  if (DT == 1) zmi_global<uint16_t>(p.dst)[o + j] = (uint16_t)zmi_pack_bf16(y[j], 0.0f);
                  else zmi_global<float>(p.dst)[o + j] = y[j];
                }
            }
          }
        } else {
          const int n = n_run[0];
          if (n >= half) continue;
          float z[4];
          if (DT == 1) {
            // the unfused path stores the GEMM result as bf16 before the activation reads it
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const uint32_t gu = zmi_pack_bf16(y0[j], y1[j]);
              const float g = __uint_as_float(gu << 16), u = __uint_as_float(gu & 0xffff0000u);
              z[j] = epi.gated_act == ZMI_ACT_SILU_AND_MUL ? zmi_act_bf16<ZMI_EK_SWISH>(g) * u
                                                           : zmi_gated(epi.gated_act, g, u);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) z[j] = zmi_gated(epi.gated_act, y0[j], y1[j]);
          }
          const int64_t o = (int64_t)m * p.ldc + n;
          if (vec_ok && n + 3 < half) {
            if (DT == 1) {
              const v2u v = {zmi_pack_bf16(z[0], z[1]), zmi_pack_bf16(z[2], z[3])};
              *zmi_global<v2u>((uint16_t *)p.dst + o) = v;
            } else {
              *zmi_global<v4f>((float *)p.dst + o) = (v4f){z[0], z[1], z[2], z[3]};
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (n + j < half) {
                if (DT == 1) zmi_global<uint16_t>(p.dst)[o + j] = (uint16_t)zmi_pack_bf16(z[j], 0.0f);
                else zmi_global<float>(p.dst)[o + j] = z[j];
              }
          }
        }
      }
    };
    using std::integral_constant;
    const bool bf16 = dst_dt == ZMI_DT_BF16;
    // interior strip: all 32 rows and all columns of the tile valid, aligned rows
    const bool interior = bf16 && vec_ok && epi.fast_kind != ZMI_EK_GENERIC && mbase + 32 <= M &&
                          (gated ? (tn + 1) * 128 <= half && epi.gated_act == ZMI_ACT_SILU_AND_MUL && epi.fast_kind == ZMI_EK_NONE
                                 : (tn + 1) * 256 <= N);
    if (interior) {
      uint16_t *d0 = (uint16_t *)p.dst + (int64_t)(mbase + r4) * p.ldc + n_run[0];
      if (gated) zmi_ring_strip_bf16<ZMI_EK_NONE, true>(stage, rsc, cc, r4, c16, d0, p.ldc, 0);
      else switch (epi.fast_kind) {
        case ZMI_EK_SWISH: zmi_ring_strip_bf16<ZMI_EK_SWISH, false>(stage, rsc, cc, r4, c16, d0, p.ldc, 64); break;
        case ZMI_EK_GELU_TANH: zmi_ring_strip_bf16<ZMI_EK_GELU_TANH, false>(stage, rsc, cc, r4, c16, d0, p.ldc, 64); break;
        case ZMI_EK_RELU: zmi_ring_strip_bf16<ZMI_EK_RELU, false>(stage, rsc, cc, r4, c16, d0, p.ldc, 64); break;
        default: zmi_ring_strip_bf16<ZMI_EK_NONE, false>(stage, rsc, cc, r4, c16, d0, p.ldc, 64); break;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      return;
    }
    const bool fast_ok = epi.fast_kind != ZMI_EK_GENERIC && (bf16 || dst_dt == ZMI_DT_F32);
    // the gated form applies no element-wise post-op of its own before the activation
    const int kind = fast_ok ? (gated && epi.fast_kind != ZMI_EK_NONE ? -1 : epi.fast_kind * 2 + (bf16 ? 1 : 0)) : -1;
    switch (kind) {
    case ZMI_EK_NONE * 2: run(integral_constant<int, ZMI_EK_NONE>{}, integral_constant<int, 0>{}); break;
    case ZMI_EK_NONE * 2 + 1: run(integral_constant<int, ZMI_EK_NONE>{}, integral_constant<int, 1>{}); break;
    case ZMI_EK_SWISH * 2: run(integral_constant<int, ZMI_EK_SWISH>{}, integral_constant<int, 0>{}); break;
    case ZMI_EK_SWISH * 2 + 1: run(integral_constant<int, ZMI_EK_SWISH>{}, integral_constant<int, 1>{}); break;
    case ZMI_EK_GELU_TANH * 2: run(integral_constant<int, ZMI_EK_GELU_TANH>{}, integral_constant<int, 0>{}); break;
    case ZMI_EK_GELU_TANH * 2 + 1: run(integral_constant<int, ZMI_EK_GELU_TANH>{}, integral_constant<int, 1>{}); break;
    case ZMI_EK_RELU * 2: run(integral_constant<int, ZMI_EK_RELU>{}, integral_constant<int, 0>{}); break;
    case ZMI_EK_RELU * 2 + 1: run(integral_constant<int, ZMI_EK_RELU>{}, integral_constant<int, 1>{}); break;
    default:
      // generic interpreter: any post-op chain, alpha / beta, destination quantization, raw s32
#pragma unroll 1
      for (int it = 0; it < 8; ++it) {
        const int r = it * 4 + r4;
        const int m = mbase + r;
        if (m >= M) continue;
        const float rs = rsc[r];
#pragma unroll 1
        for (int j = 0; j < 4; ++j) {
          const int32_t a0 = stage[r * R_EPI_LD + c16 * 4 + j];
          const int32_t a1 = stage[r * R_EPI_LD + 64 + c16 * 4 + j];
          if (!gated) {
#pragma unroll 1
            for (int h = 0; h < 2; ++h) {
              const int n = n_run[h] + j;
              if (n >= N) continue;
              const int64_t o = (int64_t)m * p.ldc + n;
              const ZmiColCtx c = zmi_col_ctx(epi, p, colsum, n, N);
              const int32_t a = h ? a1 : a0;
              if (raw) ((int32_t *)p.dst)[o] = a + c.comp;
              else zmi_store(p.dst, dst_dt, o, zmi_epilogue_value(epi, a, c, rs, m, n, p.dst, p.ldc));
            }
          } else {
            const int n = n_run[0] + j;
            if (n >= half) continue;
            const ZmiColCtx cg = zmi_col_ctx(epi, p, colsum, n, half);
            const ZmiColCtx cu = zmi_col_ctx(epi, p, colsum, n + half, N);
            float g = zmi_epilogue_value(epi, a0, cg, rs, m, n, p.dst, p.ldc);
            float u = zmi_epilogue_value(epi, a1, cu, rs, m, n + half, p.dst, p.ldc);
            if (dst_dt == ZMI_DT_BF16) {
              g = zmi_bf16_to_f32(zmi_f32_to_bf16(g));
              u = zmi_bf16_to_f32(zmi_f32_to_bf16(u));
            }
            zmi_store(p.dst, dst_dt, (int64_t)m * p.ldc + n, zmi_gated(epi.gated_act, g, u));
          }
        }
      }
    }
    (void)n_lim;
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  };
  do_strip(std::integral_constant<int, 0>{});
  if constexpr (MI > 1) do_strip(std::integral_constant<int, 1>{});
  if constexpr (MI > 2) {
    do_strip(std::integral_constant<int, 2>{});
    do_strip(std::integral_constant<int, 3>{});
  }
}

// Second step of a K-sliced launch: adds the partial tiles of the slices and finishes the
// elements (plain epilogues only: gated launches are never sliced).  One wavefront per
// 16-byte chunk column of a tile: lane l of chunk (wave w, ni, mi, g) holds row
// (w/2)*(BM/2) + mi*32 + l%32 and the four columns from (w%2)*128 + ni*32 + g*8 + (l/32)*4
// of the tile, as the MFMA left them.
template <int BM>
__global__ __launch_bounds__(R_THREADS) void zmi_ring_reduce_kernel(ZmiProblem p, int top_flags, ZmiRingSplit split,
                                                                    ZmiEpilogue epi) {
  constexpr int MI = BM / 64, NI = 4, CH = NI * MI * 4;
  const int top = top_flags & 0xffff;
  const int lane = threadIdx.x % 64;
  constexpr int units_per_tile = 4 * CH;                  // wavefront units: (w, ni, mi, g)
  const int unit = blockIdx.x * (R_THREADS / 64) + threadIdx.x / 64;
  const int tile = unit / units_per_tile;
  int full; bool rem;
  zmi_ring_rows<BM>(p.M, top_flags, full, rem);
  const int tiles_m = full + (rem ? 1 : 0);
  const int tiles_n = (p.N + 255) / 256;
  if (tile >= tiles_m * tiles_n) return;
  // same tile numbering as the GEMM kernel
  const int GM = tiles_m < 8 ? tiles_m : 8;
  const int per_group = GM * tiles_n;
  const int first_m = (tile / per_group) * GM;
  const int gm = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
  const int r = tile % per_group;
  const int tm = first_m + r % gm, tn = r / gm;
  const int m0 = tm < full ? tm * top : (p.M / top) * top;

  int u = unit % units_per_tile;
  const int g = u % 4; u /= 4;
  const int mi = u % MI; u /= MI;
  const int ni = u % NI; u /= NI;
  const int w = u, wm = w / 2, wn = w % 2;

  const int m = m0 + wm * (BM / 2) + mi * 32 + lane % 32;
  const int n0 = tn * 256 + wn * 128 + ni * 32 + g * 8 + (lane / 32) * 4;
  v4i sum = {0, 0, 0, 0};
  for (int s = 0; s < split.slices; ++s) {
    const int32_t *base = split.partial + (((int64_t)tile * split.slices + s) * 4 + w) * (CH * 256) + lane * 4;
    const v4i a = *zmi_global<const v4i>(base + ((ni * MI + mi) * 4 + g) * 256);
#pragma unroll
    for (int j = 0; j < 4; ++j) sum[j] += a[j];
  }
  if (m >= p.M) return;
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const float rs = zmi_row_scale(epi, p, m);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + j;
    if (n >= p.N) break;
    zmi_finish_element(p, epi, zmi_col_ctx(epi, p, colsum, n, p.N), rs, sum[j], m, n);
  }
}

__global__ __launch_bounds__(64) void zmi_ring_count_kernel(const ZmiProblem *probs, int n_prob, int top, int gated,
                                                             int *tab) {
  zmi_ring_fill_table(probs, n_prob, top, gated, tab, threadIdx.x);
}

hipError_t zmi_launch_ring_table(const ZmiProblem *probs_dev, int n_prob, int top, bool gated, int *tab_dev, hipStream_t stream) {
  hipLaunchKernelGGL(zmi_ring_count_kernel, dim3(1), dim3(64), 0, stream, probs_dev, n_prob, top, gated ? 1 : 0, tab_dev);
  return hipGetLastError();
}

int zmi_cu_count() {
  static const int n_cu = [] {
    int dev = 0, n = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    return n;
  }();
  return n_cu;
}

template <int BM, bool DEEP>
static hipError_t ring_launch_cfg(const ZmiProblem &p0, const ZmiProblem *probs, int n_prob, int n_items,
                                  const int *tile_tab, int top, const ZmiRingSplit &split, const ZmiEpilogue &epi,
                                  hipStream_t stream) {
  const size_t smem = RingCfg<BM, DEEP>::SMEM;
  {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_ring_kernel<BM, DEEP>, (int)smem);
    if (e != hipSuccess) return e;
  }
  const int grid = (n_items + 7) / 8 * 8;   // a multiple of 8 so the XCD renumbering applies
  hipLaunchKernelGGL((zmi_gemm_ring_kernel<BM, DEEP>), dim3(grid), dim3(R_THREADS), smem, stream, p0, probs, n_prob,
                     n_items, tile_tab, BM == 256 ? 0 : (BM == 128 ? 1 : 2), top, split, epi);
  return hipGetLastError();
}

template <int BM>
static hipError_t ring_launch(const ZmiProblem &p0, const ZmiProblem *probs, int n_prob, int n_items, bool exact,
                              const int *tile_tab, int top, const ZmiRingSplit &split, const ZmiEpilogue &epi,
                              hipStream_t stream, bool shares_cus = false) {
  if (n_items <= 0) return hipSuccess;
  n_items *= split.slices;
  // at most one workgroup per CU anyway: let it have the whole LDS for its ring -- unless the launch runs beside
  // another one and has only the CUs that one leaves free (two workgroups on each of them then)
  const int n_cu = zmi_cu_count();
  (void)exact;   // a bound that fits one workgroup per CU is as good as the exact count
  if (BM != 256 && n_items <= n_cu && !shares_cus)
    return ring_launch_cfg<BM, (BM != 256)>(p0, probs, n_prob, n_items, tile_tab, top, split, epi, stream);
  return ring_launch_cfg<BM, false>(p0, probs, n_prob, n_items, tile_tab, top, split, epi, stream);
}

// Largest tile height for a problem set: 256-row tiles once they fill the chip,
// 128-row tiles for smaller problems (more tiles, two workgroups per CU).
// Tile height of a single problem.  128-row tiles run two workgroups per CU (one's epilogue under the other's main
// loop) and, while all of them fit the CUs' slots at once, take ragged row counts as one launch with a partly filled
// last tile; 256-row tiles halve the operand traffic per multiply-add and win once their count fills the CUs.
// Measured on MI355X, K = 4096, N = 14336, whole call in us, 128- / 256-row tiles: M = 769 68 / 77, 900 72 / 70,
// 1024 74 / 70, 1025 78 / 83, 1100 80 / 94, 1536 113 / 119, 2048 134 / 127, 4096 - / 242.
int zmi_ring_pick_top(int64_t rows, int64_t out_cols) {
  const int64_t tn = (out_cols + 255) / 256;
  const int64_t t256 = ((rows + 255) / 256) * tn, t128 = ((rows + 127) / 128) * tn;
  const int n_cu = zmi_cu_count();
  if (t128 <= 2 * n_cu) {
    // one round either way: 256-row tiles only when they are whole and cover most CUs
    const bool whole256 = rows % 256 == 0 && t256 <= n_cu && t256 * 100 >= 85 * n_cu;
    return whole256 ? 256 : 128;
  }
  return t256 >= 192 ? 256 : 128;
}

// Grouped launches (n_prob problems, rows / n_prob rows each on average): every
// problem is covered by one launch whose tile height fits the typical problem
// (ZMI_RING_PAD), so its weights are streamed once and the launch count stays at
// one.  Measured on MI355X on 8 x ~128-row and 64 x 0..3900-row expert sets, the
// 128-row tile (two workgroups per CU, one's epilogue under the other's main
// loop) beats both the 256-row tile and full tiles plus right-sized remainders.
int zmi_ring_pick_top_group(int64_t rows, int n_prob, int64_t K, int64_t N, bool gated) {
  (void)K; (void)N; (void)gated;
  if (n_prob <= 0 || rows <= 0) return 128 | ZMI_RING_PAD;
  const int64_t avg = (rows + n_prob - 1) / n_prob;
  return (avg <= 64 ? 64 : 128) | ZMI_RING_PAD;
}

// One problem: tile height and K slices.  A problem whose tiles cover only a fraction of
// the CUs is bound by the latency of its few weight streams: each tile is then split over
// K, at the price of a second launch that re-reads the int32 partial tiles.  Measured on
// MI355X (K = 4096, N = 4096 / 14336, M = 32 .. 1024): four slices pay off up to a quarter
// of the CUs' worth of tiles (16 .. 64 tiles: 42 -> 34 us, 50 -> 45 us per call); two or
// eight slices, or slicing 112 and more tiles, lose to the unsliced launch.
ZmiRingPlan zmi_ring_plan(int M, int N, int K, int top_hint, int force_slices) {
  ZmiRingPlan plan;
  plan.top = top_hint ? top_hint : zmi_ring_pick_top(M, N);
  plan.slices = 1;
  plan.partial_bytes = 0;
  const int64_t tiles_n = (N + 255) / 256;
  plan.tiles = (int)(((M + (plan.top & 0xffff) - 1) / (plan.top & 0xffff)) * tiles_n);
  if (M <= 0) return plan;
  const int n_cu = zmi_cu_count();
  if ((plan.top & 0xffff) == 64 && force_slices <= 0) return plan;
  // More than 64 rows whose 64-row tiles fit the CUs at once.  A workgroup's weight stream runs at what one compute
  // unit keeps in flight (the LDS ring: about 60 GB/s at the loaded latency), so such a call lasts as long as ONE
  // workgroup's stream whatever the tile height: lower tiles put more CUs to work, and K slices shorten the stream
  // while slices x tiles still fit the CUs (one workgroup each: a second round costs more than it saves) and a slice
  // keeps 24 stages of 64 k; the slice that arrives last adds the partial tiles (64 KiB each at this height).
  // Measured, us per call, this / 128-row tiles (in four slices when few): K = 4096, N = 14336: 96 rows 29.4 / 36.7,
  // 256 rows 33.5 / 38.7; K = 8192, N = 8192: 128 rows 32.6 / 37.1, 256 rows 39.1 / 43.7; K = 14336, N = 4096:
  // 128 rows 38.2 / 47.1; K = 4096, N = 4096: 256 rows 25.7 / 32.1; K = 2048, N = 11008: 128 rows 21.0 / 28.2.
  if (!top_hint && force_slices <= 0 && M > 64) {
    const int64_t t64 = ((M + 63) / 64) * tiles_n;
    const int nk64 = (int)(zmi_blob_kpad(K) / 64);
    if (t64 <= n_cu) {
      int sl = 1;
      if (t64 * 4 <= n_cu && nk64 / 4 >= 24) sl = 4;
      else if (t64 * 2 <= n_cu && nk64 / 2 >= 24) sl = 2;
      if (sl > 1 || (t64 >= 48 && zmi_blob_kpad(K) <= 6144)) {
        plan.top = 64 | ZMI_RING_PAD;
        plan.tiles = (int)t64;
        plan.slices = sl;
        plan.partial_bytes = sl > 1 ? (size_t)t64 * sl * 64 * 256 * sizeof(int32_t) : 0;
        return plan;
      }
    }
  }
  const int nk = (int)(zmi_blob_kpad(K) / 64);
  const int top = M <= 64 || (top_hint & 0xffff) == 64 ? 64 : 128;
  const int64_t tiles = ((M + top - 1) / top) * tiles_n;
  int slices = 1;
  if (force_slices > 0) slices = force_slices;
  else if (tiles * 4 <= n_cu && nk >= 16) slices = 4;
  if (slices > nk) slices = nk;
  if (slices < 2) {
    // A remainder of rows would be a launch of its own behind the full tiles' launch, each with too few tiles to
    // fill the CUs (M = 129 .. 255, N = 14336: 38 us for 128 rows + 25 us for the rest).  While the padded count
    // still fits the CUs' workgroup slots at once, the remainder is a partly filled 128-row tile of the one launch.
    if ((plan.top & 0xffff) == 128 && M > 128 && M % 128 != 0) {
      const int64_t padded = ((M + 127) / 128) * tiles_n;
      if (padded <= 2 * n_cu) {
        plan.top = 128 | ZMI_RING_PAD;
        plan.tiles = (int)padded;
      }
    }
    return plan;
  }
  plan.top = top | ZMI_RING_PAD;
  plan.slices = slices;
  plan.tiles = (int)tiles;
  plan.partial_bytes = (size_t)tiles * slices * top * 256 * sizeof(int32_t);
  return plan;
}

// One problem, M rows in fragment-major order at p.A.
hipError_t zmi_launch_gemm_ring(const ZmiProblem &p, const ZmiEpilogue &epi, int top, const ZmiRingSplit *split,
                                hipStream_t stream, const ZmiRingSide *side) {
  if (p.M <= 0) return hipSuccess;
  const bool gated = epi.gated_act != 0;
  ZmiRingSplit sp = {1, nullptr, nullptr};
  if (split && split->slices > 1) {
    // sliced launches are one launch: the remainder rows stay with the top-height kernel
    if (!(top & ZMI_RING_PAD) || (top & 0xffff) == 256 || !split->partial || gated) return hipErrorInvalidValue;
    if (split->slices > (int)(zmi_blob_kpad(p.K) / 64)) return hipErrorInvalidValue;
    sp = *split;
  }
  hipError_t e = hipSuccess;
  // the remainder rows of a 256-row launch: on the side stream when there is one (the two launches write disjoint rows)
  hipStream_t rem_stream = stream;
  bool forked = false;
  if ((top & 0xffff) == 256) {
    const int rem_items = zmi_ring_items<128>(p.M, p.N, top, gated) + zmi_ring_items<64>(p.M, p.N, top, gated);
    if (side && side->stream && rem_items > 0 && zmi_ring_items<256>(p.M, p.N, top, gated) > 0 && sp.slices == 1) {
      e = hipEventRecord(side->fork, stream);
      if (e == hipSuccess) e = hipStreamWaitEvent(side->stream, side->fork, 0);
      if (e != hipSuccess) return e;
      rem_stream = side->stream;
      forked = true;
    }
    e = ring_launch<256>(p, nullptr, 1, zmi_ring_items<256>(p.M, p.N, top, gated), true, nullptr, top, sp, epi, stream);
    if (e != hipSuccess && !forked) return e;
  }
  if (e == hipSuccess)
    e = ring_launch<128>(p, nullptr, 1, zmi_ring_items<128>(p.M, p.N, top, gated), true, nullptr, top, sp, epi, rem_stream, forked);
  // (once forked, the join below runs whatever the launches returned: the caller's stream must stay ordered behind
  // the side stream, and a capture must not be left with an unjoined fork)
  if (e == hipSuccess)
    e = ring_launch<64>(p, nullptr, 1, zmi_ring_items<64>(p.M, p.N, top, gated), true, nullptr, top, sp, epi, rem_stream, forked);
  if (forked) {
    hipError_t j = hipEventRecord(side->join, side->stream);
    if (j == hipSuccess) j = hipStreamWaitEvent(stream, side->join, 0);
    if (e == hipSuccess) e = j;
  }
  if (e != hipSuccess || sp.slices == 1 || sp.arrivals) return e;
  // the slices' partial tiles -> finished elements
  const int th = top & 0xffff;
  const int tiles = th == 128 ? zmi_ring_items<128>(p.M, p.N, top, gated) : zmi_ring_items<64>(p.M, p.N, top, gated);
  const int units = tiles * 4 * 4 * (th / 64) * 4;
  const int grid = (units + R_THREADS / 64 - 1) / (R_THREADS / 64);
  if (th == 128) hipLaunchKernelGGL(zmi_ring_reduce_kernel<128>, dim3(grid), dim3(R_THREADS), 0, stream, p, top, sp, epi);
  else hipLaunchKernelGGL(zmi_ring_reduce_kernel<64>, dim3(grid), dim3(R_THREADS), 0, stream, p, top, sp, epi);
  return hipGetLastError();
}

// Every problem of the table.  probs_host mirrors probs_dev and sizes the grids; when it is
// null (row counts known only on the device) worst_rows / worst_cols bound them and surplus
// workgroups exit at once.  tab_dev is 4 + 3 * n_prob ints of scratch for the tile table
// (tab_ready: already filled for this table, tile height and epilogue kind by an earlier kernel).
// split (optional): K slices with arrival words (plain epilogues, padded 128- or 64-row tiles); its workspace holds
// zmi_ring_group_items(...) * slices partial tiles.
int zmi_ring_group_items(const ZmiProblem *probs_host, int n_prob, int top, int64_t worst_rows, int worst_cols, bool gated) {
  const int th = top & 0xffff;
  if (probs_host) {
    int items = 0;
    for (int e = 0; e < n_prob; ++e) {
      const ZmiProblem &q = probs_host[e];
      if (q.M <= 0) continue;
      items += th == 256 ? zmi_ring_items<256>(q.M, q.N, top, gated) : th == 128 ? zmi_ring_items<128>(q.M, q.N, top, gated)
                                                                                  : zmi_ring_items<64>(q.M, q.N, top, gated);
    }
    return items;
  }
  const int per = gated ? 128 : 256;
  const int ncols = gated ? worst_cols / 2 : worst_cols;
  return (int)(worst_rows / th + n_prob) * ((ncols + per - 1) / per);
}

hipError_t zmi_launch_gemm_ring_group(const ZmiProblem *probs_host, const ZmiProblem *probs_dev, int n_prob,
                                      int top, int64_t worst_rows, int worst_cols, int *tab_dev, bool tab_ready,
                                      const ZmiEpilogue &epi, hipStream_t stream, const ZmiRingSplit *split) {
  const bool gated = epi.gated_act != 0;
  if (!tab_dev) return hipErrorInvalidValue;
  int items[3] = {0, 0, 0};   // 256, 128, 64
  if (probs_host) {
    for (int e = 0; e < n_prob; ++e) {
      const ZmiProblem &q = probs_host[e];
      if (q.M <= 0) continue;
      items[0] += (top & 0xffff) == 256 ? zmi_ring_items<256>(q.M, q.N, top, gated) : 0;
      items[1] += zmi_ring_items<128>(q.M, q.N, top, gated);
      items[2] += zmi_ring_items<64>(q.M, q.N, top, gated);
    }
  } else {
    const int per = gated ? 128 : 256;
    const int ncols = gated ? worst_cols / 2 : worst_cols;
    const int tiles_n = (ncols + per - 1) / per;
    // at most rows/top full blocks in total and one remainder block per problem
    const int th = top & 0xffff;
    items[th == 256 ? 0 : (th == 128 ? 1 : 2)] = (int)(worst_rows / th + n_prob) * tiles_n;
    if (!(top & ZMI_RING_PAD)) {
      if (th == 256) items[1] = n_prob * tiles_n;
      if (th >= 128) items[2] = n_prob * tiles_n;
    }
  }
  if (items[0] + items[1] + items[2] <= 0) return hipSuccess;
  if (!tab_ready)
    hipLaunchKernelGGL(zmi_ring_count_kernel, dim3(1), dim3(64), 0, stream, probs_dev, n_prob, top, gated ? 1 : 0, tab_dev);
  const bool exact = probs_host != nullptr;
  ZmiProblem dummy = {};
  ZmiRingSplit whole = {1, nullptr, nullptr};
  if (split && split->slices > 1) {
    // (one launch of padded tiles, the slice that arrives last finishes the elements: no reduction launch here)
    if (gated || !(top & ZMI_RING_PAD) || (top & 0xffff) == 256 || !split->partial || !split->arrivals) return hipErrorInvalidValue;
    whole = *split;
  }
  hipError_t e = hipSuccess;
  if ((top & 0xffff) == 256) {
    e = ring_launch<256>(dummy, probs_dev, n_prob, items[0], exact, tab_dev, top, whole, epi, stream);
    if (e != hipSuccess) return e;
  }
  e = ring_launch<128>(dummy, probs_dev, n_prob, items[1], exact, tab_dev, top, whole, epi, stream);
  if (e != hipSuccess) return e;
  return ring_launch<64>(dummy, probs_dev, n_prob, items[2], exact, tab_dev, top, whole, epi, stream);
}
