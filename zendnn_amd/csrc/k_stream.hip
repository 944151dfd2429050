// Grouped int8 GEMM for experts whose GEMM is a stream of their weights (a few dozen to 256 rows each):
// the weight-traffic-bound counterpart of the MFMA-bound kernel (k_ring.hip), same tiles, same results.
//
// Reference counterpart: the per-expert GEMMs of group_matmul_run_parallel_dispatch
// (zendnnl/src/lowoha_operators/matmul/group_matmul/group_matmul_dispatch.cpp:1096) and the fused gate / up
// epilogue (group_matmul/custom_kernel/ukernel/int8_microkernel.cpp:196-606).
//
// With about 128 rows per expert every weight byte is used for 128 multiply-adds: the MFMA units need a third of
// the time the weights need to arrive, so the kernel is built around the weight stream.
//   * a workgroup of 4 wavefronts owns the tile of the MFMA-bound kernel (32 * MI rows x 256 weight columns;
//     gated: 128 outputs from 128 gate and 128 up columns), tiles numbered and ordered as there;
//   * the WEIGHTS never touch LDS: wavefront w streams its own two 32-column fragments (gated: a gate fragment and
//     the matching up fragment) from global memory straight into MFMA operand registers, D stages of 64 k ahead,
//     non-temporal (every byte is used once);
//   * the ROWS (shared by the 4 wavefronts, L2 resident: every tile of an expert reads the same rows) go through an
//     LDS ring of D + 1 stages filled by global -> LDS loads, each wavefront moving its share; row fragments
//     beyond the expert's last row cost no MFMA and no LDS read;
//   * a stage's loads are waited for by count (per-wavefront loads return in order), D - 2 stages stay in flight;
//     the wait and the one barrier per stage sit between the stage's two 32-k phases, and the LDS reads of one
//     phase run under the MFMAs of the other;
//   * gate and up accumulators of an output element sit in the same lane, so the gated activation and the scale
//     chain run on registers and the tile is stored from there (8-byte bf16 stores); the column constants and row
//     scales were parked in LDS, decoded, behind the first stages;
//   * an element is finished with the arithmetic of the MFMA-bound kernel's epilogue, so which of the two kernels
//     takes an expert does not change a bit of its result.
// K slices (128-row build, plain epilogues): a launch that would leave workgroup slots empty (few tiles, long K: a down
// projection) gives every tile to 2 .. 4 workgroups, each over its share of K; they leave int32 partial tiles in a
// workspace and zmi_stream_reduce_kernel adds them (integers: exact in any order) and finishes the elements with the
// same arithmetic.  The 256-row build has no registers to spare for it (it spilled 128 of them when it was tried, and
// two workgroups on the halves of one tile's K stream were measured slower than the MFMA-bound kernel on the same launch).
// Two builds: 128-row tiles with two workgroups per compute unit (one's start-up and epilogue run under the other's
// stream; 230 registers), and 256-row tiles with one (an expert of 129 .. 256 rows stays one row block, so its
// weights pass once).  Measured on MI355X, 8 experts of K = 4096 -> 28672 gated and 14336 -> 4096, whole fused
// block in ms, MFMA-bound kernel / this one: 11 .. 20 rows 0.358 / 0.333, 52 .. 78 rows 0.397 / 0.351,
// 88 .. 122 rows 0.391 / 0.376 (128-row tiles); 109 .. 150 rows 0.444 / 0.421, 173 .. 218 rows 0.554 / 0.479
// (256-row tiles); with the down projection in K slices: 11 .. 20 rows 0.371 / 0.298, 52 .. 78 rows 0.398 / 0.343.  In its main loop the kernel moves 5.8 TB/s of weights; what is left on the table is the
// start-up and the epilogue of every tile (17 of 63 us on a 256-row tile), which a single workgroup per compute
// unit cannot hide.
#include <type_traits>

#include "zmi_device.h"
#include "zmi_launch.h"
#include "zmi_ring_table.h"

#define S_THREADS 256

extern __shared__ __attribute__((aligned(16))) char zmi_stream_smem[];

namespace {

__device__ __forceinline__ void zmi_s_dma_pair(const void *base, uint32_t voff, uint32_t lds) {
  // two consecutive 1 KiB fragments: LDS address = m0 + offset + lane * 16
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024"
               ::"s"(lds), "v"(voff), "s"(base)
               : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void zmi_s_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// a pointer every lane holds the same value of, made visibly so (it goes to an instruction's scalar operand)
__device__ __forceinline__ const uint8_t *zmi_s_uniform(const uint8_t *p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

template <int I, int N, class F>
__device__ __forceinline__ void zmi_s_static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    zmi_s_static_for<I + 1, N>(f);
  }
}

}  // namespace

template <int MI, int D, bool GATED, int OCC, bool SPLIT>
__global__ __launch_bounds__(S_THREADS, OCC) void zmi_gemm_stream_kernel(const ZmiProblem *probs, int n_prob, int n_items,
                                                                       const int *tile_tab, int bm_idx, int top_flags,
                                                                       ZmiRingSplit split, ZmiEpilogue epi) {
  constexpr int BM = 32 * MI;
  constexpr int NPA = MI / 4;                  // row-fragment pairs a wavefront moves per stage
  constexpr int OPS = 2 * NPA + 4;             // memory operations of a wavefront per stage
  constexpr int SLOT = MI * 2048;              // bytes of a stage of rows
  constexpr int NSLOT = D + 1;
  constexpr int CST = 256 * 16 + BM * 4;       // decoded column constants of the tile's 256 weight columns, row scales
  static_assert(MI % 4 == 0 && D >= 3 && (D - 1) * OPS <= 63, "the in-flight count must fit the wait counter");
  char *smem = zmi_stream_smem + CST;          // the row ring (the constants sit in front of it)
  ZmiColCtx *cst = reinterpret_cast<ZmiColCtx *>(zmi_stream_smem);
  float *rsc = reinterpret_cast<float *>(zmi_stream_smem + 256 * 16);
  const int top = top_flags & 0xffff;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);

  // ---- which tile (the numbering of the MFMA-bound kernel's grouped launches) ----
  // (K slices of one tile are neighbours: the same XCD, their partial sums meet in one L2)
  const int n_slice = SPLIT ? split.slices : 1;   // (the 256-row build has no registers to spare for the sliced form)
  n_items = tile_tab[bm_idx] * n_slice;
  const int b = blockIdx.x;
  const int per_xcd = (n_items + 7) / 8;
  const int item = (b % 8) * per_xcd + b / 8;
  if (b / 8 >= per_xcd || item >= n_items) return;
  const int id = item / n_slice, slice = item % n_slice;
  ZmiProblem p;
  int tn, m0;
  {
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
    if (e < 0) return;
    const int Me = probs[e].M;
    int full; bool rem;
    zmi_ring_rows<BM>(Me, top_flags, full, rem);
    const int tiles_m = full + (rem ? 1 : 0);
    if (tiles_m <= 0) return;
    const int r = id - starts[e];
    const int tm = r % tiles_m;
    tn = r / tiles_m;
    m0 = tm < full ? tm * top : (Me / top) * top;
    p = probs[e];
  }
  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nk_all = K_pad / 64;
  const int k_first = (int)((int64_t)slice * nk_all / n_slice);            // this slice's stages of 64 k
  const int nk = (int)((int64_t)(slice + 1) * nk_all / n_slice) - k_first;
  const int64_t frow_bytes = (int64_t)K_pad * 32;
  const uint8_t *Afr = (const uint8_t *)p.A;
  const uint8_t *Bfr = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int a_last = (M + 31) / 32 - 1;
  const int b_last = (int)(zmi_blob_npad(N) / 32) - 1;
  const int half = N / 2;

  // ---- this wavefront's weight fragments (column blocks of 32) and its share of the rows ----
  int fc[2];
  if (!GATED) {
    fc[0] = tn * 8 + wave * 2;
    fc[1] = fc[0] + 1;
  } else {
    const int lim = half / 32 - 1;
    fc[0] = tn * 4 + wave;
    if (fc[0] > lim) fc[0] = lim;
    fc[1] = fc[0] + half / 32;
  }
  const uint8_t *bsrc[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) bsrc[ni] = zmi_s_uniform(Bfr + (int64_t)(fc[ni] < b_last ? fc[ni] : b_last) * frow_bytes);
  const uint8_t *abase[NPA];
  uint32_t a_lds[NPA];
#pragma unroll
  for (int j = 0; j < NPA; ++j) {
    const int r = wave + 4 * j;
    const int fr = m0 / 32 + r;
    abase[j] = zmi_s_uniform(Afr + (int64_t)(fr < a_last ? fr : a_last) * frow_bytes);
    a_lds[j] = CST + r * 2048;
  }
  const uint32_t lane16 = lane * 16;

  v4i bw[D][2][2];   // [stage in flight][fragment][32-k block]
  v16i acc[2][MI];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0;

  auto issue_rows = [&](int stage, int slot) {
    const int st_abs = k_first + stage < nk_all ? k_first + stage : nk_all - 1;   // (a slice without stages reads valid memory)
    const uint32_t voff = lane16 + (uint32_t)(st_abs > 0 ? st_abs : 0) * 2048u;
#pragma unroll
    for (int j = 0; j < NPA; ++j) zmi_s_dma_pair(abase[j], voff, a_lds[j] + slot * SLOT);
  };
  // The weight loads are issued by hand like the row loads, so that the one counted wait per stage below is the
  // only wait there is (the compiler cannot count the global -> LDS loads and would wait for more than it must);
  // their registers are not touched until that wait has covered them.
  auto issue_weights = [&](int u, int stage) {
    const int st_abs = k_first + stage < nk_all ? k_first + stage : nk_all - 1;   // (a slice without stages reads valid memory)
    const uint32_t voff = lane16 + (uint32_t)(st_abs > 0 ? st_abs : 0) * 2048u;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(bw[u][ni][0]) : "v"(voff), "s"(bsrc[ni]) : "memory");
      asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024 nt" : "=v"(bw[u][ni][1]) : "v"(voff), "s"(bsrc[ni]) : "memory");
    }
  };

  // ---- prologue: D stages in flight (stages past the end re-read the last one: uniform counts) ----
#pragma unroll
  for (int s = 0; s < D; ++s) {
    const int st = s < nk ? s : (nk > 0 ? nk - 1 : 0);
    issue_rows(st, s);
    issue_weights(s, st);
  }
  // The epilogue's constants, fetched behind the first stages and parked in LDS, decoded: thread t has weight column
  // t of the tile (gated: 0 .. 127 gate columns, 128 .. 255 the matching up columns) and row t of the tile.
  {
    int n, lim;
    if (GATED) {
      const int o = tn * 128 + tid % 128;
      n = tid < 128 ? o : (o < half ? o + half : N);
      lim = tid < 128 ? half : N;
    } else {
      n = tn * 256 + tid;
      lim = N;
    }
    if (n_slice == 1) {
      cst[tid] = zmi_col_ctx(epi, p, colsum, n, lim);
      if (tid < BM) rsc[tid] = m0 + tid < M ? zmi_row_scale(epi, p, m0 + tid) : 1.0f;
    }
  }
  // row fragments of this tile that hold rows at all (the others are skipped: their MFMAs and LDS reads)
  const int n_mi = __builtin_amdgcn_readfirstlane((M - m0 + 31) / 32 < MI ? (M - m0 + 31) / 32 : MI);
  v4i fa[2][MI];
  zmi_s_wait_vm<(D - 1) * OPS>();
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) fa[0][mi] = *(const v4i *)(smem + lane16 + mi * 2048);

  // One stage = two phases of 2 * MI MFMAs, one per 32-k block; every row fragment's two MFMAs are paired with the
  // LDS read of the fragment the other phase will use (second block of this stage / first block of the next), so
  // the reads run under the MFMAs.  The wait and the barrier sit between the phases: "stage s + 1 has landed" and
  // "stage s - 1 is read by no one any more" at once.
  int slot = 0;
  for (int s0 = 0; s0 < nk; s0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int s = s0 + u;
      if (s < nk) {   // (uniform)
        const int slot_next = slot + 1 == NSLOT ? 0 : slot + 1;
        const int slot_prev = slot == 0 ? NSLOT - 1 : slot - 1;
        const char *pr1 = smem + slot * SLOT + lane16 + 1024;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
          if (mi == 0 || mi < n_mi) {
            fa[1][mi] = *(const v4i *)(pr1 + mi * 2048);
            acc[0][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[u][0][0], fa[0][mi], acc[0][mi], 0, 0, 0);
            acc[1][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[u][1][0], fa[0][mi], acc[1][mi], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        zmi_s_wait_vm<(D - 2) * OPS>();
        asm volatile("s_barrier" ::: "memory");
        const int ahead = s + D < nk ? s + D : nk - 1;
        issue_rows(ahead, slot_prev);
        const char *pr0 = smem + slot_next * SLOT + lane16;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
          if (mi == 0 || mi < n_mi) {
            fa[0][mi] = *(const v4i *)(pr0 + mi * 2048);
            acc[0][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[u][0][1], fa[1][mi], acc[0][mi], 0, 0, 0);
            acc[1][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[u][1][1], fa[1][mi], acc[1][mi], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        issue_weights(u, ahead);
        slot = slot_next;
      }
    }
  }
  zmi_s_wait_vm<0>();
  // The loads of the stages past the end are never consumed.  Their registers must nevertheless stay the loads'
  // until the wait above: naming them here keeps the compiler from handing them to something else while a load
  // that it knows nothing about is still on its way to them.
#pragma unroll
  for (int u = 0; u < D; ++u)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) asm volatile("" ::"v"(bw[u][ni][kb]));

  // ---- K slices: every slice leaves its int32 partial tile in the workspace, in register order (16 bytes per lane
  // and store: whole cache lines), and is done; zmi_stream_reduce_kernel adds the slices and finishes the elements.
  if (SPLIT && n_slice > 1) {
    constexpr int CH = 2 * MI * 4;   // 16-byte chunks per lane
    int32_t *mine = split.partial + (((int64_t)id * n_slice + slice) * 4 + wave) * (int64_t)(CH * 256) + lane * 4;
    zmi_s_static_for<0, MI>([&](auto mic) {
      constexpr int mi = decltype(mic)::value;
      if (mi >= n_mi) return;   // (row fragments without rows are never read back)
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4i o = {acc[ni][mi][g * 4], acc[ni][mi][g * 4 + 1], acc[ni][mi][g * 4 + 2], acc[ni][mi][g * 4 + 3]};
          *zmi_global<v4i>(mine + ((ni * MI + mi) * 4 + g) * 256) = o;
        }
    });
    return;
  }

  // ---- epilogue.  Lane l holds row l % 32 of every 32-row fragment and, per 32-column fragment, four runs of four
  // consecutive columns starting at g * 8 + (l / 32) * 4. ----
  const int row = lane % 32, hi = lane / 32;
  // first output column of this lane's run g of fragment ni
  auto col_of = [&](int ni, int g) { return GATED ? tn * 128 + wave * 32 + g * 8 + hi * 4 : tn * 256 + wave * 64 + ni * 32 + g * 8 + hi * 4; };
  const bool has_bias = p.bias != nullptr;
  const bool vec_ok = (((uintptr_t)p.dst) % 8 == 0) && ((p.ldc * 2) % 8 == 0);
  const bool whole_tile = GATED ? (tn + 1) * 128 <= half : (tn + 1) * 256 <= N;
  const bool fast_bf16 = epi.dst_dt == ZMI_DT_BF16 && vec_ok && whole_tile &&
                         (GATED ? epi.gated_act == ZMI_ACT_SILU_AND_MUL : epi.fast_kind != ZMI_EK_GENERIC);
  if (fast_bf16) {
    // Straight-line bf16 forms on a tile without an edge, from registers, 8-byte stores (the arithmetic of the
    // MFMA-bound kernel's interior strips); column constants and row scales come from LDS.
    zmi_set_f32_flush();
    float rs[MI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) rs[mi] = rsc[mi * 32 + row];
    // (unrolled by construction: the accumulators are registers, a run-time index would move them to memory)
    zmi_s_static_for<0, (GATED ? 1 : 2)>([&](auto nic) {
      zmi_s_static_for<0, 4>([&](auto gc) {
        constexpr int ni = decltype(nic)::value, g = decltype(gc)::value;
        const int n0 = col_of(ni, g);
        const int t0 = GATED ? wave * 32 + g * 8 + hi * 4 : wave * 64 + ni * 32 + g * 8 + hi * 4;   // column within the tile
        ZmiColCtx c0[4], c1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          c0[j] = cst[t0 + j];
          if (GATED) c1[j] = cst[128 + t0 + j];
        }
        zmi_s_static_for<0, MI>([&](auto mic) {
          constexpr int mi = decltype(mic)::value;
          const int m = m0 + mi * 32 + row;
          if (m >= M) return;
          float z[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (GATED) {
              const float y0 = zmi_ring_chain(acc[0][mi][g * 4 + j], c0[j], rs[mi], has_bias);
              const float y1 = zmi_ring_chain(acc[1][mi][g * 4 + j], c1[j], rs[mi], has_bias);
              // gate and up are rounded to bf16 first, as when the activation reads a stored GEMM result
              const uint32_t gu = zmi_pack_bf16(y0, y1);
              z[j] = zmi_act_bf16<ZMI_EK_SWISH>(__uint_as_float(gu << 16)) * __uint_as_float(gu & 0xffff0000u);
            } else {
              const float y = zmi_ring_chain(acc[ni][mi][g * 4 + j], c0[j], rs[mi], has_bias);
              switch (epi.fast_kind) {
              case ZMI_EK_SWISH: z[j] = zmi_act_bf16<ZMI_EK_SWISH>(y); break;
              case ZMI_EK_GELU_TANH: z[j] = zmi_act_bf16<ZMI_EK_GELU_TANH>(y); break;
              case ZMI_EK_RELU: z[j] = zmi_act_bf16<ZMI_EK_RELU>(y); break;
              default: z[j] = y; break;
              }
            }
          }
          const v2u v = {zmi_pack_bf16(z[0], z[1]), zmi_pack_bf16(z[2], z[3])};
          *zmi_global<v2u>((uint16_t *)p.dst + (int64_t)m * p.ldc + n0) = v;
        });
      });
    });
    return;
  }

  // Every other epilogue (f32 and quantized destinations, post-op chains, tiles on the column edge): rolled loops
  // over elements.  The accumulators of one row fragment at a time go to LDS, every lane to words of its own, so
  // that the loop can index them (LDS here is the lane's indexable memory; nothing crosses lanes).
  __syncthreads();   // the row ring is read by no one any more
  int32_t *mine = reinterpret_cast<int32_t *>(smem) + wave * (32 * 64) + lane;
  zmi_s_static_for<0, MI>([&](auto mic) {
    constexpr int mi = decltype(mic)::value;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 16; ++q) mine[(ni * 16 + q) * 64] = acc[ni][mi][q];
    const int m = m0 + mi * 32 + row;
    if (m < M) {
      const float rs = rsc[mi * 32 + row];
#pragma unroll 1
      for (int x = 0; x < (GATED ? 16 : 32); ++x) {
        const int ni = x / 16, q = x % 16;
        const int c = (q / 4) * 8 + hi * 4 + q % 4;   // column within the 32-column fragment
        if (GATED) {
          const int n = tn * 128 + wave * 32 + c;
          if (n < half)
            zmi_finish_gated_ring(p, epi, cst[wave * 32 + c], cst[128 + wave * 32 + c], rs, mine[q * 64], mine[(16 + q) * 64], m, n);
        } else {
          const int n = tn * 256 + wave * 64 + ni * 32 + c;
          if (n < N) zmi_finish_element_ring(p, epi, cst[wave * 64 + ni * 32 + c], rs, mine[x * 64], m, n);
        }
      }
    }
  });
}

// Second step of a K-sliced launch (plain epilogues only: gated launches are never sliced): adds the slices' partial
// tiles and finishes the elements.  One wavefront per 16-byte chunk column of a tile: lane l of chunk (wave w, ni, mi, g)
// holds row mi * 32 + l % 32 and the four columns from w * 64 + ni * 32 + g * 8 + (l / 32) * 4 of the tile.
template <int MI>
__global__ __launch_bounds__(S_THREADS) void zmi_stream_reduce_kernel(const ZmiProblem *probs, int n_prob, const int *tile_tab,
                                                                      int bm_idx, int top_flags, ZmiRingSplit split,
                                                                      ZmiEpilogue epi) {
  constexpr int BM = 32 * MI, CH = 2 * MI * 4;
  const int top = top_flags & 0xffff;
  const int lane = threadIdx.x % 64;
  constexpr int units_per_tile = 4 * CH;
  const int unit = blockIdx.x * (S_THREADS / 64) + threadIdx.x / 64;
  const int id = unit / units_per_tile;
  if (id >= tile_tab[bm_idx]) return;
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
  if (e < 0) return;
  const ZmiProblem p = probs[e];
  int full; bool rem;
  zmi_ring_rows<BM>(p.M, top_flags, full, rem);
  const int tiles_m = full + (rem ? 1 : 0);
  if (tiles_m <= 0) return;
  const int r = id - starts[e];
  const int tm = r % tiles_m, tn = r / tiles_m;
  const int m0 = tm < full ? tm * top : (p.M / top) * top;

  int u = unit % units_per_tile;
  const int g = u % 4; u /= 4;
  const int mi = u % MI; u /= MI;
  const int ni = u % 2; u /= 2;
  const int w = u;
  const int m = m0 + mi * 32 + lane % 32;
  if (m0 + mi * 32 >= p.M) return;        // (a fragment without rows: the slices stored nothing there)
  const int n0 = tn * 256 + w * 64 + ni * 32 + g * 8 + (lane / 32) * 4;
  v4i sum = {0, 0, 0, 0};
  for (int sl = 0; sl < split.slices; ++sl) {
    const int32_t *base = split.partial + (((int64_t)id * split.slices + sl) * 4 + w) * (int64_t)(CH * 256) + lane * 4;
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
    zmi_finish_element_ring(p, epi, zmi_col_ctx(epi, p, colsum, n, p.N), rs, sum[j], m, n);
  }
}

// True when the streaming kernel can stand in for the MFMA-bound kernel on a grouped launch with this epilogue.
bool zmi_group_stream_takes(const ZmiEpilogue &epi, int N, int top_flags) {
  const int top = top_flags & 0xffff;
  if (!(top_flags & ZMI_RING_PAD) || (top != 128 && top != 256)) return false;
  if (epi.n_groups > 0) return false;
  if (epi.gated_act != 0 && ((N / 2) % 32 != 0 || epi.fast_kind != ZMI_EK_NONE)) return false;
  return zmi_env(ZE_NO_GROUP_STREAM) == nullptr;
}

template <int MI, int D, int OCC, bool SPLIT>
static hipError_t stream_launch(const ZmiProblem *probs_dev, int n_prob, int n_items, const int *tab, int top,
                                const ZmiRingSplit &split, const ZmiEpilogue &epi, hipStream_t stream) {
  if (!SPLIT && split.slices > 1) return hipErrorInvalidValue;
  const size_t smem = 256 * 16 + (size_t)MI * 32 * 4 + (size_t)(D + 1) * MI * 2048;
  const int grid = (n_items * split.slices + 7) / 8 * 8;
  const int bm_idx = MI == 8 ? 0 : 1;
  if (epi.gated_act != 0) {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_stream_kernel<MI, D, true, OCC, false>, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((zmi_gemm_stream_kernel<MI, D, true, OCC, false>), dim3(grid), dim3(S_THREADS), smem, stream, probs_dev,
                       n_prob, n_items, tab, bm_idx, top, split, epi);
  } else {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_stream_kernel<MI, D, false, OCC, SPLIT>, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((zmi_gemm_stream_kernel<MI, D, false, OCC, SPLIT>), dim3(grid), dim3(S_THREADS), smem, stream, probs_dev,
                       n_prob, n_items, tab, bm_idx, top, split, epi);
    if (SPLIT && split.slices > 1) {
      const int units = n_items * 4 * (2 * MI * 4);
      hipLaunchKernelGGL((zmi_stream_reduce_kernel<MI>), dim3((units + S_THREADS / 64 - 1) / (S_THREADS / 64)), dim3(S_THREADS), 0,
                         stream, probs_dev, n_prob, tab, bm_idx, top, split, epi);
    }
  }
  return hipGetLastError();
}

// Tiles of a launch (an upper bound when the row counts live on the device: probs_host null).
int zmi_stream_items(const ZmiProblem *probs_host, int n_prob, int top, int64_t worst_rows, int worst_cols, bool gated) {
  const int th = top & 0xffff;
  int items = 0;
  if (probs_host) {
    for (int e = 0; e < n_prob; ++e) {
      const ZmiProblem &q = probs_host[e];
      if (q.M <= 0) continue;
      items += th == 256 ? zmi_ring_items<256>(q.M, q.N, top, gated) : zmi_ring_items<128>(q.M, q.N, top, gated);
    }
  } else {
    const int per = gated ? 128 : 256;
    const int ncols = gated ? worst_cols / 2 : worst_cols;
    items = (int)(worst_rows / th + n_prob) * ((ncols + per - 1) / per);
  }
  return items;
}
// Workspace of a K-sliced launch: every (tile, slice) leaves a th x 256 int32 tile.
size_t zmi_stream_partial_bytes(int items, int slices, int top) {
  return slices > 1 ? (size_t)items * slices * (top & 0xffff) * 256 * sizeof(int32_t) : 0;
}

// Same contract as zmi_launch_gemm_ring_group for top = 128 | ZMI_RING_PAD or 256 | ZMI_RING_PAD (one launch, every
// problem's remainder rows in a partly filled tile); tab_dev must already hold the tile table (zmi_launch_ring_table
// or the kernel that built the problems).  split (may be null): K slices per tile and their workspace of
// zmi_stream_partial_bytes bytes; plain epilogues only.
hipError_t zmi_launch_gemm_stream_group(const ZmiProblem *probs_host, const ZmiProblem *probs_dev, int n_prob, int top,
                                        int64_t worst_rows, int worst_cols, const int *tab_dev, const ZmiRingSplit *split,
                                        const ZmiEpilogue &epi, hipStream_t stream) {
  const bool gated = epi.gated_act != 0;
  const int th = top & 0xffff;
  if (!tab_dev || !(top & ZMI_RING_PAD) || (th != 128 && th != 256)) return hipErrorInvalidValue;
  ZmiRingSplit sp = {1, nullptr, nullptr};
  if (split && split->slices > 1) {
    if (gated || !split->partial) return hipErrorInvalidValue;
    sp = *split;
  }
  const int items = zmi_stream_items(probs_host, n_prob, top, worst_rows, worst_cols, gated);
  if (items <= 0) return hipSuccess;
  if (th == 256) {
    sp.slices = 1;   // (not sliced: see the kernel)
    return stream_launch<8, 6, 1, false>(probs_dev, n_prob, items, tab_dev, top, sp, epi, stream);
  }
  // two workgroups per compute unit: one's epilogue and start-up run under the other's stream
  return stream_launch<4, 4, 2, true>(probs_dev, n_prob, items, tab_dev, top, sp, epi, stream);
}
