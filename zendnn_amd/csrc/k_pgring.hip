// Per-group symmetric int8 GEMM for gfx950 at large M:
//   C[M, N] = tail(sum_g (float(acc_g) * ss[m, g]) * ws[g, n]),  acc_g on v_mfma_i32_32x32x32_i8.
//
// Call site replaced: the aocl_gemm_s8s8s32o{f32,bf16}_sym_quant call with a group size
// (zendnnl/src/lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:1239-1257); semantics: the
// per-group branch of the reference's scalar kernel
// (zendnnl/src/operators/matmul/matmul_ref_kernel.cpp:917-1001) -- every group's integer sum is
// scaled by the source scale of (row, group), then by the weight scale of (group, column), each
// product rounded, and the f32 terms are added in group order.
//
// Both operands are in MFMA fragment order (1 KiB fragments of 32 rows x 32 k, zmi_device.h).  A
// workgroup of 8 wavefronts owns a 256 x 128 or a 128 x 256 tile, every wavefront 64 x 64 of it
// (2 x 2 MFMA blocks: 64 integer accumulators and 64 f32 sums per lane, so that both live in the 256
// registers a wavefront has when two share a SIMD).  K is walked in slots of 64 or 128 k that travel
// global memory -> LDS without passing through registers (global_load_lds), NS - 1 slots ahead, and
// the scales of a slot's groups ride with it ({rows of the tile} source scales, {columns of the
// tile} weight scales per group): the fold of a group needs no global load.
//
// The fold is what bounds the kernel: four VALU instructions per output element and group (convert,
// two multiplies, one add) against one MFMA per 1024 elements and 32 k.  With groups of 128 that is
// 256 VALU instructions per 16 MFMAs and wavefront, about twice the MFMAs' own time, so the MFMAs
// of a 32 x 32 block are issued between the fold instructions of the block before it and run under
// them; the second wavefront of the SIMD fills what is left.
#include <type_traits>

#include "zmi_device.h"
#include "zmi_launch.h"

#define PR_THREADS 512
#define PR_EPI_LD 68                        // words per staged row (64 + 4: rows 4 banks apart)

extern __shared__ __attribute__((aligned(16))) char zmi_pgring_smem[];

// KB: k-steps of 32 per block of MFMAs on one accumulator set: 1 (groups of 32, a fold per k-step), 2 (groups of
// 64), 4 (groups of 128 j: a fold every j-th block)
template <int BM, int KB>
struct PgRingCfg {
  static constexpr int BN = 384 - BM;
  static constexpr int AF = BM / 32, BF = BN / 32;       // fragment rows / columns of the tile: 12 together
  static constexpr int STAGE = 12 * 2048;                // 64 k of both operands
  static constexpr int SS = KB == 4 ? 2 : 1;             // stages per slot
  static constexpr int NG = KB == 1 ? 2 : 1;             // groups whose scales ride with a slot
  static constexpr int SC_GROUP = 384 * 4;               // [BM source scales][BN weight scales], f32
  static constexpr int SLOT = SS * STAGE + NG * SC_GROUP + 256;   // (+ 256 bytes that surplus wavefronts load into)
  static constexpr int NS = KB == 4 ? 3 : 5;
  static constexpr int LOADS = 3 * SS + NG;              // load instructions per wavefront and slot
  static constexpr int RING = SLOT * NS;
  static constexpr int EPI = 8 * 32 * PR_EPI_LD * 4;     // epilogue staging, reuses the ring
  static constexpr int SMEM = RING > EPI ? RING : EPI;
};

__device__ __forceinline__ void zmi_pr_dma16(const void *base, uint32_t voff, uint32_t lds) {
  // one 1 KiB fragment: LDS address = m0 + lane * 16
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void zmi_pr_dma4(const void *base, uint32_t voff, uint32_t lds) {
  // 64 floats from 64 addresses: LDS address = m0 + lane * 4
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void zmi_pr_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void zmi_pr_barrier() { asm volatile("s_barrier" ::: "memory"); }
template <class T>
__device__ __forceinline__ T zmi_pr_uniform(T p) {
  uintptr_t v = (uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (T)(((uintptr_t)hi << 32) | lo);
}

// ss: {M, G} f32 source scales; ws: {G, np} f32 weight scales, rows padded to np (a multiple of 256) columns
// MULTI (KB == 4 only): groups of more than one block (256, 384, ... k)
template <int BM, int KB, bool MULTI>
__global__ __launch_bounds__(PR_THREADS, 1) void zmi_gemm_pgring_kernel(ZmiProblem p, ZmiEpilogue epi, const float *ss,
                                                                        const float *ws, int np, int n_items, int gs) {
  using Cfg = PgRingCfg<BM, KB>;
  constexpr int BN = Cfg::BN, AF = Cfg::AF, STAGE = Cfg::STAGE, SS = Cfg::SS, NG = Cfg::NG, SLOT = Cfg::SLOT, NS = Cfg::NS;
  constexpr int WN = BN / 64;                       // wavefronts along the columns
  char *smem = zmi_pgring_smem;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / WN, wn = wave % WN;
  const int M = p.M, N = p.N, K = p.K, G = epi.n_groups;

  // ---- which tile: workgroup ids go round robin over the 8 XCDs; renumber so that every XCD gets a contiguous
  // range of tiles, ordered so that neighbours share weight columns and a band of up to 8 row tiles ----
  const int b = blockIdx.x;
  const int per_xcd = (n_items + 7) / 8;
  const int id = (b % 8) * per_xcd + b / 8;
  if (b / 8 >= per_xcd || id >= n_items) return;
  int tm, tn;
  {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int GM = tiles_m < 8 ? tiles_m : 8;
    const int per_group = GM * tiles_n;
    const int group = id / per_group;
    const int first_m = group * GM;
    const int gm = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int r = id % per_group;
    tm = first_m + r % gm;
    tn = r / gm;
  }
  const int m0 = tm * BM, n0 = tn * BN;

  const int K_pad = (int)zmi_blob_kpad(K);
  const int n_slot = K / (64 * SS);              // whole slots (the launcher checks); the blob's rows past K are not visited
  const int64_t frow_bytes = (int64_t)K_pad * 32;
  const uint8_t *Afr = (const uint8_t *)p.A;
  const uint8_t *Bfr = p.blob + zmi_blob_tiles_off(N);
  const int a_last = (M + 31) / 32 - 1;
  const int b_last = (int)(zmi_blob_npad(N) / 32) - 1;

  // ---- this wavefront's share of a stage: fragments 3 wave .. 3 wave + 2 of its 24 (12 pairs of k blocks) ----
  const uint8_t *gbase[3];
  uint32_t lds_dst[3], koff[3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int f = wave * 3 + i, r = f / 2, kb = f % 2;
    int64_t frow;
    const uint8_t *base;
    if (r < AF) {
      const int fr = m0 / 32 + r;
      frow = fr < a_last ? fr : a_last;
      base = Afr;
    } else {
      const int fc = n0 / 32 + (r - AF);
      frow = fc < b_last ? fc : b_last;
      base = Bfr;
    }
    gbase[i] = zmi_pr_uniform(base + frow * frow_bytes);
    lds_dst[i] = r * 2048 + kb * 1024;
    koff[i] = kb * 1024 + lane * 16;
  }
  // ---- and of a group's scales: six runs of 64 floats ([BM source scales][BN weight scales]), one per wavefront;
  // wavefronts 6 and 7 repeat run 0 into the spare bytes so that every wavefront counts the same loads ----
  const int job = wave < 6 ? wave : 0;
  const bool job_ss = job * 64 < BM;
  const float *sc_base = zmi_pr_uniform(job_ss ? ss : ws);
  uint32_t sc_voff, sc_step;                       // byte offset of this lane's element for group 0, step per group
  if (job_ss) {
    const int r = m0 + job * 64 + lane;
    sc_voff = (uint32_t)(((int64_t)(r < M ? r : M - 1) * G) * 4);
    sc_step = 4;
  } else {
    sc_voff = (uint32_t)((n0 + job * 64 - BM + lane) * 4);
    sc_step = (uint32_t)np * 4;
  }
  const uint32_t sc_lds = wave < 6 ? job * 256 : NG * Cfg::SC_GROUP;

  auto issue_slot = [&](int buf, int n, uint32_t mask = 0xffffffffu) {
    const uint32_t lb = buf * SLOT;
#pragma unroll
    for (int st = 0; st < SS; ++st)
#pragma unroll
      for (int i = 0; i < 3; ++i)
        zmi_pr_dma16(gbase[i], (koff[i] + (uint32_t)(n * SS + st) * 2048) & mask, lb + st * STAGE + lds_dst[i]);
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
      const int g = KB == 1 ? n * 2 + gi : KB == 2 ? n : (n * 128) / gs;
      zmi_pr_dma4(sc_base, (sc_voff + (uint32_t)g * sc_step) & mask, lb + SS * STAGE + (wave < 6 ? gi * Cfg::SC_GROUP : 0) + sc_lds);
    }
  };

  v16i acc[2][2];
  float sum[2][2][16];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) { acc[ni][mi][j] = 0; sum[ni][mi][j] = 0.0f; }

  const int hi = lane / 32, cl = lane % 32;
  // One block: KB k-steps on the four accumulator blocks, block by block.  A block that closes a group (FOLD) folds
  // every accumulator block into the f32 sums as soon as its last MFMA is issued, under the MFMAs of the next one.
  // Groups of one block start their first MFMA from zero; longer groups (MULTI) accumulate across blocks and the
  // fold clears what it has read.
  auto block = [&](auto fold_c, const char *sb, const float *sc, int ks0) {
    constexpr bool FIRST = !MULTI, FOLD = decltype(fold_c)::value;
    __builtin_amdgcn_sched_barrier(0);
    v4i fa[2][KB];
#pragma unroll
    for (int j = 0; j < KB; ++j) {
      const int ks = ks0 + j;
      const char *pr = sb + (ks / 2) * STAGE + (ks % 2) * 1024;
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i][j] = *(const v4i *)(pr + (wm * 2 + i) * 2048);
    }
    float ssv[2];
    if (FOLD) {
      ssv[0] = sc[wm * 64 + cl];
      ssv[1] = sc[wm * 64 + 32 + cl];
    }
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      v4i fb[KB];
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        const int ks = ks0 + j;
        fb[j] = *(const v4i *)(sb + (ks / 2) * STAGE + (ks % 2) * 1024 + (AF + wn * 2 + ni) * 2048);
      }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          if (FIRST && j == 0) {
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[mi][j], zero, 0, 0, 0);
          } else {
            acc[ni][mi] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[mi][j], acc[ni][mi], 0, 0, 0);
          }
        }
        if (FOLD) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const v4f w = *(const v4f *)(sc + BM + wn * 64 + ni * 32 + g * 8 + hi * 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float t = __fmul_rn((float)acc[ni][mi][g * 4 + j], ssv[mi]);
              t = __fmul_rn(t, w[j]);
              sum[ni][mi][g * 4 + j] = __fadd_rn(sum[ni][mi][g * 4 + j], t);
              if (MULTI) acc[ni][mi][g * 4 + j] = 0;
            }
          }
        }
      }
    }
    if (FOLD) {
      // instruction order: the first accumulator block's MFMAs, then every MFMA of a later block followed by its
      // share of the 64 (+ 16 clears) fold instructions of the block before, then the last block's fold
      constexpr int FV = MULTI ? 80 : 64;
      __builtin_amdgcn_sched_group_barrier(0x008, KB, 0);
#pragma unroll
      for (int t = 1; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, FV / KB, 0);
        }
      __builtin_amdgcn_sched_group_barrier(0x002, FV, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using std::integral_constant;
  const integral_constant<bool, true> yes{};
  const integral_constant<bool, false> no{};

  if (MULTI) {
    // ---- groups of several blocks: NS - 1 slots in flight (slot numbers past the end repeat the last slot: the
    // counts stay uniform); the fold of a group's last block is not overlapped (32 or more MFMAs per fold) ----
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue_slot(s, s < n_slot ? s : n_slot - 1);
    const int bpg = gs / 128;                        // blocks per group
    int buf = 0, in_group = 0;
    for (int n = 0; n < n_slot; ++n) {
      // slot n has landed (this wavefront's loads; the barrier adds everybody else's) and slot n - 1 is free
      zmi_pr_wait_vm<(NS - 2) * Cfg::LOADS>();
      zmi_pr_barrier();
      {
        const int ahead = n + NS - 1;
        issue_slot(buf == 0 ? NS - 1 : buf - 1, ahead < n_slot ? ahead : n_slot - 1);
      }
      const char *sb = smem + buf * SLOT + lane * 16;
      const float *sc = reinterpret_cast<const float *>(smem + buf * SLOT + SS * STAGE);
      const bool fold = in_group == bpg - 1;
      if (fold) block(yes, sb, sc, 0);
      else block(no, sb, sc, 0);
      in_group = fold ? 0 : in_group + 1;
      buf = buf + 1 == NS ? 0 : buf + 1;
    }
  } else {
    // ---- a fold per block: software pipeline over the four accumulator blocks t = 0 .. 3 = (ni, mi) in
    // (0,0) (0,1) (1,0) (1,1).  Every MFMA of block t is followed by a KB-th of the fold of block t - 1 (16 .. 64
    // VALU instructions, which take longer than the MFMA runs); the fold of block 3 rides under block 0 of the
    // next k block.  The LDS reads are placed by hand: weight scales of column half ni one block ahead of their
    // fold, the fragments of column half 1 during block 1, and the operands of the next k block during block 3,
    // after the slot's one barrier -- which sits before block 3, where every read of the slot has been issued,
    // so the slot's own buffer takes the loads of the slot NS ahead. ----
    constexpr int NB = KB == 1 ? 2 : 1;              // k blocks per slot
    constexpr int E = 16 / KB;                       // accumulators per fold chunk
    v16i tacc[4];
    v4f w0[4], w1[4];
    v4i fa[2][KB], fb0[KB], fb1[KB];
    float ssv[2], ssn[2], p_ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) tacc[3][i] = 0;     // (the first fold under block 0 adds zeros)
#pragma unroll
    for (int g = 0; g < 4; ++g) w1[g] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
    auto frag = [&](const char *sb, int ks, int pair) {
      return *(const v4i *)(sb + (ks / 2) * STAGE + (ks % 2) * 1024 + pair * 2048);
    };
    // The order "one MFMA, a fold chunk, one MFMA, ..." is the point of the loop, and nothing in the data flow asks
    // for it, so it is pinned: empty asm statements (no instruction) that claim to rewrite a register keep their
    // order among themselves, every MFMA sits between the one that rewrites its weight fragment and the one that
    // rewrites its accumulators, every fold chunk between the one that rewrites the accumulators it reads and the
    // ones that read the sums it wrote.  (Scheduling barriers alone are not enough: they fix the order of what
    // instruction selection hands to the scheduler, and instruction selection is free to hand over all MFMAs first.)
#define PR_PIN(x) asm volatile("" : "+v"(x)::"memory")
    auto fold_chunk = [&](auto tc, int c, v16i &a, float sv, const v4f(&w)[4]) {
      constexpr int t = decltype(tc)::value;
      PR_PIN(a);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const int i = c * E + e;
        float v = __fmul_rn((float)a[i], sv);
        v = __fmul_rn(v, w[i / 4][i % 4]);
        sum[t / 2][t % 2][i] = __fadd_rn(sum[t / 2][t % 2][i], v);
      }
#pragma unroll
      for (int e = 0; e < E; ++e) asm volatile("" ::"v"(sum[t / 2][t % 2][c * E + e]) : "memory");
    };
    auto mma = [&](v16i &a, v4i &b, const v4i &f, bool first) {
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      PR_PIN(b);
      a = first ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b, f, zero, 0, 0, 0) : __builtin_amdgcn_mfma_i32_32x32x32_i8(b, f, a, 0, 0, 0);
      PR_PIN(a);
    };
    const integral_constant<int, 0> T0{};
    const integral_constant<int, 1> T1{};
    const integral_constant<int, 2> T2{};
    const integral_constant<int, 3> T3{};
#define PR_FENCE __builtin_amdgcn_sched_barrier(0)
    // (slot numbers past the end repeat the last slot, so that the count of the first wait holds for any K)
#pragma unroll
    for (int s = 0; s < NS; ++s) issue_slot(s, s < n_slot ? s : n_slot - 1);
    zmi_pr_wait_vm<(NS - 1) * Cfg::LOADS>();
    zmi_pr_barrier();
    {
      const char *sb = smem + lane * 16;
      const float *sc = reinterpret_cast<const float *>(smem + SS * STAGE);
#pragma unroll
      for (int j = 0; j < KB; ++j) {
        fa[0][j] = frag(sb, j, wm * 2);
        fa[1][j] = frag(sb, j, wm * 2 + 1);
        fb0[j] = frag(sb, j, AF + wn * 2);
      }
      ssv[0] = sc[wm * 64 + cl];
      ssv[1] = sc[wm * 64 + 32 + cl];
    }
    int buf = 0;
    for (int n = 0; n < n_slot; ++n) {
      const int buf_next = buf + 1 == NS ? 0 : buf + 1;
#pragma unroll
      for (int bi = 0; bi < NB; ++bi) {
        const char *sb = smem + buf * SLOT + lane * 16;
        const float *scw = reinterpret_cast<const float *>(smem + buf * SLOT + SS * STAGE) + bi * 384 + BM + wn * 64 + hi * 4;
        const int ks0 = bi * KB;
        PR_FENCE;
        // block 0 under the fold of the previous k block's block 3
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          mma(tacc[0], fb0[j], fa[0][j], j == 0);
          PR_FENCE;
          fold_chunk(T3, j, tacc[3], p_ss, w1);
          if (j == 0) {
#pragma unroll
            for (int g = 0; g < 4; ++g) w0[g] = *(const v4f *)(scw + g * 8);
          }
          PR_FENCE;
        }
        // block 1; the fragments of column half 1
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          mma(tacc[1], fb0[j], fa[1][j], j == 0);
          PR_FENCE;
          fold_chunk(T0, j, tacc[0], ssv[0], w0);
          if (j == 0) {
#pragma unroll
            for (int jj = 0; jj < KB; ++jj) fb1[jj] = frag(sb, ks0 + jj, AF + wn * 2 + 1);
          }
          PR_FENCE;
        }
        // block 2; the weight scales of column half 1
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          mma(tacc[2], fb1[j], fa[0][j], j == 0);
          PR_FENCE;
          fold_chunk(T1, j, tacc[1], ssv[1], w0);
          if (j == 0) {
#pragma unroll
            for (int g = 0; g < 4; ++g) w1[g] = *(const v4f *)(scw + 32 + g * 8);
          }
          PR_FENCE;
        }
        // every LDS read of this k block has been issued.  After a slot's last k block: the next slot has landed
        // (this wavefront's loads; the barrier adds everybody else's) and this slot's buffer is free
        const char *sb_n;
        const float *sc_n;
        int ks_n;
        if (bi == NB - 1) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          zmi_pr_wait_vm<(NS - 2) * Cfg::LOADS>();
          zmi_pr_barrier();
          // (past the last slot the loads go on, so that the counts stay uniform without a branch in the loop, but
          // every lane then asks for the first bytes of its fragment row: one cache line per load)
          const bool more = n + NS < n_slot;
          issue_slot(buf, more ? n + NS : 0, more ? 0xffffffffu : 0u);
          sb_n = smem + buf_next * SLOT + lane * 16;
          sc_n = reinterpret_cast<const float *>(smem + buf_next * SLOT + SS * STAGE);
          ks_n = 0;
        } else {
          sb_n = sb;
          sc_n = reinterpret_cast<const float *>(smem + buf * SLOT + SS * STAGE) + (bi + 1) * 384;
          ks_n = (bi + 1) * KB;
        }
        PR_FENCE;
        // block 3; the next k block's operands (row half 1's fragments once block 3 has read them)
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          mma(tacc[3], fb1[j], fa[1][j], j == 0);
          PR_FENCE;
          fold_chunk(T2, j, tacc[2], ssv[0], w1);
          if (j == 0) {
#pragma unroll
            for (int jj = 0; jj < KB; ++jj) {
              fa[0][jj] = frag(sb_n, ks_n + jj, wm * 2);
              fb0[jj] = frag(sb_n, ks_n + jj, AF + wn * 2);
            }
            ssn[0] = sc_n[wm * 64 + cl];
            ssn[1] = sc_n[wm * 64 + 32 + cl];
          }
          if (j == KB - 1) {
#pragma unroll
            for (int jj = 0; jj < KB; ++jj) fa[1][jj] = frag(sb_n, ks_n + jj, wm * 2 + 1);
          }
          PR_FENCE;
        }
        p_ss = ssv[1];
        ssv[0] = ssn[0];
        ssv[1] = ssn[1];
      }
      buf = buf_next;
    }
    PR_FENCE;
#pragma unroll
    for (int j = 0; j < KB; ++j) fold_chunk(T3, j, tacc[3], p_ss, w1);
#undef PR_FENCE
#undef PR_PIN
  }
  zmi_pr_wait_vm<0>();
  zmi_pr_barrier();

  // ---- epilogue: every 32 x 64 strip goes through LDS and is read back with 16 lanes per row, 4 columns each:
  // rows are stored as 128-byte (bf16) or 256-byte (f32) runs.  alpha / beta, then the common tail. ----
  float *stage = reinterpret_cast<float *>(smem) + wave * (32 * PR_EPI_LD);
  const int c16 = lane % 16, r4 = lane / 16;
  const int dst_dt = epi.dst_dt;
  const int es = dst_dt == ZMI_DT_BF16 ? 2 : 4;
  const bool vec_ok = (((uintptr_t)p.dst) % 16 == 0) && ((p.ldc * es) % 16 == 0);
  // straight-line forms: bias (+ one activation in the MFMA-bound kernel's hardware exp / reciprocal form when the
  // store is bf16: the sums are final, so the wavefront may flush f32 denormals from here on, which makes the
  // hardware bf16 conversion the reference's) and 8- / 16-byte stores; everything else goes through the interpreter
  const bool plain = epi.fast_kind != ZMI_EK_GENERIC &&
                     (dst_dt == ZMI_DT_BF16 || (dst_dt == ZMI_DT_F32 && epi.fast_kind == ZMI_EK_NONE));
  const int act = epi.fast_kind;
  if (plain && dst_dt == ZMI_DT_BF16) zmi_set_f32_flush();
  const int nc = n0 + wn * 64 + c16 * 4;           // this lane's four output columns
  float bias[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) bias[j] = p.bias && nc + j < N ? zmi_ld_f32(p.bias, epi.bias_dt, nc + j) : 0.0f;
  auto do_strip = [&](auto mic) {
    constexpr int mi = decltype(mic)::value;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4f o = {sum[ni][mi][g * 4], sum[ni][mi][g * 4 + 1], sum[ni][mi][g * 4 + 2], sum[ni][mi][g * 4 + 3]};
        *(v4f *)&stage[cl * PR_EPI_LD + ni * 32 + g * 8 + hi * 4] = o;
      }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int mbase = m0 + wm * 64 + mi * 32;
#pragma unroll 2
    for (int it = 0; it < 8; ++it) {
      const int r = it * 4 + r4;
      const int m = mbase + r;
      const v4f a = *(const v4f *)&stage[r * PR_EPI_LD + c16 * 4];
      if (m >= M || nc >= N) continue;
      const int64_t o = (int64_t)m * p.ldc + nc;
      if (plain) {
        float y[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = __fadd_rn(a[j], bias[j]);
        if (act != ZMI_EK_NONE) {   // (uniform; bf16 stores only)
#pragma unroll
          for (int j = 0; j < 4; ++j) y[j] = zmi_act_bf16_kind(act, y[j]);
        }
        if (vec_ok && nc + 3 < N) {
          if (dst_dt == ZMI_DT_BF16) {
            const v2u v = {zmi_pack_bf16(y[0], y[1]), zmi_pack_bf16(y[2], y[3])};
            *zmi_global<v2u>((uint16_t *)p.dst + o) = v;
          } else {
            *zmi_global<v4f>((float *)p.dst + o) = (v4f){y[0], y[1], y[2], y[3]};
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (nc + j < N) {
              if (dst_dt == ZMI_DT_BF16) zmi_global<uint16_t>(p.dst)[o + j] = (uint16_t)zmi_pack_bf16(y[j], 0.0f);
              else zmi_global<float>(p.dst)[o + j] = y[j];
            }
        }
      } else {
#pragma unroll 1
        for (int j = 0; j < 4; ++j)
          if (nc + j < N) {
            float y = a[j];
            if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
            if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, dst_dt, o + j), epi.beta));
            zmi_store(p.dst, dst_dt, o + j, zmi_epilogue_tail(epi, y, bias[j], m, nc + j));
          }
      }
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
  };
  do_strip(integral_constant<int, 0>{});
  do_strip(integral_constant<int, 1>{});
}

template <int BM, int KB, bool MULTI = false>
static hipError_t pgring_launch(const ZmiProblem &p, const ZmiEpilogue &epi, const float *ss, const float *ws, int np, int gs,
                                hipStream_t stream) {
  using Cfg = PgRingCfg<BM, KB>;
  hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_pgring_kernel<BM, KB, MULTI>, Cfg::SMEM);
  if (e != hipSuccess) return e;
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + Cfg::BN - 1) / Cfg::BN);
  const dim3 grid((unsigned)((tiles + 7) / 8 * 8)), block(PR_THREADS);
  hipLaunchKernelGGL((zmi_gemm_pgring_kernel<BM, KB, MULTI>), grid, block, Cfg::SMEM, stream, p, epi, ss, ws, np, tiles, gs);
  return hipGetLastError();
}

// group sizes the kernel takes: 32 (whole slots of 64 k only), 64, multiples of 128
bool zmi_pgring_takes(int64_t M, int64_t N, int64_t K, int64_t gs) {
  if (M <= 0 || N <= 0 || K <= 0 || gs <= 0 || K % gs != 0) return false;
  if (gs == 32) return K % 64 == 0;
  return gs == 64 || gs % 128 == 0;
}

int64_t zmi_pgring_ws_cols(int64_t N) { return zmi_round_up(N, 256); }

// p.A: the s8 rows in fragment order; ss: {M, G} f32; ws: {G, zmi_pgring_ws_cols(N)} f32
hipError_t zmi_launch_gemm_pgring(const ZmiProblem &p, const ZmiEpilogue &epi, const float *ss, const float *ws,
                                  hipStream_t stream) {
  const int G = epi.n_groups;
  if (G <= 0 || !ss || !ws || p.a_is_u8 || epi.has_zp || epi.gated_act) return hipErrorInvalidValue;
  const int gs = p.K / G;
  if (!zmi_pgring_takes(p.M, p.N, p.K, gs)) return hipErrorInvalidValue;
  if (epi.dst_dt != ZMI_DT_F32 && epi.dst_dt != ZMI_DT_BF16) return hipErrorInvalidValue;
  const int np = (int)zmi_pgring_ws_cols(p.N);
  // (32-bit byte offsets into the scale arrays)
  if ((int64_t)p.M * G * 4 >= ((int64_t)1 << 31) || (int64_t)G * np * 4 >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
  // the tile shape that pads M less; 256-row tiles when both pad alike
  const bool bm128 = zmi_round_up(p.M, 128) < zmi_round_up(p.M, 256);
  const int kb = gs == 32 ? 1 : gs == 64 ? 2 : 4;
  if (bm128) {
    if (kb == 1) return pgring_launch<128, 1>(p, epi, ss, ws, np, gs, stream);
    if (kb == 2) return pgring_launch<128, 2>(p, epi, ss, ws, np, gs, stream);
    if (gs == 128) return pgring_launch<128, 4>(p, epi, ss, ws, np, gs, stream);
    return pgring_launch<128, 4, true>(p, epi, ss, ws, np, gs, stream);
  }
  if (kb == 1) return pgring_launch<256, 1>(p, epi, ss, ws, np, gs, stream);
  if (kb == 2) return pgring_launch<256, 2>(p, epi, ss, ws, np, gs, stream);
  if (gs == 128) return pgring_launch<256, 4>(p, epi, ss, ws, np, gs, stream);
  return pgring_launch<256, 4, true>(p, epi, ss, ws, np, gs, stream);
}

// ---- scales {rows, cols} (f32 or bf16) -> f32 rows of out_cols columns (zeros past cols) ----
__global__ __launch_bounds__(256) void zmi_pgring_scales_kernel(const void *src, int32_t dt, int64_t rows, int64_t cols,
                                                                int64_t out_cols, float *out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * out_cols) return;
  const int64_t r = i / out_cols, c = i % out_cols;
  out[i] = c < cols ? zmi_ld_f32(src, dt, r * cols + c) : 0.0f;
}

hipError_t zmi_launch_pgring_scales(const void *src, int32_t dt, int64_t rows, int64_t cols, int64_t out_cols, float *out,
                                    hipStream_t stream) {
  if (rows <= 0 || cols <= 0 || out_cols < cols) return hipErrorInvalidValue;
  hipLaunchKernelGGL(zmi_pgring_scales_kernel, dim3((unsigned)((rows * out_cols + 255) / 256)), dim3(256), 0, stream, src, dt,
                     rows, cols, out_cols, out);
  return hipGetLastError();
}
