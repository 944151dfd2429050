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
// ahead; the scales of the wavefront's rows and columns are staged in LDS up to 128 groups
// at a time.  Groups of 16 or 32 k share a 64-k chunk: the chunk is multiplied once per group
// with the other groups' lanes of the row operand zeroed.
#include "zmi_device.h"
#include "zmi_fused_quant.h"
#include "zmi_launch.h"
#include <cstdlib>

#define PG_WAVES 2

// RB: 16-row blocks per wavefront (1, 2 or 4); D: chunks per operand set (RB * D == 8); SUB: groups per 64-k chunk (1: groups of whole
// chunks); CPG: chunks per group when that is 1 or 2 (groups of 64 / 128), 0: any other multiple of 64,
// taken from gs at run time
template <int RB, int D, int SUB, int CPG>
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
  // ---- operands: two sets of D chunks of 64 k; one set is multiplied while the other set's requests
  // (issued before it) are in flight.  (A ring refilled chunk by chunk ends up with all its requests
  // at the end of the loop body and a wait for all of them at the top: one memory latency per D chunks.)
  // The activation rows are requested row-contiguously (D * 4 consecutive lanes, D * 64 consecutive bytes:
  // in operand order a request touches 16 rows and takes the address unit four times as long), RB * D = 8
  // requests per set, and go through this wavefront's LDS area into operand order just before they are used.
  // Rows past M repeat row M - 1 (their results are never stored); k past K reads k = 0 (the blob's rows
  // past K are zero): every request is unconditional and the loop has no divergent branch. ----
  static_assert(RB * D == 8, "eight row requests per lane and set");
  constexpr int LPR = D * 4;                      // lanes (16-byte granules) per row and set
  constexpr int RPI = 64 / LPR;                   // rows per request
  const int a_q = lane % LPR, a_s = a_q / 4, a_g = a_q % 4;
  const int8_t *arow[8];
  int a_lds[8];                                   // byte offset of this lane's granule in the staging area
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int rl = i * RPI + lane / LPR;          // row within the wavefront's 16 RB rows
    const int row = row0 + rl;
    arow[i] = (const int8_t *)p.A + (int64_t)(row < M ? row : M - 1) * p.lda;
    a_lds[i] = ((((rl / 16) * D + a_s) * 64 + a_g * 16 + ((rl % 16) ^ ((a_g * 4 + (a_s & 3)) & 15))) << 4);
  }
  __shared__ __attribute__((aligned(16))) uint8_t a_stage[PG_WAVES][RB * D * 1024];
  uint8_t *a_l = a_stage[wave];
  v4i b[2][D], raw[2][8];
  auto request_set = [&](int set, int c_first) {
    {
      const int c = c_first + a_s;
      const int cc = c < nch ? c : nch - 1;        // past the end: a valid chunk, never used
      const int k = cc * 64 + a_g * 16;
      const int ka = k < K ? k : 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) raw[set][i] = *(const v4i *)(arow[i] + ka);
    }
#pragma unroll
    for (int s = 0; s < D; ++s) {
      const int c = c_first + s;
      const int cc = c < nch ? c : nch - 1;        // (uniform)
      b[set][s] = *(const v4i *)(bsrc + (int64_t)cc * 2048);
    }
  };
  // the set's rows -> LDS in operand order (bank-swizzled like the decode kernel's staging); only this
  // wavefront's lanes touch the area and a wavefront's LDS accesses are served in order, so wavefront-scope
  // fences (no instruction) are all the synchronisation there is
  auto stage_rows = [&](int set) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) *(v4i *)(a_l + a_lds[i]) = raw[set][i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  auto operand = [&](int s, int j) {
    return *(const v4i *)(a_l + (((j * D + s) * 64 + g4 * 16 + (c16 ^ ((g4 * 4 + (s & 3)) & 15))) << 4));
  };
  request_set(0, 0);
  request_set(1, D);

  // ---- scales: this wavefront's slices ({G,16} weight scales, {16 RB, G} source scales) are staged in its own
  // LDS area GB groups at a time, all requests in flight at once; a fold then needs no global load.  (Fetching
  // them one group ahead from global memory made every fold wait for a full memory latency.) ----
  constexpr int GB = RB == 1 ? 128 : RB == 2 ? 64 : 32;   // groups per staged block: 16 / 12 / 10 KiB per wavefront
  __shared__ float scale_lds[PG_WAVES][(16 + 16 * RB) * GB];
  float *ws_l = scale_lds[wave], *ss_l = scale_lds[wave] + 16 * GB;
  auto stage_scales = [&](int gb0) {
    const int ng = G - gb0 < GB ? G - gb0 : GB;
    // (other lanes of this wavefront may still read the previous block; its LDS accesses are served in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // (no divergent branch and no type switch inside the loops, so that eight requests go out per wait;
    // columns past N and rows past M read the last valid one, their results are never stored)
    auto fill = [&](float *dst_l, const void *src, bool bf16, int count, auto index, auto slot) {
      if (bf16) {
#pragma unroll 8
        for (int i = lane; i < count; i += 64) dst_l[slot(i)] = zmi_bf16_to_f32(((const uint16_t *)src)[index(i)]);
      } else {
#pragma unroll 8
        for (int i = lane; i < count; i += 64) dst_l[slot(i)] = ((const float *)src)[index(i)];
      }
    };
    fill(ws_l, p.wei_scale_ptr, epi.wei_scale_dt == ZMI_DT_BF16, ng * 16,
         [&](int i) { const int n = cb * 16 + i % 16; return (int64_t)(gb0 + i / 16) * N + (n < N ? n : N - 1); },
         [&](int i) { return i; });
    fill(ss_l, p.src_scale_ptr, epi.src_scale_dt == ZMI_DT_BF16, ng * 16 * RB,
         [&](int i) { const int r = row0 + i / ng; return (int64_t)(r < M ? r : M - 1) * G + gb0 + i % ng; },
         [&](int i) { return (i / ng) * GB + i % ng; });
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  v4i acc[RB];
  float sum[RB][4];
#pragma unroll
  for (int j = 0; j < RB; ++j) {
    acc[j] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 4; ++q) sum[j][q] = 0.0f;
  }
  // group gi (gl within the staged block) is complete in acc:
  // sum += (float(acc) * ss[m, gi]) * ws[gi, n], each step rounded
  auto fold = [&](int gl) {
    const float wsv = ws_l[gl * 16 + c16];
#pragma unroll
    for (int j = 0; j < RB; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float t = __fmul_rn((float)acc[j][q], ss_l[(j * 16 + g4 * 4 + q) * GB + gl]);
        t = __fmul_rn(t, wsv);
        sum[j][q] = __fadd_rn(sum[j][q], t);
      }
      acc[j] = (v4i){0, 0, 0, 0};
    }
  };

  const int cpg = SUB != 1 ? 1 : CPG ? CPG : gs / 64;             // chunks per group
  const int blk_chunks = SUB == 1 ? GB * cpg : GB / SUB;        // chunks per staged block (a multiple of 2 D)
  // one chunk: multiply, fold where a group ends.  s is the chunk's position in its block of D (c % D):
  // with CPG known the fold positions are fixed at compile time and a block of D chunks is straight-line
  // code
  auto step = [&](int c, int set, int s, int gb0) {
    if (SUB == 1) {
#pragma unroll
      for (int j = 0; j < RB; ++j)
        acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(operand(s, j), b[set][s], acc[j], 0, 0, 0);
      // (K_pad may reach one chunk past K: that chunk's weights are zero and its group does not exist -- no fold,
      // its scales were never staged)
      if ((CPG ? (s + 1) % (CPG ? CPG : 1) == 0 : (c + 1) % cpg == 0) && c / cpg < G) fold(c / cpg - gb0);
    } else {
#pragma unroll
      for (int t = 0; t < SUB; ++t) {
        const int gi = c * SUB + t;
        if (gi < G) {   // (uniform; K_pad may reach past K)
          const bool mine = g4 / (4 / SUB) == t;   // this lane's 16 k belong to group t of the chunk
#pragma unroll
          for (int j = 0; j < RB; ++j) {
            const v4i am = mine ? operand(s, j) : (v4i){0, 0, 0, 0};
            acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(am, b[set][s], acc[j], 0, 0, 0);
          }
          fold(gi - gb0);
        }
      }
    }
  };
  for (int cb0 = 0; cb0 < nch; cb0 += blk_chunks) {
    const int gb0 = SUB == 1 ? cb0 / cpg : cb0 * SUB;           // first group of the block
    stage_scales(gb0);
    const int cend = cb0 + blk_chunks < nch ? cb0 + blk_chunks : nch;
    int c0 = cb0;
    for (; c0 + 2 * D <= cend; c0 += 2 * D) {
#pragma unroll
      for (int set = 0; set < 2; ++set) {
        stage_rows(set);
#pragma unroll
        for (int s = 0; s < D; ++s) step(c0 + set * D + s, set, s, gb0);
        __builtin_amdgcn_sched_barrier(0);   // the set's next requests stay between its use and the other set's
        request_set(set, c0 + set * D + 2 * D);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // (only the last block can end with fewer than 2 D chunks; nothing is requested after them)
#pragma unroll
    for (int set = 0; set < 2; ++set) {
      if (c0 + set * D >= cend) break;   // (uniform)
      stage_rows(set);
#pragma unroll
      for (int s = 0; s < D; ++s)
        if (c0 + set * D + s < cend) step(c0 + set * D + s, set, s, gb0);
    }
  }

  // ---- alpha / beta, then the common tail; acc element q of lane l is row (l / 16) * 4 + q, column l % 16 ----
  if (col >= N) return;
  const float bias = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, col) : 0.0f;
  // one straight-line activation into a bf16 store: the form of the tiled kernel for more rows (k_pgring.hip), so
  // that a row's bits do not depend on how many rows the call has
  const bool fast_act = epi.dst_dt == ZMI_DT_BF16 && epi.fast_kind != ZMI_EK_GENERIC && epi.fast_kind != ZMI_EK_NONE;
  if (fast_act) zmi_set_f32_flush();
#pragma unroll
  for (int j = 0; j < RB; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = row0 + j * 16 + g4 * 4 + q;
      if (m >= M) continue;
      const int64_t o = (int64_t)m * p.ldc + col;
      float y = sum[j][q];
      if (fast_act) {
        ((uint16_t *)p.dst)[o] = (uint16_t)zmi_pack_bf16(zmi_act_bf16_kind(epi.fast_kind, __fadd_rn(y, bias)), 0.0f);
        continue;
      }
      if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
      if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, epi.dst_dt, o), epi.beta));
      zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_tail(epi, y, bias, m, col));
    }
}

// ---- up to 16 rows: the decode kernel's shape with per-group partial tiles ---------------------
// One workgroup of 8 wavefronts per 32 weight columns, wavefront w streams the w-th eighth of K with all
// its requests in flight at once (k_decode.hip).  K may be split across wavefronts after all because what
// crosses them is INTEGER: every wavefront keeps one accumulator per group of its slice (GPW whole groups
// in CPW chunks of 64 k), the G = 8 GPW integer tiles meet in LDS, and one thread per output element then
// adds float(acc_g) * ss[m, g] * ws[g, n] in group order -- the reference's additions, in its order, with
// the weight stream of the per-token kernel.  Needs K = 512 * CPW (CPW in 1, 2, 4, 8) and whole groups of
// 64 .. 512 k per wavefront slice, or groups of 32 k (two per chunk); 16 tiles of 2 KiB meet in LDS at a time.
#define PGD_WAVES 8
#define PGD_THREADS (PGD_WAVES * 64)

__device__ __forceinline__ int pgd_lds_off(int cc, int g, int r) {   // operand granule of chunk cc, k group g, row r
  return cc * 1024 + ((g * 16 + (r ^ ((g * 4 + (cc & 3)) & 15))) << 4);
}

//
// S4: the weights are streamed as 4-bit codes, half the bytes.  tiles_s4 holds, per 32-column block, one 2 KiB
// piece per PAIR of 64-k chunks in the blob's lane order: every byte carries the code of the even chunk in its
// high nibble and the code of the odd chunk in its low nibble.  (w & 0xf0f0f0f0) and ((w << 4) & 0xf0f0f0f0) are
// then the two chunks' operands with every weight multiplied by 16 (a code in the high nibble of a byte IS
// 16 * code as a signed byte: no sign extension to compute), the integer tiles are exact multiples of 16 and
// are shifted back when they are folded.  |16 * code| <= 128, so the accumulators stay where s8 weights keep them.
template <int CPW, int GPW, bool S4>
__global__ __launch_bounds__(PGD_THREADS) void zmi_gemm_decode_pergroup_kernel(ZmiProblem p, ZmiEpilogue epi,
                                                                               ZmiFusedQuant fq, const uint8_t *tiles_s4) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  static_assert(!S4 || CPW % 2 == 0, "4-bit weights come in pairs of chunks");
  constexpr int SUB = GPW > CPW ? GPW / CPW : 1;  // groups per chunk (2: groups of 32 k)
  constexpr int CPG = GPW > CPW ? 1 : CPW / GPW;  // chunks per group
  constexpr int G = PGD_WAVES * GPW;
  constexpr int RT = G <= 32 ? G : 16;            // integer tiles (groups) that meet in LDS per round
  constexpr int WPR = RT / GPW;                   // wavefronts whose tiles make one round
  // LDS: the operand area (K * 16 bytes), which holds RT tiles of 2 KiB once the MFMAs are done; behind both,
  // the scales: [G][32] weight scales, [16][G] source scales.  (They are parked there as soon as the weight
  // requests are out: parking them only after the MFMAs, inside the freed operand area, cost 4 us -- their
  // requests end up next to the parking, a full memory latency after the last weight byte.)
  constexpr int MAIN = PGD_WAVES * CPW * 1024 > RT * 2048 ? PGD_WAVES * CPW * 1024 : RT * 2048;
  float *ws_l = reinterpret_cast<float *>(lds + MAIN);
  float *ss_l = ws_l + G * 32;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int M = p.M, N = p.N, K = p.K;
  // With fused quantization the first M workgroups quantize one source row each (per group), publish it and
  // leave; the streaming workgroups follow them in dispatch order and wait (bounded) for the M rows only after
  // their weight requests are out.  Producers wait for nothing, so the wait cannot deadlock.
  if (fq.x && (int)blockIdx.x < M) {
    if (fq.per_row) zmi_fused_quant_row(fq, blockIdx.x, K, reinterpret_cast<float *>(lds));
    else zmi_fused_quant_row_groups(fq, blockIdx.x, K, G);
    zmi_fq_publish(fq, blockIdx.x);
    return;
  }
  const int blk = fq.x ? (int)blockIdx.x - M : (int)blockIdx.x;
  const int c16 = lane % 16, g4 = lane / 16;
  const int c_begin = wave * CPW;

  // rows of this wavefront's slice: lanes 0..31 one row, lanes 32..63 the next (CPW * 64 bytes each)
  const int a_q = lane % 32;
  const bool a_live = a_q < CPW * 4;
  v4i araw[8];
  auto load_rows = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 2 * i + lane / 32;
      v4i v = {0, 0, 0, 0};
      if (a_live && row < M) v = *(const v4i *)((const int8_t *)p.A + (int64_t)row * p.lda + (c_begin * 4 + a_q) * 16);
      araw[i] = v;
    }
  };
  if (!fq.x) load_rows();
  // scales of this column block and of the rows, requested before the weight stream so that they are back
  // first (columns past N / rows past M: never stored, read as the last valid one)
  constexpr int WS_PT = (G * 32 + PGD_THREADS - 1) / PGD_THREADS;    // weight scales per thread
  constexpr int SS_PT = (16 * G + PGD_THREADS - 1) / PGD_THREADS;    // source scales per thread
  float ws_r[WS_PT], ss_r[SS_PT];
#pragma unroll
  for (int i = 0; i < WS_PT; ++i) {
    const int e0 = tid + i * PGD_THREADS, e = e0 < G * 32 ? e0 : G * 32 - 1, n = blk * 32 + e % 32;
    ws_r[i] = zmi_ld_f32(p.wei_scale_ptr, epi.wei_scale_dt, (int64_t)(e / 32) * N + (n < N ? n : N - 1));
  }
  auto load_ss = [&]() {
#pragma unroll
    for (int i = 0; i < SS_PT; ++i) {
      const int e0 = tid + i * PGD_THREADS, e = e0 < 16 * G ? e0 : 16 * G - 1, r = e / G;
      const int64_t rr = r < M ? r : M - 1;
      ss_r[i] = zmi_ld_f32(p.src_scale_ptr, epi.src_scale_dt, fq.x && fq.per_row ? rr : rr * G + e % G);
    }
  };
  if (!fq.x) load_ss();
  // the whole weight slice: NL loads of 2 KiB pieces per column group (a piece is a chunk, or a pair of chunks
  // of 4-bit codes)
  constexpr int NL = S4 ? CPW / 2 : CPW;
  const uint8_t *tiles = S4 ? tiles_s4 : p.blob + zmi_blob_tiles_off(N);
  const int64_t nb_stride = S4 ? zmi_s4_nb_stride(K) : zmi_blob_nb_stride(K);
  const int l_begin = S4 ? c_begin / 2 : c_begin;
  v4i braw[NL][2];
  const uint8_t *bsrc[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    bsrc[h] = tiles + (int64_t)blk * nb_stride + (g4 / 2) * 1024 + ((g4 % 2) * 32 + h * 16 + c16) * 16;
  // (with fused quantization three quarters of the slice go out before the wait for the rows, the rest
  // after the row requests, like the per-token decode kernel)
  constexpr int FIRST = NL >= 4 ? NL * 3 / 4 : NL;
#pragma unroll
  for (int u = 0; u < NL; ++u)
    if (u < FIRST || !fq.x) {
      braw[u][0] = *(const v4i *)(bsrc[0] + (int64_t)(l_begin + u) * 2048);
      braw[u][1] = *(const v4i *)(bsrc[1] + (int64_t)(l_begin + u) * 2048);
    }
  // operand of chunk u, column group h
  auto bop = [&](int u, int h) -> v4i {
    if (!S4) return braw[u][h];
    const v4i w = braw[u / 2][h];
    const int sh = (u % 2) * 4;
    return (v4i){(int)(((uint32_t)w[0] << sh) & 0xf0f0f0f0u), (int)(((uint32_t)w[1] << sh) & 0xf0f0f0f0u),
                 (int)(((uint32_t)w[2] << sh) & 0xf0f0f0f0u), (int)(((uint32_t)w[3] << sh) & 0xf0f0f0f0u)};
  };
  if (fq.x) {
    // the quantized rows and their scales exist once the counter says so
    // (one waiting wavefront per streaming workgroup; the others learn the outcome through LDS)
    int *ok_l = reinterpret_cast<int *>(lds);
    if (wave == 0) {
      const bool ok = zmi_fq_wait(fq, M);
      if (lane == 0) *ok_l = ok ? 1 : 0;
    }
    __syncthreads();
    const bool rows_ok = *ok_l != 0;
    __syncthreads();                 // (the operand area is written next)
    if (!rows_ok) return;            // the wait ran out: nothing is computed from unpublished rows
    asm volatile("" ::: "memory");   // the loads below stay below the wait
    load_rows();
    load_ss();
#pragma unroll
    for (int u = FIRST; u < NL; ++u) {
      braw[u][0] = *(const v4i *)(bsrc[0] + (int64_t)(l_begin + u) * 2048);
      braw[u][1] = *(const v4i *)(bsrc[1] + (int64_t)(l_begin + u) * 2048);
    }
  }
  // scales -> LDS
#pragma unroll
  for (int i = 0; i < WS_PT; ++i)
    if (tid + i * PGD_THREADS < G * 32) ws_l[tid + i * PGD_THREADS] = ws_r[i];
#pragma unroll
  for (int i = 0; i < SS_PT; ++i)
    if (tid + i * PGD_THREADS < 16 * G) ss_l[tid + i * PGD_THREADS] = ss_r[i];
  // rows -> LDS in operand order; the wavefront reads back only its own slice (wavefront-scope fences, no barrier)
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 2 * i + lane / 32;
    const int gran = c_begin * 4 + a_q;
    if (a_live) *(v4i *)(lds + pgd_lds_off(gran / 4, gran % 4, row)) = araw[i];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  v4i acc[GPW][2];
#pragma unroll
  for (int gi = 0; gi < GPW; ++gi) {
    acc[gi][0] = (v4i){0, 0, 0, 0};
    acc[gi][1] = (v4i){0, 0, 0, 0};
    if (SUB == 1) {
#pragma unroll
      for (int u = gi * CPG; u < (gi + 1) * CPG; ++u) {
        const v4i a = *(const v4i *)(lds + pgd_lds_off(c_begin + u, g4, c16));
        acc[gi][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bop(u, 0), acc[gi][0], 0, 0, 0);
        acc[gi][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bop(u, 1), acc[gi][1], 0, 0, 0);
      }
    } else {
      // two groups share a chunk: the chunk is multiplied once per group with the other group's lanes
      // (k groups of 16) of the row operand zeroed
      const int u = gi / SUB, t = gi % SUB;
      v4i a = *(const v4i *)(lds + pgd_lds_off(c_begin + u, g4, c16));
      if (g4 / (4 / SUB) != t) a = (v4i){0, 0, 0, 0};
      acc[gi][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bop(u, 0), acc[gi][0], 0, 0, 0);
      acc[gi][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bop(u, 1), acc[gi][1], 0, 0, 0);
    }
  }
  // ---- the operand area is done with ----
  __syncthreads();
  // ---- RT integer tiles at a time meet in LDS, in group order; one thread per output element adds the
  // group terms in order, each step rounded ----
  int32_t *red = (int32_t *)lds;
  const int e_row = tid / 32, e_h = (tid % 32) / 16, e_c = tid % 16;
  const int e_n = blk * 32 + e_h * 16 + e_c;
  const bool e_live = e_n < N && e_row < M;
  // acc[h][q] of lane l is row (l / 16) * 4 + q, column h * 16 + l % 16
  const int off = (e_h * 4 + e_row % 4) * 64 + (e_row / 4) * 16 + e_c;
  float sum = 0.0f;
  for (int r = 0; r < G / RT; ++r) {
    if (r > 0) __syncthreads();                    // the previous round's tiles have been read
    if (wave / WPR == r) {
#pragma unroll
      for (int gi = 0; gi < GPW; ++gi)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int q = 0; q < 4; ++q) red[((wave % WPR) * GPW + gi) * 512 + (h * 4 + q) * 64 + lane] = acc[gi][h][q];
    }
    __syncthreads();
#pragma unroll 8
    for (int t = 0; t < RT; ++t) {
      const int g = r * RT + t;
      float v = __fmul_rn((float)(S4 ? red[t * 512 + off] >> 4 : red[t * 512 + off]), ss_l[e_row * G + g]);
      v = __fmul_rn(v, ws_l[g * 32 + e_h * 16 + e_c]);
      sum = __fadd_rn(sum, v);
    }
  }
  if (!e_live) return;
  const int64_t o = (int64_t)e_row * p.ldc + e_n;
  float y = sum;
  if (epi.dst_dt == ZMI_DT_BF16 && epi.fast_kind != ZMI_EK_GENERIC && epi.fast_kind != ZMI_EK_NONE) {
    // (the same form as with more rows, see zmi_gemm_pergroup_kernel)
    const float b = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, e_n) : 0.0f;
    zmi_set_f32_flush();
    ((uint16_t *)p.dst)[o] = (uint16_t)zmi_pack_bf16(zmi_act_bf16_kind(epi.fast_kind, __fadd_rn(y, b)), 0.0f);
    return;
  }
  if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
  if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, epi.dst_dt, o), epi.beta));
  const float bias = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, e_n) : 0.0f;
  zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_tail(epi, y, bias, e_row, e_n));
}

template <int CPW, int GPW, bool S4 = false>
static hipError_t pgd_launch(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq, hipStream_t stream,
                             const uint8_t *tiles_s4 = nullptr) {
  constexpr int G = PGD_WAVES * GPW, NCH = PGD_WAVES * CPW, RT = G <= 32 ? G : 16;
  constexpr size_t main_bytes = (size_t)NCH * 1024 > (size_t)RT * 2048 ? (size_t)NCH * 1024 : (size_t)RT * 2048;
  constexpr size_t smem = main_bytes + (size_t)G * 32 * 4 + (size_t)16 * G * 4;
  {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_decode_pergroup_kernel<CPW, GPW, S4>, (int)smem);
    if (e != hipSuccess) return e;
  }
  ZmiFusedQuant none = {};
  const dim3 grid((unsigned)(zmi_blob_npad(p.N) / 32) + (fq ? p.M : 0)), block(PGD_THREADS);
  hipLaunchKernelGGL((zmi_gemm_decode_pergroup_kernel<CPW, GPW, S4>), grid, block, smem, stream, p, epi, fq ? *fq : none,
                     tiles_s4);
  return hipGetLastError();
}

// the decode-shaped kernel serves: up to 16 rows, K = 512 * CPW (CPW in 1, 2, 4, 8), whole groups per wavefront
static bool pgd_fits(const ZmiProblem &p, int G, int *cpw, int *gpw) {
  if (p.M > 16 || p.K % 512 != 0 || p.K > 4096 || G % PGD_WAVES != 0) return false;
  const int c = p.K / 512, g = G / PGD_WAVES;
  // whole groups of 64 .. 512 k per wavefront slice, or groups of 32 (two per chunk)
  if (!(c == 1 || c == 2 || c == 4 || c == 8) || !((g <= c && c % g == 0) || g == 2 * c)) return false;
  *cpw = c; *gpw = g;
  return true;
}

bool zmi_pergroup_decode_shape(const ZmiProblem &p, int G) {
  int cpw, gpw;
  return pgd_fits(p, G, &cpw, &gpw) && !zmi_env(ZE_PERGROUP_GENERIC);
}

bool zmi_pergroup_group_size_ok(int64_t gs) { return gs > 0 && (gs % 64 == 0 || gs == 32 || gs == 16); }

bool zmi_pergroup_s4_shape(const ZmiProblem &p, int G) {
  int cpw, gpw;
  return pgd_fits(p, G, &cpw, &gpw) && cpw % 2 == 0 && !zmi_env(ZE_PERGROUP_GENERIC) && !zmi_env(ZE_NO_S4_STREAM);
}

hipError_t zmi_launch_gemm_pergroup(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq,
                                    hipStream_t stream, const uint8_t *tiles_s4) {
  const int G = epi.n_groups;
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || G <= 0 || p.K % G != 0) return hipErrorInvalidValue;
  const int gs = p.K / G;
  if (!zmi_pergroup_group_size_ok(gs)) return hipErrorInvalidValue;
  if (epi.src_scale_mode != ZMI_SS_GROUP_PTR || epi.wei_scale_mode != 3 || !p.src_scale_ptr || !p.wei_scale_ptr)
    return hipErrorInvalidValue;
  if (p.a_is_u8 || epi.has_zp || epi.gated_act) return hipErrorInvalidValue;   // symmetric s8 rows only
  if (p.lda % 16 != 0 || ((uintptr_t)p.A) % 16 != 0 || p.lda < p.K) return hipErrorInvalidValue;   // 16-byte row loads
  int cpw = 0, gpw = 0;
  if (tiles_s4 && zmi_pergroup_s4_shape(p, G) && pgd_fits(p, G, &cpw, &gpw)) {
    // 4-bit codes streamed as they are (W4A8 decode shapes)
    switch (cpw * 16 + gpw) {
    case 8 * 16 + 8: return pgd_launch<8, 8, true>(p, epi, fq, stream, tiles_s4);
    case 8 * 16 + 4: return pgd_launch<8, 4, true>(p, epi, fq, stream, tiles_s4);
    case 8 * 16 + 2: return pgd_launch<8, 2, true>(p, epi, fq, stream, tiles_s4);
    case 8 * 16 + 1: return pgd_launch<8, 1, true>(p, epi, fq, stream, tiles_s4);
    case 4 * 16 + 4: return pgd_launch<4, 4, true>(p, epi, fq, stream, tiles_s4);
    case 4 * 16 + 2: return pgd_launch<4, 2, true>(p, epi, fq, stream, tiles_s4);
    case 4 * 16 + 1: return pgd_launch<4, 1, true>(p, epi, fq, stream, tiles_s4);
    case 2 * 16 + 2: return pgd_launch<2, 2, true>(p, epi, fq, stream, tiles_s4);
    case 2 * 16 + 1: return pgd_launch<2, 1, true>(p, epi, fq, stream, tiles_s4);
    case 8 * 16 + 16: return pgd_launch<8, 16, true>(p, epi, fq, stream, tiles_s4);
    case 4 * 16 + 8: return pgd_launch<4, 8, true>(p, epi, fq, stream, tiles_s4);
    case 2 * 16 + 4: return pgd_launch<2, 4, true>(p, epi, fq, stream, tiles_s4);
    default: break;
    }
  }
  if (pgd_fits(p, G, &cpw, &gpw) && !zmi_env(ZE_PERGROUP_GENERIC)) {
    switch (cpw * 16 + gpw) {
    case 8 * 16 + 8: return pgd_launch<8, 8>(p, epi, fq, stream);
    case 8 * 16 + 4: return pgd_launch<8, 4>(p, epi, fq, stream);
    case 8 * 16 + 2: return pgd_launch<8, 2>(p, epi, fq, stream);
    case 8 * 16 + 1: return pgd_launch<8, 1>(p, epi, fq, stream);
    case 4 * 16 + 4: return pgd_launch<4, 4>(p, epi, fq, stream);
    case 4 * 16 + 2: return pgd_launch<4, 2>(p, epi, fq, stream);
    case 4 * 16 + 1: return pgd_launch<4, 1>(p, epi, fq, stream);
    case 2 * 16 + 2: return pgd_launch<2, 2>(p, epi, fq, stream);
    case 2 * 16 + 1: return pgd_launch<2, 1>(p, epi, fq, stream);
    case 1 * 16 + 1: return pgd_launch<1, 1>(p, epi, fq, stream);
    case 8 * 16 + 16: return pgd_launch<8, 16>(p, epi, fq, stream);
    case 4 * 16 + 8: return pgd_launch<4, 8>(p, epi, fq, stream);
    case 2 * 16 + 4: return pgd_launch<2, 4>(p, epi, fq, stream);
    case 1 * 16 + 2: return pgd_launch<1, 2>(p, epi, fq, stream);
    default: break;
    }
  }
  if (fq) return hipErrorInvalidValue;   // fused quantization exists for the decode-shaped kernel only
  const int n_cb = (int)(zmi_blob_npad(p.N) / 16);
  // 16-row blocks per wavefront: 32 rows keep four times as many wavefronts in flight as 64 and are faster up to
  // ~96 rows (M = 64, groups of 128 / 32: 48 -> 36 us, 105 -> 63 us); beyond that the weights' re-reads from L2 win
  const int rb = p.M <= 16 ? 1 : p.M <= 96 ? 2 : 4;
  const int n_rb = (p.M + 16 * rb - 1) / (16 * rb);
  const int n_items = n_cb * n_rb;
  const dim3 grid((n_items + PG_WAVES - 1) / PG_WAVES), block(PG_WAVES * 64);
  const int sub = gs >= 64 ? 1 : 64 / gs;
#define PG_LAUNCH(RB_, D_, SUB_, CPG_) \
  hipLaunchKernelGGL((zmi_gemm_pergroup_kernel<RB_, D_, SUB_, CPG_>), grid, block, 0, stream, p, epi, n_cb, n_items, gs)
  const int cpg = sub == 1 ? (gs == 64 ? 1 : gs == 128 ? 2 : 0) : 1;
  if (rb == 1) {
    if (sub == 2) PG_LAUNCH(1, 8, 2, 1); else if (sub == 4) PG_LAUNCH(1, 8, 4, 1);
    else if (cpg == 1) PG_LAUNCH(1, 8, 1, 1); else if (cpg == 2) PG_LAUNCH(1, 8, 1, 2); else PG_LAUNCH(1, 8, 1, 0);
  } else if (rb == 2) {
    if (sub == 2) PG_LAUNCH(2, 4, 2, 1); else if (sub == 4) PG_LAUNCH(2, 4, 4, 1);
    else if (cpg == 1) PG_LAUNCH(2, 4, 1, 1); else if (cpg == 2) PG_LAUNCH(2, 4, 1, 2); else PG_LAUNCH(2, 4, 1, 0);
  } else {
    if (sub == 2) PG_LAUNCH(4, 2, 2, 1); else if (sub == 4) PG_LAUNCH(4, 2, 4, 1);
    else if (cpg == 1) PG_LAUNCH(4, 2, 1, 1); else if (cpg == 2) PG_LAUNCH(4, 2, 1, 2); else PG_LAUNCH(4, 2, 1, 0);
  }
#undef PG_LAUNCH
  return hipGetLastError();
}

// ---- per-group dynamic quantization -----------------------------------------------------------
// Reference: the per-group symmetric kernels of the dynamic reorder
// (zendnnl/src/lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/
// per_group_avx512_f32_fma_kernel.cpp:78-86 scale, :276-292 quantization): per (row, group)
// absmax over finite values, scale = max(absmax, 1e-10) / 127 clamped to >= 1e-10,
// q = (int8) nearbyint(v / scale) with the true division, non-finite -> 0; i.e. the per-token
// rule applied to every group of a row.  One wavefront per (row, group).
template <bool BF16>
__global__ __launch_bounds__(256) void zmi_quant_groups_kernel(const void *x, int64_t ldx, int M, int K, int G, int8_t *q,
                                                               int64_t ldq, float *scales, void *user_scales,
                                                               int32_t user_dt) {
  const int lane = threadIdx.x % 64;
  const int64_t item = (int64_t)blockIdx.x * 4 + threadIdx.x / 64;   // one wavefront per (row, group)
  if (item >= (int64_t)M * G) return;
  const int m = (int)(item / G), g = (int)(item % G);
  const int gs = K / G;
  const int64_t base = (int64_t)m * ldx + (int64_t)g * gs;
  auto ld = [&](int k) { return BF16 ? zmi_bf16_to_f32(((const uint16_t *)x)[base + k]) : ((const float *)x)[base + k]; };
  // (groups of up to 256 elements stay in registers between the two passes)
  float keep[4];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = lane + 64 * i;
    keep[i] = k < gs ? ld(k) : 0.0f;
    const float a = fabsf(keep[i]);
    if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
  }
  for (int k = lane + 256; k < gs; k += 64) {
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
    // (the GEMM multiplies by the scale as the scale buffer's dtype holds it: see zmi_fused_scale_as_stored)
    scales[item] = user_dt == ZMI_DT_BF16 ? zmi_bf16_to_f32(zmi_f32_to_bf16_rne(s)) : s;
    if (user_scales) {
      if (user_dt == ZMI_DT_BF16) ((uint16_t *)user_scales)[item] = zmi_f32_to_bf16_rne(s);
      else ((float *)user_scales)[item] = s;
    }
  }
  if (!q) return;   // scales only
  int8_t *dst = q + (int64_t)m * ldq + (int64_t)g * gs;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = lane + 64 * i;
    if (k < gs) dst[k] = zmi_quant_elem(keep[i], s, inv);
  }
  for (int k = lane + 256; k < gs; k += 64) dst[k] = zmi_quant_elem(ld(k), s, inv);
}

hipError_t zmi_launch_quant_groups(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, int8_t *q,
                                   int64_t ldq, float *scales, void *user_scales, int32_t user_dt, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  if (G <= 0 || K % G != 0 || (x_dt != ZMI_DT_BF16 && x_dt != ZMI_DT_F32)) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((M * G + 3) / 4));
  if (x_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_groups_kernel<true>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q,
                       ldq, scales, user_scales, user_dt);
  else
    hipLaunchKernelGGL(zmi_quant_groups_kernel<false>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q,
                       ldq, scales, user_scales, user_dt);
  return hipGetLastError();
}

// ---- asymmetric dynamic quantization: u8 rows + s32 zero-points, per token (G == 1) or per group ----
// Reference: compute_asymmetric_scale_zp (zendnnl/src/lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/
// per_token_avx512_f32_fma_kernel.cpp:89-116; the per-group twin per_group_avx512_f32_fma_kernel.cpp:91-115) and the
// quantization loops (:636-680): min / max over the finite values of the row (slice), [0, 0] when there is none, a
// range of width 0 widened to 1, scale = (max - min) / 255 clamped to >= 1e-10, zp = round(-min / scale) in double
// (half away from zero, clamped to s32), q = clamp(nearbyint(v / scale) + zp, 0, 255) with the true division,
// non-finite elements -> 0.  One wavefront per (row, group).
template <bool BF16>
__global__ __launch_bounds__(256) void zmi_quant_asym_kernel(const void *x, int64_t ldx, int M, int K, int G, uint8_t *q,
                                                             int64_t ldq, float *scales, int32_t *zps, void *user_scales,
                                                             int32_t user_dt) {
  const int lane = threadIdx.x % 64;
  const int64_t item = (int64_t)blockIdx.x * 4 + threadIdx.x / 64;
  if (item >= (int64_t)M * G) return;
  const int m = (int)(item / G), g = (int)(item % G);
  const int gs = K / G;
  const int64_t base = (int64_t)m * ldx + (int64_t)g * gs;
  auto ld = [&](int k) { return BF16 ? zmi_bf16_to_f32(((const uint16_t *)x)[base + k]) : ((const float *)x)[base + k]; };
  const float inf = __uint_as_float(0x7f800000u);
  float lo = inf, hi = -inf;
  for (int k = lane; k < gs; k += 64) {
    const float v = ld(k);
    if ((__float_as_uint(v) & 0x7f800000u) != 0x7f800000u) {
      lo = fminf(lo, v);
      hi = fmaxf(hi, v);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, o));
    hi = fmaxf(hi, __shfl_xor(hi, o));
  }
  if (lo > hi) lo = hi = 0.0f;                       // (no finite value; finite bounds are finite by construction)
  if (hi <= lo) hi = __fadd_rn(lo, 1.0f);
  float s = __fdiv_rn(__fsub_rn(hi, lo), 255.0f);
  if (s < 1e-10f) s = 1e-10f;
  const double zd = round((double)(-lo) / (double)s);
  const int32_t zp = zd < -2147483648.0 ? (int32_t)0x80000000 : zd > 2147483647.0 ? 0x7fffffff : (int32_t)zd;
  if (lane == 0) {
    scales[item] = s;
    zps[item] = zp;
    if (user_scales && user_dt == ZMI_DT_BF16) ((uint16_t *)user_scales)[item] = zmi_f32_to_bf16_rne(s);
  }
  if (!q) return;
  uint8_t *dst = q + (int64_t)m * ldq + (int64_t)g * gs;
  for (int k = lane; k < gs; k += 64) {
    const float v = ld(k);
    uint8_t out = 0;
    if ((__float_as_uint(v) & 0x7f800000u) != 0x7f800000u) {
      float t = rintf(__fdiv_rn(v, s));
      t = fminf(fmaxf(t, -4e9f), 4e9f);
      const long long qq = (long long)t + (long long)zp;
      out = (uint8_t)(qq < 0 ? 0 : qq > 255 ? 255 : qq);
    }
    dst[k] = out;
  }
}

// scales: f32 {M,G} (the caller's buffer when its dtype is f32, else scratch with the bf16 copy going to user_scales)
hipError_t zmi_launch_quant_asym(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, uint8_t *q,
                                 int64_t ldq, float *scales, int32_t *zps, void *user_scales, int32_t user_dt,
                                 hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  if (G <= 0 || K % G != 0 || (x_dt != ZMI_DT_BF16 && x_dt != ZMI_DT_F32) || !scales || !zps) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((M * G + 3) / 4));
  if (x_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_asym_kernel<true>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q, ldq, scales,
                       zps, user_scales, user_dt);
  else
    hipLaunchKernelGGL(zmi_quant_asym_kernel<false>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q, ldq, scales,
                       zps, user_scales, user_dt);
  return hipGetLastError();
}

// The same quantization for the large-M per-group GEMM: s8 rows in MFMA fragment order (zmi_afrag_off), groups of
// 32, 64 or 128.  A lane owns 16 consecutive k of one row (one 32- or 64-byte run in, one 16-byte piece of a fragment
// out); lane l of a wavefront takes row l % 8 of its 8 rows and chunk l / 8 of its 8 chunks, so that the 8 rows of a
// chunk are 128 contiguous bytes of the fragment, and a group's 2, 4 or 8 lanes meet through cross-lane exchanges.
template <bool BF16>
__global__ __launch_bounds__(256) void zmi_quant_groups_frag_kernel(const void *x, int64_t ldx, int M, int K, int G,
                                                                    int8_t *q, int64_t k_pad, float *scales,
                                                                    void *user_scales, int32_t user_dt) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int gs = K / G, L = gs / 16;                 // lanes per group: 2, 4 or 8
  const int row = (blockIdx.y * 4 + wave) * 8 + lane % 8;
  const int chunk = blockIdx.x * 8 + lane / 8;
  const int k0 = chunk * 16;
  const bool live = row < M && k0 < K;               // (K is a multiple of 16 and of the group size)
  float v[16];
  if (live) {
    if (BF16) {
      const uint16_t *src = (const uint16_t *)x + (int64_t)row * ldx + k0;
      const v4i a = *(const v4i *)src, b = *(const v4i *)(src + 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float((uint32_t)a[j] << 16);
        v[2 * j + 1] = __uint_as_float((uint32_t)a[j] & 0xffff0000u);
        v[8 + 2 * j] = __uint_as_float((uint32_t)b[j] << 16);
        v[8 + 2 * j + 1] = __uint_as_float((uint32_t)b[j] & 0xffff0000u);
      }
    } else {
      const float *src = (const float *)x + (int64_t)row * ldx + k0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v4f t = *(const v4f *)(src + 4 * j);
        v[4 * j] = t[0]; v[4 * j + 1] = t[1]; v[4 * j + 2] = t[2]; v[4 * j + 3] = t[3];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = 0.0f;
  }
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const float a = fabsf(v[j]);
    if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
  }
  // the group's lanes are 8 apart: chunks (l / 8) of one aligned run of L
  for (int o = 8; o < 8 * L; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (!live) return;
  if ((lane / 8) % L == 0) {
    const int64_t item = (int64_t)row * G + k0 / gs;
    scales[item] = user_dt == ZMI_DT_BF16 ? zmi_bf16_to_f32(zmi_f32_to_bf16_rne(s)) : s;
    if (user_scales) {
      if (user_dt == ZMI_DT_BF16) ((uint16_t *)user_scales)[item] = zmi_f32_to_bf16_rne(s);
      else ((float *)user_scales)[item] = s;
    }
  }
  v4i o;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint32_t pk = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) pk |= ((uint32_t)(uint8_t)zmi_quant_elem(v[w * 4 + j], s, inv)) << (8 * j);
    o[w] = (int)pk;
  }
  *(v4i *)(q + zmi_afrag_off(row, k0, k_pad)) = o;
}

bool zmi_quant_groups_frag_ok(const void *x, int32_t x_dt, int64_t K, int64_t ldx, int64_t G) {
  if (G <= 0 || K % G != 0) return false;
  const int64_t gs = K / G, es = x_dt == ZMI_DT_BF16 ? 2 : 4;
  if (x_dt != ZMI_DT_BF16 && x_dt != ZMI_DT_F32) return false;
  return (gs == 32 || gs == 64 || gs == 128) && ((uintptr_t)x) % 16 == 0 && (ldx * es) % 16 == 0;
}

hipError_t zmi_launch_quant_groups_frag(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, int64_t G, int8_t *q,
                                        float *scales, void *user_scales, int32_t user_dt, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  if (!zmi_quant_groups_frag_ok(x, x_dt, K, ldx, G)) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((K / 16 + 7) / 8), (unsigned)((M + 31) / 32));
  if (x_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_groups_frag_kernel<true>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q,
                       zmi_blob_kpad(K), scales, user_scales, user_dt);
  else
    hipLaunchKernelGGL(zmi_quant_groups_frag_kernel<false>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, (int)G, q,
                       zmi_blob_kpad(K), scales, user_scales, user_dt);
  return hipGetLastError();
}

// ---- 4-bit tiles for the decode-shaped kernel --------------------------------------------------
// From the blob of widened s8 weights (every byte a code in -8 .. 7): per 32-column block, the 2 KiB of chunk
// 2c and of chunk 2c + 1 become one 2 KiB piece, high nibble = even chunk, low nibble = odd chunk.
__global__ __launch_bounds__(256) void zmi_s4_tiles_kernel(const uint8_t *blob, int64_t K, int64_t N, uint8_t *out) {
  const int64_t pairs = zmi_blob_kpad(K) / 128;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;      // 16-byte granule of the output
  const int64_t per_nb = pairs * 128;
  if (i >= per_nb * (zmi_blob_npad(N) / 32)) return;
  const int64_t nb = i / per_nb, r = i % per_nb, cp = r / 128, gq = r % 128;
  const uint8_t *src = blob + zmi_blob_tiles_off(N) + nb * zmi_blob_nb_stride(K) + cp * 4096 + gq * 16;
  const v4i hi = *(const v4i *)src, lo = *(const v4i *)(src + 2048);
  v4i o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = (int)((((uint32_t)hi[j] << 4) & 0xf0f0f0f0u) | ((uint32_t)lo[j] & 0x0f0f0f0fu));
  *(v4i *)(out + nb * zmi_s4_nb_stride(K) + cp * 2048 + gq * 16) = o;
}

hipError_t zmi_launch_s4_tiles(const uint8_t *blob, int64_t K, int64_t N, uint8_t *out, hipStream_t stream) {
  const int64_t n = (zmi_blob_kpad(K) / 128) * 128 * (zmi_blob_npad(N) / 32);
  hipLaunchKernelGGL(zmi_s4_tiles_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, blob, K, N, out);
  return hipGetLastError();
}
