// Decode int8 GEMM for gfx950: C[M<=128, N] = epilogue(A[M,K] x blob), K_pad <= 4096.
//
// Same call sites as k_smallm.hip (the aocl_gemm_s8s8s32o*_sym_quant call,
// zendnnl/src/lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:1239-1257, and the
// in-house decode microkernel, matmul/group_matmul/custom_kernel/ukernel/
// int8_microkernel.cpp:196-606), specialised for K_pad <= 4096 and built around the
// one-to-sixteen-token case, where the weights are streamed once from HBM and everything
// else has to stay out of the way of that stream:
//   * one workgroup (8 wavefronts) per 32 weight columns and up to RPW groups of 16 rows;
//     wavefront w streams the w-th eighth of K with 16-byte-per-lane loads, all issued up
//     front, and keeps its weights in registers for all its row groups; with more than
//     RPW row groups the workgroups of one column block are neighbours on one XCD, so
//     the weights leave HBM once and the others find them in that XCD's L2;
//   * the activation rows are read from L2 with row-contiguous loads (32 consecutive
//     lanes, 512 consecutive bytes) BEFORE the weight loads, so they return first,
//     and are laid out in LDS in MFMA operand order (bank-swizzled); the MFMA A
//     operands then come from LDS.  Loading the operands straight from global
//     memory instead touches 16 different rows per load and costs ~2 us of the
//     ~13 us launch.  Every wavefront stages exactly the slice of K it multiplies,
//     so there is no barrier between loading, staging and multiplying: with several
//     row groups the wavefronts drift apart and the address unit, the LDS and the
//     MFMA pipe work at the same time (in lock step a group of 16 rows cost 1.8 us
//     on a compute unit: 0.7 us of load issue, 0.55 us of LDS writes, 0.35 us of MFMAs);
//   * the per-column / per-row epilogue constants are fetched before anything
//     else, so the tail after the last weight byte is LDS-only;
//   * optionally the per-token quantization of the M source rows is part of the
//     launch: M extra workgroups at the head of the grid quantize one row each and publish it,
//     every workgroup puts three quarters of its weight stream in flight, waits for the
//     rows (the wait is bounded, producers wait for nothing and are dispatched
//     first), then requests the rows and the rest of the stream.
#include "zmi_device.h"
#include "zmi_fused_quant.h"
#include "zmi_launch.h"

#define DEC_WAVES 8
#define DEC_THREADS (DEC_WAVES * 64)
#ifndef DEC_FQ_FIRST
#define DEC_FQ_FIRST 6   // chunks of the slice requested before the wait for the quantized rows (measured best of 2, 4, 6, 8)
#endif
#define DEC_RED_BYTES (DEC_WAVES * 2 * 4 * 64 * 4)   // 16 KiB of partial tiles

// Byte offset in LDS of the 16-byte operand granule of chunk cc (64 k), k group g
// (16 k), row r.  Chunk-major so that one ds_read_b128 per lane fetches a whole
// 16x64 operand; the row index is XOR-swizzled with (g, cc) so that the
// row-contiguous writes (one row, 16 consecutive granules per 16 lanes) spread
// over all banks as well.
__device__ __forceinline__ int dec_lds_off(int cc, int g, int r) {
  return cc * 1024 + ((g * 16 + (r ^ ((g * 4 + (cc & 3)) & 15))) << 4);
}

template <int RPW>
__global__ __launch_bounds__(DEC_THREADS, (RPW == 1 ? 4 : 2)) void zmi_gemm_decode_kernel(ZmiProblem p, ZmiEpilogue epi,
                                                                                       ZmiFusedQuant fq, int n_blk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);   // scalar: slice bounds and addresses stay in SGPRs
  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nchunks = K_pad / 64;
  // With fused quantization the first M workgroups only quantize one source row each,
  // publish it and leave; the streaming workgroups follow them in dispatch order.
  if (fq.x && (int)blockIdx.x < M) {
    zmi_fused_quant_row(fq, blockIdx.x, K, reinterpret_cast<float *>(lds));
    zmi_fq_publish(fq, blockIdx.x);
    return;
  }
  // column block and rows: with at most RPW row groups the workgroup index is the column
  // block; with more, the indices (dealt round robin to the 8 XCDs) are renumbered so that
  // every XCD owns a contiguous range and the workgroups of a column block stay together
  const int n_rg = (M + 16 * RPW - 1) / (16 * RPW);
  int blk = fq.x ? (int)blockIdx.x - M : (int)blockIdx.x;
  int rg = 0;
  if (n_rg > 1) {
    const int per_xcd = (n_blk * n_rg + 7) / 8;
    const int id = (blk % 8) * per_xcd + blk / 8;
    if (blk / 8 >= per_xcd || id >= n_blk * n_rg) return;
    blk = id / n_rg;
    rg = id % n_rg;
  }
  const int r0 = rg * 16 * RPW;   // first row of this workgroup; row group j starts at r0 + 16 j
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());

  // the two 16-column groups h = 0, 1 of the block
  const int wcol[2] = {blk * 32, blk * 32 + 16};

  // ---- this thread's output element: (row tid/32, column tid%32) of every row group.  With rows that
  // are given, its epilogue constants are requested BEHIND the weights, as raw words (branch-free, decoded
  // after the reduction): ahead of them, every dependent wait would hold the weight stream back by a memory
  // round trip.  With the quantization inside the launch the column constants come first, as they always
  // did: measured, the streaming workgroups' late start is what lets the quantizing workgroups' own loads
  // and stores through (M = 16, N = 14336: 14.6 against 15.1 us per call; an idle wait of the same length
  // in their place: 15.5 .. 16.2 us) ----
  const int e_row = tid / 32;
  const int e_h = (tid % 32) / 16;
  const int e_c = tid % 16;
  const int e_n = wcol[e_h] + e_c;
  const bool e_col = e_n < N;
  const int n_ok = e_col ? e_n : N - 1;
  ZmiColRaw craw = {};
  int32_t zp_word = 0;
  uint32_t rs_word[RPW];
  auto load_consts = [&]() {
    craw = zmi_col_raw(epi, p, colsum, n_ok);
    zp_word = zmi_zp_raw(p, colsum);
    #pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = r0 + j * 16 + e_row;
      rs_word[j] = zmi_row_scale_raw(epi, p, colsum, m < M ? m : M - 1);
    }
  };
  ZmiColCtx cc_first = {};
  float rs_first[RPW];
  if (fq.x) cc_first = zmi_col_ctx(epi, p, colsum, e_col ? e_n : N, N);
  auto load_rs_first = [&]() {
    #pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = r0 + j * 16 + e_row;
      rs_first[j] = zmi_row_scale(epi, p, e_col && m < M ? m : 0);
    }
  };

  // ---- activation loads: every wavefront stages its own slice of K (at most 8 chunks = 32 granules
  // of 16 bytes per row) of the group's 16 rows, so no wavefront waits for another one: lanes 0..31
  // take one row, lanes 32..63 the next (512 contiguous bytes each) ----
  const int c_begin = wave * nchunks / DEC_WAVES;
  const int c_end = (wave + 1) * nchunks / DEC_WAVES;
  const int c16 = lane % 16, g = lane / 16;
  const int a_q = lane % 32;                      // granule of the slice
  const int a_gran = c_begin * 4 + a_q;           // granule of the row
  const bool a_live = a_q < (c_end - c_begin) * 4;
  // (two register sets when a workgroup has several row groups: the rows of group j + 2 are
  // requested while group j is multiplied, which covers their L2 latency)
  constexpr int NSET = RPW > 1 ? 2 : 1;
  v4i araw[NSET][8];
  auto load_row_pair = [&](int j, int i) {
    const int8_t *A = (const int8_t *)p.A;
    const int G = ((K + 15) & ~15) / 16;   // readable 16-byte granules per row
    const int row = r0 + j * 16 + 2 * i + lane / 32;
    v4i v = {0, 0, 0, 0};
    if (a_live && row < M && a_gran < G) v = *(const v4i *)(A + (int64_t)row * p.lda + a_gran * 16);
    araw[j % NSET][i] = v;
  };
  auto load_rows = [&](int j) {
    #pragma unroll
    for (int i = 0; i < 8; ++i) load_row_pair(j, i);
  };
  // rows -> LDS in operand order
  auto store_rows = [&](int j) {
    const uint32_t xm = p.a_is_u8 ? 0x80808080u : 0u;
    #pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 2 * i + lane / 32;
      v4i v = araw[j % NSET][i];
      v[0] ^= xm; v[1] ^= xm; v[2] ^= xm; v[3] ^= xm;
      if (r0 + j * 16 + row >= M) v = (v4i){0, 0, 0, 0};
      if (a_live) *(v4i *)(lds + dec_lds_off(a_gran / 4, a_gran % 4, row)) = v;
    }
  };

  // ---- weight stream: this wavefront's slice of K, at most 8 chunks of 64 ----
  const uint8_t *bsrc[2];
  #pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t nb = wcol[h] / 32;
    const int coff = wcol[h] % 32;
    bsrc[h] = tiles + nb * zmi_blob_nb_stride(K) + (g / 2) * 1024 + ((g % 2) * 32 + coff + c16) * 16;
  }
  v4i b[8][2];
  auto load_b = [&](int u) {
    // past the end of the slice: re-read the slice's first chunk (valid memory), result unused
    const int c = c_begin + u < c_end ? c_begin + u : c_begin;
    if (RPW == 1 && n_rg == 1) {
      // read by this workgroup only: the streaming hint keeps the weights from pushing the rows out of the caches
      // (M = 16, N = 14336: 13.0 against 14.2 us); with several workgroups per column block the others
      // find the weights in L2 and the hint costs (M = 128, N = K = 4096: 13.4 against 12.8 us)
      b[u][0] = __builtin_nontemporal_load((const v4i *)(bsrc[0] + (int64_t)c * 2048));
      b[u][1] = __builtin_nontemporal_load((const v4i *)(bsrc[1] + (int64_t)c * 2048));
    } else {
      b[u][0] = *(const v4i *)(bsrc[0] + (int64_t)c * 2048);
      b[u][1] = *(const v4i *)(bsrc[1] + (int64_t)c * 2048);
    }
  };

  if (!fq.x) {
    // rows first, so they return first; then the whole slice
    load_rows(0);
    #pragma unroll
    for (int u = 0; u < 8; ++u) load_b(u);
    if (RPW > 1 && r0 + 16 < M) load_rows(1);
    load_consts();
  } else {
    #pragma unroll
    for (int u = 0; u < DEC_FQ_FIRST; ++u) load_b(u);
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
    load_rs_first();   // (the row scales exist only now)
    load_rows(0);
    #pragma unroll
    for (int u = DEC_FQ_FIRST; u < 8; ++u) load_b(u);
    if (RPW > 1 && r0 + 16 < M) load_rows(1);
  }

  // ---- per row group: rows -> LDS, then one 16x16x64 MFMA per chunk and column group; the
  // rows of the group after the next are requested before the MFMAs of this one ----
  v4i acc[RPW][2];
  #pragma unroll
  for (int j = 0; j < RPW; ++j) {
    acc[j][0] = (v4i){0, 0, 0, 0};
    acc[j][1] = (v4i){0, 0, 0, 0};
    if (j > 0 && r0 + j * 16 >= M) continue;   // (uniform) no rows left for this group
    // (the wavefront reads back only what its own lanes wrote, and a wavefront's LDS accesses are
    // served in order: no workgroup barrier between the groups; the wavefront-scope fences emit
    // no instruction, they keep the compiler from reusing operands it read for the previous group)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    store_rows(j);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool ahead = j + 2 < RPW && r0 + (j + 2) * 16 < M;   // (uniform)
    #pragma unroll
    for (int u = 0; u < 8; ++u) {
      const bool live = c_begin + u < c_end;
      const int c = live ? c_begin + u : c_begin;
      v4i a = *(const v4i *)(lds + dec_lds_off(c, g, c16));
      if (!live) a = (v4i){0, 0, 0, 0};   // whatever b holds then adds nothing
      // one row request of the group after the next per chunk: the address unit takes 16
      // cycles per request and works under the MFMAs instead of ahead of them
      if (ahead) load_row_pair(j + 2, u);
      acc[j][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[u][0], acc[j][0], 0, 0, 0);
      acc[j][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[u][1], acc[j][1], 0, 0, 0);
    }
  }

  // ---- cross-wavefront reduction through LDS (reuses the operand area) ----
  __syncthreads();
  int32_t *red = (int32_t *)lds;
  #pragma unroll
  for (int j = 0; j < RPW; ++j)
    #pragma unroll
    for (int h = 0; h < 2; ++h)
      #pragma unroll
      for (int q = 0; q < 4; ++q) red[(wave * RPW + j) * 512 + (h * 4 + q) * 64 + lane] = acc[j][h][q];
  __syncthreads();
  if (!e_col) return;

  // acc[j][h][q] of lane l is row j*16 + (l/16)*4 + q, column h*16 + l%16
  auto fetch = [&](int j, int h) -> int32_t {
    const int off = j * 512 + (h * 4 + e_row % 4) * 64 + (e_row / 4) * 16 + e_c;
    int32_t s = 0;
    #pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) s += red[w * RPW * 512 + off];
    return s;
  };
  const ZmiColCtx cc0 = fq.x ? cc_first : zmi_col_ctx_raw(epi, p, craw, zp_word, e_n, n_ok, N);
  #pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int m = r0 + j * 16 + e_row;
    if (m >= M) break;
    const float rs = fq.x ? rs_first[j] : zmi_row_scale_from_raw(epi, p, rs_word[j], m);
    zmi_finish_element(p, epi, cc0, rs, fetch(j, e_h), m, e_n);
  }
}

// ---------------------------------------------------------------------------------------
// Up to 16 rows that are given as s8 / u8 (the decode step proper): nothing stands in front of the
// weight stream.  A wavefront's loads return in order and every compute unit works its requests off
// in order, so whatever is requested ahead of the weights with a dependent wait holds the stream
// back by a memory round trip.  Here every wavefront requests
//   1. the first two chunks of its weights (memory has work while the address unit, which takes 64
//      bytes per cycle whatever they are, works the row requests off),
//   2. the rows of its own slice of K by global->LDS loads (no registers, nothing waits for them),
//   3. the rest of its 16 KiB of weights, with the streaming hint (each byte is read once; without
//      the hint the weights push the rows out of the caches: 13.3 against 12.6 us at M = 16, N = 14336),
//   4. this thread's epilogue constants as raw words (branch-free, decoded after the reduction).
// There is no barrier in front of the MFMAs: a wavefront reads back only the rows it requested.
// Rows -> LDS: one global->LDS request per chunk of 64 k.  Lane l lands at byte 16 l of the
// chunk's 1 KiB; it fetches row l / 4, and four consecutive lanes fetch the row's 64 bytes of the
// chunk (one contiguous run per row) in the order k group (l % 4) ^ (row / 4 % 4): with that twist
// the MFMA's lanes (row l % 16, k group l / 16) read the 1 KiB back without bank conflicts.  Lanes
// of rows past M request nothing (their results are never stored, and fewer rows are fewer bytes
// through L2: 11.9 / 12.2 / 12.6 us at 1 / 8 / 16 rows); bytes past the readable end of a row meet
// zero weights and are fetched from the row's last 16 bytes.
// (Measured and dropped: the rows by helper wavefronts -- their requests end up behind the weights of
// the whole compute unit; at most 2 .. 6 chunks of weights in flight per wavefront; neighbouring
// workgroups starting at different slices of K; rows and weights requested alternately.)
// The value is in a vector register at this point of the program, and later uses read that register.
template <class T>
__device__ __forceinline__ void zmi_pin_v(T &x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void zmi_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// chunks of weights requested ahead of the rows (us per call with rows that are given, M = 16, N = 14336, whole-line
// row requests: 0 chunks 12.12, 2 chunks 12.38, 4 chunks 12.20, all 8 12.50)
#define D16_W_FIRST 0
// ... ahead of the wait for rows that are quantized inside the launch (us per call at M = 16, N = 14336, one box:
// 4 chunks 14.40, 5 chunks 14.17, 6 chunks 14.41, 7 chunks 14.68, all 8 14.67)
// (with whole-line row requests: 3 chunks 13.77, 4 chunks 13.75, 5 chunks 13.51, 6 chunks 13.72, all 8 14.19)
#define D16_FQ_FIRST 5

// K beyond 4096 (n_slices > 1, blockIdx.y = slice): the workgroups of a column block take up to 64 chunks of K each
// (their rows' share fits LDS as before) and leave their int32 sums in `partial` ([slice][16][N]); integers, so the
// order of the slices does not matter.  More workgroups at once is the point as much as the LDS: K = 14336,
// N = 4096 is 128 column blocks on 256 CUs (the kernel moves 4 .. 5 TB/s there, the split-K small-M kernel 2.3).
// With `arrivals` (a zeroed word per column block, zero again when the launch is over) the slice that arrives last
// at its column block's word adds the slices and finishes the elements itself: every slice writes its sums through
// to device scope (word stores that bypass the caches) and waits for their acknowledgement before it counts itself
// in, and the last one reads them with loads of the same scope.  No fence: a release fence at device scope writes
// back the whole L2, once per workgroup (90 us per call instead of 16).  Without `arrivals`
// zmi_decode16_reduce_kernel finishes the elements in a launch of its own (+2 us).
//
// FQ (= chunks of weights requested ahead of the wait, 0: rows that are given): the per-token quantization of
// bf16 / f32 rows is part of the launch (K up to 4096).  M workgroups at the head of the grid quantize one row each
// and stamp its flag (in every copy of the flag words); every other wavefront requests most of its weights, waits
// for the flags through the scalar unit (at a copy of its own: the waiters of the device spread over the copies'
// memory channels), then requests the rows, the rest of the weights and the constants.  The scalar unit's loads do not stand in the compute unit's queue of vector
// memory requests: behind the weight stream a vector load of the flags only returns with the stream (microseconds),
// which is why the row-group kernel holds a quarter of its weights back until its wait is over.  M = 16,
// N = 14336: 14.2 us per call against 15.9 us for the row-group kernel's form and 12.8 us with rows that are given.
// What is left of the difference (timestamps inside the kernel): the rows are published 5 us after the launch
// starts (2.4 us to read and quantize a row, 1.1 us until its stores are acknowledged, 1.5 us for the flag, all
// behind the weight requests of the workgroup that shares the compute unit), a waiting wavefront sees that 1 us
// later, and its row requests then stand at the end of its compute unit's queue: the last workgroups end 11.6 us
// after they started against 9.7 us.  Sixteen copies of the flags on different memory channels bring the end of the
// wait forward by 1.3 us, and with the rows then requested ahead of the last three chunks of weights the call takes
// 14.2 us (either change alone: nothing, or 0.3 us).
#ifdef D16_TIMING
// measurement build only: per workgroup, the constant-rate clock at its start, after its MFMAs and at its end
__device__ unsigned long long d16_times[16 * 1024];
extern "C" __attribute__((visibility("default"))) int zmi_debug_d16_times(unsigned long long *out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(d16_times), sizeof(d16_times));
}
#define D16_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < 1024) d16_times[blockIdx.x * 16 + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#define D16_STAMPW(i) do { if (threadIdx.x % 64 == 0 && blockIdx.x < 1024) d16_times[blockIdx.x * 16 + (i) + threadIdx.x / 64] = __builtin_amdgcn_s_memrealtime(); } while (0)
#else
#define D16_STAMP(i)
#define D16_STAMPW(i)
#endif

// PAIR (K a multiple of 1024, one slice): the rows are staged two chunks at a time, so that a request takes whole
// 128-byte lines of eight rows instead of 64-byte halves of sixteen.  Every workgroup of the launch reads the same
// rows at the same time, and it is the number of requests the L2 channels see in the launch's first microseconds,
// not their bytes, that holds the weight stream back (M = 16 against M = 4: +1.3 us with half lines).  A pair of
// chunks is 2 KiB of LDS: [rows 0..7 | rows 8..15][row][eight 16-byte slots], slot = (chunk % 2) * 4 + k group,
// stored at position slot ^ ((row >> 1) & 7) (the MFMA's reads of sixteen rows then spread over the banks).
template <int FQ, bool PAIR>
__global__ __launch_bounds__(DEC_THREADS, 4) void zmi_gemm_decode16_kernel(ZmiProblem p, ZmiEpilogue epi, ZmiFusedQuant fq,
                                                                           int n_slices, int32_t *partial,
                                                                           unsigned int *arrivals) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  D16_STAMP(0);
  // Every argument word the straight-line path reads, requested here in one batch: the compiler otherwise fetches
  // argument words where they are first used, one scalar load and one wait after the other -- two round trips ahead
  // of the first weight request and five behind the last barrier, a microsecond of the launch in all.
  // (one statement: the loads of all its operands are issued ahead of its one wait)
  asm volatile("" ::"s"(p.A), "s"(p.lda), "s"(p.blob), "s"(p.dst), "s"(p.ldc), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.a_is_u8),
               "s"(p.src_scale_ptr), "s"(p.wei_scale_ptr), "s"(p.src_zp_ptr), "s"(p.bias), "s"(p.src_scale_val),
               "s"(p.wei_scale_val), "s"(p.src_zp_val), "s"(p.row_comp), "s"(epi.src_scale_mode), "s"(epi.src_scale_dt),
               "s"(epi.wei_scale_mode), "s"(epi.wei_scale_dt), "s"(epi.has_zp), "s"(epi.bias_dt), "s"(epi.dst_dt),
               "s"(epi.fast_kind), "s"(n_slices));
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  int blk = (int)blockIdx.x;
  if (FQ) {
    if (blk < M) {   // (producers wait for nothing and are dispatched first)
      zmi_fused_quant_row(fq, blk, K, reinterpret_cast<float *>(lds));
      zmi_fq_publish(fq, blk, fq.n_copies);
      return;
    }
    blk -= M;
  }
  const int slice = (int)blockIdx.y;
  // this workgroup's chunks of 64 k (one slice: no division in front of the first request)
  int c0 = 0, nchunks = K_pad / 64;
  if (n_slices > 1) {
    c0 = (int)((unsigned)slice * (unsigned)(K_pad / 64) / (unsigned)n_slices);
    nchunks = (int)((unsigned)(slice + 1) * (unsigned)(K_pad / 64) / (unsigned)n_slices) - c0;
  }

  // one chunk of rows -> LDS
  const int G = ((K + 15) & ~15) / 16;      // readable 16-byte granules per row
  const int a_r = lane / 4;
  const uint32_t a_row_off = (uint32_t)a_r * (uint32_t)p.lda;
  const int a_kg = (lane % 4) ^ ((a_r >> 2) & 3);
  auto stage_chunk = [&](int c) {
    const int gran = c * 4 + a_kg;
    const uint32_t voff = a_row_off + (uint32_t)(gran < G ? gran : G - 1) * 16u;
    if (a_r < M)
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"((c - c0) * 1024), "v"(voff), "s"(p.A) : "memory", "m0");
  };

  const int c_begin = c0 + wave * nchunks / DEC_WAVES;
  const int c_end = c0 + (wave + 1) * nchunks / DEC_WAVES;
  // PAIR: chunks c_begin + 2 u and + 2 u + 1, rows 8 h .. 8 h + 7 (lane: row lane / 8, slot lane % 8)
  const int p_r = lane / 8;
  auto stage_pair = [&](int u, int h) {
    const int row = h * 8 + p_r;
    const int slot = (lane % 8) ^ ((row >> 1) & 7);
    const uint32_t voff = (uint32_t)row * (uint32_t)p.lda + (uint32_t)(c_begin + 2 * u) * 64u + (uint32_t)slot * 16u;
    if (row < M)
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"((c_begin - c0) * 1024 + u * 2048 + h * 1024), "v"(voff), "s"(p.A) : "memory", "m0");
  };
  auto stage_rows = [&]() {
    if (PAIR) {
      #pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c_begin + 2 * u < c_end) { stage_pair(u, 0); stage_pair(u, 1); }
    } else {
      #pragma unroll
      for (int u = 0; u < 8; ++u)
        if (c_begin + u < c_end) stage_chunk(c_begin + u);
    }
  };
  const int c16 = lane % 16, g = lane / 16;
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  const uint8_t *bsrc[2];
  #pragma unroll
  for (int h = 0; h < 2; ++h)
    bsrc[h] = tiles + (int64_t)blk * zmi_blob_nb_stride(K) + (g / 2) * 1024 + ((g % 2) * 32 + h * 16 + c16) * 16;
  v4i b[8][2];
  auto load_b = [&](int u) {
    // past the end of the slice: re-read the slice's first chunk (valid memory), result unused
    const int c = c_begin + u < c_end ? c_begin + u : c_begin;
    b[u][0] = __builtin_nontemporal_load((const v4i *)(bsrc[0] + (int64_t)c * 2048));
    b[u][1] = __builtin_nontemporal_load((const v4i *)(bsrc[1] + (int64_t)c * 2048));
  };
  bool rows_ok = true;
  if (!FQ) {
    #pragma unroll
    for (int u = 0; u < D16_W_FIRST; ++u) load_b(u);
    stage_rows();
    #pragma unroll
    for (int u = D16_W_FIRST; u < 8; ++u) load_b(u);
  } else {
    #pragma unroll
    for (int u = 0; u < FQ; ++u) load_b(u);
    // (every wavefront for itself: there is no barrier before the MFMAs; the copies of the flags are ZMI_FQ_COPIES
    // pages apart, so that the waiting wavefronts of the device do not all read one memory channel)
    rows_ok = zmi_fq_wait_scalar(fq, M, fq.flags + (fq.n_copies > 1 ? ((blk * DEC_WAVES + wave) % fq.n_copies) * 1024 : 0));
    if (rows_ok) stage_rows();
    #pragma unroll
    for (int u = FQ; u < 8; ++u) load_b(u);
  }
  // this thread's output element (row tid / 32, column tid % 32) and its constants, as raw words
  const int e_row = tid / 32, e_col = tid % 32;
  const int e_n = blk * 32 + e_col;
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int n_ok = e_n < N ? e_n : N - 1, m_ok = e_row < M ? e_row : M - 1;
  const ZmiColRaw craw = zmi_col_raw(epi, p, colsum, n_ok);
  const int32_t zp_word = zmi_zp_raw(p, colsum);
  const uint32_t rs_word = zmi_row_scale_raw(epi, p, colsum, m_ok);
  // requests complete in order: once the rows are in LDS, at most the weight requests that followed them
  // and the 5 constant words are outstanding
  if (FQ) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (8 - (FQ ? FQ : 8)) + 5) : "memory");
  else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (8 - D16_W_FIRST) + 5) : "memory");
  const uint32_t xm = p.a_is_u8 ? 0x80808080u : 0u;

  v4i acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  #pragma unroll
  for (int u = 0; u < 8; ++u) {
    const bool live = c_begin + u < c_end;
    const int c = live ? c_begin + u : c_begin;
    v4i a;
    if (PAIR) a = *(const v4i *)(lds + (c_begin - c0) * 1024 + (u / 2) * 2048 + (c16 / 8) * 1024 + (c16 % 8) * 128 +
                                 ((((u % 2) * 4 + g) ^ ((c16 >> 1) & 7))) * 16);
    else a = *(const v4i *)(lds + (c - c0) * 1024 + (c16 * 4 + (g ^ ((c16 >> 2) & 3))) * 16);
    a[0] ^= xm; a[1] ^= xm; a[2] ^= xm; a[3] ^= xm;   // u8 rows enter the MFMA as (a - 128)
    if (!live) a = (v4i){0, 0, 0, 0};   // whatever b holds then adds nothing
    acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[u][0], acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[u][1], acc[1], 0, 0, 0);
  }

  // the element's constants, decoded while the slower wavefronts of the workgroup still multiply
  ZmiColCtx cc0 = zmi_col_ctx_raw(epi, p, craw, zp_word, e_n, n_ok, N);
  float rs0 = zmi_row_scale_from_raw(epi, p, rs_word, m_ok);
  zmi_pin_v(cc0.wscale); zmi_pin_v(cc0.bias); zmi_pin_v(cc0.comp); zmi_pin_v(cc0.shift); zmi_pin_v(rs0);
  // ---- cross-wavefront reduction through LDS (reuses the operand area) ----
  D16_STAMPW(1);
  zmi_lds_barrier();
  int32_t *red = (int32_t *)lds;
  #pragma unroll
  for (int h = 0; h < 2; ++h)
    #pragma unroll
    for (int q = 0; q < 4; ++q) red[wave * 512 + (h * 4 + q) * 64 + lane] = acc[h][q];
  if (FQ && lane == 0) red[DEC_WAVES * 512 + wave] = rows_ok ? 1 : 0;
  zmi_lds_barrier();
  if (FQ) {   // a wavefront whose wait ran out staged no rows: the workgroup stores nothing
    int all = 1;
    #pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) all &= red[DEC_WAVES * 512 + w];
    if (!all) return;
  }
  const bool e_live = e_n < N && e_row < M;
  if (!e_live && !(n_slices > 1 && arrivals)) return;

  // acc[h][q] of lane l is row (l/16)*4 + q, column h*16 + l%16
  const int off = ((e_col / 16) * 4 + e_row % 4) * 64 + (e_row / 4) * 16 + e_col % 16;
  int32_t s = 0;
  #pragma unroll
  for (int w = 0; w < DEC_WAVES; ++w) s += red[w * 512 + off];
  D16_STAMP(9);
  if (n_slices > 1) {
    if (!arrivals) {
      if (e_live) partial[((int64_t)slice * 16 + e_row) * N + e_n] = s;
      return;
    }
    if (e_live) __hip_atomic_store(partial + ((int64_t)slice * 16 + e_row) * N + e_n, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    zmi_lds_barrier();                       // (also: everybody has read its sums out of `red`)
    if (tid == 0) {
      const unsigned int before = __hip_atomic_fetch_add(arrivals + blk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = before == (unsigned int)(n_slices - 1);
      if (last) __hip_atomic_store(arrivals + blk, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      red[0] = last ? 1 : 0;
    }
    zmi_lds_barrier();
    if (red[0] == 0 || !e_live) return;
    s = 0;   // (loads that bypass this CU's and this XCD's caches: what the other slices wrote through)
    for (int sl = 0; sl < n_slices; ++sl)
      s += __hip_atomic_load(partial + ((int64_t)sl * 16 + e_row) * N + e_n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  zmi_finish_element(p, epi, cc0, rs0, s, e_row, e_n);
  D16_STAMP(10);
}

// ---------------------------------------------------------------------------------------
// Up to 16 bf16 rows, quantized per token by the workgroups that use them: no second kind of workgroup, nothing
// handed from one workgroup to another, no wait.  A workgroup of 16 wavefronts owns TWO column blocks (wavefronts
// 0 .. 7 the even one, 8 .. 15 the odd one, each streaming an eighth of K of its block as in the 16-row kernel) and
// one copy of the rows in LDS: wavefront r requests bf16 row r first (it is there long before the weights), then all
// its weights, then the constants; while the weights are on their way it takes the row's absolute maximum (a
// wavefront reduction: a row is a wavefront's), quantizes the row with the arithmetic of k_quant.hip and writes the
// s8 bytes into LDS in the order the 16-row kernel's global->LDS loads leave them.  One barrier, then every wavefront
// multiplies its slice.  A compute unit holds one such workgroup: its 16 rows are fetched and quantized once per
// compute unit (half the row traffic of two 8-wavefront workgroups), about 450 VALU instructions per wavefront, all
// of them under the weight stream.  The scales go to the caller's buffer from workgroup 0 and to the epilogue
// through LDS.  (Measured times: at zmi_decode_selfq_takes.)
#define DQ_WAVES 16
#ifndef DQ_LATE
#define DQ_LATE 2
#endif
#define DQ_THREADS (DQ_WAVES * 64)
__global__ __launch_bounds__(DQ_THREADS, 1) void zmi_gemm_decode16_selfq_kernel(ZmiProblem p, ZmiEpilogue epi, ZmiFusedQuant fq,
                                                                              int n_blk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int half = wave / DEC_WAVES, w8 = wave % DEC_WAVES;
  const int M = p.M, N = p.N, K = p.K;
  const int K_pad = (int)zmi_blob_kpad(K);
  const int nchunks = K_pad / 64;
  const int blk_raw = (int)blockIdx.x * 2 + half;
  const bool blk_live = blk_raw < n_blk;
  const int blk = blk_live ? blk_raw : n_blk - 1;   // (an odd block count: the last workgroup's second half repeats a block, stores nothing)
  const int rows_bytes = nchunks * 1024;
  // LDS: the s8 rows (reused by the partial tiles) | DQ_LATE chunks of weights per wavefront | a scale per row
  const int wl_off = rows_bytes > 2 * DEC_RED_BYTES ? rows_bytes : 2 * DEC_RED_BYTES;
  float *rs_lds = reinterpret_cast<float *>(lds + wl_off + DQ_WAVES * DQ_LATE * 2048);

  // ---- requests, in this order (a wavefront's loads return in order, so the wait below can count): the column
  // constants of this thread's output element as raw words (4 loads, nothing waits for them early), this
  // wavefront's bf16 row (8 loads of a KiB), its weights (4 global->LDS requests, 12 loads into registers) ----
  const int t2 = tid % DEC_THREADS;
  const int e_row = t2 / 32, e_col = t2 % 32;
  const int e_n = blk * 32 + e_col;
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  const int n_ok = e_n < N ? e_n : N - 1;
  const ZmiColRaw craw = zmi_col_raw(epi, p, colsum, n_ok);
  const int32_t zp_word = zmi_zp_raw(p, colsum);
  const int c_begin = w8 * nchunks / DEC_WAVES;
  const int c_end = (w8 + 1) * nchunks / DEC_WAVES;
  const int c16 = lane % 16, g = lane / 16;
  const uint8_t *tiles = p.blob + zmi_blob_tiles_off(N);
  // The row comes FIRST in the wavefront's queue (loads return in order: behind a weight request it would arrive with
  // the weights, microseconds later on the compute units memory serves last) and by loads the compiler does not
  // count (inline assembly; the wait below is explicit and hands the registers on), so that the global->LDS
  // requests behind them do not turn the compiler's own waits for the row into waits for weights.
  asm volatile("" ::: "memory");
  const int NG = K / 8;                       // granules of 8 bf16 per row
  const bool row_live = wave < M;
  const uint16_t *xrow = (const uint16_t *)fq.x + (size_t)(row_live ? wave : 0) * fq.ldx;
  v4i xr[8];
  // (rows are 8 KiB apart and every workgroup wants the same ones at the same moment: each wavefront starts at a
  // different KiB of its row, or the requests of the whole device meet in one L2 channel after the other)
  const int rot = (wave + (int)blockIdx.x) & 7;
  #pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int gi = lane + 64 * ((i + rot) & 7);
    const uint32_t voff = (uint32_t)(gi < NG ? gi : NG - 1) * 16u;   // (past the row's end: its last granule, not written below)
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(xr[i]) : "v"(voff), "s"(xrow) : "memory");
  }
  asm volatile("" ::: "memory");
  const uint8_t *wbase = tiles + (int64_t)blk * zmi_blob_nb_stride(K);
  const uint32_t wlane = (uint32_t)((g / 2) * 1024 + ((g % 2) * 32 + c16) * 16);
  #pragma unroll
  for (int u = 8 - DQ_LATE; u < 8; ++u) {
    const int c = c_begin + u < c_end ? c_begin + u : c_begin;
    #pragma unroll
    for (int h = 0; h < 2; ++h)
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   ::"s"(wl_off + (wave * DQ_LATE + (u - (8 - DQ_LATE))) * 2048 + h * 1024),
                     "v"(wlane + (uint32_t)c * 2048u + (uint32_t)h * 256u), "s"(wbase)
                   : "memory", "m0");
  }
  asm volatile("" ::: "memory");
  const uint8_t *bsrc[2];
  #pragma unroll
  for (int h = 0; h < 2; ++h)
    bsrc[h] = tiles + (int64_t)blk * zmi_blob_nb_stride(K) + (g / 2) * 1024 + ((g % 2) * 32 + h * 16 + c16) * 16;
  // (128 registers per lane at 16 wavefronts: the row's 32 and 48 of weights; the last DQ_LATE chunks of the slice
  // land in LDS instead, global->LDS loads in the lanes' own order, and are read back as MFMA operands)
  v4i b[8 - DQ_LATE][2];
  #pragma unroll
  for (int u = 0; u < 8 - DQ_LATE; ++u) {
    const int c = c_begin + u < c_end ? c_begin + u : c_begin;   // (past the slice: a valid chunk, result unused)
    b[u][0] = __builtin_nontemporal_load((const v4i *)(bsrc[0] + (int64_t)c * 2048));
    b[u][1] = __builtin_nontemporal_load((const v4i *)(bsrc[1] + (int64_t)c * 2048));
  }

  // (behind the row: the 2 * DQ_LATE global->LDS requests and the 2 * (8 - DQ_LATE) register loads = 16)
  asm volatile("s_waitcnt vmcnt(16)"
               : "+v"(xr[0]), "+v"(xr[1]), "+v"(xr[2]), "+v"(xr[3]), "+v"(xr[4]), "+v"(xr[5]), "+v"(xr[6]), "+v"(xr[7])
               :: "memory");
  __builtin_amdgcn_sched_barrier(0);
  // maximum of the absolute values: the 15-bit patterns of |bf16| order like the values, so a packed 16-bit maximum
  // over the raw words does two elements per instruction; a result in the NaN / infinity range means the row holds
  // non-finite elements, which count as zero (in the maximum and below): they are zeroed in the registers, rarely
  typedef unsigned short dq_u16x2 __attribute__((ext_vector_type(2)));
  auto row_max = [&]() {
    dq_u16x2 m = {0, 0};
    #pragma unroll
    for (int i = 0; i < 8; ++i)
      #pragma unroll
      for (int j = 0; j < 4; ++j)
        m = __builtin_elementwise_max(m, __builtin_bit_cast(dq_u16x2, (uint32_t)xr[i][j] & 0x7fff7fffu));
    uint32_t v = m[0] > m[1] ? m[0] : m[1];
    #pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t t = (uint32_t)__shfl_xor((int)v, o);
      v = t > v ? t : v;
    }
    return v;
  };
  uint32_t mbits = row_max();
  if (mbits >= 0x7f80u) {   // (uniform)
    #pragma unroll
    for (int i = 0; i < 8; ++i)
      #pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t raw = (uint32_t)xr[i][j];
        if ((raw & 0x7f80u) == 0x7f80u) raw &= 0xffff0000u;
        if ((raw & 0x7f800000u) == 0x7f800000u) raw &= 0x0000ffffu;
        xr[i][j] = (int)raw;
      }
    mbits = row_max();
  }
  float amax = __uint_as_float(mbits << 16);
  if (amax < 1e-10f) amax = 1e-10f;
  float sc = __fdiv_rn(amax, 127.0f);
  if (sc < 1e-10f) sc = 1e-10f;
  const float inv = __fdiv_rn(1.0f, sc);
  if (lane == 0 && row_live) {
    rs_lds[wave] = zmi_fused_scale_as_stored(fq, sc);
    if (blockIdx.x == 0) {
      fq.scales[wave] = zmi_fused_scale_as_stored(fq, sc);
      if (fq.user_scales) {
        if (fq.user_dt == ZMI_DT_BF16) ((uint16_t *)fq.user_scales)[wave] = zmi_f32_to_bf16_rne(sc);
        else ((float *)fq.user_scales)[wave] = sc;
      }
    }
  }
  // the s8 bytes: x * (1 / scale) rounded, and the exact quotient for the elements whose product lies within 1e-4
  // of a half-integer (the arithmetic of zmi_quant_elem: one in a thousand, looked for once per eight elements)
  if (row_live) {
    const int r = wave;
    #pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int gi = lane + 64 * ((i + rot) & 7);
      uint32_t w2[2];
      #pragma unroll
      for (int hh = 0; hh < 2; ++hh) {   // (four elements at a time: the temporaries of eight do not fit the registers)
        // q + 128 as a float: x * (1 / scale) + 128 in one fused step, rounded.  That differs from x / scale + 128 by
        // less than 5e-5 (the product's 3.8e-5 and half a unit in the last place at 256), so away from the
        // half-integers the rounded value IS rint(x / scale) + 128, and within 1e-4 of one the exact quotient decides
        float x[4], t[4], q[4];
        bool redo = false;
        #pragma unroll
        for (int j = 0; j < 2; ++j) {
          x[2 * j] = __uint_as_float(((uint32_t)xr[i][hh * 2 + j]) << 16);
          x[2 * j + 1] = __uint_as_float(((uint32_t)xr[i][hh * 2 + j]) & 0xffff0000u);
        }
        #pragma unroll
        for (int e = 0; e < 4; ++e) {
          t[e] = __builtin_fmaf(x[e], inv, 128.0f);
          q[e] = rintf(t[e]);
          redo |= fabsf(t[e] - q[e]) > 0.4999f;
        }
        if (__builtin_expect(redo, 0)) {
          #pragma unroll
          for (int e = 0; e < 4; ++e)
            if (fabsf(t[e] - q[e]) > 0.4999f) q[e] = __fadd_rn(rintf(__fdiv_rn(x[e], sc)), 128.0f);
        }
        // (the hardware's float -> byte conversion inserts the byte; the values are whole numbers in 1 .. 255)
        uint32_t w = __builtin_amdgcn_cvt_pk_u8_f32(q[0], 0, 0);
        w = __builtin_amdgcn_cvt_pk_u8_f32(q[1], 1, w);
        w = __builtin_amdgcn_cvt_pk_u8_f32(q[2], 2, w);
        w = __builtin_amdgcn_cvt_pk_u8_f32(q[3], 3, w);
        w2[hh] = w ^ 0x80808080u;
        __builtin_amdgcn_sched_barrier(0);
      }
      // granule gi = 8 k: chunk gi / 8, 16-byte k group (gi % 8) / 2, its half gi % 2
      const int c = gi >> 3, kg = (gi & 7) >> 1;
      if (gi < NG) *(v2u *)(lds + c * 1024 + (r * 4 + (kg ^ ((r >> 2) & 3))) * 16 + (gi & 1) * 8) = (v2u){w2[0], w2[1]};
      __builtin_amdgcn_sched_barrier(0);   // (one granule at a time: interleaved, their temporaries do not fit the registers)
    }
  }
  // (k past K inside the last written chunks and rows past M: whatever LDS holds meets zero weights or rows that are not stored)
  zmi_lds_barrier();   // (long before the weights are there: every wavefront then waits for its own only)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  v4i acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  #pragma unroll
  for (int u = 0; u < 8; ++u) {
    const bool live = c_begin + u < c_end;
    const int c = live ? c_begin + u : c_begin;
    v4i a = *(const v4i *)(lds + c * 1024 + (c16 * 4 + (g ^ ((c16 >> 2) & 3))) * 16);
    if (!live) a = (v4i){0, 0, 0, 0};
    v4i b0, b1;
    if (u < 8 - DQ_LATE) {
      b0 = b[u][0];
      b1 = b[u][1];
    } else {
      const uint8_t *wl = lds + wl_off + (wave * DQ_LATE + (u - (8 - DQ_LATE))) * 2048 + lane * 16;
      b0 = *(const v4i *)wl;
      b1 = *(const v4i *)(wl + 1024);
    }
    acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b0, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b1, acc[1], 0, 0, 0);
  }

  // ---- cross-wavefront reduction through LDS (reuses the operand area; one 16 KiB area per half) ----
  const float rs = rs_lds[e_row < M ? e_row : 0];
  zmi_lds_barrier();
  int32_t *red = (int32_t *)lds + half * (DEC_RED_BYTES / 4);
  #pragma unroll
  for (int h = 0; h < 2; ++h)
    #pragma unroll
    for (int q = 0; q < 4; ++q) red[w8 * 512 + (h * 4 + q) * 64 + lane] = acc[h][q];
  zmi_lds_barrier();
  if (!(blk_live && e_n < N && e_row < M)) return;
  const int off = ((e_col / 16) * 4 + e_row % 4) * 64 + (e_row / 4) * 16 + e_col % 16;
  int32_t s = 0;
  #pragma unroll
  for (int w = 0; w < DEC_WAVES; ++w) s += red[w * 512 + off];
  const ZmiColCtx cc0 = zmi_col_ctx_raw(epi, p, craw, zp_word, e_n, n_ok, N);
  zmi_finish_element(p, epi, cc0, rs, s, e_row, e_n);
}


__global__ __launch_bounds__(256) void zmi_decode16_reduce_kernel(ZmiProblem p, ZmiEpilogue epi, int n_slices,
                                                                 const int32_t *partial) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int N = p.N;
  if (e >= (int64_t)p.M * N) return;
  const int row = (int)(e / N), n = (int)(e % N);
  int32_t s = 0;
  for (int sl = 0; sl < n_slices; ++sl) s += partial[((int64_t)sl * 16 + row) * N + n];
  const int32_t *colsum = (const int32_t *)(p.blob + zmi_blob_colsum_off());
  zmi_finish_element(p, epi, zmi_col_ctx(epi, p, colsum, n, N), zmi_row_scale(epi, p, row), s, row, n);
}

int zmi_decode_grid(const ZmiProblem &p) { return (int)(zmi_blob_npad(p.N) / 32); }

bool zmi_decode_kernel_fits(const ZmiProblem &p) {
  return p.M > 0 && p.M <= 128 && zmi_blob_kpad(p.K) <= 4096;
}

// K slices of the 16-row kernel for K beyond 4096 (0: the shape is not its: more than 16 rows, or rows it cannot address)
int zmi_decode16_slices(int M, int64_t K, int64_t lda) {
  const int64_t nchunks = zmi_blob_kpad(K) / 64;
  if (M <= 0 || M > 16 || nchunks <= 64 || lda * 16 >= ((int64_t)1 << 31) || zmi_env(ZE_DECODE_ROWGROUP_KERNEL)) return 0;
  return (int)((nchunks + 63) / 64);
}
size_t zmi_decode16_partial_bytes(int M, int N, int64_t K) {
  const int64_t nchunks = zmi_blob_kpad(K) / 64;
  return M <= 16 && nchunks > 64 ? (size_t)((nchunks + 63) / 64) * 16 * (size_t)N * sizeof(int32_t) : 0;
}

// Rows given as s8 / u8, at most 16 of them: the kernel without anything in front of the weight stream.
// (ZMI_DECODE_ROWGROUP_KERNEL: the tests reach the row-group kernel with few rows through it.)
bool zmi_decode_16row_kernel(const ZmiProblem &p, bool fused_quant) {
  (void)fused_quant;
  return p.M <= 16 && (int64_t)p.lda * 16 < ((int64_t)1 << 31) && !zmi_env(ZE_DECODE_ROWGROUP_KERNEL);
}

// bf16 rows quantized by the workgroups that use them (zmi_gemm_decode16_selfq_kernel): rows of whole 16-byte
// granules, K up to 4096, and a block count whose workgroups (two blocks each, one per compute unit) are all resident.
// Up to 12 rows: every compute unit quantizes all the rows (about 75 VALU instructions per 8 elements, 4 cycles
// each), and with a wavefront per row the work of 13 .. 16 rows is four wavefronts deep on every SIMD and no longer
// hides under the weight stream.  Measured, us per call (bf16 rows, K = 4096, rotating weights), this form / the
// hand-off through the scalar unit: N = 14336: 1 row 12.06 / 12.60, 4 rows 12.09 / 12.86, 8 rows 12.71 / 13.26,
// 12 rows 13.34 / 14.02, 16 rows 15.27 / 14.58; N = 11008: 1 row 10.36 / 11.72, 8 rows 10.63 / 12.23, 16 rows
// 13.60 / 13.57; N = 4096: 1 row 8.97 / 9.25, 16 rows 11.87 / 9.15.
// ZMI_NO_DECODE_SELFQ, ZMI_DECODE_SELFQ_MAX_M, ZMI_DECODE_SELFQ_MIN_WGS: the tests reach every form through them.
bool zmi_decode_selfq_takes(const ZmiProblem &p, const ZmiFusedQuant *fq) {
  if (!fq || !fq->x || fq->x_dt != ZMI_DT_BF16 || p.M > 16 || p.a_is_u8 || !zmi_decode_kernel_fits(p)) return false;
  if (p.K % 8 != 0 || ((uintptr_t)fq->x % 16) != 0 || (fq->ldx * 2) % 16 != 0) return false;
  const int wgs = (zmi_decode_grid(p) + 1) / 2;
  int min_wgs = 64, max_m = 12;
  if (const char *e = zmi_env(ZE_DECODE_SELFQ_MIN_WGS)) min_wgs = atoi(e);
  if (const char *e = zmi_env(ZE_DECODE_SELFQ_MAX_M)) max_m = atoi(e);
  return p.M <= max_m && wgs <= zmi_cu_count() && wgs >= min_wgs && !zmi_env(ZE_NO_DECODE_SELFQ) &&
         !zmi_env(ZE_DECODE_ROWGROUP_KERNEL);
}

hipError_t zmi_launch_gemm_decode(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq,
                                  hipStream_t stream, int32_t *partial, unsigned int *arrivals) {
  if (epi.gated_act != 0) return hipErrorInvalidValue;   // gated GEMMs are grouped launches: the large-M kernel
  const int n_blk = zmi_decode_grid(p);
  if (!zmi_decode_kernel_fits(p)) {
    // K beyond 4096: up to 16 given rows, in K slices
    const int slices = fq ? 0 : zmi_decode16_slices(p.M, p.K, p.lda);
    if (slices < 2 || !partial) return hipErrorInvalidValue;
    if (n_blk <= 0) return hipSuccess;
    const int64_t per = (zmi_blob_kpad(p.K) / 64 + slices - 1) / slices + 1;   // chunks of the longest slice, rounded up
    const size_t op = (size_t)(per < 64 ? per : 64) * 1024;
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_decode16_kernel<0, false>, 4096 * 16);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((zmi_gemm_decode16_kernel<0, false>), dim3(n_blk, slices), dim3(DEC_THREADS),
                       op > DEC_RED_BYTES ? op : DEC_RED_BYTES, stream, p, epi, ZmiFusedQuant{}, slices, partial, arrivals);
    e = hipGetLastError();
    if (e != hipSuccess || arrivals) return e;
    const int64_t elems = (int64_t)p.M * p.N;
    hipLaunchKernelGGL(zmi_decode16_reduce_kernel, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, stream, p, epi, slices,
                       partial);
    return hipGetLastError();
  }
  if (n_blk <= 0) return hipSuccess;
  ZmiFusedQuant none = {};
  if (zmi_decode_selfq_takes(p, fq)) {
    // (the s8 rows, reused by the two halves' partial tiles, and a scale per row)
    const size_t op = (size_t)zmi_blob_kpad(p.K) * 16;
    const size_t smem = (op > 2 * DEC_RED_BYTES ? op : 2 * DEC_RED_BYTES) + DQ_WAVES * DQ_LATE * 2048 + 64;
    hipError_t e = zmi_func_smem_once((const void *)zmi_gemm_decode16_selfq_kernel, 4096 * 16 + DQ_WAVES * DQ_LATE * 2048 + 64);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(zmi_gemm_decode16_selfq_kernel, dim3((n_blk + 1) / 2), dim3(DQ_THREADS), smem, stream, p, epi, *fq, n_blk);
    return hipGetLastError();
  }
  if (zmi_decode_16row_kernel(p, fq != nullptr) && (!fq || fq->flags_uncached)) {
    // (the operand area, reused by the partial tiles, and with the quantization in the launch a word per wavefront)
    const size_t op = (size_t)zmi_blob_kpad(p.K) * 16;
    const size_t smem = (op > DEC_RED_BYTES ? op : DEC_RED_BYTES) + (fq ? 64 : 0);
    // (whole lines of the rows per request where every wavefront's share of K is whole pairs of chunks)
    const bool pair = p.K % 1024 == 0 && !zmi_env(ZE_DECODE_NO_ROW_PAIRS);
    const void *f = fq ? (pair ? (const void *)zmi_gemm_decode16_kernel<D16_FQ_FIRST, true> : (const void *)zmi_gemm_decode16_kernel<D16_FQ_FIRST, false>)
                       : (pair ? (const void *)zmi_gemm_decode16_kernel<0, true> : (const void *)zmi_gemm_decode16_kernel<0, false>);
    hipError_t e = zmi_func_smem_once(f, 4096 * 16 + 64);
    if (e != hipSuccess) return e;
    const dim3 grid(n_blk + (fq ? p.M : 0)), block(DEC_THREADS);
    const ZmiFusedQuant q = fq ? *fq : ZmiFusedQuant{};
    if (fq && pair) hipLaunchKernelGGL((zmi_gemm_decode16_kernel<D16_FQ_FIRST, true>), grid, block, smem, stream, p, epi, q, 1, (int32_t *)nullptr, (unsigned int *)nullptr);
    else if (fq) hipLaunchKernelGGL((zmi_gemm_decode16_kernel<D16_FQ_FIRST, false>), grid, block, smem, stream, p, epi, q, 1, (int32_t *)nullptr, (unsigned int *)nullptr);
    else if (pair) hipLaunchKernelGGL((zmi_gemm_decode16_kernel<0, true>), grid, block, smem, stream, p, epi, q, 1, (int32_t *)nullptr, (unsigned int *)nullptr);
    else hipLaunchKernelGGL((zmi_gemm_decode16_kernel<0, false>), grid, block, smem, stream, p, epi, q, 1, (int32_t *)nullptr, (unsigned int *)nullptr);
    return hipGetLastError();
  }
  // rows per workgroup: 16 up to 64 rows (more workgroups in flight: 12 / 17 us per call at
  // 32 / 64 rows, N = K = 4096, against 13 / 20 us with 64); above that, 64 rows per workgroup
  // keep the weights in registers for four row groups (128 rows: 23 against 27 us)
  // (33 .. 64 rows whose one-group workgroups would not all be resident -- more than ~1000 of them -- also take the
  // four-group form: 48 / 64 rows at N = 14336: 27.0 / 30.2 against 28.1 / 32.3 us; 64 rows at K = 2048, N = 8192: 17.7
  // against 20.3 us; ZMI_DECODE_RPW = 1 | 4 overrides the choice above 16 rows)
  int rpw = p.M <= 64 ? 1 : 4;
  if (p.M > 32 && (int64_t)n_blk * ((p.M + 15) / 16) > 1000) rpw = 4;
  if (const char *e = zmi_env(ZE_DECODE_RPW)) { const int v = atoi(e); if ((v == 1 || v == 4) && p.M > 16) rpw = v; }
  const int n_rg = (p.M + 16 * rpw - 1) / (16 * rpw);
  // (several workgroups per column block: a multiple of 8, for the renumbering over the XCDs)
  const int grid = n_rg == 1 ? n_blk : (n_blk * n_rg + 7) / 8 * 8;
  // the operand area (16 rows x K_pad) is reused by the partial tiles (16 KiB per row group)
  const size_t a_bytes = (size_t)zmi_blob_kpad(p.K) * 16;
  const size_t r_bytes = (size_t)DEC_RED_BYTES * rpw;
  const size_t smem = a_bytes > r_bytes ? a_bytes : r_bytes;
  for (const void *f : {(const void *)zmi_gemm_decode_kernel<1>, (const void *)zmi_gemm_decode_kernel<4>}) {
    hipError_t e = zmi_func_smem_once(f, 4096 * 16);
    if (e != hipSuccess) return e;
  }
  const dim3 g3(grid + (fq ? p.M : 0)), b3(DEC_THREADS);
  if (rpw == 1) hipLaunchKernelGGL(zmi_gemm_decode_kernel<1>, g3, b3, smem, stream, p, epi, fq ? *fq : none, n_blk);
  else hipLaunchKernelGGL(zmi_gemm_decode_kernel<4>, g3, b3, smem, stream, p, epi, fq ? *fq : none, n_blk);
  return hipGetLastError();
}
