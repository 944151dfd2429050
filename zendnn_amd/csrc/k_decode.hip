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
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's write-through stores have landed ...
    __syncthreads();
    if (tid == 0) atomicAdd(fq.counter, 1u);           // ... before the row is published
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

  // ---- epilogue constants of this thread's output element, fetched first ----
  // element (row tid/32, column tid%32) of every row group
  const int e_row = tid / 32;
  const int e_h = (tid % 32) / 16;
  const int e_c = tid % 16;
  const int e_n = wcol[e_h] + e_c;
  const bool e_col = e_n < N;
  const ZmiColCtx cc0 = zmi_col_ctx(epi, p, colsum, e_col ? e_n : N, N);
  // (with fused quantization the row scales exist only after the wait below)
  float rs[RPW];
  auto load_rs = [&]() {
    #pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = r0 + j * 16 + e_row;
      rs[j] = zmi_row_scale(epi, p, e_col && m < M ? m : 0);
    }
  };
  if (!fq.x) load_rs();

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
    b[u][0] = *(const v4i *)(bsrc[0] + (int64_t)c * 2048);
    b[u][1] = *(const v4i *)(bsrc[1] + (int64_t)c * 2048);
  };

  if (!fq.x) {
    // rows first, so they return first; then the whole slice
    load_rows(0);
    #pragma unroll
    for (int u = 0; u < 8; ++u) load_b(u);
    if (RPW > 1 && r0 + 16 < M) load_rows(1);
  } else {
    #pragma unroll
    for (int u = 0; u < DEC_FQ_FIRST; ++u) load_b(u);
    if (tid == 0) {
      for (int spin = 0; spin < (1 << 22); ++spin) {
        const unsigned int v = __hip_atomic_load(fq.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((int)(v - fq.target) >= 0) break;
        __builtin_amdgcn_s_sleep(1);
      }
    }
    __syncthreads();
    asm volatile("" ::: "memory");   // the loads below stay below the wait
    load_rs();
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
  #pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int m = r0 + j * 16 + e_row;
    if (m >= M) break;
    zmi_finish_element(p, epi, cc0, rs[j], fetch(j, e_h), m, e_n);
  }
}

int zmi_decode_grid(const ZmiProblem &p) { return (int)(zmi_blob_npad(p.N) / 32); }

bool zmi_decode_kernel_fits(const ZmiProblem &p) {
  return p.M > 0 && p.M <= 128 && zmi_blob_kpad(p.K) <= 4096;
}

hipError_t zmi_launch_gemm_decode(const ZmiProblem &p, const ZmiEpilogue &epi, const ZmiFusedQuant *fq,
                                  hipStream_t stream) {
  if (!zmi_decode_kernel_fits(p)) return hipErrorInvalidValue;
  if (epi.gated_act != 0) return hipErrorInvalidValue;   // gated GEMMs are grouped launches: the large-M kernel
  const int n_blk = zmi_decode_grid(p);
  if (n_blk <= 0) return hipSuccess;
  // rows per workgroup: 16 up to 64 rows (more workgroups in flight: 12 / 17 us per call at
  // 32 / 64 rows, N = K = 4096, against 13 / 20 us with 64); above that, 64 rows per workgroup
  // keep the weights in registers for four row groups (128 rows: 23 against 27 us)
  // (33 .. 64 rows whose one-group workgroups would not all be resident -- more than ~1000 of them -- also take the
  // four-group form: 48 / 64 rows at N = 14336: 27.0 / 30.2 against 28.1 / 32.3 us; 64 rows at K = 2048, N = 8192: 17.7
  // against 20.3 us; ZMI_DECODE_RPW = 1 | 4 overrides the choice above 16 rows)
  int rpw = p.M <= 64 ? 1 : 4;
  if (p.M > 32 && (int64_t)n_blk * ((p.M + 15) / 16) > 1000) rpw = 4;
  if (const char *e = getenv("ZMI_DECODE_RPW")) { const int v = atoi(e); if ((v == 1 || v == 4) && p.M > 16) rpw = v; }
  const int n_rg = (p.M + 16 * rpw - 1) / (16 * rpw);
  // (several workgroups per column block: a multiple of 8, for the renumbering over the XCDs)
  const int grid = n_rg == 1 ? n_blk : (n_blk * n_rg + 7) / 8 * 8;
  // the operand area (16 rows x K_pad) is reused by the partial tiles (16 KiB per row group)
  const size_t a_bytes = (size_t)zmi_blob_kpad(p.K) * 16;
  const size_t r_bytes = (size_t)DEC_RED_BYTES * rpw;
  const size_t smem = a_bytes > r_bytes ? a_bytes : r_bytes;
  static bool attr_done = false;
  if (!attr_done) {
    for (const void *f : {(const void *)zmi_gemm_decode_kernel<1>, (const void *)zmi_gemm_decode_kernel<4>}) {
      hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 4096 * 16);
      if (e != hipSuccess) return e;
    }
    attr_done = true;
  }
  ZmiFusedQuant none = {};
  const dim3 g3(grid + (fq ? p.M : 0)), b3(DEC_THREADS);
  if (rpw == 1) hipLaunchKernelGGL(zmi_gemm_decode_kernel<1>, g3, b3, smem, stream, p, epi, fq ? *fq : none, n_blk);
  else hipLaunchKernelGGL(zmi_gemm_decode_kernel<4>, g3, b3, smem, stream, p, epi, fq ? *fq : none, n_blk);
  return hipGetLastError();
}
