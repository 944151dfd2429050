// Weight-only quantization: C[M,N] = epilogue(A[M,K] bf16 x dequant(W[K,N] 4-bit)), f32 accumulation on the bf16 MFMA.
//
// Reference: matmul_direct with a bf16 source, s4 / u4 weights and no dynamic_quant turns every 4-bit code into a bf16
// value once (cvt_int4_to_bf16, lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:43-139:
//   f = float(code); f = (f - zp) * scale, or (f - 8) * scale + zp for u4 codes with a bf16 zero-point;
//   w = bfloat16_t(f)), caches the bf16 matrix and runs a bf16 GEMM with f32 accumulation on it.  Here the weights stay
// 4-bit in memory (a quarter of the bf16 matrix, the bound of a decode-shaped call) and every workgroup makes the
// same bf16 values in registers, with f32 operations that round like the reference's, right before the MFMA.
//
// Tiles: [N/32][K/64] pieces of 1 KiB; lane l of a wavefront owns 16 bytes of a piece = 4 dwords, dword t holding the
// 8 codes (k = 64*kc + 16*t + 8*(l/32) + j, j = 0..7 from the low nibble up; n = 32*nb + l%32): the B operand of four
// v_mfma_f32_32x32x16_bf16 in a row, one coalesced 16-byte load per lane.
//
// Kernel: one workgroup per 32 columns (and per 32 * MT rows), its wavefronts take the K chunks in turn (kc = wave,
// wave + W, ...), each keeping 8 chunks of weights in flight; the wavefronts' f32 sums meet in LDS, then alpha / beta /
// bias / post-ops / store per element (compute_matmul, operators/matmul/matmul_ref_kernel.cpp:877-896 and the post-op
// loop after it).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "../../include/zmi_lowoha.h"
#include "zmi_device.h"
#include "zmi_launch.h"

typedef __bf16 woq_bf16x8 __attribute__((ext_vector_type(8)));
typedef float woq_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t woq_u32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------------- tiles
__global__ __launch_bounds__(256) void zmi_woq_tiles_kernel(const uint8_t *packed, int64_t K, int64_t N, int64_t ldb,
                                                            int transB, uint32_t *out, int64_t n_dwords) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_dwords) return;
  const int64_t nkc = (K + 63) / 64;
  const int t = (int)(i & 3), lane = (int)((i >> 2) & 63);
  const int64_t piece = i >> 8, kc = piece % nkc, nb = piece / nkc;
  const int64_t n = nb * 32 + (lane & 31), k0 = kc * 64 + t * 16 + (lane >> 5) * 8;
  uint32_t d = 0;
  if (n < N) {
    for (int j = 0; j < 8; ++j) {
      const int64_t k = k0 + j;
      if (k >= K) break;
      const int64_t idx = transB ? n * ldb + k : k * ldb + n;
      const uint32_t byte = packed[idx >> 1];
      d |= ((idx & 1) ? (byte >> 4) : (byte & 15u)) << (4 * j);
    }
  }
  out[i] = d;
}

hipError_t zmi_launch_woq_tiles(const void *packed, int64_t K, int64_t N, int64_t ldb, bool transB, uint32_t *out,
                                hipStream_t stream) {
  const int64_t n_dwords = zmi_woq_tiles_bytes(K, N) / 4;
  hipLaunchKernelGGL(zmi_woq_tiles_kernel, dim3((unsigned)((n_dwords + 255) / 256)), dim3(256), 0, stream,
                     (const uint8_t *)packed, K, N, ldb, transB ? 1 : 0, out, n_dwords);
  return hipGetLastError();
}

// Scales and zero-points as f32, one per K group and column ([n_groups][N]), whatever their type and granularity were:
// they belong to the weights and are kept with the tiles (the reference bakes them into its cached bf16 matrix).
__global__ __launch_bounds__(256) void zmi_woq_params_kernel(ZmiWoqParamSrc s, ZmiWoqParamSrc z, int64_t G, int64_t N,
                                                             float *sf, float *zf) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= G * N) return;
  const int64_t g = i / N, n = i % N;
  sf[i] = s.ptr ? zmi_ld_f32(s.ptr, s.dt, s.mode == 0 ? 0 : s.mode == 1 ? n : g * N + n) : s.val;
  zf[i] = z.ptr ? zmi_ld_f32(z.ptr, z.dt, z.mode == 0 ? 0 : z.mode == 1 ? n : g * N + n) : z.val;
}

hipError_t zmi_launch_woq_params(const ZmiWoqParamSrc &s, const ZmiWoqParamSrc &z, int64_t G, int64_t N, float *sf,
                                 float *zf, hipStream_t stream) {
  hipLaunchKernelGGL(zmi_woq_params_kernel, dim3((unsigned)((G * N + 255) / 256)), dim3(256), 0, stream, s, z, G, N, sf, zf);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------- GEMM
// Q: 0 = s4 codes, no zero-point; 1 = s4 codes with a zero-point; 2 = u4 codes, (code - zp) * scale;
//    3 = u4 codes, (code - 8) * scale + zp
// 8 codes of one dword -> 8 bf16 values.  Q = 1 takes the codes one by one (signed field, conversion, subtraction,
// multiplication).  The others go through the byte conversions: the even and the odd nibbles are spread over the bytes
// of two words, each byte converted exactly (s4 codes after flipping their top bits: code + 8); then
//   Q = 0: fma(code + 8, s, -8 s) -- the exact product code * s rounded once, which is the reference's multiplication
//          (-8 s is exact: a power of two);
//   Q = 2: (code - zp) * s as written;  Q = 3: fma(code, s, -8 s) = the rounded (code - 8) * s, then + zp.
// byte B of a word as f32 (the conversion instruction that names its byte: the compiler finds it only for byte 0
// once it knows that the bytes hold nibbles)
template <int B>
__device__ __forceinline__ float woq_byte_f32(uint32_t x) {
  float f;
  if (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(x));
  else if (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(x));
  else if (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(x));
  else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(x));
  return f;
}

template <int Q>
__device__ __forceinline__ woq_bf16x8 woq_dequant(uint32_t d, float s, float z) {
  uint32_t o[4];
  if (Q == 1) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      float f[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int j = 2 * jj + h;
        f[h] = __fmul_rn(__fsub_rn((float)((int)(d << (28 - 4 * j)) >> 28), z), s);
      }
      o[jj] = zmi_pack_bf16(f[0], f[1]);
    }
  } else {
    if (Q == 0) d ^= 0x88888888u;
    const uint32_t ev = d & 0x0f0f0f0fu, od = (d >> 4) & 0x0f0f0f0fu;
    const float c = __fmul_rn(s, -8.0f);
    // (round to nearest even; f32 subnormals count as zero in this mode, as in the reference's bfloat16_t(float))
    auto pair = [&](float f0, float f1) {
      float f[2] = {f0, f1};
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (Q == 0) f[h] = __builtin_fmaf(f[h], s, c);
        else if (Q == 2) f[h] = __fmul_rn(__fsub_rn(f[h], z), s);
        else f[h] = __fadd_rn(__builtin_fmaf(f[h], s, c), z);
      }
      return zmi_pack_bf16(f[0], f[1]);
    };
    o[0] = pair(woq_byte_f32<0>(ev), woq_byte_f32<0>(od));
    o[1] = pair(woq_byte_f32<1>(ev), woq_byte_f32<1>(od));
    o[2] = pair(woq_byte_f32<2>(ev), woq_byte_f32<2>(od));
    o[3] = pair(woq_byte_f32<3>(ev), woq_byte_f32<3>(od));
  }
  uint4 r = {o[0], o[1], o[2], o[3]};
  return __builtin_bit_cast(woq_bf16x8, r);
}

// The main loop below has no branches: a load under a branch makes the compiler wait for every load in flight where
// the paths meet.  Rows beyond M and chunks beyond K read an address that exists; rows beyond M are never stored and
// values of k beyond K are replaced by zeros (which also makes a whole chunk beyond K add nothing).
__device__ __forceinline__ uint4 woq_load_a(const ZmiWoqProblem &p, int row, int k) {
  const uint16_t *a = (const uint16_t *)p.A;
  row = min(row, p.M - 1);
  uint32_t e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int kk = min(k + j, p.K - 1);
    const uint32_t v = a[p.transA ? (int64_t)kk * p.lda + row : (int64_t)row * p.lda + kk];
    e[j] = k + j < p.K ? v : 0u;
  }
  uint4 r;
  r.x = e[0] | (e[1] << 16); r.y = e[2] | (e[3] << 16); r.z = e[4] | (e[5] << 16); r.w = e[6] | (e[7] << 16);
  return r;
}

template <int MT> struct WoqWaves { static constexpr int W = MT <= 2 ? 8 : 4; };

// GENERAL = false: rows read 16 bytes at a time, one scale per 64-value chunk (scale groups are multiples of 64, or
// there are none).  GENERAL = true: rows element by element (any stride, transposed sources, K not a multiple of 8),
// scales looked up per 8 values.
// NB: column blocks of 32 a workgroup multiplies with each row fragment (2: the rows cross L2 once per 64 columns)
template <int MT, int Q, bool GENERAL, int NB = 1>
__global__ __launch_bounds__(WoqWaves<MT>::W * 64, (MT == 1 && !GENERAL && NB == 1) ? 4 : 1) void zmi_gemm_woq_kernel(ZmiWoqProblem p, ZmiEpilogue epi) {
  constexpr int W = WoqWaves<MT>::W, U = 8;
  extern __shared__ float woq_red[];   // [W][NB][MT * 16][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m0 = blockIdx.y * 32 * MT, kh = lane >> 5, nblk = (p.N + 31) / 32;
  const int nkc = (p.K + 63) / 64;

  woq_f32x16 acc[NB][MT];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[b][i][r] = 0.0f;

  // Requests run ahead of their use: a wavefront's next 8 chunks of weights (the whole K up to 4096), and the rows and
  // scales of the chunk after the one being multiplied (loads come back in the order they were asked for, so a
  // chunk's rows are asked for before anything that is needed later).  Addresses are a base every lane shares (kept
  // in scalar registers) plus a 32-bit offset per lane that never changes.
  constexpr int RING = !GENERAL && MT <= 2 ? 2 : 1;
  constexpr int NS = GENERAL ? 4 : 1;
  uint4 wq[NB][U];
  float sw[RING][NS][NB], zw[RING][NS][NB];
  uint4 af[RING][4][MT];
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  // (a workgroup whose last block lies beyond N multiplies the last block that exists again and stores nothing of it)
  const char *wbase[NB];
  int nc[NB];
  uint32_t noff[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const int nb = min((int)blockIdx.x * NB + b, nblk - 1);
    wbase[b] = (const char *)p.tiles + (int64_t)nb * nkc * 1024;
    nc[b] = min(nb * 32 + (lane & 31), p.N - 1);
    noff[b] = nc[b] * 4;
  }
  const uint32_t woff = lane * 16;
  uint32_t aoff[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    // rows beyond M get an offset outside the buffer: such a lane reads zeros and asks memory for nothing
    const int row = m0 + 32 * i + (lane & 31);
    aoff[i] = row < p.M ? (uint32_t)((row * (int)p.lda + kh * 8) * 2) : 0x80000000u;
  }
  // the rows as a buffer of M * lda bf16 values (untyped, 32-bit offsets, range-checked)
  const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.A, 0, GENERAL ? 0 : p.M * (int)p.lda * 2, 0x00020000);
  auto load_weights = [&](int b, int kc) { return *(const uint4 *)(wbase[b] + (int64_t)min(kc, nkc - 1) * 1024 + woff); };
  // TAIL = false: every value of the chunk lies inside K
  auto load_rows = [&](auto tail, int slot, int kc) {
    constexpr bool TAIL = decltype(tail)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        if (GENERAL) {
          af[slot][t][i] = woq_load_a(p, m0 + 32 * i + (lane & 31), kc * 64 + t * 16 + kh * 8);
        } else {
          const int k0 = kc * 64 + t * 16;
          // (with the tail handling a lane whose 8 values lie beyond K reads the last 8 inside it instead)
          const woq_u32x4 rb = TAIL ? __builtin_amdgcn_raw_buffer_load_b128(arsrc, aoff[i] - kh * 16 + min(k0 + kh * 8, p.K - 8) * 2, 0, 0)
                                    : __builtin_amdgcn_raw_buffer_load_b128(arsrc, aoff[i], k0 * 2, 0);
          uint4 r = {rb[0], rb[1], rb[2], rb[3]};
          if (TAIL) {
            const bool in = k0 + kh * 8 < p.K;
            r.x = in ? r.x : 0u; r.y = in ? r.y : 0u; r.z = in ? r.z : 0u; r.w = in ? r.w : 0u;
          }
          af[slot][t][i] = r;
        }
      }
#pragma unroll
    for (int t = 0; t < NS; ++t) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (GENERAL) {
          const int64_t gi = (int64_t)min((kc * 64 + t * 16 + kh * 8) / p.group_size, p.n_groups - 1) * p.N + nc[b];
          sw[slot][t][b] = p.sf[gi];
          zw[slot][t][b] = Q == 0 ? 0.0f : p.zf[gi];
        } else {
          const int64_t go = (int64_t)min((kc * 64) / p.group_size, p.n_groups - 1) * p.N * 4;
          sw[slot][t][b] = *(const float *)((const char *)p.sf + go + noff[b]);
          zw[slot][t][b] = Q == 0 ? 0.0f : *(const float *)((const char *)p.zf + go + noff[b]);
        }
      }
    }
  };
  auto pass = [&](auto tail, int kc0) {
    constexpr bool TAIL = decltype(tail)::value;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kc = kc0 + u * W;
      // (a chunk beyond K that a pass without the tail handling asks for ahead is never multiplied)
      if (RING == 1) load_rows(tail, 0, kc);
      else load_rows(tail, (u + 1) % RING, TAIL ? kc + W : min(kc + W, nkc - 1));
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint4 w = wq[b][u];
        wq[b][u] = load_weights(b, kc + U * W);
        const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int ts = GENERAL ? t : 0;
          const woq_bf16x8 bv = woq_dequant<Q>(wd[t], sw[u % RING][ts][b], zw[u % RING][ts][b]);
#pragma unroll
          for (int i = 0; i < MT; ++i)
            acc[b][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(woq_bf16x8, af[u % RING][t][i]), bv, acc[b][i], 0, 0, 0);
        }
      }
    }
  };
  if (RING > 1) load_rows(std::true_type{}, 0, wave_s);
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int b = 0; b < NB; ++b) wq[b][u] = load_weights(b, wave_s + u * W);
  zmi_set_f32_flush();
  for (int kc0 = wave_s; kc0 < nkc; kc0 += U * W) {
    // a pass whose 8 chunks, and the chunk it asks for ahead, lie inside K (or beyond the last chunk) needs no tail handling
    const int last = kc0 + (U - 1) * W, ahead = kc0 + U * W;
    if (!GENERAL && (last + 1) * 64 <= p.K && ((ahead + 1) * 64 <= p.K || ahead >= nkc)) pass(std::false_type{}, kc0);
    else pass(std::true_type{}, kc0);
  }
  // back to IEEE subnormals for the element-wise tail (the mode the other kernels' tails run in)
  __builtin_amdgcn_s_setreg(1 | (4 << 6) | (1 << 11), 3);

#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) woq_red[(((wave * NB + b) * MT + i) * 16 + r) * 64 + lane] = acc[b][i][r];
  __syncthreads();
  for (int sidx = threadIdx.x; sidx < NB * MT * 16 * 64; sidx += W * 64) {
    const int ln = sidx & 63, r = (sidx >> 6) & 15, i = (sidx >> 10) % MT, b = sidx / (MT * 1024);
    const int nb = (int)blockIdx.x * NB + b;
    const int m = m0 + 32 * i + 8 * (r >> 2) + 4 * (ln >> 5) + (r & 3), n = nb * 32 + (ln & 31);
    if (m >= p.M || n >= p.N || nb >= nblk) continue;
    float y = woq_red[sidx];
#pragma unroll
    for (int w = 1; w < W; ++w) y = __fadd_rn(y, woq_red[w * NB * MT * 16 * 64 + sidx]);
    const int64_t o = (int64_t)m * p.ldc + n;
    if (epi.alpha != 1.0f) y = __fmul_rn(y, epi.alpha);
    if (epi.beta != 0.0f) y = __fadd_rn(y, __fmul_rn(zmi_ld_f32(p.dst, epi.dst_dt, o), epi.beta));
    // (-0 is the one value whose addition changes nothing, not even the sign of a zero)
    const float bv = p.bias ? zmi_ld_f32(p.bias, epi.bias_dt, n) : -0.0f;
    zmi_store(p.dst, epi.dst_dt, o, zmi_epilogue_tail(epi, y, bv, m, n));
  }
}

template <int MT, bool GENERAL>
static hipError_t woq_launch_q(const ZmiWoqProblem &p, const ZmiEpilogue &epi, int q, hipStream_t stream) {
  constexpr int W = WoqWaves<MT>::W;
  const int smem = W * MT * 16 * 64 * 4;
  const dim3 grid((unsigned)((p.N + 31) / 32), (unsigned)((p.M + 32 * MT - 1) / (32 * MT)));
  const void *f = q == 0 ? (const void *)zmi_gemm_woq_kernel<MT, 0, GENERAL> : q == 1 ? (const void *)zmi_gemm_woq_kernel<MT, 1, GENERAL>
                : q == 2 ? (const void *)zmi_gemm_woq_kernel<MT, 2, GENERAL> : (const void *)zmi_gemm_woq_kernel<MT, 3, GENERAL>;
  hipError_t e = zmi_func_smem_once(f, smem);
  if (e != hipSuccess) return e;
  switch (q) {
  case 0: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 0, GENERAL>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 1: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 1, GENERAL>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 2: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 2, GENERAL>), grid, dim3(W * 64), smem, stream, p, epi); break;
  default: hipLaunchKernelGGL((zmi_gemm_woq_kernel<MT, 3, GENERAL>), grid, dim3(W * 64), smem, stream, p, epi); break;
  }
  return hipGetLastError();
}

// two column blocks per workgroup: up to 32 rows on the fast build
static hipError_t woq_launch_nb2(const ZmiWoqProblem &p, const ZmiEpilogue &epi, int q, hipStream_t stream) {
  constexpr int W = WoqWaves<1>::W;
  const int smem = W * 2 * 16 * 64 * 4;
  const dim3 grid((unsigned)(((p.N + 31) / 32 + 1) / 2), 1);
  const void *f = q == 0 ? (const void *)zmi_gemm_woq_kernel<1, 0, false, 2> : q == 1 ? (const void *)zmi_gemm_woq_kernel<1, 1, false, 2>
                : q == 2 ? (const void *)zmi_gemm_woq_kernel<1, 2, false, 2> : (const void *)zmi_gemm_woq_kernel<1, 3, false, 2>;
  hipError_t e = zmi_func_smem_once(f, smem);
  if (e != hipSuccess) return e;
  switch (q) {
  case 0: hipLaunchKernelGGL((zmi_gemm_woq_kernel<1, 0, false, 2>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 1: hipLaunchKernelGGL((zmi_gemm_woq_kernel<1, 1, false, 2>), grid, dim3(W * 64), smem, stream, p, epi); break;
  case 2: hipLaunchKernelGGL((zmi_gemm_woq_kernel<1, 2, false, 2>), grid, dim3(W * 64), smem, stream, p, epi); break;
  default: hipLaunchKernelGGL((zmi_gemm_woq_kernel<1, 3, false, 2>), grid, dim3(W * 64), smem, stream, p, epi); break;
  }
  return hipGetLastError();
}

template <bool GENERAL>
static hipError_t woq_launch_m(const ZmiWoqProblem &p, const ZmiEpilogue &epi, int q, hipStream_t stream) {
  if (p.M <= 32) return woq_launch_q<1, GENERAL>(p, epi, q, stream);
  if (p.M <= 64) return woq_launch_q<2, GENERAL>(p, epi, q, stream);
  return woq_launch_q<4, GENERAL>(p, epi, q, stream);
}

static bool woq_general(const ZmiWoqProblem &p) { return !p.a_fast || (p.n_groups > 1 && p.group_size % 64 != 0); }

// Column blocks per workgroup.  More than a few rows and enough column blocks to give every CU a workgroup of two: the
// rows cross L2 half as often (M = 16, K = 4096, N = 14336: 16.5 -> 13.5 us).  ZMI_WOQ_BLOCKS=1 / 2 forces the choice
// where the two-block build exists (up to 32 rows, the fast build); the tests use it.
int zmi_woq_blocks(const ZmiWoqProblem &p) {
  if (woq_general(p) || p.M > 32) return 1;
  if (const char *env = zmi_env(ZE_WOQ_BLOCKS)) return std::atoi(env) == 2 ? 2 : 1;
  return p.M > 4 && (p.N + 31) / 32 >= 384 ? 2 : 1;
}

hipError_t zmi_launch_gemm_woq(const ZmiWoqProblem &p, const ZmiEpilogue &epi, hipStream_t stream) {
  if (p.M <= 0 || p.N <= 0 || p.K <= 0 || !p.A || !p.tiles || !p.sf || !p.zf || !p.dst || p.group_size <= 0 ||
      p.n_groups <= 0 || (p.n_groups > 1 && (p.group_size % 8 != 0 || (int64_t)p.group_size * p.n_groups != p.K)) ||
      (p.a_fast && (p.transA || p.K % 8 != 0 || p.K < 64 || p.lda % 8 != 0 || ((uintptr_t)p.A & 15) != 0 ||
                    (int64_t)p.M * p.lda >= ((int64_t)1 << 30))) ||
      (p.M + 127) / 128 > 65535)
    return hipErrorInvalidValue;
  const int q = p.is_u4 ? (p.zp_float_domain ? 3 : 2) : (p.has_zp ? 1 : 0);
  if (p.is_u4 && !p.has_zp) return hipErrorInvalidValue;
  const bool general = woq_general(p);
  if (zmi_woq_blocks(p) == 2) return woq_launch_nb2(p, epi, q, stream);
  return general ? woq_launch_m<true>(p, epi, q, stream) : woq_launch_m<false>(p, epi, q, stream);
}
