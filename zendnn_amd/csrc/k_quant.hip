// Per-token symmetric dynamic quantization, bf16/f32 rows -> s8 rows + one f32
// scale per row.  HBM-bound: M*K*2 bytes read, M*K + 4M written.
//
// Arithmetic of the reference's dynamic_per_token_quant_bf16_s8_native
// (zendnnl/src/lowoha_operators/reorder/reorder_data_type/dynamic_quant_impl/
// per_token_avx512_f32_fma_kernel.cpp:207-303; scalar twin
// scalar_impl/dynamic_per_token_ref_kernel.cpp:70-96): absmax over the finite
// values of the row, scale = max(absmax, 1e-10) / 127 clamped to >= 1e-10,
// q = (int8) rint(v / scale) with a correctly rounded division, non-finite -> 0.
#include "zmi_device.h"
#include "zmi_launch.h"

#define QT_THREADS 256
#define QT_MAX_CHUNKS 8   // rows up to 256 * 8 * 8 = 16384 elements stay in registers

__device__ __forceinline__ float zmi_block_max(float v, float *red) {
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  const int w = threadIdx.x / 64;
  if (threadIdx.x % 64 == 0) red[w] = v;
  __syncthreads();
  float r = red[0];
  #pragma unroll
  for (int i = 1; i < QT_THREADS / 64; ++i) r = fmaxf(r, red[i]);
  __syncthreads();
  return r;
}


// dst + dst_off(k) is where element k of this row goes: k itself for K-contiguous
// rows, the fragment-major position otherwise (8 consecutive k starting at a
// multiple of 8 stay contiguous in both).
template <bool BF16>
__device__ __forceinline__ void zmi_quant_row(const void *srcv, int8_t *dst, int r_frag, int64_t frag_kpad,
                                              void *scale, int scale_dt, int K, float *red) {
  const int t = threadIdx.x;
  auto dst_off = [&](int k) -> int64_t { return frag_kpad ? zmi_afrag_off(r_frag, k, frag_kpad) : (int64_t)k; };
  const bool vec_ok = (K % 8 == 0) && (((uintptr_t)srcv) % 16 == 0) &&
                      (dst == nullptr || ((uintptr_t)dst) % 8 == 0);
  if (vec_ok && K <= QT_THREADS * 8 * QT_MAX_CHUNKS) {
    // 8 elements per thread per chunk, the row is held in registers between the passes
    float v[QT_MAX_CHUNKS][8];
    float amax = 0.0f;
    #pragma unroll
    for (int c = 0; c < QT_MAX_CHUNKS; ++c) {
      const int k = (c * QT_THREADS + t) * 8;
      if (k < K) {
        if (BF16) {
          v4i raw = *(const v4i *)((const uint16_t *)srcv + k);
          #pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[c][2 * j] = __uint_as_float(((uint32_t)raw[j]) << 16);
            v[c][2 * j + 1] = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
          }
        } else {
          const float4 *p = (const float4 *)((const float *)srcv + k);
          float4 a = p[0], b = p[1];
          v[c][0] = a.x; v[c][1] = a.y; v[c][2] = a.z; v[c][3] = a.w;
          v[c][4] = b.x; v[c][5] = b.y; v[c][6] = b.z; v[c][7] = b.w;
        }
        #pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float a = fabsf(v[c][j]);
          if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
        }
      }
    }
    amax = zmi_block_max(amax, red);
    if (amax < 1e-10f) amax = 1e-10f;
    float s = __fdiv_rn(amax, 127.0f);
    if (s < 1e-10f) s = 1e-10f;
    const float inv = __fdiv_rn(1.0f, s);
    if (t == 0) {
      if (scale_dt == ZMI_DT_BF16) *(uint16_t *)scale = zmi_f32_to_bf16_rne(s);
      else *(float *)scale = s;
    }
    if (!dst) return;
    #pragma unroll
    for (int c = 0; c < QT_MAX_CHUNKS; ++c) {
      const int k = (c * QT_THREADS + t) * 8;
      if (k < K) {
        __attribute__((aligned(8))) int8_t q[8];
        #pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = zmi_quant_elem(v[c][j], s, inv);
        *(uint2 *)(dst + dst_off(k)) = *(const uint2 *)q;
      }
    }
    return;
  }
  // generic path: any K, any alignment; the row is read twice
  float amax = 0.0f;
  for (int k = t; k < K; k += QT_THREADS) {
    float x = BF16 ? zmi_bf16_to_f32(((const uint16_t *)srcv)[k]) : ((const float *)srcv)[k];
    float a = fabsf(x);
    if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
  }
  amax = zmi_block_max(amax, red);
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (t == 0) {
    if (scale_dt == ZMI_DT_BF16) *(uint16_t *)scale = zmi_f32_to_bf16_rne(s);
    else *(float *)scale = s;
  }
  if (!dst) return;
  for (int k = t; k < K; k += QT_THREADS) {
    float x = BF16 ? zmi_bf16_to_f32(((const uint16_t *)srcv)[k]) : ((const float *)srcv)[k];
    dst[dst_off(k)] = zmi_quant_elem(x, s, inv);
  }
}

// One workgroup per row.  mats has n_mat entries (device memory when n_mat > 1,
// otherwise passed by value through mat0).
template <bool BF16>
__global__ __launch_bounds__(QT_THREADS) void zmi_quant_rows_kernel(ZmiQuantMat mat0,
                                                                    const ZmiQuantMat *mats, int n_mat,
                                                                    int scale_dt, int n_rows) {
  __shared__ float red[QT_THREADS / 64];
  // Workgroups are dealt round robin to the 8 XCDs, whose L2s are private.  Runs of 32 rows go to one XCD: in
  // fragment-major output 32 consecutive rows fill whole cache lines between them, 8 bytes per row and line,
  // and only one L2 can merge them before they go to memory.  (The grid is a multiple of 256.)
  const int xcd = blockIdx.x % 8, j = blockIdx.x / 8;
  const int row = (xcd + 8 * (j / 32)) * 32 + j % 32;
  if (row >= n_rows) return;
  ZmiQuantMat m = mat0;
  if (mats) {
    // find the matrix that owns this global row (row_start is ascending)
    int lo = 0, hi = n_mat - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) / 2;
      if (mats[mid].row_start <= row) lo = mid; else hi = mid - 1;
    }
    m = mats[lo];
  }
  const int r = row - m.row_start;
  if (r >= m.M) return;
  const size_t es = BF16 ? 2 : 4;
  const void *src = (const char *)m.src + (size_t)r * m.ld_src * es;
  int8_t *dst = m.dst ? (m.frag_kpad ? m.dst : m.dst + (size_t)r * m.ld_dst) : nullptr;
  void *sc = (char *)m.scale + (size_t)r * (scale_dt == ZMI_DT_BF16 ? 2 : 4);
  zmi_quant_row<BF16>(src, dst, r, m.frag_kpad, sc, scale_dt, m.K, red);
}

#define FR_THREADS 512
// Fragment-major destination, K a multiple of 16, 16-byte aligned rows: one
// workgroup per 8 rows.  Thread (r = t % 8, q = t / 8) owns the 16 consecutive k
// starting at 16 q + 1024 step, i.e. exactly one 16-byte chunk of the fragment
// layout, and the 8 threads of one q write 8 consecutive chunks (128 bytes).
// The rows are read twice (absmax, then quantize); the second read hits L2.
template <bool BF16, int FR_STEPS>
__global__ __launch_bounds__(FR_THREADS) void zmi_quant_frag8_kernel(ZmiQuantMat mat0, const ZmiQuantMat *mats, int n_mat,
                                                              int scale_dt) {
  __shared__ float red[FR_THREADS / 64][8];
  const int t = threadIdx.x, r8 = t % 8, q = t / 8;
  const int grp = blockIdx.x;                 // group of 8 rows in the launch's numbering
  ZmiQuantMat m = mat0;
  if (mats) {
    int lo = 0, hi = n_mat - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) / 2;
      if (mats[mid].row_start <= grp * 8) lo = mid; else hi = mid - 1;
    }
    m = mats[lo];
  }
  // row_start of every matrix is a multiple of 8 in this launch form
  const int r = grp * 8 - m.row_start + r8;
  bool live = r < m.M;
  const int K = m.K;
  const size_t es = BF16 ? 2 : 4;
  int64_t src_row = live ? r : 0;
  if (m.gather && live) {
    const int g = m.gather[r];
    live = g >= 0;
    src_row = live ? g / m.gather_div : 0;
  }
  const char *src = (const char *)m.src + (size_t)src_row * m.ld_src * es;
  // raw 32-byte (bf16) / 64-byte (f32) pieces -> 16 floats
  auto load_raw = [&](int k, v4i (&w)[4]) {
    if (BF16) {
      w[0] = *(const v4i *)(src + (size_t)k * 2);
      w[1] = *(const v4i *)(src + (size_t)k * 2 + 16);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = *(const v4i *)(src + (size_t)k * 4 + j * 16);
    }
  };
  auto unpack = [&](const v4i (&w)[4], float (&v)[16]) {
    if (BF16) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[8 * h + 2 * j] = __uint_as_float(((uint32_t)w[h][j]) << 16);
          v[8 * h + 2 * j + 1] = __uint_as_float(((uint32_t)w[h][j]) & 0xffff0000u);
        }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b) v[4 * j + b] = __int_as_float(w[j][b]);
    }
  };
  auto absmax16 = [&](const float (&v)[16], float amax) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float a = fabsf(v[j]);
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
    return amax;
  };
  auto quant_store = [&](const float (&v)[16], float s, float inv, int k) {
    v4i o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t w = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) w |= ((uint32_t)(uint8_t)zmi_quant_elem(v[4 * j + b], s, inv)) << (8 * b);
      o[j] = (int)w;
    }
    *(v4i *)(m.dst + zmi_afrag_off(r, k, m.frag_kpad)) = o;
  };
  // rows of up to FR_STEPS * FR_THREADS * 2 elements stay in registers between the two passes
  // (bf16 only: 8 registers per step; FR_STEPS is the smallest of 2 / 4 / 8 that holds the row,
  // so that short rows leave registers for more workgroups per CU); longer rows are read
  // twice, the second time from L2
  const bool in_regs = BF16 && K <= FR_STEPS * FR_THREADS * 2;
  v4i keep[FR_STEPS][2];
  float amax = 0.0f;
  if (live) {
    if (in_regs) {
#pragma unroll
      for (int st = 0; st < FR_STEPS; ++st) {
        const int k = q * 16 + st * (FR_THREADS * 2);
        if (k < K) {
          keep[st][0] = *(const v4i *)(src + (size_t)k * 2);
          keep[st][1] = *(const v4i *)(src + (size_t)k * 2 + 16);
        }
      }
#pragma unroll
      for (int st = 0; st < FR_STEPS; ++st) {
        const int k = q * 16 + st * (FR_THREADS * 2);
        if (k < K) {
          v4i w[4] = {keep[st][0], keep[st][1], keep[st][0], keep[st][1]};
          float v[16];
          unpack(w, v);
          amax = absmax16(v, amax);
        }
      }
    } else {
      for (int k = q * 16; k < K; k += FR_THREADS * 2) {
        v4i w[4];
        float v[16];
        load_raw(k, w);
        unpack(w, v);
        amax = absmax16(v, amax);
      }
    }
  }
  // the threads of one row inside a wavefront are 8 lanes apart
  amax = fmaxf(amax, __shfl_xor(amax, 8));
  amax = fmaxf(amax, __shfl_xor(amax, 16));
  amax = fmaxf(amax, __shfl_xor(amax, 32));
  if (t % 64 < 8) red[t / 64][r8] = amax;
  __syncthreads();
  amax = red[0][r8];
#pragma unroll
  for (int w = 1; w < FR_THREADS / 64; ++w) amax = fmaxf(amax, red[w][r8]);
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (!live) return;
  if (q == 0) {
    void *sc = (char *)m.scale + (size_t)r * (scale_dt == ZMI_DT_BF16 ? 2 : 4);
    if (scale_dt == ZMI_DT_BF16) *(uint16_t *)sc = zmi_f32_to_bf16_rne(s);
    else *(float *)sc = s;
  }
  if (!m.dst) return;
  if (in_regs) {
#pragma unroll
    for (int st = 0; st < FR_STEPS; ++st) {
      const int k = q * 16 + st * (FR_THREADS * 2);
      if (k < K) {
        v4i w[4] = {keep[st][0], keep[st][1], keep[st][0], keep[st][1]};
        float v[16];
        unpack(w, v);
        quant_store(v, s, inv, k);
      }
    }
  } else {
    for (int k = q * 16; k < K; k += FR_THREADS * 2) {
      v4i w[4];
      float v[16];
      load_raw(k, w);
      unpack(w, v);
      quant_store(v, s, inv, k);
    }
  }
}

// launches the 8-row kernel with the smallest register window that holds a row
template <bool BF16>
static void zmi_quant_frag8_launch(unsigned grid, hipStream_t stream, const ZmiQuantMat &m0, const ZmiQuantMat *mats,
                                   int n_mat, int scale_dt, int64_t k_max) {
  if (k_max <= 2 * FR_THREADS * 2)
    hipLaunchKernelGGL((zmi_quant_frag8_kernel<BF16, 2>), dim3(grid), dim3(FR_THREADS), 0, stream, m0, mats, n_mat, scale_dt);
  else if (k_max <= 4 * FR_THREADS * 2)
    hipLaunchKernelGGL((zmi_quant_frag8_kernel<BF16, 4>), dim3(grid), dim3(FR_THREADS), 0, stream, m0, mats, n_mat, scale_dt);
  else
    hipLaunchKernelGGL((zmi_quant_frag8_kernel<BF16, 8>), dim3(grid), dim3(FR_THREADS), 0, stream, m0, mats, n_mat, scale_dt);
}

static bool zmi_quant_frag8_ok(const void *src, int64_t K, int64_t ld_src, int32_t src_dt) {
  const int64_t es = src_dt == ZMI_DT_BF16 ? 2 : 4;
  return K % 16 == 0 && ((uintptr_t)src) % 16 == 0 && (ld_src * es) % 16 == 0;
}

hipError_t zmi_launch_quant_rows(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t ld_src,
                                 int8_t *dst, int64_t ld_dst, int64_t frag_kpad, void *scales, int32_t scale_dt,
                                 hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  ZmiQuantMat m;
  m.src = src; m.dst = dst; m.scale = scales; m.ld_src = ld_src; m.ld_dst = ld_dst;
  m.M = (int32_t)M; m.K = (int32_t)K; m.row_start = 0; m.frag_kpad = (int32_t)frag_kpad;
  m.gather = nullptr; m.gather_div = 1;
  // Up to a few thousand rows one workgroup per row wins, also for fragment-major output
  // (measured on MI355X, K = 4096: 4 .. 5 us per call less at 128 .. 1024 rows, 1 us less at
  // 2048); the wider stores of the 8-rows-per-workgroup kernel pay once the launch is large
  // (26000 rows x 1408: 40 us against 63 us).
  if (frag_kpad && M > 2048 && zmi_quant_frag8_ok(src, K, ld_src, src_dt)) {
    const unsigned grid = (unsigned)((M + 7) / 8);
    if (src_dt == ZMI_DT_BF16) zmi_quant_frag8_launch<true>(grid, stream, m, nullptr, 1, scale_dt, K);
    else zmi_quant_frag8_launch<false>(grid, stream, m, nullptr, 1, scale_dt, K);
    return hipGetLastError();
  }
  if (src_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_rows_kernel<true>, dim3((unsigned)((M + 255) / 256 * 256)), dim3(QT_THREADS), 0, stream, m,
                       (const ZmiQuantMat *)nullptr, 1, scale_dt, (int)M);
  else
    hipLaunchKernelGGL(zmi_quant_rows_kernel<false>, dim3((unsigned)((M + 255) / 256 * 256)), dim3(QT_THREADS), 0, stream, m,
                       (const ZmiQuantMat *)nullptr, 1, scale_dt, (int)M);
  return hipGetLastError();
}

bool zmi_quant_mat_frag8_ok(const ZmiQuantMat &m, int32_t src_dt) {
  return m.frag_kpad > 0 && zmi_quant_frag8_ok(m.src, m.K, m.ld_src, src_dt);
}

hipError_t zmi_launch_quant_group(const ZmiQuantMat *mats_dev, int n_mat, int64_t total_rows,
                                  int32_t src_dt, int32_t scale_dt, int rows8, hipStream_t stream) {
  if (total_rows <= 0) return hipSuccess;
  ZmiQuantMat m0 = {};
  if (rows8) {
    // every matrix is fragment-major, eligible for the 8-row kernel, and starts at a multiple of 8 rows
    const unsigned grid = (unsigned)((total_rows + 7) / 8);
    // (the row lengths live on the device: the widest register window serves them all)
    if (src_dt == ZMI_DT_BF16) zmi_quant_frag8_launch<true>(grid, stream, m0, mats_dev, n_mat, scale_dt, 1 << 30);
    else zmi_quant_frag8_launch<false>(grid, stream, m0, mats_dev, n_mat, scale_dt, 1 << 30);
    return hipGetLastError();
  }
  if (src_dt == ZMI_DT_BF16)
    hipLaunchKernelGGL(zmi_quant_rows_kernel<true>, dim3((unsigned)((total_rows + 255) / 256 * 256)), dim3(QT_THREADS), 0,
                       stream, m0, mats_dev, n_mat, scale_dt, (int)total_rows);
  else
    hipLaunchKernelGGL(zmi_quant_rows_kernel<false>, dim3((unsigned)((total_rows + 255) / 256 * 256)), dim3(QT_THREADS), 0,
                       stream, m0, mats_dev, n_mat, scale_dt, (int)total_rows);
  return hipGetLastError();
}

// Per-tensor dynamic scale (src_scale dims {1} / {1,1}): absmax over the whole
// tensor, then every row is quantized with that one scale (reference:
// zendnnl/src/lowoha_operators/reorder/lowoha_reorder_utils.cpp:724-761).  Two
// small kernels: a grid-wide max through an ordered-int atomicMax, then the
// element-wise quantization; scales[m] is filled for every row so the GEMM can
// treat the result as per-token.
template <bool BF16>
__global__ __launch_bounds__(QT_THREADS) void zmi_absmax_kernel(const void *src, int64_t M, int64_t K,
                                                                int64_t ld, unsigned int *amax_bits) {
  __shared__ float red[QT_THREADS / 64];
  const int64_t row = blockIdx.x;
  float amax = 0.0f;
  for (int64_t k = threadIdx.x; k < K; k += QT_THREADS) {
    float x = BF16 ? zmi_bf16_to_f32(((const uint16_t *)src)[row * ld + k]) : ((const float *)src)[row * ld + k];
    float a = fabsf(x);
    if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
  }
  amax = zmi_block_max(amax, red);
  // non-negative floats order like their bit patterns
  if (threadIdx.x == 0) atomicMax(amax_bits, __float_as_uint(amax));
}

template <bool BF16>
__global__ __launch_bounds__(QT_THREADS) void zmi_quant_tensor_kernel(const void *src, int64_t M, int64_t K,
                                                                      int64_t ld, int8_t *dst, int64_t ld_dst,
                                                                      int64_t frag_kpad, float *scales,
                                                                      const unsigned int *amax_bits) {
  const int64_t row = blockIdx.x;
  float amax = __uint_as_float(*amax_bits);
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (threadIdx.x == 0) scales[row] = s;
  if (!dst) return;
  for (int64_t k = threadIdx.x; k < K; k += QT_THREADS) {
    float x = BF16 ? zmi_bf16_to_f32(((const uint16_t *)src)[row * ld + k]) : ((const float *)src)[row * ld + k];
    dst[frag_kpad ? zmi_afrag_off(row, k, frag_kpad) : row * ld_dst + k] = zmi_quant_elem(x, s, inv);
  }
}

__global__ void zmi_zero_u32_kernel(unsigned int *p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

hipError_t zmi_launch_quant_tensor(const void *src, int32_t src_dt, int64_t M, int64_t K, int64_t ld_src,
                                   int8_t *dst, int64_t ld_dst, int64_t frag_kpad, float *scales,
                                   unsigned int *amax_scratch, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_zero_u32_kernel, dim3(1), dim3(64), 0, stream, amax_scratch, 1);
  if (src_dt == ZMI_DT_BF16) {
    hipLaunchKernelGGL(zmi_absmax_kernel<true>, dim3((unsigned)M), dim3(QT_THREADS), 0, stream, src, M, K,
                       ld_src, amax_scratch);
    hipLaunchKernelGGL(zmi_quant_tensor_kernel<true>, dim3((unsigned)M), dim3(QT_THREADS), 0, stream, src,
                       M, K, ld_src, dst, ld_dst, frag_kpad, scales, amax_scratch);
  } else {
    hipLaunchKernelGGL(zmi_absmax_kernel<false>, dim3((unsigned)M), dim3(QT_THREADS), 0, stream, src, M, K,
                       ld_src, amax_scratch);
    hipLaunchKernelGGL(zmi_quant_tensor_kernel<false>, dim3((unsigned)M), dim3(QT_THREADS), 0, stream, src,
                       M, K, ld_src, dst, ld_dst, frag_kpad, scales, amax_scratch);
  }
  return hipGetLastError();
}

// Fragment-major per-token quantization with a row gather: destination row r (of n_rows) takes
// source row gather[r] / gather_div of x; rows with gather[r] < 0 are left alone.
hipError_t zmi_launch_quant_gather(const void *x, int32_t x_dt, int64_t ldx, int64_t K, const int32_t *gather,
                                   int32_t gather_div, int64_t n_rows, int8_t *dst, int64_t frag_kpad, float *scales,
                                   hipStream_t stream) {
  if (n_rows <= 0) return hipSuccess;
  if (!zmi_quant_frag8_ok(x, K, ldx, x_dt) || !frag_kpad) return hipErrorInvalidValue;
  ZmiQuantMat m = {};
  m.src = x; m.dst = dst; m.scale = scales; m.ld_src = ldx; m.ld_dst = frag_kpad;
  m.M = (int32_t)n_rows; m.K = (int32_t)K; m.row_start = 0; m.frag_kpad = (int32_t)frag_kpad;
  m.gather = gather; m.gather_div = gather_div;
  const unsigned grid = (unsigned)((n_rows + 7) / 8);
  if (x_dt == ZMI_DT_BF16) zmi_quant_frag8_launch<true>(grid, stream, m, nullptr, 1, ZMI_DT_F32, K);
  else zmi_quant_frag8_launch<false>(grid, stream, m, nullptr, 1, ZMI_DT_F32, K);
  return hipGetLastError();
}
