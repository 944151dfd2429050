// Layout fix-ups that let the fast GEMM kernels assume 16-byte aligned,
// K-contiguous activation rows: copies A[M,K] (or its transpose) into a scratch
// buffer whose row stride is a multiple of 16, zero-filling the tail.
#include "zmi_device.h"
#include "zmi_launch.h"

__global__ __launch_bounds__(256) void zmi_pad_rows_kernel(const int8_t *src, int64_t M, int64_t K,
                                                           int64_t ld_src, int trans, int8_t *dst,
                                                           int64_t ld_dst) {
  const int64_t m = blockIdx.x;
  for (int64_t k = threadIdx.x; k < ld_dst; k += blockDim.x) {
    int8_t v = 0;
    if (k < K) v = trans ? src[k * ld_src + m] : src[m * ld_src + k];
    dst[m * ld_dst + k] = v;
  }
}

hipError_t zmi_launch_pad_rows(const void *src, int64_t M, int64_t K, int64_t ld_src, int trans,
                               int8_t *dst, int64_t ld_dst, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_pad_rows_kernel, dim3((unsigned)M), dim3(256), 0, stream, (const int8_t *)src, M, K,
                     ld_src, trans, dst, ld_dst);
  return hipGetLastError();
}

// Fragment-major copy for the large-M kernel: one workgroup per 32-row block and segment of
// RF_SEG_KB fragments along K (so that a few hundred rows already fill the device), one
// 16-byte chunk per thread and step, written in fragment order (coalesced).
#define RF_SEG_KB 16
__global__ __launch_bounds__(256) void zmi_repack_frag_kernel(const int8_t *src, int64_t M, int64_t K,
                                                              int64_t ld_src, int trans, int is_u8, int8_t *dst,
                                                              int64_t k_pad) {
  const int64_t fr = blockIdx.x;
  const int64_t kb_first = (int64_t)blockIdx.y * RF_SEG_KB;
  const int64_t kb_left = k_pad / 32 - kb_first;
  const int64_t chunks = (kb_left < RF_SEG_KB ? kb_left : RF_SEG_KB) * 64;
  for (int64_t idx = threadIdx.x; idx < chunks; idx += blockDim.x) {
    const int64_t kb = kb_first + idx / 64;
    const int l = (int)(idx % 64);
    const int64_t row = fr * 32 + l % 32;
    const int64_t k0 = kb * 32 + (l / 32) * 16;
    __attribute__((aligned(16))) int8_t v[16];
    if (!trans && row < M && k0 + 16 <= K && ((uintptr_t)(src + row * ld_src + k0)) % 16 == 0) {
      *(v4i *)v = *(const v4i *)(src + row * ld_src + k0);
    } else {
#pragma unroll
      for (int b = 0; b < 16; ++b) {
        const int64_t k = k0 + b;
        int8_t x = is_u8 ? (int8_t)0x80 : 0;   // becomes 0 after the shift
        if (row < M && k < K) x = trans ? src[k * ld_src + row] : src[row * ld_src + k];
        v[b] = x;
      }
    }
    v4i w = *(const v4i *)v;
    if (is_u8) { w[0] ^= 0x80808080; w[1] ^= 0x80808080; w[2] ^= 0x80808080; w[3] ^= 0x80808080; }
    *(v4i *)(dst + (fr * (k_pad / 32) + kb) * 1024 + l * 16) = w;
  }
}

hipError_t zmi_launch_repack_frag(const void *src, int64_t M, int64_t K, int64_t ld_src, int trans, int is_u8,
                                  int8_t *dst, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  const int64_t k_pad = zmi_blob_kpad(K);
  const unsigned segs = (unsigned)((k_pad / 32 + RF_SEG_KB - 1) / RF_SEG_KB);
  hipLaunchKernelGGL(zmi_repack_frag_kernel, dim3((unsigned)((M + 31) / 32), segs), dim3(256), 0, stream,
                     (const int8_t *)src, M, K, ld_src, trans, is_u8, dst, k_pad);
  return hipGetLastError();
}

// ---- GGML Q8_0 weights -> s8 rows [N, K] + bf16 scales {K / 32, N} ---------------------------------
// Reference: ggml_unpack_weight_buffer, Q8_0 branch
// (zendnnl/src/lowoha_operators/matmul/ggml_weight_unpack.cpp:190-236): the packed buffer is
// N * (K / 32) blocks of { fp16 d; int8 qs[32] } (34 bytes, row-major over [N][K / 32]); the int8 values are
// copied as they are and the scale of block (n, g) goes to scales[g * N + n], converted fp16 -> f32 -> bf16
// (round to nearest even, NaN quieted; :66-73) -- unpack_ggml_weights_and_cache asks for bf16 scales (:412-420).
__global__ __launch_bounds__(256) void zmi_ggml_q8_0_unpack_kernel(const uint8_t *blocks, int64_t N, int64_t K,
                                                                   int8_t *rows, uint16_t *scales) {
  const int64_t ng = K / 32;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;   // block index n * ng + g
  if (i >= N * ng) return;
  const int64_t n = i / ng, g = i % ng;
  const uint16_t *b = (const uint16_t *)(blocks + i * 34);     // 34-byte blocks: 2-byte aligned
  const uint16_t hb = b[0];
  const float d = (float)__builtin_bit_cast(_Float16, hb);   // exact (fp16 subnormals included)
  const uint32_t u = __float_as_uint(d);
  scales[g * N + n] = (u & 0x7fffffffu) > 0x7f800000u ? (uint16_t)((u >> 16) | 64u)
                                                       : (uint16_t)((u + (0x7fffu + ((u >> 16) & 1u))) >> 16);
  uint16_t *dst = (uint16_t *)(rows + n * K + g * 32);         // K % 32 == 0: even offsets
#pragma unroll
  for (int j = 0; j < 16; ++j) dst[j] = b[1 + j];
}

hipError_t zmi_launch_ggml_q8_0_unpack(const void *blocks, int64_t N, int64_t K, int8_t *rows, uint16_t *scales,
                                       hipStream_t stream) {
  if (N <= 0 || K <= 0 || K % 32 != 0) return hipErrorInvalidValue;
  const int64_t nb = N * (K / 32);
  hipLaunchKernelGGL(zmi_ggml_q8_0_unpack_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, stream,
                     (const uint8_t *)blocks, N, K, rows, scales);
  return hipGetLastError();
}

// ---- packed s4 weights -> s8, same orientation ------------------------------------------------------
// Reference: cvt_s4_to_s8 with extract_4bit_nibble
// (zendnnl/src/lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:33-41, 144-163): nibble i of the packed
// buffer (two per byte, even index = low nibble) is element i of a [rows, ld] matrix of 4-bit codes,
// sign-extended from bit 3.  The orientation is kept (rows x cols out of rows x ld), so consecutive threads
// read consecutive nibbles whichever way the weights lie; the prepack kernel transposes if it has to.
__global__ __launch_bounds__(256) void zmi_s4_widen_kernel(const uint8_t *packed, int64_t rows, int64_t cols, int64_t ld,
                                                           int8_t *out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;   // output element r * cols + c
  if (i >= rows * cols) return;
  const int64_t r = i / cols, c = i % cols;
  const int64_t idx = r * ld + c;
  const uint32_t byte = packed[idx >> 1];
  const int32_t nib = (idx & 1) ? (int32_t)(byte >> 4) : (int32_t)(byte & 15u);
  out[i] = (int8_t)((nib ^ 8) - 8);
}

hipError_t zmi_launch_s4_widen(const void *packed, int64_t rows, int64_t cols, int64_t ld, int8_t *out, hipStream_t stream) {
  if (rows <= 0 || cols <= 0 || ld < cols) return hipErrorInvalidValue;
  const int64_t n = rows * cols;
  hipLaunchKernelGGL(zmi_s4_widen_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                     (const uint8_t *)packed, rows, cols, ld, out);
  return hipGetLastError();
}

// ---- one scale per tensor / per row -> {M, G} f32 ---------------------------------------------------
// Reference: broadcast_w4a8_src_scale (backends/aocl/aocl_kernel.cpp:167-236): compact source scales are
// repeated over the G groups before the per-group GEMM.
__global__ __launch_bounds__(256) void zmi_broadcast_scales_kernel(const void *src, int32_t dt, int per_tensor, int64_t M,
                                                                  int64_t G, float *out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * G) return;
  const int64_t m = per_tensor ? 0 : i / G;
  out[i] = dt == ZMI_DT_BF16 ? __uint_as_float((uint32_t)((const uint16_t *)src)[m] << 16) : ((const float *)src)[m];
}

hipError_t zmi_launch_broadcast_scales(const void *src, int32_t dt, int per_tensor, int64_t M, int64_t G, float *out,
                                       hipStream_t stream) {
  if (M <= 0 || G <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(zmi_broadcast_scales_kernel, dim3((unsigned)((M * G + 255) / 256)), dim3(256), 0, stream, src, dt,
                     per_tensor, M, G, out);
  return hipGetLastError();
}

// ---- f32 scales -> the values a bf16 scale buffer holds ---------------------------------------------
// The reference narrows computed scales into the buffer's dtype and its GEMM reads them back
// (lowoha_operators/reorder/lowoha_reorder_utils.cpp:600-628): sc[i] becomes bf16(sc[i]) as f32 for i < n, and the
// first n_user narrowed values go to the caller's bf16 buffer when there is one.
__global__ __launch_bounds__(256) void zmi_narrow_scales_kernel(float *sc, int64_t n, uint16_t *user, int64_t n_user) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint16_t h = zmi_f32_to_bf16_rne(sc[i]);
  sc[i] = zmi_bf16_to_f32(h);
  if (user && i < n_user) user[i] = h;
}

hipError_t zmi_launch_narrow_scales(float *sc, int64_t n, void *user_bf16, int64_t n_user, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_narrow_scales_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, sc, n,
                     (uint16_t *)user_bf16, n_user);
  return hipGetLastError();
}


// ---- weight zero-point: one compensation word per source row ------------------------------------------
// row_comp[m] = -wei_zp * sum_k A[m, k] + src_zp * wei_zp * K in int32 (two's complement wrap), the source as the
// caller gave it (u8 / s8, row- or column-major).  Reference: cache_or_compute_zp_compensation,
// lowoha_operators/matmul/lru_cache/lowoha_cache.hpp:151-232 (its column term is the blob's colsum).  One wavefront per row.
__global__ __launch_bounds__(256) void zmi_row_comp_kernel(const void *A, int64_t lda, int transA, int is_u8, int M, int K,
                                                           int32_t wei_zp_val, const void *wei_zp_ptr, int32_t wei_zp_dt,
                                                           int32_t src_zp_val, const int32_t *src_zp_ptr, int32_t *out) {
  const int lane = threadIdx.x % 64;
  const int m = blockIdx.x * 4 + threadIdx.x / 64;
  if (m >= M) return;
  int32_t wz = wei_zp_val;
  if (wei_zp_ptr) wz = wei_zp_dt == ZMI_DT_S8 ? (int32_t)*(const int8_t *)wei_zp_ptr
                     : wei_zp_dt == ZMI_DT_U8 ? (int32_t)*(const uint8_t *)wei_zp_ptr : *(const int32_t *)wei_zp_ptr;
  const int32_t sz = src_zp_ptr ? *src_zp_ptr : src_zp_val;
  uint32_t sum = 0;
  for (int k = lane; k < K; k += 64) {
    const int64_t i = transA ? (int64_t)k * lda + m : (int64_t)m * lda + k;
    sum += is_u8 ? (uint32_t)((const uint8_t *)A)[i] : (uint32_t)(int32_t)((const int8_t *)A)[i];
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += (uint32_t)__shfl_xor((int)sum, o);
  if (lane == 0) out[m] = (int32_t)((uint32_t)sz * (uint32_t)wz * (uint32_t)K - (uint32_t)wz * sum);
}

hipError_t zmi_launch_row_comp(const void *A, int64_t lda, bool transA, bool is_u8, int M, int K, int32_t wei_zp_val,
                               const void *wei_zp_ptr, int32_t wei_zp_dt, int32_t src_zp_val, const int32_t *src_zp_ptr,
                               int32_t *out, hipStream_t stream) {
  if (M <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_row_comp_kernel, dim3((M + 3) / 4), dim3(256), 0, stream, A, lda, transA ? 1 : 0, is_u8 ? 1 : 0, M, K,
                     wei_zp_val, wei_zp_ptr, wei_zp_dt, src_zp_val, src_zp_ptr, out);
  return hipGetLastError();
}
