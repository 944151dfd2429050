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
