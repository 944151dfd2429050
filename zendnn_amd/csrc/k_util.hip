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
