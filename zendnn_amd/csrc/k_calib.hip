// What this device sustains, measured with nothing in the way: the two denominators the
// kernels of this library are judged against besides the nominal peaks.
//   * zmi_calib_hbm_read: a kernel that only reads -- the decode kernels' launch shape (one
//     workgroup of 8 wavefronts per 128 KiB, 16 requests of 16 bytes per lane, all in flight),
//     over buffers the caller rotates so that every launch comes from HBM.  Launch to launch
//     between two events, like the decode benchmark, and as the span from the first
//     wavefront's start to the last one's end inside the kernel.
//   * zmi_calib_mfma_i8: a loop of nothing but v_mfma_i32_32x32x32_i8 on every compute unit,
//     with operands that are constant, or that change from one instruction to the next like the
//     operands of a GEMM on random int8 data do (what the multipliers toggle sets the power they
//     draw, and the shader clock follows the power).  Reports the rate and the average shader
//     clock over the loop (the shader-clock counter against the 100 MHz real-time counter).
// Nothing here is on the path of any LowOHA call; bench.py --calib is the caller.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <vector>

#include "zmi_device.h"

#define CALIB_API extern "C" __attribute__((visibility("default")))

namespace {

__device__ unsigned long long g_calib_ts[2 * 8192];
__device__ unsigned long long g_calib_clk[4 * 2048];

__global__ __launch_bounds__(512) void zmi_calib_read_kernel(const v4i *__restrict__ p, int *sink) {
  const unsigned long long t0 = wall_clock64();
  // wavefront w of the workgroup reads its own 16 KiB, 1 KiB per request
  const v4i *base = p + ((size_t)blockIdx.x * 512 * 16) + (threadIdx.x / 64) * 64 * 16 + threadIdx.x % 64;
  v4i v[16];
#pragma unroll
  for (int i = 0; i < 16; i++) v[i] = __builtin_nontemporal_load(base + (size_t)i * 64);
  v4i acc = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 16; i++) { acc[0] ^= v[i][0]; acc[1] ^= v[i][1]; acc[2] ^= v[i][2]; acc[3] ^= v[i][3]; }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) sink[0] = 1;   // (keeps the loads)
  __syncthreads();
  if (threadIdx.x == 0 && blockIdx.x < 8192) {
    g_calib_ts[blockIdx.x * 2] = t0;
    g_calib_ts[blockIdx.x * 2 + 1] = wall_clock64();
  }
}

// The same read with the launch shape as a parameter: `grid` workgroups of THREADS threads, every lane REQ requests of
// 16 bytes, all in flight (grid * THREADS * REQ * 16 bytes in all; workgroup b reads its own contiguous range).
template <int THREADS, int REQ>
__global__ __launch_bounds__(THREADS) void zmi_calib_read_shape_kernel(const v4i *__restrict__ p, int *sink) {
  const unsigned long long t0 = wall_clock64();
  const v4i *base = p + ((size_t)blockIdx.x * THREADS * REQ) + (threadIdx.x / 64) * 64 * REQ + threadIdx.x % 64;
  v4i v[REQ];
#pragma unroll
  for (int i = 0; i < REQ; i++) v[i] = __builtin_nontemporal_load(base + (size_t)i * 64);
  v4i acc = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < REQ; i++) { acc[0] ^= v[i][0]; acc[1] ^= v[i][1]; acc[2] ^= v[i][2]; acc[3] ^= v[i][3]; }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) sink[0] = 1;   // (keeps the loads)
  __syncthreads();
  if (threadIdx.x == 0 && blockIdx.x < 8192) {
    g_calib_ts[blockIdx.x * 2] = t0;
    g_calib_ts[blockIdx.x * 2 + 1] = wall_clock64();
  }
}

// 8 independent accumulators per wavefront; with VARY the operands of consecutive instructions differ
template <bool VARY>
__global__ __launch_bounds__(256) void zmi_calib_mfma_kernel(const v4i *__restrict__ operands, int iters, int *sink) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  v4i a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = operands[(VARY ? i : 0) * 64 + lane];
#pragma unroll
  for (int i = 0; i < 2; ++i) b[i] = operands[(4 + (VARY ? i : 0)) * 64 + lane];
  v16i acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0;
  const unsigned long long c0 = clock64(), r0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i % 4], b[i / 4], acc[i], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), r1 = wall_clock64();
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  if (s == 0x12345678) sink[0] = s;
  if (lane == 0 && wave == 0 && blockIdx.x < 2048) {
    g_calib_clk[blockIdx.x * 2] = c1 - c0;
    g_calib_clk[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

}  // namespace

// bufs: n_bufs device buffers of `bytes` bytes each (a multiple of 128 KiB), read in turn by `launches` launches
// after `warm` untimed ones on `stream`.  us_per_launch: between two events; span_us: first wavefront's start to
// the last one's end inside a launch, the largest of the 8 XCDs (their counters are not aligned with each other).
CALIB_API int32_t zmi_calib_hbm_read(void *const *bufs, int32_t n_bufs, uint64_t bytes, int32_t warm, int32_t launches,
                                     void *stream, float *us_per_launch, float *span_us) {
  if (!bufs || n_bufs <= 0 || bytes == 0 || bytes % (128 * 1024) != 0 || launches <= 0) return ZMI_FAILURE;
  hipStream_t st = (hipStream_t)stream;
  const int grid = (int)(bytes / (128 * 1024));
  int *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipMalloc(&sink, 256) != hipSuccess) return ZMI_FAILURE;
  bool ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
  for (int i = 0; ok && i < warm; ++i)
    hipLaunchKernelGGL(zmi_calib_read_kernel, dim3(grid), dim3(512), 0, st, (const v4i *)bufs[i % n_bufs], sink);
  ok = ok && hipStreamSynchronize(st) == hipSuccess && hipEventRecord(e0, st) == hipSuccess;
  for (int i = 0; ok && i < launches; ++i)
    hipLaunchKernelGGL(zmi_calib_read_kernel, dim3(grid), dim3(512), 0, st, (const v4i *)bufs[i % n_bufs], sink);
  float ms = 0.0f;
  ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
       hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
  if (ok && us_per_launch) *us_per_launch = ms * 1e3f / launches;
  if (ok && span_us) {
    const int n = grid < 8192 ? grid : 8192;
    std::vector<unsigned long long> ts(2 * (size_t)n);
    ok = hipMemcpyFromSymbol(ts.data(), HIP_SYMBOL(g_calib_ts), ts.size() * 8) == hipSuccess;
    double worst = 0.0;
    for (int x = 0; ok && x < 8; ++x) {
      unsigned long long a = ~0ull, b = 0;
      for (int i = x; i < n; i += 8) { a = std::min(a, ts[i * 2]); b = std::max(b, ts[i * 2 + 1]); }
      if (b > a) worst = std::max(worst, (double)(b - a) * 0.01);
    }
    *span_us = (float)worst;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  return ok ? ZMI_SUCCESS : ZMI_FAILURE;
}

// zmi_calib_hbm_read with the launch shape given: threads per workgroup (256, 512 or 1024) and requests per lane
// (8, 14 or 16); bytes must be a multiple of threads * requests * 16.  What the best shape reaches is the ceiling a
// streaming kernel can be held against; the shape of the default entry point is the decode kernels' own.
CALIB_API int32_t zmi_calib_hbm_read_shape(void *const *bufs, int32_t n_bufs, uint64_t bytes, int32_t threads, int32_t requests,
                                           int32_t warm, int32_t launches, void *stream, float *us_per_launch, float *span_us) {
  if (!bufs || n_bufs <= 0 || bytes == 0 || launches <= 0 || threads <= 0 || requests <= 0) return ZMI_FAILURE;
  const uint64_t per_wg = (uint64_t)threads * requests * 16;
  if (bytes % per_wg != 0) return ZMI_FAILURE;
  hipStream_t st = (hipStream_t)stream;
  const int grid = (int)(bytes / per_wg);
  int *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipMalloc(&sink, 256) != hipSuccess) return ZMI_FAILURE;
  bool ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
  bool known = true;
  auto launch = [&](const void *buf) {
    const v4i *p = (const v4i *)buf;
#define ZMI_CALIB_SHAPE(T, R) \
    if (threads == T && requests == R) { hipLaunchKernelGGL((zmi_calib_read_shape_kernel<T, R>), dim3(grid), dim3(T), 0, st, p, sink); return; }
    ZMI_CALIB_SHAPE(256, 8) ZMI_CALIB_SHAPE(256, 14) ZMI_CALIB_SHAPE(256, 16) ZMI_CALIB_SHAPE(512, 8) ZMI_CALIB_SHAPE(512, 14)
    ZMI_CALIB_SHAPE(512, 16) ZMI_CALIB_SHAPE(1024, 8) ZMI_CALIB_SHAPE(1024, 14) ZMI_CALIB_SHAPE(1024, 16)
#undef ZMI_CALIB_SHAPE
    known = false;
  };
  for (int i = 0; ok && known && i < warm; ++i) launch(bufs[i % n_bufs]);
  ok = ok && known && hipStreamSynchronize(st) == hipSuccess && hipEventRecord(e0, st) == hipSuccess;
  for (int i = 0; ok && i < launches; ++i) launch(bufs[i % n_bufs]);
  float ms = 0.0f;
  ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
       hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
  if (ok && us_per_launch) *us_per_launch = ms * 1e3f / launches;
  if (ok && span_us) {
    const int n = grid < 8192 ? grid : 8192;
    std::vector<unsigned long long> ts(2 * (size_t)n);
    ok = hipMemcpyFromSymbol(ts.data(), HIP_SYMBOL(g_calib_ts), ts.size() * 8) == hipSuccess;
    double worst = 0.0;
    for (int x = 0; ok && x < 8; ++x) {
      unsigned long long a = ~0ull, b = 0;
      for (int i = x; i < n; i += 8) { a = std::min(a, ts[i * 2]); b = std::max(b, ts[i * 2 + 1]); }
      if (b > a) worst = std::max(worst, (double)(b - a) * 0.01);
    }
    *span_us = (float)worst;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  return ok ? ZMI_SUCCESS : ZMI_FAILURE;
}

// One launch of `iters` x 8 MFMAs per wavefront on wgs_per_cu x (number of CUs) workgroups of 4 wavefronts.
// operands: 6 x 1 KiB of int8 operand fragments in device memory (what the caller puts there is what the multipliers see).
// tops: int8 operations (2 per multiply-add) per second / 1e12; shader_mhz: average shader clock inside the loop.
CALIB_API int32_t zmi_calib_mfma_i8(const void *operands, int32_t vary_operands, int32_t wgs_per_cu, int32_t iters,
                                    void *stream, float *tops, float *shader_mhz) {
  if (!operands || iters <= 0 || wgs_per_cu <= 0) return ZMI_FAILURE;
  hipStream_t st = (hipStream_t)stream;
  int dev = 0, n_cu = 256;
  if (hipGetDevice(&dev) != hipSuccess) return ZMI_FAILURE;
  (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
  const int grid = n_cu * wgs_per_cu;
  int *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipMalloc(&sink, 256) != hipSuccess) return ZMI_FAILURE;
  bool ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
  auto launch = [&](int n) {
    if (vary_operands) hipLaunchKernelGGL(zmi_calib_mfma_kernel<true>, dim3(grid), dim3(256), 0, st, (const v4i *)operands, n, sink);
    else hipLaunchKernelGGL(zmi_calib_mfma_kernel<false>, dim3(grid), dim3(256), 0, st, (const v4i *)operands, n, sink);
  };
  if (ok) launch(iters / 4 + 1);   // untimed
  ok = ok && hipStreamSynchronize(st) == hipSuccess && hipEventRecord(e0, st) == hipSuccess;
  if (ok) launch(iters);
  float ms = 0.0f;
  ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
       hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
  if (ok && tops) *tops = (float)(2.0 * 32 * 32 * 32 * 8.0 * iters * 4.0 * grid / (ms * 1e-3) / 1e12);
  if (ok && shader_mhz) {
    const int n = grid < 2048 ? grid : 2048;
    std::vector<unsigned long long> ck(2 * (size_t)n);
    ok = hipMemcpyFromSymbol(ck.data(), HIP_SYMBOL(g_calib_clk), ck.size() * 8) == hipSuccess;
    double c = 0.0, r = 0.0;
    for (int i = 0; ok && i < n; ++i) { c += (double)ck[i * 2]; r += (double)ck[i * 2 + 1]; }
    *shader_mhz = r > 0.0 ? (float)(c / r * 100.0) : 0.0f;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  return ok ? ZMI_SUCCESS : ZMI_FAILURE;
}
