// Dynamic asymmetric quantization of a whole source tensor to u8 (one scale, one zero-point), the pre-pass of
// matmul_direct with dynamic_quant and a u8 compute type.
//
// Reference: reorder_quantization_wrapper (lowoha_operators/matmul/quantization/reorder_quantization.cpp:43-280) runs
// the reorder operator on the source; with scale and zero-point of one element each that is its per-tensor branch,
// lowoha_operators/reorder/lowoha_reorder_utils.cpp:708-813: min / max over the finite values ([0, 0] when there is
// none), max = min + 1 when max <= min, scale = (max - min) / 255, zp = round(-min / scale) in double (half away from
// zero, clamped to s32) with the scale as computed, then scale = max(scale, 1e-10); elements
// q = clamp(int32(nearbyint(v / scale)) + zp, 0, 255) (reorder_data_type/scalar_impl/scalar_ref_kernels.cpp:36-40).
// Non-finite elements, whose conversion the reference leaves undefined, give 0 as in its per-token kernels.
//
// Three small launches: per-row bounds (one wavefront per row), the parameters (one workgroup), the codes (one
// wavefront per row).  HBM-bound: the source is read twice (2 or 4 bytes per element each time) and one byte written.
#include <hip/hip_runtime.h>

#include "../../include/zmi_lowoha.h"
#include "zmi_device.h"
#include "zmi_launch.h"

template <bool BF16>
__device__ __forceinline__ float asym_ld(const void *x, int64_t i) {
  return BF16 ? zmi_bf16_to_f32(((const uint16_t *)x)[i]) : ((const float *)x)[i];
}
__device__ __forceinline__ bool asym_finite(float v) { return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u; }

template <bool BF16>
__global__ __launch_bounds__(256) void zmi_asym_tensor_bounds_kernel(const void *x, int64_t ldx, int M, int K, float *lohi) {
  const int lane = threadIdx.x % 64;
  const int m = blockIdx.x * 4 + threadIdx.x / 64;
  if (m >= M) return;
  const float big = 3.402823466e+38f;
  float lo = big, hi = -big;
  for (int k = lane; k < K; k += 64) {
    const float v = asym_ld<BF16>(x, (int64_t)m * ldx + k);
    if (asym_finite(v)) {
      lo = fminf(lo, v);
      hi = fmaxf(hi, v);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, o));
    hi = fmaxf(hi, __shfl_xor(hi, o));
  }
  if (lane == 0) {
    lohi[2 * m] = lo;
    lohi[2 * m + 1] = hi;
  }
}

__global__ __launch_bounds__(256) void zmi_asym_tensor_params_kernel(const float *lohi, int M, float *scale, int32_t *zp,
                                                                     void *user_scale, int32_t user_dt) {
  __shared__ float s_lo[4], s_hi[4];
  const float big = 3.402823466e+38f;
  float lo = big, hi = -big;
  for (int m = threadIdx.x; m < M; m += 256) {
    lo = fminf(lo, lohi[2 * m]);
    hi = fmaxf(hi, lohi[2 * m + 1]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, o));
    hi = fmaxf(hi, __shfl_xor(hi, o));
  }
  if (threadIdx.x % 64 == 0) {
    s_lo[threadIdx.x / 64] = lo;
    s_hi[threadIdx.x / 64] = hi;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  lo = fminf(fminf(s_lo[0], s_lo[1]), fminf(s_lo[2], s_lo[3]));
  hi = fmaxf(fmaxf(s_hi[0], s_hi[1]), fmaxf(s_hi[2], s_hi[3]));
  if (lo == big && hi == -big) lo = hi = 0.0f;
  if (hi <= lo) hi = __fadd_rn(lo, 1.0f);
  float s = __fdiv_rn(__fsub_rn(hi, lo), 255.0f);
  const double zd = round((double)(-lo) / (double)s);
  *zp = zd < -2147483648.0 ? (int32_t)0x80000000 : zd > 2147483647.0 ? 0x7fffffff : (int32_t)zd;
  if (s < 1e-10f) s = 1e-10f;
  // A bf16 scale buffer holds the narrowed value, and the codes are made with what that buffer reads back as: the
  // reference computes the parameters, stores them, and then runs its static reorder on the stored parameters
  // (lowoha_reorder.cpp:186-205 after compute_dynamic_quant_params, lowoha_reorder_utils.cpp:600-628, 810).  The
  // zero-point above comes from the scale as computed, as there.
  if (user_scale && user_dt == ZMI_DT_BF16) {
    const uint16_t h = zmi_f32_to_bf16_rne(s);
    *(uint16_t *)user_scale = h;
    s = zmi_bf16_to_f32(h);
  }
  *scale = s;
}

template <bool BF16>
__global__ __launch_bounds__(256) void zmi_asym_tensor_quant_kernel(const void *x, int64_t ldx, int M, int K,
                                                                    const float *scale, const int32_t *zp, uint8_t *q,
                                                                    int64_t ldq) {
  const int lane = threadIdx.x % 64;
  const int m = blockIdx.x * 4 + threadIdx.x / 64;
  if (m >= M) return;
  const float s = *scale;
  const long long z = *zp;
  for (int k = lane; k < K; k += 64) {
    const float v = asym_ld<BF16>(x, (int64_t)m * ldx + k);
    uint8_t out = 0;
    if (asym_finite(v)) {
      float t = rintf(__fdiv_rn(v, s));
      t = fminf(fmaxf(t, -4e9f), 4e9f);
      const long long qq = (long long)t + z;
      out = (uint8_t)(qq < 0 ? 0 : qq > 255 ? 255 : qq);
    }
    q[(int64_t)m * ldq + k] = out;
  }
}

// scale: the f32 the codes are made with (the caller's buffer when its type is f32; with a bf16 scale buffer scratch
// that receives the narrowed value widened again, the bf16 itself going to user_scale); lohi: 2 * M floats of scratch
hipError_t zmi_launch_quant_asym_tensor(const void *x, int32_t x_dt, int64_t M, int64_t K, int64_t ldx, uint8_t *q,
                                        int64_t ldq, float *lohi, float *scale, int32_t *zp, void *user_scale,
                                        int32_t user_dt, hipStream_t stream) {
  if (M <= 0 || K <= 0 || (x_dt != ZMI_DT_BF16 && x_dt != ZMI_DT_F32) || !q || !lohi || !scale || !zp || ldx < K || ldq < K)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)((M + 3) / 4));
  if (x_dt == ZMI_DT_BF16) {
    hipLaunchKernelGGL(zmi_asym_tensor_bounds_kernel<true>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, lohi);
    hipLaunchKernelGGL(zmi_asym_tensor_params_kernel, dim3(1), dim3(256), 0, stream, lohi, (int)M, scale, zp, user_scale, user_dt);
    hipLaunchKernelGGL(zmi_asym_tensor_quant_kernel<true>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, scale, zp, q, ldq);
  } else {
    hipLaunchKernelGGL(zmi_asym_tensor_bounds_kernel<false>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, lohi);
    hipLaunchKernelGGL(zmi_asym_tensor_params_kernel, dim3(1), dim3(256), 0, stream, lohi, (int)M, scale, zp, user_scale, user_dt);
    hipLaunchKernelGGL(zmi_asym_tensor_quant_kernel<false>, grid, dim3(256), 0, stream, x, ldx, (int)M, (int)K, scale, zp, q, ldq);
  }
  return hipGetLastError();
}
