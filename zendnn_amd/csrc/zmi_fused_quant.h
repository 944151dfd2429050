// Per-token quantization of one source row by a whole workgroup, used by the
// small-M kernels that fuse the quantization into the GEMM launch: the
// workgroups with the lowest indices quantize one row each and publish it through
// the row's device-scope flag, and every workgroup waits for the flags of all rows
// before it reads the s8 rows (same arithmetic as k_quant.hip).
#pragma once
#include "zmi_device.h"
#include "zmi_launch.h"

// Quantizes one source row with the whole workgroup.  The s8 row and its scale
// are written with device-scope (write-through) stores: the eight XCDs have
// private, mutually non-coherent L2s, and a full release / acquire fence pair
// would write back and invalidate whole caches in the middle of the weight
// stream.  Readers on other XCDs miss in their own L2 (invalidated when the
// kernel started) and fetch the fresh bytes.
// The scale the GEMM multiplies by is the one the scale buffer holds: with a bf16 scale dtype the reference narrows the
// computed f32 scale (bfloat16_t::f32_to_bf16_val, lowoha_operators/reorder/lowoha_reorder_utils.cpp:600-628) and its
// GEMM reads the narrowed value back, while the rows were quantized with the f32 scale.
static __device__ __forceinline__ float zmi_fused_scale_as_stored(const ZmiFusedQuant &fq, float s) {
  return fq.user_dt == ZMI_DT_BF16 ? zmi_bf16_to_f32(zmi_f32_to_bf16_rne(s)) : s;
}

// ---- hand-off --------------------------------------------------------------------------
// Producer side, called by every thread of a workgroup that has just quantized row `row`: the
// row's flag takes the launch's epoch once all the workgroup's write-through stores have landed.
// (copies > 1: the flag goes to that many copies of the flag words, a page apart; waiters through the scalar unit
// spread over them, everybody else reads copy 0)
static __device__ __forceinline__ void zmi_fq_publish(const ZmiFusedQuant &fq, int row, int copies = 1) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if ((int)threadIdx.x < copies)
    __hip_atomic_store(&fq.flags[threadIdx.x * 1024 + row], fq.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Consumer side, called by whole wavefronts (every lane): polls the flags of rows 0 .. rows-1
// (lane l looks at rows l and l + 64; rows <= 128) until all carry the launch's epoch or the time
// limit passes.  Returns true when the rows are there.  When the limit ran out the error word is
// set and the caller must not touch the rows: the host reports the failure on the thread's next call.
static __device__ __forceinline__ bool zmi_fq_wait(const ZmiFusedQuant &fq, int rows) {
  const int lane = threadIdx.x % 64;
  const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
  const unsigned int *f0 = &fq.flags[lane < rows ? lane : 0];
  const unsigned int *f1 = &fq.flags[lane + 64 < rows ? lane + 64 : 0];
  const bool two = rows > 64;   // (uniform)
  bool ok = false;
  // A look at the flags is a trip to memory behind everything the compute unit has already asked for (microseconds
  // under load), so several looks are kept in flight, a fraction of a microsecond apart, and examined oldest first.
  constexpr int NP = 4;
  unsigned int v0[NP], v1[NP];
  if (fq.wait_ticks != 0) {
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      v0[j] = __hip_atomic_load(f0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v1[j] = two ? __hip_atomic_load(f1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : fq.epoch;
      __builtin_amdgcn_s_sleep(4);
    }
    for (;;) {
      bool done = false;
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        if (__all(v0[j] == fq.epoch && v1[j] == fq.epoch)) { ok = true; done = true; break; }
        if (__builtin_amdgcn_s_memrealtime() - t0 > (uint64_t)fq.wait_ticks) { done = true; break; }
        v0[j] = __hip_atomic_load(f0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v1[j] = two ? __hip_atomic_load(f1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : fq.epoch;
      }
      if (done) break;
    }
  }
  if (!ok && lane == 0) __hip_atomic_store(fq.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  return ok;
}

// The same wait through the scalar unit, called by a whole wavefront: a scalar load does not stand in the compute
// unit's queue of vector memory requests, so a wavefront may have its whole weight stream in flight while it waits
// (behind the stream, a vector load of the flags returns with the stream).  A scalar load cannot ask for device
// scope; the flags lie in uncached device memory for it (in cached memory the XCD's L2 would keep answering with
// the line it fetched first), and `glc` makes the load miss in the scalar cache.
static __device__ __forceinline__ bool zmi_fq_wait_scalar(const ZmiFusedQuant &fq, int rows, const unsigned int *flags) {
  typedef unsigned int zmi_u16v __attribute__((ext_vector_type(16)));
  const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
  bool ok = false;
  if (fq.wait_ticks != 0) {
    for (;;) {
      bool all = true;
      for (int r0 = 0; r0 < rows; r0 += 16) {   // (rows <= 128: at most 8 loads of 16 flags)
        zmi_u16v v;
        asm volatile("s_load_dwordx16 %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=&s"(v) : "s"(flags + r0) : "memory");
#pragma unroll
        for (int i = 0; i < 16; ++i) all &= (r0 + i >= rows) | (v[i] == fq.epoch);
      }
      if (all) { ok = true; break; }
      if (__builtin_amdgcn_s_memrealtime() - t0 > (uint64_t)fq.wait_ticks) break;
      __builtin_amdgcn_s_sleep(2);
    }
  }
  if (!ok && threadIdx.x % 64 == 0) __hip_atomic_store(fq.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  return ok;
}

static __device__ void zmi_fused_quant_row(const ZmiFusedQuant &fq, int row, int K, float *red) {
  const int t = threadIdx.x, nt = blockDim.x;
  const bool bf16 = fq.x_dt == ZMI_DT_BF16;
  const char *src = (const char *)fq.x + (size_t)row * fq.ldx * (bf16 ? 2 : 4);
  auto ld = [&](int k) { return bf16 ? zmi_bf16_to_f32(((const uint16_t *)src)[k]) : ((const float *)src)[k]; };
  // one 16-byte chunk (8 bf16) per thread held in registers when the row fits
  const bool vec = bf16 && K % 8 == 0 && K <= nt * 8 && ((uintptr_t)src % 16) == 0;
  float v8[8];
  float amax = 0.0f;
  if (vec) {
    #pragma unroll
    for (int j = 0; j < 8; ++j) v8[j] = 0.0f;
    if (t * 8 < K) {
      const v4i raw = *(const v4i *)((const uint16_t *)src + t * 8);
      #pragma unroll
      for (int j = 0; j < 4; ++j) {
        v8[2 * j] = __uint_as_float(((uint32_t)raw[j]) << 16);
        v8[2 * j + 1] = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
      }
    }
    #pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = fabsf(v8[j]);
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
  } else {
    for (int k = t; k < K; k += nt) {
      const float a = fabsf(ld(k));
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
  }
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if (t % 64 == 0) red[t / 64] = amax;
  __syncthreads();
  amax = red[0];
  for (int i = 1; i < nt / 64; ++i) amax = fmaxf(amax, red[i]);
  __syncthreads();
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (t == 0) {
    __hip_atomic_store((unsigned int *)&fq.scales[row], __float_as_uint(zmi_fused_scale_as_stored(fq, s)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (fq.user_scales) {
      if (fq.user_dt == ZMI_DT_BF16) ((uint16_t *)fq.user_scales)[row] = zmi_f32_to_bf16_rne(s);
      else ((float *)fq.user_scales)[row] = s;
    }
  }
  unsigned int *dst = (unsigned int *)(fq.q + (size_t)row * fq.ldq);
  if (vec) {
    if (t * 8 < K) {
      #pragma unroll
      for (int h = 0; h < 2; ++h) {
        unsigned int w = 0;
        #pragma unroll
        for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(v8[h * 4 + j], s, inv)) << (8 * j);
        __hip_atomic_store(&dst[t * 2 + h], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    return;
  }
  for (int k4 = t; k4 < K / 4; k4 += nt) {
    unsigned int w = 0;
    #pragma unroll
    for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(ld(k4 * 4 + j), s, inv)) << (8 * j);
    __hip_atomic_store(&dst[k4], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}


// The same by a single wavefront (no workgroup barrier), for kernels whose other
// wavefronts must not wait for the quantization: two passes over the row, the
// second one re-reads it from L2.  K must be a multiple of 4.
static __device__ void zmi_fused_quant_row_wave(const ZmiFusedQuant &fq, int row, int K) {
  const int lane = threadIdx.x % 64;
  const bool bf16 = fq.x_dt == ZMI_DT_BF16;
  const char *src = (const char *)fq.x + (size_t)row * fq.ldx * (bf16 ? 2 : 4);
  const bool vec = bf16 && K % 8 == 0 && ((uintptr_t)src % 16) == 0;
  auto ld = [&](int k) { return bf16 ? zmi_bf16_to_f32(((const uint16_t *)src)[k]) : ((const float *)src)[k]; };
  auto ld8 = [&](int k, float (&v)[8]) {
    const v4i raw = *(const v4i *)((const uint16_t *)src + k);
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = __uint_as_float(((uint32_t)raw[j]) << 16);
      v[2 * j + 1] = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
    }
  };
  float amax = 0.0f;
  if (vec) {
    for (int k = lane * 8; k < K; k += 512) {
      float v[8];
      ld8(k, v);
      #pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float a = fabsf(v[j]);
        if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
      }
    }
  } else {
    for (int k = lane; k < K; k += 64) {
      const float a = fabsf(ld(k));
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
  }
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  if (lane == 0) {
    __hip_atomic_store((unsigned int *)&fq.scales[row], __float_as_uint(zmi_fused_scale_as_stored(fq, s)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (fq.user_scales) {
      if (fq.user_dt == ZMI_DT_BF16) ((uint16_t *)fq.user_scales)[row] = zmi_f32_to_bf16_rne(s);
      else ((float *)fq.user_scales)[row] = s;
    }
  }
  unsigned int *dst = (unsigned int *)(fq.q + (size_t)row * fq.ldq);
  if (vec) {
    for (int k = lane * 8; k < K; k += 512) {
      float v[8];
      ld8(k, v);
      #pragma unroll
      for (int h = 0; h < 2; ++h) {
        unsigned int w = 0;
        #pragma unroll
        for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(v[h * 4 + j], s, inv)) << (8 * j);
        __hip_atomic_store(&dst[k / 4 + h], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    return;
  }
  for (int k4 = lane; k4 < K / 4; k4 += 64) {
    unsigned int w = 0;
    #pragma unroll
    for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(ld(k4 * 4 + j), s, inv)) << (8 * j);
    __hip_atomic_store(&dst[k4], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}


// Per-group form: one source row, G groups of K / G elements, every wavefront of the workgroup takes the
// groups w, w + n_waves, ... (same arithmetic as zmi_quant_groups_kernel; K / G must be a multiple of 4).
// Scales go to fq.scales[row * G + g]; published like the rows, with device-scope stores.
static __device__ void zmi_fused_quant_row_groups(const ZmiFusedQuant &fq, int row, int K, int G) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64, n_waves = blockDim.x / 64;
  const bool bf16 = fq.x_dt == ZMI_DT_BF16;
  const int gs = K / G;
  // Fast form: the row fits the workgroup at 8 elements per thread and a group is a power-of-two run of
  // lanes inside one wavefront (groups of 64 .. 512): one 16-byte request per thread (two for f32), the
  // group maximum by lane exchanges, one 8-byte store -- a single trip to memory.
  const int es = bf16 ? 2 : 4;
  const char *rowp = (const char *)fq.x + (size_t)row * fq.ldx * es;
  if (K % 8 == 0 && K <= (int)blockDim.x * 8 && gs >= 8 && gs <= 512 && (gs & (gs - 1)) == 0 &&
      ((uintptr_t)rowp % 16) == 0) {
    const int t = threadIdx.x;
    float v8[8];
    #pragma unroll
    for (int j = 0; j < 8; ++j) v8[j] = 0.0f;
    if (t * 8 < K) {
      if (bf16) {
        const v4i raw = *(const v4i *)(rowp + (size_t)t * 16);
        #pragma unroll
        for (int j = 0; j < 4; ++j) {
          v8[2 * j] = __uint_as_float(((uint32_t)raw[j]) << 16);
          v8[2 * j + 1] = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
        }
      } else {
        const v4i r0 = *(const v4i *)(rowp + (size_t)t * 32), r1 = *(const v4i *)(rowp + (size_t)t * 32 + 16);
        #pragma unroll
        for (int j = 0; j < 4; ++j) { v8[j] = __int_as_float(r0[j]); v8[4 + j] = __int_as_float(r1[j]); }
      }
    }
    float amax = 0.0f;
    #pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = fabsf(v8[j]);
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
    const int lpg = gs / 8;   // lanes per group: 1 .. 64
    #pragma unroll
    for (int o = 32; o > 0; o >>= 1)
      if (o < lpg) amax = fmaxf(amax, __shfl_xor(amax, o));
    if (amax < 1e-10f) amax = 1e-10f;
    float s = __fdiv_rn(amax, 127.0f);
    if (s < 1e-10f) s = 1e-10f;
    const float inv = __fdiv_rn(1.0f, s);
    if (t * 8 < K) {
      const int g = t * 8 / gs;
      if (t % lpg == 0) {
        __hip_atomic_store((unsigned int *)&fq.scales[(int64_t)row * G + g], __float_as_uint(zmi_fused_scale_as_stored(fq, s)), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        if (fq.user_scales) {
          if (fq.user_dt == ZMI_DT_BF16) ((uint16_t *)fq.user_scales)[(int64_t)row * G + g] = zmi_f32_to_bf16_rne(s);
          else ((float *)fq.user_scales)[(int64_t)row * G + g] = s;
        }
      }
      unsigned int *dst = (unsigned int *)(fq.q + (int64_t)row * fq.ldq);
      #pragma unroll
      for (int h = 0; h < 2; ++h) {
        unsigned int w = 0;
        #pragma unroll
        for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(v8[h * 4 + j], s, inv)) << (8 * j);
        __hip_atomic_store(&dst[t * 2 + h], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    return;
  }
  for (int g = wave; g < G; g += n_waves) {
    const int64_t base = (int64_t)row * fq.ldx + (int64_t)g * gs;
    auto ld = [&](int k) { return bf16 ? zmi_bf16_to_f32(((const uint16_t *)fq.x)[base + k]) : ((const float *)fq.x)[base + k]; };
    float amax = 0.0f;
    for (int k = lane; k < gs; k += 64) {
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
      __hip_atomic_store((unsigned int *)&fq.scales[(int64_t)row * G + g], __float_as_uint(zmi_fused_scale_as_stored(fq, s)), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      if (fq.user_scales) {
        if (fq.user_dt == ZMI_DT_BF16) ((uint16_t *)fq.user_scales)[(int64_t)row * G + g] = zmi_f32_to_bf16_rne(s);
        else ((float *)fq.user_scales)[(int64_t)row * G + g] = s;
      }
    }
    unsigned int *dst = (unsigned int *)(fq.q + (int64_t)row * fq.ldq + (int64_t)g * gs);
    for (int k4 = lane; k4 < gs / 4; k4 += 64) {
      unsigned int w = 0;
      #pragma unroll
      for (int j = 0; j < 4; ++j) w |= ((unsigned int)(uint8_t)zmi_quant_elem(ld(k4 * 4 + j), s, inv)) << (8 * j);
      __hip_atomic_store(&dst[k4], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}
