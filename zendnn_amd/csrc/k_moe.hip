// MoE glue kernels for gfx950: stand-alone gated activation, weighted reduce
// (combine), device-side routing (histogram / scan / stable slot assignment),
// quantize-and-scatter, and the per-expert problem table.  All HBM-bound.
#include "zmi_device.h"
#include "zmi_launch.h"
#include "zmi_ring_table.h"

// ---------------------------------------------------------------------------
// Gated activation in place: buf[m, 0:dim] = act(gate) * up, dim = N/2.
// Reference: group_matmul_moe_act_execute / apply_gated_act_inplace
// (zendnnl/src/lowoha_operators/matmul/group_matmul/group_matmul_moe_act.cpp:88-254).
// One workgroup per row.  Results are staged in LDS and written after a
// barrier because swiglu_oai's interleaved layout overlaps reads and writes.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void zmi_gated_act_kernel(ZmiActMat m0, const ZmiActMat *mats, int n_mat,
                                                            int act, int dt) {
  extern __shared__ float res[];
  const int row = blockIdx.x;
  ZmiActMat m = m0;
  if (mats) {
    int lo = 0, hi = n_mat - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) / 2;
      if (mats[mid].row_start <= row) lo = mid; else hi = mid - 1;
    }
    m = mats[lo];
  }
  const int r = row - m.row_start;
  if (r >= m.M) return;
  const int dim = m.N / 2;
  const int64_t base = (int64_t)r * m.ld;
  for (int n = threadIdx.x; n < dim; n += blockDim.x) {
    float g, u;
    if (act == ZMI_ACT_SWIGLU_OAI_MUL) {
      g = zmi_ld_f32(m.buf, dt, base + 2 * n);
      u = zmi_ld_f32(m.buf, dt, base + 2 * n + 1);
    } else {
      g = zmi_ld_f32(m.buf, dt, base + n);
      u = zmi_ld_f32(m.buf, dt, base + dim + n);
    }
    res[n] = zmi_gated(act, g, u);
  }
  __syncthreads();
  for (int n = threadIdx.x; n < dim; n += blockDim.x) {
    if (dt == ZMI_DT_BF16) ((uint16_t *)m.buf)[base + n] = zmi_f32_to_bf16(res[n]);
    else if (dt == ZMI_DT_F16) ((uint16_t *)m.buf)[base + n] = zmi_f32_to_f16(res[n]);   // (float16_t(value), group_matmul_moe_act.cpp:165-182)
    else ((float *)m.buf)[base + n] = res[n];
  }
}

hipError_t zmi_launch_gated_act(const ZmiActMat *mats_dev, const ZmiActMat *mat0, int n_mat,
                                int64_t total_rows, int max_N, int32_t act, int32_t dt, hipStream_t stream) {
  if (total_rows <= 0) return hipSuccess;
  const size_t smem = (size_t)(max_N / 2) * sizeof(float);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  {
    hipError_t e = zmi_func_smem_once((const void *)zmi_gated_act_kernel, (int)smem);
    if (e != hipSuccess) return e;
  }
  ZmiActMat m0 = {};
  if (mat0) m0 = *mat0;
  hipLaunchKernelGGL(zmi_gated_act_kernel, dim3((unsigned)total_rows), dim3(256), smem, stream, m0, mats_dev,
                     n_mat, act, dt);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Weighted reduce: out[t, d] = sum_k w[t,k] * row(t,k)[d], f32 accumulation in
// k order, first term a plain product, then fused multiply-adds; bf16 store
// with the plain round-to-nearest-even bit trick.
// Reference: moe_weighted_reduce_avx512_{bf16,f32}
// (group_matmul/group_matmul_moe_postop.cpp:191-286).
// Rows come either from a table of pointers (the reference's row_ptrs) or from
// rows_base + slot_of[t*topk+k] * row_ld (device-side routing).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void zmi_moe_combine_kernel(const void *const *row_ptrs, const void *rows_base,
                                                              int64_t row_ld, const int32_t *slot_of,
                                                              const float *weights, int skip_weighted, int topk,
                                                              int D, int dt, void *out, int64_t ldo) {
  const int t = blockIdx.x;
  const size_t es = dt == ZMI_DT_BF16 || dt == ZMI_DT_F16 ? 2 : 4;
  auto row_of = [&](int k) -> const void * {
    const int s = t * topk + k;
    return row_ptrs ? row_ptrs[s] : (const void *)((const char *)rows_base + (int64_t)slot_of[s] * row_ld * es);
  };
  // bf16 rows, 8 columns (16 bytes) per thread and step, when everything is 16-byte aligned
  bool vec = dt == ZMI_DT_BF16 && D % 8 == 0 && ldo % 8 == 0 && ((uintptr_t)out) % 16 == 0;
  for (int k = 0; k < topk && vec; ++k) vec = ((uintptr_t)row_of(k)) % 16 == 0;
  if (vec) {
    for (int d = threadIdx.x * 8; d < D; d += blockDim.x * 8) {
      float acc[8];
      for (int k = 0; k < topk; ++k) {
        const v4i raw = *(const v4i *)((const uint16_t *)row_of(k) + d);
        const float w = skip_weighted ? 1.0f : weights[t * topk + k];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float x0 = __uint_as_float(((uint32_t)raw[j]) << 16);
          const float x1 = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
          acc[2 * j] = (k == 0) ? __fmul_rn(w, x0) : __builtin_fmaf(w, x0, acc[2 * j]);
          acc[2 * j + 1] = (k == 0) ? __fmul_rn(w, x1) : __builtin_fmaf(w, x1, acc[2 * j + 1]);
        }
      }
      v4i o;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[j] = (int)((uint32_t)zmi_f32_to_bf16_rne(acc[2 * j]) | ((uint32_t)zmi_f32_to_bf16_rne(acc[2 * j + 1]) << 16));
      *(v4i *)((uint16_t *)out + (int64_t)t * ldo + d) = o;
    }
    return;
  }
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = 0.0f;
    for (int k = 0; k < topk; ++k) {
      const float w = skip_weighted ? 1.0f : weights[t * topk + k];
      const float x = zmi_ld_f32(row_of(k), dt, d);
      acc = (k == 0) ? __fmul_rn(w, x) : __builtin_fmaf(w, x, acc);
    }
    if (dt == ZMI_DT_BF16) ((uint16_t *)out)[(int64_t)t * ldo + d] = zmi_f32_to_bf16_rne(acc);
    else if (dt == ZMI_DT_F16) ((uint16_t *)out)[(int64_t)t * ldo + d] = zmi_f32_to_f16(acc);   // (store_from_f32, group_matmul_moe_postop.cpp:84-100)
    else ((float *)out)[(int64_t)t * ldo + d] = acc;
  }
}

hipError_t zmi_launch_moe_combine(const void *const *row_ptrs_dev, const void *rows_base, int64_t row_ld,
                                  const int32_t *slot_of, const float *weights, int skip_weighted, int T,
                                  int topk, int D, int32_t dt, void *out, int64_t ldo, hipStream_t stream) {
  if (T <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_moe_combine_kernel, dim3((unsigned)T), dim3(256), 0, stream, row_ptrs_dev, rows_base,
                     row_ld, slot_of, weights, skip_weighted, topk, D, dt, out, ldo);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Routing.  G workgroups of 16 wavefronts; wavefront u = 16 g + w owns the
// contiguous segment u of the flat (t,k) index space.
//   A: per-wavefront histograms hist[u][e] (LDS atomics);
//   B: counts / exclusive offsets per expert, and cursor[u][e] = offsets[e] +
//      sum of hist[u'][e] for u' < u;
//   C: every wavefront walks its segment in order, 64 entries at a time; an
//      entry's slot is cursor + (number of lower lanes with the same expert).
// The order inside an expert is therefore the (t,k) order: deterministic.
// One workgroup does A, B and C in one launch.  Several workgroups (long id lists: one
// workgroup would walk them 1024 entries at a time) take two launches: `phase` 0 is pass A,
// whose histograms go to ghist[16 G][E] in device memory; `phase` 1 reads all of them back
// for pass B (every workgroup computes the offsets for itself) and runs pass C.
// ---------------------------------------------------------------------------
#define RT_WAVES 16
#define RT_KEEP 8    // ids kept per lane between the passes of one launch: 8 x 64 x 16 = 8192 entries per workgroup

__global__ __launch_bounds__(RT_WAVES * 64) void zmi_moe_route_kernel(const int32_t *topk_ids, int n, int E,
                                                                      int align, int32_t *counts,
                                                                      int32_t *offsets, int32_t *slot_of,
                                                                      int32_t *src_of, int n_slots, int32_t *ghist,
                                                                      int phase) {
  extern __shared__ int32_t sh[];   // hist[RT_WAVES][E], off[E+1], then (several workgroups) all histograms
  int32_t *hist = sh;
  int32_t *off = sh + RT_WAVES * E;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int G = gridDim.x, g = blockIdx.x;
  const bool multi = G > 1;
  int ebits = 1;
  while ((1 << ebits) < E) ++ebits;          // expert ids fit in ebits bits
  const int seg = (n + G * RT_WAVES - 1) / (G * RT_WAVES);
  const int s0 = (g * RT_WAVES + wave) * seg < n ? (g * RT_WAVES + wave) * seg : n;
  const int s1 = (s0 + seg < n) ? s0 + seg : n;
  // The segment's ids are read once, all loads in flight together, and kept in registers
  // (RT_KEEP x 64 per wavefront; what a longer segment has beyond that is read again).
  int keep[RT_KEEP];
#pragma unroll
  for (int it = 0; it < RT_KEEP; ++it) {
    const int i = s0 + it * 64 + lane;
    keep[it] = i < s1 ? topk_ids[i] : -1;
  }
  if (!multi || phase == 0) {
    if (src_of)
      for (int i = g * blockDim.x + tid; i < n_slots; i += G * blockDim.x) src_of[i] = -1;
    for (int i = tid; i < RT_WAVES * E; i += blockDim.x) hist[i] = 0;
    __syncthreads();
    auto count = [&](int e) {
      if (e >= 0 && e < E) atomicAdd(&hist[wave * E + e], 1);
    };
#pragma unroll
    for (int it = 0; it < RT_KEEP; ++it)
      if (s0 + it * 64 < s1) count(keep[it]);
    for (int i0 = s0 + RT_KEEP * 64; i0 < s1; i0 += 64) count(i0 + lane < s1 ? topk_ids[i0 + lane] : -1);
    __syncthreads();
    if (multi) {
      for (int i = tid; i < RT_WAVES * E; i += blockDim.x) ghist[(size_t)g * RT_WAVES * E + i] = hist[i];
      return;
    }
  }
  // per-expert totals and the per-wavefront running starts (thread e handles expert e);
  // several workgroups: all their histograms come into LDS first, in one sweep of loads
  int32_t *gh = off + E + 1;
  if (multi) {
    for (int i = tid; i < G * RT_WAVES * E; i += blockDim.x) gh[i] = ghist[i];
    __syncthreads();
  }
  for (int e = tid; e < E; e += blockDim.x) {
    int run = 0;
    if (!multi) {
      for (int w = 0; w < RT_WAVES; ++w) {
        const int c = hist[w * E + e];
        hist[w * E + e] = run;
        run += c;
      }
    } else {
      for (int u = 0; u < G * RT_WAVES; ++u) {
        if (u == g * RT_WAVES) {
          // this workgroup's wavefronts start here
          int r2 = run;
          for (int w = 0; w < RT_WAVES; ++w) {
            hist[w * E + e] = r2;
            r2 += gh[(u + w) * E + e];
          }
        }
        run += gh[u * E + e];
      }
    }
    off[e] = run;
    if (g == 0) counts[e] = run;
  }
  __syncthreads();
  // exclusive offsets of the aligned counts: wavefront 0 scans 64 experts per step
  if (wave == 0) {
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int c = e < E ? (off[e] + align - 1) / align * align : 0;
      int x = c;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int y = __shfl_up(x, o);
        if (lane >= o) x += y;
      }
      if (e < E) {
        off[e] = carry + x - c;
        if (g == 0) offsets[e] = carry + x - c;
      }
      carry += __shfl(x, 63);
    }
    if (lane == 0) {
      off[E] = carry;
      if (g == 0) offsets[E] = carry;
    }
  }
  __syncthreads();
  auto place = [&](int i, int e) {
    const bool live = i < s1;
    const bool ok = live && e >= 0 && e < E;
    if (!ok) e = -1;
    // lanes holding the same expert as this lane
    unsigned long long same = __ballot(ok);
    for (int bit = 0; bit < ebits; ++bit) {
      const unsigned long long b = __ballot((e >> bit) & 1);
      same &= ((e >> bit) & 1) ? b : ~b;
    }
    if (ok) {
      const int rank = __popcll(same & ((1ull << lane) - 1ull));
      const int total = __popcll(same);
      const int start = hist[wave * E + e];
      slot_of[i] = off[e] + start + rank;
      if (src_of) src_of[off[e] + start + rank] = i;
      // the last lane of each expert group advances the cursor for the next 64 entries
      if (rank == total - 1) hist[wave * E + e] = start + total;
    } else if (live) {
      slot_of[i] = -1;
    }
    __builtin_amdgcn_wave_barrier();
  };
#pragma unroll
  for (int it = 0; it < RT_KEEP; ++it)
    if (s0 + it * 64 < s1) place(s0 + it * 64 + lane, keep[it]);
  for (int i0 = s0 + RT_KEEP * 64; i0 < s1; i0 += 64) {
    const int i = i0 + lane;
    place(i, i < s1 ? topk_ids[i] : -1);
  }
}

// workgroups of a routing launch: 4096 entries each (4 steps of 64 per wavefront), at most 16,
// and no more than keep all the per-wavefront histograms within 64 KiB of LDS
static int zmi_moe_route_groups(int64_t n, int E) {
  int64_t G = (n + 4095) / 4096;
  if (G > 16) G = 16;
  const int64_t cap = 16384 / ((int64_t)RT_WAVES * E);
  if (G > cap) G = cap;
  return G < 1 ? 1 : (int)G;
}

// hist_scratch: zmi_moe_route_scratch_ints(T * topk, E) ints of device memory for the
// several-workgroup form (null: one workgroup whatever the size).
size_t zmi_moe_route_scratch_ints(int64_t n, int E) {
  const int G = zmi_moe_route_groups(n, E);
  return G > 1 ? (size_t)G * RT_WAVES * E : 0;
}

hipError_t zmi_launch_moe_route(const int32_t *topk_ids, int T, int topk, int E, int align, int32_t *counts,
                                int32_t *offsets, int32_t *slot_of, int32_t *src_of, int n_slots,
                                int32_t *hist_scratch, hipStream_t stream) {
  if (E > 2047 || E <= 0) return hipErrorInvalidValue;
  const int n = T * topk;
  const int G = hist_scratch ? zmi_moe_route_groups(n, E) : 1;
  const size_t smem = ((size_t)RT_WAVES * E + E + 1 + (G > 1 ? (size_t)G * RT_WAVES * E : 0)) * sizeof(int32_t);
  {
    hipError_t e = zmi_func_smem_once((const void *)zmi_moe_route_kernel, (int)smem);
    if (e != hipSuccess) return e;
  }
  const int al = align < 1 ? 1 : align;
  if (G > 1)
    hipLaunchKernelGGL(zmi_moe_route_kernel, dim3(G), dim3(RT_WAVES * 64), smem, stream, topk_ids, n, E, al, counts,
                       offsets, slot_of, src_of, n_slots, hist_scratch, 0);
  hipLaunchKernelGGL(zmi_moe_route_kernel, dim3(G), dim3(RT_WAVES * 64), smem, stream, topk_ids, n, E, al, counts,
                     offsets, slot_of, src_of, n_slots, hist_scratch, 1);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Quantize token t once (per-token symmetric s8, same arithmetic as
// k_quant.hip) and write the row (fragment-major over the slot numbering) and
// its scale to each of its topk slots.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void zmi_moe_quant_scatter_kernel(const uint16_t *x, int64_t ldx, int H, int topk,
                                                                    const int32_t *slot_of, int8_t *A1, float *s1) {
  const int64_t k_pad = zmi_blob_kpad(H);
  __shared__ float red[4];
  const int t = blockIdx.x;
  const uint16_t *row = x + (int64_t)t * ldx;
  // 8 consecutive elements per thread and step (H is a multiple of 16); 16-byte loads when the row allows
  const bool vec = ((uintptr_t)row) % 16 == 0;
  auto load8 = [&](int k, float (&v)[8]) {
    if (vec) {
      const v4i raw = *(const v4i *)(row + k);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(((uint32_t)raw[j]) << 16);
        v[2 * j + 1] = __uint_as_float(((uint32_t)raw[j]) & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = zmi_bf16_to_f32(row[k + j]);
    }
  };
  float amax = 0.0f;
  for (int k = threadIdx.x * 8; k < H; k += blockDim.x * 8) {
    float v[8];
    load8(k, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = fabsf(v[j]);
      if ((__float_as_uint(a) & 0x7f800000u) != 0x7f800000u) amax = fmaxf(amax, a);
    }
  }
  #pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  if (amax < 1e-10f) amax = 1e-10f;
  float s = __fdiv_rn(amax, 127.0f);
  if (s < 1e-10f) s = 1e-10f;
  const float inv = __fdiv_rn(1.0f, s);
  for (int k = threadIdx.x * 8; k < H; k += blockDim.x * 8) {
    float v[8];
    load8(k, v);
    __attribute__((aligned(8))) int8_t q[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = zmi_quant_elem(v[j], s, inv);
    for (int j = 0; j < topk; ++j) {
      const int slot = slot_of[t * topk + j];
      // 8 consecutive k starting at a multiple of 8 are contiguous in fragment order
      if (slot >= 0) *(uint2 *)(A1 + zmi_afrag_off(slot, k, k_pad)) = *(const uint2 *)q;
    }
  }
  if (threadIdx.x < topk) {
    const int slot = slot_of[t * topk + threadIdx.x];
    if (slot >= 0) s1[slot] = s;
  }
}

hipError_t zmi_launch_moe_quant_scatter(const void *x, int64_t ldx, int T, int H, int topk,
                                        const int32_t *slot_of, int8_t *A1, float *s1, hipStream_t stream) {
  if (T <= 0) return hipSuccess;
  hipLaunchKernelGGL(zmi_moe_quant_scatter_kernel, dim3((unsigned)T), dim3(256), 0, stream, (const uint16_t *)x,
                     ldx, H, topk, slot_of, A1, s1);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Per-expert problem tables for Op1 (gate|up) and Op2 (down) from the device
// side counts / offsets.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void zmi_moe_build_problems_kernel(ZmiMoeTables tb, int E, int H, int I,
                                                                     const int32_t *counts, const int32_t *offsets,
                                                                     const int8_t *A1, const float *s1, uint16_t *act,
                                                                     const int8_t *A2, const float *s2, uint16_t *Y,
                                                                     ZmiProblem *op1, ZmiProblem *op2, int top1,
                                                                     int top2, int *tab1, int *tab2) {
  // one workgroup: the problem tables first, then (their rows are visible to the whole workgroup
  // after the barrier) wavefronts 0 and 1 fill the tile tables of the two grouped GEMM launches
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    const int64_t o = offsets[e];   // a multiple of 32: every expert starts on a fragment row
    ZmiProblem a = {};
    a.A = A1 + o * zmi_blob_kpad(H); a.lda = H; a.blob = (const uint8_t *)tb.w13_blob[e];
    a.dst = act + o * I; a.ldc = I; a.M = counts[e]; a.N = 2 * I; a.K = H; a.a_is_u8 = 0;
    a.src_scale_ptr = s1 + o; a.wei_scale_ptr = tb.w13_scale[e];
    op1[e] = a;
    ZmiProblem b = {};
    b.A = A2 + o * zmi_blob_kpad(I); b.lda = I; b.blob = (const uint8_t *)tb.w2_blob[e];
    b.dst = Y + o * H; b.ldc = H; b.M = counts[e]; b.N = H; b.K = I; b.a_is_u8 = 0;
    b.src_scale_ptr = s2 + o; b.wei_scale_ptr = tb.w2_scale[e];
    op2[e] = b;
  }
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  if (wave == 0 && tab1) zmi_ring_fill_table(op1, E, top1, 1, tab1, lane);
  if (wave == 1 && tab2) zmi_ring_fill_table(op2, E, top2, 0, tab2, lane);
}

// top1 / top2, tab1 / tab2: tile heights and tile tables of the Op1 (gated) and Op2 grouped launches
// (zmi_launch_gemm_ring_group with tab_ready = true then skips its own table launch).
hipError_t zmi_launch_moe_build_problems(ZmiMoeTables tb, int E, int H, int I, const int32_t *counts,
                                         const int32_t *offsets, const int8_t *A1, const float *s1, void *act,
                                         const int8_t *A2, const float *s2, void *Y, ZmiProblem *op1,
                                         ZmiProblem *op2, int top1, int top2, int *tab1, int *tab2,
                                         hipStream_t stream) {
  hipLaunchKernelGGL(zmi_moe_build_problems_kernel, dim3(1), dim3(256), 0, stream, tb, E, H, I, counts, offsets, A1,
                     s1, (uint16_t *)act, A2, s2, (uint16_t *)Y, op1, op2, top1, top2, tab1, tab2);
  return hipGetLastError();
}
