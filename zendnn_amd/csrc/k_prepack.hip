// Weight prepack for gfx950: [K,N] (or transposed [N,K]) s8 weights -> the
// MFMA-fragment blob described in zmi_device.h.  HBM-bound: K*N bytes read,
// K_pad*N_pad bytes written.
//
// Replaces the reference's aocl_reorder_{u8s8s32os32,s8s8s32os32,
// s8s8s32os32_sym_quant} calls (zendnnl/src/lowoha_operators/reorder/prepack/
// lowoha_prepack.cpp:173-252), which emit AVX-512 VNNI panels.
#include "zmi_device.h"
#include "zmi_launch.h"

// One workgroup packs a 64(k) x 64(n) patch: it is read with row-contiguous
// 16-byte loads, staged in LDS, and written as 2x2 fragments of 1 KiB, each
// thread writing one 16-byte chunk per fragment.
#define PP_TK 64
#define PP_TN 64

template <bool TRANSPOSED>
__global__ __launch_bounds__(256) void zmi_prepack_kernel(const int8_t *__restrict__ B, int64_t K,
                                                           int64_t N, int64_t ldb,
                                                           uint8_t *__restrict__ tiles,
                                                           int64_t kblocks) {
  // patch[k][n] with one pad byte column group to spread banks
  __shared__ int8_t patch[PP_TK][PP_TN + 4];
  const int t = threadIdx.x;
  const int64_t k0 = (int64_t)blockIdx.x * PP_TK;
  const int64_t n0 = (int64_t)blockIdx.y * PP_TN;

  if (!TRANSPOSED) {
    // source rows are k, contiguous in n: 64 rows x 64 bytes, 16 threads per row of 4 bytes
    for (int i = t; i < PP_TK * (PP_TN / 4); i += 256) {
      int kk = i / (PP_TN / 4), nn = (i % (PP_TN / 4)) * 4;
      int64_t k = k0 + kk, n = n0 + nn;
      int8_t v[4] = {0, 0, 0, 0};
      if (k < K) {
        for (int j = 0; j < 4; ++j)
          if (n + j < N) v[j] = B[k * ldb + n + j];
      }
      for (int j = 0; j < 4; ++j) patch[kk][nn + j] = v[j];
    }
  } else {
    // source rows are n, contiguous in k
    for (int i = t; i < PP_TN * (PP_TK / 4); i += 256) {
      int nn = i / (PP_TK / 4), kk = (i % (PP_TK / 4)) * 4;
      int64_t k = k0 + kk, n = n0 + nn;
      int8_t v[4] = {0, 0, 0, 0};
      if (n < N) {
        for (int j = 0; j < 4; ++j)
          if (k + j < K) v[j] = B[n * ldb + k + j];
      }
      for (int j = 0; j < 4; ++j) patch[kk + j][nn] = v[j];
    }
  }
  __syncthreads();

  // 4 fragments (2 column blocks x 2 k blocks), 64 lanes each: thread t writes
  // lane (t % 64) of fragment (t / 64).
  const int frag = t / 64, lane = t % 64;
  const int fnb = frag / 2, fkb = frag % 2;
  const int col = fnb * 32 + lane % 32;
  const int krow = fkb * 32 + (lane / 32) * 16;
  __attribute__((aligned(16))) int8_t out[16];
  #pragma unroll
  for (int b = 0; b < 16; ++b) out[b] = patch[krow + b][col];
  const int64_t nb = n0 / 32 + fnb, kb = k0 / 32 + fkb;
  uint8_t *dst = tiles + nb * zmi_blob_nb_stride(K) + kb * 1024 + lane * 16;
  *(v4i *)dst = *(const v4i *)out;
}

// colsum[n] = sum_k B[k][n], read back from the fragments: one wavefront per
// 32-column block; lane i adds its 16 bytes of every fragment, lanes i and
// i+32 hold the two k halves of the same column.
__global__ __launch_bounds__(64) void zmi_colsum_kernel(const uint8_t *__restrict__ tiles,
                                                        int64_t kblocks, int64_t nb_stride,
                                                        int32_t *__restrict__ colsum) {
  const int lane = threadIdx.x;
  const int64_t nb = blockIdx.x;
  const uint8_t *p = tiles + nb * nb_stride + lane * 16;
  int32_t s = 0;
  for (int64_t kb = 0; kb < kblocks; ++kb) {
    v4i v = *(const v4i *)(p + kb * 1024);
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      int32_t w = v[j];
      s += (int8_t)(w & 0xff) + (int8_t)((w >> 8) & 0xff) + (int8_t)((w >> 16) & 0xff) + (w >> 24);
    }
  }
  s += __shfl_xor(s, 32);
  if (lane < 32) colsum[nb * 32 + lane] = s;
}

__global__ void zmi_blob_header_kernel(ZmiBlobHeader *h, int64_t K, int64_t N, int32_t src_dtype,
                                       int32_t sym_group_size) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    h->magic = ZMI_BLOB_MAGIC;
    h->version = 1;
    h->flags = 0;
    h->K = K;
    h->N = N;
    h->K_pad = zmi_blob_kpad(K);
    h->N_pad = zmi_blob_npad(N);
    h->colsum_off = zmi_blob_colsum_off();
    h->tiles_off = zmi_blob_tiles_off(N);
    h->total_bytes = zmi_blob_bytes(K, N);
    h->src_dtype = src_dtype;
    h->sym_group_size = sym_group_size;
  }
}

hipError_t zmi_launch_prepack(const int8_t *B, int64_t K, int64_t N, int64_t ldb, int transposed,
                              int32_t src_dtype, int32_t sym_group_size, uint8_t *blob,
                              hipStream_t stream) {
  const int64_t K_pad = zmi_blob_kpad(K), N_pad = zmi_blob_npad(N);
  const int64_t kblocks = K_pad / 32;
  uint8_t *tiles = blob + zmi_blob_tiles_off(N);
  int32_t *colsum = (int32_t *)(blob + zmi_blob_colsum_off());
  dim3 grid((unsigned)(K_pad / PP_TK), (unsigned)(N_pad / PP_TN));
  if (transposed)
    hipLaunchKernelGGL(zmi_prepack_kernel<true>, grid, dim3(256), 0, stream, B, K, N, ldb, tiles, kblocks);
  else
    hipLaunchKernelGGL(zmi_prepack_kernel<false>, grid, dim3(256), 0, stream, B, K, N, ldb, tiles, kblocks);
  hipLaunchKernelGGL(zmi_colsum_kernel, dim3((unsigned)(N_pad / 32)), dim3(64), 0, stream, tiles, kblocks,
                     zmi_blob_nb_stride(K), colsum);
  hipLaunchKernelGGL(zmi_blob_header_kernel, dim3(1), dim3(64), 0, stream, (ZmiBlobHeader *)blob, K, N,
                     src_dtype, sym_group_size);
  return hipGetLastError();
}
