// Drives the C++ LowOHA front end (zendnnl_lowoha.hpp) the way a framework plugin
// or the reference's own examples would.  With --validate-only it needs no GPU:
// every call is rejected by validation.  Without it, it runs the deterministic
// recipe of the reference's int8 example (examples/lowoha_matmul_example.cpp:509-535:
// w = (i % 7) - 3, a = (i + 17 * iter) % 256) through matmul_direct, with plain and
// with prepacked weights, and compares the s32 result with a host triple loop.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <vector>

#include "zendnnl_lowoha.hpp"

using namespace zendnnl::lowoha::matmul;
using namespace zendnnl::lowoha::reorder;
using zendnnl::memory::data_type_t;
using zendnnl::memory::status_t;

static int fails = 0;
#define CHECK(cond)                                                   \
  do {                                                                \
    if (!(cond)) {                                                    \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
      ++fails;                                                        \
    }                                                                 \
  } while (0)

static void validate_only() {
  void *fake = reinterpret_cast<void *>(0x1000);
  matmul_params p;
  p.dtypes.src = data_type_t::u8;
  p.dtypes.wei = data_type_t::s8;
  p.dtypes.dst = data_type_t::f32;
  matmul_batch_params_t b;
  CHECK(matmul_direct('r', false, false, 4, 8, 16, 1.f, nullptr, 16, fake, 8, nullptr, 0.f, fake, 8, true, b, p) == status_t::failure);
  CHECK(matmul_direct('r', false, false, 0, 8, 16, 1.f, fake, 16, fake, 8, nullptr, 0.f, fake, 8, true, b, p) == status_t::failure);
  matmul_params q = p;
  q.postop_.resize(1);
  q.postop_[0].po_type = zendnnl::ops::post_op_type_t::mish;
  CHECK(matmul_direct('r', false, false, 4, 8, 16, 1.f, fake, 16, fake, 8, nullptr, 0.f, fake, 8, true, b, q) == status_t::failure);
  matmul_params bf;
  bf.dtypes.src = bf.dtypes.wei = bf.dtypes.dst = data_type_t::bf16;
  CHECK(matmul_direct('r', false, false, 4, 8, 16, 1.f, fake, 16, fake, 8, nullptr, 0.f, fake, 8, true, b, bf) == status_t::unimplemented);
  reorder_params_t rp;
  rp.is_prepack = true;
  rp.prepack.algo = zendnnl::ops::matmul_algo_t::aocl_dlp_blocked;
  rp.prepack.wei_dtype = data_type_t::s8;
  rp.prepack.src_dtype = data_type_t::u8;
  rp.prepack.K = 100; rp.prepack.N = 37; rp.prepack.ldb = 37;
  size_t sz = weight_prepack_size(rp);
  CHECK(sz > 0 && sz % 64 == 0 && rp.prepack.cached_size == sz);
  rp.prepack.ldb = 10;
  CHECK(weight_prepack_size(rp) == 0);
  CHECK(reorder_direct(fake, fake, rp) == status_t::failure);
  // group call: vector size mismatch
  std::vector<matmul_params> ps(2, p);
  CHECK(group_matmul_direct({'r', 'r'}, {false, false}, {false, false}, {4, 4}, {8}, {16, 16}, {1.f, 1.f},
                            {fake, fake}, {16, 16}, {fake, fake}, {8, 8}, {nullptr, nullptr}, {0.f, 0.f},
                            {fake, fake}, {8, 8}, {true, true}, ps) == status_t::failure);
}

static void gpu_example() {
  const int M = 48, K = 320, N = 200;
  std::vector<int8_t> w(K * N);
  for (int i = 0; i < K * N; ++i) w[i] = static_cast<int8_t>((i % 7) - 3);
  int8_t *w_d; uint8_t *a_d; int32_t *c_d;
  hipMalloc(&w_d, w.size()); hipMalloc(&a_d, M * K); hipMalloc(&c_d, M * N * 4);
  hipMemcpy(w_d, w.data(), w.size(), hipMemcpyHostToDevice);
  reorder_params_t rp;
  rp.is_prepack = true;
  rp.prepack.algo = zendnnl::ops::matmul_algo_t::aocl_dlp_blocked;
  rp.prepack.wei_dtype = data_type_t::s8;
  rp.prepack.src_dtype = data_type_t::u8;
  rp.prepack.K = K; rp.prepack.N = N; rp.prepack.ldb = N;
  const size_t sz = weight_prepack_size(rp);
  void *blob; hipMalloc(&blob, sz);
  CHECK(reorder_direct(w_d, blob, rp) == status_t::success);
  int32_t zp = 128;
  for (int iter = 0; iter < 3; ++iter) {
    std::vector<uint8_t> a(M * K);
    for (int i = 0; i < M * K; ++i) a[i] = static_cast<uint8_t>((i + 17 * iter) % 256);
    hipMemcpy(a_d, a.data(), a.size(), hipMemcpyHostToDevice);
    for (int packed = 0; packed < 2; ++packed) {
      matmul_params p;
      p.dtypes.src = data_type_t::u8; p.dtypes.wei = data_type_t::s8; p.dtypes.dst = data_type_t::s32;
      p.quant_params.src_zp.buff = &zp; p.quant_params.src_zp.dt = data_type_t::s32; p.quant_params.src_zp.dims = {1};
      if (packed) { p.mem_format_b = 'r'; p.lowoha_algo = zendnnl::ops::matmul_algo_t::aocl_dlp_blocked; }
      matmul_batch_params_t b;
      hipMemset(c_d, 0xff, M * N * 4);
      status_t st = matmul_direct('r', false, false, M, N, K, 1.f, a_d, K, packed ? blob : (void *)w_d, N, nullptr, 0.f,
                                  c_d, N, true, b, p);
      CHECK(st == status_t::success);
      std::vector<int32_t> c(M * N);
      hipMemcpy(c.data(), c_d, c.size() * 4, hipMemcpyDeviceToHost);
      int bad = 0;
      for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
          int64_t s = 0;
          for (int k = 0; k < K; ++k) s += (int64_t)((int)a[m * K + k] - 128) * w[k * N + n];
          if (c[m * N + n] != (int32_t)s) ++bad;
        }
      CHECK(bad == 0);
    }
  }
  clear_matmul_weight_caches();
  hipFree(w_d); hipFree(a_d); hipFree(c_d); hipFree(blob);
}

int main(int argc, char **argv) {
  validate_only();
  if (!(argc > 1 && std::strcmp(argv[1], "--validate-only") == 0)) gpu_example();
  std::printf(fails ? "adapter example: %d check(s) failed\n" : "adapter example: ok\n", fails);
  return fails ? 1 : 0;
}
