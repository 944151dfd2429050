// Drives the C++ LowOHA front end (zendnnl_lowoha.hpp) the way a framework plugin
// or the reference's own examples would.  With --validate-only it needs no GPU:
// every call is rejected by validation.  Without it, it runs the deterministic
// recipe of the reference's int8 example (examples/lowoha_matmul_example.cpp:509-535:
// w = (i % 7) - 3, a = (i + 17 * iter) % 256) through matmul_direct, with plain and
// with prepacked weights, and compares the s32 result with a host triple loop; then the reference's W4A8 example.
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
  // (mish on the static scale chain is accepted: what stops this call is the leading dimension, before any launch)
  CHECK(matmul_direct('r', false, false, 4, 8, 16, 1.f, fake, 8, fake, 8, nullptr, 0.f, fake, 8, true, b, q) == status_t::failure);
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

// The reference's W4A8 example as its caller writes it (examples/lowoha_matmul_example.cpp:370-457): M = 8, K = 128,
// N = 64, groups of 32, bf16 ones as activations, every s4 code 1, bf16 weight scales 1 + 0.05 g, a bf16 {M,1}
// source-scale buffer that the dynamic quantization overwrites.  Every row quantizes to 127 with scale 1/127, so the
// output is 32 * sum_g bf16(1 + 0.05 g) = 137.5 up to f32 rounding: 137 or 138 in bf16 (0x4309 / 0x430a).
static uint16_t to_bf16(float f) {
  uint32_t u; std::memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

static void gpu_w4a8_example() {
  const int M = 8, K = 128, N = 64, G = 4;
  std::vector<uint16_t> src_scale(M), wei_scale(G * N), input(M * K, 0x3F80), output(M * N, 0);
  for (int m = 0; m < M; ++m) src_scale[m] = to_bf16(0.02f + 0.001f * m);
  for (int g = 0; g < G; ++g)
    for (int n = 0; n < N; ++n) wei_scale[g * N + n] = to_bf16(1.0f + 0.05f * g);
  std::vector<int8_t> weights((K * N + 1) / 2, (int8_t)0x11);
  void *ss_d, *ws_d, *w_d, *x_d, *y_d;
  hipMalloc(&ss_d, M * 2); hipMalloc(&ws_d, G * N * 2); hipMalloc(&w_d, weights.size()); hipMalloc(&x_d, M * K * 2); hipMalloc(&y_d, M * N * 2);
  hipMemcpy(ss_d, src_scale.data(), M * 2, hipMemcpyHostToDevice);
  hipMemcpy(ws_d, wei_scale.data(), G * N * 2, hipMemcpyHostToDevice);
  hipMemcpy(w_d, weights.data(), weights.size(), hipMemcpyHostToDevice);
  hipMemcpy(x_d, input.data(), M * K * 2, hipMemcpyHostToDevice);
  matmul_params params;
  params.dtypes.src = data_type_t::bf16;
  params.dtypes.wei = data_type_t::s4;
  params.dtypes.dst = data_type_t::bf16;
  params.dtypes.bias = data_type_t::none;
  params.dtypes.compute = data_type_t::s8;
  params.dynamic_quant = true;
  params.lowoha_algo = zendnnl::ops::matmul_algo_t::aocl_dlp_blocked;
  params.quant_params.src_scale.buff = ss_d;
  params.quant_params.src_scale.dt = data_type_t::bf16;
  params.quant_params.src_scale.dims = {M, 1};
  params.quant_params.wei_scale.buff = ws_d;
  params.quant_params.wei_scale.dt = data_type_t::bf16;
  params.quant_params.wei_scale.dims = {G, N};
  matmul_batch_params_t batch_params;
  CHECK(matmul_direct('r', false, false, M, N, K, 1.0f, x_d, K, w_d, N, nullptr, 0.0f, y_d, N, true, batch_params, params) ==
        status_t::success);
  hipMemcpy(output.data(), y_d, M * N * 2, hipMemcpyDeviceToHost);
  hipMemcpy(src_scale.data(), ss_d, M * 2, hipMemcpyDeviceToHost);
  int bad = 0;
  for (int i = 0; i < M * N; ++i) if (output[i] != 0x4309 && output[i] != 0x430a) ++bad;
  CHECK(bad == 0);
  for (int m = 0; m < M; ++m) CHECK(src_scale[m] == to_bf16(1.0f / 127.0f));
  // the validator's outcomes for this path (lowoha_matmul_utils.cpp:72-176)
  params.dtypes.dst = data_type_t::f32;
  CHECK(matmul_direct('r', false, false, M, N, K, 1.0f, x_d, K, w_d, N, nullptr, 0.0f, y_d, N, true, batch_params, params) ==
        status_t::failure);
  params.dtypes.dst = data_type_t::bf16;
  params.dynamic_quant = false;    // bf16 x s4 without dynamic quantization is weight-only quantization: no source scale
  CHECK(matmul_direct('r', false, false, M, N, K, 1.0f, x_d, K, w_d, N, nullptr, 0.0f, y_d, N, true, batch_params, params) ==
        status_t::failure);
  params.quant_params.src_scale.buff = nullptr;
  params.quant_params.src_scale.dims.clear();
  params.dtypes.compute = data_type_t::none;
  CHECK(matmul_direct('r', false, false, M, N, K, 1.0f, x_d, K, w_d, N, nullptr, 0.0f, y_d, N, true, batch_params, params) ==
        status_t::success);
  clear_matmul_weight_caches();
  hipFree(ss_d); hipFree(ws_d); hipFree(w_d); hipFree(x_d); hipFree(y_d);
}

int main(int argc, char **argv) {
  // The validation cases hand the library addresses that are no memory: they run where no device can be launched on
  // (a case that slipped past the validators then stops at the device check), never in front of the GPU examples.
  if (argc > 1 && std::strcmp(argv[1], "--validate-only") == 0) validate_only();
  else { gpu_example(); gpu_w4a8_example(); }
  std::printf(fails ? "adapter example: %d check(s) failed\n" : "adapter example: ok\n", fails);
  return fails ? 1 : 0;
}
