// zmi_matmul_direct_noalloc: the decode-shaped matmul_direct call with run-time (per-token) quantization
// of its source rows, for callers that must not allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid it).  Same arithmetic and kernels as zmi_matmul_direct on
// the same arguments; the only difference is where the quantized rows and their scales live between
// the quantization launch and the GEMM launch: in a fixed array inside the library's device image
// instead of the calling thread's grow-only arena.
#include <cstring>
#include <mutex>

#include "zmi_api.h"
#include "zmi_host.h"

#define ZMI_NOALLOC_MAX_M 128
#define ZMI_NOALLOC_MAX_KPAD 4096

namespace {

constexpr size_t kRowsBytes = (size_t)ZMI_NOALLOC_MAX_M * ZMI_NOALLOC_MAX_KPAD;   // s8 rows, leading dimension K16
constexpr size_t kScalesOff = kRowsBytes;                                         // 128 f32 scales
constexpr size_t kAmaxOff = kScalesOff + 1024;                                    // per-tensor maximum (one word)
constexpr size_t kScratchBytes = kAmaxOff + 1024;

// Every GPU the library runs on holds its own copy of this array until the process ends.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

// Device address of the current device's copy of the array (its name is only a host-side stand-in).
unsigned char *scratch_of_current_device() {
  int dev = 0;
  if (!zmi::hip_ok(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) { zmi::set_error("device index out of range"); return nullptr; }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    if (!zmi::hip_ok(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
    g_scratch_ptr[dev] = (unsigned char *)p;
  }
  return g_scratch_ptr[dev];
}

}  // namespace

namespace zmi {
bool noalloc_setup() { return scratch_of_current_device() != nullptr; }
}  // namespace zmi

using namespace zmi;

extern "C" int32_t zmi_matmul_direct_noalloc(char layout, int32_t transA, int32_t transB, int32_t M, int32_t N, int32_t K,
                                             float alpha, const void *src, int32_t lda, const void *weight, int32_t ldb,
                                             const void *bias, float beta, void *dst, int32_t ldc, int32_t is_weights_const,
                                             const zmi_batch_params_t *batch_params, const zmi_matmul_params_t *params) {
  clear_error();
  (void)ldb;
  note_operand(src); note_operand(weight); note_operand(dst); note_operand(bias);
  // a hand-off of an earlier launch on this thread that gave up is reported here, as zmi_matmul_direct does
  if (async_failure_pending()) return ZMI_FAILURE;
  if (!params) { set_error("null params"); return ZMI_FAILURE; }
  const zmi_matmul_params_t &p = *params;
  const int Batch_A = batch_params ? batch_params->Batch_A : 1;
  const int Batch_B = batch_params ? batch_params->Batch_B : 1;
  int32_t st = validate_matmul(src, weight, dst, M, N, K, Batch_A, Batch_B, p, is_weights_const != 0);
  if (st != ZMI_SUCCESS) return st;
  // ---- the part of matmul_direct this entry point serves ----
  if (layout != 'r' && layout != 'R') { set_error("only row-major layout is implemented"); return ZMI_UNIMPLEMENTED; }
  if (Batch_A != 1 || Batch_B != 1) { set_error("batched matmul is not implemented"); return ZMI_UNIMPLEMENTED; }
  if (!is_dynamic_quant_config(p) || p.dt_compute != ZMI_DT_S8) {
    set_error("zmi_matmul_direct_noalloc serves bf16 / f32 sources with dynamic_quant and s8 compute");
    return ZMI_UNIMPLEMENTED;
  }
  if (p.mem_format_b != 'r' || p.pack_format_b != 0) {
    set_error("zmi_matmul_direct_noalloc takes prepacked weights only (mem_format_b 'r': packing would allocate)");
    return ZMI_UNIMPLEMENTED;
  }
  if (p.lowoha_algo != ZMI_ALGO_AOCL_DLP_BLOCKED) { set_error("mem_format_b == 'r' requires lowoha_algo == aocl_dlp_blocked"); return ZMI_FAILURE; }
  if (transA || transB) { set_error("zmi_matmul_direct_noalloc: no transposed operands"); return ZMI_UNIMPLEMENTED; }
  if (M > ZMI_NOALLOC_MAX_M || zmi_blob_kpad(K) > ZMI_NOALLOC_MAX_KPAD) {
    set_error("zmi_matmul_direct_noalloc: at most 128 rows and K <= 4096 (the fixed scratch array holds no more)");
    return ZMI_FAILURE;
  }
  if (lda < K || ldc < N) { set_error("leading dimension too small"); return ZMI_FAILURE; }
  if (p.src_zp.buff) { set_error("dynamic quantization is symmetric: no source zero-point"); return ZMI_FAILURE; }
  int64_t scale_n = 1;
  for (int i = 0; i < p.src_scale.ndims; ++i) scale_n *= p.src_scale.dims[i];
  if (!(scale_n == 1 || scale_n == M)) {
    set_error("zmi_matmul_direct_noalloc: source scale dims must be {1} or {M,1}");
    return scale_n > M ? ZMI_UNIMPLEMENTED : ZMI_FAILURE;
  }
  const int32_t sdt = p.src_scale.dt == ZMI_DT_NONE ? ZMI_DT_F32 : p.src_scale.dt;
  if (sdt != ZMI_DT_F32 && sdt != ZMI_DT_BF16) { set_error("source scale must be f32 or bf16"); return ZMI_FAILURE; }
  if (!ensure_device()) return ZMI_FAILURE;
  if (p.src_scale.buff && !is_device_pointer(p.src_scale.buff)) {
    set_error("dynamic_quant: src_scale.buff receives the computed scales and must be device memory (or null)");
    return ZMI_FAILURE;
  }
  if (!blob_matches(weight, K, N)) return ZMI_FAILURE;   // (the first call with a blob reads its header back; later ones do not)

  unsigned char *sc = scratch_of_current_device();
  if (!sc) return ZMI_FAILURE;
  int8_t *q = (int8_t *)sc;
  float *scales = (float *)(sc + kScalesOff);
  unsigned int *amax = (unsigned int *)(sc + kAmaxOff);
  const int64_t K16 = zmi_round_up(K, 16);

  zmi_matmul_params_t ep = p;   // working copy
  ZmiProblem prob;
  std::memset(&prob, 0, sizeof(prob));
  prob.blob = (const uint8_t *)weight;
  prob.dst = dst; prob.ldc = ldc;
  prob.M = M; prob.N = N; prob.K = K;
  prob.A = q; prob.lda = K16; prob.a_is_u8 = 0;
  // (bytes of a row between K and K16 keep what an earlier call left there: they meet the blob's zero rows)
  if (scale_n == M && M > 1) {
    // the scales go to the caller's buffer when there is one, in the dtype the params name; the GEMM reads them there
    void *scale_out = p.src_scale.buff ? (void *)p.src_scale.buff : (void *)scales;
    if (!hip_ok(zmi_launch_quant_rows(src, p.dt_src, M, K, lda, q, K16, 0, scale_out, sdt, stream()), "quant launch")) return ZMI_FAILURE;
    ep.src_scale.buff = scale_out;
    ep.src_scale.dt = sdt;
    ep.src_scale.ndims = 2; ep.src_scale.dims[0] = M; ep.src_scale.dims[1] = 1;
  } else {
    // one scale for the whole tensor (M == 1 included); the word the maximum is collected in is cleared by the launch itself
    if (!hip_ok(zmi_launch_quant_tensor(src, p.dt_src, M, K, lda, q, K16, 0, scales, amax, stream()), "quant launch")) return ZMI_FAILURE;
    if (sdt == ZMI_DT_BF16) {
      if (!hip_ok(zmi_launch_narrow_scales(scales, M, (void *)p.src_scale.buff, 1, stream()), "scale narrowing launch")) return ZMI_FAILURE;
    } else if (p.src_scale.buff) {
      if (!hip_ok(hipMemcpyAsync((void *)p.src_scale.buff, scales, sizeof(float), hipMemcpyDeviceToDevice, stream()), "hipMemcpyAsync(scale)"))
        return ZMI_FAILURE;
    }
    ep.src_scale.buff = scales;
    ep.src_scale.dt = ZMI_DT_F32;
    ep.src_scale.ndims = 1; ep.src_scale.dims[0] = 1;
  }
  ep.dt_src = ZMI_DT_S8;
  ZmiEpilogue epi;
  st = build_epilogue(ep, M, N, alpha, beta, bias, &epi, &prob);
  if (st != ZMI_SUCCESS) return st;
  set_kernel_name(zmi_decode_16row_kernel(prob, false) ? "decode16_dma_rows_mfma16x16x64 (static scratch)"
                                                       : "decode_lds_rows_mfma16x16x64 (static scratch)");
  if (!hip_ok(zmi_launch_gemm_decode(prob, epi, nullptr, stream()), "decode GEMM launch")) return ZMI_FAILURE;
  return ZMI_SUCCESS;
}
