// Internals shared by the C ABI translation units.
#pragma once
#include "zmi_host.h"

namespace zmi {
int32_t validate_matmul(const void *src, const void *weight, const void *dst, int M, int N, int K,
                        int Batch_A, int Batch_B, const zmi_matmul_params_t &p, bool is_weights_const);
bool is_dynamic_quant_config(const zmi_matmul_params_t &p);
int32_t build_epilogue(const zmi_matmul_params_t &p, int M, int N, float alpha, float beta, const void *bias,
                       ZmiEpilogue *out, ZmiProblem *prob, bool allow_wei_zp = false);
int32_t run_single_gemm(const ZmiProblem &prob, const ZmiEpilogue &epi, const ZmiRingPlan *plan);
bool a_needs_repack(const void *A, int64_t lda, int K, bool transA);
bool use_ring_kernel(int M, int N, int K);
// weight-only quantization (zmi_api_woq.hip): bf16 source, s4 / u4 weights, no dynamic_quant
bool is_woq_config(const zmi_matmul_params_t &p);
int32_t matmul_woq(char layout, int32_t transA, int32_t transB, int32_t M, int32_t N, int32_t K, float alpha,
                   const void *src, int32_t lda, const void *weight, int32_t ldb, const void *bias, float beta, void *dst,
                   int32_t ldc, int32_t is_weights_const, const zmi_matmul_params_t &p);
}  // namespace zmi
