"""GPU parity of matmul_direct with GGML Q8_0 packed weights (pack_format_b = 1): the library unpacks the
[N][K/32] blocks of {fp16 d, int8 qs[32]} into s8 rows and bf16 {K/32, N} scales, caches the reordered
weights per pointer, and runs the per-group symmetric GEMM with groups of 32 (reference:
lowoha_operators/matmul/ggml_weight_unpack.cpp:155-236, 367-480; lowoha_matmul.cpp:389-401)."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _pack(rows, d16):
    N, K = rows.shape
    blk = np.zeros((N, K // 32, 34), dtype=np.uint8)
    blk[:, :, :2] = d16.view(np.uint16).reshape(N, K // 32, 1).view(np.uint8)
    blk[:, :, 2:] = rows.reshape(N, K // 32, 32).view(np.uint8)
    return blk.reshape(-1)


def _weights(rng, N, K):
    rows = rng.integers(-127, 128, (N, K), dtype=np.int8)
    d16 = rng.uniform(1e-3, 0.02, (N, K // 32)).astype(np.float16)
    return rows, d16, _pack(rows, d16)


@pytest.mark.parametrize("M,K,N", [(1, 64, 16), (16, 4096, 96), (5, 512, 33), (40, 256, 70), (130, 1024, 48), (7, 32, 50),
                                   (300, 512, 260)])   # (the last one: the MFMA-tiled per-group kernel, groups of 32)
@pytest.mark.parametrize("dst_dt", [capi.DT_F32, capi.DT_BF16])
def test_static_s8_rows_with_q8_0_weights(zo, M, K, N, dst_dt):
    rng = np.random.default_rng(M + K + N)
    G = K // 32
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    rows, d16, packed = _weights(rng, N, K)
    ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    a_d, w_d, ss_d = H.to_dev(a), H.to_dev(packed), H.to_dev(ss)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
    p.pack_format_b = 1
    dst = torch.zeros((M, N), dtype=torch.float32 if dst_dt == capi.DT_F32 else torch.bfloat16, device=H.DEV)
    for _ in range(2):                          # the second call finds the unpacked weights in the cache
        dst.zero_()
        st = lowoha.matmul_direct("r", False, True, M, N, K, 1.0, a_d, K, w_d, K, H.to_dev(bias), 0.0, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        assert lowoha.last_kernel().startswith("pergroup_") or K == 32   # (one group: the per-token chain is the same arithmetic)
        ph = H.host_params(p, src_scale=ss)
        keep = []
        st, want, _, _ = zo.matmul_int8(a, packed, ph.flat(keep), M, N, K, bias=bias, transB=True, ldb=K)
        assert st == capi.SUCCESS
        assert np.array_equal(H.to_host(dst), want)     # no activation: every step is a correctly rounded f32 operation
    capi.load().zmi_clear_weight_cache()


@pytest.mark.parametrize("M,K,N", [(16, 4096, 256), (3, 128, 40), (70, 512, 64), (20, 32, 36), (257, 1024, 130)])
def test_dynamic_bf16_rows_with_q8_0_weights(zo, M, K, N):
    rng = np.random.default_rng(M * 3 + K + N)
    G = K // 32
    x = H.bf16_bits((rng.standard_normal((M, K)) * 2).astype(np.float32))
    rows, d16, packed = _weights(rng, N, K)
    x_d, w_d = H.to_dev(x), H.to_dev(packed)
    scales_d = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, G))
    p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    p.pack_format_b = 1
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, True, M, N, K, 1.0, x_d, K, w_d, K, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=None)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, packed, ph.flat(keep), M, N, K, transB=True, ldb=K, want_scales=True,
                                         n_scales=M * G)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(scales_d), scales)
    H.check_bf16(H.to_host(dst), want, max_frac=1e-2)
    if M >= 129:
        assert lowoha.last_kernel() == "pergroup_ring_mfma32x32x32"
    capi.load().zmi_clear_weight_cache()


def test_q8_0_rejections(zo):
    M, K, N = 4, 64, 8
    G = K // 32
    rng = np.random.default_rng(1)
    rows, d16, packed = _weights(rng, N, K)
    a_d, w_d = H.to_dev(np.ones((M, K), dtype=np.int8)), H.to_dev(packed)
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)

    def call(transB=True, const=True, scale_dims=(M, G), src=capi.DT_S8, K_=K):
        ss_d = torch.ones(int(np.prod(scale_dims)), dtype=torch.float32, device=H.DEV)
        p = lowoha.MatmulParams(src=src, wei=capi.DT_S8, dst=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, scale_dims)
        p.pack_format_b = 1
        return lowoha.matmul_direct("r", False, transB, M, N, K_, 1.0, a_d, K, w_d, K, None, 0.0, dst, N, const, p)

    assert call() == capi.SUCCESS
    assert call(transB=False) == capi.FAILURE              # the packed layout is N x K
    assert call(const=False) == capi.FAILURE               # cached unpack needs constant weights
    assert call(scale_dims=(1,)) == capi.FAILURE           # per-group symmetric int8 only
    assert call(src=capi.DT_U8) == capi.FAILURE
    assert call(scale_dims=(M, 1)) == capi.UNIMPLEMENTED   # per-token rows with packed per-group weights: not in this build
    assert call(K_=48, scale_dims=(M, 1)) == capi.FAILURE  # K % 32 != 0
    capi.load().zmi_clear_weight_cache()
