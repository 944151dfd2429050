"""GPU parity of the batched form of matmul_direct (Batch_A / Batch_B > 1) through the C ABI.

Reference: bmm_execute, zendnnl/src/lowoha_operators/matmul/partitioning/bmm/looper/bmm_looper.cpp:192-223
(strides) and :326-340 (batch b = src batch b % Batch_A, weight batch b % Batch_B, dst batch b);
apply_bmm_postop_offsets, matmul/lowoha_matmul_utils.cpp:36-70 (3-D binary operands advance per batch).
The expected values are the oracle's single product on each batch's slices, taken by numpy indexing
(so the stride arithmetic of the library is checked against an independent one).  Bars as for the
single product: s32 bit-exact, f32 identical chain, bf16 within one ulp."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _oracle(zo, p_host, src, w, M, N, K, **kw):
    keep = []
    flat = p_host.flat(keep)
    st, dst, acc, scales = zo.matmul_int8(np.ascontiguousarray(src), np.ascontiguousarray(w), flat, M, N, K, **kw)
    assert st == capi.SUCCESS
    return dst


@pytest.mark.parametrize("BA,BB", [(4, 4), (1, 3), (3, 1), (4, 2), (2, 6)])
@pytest.mark.parametrize("M,K,N", [(8, 128, 96), (130, 256, 64), (64, 64, 200)])
def test_s8_batches_s32_bit_exact_with_broadcast(zo, BA, BB, M, K, N):
    rng = np.random.default_rng(BA * 100 + BB * 10 + M)
    B = max(BA, BB)
    a = rng.integers(-128, 128, (BA, M, K), dtype=np.int8)
    w = rng.integers(-127, 128, (BB, K, N), dtype=np.int8)
    dst = torch.full((B, M, N), -7, dtype=torch.int32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N,
                              False, p, batch_a=BA, batch_b=BB)
    assert st == capi.SUCCESS, lowoha.last_error()
    got = H.to_host(dst)
    for b in range(B):
        want, ov = zo.gemm_s32(a[b % BA], w[b % BB])
        assert ov == 0
        assert np.array_equal(got[b], want), f"batch {b}"


def test_explicit_strides_transposed_weights_and_padding(zo):
    """Strides in elements larger than the matrices, leading dimensions larger than the rows, transB
    (attention-score shape: Q x K^T per head) and a destination with gaps that must stay untouched."""
    rng = np.random.default_rng(11)
    B, M, K, N = 5, 40, 64, 72
    lda, ldb, ldc = K + 16, K + 32, N + 8
    s_src, s_wei, s_dst = M * lda + 64, N * ldb + 128, M * ldc + 24
    a = rng.integers(-128, 128, (B, s_src), dtype=np.int8)
    w = rng.integers(-127, 128, (B, s_wei), dtype=np.int8)
    dst = torch.full((B, s_dst), 12345, dtype=torch.int32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    st = lowoha.matmul_direct("r", False, True, M, N, K, 1.0, H.to_dev(a), lda, H.to_dev(w), ldb, None, 0.0, dst, ldc,
                              False, p, batch_a=B, batch_b=B, batch_strides=(s_src, s_wei, s_dst))
    assert st == capi.SUCCESS, lowoha.last_error()
    got = H.to_host(dst)
    for b in range(B):
        ab = a[b, :M * lda].reshape(M, lda)[:, :K]
        wb = w[b, :N * ldb].reshape(N, ldb)[:, :K].T              # stored [N, K]: the product uses its transpose
        want, ov = zo.gemm_s32(np.ascontiguousarray(ab), np.ascontiguousarray(wb))
        assert ov == 0
        full = got[b, :M * ldc].reshape(M, ldc)
        assert np.array_equal(full[:, :N], want), f"batch {b}"
        assert np.all(full[:, N:] == 12345) and np.all(got[b, M * ldc:] == 12345)


@pytest.mark.parametrize("dst_dt", [capi.DT_F32, capi.DT_BF16])
def test_u8_batches_scales_bias_and_3d_binary_post_ops(zo, dst_dt):
    """Static u8 quantization shared by all batches, a bias, a 3-D add operand with one slice per batch,
    a 3-D mul operand with batch dimension 1 (shared) and an element-wise op behind them."""
    rng = np.random.default_rng(23)
    BA, BB, M, K, N = 3, 1, 24, 192, 128
    a = rng.integers(0, 256, (BA, M, K), dtype=np.uint8)
    w = rng.integers(-127, 128, (BB, K, N), dtype=np.int8)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ss = np.array([0.03], dtype=np.float32)
    zp = np.array([121], dtype=np.int32)
    bias = rng.standard_normal(N).astype(np.float32)
    add = rng.standard_normal((BA, M, N)).astype(np.float32)
    mul = rng.uniform(0.5, 1.5, (1, M, N)).astype(np.float32)
    ws_d, ss_d, zp_d, bias_d, add_d, mul_d = (H.to_dev(x) for x in (ws, ss, zp, bias, add, mul))
    tdt = torch.float32 if dst_dt == capi.DT_F32 else torch.bfloat16
    dst = torch.zeros((BA, M, N), dtype=tdt, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (1,))
    p.src_zp = lowoha.QuantParam(zp_d, capi.DT_S32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add_d, capi.DT_F32, (BA, M, N)),
                 lowoha.PostOp(capi.PO_BINARY_MUL, mul_d, capi.DT_F32, (1, M, N)),
                 lowoha.PostOp(capi.PO_RELU)]
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, bias_d, 0.0, dst, N,
                              True, p, batch_a=BA, batch_b=BB)
    assert st == capi.SUCCESS, lowoha.last_error()
    for b in range(BA):
        ph = H.host_params(p, src_scale=ss, src_zp=zp, wei_scale=ws)
        ab, mb = np.ascontiguousarray(add[b]), np.ascontiguousarray(mul[0])
        ph.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, ab.ctypes.data, capi.DT_F32, (M, N)),
                      lowoha.PostOp(capi.PO_BINARY_MUL, mb.ctypes.data, capi.DT_F32, (M, N)),
                      lowoha.PostOp(capi.PO_RELU)]
        want = _oracle(zo, ph, a[b], w[0], M, N, K, bias=bias)
        if dst_dt == capi.DT_F32:
            assert np.array_equal(H.to_host(dst[b]), want), f"batch {b}"
        else:
            H.check_bf16(H.to_host(dst[b]), want)


def test_one_batch_with_3d_operand_reads_like_2d(zo):
    rng = np.random.default_rng(5)
    M, K, N = 16, 64, 64
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    add = rng.standard_normal((1, M, N)).astype(np.float32)
    add_d = H.to_dev(add)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    p.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add_d, capi.DT_F32, (1, M, N))]
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    acc, _ = zo.gemm_s32(a, w)
    assert np.array_equal(H.to_host(dst), acc.astype(np.float32) + add[0])


def test_batched_forms_that_are_refused():
    rng = np.random.default_rng(1)
    M, K, N = 8, 64, 64
    a = H.to_dev(rng.integers(-128, 128, (6, M, K), dtype=np.int8))
    w = H.to_dev(rng.integers(-127, 128, (4, K, N), dtype=np.int8))
    dst = torch.zeros((6, M, N), dtype=torch.int32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a, K, w, N, None, 0.0, dst, N, False, p, batch_a=6, batch_b=4)
    assert st == capi.FAILURE and "broadcast" in lowoha.last_error()
    x = torch.zeros((2, M, K), dtype=torch.bfloat16, device=H.DEV)
    pd = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    pd.dynamic_quant = True
    pd.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    pd.wei_scale = lowoha.QuantParam(torch.ones(N, device=H.DEV), capi.DT_F32, (1, N))
    out = torch.zeros((2, M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, K, w, N, None, 0.0, out, N, True, pd, batch_a=2, batch_b=1)
    assert st == capi.UNIMPLEMENTED
    # a 3-D operand with fewer slices than batches
    add = torch.zeros((2, M, N), dtype=torch.float32, device=H.DEV)
    pf = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    pf.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add, capi.DT_F32, (2, M, N))]
    outf = torch.zeros((4, M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a, K, w, N, None, 0.0, outf, N, False, pf, batch_a=4, batch_b=4)
    assert st == capi.FAILURE
