"""GPU parity of the per-group GEMM at large M (the MFMA-tiled kernel with the scales staged through LDS):
against the oracle bit for bit on f32 results (reference arithmetic: operators/matmul/matmul_ref_kernel.cpp:917-1001,
every group's term rounded at each step and added in group order), and against the library's own
one-wavefront-per-column-block kernel, which the environment switch ZMI_PGRING_MIN_M=0 brings back."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.test_gpu_reorder_edges import _run_both

pytestmark = pytest.mark.gpu

RING = "pergroup_ring_mfma32x32x32"


@pytest.fixture(autouse=True)
def _tiled_kernel_from_96_rows(monkeypatch):
    """The library takes the tiled kernel from 129 rows (below that its few tiles leave most compute units idle);
    these tests reach its 128-row tile and ragged single tiles by lowering the switch."""
    monkeypatch.setenv("ZMI_PGRING_MIN_M", "96")


def _scales(rng, M, N, G):
    ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    return ss, ws


# (M, K, N, G): groups of 32 (two per 64-k slot), 64, 128, 256, 384 and 512; 128- and 256-row tiles with ragged last
# tiles in both directions; one and several slots; more slots than the ring holds
SHAPES = [(96, 64, 32, 2), (97, 128, 100, 4), (128, 256, 256, 8), (129, 512, 130, 16), (300, 1024, 257, 32),
          (257, 128, 515, 2), (130, 192, 48, 3), (513, 640, 129, 10), (256, 128, 128, 2),
          (100, 256, 70, 2), (255, 1024, 384, 8), (260, 2048, 200, 16), (1000, 512, 300, 4),
          (200, 512, 96, 2), (131, 768, 260, 3), (400, 768, 64, 2), (150, 1536, 33, 3), (99, 2048, 512, 4)]


@pytest.mark.parametrize("M,K,N,G", SHAPES)
def test_static_f32_bit_exact_against_the_oracle(zo, M, K, N, G):
    rng = np.random.default_rng(M * 7 + K + N + G)
    ss, ws = _scales(rng, M, N, G)
    bias = rng.standard_normal(N).astype(np.float32)
    for transA, transB, pad, with_bias in ((False, False, 0, True), (True, True, 3, False)):
        a = rng.integers(-128, 128, (K, M + pad) if transA else (M, K + pad), dtype=np.int8)
        w = rng.integers(-127, 128, (N, K + pad) if transB else (K, N + pad), dtype=np.int8)
        ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32,
                                bias=capi.DT_F32 if with_bias else capi.DT_NONE)
        p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
        p.weight_cache_type = 0
        got, want = _run_both(zo, p, a, w, M, N, K, bias=bias if with_bias else None,
                              host_bufs={"src_scale": ss, "wei_scale": ws}, lda=a.shape[1], ldb=w.shape[1],
                              ldc=N + 3, transA=transA, transB=transB)
        assert lowoha.last_kernel() == RING
        bad = np.argwhere(got[:, :N] != want[:, :N])
        assert len(bad) == 0, (M, K, N, G, transA, transB, len(bad), bad[:8].tolist())
        assert np.all(got[:, N:] == 0)


def _dyn_call(x_d, w_d, ws_d, ws_dt, bias_d, M, K, N, G, src_dt, dst_dt, postops=(), alpha=1.0, beta=0.0, dst0=None,
              scale_dt=capi.DT_F32):
    scales_d = torch.zeros(M * G, dtype=torch.float32 if scale_dt == capi.DT_F32 else torch.bfloat16, device=H.DEV)
    p = lowoha.MatmulParams(src=src_dt, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_S8,
                            bias=capi.DT_F32 if bias_d is not None else capi.DT_NONE)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, scale_dt, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, ws_dt, (G, N))
    p.postop_ = list(postops)
    p.weight_cache_type = 0
    dst = dst0.clone() if dst0 is not None else torch.zeros((M, N), dtype=torch.float32 if dst_dt == capi.DT_F32
                                                            else torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, alpha, x_d, K, w_d, N, bias_d, beta, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    return dst, scales_d, lowoha.last_kernel()


@pytest.mark.parametrize("M,K,N,G", [(150, 1024, 96, 8), (300, 512, 200, 16), (128, 4096, 320, 32), (2048, 1024, 256, 8),
                                     (257, 512, 130, 2)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_dynamic_per_group_against_the_oracle(zo, M, K, N, G, src_dt):
    """Rows quantized per (row, group) by the library, then the per-group GEMM: scales and f32 output bit-exact."""
    rng = np.random.default_rng(M + K + G)
    x32 = (rng.standard_normal((M, K)) * rng.uniform(0.2, 3.0, (M, 1))).astype(np.float32)
    x32[0, 3] = np.nan
    x = H.bf16_bits(x32) if src_dt == capi.DT_BF16 else x32
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    dst, scales_d, kernel = _dyn_call(x_d, w_d, ws_d, capi.DT_F32, H.to_dev(bias), M, K, N, G, src_dt, capi.DT_F32)
    assert kernel == RING
    p = lowoha.MatmulParams(src=src_dt, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8, bias=capi.DT_F32)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, w, ph.flat(keep), M, N, K, bias=bias, want_scales=True, n_scales=M * G)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(scales_d), scales)
    assert np.array_equal(H.to_host(dst), want)


CASES = [
    # (M, K, N, G, dst, weight scale dtype, source scale dtype, post-ops, alpha, beta)
    (200, 512, 300, 4, capi.DT_BF16, capi.DT_F32, capi.DT_F32, (), 1.0, 0.0),
    (200, 512, 300, 4, capi.DT_BF16, capi.DT_BF16, capi.DT_BF16, (capi.PO_SWISH,), 1.0, 0.0),
    (130, 256, 101, 8, capi.DT_F32, capi.DT_BF16, capi.DT_F32, (capi.PO_GELU_TANH,), 1.0, 0.0),
    (300, 1024, 64, 16, capi.DT_F32, capi.DT_F32, capi.DT_F32, (capi.PO_RELU,), 0.5, 1.5),
    (257, 768, 258, 2, capi.DT_BF16, capi.DT_F32, capi.DT_F32, (capi.PO_GELU_ERF, capi.PO_TANH), 1.0, 0.25),
    (512, 2048, 512, 16, capi.DT_BF16, capi.DT_F32, capi.DT_F32, (), 1.0, 0.0),
    (1024, 4096, 256, 128, capi.DT_F32, capi.DT_F32, capi.DT_F32, (), 1.0, 0.0),
]


@pytest.mark.parametrize("M,K,N,G,dst_dt,ws_dt,ss_dt,pos,alpha,beta", CASES)
def test_same_bits_as_the_column_block_kernel(monkeypatch, M, K, N, G, dst_dt, ws_dt, ss_dt, pos, alpha, beta):
    """Dynamic quantization, both destinations, bf16 scales, bias, post-ops, alpha / beta: the two kernels run the
    same arithmetic in the same order, so every stored bit agrees."""
    rng = np.random.default_rng(M + K + N + G)
    x = H.gen_bf16_normal(rng, (M, K), std=1.5)
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    x_d, w_d, bias_d = H.to_dev(x), H.to_dev(w), H.to_dev(bias)
    ws_d = H.to_dev(H.bf16_bits(ws) if ws_dt == capi.DT_BF16 else ws)
    tdt = torch.float32 if dst_dt == capi.DT_F32 else torch.bfloat16
    dst0 = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).to(H.DEV).to(tdt)
    postops = [lowoha.PostOp(po) for po in pos]
    args = (x_d, w_d, ws_d, ws_dt, bias_d, M, K, N, G, capi.DT_BF16, dst_dt, postops, alpha, beta, dst0, ss_dt)
    got, sc_got, kernel = _dyn_call(*args)
    assert kernel == RING
    monkeypatch.setenv("ZMI_PGRING_MIN_M", "0")
    want, sc_want, kernel = _dyn_call(*args)
    assert kernel == "pergroup_mfma16x16x64"
    assert torch.equal(sc_got.view(torch.uint8), sc_want.view(torch.uint8))
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))


def test_binary_post_ops_and_rows_below_the_switch(zo, monkeypatch):
    """A {M,N} binary add and a {1,N} binary multiply through the tile epilogue; the row count from which the tiled
    kernel is taken can be lowered through the environment."""
    rng = np.random.default_rng(11)
    M, K, N, G = 140, 256, 90, 2
    ss, ws = _scales(rng, M, N, G)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    add = rng.standard_normal((M, N)).astype(np.float32)
    mul = rng.uniform(0.5, 1.5, (1, N)).astype(np.float32)
    add_d, mul_d = H.to_dev(add), H.to_dev(mul)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    p.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add_d, capi.DT_F32, (M, N)),
                 lowoha.PostOp(capi.PO_BINARY_MUL, mul_d, capi.DT_F32, (1, N))]
    p.weight_cache_type = 0
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == RING
    ph = H.host_params(p, src_scale=ss, wei_scale=ws)
    ph.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add.ctypes.data, capi.DT_F32, (M, N)),
                  lowoha.PostOp(capi.PO_BINARY_MUL, mul.ctypes.data, capi.DT_F32, (1, N))]
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(dst), want)
    # the default switch: 129 rows
    monkeypatch.delenv("ZMI_PGRING_MIN_M")
    for rows, name in ((128, "pergroup_mfma16x16x64"), (129, RING)):
        pr = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
        ssr = rng.uniform(0.005, 0.03, (rows, G)).astype(np.float32)
        ssr_d = H.to_dev(ssr)
        pr.src_scale = lowoha.QuantParam(ssr_d, capi.DT_F32, (rows, G))
        pr.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
        pr.weight_cache_type = 0
        ar = rng.integers(-128, 128, (rows, K), dtype=np.int8)
        got, want = _run_both(zo, pr, ar, w, rows, N, K, host_bufs={"src_scale": ssr, "wei_scale": ws})
        assert lowoha.last_kernel() == name and np.array_equal(got, want)
    # 40 rows: the column-block kernel by default, the tiled one when the switch says so
    M2 = 40
    p2 = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    ss2_d = H.to_dev(ss[:M2].copy())
    p2.src_scale = lowoha.QuantParam(ss2_d, capi.DT_F32, (M2, G))
    p2.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    p2.weight_cache_type = 0
    hb = {"src_scale": ss[:M2].copy(), "wei_scale": ws}
    got, want = _run_both(zo, p2, a[:M2].copy(), w, M2, N, K, host_bufs=hb)
    assert lowoha.last_kernel() == "pergroup_mfma16x16x64" and np.array_equal(got, want)
    monkeypatch.setenv("ZMI_PGRING_MIN_M", "17")
    got, want = _run_both(zo, p2, a[:M2].copy(), w, M2, N, K, host_bufs=hb)
    assert lowoha.last_kernel() == RING and np.array_equal(got, want)
