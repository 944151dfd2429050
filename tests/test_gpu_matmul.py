"""GPU parity of matmul_direct (through the C ABI) against the CPU oracle on
the same seeded inputs.  Bars: s32 accumulators bit-exact; f32 within 1e-5
relative; bf16 within one bf16 ulp."""
import os

import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _oracle(zo, p_host, src, w, M, N, K, **kw):
    keep = []
    flat = p_host.flat(keep)
    st, dst, acc, scales = zo.matmul_int8(src, w, flat, M, N, K, **kw)
    assert st == capi.SUCCESS
    return dst, acc, scales


# ------------------------------------------------------------------ config 1
@pytest.mark.parametrize("M,K,N", [(128, 4096, 4096), (32, 256, 128), (128, 512, 192)])
@pytest.mark.parametrize("packed", [False, True])
def test_u8s8_zero_point_s32_and_f32(zo, small_m_kernel, M, K, N, packed):
    rng = np.random.default_rng(0x5EED0001)
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([128], dtype=np.int32)
    a_d, w_d, ws_d, bias_d = H.to_dev(a), H.to_dev(w), H.to_dev(ws), H.to_dev(bias)
    wt = H.prepack(w_d, K, N, src_dtype=capi.DT_U8) if packed else w_d

    # (a) raw accumulator: s32 destination, zero-point compensation only
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))      # one-element host buffer
    if packed:
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, wt, N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    acc, ov = zo.gemm_s32(a, w)
    assert ov == 0
    want = acc.astype(np.int64) - 128 * w.astype(np.int64).sum(axis=0)[None, :]
    assert np.array_equal(H.to_host(dst).astype(np.int64), want)        # bit-exact

    # (b) the dequantised f32 result with per-channel scales and bias
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
    zp_d = H.to_dev(zp)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.src_zp = lowoha.QuantParam(zp_d, capi.DT_S32, (1,))                # one-element device buffer
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    if packed:
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dstf = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, wt, N, bias_d, 0.0, dstf, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=ss, src_zp=zp, wei_scale=ws)
    ph.mem_format_b = "n"
    want_f, _, _ = _oracle(zo, ph, a, w, M, N, K, bias=bias)
    got = H.to_host(dstf)
    H.check_f32(got, want_f)
    # the chain is the same sequence of correctly rounded f32 operations on both sides
    assert np.array_equal(got, want_f)


# ------------------------------------------------------------------ config 2
@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("K,N", [(4096, 14336), (512, 320)])
def test_decode_dynamic_quant_bf16_silu(zo, M, K, N):
    rng = np.random.default_rng(0x5EED0002 + M)
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    blob = H.prepack(w_d, K, N)
    scales_d = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, 1))      # library writes the scales here
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, blob, N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "decode" in lowoha.last_kernel() or "smallm" in lowoha.last_kernel()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    want, _, scales = _oracle(zo, ph, x, w, M, N, K, want_scales=True)
    if M > 1:
        assert np.array_equal(H.to_host(scales_d), scales)              # per-token scales bit-exact
    else:
        assert H.to_host(scales_d)[0] == scales[0]
    H.check_bf16(H.to_host(dst), want)

    # same call with the scratch-allocated scale buffer and unpacked weights gives the same bits
    p2 = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p2.dynamic_quant = True
    p2.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p2.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p2.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    dst2 = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, None, 0.0, dst2, N, True, p2)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert torch.equal(dst.view(torch.int16), dst2.view(torch.int16))


# ------------------------------------------------------------------ config 3
@pytest.mark.parametrize("M,K,N,rows", [(2048, 4096, 4096, None), (2048, 4096, 14336, 96), (300, 384, 520, None)])
def test_prefill_dynamic_quant_bias_gelu(zo, M, K, N, rows):
    rng = np.random.default_rng(0x5EED0003)
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    x_d, w_d, ws_d, bias_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws), H.to_dev(bias)
    blob = H.prepack(w_d, K, N)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_GELU_TANH)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, blob, N, bias_d, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "mfma32x32x32" in lowoha.last_kernel()
    got = H.to_host(dst)
    # rows are independent (per-token quantization), so the oracle may run on a sample of them
    sel = np.arange(M) if rows is None else np.sort(rng.choice(M, rows, replace=False))
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    ph.src_scale = lowoha.QuantParam(None, capi.DT_F32, (len(sel), 1))
    want, _, _ = _oracle(zo, ph, np.ascontiguousarray(x[sel]), w, len(sel), N, K, bias=bias)
    H.check_bf16(got[sel], want, atol=1e-6, max_frac=5e-3)

    # s32 accumulators of the same kernel, bit-exact, on pre-quantized rows
    q, s = zo.quant_per_token(np.ascontiguousarray(x[sel]), capi.DT_BF16)
    q_d = H.to_dev(q)
    p3 = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    p3.mem_format_b = "r"
    p3.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    acc_d = torch.zeros((len(sel), N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, len(sel), N, K, 1.0, q_d, K, blob, N, None, 0.0, acc_d, N, True, p3)
    assert st == capi.SUCCESS, lowoha.last_error()
    if len(sel) * N * K <= 2048 * 4096 * 4096:
        import ctypes as C
        Bt = np.ascontiguousarray(w.T)
        acc = np.empty((len(sel), N), dtype=np.int32)
        zo.lib().zo_gemm_s32_bt(q.ctypes.data, capi.DT_S8, K, Bt.ctypes.data, K, len(sel), N, K, acc.ctypes.data, N)
        assert np.array_equal(H.to_host(acc_d), acc)


# ------------------------------------------------------------------ 17 .. 128 rows
@pytest.fixture(params=["fused", "separate"])
def quant_launch(request):
    """Per-token quantization inside the GEMM launch (the default where a kernel offers it) or in a launch of its own."""
    old = os.environ.get("ZMI_NO_FUSED_QUANT")
    if request.param == "separate":
        os.environ["ZMI_NO_FUSED_QUANT"] = "1"
    else:
        os.environ.pop("ZMI_NO_FUSED_QUANT", None)
    yield request.param
    if old is None:
        os.environ.pop("ZMI_NO_FUSED_QUANT", None)
    else:
        os.environ["ZMI_NO_FUSED_QUANT"] = old


@pytest.mark.parametrize("M", [17, 40, 64, 100, 128])
@pytest.mark.parametrize("K,N", [(4096, 1000), (520, 96)])
def test_row_groups_dynamic_quant_bf16_silu(zo, small_m_kernel, quant_launch, M, K, N):
    """More than one 16-row group: a partly filled last group, a column edge inside a block,
    fused per-token quantization (scales bit-exact) and the bf16 SiLU epilogue."""
    rng = np.random.default_rng(M * 31 + N)
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    blob = H.prepack(w_d, K, N)
    scales_d = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    for _ in range(2):
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, blob, N, None, 0.0, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
    assert small_m_kernel in lowoha.last_kernel() or "ring" in lowoha.last_kernel()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    want, _, scales = _oracle(zo, ph, x, w, M, N, K, want_scales=True)
    assert np.array_equal(H.to_host(scales_d), scales)
    H.check_bf16(H.to_host(dst), want)


@pytest.mark.parametrize("M,K,N", [(33, 1000, 300), (128, 4096, 512)])
def test_row_groups_s32_accumulators_bit_exact(zo, small_m_kernel, M, K, N):
    rng = np.random.default_rng(M + K + N)
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    zp = np.array([77], dtype=np.int32)
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
    dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert small_m_kernel in lowoha.last_kernel() or "ring" in lowoha.last_kernel()
    want = (a.astype(np.int64) - 77) @ w.astype(np.int64)
    assert np.array_equal(H.to_host(dst).astype(np.int64), want)


@pytest.mark.parametrize("M,K,N,force", [(40, 520, 96, True), (64, 4096, 1000, True), (33, 256, 300, True),
                                         (48, 256, 10752, False), (64, 128, 8192, False)])
def test_four_row_groups_per_workgroup_below_65_rows(zo, quant_launch, M, K, N, force, monkeypatch):
    """33 .. 64 rows on the decode kernel's four-groups-per-workgroup form (weights kept in registers for all row
    groups): taken by itself when the one-group form would need more than ~1000 workgroups, forced here on the small
    shapes through ZMI_DECODE_RPW."""
    if force:
        monkeypatch.setenv("ZMI_DECODE_RPW", "4")
    rng = np.random.default_rng(M * 17 + N)
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    blob = H.prepack(w_d, K, N)
    scales_d = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8, bias=capi.DT_F32)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, blob, N, H.to_dev(b), 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "decode_lds_rows" in lowoha.last_kernel()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    keep = []
    st, want, _, scales = zo.matmul_int8(x, w, ph.flat(keep), M, N, K, bias=b, want_scales=True)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(scales_d), scales)
    assert np.array_equal(H.to_host(dst), want)      # no activation: bit-identical f32
