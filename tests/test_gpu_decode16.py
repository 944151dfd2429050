"""Decode calls with at most 16 rows: the kernel that fetches the rows by global->LDS loads
(rows given as s8 / u8) against the oracle and against the row-group kernel, and the hand-off
of the launches that quantize their own rows (failure path, stream hand-over, argument checks).
Every call goes through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _static_call(M, K, N, u8, dst_dt, rng, bias=False, po=None, lda=None):
    lda = lda or K
    if u8:
        a = rng.integers(0, 256, (M, lda), dtype=np.uint8)
    else:
        a = rng.integers(-127, 128, (M, lda), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ss = rng.uniform(0.01, 0.03, M).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    zp = np.array([131], dtype=np.int32)
    p = lowoha.MatmulParams(src=capi.DT_U8 if u8 else capi.DT_S8, wei=capi.DT_S8, dst=dst_dt,
                            bias=capi.DT_F32 if bias else capi.DT_NONE)
    dev = {}
    if dst_dt != capi.DT_S32:
        if u8:
            # (a source zero-point allows per-tensor source scales only)
            p.src_scale = lowoha.QuantParam(ss[:1].ctypes.data, capi.DT_F32, (1,))
        else:
            dev["ss"] = H.to_dev(ss)
            p.src_scale = lowoha.QuantParam(dev["ss"], capi.DT_F32, (M, 1) if M > 1 else (1,))
        dev["ws"] = H.to_dev(ws)
        p.wei_scale = lowoha.QuantParam(dev["ws"], capi.DT_F32, (1, N))
    if u8:
        p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
    if po is not None:
        p.postop_ = [lowoha.PostOp(po)]
    return a, w, ws, ss, b, zp, p, dev


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("K,N", [(4096, 1000), (1000, 333), (64, 32), (16, 70), (2048, 4096)])
@pytest.mark.parametrize("u8", [False, True])
def test_s32_accumulators_bit_exact_both_kernels(M, K, N, u8, monkeypatch):
    """Raw s32 destination (accumulator + zero-point compensation) on the 16-row kernel and, forced, on the
    row-group kernel: both equal the integer product; K that is no multiple of 64 or 16, column edges."""
    rng = np.random.default_rng(M * 1000 + K + N + int(u8))
    a, w, _, _, _, zp, p, _ = _static_call(M, K, N, u8, capi.DT_S32, rng)
    want = (a.astype(np.int64) - (131 if u8 else 0)) @ w.astype(np.int64)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    for forced in (False, True):
        if forced:
            monkeypatch.setenv("ZMI_DECODE_ROWGROUP_KERNEL", "1")
        dst = torch.full((M, N), -7, dtype=torch.int32, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, False, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        name = lowoha.last_kernel()
        assert ("decode16" in name) == (not forced), name
        assert np.array_equal(H.to_host(dst).astype(np.int64), want), name


@pytest.mark.parametrize("M,K,N,lda", [(16, 4096, 14336, 4096), (5, 1024, 96, 1040), (16, 512, 2048, 512), (2, 128, 64, 256)])
@pytest.mark.parametrize("u8", [False, True])
def test_f32_chain_bit_identical_to_oracle(zo, M, K, N, lda, u8):
    """Scales + bias, f32 out, no activation: bit-identical to the oracle (padded leading dimension included)."""
    rng = np.random.default_rng(M + K + N + lda)
    a, w, ws, ss, b, zp, p, dev = _static_call(M, K, N, u8, capi.DT_F32, rng, bias=True, lda=lda)
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), lda, H.to_dev(w), N, H.to_dev(b), 0.0, dst, N,
                              False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "decode16" in lowoha.last_kernel()
    ph = H.host_params(p, src_scale=ss[:1] if u8 or M == 1 else ss, wei_scale=ws, src_zp=zp if u8 else None)
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K, bias=b, lda=lda)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(dst), want)


def test_bf16_silu_matches_row_group_kernel_bit_for_bit(zo, monkeypatch):
    """The two decode kernels share the epilogue code: identical bf16 bits, and within the activation tolerance of the oracle."""
    rng = np.random.default_rng(99)
    M, K, N = 16, 4096, 1536
    a, w, ws, ss, _, _, p, dev = _static_call(M, K, N, False, capi.DT_BF16, rng, po=capi.PO_SWISH)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    outs = []
    for forced in (False, True):
        if forced:
            monkeypatch.setenv("ZMI_DECODE_ROWGROUP_KERNEL", "1")
        dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, False, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        outs.append(H.to_host(dst))
    assert np.array_equal(outs[0], outs[1])
    ph = H.host_params(p, src_scale=ss, wei_scale=ws)
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
    assert st == capi.SUCCESS
    H.check_bf16(outs[0], want)


def _fused_call(M, K, N, rng):
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    keep = {"x": H.to_dev(x), "ws": H.to_dev(ws), "blob": H.prepack(H.to_dev(w), K, N)}
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(keep["ws"], capi.DT_F32, (1, N))
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.full((M, N), 12345.0, dtype=torch.float32, device=H.DEV)

    def call():
        return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, keep["x"], K, keep["blob"], N, None, 0.0, dst, N, True, p)
    return x, w, ws, p, dst, call, keep


FUSED_NAMES = {
    "selfq": "decode16x2_selfquant_mfma16x16x64 (per-token quant in the workgroup)",
    "handoff16": "decode16_dma_rows_mfma16x16x64 (fused per-token quant)",
    "rowgroup": "decode_lds_rows_mfma16x16x64 (fused per-token quant)",
}


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("K,N", [(4096, 14336), (4096, 1000), (1000, 333), (64, 32), (24, 70), (2048, 4096), (4096, 2080)])
def test_fused_quantization_three_forms_bit_exact(zo, M, K, N, monkeypatch):
    """bf16 rows quantized per token inside the decode launch, in its three forms: by the workgroups that use the
    rows (16 wavefronts, two column blocks; odd block counts included), by quantizing workgroups whose rows the
    16-row kernel waits for through the scalar unit, and the row-group kernel's hand-off.  Each bit-identical to the
    oracle on repeated calls; rows with NaN / infinite elements (they count as zero) give the same bits in all three."""
    rng = np.random.default_rng(M * 100 + K + N)
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    hk = []
    st, want, _, _ = zo.matmul_int8(x, w, ph.flat(hk), M, N, K)
    assert st == capi.SUCCESS
    xbad = x.copy()
    xbad[0, 0] = 0x7f80          # +inf
    xbad[M - 1, K - 1] = 0xffc0  # NaN
    xbad[M // 2, K // 2] = 0xff80  # -inf
    xbad_d = H.to_dev(xbad)
    bad = []
    for mode in ("selfq", "handoff16", "rowgroup"):
        monkeypatch.delenv("ZMI_NO_DECODE_SELFQ", raising=False)
        monkeypatch.delenv("ZMI_DECODE_ROWGROUP_KERNEL", raising=False)
        monkeypatch.setenv("ZMI_DECODE_SELFQ_MIN_WGS", "1")
        monkeypatch.setenv("ZMI_DECODE_SELFQ_MAX_M", "16")
        if mode != "selfq":
            monkeypatch.setenv("ZMI_NO_DECODE_SELFQ", "1")
        if mode == "rowgroup":
            monkeypatch.setenv("ZMI_DECODE_ROWGROUP_KERNEL", "1")
        for rep in range(2):
            dst.fill_(12345.0)
            assert call() == capi.SUCCESS, lowoha.last_error()
            assert lowoha.last_kernel() == FUSED_NAMES[mode]
            assert np.array_equal(H.to_host(dst), want), (mode, rep)
        d2 = torch.full((M, N), 12345.0, dtype=torch.float32, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, xbad_d, K, keep["blob"], N, None, 0.0, d2, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        bad.append(H.to_host(d2))
    assert np.array_equal(bad[0], bad[1]) and np.array_equal(bad[1], bad[2])
    assert np.all(np.isfinite(bad[0]))


@pytest.mark.parametrize("M,K,N", [(16, 4096, 2080), (13, 1000, 333)])
def test_handoff_flags_in_ordinary_memory(zo, M, K, N, monkeypatch):
    """ZMI_NO_UNCACHED_FLAGS: the hand-off words live in ordinary device memory, as on a device that refuses the
    uncached kind; the launch that would wait through the scalar unit takes the row-group kernel's form, which waits
    with device-scope vector loads.  Bit-identical to the oracle, and switching back works."""
    rng = np.random.default_rng(M + K + N)
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    hk = []
    st, want, _, _ = zo.matmul_int8(x, w, ph.flat(hk), M, N, K)
    assert st == capi.SUCCESS
    monkeypatch.setenv("ZMI_NO_DECODE_SELFQ", "1")
    for plain in (True, False, True):
        if plain:
            monkeypatch.setenv("ZMI_NO_UNCACHED_FLAGS", "1")
        else:
            monkeypatch.delenv("ZMI_NO_UNCACHED_FLAGS", raising=False)
        for rep in range(2):
            dst.fill_(12345.0)
            assert call() == capi.SUCCESS, lowoha.last_error()
            assert lowoha.last_kernel() == FUSED_NAMES["rowgroup" if plain else "handoff16"]
            assert np.array_equal(H.to_host(dst), want), (plain, rep)


def test_fused_quantization_default_form_by_width(zo, monkeypatch):
    """Which form a call takes by itself: up to 12 rows and an output wide enough for 64 two-block workgroups (at
    most one per compute unit) quantize in the workgroups, the others keep the hand-off."""
    monkeypatch.delenv("ZMI_DECODE_SELFQ_MIN_WGS", raising=False)
    monkeypatch.delenv("ZMI_DECODE_SELFQ_MAX_M", raising=False)
    rng = np.random.default_rng(3)
    for M, N, mode in ((8, 14336, "selfq"), (12, 4096, "selfq"), (13, 14336, "handoff16"), (16, 14336, "handoff16"),
                       (4, 2048, "handoff16"), (1, 20480, "handoff16")):
        x, w, ws, p, dst, call, keep = _fused_call(M, 512, N, rng)
        assert call() == capi.SUCCESS, lowoha.last_error()
        assert lowoha.last_kernel() == FUSED_NAMES[mode], N
        capi.load().zmi_clear_weight_cache()


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("K,N", [(4160, 96), (8192, 1000), (14336, 333), (20000, 64)])
@pytest.mark.parametrize("mode", ["arrivals", "reduce_kernel"])
def test_long_k_in_slices_bit_exact(zo, M, K, N, mode, monkeypatch):
    """K beyond 4096 with at most 16 rows: the 16-row kernel in K slices (2, 2, 4 and 5 of them; K that is no multiple
    of 64), finished by the last slice to arrive or, without the arrival words, by a reduction kernel.  Raw s32 sums
    against the integer product, the f32 chain and dynamically quantized bf16 rows against the oracle; repeated
    calls (the arrival words must be zero again)."""
    if mode == "reduce_kernel":
        monkeypatch.setenv("ZMI_NO_SLICE_ARRIVALS", "1")
    rng = np.random.default_rng(M * 1000 + K + N)
    for u8 in (False, True):
        a, w, _, _, _, zp, p, _ = _static_call(M, K, N, u8, capi.DT_S32, rng)
        want = (a.astype(np.int64) - (131 if u8 else 0)) @ w.astype(np.int64)
        a_d, w_d = H.to_dev(a), H.to_dev(w)
        for rep in range(2):
            dst = torch.full((M, N), -7, dtype=torch.int32, device=H.DEV)
            st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, True, p)
            assert st == capi.SUCCESS, lowoha.last_error()
            assert lowoha.last_kernel() == "decode16_ksliced_dma_rows_mfma16x16x64"
            assert np.array_equal(H.to_host(dst).astype(np.int64), want), (u8, rep)
        capi.load().zmi_clear_weight_cache()
    # f32 chain with bias, rows given
    a, w, ws, ss, b, zp, p, dev = _static_call(M, K, N, False, capi.DT_F32, rng, bias=True)
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, H.to_dev(b), 0.0, dst, N, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=ss if M > 1 else ss[:1], wei_scale=ws)
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K, bias=b)
    assert st == capi.SUCCESS and np.array_equal(H.to_host(dst), want)
    # bf16 rows quantized per token by the call (a launch of its own in front of the sliced kernel)
    x = H.gen_bf16_normal(rng, (M, K), std=2.0)
    ws_d = H.to_dev(ws)
    sc_d = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    pd = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
    pd.dynamic_quant = True
    pd.src_scale = lowoha.QuantParam(sc_d, capi.DT_F32, (M, 1))
    pd.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(x), K, H.to_dev(w), N, None, 0.0, dst, N, False, pd)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == "decode16_ksliced_dma_rows_mfma16x16x64"
    ph = H.host_params(pd, src_scale=None, wei_scale=ws)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, w, ph.flat(keep), M, N, K, want_scales=True, n_scales=M)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(sc_d), scales[:M]) and np.array_equal(H.to_host(dst), want)
    # the small-M kernel on the same call (environment switch): the same bits
    monkeypatch.setenv("ZMI_NO_DECODE_SLICED", "1")
    dst2 = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(x), K, H.to_dev(w), N, None, 0.0, dst2, N, False, pd)
    assert st == capi.SUCCESS and lowoha.last_kernel().startswith("smallm_splitk")
    assert torch.equal(dst2, dst)


@pytest.mark.parametrize("M,K,N", [(16, 4096, 2048), (4, 512, 320), (40, 1024, 256)])
def test_handoff_timeout_fails_loudly_and_recovers(zo, M, K, N, monkeypatch):
    """A streaming workgroup whose wait for the quantized rows runs out computes nothing: the output keeps its
    old contents, the thread's next call returns failure with a message, and the call after that is correct again.
    The limit is forced to zero from the host (every wait gives up at once); all kernels exit normally."""
    rng = np.random.default_rng(M + K)
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    assert call() == capi.SUCCESS, lowoha.last_error()
    assert "fused" in lowoha.last_kernel()
    good = H.to_host(dst).copy()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    hk = []
    st, want, _, _ = zo.matmul_int8(x, w, ph.flat(hk), M, N, K)
    assert st == capi.SUCCESS and np.array_equal(good, want)

    dst.fill_(12345.0)
    monkeypatch.setenv("ZMI_FUSED_WAIT_US", "0")
    assert call() == capi.SUCCESS          # (queued: the failure is found by the kernel, later)
    torch.cuda.synchronize()
    monkeypatch.delenv("ZMI_FUSED_WAIT_US")
    assert np.all(H.to_host(dst) == 12345.0), "a workgroup stored results computed from unpublished rows"
    assert call() == capi.FAILURE
    assert "quantized rows" in lowoha.last_error()
    assert call() == capi.SUCCESS, lowoha.last_error()
    assert np.array_equal(H.to_host(dst), want)


def test_unimplemented_call_leaves_the_handoff_intact(zo):
    """A call that is refused after the fused path was planned (an unimplemented post-op) must not disturb later
    fused calls: the hand-off carries no count from one launch to the next."""
    rng = np.random.default_rng(5)
    M, K, N = 8, 1024, 512
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    assert call() == capi.SUCCESS, lowoha.last_error()
    good = H.to_host(dst).copy()
    p.postop_ = [lowoha.PostOp(capi.PO_SOFTMAX)]
    assert call() == capi.UNIMPLEMENTED
    p.postop_ = []
    import time
    t0 = time.perf_counter()
    for _ in range(3):
        dst.fill_(0.0)
        assert call() == capi.SUCCESS, lowoha.last_error()
        assert np.array_equal(H.to_host(dst), good)
    assert time.perf_counter() - t0 < 1.0, "fused calls after a refused one wait for rows that never come"


def test_stream_handover_orders_scratch_reuse(zo):
    """zmi_set_stream between two asynchronous calls: the second call's scratch (quantized rows, hand-off words)
    is the first call's, so the new stream is made to wait for the old one."""
    lib = capi.load()
    rng = np.random.default_rng(17)
    M, K, N = 16, 4096, 4096
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    x2 = H.gen_bf16_normal(rng, (M, K))
    x2_d = H.to_dev(x2)
    dst2 = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    hk = []
    _, want1, _, _ = zo.matmul_int8(x, w, ph.flat(hk), M, N, K)
    _, want2, _, _ = zo.matmul_int8(x2, w, ph.flat(hk), M, N, K)
    s_a, s_b = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    old = lib.zmi_get_stream()
    try:
        for _ in range(20):
            lib.zmi_set_stream(ctypes.c_void_p(s_a.cuda_stream))
            assert call() == capi.SUCCESS, lowoha.last_error()
            lib.zmi_set_stream(ctypes.c_void_p(s_b.cuda_stream))
            st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x2_d, K, keep["blob"], N, None, 0.0, dst2, N, True, p)
            assert st == capi.SUCCESS, lowoha.last_error()
        torch.cuda.synchronize()
        assert np.array_equal(H.to_host(dst), want1)
        assert np.array_equal(H.to_host(dst2), want2)
    finally:
        lib.zmi_set_stream(ctypes.c_void_p(old))


def test_dynamic_scale_buffer_in_host_memory_is_refused():
    """With dynamic_quant the scale buffer is an output the kernels write: a host pointer is refused up front."""
    rng = np.random.default_rng(3)
    M, K, N = 1, 256, 64
    x, w, ws, p, dst, call, keep = _fused_call(M, K, N, rng)
    host_scale = np.zeros(1, dtype=np.float32)
    p.src_scale = lowoha.QuantParam(host_scale.ctypes.data, capi.DT_F32, (1, 1))
    assert call() == capi.FAILURE
    assert "device memory" in lowoha.last_error()
    dev_scale = torch.zeros(1, dtype=torch.float32, device=H.DEV)
    p.src_scale = lowoha.QuantParam(dev_scale, capi.DT_F32, (1, 1))
    assert call() == capi.SUCCESS, lowoha.last_error()
    assert float(H.to_host(dev_scale)[0]) > 0.0
