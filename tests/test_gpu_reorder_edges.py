"""GPU parity of reorder_direct (prepack and dynamic per-token modes) and of the
edge cases of matmul_direct: odd shapes and alignments, transposed operands,
padded leading dimensions, every post-op and destination dtype, alpha / beta."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("small_m_kernel")]


def _dq_params(M, K, src_dt, scale_buf, dims):
    rp = lowoha.ReorderParams()
    rp.src_dtype, rp.dst_dtype = src_dt, capi.DT_S8
    rp.dynamic_quant = True
    rp.algo = 1
    rp.src_shape = rp.dst_shape = (M, K)
    rp.scale = lowoha.QuantParam(scale_buf, capi.DT_F32, dims)
    return rp


@pytest.mark.parametrize("M,K", [(1, 64), (7, 515), (33, 4096), (5, 20000), (2048, 1408)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_dynamic_per_token_quant_bit_exact(zo, M, K, src_dt):
    rng = np.random.default_rng(M * 131 + K)
    xf = (rng.standard_normal((M, K)) * rng.uniform(0.01, 30, (M, 1))).astype(np.float32)
    if M > 3:
        xf[1, :] = 0.0                       # zero row -> scale clamps to 1e-10
        xf[2, 3] = np.inf
        xf[2, 5] = np.nan
        xf[3, 0] = -np.inf
    x = H.bf16_bits(xf) if src_dt == capi.DT_BF16 else xf
    x_d = H.to_dev(x)
    q_d = torch.zeros((M, K), dtype=torch.int8, device=H.DEV)
    s_d = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q_d, _dq_params(M, K, src_dt, s_d, (M, 1)))
    assert st == capi.SUCCESS, lowoha.last_error()
    q, s = zo.quant_per_token(x, src_dt)
    assert np.array_equal(H.to_host(s_d), s)
    assert np.array_equal(H.to_host(q_d), q)
    # quantize -> dequantize stays within half a step of the source (the reference's own round-trip test)
    src_f = zo.bf16_to_f32(x) if src_dt == capi.DT_BF16 else x
    fin = np.isfinite(src_f)
    back = q.astype(np.float32) * s[:, None]
    assert np.all(np.abs(back - src_f)[fin] <= 0.50002 * s[:, None].repeat(K, 1)[fin] + 1e-12)
    # scales only (dst == nullptr)
    s2 = torch.zeros(M, dtype=torch.float32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, None, _dq_params(M, K, src_dt, s2, (M, 1)))
    assert st == capi.SUCCESS and torch.equal(s2, s_d)


def test_dynamic_per_tensor_quant(zo):
    rng = np.random.default_rng(5)
    M, K = 9, 300
    x = H.gen_bf16_normal(rng, (M, K), std=3.0)
    x_d = H.to_dev(x)
    q_d = torch.zeros((M, K), dtype=torch.int8, device=H.DEV)
    s_d = torch.zeros(1, dtype=torch.float32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q_d, _dq_params(M, K, capi.DT_BF16, s_d, (1, 1)))
    assert st == capi.SUCCESS, lowoha.last_error()
    xf = zo.bf16_to_f32(x)
    s = np.float32(np.abs(xf).max()) / np.float32(127.0)
    assert H.to_host(s_d)[0] == s
    assert np.array_equal(H.to_host(q_d), np.rint(xf / s).astype(np.int8))


@pytest.mark.parametrize("K,N,transposed,ldpad", [(64, 64, False, 0), (100, 37, False, 3), (4096, 192, True, 0),
                                                 (130, 70, True, 5), (1408, 2048, False, 0)])
def test_prepack_round_trip_and_size(zo, K, N, transposed, ldpad):
    """The blob is opaque: what is checkable is matmul(prepack(B)) == matmul(B) bit-exactly,
    the size query (multiple of 64, >= payload), and the zero-point column sums it carries."""
    rng = np.random.default_rng(K + N)
    w = H.gen_weights(rng, K, N)
    if transposed:
        buf = np.zeros((N, K + ldpad), dtype=np.int8)
        buf[:, :K] = w.T
    else:
        buf = np.zeros((K, N + ldpad), dtype=np.int8)
        buf[:, :N] = w
    ldb = buf.shape[1]
    w_d = H.to_dev(buf)
    blob = H.prepack(w_d, K, N, ldb=ldb, transposed=transposed, src_dtype=capi.DT_U8)
    assert blob.numel() % 64 == 0 and blob.numel() >= K * N
    M = 19
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    zp = np.array([77], dtype=np.int32)
    outs = []
    for fmt, wt in (("r", blob), ("n", w_d)):
        p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
        p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
        p.mem_format_b = fmt
        if fmt == "r":
            p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
        st = lowoha.matmul_direct("r", False, transposed if fmt == "n" else False, M, N, K, 1.0, H.to_dev(a), K,
                                  wt, ldb if fmt == "n" else N, None, 0.0, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        outs.append(H.to_host(dst))
    want = (a.astype(np.int64) - 77) @ w.astype(np.int64)
    assert np.array_equal(outs[0].astype(np.int64), want)
    assert np.array_equal(outs[1].astype(np.int64), want)


def test_wrong_blob_is_rejected():
    w = torch.zeros((64, 64), dtype=torch.int8, device=H.DEV)
    blob = H.prepack(w, 64, 64)
    a = torch.zeros((4, 128), dtype=torch.int8, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((4, 64), dtype=torch.int32, device=H.DEV)
    # K does not match what the blob was packed for
    assert lowoha.matmul_direct("r", False, False, 4, 64, 128, 1.0, a, 128, blob, 64, None, 0.0, dst, 64, True, p) == capi.FAILURE
    # a plain weight buffer passed as a blob
    big = torch.zeros(1 << 16, dtype=torch.int8, device=H.DEV)
    assert lowoha.matmul_direct("r", False, False, 4, 64, 64, 1.0, a, 128, big, 64, None, 0.0, dst, 64, True, p) == capi.FAILURE


def _run_both(zo, p, a, w, M, N, K, *, bias=None, host_bufs=None, dst_np=None, lda=None, ldb=None, ldc=None,
              transA=False, transB=False, alpha=1.0, beta=0.0):
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    ldc_ = ldc or N
    np_dt = zo.NP_OF_DT[p.dt_dst]
    dst0 = dst_np if dst_np is not None else np.zeros((M, ldc_), dtype=np_dt)
    dst_d = H.to_dev(dst0.copy())
    bias_d = H.to_dev(bias) if bias is not None else None
    st = lowoha.matmul_direct("r", transA, transB, M, N, K, alpha, a_d, lda or a.shape[1], w_d, ldb or w.shape[1],
                              bias_d, beta, dst_d, ldc_, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    keep = []
    ph = H.host_params(p, **(host_bufs or {}))
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K, bias=bias, dst=dst0.copy(), lda=lda, ldb=ldb,
                                    ldc=ldc_, transA=transA, transB=transB, alpha=alpha, beta=beta)
    assert st == capi.SUCCESS
    return H.to_host(dst_d), want


@pytest.mark.parametrize("M,K,N", [(5, 100, 37), (1, 17, 1), (129, 72, 65), (200, 1000, 300)])
def test_odd_shapes_strides_and_transposes(zo, M, K, N):
    rng = np.random.default_rng(M + K + N)
    ss = np.array([0.03], dtype=np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    for transA, transB, pad in ((False, False, 0), (False, True, 3), (True, False, 5), (True, True, 1)):
        a = rng.integers(-128, 128, (K, M + pad) if transA else (M, K + pad), dtype=np.int8)
        w = rng.integers(-127, 128, (N, K + pad) if transB else (K, N + pad), dtype=np.int8)
        ws_d = H.to_dev(ws)
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
        p.weight_cache_type = 0
        got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws},
                              lda=a.shape[1], ldb=w.shape[1], ldc=N + 7, transA=transA, transB=transB)
        assert np.array_equal(got[:, :N], want[:, :N])
        assert np.all(got[:, N:] == 0)          # padding columns of dst are left alone


@pytest.mark.parametrize("po", [capi.PO_RELU, capi.PO_LEAKY_RELU, capi.PO_GELU_TANH, capi.PO_GELU_ERF,
                                capi.PO_SIGMOID, capi.PO_SWISH, capi.PO_TANH, capi.PO_CLIP])
@pytest.mark.parametrize("M", [24, 200])
def test_every_eltwise_post_op_f32(zo, po, M):
    rng = np.random.default_rng(po)
    K, N = 256, 96
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.01], dtype=np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(po, alpha=1.5, beta=-0.5)]     # reversed clip bounds are swapped, as in the reference
    got, want = _run_both(zo, p, a, w, M, N, K, host_bufs={"src_scale": ss, "wei_scale": ws})
    if po == capi.PO_CLIP:
        ph = H.host_params(p, src_scale=ss, wei_scale=ws)
        ph.postop_ = [lowoha.PostOp(po, alpha=-0.5, beta=1.5)]
        keep = []
        _, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
    H.check_f32(got, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("po", [capi.PO_ELU, capi.PO_SQUARE, capi.PO_ABS, capi.PO_SQRT, capi.PO_EXP, capi.PO_LOG, capi.PO_MISH])
@pytest.mark.parametrize("M,dst_dt", [(7, capi.DT_F32), (24, capi.DT_BF16), (200, capi.DT_F32), (200, capi.DT_BF16)])
def test_remaining_eltwise_post_ops(zo, po, M, dst_dt):
    """elu (alpha from the post-op) / square / abs / sqrt / exp / log / mish through the interpreter of every kernel that can
    take the call: f32 within 1e-5 relative, bf16 within one ulp.  sqrt and log see a chain whose result is positive
    (ReLU + a bias in front of them keeps them off the reference's NaN / -inf cases, which are compared too: NaN == NaN)."""
    rng = np.random.default_rng(po * 100 + M)
    K, N = 256, 96
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.01], dtype=np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.uniform(0.5, 1.5, N).astype(np.float32)
    ws_d, b_d = H.to_dev(ws), H.to_dev(b)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    chain = [lowoha.PostOp(po, alpha=1.7)]
    if po in (capi.PO_SQRT, capi.PO_LOG):
        add = np.full((1, N), 0.25, dtype=np.float32)
        add_d = H.to_dev(add)
        chain = [lowoha.PostOp(capi.PO_RELU), lowoha.PostOp(capi.PO_BINARY_ADD, add_d, capi.DT_F32, (1, N)), lowoha.PostOp(po)]
    p.postop_ = chain
    dst = torch.zeros((M, N), dtype=torch.float32 if dst_dt == capi.DT_F32 else torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, b_d, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=ss, wei_scale=ws)
    if po in (capi.PO_SQRT, capi.PO_LOG):
        ph.postop_ = [lowoha.PostOp(capi.PO_RELU), lowoha.PostOp(capi.PO_BINARY_ADD, add.ctypes.data, capi.DT_F32, (1, N)),
                      lowoha.PostOp(po)]
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K, bias=b)
    assert st == capi.SUCCESS
    if dst_dt == capi.DT_F32:
        H.check_f32(H.to_host(dst), want, rtol=1e-5, atol=1e-6)
    else:
        H.check_bf16(H.to_host(dst), want, max_frac=5e-3)


def test_softmax_post_op_is_refused():
    rng = np.random.default_rng(1)
    M, K, N = 8, 64, 32
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    p.postop_ = [lowoha.PostOp(capi.PO_SOFTMAX)]
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(rng.integers(-128, 128, (M, K), dtype=np.int8)), K,
                              H.to_dev(H.gen_weights(rng, K, N)), N, None, 0.0, dst, N, True, p)
    assert st == capi.UNIMPLEMENTED


def test_binary_post_ops_chain_and_dst_quant(zo):
    rng = np.random.default_rng(99)
    M, K, N = 40, 128, 80
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([120], dtype=np.int32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    add = rng.standard_normal((M, N)).astype(np.float32)
    mul = rng.uniform(0.5, 1.5, (1, N)).astype(np.float32)
    ds = np.array([7.5], dtype=np.float32)
    dz = np.array([3], dtype=np.int32)
    ws_d, add_d, mul_d = H.to_dev(ws), H.to_dev(add), H.to_dev(mul)
    for dst_dt in (capi.DT_S8, capi.DT_U8, capi.DT_F32, capi.DT_BF16):
        p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=dst_dt)
        p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
        p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
        p.dst_scale = lowoha.QuantParam(ds.ctypes.data, capi.DT_F32, (1,))
        p.dst_zp = lowoha.QuantParam(dz.ctypes.data, capi.DT_S32, (1,))
        p.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add_d, capi.DT_F32, (M, N)),
                     lowoha.PostOp(capi.PO_RELU),
                     lowoha.PostOp(capi.PO_BINARY_MUL, mul_d, capi.DT_F32, (1, N))]
        ph_bufs = {"src_scale": ss, "src_zp": zp, "wei_scale": ws, "dst_scale": ds, "dst_zp": dz}
        a_d, w_d = H.to_dev(a), H.to_dev(w)
        dst_d = torch.zeros((M, N), dtype={capi.DT_S8: torch.int8, capi.DT_U8: torch.uint8, capi.DT_F32: torch.float32,
                                           capi.DT_BF16: torch.bfloat16}[dst_dt], device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst_d, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        ph = H.host_params(p, **ph_bufs)
        ph.postop_ = [lowoha.PostOp(capi.PO_BINARY_ADD, add.ctypes.data, capi.DT_F32, (M, N)),
                      lowoha.PostOp(capi.PO_RELU),
                      lowoha.PostOp(capi.PO_BINARY_MUL, mul.ctypes.data, capi.DT_F32, (1, N))]
        keep = []
        _, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
        assert np.array_equal(H.to_host(dst_d), want)


def test_alpha_beta(zo):
    rng = np.random.default_rng(3)
    M, K, N = 150, 192, 130
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([100], dtype=np.int32)
    c0 = rng.standard_normal((M, N)).astype(np.float32)
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
    got, want = _run_both(zo, p, a, w, M, N, K, host_bufs={"src_scale": ss, "src_zp": zp}, dst_np=c0,
                          alpha=0.5, beta=2.0)
    assert np.array_equal(got, want)


def test_weight_cache_modes_agree():
    rng = np.random.default_rng(8)
    M, K, N = 20, 256, 128
    a = H.to_dev(rng.integers(-128, 128, (M, K), dtype=np.int8))
    w = H.to_dev(H.gen_weights(rng, K, N))
    outs = []
    for wct, const in ((0, True), (1, True), (2, True), (2, False)):
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
        p.weight_cache_type = wct
        dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
        for _ in range(2):      # second call hits the cache where one is kept
            assert lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a, K, w, N, None, 0.0, dst, N, const, p) == capi.SUCCESS
        outs.append(dst)
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert torch.equal(outs[0], (a.cpu().int() @ w.cpu().int()).to(H.DEV))


def test_mish_refused_where_the_reference_refuses_it():
    """mish with per-row source scales on s8 rows and with dynamic quantization: failure before any launch
    (lowoha_matmul_utils.cpp:379-408); the static per-tensor chain above computes it."""
    rng = np.random.default_rng(5)
    M, K, N = 8, 64, 32
    ws_d = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    ss_d = H.to_dev(rng.uniform(0.01, 0.02, M).astype(np.float32))
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    w_d = H.to_dev(H.gen_weights(rng, K, N))
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    a_d = H.to_dev(rng.integers(-128, 128, (M, K), dtype=np.int8))
    assert lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, True, p) == capi.FAILURE
    assert "mish" in lowoha.last_error()
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    x_d = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
    assert lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, None, 0.0, dst, N, True, p) == capi.FAILURE
    assert "mish" in lowoha.last_error()
