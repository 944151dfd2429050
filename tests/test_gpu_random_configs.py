"""GPU parity of matmul_direct on seeded random configurations: shapes that land on every
kernel (1 .. 700 rows, K on both sides of the decode kernel's limit, ragged columns), source
and destination types, strides, transposes, zero-points, bias types and single post-ops.
Every case is compared with the CPU oracle on the same inputs; the seed is the case."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.test_gpu_reorder_edges import _run_both

pytestmark = pytest.mark.gpu

_POSTOPS = [None, capi.PO_RELU, capi.PO_SWISH, capi.PO_GELU_TANH, capi.PO_SIGMOID, capi.PO_TANH]


def _pick(rng, seq):
    return seq[int(rng.integers(len(seq)))]


@pytest.mark.parametrize("seed", range(48))
def test_static_quant_random_configuration(zo, seed):
    rng = np.random.default_rng(1000 + seed)
    M = int(_pick(rng, [1, 3, 16, 17, 31, 48, 64, 65, 100, 128, 129, 190, 257, 400, 700]))
    K = int(_pick(rng, [1, 15, 16, 33, 64, 200, 512, 1000, 4096, 4100, 6000]))
    N = int(_pick(rng, [1, 7, 32, 33, 100, 256, 257, 515, 1100]))
    if M * K * N > 300 * 4100 * 600:          # keep the oracle's part of a case within a second or two
        N = min(N, 257)
    u8 = bool(rng.integers(2))
    transA, transB = bool(rng.integers(4) == 0), bool(rng.integers(3) == 0)
    pad_a, pad_w, pad_c = (int(x) for x in rng.integers(0, 9, 3))
    dst_dt = _pick(rng, [capi.DT_F32, capi.DT_BF16, capi.DT_S32, capi.DT_S8, capi.DT_U8])
    po = _pick(rng, _POSTOPS)
    a = rng.integers(0, 256, (K, M + pad_a) if transA else (M, K + pad_a), dtype=np.uint8)
    if not u8:
        a = a.view(np.int8)
    w = rng.integers(-127, 128, (N, K + pad_w) if transB else (K, N + pad_w), dtype=np.int8)
    bufs = {}
    p = lowoha.MatmulParams(src=capi.DT_U8 if u8 else capi.DT_S8, wei=capi.DT_S8, dst=dst_dt)
    if dst_dt == capi.DT_S32:
        # the raw accumulator (with the zero-point compensation): no scales, bias or post-op
        bias = None
        if u8 or rng.integers(2):
            zp = np.array([int(rng.integers(0, 256)) if u8 else int(rng.integers(-20, 20))], dtype=np.int32)
            p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
            bufs["src_zp"] = zp
    else:
        # the reference takes per-token source scales only for s8 sources without a zero-point and f32 / bf16 outputs
        use_zp = u8 or rng.integers(3) == 0
        per_token = bool(rng.integers(2)) and not use_zp and dst_dt in (capi.DT_F32, capi.DT_BF16)
        ss = rng.uniform(0.005, 0.03, M if per_token else 1).astype(np.float32)
        ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
        ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
        p.src_scale = lowoha.QuantParam(ss_d if per_token else ss.ctypes.data, capi.DT_F32, (M, 1) if per_token else (1,))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
        bufs.update(src_scale=ss, wei_scale=ws)
        if use_zp:
            zp = np.array([int(rng.integers(100, 156)) if u8 else int(rng.integers(-9, 9))], dtype=np.int32)
            p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
            bufs["src_zp"] = zp
        bias = rng.standard_normal(N).astype(np.float32) if rng.integers(3) else None
        if bias is not None:
            p.dt_bias = capi.DT_F32
        if dst_dt in (capi.DT_S8, capi.DT_U8):
            ds = np.array([float(rng.uniform(3.0, 9.0))], dtype=np.float32)
            dz = np.array([int(rng.integers(-3, 4)) + (64 if dst_dt == capi.DT_U8 else 0)], dtype=np.int32)
            p.dst_scale = lowoha.QuantParam(ds.ctypes.data, capi.DT_F32, (1,))
            p.dst_zp = lowoha.QuantParam(dz.ctypes.data, capi.DT_S32, (1,))
            bufs.update(dst_scale=ds, dst_zp=dz)
            po = _pick(rng, [None, capi.PO_RELU])      # rounding to integers: keep the chain exactly reproducible
        if po is not None:
            p.postop_ = [lowoha.PostOp(po)]
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs=bufs, lda=a.shape[1], ldb=w.shape[1],
                          ldc=N + pad_c, transA=transA, transB=transB)
    what = f"seed {seed}: M={M} K={K} N={N} u8={u8} tA={transA} tB={transB} dst={dst_dt} po={po} [{lowoha.last_kernel()}]"
    g, wv = got[:, :N], want[:, :N]
    if dst_dt == capi.DT_BF16:
        if po is None or po == capi.PO_RELU:
            assert np.array_equal(g, wv), what         # every step of the chain is a correctly rounded f32 operation
        else:
            H.check_bf16(g, wv, atol=1e-6 if po == capi.PO_GELU_TANH else 0.0, max_frac=1e-2)
    elif dst_dt == capi.DT_F32:
        if po is None or po == capi.PO_RELU:
            assert np.array_equal(g, wv), what
        else:
            H.check_f32(g, wv, rtol=1e-5, atol=1e-6)
    else:
        assert np.array_equal(g, wv), what
    assert np.all(got[:, N:] == 0), what          # padding columns of dst are left alone


@pytest.mark.parametrize("seed", range(32))
def test_dynamic_quant_random_configuration(zo, seed):
    """bf16 / f32 rows quantized by the library (per token, or one scale for the tensor): the scales it
    writes are bit-exact, the output within the bf16 / f32 bars."""
    from tests.test_gpu_matmul import _oracle
    rng = np.random.default_rng(5000 + seed)
    M = int(_pick(rng, [1, 2, 16, 17, 40, 64, 65, 128, 129, 200, 333]))
    K = int(_pick(rng, [16, 20, 100, 512, 1024, 4096, 4352]))
    N = int(_pick(rng, [5, 32, 96, 300, 1000]))
    src_dt = _pick(rng, [capi.DT_BF16, capi.DT_F32])
    dst_dt = _pick(rng, [capi.DT_BF16, capi.DT_F32])
    if src_dt == capi.DT_F32:
        dst_dt = capi.DT_F32                 # (the reference rejects an f32 source with a bf16 destination)
    per_token = bool(rng.integers(4)) or M == 1
    po = _pick(rng, [None, capi.PO_SWISH, capi.PO_GELU_TANH, capi.PO_RELU])
    packed = bool(rng.integers(2))
    x32 = (rng.standard_normal((M, K)) * float(rng.uniform(0.2, 3.0))).astype(np.float32)
    x = H.bf16_bits(x32) if src_dt == capi.DT_BF16 else x32
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32) if rng.integers(2) else None
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    n_sc = M if per_token else 1
    scales_d = torch.zeros(n_sc, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=src_dt, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_S8,
                            bias=capi.DT_F32 if bias is not None else capi.DT_NONE)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, 1) if per_token else (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    if po is not None:
        p.postop_ = [lowoha.PostOp(po)]
    wt = w_d
    if packed:
        wt = H.prepack(w_d, K, N)
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    p.weight_cache_type = 0
    dst = torch.zeros((M, N), dtype=torch.bfloat16 if dst_dt == capi.DT_BF16 else torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, wt, N, H.to_dev(bias), 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    want, _, scales = _oracle(zo, ph, x, w, M, N, K, bias=bias, want_scales=True)
    what = f"seed {seed}: M={M} K={K} N={N} src={src_dt} dst={dst_dt} per_token={per_token} po={po} [{lowoha.last_kernel()}]"
    got_sc = H.to_host(scales_d)
    assert np.array_equal(got_sc, np.asarray(scales, dtype=np.float32).reshape(-1)[:n_sc]), what
    if po is None or po == capi.PO_RELU:
        assert np.array_equal(H.to_host(dst), want), what   # exact scales, exact quantization, correctly rounded f32 chain
    elif dst_dt == capi.DT_BF16:
        H.check_bf16(H.to_host(dst), want, atol=1e-6 if po == capi.PO_GELU_TANH else 0.0, max_frac=1e-2)
    else:
        H.check_f32(H.to_host(dst), want, rtol=1e-5, atol=1e-6)
