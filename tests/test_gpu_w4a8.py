"""GPU parity of matmul_direct for W4A8: bf16 rows quantized at run time to s8 (one scale per tensor, per row or
per (row, group)), packed s4 weights with {G, N} scales, bf16 out.  The library widens the s4 codes to s8, reorders
and caches them per weight pointer, repeats compact source scales over the groups and runs the per-group symmetric
GEMM (reference: lowoha_operators/matmul/lowoha_matmul_utils.cpp:72-176 for the contract,
matmul/backends/aocl/aocl_kernel.cpp:144-236, 704-793 for the widening, the scale broadcast and the cache)."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _s4_pack(codes, ld):
    R, C = codes.shape
    full = np.full((R, ld), 5, dtype=np.int64)
    full[:, :C] = codes
    flat = full.reshape(-1) & 15
    if flat.size % 2:
        flat = np.append(flat, 0)
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)


def _case(rng, M, K, N, G, transB, pad=0):
    x = H.bf16_bits((rng.standard_normal((M, K)) * 2).astype(np.float32))
    w = rng.integers(-8, 8, (K, N), dtype=np.int8)
    ldb = (K if transB else N) + pad
    packed = _s4_pack(w.T.copy(), ldb) if transB else _s4_pack(w, ldb)
    ws = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
    return x, packed, ldb, ws


def _run(zo, M, K, N, G, sdims, *, transB=False, const=True, postop=None, bias=False, ws_bf16=False, pad=0, calls=1,
         want_kernel=None):
    rng = np.random.default_rng(M * 7 + K + N * 3 + G)
    x, packed, ldb, ws = _case(rng, M, K, N, G, transB, pad)
    if ws_bf16:
        ws_h = H.bf16_bits(ws)
        ws_dt = capi.DT_BF16
    else:
        ws_h, ws_dt = ws, capi.DT_F32
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    n_sc = int(np.prod(sdims))
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(packed), H.to_dev(ws_h)
    sc_d = torch.zeros(n_sc, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8,
                            bias=capi.DT_F32 if bias else capi.DT_NONE)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(sc_d, capi.DT_F32, sdims)
    p.wei_scale = lowoha.QuantParam(ws_d, ws_dt, (G, N))
    if postop is not None:
        p.postop_ = [lowoha.PostOp(postop)]
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    b_d = H.to_dev(b) if bias else None
    for _ in range(calls):                       # a second call finds the widened weights in the cache
        dst.zero_()
        st = lowoha.matmul_direct("r", False, transB, M, N, K, 1.0, x_d, K, w_d, ldb, b_d, 0.0, dst, N, const, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        if want_kernel:
            assert lowoha.last_kernel().startswith(want_kernel), lowoha.last_kernel()
    ph = H.host_params(p, src_scale=None, wei_scale=ws_h)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, packed, ph.flat(keep), M, N, K, bias=b, transB=transB, ldb=ldb,
                                         want_scales=True, n_scales=max(n_sc, M))
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(sc_d), scales[:n_sc])
    if postop is None:
        assert np.array_equal(H.to_host(dst), want)     # every step is a correctly rounded f32 operation
    else:
        H.check_bf16(H.to_host(dst), want, max_frac=1e-2)
    capi.load().zmi_clear_weight_cache()


@pytest.mark.parametrize("M,K,N,G", [(16, 4096, 512, 32), (4, 4096, 14336, 32), (1, 4096, 96, 128), (16, 1024, 100, 16),
                                     (5, 256, 33, 4), (40, 512, 70, 8), (130, 1024, 48, 32), (3, 128, 16, 8),
                                     (260, 1024, 200, 8), (192, 512, 64, 16)])   # (the MFMA-tiled per-group kernel)
@pytest.mark.parametrize("kind", ["tensor", "token", "group"])
def test_w4a8_scale_granularities(zo, M, K, N, G, kind):
    sdims = {"tensor": (1, 1), "token": (M, 1), "group": (M, G)}[kind]
    _run(zo, M, K, N, G, sdims, want_kernel="pergroup_", calls=2)


@pytest.mark.parametrize("transB", [False, True])
@pytest.mark.parametrize("const", [False, True])
def test_w4a8_orientations_padding_and_uncached_weights(zo, transB, const):
    _run(zo, 7, 512, 45, 8, (7, 1), transB=transB, const=const, pad=3 if transB else 1, bias=True)
    _run(zo, 16, 2048, 64, 16, (16, 16), transB=transB, const=const, bias=True, ws_bf16=True)


@pytest.mark.parametrize("postop", [capi.PO_SWISH, capi.PO_GELU_TANH, capi.PO_RELU])
def test_w4a8_post_ops(zo, postop):
    _run(zo, 16, 4096, 320, 32, (16, 1), postop=postop, bias=True)
    _run(zo, 9, 1024, 64, 32, (9, 32), postop=postop)


@pytest.mark.parametrize("kind", ["tensor", "token", "group"])
@pytest.mark.parametrize("M,K,N,G", [(16, 4096, 200, 32), (16, 4096, 64, 128), (7, 2048, 40, 8), (2, 1024, 96, 32),
                                     (16, 1024, 33, 8)])
def test_w4a8_decode_shapes_stream_the_4_bit_tiles(zo, M, K, N, G, kind):
    # up to 16 rows, K = 1024 / 2048 / 4096, cached weights: the decode-shaped kernel reads 4-bit tiles; with one
    # scale per row or per (row, group) the quantization is part of the same launch
    sdims = {"tensor": (1, 1), "token": (M, 1), "group": (M, G)}[kind]
    name = "pergroup_decode_s4_mfma16x16x64" + {"tensor": "", "token": " (fused per-token quant)",
                                                "group": " (fused per-group quant)"}[kind]
    _run(zo, M, K, N, G, sdims, want_kernel=name, calls=2, postop=capi.PO_SWISH if N == 200 else None, bias=N == 64)


def test_w4a8_one_group_is_the_per_channel_chain(zo):
    # G = 1: {1, N} weight scales, the plain per-token chain on the widened weights
    _run(zo, 8, 512, 64, 1, (8, 1))
    _run(zo, 200, 256, 300, 1, (200, 1))


def test_w4a8_rejections(zo):
    M, K, N, G = 4, 64, 8, 2
    x_d = H.to_dev(np.zeros((M, K), dtype=np.uint16))
    w_d = H.to_dev(np.zeros(K * N // 2, dtype=np.uint8))
    ws_d = torch.ones(G * N, dtype=torch.float32, device=H.DEV)

    def call(src=capi.DT_BF16, dst_dt=capi.DT_BF16, compute=capi.DT_S8, dyn=True, sdims=(M, 1), wdims=(G, N), fmt="n"):
        p = lowoha.MatmulParams(src=src, wei=capi.DT_S4, dst=dst_dt, compute=compute)
        p.dynamic_quant = dyn
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, sdims)
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, wdims)
        p.mem_format_b = fmt
        if fmt == "r":
            p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        dst = torch.zeros((M, N), dtype=torch.bfloat16 if dst_dt == capi.DT_BF16 else torch.float32, device=H.DEV)
        return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, None, 0.0, dst, N, True, p)

    assert call() == capi.SUCCESS
    assert call(src=capi.DT_S8) == capi.FAILURE
    assert call(src=capi.DT_F32) == capi.FAILURE
    assert call(dst_dt=capi.DT_F32) == capi.FAILURE
    assert call(compute=capi.DT_BF16) == capi.FAILURE
    assert call(dyn=False) == capi.SUCCESS                 # weight-only quantization: another path (test_gpu_woq.py)
    assert call(sdims=(M, 3)) == capi.FAILURE
    assert call(wdims=(G, N - 1)) == capi.FAILURE
    assert call(wdims=(3, N)) == capi.FAILURE
    assert call(wdims=(32, N)) == capi.FAILURE             # groups of 2
    assert call(fmt="r") == capi.FAILURE                   # no prepacked form of s4 weights
    capi.load().zmi_clear_weight_cache()


def test_w4a8_reference_example_recipe(zo):
    """The reference's W4A8 example (examples/lowoha_matmul_example.cpp:370-457): M=8 K=128 N=64, groups of 32, bf16
    ones as activations, every s4 code 1, bf16 weight scales 1 + 0.05 g, bf16 {M,1} source-scale buffer (overwritten
    by the dynamic quantization).  Every row quantizes to 127 with scale 1/127, every group sum is 32 * 127, so the
    output is 32 * sum_g bf16(1 + 0.05 g) = 137.5 up to f32 rounding: 137 or 138 in bf16."""
    M, K, N, G = 8, 128, 64, 4
    x = np.full((M, K), 0x3F80, dtype=np.uint16)
    packed = np.full(K * N // 2, 0x11, dtype=np.uint8)
    ws = H.bf16_bits(np.repeat((1.0 + 0.05 * np.arange(G, dtype=np.float32))[:, None], N, axis=1))
    sc_d = H.to_dev(H.bf16_bits((0.02 + 0.001 * np.arange(M)).astype(np.float32)))
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    p.src_scale = lowoha.QuantParam(sc_d, capi.DT_BF16, (M, 1))
    p.wei_scale = lowoha.QuantParam(H.to_dev(ws), capi.DT_BF16, (G, N))
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(x), K, H.to_dev(packed), N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    got = H.to_host(dst)
    vals = (got.astype(np.uint32) << 16).view(np.float32)
    assert np.all((vals == 137.0) | (vals == 138.0)), np.unique(vals)
    # the computed scales replace the caller's: bf16(1 / 127)
    want_s = H.bf16_bits(np.full(M, np.float32(1.0) / np.float32(127.0), dtype=np.float32))
    assert np.array_equal(H.to_host(sc_d), want_s)
    capi.load().zmi_clear_weight_cache()


@pytest.mark.parametrize("with_buffer", [True, False])
@pytest.mark.parametrize("wei,M,K,N,G,sdims", [
    (capi.DT_S4, 16, 4096, 200, 32, "token"), (capi.DT_S4, 16, 4096, 72, 32, "group"), (capi.DT_S4, 40, 512, 64, 8, "token"),
    (capi.DT_S4, 9, 256, 48, 4, "group"), (capi.DT_S4, 1, 256, 254, 16, "token"), (capi.DT_S4, 1, 4096, 64, 32, "token"),
    (capi.DT_S8, 1, 520, 96, 1, "token"), (capi.DT_S8, 1, 8192, 40, 1, "token"),
    (capi.DT_S8, 16, 4096, 320, 1, "token"), (capi.DT_S8, 4, 512, 96, 1, "token"), (capi.DT_S8, 100, 1024, 64, 1, "token"),
    (capi.DT_S8, 300, 256, 300, 1, "token"), (capi.DT_S8, 16, 4096, 64, 32, "group"), (capi.DT_S8, 33, 512, 40, 8, "group")])
def test_bf16_source_scale_dtype_is_what_the_gemm_multiplies_by(zo, wei, M, K, N, G, sdims, with_buffer):
    """src_scale.dt = bf16 (as in the reference's W4A8 example): the computed f32 scales are narrowed into the scale
    buffer -- the caller's, or the library's own of that dtype -- and the GEMM reads the narrowed values, while the
    rows are quantized with the f32 scales (lowoha_reorder_utils.cpp:600-628, 835-856; reorder_quantization.cpp:103-117).
    Covers W4A8 and s8 weights, per-token and per-group scales, the fused decode launches and the separate ones."""
    rng = np.random.default_rng(M + K + N + G + int(with_buffer))
    x = H.bf16_bits((rng.standard_normal((M, K)) * 2).astype(np.float32))
    if wei == capi.DT_S4:
        w = rng.integers(0, 256, K * N // 2, dtype=np.uint8)
        ws = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
    else:
        w = H.gen_weights(rng, K, N)
        ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    dims = (M, 1) if sdims == "token" else (M, G)
    n_sc = int(np.prod(dims))
    sc_d = torch.zeros(n_sc, dtype=torch.bfloat16, device=H.DEV) if with_buffer else None
    dst_dt = capi.DT_BF16 if wei == capi.DT_S4 else capi.DT_F32
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=wei, dst=dst_dt, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(sc_d, capi.DT_BF16, dims)
    p.wei_scale = lowoha.QuantParam(H.to_dev(ws), capi.DT_F32, (G, N) if G > 1 else (1, N))
    dst = torch.zeros((M, N), dtype=torch.bfloat16 if dst_dt == capi.DT_BF16 else torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(x), K, H.to_dev(w), N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, w, ph.flat(keep), M, N, K, ldb=N, want_scales=True, n_scales=max(n_sc, M))
    assert st == capi.SUCCESS
    if with_buffer:
        assert np.array_equal(H.to_host(sc_d), H.bf16_bits(scales[:n_sc]))      # (the oracle's are bf16 values held in f32)
    assert np.array_equal(H.to_host(dst), want), lowoha.last_kernel()
    capi.load().zmi_clear_weight_cache()
