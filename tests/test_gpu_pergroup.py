"""GPU parity of matmul_direct with per-group symmetric scales: source scales {M,G}, weight scales {G,N}
(reference: validation lowoha_operators/matmul/lowoha_matmul_utils.cpp:253-301, arithmetic
operators/matmul/matmul_ref_kernel.cpp:917-1001).  The kernel adds the group terms in the reference's order
with one rounding per step, so f32 results without an activation are compared bit for bit."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.test_gpu_reorder_edges import _run_both

pytestmark = pytest.mark.gpu


def _scales(rng, M, N, G):
    ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    return ss, ws


# (M, K, N, G): group sizes 64, 128, 256, 32 and 16; one row .. several 64-row blocks; ragged N
SHAPES = [(2, 192, 354, 3), (40, 192, 154, 3), (200, 320, 294, 5),   # K = 64 x odd: K_pad holds one chunk past K
          (1, 128, 32, 2), (5, 256, 33, 4), (16, 4096, 512, 32), (16, 1024, 100, 4), (40, 512, 100, 16),
          (70, 192, 64, 12), (17, 64, 16, 4), (300, 1024, 260, 8), (130, 2048, 48, 32), (3, 32, 5, 2),
          # up to 16 rows with K = 512 .. 4096 and whole groups per eighth of K: the decode-shaped kernel, every
          # (chunks, groups) per wavefront pair it is built for
          (16, 4096, 40, 64), (9, 4096, 33, 16), (2, 4096, 64, 8), (16, 2048, 96, 32), (5, 2048, 32, 16),
          (1, 2048, 70, 8), (16, 1024, 64, 16), (3, 1024, 31, 8), (12, 512, 50, 8),
          # groups of 32 on it (two per chunk, 16 integer tiles per round)
          (16, 4096, 64, 128), (7, 2048, 40, 64), (16, 1024, 33, 32), (2, 512, 96, 16)]


@pytest.mark.parametrize("M,K,N,G", SHAPES)
def test_static_per_group_f32_bit_exact(zo, M, K, N, G):
    rng = np.random.default_rng(M * 7 + K + N + G)
    ss, ws = _scales(rng, M, N, G)
    bias = rng.standard_normal(N).astype(np.float32)
    for transA, transB, pad, with_bias in ((False, False, 0, True), (False, True, 3, False), (True, False, 5, True)):
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
        assert lowoha.last_kernel().startswith("pergroup_")
        assert np.array_equal(got[:, :N], want[:, :N]), (M, K, N, G, transA, transB)
        assert np.all(got[:, N:] == 0)


@pytest.mark.parametrize("M,K,N,G", [(16, 4096, 512, 32), (40, 512, 100, 16), (200, 256, 64, 2)])
@pytest.mark.parametrize("po", [capi.PO_SWISH, capi.PO_GELU_TANH, capi.PO_RELU])
def test_static_per_group_bf16_post_ops_prepacked_bf16_scales(zo, M, K, N, G, po):
    """bf16 destination, one activation, prepacked weights, scales stored as bf16."""
    rng = np.random.default_rng(po * 100 + M)
    ss, ws = _scales(rng, M, N, G)
    ss_b, ws_b = H.bf16_bits(ss), H.bf16_bits(ws)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    ss_d, ws_d = H.to_dev(ss_b), H.to_dev(ws_b)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_BF16, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_BF16, (G, N))
    p.postop_ = [lowoha.PostOp(po)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, H.prepack(w_d, K, N), N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=ss_b, wei_scale=ws_b)
    ph.mem_format_b = "n"
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
    assert st == capi.SUCCESS
    if po == capi.PO_RELU:
        assert np.array_equal(H.to_host(dst), want)
    else:
        H.check_bf16(H.to_host(dst), want, atol=1e-6 if po == capi.PO_GELU_TANH else 0.0, max_frac=1e-2)


def test_generic_kernel_on_a_decode_shaped_problem(zo, monkeypatch):
    """The one-wavefront-per-column-block kernel on a shape the decode-shaped kernel would take (env switch)."""
    monkeypatch.setenv("ZMI_PERGROUP_GENERIC", "1")
    rng = np.random.default_rng(5)
    M, K, N, G = 16, 2048, 96, 16
    ss, ws = _scales(rng, M, N, G)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, host_bufs={"src_scale": ss, "wei_scale": ws})
    assert lowoha.last_kernel() == "pergroup_mfma16x16x64"
    assert np.array_equal(got, want)


def test_static_per_group_alpha_beta(zo):
    rng = np.random.default_rng(77)
    M, K, N, G = 20, 256, 40, 4
    ss, ws = _scales(rng, M, N, G)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    c0 = rng.standard_normal((M, N)).astype(np.float32)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, host_bufs={"src_scale": ss, "wei_scale": ws}, dst_np=c0,
                          alpha=0.5, beta=1.5)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,K,N,G", [(16, 4096, 14336, 32), (4, 4096, 1024, 64), (1, 512, 64, 8), (33, 256, 40, 16),
                                     (16, 4096, 320, 128), (9, 1024, 64, 32),
                                     (150, 1024, 96, 8)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_dynamic_per_group(zo, M, K, N, G, src_dt):
    """bf16 / f32 rows quantized per (row, group) by the library: the {M,G} scales it writes are bit-exact, and so
    is the f32 output (exact scales, exact s8 rows, the reference's order of additions).  The first case has
    the shape of the headline decode configuration."""
    if src_dt == capi.DT_F32 and N > 2000:
        pytest.skip("one full-size case is enough")
    rng = np.random.default_rng(M + K + G)
    x32 = (rng.standard_normal((M, K)) * rng.uniform(0.2, 3.0, (M, 1))).astype(np.float32)
    x32[0, 3] = np.nan
    x = H.bf16_bits(x32) if src_dt == capi.DT_BF16 else x32
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    scales_d = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    p = lowoha.MatmulParams(src=src_dt, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8, bias=capi.DT_F32)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(scales_d, capi.DT_F32, (M, G))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
    p.weight_cache_type = 0
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, H.to_dev(bias), 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel().startswith("pergroup_")
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    keep = []
    st, want, _, scales = zo.matmul_int8(x, w, ph.flat(keep), M, N, K, bias=bias, want_scales=True, n_scales=M * G)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(scales_d), scales)
    assert np.array_equal(H.to_host(dst), want)


def test_per_group_rejections(zo):
    M, K, N = 4, 192, 16
    a_d = H.to_dev(np.ones((M, K), dtype=np.int8))
    w_d = H.to_dev(np.ones((K, N), dtype=np.int8))
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)

    def call(G, wei_dims, src=capi.DT_S8, dst_dt=capi.DT_F32, zp=False):
        ss_d = torch.ones(M * G, dtype=torch.float32, device=H.DEV)
        ws_d = torch.ones(int(np.prod(wei_dims)), dtype=torch.float32, device=H.DEV)
        p = lowoha.MatmulParams(src=src, wei=capi.DT_S8, dst=dst_dt)
        p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, G))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, wei_dims)
        if zp:
            z = np.array([3], dtype=np.int32)
            p.src_zp = lowoha.QuantParam(z.ctypes.data, capi.DT_S32, (1,))
        p.weight_cache_type = 0
        return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, False, p)

    assert call(3, (3, N)) == capi.SUCCESS                       # group size 64
    assert call(4, (4, N)) == capi.UNIMPLEMENTED                 # group size 48: documented limit of this build
    assert call(3, (1, N)) == capi.FAILURE                       # per-channel weight scale (reference: failure)
    assert call(3, (2, N)) == capi.FAILURE                       # group counts differ
    assert call(5, (5, N)) == capi.FAILURE                       # K % G != 0
    assert call(3, (3, N), zp=True) == capi.FAILURE              # symmetric only
    assert call(3, (3, N), src=capi.DT_U8) == capi.FAILURE       # s8 / bf16 / f32 sources only
    assert call(3, (3, N), dst_dt=capi.DT_S8) == capi.FAILURE    # f32 / bf16 destinations only


# ---------------------------------------------------------------- the quantization entry points
@pytest.mark.parametrize("M,K,G", [(1, 64, 2), (7, 512, 16), (33, 4096, 32), (5, 20000, 4), (300, 1408, 11)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_reorder_direct_dynamic_per_group_bit_exact(zo, M, K, G, src_dt):
    """reorder_direct with {M,G} scale dims (lowoha_reorder.cpp:167-171): s8 rows and scales equal the oracle's,
    with zero groups, NaN and infinities; scales as f32 and as bf16; scales only (dst == nullptr)."""
    rng = np.random.default_rng(M * 131 + K + G)
    xf = (rng.standard_normal((M, K)) * rng.uniform(0.01, 30, (M, 1))).astype(np.float32)
    gs = K // G
    xf[0, :gs] = 0.0                        # a zero group: scale clamps to 1e-10
    xf[M - 1, K - 1] = np.inf
    xf[M // 2, 1] = np.nan
    x = H.bf16_bits(xf) if src_dt == capi.DT_BF16 else xf
    x_d = H.to_dev(x)
    q, s = zo.quant_per_group(x, src_dt, G)

    def params(scale_buf, scale_dt):
        rp = lowoha.ReorderParams()
        rp.src_dtype, rp.dst_dtype = src_dt, capi.DT_S8
        rp.dynamic_quant = True
        rp.algo = 1
        rp.src_shape = rp.dst_shape = (M, K)
        rp.scale = lowoha.QuantParam(scale_buf, scale_dt, (M, G))
        return rp

    q_d = torch.zeros((M, K), dtype=torch.int8, device=H.DEV)
    s_d = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q_d, params(s_d, capi.DT_F32))
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == "quant_groups"
    assert np.array_equal(H.to_host(s_d).reshape(M, G), s)
    assert np.array_equal(H.to_host(q_d), q)
    # bf16 scales: the f32 scale rounded to nearest even; the rows are quantized with the f32 scale
    sb_d = torch.zeros(M * G, dtype=torch.bfloat16, device=H.DEV)
    q2_d = torch.zeros((M, K), dtype=torch.int8, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q2_d, params(sb_d, capi.DT_BF16))
    assert st == capi.SUCCESS, lowoha.last_error()
    assert np.array_equal(H.to_host(sb_d).reshape(M, G), H.bf16_bits(s))
    assert torch.equal(q2_d, q_d)
    # scales only
    s2 = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, None, params(s2, capi.DT_F32))
    assert st == capi.SUCCESS and torch.equal(s2, s_d)


def test_reorder_direct_per_group_needs_divisible_k(zo):
    M, K = 4, 100
    x_d = torch.zeros((M, K), dtype=torch.float32, device=H.DEV)
    q_d = torch.zeros((M, K), dtype=torch.int8, device=H.DEV)
    s_d = torch.zeros(M * 3, dtype=torch.float32, device=H.DEV)
    rp = lowoha.ReorderParams()
    rp.src_dtype, rp.dst_dtype = capi.DT_F32, capi.DT_S8
    rp.dynamic_quant = True
    rp.algo = 1
    rp.src_shape = rp.dst_shape = (M, K)
    rp.scale = lowoha.QuantParam(s_d, capi.DT_F32, (M, 3))
    assert lowoha.reorder_direct(x_d, q_d, rp) == capi.FAILURE


@pytest.mark.parametrize("M,K,G", [(1, 64, 1), (7, 515, 1), (33, 4096, 1), (5, 20000, 1), (9, 512, 16), (300, 1408, 11)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_reorder_direct_asymmetric_dynamic_quantization_bit_exact(zo, M, K, G, src_dt):
    """reorder_direct with a zero-point buffer: u8 rows, f32 (or bf16) scales and s32 zero-points per token ({M,1}) or
    per group ({M,G}) equal the oracle's (reference: compute_asymmetric_scale_zp and the u8 kernels,
    dynamic_quant_impl/per_token_avx512_f32_fma_kernel.cpp:89-116, :565-680), with constant slices, shifted rows, NaN
    and infinities."""
    rng = np.random.default_rng(M * 17 + K + G)
    xf = (rng.standard_normal((M, K)) * rng.uniform(0.01, 30, (M, 1)) + rng.uniform(-40, 40, (M, 1))).astype(np.float32)
    gs = K // G
    xf[0, :gs] = 2.5                         # a constant slice: its range is widened to 1
    xf[M - 1, K - 1] = np.inf
    xf[M // 2, 1] = np.nan
    if M > 3:
        xf[3, :] = np.nan                    # nothing finite: range [0, 1], zero-point 0, codes 0
    x = H.bf16_bits(xf) if src_dt == capi.DT_BF16 else xf
    x_d = H.to_dev(x)
    q, s, z = zo.quant_asym(x, src_dt, G)

    def params(scale_buf, scale_dt, zp_buf):
        rp = lowoha.ReorderParams()
        rp.src_dtype, rp.dst_dtype = src_dt, capi.DT_U8
        rp.dynamic_quant = True
        rp.algo = 1
        rp.src_shape = rp.dst_shape = (M, K)
        rp.scale = lowoha.QuantParam(scale_buf, scale_dt, (M, G))
        rp.zero_point = lowoha.QuantParam(zp_buf, capi.DT_S32, (M, G))
        return rp

    q_d = torch.zeros((M, K), dtype=torch.uint8, device=H.DEV)
    s_d = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    z_d = torch.zeros(M * G, dtype=torch.int32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q_d, params(s_d, capi.DT_F32, z_d))
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == ("quant_asym_per_token" if G == 1 else "quant_asym_groups")
    assert np.array_equal(H.to_host(s_d).reshape(M, G), s)
    assert np.array_equal(H.to_host(z_d).reshape(M, G), z)
    assert np.array_equal(H.to_host(q_d), q)
    # bf16 scales: the f32 scale narrowed for the caller, the rows quantized with the f32 scale; scales only
    sb_d = torch.zeros(M * G, dtype=torch.bfloat16, device=H.DEV)
    z2_d = torch.zeros(M * G, dtype=torch.int32, device=H.DEV)
    q2_d = torch.zeros((M, K), dtype=torch.uint8, device=H.DEV)
    st = lowoha.reorder_direct(x_d, q2_d, params(sb_d, capi.DT_BF16, z2_d))
    assert st == capi.SUCCESS, lowoha.last_error()
    assert np.array_equal(H.to_host(sb_d).reshape(M, G), H.bf16_bits(s))
    assert torch.equal(q2_d, q_d) and torch.equal(z2_d, z_d)
    s3 = torch.zeros(M * G, dtype=torch.float32, device=H.DEV)
    z3 = torch.zeros(M * G, dtype=torch.int32, device=H.DEV)
    st = lowoha.reorder_direct(x_d, None, params(s3, capi.DT_F32, z3))
    assert st == capi.SUCCESS and torch.equal(s3, s_d) and torch.equal(z3, z_d)
    # scale and zero-point dims must agree
    bad = params(s_d, capi.DT_F32, z_d)
    bad.zero_point = lowoha.QuantParam(z_d, capi.DT_S32, (M * G, 1) if G > 1 else (1, M))
    if bad.zero_point.dims != bad.scale.dims:
        assert lowoha.reorder_direct(x_d, q_d, bad) == capi.FAILURE


@pytest.mark.parametrize("G", [1, 8])
def test_group_dynamic_quant_per_token_and_per_group(zo, G):
    """group_dynamic_quant (lowoha_reorder.cpp:279-404) through the C ABI: several matrices, one with no rows, padded
    row strides; num_groups <= 1 is per token, > 1 per group."""
    import ctypes as C
    rng = np.random.default_rng(40 + G)
    shapes = [(5, 64), (0, 128), (33, 512), (2, 1024)]
    lib = capi.load()
    n = len(shapes)
    keep, want = [], []
    srcs, dsts, scales = (C.c_void_p * n)(), (C.c_void_p * n)(), (C.c_void_p * n)()
    Ms, Ks = (C.c_int32 * n)(), (C.c_int32 * n)()
    lds, ldd = (C.c_int64 * n)(), (C.c_int64 * n)()
    for i, (M, K) in enumerate(shapes):
        pad = 8 * (i % 2)
        xf = (rng.standard_normal((max(M, 1), K + pad)) * 3).astype(np.float32)
        x = H.bf16_bits(xf)
        x_d = H.to_dev(x)
        q_d = torch.zeros((max(M, 1), K + pad), dtype=torch.int8, device=H.DEV)
        s_d = torch.zeros(max(M, 1) * G, dtype=torch.float32, device=H.DEV)
        keep += [x_d, q_d, s_d]
        srcs[i], dsts[i], scales[i] = x_d.data_ptr(), q_d.data_ptr(), s_d.data_ptr()
        Ms[i], Ks[i], lds[i], ldd[i] = M, K, K + pad, K + pad
        xs = np.ascontiguousarray(x[:, :K])
        want.append(zo.quant_per_group(xs, capi.DT_BF16, G) if G > 1 else zo.quant_per_token(xs, capi.DT_BF16))
    gp = capi.GroupDqParamsT(capi.DT_BF16, capi.DT_S8, capi.DT_F32, 0, G)
    st = lib.zmi_group_dynamic_quant(n, srcs, Ms, Ks, lds, dsts, ldd, scales, C.byref(gp))
    assert st == capi.SUCCESS, lowoha.last_error()
    for i, (M, K) in enumerate(shapes):
        if M == 0:
            continue
        q, s = want[i]
        assert np.array_equal(H.to_host(keep[3 * i + 1])[:M, :K], q[:M])
        assert np.array_equal(H.to_host(keep[3 * i + 2])[:M * G], np.asarray(s).reshape(-1)[:M * G])
        assert np.all(H.to_host(keep[3 * i + 1])[:, K:] == 0)          # padding bytes of dst are left alone


def test_grouped_call_with_per_group_ggml_and_s4_experts(zo):
    """group_matmul_direct with experts the grouped kernels do not take -- per-group scales on static s8 rows, per-group
    dynamic quantization, GGML Q8_0 packed weights, W4A8 -- runs them on the matmul_direct path (reference:
    group_matmul/group_matmul_dispatch.cpp:472-515, group_matmul_direct.cpp:1222-1260); followed here by the
    weighted reduce over the f32 expert outputs, and by a gated activation over them."""
    rng = np.random.default_rng(77)
    K, N, T = 256, 48, 6
    G = K // 32
    E = 3
    # expert 0: static s8 rows, {T,G} x {G,N} f32 scales
    a0 = rng.integers(-128, 128, (T, K), dtype=np.int8)
    w0 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ss0 = rng.uniform(0.005, 0.03, (T, G)).astype(np.float32)
    ws0 = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    p0 = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    ss0_d, ws0_d = H.to_dev(ss0), H.to_dev(ws0)
    p0.src_scale = lowoha.QuantParam(ss0_d, capi.DT_F32, (T, G))
    p0.wei_scale = lowoha.QuantParam(ws0_d, capi.DT_F32, (G, N))
    # expert 1: bf16 rows quantized per group, f32 out
    x1 = H.bf16_bits(rng.standard_normal((T, K)).astype(np.float32))
    w1 = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ws1 = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    ws1_d = H.to_dev(ws1)
    p1 = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
    p1.dynamic_quant = True
    p1.src_scale = lowoha.QuantParam(None, capi.DT_F32, (T, G))
    p1.wei_scale = lowoha.QuantParam(ws1_d, capi.DT_F32, (G, N))
    # expert 2: static s8 rows, GGML Q8_0 packed weights ([N][K/32] blocks of {fp16 d, int8 qs[32]})
    a2 = rng.integers(-128, 128, (T, K), dtype=np.int8)
    rows2 = rng.integers(-127, 128, (N, K), dtype=np.int8)
    d16 = rng.uniform(1e-3, 0.02, (N, G)).astype(np.float16)
    blk = np.zeros((N, G, 34), dtype=np.uint8)
    blk[:, :, :2] = d16.view(np.uint16).reshape(N, G, 1).view(np.uint8)
    blk[:, :, 2:] = rows2.reshape(N, G, 32).view(np.uint8)
    packed2 = blk.reshape(-1)
    ss2 = rng.uniform(0.005, 0.03, (T, G)).astype(np.float32)
    ss2_d = H.to_dev(ss2)
    p2 = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
    p2.src_scale = lowoha.QuantParam(ss2_d, capi.DT_F32, (T, G))
    p2.pack_format_b = 1

    srcs = [H.to_dev(a0), H.to_dev(x1), H.to_dev(a2)]
    weis = [H.to_dev(w0), H.to_dev(w1), H.to_dev(packed2)]
    dst = [torch.zeros((T, N), dtype=torch.float32, device=H.DEV) for _ in range(E)]
    ids = [(t % E, (t + 1) % E) for t in range(T)]
    rp = [dst[e].data_ptr() + t * N * 4 for t in range(T) for e in ids[t]]
    tw_h = rng.uniform(0.2, 0.8, (T, 2)).astype(np.float32)
    out = torch.zeros((T, N), dtype=torch.float32, device=H.DEV)
    pp = lowoha.MoePostop(T, 2, out, N, H.to_dev(tw_h), rp)
    args = (["r"] * E, [False] * E, [False, False, True], [T] * E, [N] * E, [K] * E, [1.0] * E,
            srcs, [K] * E, weis, [N, N, K], [None] * E, [0.0] * E, dst, [N] * E, [True] * E, [p0, p1, p2])
    st = lowoha.group_matmul_direct(*args, moe_postop=pp)
    assert st == capi.SUCCESS, lowoha.last_error()

    want = []
    keep = []
    st, y, _, _ = zo.matmul_int8(a0, w0, H.host_params(p0, src_scale=ss0, wei_scale=ws0).flat(keep), T, N, K)
    assert st == capi.SUCCESS
    want.append(y)
    st, y, _, _ = zo.matmul_int8(x1, w1, H.host_params(p1, src_scale=None, wei_scale=ws1).flat(keep), T, N, K)
    assert st == capi.SUCCESS
    want.append(y)
    st, y, _, _ = zo.matmul_int8(a2, packed2, H.host_params(p2, src_scale=ss2).flat(keep), T, N, K, transB=True, ldb=K)
    assert st == capi.SUCCESS
    want.append(y)
    for e in range(E):
        assert np.array_equal(H.to_host(dst[e]), want[e])
    red = zo.moe_reduce([want[e][t] for t in range(T) for e in ids[t]], tw_h, capi.DT_F32, N)
    assert np.array_equal(H.to_host(out), red)

    # a gated activation on top: the stand-alone activation pass over the experts' (wide, f32) outputs
    st = lowoha.group_matmul_direct(*args, gated_act=capi.ACT_SILU_AND_MUL)
    assert st == capi.SUCCESS, lowoha.last_error()
    for e in range(E):
        act = zo.gated_act(capi.ACT_SILU_AND_MUL, want[e].copy(), capi.DT_F32)
        H.check_f32(H.to_host(dst[e])[:, :N // 2], act[:, :N // 2], rtol=2e-6, atol=1e-7)

    # two W4A8 experts (bf16 rows, packed s4 weights, bf16 out), ragged row counts
    Ms = [5, 9]
    xs, w4s, wss, ps, dsts = [], [], [], [], []
    for e, m in enumerate(Ms):
        xs.append(H.bf16_bits(rng.standard_normal((m, K)).astype(np.float32)))
        codes = rng.integers(0, 256, K * N // 2, dtype=np.uint8)
        w4s.append(codes)
        wss.append(rng.uniform(0.01, 0.1, (G, N)).astype(np.float32))
        pe = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8)
        pe.dynamic_quant = True
        pe.src_scale = lowoha.QuantParam(None, capi.DT_F32, (m, 1))
        pe.wei_scale = lowoha.QuantParam(H.to_dev(wss[e]), capi.DT_F32, (G, N))
        ps.append(pe)
        dsts.append(torch.zeros((m, N), dtype=torch.bfloat16, device=H.DEV))
    st = lowoha.group_matmul_direct(["r"] * 2, [False] * 2, [False] * 2, Ms, [N] * 2, [K] * 2, [1.0] * 2,
                                    [H.to_dev(x) for x in xs], [K] * 2, [H.to_dev(w) for w in w4s], [N] * 2, [None] * 2,
                                    [0.0] * 2, dsts, [N] * 2, [True] * 2, ps)
    assert st == capi.SUCCESS, lowoha.last_error()
    for e, m in enumerate(Ms):
        st, y, _, _ = zo.matmul_int8(xs[e], w4s[e], H.host_params(ps[e], src_scale=None, wei_scale=wss[e]).flat(keep), m, N, K,
                                     ldb=N)
        assert st == capi.SUCCESS
        assert np.array_equal(H.to_host(dsts[e]), y)
    capi.load().zmi_clear_weight_cache()
