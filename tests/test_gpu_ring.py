"""GPU parity of the large-M (fragment-major, MFMA-bound) kernel through matmul_direct:
tile-edge shapes for every tile height, the straight-line bf16 epilogues next to
their edge forms, unaligned destinations, u8 sources, the destination dtypes
that go through its generic epilogue, and the K-sliced launch (partial tiles + reduction
kernel) for both of its tile heights."""
import os

import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.test_gpu_reorder_edges import _run_both

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["128", "256"])
def top(request):
    """Forces the largest tile height of the single-problem launch."""
    old = os.environ.get("ZMI_GEMM_TOP")
    os.environ["ZMI_GEMM_TOP"] = request.param
    yield int(request.param)
    if old is None:
        del os.environ["ZMI_GEMM_TOP"]
    else:
        os.environ["ZMI_GEMM_TOP"] = old


# rows: one full tile + remainders that land in each of the 64 / 128 / 256 row kernels;
# columns: inside one tile, across tiles, not a multiple of 4, not a multiple of 32
@pytest.mark.parametrize("M,K,N", [(129, 64, 256), (192, 130, 260), (257, 96, 513), (320, 200, 31), (449, 1024, 300),
                                   (513, 48, 770)])
def test_s32_accumulators_bit_exact_every_tile_height(zo, top, M, K, N):
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    zp = np.array([131], dtype=np.int32)
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
    dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "ring" in lowoha.last_kernel()
    want = (a.astype(np.int64) - 131) @ w.astype(np.int64)
    assert np.array_equal(H.to_host(dst).astype(np.int64), want)


@pytest.mark.parametrize("po", [None, capi.PO_RELU, capi.PO_SWISH, capi.PO_GELU_TANH])
@pytest.mark.parametrize("M,K,N,ldc_pad", [(300, 256, 512, 0),      # interior strips + a row remainder
                                           (260, 192, 322, 0),      # column edge inside a tile, 8-byte stores misaligned rows
                                           (384, 128, 256, 3)])     # padded leading dimension: scalar stores
def test_bf16_epilogues_interior_and_edges(zo, top, po, M, K, N, ldc_pad):
    rng = np.random.default_rng(M + N + (po or 0))
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = rng.uniform(0.01, 0.03, M).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    if po is not None:
        p.postop_ = [lowoha.PostOp(po)]
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws}, ldc=N + ldc_pad)
    H.check_bf16(got[:, :N], want[:, :N], atol=1e-6 if po == capi.PO_GELU_TANH else 0.0, max_frac=5e-3)
    assert np.all(got[:, N:] == 0)


@pytest.mark.parametrize("dst_dt", [capi.DT_F32, capi.DT_S8, capi.DT_U8])
def test_f32_exact_and_quantized_destinations(zo, top, dst_dt):
    rng = np.random.default_rng(dst_dt)
    M, K, N = 270, 160, 290
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.02], dtype=np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    bufs = {"src_scale": ss, "wei_scale": ws}
    if dst_dt != capi.DT_F32:
        ds = np.array([7.5], dtype=np.float32)
        dz = np.array([3], dtype=np.int32)
        p.dst_scale = lowoha.QuantParam(ds.ctypes.data, capi.DT_F32, (1,))
        p.dst_zp = lowoha.QuantParam(dz.ctypes.data, capi.DT_S32, (1,))
        bufs.update(dst_scale=ds, dst_zp=dz)
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs=bufs)
    # separately rounded f32 steps in the reference's order on both sides
    assert np.array_equal(got, want)


def test_transposed_source_and_weights(zo, top):
    rng = np.random.default_rng(11)
    M, K, N = 200, 90, 140
    a = rng.integers(-128, 128, (K, M + 2), dtype=np.int8)      # A^T with padding
    w = rng.integers(-127, 128, (N, K + 6), dtype=np.int8)      # B^T with padding
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, lda=M + 2, ldb=K + 6, transA=True, transB=True)
    assert np.array_equal(got, want)


@pytest.fixture
def env():
    """Sets environment switches for one test and restores them afterwards."""
    saved = {}

    def set_(**kv):
        for k, v in kv.items():
            saved.setdefault(k, os.environ.get(k))
            os.environ[k] = str(v)

    yield set_
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


# 64-row tiles (M <= 64) and 128-row tiles; K not a multiple of the slice count, fewer
# 64-k stages than slices asked for (K = 100: two stages), several row and column tiles
# finished by the slice that arrives last at its tile's word, or (without the arrival words) by a reduction launch
@pytest.mark.parametrize("arrivals", [True, False])
@pytest.mark.parametrize("slices", [2, 3, 8])
@pytest.mark.parametrize("M,K,N", [(20, 256, 256), (64, 1000, 700), (100, 100, 300), (129, 512, 256), (300, 640, 515)])
def test_k_sliced_s32_accumulators_bit_exact(zo, env, M, K, N, slices, arrivals):
    env(ZMI_DECODE_MAX_M=16, ZMI_RING_MIN_M=17, ZMI_RING_SPLITK=slices)
    if not arrivals:
        env(ZMI_NO_SLICE_ARRIVALS=1)
    rng = np.random.default_rng(M + K + N)
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    zp = np.array([131], dtype=np.int32)
    want = (a.astype(np.int64) - 131) @ w.astype(np.int64)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    for _ in range(2):   # the partial-tile scratch is reused call after call
        p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
        p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
        dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, False, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        assert "ksliced" in lowoha.last_kernel()
        assert np.array_equal(H.to_host(dst).astype(np.int64), want)


@pytest.mark.parametrize("arrivals", [True, False])
@pytest.mark.parametrize("po", [None, capi.PO_SWISH, capi.PO_GELU_TANH])
@pytest.mark.parametrize("M,K,N,ldc_pad", [(48, 512, 320, 0), (200, 384, 322, 3)])
def test_k_sliced_bf16_epilogues(zo, env, po, M, K, N, ldc_pad, arrivals):
    env(ZMI_DECODE_MAX_M=16, ZMI_RING_MIN_M=17, ZMI_RING_SPLITK=3)
    if not arrivals:
        env(ZMI_NO_SLICE_ARRIVALS=1)
    rng = np.random.default_rng(M + N + (po or 0))
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = rng.uniform(0.01, 0.03, M).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    if po is not None:
        p.postop_ = [lowoha.PostOp(po)]
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws}, ldc=N + ldc_pad)
    assert "ksliced" in lowoha.last_kernel()
    H.check_bf16(got[:, :N], want[:, :N], atol=1e-6 if po == capi.PO_GELU_TANH else 0.0, max_frac=5e-3)
    assert np.all(got[:, N:] == 0)


@pytest.mark.parametrize("M,K,N", [(100, 256, 6200), (200, 192, 3300), (256, 320, 3100)])
def test_unsliced_64_row_tiles_for_a_wide_problem_with_few_rows(zo, env, M, K, N):
    """65 .. 256 rows against many weight columns and a short K: the launch plan takes 64-row tiles, unsliced (a
    partly filled last tile included).  Raw s32 sums against the integer product, bf16 + SiLU against the oracle."""
    env(ZMI_DECODE_MAX_M=16, ZMI_RING_MIN_M=17)
    rng = np.random.default_rng(M + K + N)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    want = a.astype(np.int64) @ w.astype(np.int64)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, None, 0.0, dst, N, False, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == "ring_mfma32x32x32_top64"
    assert np.array_equal(H.to_host(dst).astype(np.int64), want)
    ss = rng.uniform(0.01, 0.03, M).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws})
    assert lowoha.last_kernel() == "ring_mfma32x32x32_top64"
    H.check_bf16(got, want, max_frac=5e-3)


@pytest.mark.parametrize("M,K,N,slices", [(100, 3100, 1500, 2), (130, 6200, 700, 4), (257, 1600, 2600, 1)])
def test_plan_takes_64_row_tiles_in_k_slices_by_itself(zo, env, M, K, N, slices):
    """More than 64 rows, few tiles: the plan picks 64-row tiles and as many K slices (4, 2 or 1) as leave a slice 24
    stages of 64 k; partly filled last row tile, K that is no multiple of 64.  s32 sums against the integer product,
    the f32 chain with a bias against the oracle, twice (the arrival words must be zero again)."""
    env(ZMI_DECODE_MAX_M=16, ZMI_RING_MIN_M=17)
    rng = np.random.default_rng(M + K + N)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    want = a.astype(np.int64) @ w.astype(np.int64)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    name = "ring_mfma32x32x32_top64_ksliced" if slices > 1 else "ring_mfma32x32x32_top64"
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    for rep in range(2):
        dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        assert lowoha.last_kernel() == name
        assert np.array_equal(H.to_host(dst).astype(np.int64), want), rep
    ss = rng.uniform(0.01, 0.03, M).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws})
    assert lowoha.last_kernel() == name
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dst_dt", [capi.DT_F32, capi.DT_S8, capi.DT_U8])
def test_k_sliced_f32_exact_and_quantized_destinations(zo, env, dst_dt):
    env(ZMI_DECODE_MAX_M=16, ZMI_RING_MIN_M=17, ZMI_RING_SPLITK=4)
    rng = np.random.default_rng(100 + dst_dt)
    M, K, N = 150, 320, 290
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.02], dtype=np.float32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    bufs = {"src_scale": ss, "wei_scale": ws}
    if dst_dt != capi.DT_F32:
        ds = np.array([7.5], dtype=np.float32)
        dz = np.array([3], dtype=np.int32)
        p.dst_scale = lowoha.QuantParam(ds.ctypes.data, capi.DT_F32, (1,))
        p.dst_zp = lowoha.QuantParam(dz.ctypes.data, capi.DT_S32, (1,))
        bufs.update(dst_scale=ds, dst_zp=dz)
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs=bufs)
    assert "ksliced" in lowoha.last_kernel()
    assert np.array_equal(got, want)


def test_k_slices_chosen_for_a_problem_with_few_tiles(zo):
    """M = 192, N = 2048, K = 4096 (16 tiles): the launch plan slices K without being told to,
    and the dynamic-quantization call agrees with the oracle."""
    from tests.test_gpu_matmul import _oracle
    rng = np.random.default_rng(5)
    M, K, N = 192, 4096, 2048
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    x_d, w_d, ws_d = H.to_dev(x), H.to_dev(w), H.to_dev(ws)
    blob = H.prepack(w_d, K, N)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, blob, N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert "ksliced" in lowoha.last_kernel()
    sel = np.sort(rng.choice(M, 24, replace=False))
    ph = H.host_params(p, src_scale=None, wei_scale=ws)
    ph.mem_format_b = "n"
    ph.src_scale = lowoha.QuantParam(None, capi.DT_F32, (len(sel), 1))
    want, _, _ = _oracle(zo, ph, np.ascontiguousarray(x[sel]), w, len(sel), N, K)
    H.check_bf16(H.to_host(dst)[sel], want)


def test_remainder_tiles_beside_the_256_row_tiles_keep_stream_order(zo, monkeypatch):
    """With 256-row tiles the remainder rows' tiles are a launch of their own on the library's side stream, between a
    fork and a join on the caller's stream.  Calls that reuse one destination back to back, with a torch kernel
    on the same stream in between, must see each other's results in stream order."""
    monkeypatch.setenv("ZMI_GEMM_TOP", "256")
    rng = np.random.default_rng(21)
    K, N = 320, 300
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    w_d, ws_d = H.to_dev(w), H.to_dev(ws)
    ss = np.array([0.02], dtype=np.float32)
    Ms = (300, 257, 600, 449)     # remainders of 44, 1, 88 and 193 rows (64-, 64-, 128- and 256-row tiles)
    dst = torch.zeros((max(Ms), N), dtype=torch.float32, device=H.DEV)
    for rep in range(3):
        for M in Ms:
            a = rng.integers(-128, 128, (M, K), dtype=np.int8)
            p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
            p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
            p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
            dst.fill_(7.0)                    # (a torch kernel on the same stream between the calls)
            st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, w_d, N, None, 0.0, dst, N, True, p)
            assert st == capi.SUCCESS, lowoha.last_error()
            assert lowoha.last_kernel() == "ring_mfma32x32x32_top256"
            got = dst[:M].clone()             # (reads the destination on the same stream, right behind the call)
            ph = H.host_params(p, src_scale=ss, wei_scale=ws)
            keep = []
            st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K)
            assert st == capi.SUCCESS
            assert np.array_equal(H.to_host(got), want), (rep, M)
            assert torch.all(dst[M:] == 7.0)
    capi.load().zmi_clear_weight_cache()
