"""GPU parity of the large-M (fragment-major, MFMA-bound) kernel through matmul_direct:
tile-edge shapes for every tile height, the straight-line bf16 epilogues next to
their edge forms, unaligned destinations, u8 sources, and the destination dtypes
that go through its generic epilogue."""
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
