"""GPU parity of the persistent form of the large-M kernel (k_pring.hip) through matmul_direct: every tile width
(256 x 64 .. 256 x 256 outputs), several tiles per workgroup, partly filled bands, column edges, the straight-line
epilogues, static and dynamically quantized sources.  ZMI_PRING=1 sends shapes below the size rule to it and
ZMI_PRING_GRID shrinks its grid so that small shapes give a workgroup several tiles."""
import os

import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.test_gpu_reorder_edges import _run_both

pytestmark = pytest.mark.gpu


@pytest.fixture
def env():
    saved = {}

    def set_(**kv):
        for k, v in kv.items():
            saved.setdefault(k, os.environ.get(k))
            if v is None:
                os.environ.pop(k, None)      # (the switches are on when the variable exists, whatever it holds)
            else:
                os.environ[k] = str(v)

    yield set_
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


# N / 64 units per band split over 8 XCDs: 3584 -> 7 per XCD (tiles of 4 + 3 units), 2560 -> 5 (3 + 2), 4608 -> 9
# (3 + 3 + 3), 1408 -> 2 or 3, 516 -> one unit on most XCDs and a column edge; grid 8: one workgroup per XCD walks
# all its bands; grid 16 / 24: runs that start and end inside a band
@pytest.mark.parametrize("M,K,N,grid", [(600, 192, 3584, 8), (257, 128, 2560, 8), (512, 64, 4608, 16), (300, 320, 1408, 8),
                                        (700, 96, 516, 24), (1024, 256, 3584, 32), (256, 4096, 512, 8)])
@pytest.mark.parametrize("po", [None, capi.PO_GELU_TANH])
def test_static_rows_every_tile_width(zo, env, M, K, N, grid, po):
    env(ZMI_PRING=1, ZMI_PRING_GRID=grid, ZMI_RING_MIN_M=1, ZMI_NO_DECODE_KERNEL=1, ZMI_RING_SPLITK=1)
    rng = np.random.default_rng(M + K + N + grid)
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
    got, want = _run_both(zo, p, a, w, M, N, K, bias=bias, host_bufs={"src_scale": ss, "wei_scale": ws},
                          ldc=(N + 7) // 8 * 8 + 8)        # (rows of the destination 16-byte aligned)
    assert "pring" in lowoha.last_kernel(), lowoha.last_kernel()
    if po is None:
        assert np.array_equal(got[:, :N], want[:, :N])        # the separately rounded scale chain: bit-identical
    else:
        H.check_bf16(got[:, :N], want[:, :N], atol=1e-6, max_frac=5e-3)
    assert np.all(got[:, N:] == 0)


@pytest.mark.parametrize("po", [capi.PO_SWISH, capi.PO_RELU])
def test_u8_source_with_zero_point_and_other_activations(zo, env, po):
    env(ZMI_PRING=1, ZMI_PRING_GRID=8)
    rng = np.random.default_rng(po)
    M, K, N = 384, 160, 1024
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    w = H.gen_weights(rng, K, N)
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([117], dtype=np.int32)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_BF16)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(po)]
    p.weight_cache_type = 0
    got, want = _run_both(zo, p, a, w, M, N, K, host_bufs={"src_scale": ss, "src_zp": zp, "wei_scale": ws})
    assert "pring" in lowoha.last_kernel(), lowoha.last_kernel()
    H.check_bf16(got, want, max_frac=5e-3)


def test_dynamic_quant_rows_match_the_tiled_kernel_bit_for_bit(env):
    """The same call through the persistent form and through the tiled kernel: the same integers go through the same
    element arithmetic, so the bf16 outputs are identical (full-size check of BASELINE config 3's shape is in
    test_gpu_matmul.py)."""
    rng = np.random.default_rng(3)
    M, K, N = 1100, 512, 3584
    x = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
    w = H.to_dev(H.gen_weights(rng, K, N))
    blob = H.prepack(w, K, N)
    ws = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    b = H.to_dev((rng.standard_normal(N) * 0.1).astype(np.float32))
    outs = []
    for pring in (1, 0):
        env(ZMI_PRING=pring, ZMI_PRING_GRID=64)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
        p.postop_ = [lowoha.PostOp(capi.PO_GELU_TANH)]
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, K, blob, N, b, 0.0, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        assert ("pring" in lowoha.last_kernel()) == bool(pring), lowoha.last_kernel()
        outs.append(H.to_host(dst))
    assert np.array_equal(outs[0], outs[1])

