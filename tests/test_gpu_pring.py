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


def _dyn_call(x, blob, ws, b, M, K, N, sbuf, po=capi.PO_SWISH):
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(sbuf, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
    p.postop_ = [lowoha.PostOp(po)]
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, x.shape[1], blob, N, b, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    return H.to_host(dst), lowoha.last_kernel()


# bands that are partly filled, chunks of fewer than eight rows, K from one 16-value piece per row to the largest the
# launch takes, a source with a row stride, the default grid at BASELINE config 3's row count
@pytest.mark.parametrize("M,K,N,ldx,grid", [(1100, 512, 3584, 512, 64), (257, 4096, 1024, 4104, 8), (520, 8192, 512, 8192, 16),
                                            (300, 16, 640, 16, 8), (2048, 4096, 2048, 4096, 0), (1027, 1008, 1536, 1008, 24)])
def test_rows_quantized_inside_the_launch_match_the_separate_launch(env, M, K, N, ldx, grid):
    """Per-token quantization inside the persistent kernel's launch against the quantization launch followed by the
    same kernel: scales and outputs bit-identical, also on a repeated call (the flags then hold the numbers of earlier
    launches) and after a call of another shape; the scales against their closed form amax / 127."""
    env(ZMI_PRING=1, ZMI_RING_MIN_M=1, ZMI_NO_DECODE_KERNEL=1, ZMI_RING_SPLITK=1)
    if grid:
        env(ZMI_PRING_GRID=grid)
    rng = np.random.default_rng(M * 7 + K)
    xh = np.zeros((M, ldx), dtype=np.uint16)
    xh[:, :K] = H.gen_bf16_normal(rng, (M, K))
    xh[:, K:] = 0x7fc0                       # (a NaN pattern in the stride's gap: never read)
    if M > 40:
        xh[33, :K] = 0                        # an all-zero row: the floor of the scale
        xh[34, 3 % K] = 0x7f80                # an infinity: left out of the maximum, saturates
    x = H.to_dev(xh)
    w = H.to_dev(H.gen_weights(rng, K, N))
    blob = H.prepack(w, K, N)
    ws = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    b = H.to_dev((rng.standard_normal(N) * 0.1).astype(np.float32))
    res = []
    for no_fuse in (1, 0, 0):
        env(ZMI_NO_PRING_QUANT=1 if no_fuse else None)
        sbuf = torch.zeros(M, dtype=torch.float32, device=H.DEV)
        out, name = _dyn_call(x, blob, ws, b, M, K, N, sbuf)
        assert "pring" in name and (("quant in the launch" in name) == (not no_fuse)), name
        res.append((out, H.to_host(sbuf)))
        if no_fuse == 0 and len(res) == 2:
            # another shape in between: the words of the first chunks are reused with other launch numbers
            x2 = H.to_dev(H.gen_bf16_normal(rng, (264, 64)))
            w2 = H.to_dev(H.gen_weights(rng, 64, 512))
            _dyn_call(x2, H.prepack(w2, 64, 512), ws[:512].contiguous(), b[:512].contiguous(), 264, 64, 512, None)
    for out, sc in res[1:]:
        assert np.array_equal(sc.view(np.uint32), res[0][1].view(np.uint32))
        assert np.array_equal(out, res[0][0])
    vals = (xh[:, :K].astype(np.uint32) << 16).view(np.float32)
    amax = np.max(np.where(np.isfinite(vals), np.abs(vals), np.float32(0)), axis=1).astype(np.float32)
    want = np.maximum(np.maximum(amax, np.float32(1e-10)) / np.float32(127.0), np.float32(1e-10)).astype(np.float32)
    assert np.array_equal(res[1][1].view(np.uint32), want.view(np.uint32))


def test_scale_buffer_that_shares_cache_lines_between_bands_takes_the_separate_launch(env):
    env(ZMI_PRING=1, ZMI_PRING_GRID=8, ZMI_RING_MIN_M=1, ZMI_RING_SPLITK=1)
    rng = np.random.default_rng(11)
    M, K, N = 520, 256, 512
    x = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
    blob = H.prepack(H.to_dev(H.gen_weights(rng, K, N)), K, N)
    ws = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    b = H.to_dev(np.zeros(N, dtype=np.float32))
    whole = torch.zeros(M + 8, dtype=torch.float32, device=H.DEV)
    out_a, name_a = _dyn_call(x, blob, ws, b, M, K, N, whole[1:M + 1])
    out_b, name_b = _dyn_call(x, blob, ws, b, M, K, N, whole[:M])
    assert "quant in the launch" not in name_a and "quant in the launch" in name_b
    assert np.array_equal(out_a, out_b)
