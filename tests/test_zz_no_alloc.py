"""zmi_matmul_direct_noalloc (the entry point that allocates no device memory) against zmi_matmul_direct on the
same arguments, through the C ABI: bit-identical outputs and scales, on two calls in a row, the second with a
smaller input (the scratch array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _case(M, K, N, rng, dst_dt, po, per_tensor=False, scale_buf=False, scale_dt=capi.DT_F32):
    x = H.gen_bf16_normal(rng, (M, K))
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    keep = {"x": H.to_dev(x), "ws": H.to_dev(ws), "b": H.to_dev(b), "blob": H.prepack(H.to_dev(w), K, N)}
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_S8, bias=capi.DT_F32)
    p.dynamic_quant = True
    n_sc = 1 if per_tensor else M
    tdt = torch.float32 if scale_dt == capi.DT_F32 else torch.bfloat16
    outs = []
    for noalloc in (False, True):
        sbuf = torch.zeros(n_sc, dtype=tdt, device=H.DEV) if scale_buf else None
        p.src_scale = lowoha.QuantParam(sbuf, scale_dt, (1,) if per_tensor else (M, 1))
        p.wei_scale = lowoha.QuantParam(keep["ws"], capi.DT_F32, (1, N))
        p.postop_ = [lowoha.PostOp(po)] if po else []
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        dst = torch.zeros((M, N), dtype=torch.float32 if dst_dt == capi.DT_F32 else torch.bfloat16, device=H.DEV)
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, keep["x"], K, keep["blob"], N, keep["b"], 0.0, dst, N,
                                  True, p, noalloc=noalloc)
        assert st == capi.SUCCESS, lowoha.last_error()
        if noalloc:
            assert "static scratch" in lowoha.last_kernel()
        outs.append((H.to_host(dst), H.to_host(sbuf) if scale_buf else None))
    assert np.array_equal(outs[0][0], outs[1][0])
    if scale_buf:
        assert np.array_equal(outs[0][1], outs[1][1])


def test_noalloc_matches_matmul_direct_two_calls_in_a_row():
    rng = np.random.default_rng(2024)
    # the headline decode shape, then a smaller call that reuses the array's head
    _case(16, 4096, 14336, rng, capi.DT_BF16, capi.PO_SWISH)
    _case(5, 1000, 300, rng, capi.DT_F32, None, scale_buf=True)
    # more rows than one group, per-tensor scale, bf16 scale buffer, one row
    _case(128, 4096, 512, rng, capi.DT_BF16, capi.PO_GELU_TANH, scale_buf=True, scale_dt=capi.DT_BF16)
    _case(40, 520, 96, rng, capi.DT_F32, None, per_tensor=True, scale_buf=True)
    _case(1, 4096, 1024, rng, capi.DT_BF16, capi.PO_SWISH)
    # 13 .. 16 rows on the 16-row kernel with K that is no multiple of 16 (the rows' stride in the array is)
    _case(16, 1000, 300, rng, capi.DT_BF16, capi.PO_SWISH)
    _case(13, 4090, 200, rng, capi.DT_F32, None, scale_buf=True)


def test_noalloc_calls_leave_the_free_device_memory_unchanged():
    """The entry point's defining property: after a first call (which may load code objects), calls with new shapes
    under its limits change neither the free device memory nor the caching allocator's reservation -- every buffer of
    the calls below exists before the first measurement."""
    rng = np.random.default_rng(99)
    shapes = [(16, 4096, 2048), (3, 520, 96), (128, 4096, 512), (64, 1024, 300), (1, 256, 64)]
    cases = []
    for M, K, N in shapes:
        x = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
        blob = H.prepack(H.to_dev(H.gen_weights(rng, K, N)), K, N)
        ws = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
        dst = torch.zeros((M, N), dtype=torch.bfloat16, device=H.DEV)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        cases.append((M, K, N, x, blob, dst, p, ws))

    def call(c):
        M, K, N, x, blob, dst, p, _ = c
        st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, K, blob, N, None, 0.0, dst, N, True, p, noalloc=True)
        assert st == capi.SUCCESS, lowoha.last_error()

    for c in cases:        # first calls: code objects, the blob header checks
        call(c)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(3):
        for c in cases:
            call(c)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_reserved() == reserved0


def test_noalloc_rejects_what_the_array_cannot_hold():
    rng = np.random.default_rng(7)
    M, K, N = 129, 256, 64
    x = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
    w = H.to_dev(H.gen_weights(rng, K, N))
    ws = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    blob = H.prepack(w, K, N)
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
    p.mem_format_b = "r"
    p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, K, blob, N, None, 0.0, dst, N, True, p, noalloc=True)
    assert st == capi.FAILURE and "128 rows" in lowoha.last_error()
    p.mem_format_b = "n"
    p.lowoha_algo = capi.ALGO_NONE
    st = lowoha.matmul_direct("r", False, False, 16, N, K, 1.0, x, K, w, N, None, 0.0, dst, N, True, p, noalloc=True)
    assert st == capi.UNIMPLEMENTED
