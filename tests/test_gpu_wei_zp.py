"""A weight zero-point on matmul_direct (reference: the 2-D zero-point compensation, lowoha_operators/matmul/
lru_cache/lowoha_cache.hpp:151-232): every kernel family a single problem can reach, against the integer product of the
shifted operands (s32 destination) and against the oracle (f32 chain).  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu

# (M, K, N, substring of the kernel's name)
SHAPES = [
    (8, 512, 300, "decode16"), (1, 4096, 64, "decode16"), (40, 1024, 200, "decode_lds_rows"), (100, 520, 96, "decode_lds_rows"),
    (8, 4200, 100, "decode16_ksliced"), (24, 4200, 100, "smallm"), (200, 512, 300, "ksliced"), (300, 64, 515, "ksliced"),
    (130, 100, 70, "ksliced"), (1000, 256, 260, "ksliced"),
]


def _zp(value, dt, device):
    a = np.array([value], dtype=np.int8 if dt == capi.DT_S8 else np.int32)
    return a, (H.to_dev(a) if device else a.ctypes.data)


@pytest.mark.parametrize("M,K,N,kname", SHAPES)
@pytest.mark.parametrize("u8", [False, True])
def test_s32_destination_is_the_product_of_the_shifted_operands(M, K, N, kname, u8):
    rng = np.random.default_rng(M + K + N + int(u8))
    a = rng.integers(0, 256, (M, K), dtype=np.uint8) if u8 else rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    a_zp, w_zp = (131, -9) if u8 else (0, 6)
    want = (a.astype(np.int64) - a_zp) @ (w.astype(np.int64) - w_zp)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    azp = np.array([a_zp], dtype=np.int32)
    for w_dt, on_device in ((capi.DT_S8, False), (capi.DT_S32, True)):
        wz, wz_buf = _zp(w_zp, w_dt, on_device)
        p = lowoha.MatmulParams(src=capi.DT_U8 if u8 else capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
        p.wei_zp = lowoha.QuantParam(wz_buf, w_dt, (1,))
        if u8:
            p.src_zp = lowoha.QuantParam(azp.ctypes.data, capi.DT_S32, (1,))
        for rep in range(2):
            dst = torch.full((M, N), -7, dtype=torch.int32, device=H.DEV)
            st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, True, p)
            assert st == capi.SUCCESS, lowoha.last_error()
            assert kname in lowoha.last_kernel(), lowoha.last_kernel()
            assert np.array_equal(H.to_host(dst).astype(np.int64), want), (w_dt, rep, lowoha.last_kernel())


@pytest.mark.parametrize("M,K,N,kname", [(8, 512, 300, "decode16"), (40, 1024, 200, "decode_lds_rows"), (24, 4200, 100, "smallm"),
                                         (200, 512, 300, "ksliced")])
@pytest.mark.parametrize("u8,transA", [(False, False), (True, False), (False, True)])
def test_f32_chain_bit_identical_to_the_oracle(zo, M, K, N, kname, u8, transA):
    rng = np.random.default_rng(M + K + N + int(u8) + 2 * int(transA))
    a = rng.integers(0, 256, (M, K), dtype=np.uint8) if u8 else rng.integers(-128, 128, (M, K), dtype=np.int8)
    src = np.ascontiguousarray(a.T) if transA else a
    lda = M if transA else K
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    ss = np.array([0.02], dtype=np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    azp = np.array([120], dtype=np.int32)
    wzp = np.array([-5], dtype=np.int8)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_U8 if u8 else capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    p.wei_zp = lowoha.QuantParam(wzp.ctypes.data, capi.DT_S8, (1,))
    if u8:
        p.src_zp = lowoha.QuantParam(azp.ctypes.data, capi.DT_S32, (1,))
    p.postop_ = [lowoha.PostOp(capi.PO_RELU)]
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", transA, False, M, N, K, 1.0, H.to_dev(src), lda, H.to_dev(w), N, H.to_dev(bias), 0.0, dst, N,
                              True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert kname in lowoha.last_kernel(), lowoha.last_kernel()
    ph = H.host_params(p, wei_scale=ws)
    keep = []
    st, want, _, _ = zo.matmul_int8(src, w, ph.flat(keep), M, N, K, bias=bias, transA=transA, lda=lda)
    assert st == capi.SUCCESS
    assert np.array_equal(H.to_host(dst), want)


def test_zero_valued_weight_zero_point_changes_nothing_and_unsupported_forms_say_so(zo):
    rng = np.random.default_rng(2)
    M, K, N = 8, 256, 96
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    a_d, w_d = H.to_dev(a), H.to_dev(w)
    zero = np.array([0], dtype=np.int8)
    p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32)
    p.wei_zp = lowoha.QuantParam(zero.ctypes.data, capi.DT_S8, (1,))
    dst = torch.zeros((M, N), dtype=torch.int32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, a_d, K, w_d, N, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert np.array_equal(H.to_host(dst).astype(np.int64), a.astype(np.int64) @ w.astype(np.int64))
    # bf16 rows quantized by the call: the weight zero-point is not taken there
    five = np.array([5], dtype=np.int8)
    x = H.to_dev(H.gen_bf16_normal(rng, (M, K)))
    ws_d = H.to_dev(rng.uniform(0.001, 0.01, N).astype(np.float32))
    pd = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
    pd.dynamic_quant = True
    pd.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
    pd.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    pd.wei_zp = lowoha.QuantParam(five.ctypes.data, capi.DT_S8, (1,))
    d2 = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x, K, w_d, N, None, 0.0, d2, N, True, pd)
    assert st == capi.UNIMPLEMENTED and "zero-point" in lowoha.last_error()
