"""Half-precision destinations (reference: aocl_gemm_s8s8s32of16 / u8s8s32of16, aocl_kernel.cpp:1224-1229, :1290-1294;
the store conversion is float16_t(float), common/float16.cpp:124-205): every kernel family against the oracle, bit
for bit, including accumulation into a half-precision destination (beta).  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _f16_dev(bits):
    return torch.from_numpy(bits.view(np.int16)).to(H.DEV)


def _f16_host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("M,K,N", [(8, 512, 300), (40, 1024, 200), (24, 4200, 100), (8, 4200, 64), (200, 512, 300), (300, 640, 515)])
@pytest.mark.parametrize("u8", [False, True])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_f16_destination_bit_identical_to_the_oracle(zo, M, K, N, u8, beta):
    rng = np.random.default_rng(M + K + N + int(u8) + int(beta * 10))
    a = rng.integers(0, 256, (M, K), dtype=np.uint8) if u8 else rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    # (scales that take results beyond 65504 at 8 rows and below the smallest normal half at 24 rows)
    ss = np.array([30.0 if M == 8 else 3e-7 if M == 24 else 0.02], dtype=np.float32)
    bias = (rng.standard_normal(N) * (1e-4 if M == 24 else 1.0)).astype(np.float32)
    azp = np.array([128], dtype=np.int32)
    dst0 = rng.standard_normal((M, N)).astype(np.float16).view(np.uint16)
    ws_d = H.to_dev(ws)
    p = lowoha.MatmulParams(src=capi.DT_U8 if u8 else capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F16, bias=capi.DT_F32)
    p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
    p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (1, N))
    if u8:
        p.src_zp = lowoha.QuantParam(azp.ctypes.data, capi.DT_S32, (1,))
    p.postop_ = [lowoha.PostOp(capi.PO_GELU_TANH)] if M == 40 else []
    dst = _f16_dev(dst0.copy())
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(a), K, H.to_dev(w), N, H.to_dev(bias), beta, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, wei_scale=ws)
    keep = []
    st, want, _, _ = zo.matmul_int8(a, w, ph.flat(keep), M, N, K, bias=bias, beta=beta, dst=dst0.copy())
    assert st == capi.SUCCESS
    got = _f16_host(dst)
    if p.postop_:
        # (the activation's last f32 bit differs between the device and libm: at most one half-precision step, rarely)
        d = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() < 2e-3, lowoha.last_kernel()
    else:
        assert np.array_equal(got, want), lowoha.last_kernel()
    f = np.abs(got.view(np.float16).astype(np.float32))
    if M == 8 and beta == 0.0:
        assert np.isinf(f).any()
    if M == 24 and beta == 0.0:
        assert ((f > 0) & (f < 6.0e-5)).any()
