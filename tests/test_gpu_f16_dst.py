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


@pytest.mark.parametrize("act", [capi.ACT_SILU_AND_MUL, capi.ACT_SWIGLU_OAI_MUL])
def test_group_call_with_f16_destinations_gated_activation_and_weighted_reduce(zo, act):
    """group_matmul_direct with half-precision expert outputs: the GEMMs, the gated activation (float16_t(value),
    group_matmul_moe_act.cpp:165-182) and the weighted reduce over half-precision rows (store_from_f32,
    group_matmul_moe_postop.cpp:84-100).  Before, the activation and the reduce treated f16 as f32 words."""
    rng = np.random.default_rng(31 + act)
    E, T, K, I = 3, 10, 192, 40
    N = 2 * I
    Ms = [T, T, T]
    srcs = [rng.integers(-128, 128, (T, K), dtype=np.int8) for _ in range(E)]
    ws = [H.gen_weights(rng, K, N) for _ in range(E)]
    sscale = np.array([0.01], dtype=np.float32)
    wscale = [rng.uniform(0.001, 0.004, N).astype(np.float32) for _ in range(E)]
    src_d = [H.to_dev(s) for s in srcs]
    w_d = [H.to_dev(w) for w in ws]
    wsc_d = [H.to_dev(x) for x in wscale]
    dst = [torch.zeros((T, N), dtype=torch.int16, device=H.DEV) for _ in range(E)]
    params = []
    for e in range(E):
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F16)
        p.src_scale = lowoha.QuantParam(sscale.ctypes.data, capi.DT_F32, (1,))
        p.wei_scale = lowoha.QuantParam(wsc_d[e], capi.DT_F32, (1, N))
        params.append(p)
    ids = [(t % E, (t + 1) % E) for t in range(T)]
    rp = [dst[e].data_ptr() + t * N * 2 for t in range(T) for e in ids[t]]
    tw_h = rng.uniform(0.2, 0.8, (T, 2)).astype(np.float32)
    tw = H.to_dev(tw_h)
    out = torch.zeros((T, N), dtype=torch.int16, device=H.DEV)   # (without fused_moe the reduce takes whole rows)
    pp = lowoha.MoePostop(T, 2, out, N, tw, rp)
    st = lowoha.group_matmul_direct(
        ["r"] * E, [False] * E, [False] * E, Ms, [N] * E, [K] * E, [1.0] * E,
        src_d, [K] * E, w_d, [N] * E, [None] * E, [0.0] * E, dst, [N] * E, [True] * E, params,
        gated_act=act, moe_postop=pp)
    assert st == capi.SUCCESS, lowoha.last_error()
    got = [_f16_host(d) for d in dst]
    for e in range(E):
        ph = H.host_params(params[e], wei_scale=wscale[e])
        keep = []
        st, y, _, _ = zo.matmul_int8(srcs[e], ws[e], ph.flat(keep), T, N, K)
        assert st == capi.SUCCESS
        zo.gated_act(act, y, capi.DT_F16)
        d = np.abs(got[e][:, :I].view(np.int16).astype(np.int32) - y[:, :I].view(np.int16).astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() < 5e-3, (e, d.max())
    # the reduce over the device's own rows: bit-identical
    rows = [got[e][t].copy() for t in range(T) for e in ids[t]]
    want = zo.moe_reduce(rows, tw_h, capi.DT_F16, N)
    assert np.array_equal(_f16_host(out), want)
