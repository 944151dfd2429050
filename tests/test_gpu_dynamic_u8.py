"""GPU parity of matmul_direct with dynamic_quant and a u8 compute type: the bf16 / f32 source is quantized
asymmetrically per tensor (one scale, one s32 zero-point; lowoha_operators/reorder/lowoha_reorder_utils.cpp:708-813,
reached through matmul/quantization/reorder_quantization.cpp:43-280), then the u8 x s8 GEMM with the zero-point
compensation and the dequantization chain follow.  Scale, zero-point and (through an s32 destination) the
accumulator are compared bit for bit with the oracle; bf16 activations by the usual one-ulp rule."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _run(zo, M, K, N, *, src_dt=capi.DT_BF16, dst_dt=capi.DT_BF16, scale_dt=capi.DT_F32, user_bufs=True, postop=None,
         bias=False, x=None, lda=None, seed=0):
    rng = np.random.default_rng(seed + M * 5 + K + N)
    if x is None:
        x = (rng.standard_normal((M, K)) * 3 + 0.7).astype(np.float32)
    lda = lda or K
    xs = np.zeros((M, lda), dtype=np.float32)
    xs[:, :K] = x
    xh = H.bf16_bits(xs) if src_dt == capi.DT_BF16 else xs
    w = H.gen_weights(rng, K, N)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    sc_d = torch.zeros(1, dtype=torch.float32 if scale_dt == capi.DT_F32 else torch.bfloat16, device=H.DEV) if user_bufs else None
    zp_d = torch.zeros(1, dtype=torch.int32, device=H.DEV) if user_bufs else None
    p = lowoha.MatmulParams(src=src_dt, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_U8,
                            bias=capi.DT_F32 if bias else capi.DT_NONE)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(sc_d, scale_dt, (1, 1))
    p.src_zp = lowoha.QuantParam(zp_d, capi.DT_S32, (1, 1))
    if dst_dt != capi.DT_S32:
        p.wei_scale = lowoha.QuantParam(H.to_dev(ws), capi.DT_F32, (1, N))
    if postop is not None:
        p.postop_ = [lowoha.PostOp(postop)]
    tdt = {capi.DT_BF16: torch.bfloat16, capi.DT_F32: torch.float32, capi.DT_S32: torch.int32}[dst_dt]
    dst = torch.zeros((M, N), dtype=tdt, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, K, 1.0, H.to_dev(xh), lda, H.to_dev(w), N, H.to_dev(b), 0.0, dst, N,
                              True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    ph = H.host_params(p, src_scale=None, src_zp=None, **({"wei_scale": ws} if dst_dt != capi.DT_S32 else {}))
    keep = []
    zp_want = np.zeros(1, dtype=np.int32)
    st, want, _, scales = zo.matmul_int8(xh, w, ph.flat(keep), M, N, K, bias=b, lda=lda, want_scales=True, zp_out=zp_want)
    assert st == capi.SUCCESS
    if user_bufs:
        got_s = H.to_host(sc_d)
        got_s = zo.bf16_to_f32(got_s) if scale_dt == capi.DT_BF16 else got_s
        assert got_s[0] == scales[0]
        assert H.to_host(zp_d)[0] == zp_want[0]
    got = H.to_host(dst)
    if dst_dt == capi.DT_S32 or (postop is None and dst_dt == capi.DT_F32):
        assert np.array_equal(got, want)
    elif dst_dt == capi.DT_F32:
        H.check_f32(got, want)
    else:
        H.check_bf16(got, want, max_frac=1e-2)
    return zp_want[0]


@pytest.mark.parametrize("M,K,N", [(1, 512, 96), (16, 4096, 320), (40, 1000, 70), (130, 2048, 256), (300, 512, 512)])
@pytest.mark.parametrize("src_dt", [capi.DT_BF16, capi.DT_F32])
def test_accumulator_scale_and_zero_point_bit_exact(zo, M, K, N, src_dt):
    # s32 destination without scales: the accumulator plus the zero-point compensation, which is exact
    zp = _run(zo, M, K, N, src_dt=src_dt, dst_dt=capi.DT_S32)
    assert 0 < zp < 255


@pytest.mark.parametrize("scale_dt", [capi.DT_F32, capi.DT_BF16])
@pytest.mark.parametrize("user_bufs", [True, False])
def test_dequantization_chain_and_where_the_parameters_live(zo, scale_dt, user_bufs):
    _run(zo, 16, 4096, 320, dst_dt=capi.DT_F32, scale_dt=scale_dt, user_bufs=user_bufs, bias=True)
    _run(zo, 70, 512, 100, dst_dt=capi.DT_BF16, scale_dt=scale_dt, user_bufs=user_bufs, postop=capi.PO_SWISH, bias=True)


def test_non_finite_elements_constant_tensors_and_padded_rows(zo):
    x = np.random.default_rng(3).standard_normal((8, 256)).astype(np.float32)
    x[0, 0], x[3, 7], x[5, 100] = np.nan, np.inf, -np.inf
    _run(zo, 8, 256, 64, dst_dt=capi.DT_S32, src_dt=capi.DT_F32, x=x)
    _run(zo, 4, 128, 32, dst_dt=capi.DT_S32, x=np.full((4, 128), 2.5, dtype=np.float32))     # max == min: range [2.5, 3.5]
    _run(zo, 4, 128, 32, dst_dt=capi.DT_S32, x=np.zeros((4, 128), dtype=np.float32))
    _run(zo, 9, 200, 48, dst_dt=capi.DT_F32, lda=211)


def test_rejections():
    M, K, N = 4, 64, 16
    x_d = H.to_dev(np.zeros((M, K), dtype=np.uint16))
    w_d = H.to_dev(np.zeros((K, N), dtype=np.int8))

    def call(sdims=(1, 1), zdims=(1, 1), zdt=capi.DT_S32):
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_U8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, sdims)
        p.src_zp = lowoha.QuantParam(None, zdt, zdims)
        dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
        return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, None, 0.0, dst, N, True, p)

    assert call() == capi.SUCCESS
    assert call(sdims=(M, 1)) == capi.UNIMPLEMENTED         # the GEMM reads one zero-point: per-tensor only
    assert call(zdims=(M, 1)) == capi.UNIMPLEMENTED
    assert call(zdims=()) == capi.UNIMPLEMENTED             # zero-point dims are required
    assert call(zdt=capi.DT_S8) == capi.FAILURE
