"""GPU tests of the weight-traffic-bound grouped kernel (k_stream.hip) through group_matmul_direct and the
device-routed fused block: against the oracle, and bit for bit against the MFMA-bound kernel on the same
call (both finish an element with the same arithmetic, so which kernel takes an expert must not show).

The kernel takes a grouped launch by itself only when the launch has at least two tiles per compute unit;
the small shapes here force it through ZMI_GROUP_STREAM_TOP (tile height | 0x10000) and switch it off
through ZMI_NO_GROUP_STREAM."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests import moe_helpers as MH

pytestmark = pytest.mark.gpu

TOP128, TOP256 = str(128 | 0x10000), str(256 | 0x10000)


def _with_kernel(monkeypatch, top, slices=None):
    monkeypatch.delenv("ZMI_NO_GROUP_STREAM", raising=False)
    monkeypatch.delenv("ZMI_GROUP_STREAM_TOP", raising=False)
    monkeypatch.delenv("ZMI_GROUP_STREAM_SLICES", raising=False)
    if top is None:
        monkeypatch.setenv("ZMI_NO_GROUP_STREAM", "1")
    else:
        monkeypatch.setenv("ZMI_GROUP_STREAM_TOP", top)
        if slices:
            monkeypatch.setenv("ZMI_GROUP_STREAM_SLICES", str(slices))


def _grouped(Ms, K, N, dst_dt, post=None, bias=False, gated=None, rng=None, static_u8=False):
    """A grouped call on fresh seeded inputs; returns a closure that runs it into new destinations."""
    E = len(Ms)
    if static_u8:
        xs = [rng.integers(0, 256, (max(m, 1), K), dtype=np.uint8) for m in Ms]
    else:
        xs = [H.gen_bf16_normal(rng, (max(m, 1), K)) for m in Ms]
    ws = [H.gen_weights(rng, K, N) for _ in Ms]
    wsc = [rng.uniform(0.001, 0.01, N).astype(np.float32) for _ in Ms]
    bs = [rng.standard_normal(N).astype(np.float32) if bias else None for _ in Ms]
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([128], dtype=np.int32)
    xs_d, ws_d, wsc_d = [H.to_dev(x) for x in xs], [H.to_dev(w) for w in ws], [H.to_dev(s) for s in wsc]
    bs_d = [H.to_dev(b) for b in bs]
    ss_d, zp_d = H.to_dev(ss), H.to_dev(zp)
    tdt = {capi.DT_BF16: torch.bfloat16, capi.DT_F32: torch.float32}[dst_dt]
    params = []
    for e, m in enumerate(Ms):
        if static_u8:
            p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=dst_dt, bias=capi.DT_F32 if bias else capi.DT_NONE)
            p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (1,))
            p.src_zp = lowoha.QuantParam(zp_d, capi.DT_S32, (1,))
        else:
            p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_S8,
                                    bias=capi.DT_F32 if bias else capi.DT_NONE)
            p.dynamic_quant = True
            p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (m, 1))
        p.wei_scale = lowoha.QuantParam(wsc_d[e], capi.DT_F32, (1, N))
        if post is not None:
            p.postop_ = [lowoha.PostOp(post)]
        params.append(p)

    def run():
        dst = [torch.full((max(m, 1), N), 7.0, dtype=tdt, device=H.DEV) for m in Ms]
        st = lowoha.group_matmul_direct(["r"] * E, [False] * E, [False] * E, Ms, [N] * E, [K] * E, [1.0] * E,
                                        [x if m else None for x, m in zip(xs_d, Ms)], [K] * E, ws_d, [N] * E, bs_d,
                                        [0.0] * E, dst, [N] * E, [True] * E, params, gated_act=gated)
        assert st == capi.SUCCESS, lowoha.last_error()
        return [H.to_host(d) for d in dst], lowoha.last_kernel()

    host = dict(xs=xs, ws=ws, wsc=wsc, bs=bs, ss=ss, zp=zp, params=params)
    return run, host


@pytest.mark.parametrize("top", [TOP128, TOP256])
@pytest.mark.parametrize("Ms", [[100, 0, 128, 17, 33], [130, 250, 5, 129], [300, 64, 513]])
@pytest.mark.parametrize("dst_dt,post", [(capi.DT_BF16, None), (capi.DT_BF16, capi.PO_SWISH), (capi.DT_BF16, capi.PO_GELU_TANH),
                                         (capi.DT_BF16, capi.PO_RELU), (capi.DT_F32, None), (capi.DT_F32, capi.PO_SWISH)])
def test_plain_grouped_gemms_match_the_mfma_bound_kernel_bit_for_bit(zo, monkeypatch, top, Ms, dst_dt, post):
    """Row counts on both sides of the tile heights (row fragments without rows, several row blocks, experts
    without rows, experts of at most 16 rows), N with a column edge inside a tile, bias; bf16 stores from registers
    and the rolled-loop epilogue (f32)."""
    rng = np.random.default_rng(len(Ms) * 1000 + sum(Ms) + (post or 0))
    K, N = 320, 600                  # 600 = 2 * 256 + 88: the third tile has a column edge
    run, host = _grouped(Ms, K, N, dst_dt, post=post, bias=True, rng=rng)
    _with_kernel(monkeypatch, None)
    ref, name_ref = run()
    assert "ring" in name_ref
    _with_kernel(monkeypatch, top)
    got, name = run()
    assert "stream" in name
    for e, m in enumerate(Ms):
        assert np.array_equal(got[e], ref[e]), f"expert {e} ({m} rows)"   # (rows beyond m keep the fill value on both)
    # and against the oracle, one expert
    e = 0
    keep = []
    ph = H.host_params(host["params"][e], src_scale=None, wei_scale=host["wsc"][e])
    st, want, _, _ = zo.matmul_int8(host["xs"][e][:Ms[e]], host["ws"][e], ph.flat(keep), Ms[e], N, K, bias=host["bs"][e])
    assert st == capi.SUCCESS
    if dst_dt == capi.DT_F32:
        H.check_f32(got[e][:Ms[e]], want)
    else:
        H.check_bf16(got[e][:Ms[e]], want, max_frac=5e-3, atol=1e-6 if post == capi.PO_GELU_TANH else 0.0)


@pytest.mark.parametrize("Ms", [[100, 0, 128, 70], [130, 40, 129], [20, 64, 33, 17, 50]])
@pytest.mark.parametrize("dst_dt,post", [(capi.DT_BF16, None), (capi.DT_BF16, capi.PO_GELU_TANH), (capi.DT_F32, None)])
def test_mfma_bound_kernel_in_k_slices_is_bit_identical(zo, monkeypatch, Ms, dst_dt, post):
    """A grouped launch of the MFMA-bound kernel with few tiles and a long K goes out in K slices: the slice that
    arrives last at its tile's word adds the others' int32 partial tiles and finishes the elements.  Bit-identical
    to the unsliced launch (ZMI_NO_GROUP_RING_SLICES) on repeated calls -- the arrival words are zero again after
    every launch -- and equal to the oracle.  Row counts: partly filled tiles, two row blocks per expert, experts
    without rows, 64-row tiles (the last list)."""
    rng = np.random.default_rng(sum(Ms) + (post or 0) + dst_dt)
    K, N = 3200, 600                 # 50 stages of 64 k: two slices of 25; a column edge inside the third tile
    run, host = _grouped(Ms, K, N, dst_dt, post=post, bias=True, rng=rng)
    _with_kernel(monkeypatch, None)
    monkeypatch.setenv("ZMI_NO_GROUP_RING_SLICES", "1")
    ref, name_ref = run()
    assert name_ref == "group: ring_mfma32x32x32"
    monkeypatch.delenv("ZMI_NO_GROUP_RING_SLICES")
    for rep in range(3):
        got, name = run()
        assert name == "group: ring_mfma32x32x32 (K slices)"
        for e, m in enumerate(Ms):
            assert np.array_equal(got[e], ref[e]), f"call {rep}, expert {e} ({m} rows)"
    e = 0
    keep = []
    ph = H.host_params(host["params"][e], src_scale=None, wei_scale=host["wsc"][e])
    st, want, _, _ = zo.matmul_int8(host["xs"][e][:Ms[e]], host["ws"][e], ph.flat(keep), Ms[e], N, K, bias=host["bs"][e])
    assert st == capi.SUCCESS
    if dst_dt == capi.DT_F32:
        H.check_f32(got[e][:Ms[e]], want)
    else:
        H.check_bf16(got[e][:Ms[e]], want, max_frac=5e-3, atol=1e-6 if post == capi.PO_GELU_TANH else 0.0)


@pytest.mark.parametrize("top", [TOP128, TOP256])
def test_static_u8_rows_with_zero_point(zo, monkeypatch, top):
    """u8 rows with a source zero-point: the compensation term travels through the parked column constants."""
    rng = np.random.default_rng(8)
    Ms, K, N = [70, 140], 256, 512
    run, host = _grouped(Ms, K, N, capi.DT_F32, bias=True, rng=rng, static_u8=True)
    _with_kernel(monkeypatch, None)
    ref, _ = run()
    _with_kernel(monkeypatch, top)
    got, name = run()
    assert "stream" in name
    keep = []
    for e, m in enumerate(Ms):
        assert np.array_equal(got[e], ref[e])
        ph = H.host_params(host["params"][e], src_scale=host["ss"], src_zp=host["zp"], wei_scale=host["wsc"][e])
        st, want, _, _ = zo.matmul_int8(host["xs"][e][:m], host["ws"][e], ph.flat(keep), m, N, K, bias=host["bs"][e])
        assert st == capi.SUCCESS
        assert np.array_equal(got[e][:m], want)


@pytest.mark.parametrize("top", [TOP128, TOP256])
@pytest.mark.parametrize("T,Hd,I,E,topk,skew", [(96, 512, 320, 8, 2, False),     # I = 320: gated tiles with a column edge
                                                (300, 256, 128, 4, 2, False),    # ~150 rows per expert
                                                (600, 256, 384, 3, 2, True)])    # several row blocks
def test_fused_block_matches_the_mfma_bound_kernel_and_the_oracle(zo, monkeypatch, top, T, Hd, I, E, topk, skew):
    c = MH.make_case(0x5EED0D00 + T, T, Hd, I, E, topk, skew)
    outs = {}
    for which in (None, top):
        _with_kernel(monkeypatch, which)
        d = MH.DeviceMoe(c)
        st = d.call_fused()
        assert st == capi.SUCCESS, lowoha.last_error()
        ids_d = H.to_dev(c.ids)
        w13b = [H.prepack(w, c.H, 2 * c.I) for w in d.w13]
        w2b = [H.prepack(w, c.I, c.H) for w in d.w2]
        out2 = torch.zeros((c.T, c.H), dtype=torch.bfloat16, device=H.DEV)
        st = lowoha.moe_fused_device(d.x, ids_d, d.topk_w, w13b, w2b, d.s13, d.s2, c.I, capi.ACT_SILU_AND_MUL, out2)
        assert st == capi.SUCCESS, lowoha.last_error()
        outs[which] = (H.to_host(d.out), H.to_host(out2), [H.to_host(t) if t is not None else None for t in d.dst_down])
    a, b = outs[None], outs[top]
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert (x is None and y is None) or np.array_equal(x, y)
    assert np.array_equal(b[0], b[1])                       # caller-scattered and device-routed forms agree
    want = MH.oracle_moe(zo, c, list(range(T)))
    MH.check_moe_out(b[0], want, flipped_rows=max(1, T // 50))


def test_gelu_gate_takes_the_rolled_epilogue(zo, monkeypatch):
    """gelu_and_mul has no straight-line form in the kernel: every tile goes through the rolled loop."""
    c = MH.make_case(0x5EED0E00, 80, 256, 128, 4, 2)
    outs = {}
    for which in (None, TOP128):
        _with_kernel(monkeypatch, which)
        d = MH.DeviceMoe(c)
        st = d.call_fused(act=capi.ACT_GELU_AND_MUL)
        assert st == capi.SUCCESS, lowoha.last_error()
        outs[which] = H.to_host(d.out)
    assert np.array_equal(outs[None], outs[TOP128])


def test_the_kernel_takes_a_large_enough_launch_by_itself(monkeypatch):
    """8 experts of ~100 rows, K = 512 -> 2 * 4096 gated: 8 * 32 = 256 ... below two tiles per compute unit the
    MFMA-bound kernel keeps the launch; with 2 * 8192 gated columns (512 tiles) the streaming kernel takes it."""
    monkeypatch.delenv("ZMI_NO_GROUP_STREAM", raising=False)
    monkeypatch.delenv("ZMI_GROUP_STREAM_TOP", raising=False)
    rng = np.random.default_rng(3)
    names = {}
    for I in (4096, 8192):
        run, _ = _grouped([100] * 8, 512, 2 * I, capi.DT_BF16, rng=rng, gated=capi.ACT_SILU_AND_MUL)
        _, names[I] = run()
    assert "ring" in names[4096] and "stream" in names[8192]


@pytest.mark.parametrize("top", [TOP128, TOP256])    # (the 256-row build ignores the request and runs unsliced)
@pytest.mark.parametrize("slices", [2, 3, 4])
@pytest.mark.parametrize("dst_dt,post", [(capi.DT_BF16, capi.PO_SWISH), (capi.DT_F32, None)])
def test_k_slices_leave_every_bit_where_it_was(zo, monkeypatch, top, slices, dst_dt, post):
    """Plain grouped launches cut into K slices (int32 partial tiles in a workspace, a second kernel adds them and
    finishes the elements): bit-identical to the unsliced MFMA-bound kernel; K_pad / 64 = 12 stages, so 3 and 4 slices
    divide evenly and unevenly, and the row counts leave row fragments and whole row blocks without rows."""
    rng = np.random.default_rng(slices * 10 + (post or 0))
    Ms, K, N = [100, 0, 129, 40, 300], 704, 600
    run, _ = _grouped(Ms, K, N, dst_dt, post=post, bias=True, rng=rng)
    _with_kernel(monkeypatch, None)
    ref, _ = run()
    _with_kernel(monkeypatch, top, slices)
    got, name = run()
    assert "stream" in name
    for e, m in enumerate(Ms):
        assert np.array_equal(got[e], ref[e]), f"expert {e} ({m} rows)"


def test_fused_block_with_a_sliced_down_projection(zo, monkeypatch):
    """The device-routed block whose down projection has few tiles and a long K takes K slices by itself
    (8 experts x ~32 rows, 2048 -> 512: 16 tiles of 128 rows on a device that holds hundreds of workgroups)."""
    c = MH.make_case(0x5EED0F00, 128, 512, 2048, 8, 2)
    outs = {}
    for which in (None, "auto"):
        monkeypatch.delenv("ZMI_GROUP_STREAM_TOP", raising=False)
        monkeypatch.delenv("ZMI_GROUP_STREAM_SLICES", raising=False)
        monkeypatch.delenv("ZMI_NO_GROUP_STREAM", raising=False)
        if which is None:
            monkeypatch.setenv("ZMI_NO_GROUP_STREAM", "1")
        d = MH.DeviceMoe(c)
        w13b = [H.prepack(w, c.H, 2 * c.I) for w in d.w13]
        w2b = [H.prepack(w, c.I, c.H) for w in d.w2]
        out2 = torch.zeros((c.T, c.H), dtype=torch.bfloat16, device=H.DEV)
        st = lowoha.moe_fused_device(d.x, H.to_dev(c.ids), d.topk_w, w13b, w2b, d.s13, d.s2, c.I, capi.ACT_SILU_AND_MUL, out2)
        assert st == capi.SUCCESS, lowoha.last_error()
        outs[which] = H.to_host(out2)
    assert np.array_equal(outs[None], outs["auto"])
    want = MH.oracle_moe(zo, c, list(range(c.T)))
    MH.check_moe_out(outs["auto"], want, flipped_rows=2)
