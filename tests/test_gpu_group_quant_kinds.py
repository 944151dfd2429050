"""GPU parity of gated_act and fused_moe on the experts the grouped kernels do not take: per-group
scales, GGML Q8_0 packed weights and W4A8 (s4 weights).

Reference: the two-pass composition (run_fused_moe_legacy_two_pass,
zendnnl/src/lowoha_operators/matmul/group_matmul/group_matmul_fused_moe.cpp:906-1078) with Op2's
parameters derived by setup_op2_dispatch_scratch (same file :761-880): Op2 keeps Op1's
dynamic_quant / compute / weight dtypes and scale dtype; with per-group source scales its group count
comes from the down projection's weight scale {G2, N_down}; a GGML expert has both projections
packed.  Its own tests of these kinds: gtests/group_matmul/test_quant.cpp:363-1121 (gated activation
on per-group experts at :470-560).

Expected values: the oracle's single products composed on the host in that order.  Bars: the stage
results that involve no exp (Op1 alone; Op2 on the oracle's intermediate is covered for the plain
kind elsewhere) are identical; after the activation one bf16 ulp; after the re-quantizing Op2 the
propagated two-ulp bound of the plain fused block."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests.moe_helpers import check_moe_out

pytestmark = pytest.mark.gpu


def _q8_0(rng, N, K):
    """[N][K/32] blocks of {fp16 d, int8 qs[32]} as a flat byte array."""
    G = K // 32
    rows = rng.integers(-127, 128, (N, K), dtype=np.int8)
    d16 = rng.uniform(1e-3, 0.02, (N, G)).astype(np.float16)
    blk = np.zeros((N, G, 34), dtype=np.uint8)
    blk[:, :, :2] = d16.view(np.uint16).reshape(N, G, 1).view(np.uint8)
    blk[:, :, 2:] = rows.reshape(N, G, 32).view(np.uint8)
    return blk.reshape(-1)


class Kind:
    """One quantization kind: builds an expert's weights / scales and the params of either projection."""

    def __init__(self, name):
        self.name = name

    def weights(self, rng, K, N, gs):
        G = K // gs
        if self.name == "ggml":
            return _q8_0(rng, N, K), None
        if self.name == "w4a8":
            return rng.integers(0, 256, K * N // 2, dtype=np.uint8), rng.uniform(0.01, 0.05, (G, N)).astype(np.float32)
        return rng.integers(-127, 128, (K, N), dtype=np.int8), rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)

    def params(self, M, K, N, gs, ws_buf, per_group_src=True):
        G = K // gs
        wei = capi.DT_S4 if self.name == "w4a8" else capi.DT_S8
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=wei, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, G) if per_group_src else (M, 1))
        if self.name == "ggml":
            p.pack_format_b = 1
        else:
            p.wei_scale = lowoha.QuantParam(ws_buf, capi.DT_F32, (G, N))
        return p

    @property
    def transB(self):
        return self.name == "ggml"

    def ldb(self, K, N):
        return K if self.name == "ggml" else N


def _oracle_product(zo, kind, x, w, ws, M, K, N, gs, per_group_src=True):
    keep = []
    p = kind.params(M, K, N, gs, None, per_group_src)
    if ws is not None:
        p.wei_scale = lowoha.QuantParam(ws.ctypes.data, capi.DT_F32, p.wei_scale.dims)
    st, y, _, _ = zo.matmul_int8(x, w, p.flat(keep), M, N, K, transB=kind.transB, ldb=kind.ldb(K, N))
    assert st == capi.SUCCESS
    return y


@pytest.mark.parametrize("kind,per_group_src", [("pergroup", True), ("ggml", True), ("w4a8", True), ("w4a8", False)])
@pytest.mark.parametrize("act", [capi.ACT_SILU_AND_MUL, capi.ACT_GELU_AND_MUL])
def test_fused_moe_on_per_group_ggml_and_s4_experts(zo, kind, per_group_src, act):
    kind = Kind(kind)
    rng = np.random.default_rng(sum(map(ord, kind.name)) * 8 + int(per_group_src) * 4 + int(act))
    T, Hd, I, E, topk = 24, 256, 128, 4, 2
    gs1, gs2 = 32, 32                       # group sizes of Op1 (over Hd) and Op2 (over I)
    x = H.bf16_bits(rng.standard_normal((T, Hd)).astype(np.float32))
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32)
    ids[:, :] = np.where(ids == 3, 0, ids)  # expert 3 gets no rows; expert 0 may be picked twice by a token
    tw = rng.uniform(0.2, 0.8, (T, topk)).astype(np.float32)
    rows_of = [[] for _ in range(E)]
    slot = {}
    for t in range(T):
        for k in range(topk):
            e = int(ids[t, k])
            slot[(t, k)] = (e, len(rows_of[e]))
            rows_of[e].append(t)
    Ms = [len(r) for r in rows_of]
    assert Ms[3] == 0 and min(Ms[:3]) > 0
    w13, s13, w2, s2 = [], [], [], []
    for e in range(E):
        w, s = kind.weights(rng, Hd, 2 * I, gs1)
        w13.append(w)
        s13.append(s)
        w, s = kind.weights(rng, I, Hd, gs2)
        w2.append(w)
        s2.append(s)
    src = [H.to_dev(np.ascontiguousarray(x[rows_of[e]])) if Ms[e] else None for e in range(E)]
    dst = [torch.zeros((max(Ms[e], 1), 2 * I), dtype=torch.bfloat16, device=H.DEV) for e in range(E)]
    dst_down = [torch.zeros((max(Ms[e], 1), Hd), dtype=torch.bfloat16, device=H.DEV) for e in range(E)]
    s13_d = [H.to_dev(s) for s in s13]
    s2_d = [H.to_dev(s) for s in s2]
    params = [kind.params(Ms[e], Hd, 2 * I, gs1, s13_d[e], per_group_src) for e in range(E)]
    down_scale = None
    if kind.name != "ggml":
        down_scale = [lowoha.QuantParam(s2_d[e], capi.DT_F32, (I // gs2, Hd)) for e in range(E)]
    fm = lowoha.FusedMoe(down_weight=[H.to_dev(w) for w in w2], N_down=[Hd] * E, ldb_down=[kind.ldb(I, Hd)] * E,
                         down_scale=down_scale, dst_down=dst_down, ldc_down=[Hd] * E)
    out = torch.zeros((T, Hd), dtype=torch.bfloat16, device=H.DEV)
    rp = [dst_down[slot[(t, k)][0]].data_ptr() + slot[(t, k)][1] * Hd * 2 for t in range(T) for k in range(topk)]
    pp = lowoha.MoePostop(T, topk, out, Hd, H.to_dev(tw), rp)
    st = lowoha.group_matmul_direct(
        ["r"] * E, [False] * E, [kind.transB] * E, Ms, [2 * I] * E, [Hd] * E, [1.0] * E,
        src, [Hd] * E, [H.to_dev(w) for w in w13], [kind.ldb(Hd, 2 * I)] * E, [None] * E, [0.0] * E,
        dst, [2 * I] * E, [True] * E, params, moe_postop=pp, gated_act=act, fused_moe=fm)
    assert st == capi.SUCCESS, lowoha.last_error()

    y2 = {}
    for e in range(E):
        if Ms[e] == 0:
            continue
        xe = np.ascontiguousarray(x[rows_of[e]])
        y1 = _oracle_product(zo, kind, xe, w13[e], s13[e], Ms[e], Hd, 2 * I, gs1, per_group_src)
        zo.gated_act(act, y1, capi.DT_BF16)
        a = np.ascontiguousarray(y1[:, :I])
        # stage 1 (Op1 + activation) as the library left it in the caller's dst
        H.check_bf16(H.to_host(dst[e])[:Ms[e], :I], a, max_frac=5e-3, atol=1e-6 if act == capi.ACT_GELU_AND_MUL else 0.0)
        y2[e] = _oracle_product(zo, kind, a, w2[e], s2[e], Ms[e], I, Hd, gs2, per_group_src)
        check_moe_out(H.to_host(dst_down[e])[:Ms[e]], y2[e], flipped_rows=1)
    rows = [np.ascontiguousarray(y2[slot[(t, k)][0]][slot[(t, k)][1]]) for t in range(T) for k in range(topk)]
    want = zo.moe_reduce(rows, tw, capi.DT_BF16, Hd)
    check_moe_out(H.to_host(out), want, flipped_rows=1)
    capi.load().zmi_clear_weight_cache()


def test_gated_act_on_static_per_group_experts(zo):
    """The reference's own case (gtests/group_matmul/test_quant.cpp:470-560): static s8 rows with {M,G} x {G,N}
    scales, bf16 destination, a gated activation over the grouped call."""
    rng = np.random.default_rng(470)
    Ms, K, N, gs = [9, 0, 33], 128, 96, 16
    G = K // gs
    E = len(Ms)
    srcs, weis, dsts, params, host = [], [], [], [], []
    for m in Ms:
        a = rng.integers(-128, 128, (max(m, 1), K), dtype=np.int8)
        w = rng.integers(-127, 128, (K, N), dtype=np.int8)
        ss = rng.uniform(0.005, 0.03, (max(m, 1), G)).astype(np.float32)
        ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
        ss_d, ws_d = H.to_dev(ss), H.to_dev(ws)
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16)
        p.src_scale = lowoha.QuantParam(ss_d, capi.DT_F32, (m, G))
        p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, (G, N))
        srcs.append(H.to_dev(a) if m else None)
        weis.append(H.to_dev(w))
        dsts.append(torch.zeros((max(m, 1), N), dtype=torch.bfloat16, device=H.DEV))
        params.append(p)
        host.append((a, w, ss, ws))
    st = lowoha.group_matmul_direct(["r"] * E, [False] * E, [False] * E, Ms, [N] * E, [K] * E, [1.0] * E,
                                    srcs, [K] * E, weis, [N] * E, [None] * E, [0.0] * E, dsts, [N] * E, [True] * E, params,
                                    gated_act=capi.ACT_SILU_AND_MUL)
    assert st == capi.SUCCESS, lowoha.last_error()
    keep = []
    for e, m in enumerate(Ms):
        if m == 0:
            continue
        a, w, ss, ws = host[e]
        ph = H.host_params(params[e], src_scale=ss, wei_scale=ws)
        st, y, _, _ = zo.matmul_int8(a[:m], w, ph.flat(keep), m, N, K)
        assert st == capi.SUCCESS
        zo.gated_act(capi.ACT_SILU_AND_MUL, y, capi.DT_BF16)
        H.check_bf16(H.to_host(dsts[e])[:m, :N // 2], y[:, :N // 2], max_frac=5e-3)
    # a tight destination (ldc = N / 2) cannot hold Op1's full rows on this path
    st = lowoha.group_matmul_direct(["r"] * E, [False] * E, [False] * E, Ms, [N] * E, [K] * E, [1.0] * E,
                                    srcs, [K] * E, weis, [N] * E, [None] * E, [0.0] * E, dsts, [N // 2] * E, [True] * E, params,
                                    gated_act=capi.ACT_SILU_AND_MUL)
    assert st == capi.UNIMPLEMENTED
