"""GPU tests of zmi_moe_router_topk (through the C ABI): expert ids bit-exact against a stable
descending sort of the logits on the host, weights against a float64 softmax (<= 1e-6 relative).

The reference has no router (the framework builds topk ids / weights on the host,
docs/operator/low_overhead_operator/lowoha_group_matmul_operator.md:238-259), so there is no
reference output to compare with: the expected values are what the mathematics fixes (the head of a
stable sort; softmax in float64)."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu

REL_TOL = 1e-6


def expect(logits_f32, topk, renormalize):
    x = logits_f32.astype(np.float64)
    ids = np.argsort(-logits_f32, axis=1, kind="stable")[:, :topk]        # -(+0) == -0 == +0: equal, index order
    p = np.exp(x - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    w = np.take_along_axis(p, ids, axis=1)
    if renormalize:
        w = w / w.sum(axis=1, keepdims=True)
    return ids.astype(np.int32), w


def run(logits_t, topk, renormalize):
    st, ids, w = lowoha.moe_router_topk(logits_t, topk, renormalize)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert lowoha.last_kernel() == "moe_router_topk"
    return H.to_host(ids), H.to_host(w)


@pytest.mark.parametrize("T,E,topk", [(1, 1, 1), (1, 8, 2), (5, 8, 2), (512, 8, 2), (4096, 64, 6), (33, 60, 8),
                                      (130, 128, 8), (77, 65, 4), (40, 512, 64), (9, 300, 1), (3, 16, 16)])
@pytest.mark.parametrize("renormalize", [False, True])
def test_random_logits_f32(T, E, topk, renormalize):
    rng = np.random.default_rng(T * 1000 + E * 10 + topk)
    x = (rng.standard_normal((T, E)) * 3.0).astype(np.float32)
    got_ids, got_w = run(H.to_dev(x), topk, renormalize)
    want_ids, want_w = expect(x, topk, renormalize)
    assert np.array_equal(got_ids, want_ids)
    assert np.all(np.abs(got_w - want_w) <= REL_TOL * want_w)
    if renormalize:
        assert np.all(np.abs(got_w.astype(np.float64).sum(axis=1) - 1.0) <= 1e-6)


@pytest.mark.parametrize("E,topk", [(8, 2), (64, 6), (200, 8)])
def test_ties_go_to_the_lower_expert(E, topk):
    """Logits on a coarse grid (many equal values), all-equal rows, and +0 / -0 mixes."""
    rng = np.random.default_rng(E + topk)
    T = 300
    x = rng.integers(-2, 3, size=(T, E)).astype(np.float32) * 0.5
    x[0, :] = 1.25                                          # all equal: experts 0 .. topk-1, weights 1/E each
    x[1, :] = np.where(rng.random(E) < 0.5, 0.0, -0.0)      # signed zeros are one value
    x[2, :] = -3.0
    x[2, E - 1] = 7.0                                       # a single winner in the last position
    got_ids, got_w = run(H.to_dev(x), topk, False)
    want_ids, want_w = expect(x, topk, False)
    assert np.array_equal(got_ids, want_ids)
    assert got_ids[0].tolist() == list(range(topk)) and got_ids[1].tolist() == list(range(topk))
    assert got_ids[2, 0] == E - 1
    assert np.all(np.abs(got_w - want_w) <= REL_TOL * want_w)
    assert np.all(np.abs(got_w[0] - 1.0 / E) <= REL_TOL / E)


def test_bf16_logits_and_row_stride():
    """bf16 logits (what a bf16 gate projection leaves), read from a wider buffer (ldl > E)."""
    rng = np.random.default_rng(42)
    T, E, ld, topk = 257, 64, 80, 6
    buf = torch.from_numpy((rng.standard_normal((T, ld)) * 4.0).astype(np.float32)).to(torch.bfloat16).to(H.DEV)
    view = buf[:, :E]
    assert view.stride(0) == ld
    got_ids, got_w = run(view, topk, True)
    x = view.float().cpu().numpy()                          # (bf16 values are exactly representable in f32)
    want_ids, want_w = expect(x, topk, True)
    assert np.array_equal(got_ids, want_ids)
    assert np.all(np.abs(got_w - want_w) <= REL_TOL * want_w)


def test_extreme_logits():
    """Large spread (probabilities underflow to 0 beside the winner), -inf entries, and a NaN that must
    sort behind every number."""
    E, topk = 32, 4
    x = np.zeros((4, E), dtype=np.float32)
    x[0] = np.linspace(-200.0, 200.0, E)
    x[1] = -np.inf
    x[1, [3, 9, 20, 21, 22]] = [1.0, 5.0, -2.0, 5.0, 0.5]
    x[2] = np.linspace(1e30, -1e30, E)
    x[3] = np.arange(E, dtype=np.float32)
    got_ids, got_w = run(H.to_dev(x), topk, False)
    want_ids, want_w = expect(x, topk, False)
    assert np.array_equal(got_ids, want_ids)
    assert got_ids[1].tolist() == [9, 21, 3, 22]
    assert np.all(np.abs(got_w - want_w) <= REL_TOL * want_w + 1e-45)
    y = x[3:4].copy()
    y[0, 31] = np.nan
    ids_nan, _ = run(H.to_dev(y), topk, False)
    assert ids_nan[0].tolist() == [30, 29, 28, 27]


def test_router_feeds_route_and_fused_block_shapes():
    """The ids this kernel writes are what zmi_moe_route consumes: counts add up, every expert id in range."""
    rng = np.random.default_rng(7)
    T, E, topk = 1000, 64, 6
    x = H.to_dev(rng.standard_normal((T, E)).astype(np.float32))
    st, ids, w = lowoha.moe_router_topk(x, topk, True)
    assert st == capi.SUCCESS, lowoha.last_error()
    st, counts, offsets, slot_of = lowoha.moe_route(ids, E)
    assert st == capi.SUCCESS, lowoha.last_error()
    assert int(H.to_host(counts).sum()) == T * topk
    so = np.sort(H.to_host(slot_of))
    assert np.array_equal(so, np.arange(T * topk))
    # a token never selects one expert twice
    hid = np.sort(H.to_host(ids), axis=1)
    assert np.all(hid[:, 1:] != hid[:, :-1])


def test_argument_checks():
    x = H.to_dev(np.zeros((4, 8), dtype=np.float32))
    st, _, _ = lowoha.moe_router_topk(x, 9)
    assert st == capi.FAILURE and "topk" in lowoha.last_error()
    big = H.to_dev(np.zeros((2, 600), dtype=np.float32))
    st, _, _ = lowoha.moe_router_topk(big, 2)
    assert st == capi.UNIMPLEMENTED
    lib = capi.load()
    ids = torch.empty(8, dtype=torch.int32, device=H.DEV)
    w = torch.empty(8, dtype=torch.float32, device=H.DEV)
    assert lib.zmi_moe_router_topk(x.data_ptr(), capi.DT_S8, 8, 4, 8, 2, 0, ids.data_ptr(), w.data_ptr()) == capi.FAILURE
    assert lib.zmi_moe_router_topk(x.data_ptr(), capi.DT_F32, 4, 4, 8, 2, 0, ids.data_ptr(), w.data_ptr()) == capi.FAILURE
    assert lib.zmi_moe_router_topk(None, capi.DT_F32, 8, 4, 8, 2, 0, ids.data_ptr(), w.data_ptr()) == capi.FAILURE
