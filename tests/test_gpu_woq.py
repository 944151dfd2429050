"""GPU parity of matmul_direct for weight-only quantization: a bf16 source, packed s4 / u4 weights with scales (and
zero-points), no dynamic_quant.  The reference makes a bf16 weight matrix from the codes once and runs a bf16 GEMM with
f32 accumulation on it (lowoha_operators/matmul/backends/aocl/aocl_kernel.cpp:43-139, 640-702, 944-966); the library
keeps the codes 4-bit and makes the same bf16 values in registers.

Two bars.  The dequantized weights are compared bit for bit: a source of one-hot rows makes the product the weight
matrix itself.  Whole products are sums of the same exact bf16 x bf16 products in f32, in an order that is the
GEMM's own on both sides (the reference's is AOCL's), so they are compared to a tolerance stated in `_check`."""
import numpy as np
import pytest
import torch

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H

pytestmark = pytest.mark.gpu


def _pack4(codes, ld):
    R, C = codes.shape
    full = np.full((R, ld), 5, dtype=np.int64)
    full[:, :C] = codes
    flat = full.reshape(-1) & 15
    if flat.size % 2:
        flat = np.append(flat, 0)
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)


KINDS = {"s4": (capi.DT_S4, None), "s4_zp": (capi.DT_S4, capi.DT_S8), "u4_s8": (capi.DT_U4, capi.DT_S8),
         "u4_bf16": (capi.DT_U4, capi.DT_BF16)}


def _weights(rng, K, N, kind, gran, G, transB, pad, ws_bf16):
    wdt, zdt = KINDS[kind]
    codes = rng.integers(0, 16, (K, N)) if wdt == capi.DT_U4 else rng.integers(-8, 8, (K, N))
    ldb = (K if transB else N) + pad
    packed = _pack4(codes.T.copy(), ldb) if transB else _pack4(codes, ldb)
    dims = {"tensor": (1, 1), "channel": (1, N), "group": (G, N)}[gran]
    ws = rng.uniform(0.01, 0.1, dims).astype(np.float32)
    ws_h, ws_dt = (H.bf16_bits(ws), capi.DT_BF16) if ws_bf16 else (ws, capi.DT_F32)
    zp_h = None
    if zdt == capi.DT_S8:
        zp_h = rng.integers(0 if wdt == capi.DT_U4 else -3, 16 if wdt == capi.DT_U4 else 4, dims).astype(np.int8)
    elif zdt == capi.DT_BF16:
        zp_h = H.bf16_bits(rng.uniform(-0.2, 0.2, dims).astype(np.float32))
    return wdt, zdt, packed, ldb, dims, ws_h, ws_dt, zp_h


def _params(wdt, zdt, dims, ws_d, ws_dt, zp_d, dst_dt, bias, postops):
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=wdt, dst=dst_dt, compute=capi.DT_NONE,
                            bias=capi.DT_F32 if bias else capi.DT_NONE)
    p.wei_scale = lowoha.QuantParam(ws_d, ws_dt, dims)
    if zdt is not None:
        p.wei_zp = lowoha.QuantParam(zp_d, zdt, dims)
    p.postop_ = list(postops)
    return p


def _dev_or_host(a, dims):
    """One-element parameters may stay in host memory; the others must be device memory."""
    if a is None:
        return None
    if int(np.prod(dims)) == 1:
        return a.ctypes.data
    return H.to_dev(a.reshape(-1))


def _check(got, want, mag, dst_dt):
    """f32 results: |got - want| <= 1e-5 * sum_k |a||w| (K up to 4096 f32 additions in two different orders);
    bf16 results: the same bound, or one bf16 unit in the last place."""
    if dst_dt == capi.DT_F32:
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        assert (err <= 1e-5 * mag + 1e-30).all(), f"worst {np.max(err / (mag + 1e-30)):.3e} of the magnitude sum"
        return
    g = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    w = (want.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ok = (H.bf16_ulp_diff(got, want) <= 1) | (np.abs(g - w) <= 1e-5 * mag)
    assert ok.all(), f"{(~ok).sum()} elements outside one bf16 ulp and the f32 accumulation bound"
    assert (H.bf16_ulp_diff(got, want) != 0).mean() <= 0.02


def _run(zo, M, K, N, kind, gran="group", G=None, *, transB=False, pad=0, ws_bf16=False, dst_dt=capi.DT_BF16, bias=False,
         postops=(), alpha=1.0, beta=0.0, lda=None, transA=False, cache=True, calls=1, x=None, exact=False, seed=0):
    rng = np.random.default_rng(seed + M * 7 + K + N * 3)
    G = G or max(1, K // 64)
    wdt, zdt, packed, ldb, dims, ws_h, ws_dt, zp_h = _weights(rng, K, N, kind, gran, G, transB, pad, ws_bf16)
    if x is None:
        x = H.bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    lda = lda or (M if transA else K)
    xs = np.zeros((K, lda) if transA else (M, lda), dtype=np.uint16)
    if transA:
        xs[:, :M] = x.T
    else:
        xs[:, :K] = x
    b = rng.standard_normal(N).astype(np.float32) if bias else None
    keepalive = [ws_h, zp_h]
    ws_d, zp_d = _dev_or_host(ws_h, dims), _dev_or_host(zp_h, dims)
    p = _params(wdt, zdt, dims, ws_d, ws_dt, zp_d, dst_dt, bias, postops)
    p.weight_cache_type = 2 if cache else 0
    tdt = torch.bfloat16 if dst_dt == capi.DT_BF16 else torch.float32
    c0 = rng.standard_normal((M, N)).astype(np.float32)
    c0 = H.bf16_bits(c0) if dst_dt == capi.DT_BF16 else c0
    x_d, w_d, b_d = H.to_dev(xs), H.to_dev(packed), H.to_dev(b)
    for _ in range(calls):
        dst = H.to_dev(c0.copy())
        st = lowoha.matmul_direct("r", transA, transB, M, N, K, alpha, x_d, lda, w_d, ldb, b_d, beta, dst, N, True, p)
        assert st == capi.SUCCESS, lowoha.last_error()
        assert lowoha.last_kernel().startswith("woq_u4" if wdt == capi.DT_U4 else "woq_s4"), lowoha.last_kernel()
    assert dst.dtype == tdt
    ph = H.host_params(p, wei_scale=ws_h, **({"wei_zp": zp_h} if zp_h is not None else {}))
    keep = []
    st, want = zo.matmul_woq(xs, packed, ph.flat(keep), M, N, K, bias=b, dst=c0.copy(), lda=lda, ldb=ldb, transA=transA,
                             transB=transB, alpha=alpha, beta=beta)
    assert st == capi.SUCCESS
    got = H.to_host(dst)
    if exact:
        assert np.array_equal(got, want)
    else:
        wb = zo.woq_dequant(packed, K, N, wdt, ws_h, ws_dt, zp_h, zdt or 0, ldb=ldb, transposed=transB)
        mag = np.abs(zo.bf16_to_f32(x).astype(np.float64)) @ np.abs(zo.bf16_to_f32(wb).astype(np.float64)) * abs(alpha)
        if beta:
            mag = mag + np.abs((zo.bf16_to_f32(c0) if dst_dt == capi.DT_BF16 else c0).astype(np.float64)) * abs(beta)
        if postops:
            # the activations used here have slope <= ~1.1: the bound carries over; their own last-ulp rule is check_bf16's
            mag = mag * 1.2 + 1e-6
        _check(got, want, mag, dst_dt)
    del keepalive
    capi.load().zmi_clear_weight_cache()


def _one_hot(K):
    x = np.zeros((K, K), dtype=np.float32)
    x[np.arange(K), np.arange(K)] = 1.0
    return H.bf16_bits(x)


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("gran,G", [("tensor", 1), ("channel", 1), ("group", 2), ("group", 4), ("group", 32)])
def test_dequantized_weights_are_the_reference_values_bit_for_bit(zo, kind, gran, G):
    # one-hot rows: row k of the product is row k of the bf16 weight matrix, plus zeros
    K, N = 256, 70
    _run(zo, K, K, N, kind, gran, G, x=_one_hot(K), dst_dt=capi.DT_F32, exact=True)


@pytest.mark.parametrize("kind", ["s4", "u4_bf16"])
@pytest.mark.parametrize("transB,pad", [(False, 0), (False, 3), (True, 0), (True, 5)])
def test_dequantized_weights_any_orientation_and_scale_type(zo, kind, transB, pad):
    K, N = 192, 45          # K is not a multiple of the 64-value tile
    _run(zo, K, K, N, kind, "group", 8, x=_one_hot(K), dst_dt=capi.DT_F32, exact=True, transB=transB, pad=pad, ws_bf16=True)
    _run(zo, K, K, N, kind, "group", 3, x=_one_hot(K), dst_dt=capi.DT_BF16, exact=True, transB=transB, pad=pad)


@pytest.mark.parametrize("M", [1, 4, 16, 33, 64, 100, 130, 300])
@pytest.mark.parametrize("kind", ["s4", "u4_s8"])
def test_products_by_row_count(zo, M, kind):
    _run(zo, M, 1024, 200, kind, "group", 8, calls=2)
    _run(zo, M, 520, 64, kind, "channel", dst_dt=capi.DT_F32, bias=True)


@pytest.mark.parametrize("kind", list(KINDS))
def test_decode_shape_of_the_headline_layer(zo, kind):
    _run(zo, 16, 4096, 14336, kind, "group", 32, bias=True, postops=[lowoha.PostOp(capi.PO_SWISH)])


@pytest.mark.parametrize("postop", [capi.PO_GELU_TANH, capi.PO_RELU, capi.PO_SWISH])
def test_post_ops_alpha_beta(zo, postop):
    _run(zo, 9, 512, 96, "s4", "group", 4, postops=[lowoha.PostOp(postop)], bias=True)
    _run(zo, 40, 512, 96, "u4_bf16", "group", 4, alpha=0.5, beta=0.25, dst_dt=capi.DT_F32)
    _run(zo, 40, 512, 96, "u4_s8", "tensor", alpha=2.0, beta=1.0, bias=True)


def test_binary_post_ops(zo):
    rng = np.random.default_rng(5)
    M, N = 20, 72
    add = H.to_dev(rng.standard_normal((M, N)).astype(np.float32))
    mul = H.to_dev(rng.standard_normal((1, N)).astype(np.float32))
    pos = [lowoha.PostOp(capi.PO_BINARY_ADD, buff=add, dtype=capi.DT_F32, dims=(M, N)),
           lowoha.PostOp(capi.PO_BINARY_MUL, buff=mul, dtype=capi.DT_F32, dims=(1, N))]
    rngw = np.random.default_rng(M * 7 + 256 + N * 3)
    wdt, zdt, packed, ldb, dims, ws_h, ws_dt, zp_h = _weights(rngw, 256, N, "s4", "group", 4, False, 0, False)
    x = H.bf16_bits(rngw.standard_normal((M, 256)).astype(np.float32))
    p = _params(wdt, zdt, dims, H.to_dev(ws_h.reshape(-1)), ws_dt, None, capi.DT_F32, False, pos)
    dst = torch.zeros((M, N), dtype=torch.float32, device=H.DEV)
    st = lowoha.matmul_direct("r", False, False, M, N, 256, 1.0, H.to_dev(x), 256, H.to_dev(packed), ldb, None, 0.0, dst, N, True, p)
    assert st == capi.SUCCESS, lowoha.last_error()
    wb = zo.bf16_to_f32(zo.woq_dequant(packed, 256, N, wdt, ws_h, ws_dt)).astype(np.float64)
    full = zo.bf16_to_f32(x).astype(np.float64) @ wb
    want = (full + H.to_host(add)) * H.to_host(mul)
    assert np.abs(H.to_host(dst) - want).max() <= 1e-5 * (np.abs(zo.bf16_to_f32(x)).astype(np.float64) @ np.abs(wb)).max() * 4
    capi.load().zmi_clear_weight_cache()


def test_sources_the_fast_row_loads_do_not_take(zo):
    _run(zo, 7, 100, 40, "s4", "channel", dst_dt=capi.DT_F32)              # K is not a multiple of 8
    _run(zo, 40, 36, 70, "u4_s8", "tensor")


def test_source_strides_and_transposed_sources(zo):
    _run(zo, 7, 96, 40, "s4", "group", 4, lda=101, dst_dt=capi.DT_F32)     # odd leading dimension
    _run(zo, 7, 96, 40, "u4_s8", "group", 4, lda=104)                       # padded, still 16-byte rows
    _run(zo, 12, 128, 33, "s4", "channel", transA=True, lda=14, dst_dt=capi.DT_F32)


def test_uncached_weights(zo):
    _run(zo, 16, 512, 100, "s4", "group", 8, cache=False, calls=2)
    _run(zo, 70, 512, 100, "u4_bf16", "group", 8, cache=False, calls=2)


def test_rejections():
    M, K, N, G = 4, 64, 8, 2
    x_d = H.to_dev(np.zeros((M, K), dtype=np.uint16))
    w_d = H.to_dev(np.zeros(K * N // 2, dtype=np.uint8))
    ws_d = torch.ones(G * N, dtype=torch.float32, device=H.DEV)
    zp_d = torch.zeros(G * N, dtype=torch.int8, device=H.DEV)
    one = np.ones(1, dtype=np.float32)

    def call(wei=capi.DT_S4, dst_dt=capi.DT_BF16, const=True, wdims=(G, N), zp=None, zp_dt=capi.DT_S8, zdims=(G, N),
             scale=True, src_scale=False, fmt="n"):
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=wei, dst=dst_dt, compute=capi.DT_NONE)
        if scale:
            p.wei_scale = lowoha.QuantParam(ws_d, capi.DT_F32, wdims)
        if zp is not None:
            p.wei_zp = lowoha.QuantParam(zp, zp_dt, zdims)
        if src_scale:
            p.src_scale = lowoha.QuantParam(one.ctypes.data, capi.DT_F32, (1, 1))
        p.mem_format_b = fmt
        if fmt == "r":
            p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        tdt = {capi.DT_BF16: torch.bfloat16, capi.DT_F32: torch.float32, capi.DT_F16: torch.float16, capi.DT_S8: torch.int8}[dst_dt]
        dst = torch.zeros((M, N), dtype=tdt, device=H.DEV)
        return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, x_d, K, w_d, N, None, 0.0, dst, N, const, p)

    assert call() == capi.SUCCESS
    assert call(zp=zp_d) == capi.SUCCESS
    assert call(wei=capi.DT_U4, zp=zp_d) == capi.SUCCESS
    assert call(const=False) == capi.FAILURE                        # the weights must be constant
    assert call(src_scale=True) == capi.FAILURE                     # no source / destination quantization
    assert call(wei=capi.DT_U4) == capi.FAILURE                     # u4 needs a zero-point
    assert call(wei=capi.DT_U4, zp=zp_d, zp_dt=capi.DT_S32) == capi.FAILURE
    assert call(dst_dt=capi.DT_F16) == capi.FAILURE
    assert call(scale=False) == capi.FAILURE
    assert call(wdims=(3, N)) == capi.FAILURE                       # groups do not divide K
    assert call(wdims=(G, N - 1)) == capi.FAILURE
    assert call(zp=zp_d, zdims=(1, 3)) == capi.FAILURE
    assert call(fmt="r") == capi.FAILURE
    assert call(wdims=(16, N)) == capi.UNIMPLEMENTED                # groups of 4 values of K
    assert call(dst_dt=capi.DT_S8) == capi.UNIMPLEMENTED
    capi.load().zmi_clear_weight_cache()


@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_kinds_and_granularities(zo, seed):
    rng = np.random.default_rng(9000 + seed)
    M = int(rng.choice([1, 2, 5, 16, 17, 32, 33, 63, 64, 65, 100, 129, 200]))
    K = int(rng.choice([8, 24, 64, 72, 120, 128, 192, 520, 1000, 1024, 1536, 4104]))
    N = int(rng.integers(1, 150))
    kind = list(KINDS)[int(rng.integers(0, 4))]
    gran = ["tensor", "channel", "group"][int(rng.integers(0, 3))]
    G = 1
    if gran == "group":
        divs = [g for g in (2, 3, 4, 5, 8, 13, 16, 24) if K % g == 0 and (K // g) % 8 == 0]
        if not divs:
            gran = "channel"
        else:
            G = int(rng.choice(divs))
    _run(zo, M, K, N, kind, gran, G, ws_bf16=bool(rng.integers(0, 2)), dst_dt=[capi.DT_BF16, capi.DT_F32][int(rng.integers(0, 2))],
         bias=bool(rng.integers(0, 2)), transB=bool(rng.integers(0, 2)), pad=int(rng.integers(0, 2)) * 2,
         cache=bool(rng.integers(0, 4)), seed=seed)


@pytest.mark.parametrize("kind", list(KINDS))
def test_two_column_blocks_per_workgroup(zo, kind, monkeypatch):
    # the form wide decode-shaped calls take by themselves (more than 4 rows, at least 384 column blocks), forced here
    # on small shapes: odd block counts, one block, a K tail, one-hot sources (bit-exact)
    monkeypatch.setenv("ZMI_WOQ_BLOCKS", "2")
    _run(zo, 32, 256, 70, kind, "group", 4, x=_one_hot(256)[:32], dst_dt=capi.DT_F32, exact=True)
    _run(zo, 16, 1000, 33, kind, "channel", bias=True)
    _run(zo, 1, 512, 20, kind, "tensor", dst_dt=capi.DT_F32)
    _run(zo, 9, 1024, 200, kind, "group", 8, calls=2)
    _run(zo, 40, 512, 100, kind, "group", 8)          # more than 32 rows: the one-block form whatever the switch says


def test_wide_decode_calls_take_two_column_blocks_by_themselves(zo):
    _run(zo, 16, 1024, 12288, "s4", "group", 8, bias=True)
    assert "two column blocks" in lowoha.last_kernel()
    _run(zo, 16, 1024, 12360, "u4_bf16", "group", 8)      # 387 column blocks: the last workgroup has one
    assert "two column blocks" in lowoha.last_kernel()
    _run(zo, 4, 1024, 12288, "s4", "group", 8)
    assert "two column blocks" not in lowoha.last_kernel()
