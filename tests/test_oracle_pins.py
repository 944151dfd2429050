"""Pins the CPU oracle against facts that do not come from the oracle itself:
closed forms, integer identities, brute force in Python integers, libm in
double precision, torch's bfloat16, and the deterministic recipes the
reference's examples use.  A dropped term, a wrong sign or index, or a
transposed operand fails at least one of these."""
import math

import numpy as np
import pytest
import torch

from zendnn_amd import capi


# ---------------------------------------------------------------- bf16
def test_bf16_ctor_matches_torch_on_normals(zo):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 200000).astype(np.float32)
    ours = zo.f32_to_bf16(x, ctor=True)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    assert np.array_equal(zo.f32_to_bf16(x, ctor=False), ref)


def test_bf16_exhaustive_high_half_and_ties(zo):
    hi = np.arange(65536, dtype=np.uint32) << 16
    # exact, just-below-tie, tie, just-above-tie, all-ones low half
    for lo in (0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        bits = (hi | lo).astype(np.uint32)
        x = bits.view(np.float32)
        got = zo.f32_to_bf16(x, ctor=True).astype(np.uint32)
        exp_field = (bits >> 23) & 0xFF
        man = bits & 0x7FFFFF
        normal = (exp_field != 0) & (exp_field != 0xFF)
        up = (lo > 0x8000) | ((lo == 0x8000) & (((bits >> 16) & 1) == 1))
        want_normal = ((bits >> 16) + up.astype(np.uint32)) & 0xFFFF
        assert np.array_equal(got[normal], want_normal[normal])
        sub = exp_field == 0                       # zero / subnormal -> signed zero
        assert np.array_equal(got[sub], (bits[sub] >> 16) & 0x8000)
        inf = (exp_field == 0xFF) & (man == 0)
        assert np.array_equal(got[inf], bits[inf] >> 16)
        nan = (exp_field == 0xFF) & (man != 0)
        assert np.array_equal(got[nan], (bits[nan] >> 16) | 0x40)
        # the plain bit trick has no special cases
        got2 = zo.f32_to_bf16(x, ctor=False).astype(np.uint32)
        want2 = ((bits.astype(np.uint64) + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF
        assert np.array_equal(got2, want2.astype(np.uint32))


def test_bf16_round_trip(zo):
    h = np.arange(65536, dtype=np.uint16)
    f = zo.bf16_to_f32(h)
    ok = ~np.isnan(f) & ((h & 0x7F80) != 0)
    assert np.array_equal(zo.f32_to_bf16(f[ok]), h[ok])


# ------------------------------------------------------- per-token quant
def _bf16(x, zo):
    return zo.f32_to_bf16(np.asarray(x, dtype=np.float32))


def test_quant_constant_row_closed_form(zo):
    for c in (0.5, -3.0, 127.0, 1e-3):
        src = _bf16(np.full((1, 64), c), zo)
        cb = float(zo.bf16_to_f32(src[0, :1])[0])
        q, s = zo.quant_per_token(src, capi.DT_BF16)
        assert s[0] == np.float32(abs(cb)) / np.float32(127.0)
        assert np.all(q == (127 if c > 0 else -127))


def test_quant_zero_row_and_nonfinite(zo):
    src = np.zeros((3, 32), dtype=np.float32)
    src[1, 3] = np.inf
    src[1, 4] = np.nan
    src[1, 5] = -np.inf
    src[1, 6] = 2.0
    src[2, :] = np.nan
    q, s = zo.quant_per_token(src, capi.DT_F32)
    assert s[0] == np.float32(1e-10)          # 1e-10/127 clamped back up to 1e-10
    assert np.all(q[0] == 0)
    assert s[1] == np.float32(2.0) / np.float32(127.0)   # non-finite excluded from absmax
    assert q[1, 3] == 0 and q[1, 4] == 0 and q[1, 5] == 0 and q[1, 6] == 127
    assert s[2] == np.float32(1e-10) and np.all(q[2] == 0)


def test_quant_ties_round_to_even(zo):
    # absmax 127 -> scale exactly 1 -> v/scale == v; halves must go to even
    vals = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5, -126.5], dtype=np.float32)
    q, s = zo.quant_per_token(vals[None, :], capi.DT_F32)
    assert s[0] == 1.0
    assert q[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 4, 126, -126]


def test_quant_invariants_random(zo):
    rng = np.random.default_rng(7)
    x = _bf16(rng.standard_normal((37, 515)), zo)
    q, s = zo.quant_per_token(x, capi.DT_BF16)
    xf = zo.bf16_to_f32(x)
    assert np.all(np.abs(q.astype(np.int32)).max(axis=1) == 127)
    assert np.array_equal(s, (np.abs(xf).max(axis=1) / np.float32(127.0)).astype(np.float32))
    # what "quantized" means, in float64 and without the oracle's rounding routine: q is an integer nearest
    # to x / s (the f32 quotient the oracle rounds is within 2^-24 relative of the exact one, i.e. 127 * 2^-24
    # absolute), it keeps the sign and the order of x within a row, and x -> q * s loses at most half a step
    r = xf.astype(np.float64) / s.astype(np.float64)[:, None]
    assert np.all(np.abs(q.astype(np.float64) - r) <= 0.5 + 127.0 * 2.0 ** -24)
    assert np.all((q.astype(np.int32) * np.sign(xf).astype(np.int32)) >= 0)
    order = np.argsort(xf, axis=1, kind="stable")
    assert np.all(np.diff(np.take_along_axis(q.astype(np.int32), order, axis=1), axis=1) >= 0)
    assert np.all(np.abs(xf.astype(np.float64) - q.astype(np.float64) * s.astype(np.float64)[:, None])
                  <= 0.5 * s.astype(np.float64)[:, None] * (1.0 + 1e-5))


# ------------------------------------------------------------ s32 GEMM
def test_gemm_all_ones_closed_form(zo):
    A = np.ones((5, 77), dtype=np.uint8)
    B = np.ones((77, 9), dtype=np.int8)
    acc, ov = zo.gemm_s32(A, B)
    assert ov == 0 and np.all(acc == 77)


def test_gemm_brute_force_python_ints_and_transposes(zo):
    rng = np.random.default_rng(3)
    M, K, N = 7, 19, 5
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    As = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    for a in (A, As):
        want = [[sum(int(a[m, k]) * int(B[k, n]) for k in range(K)) for n in range(N)] for m in range(M)]
        acc, ov = zo.gemm_s32(a, B)
        assert ov == 0 and acc.tolist() == want
        acc_t, _ = zo.gemm_s32(np.ascontiguousarray(a.T), np.ascontiguousarray(B.T), transA=True, transB=True)
        assert acc_t.tolist() == want
    # a non-symmetric case catches swapped operands: A @ B != (B.T @ A.T) elementwise unless transposed
    assert acc.shape == (M, N)


def test_gemm_reference_example_recipe(zo):
    # deterministic recipe of the reference's int8 example
    # (examples/lowoha_matmul_example.cpp:509-535): w = (i % 7) - 3, a = (i + 17*iter) % 256
    M, K, N = 4, 64, 8
    w = np.array([(i % 7) - 3 for i in range(K * N)], dtype=np.int8).reshape(K, N)
    for it in range(3):
        a = np.array([(i + 17 * it) % 256 for i in range(M * K)], dtype=np.uint8).reshape(M, K)
        acc, ov = zo.gemm_s32(a, w)
        want = a.astype(np.int64) @ w.astype(np.int64)
        assert ov == 0 and np.array_equal(acc.astype(np.int64), want)


def test_gemm_extremes_fit_int32(zo):
    K = 14336
    A = np.full((1, K), -128, dtype=np.int8)
    B = np.full((K, 1), -127, dtype=np.int8)
    acc, ov = zo.gemm_s32(A, B)
    assert ov == 0 and acc[0, 0] == 128 * 127 * K


def test_fast_and_general_gemm_agree(zo):
    import ctypes as C
    rng = np.random.default_rng(11)
    M, K, N = 9, 300, 33
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    Bt = np.empty((N, K), dtype=np.int8)
    L = zo.lib()
    L.zo_transpose_s8(B.ctypes.data, K, N, N, Bt.ctypes.data)
    assert np.array_equal(Bt, B.T)
    acc = np.empty((M, N), dtype=np.int32)
    L.zo_gemm_s32_bt(A.ctypes.data, capi.DT_S8, K, Bt.ctypes.data, K, M, N, K, acc.ctypes.data, N)
    assert np.array_equal(acc, A.astype(np.int32) @ B.astype(np.int32))


# ------------------------------------------------- zero-point compensation
def test_zp_identity(zo):
    rng = np.random.default_rng(5)
    M, K, N, zp = 6, 40, 11, 128
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    comp = np.empty(N, dtype=np.int32)
    zo.lib().zo_zp_comp(B.ctypes.data, 0, N, K, N, zp, comp.ctypes.data)
    acc, _ = zo.gemm_s32(A, B)
    want = (A.astype(np.int64) - zp) @ B.astype(np.int64)
    assert np.array_equal(acc.astype(np.int64) + comp[None, :], want)
    comp0 = np.empty(N, dtype=np.int32)
    zo.lib().zo_zp_comp(B.ctypes.data, 0, N, K, N, 0, comp0.ctypes.data)
    assert np.all(comp0 == 0)


@pytest.mark.parametrize("u8", [False, True])
@pytest.mark.parametrize("transA", [False, True])
def test_weight_zero_point_is_the_integer_product_of_the_shifted_operands(zo, u8, transA):
    """(A - a_zp)(W - w_zp) evaluated in Python integers equals the oracle's s32 result with a source and a weight
    zero-point (either alone as well): the 2-D compensation's three terms, none dropped, no sign wrong."""
    rng = np.random.default_rng(12 + int(u8) + 2 * int(transA))
    M, K, N = 7, 45, 13
    A = rng.integers(0, 256, (M, K), dtype=np.uint8) if u8 else rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    src = np.ascontiguousarray(A.T) if transA else A
    for a_zp, w_zp, w_dt in ((0, 5, np.int8), (3 if not u8 else 131, -7, np.int32), (-2 if not u8 else 17, 0, np.int8)):
        azp = np.array([a_zp], dtype=np.int32)
        wzp = np.array([w_zp], dtype=w_dt)
        p = _params(dt_src=capi.DT_U8 if u8 else capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_S32,
                    src_zp=capi.quant(azp.ctypes.data, capi.DT_S32, (1,)) if a_zp else capi.quant(),
                    wei_zp=capi.quant(wzp.ctypes.data, capi.DT_S8 if w_dt == np.int8 else capi.DT_S32, (1,)) if w_zp else capi.quant())
        st, dst, _, _ = zo.matmul_int8(src, B, p, M, N, K, transA=transA, lda=M if transA else K)
        assert st == capi.SUCCESS
        want = (A.astype(np.int64) - a_zp) @ (B.astype(np.int64) - w_zp)
        assert np.array_equal(dst[:, :N].astype(np.int64), want), (a_zp, w_zp)


# ------------------------------------------------------ dequant chain
def _params(**kw):
    p = capi.MatmulParamsT()
    p.mem_format_a = b"n"
    p.mem_format_b = b"n"
    p.lowoha_algo = capi.ALGO_NONE
    p.weight_cache_type = 2
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def test_chain_unit_scales_equals_accumulator(zo):
    rng = np.random.default_rng(9)
    M, K, N = 5, 48, 12
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    one = np.ones(1, dtype=np.float32)
    p = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32,
                src_scale=capi.quant(one.ctypes.data, capi.DT_F32, (1,)),
                wei_scale=capi.quant(one.ctypes.data, capi.DT_F32, (1,)))
    st, dst, acc, _ = zo.matmul_int8(A, B, p, M, N, K, want_acc=True)
    assert st == capi.SUCCESS
    assert np.array_equal(dst[:, :N], acc.astype(np.float32))
    # s32 destination without scales is the accumulator itself
    p2 = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_S32)
    st, dst2, _, _ = zo.matmul_int8(A, B, p2, M, N, K)
    assert np.array_equal(dst2[:, :N], acc)


def test_chain_per_channel_equal_is_per_tensor_and_order(zo):
    rng = np.random.default_rng(10)
    M, K, N = 4, 32, 10
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ss = np.array([0.02], dtype=np.float32)
    zp = np.array([128], dtype=np.int32)
    ws1 = np.array([0.005], dtype=np.float32)
    wsN = np.full(N, 0.005, dtype=np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    outs = []
    for ws, dims in ((ws1, (1,)), (wsN, (1, N))):
        p = _params(dt_src=capi.DT_U8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, dt_bias=capi.DT_F32,
                    src_scale=capi.quant(ss.ctypes.data, capi.DT_F32, (1,)),
                    src_zp=capi.quant(zp.ctypes.data, capi.DT_S32, (1,)),
                    wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, dims))
        st, dst, acc, _ = zo.matmul_int8(A, B, p, M, N, K, bias=bias, want_acc=True)
        assert st == capi.SUCCESS
        outs.append(dst.copy())
    assert np.array_equal(outs[0], outs[1])
    # independent statement of the chain, one float32 rounding per step
    comp = (-128 * B.astype(np.int64).sum(axis=0)).astype(np.float32)
    y = acc.astype(np.float32) + comp[None, :]
    y = (y * np.float32(0.02)).astype(np.float32)
    y = (y * wsN[None, :]).astype(np.float32)
    y = (y + bias[None, :]).astype(np.float32)
    assert np.array_equal(outs[0], y)
    # and it is the dequantised product to float accuracy
    exact = ((A.astype(np.float64) - 128) @ B.astype(np.float64)) * 0.02 * 0.005 + bias
    assert np.allclose(outs[0], exact, rtol=1e-5, atol=1e-5)


def test_chain_dynamic_quant_per_token(zo):
    rng = np.random.default_rng(12)
    M, K, N = 6, 64, 16
    x = zo.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    p = _params(dt_src=capi.DT_BF16, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, dt_compute=capi.DT_S8,
                dynamic_quant=1,
                src_scale=capi.quant(None, capi.DT_F32, (M, 1)),
                wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, (1, N)))
    st, dst, acc, scales = zo.matmul_int8(x, B, p, M, N, K, want_acc=True, want_scales=True)
    assert st == capi.SUCCESS
    q, s = zo.quant_per_token(x, capi.DT_BF16)
    assert np.array_equal(s, scales)
    assert np.array_equal(acc, q.astype(np.int32) @ B.astype(np.int32))
    y = ((acc.astype(np.float32) * s[:, None]).astype(np.float32) * ws[None, :]).astype(np.float32)
    assert np.array_equal(dst, y)
    # close to the unquantised product (what the reference's dynamic-quant tests compare with)
    full = zo.bf16_to_f32(x).astype(np.float64) @ (B.astype(np.float64) * ws[None, :])
    assert np.abs(dst - full).max() < 0.02 * np.abs(full).max()


# ------------------------------------------------------- per-group scales
def _pg_params(ss, ws, M, N, G, dst=capi.DT_F32, **kw):
    return _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=dst,
                   src_scale=capi.quant(ss.ctypes.data, capi.DT_F32, (M, G)),
                   wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, (G, N)), **kw)


def test_per_group_closed_form_with_power_of_two_scales(zo):
    """All-ones operands: every group sum is K/G; with scales 2^-(..) every product and every partial sum
    is exact, so the result is the closed form sum_g (K/G) ss[m,g] ws[g,n].  The scale patterns differ
    along every axis, so a transposed or mis-strided scale index changes the answer."""
    M, K, N, G = 3, 64, 5, 4
    A = np.ones((M, K), dtype=np.int8)
    B = np.ones((K, N), dtype=np.int8)
    ss = np.array([[2.0 ** -(m + 2 * g) for g in range(G)] for m in range(M)], dtype=np.float32)
    ws = np.array([[2.0 ** -(3 * g + n) for n in range(N)] for g in range(G)], dtype=np.float32)
    st, dst, _, _ = zo.matmul_int8(A, B, _pg_params(ss, ws, M, N, G), M, N, K)
    assert st == capi.SUCCESS
    want = np.array([[sum((K // G) * float(ss[m, g]) * float(ws[g, n]) for g in range(G)) for n in range(N)]
                     for m in range(M)])
    assert np.array_equal(dst[:, :N].astype(np.float64), want)


def test_per_group_with_equal_power_of_two_group_scales_is_the_per_token_chain(zo):
    """ss[m,g] = s_m and ws[g,n] = w_n (powers of two, so nothing rounds): the group terms add up to
    float(acc) s_m w_n exactly, i.e. the per-token / per-channel result bit for bit."""
    rng = np.random.default_rng(21)
    M, K, N, G = 4, 96, 7, 3
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    sm = (2.0 ** -rng.integers(2, 8, M)).astype(np.float32)
    wn = (2.0 ** -rng.integers(4, 10, N)).astype(np.float32)
    ss = np.repeat(sm[:, None], G, axis=1).copy()
    ws = np.repeat(wn[None, :], G, axis=0).copy()
    bias = rng.standard_normal(N).astype(np.float32)
    st, got, _, _ = zo.matmul_int8(A, B, _pg_params(ss, ws, M, N, G, dt_bias=capi.DT_F32), M, N, K, bias=bias)
    assert st == capi.SUCCESS
    p = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, dt_bias=capi.DT_F32,
                src_scale=capi.quant(sm.ctypes.data, capi.DT_F32, (M, 1)),
                wei_scale=capi.quant(wn.ctypes.data, capi.DT_F32, (1, N)))
    st, want, _, _ = zo.matmul_int8(A, B, p, M, N, K, bias=bias)
    assert st == capi.SUCCESS
    assert np.array_equal(got, want)


@pytest.mark.parametrize("transB", [False, True])
def test_per_group_numpy_float32_brute_force(zo, transB):
    """Independent statement on a small random case: integer group sums by numpy, then one float32
    rounding per step in the reference's order (scale by ss, scale by ws, add in group order, bias)."""
    rng = np.random.default_rng(22)
    M, K, N, G = 5, 128, 9, 8
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    Bw = np.ascontiguousarray(B.T) if transB else B
    st, got, _, _ = zo.matmul_int8(A, Bw, _pg_params(ss, ws, M, N, G, dt_bias=capi.DT_F32), M, N, K, bias=bias,
                                   transB=transB)
    assert st == capi.SUCCESS
    gs = K // G
    gsum = np.einsum("mgk,gkn->mgn", A.reshape(M, G, gs).astype(np.int64), B.reshape(G, gs, N).astype(np.int64))
    y = np.zeros((M, N), dtype=np.float32)
    for g in range(G):
        t = (gsum[:, g, :].astype(np.float32) * ss[:, g][:, None]).astype(np.float32)
        t = (t * ws[g][None, :]).astype(np.float32)
        y = (y + t).astype(np.float32)
    y = (y + bias[None, :]).astype(np.float32)
    assert np.array_equal(got[:, :N], y)
    # a wrong group order would still pass the closed forms above; it fails here unless float addition commuted
    exact = np.einsum("mgn,mg,gn->mn", gsum.astype(np.float64), ss.astype(np.float64), ws.astype(np.float64)) + bias
    assert np.allclose(got[:, :N], exact, rtol=1e-5, atol=1e-5)


def test_per_group_rejects_what_the_reference_validator_rejects(zo):
    M, K, N, G = 2, 64, 4, 2
    A = np.ones((M, K), dtype=np.int8)
    B = np.ones((K, N), dtype=np.int8)
    ss = np.ones((M, G), dtype=np.float32)
    ws_bad = np.ones((1, N), dtype=np.float32)           # per-channel weight scale with a per-group source scale
    p = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32,
                src_scale=capi.quant(ss.ctypes.data, capi.DT_F32, (M, G)),
                wei_scale=capi.quant(ws_bad.ctypes.data, capi.DT_F32, (1, N)))
    st, _, _, _ = zo.matmul_int8(A, B, p, M, N, K)
    assert st == capi.FAILURE


def test_quant_per_group_closed_form_and_per_token_view(zo):
    """Every group of a row holds its own constant: scale = |c| / 127 and q = +-127 per group; and the whole
    thing equals the per-token rule on the [M*G, K/G] view of the rows."""
    M, K, G = 3, 96, 6
    gs = K // G
    c = np.array([[(-1.0) ** (m + g) * (0.25 + m + 3 * g) for g in range(G)] for m in range(M)], dtype=np.float32)
    x = np.repeat(c, gs, axis=1)
    q, s = zo.quant_per_group(x, capi.DT_F32, G)
    assert np.array_equal(s, (np.abs(c) / np.float32(127.0)).astype(np.float32))
    assert np.array_equal(q, np.repeat(np.where(c > 0, 127, -127).astype(np.int8), gs, axis=1))
    rng = np.random.default_rng(23)
    x = (rng.standard_normal((M, K)) * rng.uniform(0.1, 5.0, (M, K))).astype(np.float32)
    x[1, 40] = np.nan
    x[2, 3] = np.inf
    q, s = zo.quant_per_group(x, capi.DT_F32, G)
    qv, sv = zo.quant_per_token(x.reshape(M * G, gs), capi.DT_F32)
    assert np.array_equal(q.reshape(M * G, gs), qv) and np.array_equal(s.reshape(-1), sv)
    assert q[1, 40] == 0 and q[2, 3] == 0


def test_asymmetric_quant_closed_forms_and_properties(zo):
    """zo_quant_asym (u8 rows + s32 zero-points; reference: compute_asymmetric_scale_zp,
    per_token_avx512_f32_fma_kernel.cpp:89-116, quantization :636-680).  Rows of integers times a power of two make
    every step exact, so scale, zero-point and every code are known without evaluating the formula; the other checks
    are properties (dequantization within half a step, the codes of the row's extremes, the zero-point against exact
    fractions)."""
    from fractions import Fraction
    # rows k * s, k = lo .. lo + 255: range 255 s, scale = s exactly, zp = -lo, code = k - lo
    for lo, e in ((0, -3), (-100, -5), (-255, 0), (-17, -10)):
        s_ = np.float32(2.0 ** e)
        k = np.arange(lo, lo + 256, dtype=np.int64)
        rng = np.random.default_rng(lo + 1000)
        row = (rng.permutation(k).astype(np.float32) * s_)[None, :]
        q, sc, zp = zo.quant_asym(row, capi.DT_F32)
        assert sc[0, 0] == s_ and zp[0, 0] == -lo
        assert np.array_equal(q[0].astype(np.int64), np.rint(row[0] / s_).astype(np.int64) - lo)
    # a constant row: the range becomes [c, c + 1] (c = 0.25: c + 1 and the width are exact), scale = 1/255 as f32,
    # every code is 0 (c * 255 = 63.75 is no tie)
    row = np.full((1, 40), 0.25, dtype=np.float32)
    q, sc, zp = zo.quant_asym(row, capi.DT_F32)
    assert sc[0, 0] == np.float32(1.0) / np.float32(255.0) and np.all(q == 0)
    assert zp[0, 0] == -round(Fraction(0.25) / Fraction(float(sc[0, 0]))) == -64
    # no finite value at all: range [0, 1], zero-point 0, every code 0; non-finite elements of a mixed row give 0
    row = np.array([[np.nan, np.inf, -np.inf, np.nan]], dtype=np.float32)
    q, sc, zp = zo.quant_asym(row, capi.DT_F32)
    assert sc[0, 0] == np.float32(1.0) / np.float32(255.0) and zp[0, 0] == 0 and np.all(q == 0)
    row = np.array([[1.0, np.nan, 3.0, np.inf, 2.0, -np.inf]], dtype=np.float32)
    q, sc, zp = zo.quant_asym(row, capi.DT_F32)
    assert sc[0, 0] == np.float32(2.0) / np.float32(255.0)
    assert q[0, 0] == 0 and q[0, 2] == 255 and q[0, 1] == 0 and q[0, 3] == 0 and q[0, 5] == 0
    # random rows, bf16 and f32, per token and per group
    rng = np.random.default_rng(3)
    for src_dt, G in ((capi.DT_F32, 1), (capi.DT_BF16, 1), (capi.DT_F32, 4), (capi.DT_BF16, 8)):
        M, K = 13, 256
        xf = (rng.standard_normal((M, K)) * rng.uniform(0.01, 20, (M, 1)) + rng.uniform(-5, 5, (M, 1))).astype(np.float32)
        x = zo.f32_to_bf16(xf) if src_dt == capi.DT_BF16 else xf
        v = zo.bf16_to_f32(x) if src_dt == capi.DT_BF16 else xf
        q, sc, zp = zo.quant_asym(x, src_dt, G)
        vg = v.reshape(M, G, K // G)
        qg = q.reshape(M, G, K // G).astype(np.int64)
        lo, hi = vg.min(axis=2), vg.max(axis=2)
        assert np.array_equal(sc, ((hi - lo) / np.float32(255.0)).astype(np.float32))     # one f32 subtraction, one division
        for m in range(M):
            for g in range(G):
                exact = Fraction(float(-lo[m, g])) / Fraction(float(sc[m, g]))
                # (round half away from zero of the double quotient: within 1 of the exact quotient's rounding)
                assert abs(int(zp[m, g]) - round(exact)) <= 1
        back = (qg - zp[:, :, None]).astype(np.float64) * sc[:, :, None].astype(np.float64)
        assert np.all(np.abs(back - vg) <= 0.5001 * sc[:, :, None] + 1e-12)                  # within half a step
        at_lo = np.take_along_axis(qg, vg.argmin(axis=2)[:, :, None], axis=2)[:, :, 0]
        at_hi = np.take_along_axis(qg, vg.argmax(axis=2)[:, :, None], axis=2)[:, :, 0]
        assert np.all(at_lo <= 1) and np.all(at_hi >= 254)
        # per group == per token on the [M * G, K / G] view
        q2, sc2, zp2 = zo.quant_asym(np.ascontiguousarray(x.reshape(M * G, K // G)), src_dt, 1)
        assert np.array_equal(q2.reshape(M, K), q) and np.array_equal(sc2.reshape(M, G), sc) and np.array_equal(zp2.reshape(M, G), zp)


def test_chain_dynamic_quant_per_group(zo):
    rng = np.random.default_rng(24)
    M, K, N, G = 4, 128, 6, 4
    x = zo.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
    p = _params(dt_src=capi.DT_BF16, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, dt_compute=capi.DT_S8, dynamic_quant=1,
                src_scale=capi.quant(None, capi.DT_F32, (M, G)),
                wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, (G, N)))
    st, dst, _, scales = zo.matmul_int8(x, B, p, M, N, K, want_scales=True, n_scales=M * G)
    assert st == capi.SUCCESS
    q, s = zo.quant_per_group(x, capi.DT_BF16, G)
    assert np.array_equal(s.reshape(-1), scales)
    st, want, _, _ = zo.matmul_int8(q, B, _pg_params(s, ws, M, N, G), M, N, K)
    assert np.array_equal(dst, want)
    full = zo.bf16_to_f32(x).astype(np.float64) @ (B.astype(np.float64) * np.repeat(ws, K // G, axis=0))
    assert np.abs(dst - full).max() < 0.02 * np.abs(full).max()


# ------------------------------------------------------------- GGML Q8_0
def _q8_0_pack(rows, d16):
    """rows int8 [N,K], d16 float16 [N, K/32] -> the packed buffer: [N][K/32] blocks of {fp16 d, int8 qs[32]}."""
    N, K = rows.shape
    blk = np.zeros((N, K // 32, 34), dtype=np.uint8)
    blk[:, :, :2] = d16.view(np.uint16).reshape(N, K // 32, 1).view(np.uint8)
    blk[:, :, 2:] = rows.reshape(N, K // 32, 32).view(np.uint8)
    return blk.reshape(-1)


def test_f32_to_fp16_round_trip_numpy_and_the_reference_carry_case(zo):
    """Narrowing to half precision: every half value survives the round trip; 300 000 random f32 bit patterns and
    every tie / boundary neighbourhood agree with numpy's float16 (IEEE round to nearest even), except where the
    reference's own code departs from IEEE: magnitudes in [2^-14 - 2^-25, 2^-14) round up to the smallest normal
    half in IEEE and to a signed zero in the reference (it masks the carried mantissa) -- known answers there."""
    L = zo.lib()
    conv = np.frompyfunc(lambda v: L.zo_f32_to_f16(float(v)), 1, 1)
    halves = np.arange(65536, dtype=np.uint16)
    vals = halves.view(np.float16).astype(np.float32)
    ok = ~np.isnan(vals)
    got = conv(vals[ok]).astype(np.uint16)
    assert np.array_equal(got, halves[ok])
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2 ** 32, 300000, dtype=np.uint64).astype(np.uint32)
    # neighbourhoods of every half value's midpoints (ties) and of the range ends
    mid = ((halves[ok].astype(np.uint32) & 0x7fff) < 0x7bff)
    h32 = vals[ok][mid].view(np.uint32)
    h64 = h32.astype(np.int64)
    ties = np.concatenate([h64 + 0x1000 + d for d in (-1, 0, 1)] + [np.array([0x477fe000 + d for d in range(-3, 4)], dtype=np.int64)])
    x = np.concatenate([bits, ties.astype(np.uint32)]).view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = conv(x).astype(np.uint16)
    a = np.abs(x.astype(np.float64))
    carry = (a >= 2.0 ** -14 - 2.0 ** -25) & (a < 2.0 ** -14)
    tiny = a < 2.0 ** -126          # f32 subnormals: signed zero in both
    assert np.array_equal(got[~carry], want[~carry])
    assert np.all(got[tiny] == (x[tiny].view(np.uint32) >> 16 & 0x8000))
    # the carry case: IEEE gives the smallest normal, the reference a signed zero
    for v in (np.float32(2.0 ** -14 - 2.0 ** -25), np.float32(2.0 ** -14 - 2.0 ** -26), np.float32(-(2.0 ** -14) * (1 - 2.0 ** -13))):
        assert np.float16(v).view(np.uint16) & 0x7fff == 0x0400
        assert L.zo_f32_to_f16(float(v)) == (0x8000 if v < 0 else 0)
    # NaN: quiet, sign and top mantissa bits kept
    nan = np.array([0x7fa00000], dtype=np.uint32).view(np.float32)[0]
    assert L.zo_f32_to_f16(float(nan)) & 0x7e00 == 0x7e00


def test_fp16_conversion_against_numpy_for_every_half_value(zo):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([zo.lib().zo_fp16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_ggml_q8_0_unpack_layout_and_bf16_scales(zo):
    rng = np.random.default_rng(31)
    N, K = 7, 96
    rows = rng.integers(-128, 128, (N, K), dtype=np.int8)
    d16 = rng.uniform(1e-4, 0.05, (N, K // 32)).astype(np.float16)
    d16[0, 0] = np.float16(6e-8)               # an fp16 subnormal
    got_rows, got_scales = zo.ggml_q8_0_unpack(_q8_0_pack(rows, d16), N, K)
    assert np.array_equal(got_rows, rows)
    want = torch.from_numpy(d16.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got_scales, want.T)  # scales[g, n] = bf16(f32(d[n, g]))


def test_ggml_matmul_is_the_per_group_matmul_on_the_unpacked_weights(zo):
    rng = np.random.default_rng(32)
    M, K, N = 5, 128, 9
    G = K // 32
    A = rng.integers(-128, 128, (M, K), dtype=np.int8)
    rows = rng.integers(-127, 128, (N, K), dtype=np.int8)
    d16 = rng.uniform(1e-3, 0.02, (N, G)).astype(np.float16)
    ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
    packed = _q8_0_pack(rows, d16)
    p = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, pack_format_b=1,
                src_scale=capi.quant(ss.ctypes.data, capi.DT_F32, (M, G)))
    st, got, _, _ = zo.matmul_int8(A, packed, p, M, N, K, transB=True, ldb=K)
    assert st == capi.SUCCESS
    ws = zo.ggml_q8_0_unpack(packed, N, K)[1]
    p2 = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32,
                 src_scale=capi.quant(ss.ctypes.data, capi.DT_F32, (M, G)),
                 wei_scale=capi.quant(ws.ctypes.data, capi.DT_BF16, (G, N)))
    st, want, _, _ = zo.matmul_int8(A, rows, p2, M, N, K, transB=True, ldb=K)
    assert st == capi.SUCCESS
    assert np.array_equal(got, want)
    # and it is the dequantised product to the scales' accuracy
    wf = zo.bf16_to_f32(ws)                                             # [G, N]
    full = np.einsum("mgk,ngk,mg,gn->mn", A.reshape(M, G, 32).astype(np.float64), rows.reshape(N, G, 32).astype(np.float64),
                     ss.astype(np.float64), wf.astype(np.float64))
    assert np.allclose(got, full, rtol=1e-5, atol=1e-5)
    # transB = false is refused (the packed layout is N x K)
    st, _, _, _ = zo.matmul_int8(A, packed, p, M, N, K, transB=False, ldb=K)
    assert st == capi.FAILURE


# ------------------------------------------------------------- W4A8 (s4 weights)
def _s4_pack(codes, ld):
    """codes int8 [R, C] in -8..7 -> packed nibbles of a [R, ld] matrix (pad columns hold 5): element i of the
    flattened matrix is the low nibble of byte i // 2 when i is even, else the high nibble."""
    R, C = codes.shape
    full = np.full((R, ld), 5, dtype=np.int64)
    full[:, :C] = codes
    flat = full.reshape(-1) & 15
    if flat.size % 2:
        flat = np.append(flat, 0)
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)


def test_s4_widening_known_answers_and_numpy_restatement(zo):
    # every code in both nibble positions: byte (hi << 4 | lo) -> [lo, hi], sign-extended from bit 3
    for lo in range(16):
        for hi in range(16):
            got = zo.s4_to_s8(np.array([(hi << 4) | lo], dtype=np.uint8), 1, 2)
            assert got.tolist() == [[lo - 16 if lo >= 8 else lo, hi - 16 if hi >= 8 else hi]]
    assert zo.s4_to_s8(np.array([0x87, 0xF0, 0x1E], dtype=np.uint8), 2, 3).tolist() == [[7, -8, 0], [-1, -2, 1]]
    # random matrices, both orientations, padded (odd) leading dimension: the layout by construction
    rng = np.random.default_rng(41)
    for K, N, pad in [(8, 6, 0), (12, 5, 3), (7, 9, 1)]:
        w = rng.integers(-8, 8, (K, N), dtype=np.int8)
        assert np.array_equal(zo.s4_to_s8(_s4_pack(w, N + pad), K, N, ldb=N + pad), w)
        assert np.array_equal(zo.s4_to_s8(_s4_pack(w.T.copy(), K + pad), K, N, ldb=K + pad, transposed=True), w)


@pytest.mark.parametrize("scale_dims", ["tensor", "token", "group"])
@pytest.mark.parametrize("transB", [False, True])
def test_w4a8_is_the_per_group_matmul_on_the_widened_weights(zo, scale_dims, transB):
    rng = np.random.default_rng(42)
    M, K, N, G = 5, 128, 10, 4
    x = zo.f32_to_bf16((rng.standard_normal((M, K)) * 3).astype(np.float32))
    w = rng.integers(-8, 8, (K, N), dtype=np.int8)
    packed = _s4_pack(w.T.copy(), K) if transB else _s4_pack(w, N)
    ws = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
    dims = {"tensor": (1, 1), "token": (M, 1), "group": (M, G)}[scale_dims]
    p = _params(dt_src=capi.DT_BF16, dt_wei=capi.DT_S4, dt_dst=capi.DT_BF16, dt_compute=capi.DT_S8, dynamic_quant=1,
                src_scale=capi.quant(None, capi.DT_F32, dims),
                wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, (G, N)))
    st, got, _, scales = zo.matmul_int8(x, packed, p, M, N, K, transB=transB, ldb=K if transB else N,
                                        want_scales=True, n_scales=M * G)
    assert st == capi.SUCCESS
    # the same source quantization as the s8-weight path, its scales repeated over the groups, then the per-group GEMM
    if scale_dims == "group":
        q, s = zo.quant_per_group(x, capi.DT_BF16, G)
    elif scale_dims == "token":
        q, s1 = zo.quant_per_token(x, capi.DT_BF16)
        s = np.repeat(s1.reshape(M, 1), G, axis=1)
    else:
        xf = zo.bf16_to_f32(x)
        s0 = np.float32(np.abs(xf).max()) / np.float32(127.0)
        q = np.rint(xf / s0).astype(np.int8)
        s = np.full((M, G), s0, dtype=np.float32)
    s = np.ascontiguousarray(s, dtype=np.float32)
    p2 = _params(dt_src=capi.DT_S8, dt_wei=capi.DT_S8, dt_dst=capi.DT_BF16,
                 src_scale=capi.quant(s.ctypes.data, capi.DT_F32, (M, G)),
                 wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, (G, N)))
    st, want, _, _ = zo.matmul_int8(q, w, p2, M, N, K)
    assert st == capi.SUCCESS
    assert np.array_equal(got, want)
    # and it is the dequantised product to the quantization's accuracy
    full = zo.bf16_to_f32(x).astype(np.float64) @ (w.astype(np.float64) * np.repeat(ws, K // G, axis=0))
    assert np.abs(zo.bf16_to_f32(got) - full).max() < 0.03 * np.abs(full).max()


def test_w4a8_rejections_follow_the_reference_validator(zo):
    M, K, N, G = 4, 64, 8, 2
    x = np.zeros((M, K), dtype=np.uint16)
    packed = np.zeros(K * N // 2, dtype=np.uint8)
    ws = np.ones((G, N), dtype=np.float32)

    def call(src=capi.DT_BF16, dst=capi.DT_BF16, compute=capi.DT_S8, dyn=1, sdims=(M, 1), wdims=(G, N), K_=K):
        p = _params(dt_src=src, dt_wei=capi.DT_S4, dt_dst=dst, dt_compute=compute, dynamic_quant=dyn,
                    src_scale=capi.quant(None, capi.DT_F32, sdims),
                    wei_scale=capi.quant(ws.ctypes.data, capi.DT_F32, wdims))
        return zo.matmul_int8(x, packed, p, M, N, K_)[0]

    assert call() == capi.SUCCESS
    assert call(src=capi.DT_S8) == capi.FAILURE                 # pre-quantized sources are not W4A8
    assert call(src=capi.DT_F32) == capi.FAILURE
    assert call(dst=capi.DT_F32) == capi.FAILURE
    assert call(compute=capi.DT_BF16) == capi.FAILURE
    assert call(dyn=0) == capi.UNIMPLEMENTED                    # weight-only quantization: another path
    assert call(sdims=(M, 3)) == capi.FAILURE
    assert call(wdims=(G, N - 1)) == capi.FAILURE
    assert call(wdims=(3, N)) == capi.FAILURE                   # K not divisible by G
    assert call(wdims=(32, N)) == capi.FAILURE                  # groups of 2: not a multiple of 4


# ------------------------------------------------------------- post-ops
def test_eltwise_against_libm_double(zo):
    xs = np.concatenate([np.linspace(-12, 12, 4001), [0.0, -0.0, 1e-6, -1e-6, 30.0, -30.0]]).astype(np.float32)
    def ulp(a, b):
        a = np.float32(a); b = np.float32(b)
        sp = np.spacing(np.abs(b)) if b != 0 else np.float32(1e-45)
        return abs(float(a) - float(b)) / float(sp)
    silu = zo.eltwise(capi.PO_SWISH, xs)
    gelu = zo.eltwise(capi.PO_GELU_TANH, xs)
    gerf = zo.eltwise(capi.PO_GELU_ERF, xs)
    sig = zo.eltwise(capi.PO_SIGMOID, xs)
    for i, x in enumerate(xs.astype(np.float64)):
        assert ulp(silu[i], x / (1 + math.exp(-x))) <= 2
        assert ulp(sig[i], 1 / (1 + math.exp(-x))) <= 2
        t = math.tanh(math.sqrt(2 / math.pi) * x * (1 + 0.044715 * x * x))
        want = 0.5 * x * (1 + t)
        # near the negative tail 1+tanh cancels; bound the absolute error there instead
        assert ulp(gelu[i], want) <= 4 or abs(float(gelu[i]) - want) < 2e-7 * max(1.0, abs(x))
        want_e = 0.5 * x * (1 + math.erf(x / math.sqrt(2)))
        assert ulp(gerf[i], want_e) <= 4 or abs(float(gerf[i]) - want_e) < 2e-7 * max(1.0, abs(x))
    assert np.array_equal(zo.eltwise(capi.PO_RELU, xs), np.maximum(xs, 0))
    assert np.array_equal(zo.eltwise(capi.PO_CLIP, xs, -1.0, 2.0), np.clip(xs, -1.0, 2.0))
    lr = zo.eltwise(capi.PO_LEAKY_RELU, xs)
    assert np.array_equal(lr, np.where(xs > 0, xs, np.float32(0.01) * xs))


def test_remaining_eltwise_types_closed_forms_and_libm(zo):
    """elu / square / abs / sqrt / exp / log (matmul_ref_kernel.cpp:694-751): exact where the mathematics fixes
    the float (squares and roots of small integers, |x|, elu above zero, exp(0), log(1)), libm in double elsewhere."""
    ints = np.arange(-20, 21, dtype=np.float32)
    assert np.array_equal(zo.eltwise(capi.PO_SQUARE, ints), ints * ints)
    assert np.array_equal(zo.eltwise(capi.PO_ABS, ints), np.abs(ints))
    assert np.signbit(zo.eltwise(capi.PO_ABS, np.array([-0.0], dtype=np.float32)))[0] == False   # noqa: E712  (-(-0) = +0)
    sq = np.arange(0, 40, dtype=np.float32)
    assert np.array_equal(zo.eltwise(capi.PO_SQRT, sq * sq), sq)
    assert np.isnan(zo.eltwise(capi.PO_SQRT, np.array([-1.0], dtype=np.float32)))[0]
    assert zo.eltwise(capi.PO_EXP, np.array([0.0], dtype=np.float32))[0] == 1.0
    assert zo.eltwise(capi.PO_LOG, np.array([1.0], dtype=np.float32))[0] == 0.0
    pos = np.linspace(0.001, 9, 200).astype(np.float32)
    assert np.array_equal(zo.eltwise(capi.PO_ELU, pos, 1.7), pos)                  # identity above zero
    xs = np.linspace(-15, 15, 2001).astype(np.float32)
    ex = zo.eltwise(capi.PO_EXP, xs)
    el = zo.eltwise(capi.PO_ELU, xs, 1.7)
    lg = zo.eltwise(capi.PO_LOG, np.abs(xs) + np.float32(1e-3))
    for i, x in enumerate(xs.astype(np.float64)):
        assert abs(float(ex[i]) - math.exp(x)) <= 2 * float(np.spacing(np.float32(math.exp(x))))
        if x <= 0:
            # alpha * (float(e^x) - 1) in double: the float rounding of e^x is the only error before the final rounding
            want = 1.7 * (math.exp(x) - 1.0)
            assert abs(float(el[i]) - want) <= 1.7 * 6e-8 + abs(want) * 1.2e-7
        v = float(np.abs(xs[i]) + np.float32(1e-3))
        assert abs(float(lg[i]) - math.log(v)) <= 2 * float(np.spacing(np.float32(abs(math.log(v))))) + 1e-45


# ---------------------------------------------------- gated act / reduce
def test_mish_against_libm_double_and_limits(zo):
    """mish_fwd (matmul_ref_kernel.cpp:755-760) = x tanh(ln(1 + e^x)): libm in double on a grid, the limits the
    mathematics fixes (mish(0) = 0, mish(x) -> x for large x, -> 0 from below for very negative x) and the identity
    tanh(softplus(x)) = ((1 + e^x)^2 - 1) / ((1 + e^x)^2 + 1), which a dropped max(x, 0) or a wrong sign of |x| fails."""
    xs = np.concatenate([np.linspace(-30, 30, 1201), [0.0, -0.0, 1e-6, -1e-6, 88.0, -88.0, 20.0]]).astype(np.float32)
    got = zo.eltwise(capi.PO_MISH, xs)
    for i, x in enumerate(xs.astype(np.float64)):
        want = x * math.tanh(math.log1p(math.exp(x))) if x < 30 else x
        n = (1.0 + math.exp(x)) ** 2 if x < 30 else float("inf")
        alt = x * ((n - 1.0) / (n + 1.0)) if n != float("inf") else x
        assert abs(want - alt) <= 1e-12 * max(1.0, abs(want)) + 1e-300
        assert abs(float(got[i]) - want) <= 4 * float(np.spacing(np.float32(abs(want)))) + 1e-37, (x, got[i], want)
    assert float(zo.eltwise(capi.PO_MISH, np.array([0.0], dtype=np.float32))[0]) == 0.0
    assert float(zo.eltwise(capi.PO_MISH, np.array([50.0], dtype=np.float32))[0]) == 50.0
    tail = float(zo.eltwise(capi.PO_MISH, np.array([-25.0], dtype=np.float32))[0])
    assert -1e-9 < tail < 0.0


def test_gated_act_brute_force(zo):
    rng = np.random.default_rng(13)
    M, dim = 5, 24
    buf = zo.f32_to_bf16(rng.standard_normal((M, 2 * dim)).astype(np.float32) * 3)
    f = zo.bf16_to_f32(buf).astype(np.float64)
    out = zo.gated_act(capi.ACT_SILU_AND_MUL, buf.copy(), capi.DT_BF16)
    g, u = f[:, :dim], f[:, dim:]
    want = zo.f32_to_bf16((g / (1 + np.exp(-g)) * u).astype(np.float32))
    got = out[:, :dim]
    d = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 0.02       # double vs float evaluation: rare 1-ulp flips
    assert np.array_equal(out[:, dim:], buf[:, dim:])    # the up half is left untouched
    f32 = rng.standard_normal((M, 2 * dim)).astype(np.float32)
    o32 = zo.gated_act(capi.ACT_SILU_AND_MUL, f32.copy(), capi.DT_F32)
    w32 = f32[:, :dim].astype(np.float64)
    assert np.allclose(o32[:, :dim], w32 / (1 + np.exp(-w32)) * f32[:, dim:], rtol=3e-7, atol=1e-7)


def test_moe_reduce_closed_form_and_brute_force(zo):
    # closed form of the reference example (examples/lowoha_group_matmul_example.cpp:320):
    # all-ones src, expert e weight (e+1), K wide, routing weights 0.5/0.5
    K, D = 64, 8
    e0, e1 = 2, 5
    rows = [np.full(D, K * (e0 + 1), dtype=np.float32), np.full(D, K * (e1 + 1), dtype=np.float32)]
    out = zo.moe_reduce(rows, np.array([[0.5, 0.5]], dtype=np.float32), capi.DT_F32, D)
    assert np.all(out == 0.5 * K * (e0 + 1) + 0.5 * K * (e1 + 1))
    rng = np.random.default_rng(14)
    T, topk, D = 6, 3, 20
    rows = [zo.f32_to_bf16(rng.standard_normal(D).astype(np.float32)) for _ in range(T * topk)]
    w = rng.uniform(0, 1, (T, topk)).astype(np.float32)
    out = zo.moe_reduce(rows, w, capi.DT_BF16, D)
    for t in range(T):
        acc = np.zeros(D, dtype=np.float64)
        for k in range(topk):
            acc += float(w[t, k]) * zo.bf16_to_f32(rows[t * topk + k]).astype(np.float64)
        want = zo.f32_to_bf16(acc.astype(np.float32), ctor=False)
        d = np.abs(out[t].astype(np.int32) - want.astype(np.int32))
        assert d.max() <= 1
    ones = zo.moe_reduce(rows, w, capi.DT_BF16, D, skip_weighted=True)
    t0 = sum(zo.bf16_to_f32(rows[k]).astype(np.float64) for k in range(topk))
    assert np.abs(zo.bf16_to_f32(ones[0]) - t0).max() < 0.05


# ------------------------------------------------- weight-only quantization
def _nib_pack(flat):
    flat = np.asarray(flat, dtype=np.int64) & 15
    if flat.size % 2:
        flat = np.append(flat, 0)
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)


def test_woq_nibble_order_sign_extension_and_orientation(zo):
    # byte 0x21 holds index 0 -> 1 (low nibble) and index 1 -> 2; 0xF8 holds 8 -> -8 (s4) / 8 (u4) and 15 -> -1 / 15
    packed = np.array([0x21, 0xF8], dtype=np.uint8)
    one = np.ones(1, dtype=np.float32)
    got = zo.bf16_to_f32(zo.woq_dequant(packed, 2, 2, capi.DT_S4, one, capi.DT_F32))
    assert got.tolist() == [[1.0, 2.0], [-8.0, -1.0]]
    got = zo.bf16_to_f32(zo.woq_dequant(packed, 2, 2, capi.DT_U4, one, capi.DT_F32))
    assert got.tolist() == [[1.0, 2.0], [8.0, 15.0]]
    # transposed: element (row, col) sits at nibble col * ldb + row
    got = zo.bf16_to_f32(zo.woq_dequant(packed, 2, 2, capi.DT_S4, one, capi.DT_F32, transposed=True))
    assert got.tolist() == [[1.0, -8.0], [2.0, -1.0]]
    # a leading dimension of 3 nibbles: rows start at nibbles 0 and 3
    packed = _nib_pack([1, 2, 7, 3, 4, 7])
    got = zo.bf16_to_f32(zo.woq_dequant(packed, 2, 2, capi.DT_S4, one, capi.DT_F32, ldb=3))
    assert got.tolist() == [[1.0, 2.0], [3.0, 4.0]]


def test_woq_dequantization_formulas_where_every_step_is_exact(zo):
    # scales and zero-points that keep every operation exact: the two formulas give different, known values
    codes = np.arange(16).reshape(16, 1)
    packed = _nib_pack(np.repeat(codes, 2, axis=1).reshape(-1))     # [16, 2], both columns the same code
    scale = np.array([0.25], dtype=np.float32)
    zp8 = np.array([3], dtype=np.int8)
    zpf = zo.f32_to_bf16(np.array([0.5], dtype=np.float32))
    u = np.arange(16, dtype=np.float64)
    s = np.where(u >= 8, u - 16, u)
    col = lambda a: zo.bf16_to_f32(a)[:, 0].astype(np.float64)
    assert np.array_equal(col(zo.woq_dequant(packed, 16, 2, capi.DT_S4, scale, capi.DT_F32)), s * 0.25)
    assert np.array_equal(col(zo.woq_dequant(packed, 16, 2, capi.DT_S4, scale, capi.DT_F32, zp8, capi.DT_S8)), (s - 3) * 0.25)
    assert np.array_equal(col(zo.woq_dequant(packed, 16, 2, capi.DT_U4, scale, capi.DT_F32, zp8, capi.DT_S8)), (u - 3) * 0.25)
    # u4 codes with a bf16 zero-point: the midpoint 8 comes off, the zero-point is added after the scale
    assert np.array_equal(col(zo.woq_dequant(packed, 16, 2, capi.DT_U4, scale, capi.DT_F32, zpf, capi.DT_BF16)), (u - 8) * 0.25 + 0.5)
    # s4 codes with a bf16 zero-point stay on the first formula
    assert np.array_equal(col(zo.woq_dequant(packed, 16, 2, capi.DT_S4, scale, capi.DT_F32, zpf, capi.DT_BF16)), (s - 0.5) * 0.25)


def test_woq_dequantization_granularities_and_rounding_against_torch(zo):
    # bf16-valued scales: (code - zp) * scale has at most 14 significant bits, so the f32 product is exact and the
    # one rounding left is the bf16 one, which torch does from the exact double product
    rng = np.random.default_rng(77)
    K, N, G = 48, 10, 3
    codes = rng.integers(-8, 8, (K, N))
    packed = _nib_pack(codes.reshape(-1))
    for dims in ((1, 1), (1, N), (G, N)):
        sc_bits = zo.f32_to_bf16(rng.uniform(0.01, 0.3, dims).astype(np.float32))
        sc = zo.bf16_to_f32(sc_bits).astype(np.float64)
        zp = rng.integers(-4, 5, dims).astype(np.int8)
        rows = np.arange(K) // (K // dims[0]) if dims[0] > 1 else np.zeros(K, dtype=np.int64)
        sc_full = np.broadcast_to(sc, (dims[0], N))[rows]
        zp_full = np.broadcast_to(zp, (dims[0], N))[rows].astype(np.float64)
        exact = (codes - zp_full) * sc_full
        want = torch.from_numpy(exact).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        got = zo.woq_dequant(packed, K, N, capi.DT_S4, sc_bits.reshape(-1), capi.DT_BF16, zp.reshape(-1), capi.DT_S8)
        assert np.array_equal(got, want), dims


def test_woq_product_is_the_double_precision_product_of_the_bf16_operands(zo):
    rng = np.random.default_rng(78)
    M, K, N, G = 6, 96, 20, 4
    codes = rng.integers(0, 16, (K, N))
    packed = _nib_pack(codes.reshape(-1))
    sc = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
    zp = zo.f32_to_bf16(rng.uniform(-0.2, 0.2, (G, N)).astype(np.float32))
    x = zo.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    bias = rng.standard_normal(N).astype(np.float32)
    c0 = rng.standard_normal((M, N)).astype(np.float32)
    p = _params(dt_src=capi.DT_BF16, dt_wei=capi.DT_U4, dt_dst=capi.DT_F32, dt_bias=capi.DT_F32,
                wei_scale=capi.quant(sc.ctypes.data, capi.DT_F32, (G, N)),
                wei_zp=capi.quant(zp.ctypes.data, capi.DT_BF16, (G, N)))
    st, got = zo.matmul_woq(x, packed, p, M, N, K, bias=bias, dst=c0.copy(), alpha=0.5, beta=2.0)
    assert st == capi.SUCCESS
    wb = zo.bf16_to_f32(zo.woq_dequant(packed, K, N, capi.DT_U4, sc.reshape(-1), capi.DT_F32, zp.reshape(-1), capi.DT_BF16))
    xf = zo.bf16_to_f32(x).astype(np.float64)
    want = 0.5 * (xf @ wb.astype(np.float64)) + 2.0 * c0 + bias
    mag = 0.5 * (np.abs(xf) @ np.abs(wb.astype(np.float64))) + 2.0 * np.abs(c0) + np.abs(bias)
    assert (np.abs(got - want) <= 2e-6 * mag).all()
    # integer-valued operands and a power-of-two scale: every partial sum is exact in f32, any order gives this
    xi = zo.f32_to_bf16(rng.integers(-4, 5, (M, K)).astype(np.float32))
    half = np.array([0.5], dtype=np.float32)
    z8 = np.array([7], dtype=np.int8)
    p = _params(dt_src=capi.DT_BF16, dt_wei=capi.DT_U4, dt_dst=capi.DT_F32,
                wei_scale=capi.quant(half.ctypes.data, capi.DT_F32, (1, 1)), wei_zp=capi.quant(z8.ctypes.data, capi.DT_S8, (1, 1)))
    st, got = zo.matmul_woq(xi, packed, p, M, N, K)
    assert st == capi.SUCCESS
    assert np.array_equal(got, zo.bf16_to_f32(xi).astype(np.float64) @ ((codes - 7) * 0.5))


def test_woq_rejections_follow_the_reference_validator(zo):
    M, K, N, G = 2, 32, 4, 2
    x = np.zeros((M, K), dtype=np.uint16)
    packed = np.zeros(K * N // 2, dtype=np.uint8)
    ws = np.ones((G, N), dtype=np.float32)
    z8 = np.zeros((G, N), dtype=np.int8)

    def call(wei=capi.DT_S4, dst=capi.DT_BF16, const=True, zp=None, zp_dt=capi.DT_S8, extra=None, scale=True, dyn=0):
        kw = dict(dt_src=capi.DT_BF16, dt_wei=wei, dt_dst=dst, dynamic_quant=dyn)
        if scale:
            kw["wei_scale"] = capi.quant(ws.ctypes.data, capi.DT_F32, (G, N))
        if zp is not None:
            kw["wei_zp"] = capi.quant(zp.ctypes.data, zp_dt, (G, N))
        if extra:
            kw[extra] = capi.quant(ws.ctypes.data, capi.DT_F32, (1, 1))
        return zo.matmul_woq(x, packed, _params(**kw), M, N, K, is_weights_const=const)[0]

    assert call() == capi.SUCCESS
    assert call(wei=capi.DT_U4, zp=z8) == capi.SUCCESS
    assert call(const=False) == capi.FAILURE
    assert call(extra="src_scale") == capi.FAILURE
    assert call(extra="dst_scale") == capi.FAILURE
    assert call(wei=capi.DT_U4) == capi.FAILURE                      # u4 without a zero-point
    assert call(wei=capi.DT_U4, zp=z8, zp_dt=capi.DT_S32) == capi.FAILURE
    assert call(dst=capi.DT_F16) == capi.FAILURE
    assert call(scale=False) == capi.FAILURE
    assert call(dyn=1) == capi.UNIMPLEMENTED                         # W4A8: zo_matmul_int8's


# ------------------------------------------------- dynamic quantization to u8 (per tensor)
def test_dynamic_u8_per_tensor_closed_forms(zo):
    # values k / 4 for k = -100 .. 155: min -25, max 38.75, scale = 63.75 / 255 = 0.25 exactly, zp = round(25 / 0.25) = 100,
    # codes k + 100; the product with all-ones weights and unit weight scale is then a known integer
    M, K, N = 2, 128, 3
    k = np.arange(-100, 156, dtype=np.float32).reshape(M, K)
    x = k / 4
    w = np.ones((K, N), dtype=np.int8)
    p = _params(dt_src=capi.DT_F32, dt_wei=capi.DT_S8, dt_dst=capi.DT_S32, dt_compute=capi.DT_U8, dynamic_quant=1,
                src_scale=capi.quant(None, capi.DT_F32, (1, 1)), src_zp=capi.quant(None, capi.DT_S32, (1, 1)))
    zp = np.zeros(1, dtype=np.int32)
    st, dst, acc, scales = zo.matmul_int8(x, w, p, M, N, K, want_acc=True, want_scales=True, zp_out=zp)
    assert st == capi.SUCCESS
    assert scales[0] == np.float32(0.25) and zp[0] == 100
    assert np.array_equal(acc, np.repeat((k + 100).sum(axis=1).astype(np.int32)[:, None], N, axis=1))   # u8 codes k + 100
    # minus zp * colsum, times the source scale (the chain applies it whatever the destination type)
    assert np.array_equal(dst[:, :N], np.repeat((k.sum(axis=1) / 4).astype(np.int32)[:, None], N, axis=1))
    # a constant tensor: range [c, c + 1], scale 1 / 255, zp = round(-c * 255); no finite value: [0, 0] -> [0, 1], zp 0
    # (2.5 * 255 is the tie 637.5 for the real 1 / 255; the f32 scale lies above 1 / 255, so the quotient lies below it)
    for c, want_zp in ((2.0, -510), (-1.0, 255), (0.0, 0), (2.5, -637)):
        xc = np.full((M, K), c, dtype=np.float32)
        st, _, _, scales = zo.matmul_int8(xc, w, p, M, N, K, want_scales=True, zp_out=zp)
        assert st == capi.SUCCESS and scales[0] == np.float32(1.0) / np.float32(255.0)
        assert zp[0] == want_zp, (c, zp[0])
    xn = np.full((M, K), np.nan, dtype=np.float32)
    st, dst, acc, scales = zo.matmul_int8(xn, w, p, M, N, K, want_acc=True, want_scales=True, zp_out=zp)
    assert st == capi.SUCCESS and zp[0] == 0 and not acc.any()
    # per-token dims: the GEMM has one zero-point to read
    p2 = _params(dt_src=capi.DT_F32, dt_wei=capi.DT_S8, dt_dst=capi.DT_S32, dt_compute=capi.DT_U8, dynamic_quant=1,
                 src_scale=capi.quant(None, capi.DT_F32, (M, 1)), src_zp=capi.quant(None, capi.DT_S32, (M, 1)))
    assert zo.matmul_int8(x, w, p2, M, N, K)[0] == capi.UNIMPLEMENTED


def test_dynamic_u8_dequantizes_to_the_source_within_half_a_step(zo):
    rng = np.random.default_rng(5)
    M, K = 6, 64
    x = (rng.standard_normal((M, K)) * 2 + 1).astype(np.float32)
    eye = np.eye(K, dtype=np.int8)
    one = np.ones(1, dtype=np.float32)
    p = _params(dt_src=capi.DT_F32, dt_wei=capi.DT_S8, dt_dst=capi.DT_F32, dt_compute=capi.DT_U8, dynamic_quant=1,
                src_scale=capi.quant(None, capi.DT_F32, (1, 1)), src_zp=capi.quant(None, capi.DT_S32, (1, 1)),
                wei_scale=capi.quant(one.ctypes.data, capi.DT_F32, (1,)))
    zp = np.zeros(1, dtype=np.int32)
    st, dst, _, scales = zo.matmul_int8(x, eye, p, M, K, K, want_scales=True, zp_out=zp)
    assert st == capi.SUCCESS
    # identity weights: dst = (q - zp) * scale, the dequantized source
    assert np.abs(dst[:, :K] - x).max() <= 0.5 * scales[0] * (1 + 1e-5) + 1e-6
    assert scales[0] == (x.max() - x.min()) / np.float32(255.0)


def test_dynamic_u8_with_a_bf16_scale_buffer_quantizes_with_the_narrowed_scale(zo):
    """Range [0, 76.5]: scale 76.5 / 255 = 0.3 in f32, which a bf16 buffer stores as 0.30078125; the reference stores the
    parameters and then quantizes with what the buffer reads back as (lowoha_reorder.cpp:186-205), so 76.5 becomes
    code 254 (255 with the f32 scale) and 60 becomes 199 (200); the zero-point comes from the scale as computed."""
    K = 64
    x = np.zeros((1, K), dtype=np.float32)
    x[0, :5] = [0.0, 30.0, 45.0, 60.0, 76.5]
    eye = np.eye(K, dtype=np.int8)
    zp = np.zeros(1, dtype=np.int32)
    codes = {}
    for sdt in (capi.DT_F32, capi.DT_BF16):
        p = _params(dt_src=capi.DT_F32, dt_wei=capi.DT_S8, dt_dst=capi.DT_S32, dt_compute=capi.DT_U8, dynamic_quant=1,
                    src_scale=capi.quant(None, sdt, (1, 1)), src_zp=capi.quant(None, capi.DT_S32, (1, 1)))
        st, _, acc, scales = zo.matmul_int8(x, eye, p, 1, K, K, want_acc=True, want_scales=True, zp_out=zp)
        assert st == capi.SUCCESS and zp[0] == 0
        codes[sdt] = (acc[0, :5].tolist(), float(scales[0]))
    assert codes[capi.DT_F32] == ([0, 100, 150, 200, 255], float(np.float32(76.5) / np.float32(255.0)))
    assert codes[capi.DT_BF16] == ([0, 100, 150, 199, 254], 0.30078125)
