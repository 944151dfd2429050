"""Golden cases of the LowOHA int8 path at reduced size: one per BASELINE configuration plus the adjacent formats
(per-group scales, GGML Q8_0, W4A8).  Every case is a seed and a shape; the inputs are regenerated from the seed
(numpy's PCG64 streams are stable across versions), run(case, backend) pushes them through either the CPU oracle or the
C ABI on the GPU with the same parameter structs, and returns named outputs.  make_golden.py stores the oracle's
outputs (SHA-256 for bit-exact outputs, the bf16 bit patterns for outputs compared within one unit in the last
place); tests/test_golden.py checks both backends against the stored values.

The reference holds no golden vectors for this path (its own tests are differential: AOCL against its scalar kernel,
gtests/test_matmul.cpp:975-1549, gtests/group_matmul/test_fused_moe.cpp:2491), so the fixtures come from this
repository's oracle, which is pinned separately (tests/test_oracle_pins.py)."""
import hashlib

import numpy as np

from zendnn_amd import capi, lowoha
from tests import gpu_helpers as H
from tests import moe_helpers as MH

EXACT, BF16_ULP = "exact", "bf16_ulp"

# name -> (kind, seed, dims ...)
CASES = {
    "cfg1_u8s8_zp128": ("u8", 0x5EED0001, 32, 256, 128),
    "cfg2_decode_M1": ("decode", 0x5EED0002, 1, 512, 320),
    "cfg2_decode_M4": ("decode", 0x5EED0002, 4, 512, 320),
    "cfg2_decode_M16": ("decode", 0x5EED0002, 16, 512, 320),
    "cfg3_prefill": ("prefill", 0x5EED0003, 160, 512, 256),
    "cfg4_moe_top2": ("moe", 0x5EED0004, 48, 256, 128, 4, 2, False),
    "cfg5_moe_top6_skewed": ("moe", 0x5EED0005, 96, 128, 96, 16, 6, True),
    "per_group_scales": ("per_group", 0x5EED0006, 9, 512, 72, 8),
    "ggml_q8_0": ("ggml", 0x5EED0007, 6, 256, 40),
    "w4a8": ("w4a8", 0x5EED0008, 12, 1024, 56, 8),
    "weight_only_4bit": ("woq", 0x5EED0009, 192, 40, 3),
}


def sha(a):
    a = np.ascontiguousarray(a)
    return hashlib.sha256(a.tobytes()).hexdigest()


class _Backend:
    """matmul_direct on host arrays through the oracle ("cpu") or the C ABI ("gpu")."""

    def __init__(self, name, zo=None):
        self.name, self.zo = name, zo

    def matmul(self, p, src, weight, M, N, K, *, bias=None, transB=False, ldb=None, host=None, scales_n=0,
               const=True):
        """p: lowoha.MatmulParams whose quant buffers are given as host arrays in `host` (name -> array or None)."""
        host = host or {}
        ldb = ldb if ldb is not None else (K if transB else N)
        np_dt = {capi.DT_F32: np.float32, capi.DT_BF16: np.uint16, capi.DT_S32: np.int32}[p.dt_dst]
        if self.name == "cpu":
            keep = []
            ph = H.host_params(p, **host)
            if p.dt_wei in (capi.DT_S4, capi.DT_U4) and not p.dynamic_quant:
                st, dst = self.zo.matmul_woq(src, weight, ph.flat(keep), M, N, K, bias=bias, transB=transB, ldb=ldb)
                assert st == capi.SUCCESS
                return dst[:, :N].astype(np_dt, copy=False), None
            st, dst, _, scales = self.zo.matmul_int8(src, weight, ph.flat(keep), M, N, K, bias=bias, transB=transB, ldb=ldb,
                                                     want_scales=scales_n > 0, n_scales=scales_n or None)
            assert st == capi.SUCCESS
            return dst[:, :N].astype(np_dt, copy=False), (scales[:scales_n] if scales_n else None)
        import torch
        keep = []
        pd = H.host_params(p)          # shallow copy; device buffers below
        sc_d = None
        for name, arr in host.items():
            q = getattr(p, name)
            if arr is None and name == "src_scale" and scales_n:
                sc_d = torch.zeros(scales_n, dtype=torch.float32, device=H.DEV)
                setattr(pd, name, lowoha.QuantParam(sc_d, q.dt, q.dims))
            elif arr is None:
                setattr(pd, name, lowoha.QuantParam(None, q.dt, q.dims))
            elif arr.size == 1:
                keep.append(arr)
                setattr(pd, name, lowoha.QuantParam(arr.ctypes.data, q.dt, q.dims))   # one element: host memory
            else:
                t = H.to_dev(arr)
                keep.append(t)
                setattr(pd, name, lowoha.QuantParam(t, q.dt, q.dims))
        tdt = {capi.DT_F32: torch.float32, capi.DT_BF16: torch.bfloat16, capi.DT_S32: torch.int32}[p.dt_dst]
        dst = torch.zeros((M, N), dtype=tdt, device=H.DEV)
        st = lowoha.matmul_direct("r", False, transB, M, N, K, 1.0, H.to_dev(src), src.shape[-1], H.to_dev(weight), ldb,
                                  H.to_dev(bias), 0.0, dst, N, const, pd)
        assert st == capi.SUCCESS, lowoha.last_error()
        return H.to_host(dst), (H.to_host(sc_d) if sc_d is not None else None)


def run(name, backend, zo=None):
    """-> {output name: (array, EXACT | BF16_ULP)}"""
    spec = CASES[name]
    kind, seed = spec[0], spec[1]
    rng = np.random.default_rng(seed)
    be = _Backend(backend, zo)
    out = {}
    if kind == "u8":
        # BASELINE config 1: u8 x s8, zero-point 128, scale 0.02, per-channel weight scales, f32 bias, no post-op;
        # a second call with an s32 destination and no scales stores the accumulator (+ compensation) itself
        M, K, N = spec[2:]
        a = rng.integers(0, 256, (M, K), dtype=np.uint8)
        w = H.gen_weights(rng, K, N)
        ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        zp, ss = np.array([128], dtype=np.int32), np.array([0.02], dtype=np.float32)
        p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (1,))
        p.src_zp = lowoha.QuantParam(None, capi.DT_S32, (1,))
        p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (1, N))
        out["dst_f32"] = (be.matmul(p, a, w, M, N, K, bias=bias, host=dict(src_scale=ss, src_zp=zp, wei_scale=ws))[0], EXACT)
        p2 = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_S32)
        p2.src_zp = lowoha.QuantParam(None, capi.DT_S32, (1,))
        out["acc_s32"] = (be.matmul(p2, a, w, M, N, K, host=dict(src_zp=zp))[0], EXACT)
    elif kind in ("decode", "prefill"):
        # BASELINE configs 2 / 3: bf16 rows quantized per token, per-channel weight scales; f32 without an
        # activation is bit-exact, the bf16 SiLU (decode) / bias + GELU-tanh (prefill) outputs within one ulp
        M, K, N = spec[2:]
        x = H.gen_bf16_normal(rng, (M, K))
        w = H.gen_weights(rng, K, N)
        ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
        bias = (rng.standard_normal(N) * 0.1).astype(np.float32) if kind == "prefill" else None

        def params(dst_dt, po):
            p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=dst_dt, compute=capi.DT_S8,
                                    bias=capi.DT_F32 if bias is not None else capi.DT_NONE)
            p.dynamic_quant = True
            p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
            p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (1, N))
            if po is not None:
                p.postop_ = [lowoha.PostOp(po)]
            return p
        y, sc = be.matmul(params(capi.DT_F32, None), x, w, M, N, K, bias=bias, host=dict(src_scale=None, wei_scale=ws),
                          scales_n=M)
        out["dst_f32_no_act"] = (y, EXACT)
        out["src_scales"] = (sc, EXACT)
        po = capi.PO_SWISH if kind == "decode" else capi.PO_GELU_TANH
        y, _ = be.matmul(params(capi.DT_BF16, po), x, w, M, N, K, bias=bias, host=dict(src_scale=None, wei_scale=ws))
        out["dst_bf16_act"] = (y, BF16_ULP)
    elif kind == "moe":
        # BASELINE configs 4 / 5: fused MoE block, softmax top-k routing (skewed by a per-expert bias in config 5,
        # which leaves some experts without rows), SiLU-gated Op1, Op2, weighted reduce to bf16
        T, Hd, I, E, topk, skew = spec[2:]
        c = MH.make_case(seed, T, Hd, I, E, topk, skew=skew)
        out["expert_rows"] = (np.array(c.M, dtype=np.int32), EXACT)
        if backend == "cpu":
            out["out_bf16"] = (MH.oracle_moe(zo, c, list(range(T))), BF16_ULP)
        else:
            d = MH.DeviceMoe(c)
            st = d.call_fused()
            assert st == capi.SUCCESS, lowoha.last_error()
            out["out_bf16"] = (H.to_host(d.out), BF16_ULP)
    elif kind == "per_group":
        M, K, N, G = spec[2:]
        a = rng.integers(-128, 128, (M, K), dtype=np.int8)
        w = H.gen_weights(rng, K, N)
        ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
        ws = rng.uniform(0.001, 0.01, (G, N)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, G))
        p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (G, N))
        out["dst_f32"] = (be.matmul(p, a, w, M, N, K, bias=bias, host=dict(src_scale=ss, wei_scale=ws))[0], EXACT)
        x = H.gen_bf16_normal(rng, (M, K))
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_F32, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, G))
        p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (G, N))
        y, sc = be.matmul(p, x, w, M, N, K, host=dict(src_scale=None, wei_scale=ws), scales_n=M * G)
        out["dyn_dst_f32"] = (y, EXACT)
        out["dyn_src_scales"] = (sc, EXACT)
    elif kind == "ggml":
        M, K, N = spec[2:]
        G = K // 32
        a = rng.integers(-128, 128, (M, K), dtype=np.int8)
        rows = rng.integers(-127, 128, (N, K), dtype=np.int8)
        d16 = rng.uniform(1e-3, 0.02, (N, G)).astype(np.float16)
        blk = np.zeros((N, G, 34), dtype=np.uint8)
        blk[:, :, :2] = d16.view(np.uint16).reshape(N, G, 1).view(np.uint8)
        blk[:, :, 2:] = rows.reshape(N, G, 32).view(np.uint8)
        ss = rng.uniform(0.005, 0.03, (M, G)).astype(np.float32)
        p = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, G))
        p.pack_format_b = 1
        out["dst_f32"] = (be.matmul(p, a, blk.reshape(-1), M, N, K, transB=True, ldb=K, host=dict(src_scale=ss))[0], EXACT)
    elif kind == "w4a8":
        M, K, N, G = spec[2:]
        x = H.gen_bf16_normal(rng, (M, K), std=2.0)
        packed = rng.integers(0, 256, K * N // 2, dtype=np.uint8)      # [K, N] nibbles, even index = low nibble
        ws = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
        for tag, dims in (("per_token", (M, 1)), ("per_group", (M, G))):
            p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8)
            p.dynamic_quant = True
            p.src_scale = lowoha.QuantParam(None, capi.DT_F32, dims)
            p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (G, N))
            y, sc = be.matmul(p, x, packed, M, N, K, ldb=N, host=dict(src_scale=None, wei_scale=ws),
                              scales_n=int(np.prod(dims)))
            out["dst_bf16_" + tag] = (y, EXACT)
            out["src_scales_" + tag] = (sc, EXACT)
    elif kind == "woq":
        # weight-only quantization: one-hot bf16 rows make the product the dequantized bf16 weight matrix itself
        # (every sum is one value plus zeros, exact in any order): s4 codes with f32 {G,N} scales, and u4 codes with
        # bf16 {G,N} zero-points, the (code - 8) * scale + zp form
        K, N, G = spec[2:]
        eye = np.zeros((K, K), dtype=np.uint16)
        eye[np.arange(K), np.arange(K)] = 0x3F80
        packed = rng.integers(0, 256, K * N // 2, dtype=np.uint8)
        ws = rng.uniform(0.01, 0.1, (G, N)).astype(np.float32)
        zp = H.bf16_bits(rng.uniform(-0.2, 0.2, (G, N)).astype(np.float32))
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16)
        p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (G, N))
        out["weights_bf16_s4"] = (be.matmul(p, eye, packed, K, N, K, ldb=N, host=dict(wei_scale=ws))[0], EXACT)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_U4, dst=capi.DT_F32)
        p.wei_scale = lowoha.QuantParam(None, capi.DT_F32, (G, N))
        p.wei_zp = lowoha.QuantParam(None, capi.DT_BF16, (G, N))
        out["weights_f32_u4_bf16_zp"] = (be.matmul(p, eye, packed, K, N, K, ldb=N, host=dict(wei_scale=ws, wei_zp=zp))[0], EXACT)
    else:
        raise KeyError(kind)
    return out


def bf16_table(zo):
    """Both f32 -> bf16 rules of the reference (common/bfloat16.cpp:27-51 constructor, :69-79 bit trick) on every
    high half with the low halves that decide the rounding."""
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    f = bits.view(np.float32)
    return {"ctor": zo.f32_to_bf16(f, ctor=True), "rne": zo.f32_to_bf16(f, ctor=False)}


def quant_ties(zo):
    """Per-token quantization on rows built so that v / scale lands on n + 0.5 (ties go to even), with a NaN, an
    infinity and a zero row."""
    rows = np.zeros((4, 64), dtype=np.float32)
    rows[0, :] = np.arange(64, dtype=np.float32) * 0.5          # absmax 31.5 ... scale = 31.5 / 127
    rows[0, 63] = 127.0                                          # scale exactly 1: 0.5, 1.5, 2.5 ... are ties
    rows[1, :] = -rows[0, :]
    rows[2, :8] = [np.nan, np.inf, -np.inf, 2.5, -3.5, 4.5, 127.0, 0.0]
    q, s = zo.quant_per_token(rows, capi.DT_F32)
    return {"q": q, "scales": s}
