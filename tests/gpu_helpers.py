"""Shared plumbing of the GPU parity tests: seeded inputs, host<->device copies,
and the comparison rules."""
import numpy as np
import torch

from zendnn_amd import capi, lowoha

DEV = "cuda:0"


def to_dev(a):
    """numpy array (uint16 carries bf16 bits) -> torch tensor on the GPU."""
    if a is None:
        return None
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(a).to(DEV)


def to_host(t):
    torch.cuda.synchronize()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def bf16_bits(x):
    """float32 numpy -> bf16 bit patterns (round to nearest even), via torch on the host."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def bf16_ulp_diff(a_bits, b_bits):
    """Distance in bf16 units of last place between two arrays of bit patterns
    (sign-magnitude mapped onto a monotone integer line)."""
    def key(h):
        h = h.astype(np.int32)
        return np.where(h & 0x8000, -(h & 0x7FFF), h & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def check_bf16(got_bits, want_bits, max_frac=2e-3, underflow=1e-30, atol=0.0):
    """<= 1 bf16 ulp everywhere, and only a small fraction of elements may differ
    at all (the device's exp / reciprocal differ from libm in the last f32 ulps,
    which moves a bf16 rounding only when the value sits next to a tie).
    Where both values are below `underflow` in magnitude (an activation of a
    hugely negative input: the f32 reciprocal underflows to zero on the device
    while the reference's double-precision step keeps ~1e-37) the ulp metric is
    meaningless and the absolute difference, < 1e-30, is the check.
    atol > 0 additionally accepts |got - want| <= atol: GELU's "1 + tanh(u)"
    (and "1 + erf") cancels in the negative tail, where the reference's own
    value is only good to about |x| * 6e-8 absolute and depends on libm's last
    bit of tanhf, so a bound in ulps of the (tiny) result cannot hold there."""
    d = bf16_ulp_diff(got_bits, want_bits)
    g = (got_bits.astype(np.uint32) << 16).view(np.float32)
    w = (want_bits.astype(np.uint32) << 16).view(np.float32)
    tiny = (np.abs(g) < underflow) & (np.abs(w) < underflow)
    d = np.where(tiny, 0, d)
    if atol > 0:
        d = np.where(np.abs(g.astype(np.float64) - w.astype(np.float64)) <= atol, np.minimum(d, 1), d)
    assert d.max() <= 1, f"max bf16 ulp diff {d.max()} at {np.unravel_index(d.argmax(), d.shape)}"
    frac = float((d != 0).mean())
    assert frac <= max_frac, f"{frac:.2e} of the elements differ by one bf16 ulp"
    return frac


def check_f32(got, want, rtol=1e-5, atol=1e-6):
    """|got - want| <= rtol * |want| + atol (atol covers results that cancel to
    near zero, where a relative bound on the result is meaningless)."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = rtol * np.abs(want.astype(np.float64)) + atol
    bad = err > bound
    assert not bad.any(), f"{bad.sum()} elements outside tolerance, worst {err.max():.3e}"


def gen_weights(rng, K, N):
    return rng.integers(-127, 128, (K, N), dtype=np.int8)


def gen_bf16_normal(rng, shape, std=1.0):
    return bf16_bits(rng.standard_normal(shape).astype(np.float32) * std)


def host_params(p_dev, **host_buffs):
    """A MatmulParams copy whose quant buffers point at host numpy arrays (for the oracle).
    host_buffs maps field name -> numpy array or None."""
    import copy
    p = copy.copy(p_dev)
    p.postop_ = list(p_dev.postop_)
    for name, arr in host_buffs.items():
        q = getattr(p_dev, name)
        setattr(p, name, lowoha.QuantParam(arr.ctypes.data if arr is not None else None, q.dt, q.dims))
    return p


def prepack(w_dev, K, N, ldb=None, transposed=False, src_dtype=capi.DT_S8):
    rp = lowoha.ReorderParams()
    rp.is_prepack = True
    rp.prepack_algo = capi.ALGO_AOCL_DLP_BLOCKED
    rp.prepack_wei_dtype = capi.DT_S8
    rp.prepack_src_dtype = src_dtype
    rp.prepack_K, rp.prepack_N = K, N
    rp.prepack_ldb = ldb if ldb is not None else (K if transposed else N)
    rp.prepack_transposed = transposed
    size = lowoha.weight_prepack_size(rp)
    assert size > 0 and size % 64 == 0
    blob = torch.empty(size, dtype=torch.uint8, device=DEV)
    st = lowoha.reorder_direct(w_dev, blob, rp)
    assert st == capi.SUCCESS, lowoha.last_error()
    return blob
