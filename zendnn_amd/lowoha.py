"""Python mirror of the LowOHA entry points over the C ABI.

Names, argument order and meaning follow the reference's C++ interface
(matmul_direct / group_matmul_direct: zendnnl/src/lowoha_operators/matmul/
lowoha_matmul.hpp:104-223; reorder_direct / weight_prepack_size:
lowoha_operators/reorder/lowoha_reorder.hpp:103, reorder/prepack/
lowoha_prepack.hpp:165).  Buffers are torch tensors on the GPU (or raw
integer device addresses); torch only owns the memory, every computation
happens in libzmi_lowoha.so.
"""
import ctypes as C

from . import capi
from .capi import (DT_BF16, DT_F32, DT_NONE, DT_S8, DT_S32, DT_U8,  # noqa: F401
                   SUCCESS, FAILURE, UNIMPLEMENTED)


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def torch_dt(t):
    import torch
    return {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.int8: DT_S8,
            torch.uint8: DT_U8, torch.int32: DT_S32}[t.dtype]


class QuantParam:
    """matmul_quantization_params_t::matmul_quant_t: {buff, dt, dims}."""

    def __init__(self, buff=None, dt=DT_NONE, dims=()):
        self.buff, self.dt, self.dims = buff, dt, tuple(dims)

    def flat(self):
        return capi.quant(_ptr(self.buff), self.dt, self.dims)


class PostOp:
    """matmul_post_op: {po_type, buff, dtype, dims, alpha, beta, leading_dim}."""

    def __init__(self, po_type, buff=None, dtype=DT_NONE, dims=(), alpha=0.0, beta=0.0, leading_dim=-1):
        self.po_type, self.buff, self.dtype = po_type, buff, dtype
        self.dims, self.alpha, self.beta, self.leading_dim = tuple(dims), alpha, beta, leading_dim


class MatmulParams:
    """matmul_params with the reference's defaults (matmul/lowoha_common.hpp:223-226)."""

    def __init__(self, src=DT_NONE, wei=DT_NONE, dst=DT_NONE, bias=DT_NONE, compute=DT_NONE):
        self.dt_src, self.dt_wei, self.dt_dst, self.dt_bias, self.dt_compute = src, wei, dst, bias, compute
        self.postop_ = []
        self.src_scale = QuantParam()
        self.wei_scale = QuantParam()
        self.dst_scale = QuantParam()
        self.src_zp = QuantParam()
        self.wei_zp = QuantParam()
        self.dst_zp = QuantParam()
        self.mem_format_a = "n"
        self.mem_format_b = "n"
        self.lowoha_algo = capi.ALGO_NONE
        self.num_threads = 0
        self.dynamic_quant = False
        self.pack_format_b = 0
        self.total_matmul = 0
        self.active_matmul = 0
        self.weight_cache_type = 2

    def flat(self, keep):
        """Flattens into capi.MatmulParamsT; objects that must outlive the call go to keep."""
        p = capi.MatmulParamsT()
        p.dt_src, p.dt_wei, p.dt_dst, p.dt_bias, p.dt_compute = (
            self.dt_src, self.dt_wei, self.dt_dst, self.dt_bias, self.dt_compute)
        n = len(self.postop_)
        p.n_postops = n
        if n:
            arr = (capi.PostOpT * n)()
            for i, po in enumerate(self.postop_):
                arr[i].po_type = po.po_type
                arr[i].dtype = po.dtype
                arr[i].buff = _ptr(po.buff)
                arr[i].ndims = len(po.dims)
                for j, d in enumerate(po.dims):
                    arr[i].dims[j] = d
                arr[i].leading_dim = po.leading_dim
                arr[i].alpha, arr[i].beta = po.alpha, po.beta
            keep.append(arr)
            p.postops = arr
        for name in ("src_scale", "wei_scale", "dst_scale", "src_zp", "wei_zp", "dst_zp"):
            setattr(p, name, getattr(self, name).flat())
        p.mem_format_a = self.mem_format_a.encode()
        p.mem_format_b = self.mem_format_b.encode()
        p.lowoha_algo = self.lowoha_algo
        p.num_threads = self.num_threads
        p.dynamic_quant = int(self.dynamic_quant)
        p.pack_format_b = self.pack_format_b
        p.total_matmul, p.active_matmul = self.total_matmul, self.active_matmul
        p.weight_cache_type = self.weight_cache_type
        return p


def last_error():
    return capi.load().zmi_last_error().decode()


def last_kernel():
    return capi.load().zmi_last_kernel().decode()


def matmul_direct(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc,
                  is_weights_const, params, batch_a=1, batch_b=1, noalloc=False, batch_strides=None):
    """noalloc=True: the entry point that allocates no device memory (zmi_matmul_direct_noalloc).
    batch_strides: (src, wei, dst) strides in elements, None entries (or no tuple) derive them from the
    dimensions like matmul_batch_params_t's default of (size_t)-1."""
    lib = capi.load()
    keep = []
    p = params.flat(keep)
    b = capi.BatchParamsT()
    lib.zmi_batch_params_init(C.byref(b))
    b.Batch_A, b.Batch_B = batch_a, batch_b
    if batch_strides is not None:
        for name, v in zip(("batch_stride_src", "batch_stride_wei", "batch_stride_dst"), batch_strides):
            if v is not None:
                setattr(b, name, int(v))
    fn = lib.zmi_matmul_direct_noalloc if noalloc else lib.zmi_matmul_direct
    return fn(layout.encode(), int(transA), int(transB), M, N, K, alpha, _ptr(src), lda,
                                 _ptr(weight), ldb, _ptr(bias), beta, _ptr(dst), ldc, int(is_weights_const),
                                 C.byref(b), C.byref(p))


def prepared_matmul(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc,
                    is_weights_const, params):
    """Flattens the arguments once and returns (call, rebind): call() issues the same
    matmul_direct with no per-call Python work beyond the foreign call; rebind(weight=...)
    swaps the weight pointer.  For timing loops and serving loops."""
    lib = capi.load()
    keep = []
    p = params.flat(keep)
    b = capi.BatchParamsT()
    lib.zmi_batch_params_init(C.byref(b))
    state = {"w": C.c_void_p(_ptr(weight)), "keep": (keep, params, src, bias, dst, weight)}
    fixed_a = (layout.encode(), int(transA), int(transB), M, N, K, alpha, C.c_void_p(_ptr(src)), lda)
    fixed_b = (ldb, C.c_void_p(_ptr(bias)), beta, C.c_void_p(_ptr(dst)), ldc, int(is_weights_const),
               C.byref(b), C.byref(p))
    fn = lib.zmi_matmul_direct

    def call():
        return fn(*fixed_a, state["w"], *fixed_b)

    def rebind(weight):
        state["w"] = C.c_void_p(_ptr(weight))

    return call, rebind


class ReorderParams:
    """reorder_params_t (prepack and dynamic per-token fields)."""

    def __init__(self):
        self.src_dtype = DT_NONE
        self.dst_dtype = DT_NONE
        self.scale = QuantParam()
        self.zero_point = QuantParam()
        self.algo = 0
        self.num_threads = 0
        self.src_shape = ()
        self.dst_shape = ()
        self.src_strides = ()
        self.dst_strides = ()
        self.dynamic_quant = False
        self.is_prepack = False
        # prepack_params_t
        self.prepack_algo = capi.ALGO_NONE
        self.prepack_wei_dtype = DT_NONE
        self.prepack_src_dtype = DT_NONE
        self.prepack_K = 0
        self.prepack_N = 0
        self.prepack_ldb = 0
        self.prepack_transposed = False
        self.prepack_sym_group_size = 0
        self.cached_size = 0

    def flat(self):
        lib = capi.load()
        r = capi.ReorderParamsT()
        lib.zmi_reorder_params_init(C.byref(r))
        r.src_dtype, r.dst_dtype = self.src_dtype, self.dst_dtype
        r.scale = self.scale.flat()
        r.zero_point = self.zero_point.flat()
        r.algo, r.num_threads = self.algo, self.num_threads
        for name in ("src_shape", "dst_shape", "src_strides", "dst_strides"):
            v = getattr(self, name)
            setattr(r, "n_" + name, len(v))
            arr = getattr(r, name)
            for i, d in enumerate(v):
                arr[i] = d
        r.dynamic_quant, r.is_prepack = int(self.dynamic_quant), int(self.is_prepack)
        r.prepack.algo = self.prepack_algo
        r.prepack.wei_dtype = self.prepack_wei_dtype
        r.prepack.src_dtype = self.prepack_src_dtype
        r.prepack.K, r.prepack.N, r.prepack.ldb = self.prepack_K, self.prepack_N, self.prepack_ldb
        r.prepack.transposed = int(self.prepack_transposed)
        r.prepack.sym_group_size = self.prepack_sym_group_size
        return r


def weight_prepack_size(rp):
    r = rp.flat()
    n = capi.load().zmi_weight_prepack_size(C.byref(r))
    rp.cached_size = r.prepack.cached_size
    return n


def reorder_direct(src, dst, rp):
    r = rp.flat()
    return capi.load().zmi_reorder_direct(_ptr(src), _ptr(dst), C.byref(r))


def _arr(ctype, values):
    n = len(values)
    if n == 0:
        return 0, None
    return n, (ctype * n)(*values)


class MoePostop:
    """group_matmul_moe_postop_params."""

    def __init__(self, num_tokens, topk, output, ldc_output, topk_weights, row_ptrs, skip_weighted=False):
        self.num_tokens, self.topk, self.output, self.ldc_output = num_tokens, topk, output, ldc_output
        self.topk_weights, self.row_ptrs, self.skip_weighted = topk_weights, row_ptrs, skip_weighted


class FusedMoe:
    """grp_matmul_fused_moe_params."""

    def __init__(self, down_weight, N_down, ldb_down, bias_down=None, bias_dt_down=DT_NONE,
                 down_scale=None, down_zp=None, dst_down=None, ldc_down=None):
        n = len(down_weight)
        self.down_weight, self.N_down, self.ldb_down = down_weight, N_down, ldb_down
        self.bias_down = bias_down if bias_down is not None else [None] * n
        self.bias_dt_down = bias_dt_down
        self.down_scale = down_scale or []
        self.down_zp = down_zp or []
        self.dst_down = dst_down or []
        self.ldc_down = ldc_down or []


def group_matmul_direct(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc,
                        is_weights_const, params, moe_postop=None, gated_act=None, fused_moe=None):
    """All per-expert arguments are Python lists, as the reference's std::vector arguments."""
    return prepared_group_matmul(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc,
                                 is_weights_const, params, moe_postop, gated_act, fused_moe)[0]()


def prepared_group_matmul(layout, transA, transB, M, N, K, alpha, src, lda, weight, ldb, bias, beta, dst, ldc,
                          is_weights_const, params, moe_postop=None, gated_act=None, fused_moe=None):
    """The flattened arguments of group_matmul_direct, marshalled once: returns (call, keep); call() is one foreign
    call with the same argument block every time (what a C++ caller's vectors cost: nothing per call)."""
    lib = capi.load()
    keep = []
    g = capi.GroupArgsT()

    def put(name, ctype, values, conv=lambda v: v):
        n, arr = _arr(ctype, [conv(v) for v in values])
        keep.append(arr)
        setattr(g, "n_" + name, n)
        if arr is not None:
            setattr(g, name, arr)

    lay = "".join(layout).encode()
    keep.append(lay)
    g.n_layout, g.layout = len(layout), lay
    put("transA", C.c_uint8, transA, int)
    put("transB", C.c_uint8, transB, int)
    put("M", C.c_int32, M)
    put("N", C.c_int32, N)
    put("K", C.c_int32, K)
    put("alpha", C.c_float, alpha)
    put("src", C.c_void_p, src, _ptr)
    put("lda", C.c_int32, lda)
    put("weight", C.c_void_p, weight, _ptr)
    put("ldb", C.c_int32, ldb)
    put("bias", C.c_void_p, bias, _ptr)
    put("beta", C.c_float, beta)
    put("dst", C.c_void_p, dst, _ptr)
    put("ldc", C.c_int32, ldc)
    put("is_weights_const", C.c_uint8, is_weights_const, int)
    n = len(params)
    parr = (capi.MatmulParamsT * max(n, 1))()
    for i, p in enumerate(params):
        parr[i] = p.flat(keep)
    keep.append(parr)
    g.n_params, g.params = n, parr

    pp = None
    if moe_postop is not None:
        pp = capi.MoePostopT()
        pp.num_tokens, pp.topk = moe_postop.num_tokens, moe_postop.topk
        pp.output, pp.ldc_output = _ptr(moe_postop.output), moe_postop.ldc_output
        pp.topk_weights = _ptr(moe_postop.topk_weights)
        pp.skip_weighted = int(moe_postop.skip_weighted)
        if moe_postop.row_ptrs is not None:
            nrp, rp = _arr(C.c_void_p, [_ptr(v) for v in moe_postop.row_ptrs])
            keep.append(rp)
            pp.row_ptrs = rp
    fm = None
    if fused_moe is not None:
        fm = capi.FusedMoeT()

        def putf(name, ctype, values, conv=lambda v: v):
            nn, arr = _arr(ctype, [conv(v) for v in values])
            keep.append(arr)
            setattr(fm, "n_" + name, nn)
            if arr is not None:
                setattr(fm, name, arr)

        putf("down_weight", C.c_void_p, fused_moe.down_weight, _ptr)
        putf("N_down", C.c_int32, fused_moe.N_down)
        putf("ldb_down", C.c_int32, fused_moe.ldb_down)
        putf("bias_down", C.c_void_p, fused_moe.bias_down, _ptr)
        fm.bias_dt_down = fused_moe.bias_dt_down
        for name in ("down_scale", "down_zp"):
            vals = getattr(fused_moe, name)
            setattr(fm, "n_" + name, len(vals))
            if vals:
                arr = (capi.QuantT * len(vals))(*[v.flat() for v in vals])
                keep.append(arr)
                setattr(fm, name, arr)
        putf("dst_down", C.c_void_p, fused_moe.dst_down, _ptr)
        putf("ldc_down", C.c_int32, fused_moe.ldc_down)
    keep.extend([g, pp, fm])
    a_g, a_pp, a_fm, act = C.byref(g), (C.byref(pp) if pp is not None else None), (C.byref(fm) if fm is not None else None), int(gated_act or 0)
    fn = lib.zmi_group_matmul_direct
    # (the closure holds `keep`: the argument block points into buffers only that list owns)
    return (lambda _keep=keep: fn(a_g, a_pp, act, a_fm)), keep


def moe_route(topk_ids, E):
    """topk_ids: int32 tensor [T, topk] on the GPU -> (counts[E], offsets[E+1], slot_of[T*topk])."""
    import torch
    T, topk = topk_ids.shape
    counts = torch.empty(E, dtype=torch.int32, device=topk_ids.device)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=topk_ids.device)
    slot_of = torch.empty(T * topk, dtype=torch.int32, device=topk_ids.device)
    st = capi.load().zmi_moe_route(topk_ids.data_ptr(), T, topk, E, counts.data_ptr(), offsets.data_ptr(),
                                   slot_of.data_ptr())
    return st, counts, offsets, slot_of


def moe_router_topk(logits, topk, renormalize=False):
    """logits: f32 / bf16 tensor [T, E] on the GPU -> (status, topk_ids int32 [T, topk], topk_weights f32 [T, topk])."""
    import torch
    T, E = logits.shape
    ids = torch.empty(T, topk, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, topk, dtype=torch.float32, device=logits.device)
    dt = {torch.float32: capi.DT_F32, torch.bfloat16: capi.DT_BF16}[logits.dtype]
    st = capi.load().zmi_moe_router_topk(logits.data_ptr(), dt, logits.stride(0), T, E, topk, int(bool(renormalize)),
                                         ids.data_ptr(), w.data_ptr())
    return st, ids, w


def moe_fused_device(x, topk_ids, topk_weights, w13_blobs, w2_blobs, w13_scales, w2_scales, I, gated_act, out):
    T, H = x.shape
    E = len(w13_blobs)
    d = capi.MoeDeviceT()
    d.T, d.H, d.I, d.E, d.topk = T, H, I, E, topk_ids.shape[1]
    d.x, d.ldx = x.data_ptr(), x.stride(0)
    d.topk_ids, d.topk_weights = topk_ids.data_ptr(), topk_weights.data_ptr()
    keep = []
    for name, vals in (("w13_blob", w13_blobs), ("w2_blob", w2_blobs), ("w13_scale", w13_scales),
                       ("w2_scale", w2_scales)):
        arr = (C.c_void_p * E)(*[_ptr(v) for v in vals])
        keep.append(arr)
        setattr(d, name, arr)
    d.gated_act = gated_act
    d.out, d.ldo = out.data_ptr(), out.stride(0)
    return capi.load().zmi_moe_fused_device(C.byref(d))
