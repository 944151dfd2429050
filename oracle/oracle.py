"""numpy front end of the CPU oracle (test infrastructure only).

Every function takes and returns numpy arrays in host memory and calls
libzmi_oracle.so (zmi_oracle.c).  bf16 tensors are carried as uint16 arrays.
"""
import ctypes as C
import os

import numpy as np

from zendnn_amd import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class MatmulCall(C.Structure):
    _fields_ = [("layout", C.c_char), ("transA", C.c_int32), ("transB", C.c_int32),
                ("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("alpha", C.c_float),
                ("src", C.c_void_p), ("lda", C.c_int32), ("weight", C.c_void_p),
                ("ldb", C.c_int32), ("bias", C.c_void_p), ("beta", C.c_float),
                ("dst", C.c_void_p), ("ldc", C.c_int32),
                ("params", C.POINTER(capi.MatmulParamsT)),
                ("acc_out", C.c_void_p), ("scale_out", C.c_void_p), ("zp_out", C.c_void_p)]


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libzmi_oracle.so")
        if not os.path.exists(path):
            from oracle import build
            build.build()
        L = C.CDLL(path)
        L.zo_f32_to_bf16_ctor.restype = C.c_uint16
        L.zo_f32_to_bf16_ctor.argtypes = [C.c_float]
        L.zo_f32_to_bf16_rne.restype = C.c_uint16
        L.zo_f32_to_bf16_rne.argtypes = [C.c_float]
        L.zo_bf16_to_f32.restype = C.c_float
        L.zo_bf16_to_f32.argtypes = [C.c_uint16]
        L.zo_f32_to_bf16_buf.restype = None
        L.zo_f32_to_bf16_buf.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.zo_quant_per_token.restype = None
        L.zo_quant_per_token.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64,
                                         C.c_void_p, C.c_int64, C.c_void_p]
        L.zo_quant_per_group.restype = None
        L.zo_quant_per_group.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                         C.c_void_p, C.c_int64, C.c_void_p]
        L.zo_quant_asym.restype = None
        L.zo_quant_asym.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                    C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
        L.zo_fp16_to_f32.restype = C.c_float
        L.zo_fp16_to_f32.argtypes = [C.c_uint16]
        L.zo_f32_to_f16.restype = C.c_uint16
        L.zo_f32_to_f16.argtypes = [C.c_float]
        L.zo_ggml_q8_0_unpack.restype = None
        L.zo_ggml_q8_0_unpack.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
        L.zo_s4_to_s8.restype = None
        L.zo_s4_to_s8.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p]
        L.zo_gemm_s32.restype = C.c_int64
        L.zo_gemm_s32.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p,
                                  C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                  C.c_void_p, C.c_int64]
        L.zo_gemm_s32_bt.restype = None
        L.zo_gemm_s32_bt.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_void_p, C.c_int64,
                                     C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int64]
        L.zo_transpose_s8.restype = None
        L.zo_transpose_s8.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]
        L.zo_zp_comp.restype = None
        L.zo_zp_comp.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64,
                                 C.c_int32, C.c_void_p]
        L.zo_eltwise.restype = C.c_float
        L.zo_eltwise.argtypes = [C.c_int32, C.c_float, C.c_float, C.c_float]
        L.zo_matmul_int8.restype = C.c_int32
        L.zo_matmul_int8.argtypes = [C.POINTER(MatmulCall)]
        L.zo_matmul_woq.restype = C.c_int32
        L.zo_matmul_woq.argtypes = [C.POINTER(MatmulCall), C.c_int32]
        L.zo_woq_dequant.restype = None
        L.zo_woq_dequant.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32,
                                     C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]
        L.zo_gated_act.restype = None
        L.zo_gated_act.argtypes = [C.c_int32, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64]
        L.zo_moe_reduce.restype = None
        L.zo_moe_reduce.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_int32, C.c_int64,
                                    C.c_int32, C.c_int64, C.c_int32, C.c_void_p, C.c_int64]
        L.zo_bench_s8_gemm.restype = None
        L.zo_bench_s8_gemm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                       C.c_int64, C.c_int64, C.c_int32, C.c_void_p]
        _LIB = L
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


NP_OF_DT = {capi.DT_F32: np.float32, capi.DT_BF16: np.uint16, capi.DT_S32: np.int32,
            capi.DT_S8: np.int8, capi.DT_U8: np.uint8, capi.DT_F16: np.uint16}


def f32_to_bf16(x, ctor=True):
    """float32 array -> uint16 array of bf16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().zo_f32_to_bf16_buf(_p(x), _p(out), x.size, 1 if ctor else 0)
    return out


def bf16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    return (h.astype(np.uint32) << 16).view(np.float32)


def quant_per_token(src, src_dt):
    """src [M,K] (float32, or uint16 bf16 bits) -> (q int8 [M,K], scales f32 [M])."""
    src = np.ascontiguousarray(src)
    M, K = src.shape
    q = np.empty((M, K), dtype=np.int8)
    s = np.empty((M,), dtype=np.float32)
    lib().zo_quant_per_token(_p(src), src_dt, M, K, K, _p(q), K, _p(s))
    return q, s


def quant_per_group(src, src_dt, G):
    """src [M,K] (float32, or uint16 bf16 bits) -> (q int8 [M,K], scales f32 [M,G]); K % G == 0."""
    src = np.ascontiguousarray(src)
    M, K = src.shape
    q = np.empty((M, K), dtype=np.int8)
    s = np.empty((M, G), dtype=np.float32)
    lib().zo_quant_per_group(_p(src), src_dt, M, K, G, K, _p(q), K, _p(s))
    return q, s


def quant_asym(src, src_dt, G=1):
    """src [M,K] (float32, or uint16 bf16 bits) -> (q uint8 [M,K], scales f32 [M,G], zero-points int32 [M,G])."""
    src = np.ascontiguousarray(src)
    M, K = src.shape
    q = np.empty((M, K), dtype=np.uint8)
    s = np.empty((M, G), dtype=np.float32)
    z = np.empty((M, G), dtype=np.int32)
    lib().zo_quant_asym(_p(src), src_dt, M, K, G, K, _p(q), K, _p(s), _p(z))
    return q, s, z


def ggml_q8_0_unpack(blocks, N, K):
    """blocks: uint8 [N * (K/32) * 34] -> (rows int8 [N,K], scales bf16 bits uint16 [K/32, N])."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    rows = np.empty((N, K), dtype=np.int8)
    scales = np.empty((K // 32, N), dtype=np.uint16)
    lib().zo_ggml_q8_0_unpack(_p(blocks), N, K, _p(rows), _p(scales))
    return rows, scales


def s4_to_s8(packed, K, N, ldb=None, transposed=False):
    """packed: uint8 nibble pairs of a [K, ldb] (or [N, ldb] when transposed) s4 matrix -> int8 [K, N]."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    if ldb is None:
        ldb = K if transposed else N
    out = np.empty((K, N), dtype=np.int8)
    lib().zo_s4_to_s8(_p(packed), K, N, ldb, int(transposed), _p(out))
    return out


def gemm_s32(A, B, transA=False, transB=False):
    """Exact s32 accumulator; A u8/s8 [M,K] (or [K,M] if transA), B s8 [K,N]
    (or [N,K] if transB).  Returns (acc [M,N] int32, overflow_count)."""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    acc = np.empty((M, N), dtype=np.int32)
    a_dt = capi.DT_U8 if A.dtype == np.uint8 else capi.DT_S8
    ov = lib().zo_gemm_s32(_p(A), a_dt, int(transA), A.shape[1], _p(B), int(transB), B.shape[1],
                           M, N, K, _p(acc), N)
    return acc, ov


def matmul_int8(src, weight, params, M, N, K, *, bias=None, dst=None, lda=None, ldb=None,
                ldc=None, transA=False, transB=False, alpha=1.0, beta=0.0, want_acc=False,
                want_scales=False, n_scales=None, zp_out=None):
    """Runs the oracle's matmul_direct on host arrays.  params is a
    capi.MatmulParamsT whose buff pointers reference host memory.  Returns
    (status, dst array, acc or None, scales or None)."""
    src = np.ascontiguousarray(src)
    weight = np.ascontiguousarray(weight)
    lda = lda if lda is not None else src.shape[-1]
    ldb = ldb if ldb is not None else weight.shape[-1]
    ldc = ldc if ldc is not None else N
    if dst is None:
        dst = np.zeros((M, ldc), dtype=NP_OF_DT[params.dt_dst])
    acc = np.empty((M, N), dtype=np.int32) if want_acc else None
    scales = np.empty((n_scales or M,), dtype=np.float32) if want_scales else None   # (M * G with per-group scales)
    call = MatmulCall()
    call.layout = b"r"
    call.transA, call.transB = int(transA), int(transB)
    call.M, call.N, call.K = M, N, K
    call.alpha, call.beta = alpha, beta
    call.src, call.lda = _p(src), lda
    call.weight, call.ldb = _p(weight), ldb
    call.bias = _p(bias)
    call.dst, call.ldc = _p(dst), ldc
    call.params = C.pointer(params)
    call.acc_out = _p(acc)
    call.scale_out = _p(scales)
    call.zp_out = _p(zp_out)   # int32 [1]: receives the zero-point of a dynamic quantization to u8
    st = lib().zo_matmul_int8(C.byref(call))
    return st, dst, acc, scales


def woq_dequant(packed, K, N, wei_dt, scales, scale_dt, zp=None, zp_dt=0, ldb=None, transposed=False):
    """4-bit codes -> the bf16 weight matrix [K, N] (bits) the weight-only path multiplies with."""
    packed = np.ascontiguousarray(packed)
    out = np.empty((K, N), dtype=np.uint16)
    ldb = ldb if ldb is not None else (K if transposed else N)
    lib().zo_woq_dequant(_p(packed), K, N, ldb, int(transposed), wei_dt, _p(scales), scales.size, scale_dt,
                         _p(zp), 0 if zp is None else zp.size, zp_dt, _p(out))
    return out


def matmul_woq(src, weight, params, M, N, K, *, bias=None, dst=None, lda=None, ldb=None, ldc=None,
               transA=False, transB=False, alpha=1.0, beta=0.0, is_weights_const=True):
    """The oracle's matmul_direct for a bf16 source with s4 / u4 weights (weight-only quantization) on host
    arrays.  Returns (status, dst array)."""
    src = np.ascontiguousarray(src)
    weight = np.ascontiguousarray(weight)
    lda = lda if lda is not None else src.shape[-1]
    ldb = ldb if ldb is not None else (K if transB else N)
    ldc = ldc if ldc is not None else N
    if dst is None:
        dst = np.zeros((M, ldc), dtype=NP_OF_DT[params.dt_dst])
    call = MatmulCall()
    call.layout = b"r"
    call.transA, call.transB = int(transA), int(transB)
    call.M, call.N, call.K = M, N, K
    call.alpha, call.beta = alpha, beta
    call.src, call.lda = _p(src), lda
    call.weight, call.ldb = _p(weight), ldb
    call.bias = _p(bias)
    call.dst, call.ldc = _p(dst), ldc
    call.params = C.pointer(params)
    st = lib().zo_matmul_woq(C.byref(call), int(is_weights_const))
    return st, dst


def gated_act(act, buf, dt):
    """In place on buf [M, N] (float32 or bf16 bits): buf[:, :N/2] = act(gate) * up."""
    assert buf.flags.c_contiguous
    M, N = buf.shape
    lib().zo_gated_act(act, _p(buf), dt, M, N, N)
    return buf


def moe_reduce(rows, weights, dt, D, skip_weighted=False):
    """rows: list of T*topk 1-D host arrays (the gathered expert rows);
    weights f32 [T, topk].  Returns out [T, D]."""
    T, topk = weights.shape
    ptrs = (C.c_void_p * (T * topk))(*[r.ctypes.data for r in rows])
    out = np.empty((T, D), dtype=NP_OF_DT[dt])
    w = np.ascontiguousarray(weights, dtype=np.float32)
    lib().zo_moe_reduce(ptrs, _p(w), int(skip_weighted), T, topk, D, dt, _p(out), D)
    return out


def eltwise(po, x, alpha=0.0, beta=0.0):
    L = lib()
    x = np.asarray(x, dtype=np.float32)
    return np.array([L.zo_eltwise(po, float(v), alpha, beta) for v in x.ravel()],
                    dtype=np.float32).reshape(x.shape)
