"""ctypes description of the C ABI declared in include/zmi_lowoha.h.

This module is plumbing: it mirrors the flat structs field for field and loads
libzmi_lowoha.so.  It computes nothing.  If the library has not been built the
loader raises; there is no CPU fallback.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libzmi_lowoha.so")
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libzendnnl_mi355x.so")

# status_t
SUCCESS, FAILURE, UNIMPLEMENTED, ISA_UNSUPPORTED = 1, 0, -1, -21

# data_type_t
DT_NONE, DT_F32, DT_F16, DT_BF16, DT_S32, DT_S64, DT_S16, DT_S8, DT_S4, \
    DT_U32, DT_U16, DT_U8, DT_U4 = range(13)

# post_op_type_t
(PO_NONE, PO_ELU, PO_RELU, PO_LEAKY_RELU, PO_GELU_TANH, PO_GELU_ERF, PO_SIGMOID,
 PO_SWISH, PO_TANH, PO_SOFTMAX, PO_POOLING, PO_SQUARE, PO_ABS, PO_SQRT, PO_EXP,
 PO_LOG, PO_CLIP, PO_BINARY_ADD, PO_BINARY_MUL, PO_MISH) = range(20)

ALGO_NONE, ALGO_DYNAMIC_DISPATCH, ALGO_AOCL_DLP_BLOCKED = -1, 0, 1
ALGO_ONEDNN_BLOCKED, ALGO_LIBXSMM_BLOCKED = 2, 3

ACT_NONE, ACT_SILU_AND_MUL, ACT_GELU_AND_MUL, ACT_SWIGLU_OAI_MUL = range(4)

MAX_DIMS = 4


class QuantT(C.Structure):
    _fields_ = [("buff", C.c_void_p), ("dt", C.c_int32), ("ndims", C.c_int32),
                ("dims", C.c_int64 * MAX_DIMS)]


class PostOpT(C.Structure):
    _fields_ = [("po_type", C.c_int32), ("dtype", C.c_int32), ("buff", C.c_void_p),
                ("ndims", C.c_int32), ("leading_dim", C.c_int32),
                ("dims", C.c_int64 * MAX_DIMS), ("alpha", C.c_float), ("beta", C.c_float)]


class BatchParamsT(C.Structure):
    _fields_ = [("Batch_A", C.c_int32), ("Batch_B", C.c_int32),
                ("batch_stride_src", C.c_uint64), ("batch_stride_wei", C.c_uint64),
                ("batch_stride_dst", C.c_uint64)]


class MatmulParamsT(C.Structure):
    _fields_ = [("dt_src", C.c_int32), ("dt_wei", C.c_int32), ("dt_dst", C.c_int32),
                ("dt_bias", C.c_int32), ("dt_compute", C.c_int32),
                ("n_postops", C.c_int32), ("postops", C.POINTER(PostOpT)),
                ("src_scale", QuantT), ("wei_scale", QuantT), ("dst_scale", QuantT),
                ("src_zp", QuantT), ("wei_zp", QuantT), ("dst_zp", QuantT),
                ("mem_format_a", C.c_char), ("mem_format_b", C.c_char),
                ("lowoha_algo", C.c_int32), ("num_threads", C.c_int32),
                ("dynamic_quant", C.c_int32), ("pack_format_b", C.c_int32),
                ("total_matmul", C.c_uint32), ("active_matmul", C.c_uint32),
                ("weight_cache_type", C.c_int32)]


class MoePostopT(C.Structure):
    _fields_ = [("num_tokens", C.c_int32), ("topk", C.c_int32), ("output", C.c_void_p),
                ("ldc_output", C.c_int32), ("topk_weights", C.c_void_p),
                ("skip_weighted", C.c_int32), ("row_ptrs", C.POINTER(C.c_void_p))]


class FusedMoeT(C.Structure):
    _fields_ = [("n_down_weight", C.c_int32), ("down_weight", C.POINTER(C.c_void_p)),
                ("n_N_down", C.c_int32), ("N_down", C.POINTER(C.c_int32)),
                ("n_ldb_down", C.c_int32), ("ldb_down", C.POINTER(C.c_int32)),
                ("n_bias_down", C.c_int32), ("bias_down", C.POINTER(C.c_void_p)),
                ("bias_dt_down", C.c_int32),
                ("n_down_scale", C.c_int32), ("down_scale", C.POINTER(QuantT)),
                ("n_down_zp", C.c_int32), ("down_zp", C.POINTER(QuantT)),
                ("n_dst_down", C.c_int32), ("dst_down", C.POINTER(C.c_void_p)),
                ("n_ldc_down", C.c_int32), ("ldc_down", C.POINTER(C.c_int32))]


class GroupArgsT(C.Structure):
    _fields_ = [("n_layout", C.c_int32), ("layout", C.c_char_p),
                ("n_transA", C.c_int32), ("transA", C.POINTER(C.c_uint8)),
                ("n_transB", C.c_int32), ("transB", C.POINTER(C.c_uint8)),
                ("n_M", C.c_int32), ("M", C.POINTER(C.c_int32)),
                ("n_N", C.c_int32), ("N", C.POINTER(C.c_int32)),
                ("n_K", C.c_int32), ("K", C.POINTER(C.c_int32)),
                ("n_alpha", C.c_int32), ("alpha", C.POINTER(C.c_float)),
                ("n_src", C.c_int32), ("src", C.POINTER(C.c_void_p)),
                ("n_lda", C.c_int32), ("lda", C.POINTER(C.c_int32)),
                ("n_weight", C.c_int32), ("weight", C.POINTER(C.c_void_p)),
                ("n_ldb", C.c_int32), ("ldb", C.POINTER(C.c_int32)),
                ("n_bias", C.c_int32), ("bias", C.POINTER(C.c_void_p)),
                ("n_beta", C.c_int32), ("beta", C.POINTER(C.c_float)),
                ("n_dst", C.c_int32), ("dst", C.POINTER(C.c_void_p)),
                ("n_ldc", C.c_int32), ("ldc", C.POINTER(C.c_int32)),
                ("n_is_weights_const", C.c_int32), ("is_weights_const", C.POINTER(C.c_uint8)),
                ("n_params", C.c_int32), ("params", C.POINTER(MatmulParamsT))]


class PrepackParamsT(C.Structure):
    _fields_ = [("algo", C.c_int32), ("wei_dtype", C.c_int32), ("src_dtype", C.c_int32),
                ("K", C.c_int64), ("N", C.c_int64), ("ldb", C.c_int64),
                ("transposed", C.c_int32), ("sym_group_size", C.c_int32),
                ("cached_size", C.c_size_t)]


class ReorderParamsT(C.Structure):
    _fields_ = [("src_dtype", C.c_int32), ("dst_dtype", C.c_int32),
                ("scale", QuantT), ("zero_point", QuantT),
                ("algo", C.c_int32), ("num_threads", C.c_int32),
                ("n_src_shape", C.c_int32), ("src_shape", C.c_int64 * MAX_DIMS),
                ("n_dst_shape", C.c_int32), ("dst_shape", C.c_int64 * MAX_DIMS),
                ("n_src_strides", C.c_int32), ("src_strides", C.c_int64 * MAX_DIMS),
                ("n_dst_strides", C.c_int32), ("dst_strides", C.c_int64 * MAX_DIMS),
                ("dynamic_quant", C.c_int32), ("is_prepack", C.c_int32),
                ("prepack", PrepackParamsT)]


class GroupDqParamsT(C.Structure):
    _fields_ = [("src_dtype", C.c_int32), ("dst_dtype", C.c_int32), ("scale_dtype", C.c_int32),
                ("num_threads", C.c_int32), ("num_groups", C.c_int32)]


class MoeDeviceT(C.Structure):
    _fields_ = [("T", C.c_int32), ("H", C.c_int32), ("I", C.c_int32), ("E", C.c_int32),
                ("topk", C.c_int32),
                ("x", C.c_void_p), ("ldx", C.c_int32),
                ("topk_ids", C.c_void_p), ("topk_weights", C.c_void_p),
                ("w13_blob", C.POINTER(C.c_void_p)), ("w2_blob", C.POINTER(C.c_void_p)),
                ("w13_scale", C.POINTER(C.c_void_p)), ("w2_scale", C.POINTER(C.c_void_p)),
                ("gated_act", C.c_int32),
                ("out", C.c_void_p), ("ldo", C.c_int32)]


# name -> (restype, argtypes); every symbol include/zmi_lowoha.h declares.
SIGNATURES = {
    "zmi_matmul_params_init": (None, [C.POINTER(MatmulParamsT)]),
    "zmi_batch_params_init": (None, [C.POINTER(BatchParamsT)]),
    "zmi_matmul_direct": (C.c_int32, [C.c_char, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                      C.c_int32, C.c_float, C.c_void_p, C.c_int32, C.c_void_p,
                                      C.c_int32, C.c_void_p, C.c_float, C.c_void_p, C.c_int32,
                                      C.c_int32, C.POINTER(BatchParamsT),
                                      C.POINTER(MatmulParamsT)]),
    "zmi_matmul_direct_noalloc": (C.c_int32, [C.c_char, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                              C.c_int32, C.c_float, C.c_void_p, C.c_int32, C.c_void_p,
                                              C.c_int32, C.c_void_p, C.c_float, C.c_void_p, C.c_int32,
                                              C.c_int32, C.POINTER(BatchParamsT),
                                              C.POINTER(MatmulParamsT)]),
    "zmi_group_matmul_direct": (C.c_int32, [C.POINTER(GroupArgsT), C.POINTER(MoePostopT),
                                            C.c_int32, C.POINTER(FusedMoeT)]),
    "zmi_reorder_params_init": (None, [C.POINTER(ReorderParamsT)]),
    "zmi_weight_prepack_size": (C.c_size_t, [C.POINTER(ReorderParamsT)]),
    "zmi_reorder_direct": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(ReorderParamsT)]),
    "zmi_group_dynamic_quant": (C.c_int32, [C.c_int32, C.POINTER(C.c_void_p),
                                            C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                            C.POINTER(C.c_int64), C.POINTER(C.c_void_p),
                                            C.POINTER(C.c_int64), C.POINTER(C.c_void_p),
                                            C.POINTER(GroupDqParamsT)]),
    "zmi_init": (C.c_int32, [C.c_int32]),
    "zmi_set_stream": (None, [C.c_void_p]),
    "zmi_get_stream": (C.c_void_p, []),
    "zmi_last_error": (C.c_char_p, []),
    "zmi_last_kernel": (C.c_char_p, []),
    "zmi_clear_weight_cache": (None, []),
    "zmi_clear_scratch": (None, []),
    "zmi_reload_env": (None, []),
    "zmi_version": (C.c_char_p, []),
    "zmi_moe_route": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                  C.c_void_p, C.c_void_p]),
    "zmi_moe_router_topk": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                        C.c_void_p, C.c_void_p]),
    "zmi_moe_fused_device": (C.c_int32, [C.POINTER(MoeDeviceT)]),
    "zmi_calib_hbm_read": (C.c_int32, [C.POINTER(C.c_void_p), C.c_int32, C.c_uint64, C.c_int32, C.c_int32,
                                       C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "zmi_calib_hbm_read_shape": (C.c_int32, [C.POINTER(C.c_void_p), C.c_int32, C.c_uint64, C.c_int32, C.c_int32, C.c_int32,
                                             C.c_int32, C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "zmi_large_m_plan": (C.c_int32, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                     C.POINTER(C.c_int32)]),
    "zmi_calib_mfma_i8": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                      C.POINTER(C.c_float), C.POINTER(C.c_float)]),
}

_lib = None


def load():
    """Loads libzmi_lowoha.so and binds every declared symbol.  Raises if the
    library is missing or a symbol is not exported."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "from the repository root (there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def quant(buff=None, dt=DT_NONE, dims=()):
    q = QuantT()
    q.buff = buff
    q.dt = dt
    q.ndims = len(dims)
    for i, d in enumerate(dims):
        q.dims[i] = d
    return q
