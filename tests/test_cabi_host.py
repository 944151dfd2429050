"""CPU-side tests of the C ABI: the library loads, exports every symbol the
header declares, and reproduces the reference's validation outcomes (status
codes) for matmul_direct, group_matmul_direct, reorder_direct and
weight_prepack_size.  Every case here is rejected before any GPU call, so the
tests need no GPU (reference rules: lowoha_matmul_utils.cpp:180-411,
group_matmul_direct.cpp:185-699, lowoha_prepack.cpp:53-96)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from zendnn_amd import capi, lowoha

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x1000   # non-null placeholder; validation fails before anything dereferences it


def _device_present():
    try:
        import torch
        return torch.cuda.device_count() > 0
    except Exception:
        return False


# The validation tests hand the library addresses that are no memory: they belong on a machine without a device,
# where a case that slipped past the validators fails at the device check instead of launching on such an address.
fake_pointers = pytest.mark.skipif(_device_present(), reason="placeholder addresses: run where no device can be launched on")


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    hdr = open(os.path.join(ROOT, "include", "zmi_lowoha.h")).read()
    declared = set(re.findall(r"ZMI_API[^;]*?\b(zmi_\w+)\s*\(", hdr))
    assert declared, "no declarations found"
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None
    assert b"gfx950" in lib.zmi_version()


def test_params_init_matches_reference_defaults():
    lib = capi.load()
    p = capi.MatmulParamsT()
    lib.zmi_matmul_params_init(C.byref(p))
    assert (p.mem_format_a, p.mem_format_b) == (b"n", b"n")
    assert p.lowoha_algo == -1 and p.num_threads == 0 and p.dynamic_quant == 0
    assert p.weight_cache_type == 2 and p.total_matmul == 0 and p.active_matmul == 0
    b = capi.BatchParamsT()
    lib.zmi_batch_params_init(C.byref(b))
    assert (b.Batch_A, b.Batch_B) == (1, 1) and b.batch_stride_src == 2**64 - 1


def _mm(p, src=FAKE, wei=FAKE, dst=FAKE, M=4, N=8, K=16, **kw):
    return lowoha.matmul_direct("r", False, False, M, N, K, 1.0, src, K, wei, N, None, 0.0, dst, N, True, p, **kw)


def _int8_params(**kw):
    p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_F32)
    for k, v in kw.items():
        setattr(p, k, v)
    return p


@fake_pointers
def test_matmul_validation_status_codes():
    one = np.ones(4, dtype=np.float32)
    q = lambda dims, dt=capi.DT_F32: lowoha.QuantParam(one.ctypes.data, dt, dims)
    assert _mm(_int8_params(), src=None) == capi.FAILURE
    assert _mm(_int8_params(), wei=None) == capi.FAILURE
    assert _mm(_int8_params(), dst=None) == capi.FAILURE
    assert _mm(_int8_params(), M=0) == capi.FAILURE
    assert _mm(_int8_params(), K=-1) == capi.FAILURE
    assert _mm(_int8_params(), batch_a=0) == capi.FAILURE
    assert _mm(_int8_params(), batch_a=3, batch_b=2) == capi.FAILURE
    # source quant params without s8 weights
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_BF16, dst=capi.DT_BF16)
    p.src_scale = q((1,))
    assert _mm(p) == capi.FAILURE
    # per-token source scale: needs symmetric s8/bf16/f32 source, f32/bf16 dst, per-channel weight scale
    p = _int8_params(dt_src=capi.DT_S8, src_scale=q((4, 1)))
    assert _mm(p) == capi.FAILURE                                   # no per-channel weight scale
    p = _int8_params(dt_src=capi.DT_S8, src_scale=q((4, 1)), wei_scale=q((1, 8)), src_zp=q((1,), capi.DT_S32))
    assert _mm(p) == capi.FAILURE                                   # zero-point with per-token scale
    p = _int8_params(dt_src=capi.DT_U8, src_scale=q((4, 1)), wei_scale=q((1, 8)))
    assert _mm(p) == capi.FAILURE                                   # u8 source with per-token scale
    p = _int8_params(dt_src=capi.DT_S8, dt_dst=capi.DT_S8, src_scale=q((4, 1)), wei_scale=q((1, 8)))
    assert _mm(p) == capi.FAILURE                                   # s8 dst with per-token scale
    # src_zp / dst_scale / dst_zp must be per-tensor
    assert _mm(_int8_params(src_zp=q((4,), capi.DT_S32))) == capi.FAILURE
    assert _mm(_int8_params(dst_scale=q((1, 8)))) == capi.FAILURE
    # dtype combinations
    assert _mm(_int8_params(dt_src=capi.DT_S32)) == capi.FAILURE
    assert _mm(_int8_params(dt_dst=capi.DT_S16)) == capi.FAILURE
    assert _mm(lowoha.MatmulParams(src=capi.DT_F32, wei=capi.DT_S8, dst=capi.DT_BF16)) == capi.FAILURE
    # post-ops: non-finite clip bounds, mish on the int8 paths
    p = _int8_params()
    p.postop_ = [lowoha.PostOp(capi.PO_CLIP, alpha=float("nan"), beta=1.0)]
    assert _mm(p) == capi.FAILURE
    # mish: refused with per-row source scales on s8 rows, with dynamic quantization and on W4A8
    # (lowoha_matmul_utils.cpp:379-408); the static scale chain takes it
    p = _int8_params(dt_src=capi.DT_S8, dt_dst=capi.DT_BF16, src_scale=q((4, 1)), wei_scale=q((1, 8)))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    assert _mm(p) == capi.FAILURE and "mish" in lowoha.last_error()
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (4, 1))
    p.wei_scale = q((1, 8))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    assert _mm(p) == capi.FAILURE and "mish" in lowoha.last_error()
    p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8)
    p.dynamic_quant = True
    p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (4, 1))
    p.wei_scale = q((1, 8))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    assert _mm(p) == capi.FAILURE and "mish" in lowoha.last_error()
    # (the static chain accepts it: the call gets as far as the next check -- a leading dimension that is too small,
    # so that this case, like every case of this file, is refused before anything touches the placeholder pointers)
    p = _int8_params(src_scale=q((1,)), wei_scale=q((1, 8)))
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    assert lowoha.matmul_direct("r", False, False, 4, 8, 16, 1.0, FAKE, 8, FAKE, 8, None, 0.0, FAKE, 8, True, p) == capi.FAILURE
    assert "mish" not in lowoha.last_error() and "leading dimension" in lowoha.last_error()
    # outside the implemented path: status unimplemented, not failure
    assert _mm(lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_BF16, dst=capi.DT_BF16)) == capi.UNIMPLEMENTED
    # GGML-packed weights: transB = true is required (the packed layout is N x K), as in the reference
    assert _mm(_int8_params(pack_format_b=1)) == capi.FAILURE
    assert _mm(_int8_params(pack_format_b=2)) == capi.FAILURE
    assert _mm(lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16)) == capi.UNIMPLEMENTED
    assert lowoha.matmul_direct("c", False, False, 4, 8, 16, 1.0, FAKE, 16, FAKE, 8, None, 0.0, FAKE, 8, True,
                                _int8_params()) == capi.UNIMPLEMENTED
    # prepacked weights demand the blocked algo, as in the reference
    assert _mm(_int8_params(mem_format_b="r")) == capi.FAILURE
    assert "aocl_dlp_blocked" in lowoha.last_error()
    # leading dimensions
    assert lowoha.matmul_direct("r", False, False, 4, 8, 16, 1.0, FAKE, 8, FAKE, 8, None, 0.0, FAKE, 8, True,
                                _int8_params()) == capi.FAILURE


def test_diagnostics_gate(monkeypatch):
    # ZENDNNL_DIAGNOSTICS_ENABLE=0 skips the validator but never the memory-safety subset
    monkeypatch.setenv("ZENDNNL_DIAGNOSTICS_ENABLE", "0")
    assert _mm(_int8_params(), src=None) == capi.FAILURE
    assert _mm(_int8_params(), M=0) == capi.FAILURE


def _prepack_rp(**kw):
    rp = lowoha.ReorderParams()
    rp.is_prepack = True
    rp.prepack_algo = capi.ALGO_AOCL_DLP_BLOCKED
    rp.prepack_wei_dtype = capi.DT_S8
    rp.prepack_src_dtype = capi.DT_S8
    rp.prepack_K, rp.prepack_N, rp.prepack_ldb = 100, 37, 37
    for k, v in kw.items():
        setattr(rp, k, v)
    return rp


@fake_pointers
def test_prepack_size_and_validation():
    rp = _prepack_rp()
    n = lowoha.weight_prepack_size(rp)
    assert n > 0 and n % 64 == 0 and n >= 100 * 37 and rp.cached_size == n
    # deterministic in (K, N) only
    assert lowoha.weight_prepack_size(_prepack_rp(prepack_ldb=64)) == n
    # size grows with the padded shape
    assert lowoha.weight_prepack_size(_prepack_rp(prepack_K=4096, prepack_N=14336, prepack_ldb=14336)) >= 4096 * 14336
    for bad in (dict(prepack_K=0), dict(prepack_N=-3), dict(prepack_ldb=36),
                dict(prepack_transposed=True, prepack_ldb=99)):
        rp = _prepack_rp(**bad)
        assert lowoha.weight_prepack_size(rp) == 0 and rp.cached_size == 0
        assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE
    rp = _prepack_rp(prepack_algo=capi.ALGO_ONEDNN_BLOCKED)
    assert lowoha.weight_prepack_size(rp) == 0
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.UNIMPLEMENTED
    rp = _prepack_rp(prepack_wei_dtype=capi.DT_BF16)
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.UNIMPLEMENTED
    assert lowoha.reorder_direct(None, FAKE, _prepack_rp()) == capi.FAILURE


@fake_pointers
def test_reorder_dynamic_validation():
    rp = lowoha.ReorderParams()
    rp.dynamic_quant = True
    rp.src_dtype, rp.dst_dtype = capi.DT_BF16, capi.DT_S8
    rp.src_shape, rp.dst_shape = (4, 16), (4, 8)
    rp.scale = lowoha.QuantParam(FAKE, capi.DT_F32, (4, 1))
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # shapes differ
    rp.dst_shape = (4, 16)
    assert lowoha.reorder_direct(None, FAKE, rp) == capi.FAILURE
    rp.scale = lowoha.QuantParam(None, capi.DT_F32, (4, 1))
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # no scale buffer
    rp.scale = lowoha.QuantParam(FAKE, capi.DT_F32, (4, 1))
    # a zero-point buffer selects the asymmetric form (reference: validate_dynamic_quant_params,
    # reorder/lowoha_reorder_utils.cpp:549-580): u8 destination, s32 zero-points, dims given
    rp.zero_point = lowoha.QuantParam(FAKE, capi.DT_S32, (4, 1))
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # asymmetric needs a u8 destination
    rp.dst_dtype = capi.DT_U8
    rp.zero_point = lowoha.QuantParam(FAKE, capi.DT_S8, (4, 1))
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # zero-points are s32
    rp.zero_point = lowoha.QuantParam(FAKE, capi.DT_S32, ())
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # zero_point dims are required
    rp.zero_point = lowoha.QuantParam()
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # symmetric needs an s8 destination
    rp.dst_dtype = capi.DT_BF16
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE          # s8 or u8 only
    rp2 = lowoha.ReorderParams()                                          # static conversion modes
    assert lowoha.reorder_direct(FAKE, FAKE, rp2) == capi.UNIMPLEMENTED


def _group(E=3, **over):
    a = dict(layout=["r"] * E, transA=[False] * E, transB=[False] * E, M=[4] * E, N=[8] * E, K=[16] * E,
             alpha=[1.0] * E, src=[FAKE] * E, lda=[16] * E, weight=[FAKE] * E, ldb=[8] * E, bias=[None] * E,
             beta=[0.0] * E, dst=[FAKE] * E, ldc=[8] * E, is_weights_const=[True] * E,
             params=[lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_BF16, dst=capi.DT_BF16) for _ in range(E)])
    extra = {k: over.pop(k) for k in ("moe_postop", "gated_act", "fused_moe") if k in over}
    a.update(over)
    return lowoha.group_matmul_direct(a["layout"], a["transA"], a["transB"], a["M"], a["N"], a["K"], a["alpha"],
                                      a["src"], a["lda"], a["weight"], a["ldb"], a["bias"], a["beta"], a["dst"],
                                      a["ldc"], a["is_weights_const"], a["params"], **extra)


@fake_pointers
def test_group_validation_status_codes():
    E = 3
    assert _group(M=[]) == capi.FAILURE
    assert _group(N=[8, 8]) == capi.FAILURE                      # vector size mismatch
    assert _group(src=[FAKE, FAKE]) == capi.FAILURE              # src.size() must be 1 or num_ops
    assert _group(M=[4, -1, 4]) == capi.FAILURE
    assert _group(src=[FAKE, None, FAKE]) == capi.FAILURE        # null src at an active expert
    assert _group(M=[4, 0, 4], src=[FAKE, None, FAKE], dst=[FAKE, None, FAKE]) == capi.UNIMPLEMENTED  # bf16 weights: past validation
    # sequential chain (src.size() == 1) refuses the MoE extras and checks the chaining dims
    pp = lowoha.MoePostop(4, 2, FAKE, 8, FAKE, [FAKE] * 8)
    assert _group(src=[FAKE], moe_postop=pp) == capi.FAILURE
    assert _group(src=[FAKE], gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE
    assert _group(src=[FAKE], K=[16, 9, 8]) == capi.FAILURE      # K[i] != N[i-1]
    # gated activation: even N, float dst, row-major
    assert _group(N=[7] * E, ldb=[7] * E, ldc=[7] * E, gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE
    assert _group(layout=["c"] * E, gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE
    ps = [lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_S32) for _ in range(E)]
    assert _group(params=ps, gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE
    assert _group(ldc=[8, 4, 8], gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE   # mixed tight / wide dst
    # fused MoE
    fm = lowoha.FusedMoe(down_weight=[], N_down=[], ldb_down=[])
    assert _group(fused_moe=fm) == capi.FAILURE                  # non-null but empty
    fm = lowoha.FusedMoe(down_weight=[FAKE] * E, N_down=[16] * E, ldb_down=[4] * E, dst_down=[FAKE] * E, ldc_down=[16] * E)
    assert _group(fused_moe=fm, gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE    # ldb_down too small
    fm = lowoha.FusedMoe(down_weight=[FAKE] * E, N_down=[16] * E, ldb_down=[16] * E, dst_down=[FAKE] * E, ldc_down=[8] * E)
    assert _group(fused_moe=fm, gated_act=capi.ACT_SILU_AND_MUL) == capi.FAILURE    # ldc_down < N_down
    fm = lowoha.FusedMoe(down_weight=[FAKE] * E, N_down=[32] * E, ldb_down=[32] * E)
    assert _group(fused_moe=fm, gated_act=capi.ACT_SILU_AND_MUL, dst=[None] * E) == capi.FAILURE  # Op2 into src needs lda >= N_down
    fm = lowoha.FusedMoe(down_weight=[FAKE] * E, N_down=[16, 16, 8], ldb_down=[16] * E, dst_down=[FAKE] * E, ldc_down=[16] * E)
    assert _group(fused_moe=fm, gated_act=capi.ACT_SILU_AND_MUL, moe_postop=pp) == capi.FAILURE   # non-uniform N_down
    # weighted reduce
    assert _group(moe_postop=lowoha.MoePostop(0, 2, FAKE, 8, FAKE, [FAKE])) == capi.FAILURE
    assert _group(moe_postop=lowoha.MoePostop(4, 2, FAKE, 4, FAKE, [FAKE] * 8)) == capi.FAILURE   # ldc_output < D
    assert _group(moe_postop=lowoha.MoePostop(4, 2, FAKE, 8, None, [FAKE] * 8)) == capi.FAILURE   # weights required
    assert _group(N=[8, 8, 16], ldb=[8, 8, 16], ldc=[8, 8, 16], moe_postop=pp) == capi.FAILURE
    # prepack-extras contract
    ps = [lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_BF16, dst=capi.DT_BF16) for _ in range(E)]
    ps[0].active_matmul, ps[0].total_matmul = 4, 4
    assert _group(params=ps) == capi.FAILURE                     # active_matmul > M.size()
    ps[0].active_matmul, ps[0].total_matmul = 2, 1
    assert _group(params=ps) == capi.FAILURE                     # total < active
    ps[0].active_matmul, ps[0].total_matmul = 2, 5
    assert _group(params=ps) == capi.FAILURE                     # weight-side vectors shorter than total_matmul


def test_product_does_not_touch_the_oracle():
    """No product source may import, link or name anything under oracle/."""
    bad = []
    for base in ("zendnn_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            if os.path.basename(dirpath) in ("build", "lib", "__pycache__"):
                continue
            for f in files:
                if f.endswith((".py", ".h", ".hpp", ".hip", ".cpp")):
                    text = open(os.path.join(dirpath, f), errors="ignore").read()
                    if re.search(r"zmi_oracle|libzmi_oracle|from oracle|import oracle|oracle/", text):
                        bad.append(os.path.join(dirpath, f))
    assert not bad, bad


def test_environment_switches_are_read_once_and_reloadable(monkeypatch):
    """The switches are cached per process (zmi_reload_env reads them again); under ZMI_ENV_LIVE, which the test
    session sets, every look goes to the environment -- the diagnostics gate above relies on it."""
    lib = capi.load()
    assert os.environ.get("ZMI_ENV_LIVE") == "1"
    lib.zmi_reload_env()
    monkeypatch.setenv("ZENDNNL_DIAGNOSTICS_ENABLE", "0")
    lib.zmi_reload_env()
    assert _mm(_int8_params(), M=0) == capi.FAILURE


def _plan(lib, M, N, K):
    t, s, p = C.c_int32(), C.c_int32(), C.c_int32()
    assert lib.zmi_large_m_plan(M, N, K, C.byref(t), C.byref(s), C.byref(p)) == capi.SUCCESS
    return t.value, s.value, p.value


def test_large_m_plan_follows_the_measurements(monkeypatch):
    """Which form of the large-M kernel takes a call is decided on the host from prices that came out of measurements
    on MI355X (whole call, tiled / persistent, K = 4096): the shapes below are those measurements, and the plan must
    pick the faster form for each -- except 900 x 14336 (71.8 / 67.8 us), which the prices are known to get wrong.
    Without a device the planner assumes 256 compute units, the MI355X figure."""
    for v in ("ZMI_PRING", "ZMI_GEMM_TOP", "ZMI_RING_SPLITK", "ZMI_RING_MIN_M", "ZMI_DECODE_MAX_M", "ZMI_NO_DECODE_KERNEL"):
        monkeypatch.delenv(v, raising=False)
    lib = capi.load()
    lib.zmi_reload_env()
    persistent_wins = [(2048, 4096), (1024, 4096), (1024, 8192), (2048, 2048), (512, 14336), (768, 14336), (1300, 14336),
                       (1536, 14336), (1792, 14336), (2048, 14336), (4096, 14336), (2048, 5000), (256, 14336), (4096, 4096),
                       (1024, 14336), (2048, 8192)]
    tiled_wins = [(1536, 4096), (1100, 4096), (600, 8192), (1100, 14336), (300, 14336)]
    for M, N in persistent_wins:
        assert _plan(lib, M, N, 4096) == (256, 1, 1), (M, N)
    for M, N in tiled_wins:
        t, s, p = _plan(lib, M, N, 4096)
        assert p == 0 and t in (64, 128, 256) and s == 1, (M, N, t, s, p)
    # the decode-shaped kernels keep their calls; few rows against many columns go out in K slices of 64-row tiles
    assert _plan(lib, 16, 14336, 4096) == (0, 0, 0)
    t, s, p = _plan(lib, 128, 14336, 4096)
    assert (t, p) == (64, 0) and s >= 2
    # few rows: 64-row tiles in as many K slices as leave a slice 24 stages and fit one workgroup per compute unit
    # (the shapes of the planner's own measurements)
    assert _plan(lib, 96, 14336, 4096) == (64, 2, 0)
    assert _plan(lib, 128, 8192, 8192) == (64, 4, 0)
    assert _plan(lib, 128, 4096, 14336) == (64, 4, 0)
    assert _plan(lib, 256, 4096, 4096) == (64, 2, 0)
    # the overrides
    monkeypatch.setenv("ZMI_PRING", "0")
    lib.zmi_reload_env()
    assert _plan(lib, 2048, 14336, 4096)[2] == 0
    monkeypatch.setenv("ZMI_PRING", "1")
    lib.zmi_reload_env()
    assert _plan(lib, 1100, 4096, 4096)[2] == 1
    monkeypatch.delenv("ZMI_PRING")
    monkeypatch.setenv("ZMI_GEMM_TOP", "256")
    lib.zmi_reload_env()
    assert _plan(lib, 2048, 14336, 4096) == (256, 1, 0)
    monkeypatch.delenv("ZMI_GEMM_TOP")
    lib.zmi_reload_env()
    assert lib.zmi_large_m_plan(0, 8, 8, None, None, None) == capi.FAILURE


def test_environment_table_names_follow_the_enum():
    """The switches are looked up by position: the enum in zmi_launch.h and the name table in zmi_host.hip must list
    the same switches in the same order, and nothing else in the sources may read the environment itself."""
    src = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "zendnn_amd", "csrc")
    head = open(os.path.join(src, "zmi_launch.h")).read()
    enum = head[head.index("enum ZmiEnvVar {"):head.index("ZE_COUNT")]
    enums = re.findall(r"\bZE_[A-Z0-9_]+", enum)
    host = open(os.path.join(src, "zmi_host.hip")).read()
    table = host[host.index("kEnvNames"):]
    names = re.findall(r'"([A-Z0-9_]+)"', table[:table.index("};")])
    assert len(enums) == len(names) > 20
    for e, n in zip(enums, names):
        assert e[3:] == (n[4:] if n.startswith("ZMI_") else n), (e, n)
    for f in os.listdir(src):
        text = open(os.path.join(src, f)).read()
        if f != "zmi_host.hip":
            assert "getenv(" not in text, f


@fake_pointers
def test_placeholder_addresses_are_refused_before_anything_is_queued():
    """A call that passes every validator with an operand address in the first 64 KiB (here the accepted form of the
    mish post-op on the static scale chain) is refused by the library itself, with or without a device: such an
    address is no memory, and a kernel launched on it faults the device."""
    p = _int8_params()
    p.postop_ = [lowoha.PostOp(capi.PO_MISH)]
    st = lowoha.matmul_direct("r", False, False, 4, 8, 16, 1.0, FAKE, 16, FAKE, 8, None, 0.0, FAKE, 8, True, p)
    assert st == capi.FAILURE and "first 64 KiB" in lowoha.last_error(), lowoha.last_error()
    rp = _prepack_rp()
    assert lowoha.reorder_direct(FAKE, FAKE, rp) == capi.FAILURE and "first 64 KiB" in lowoha.last_error()
