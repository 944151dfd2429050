#!/usr/bin/env python3
"""Benchmark of the LowOHA int8 matmul path on one MI355X.

Headline workload (BASELINE.json configs[1], the decode shape): one
matmul_direct call per step, M=16, K=4096, N=14336, bf16 activations quantized
per token to s8 inside the call, prepacked s8 weights with per-channel scales,
fused SiLU, bf16 output.  The metric is the algorithmic bytes of one call
(weights K*N + activations M*K*2 + scales N*4 + output M*N*2) divided by the
time of one call, in GB/s; the roofline that bounds it is HBM (8 TB/s).

Weights rotate through enough prepacked copies to exceed the 256 MB on-die
cache, so every step streams its weights from HBM (the reference's "warm"
benchmark mode, benchdnn/doc/matmul.md:171-181).  Inputs are resident in HBM
before the timed region.

Prints ONE JSON line.  The other BASELINE.json configs are timed briefly and
reported under "other_configs" in the same line.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
INT8_PEAK_TOPS = 5000.0
K_DEC, N_DEC = 4096, 14336
# HBM bytes per launch of the headline kernel (FETCH_SIZE + WRITE_SIZE, scaled by a plain copy of known
# size), measured with the commands recorded in profiles/zmi_gemm_decode16_kernel_decode_M16_K4096_N14336.md.
# The counters were last read on the kernel's earlier form (rows staged in half lines): the current form has no
# measurement of its own, so the line reports null and keeps the earlier figure beside it.
DECODE_TRAFFIC_BYTES = None
DECODE_TRAFFIC_BYTES_EARLIER_FORM = 60346524


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extras", action="store_true", help="skip the other configs and the CPU baseline")
    ap.add_argument("--only", default=None,
                    choices=["decode_M1", "decode_M4", "decode_M64", "decode_M128", "decode_M16_per_group128", "decode_M16_per_group32", "decode_M16_w4a8_group128", "decode_M16_w4a8_group128_per_token_rows", "decode_M16_woq_s4_group128", "decode_M16_woq_u4_group128", "decode_M1_woq_s4_group128", "prefill_N4096", "prefill_N14336", "config1_u8s8_M128",
                             "decode_M16_K14336_N4096", "prefill_N14336_per_group128", "prefill_N14336_per_group32",
                             "moe_decode_T16", "moe_config4", "moe_config5", "moe_config4_group_matmul_direct",
                             "moe_config5_group_matmul_direct"],
                    help="run one of the other configs alone and print its entry (for profiler runs)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy, the known-size kernel that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run")
    ap.add_argument("--no-calib", action="store_true",
                    help="skip the measured ceilings (read-only streaming kernel, pure MFMA loop)")
    ap.add_argument("--calib", action="store_true", help="run the measured ceilings alone and print them")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the path has no multi-GPU part (--gpus must be 1)",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from zendnn_amd import capi, lowoha

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = capi.load()      # raises if the HIP library is not built: there is no fallback
    dev = "cuda:0"
    torch.cuda.set_device(0)
    lib.zmi_set_stream(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    g = torch.Generator(device=dev)
    g.manual_seed(0x5EED0002)

    def prepack(w, K, N, src_dt=capi.DT_S8):
        rp = lowoha.ReorderParams()
        rp.is_prepack = True
        rp.prepack_algo = capi.ALGO_AOCL_DLP_BLOCKED
        rp.prepack_wei_dtype = capi.DT_S8
        rp.prepack_src_dtype = src_dt
        rp.prepack_K, rp.prepack_N, rp.prepack_ldb = K, N, N
        size = lowoha.weight_prepack_size(rp)
        blob = torch.empty(size, dtype=torch.uint8, device=dev)
        assert lowoha.reorder_direct(w, blob, rp) == capi.SUCCESS, lowoha.last_error()
        return blob

    def rand_w(K, N):
        return torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev, generator=g)

    def ev_time(fn, steps, warmup, ramp_ms=30.0):
        """Average milliseconds per call: warmup untimed calls, then `steps` calls between two
        events on the library's stream, synchronised on both sides.  The untimed part lasts at
        least ramp_ms of wall clock whatever `warmup` says: after the set-up the device sits in a
        low power state, and a handful of 15 us calls does not bring its clocks up (20 timed steps
        right after 5 warm-up calls read 25 % slow)."""
        t_end = time.perf_counter() + ramp_ms * 1e-3
        n = 0
        while n < warmup or time.perf_counter() < t_end:
            fn()
            n += 1
            if n % 64 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    # ------------------------------------------------------------ decode (headline)
    def decode_setup(M, n_sets):
        blobs = [prepack(rand_w(K_DEC, N_DEC), K_DEC, N_DEC) for _ in range(n_sets)]
        ws = torch.rand(N_DEC, device=dev, generator=g) * 0.009 + 0.001
        x = torch.randn((M, K_DEC), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((M, N_DEC), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (M, 1))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N_DEC))
        p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        state = {"i": 0}
        # arguments are flattened once per weight set: the timed loop is one foreign call per step
        calls = [lowoha.prepared_matmul("r", False, False, M, N_DEC, K_DEC, 1.0, x, K_DEC, blob, N_DEC, None, 0.0,
                                        dst, N_DEC, True, p)[0] for blob in blobs]

        def step():
            st = calls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        # the GEMM kernel alone: the same call on rows that are already s8 with given scales
        xq = torch.randint(-127, 128, (M, K_DEC), dtype=torch.int8, device=dev, generator=g)
        xs = torch.rand(M, device=dev, generator=g) * 0.02 + 0.01
        pk = lowoha.MatmulParams(src=capi.DT_S8, wei=capi.DT_S8, dst=capi.DT_BF16)
        pk.src_scale = lowoha.QuantParam(xs, capi.DT_F32, (M, 1) if M > 1 else (1,))
        pk.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N_DEC))
        pk.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
        pk.mem_format_b = "r"
        pk.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED

        kcalls = [lowoha.prepared_matmul("r", False, False, M, N_DEC, K_DEC, 1.0, xq, K_DEC, blob, N_DEC, None, 0.0,
                                         dst, N_DEC, True, pk)[0] for blob in blobs]

        def kernel_only():
            st = kcalls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        keep = (blobs, ws, x, dst, xq, xs, calls, kcalls)
        return step, kernel_only, keep

    def decode_bytes(M):
        return K_DEC * N_DEC + M * K_DEC * 2 + N_DEC * 4 + M * N_DEC * 2

    if args.calib_copy:
        ca = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        cb_ = torch.empty_like(ca)
        cb_.copy_(ca)
        torch.cuda.synchronize()
        del ca, cb_
        torch.cuda.empty_cache()

    def run_calib():
        """What this device sustains with nothing in the way (hand-written kernels in csrc/k_calib.hip)."""
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        out = {}
        us = ctypes.c_float()
        span = ctypes.c_float()
        nbytes = K_DEC * N_DEC
        bufs = [torch.randint(-127, 128, (nbytes,), dtype=torch.int8, device=dev, generator=g) for _ in range(8)]
        arr = (ctypes.c_void_p * 8)(*[b.data_ptr() for b in bufs])
        best = None
        for _ in range(3):
            st = lib.zmi_calib_hbm_read(arr, 8, nbytes, 200, 400, stream, ctypes.byref(us), ctypes.byref(span))
            assert st == capi.SUCCESS
            if best is None or us.value < best[0]:
                best = (us.value, span.value)
        out["hbm_read_decode_shape"] = {
            "bytes_per_launch": nbytes, "buffers_rotated": 8, "us_per_launch": round(best[0], 2),
            "GBps": round(nbytes / best[0] / 1e3, 1), "in_kernel_span_us": round(best[1], 2),
            "GBps_in_kernel": round(nbytes / best[1] / 1e3, 1),
            "what": "a kernel that only reads the 58.7 MB of one decode call's weights (448 workgroups x 8 wavefronts x 16 "
                    "requests of 16 B per lane, all in flight), launched back to back over 8 rotating buffers"}
        # the same read with other launch shapes (threads per workgroup, requests per lane): what the best of them
        # reaches is the ceiling a streaming kernel of this size can be held against
        shapes = {}
        for (thr, req) in ((512, 16), (512, 14), (1024, 14), (256, 8), (1024, 8), (512, 8)):
            b2 = None
            for _ in range(2):
                st = lib.zmi_calib_hbm_read_shape(arr, 8, nbytes, thr, req, 200, 400, stream, ctypes.byref(us), ctypes.byref(span))
                assert st == capi.SUCCESS
                if b2 is None or us.value < b2:
                    b2 = us.value
            shapes["%dx%d_threads_x%d_requests" % (nbytes // (thr * req * 16), thr, req)] = round(b2, 2)
        best_shape = min(shapes, key=shapes.get)
        out["hbm_read_best_shape"] = {"shape": best_shape, "us_per_launch": shapes[best_shape],
                                      "GBps": round(nbytes / shapes[best_shape] / 1e3, 1), "all_shapes_us": shapes}
        del bufs
        big = torch.randint(-127, 128, (1 << 30,), dtype=torch.int8, device=dev, generator=g)
        arr1 = (ctypes.c_void_p * 1)(big.data_ptr())
        st = lib.zmi_calib_hbm_read(arr1, 1, 1 << 30, 3, 10, stream, ctypes.byref(us), ctypes.byref(span))
        assert st == capi.SUCCESS
        out["hbm_read_1GiB"] = {"us_per_launch": round(us.value, 1), "GBps": round((1 << 30) / us.value / 1e3, 1)}
        del big
        torch.cuda.empty_cache()
        ops = torch.randint(-127, 128, (6 * 1024,), dtype=torch.int8, device=dev, generator=g)
        tops = ctypes.c_float()
        mhz = ctypes.c_float()
        for name, vary, per_cu in (("constant_operands_1wg_per_cu", 0, 1), ("varying_operands_1wg_per_cu", 1, 1),
                                   ("varying_operands_2wg_per_cu", 1, 2)):
            st = lib.zmi_calib_mfma_i8(ctypes.c_void_p(ops.data_ptr()), vary, per_cu, 6000, stream,
                                       ctypes.byref(tops), ctypes.byref(mhz))
            assert st == capi.SUCCESS
            out["mfma_i8_" + name] = {"TOPS": round(tops.value, 1), "shader_MHz": round(mhz.value, 0),
                                      "pct_of_nominal": round(100 * tops.value / INT8_PEAK_TOPS, 1)}
        out["mfma_i8_what"] = ("a loop of nothing but v_mfma_i32_32x32x32_i8, 4 wavefronts per workgroup on every compute "
                               "unit, about 1 ms per timed launch; 'varying': consecutive instructions get different random int8 operand "
                               "fragments, as in a GEMM on random data (the multipliers' toggling sets the power, the clock follows)")
        return out

    calib = None
    if args.calib or not (args.no_calib or args.only):
        calib = run_calib()
        torch.cuda.empty_cache()
        if args.calib:
            print(json.dumps({"calibration": calib}))
            return

    M = 16
    n_sets = 8
    keep = None
    result = None
    if not args.only:
        step, kernel_only, keep = decode_setup(M, n_sets)
        ms = ev_time(step, args.steps, args.warmup)
        step_kernel = lowoha.last_kernel()
        value = decode_bytes(M) / (ms * 1e-3) / 1e9
        ms_k = ev_time(kernel_only, args.steps, args.warmup)
        gemm_kernel = lowoha.last_kernel()
        # One step is ONE launch: the decode kernel with the per-token quantization inside it (by the
        # workgroups that use the rows, or by quantizing workgroups at the head of the grid).  The timed region
        # above is therefore already "that kernel launched back to back between two events on its stream".
        fused = "fused" in step_kernel or "selfquant" in step_kernel
        achieved = value if fused else None
        # the same kernel on rows that are already s8 (no quantization part), for comparison
        kbytes = K_DEC * N_DEC + M * K_DEC + M * 4 + N_DEC * 4 + M * N_DEC * 2
        gemm_only = kbytes / (ms_k * 1e-3) / 1e9
        if achieved is None:
            achieved = gemm_only

        result = {
            "metric": "decode_int8_gemm_weight_streaming",
            "value": round(value, 1),
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "untimed_ramp_ms": 30.0,
            "ms_per_step": round(ms, 5),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "s8 x s8 -> s32 (f32 epilogue, bf16 store)",
            "data": "synthetic",
            "config": {"workload": "matmul_direct decode: M=16 K=4096 N=14336, bf16 -> per-token s8, "
                                   "prepacked s8 weights, per-channel scales, SiLU, bf16 out",
                       "weight_sets_rotated": n_sets, "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 1)},
            "roofline": {"bound": "hbm", "kernel": ("zmi_gemm_decode16_selfq_kernel: " if "selfquant" in step_kernel and fused
                                                      else "zmi_gemm_decode16_kernel: ") + (step_kernel if fused else gemm_kernel),
                         "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": DECODE_TRAFFIC_BYTES,
                         "traffic_earlier_form_of_the_kernel": DECODE_TRAFFIC_BYTES_EARLIER_FORM,
                         "algorithmic_bytes_per_launch": decode_bytes(M) if fused else kbytes,
                         "avg_launch_us": round((ms if fused else ms_k) * 1e3, 2),
                         "gemm_only": {"kernel": gemm_kernel, "us": round(ms_k * 1e3, 2), "GBps": round(gemm_only, 1),
                                       "algorithmic_bytes": kbytes},
                         "note": "launches timed back to back between two events on the kernel's stream, so the "
                                 "figure includes the dispatch gap; traffic is FETCH_SIZE + WRITE_SIZE per launch "
                                 "from the rocprofv3 --pmc runs summarised under profiles/ (null if not measured "
                                 "for this build)"},
        }
        if calib:
            ceil = max(calib["hbm_read_decode_shape"]["GBps"], calib["hbm_read_best_shape"]["GBps"])
            result["roofline"]["measured_peak"] = {
                "value": ceil, "unit": "GB/s", "frac_of_measured": round(achieved / ceil, 4),
                "gemm_only_frac_of_measured": round(gemm_only / ceil, 4),
                "what": "a kernel that does nothing but read the bytes, over the same 8 rotating buffers, launch to launch: "
                        "the best of the launch shapes tried (calibration.hbm_read_best_shape, .hbm_read_decode_shape)"}
            result["calibration"] = calib

    # ---------------------------------------------------------------- other configs
    def run_decode_m(m):
        s_, k_, kp_ = decode_setup(m, n_sets)
        t = ev_time(s_, 100, 10)
        step_name = lowoha.last_kernel()
        tk = ev_time(k_, 100, 10)
        return {"GBps": round(decode_bytes(m) / (t * 1e-3) / 1e9, 1), "us_per_call": round(t * 1e3, 2),
                "gemm_only_GBps": round((K_DEC * N_DEC + m * K_DEC + m * 4 + N_DEC * 4 + m * N_DEC * 2) / (tk * 1e-3) / 1e9, 1),
                "kernel": step_name, "gemm_only_kernel": lowoha.last_kernel()}

    def run_decode_per_group(m, gs):
        # the decode call with per-group scales: {M,G} source scales computed by the library, {G,N} weight scales,
        # G = K / gs; one launch (the per-group quantization is part of the decode-shaped GEMM launch); bytes = the
        # per-token call's + the scales
        G = K_DEC // gs
        blobs = [prepack(rand_w(K_DEC, N_DEC), K_DEC, N_DEC) for _ in range(n_sets)]
        ws = torch.rand((G, N_DEC), device=dev, generator=g) * 0.009 + 0.001
        x = torch.randn((m, K_DEC), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((m, N_DEC), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (m, G))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (G, N_DEC))
        p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        calls = [lowoha.prepared_matmul("r", False, False, m, N_DEC, K_DEC, 1.0, x, K_DEC, blob, N_DEC, None, 0.0,
                                        dst, N_DEC, True, p)[0] for blob in blobs]
        state = {"i": 0}

        def step():
            st = calls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        t = ev_time(step, 100, 10)
        nbytes = K_DEC * N_DEC + m * K_DEC * 2 + G * N_DEC * 4 + m * G * 4 + m * N_DEC * 2
        return {"GBps": round(nbytes / (t * 1e-3) / 1e9, 1), "us_per_call": round(t * 1e3, 2), "group_size": gs,
                "kernel": lowoha.last_kernel()}

    def run_decode_w4a8(m, gs, per_token):
        # W4A8 decode: bf16 rows quantized by the library ({M,G} scales, or one per row repeated over the groups),
        # packed s4 weights (K*N/2 bytes) with {G,N} scales; the library widens, reorders and caches them on the
        # first call per weight pointer (outside the timed region) and then streams the 4-bit tiles.
        # bytes = the 4-bit weights + rows + scales + output.
        G = K_DEC // gs
        ws4 = [torch.randint(0, 256, (K_DEC * N_DEC // 2,), dtype=torch.uint8, device=dev, generator=g) for _ in range(n_sets)]
        ws = torch.rand((G, N_DEC), device=dev, generator=g) * 0.009 + 0.001
        x = torch.randn((m, K_DEC), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((m, N_DEC), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S4, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (m, 1) if per_token else (m, G))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (G, N_DEC))
        p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
        calls = [lowoha.prepared_matmul("r", False, False, m, N_DEC, K_DEC, 1.0, x, K_DEC, w4, N_DEC, None, 0.0,
                                        dst, N_DEC, True, p)[0] for w4 in ws4]
        state = {"i": 0}

        def step():
            st = calls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        t = ev_time(step, 100, 2 * n_sets)
        nbytes = K_DEC * N_DEC // 2 + m * K_DEC * 2 + G * N_DEC * 4 + m * G * 4 + m * N_DEC * 2
        out = {"GBps": round(nbytes / (t * 1e-3) / 1e9, 1), "us_per_call": round(t * 1e3, 2), "group_size": gs,
               "source_scales": "per token" if per_token else "per group", "kernel": lowoha.last_kernel()}
        capi.load().zmi_clear_weight_cache()
        return out

    def run_decode_woq(m, gs, u4):
        # weight-only quantization at decode: bf16 rows as they are, packed s4 (or u4 with bf16 zero-points) weights with
        # {G,N} scales, dequantized to bf16 in registers in front of the bf16 MFMA; the 4-bit tiles are made and cached
        # on the first call per weight pointer (outside the timed region).  bytes = 4-bit weights + rows + scales
        # (+ zero-points) + output.
        G = K_DEC // gs
        ws4 = [torch.randint(0, 256, (K_DEC * N_DEC // 2,), dtype=torch.uint8, device=dev, generator=g) for _ in range(n_sets)]
        ws = torch.rand((G, N_DEC), device=dev, generator=g) * 0.009 + 0.001
        zp = (torch.rand((G, N_DEC), device=dev, generator=g) * 0.1).to(torch.bfloat16)
        x = torch.randn((m, K_DEC), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((m, N_DEC), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_U4 if u4 else capi.DT_S4, dst=capi.DT_BF16)
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (G, N_DEC))
        if u4:
            p.wei_zp = lowoha.QuantParam(zp, capi.DT_BF16, (G, N_DEC))
        p.postop_ = [lowoha.PostOp(capi.PO_SWISH)]
        calls = [lowoha.prepared_matmul("r", False, False, m, N_DEC, K_DEC, 1.0, x, K_DEC, w4, N_DEC, None, 0.0,
                                        dst, N_DEC, True, p)[0] for w4 in ws4]
        state = {"i": 0}

        def step():
            st = calls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        t = ev_time(step, 100, 2 * n_sets)
        nbytes = K_DEC * N_DEC // 2 + m * K_DEC * 2 + G * N_DEC * (6 if u4 else 4) + m * N_DEC * 2
        out = {"GBps": round(nbytes / (t * 1e-3) / 1e9, 1), "us_per_call": round(t * 1e3, 2), "group_size": gs,
               "weights": "u4, bf16 zero-points" if u4 else "s4", "kernel": lowoha.last_kernel()}
        capi.load().zmi_clear_weight_cache()
        return out

    def run_decode_down(m):
        # the down projection of the same block at decode: K = 14336, N = 4096, bf16 rows quantized per token by the
        # call (a launch of its own), then the 16-row kernel in K slices; bytes = weights + rows + scales + output
        K, N = N_DEC, K_DEC
        blobs = [prepack(rand_w(K, N), K, N) for _ in range(n_sets)]
        ws = torch.rand(N, device=dev, generator=g) * 0.009 + 0.001
        x = torch.randn((m, K), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((m, N), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (m, 1))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        calls = [lowoha.prepared_matmul("r", False, False, m, N, K, 1.0, x, K, blob, N, None, 0.0, dst, N, True, p)[0]
                 for blob in blobs]
        state = {"i": 0}

        def step():
            st = calls[state["i"] % n_sets]()
            state["i"] += 1
            if st != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())

        t = ev_time(step, 100, 10)
        nbytes = K * N + m * K * 2 + m * 4 + N * 4 + m * N * 2
        return {"GBps": round(nbytes / (t * 1e-3) / 1e9, 1), "us_per_call": round(t * 1e3, 2), "kernel": lowoha.last_kernel()}

    def run_prefill(N, gs=None):
        # config 3: whole call = per-token quantization launch (rows written in MFMA fragment order) + GEMM launch;
        # the per-kernel split is in the rocprofv3 summaries under profiles/
        # gs: per-group scales instead ({M, K/gs} source scales computed by the call, {K/gs, N} weight scales)
        Mp, K = 2048, 4096
        blob = prepack(rand_w(K, N), K, N)
        ws = torch.rand(N if gs is None else (K // gs, N), device=dev, generator=g) * 0.009 + 0.001
        bias = torch.randn(N, device=dev, generator=g) * 0.1
        x = torch.randn((Mp, K), device=dev, generator=g).to(torch.bfloat16)
        dst = torch.zeros((Mp, N), dtype=torch.bfloat16, device=dev)
        p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, bias=capi.DT_F32, compute=capi.DT_S8)
        p.dynamic_quant = True
        p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (Mp, 1) if gs is None else (Mp, K // gs))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N) if gs is None else (K // gs, N))
        p.postop_ = [lowoha.PostOp(capi.PO_GELU_TANH)]
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        t = ev_time(lambda: lowoha.matmul_direct("r", False, False, Mp, N, K, 1.0, x, K, blob, N, bias, 0.0, dst, N, True, p), 30, 5)
        ops = 2.0 * Mp * N * K
        r = {"TOPS_whole_call": round(ops / (t * 1e-3) / 1e12, 1),
             "pct_of_int8_mfma_peak": round(100 * ops / (t * 1e-3) / 1e12 / INT8_PEAK_TOPS, 1),
             "us_whole_call": round(t * 1e3, 1), "kernel": lowoha.last_kernel()}
        if calib:
            r["pct_of_measured_mfma_loop"] = round(100 * ops / (t * 1e-3) / 1e12 /
                                                   calib["mfma_i8_varying_operands_1wg_per_cu"]["TOPS"], 1)
        return r

    def run_config1():
        Mc, K, N = 128, 4096, 4096
        blobs = [prepack(rand_w(K, N), K, N, capi.DT_U8) for _ in range(20)]
        a = torch.randint(0, 256, (Mc, K), dtype=torch.uint8, device=dev, generator=g)
        ws = torch.rand(N, device=dev, generator=g) * 0.009 + 0.001
        bias = torch.randn(N, device=dev, generator=g)
        dst = torch.zeros((Mc, N), dtype=torch.float32, device=dev)
        ss = np.array([0.02], dtype=np.float32)
        zp = np.array([128], dtype=np.int32)
        p = lowoha.MatmulParams(src=capi.DT_U8, wei=capi.DT_S8, dst=capi.DT_F32, bias=capi.DT_F32)
        p.src_scale = lowoha.QuantParam(ss.ctypes.data, capi.DT_F32, (1,))
        p.src_zp = lowoha.QuantParam(zp.ctypes.data, capi.DT_S32, (1,))
        p.wei_scale = lowoha.QuantParam(ws, capi.DT_F32, (1, N))
        p.mem_format_b = "r"
        p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
        st = {"i": 0}

        def c1():
            b = blobs[st["i"] % len(blobs)]
            st["i"] += 1
            lowoha.matmul_direct("r", False, False, Mc, N, K, 1.0, a, K, b, N, bias, 0.0, dst, N, True, p)
        t = ev_time(c1, 100, 10)
        return {"us_per_call": round(t * 1e3, 2), "GBps": round(19431424 / (t * 1e-3) / 1e9, 1),
                "TOPS": round(2.0 * Mc * N * K / (t * 1e-3) / 1e12, 1), "kernel": lowoha.last_kernel()}

    def run_moe(T, Hd, I, E, topk, skew):
        # configs 4 and 5: tokens/s through the device-routed fused block
        w13 = [prepack(rand_w(Hd, 2 * I), Hd, 2 * I) for _ in range(E)]
        w2 = [prepack(rand_w(I, Hd), I, Hd) for _ in range(E)]
        s13 = [torch.rand(2 * I, device=dev, generator=g) * 0.009 + 0.001 for _ in range(E)]
        s2 = [torch.rand(Hd, device=dev, generator=g) * 0.009 + 0.001 for _ in range(E)]
        x = torch.randn((T, Hd), device=dev, generator=g).to(torch.bfloat16)
        logits = torch.randn((T, E), device=dev, generator=g)
        if skew:
            logits = logits + torch.randn(E, device=dev, generator=g) * 1.5
        prob = torch.softmax(logits, dim=1)
        tw, ids = torch.topk(prob, topk, dim=1)
        ids = ids.to(torch.int32).contiguous()
        tw = tw.contiguous()
        out = torch.zeros((T, Hd), dtype=torch.bfloat16, device=dev)

        def moe():
            r = lowoha.moe_fused_device(x, ids, tw, w13, w2, s13, s2, I, capi.ACT_SILU_AND_MUL, out)
            if r != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())
        t = ev_time(moe, 10, 3)
        cnt = torch.bincount(ids.flatten().long(), minlength=E)
        ops = 2.0 * T * topk * 3 * Hd * I
        touched = int((cnt > 0).sum())
        return {"tokens_per_s": round(T / (t * 1e-3), 0), "ms_per_call": round(t, 4),
                "TOPS": round(ops / (t * 1e-3) / 1e12, 1),
                "weight_GBps": round(touched * 3 * Hd * I / (t * 1e-3) / 1e9, 1),
                "expert_rows_min_max": [int(cnt.min()), int(cnt.max())],
                "experts_under_8_rows": int((cnt < 8).sum()), "experts_over_1000_rows": int((cnt > 1000).sum())}

    def run_moe_group_api(T, Hd, I, E, topk, skew):
        # the same block through the reference-shaped entry point, group_matmul_direct with fused_moe + moe_postop
        # (lowoha_matmul.hpp:204-223): the caller scatters the tokens into one source matrix per expert and builds
        # row_ptrs outside the timed region, as a framework does once per routing
        # (benchdnn/grp_matmul/grp_matmul_benchdnn.cpp:625-712); the call uploads its pointer tables every time
        w13 = [prepack(rand_w(Hd, 2 * I), Hd, 2 * I) for _ in range(E)]
        w2 = [prepack(rand_w(I, Hd), I, Hd) for _ in range(E)]
        s13 = [torch.rand(2 * I, device=dev, generator=g) * 0.009 + 0.001 for _ in range(E)]
        s2 = [torch.rand(Hd, device=dev, generator=g) * 0.009 + 0.001 for _ in range(E)]
        x = torch.randn((T, Hd), device=dev, generator=g).to(torch.bfloat16)
        logits = torch.randn((T, E), device=dev, generator=g)
        if skew:
            logits = logits + torch.randn(E, device=dev, generator=g) * 1.5
        tw, ids = torch.topk(torch.softmax(logits, dim=1), topk, dim=1)
        tw = tw.contiguous()
        ids_h = ids.cpu().numpy()
        rows_of = [[] for _ in range(E)]
        slot = {}
        for t in range(T):
            for k in range(topk):
                e = int(ids_h[t, k])
                slot[(t, k)] = (e, len(rows_of[e]))
                rows_of[e].append(t)
        Ms = [len(r) for r in rows_of]
        src = [x.index_select(0, torch.tensor(r, dtype=torch.long, device=dev)).contiguous() if r else None for r in rows_of]
        dst_down = [torch.zeros((m, Hd), dtype=torch.bfloat16, device=dev) if m else None for m in Ms]
        out = torch.zeros((T, Hd), dtype=torch.bfloat16, device=dev)
        row_ptrs = []
        for t in range(T):
            for k in range(topk):
                e, j = slot[(t, k)]
                row_ptrs.append(dst_down[e].data_ptr() + j * Hd * 2)
        params = []
        for e in range(E):
            p = lowoha.MatmulParams(src=capi.DT_BF16, wei=capi.DT_S8, dst=capi.DT_BF16, compute=capi.DT_S8)
            p.dynamic_quant = True
            p.src_scale = lowoha.QuantParam(None, capi.DT_F32, (Ms[e], 1))
            p.wei_scale = lowoha.QuantParam(s13[e], capi.DT_F32, (1, 2 * I))
            p.mem_format_b = "r"
            p.lowoha_algo = capi.ALGO_AOCL_DLP_BLOCKED
            params.append(p)
        fm = lowoha.FusedMoe(down_weight=w2, N_down=[Hd] * E, ldb_down=[Hd] * E,
                             down_scale=[lowoha.QuantParam(s2[e], capi.DT_F32, (1, Hd)) for e in range(E)],
                             dst_down=dst_down, ldc_down=[Hd] * E)
        pp = lowoha.MoePostop(T, topk, out, Hd, tw, row_ptrs)
        call, keep_ = lowoha.prepared_group_matmul(
            ["r"] * E, [False] * E, [False] * E, Ms, [2 * I] * E, [Hd] * E, [1.0] * E, src, [Hd] * E, w13, [2 * I] * E,
            [None] * E, [0.0] * E, [None] * E, [2 * I] * E, [True] * E, params, moe_postop=pp,
            gated_act=capi.ACT_SILU_AND_MUL, fused_moe=fm)

        def moe():
            if call() != capi.SUCCESS:
                raise RuntimeError(lowoha.last_error())
        t = ev_time(moe, 10, 3)
        touched = sum(1 for m in Ms if m > 0)
        return {"tokens_per_s": round(T / (t * 1e-3), 0), "ms_per_call": round(t, 4),
                "TOPS": round(2.0 * T * topk * 3 * Hd * I / (t * 1e-3) / 1e12, 1),
                "weight_GBps": round(touched * 3 * Hd * I / (t * 1e-3) / 1e9, 1),
                "entry": "zmi_group_matmul_direct (fused_moe + moe_postop; tokens scattered and row_ptrs built by the caller "
                         "outside the timed region)"}

    extras = {
        "decode_M1": lambda: run_decode_m(1),
        "decode_M4": lambda: run_decode_m(4),
        # the same call with more rows than a decode step proper: 16-row groups of the decode kernel
        # (64 rows) and the K-sliced large-M kernel (128 rows)
        "decode_M64": lambda: run_decode_m(64),
        "decode_M128": lambda: run_decode_m(128),
        "decode_M16_per_group128": lambda: run_decode_per_group(16, 128),
        "decode_M16_per_group32": lambda: run_decode_per_group(16, 32),
        "decode_M16_w4a8_group128": lambda: run_decode_w4a8(16, 128, False),
        "decode_M16_w4a8_group128_per_token_rows": lambda: run_decode_w4a8(16, 128, True),
        "decode_M16_woq_s4_group128": lambda: run_decode_woq(16, 128, False),
        "decode_M16_woq_u4_group128": lambda: run_decode_woq(16, 128, True),
        "decode_M1_woq_s4_group128": lambda: run_decode_woq(1, 128, False),
        "prefill_N4096": lambda: run_prefill(4096),
        "prefill_N14336": lambda: run_prefill(14336),
        "config1_u8s8_M128": run_config1,
        "decode_M16_K14336_N4096": lambda: run_decode_down(16),
        # config 3's shape with per-group scales (the VALU-bound tiled kernel: every group's sums are scaled and added in f32)
        "prefill_N14336_per_group128": lambda: run_prefill(14336, 128),
        "prefill_N14336_per_group32": lambda: run_prefill(14336, 32),
        # a decode step of configuration 4's block: 16 tokens, every expert has a handful of rows (decode-shaped grouped kernel)
        "moe_decode_T16": lambda: run_moe(16, 4096, 14336, 8, 2, False),
        "moe_config4": lambda: run_moe(512, 4096, 14336, 8, 2, False),
        "moe_config5": lambda: run_moe(4096, 2048, 1408, 64, 6, True),
        "moe_config4_group_matmul_direct": lambda: run_moe_group_api(512, 4096, 14336, 8, 2, False),
        "moe_config5_group_matmul_direct": lambda: run_moe_group_api(4096, 2048, 1408, 64, 6, True),
    }
    if args.only:
        # one of the other configs alone (the form the profiler runs use); prints its entry only
        print(json.dumps({args.only: extras[args.only]()}))
        return

    if not args.no_extras:
        other = {}
        del keep
        torch.cuda.empty_cache()
        for name, fn in extras.items():
            other[name] = fn()
            torch.cuda.empty_cache()
        result["other_configs"] = other
        # the MFMA-bound kernel of the path (BASELINE config 3) beside the HBM-bound headline
        pf = other["prefill_N14336"]
        result["roofline"]["mfma"] = {
            "bound": "mfma", "workload": "matmul_direct prefill: M=2048 K=4096 N=14336, bf16 -> per-token s8, bias, GELU-tanh, bf16 out "
                                         "(whole call: quantization launch + GEMM launch)",
            "kernel": pf["kernel"], "achieved": pf["TOPS_whole_call"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
            "frac": round(pf["TOPS_whole_call"] / INT8_PEAK_TOPS, 4), "us_whole_call": pf["us_whole_call"],
            "measured_peak": ({"value": calib["mfma_i8_varying_operands_1wg_per_cu"]["TOPS"], "unit": "TOP/s",
                               "frac_of_measured": round(pf["TOPS_whole_call"] / calib["mfma_i8_varying_operands_1wg_per_cu"]["TOPS"], 4),
                               "what": "a loop of nothing but v_mfma_i32_32x32x32_i8 on random operands on every compute unit "
                                       "(calibration.mfma_i8_varying_operands_1wg_per_cu): the rate the power limit leaves"}
                              if calib else None),
            "N4096": other["prefill_N4096"]}

        # ------------------------------------------------------ CPU baseline (oracle port)
        from oracle import build as obuild, oracle as zo
        obuild.build(force=False)
        rng = np.random.default_rng(1)
        L = zo.lib()
        L.zo_omp_threads.restype = ctypes.c_int32
        cores = int(L.zo_omp_threads())     # threads the port's OpenMP regions really run on

        def cpu_gemm(Mb, Nb, Kb, po, seconds):
            A = rng.integers(-127, 128, (Mb, Kb), dtype=np.int8)
            Bt = rng.integers(-127, 128, (Nb, Kb), dtype=np.int8)   # pre-transposed: the packed form of the CPU path
            sa = rng.uniform(0.01, 0.03, Mb).astype(np.float32)
            sb = rng.uniform(0.001, 0.01, Nb).astype(np.float32)
            out = np.zeros((Mb, Nb), dtype=np.uint16)

            def call():
                L.zo_bench_s8_gemm(A.ctypes.data, Bt.ctypes.data, sa.ctypes.data, sb.ctypes.data, Mb, Nb, Kb, po,
                                   out.ctypes.data)
            call()
            t0 = time.perf_counter()
            n = 0
            while time.perf_counter() - t0 < seconds:
                call()
                n += 1
            return (time.perf_counter() - t0) / n, n

        dt, n = cpu_gemm(16, N_DEC, K_DEC, capi.PO_SWISH, 8.0)
        cb = K_DEC * N_DEC + 16 * K_DEC + 16 * 4 + N_DEC * 4 + 16 * N_DEC * 2
        result["cpu_baseline"] = {"value": round(cb / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                                  "sample": f"{n} calls of the same M=16 K=4096 N=14336 s8 x s8 GEMM + scales + SiLU + bf16 "
                                            f"store through the oracle's OpenMP port (about 8 s); not AOCL-DLP",
                                  "ms_per_call": round(dt * 1e3, 3)}
        # the other workloads, each on a bounded sample through the same port
        dtp, n = cpu_gemm(64, 4096, 4096, capi.PO_GELU_TANH, 5.0)
        dtm1, n1 = cpu_gemm(32, 28672, 4096, 0, 4.0)
        dtm2, n2 = cpu_gemm(32, 4096, 14336, 0, 3.0)
        result["cpu_baseline"]["other_workloads"] = {
            "prefill_N4096": {"TOPS": round(2.0 * 64 * 4096 * 4096 / dtp / 1e12, 3), "cores": cores,
                              "sample": f"{n} calls on 64 of the 2048 rows (GEMM + scales + GELU-tanh + bf16 store); rows are independent"},
            "moe_config4": {"tokens_per_s": round(16 / (dtm1 + dtm2), 1), "cores": cores,
                            "sample": f"the two GEMMs of one expert on the 32 routed rows of 16 tokens ({n1} + {n2} calls; "
                                      "4096 -> 28672 and 14336 -> 4096), without activation, re-quantization and reduce"}}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
    # leave nothing behind: no worker thread of the BLAS / OpenMP pools or of the runtime keeps the process alive once
    # the line is out (a profiler that writes its files when the process exits normally gets the normal exit)
    sys.stdout.flush()
    sys.stderr.flush()
    profiled = any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ) or "rocprof" in os.environ.get("LD_PRELOAD", "")
    if not profiled:
        os._exit(0)
