"""Compiles the gfx950 kernels and the C ABI into zendnn_amd/lib/libzmi_lowoha.so
and the C++ adapter into zendnn_amd/lib/libzendnnl_mi355x.so.

hipcc cross-compiles for gfx950 without a GPU.  Every translation unit is
compiled on its own (in parallel) and the objects are linked once.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")

HIP_SOURCES = ["k_prepack.hip", "k_quant.hip", "k_ring.hip", "k_pring.hip", "k_smallm.hip", "k_decode.hip", "k_pergroup.hip", "k_moe.hip", "k_util.hip", "k_calib.hip", "k_group_decode.hip", "k_router.hip", "k_stream.hip", "k_pgring.hip", "k_woq.hip", "k_asym.hip",
               "zmi_host.hip", "zmi_api.hip", "zmi_api_group.hip", "zmi_api_noalloc.hip", "zmi_api_woq.hip"]
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-ffp-contract=off", "-Wall", "-Wno-unused-function"]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    return r


def _newest_header():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(HERE, "..", "include", "zmi_lowoha.h"))
    return max(os.path.getmtime(h) for h in hs)


def build(verbose=False, force=True):
    """force=False recompiles only translation units older than their source or any header."""
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    objs = []
    jobs = []
    hdr = _newest_header()
    for src in HIP_SOURCES:
        obj = os.path.join(OBJDIR, src + ".o")
        objs.append(obj)
        path = os.path.join(CSRC, src)
        if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), hdr):
            continue
        jobs.append(["hipcc"] + HIPCC_FLAGS + ["-c", path, "-o", obj])
    if jobs:
        with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
            list(ex.map(_run, jobs))
    lib = os.path.join(LIBDIR, "libzmi_lowoha.so")
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    # C++ adapter: plain g++, sees only the C ABI header
    host_src = os.path.join(HOST, "lowoha_adapter.cpp")
    host_lib = os.path.join(LIBDIR, "libzendnnl_mi355x.so")
    if os.path.exists(host_src):
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(HERE, "..", "include"),
              "-I", HOST, host_src, "-o", host_lib, "-L", LIBDIR, "-lzmi_lowoha", "-Wl,-rpath,$ORIGIN"])
        # C++ usage example / adapter test (host code only; hipcc for the HIP runtime headers)
        ex_src = os.path.join(HERE, "..", "tests", "cpp", "adapter_example.cpp")
        if os.path.exists(ex_src):
            _run(["hipcc", "-O1", "-std=c++17", "-w", "-I", HOST, "-I", os.path.join(HERE, "..", "include"), ex_src,
                  "-o", os.path.join(LIBDIR, "adapter_example"), "-L", LIBDIR, "-lzendnnl_mi355x", "-lzmi_lowoha",
                  "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", lib)
    return lib


if __name__ == "__main__":
    build(verbose=True, force="--force" in sys.argv)
