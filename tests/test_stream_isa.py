"""Build-time checks of the weight-traffic-bound grouped kernel's machine code (no GPU needed).

k_stream.hip issues its weight loads by hand (inline asm) and waits for them by count, so the compiler does not know
that a loaded register is not valid until that wait.  That is sound only while the compiler neither copies nor reuses
such a register between the load's issue and its use, and while nothing spills: with spills it might move exactly those
registers.  Both are properties of the generated code, so they are checked on the generated code: every stream kernel
must have no scratch and no spilled registers, and between the first hand-issued load and the final wait nothing but
MFMAs may touch a register that a hand-issued load has targeted."""
import os
import re
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "zendnn_amd", "csrc")


def _compile(source):
    from zendnn_amd import build
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, source.replace(".hip", ".s"))
        flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC"]
        cmd = ["hipcc"] + flags + ["-I", os.path.join(HERE, "..", "include"), "-S", "--cuda-device-only",
                                   os.path.join(CSRC, source), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        return open(out).read()


@pytest.fixture(scope="module")
def isa():
    return _compile("k_stream.hip")


@pytest.fixture(scope="module")
def isa_pgring():
    return _compile("k_pgring.hip")


def _kernels(isa):
    parts = re.split(r"\n(?=_Z22zmi_gemm_stream_kernel)", isa)[1:]
    assert len(parts) >= 4
    return [(p.split(":")[0], p.split("s_endpgm")[0]) for p in parts]


def test_no_scratch_and_no_spills(isa):
    names = re.findall(r"\.name:\s+(_Z22zmi_gemm_stream_kernel\S+)", isa)
    assert len(names) >= 4
    for meta in re.split(r"\n\s*- \.agpr_count", isa)[1:]:
        m = re.search(r"\.name:\s+(\S+)", meta)
        if not m or "zmi_gemm_stream_kernel" not in m.group(1):
            continue
        assert int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", meta).group(1)) == 0, m.group(1)
        assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", meta).group(1)) == 0, m.group(1)
        assert int(re.search(r"\.sgpr_spill_count:\s+(\d+)", meta).group(1)) == 0, m.group(1)


def test_in_flight_registers_are_touched_by_mfmas_only(isa):
    for name, body in _kernels(isa):
        i0 = body.index("global_load_dwordx4 v[")
        i1 = body.index("s_waitcnt vmcnt(0)", i0)
        inflight = set()
        n_loads = 0
        for line in body[i0:i1].split("\n"):
            line = line.strip()
            if not line or line[0] in ";." or line.endswith(":"):
                continue
            m = re.match(r"global_load_dwordx4 v\[(\d+):(\d+)\], v(\d+)", line)
            if m:
                inflight.update(range(int(m.group(1)), int(m.group(2)) + 1))
                n_loads += 1
                continue
            op, _, rest = line.partition(" ")
            regs = set()
            for m in re.finditer(r"\bv\[(\d+):(\d+)\]", rest):
                regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
            for m in re.finditer(r"\bv(\d+)\b", rest):
                regs.add(int(m.group(1)))
            assert not (regs & inflight) or op.startswith("v_mfma"), f"{name}: {line}"
        assert n_loads >= 16 and len(inflight) >= 64, name


def test_pergroup_tiled_kernel_has_no_spills_and_interleaves_its_fold(isa_pgring):
    """k_pgring.hip: two wavefronts share a SIMD, so every variant must fit 256 registers without scratch (a spill in
    the k loop costs more than the kernel gains); and in the variants that fold every block, the loop must issue
    the fold's VALU instructions between the MFMAs (never two MFMAs in a row, never a run of 3 x 64 fold
    instructions): that order is what lets the MFMAs run under the fold."""
    metas = [m for m in re.split(r"\n\s*- \.agpr_count", isa_pgring)[1:] if "zmi_gemm_pgring_kernel" in m]
    assert len(metas) == 8
    for meta in metas:
        name = re.search(r"\.name:\s+(\S+)", meta).group(1)
        assert int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", meta).group(1)) == 0, name
        assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", meta).group(1)) == 0, name
        assert int(re.search(r"\.vgpr_count:\s+(\d+)", meta).group(1)) <= 256, name
    bodies = re.split(r"\n(?=_Z22zmi_gemm_pgring_kernel)", isa_pgring)[1:]
    checked = 0
    for body in bodies:
        name = body.split(":")[0]
        if "Lb1E" in name:          # groups of several blocks: the fold is not pipelined
            continue
        body = body.split("s_endpgm")[0]
        start = body.index("Inner Loop Header")
        loop = body[start:body.index("s_cbranch_scc", start)]
        ops = [ln.split()[0] for ln in loop.split("\n") if ln.startswith("\t") and ln.strip() and not ln.strip().startswith(";")]
        seq = [o for o in ops if o.startswith("v_mfma") or o.startswith(("v_cvt_f32_i32", "v_mul_f32", "v_add_f32"))]
        run_valu = run_mfma = worst_valu = worst_mfma = 0
        for o in seq:
            if o.startswith("v_mfma"):
                run_mfma += 1
                run_valu = 0
            else:
                run_valu += 1
                run_mfma = 0
            worst_valu, worst_mfma = max(worst_valu, run_valu), max(worst_mfma, run_mfma)
        assert sum(o.startswith("v_mfma") for o in seq) in (8, 16), name
        assert worst_mfma == 1 and worst_valu <= 64, (name, worst_mfma, worst_valu)
        checked += 1
    assert checked == 6
