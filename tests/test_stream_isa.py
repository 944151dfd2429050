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


@pytest.fixture(scope="module")
def isa():
    from zendnn_amd import build
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k_stream.s")
        flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC"]
        cmd = ["hipcc"] + flags + ["-I", os.path.join(HERE, "..", "include"), "-S", "--cuda-device-only",
                                   os.path.join(CSRC, "k_stream.hip"), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        return open(out).read()


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
