"""The committed golden fixtures (tests/golden/golden.json, golden_bf16.npz; written by tests/golden/make_golden.py from
the CPU oracle) against the oracle as it is now (CPU) and against the HIP path through the C ABI (GPU): one reduced
case per BASELINE configuration plus per-group scales, GGML Q8_0, W4A8 and the dequantized weights of the weight-only path.  Bit-exact outputs are compared by SHA-256,
activation outputs within one bf16 unit in the last place (two for the fused MoE block, whose re-quantized
intermediate may move by one count)."""
import json
import os

import numpy as np
import pytest

from tests import gpu_helpers as H
from tests.golden import cases

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
META = json.load(open(os.path.join(HERE, "golden.json")))
BF16 = np.load(os.path.join(HERE, "golden_bf16.npz"))


def _check(name, outs, exact_only=False):
    assert set(outs) == set(META[name])
    for key, (arr, mode) in outs.items():
        want = META[name][key]
        arr = np.ascontiguousarray(arr)
        assert list(arr.shape) == want["shape"] and str(arr.dtype) == want["dtype"], (name, key)
        if mode == cases.EXACT or exact_only:
            assert cases.sha(arr) == want["sha256"], (name, key)
        else:
            ref = BF16[name + "/" + key]
            if name.startswith("cfg4") or name.startswith("cfg5"):
                d = H.bf16_ulp_diff(arr, ref)
                assert d.max() <= 2 and (d > 1).mean() <= 1e-4, (name, key, int(d.max()))
            else:
                H.check_bf16(arr, ref, max_frac=5e-3, atol=1e-6 if name == "cfg3_prefill" else 0.0)


@pytest.mark.parametrize("name", list(cases.CASES))
def test_oracle_reproduces_the_golden_outputs(zo, name):
    _check(name, cases.run(name, "cpu", zo), exact_only=True)


def test_oracle_reproduces_the_bf16_table_and_the_quantization_ties(zo):
    for tag, fn in (("bf16_table", cases.bf16_table), ("quant_ties", cases.quant_ties)):
        got = fn(zo)
        assert set(got) == set(META[tag])
        for k, v in got.items():
            assert cases.sha(v) == META[tag][k]["sha256"], (tag, k)
    # the ties themselves, spelled out: scale 1, 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, 3.5 -> 4 (half to even); non-finite -> 0
    q, s = cases.quant_ties(zo)["q"], cases.quant_ties(zo)["scales"]
    assert s[0] == 1.0 and q[0, 1:8].tolist() == [0, 1, 2, 2, 2, 3, 4]
    assert q[1, 1:8].tolist() == [0, -1, -2, -2, -2, -3, -4]
    assert q[2, :8].tolist() == [0, 0, 0, 2, -4, 4, 127, 0]
    assert s[3] == np.float32(1e-10) and not q[3].any()


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.CASES))
def test_hip_path_matches_the_golden_outputs(name):
    _check(name, cases.run(name, "gpu"))
