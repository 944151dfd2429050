"""Writes tests/golden/golden.json (+ golden_bf16.npz) from the CPU oracle:  python -m tests.golden.make_golden
Bit-exact outputs are stored as SHA-256 of their bytes with shape and dtype; outputs the GPU may round differently in
the last place (activations) as bf16 bit patterns."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def main():
    from oracle import build, oracle as zo
    from tests.golden import cases
    build.build(force=False)
    meta, arrays = {}, {}
    for name in cases.CASES:
        meta[name] = {}
        for key, (arr, mode) in cases.run(name, "cpu", zo).items():
            arr = np.ascontiguousarray(arr)
            meta[name][key] = {"mode": mode, "shape": list(arr.shape), "dtype": str(arr.dtype), "sha256": cases.sha(arr)}
            if mode == cases.BF16_ULP:
                arrays[name + "/" + key] = arr
    for fn, tag in ((cases.bf16_table, "bf16_table"), (cases.quant_ties, "quant_ties")):
        meta[tag] = {k: {"mode": cases.EXACT, "shape": list(v.shape), "dtype": str(v.dtype), "sha256": cases.sha(v)}
                     for k, v in fn(zo).items()}
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
        f.write("\n")
    np.savez_compressed(os.path.join(HERE, "golden_bf16.npz"), **arrays)
    print("wrote", len(meta), "cases;", sum(a.nbytes for a in arrays.values()), "bytes of bf16 outputs")


if __name__ == "__main__":
    main()
