"""Builds the CPU oracle (test infrastructure) into oracle/libzmi_oracle.so.

The reference's own implementation of this path cannot be compiled here: its
arithmetic lives in AOCL-DLP, which the reference fetches over the network at
configure time and does not vendor, and its common layer needs aocl-utils
headers that are absent too.  So there is no oracle/_ref build; the oracle is
the restatement in zmi_oracle.c, pinned by tests/test_oracle_*.py.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "zmi_oracle.c")
OUT = os.path.join(HERE, "libzmi_oracle.so")


def build(force=True):
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = ["gcc", "-O3", "-ffp-contract=off", "-fopenmp", "-fvisibility=hidden", "-shared",
           "-fPIC", "-Wall", "-o", OUT, SRC, "-lm"]
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build())
