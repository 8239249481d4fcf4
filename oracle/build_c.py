"""Builds the C restatement of the oracle (oracle/terrace_oracle.c) into oracle/_c/libterrace_oracle.so.

    python oracle/build_c.py

Test infrastructure: the library is the multi-core CPU baseline of bench.py and a second checker.
"""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_c")
LIB = os.path.join(OUT_DIR, "libterrace_oracle.so")


def build(verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    cmd = ["gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-ffp-contract=off", "-fno-fast-math", "-shared", "-fPIC",
           "-fvisibility=hidden", "-Wall", "-o", LIB, os.path.join(HERE, "terrace_oracle.c"), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode:
        raise RuntimeError(f"gcc failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
