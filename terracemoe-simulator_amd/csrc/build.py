"""Builds libterrace_hip.so for gfx950 with hipcc alone (no torch headers).

    python terracemoe-simulator_amd/csrc/build.py [--force]

Sources are compiled one translation unit per process, in parallel; the library lands in
terracemoe-simulator_amd/lib/ where the ``terrace`` package looks for it.
"""
from __future__ import annotations

import glob
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(os.path.dirname(HERE), "lib")
OBJ_DIR = os.path.join(HERE, "build")
SOURCES = ["rows.hip", "sort.hip", "pack.hip", "expand.hip", "route.hip", "noalloc.hip", "api.hip"]
LIB = os.path.join(LIB_DIR, "libterrace_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
    "-I", os.path.join(ROOT, "include"), "-I", HERE,
    "-Wall", "-Wno-unused-function",
]


def source_hash() -> str:
    """Digest of everything the library is compiled from; build() stamps it into the library
    (terrace_version() ends with it) so that a library older than its sources can be told apart."""
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(HERE, "*.hip")) + glob.glob(os.path.join(HERE, "*.hpp")) +
                   glob.glob(os.path.join(ROOT, "include", "*.h")))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    stamp = [f'-DTERRACE_SOURCE_HASH="{source_hash()}"'] if src == "api.hip" else []
    cmd = [HIPCC, *FLAGS, *stamp, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
