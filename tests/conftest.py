"""Shared test plumbing: import paths, the ``gpu`` marker, seeded routing generators."""
from __future__ import annotations

import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "terracemoe-simulator_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm device (run on the MI355X box)")


def pytest_sessionstart(session):
    """A library built before its sources were last edited must not be tested (least of all on a GPU, where
    a kernel that lacks a check its test relies on can fault the card): build.py stamps the digest of the
    sources into the library, and the session stops here when the two differ."""
    import glob
    import importlib.util
    import re
    libs = sorted(glob.glob(os.path.join(PKG, "lib", "libterrace_hip*.so")))
    if not libs or os.environ.get("TERRACE_OPS_LIB"):
        return
    spec = importlib.util.spec_from_file_location("terrace_build", os.path.join(PKG, "csrc", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    # read the stamp out of the file: loading a HIP library here, before torch has brought in the HIP runtime it
    # ships, would bind the library to another copy of the runtime and every launch would fail
    with open(libs[0], "rb") as f:
        found = re.search(rb"\(gfx950\) src:([0-9a-z]+)", f.read())
    stamped = found.group(1).decode() if found else "none"
    if stamped != build.source_hash():
        pytest.exit(f"{libs[0]} was built from other sources (stamp {stamped}, sources {build.source_hash()}): "
                    f"run python terracemoe-simulator_amd/csrc/build.py", returncode=3)


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:                                   # pragma: no cover
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no ROCm device in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def literals():
    with open(os.path.join(ROOT, "tests", "golden", "reference_literals.json")) as f:
        return json.load(f)


def equal_quota_routing(T, k, n_experts, n_nodes, m, seed, sort_rows=False):
    """Seeded routing with exactly ``m`` nodes per token and ``k//m`` experts on each
    (the generator shape of the reference's tests/test_terrace_k2_ref.py:64-75)."""
    rng = np.random.default_rng(seed)
    per, quota = n_experts // n_nodes, k // m
    out = np.empty((T, k), dtype=np.int64)
    for t in range(T):
        nodes = rng.permutation(n_nodes)[:m]
        out[t] = np.concatenate([a * per + rng.permutation(per)[:quota] for a in nodes])
    return np.sort(out, axis=1) if sort_rows else out


def arrival_plane(R, quota, epr, rpn, seed, degenerate=False):
    """Seeded arrival slot table: ascending distinct slot ids per row, or all-zero rows
    (input shape of the reference's tests/test_terrace_k1_arrival.py:84-99)."""
    rng = np.random.default_rng(seed)
    slots = epr * rpn
    if degenerate:
        return np.zeros((R, quota), dtype=np.int64)
    out = np.empty((R, quota), dtype=np.int64)
    for r in range(R):
        out[r] = np.sort(rng.permutation(slots)[:quota])
    return out
