"""The oracle against its committed fixture: tests/golden/oracle_digests.json holds the digest of every plane of
the path for six formula-made cases (tests/golden_cases.py).  A change of the oracle that moves any bit of any
plane shows here, whatever the kernels do; the GPU suite holds the kernels to the same file."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import golden_cases as gc

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def digests():
    with open(os.path.join(HERE, "golden", "oracle_digests.json")) as f:
        return json.load(f)


def test_inputs_are_the_same_bits_everywhere():
    """The generator is integer arithmetic only; three spot values pin it."""
    c = gc.inputs("reference_shape")
    assert c["logits"].dtype == np.float32 and c["logits"].shape == (192, 64)
    assert gc.digest(c["logits"]) == gc.digest(gc.inputs("reference_shape")["logits"])
    assert float(np.abs(c["logits"]).max()) <= 0.5 and len(np.unique(c["logits"])) > 12000
    assert [int(v) for v in (c["logits"][:2, :2] * (1 << 24)).astype(np.int64).reshape(-1)] == \
           [int(v) for v in (gc._mixed(2, 2, 1) * (1 << 24)).astype(np.int64).reshape(-1)]


@pytest.mark.parametrize("name", list(gc.CASES))
def test_oracle_reproduces_its_fixture(name, digests):
    planes = gc.oracle_planes(name)
    assert sorted(planes) == sorted(digests[name]), "the set of planes changed: regenerate the fixture on purpose"
    wrong = [k for k, v in planes.items() if gc.digest(v) != digests[name][k]]
    assert not wrong, f"{name}: the oracle no longer reproduces {wrong}"


@pytest.mark.parametrize("name", list(gc.CASES))
def test_fixture_cases_are_not_degenerate(name):
    p = gc.oracle_planes(name)
    c = gc.inputs(name)
    assert len(np.unique(p["expert_idx"])) > c["E"] // 2           # the routing spreads over the experts
    assert (p["node_counts"] > 0).all() and (p["i_send"] > 0).all()
    if c["capacity"] is not None:
        assert 0 < p["kept"].sum() < p["kept"].size               # some rows are dropped, some kept
