"""Writes tests/golden/oracle_digests.json: the digest of every plane the CPU oracle produces for the formula-made
cases of tests/golden_cases.py.  Run from the repository root:  python tests/golden/make_oracle_digests.py"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

import golden_cases as gc  # noqa: E402

out = {"_about": "sha256 (first 24 hex digits) over dtype, shape and bytes of each plane; made by "
                 "tests/golden/make_oracle_digests.py from the oracle, inputs by formula (tests/golden_cases.py)"}
for name in gc.CASES:
    out[name] = {k: gc.digest(v) for k, v in gc.oracle_planes(name).items()}
with open(os.path.join(HERE, "oracle_digests.json"), "w") as f:
    json.dump(out, f, indent=1, sort_keys=True)
    f.write("\n")
print("wrote", len(out) - 1, "cases")
