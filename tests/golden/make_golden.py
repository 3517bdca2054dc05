"""Writes tests/golden/policyA_*.json: expected ids, distance bit patterns and
counters of the reference's CPU search on tiny seeded inputs.

The expected values come from oracle/_ref (the reference's own neighbor.h and
distance.h compiled in place around oracle/ref_harness.cpp), so this script only
runs where the reference tree is mounted.  Inputs are regenerated from seeds by
tests/util.py; each fixture carries a SHA-256 of the input bytes.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from test_oracle_policy import golden_inputs  # noqa: E402
from util import digest  # noqa: E402

CASES = [
    dict(name="policyA_gauss_n200_d8", kind="gauss", n=200, dim=8, R=8, seed=101, n_start=2, ragged_seed=4,
         Q=6, L=16, k=5, M=2),
    dict(name="policyA_gauss_n256_d200", kind="gauss", n=256, dim=200, R=32, seed=202, n_start=16, Q=4, L=32,
         k=10, M=16),
    dict(name="policyA_gauss_n150_d36_m1", kind="gauss", n=150, dim=36, R=6, seed=303, n_start=3, ragged_seed=8,
         Q=5, L=8, k=8, M=1),
    dict(name="policyA_lattice_ties", kind="lattice", side=4, dim=4, R=8, starts=[0, 255], Q=3, L=12, k=12, M=2,
         queries=[[1.5, 1.5, 1.5, 1.5], [0, 0, 0, 0], [3, 0.5, 2, 1]]),
]


def main():
    if oracle.ref() is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle` where the reference tree is present")
    for case in CASES:
        base, nbrs, starts, q = golden_inputs(case)
        prob = oracle.Problem(base, nbrs, starts)
        ids, dists, stats, _ = oracle.ref_search_in_cpu(prob, q, case["k"], case["L"], M=case["M"])
        out = dict(case)
        out["input_sha256"] = digest(base, nbrs, starts, q)
        out["ids"] = ids.tolist()
        out["dist_bits"] = dists.view(np.uint32).tolist()
        out["stats"] = stats.tolist()
        with open(os.path.join(HERE, case["name"] + ".json"), "w") as f:
            json.dump(out, f, indent=None, separators=(",", ":"))
            f.write("\n")
        print("wrote", case["name"])


if __name__ == "__main__":
    main()
