#!/usr/bin/env python3
"""Writes the golden fixtures from the REAL reference.

Needs oracle/_ref (the reference's OMP and CPP device systems compiled from its own
headers by oracle/Makefile, which in turn needs the reference tree).  Outputs, data only:
  tests/golden/small.npz     full outputs of every case at small N (exact arrays)
  tests/golden/digests.json  sha256 of every output at a larger N, plus provenance
Sort cases use the sequential CPP system (thread-count independent); all others are
written from the OMP system and cross-checked against CPP before being accepted, except
float32 sums, where both are checked to agree bit for bit as well (the OMP system's scan
is sequential).
Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import cases  # noqa: E402
from oracle import cpu  # noqa: E402


def run_all(sizes):
    omp, cpp = cpu.Reference("omp"), cpu.Reference("cpp")
    out = {}
    for name, fn in cases.CASES.items():
        n = sizes[name]
        a = fn(cpp, n)
        if name != "c2":  # c2 float layout is defined by the sequential system only
            b = fn(omp, n)
            for k in a:
                if not np.array_equal(np.ascontiguousarray(a[k]).view(np.uint8),
                                      np.ascontiguousarray(b[k]).view(np.uint8)):
                    raise SystemExit(f"OMP and CPP systems disagree on {k} at n={n}")
        out.update(a)
    return out


def main():
    small = run_all(cases.SMALL)
    np.savez_compressed(os.path.join(HERE, "small.npz"), **small)
    large = run_all(cases.LARGE)
    doc = {
        "_comment": "sha256 of the reference's outputs (raw little-endian bytes); written by make_fixtures.py",
        "reference": "Thrust 1.14.0, OMP and CPP device systems, g++ -O3",
        "sizes": cases.LARGE,
        "sha256": {k: cases.digest(v) for k, v in sorted(large.items())},
        "elements": {k: int(np.asarray(v).size) for k, v in sorted(large.items())},
    }
    with open(os.path.join(HERE, "digests.json"), "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
    print("wrote", len(small), "small arrays and", len(large), "digests")


if __name__ == "__main__":
    main()
