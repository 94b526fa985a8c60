"""Writes tests/golden/shuffle_permutations.npz: what thrust::shuffle_copy of the real reference
(its sequential CPP system, compiled by oracle/Makefile into oracle/_ref/libref_cpp.so) makes of
0, 1, ..., n-1 with thrust::default_random_engine(seed), for a few n and seeds.  Run from the
repository root where the reference build exists: python tests/golden/make_shuffle_vectors.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import cpu  # noqa: E402

CASES = [(0, 1), (1, 1), (2, 5), (3, 0xD5), (5, 2), (8, 7), (17, 183), (64, 1), (100, 42), (1000, 183), (4097, 9),
         (70000, 12345)]


def main():
    ref = cpu.Reference("cpp")
    out = {}
    for n, seed in CASES:
        out["n%d_seed%d" % (n, seed)] = ref.shuffle_copy(np.arange(n, dtype=np.uint32), seed)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "shuffle_permutations.npz"), **out)
    print("wrote", len(out), "permutations")


if __name__ == "__main__":
    main()
