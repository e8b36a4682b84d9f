"""Writes tests/golden/scipy_correlate2d.npz: inputs and expected outputs that pin
the oracle's definition (validate.hpp:94-132) against an independent library
routine, scipy.signal.correlate2d(ref, target, mode='full').

Two kinds of cases: small-integer-valued matrices, whose products and sums are
exact in fp32 and fp64 (compared bit for bit), and real-valued fp64 matrices
(compared to 1e-12). Shapes cover square, non-square, odd, single row, single
column and 1x1.

Run from the repo root:  python tests/golden/make_scipy_fixtures.py
"""
import os

import numpy as np
from scipy.signal import correlate2d

SHAPES = [(1, 1), (1, 7), (6, 1), (2, 2), (3, 5), (5, 3), (4, 4), (7, 9), (8, 8), (16, 11), (13, 32)]


def main():
    rng = np.random.default_rng(20231)
    out = {}
    for i, (rows, cols) in enumerate(SHAPES):
        ref_i = rng.integers(-8, 9, size=(rows, cols)).astype(np.float64)
        tgt_i = rng.integers(-8, 9, size=(rows, cols)).astype(np.float64)
        out[f"int_{i}_ref"] = ref_i
        out[f"int_{i}_target"] = tgt_i
        out[f"int_{i}_expected"] = correlate2d(ref_i, tgt_i, mode="full")
        ref_r = rng.standard_normal((rows, cols))
        tgt_r = rng.random((rows, cols))
        out[f"real_{i}_ref"] = ref_r
        out[f"real_{i}_target"] = tgt_r
        out[f"real_{i}_expected"] = correlate2d(ref_r, tgt_r, mode="full")
    out["num_cases"] = np.array(len(SHAPES))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scipy_correlate2d.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
