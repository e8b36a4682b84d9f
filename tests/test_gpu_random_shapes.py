"""Seeded random sweep over shapes, matrix counts, families and dtypes: every case is compared
bit for bit with the oracle on small integer-valued inputs. Complements the fixed shapes of
test_gpu_parity.py with sizes nobody chose (odd widths that are no multiple of the 128-bit
pieces, matrices smaller than a tile, counts that do not fill the matrix lanes)."""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def ints(rng, shape, dtype):
    return rng.integers(-4, 5, size=shape).astype(dtype)


CASES_PER_MODE = 24


def test_random_one_to_one_and_one_to_many(oracle):
    xc = load_package()
    rng = np.random.default_rng(20231)
    pair = ["overlap_wise", "warp_per_overlap", "warp_per_overlap_lds", "block_per_overlap", "shuffle", "split_row",
            "grouped_overlap", "multimat_right", "multimat_right_grouped", "multimat_both", "multimat_both_grouped"]
    many = ["warp_per_overlap_lds", "multimat_right", "multimat_right_grouped", "multimat_both", "multimat_both_grouped"]
    for case in range(CASES_PER_MODE):
        dtype = (np.float32, np.float64)[case % 2]
        rows, cols = int(rng.integers(1, 90)), int(rng.integers(1, 140))
        n_right = int(rng.integers(1, 12))
        left = ints(rng, (1, rows, cols), dtype)
        right = ints(rng, (n_right, rows, cols), dtype)
        exp = oracle.one_to_many(left, right, threads=4)
        fam = pair[case % len(pair)]
        print("case", case, np.dtype(dtype).name, rows, cols, "one_to_one", fam, flush=True)
        got = xc.run(fam, left[0], right[0], 1)
        assert np.array_equal(got[0], exp[0]), (case, fam, rows, cols, xc.last_launch()["kernel"])
        fam = many[case % len(many)]
        print("case", case, np.dtype(dtype).name, rows, cols, n_right, "one_to_many", fam, flush=True)
        got = xc.run(fam, left, right, n_right, n_left=1, n_right=n_right)
        assert np.array_equal(got, exp), (case, fam, rows, cols, n_right, xc.last_launch()["kernel"])


def test_random_n_to_mn_and_n_to_m(oracle):
    xc = load_package()
    rng = np.random.default_rng(20232)
    for case in range(CASES_PER_MODE):
        dtype = (np.float64, np.float32)[case % 2]
        rows, cols = int(rng.integers(1, 70)), int(rng.integers(1, 100))
        n_left, per_left = int(rng.integers(1, 7)), int(rng.integers(1, 10))
        left = ints(rng, (n_left, rows, cols), dtype)
        # n_to_mn in the grouped device layout: the right matrices of left l are [l*m, (l+1)*m)
        right = ints(rng, (n_left * per_left, rows, cols), dtype)
        print("case", case, np.dtype(dtype).name, rows, cols, n_left, per_left, "n_to_mn", flush=True)
        got = xc.run("multimat_right_grouped", left, right, n_left * per_left, n_left=n_left, n_right=per_left)
        for l in range(n_left):
            exp = oracle.one_to_many(left[l:l + 1], right[l * per_left:(l + 1) * per_left], threads=4)
            assert np.array_equal(got[l * per_left:(l + 1) * per_left], exp), (case, l, rows, cols, xc.last_launch()["kernel"])
        n_right = int(rng.integers(1, 12))
        right = ints(rng, (n_right, rows, cols), dtype)
        exp = oracle.n_to_m(left, right, threads=4)
        for fam in ("multimat_both", "multimat_both_grouped"):
            print("case", case, np.dtype(dtype).name, rows, cols, n_left, n_right, "n_to_m", fam, flush=True)
            got = xc.run(fam, left, right, n_left * n_right, n_left=n_left, n_right=n_right)
            assert np.array_equal(got, exp), (case, fam, rows, cols, n_left, n_right, xc.last_launch()["kernel"])
