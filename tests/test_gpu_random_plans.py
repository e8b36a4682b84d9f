"""GPU parity on seeded random requests: family, shape, matrix counts and tuning fields are drawn at random, so
the launcher's planner is exercised on combinations no hand-written case lists (tiny and ragged matrices, chunk
sizes that do not divide anything, column chunks, tile requests that have no exact match). Integer-valued inputs:
every result must equal the CPU oracle bit for bit, whatever plan the launcher chose; the plan is printed before
each launch so that a failure names its case."""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


PAIR_FAMILIES = ["shuffle", "split_row", "grouped_overlap"]
RIGHT_FAMILIES = ["multimat_right", "multimat_right_grouped"]
BOTH_FAMILIES = ["multimat_both", "multimat_both_grouped"]
GROUP_FAMILIES = ["multimat_right_groups", "multimat_right_grouped"]


def draw_params(rng, family, rows):
    kw = {}
    if rng.random() < 0.6:
        kw["rows_per_thread"] = int(rng.choice([1, 2, 3, 5, 7, 10, 16, 33, rows, rows + 5]))
    if rng.random() < 0.6:
        kw["distribution_type"] = str(rng.choice(["none", "rectangle", "triangle"]))
    if rng.random() < 0.3:
        kw["column_chunks"] = int(rng.choice([1, 2, 3, 5]))
    if rng.random() < 0.3:
        kw["warps_per_thread_block"] = int(rng.choice([1, 4, 8, 32]))
    if "grouped" in family:
        if rng.random() < 0.5:
            kw["matrix_cores"] = int(rng.choice([1, 2]))
        if rng.random() < 0.5:
            key = "shifts_per_thread" if family == "grouped_overlap" else "shifts_per_thread_right_matrix"
            kw[key] = int(rng.integers(1, 9 if family == "grouped_overlap" else 5))
        if rng.random() < 0.3:
            kw["left_rows_per_iteration"] = int(rng.integers(1, 5))
    if family != "grouped_overlap" and family not in ("shuffle", "split_row"):
        limit = 4 if "grouped" in family else 8
        if rng.random() < 0.5:
            kw["right_matrices_per_thread"] = int(rng.integers(1, limit + 1))
        if "both" in family and rng.random() < 0.5:
            kw["left_matrices_per_thread"] = int(rng.integers(1, limit + 1))
    return kw


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_random_requests_match_the_oracle(oracle, dtype):
    xc = load_package()
    rng = np.random.default_rng(20231 if dtype == np.float32 else 20232)
    plans = set()
    for case in range(300):
        rows, cols = (int(v) for v in rng.choice([1, 2, 3, 5, 8, 13, 16, 21, 31, 32, 33, 47, 64, 70, 97, 130], size=2))
        mode = rng.choice(["pair", "right", "both", "groups"])
        if mode == "pair":
            family, n_left, n_right = str(rng.choice(PAIR_FAMILIES)), 1, 1
        elif mode == "right":
            family, n_left, n_right = str(rng.choice(RIGHT_FAMILIES)), 1, int(rng.integers(1, 12))
        elif mode == "both":
            family, n_left, n_right = str(rng.choice(BOTH_FAMILIES)), int(rng.integers(1, 7)), int(rng.integers(1, 9))
        else:
            family, n_left, n_right = str(rng.choice(GROUP_FAMILIES)), int(rng.integers(2, 6)), int(rng.integers(1, 6))
        kw = draw_params(rng, family, rows)
        left = rng.integers(-3, 4, (n_left, rows, cols)).astype(dtype)
        n_right_total = n_left * n_right if mode == "groups" else n_right
        right = rng.integers(-3, 4, (n_right_total, rows, cols)).astype(dtype)
        if mode == "groups":
            exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * n_right:(l + 1) * n_right]) for l in range(n_left)])
            n_results = n_left * n_right
        elif mode == "both":
            exp, n_results = oracle.n_to_m(left, right), n_left * n_right
        else:
            exp, n_results = oracle.one_to_many(left, right), n_right
        say("case", case, np.dtype(dtype).name, family, (rows, cols), n_left, n_right, kw)
        params = xc.make_params(**kw)
        got = xc.run(family, left, right, n_results, n_left=n_left, n_right=n_right, params=params)
        rec = xc.last_launch()
        plans.add((rec["kernel"], rec["uses_atomics"], rec["column_chunks"] > 1))
        assert np.isfinite(got).all(), (case, family, kw, rec["kernel"])
        bad = np.argwhere(got != exp)
        assert bad.size == 0, (case, family, (rows, cols), n_left, n_right, kw, rec, bad[:3].tolist())
    say(len(plans), "distinct (kernel, atomics, column chunks) combinations")
    assert len(plans) >= 20
