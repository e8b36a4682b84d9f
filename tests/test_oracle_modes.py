"""Pins the oracle's mode drivers (validate.hpp:216-298), validation statistic
(validate.hpp:134-188), interleave map (matrix.hpp:614-618) and split-row worker
maps (row_distribution.cuh)."""
import math

import numpy as np
import pytest


def const_matrices(values, rows=3, cols=4, dtype=np.float32):
    return np.stack([np.full((rows, cols), v, dtype=dtype) for v in values])


def centre(res):
    return res[:, res.shape[1] // 2, res.shape[2] // 2]


def test_one_to_one(oracle):
    rng = np.random.default_rng(1)
    a = rng.random((5, 6), dtype=np.float32)
    b = rng.random((5, 6), dtype=np.float32)
    res = oracle.one_to_one(a, b)
    assert res.shape == (1, 9, 11)
    np.testing.assert_array_equal(res[0], oracle.cross_corr(a, b))


def test_one_to_many_pairs(oracle):
    left = const_matrices([2])
    right = const_matrices([10, 20, 30, 40, 50])
    res = oracle.one_to_many(left, right)
    assert res.shape[0] == 5
    np.testing.assert_array_equal(centre(res), 12 * 2 * np.array([10, 20, 30, 40, 50], dtype=np.float32))


def test_n_to_mn_file_order(oracle):
    # validate.hpp:264-269: target t*n + r pairs with ref r; result at the same index
    n, m = 3, 4
    left = const_matrices([1, 2, 3])
    right = const_matrices([10 * (i + 1) for i in range(n * m)])
    res = oracle.n_to_mn(left, right)
    exp = [12 * (i % n + 1) * 10 * (i + 1) for i in range(n * m)]
    np.testing.assert_array_equal(centre(res), np.array(exp, dtype=np.float32))


def test_n_to_m_index(oracle):
    # validate.hpp:285-289: result r * n_target + t
    left = const_matrices([1, 2, 3], dtype=np.float64)
    right = const_matrices([10, 20], dtype=np.float64)
    res = oracle.n_to_m(left, right)
    assert res.shape[0] == 6
    exp = [12 * l * r for l in (1, 2, 3) for r in (10, 20)]
    np.testing.assert_array_equal(centre(res), np.array(exp, dtype=np.float64))


def test_mode_drivers_match_pairwise(oracle):
    rng = np.random.default_rng(2)
    left = rng.standard_normal((2, 4, 5))
    right = rng.standard_normal((6, 4, 5))
    nm = oracle.n_to_m(left, right, threads=2)
    mn = oracle.n_to_mn(left, right)
    for r in range(2):
        for t in range(6):
            np.testing.assert_array_equal(nm[r * 6 + t], oracle.cross_corr(left[r], right[t]))
    for i in range(6):
        np.testing.assert_array_equal(mn[i], oracle.cross_corr(left[i % 2], right[i]))


def test_mode_errors(oracle):
    a = np.zeros((2, 3, 3), dtype=np.float32)
    b = np.zeros((3, 3, 3), dtype=np.float32)
    with pytest.raises(RuntimeError, match="not divisible"):
        oracle.n_to_mn(a, b)
    with pytest.raises(RuntimeError, match="Invalid result matrix size"):
        oracle.one_to_one(a[0], b[0], result_shape=(1, 5, 6))
    with pytest.raises(RuntimeError, match="Invalid number of result matrices"):
        oracle.one_to_many(a[0], b, result_shape=(2, 5, 5))
    with pytest.raises(RuntimeError, match="Invalid number of result matrices"):
        oracle.n_to_m(a, b, result_shape=(5, 5, 5))


def test_validate_result_hand_cases(oracle):
    result = np.array([1.0, 2.0, 4e-6, 0.0], dtype=np.float32)
    valid = np.array([1.0, 4.0, 9e-6, 1.0], dtype=np.float32)
    v = oracle.validate_result(result, valid)
    # differences: 0, |2-4|/4 = 0.5, both <= 1e-5 -> 0, |0-1|/1 = 1
    assert v.diff_max == 1.0
    assert v.diff_mean == pytest.approx(1.5 / 4)
    assert v.diff_stddev == pytest.approx(math.sqrt((0.25 + 1.0) / 4 - (1.5 / 4) ** 2))
    assert (v.at_max_result, v.at_max_valid) == (0.0, 1.0)
    # only one of the two is tiny: not zeroed
    v = oracle.validate_result(np.array([5e-6]), np.array([2e-5]))
    assert v.diff_max == pytest.approx(1.5e-5 / 2e-5)
    # first occurrence of the maximum is reported
    v = oracle.validate_result(np.array([1.0, 3.0, 5.0]), np.array([2.0, 6.0, 5.0]))
    assert v.diff_max == 0.5 and (v.at_max_result, v.at_max_valid) == (1.0, 2.0)
    # identical inputs
    v = oracle.validate_result(valid, valid)
    assert (v.diff_max, v.diff_mean, v.diff_stddev) == (0.0, 0.0, 0.0)
    with pytest.raises(RuntimeError, match="different sizes"):
        oracle.validate_result(np.zeros(3), np.zeros(4))


def test_errors_measures(oracle):
    a = np.array([3.0, 4.0, 0.0])
    b = np.array([3.0, 0.0, 0.0])
    e = oracle.errors(a, b)
    assert e.rel_frobenius == pytest.approx(4.0 / 3.0)
    assert e.max_abs == 4.0 and e.max_rel == 1.0


def test_interleave_index(oracle):
    # n = 2 refs, m = 3 targets each: file order t*n + r -> slot r*m + t
    assert [oracle.interleave_index(i, 6, 2) for i in range(6)] == [0, 3, 1, 4, 2, 5]
    for total, group in [(12, 3), (128, 8), (7, 7), (5, 1)]:
        slots = [oracle.interleave_index(i, total, group) for i in range(total)]
        assert sorted(slots) == list(range(total))
        for i, s in enumerate(slots):
            assert s == (i % group) * (total // group) + i // group


@pytest.mark.parametrize("dist", ["none", "rectangle", "triangle"])
@pytest.mark.parametrize("rows,max_rows", [(1, 1), (4, 1), (8, 3), (16, 4), (64, 4), (64, 10), (33, 5), (100, 7)])
def test_distribution_covers_every_row_part_once(oracle, dist, rows, max_rows):
    """row_distribution.cuh: the active workers (worker_idx < workers_for_row and a valid
    output row) enumerate every (output row, part) exactly once, and workers_for_row is
    ceil(overlap rows / max rows) (1 for 'none')."""
    search = 2 * rows - 1
    total = oracle.dist_num_workers(dist, max_rows, rows, search)
    seen = {}
    # a launch rounds the worker count up to whole blocks: surplus ids must be inactive
    for wid in range(total + 40):
        row, idx, per_row = oracle.dist_distribute_rows(dist, wid, max_rows, rows, search)
        if row >= search or idx >= per_row:
            continue
        assert wid < total
        overlap_rows = rows - abs(row - (rows - 1))
        assert per_row == (1 if dist == "none" else -(-overlap_rows // max_rows))
        assert (row, idx) not in seen
        seen[(row, idx)] = wid
    expected = 0
    for row in range(search):
        overlap_rows = rows - abs(row - (rows - 1))
        expected += 1 if dist == "none" else -(-overlap_rows // max_rows)
    assert len(seen) == expected


def test_distribution_worker_counts(oracle):
    assert oracle.dist_num_workers("none", 4, 64, 127) == 127
    assert oracle.dist_num_workers("rectangle", 4, 64, 127) == 127 * 16
    # triangle packs densely: exactly the number of (row, part) pairs when rows % max_rows == 0
    assert oracle.dist_num_workers("triangle", 4, 64, 127) == sum(-(-(64 - abs(r - 63)) // 4) for r in range(127))
