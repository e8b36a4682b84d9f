"""Pins the oracle's definition functions (xo_hadamard_and_sum_*, xo_naive_cross_corr_*,
restating validate.hpp:94-132) against closed forms, an independent library routine
(scipy fixtures), a textbook brute force, symmetry and linearity."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scipy_correlate2d.npz")


def brute_force(ref, target):
    """out[sy + H-1][sx + W-1] = sum over all (y, x) with both indices valid of
    ref[y][x] * target[y - sy][x - sx], written from the definition."""
    rows, cols = ref.shape
    out = np.zeros((2 * rows - 1, 2 * cols - 1), dtype=np.float64)
    for sy in range(-(rows - 1), rows):
        for sx in range(-(cols - 1), cols):
            s = 0.0
            for y in range(rows):
                for x in range(cols):
                    ty, tx = y - sy, x - sx
                    if 0 <= ty < rows and 0 <= tx < cols:
                        s += float(ref[y, x]) * float(target[ty, tx])
            out[sy + rows - 1, sx + cols - 1] = s
    return out


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_scipy_integer_fixtures_bit_exact(oracle, dtype):
    g = np.load(GOLDEN)
    for i in range(int(g["num_cases"])):
        ref = g[f"int_{i}_ref"].astype(dtype)
        target = g[f"int_{i}_target"].astype(dtype)
        got = oracle.cross_corr(ref, target)
        assert got.dtype == dtype
        np.testing.assert_array_equal(got, g[f"int_{i}_expected"].astype(dtype))
        # accumulate-in-double variant
        if dtype == np.float32:
            np.testing.assert_array_equal(oracle.cross_corr(ref, target, acc64=True), g[f"int_{i}_expected"])


def test_scipy_real_fixtures_fp64(oracle):
    g = np.load(GOLDEN)
    for i in range(int(g["num_cases"])):
        got = oracle.cross_corr(g[f"real_{i}_ref"], g[f"real_{i}_target"])
        exp = g[f"real_{i}_expected"]
        assert np.linalg.norm(got - exp) <= 1e-12 * max(np.linalg.norm(exp), 1e-300)
        got32 = oracle.cross_corr(g[f"real_{i}_ref"].astype(np.float32), g[f"real_{i}_target"].astype(np.float32))
        assert np.linalg.norm(got32 - exp) <= 1e-5 * np.linalg.norm(exp) + 1e-6


@pytest.mark.parametrize("shape", [(1, 1), (2, 3), (5, 4), (8, 8)])
def test_brute_force(oracle, shape):
    rng = np.random.default_rng(7)
    ref = rng.integers(-5, 6, size=shape).astype(np.float64)
    target = rng.integers(-5, 6, size=shape).astype(np.float64)
    np.testing.assert_array_equal(oracle.cross_corr(ref, target), brute_force(ref, target))
    np.testing.assert_array_equal(
        oracle.cross_corr(ref.astype(np.float32), target.astype(np.float32)),
        brute_force(ref, target).astype(np.float32),
    )


@pytest.mark.parametrize("shape", [(1, 9), (6, 6), (17, 5), (64, 64)])
def test_all_ones_closed_form(oracle, shape):
    rows, cols = shape
    ones = np.ones(shape, dtype=np.float32)
    got = oracle.cross_corr(ones, ones)
    oy = np.arange(2 * rows - 1)[:, None]
    ox = np.arange(2 * cols - 1)[None, :]
    exp = (rows - np.abs(oy - (rows - 1))) * (cols - np.abs(ox - (cols - 1)))
    np.testing.assert_array_equal(got, exp.astype(np.float32))


def test_delta_places_the_other_matrix(oracle):
    rng = np.random.default_rng(3)
    rows, cols = 5, 7
    other = rng.standard_normal((rows, cols))
    # delta as target at (py, px): res[sy][sx] = ref[py + sy][px + sx]
    for py, px in [(0, 0), (2, 3), (4, 6)]:
        delta = np.zeros((rows, cols))
        delta[py, px] = 1.0
        got = oracle.cross_corr(other, delta)
        exp = np.zeros_like(got)
        for sy in range(-(rows - 1), rows):
            for sx in range(-(cols - 1), cols):
                y, x = py + sy, px + sx
                if 0 <= y < rows and 0 <= x < cols:
                    exp[sy + rows - 1, sx + cols - 1] = other[y, x]
        np.testing.assert_array_equal(got, exp)
        # delta as ref at (py, px): res[sy][sx] = target[py - sy][px - sx] (flipped placement)
        got = oracle.cross_corr(delta, other)
        exp = np.zeros_like(got)
        for sy in range(-(rows - 1), rows):
            for sx in range(-(cols - 1), cols):
                y, x = py - sy, px - sx
                if 0 <= y < rows and 0 <= x < cols:
                    exp[sy + rows - 1, sx + cols - 1] = other[y, x]
        np.testing.assert_array_equal(got, exp)


def test_centre_and_corners(oracle):
    rng = np.random.default_rng(11)
    rows, cols = 6, 9
    ref = rng.standard_normal((rows, cols))
    target = rng.standard_normal((rows, cols))
    got = oracle.cross_corr(ref, target)
    assert got[rows - 1, cols - 1] == pytest.approx(float(np.sum(ref * target)), rel=1e-13)
    assert got[0, 0] == ref[0, 0] * target[rows - 1, cols - 1]
    assert got[0, -1] == ref[0, cols - 1] * target[rows - 1, 0]
    assert got[-1, 0] == ref[rows - 1, 0] * target[0, cols - 1]
    assert got[-1, -1] == ref[rows - 1, cols - 1] * target[0, 0]
    # hadamard_and_sum addresses shifts directly
    assert oracle.hadamard_and_sum(ref, target, 0, 0) == got[rows - 1, cols - 1]
    assert oracle.hadamard_and_sum(ref, target, -(cols - 1), -(rows - 1)) == got[0, 0]
    assert oracle.hadamard_and_sum(ref, target, 2, -1) == got[rows - 2, cols + 1]
    assert oracle.hadamard_and_sum(ref, target, cols, 0) == 0.0  # empty overlap


def test_swap_flips_result(oracle):
    rng = np.random.default_rng(5)
    a = rng.integers(-9, 10, size=(7, 4)).astype(np.float32)
    b = rng.integers(-9, 10, size=(7, 4)).astype(np.float32)
    np.testing.assert_array_equal(oracle.cross_corr(a, b), oracle.cross_corr(b, a)[::-1, ::-1])


def test_linearity(oracle):
    rng = np.random.default_rng(6)
    a, b, c = (rng.integers(-4, 5, size=(6, 6)).astype(np.float64) for _ in range(3))
    np.testing.assert_array_equal(
        oracle.cross_corr(a + 3 * b, c), oracle.cross_corr(a, c) + 3 * oracle.cross_corr(b, c)
    )
    np.testing.assert_array_equal(
        oracle.cross_corr(c, a - 2 * b), oracle.cross_corr(c, a) - 2 * oracle.cross_corr(c, b)
    )


def test_sequential_fp32_accumulation_order(oracle):
    """The fp32 oracle adds products one by one in row-major order in fp32
    (validate.hpp:102-111): reproduce that order with numpy scalars on one shift."""
    rng = np.random.default_rng(8)
    ref = rng.random((9, 13), dtype=np.float32)
    target = rng.random((9, 13), dtype=np.float32)
    for sx, sy in [(0, 0), (3, -2), (-5, 4)]:
        s = np.float32(0)
        for y in range(max(sy, 0), min(9 + sy, 9)):
            for x in range(max(sx, 0), min(13 + sx, 13)):
                s = np.float32(s + np.float32(target[y - sy, x - sx] * ref[y, x]))
        assert oracle.hadamard_and_sum(ref, target, sx, sy) == s


def test_threads_and_bands_bit_identical(oracle):
    rng = np.random.default_rng(9)
    ref = rng.random((24, 20), dtype=np.float32)
    target = rng.random((24, 20), dtype=np.float32)
    full = oracle.cross_corr(ref, target)
    np.testing.assert_array_equal(oracle.cross_corr(ref, target, threads=4), full)
    band = oracle.cross_corr(ref, target, row_begin=10, row_end=17, threads=3)
    np.testing.assert_array_equal(band[10:17], full[10:17])
    assert not band[:10].any() and not band[17:].any()
