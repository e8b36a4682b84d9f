"""GPU parity of the matrix-core tiles (xcorr_params.matrix_cores = 1 keeps the launcher to them): every mode of the
grouped families on shapes that do not divide the 32 x 32 / 16 x 16 result tiles, the 8-column steps or the staged bands,
whole and with the reduction cut into atomically added chunks of rows and columns, against the CPU oracle.
Integer-valued inputs must match bit for bit, real-valued ones to 1e-5 (fp32) / 1e-12 (fp64) relative Frobenius error."""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
SHAPES = [(1, 1), (1, 9), (7, 1), (5, 3), (16, 16), (31, 33), (33, 17), (64, 64), (70, 130), (150, 41)]
CHUNKINGS = [{}, dict(rows_per_thread=8), dict(rows_per_thread=24, distribution_type="rectangle"), dict(rows_per_thread=40, column_chunks=2),
             dict(distribution_type="none")]


def say(*a):
    print(*a, flush=True)


def ints(rng, shape, dtype, amp=4):
    return rng.integers(-amp, amp + 1, size=shape).astype(dtype)


def rel_frob(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    den = np.linalg.norm(b)
    return np.linalg.norm(a - b) / (den if den > 0 else 1.0)


def launch_and_check(xc, family, left, right, n_results, n_left, n_right, exp, exact, kw, seen):
    got = xc.run(family, left, right, n_results, n_left=n_left, n_right=n_right, params=xc.make_params(matrix_cores=1, **kw))
    rec = xc.last_launch()
    what = f"{family} {left.shape} x {right.shape} {kw} {rec['kernel']} rows={rec['rows_per_worker']} atomics={rec['uses_atomics']}"
    assert rec["matrix_cores"] == 1, what
    seen.add(rec["kernel"].split("/")[1])
    assert np.isfinite(got).all(), what
    if exact:
        bad = np.argwhere(got != exp)
        assert bad.size == 0, f"{what}: {len(bad)} elements differ, first {bad[:3].tolist()}"
    else:
        err = rel_frob(got, exp)
        assert err <= TOL[got.dtype], f"{what}: rel frobenius {err:.3e}"


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_one_pair(oracle, dtype):
    xc = load_package()
    rng = np.random.default_rng(900)
    seen = set()
    for shape in SHAPES + [(200, 260)]:
        left, right = ints(rng, shape, dtype), ints(rng, shape, dtype)
        exp = oracle.one_to_one(left, right, threads=4)
        for kw in CHUNKINGS:
            say("one pair", np.dtype(dtype).name, shape, kw)
            launch_and_check(xc, "grouped_overlap", left, right, 1, 1, 1, exp, True, kw, seen)
    left, right = rng.standard_normal((130, 150)).astype(dtype), rng.standard_normal((130, 150)).astype(dtype)
    launch_and_check(xc, "grouped_overlap", left, right, 1, 1, 1, oracle.one_to_one(left, right, threads=4), False, {}, seen)
    say(sorted(seen))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_one_to_many_and_groups(oracle, dtype):
    xc = load_package()
    rng = np.random.default_rng(901)
    seen = set()
    for shape in [(1, 1), (5, 3), (16, 16), (33, 17), (40, 70), (64, 64)]:
        for n_right in (1, 3, 4, 9, 17):
            left, right = ints(rng, (1,) + shape, dtype), ints(rng, (n_right,) + shape, dtype)
            exp = oracle.one_to_many(left, right)
            for kw in CHUNKINGS[:3] + [dict(right_matrices_per_thread=4)]:
                say("one_to_many", np.dtype(dtype).name, shape, n_right, kw)
                launch_and_check(xc, "multimat_right_grouped", left, right, n_right, 1, n_right, exp, True, kw, seen)
        # every left matrix with its own group of right matrices, one launch
        for n_left, per_left in [(2, 1), (3, 5), (7, 4), (4, 9)]:
            left, right = ints(rng, (n_left,) + shape, dtype), ints(rng, (n_left * per_left,) + shape, dtype)
            exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * per_left:(l + 1) * per_left]) for l in range(n_left)])
            for kw in CHUNKINGS[:2]:
                say("n_to_mn", np.dtype(dtype).name, shape, n_left, per_left, kw)
                launch_and_check(xc, "multimat_right_grouped", left, right, n_left * per_left, n_left, per_left, exp, True, kw, seen)
    left, right = rng.random((1, 90, 75)).astype(dtype), rng.random((6, 90, 75)).astype(dtype)
    launch_and_check(xc, "multimat_right_grouped", left, right, 6, 1, 6, oracle.one_to_many(left, right, threads=4), False, {}, seen)
    say(sorted(seen))
    assert any("_r" in k for k in seen), seen  # tiles with right matrices over the rows of a result tile were used


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_all_pairs(oracle, dtype):
    xc = load_package()
    rng = np.random.default_rng(902)
    seen = set()
    for shape in [(1, 1), (3, 5), (16, 16), (19, 23), (33, 40), (64, 64)]:
        for n_left, n_right in [(1, 1), (2, 3), (4, 4), (5, 9), (9, 5), (13, 2)]:
            left, right = ints(rng, (n_left,) + shape, dtype), ints(rng, (n_right,) + shape, dtype)
            exp = oracle.n_to_m(left, right, threads=4)
            for kw in CHUNKINGS[:3] + [dict(left_matrices_per_thread=4, right_matrices_per_thread=4)]:
                say("n_to_m", np.dtype(dtype).name, shape, n_left, n_right, kw)
                launch_and_check(xc, "multimat_both_grouped", left, right, n_left * n_right, n_left, n_right, exp, True, kw, seen)
    left, right = rng.standard_normal((5, 50, 60)).astype(dtype), rng.standard_normal((7, 50, 60)).astype(dtype)
    launch_and_check(xc, "multimat_both_grouped", left, right, 35, 5, 7, oracle.n_to_m(left, right, threads=4), False, {}, seen)
    say(sorted(seen))
    assert any("_l" in k for k in seen), seen  # tiles with left matrices over the columns of a result tile were used


def test_tiles_with_copies_of_the_x_shifts(oracle):
    """The fp32 tiles whose result columns hold 16 x shifts twice, 8 left rows apart (16 x 16 shifts of 4 right matrices): forced by
    index on shapes around their 8-row offset, the 32-row stages and the 64-bit-aligned rows of their left band, whole and in chunks
    of left rows that start and end anywhere; the launcher's own choice on a launch they are best for."""
    xc = load_package()
    rng = np.random.default_rng(905)
    indices = []
    probe = ints(rng, (1, 4, 4), np.float32)
    for index in range(1, 64):
        try:
            xc.run("multimat_right_grouped", probe, probe, 1, n_left=1, n_right=1, params=xc.make_params(specialisation=index))
        except xc.XcorrError as e:
            if "does not exist" in e.message:
                break
            continue
        if "_m16x16_" in xc.last_launch()["kernel"] and not xc.last_launch()["kernel"].endswith("_s4"):
            indices.append(index)
    assert len(indices) == 2, indices
    for index in indices:
        for shape in [(1, 1), (5, 3), (7, 9), (8, 8), (9, 16), (16, 16), (19, 23), (31, 33), (33, 17), (40, 40), (64, 64), (70, 130), (150, 41)]:
            for n_right in (1, 3, 4, 9):
                left, right = ints(rng, (1,) + shape, np.float32), ints(rng, (n_right,) + shape, np.float32)
                exp = oracle.one_to_many(left, right, threads=4)
                for kw in [{}, dict(rows_per_thread=3), dict(rows_per_thread=8), dict(rows_per_thread=24), dict(rows_per_thread=40, column_chunks=2)]:
                    say("copies", index, shape, n_right, kw)
                    got = xc.run("multimat_right_grouped", left, right, n_right, n_left=1, n_right=n_right, params=xc.make_params(specialisation=index, **kw))
                    rec = xc.last_launch()
                    bad = np.argwhere(got != exp)
                    assert bad.size == 0, (index, shape, n_right, kw, rec["kernel"], bad[:3].tolist())
        left, right = ints(rng, (3, 40, 70), np.float32), ints(rng, (15, 40, 70), np.float32)
        exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * 5:(l + 1) * 5]) for l in range(3)])
        assert np.array_equal(xc.run("multimat_right_grouped", left, right, 15, n_left=3, n_right=5, params=xc.make_params(specialisation=index)), exp)
        exp = oracle.n_to_m(left, right, threads=4)
        assert np.array_equal(xc.run("multimat_both_grouped", left, right, 45, n_left=3, n_right=15, params=xc.make_params(specialisation=index, rows_per_thread=16)), exp)
    left, right = rng.standard_normal((1, 128, 128)).astype(np.float32), rng.standard_normal((64, 128, 128)).astype(np.float32)
    got = xc.run("multimat_right_grouped", left, right, 64, n_left=1, n_right=64)
    assert "_m16x16_r4" in xc.last_launch()["kernel"], xc.last_launch()["kernel"]
    sample = [0, 17, 63]
    assert rel_frob(got[sample], oracle.one_to_many(left, right[sample], threads=4)) <= 1e-5


def test_never_and_only(oracle):
    """matrix_cores = 2 keeps the register tiles; both settings give the same integers."""
    xc = load_package()
    rng = np.random.default_rng(903)
    left, right = ints(rng, (300, 280), np.float32), ints(rng, (300, 280), np.float32)
    exp = oracle.one_to_one(left, right, threads=4)
    for setting, flag in [(1, 1), (2, 0)]:
        got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(matrix_cores=setting))
        assert xc.last_launch()["matrix_cores"] == flag
        assert np.array_equal(got, exp)
    with pytest.raises(xc.XcorrError, match="matrix_cores must be 0, 1 or 2"):
        xc.run("grouped_overlap", left, right, 1, params=xc.make_params(matrix_cores=7))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_one_output_row_families_on_matrix_core_tiles(oracle, dtype):
    """shuffle, split_row, multimat_right(_groups) and multimat_both served by matrix-core tiles under their own contracts
    (who clears the output, rows per worker, distribution): forced with matrix_cores = 1 on small shapes, chosen by the
    launcher on larger ones."""
    xc = load_package()
    rng = np.random.default_rng(904)
    seen = set()
    contracts = [{}, dict(rows_per_thread=16), dict(rows_per_thread=40, distribution_type="rectangle"), dict(distribution_type="triangle"),
                 dict(distribution_type="none")]
    for shape in [(5, 3), (31, 33), (64, 64), (70, 130)]:
        left, right = ints(rng, shape, dtype), ints(rng, shape, dtype)
        exp = oracle.one_to_one(left, right, threads=4)
        for family in ("shuffle", "split_row"):
            for kw in contracts:
                if family == "shuffle" and "rows_per_thread" in kw:
                    continue
                say(family, np.dtype(dtype).name, shape, kw)
                launch_and_check(xc, family, left, right, 1, 1, 1, exp, True, kw, seen)
        for n_right in (3, 9):
            many = ints(rng, (n_right,) + shape, dtype)
            exp_many = oracle.one_to_many(left[None], many)
            for kw in contracts:
                say("multimat_right", np.dtype(dtype).name, shape, n_right, kw)
                launch_and_check(xc, "multimat_right", left[None], many, n_right, 1, n_right, exp_many, True, kw, seen)
        lefts, rights = ints(rng, (3,) + shape, dtype), ints(rng, (6,) + shape, dtype)
        exp_groups = np.concatenate([oracle.one_to_many(lefts[l:l + 1], rights[2 * l:2 * l + 2]) for l in range(3)])
        exp_all = oracle.n_to_m(lefts, rights, threads=4)
        for kw in contracts[:4]:
            say("multimat_right_groups / multimat_both", np.dtype(dtype).name, shape, kw)
            launch_and_check(xc, "multimat_right_groups", lefts, rights, 6, 3, 2, exp_groups, True, kw, seen)
            launch_and_check(xc, "multimat_both", lefts, rights, 18, 3, 6, exp_all, True, kw, seen)
    # the launcher's own choice on a launch that is large enough, and the cases it leaves to the one-row tiles
    left, right = ints(rng, (150, 140), dtype), ints(rng, (150, 140), dtype)
    exp = oracle.one_to_one(left, right, threads=4)
    for family, kw, routed in [("split_row", {}, 1), ("shuffle", {}, 1), ("split_row", dict(rows_per_thread=7), 0), ("shuffle", dict(distribution_type="none"), 0),
                               ("split_row", dict(matrix_cores=2), 0)]:
        got = xc.run(family, left, right, 1, params=xc.make_params(**kw))
        rec = xc.last_launch()
        assert rec["matrix_cores"] == routed, (family, kw, rec["kernel"])
        assert np.array_equal(got, exp), (family, kw, rec["kernel"])
    say(sorted(seen))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_tiles_swept_result_tile_by_result_tile(oracle, dtype):
    """The tiles whose sweep trims every result tile of a block to its own overlap (`_s16`: one pair, 16 x 16 shifts at a time;
    `_r4_s4`: four right matrices, 16 x 4 shifts at a time), forced by index: shapes below, at and above the extents of a result tile
    and of a block tile, one-row and one-column matrices, whole reductions and chunks of left rows and right columns that start
    and end anywhere (atomic adds), one left matrix against several right ones, groups, all pairs; the launcher's own choice on
    launches they are best for. Bit-exact on integers."""
    xc = load_package()
    rng = np.random.default_rng(906)
    indices = {}
    probe = ints(rng, (1, 4, 4), dtype)
    for index in range(1, 80):
        try:
            xc.run("multimat_right_grouped", probe, probe, 1, n_left=1, n_right=1, params=xc.make_params(specialisation=index))
        except xc.XcorrError as e:
            if "does not exist" in e.message:
                break
            continue
        kernel = xc.last_launch()["kernel"].split("/")[1]
        if kernel.endswith("_s16") or kernel.endswith("_s4"):
            indices[kernel] = index
    say("tiles:", indices)
    assert len(indices) == (3 if dtype == np.float32 else 2), indices
    for kernel, index in indices.items():
        for shape in [(1, 1), (1, 40), (37, 1), (5, 3), (15, 17), (16, 16), (17, 31), (32, 32), (33, 47), (64, 64), (65, 63), (70, 130), (150, 41)]:
            for n_right in (1, 3, 4, 9) if "_r4" in kernel else (1, 2):
                left, right = ints(rng, (1,) + shape, dtype), ints(rng, (n_right,) + shape, dtype)
                exp = oracle.one_to_many(left, right)
                for kw in [{}, dict(rows_per_thread=3), dict(rows_per_thread=8), dict(rows_per_thread=24), dict(rows_per_thread=40, column_chunks=2)]:
                    got = xc.run("multimat_right_grouped", left, right, n_right, n_left=1, n_right=n_right, params=xc.make_params(specialisation=index, **kw))
                    rec = xc.last_launch()
                    assert rec["kernel"].endswith(kernel)
                    bad = np.argwhere(got != exp)
                    assert bad.size == 0, (kernel, shape, n_right, kw, bad[:3].tolist())
        left, right = ints(rng, (3, 21, 45), dtype), ints(rng, (15, 21, 45), dtype)
        exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * 5:(l + 1) * 5]) for l in range(3)])
        assert np.array_equal(xc.run("multimat_right_grouped", left, right, 15, n_left=3, n_right=5, params=xc.make_params(specialisation=index)), exp)
        exp = oracle.n_to_m(left, right)
        assert np.array_equal(xc.run("multimat_both_grouped", left, right, 45, n_left=3, n_right=15, params=xc.make_params(specialisation=index, rows_per_thread=16)), exp)
        left, right = ints(rng, (1, 100, 90), dtype), ints(rng, (1, 100, 90), dtype)
        assert np.array_equal(xc.run("grouped_overlap", left, right, 1, params=xc.make_params(specialisation=index)), oracle.one_to_one(left[0], right[0]))
    # the launcher's own choice: many independent pairs; one left matrix against many right ones
    left, right = ints(rng, (600, 48, 48), dtype), ints(rng, (600, 48, 48), dtype)
    got = xc.run("multimat_right_grouped", left, right, 600, n_left=600, n_right=1)
    assert xc.last_launch()["kernel"].endswith("_s16"), xc.last_launch()["kernel"]
    assert np.array_equal(got, oracle.n_to_mn(left, right, threads=8))
    left, right = ints(rng, (1, 128, 128), dtype), ints(rng, (64, 128, 128), dtype)
    got = xc.run("multimat_right_grouped", left, right, 64, n_left=1, n_right=64)
    assert xc.last_launch()["kernel"].endswith("_r4_s4"), xc.last_launch()["kernel"]
    sample = [0, 17, 63]
    assert np.array_equal(got[sample], oracle.one_to_many(left, right[sample], threads=4))
