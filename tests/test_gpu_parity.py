"""GPU parity: every kernel family, called through the C ABI, against the CPU oracle on
the same seeded inputs.

Bars: integer-valued inputs (every product and sum exact) must match bit for bit in
fp32 and fp64; real-valued inputs must match the oracle to a relative Frobenius error
of 1e-5 (fp32) / 1e-12 (fp64), the tolerances of the build's brief. The GPU kernels add
the same products in a different order than the oracle's sequential loop, so real-valued
results are not expected to be bit-identical (nor are the reference's own kernels).
"""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}

SHAPES = [(1, 1), (1, 7), (6, 1), (3, 5), (16, 16), (17, 33), (33, 17), (64, 64), (70, 130)]


def say(*a):
    print(*a, flush=True)


def ints(rng, shape, dtype, amp=4):
    return rng.integers(-amp, amp + 1, size=shape).astype(dtype)


def rel_frob(a, b):
    a = a.astype(np.float64).ravel()
    b = b.astype(np.float64).ravel()
    den = np.linalg.norm(b)
    return np.linalg.norm(a - b) / (den if den > 0 else 1.0)


def check(got, exp, exact, what):
    assert got.shape == exp.shape, what
    assert np.isfinite(got).all(), f"{what}: unwritten or non-finite output elements"
    if exact:
        bad = np.argwhere(got != exp)
        assert bad.size == 0, f"{what}: {len(bad)} elements differ, first {bad[:3].tolist()}"
    else:
        err = rel_frob(got, exp)
        assert err <= TOL[got.dtype], f"{what}: rel frobenius {err:.3e}"


ONE_TO_ONE_CASES = [
    ("overlap_wise", {}),
    ("warp_per_overlap", dict(warp_per_overlap_variant="base")),
    ("warp_per_overlap", dict(warp_per_overlap_variant="base", shifts_per_thread_block=3)),
    ("warp_per_overlap", dict(warp_per_overlap_variant="simple_indexing", shifts_per_thread_block=32)),
    ("warp_per_overlap", dict(warp_per_overlap_variant="work_distribution", distribution_type="none")),
    ("warp_per_overlap", dict(warp_per_overlap_variant="work_distribution", distribution_type="rectangle", rows_per_thread=3)),
    ("warp_per_overlap", dict(warp_per_overlap_variant="work_distribution", distribution_type="triangle", rows_per_thread=5)),
    ("shuffle", {}),
    ("shuffle", dict(whole_pair_in_lds=2)),
    ("shuffle", dict(warps_per_thread_block=4, whole_pair_in_lds=2)),
    ("shuffle", dict(distribution_type="none")),
    ("split_row", {}),
    ("split_row", dict(whole_pair_in_lds=2)),
    ("split_row", dict(distribution_type="none", whole_pair_in_lds=2)),
    ("split_row", dict(distribution_type="none", column_chunks=3)),
    ("split_row", dict(distribution_type="triangle", rows_per_thread=6, column_chunks=2)),
    ("warp_per_overlap", dict(warp_per_overlap_variant="work_distribution")),
    ("split_row", dict(distribution_type="rectangle", rows_per_thread=10)),
    ("split_row", dict(distribution_type="triangle", rows_per_thread=4)),
    ("split_row", dict(distribution_type="triangle", rows_per_thread=1)),
    ("grouped_overlap", {}),
    ("grouped_overlap", dict(whole_pair_in_lds=1)),
    ("grouped_overlap", dict(whole_pair_in_lds=2)),
    ("grouped_overlap", dict(shifts_per_thread=4, left_rows_per_iteration=3, warps_per_thread_block=8)),
    ("grouped_overlap", dict(shifts_per_thread=8)),
    ("grouped_overlap", dict(shifts_per_thread=1)),
    ("grouped_overlap", dict(shifts_per_thread=8, rows_per_thread=16)),
    ("grouped_overlap", dict(shifts_per_thread=4, rows_per_thread=7, distribution_type="rectangle")),
    ("multimat_right", {}),
    ("multimat_right", dict(whole_pair_in_lds=2)),
    ("multimat_right_grouped", {}),
    ("multimat_both", {}),
    ("multimat_both", dict(whole_pair_in_lds=2)),
    ("multimat_both_grouped", {}),
    ("warp_per_overlap_lds", {}),
    ("warp_per_overlap_lds", dict(whole_pair_in_lds=2)),
    ("warp_per_overlap_lds", dict(shifts_per_thread_block=32, shared_mem_rows=32)),
    ("warp_per_overlap_lds", dict(shifts_per_thread_block=3, shared_mem_rows=7)),
    ("warp_per_overlap_lds", dict(shifts_per_thread_block=8, column_group_per_block=1)),
    ("block_per_overlap", {}),
    ("block_per_overlap", dict(block_size=64)),
    ("block_per_overlap", dict(block_size=1024)),
    ("block_per_overlap", dict(block_size=200)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("family,kw", ONE_TO_ONE_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_one_to_one_all_families(oracle, dtype, family, kw):
    xc = load_package()
    rng = np.random.default_rng(100)
    for shape in SHAPES:
        say("one_to_one", family, kw, np.dtype(dtype).name, shape)
        left, right = ints(rng, shape, dtype), ints(rng, shape, dtype)
        exp = oracle.one_to_one(left, right)
        got = xc.run(family, left, right, 1, params=xc.make_params(**kw))
        check(got, exp, True, f"{family} {kw} {shape} int")
        left = rng.standard_normal(shape).astype(dtype)
        right = rng.random(shape).astype(dtype)
        exp = oracle.one_to_one(left, right)
        got = xc.run(family, left, right, 1, params=xc.make_params(**kw))
        check(got, exp, False, f"{family} {kw} {shape} real")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_whole_pair_in_lds(oracle, dtype):
    """The kernel that keeps both matrices of a small pair in LDS (the default of grouped_overlap up to
    96 x 96 fp32 / 64 x 64 fp64): every size 1 ... 12 squared, sizes around the 64-column chunk of its lanes,
    ragged non-square shapes and the largest pairs that fit; bit-exact on integers, within tolerance on real
    values; the launcher picks it by itself for small pairs and leaves larger ones to the engine; a pair that
    does not fit is an error when the kernel is forced."""
    xc = load_package()
    rng = np.random.default_rng(321)
    shapes = [(n, n) for n in range(1, 13)] + [(1, 64), (64, 1), (63, 64), (64, 65), (65, 63), (5, 128), (128, 5), (2, 129), (31, 97),
                                                (80, 80), (96, 96), (90, 101)]
    shapes += [(128, 128), (136, 130)] if dtype == np.float32 else [(98, 94)]
    for shape in shapes:
        say("whole pair in LDS", np.dtype(dtype).name, shape)
        left, right = ints(rng, shape, dtype), ints(rng, shape, dtype)
        got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(whole_pair_in_lds=1))
        assert "pair_in_lds" in xc.last_launch()["kernel"]
        assert xc.last_launch()["uses_atomics"] == 0
        check(got, oracle.one_to_one(left, right), True, f"whole pair {shape} int")
        left, right = rng.standard_normal(shape).astype(dtype), rng.random(shape).astype(dtype)
        got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(whole_pair_in_lds=1))
        check(got, oracle.one_to_one(left, right), False, f"whole pair {shape} real")
    # the launcher's own choice
    for shape, expect in [((64, 64), True), ((40, 90), True), ((90, 100), np.dtype(dtype) == np.float32), ((110, 100), False),
                          ((200, 200), False), ((3, 300), False)]:
        left, right = ints(rng, shape, dtype), ints(rng, shape, dtype)
        got = xc.run("grouped_overlap", left, right, 1)
        assert ("pair_in_lds" in xc.last_launch()["kernel"]) == expect, (shape, xc.last_launch()["kernel"])
        check(got, oracle.one_to_one(left, right), True, f"default {shape}")
        got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(whole_pair_in_lds=2))
        assert "pair_in_lds" not in xc.last_launch()["kernel"]
        check(got, oracle.one_to_one(left, right), True, f"engine {shape}")
    # asking for a tile keeps the engine
    left, right = ints(rng, (32, 32), dtype), ints(rng, (32, 32), dtype)
    xc.run("grouped_overlap", left, right, 1, params=xc.make_params(shifts_per_thread=4))
    assert "pair_in_lds" not in xc.last_launch()["kernel"]
    big = (300, 300)
    with pytest.raises(xc.XcorrError) as err:
        xc.run("grouped_overlap", ints(rng, big, dtype), ints(rng, big, dtype), 1, params=xc.make_params(whole_pair_in_lds=1))
    assert err.value.code == 3 and "does not fit" in err.value.message
    with pytest.raises(xc.XcorrError) as err:
        xc.run("grouped_overlap", left, right, 1, params=xc.make_params(whole_pair_in_lds=3))
    assert err.value.code == 1


def run_as_planned(xc, family, left, right, n_results, n_left, n_right, params):
    """What a caller that asks first does: a planning call, then the launch into an output that is zeroed only when the
    record says that the launch adds into it (filled with a NaN pattern otherwise). Returns (result, record)."""
    rows, cols = left.shape[-2:]
    out_shape = (n_results, 2 * rows - 1, 2 * cols - 1)
    d_left, d_right = xc.DeviceBuffer.from_numpy(left), xc.DeviceBuffer.from_numpy(right)
    d_out = xc.DeviceBuffer(int(np.prod(out_shape)) * left.dtype.itemsize)
    try:
        assert xc.lib().xcorr_plan_only(1) == 0
        try:
            xc.launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, left.dtype, params)
            planned = xc.last_launch()
        finally:
            xc.lib().xcorr_plan_only(0)
        if planned["uses_atomics"]:
            d_out.zero()
        else:
            d_out.fill_bytes(0xFF)
        xc.launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, left.dtype, params)
        xc.sync()
        rec = xc.last_launch()
        assert rec["kernel"] == planned["kernel"] and rec["uses_atomics"] == planned["uses_atomics"] and rec["grid"] == planned["grid"]
        return d_out.to_numpy(out_shape, left.dtype), rec
    finally:
        d_left.free()
        d_right.free()
        d_out.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_few_small_pairs_whole_in_lds(oracle, dtype):
    """The one-output-row families on few small matrices with no tile or chunk named: every pair whole in LDS, one launch,
    plain stores into an output that nobody zeroed - one pair, one left against many, groups, all pairs; ragged shapes, more
    pairs than the device has CUs for a block each is not possible (at most 64 pairs), a count of pairs that does not divide
    the CUs is. A named chunk, more pairs or larger matrices keep the engine, and the planning call says which."""
    xc = load_package()
    rng = np.random.default_rng(777)
    wd = dict(warp_per_overlap_variant="work_distribution")
    one_pair = [("shuffle", {}), ("split_row", {}), ("split_row", dict(distribution_type="triangle")), ("multimat_right", {}),
                ("multimat_right", dict(distribution_type="rectangle")), ("multimat_both", {}), ("warp_per_overlap", wd),
                ("warp_per_overlap", dict(shifts_per_thread_block=8, distribution_type="rectangle", **wd))]
    for family, kw in one_pair:
        for shape in [(1, 1), (3, 5), (16, 16), (33, 17), (64, 64), (31, 97)]:
            say("one small pair", family, kw, np.dtype(dtype).name, shape)
            left, right = ints(rng, (1,) + shape, dtype), ints(rng, (1,) + shape, dtype)
            got, rec = run_as_planned(xc, family, left, right, 1, 1, 1, xc.make_params(**kw))
            assert "pair_in_lds" in rec["kernel"] and rec["uses_atomics"] == 0, rec
            check(got, oracle.one_to_one(left[0], right[0]), True, f"{family} {kw} {shape}")
    for shape, counts in [((16, 16), [(1, 2), (1, 32), (4, 4), (7, 9), (64, 1), (3, 1)]), ((32, 32), [(1, 8), (2, 8), (4, 4), (5, 3)]),
                          ((13, 7), [(1, 5), (6, 6)]), ((1, 1), [(2, 2)]), ((32, 9), [(3, 7)])]:
        for n_left, n_right in counts:
            say("few small pairs", np.dtype(dtype).name, shape, n_left, n_right)
            left = rng.standard_normal((n_left,) + shape).astype(dtype)
            right_all = rng.standard_normal((n_left * n_right,) + shape).astype(dtype)
            left_i, right_i = ints(rng, left.shape, dtype), ints(rng, right_all.shape, dtype)
            for l, r, exact in ((left_i, right_i, True), (left, right_all, False)):
                # groups: left l against its own n_right right matrices
                exp = np.concatenate([oracle.one_to_many(l[i:i + 1], r[i * n_right:(i + 1) * n_right]) for i in range(n_left)])
                family = "multimat_right_groups" if n_left > 1 else "multimat_right"
                for fam, kw in ((family, {}), (family, dict(distribution_type="triangle")), ("multimat_right_grouped", {})):
                    got, rec = run_as_planned(xc, fam, l, r, n_left * n_right, n_left, n_right, xc.make_params(**kw))
                    assert "pair_in_lds" in rec["kernel"] and rec["uses_atomics"] == 0, rec
                    check(got, exp, exact, f"{fam} {kw} {n_left}x{n_right} {shape}")
                # all pairs: every left against the first n_right right matrices
                exp = oracle.n_to_m(l, r[:n_right])
                for fam in ("multimat_both", "multimat_both_grouped"):
                    got, rec = run_as_planned(xc, fam, l, r[:n_right], n_left * n_right, n_left, n_right, xc.make_params())
                    assert "pair_in_lds" in rec["kernel"] and rec["uses_atomics"] == 0, rec
                    check(got, exp, exact, f"{fam} {n_left}x{n_right} {shape}")
    # what keeps the engine: a chunk or a tile named, whole_pair_in_lds = 2, more than 64 pairs, matrices beyond 32 x 32
    left, right = ints(rng, (8, 16, 16), dtype), ints(rng, (72, 16, 16), dtype)
    for family, n_left, n_right, kw in [("multimat_both", 8, 8, dict(rows_per_thread=8)), ("multimat_both", 8, 8, dict(whole_pair_in_lds=2)),
                                        ("multimat_both", 8, 8, dict(left_matrices_per_thread=2)), ("multimat_both", 8, 9, {}),
                                        ("multimat_right", 1, 72, {}), ("multimat_right", 1, 8, dict(right_matrices_per_thread=2)),
                                        ("multimat_both_grouped", 8, 8, dict(shifts_per_thread_right_matrix=4)), ("multimat_both_grouped", 8, 9, {})]:
        got, rec = run_as_planned(xc, family, left[:n_left], right[:n_right], n_left * n_right, n_left, n_right, xc.make_params(**kw))
        assert "pair_in_lds" not in rec["kernel"], (family, kw, rec)
        exp = oracle.n_to_m(left[:n_left], right[:n_right])
        check(got, exp, True, f"engine {family} {kw}")
    for shape, n in [((40, 40), 2), ((32, 32), 8)]:  # (64 pairs of 32x32 are more work than the whole-pair kernel is good for)
        left, right = ints(rng, (n,) + shape, dtype), ints(rng, (n,) + shape, dtype)
        got, rec = run_as_planned(xc, "multimat_both", left, right, n * n, n, n, xc.make_params())
        assert "pair_in_lds" not in rec["kernel"]
        check(got, oracle.n_to_m(left, right), True, f"engine {shape} {n}x{n}")
    # the LDS-staged wavefront-per-overlap family: the same route while none of its staging parameters is named
    left, right = ints(rng, (1, 24, 24), dtype), ints(rng, (8, 24, 24), dtype)
    for kw, routed in [({}, True), (dict(right_matrices_per_block=2), False), (dict(column_group_per_block=1), False), (dict(whole_pair_in_lds=2), False)]:
        got, rec = run_as_planned(xc, "warp_per_overlap_lds", left, right, 8, 1, 8, xc.make_params(**kw))
        assert ("pair_in_lds" in rec["kernel"]) == routed, (kw, rec)
        check(got, oracle.one_to_many(left, right), True, f"warp_per_overlap_lds {kw}")
    # forced (whole_pair_in_lds = 1): also beyond the sizes the launcher would pick it for
    left, right = ints(rng, (3, 20, 36), dtype), ints(rng, (70, 20, 36), dtype)
    got, rec = run_as_planned(xc, "multimat_both", left, right, 210, 3, 70, xc.make_params(whole_pair_in_lds=1))
    assert "pair_in_lds" in rec["kernel"], rec
    check(got, oracle.n_to_m(left, right), True, "forced multimat_both 3x70")
    got, rec = run_as_planned(xc, "warp_per_overlap_lds", left[:1], right, 70, 1, 70, xc.make_params(whole_pair_in_lds=1))
    assert "pair_in_lds" in rec["kernel"], rec
    check(got, oracle.one_to_many(left[:1], right), True, "forced warp_per_overlap_lds 1x70")


ONE_TO_MANY_CASES = [
    ("multimat_right", {}),
    ("multimat_right", dict(whole_pair_in_lds=2)),
    ("multimat_right", dict(right_matrices_per_thread=1)),
    ("multimat_right", dict(right_matrices_per_thread=8, warps_per_thread_block=4)),
    ("multimat_right", dict(right_matrices_per_thread=2, rows_per_thread=10, distribution_type="rectangle")),
    ("multimat_right", dict(right_matrices_per_thread=4, rows_per_thread=3, distribution_type="triangle")),
    ("multimat_right", dict(distribution_type="none", whole_pair_in_lds=2)),
    ("multimat_right", dict(distribution_type="triangle", whole_pair_in_lds=2)),
    ("multimat_right", dict(rows_per_thread=1, distribution_type="none")),
    ("multimat_right_grouped", {}),
    ("multimat_right_grouped", dict(shifts_per_thread_right_matrix=4, right_matrices_per_thread=4, left_rows_per_iteration=4)),
    ("multimat_right_grouped", dict(shifts_per_thread_right_matrix=2, right_matrices_per_thread=2, rows_per_thread=16)),
    ("multimat_both", dict(left_matrices_per_thread=1, right_matrices_per_thread=4)),
    ("multimat_both_grouped", {}),
    ("warp_per_overlap_lds", dict(right_matrices_per_block=1)),
    ("warp_per_overlap_lds", dict(right_matrices_per_block=8, shifts_per_thread_block=16)),
    ("warp_per_overlap_lds", dict(right_matrices_per_block=3, shifts_per_thread_block=5, shared_mem_rows=9)),
    ("warp_per_overlap_lds", dict(right_matrices_per_block=4, shifts_per_thread_block=8, column_group_per_block=1)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("family,kw", ONE_TO_MANY_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_one_to_many(oracle, dtype, family, kw):
    xc = load_package()
    rng = np.random.default_rng(200)
    for shape, n_right in [((5, 9), 1), ((16, 16), 3), ((33, 20), 7), ((64, 64), 19)]:
        say("one_to_many", family, kw, np.dtype(dtype).name, shape, n_right)
        left = ints(rng, (1,) + shape, dtype)
        right = ints(rng, (n_right,) + shape, dtype)
        exp = oracle.one_to_many(left, right)
        got = xc.run(family, left, right, n_right, n_left=1, n_right=n_right, params=xc.make_params(**kw))
        check(got, exp, True, f"{family} {kw} {shape}x{n_right} int")
        left = rng.standard_normal((1,) + shape).astype(dtype)
        right = rng.standard_normal((n_right,) + shape).astype(dtype)
        exp = oracle.one_to_many(left, right, threads=4)
        got = xc.run(family, left, right, n_right, n_left=1, n_right=n_right, params=xc.make_params(**kw))
        check(got, exp, False, f"{family} {kw} {shape}x{n_right} real")


def test_overlap_wise_batches(oracle):
    """run_cross_corr_naive_original's (subregions_per_pic, batch_size) layout: right matrix
    b*n + i pairs with left i, i.e. the n_to_mn file order of validate.hpp:264-269."""
    xc = load_package()
    rng = np.random.default_rng(300)
    for dtype in (np.float32, np.float64):
        for n_left, batch, shape in [(1, 5, (9, 6)), (3, 1, (8, 8)), (4, 3, (12, 17))]:
            say("overlap_wise batches", np.dtype(dtype).name, n_left, batch, shape)
            left = ints(rng, (n_left,) + shape, dtype)
            right = ints(rng, (n_left * batch,) + shape, dtype)
            exp = oracle.n_to_mn(left, right)
            got = xc.run("overlap_wise", left, right, n_left * batch, n_left=n_left, n_right=batch)
            check(got, exp, True, f"overlap_wise {n_left}x{batch}")
        # every right matrix with every left matrix in one launch (what the reference's host loops over, n_to_m.hpp:198-212)
        for n_left, n_right, shape in [(1, 4, (7, 9)), (3, 5, (16, 11)), (6, 2, (33, 20)), (3, 4, (10, 70))]:
            say("overlap_wise all pairs", np.dtype(dtype).name, n_left, n_right, shape)
            left = ints(rng, (n_left,) + shape, dtype)
            right = ints(rng, (n_right,) + shape, dtype)
            got = xc.run("overlap_wise_all_pairs", left, right, n_left * n_right, n_left=n_left, n_right=n_right)
            check(got, oracle.n_to_m(left, right), True, f"overlap_wise all pairs {n_left}x{n_right}")


N_TO_MN_CASES = [
    {},
    dict(shifts_per_thread_right_matrix=4, right_matrices_per_thread=4, left_rows_per_iteration=4),
    dict(shifts_per_thread_right_matrix=2, right_matrices_per_thread=1),
    dict(rows_per_thread=8, distribution_type="rectangle"),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kw", N_TO_MN_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_n_to_mn_one_launch(oracle, dtype, kw):
    """multimat_right_grouped with n_left > 1 takes the right matrices de-interleaved (left l
    owns [l*m, (l+1)*m), as the reference's n_to_mn classes arrange them, n_to_mn.hpp:165-172);
    the oracle works in file order, so the test interleaves around it with the reference's
    index map (matrix.hpp:614-618)."""
    xc = load_package()
    rng = np.random.default_rng(400)
    for n, m, shape in [(2, 3, (8, 8)), (3, 5, (20, 13)), (8, 4, (32, 32))]:
        say("n_to_mn", kw, np.dtype(dtype).name, n, m, shape)
        left = ints(rng, (n,) + shape, dtype)
        right_file = ints(rng, (n * m,) + shape, dtype)
        slot = [oracle.interleave_index(i, n * m, n) for i in range(n * m)]
        right_dev = np.empty_like(right_file)
        for i, s in enumerate(slot):
            right_dev[s] = right_file[i]
        exp_file = oracle.n_to_mn(left, right_file)
        got_dev = xc.run("multimat_right_grouped", left, right_dev, n * m, n_left=n, n_right=m, params=xc.make_params(**kw))
        got_file = np.stack([got_dev[slot[i]] for i in range(n * m)])
        check(got_file, exp_file, True, f"n_to_mn {n}x{m} {shape}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_many_left_matrices_with_few_right_ones_each(oracle, dtype):
    """n_to_mn with one or two right matrices per left matrix (independent pairs): no tile that lays lanes over the right
    matrices of ONE left matrix has anything to share. The launcher's pick for thousands of small fp32 pairs is a matrix-core
    tile whose sweep trims each 16 x 16 result tile to its own overlap (the register tile that lays eight lanes over left
    matrices with their own groups is what `matrix_cores` = 2 runs); bit-exact whatever it picks."""
    xc = load_package()
    rng = np.random.default_rng(420)
    picked = set()
    for n, m, shape in [(2000, 1, (32, 32)), (1000, 2, (32, 32)), (301, 1, (40, 36)), (77, 3, (33, 31)), (1500, 1, (20, 24)), (500, 1, (64, 64)),
                        (40, 1, (100, 90)), (1200, 1, (16, 16)), (900, 1, (17, 18))]:
        say("n_to_mn, few right matrices per left", np.dtype(dtype).name, n, m, shape)
        left = ints(rng, (n,) + shape, dtype)
        right = ints(rng, (n * m,) + shape, dtype)
        exp = oracle.n_to_mn(left, right, threads=16)          # file order: right i pairs with left i % n
        slot = [oracle.interleave_index(i, n * m, n) for i in range(n * m)]
        right_dev = np.empty_like(right)
        right_dev[slot] = right
        got_dev = xc.run("multimat_right_grouped", left, right_dev, n * m, n_left=n, n_right=m)
        picked.add(xc.last_launch()["kernel"])
        check(got_dev[slot], exp, True, f"n_to_mn {n}x{m} {shape}")
        if dtype == np.float32 and shape[0] <= 40:
            got_dev = xc.run("multimat_right_grouped", left, right_dev, n * m, n_left=n, n_right=m, params=xc.make_params(matrix_cores=2))
            picked.add(xc.last_launch()["kernel"])
            check(got_dev[slot], exp, True, f"n_to_mn {n}x{m} {shape}, vector FMAs")
    say("kernels:", sorted(picked))
    if dtype == np.float32:  # (fp64 has neither: the paired tile measured slower than the single-matrix tiles there)
        assert any("pairs8" in k for k in picked) and any("m64x64_s16" in k for k in picked) and any("m32x32_s16" in k for k in picked), picked


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kw", [{}, dict(whole_pair_in_lds=2), dict(distribution_type="none", whole_pair_in_lds=2),
                                dict(right_matrices_per_thread=4, distribution_type="rectangle"),
                                dict(right_matrices_per_thread=2, rows_per_thread=5, distribution_type="triangle"),
                                dict(rows_per_thread=1, distribution_type="none")], ids=lambda v: str(v).replace(" ", ""))
def test_multimat_right_groups(oracle, dtype, kw):
    """xcorr_multimat_right_groups: the one-output-row family over n_left groups in one launch gives what n_left calls of
    xcorr_multimat_right on the consecutive groups give (the loop of the reference's host, n_to_mn.hpp:286-300)."""
    xc = load_package()
    rng = np.random.default_rng(410)
    for n, m, shape in [(2, 3, (8, 8)), (3, 5, (20, 13)), (8, 4, (32, 32)), (5, 1, (17, 40))]:
        say("multimat_right_groups", kw, np.dtype(dtype).name, n, m, shape)
        left = ints(rng, (n,) + shape, dtype)
        right = ints(rng, (n * m,) + shape, dtype)
        exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * m:(l + 1) * m]) for l in range(n)])
        got = xc.run("multimat_right_groups", left, right, n * m, n_left=n, n_right=m, params=xc.make_params(**kw))
        check(got, exp, True, f"groups {n}x{m} {shape}")
        one_by_one = np.concatenate([xc.run("multimat_right", left[l:l + 1], right[l * m:(l + 1) * m], m, n_left=1, n_right=m,
                                            params=xc.make_params(**kw)) for l in range(n)])
        np.testing.assert_array_equal(got, one_by_one)


N_TO_M_CASES = [
    ("multimat_both", {}),
    ("multimat_both", dict(whole_pair_in_lds=2)),
    ("multimat_both", dict(left_matrices_per_thread=2, right_matrices_per_thread=2, rows_per_thread=10, distribution_type="triangle")),
    ("multimat_both", dict(left_matrices_per_thread=8, right_matrices_per_thread=8, rows_per_thread=3, distribution_type="rectangle")),
    ("multimat_both", dict(left_matrices_per_thread=1, right_matrices_per_thread=1, distribution_type="none")),
    ("multimat_both_grouped", {}),
    ("multimat_both_grouped", dict(shifts_per_thread_right_matrix=2, left_matrices_per_thread=2, right_matrices_per_thread=2, left_rows_per_iteration=2)),
    ("multimat_both_grouped", dict(shifts_per_thread_right_matrix=4, left_matrices_per_thread=4, right_matrices_per_thread=4)),
    ("multimat_both_grouped", dict(rows_per_thread=5)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("family,kw", N_TO_M_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_n_to_m(oracle, dtype, family, kw):
    xc = load_package()
    rng = np.random.default_rng(500)
    for n_left, n_right, shape in [(1, 1, (7, 7)), (2, 3, (16, 16)), (5, 9, (24, 31)), (16, 11, (32, 32))]:
        say("n_to_m", family, kw, np.dtype(dtype).name, n_left, n_right, shape)
        left = ints(rng, (n_left,) + shape, dtype)
        right = ints(rng, (n_right,) + shape, dtype)
        exp = oracle.n_to_m(left, right)
        got = xc.run(family, left, right, n_left * n_right, n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
        check(got, exp, True, f"{family} {kw} {n_left}x{n_right} {shape} int")
        left = rng.standard_normal((n_left,) + shape).astype(dtype)
        right = rng.standard_normal((n_right,) + shape).astype(dtype)
        exp = oracle.n_to_m(left, right, threads=4)
        got = xc.run(family, left, right, n_left * n_right, n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
        check(got, exp, False, f"{family} {kw} {n_left}x{n_right} {shape} real")


def test_every_tile_specialisation(oracle):
    """Forces each lane layout / register tile through the geometry fields and checks it on
    shapes that do not divide the tiles."""
    xc = load_package()
    rng = np.random.default_rng(600)
    layouts = [dict(lanes_x=8, lanes_y=8), dict(lanes_x=4, lanes_y=4), dict(lanes_x=2, lanes_y=2), dict(lanes_x=1, lanes_y=1)]
    for dtype in (np.float32, np.float64):
        for lay in layouts:
            for xs in (4, 8):
                for n_left, n_right, shape in [(3, 5, (19, 23)), (9, 17, (40, 36))]:
                    kw = dict(lay, x_shifts_per_thread=xs)
                    left = ints(rng, (n_left,) + shape, dtype)
                    right = ints(rng, (n_right,) + shape, dtype)
                    try:
                        got = xc.run("multimat_both_grouped", left, right, n_left * n_right, n_left=n_left, n_right=n_right,
                                     params=xc.make_params(**kw))
                    except xc.XcorrError as e:
                        assert e.code == 3, e  # no such specialisation compiled
                        continue
                    say("tile", np.dtype(dtype).name, kw, xc.last_launch()["kernel"], n_left, n_right, shape)
                    check(got, oracle.n_to_m(left, right), True, f"tile {kw} {shape}")


def test_every_compiled_specialisation_by_index(oracle):
    """Runs every entry of the specialisation tables (all register tiles, lane layouts and the
    ways wavefronts share a tile), unsplit and with the reduction split into atomically added
    chunks, on shapes that span several staged bands and do not divide any tile."""
    xc = load_package()
    rng = np.random.default_rng(650)
    for dtype in (np.float32, np.float64):
        cases = []
        for n_left, n_right, shape in [(3, 5, (19, 23)), (2, 3, (75, 45))]:
            left = ints(rng, (n_left,) + shape, dtype)
            right = ints(rng, (n_right,) + shape, dtype)
            cases.append((n_left, n_right, shape, left, right, oracle.n_to_m(left, right, threads=4)))
        # the tiles that pair every left matrix with its own group of right matrices only serve the n_to_mn layout
        group_cases = []
        for n_left, per_left, shape in [(11, 1, (19, 23)), (5, 3, (75, 45)), (9, 2, (33, 40))]:
            left = ints(rng, (n_left,) + shape, dtype)
            right = ints(rng, (n_left * per_left,) + shape, dtype)
            exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * per_left:(l + 1) * per_left]) for l in range(n_left)])
            group_cases.append((n_left, per_left, shape, left, right, exp))
        index, names = 1, []
        while True:
            try:
                for n_left, n_right, shape, left, right, exp in cases:
                    for rows in (0, 20):
                        kw = dict(specialisation=index, rows_per_thread=rows)
                        got = xc.run("multimat_both_grouped", left, right, n_left * n_right, n_left=n_left, n_right=n_right,
                                     params=xc.make_params(**kw))
                        rec = xc.last_launch()
                        check(got, exp, True, f"spec {index} {rec['kernel']} rows={rows} {shape}")
                names.append(rec["kernel"])
            except xc.XcorrError as e:
                if "own group only" in e.message:
                    for n_left, per_left, shape, left, right, exp in group_cases:
                        for rows in (0, 20):
                            kw = dict(specialisation=index, rows_per_thread=rows)
                            got = xc.run("multimat_right_grouped", left, right, n_left * per_left, n_left=n_left, n_right=per_left,
                                         params=xc.make_params(**kw))
                            rec = xc.last_launch()
                            check(got, exp, True, f"spec {index} {rec['kernel']} rows={rows} {n_left}x{per_left} {shape}")
                    names.append(rec["kernel"])
                else:
                    assert "does not exist" in e.message, e
                    break
            index += 1
        say(np.dtype(dtype).name, len(names), "specialisations:", " ".join(n.split("/")[1] for n in names))
        assert len(names) >= 9


def test_tuning_integers_are_exact_requests(oracle):
    """The reference's shifts / matrices per thread, when non-zero, pick the nearest compiled tile at or above them
    (xcorr_last_launch tells which); zero leaves the choice to the launcher. Results do not depend on the tile."""
    xc = load_package()
    rng = np.random.default_rng(11)
    left, right = ints(rng, (130, 150), np.float32), ints(rng, (130, 150), np.float32)
    exp = oracle.one_to_one(left, right)
    for asked, want in [(1, 4), (2, 4), (4, 4), (5, 8), (8, 8)]:
        got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(shifts_per_thread=asked))
        rec = xc.last_launch()
        assert rec["y_shifts_per_thread"] == want, (asked, rec)
        check(got, exp, True, f"grouped shifts_per_thread={asked}")
    for dtype in (np.float32, np.float64):
        left, right = ints(rng, (1, 40, 40), dtype), ints(rng, (20, 40, 40), dtype)
        exp = oracle.one_to_many(left[0], right)
        for asked in (1, 2, 4):
            got = xc.run("multimat_right_grouped", left, right, 20, n_left=1, n_right=20, params=xc.make_params(right_matrices_per_thread=asked))
            rec = xc.last_launch()
            have = rec["right_matrices_per_thread"] * rec["lanes_right"]
            assert have == (1 if asked == 1 else 4), (asked, rec)
            check(got, exp, True, f"right_matrices_per_thread={asked}")
        left, right = ints(rng, (6, 24, 24), dtype), ints(rng, (9, 24, 24), dtype)
        exp = oracle.n_to_m(left, right)
        for lm, rm in [(1, 1), (4, 4), (3, 2), (4, 1)]:
            got = xc.run("multimat_both_grouped", left, right, 54, n_left=6, n_right=9,
                         params=xc.make_params(left_matrices_per_thread=lm, right_matrices_per_thread=rm))
            rec = xc.last_launch()
            assert rec["right_matrices_per_thread"] * rec["lanes_right"] >= rm and rec["left_matrices_per_thread"] * rec["lanes_left"] >= lm, (lm, rm, rec)
            if (lm, rm) == (1, 1):
                assert rec["lanes_right"] == 1 and rec["lanes_left"] == 1, rec
            check(got, exp, True, f"left/right matrices per thread {lm}/{rm}")
        # one-output-row families
        got = xc.run("multimat_both", left, right, 54, n_left=6, n_right=9, params=xc.make_params(left_matrices_per_thread=2, right_matrices_per_thread=2, rows_per_thread=8))
        rec = xc.last_launch()
        assert rec["left_matrices_per_thread"] == 2 and rec["right_matrices_per_thread"] == 2, rec
        check(got, exp, True, "multimat_both 2/2")
        got = xc.run("multimat_both", left, right, 54, n_left=6, n_right=9, params=xc.make_params(left_matrices_per_thread=1, right_matrices_per_thread=1, rows_per_thread=8))
        rec = xc.last_launch()
        assert rec["left_matrices_per_thread"] == 1 and rec["right_matrices_per_thread"] == 1, rec
        check(got, exp, True, "multimat_both 1/1")


def test_launch_record_and_errors(oracle):
    xc = load_package()
    rng = np.random.default_rng(700)
    left = ints(rng, (32, 32), np.float32)
    xc.run("grouped_overlap", left, left, 1, params=xc.make_params(shifts_per_thread=8))
    rec = xc.last_launch()
    say(rec)
    assert rec["kernel"].startswith("grouped_overlap/")
    assert rec["y_shifts_per_thread"] in (4, 8) and rec["block"][0] % 64 == 0 and rec["grid"][0] >= 1
    assert 1 <= rec["blocks_per_cu"] <= 16  # occupancy the planner's run-time model works with
    # the geometry fields select a tile exactly
    xc.run("grouped_overlap", left, left, 1, params=xc.make_params(x_shifts_per_thread=8, lanes_x=8, lanes_y=8))
    rec = xc.last_launch()
    assert rec["x_shifts_per_thread"] == 8 and rec["lanes_x"] == 8 and rec["lanes_y"] == 8
    # the planner cuts the reduction of a small multi-matrix problem into chunks (atomic adds into an output it
    # clears itself) also for tiles whose lanes lie over matrices; an explicit rows_per_thread is taken as it is
    one, many = ints(rng, (1, 96, 96), np.float32), ints(rng, (8, 96, 96), np.float32)
    got = xc.run("multimat_right_grouped", one, many, 8, n_left=1, n_right=8, params=xc.make_params(specialisation=14, rows_per_thread=36))
    rec = xc.last_launch()
    assert rec["lanes_right"] == 8 and rec["uses_atomics"] == 1 and rec["rows_per_worker"] == 36
    np.testing.assert_array_equal(got, oracle.one_to_many(one, many))
    with pytest.raises(xc.XcorrError, match="Too many shifts per thread"):
        xc.run("grouped_overlap", left, left, 1, params=xc.make_params(shifts_per_thread=9))
    with pytest.raises(xc.XcorrError, match="Too many warps"):
        xc.run("split_row", left, left, 1, params=xc.make_params(warps_per_thread_block=64))
    info = xc.device_info()
    say(info.name, info.arch, info.compute_units, info.clock_khz, info.fp32_vector_peak_tflops)
    assert b"gfx950" in info.arch


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_planner_choices_for_few_matrices_of_medium_size(oracle, dtype):
    """Problems with too few tiles to fill the GPU: the planner's run-time model cuts the reduction over
    left rows into chunks (atomic adds into an output it clears itself), also for tiles whose lanes lie
    over matrices, or falls back to the small tile. Whatever it picks, integer-valued inputs must match
    the oracle exactly; the plan is printed."""
    xc = load_package()
    rng = np.random.default_rng(800)
    for family, mode, n_left, n_right, shape in [("multimat_right_grouped", "one_to_many", 1, 32, (96, 80)),
                                                 ("multimat_right_grouped", "one_to_many", 1, 8, (128, 128)),
                                                 ("multimat_both_grouped", "n_to_m", 4, 8, (96, 96)),
                                                 ("multimat_both_grouped", "n_to_m", 16, 16, (40, 24))]:
        left = ints(rng, (n_left,) + shape, dtype)
        right = ints(rng, (n_right,) + shape, dtype)
        n_out = n_left * n_right if mode == "n_to_m" else n_right
        exp = getattr(oracle, mode)(left, right, threads=8)
        for kw in ({}, dict(rows_per_thread=27), dict(rows_per_thread=1000)):
            got = xc.run(family, left, right, n_out, n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
            rec = xc.last_launch()
            say(mode, np.dtype(dtype).name, n_left, n_right, shape, kw, rec["kernel"], "rows", rec["rows_per_worker"], "grid", rec["grid"][0],
                "atomics", rec["uses_atomics"])
            if kw.get("rows_per_thread") == 27:
                assert rec["rows_per_worker"] == 27 and rec["uses_atomics"] == 1
            if kw.get("rows_per_thread") == 1000:
                assert rec["rows_per_worker"] == shape[0] and rec["uses_atomics"] == 0
            check(got, exp, True, f"{mode} {n_left}x{n_right} {shape} {kw}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reduction_cut_over_columns(oracle, dtype):
    """column_chunks cuts the reduction over right columns into work items that add atomically (on top of, or
    instead of, the cut over left rows); every grouped tile, more chunks than columns allow, ragged widths."""
    xc = load_package()
    rng = np.random.default_rng(900)
    n_specs = 17 if dtype == np.float32 else 14
    first_grouped = 4 if dtype == np.float32 else 3
    for family, mode, n_left, n_right, shape in [("grouped_overlap", "one_to_one", 1, 1, (40, 70)),
                                                 ("multimat_right_grouped", "one_to_many", 1, 5, (33, 18)),
                                                 ("multimat_both_grouped", "n_to_m", 3, 4, (21, 47))]:
        left = ints(rng, (n_left,) + shape, dtype)
        right = ints(rng, (n_right,) + shape, dtype)
        n_out = n_left * n_right if mode == "n_to_m" else n_right
        exp = getattr(oracle, mode)(left, right)
        for spec in range(first_grouped, n_specs + 1):
            for chunks, rows in [(2, 0), (3, 9), (8, 1000), (64, 0)]:
                got = xc.run(family, left, right, n_out, n_left=n_left, n_right=n_right,
                             params=xc.make_params(specialisation=spec, column_chunks=chunks, rows_per_thread=rows))
                rec = xc.last_launch()
                say(mode, np.dtype(dtype).name, shape, "spec", spec, rec["kernel"], "column chunks", rec["column_chunks"], "rows", rec["rows_per_worker"],
                    "grid", rec["grid"][0])
                assert rec["uses_atomics"] == 1 and 2 <= rec["column_chunks"] <= chunks
                check(got, exp, True, f"{mode} spec {spec} chunks {chunks} rows {rows}")
        # left to the planner, small problems are cut over columns too
        got = xc.run(family, left, right, n_out, n_left=n_left, n_right=n_right)
        say(mode, "planner", xc.last_launch())
        check(got, exp, True, f"{mode} planner")
