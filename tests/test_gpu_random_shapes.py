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


def test_random_parameters(oracle):
    """Random legal values of the reference's per-algorithm arguments (variants, block sizes, rows per
    thread, matrices per thread, distributions, shared-memory geometry) on random shapes. A combination
    the library rejects must be rejected with an argument error, never computed wrongly."""
    xc = load_package()
    rng = np.random.default_rng(20233)
    fams = ["overlap_wise", "warp_per_overlap", "warp_per_overlap_lds", "block_per_overlap", "shuffle", "split_row",
            "multimat_right", "multimat_both", "grouped_overlap", "multimat_right_grouped", "multimat_both_grouped"]

    def ri(a, b):
        return int(rng.integers(a, b))

    rejected = 0
    for case in range(8 * len(fams)):
        fam = fams[case % len(fams)]
        dtype = (np.float32, np.float64)[(case // len(fams)) % 2]
        small = fam in ("overlap_wise", "warp_per_overlap", "warp_per_overlap_lds", "block_per_overlap")
        rows, cols = ri(1, 60 if small else 150), ri(1, 60 if small else 150)
        n_left = n_right = 1
        kw = {}
        if fam == "overlap_wise":
            n_left, n_right = ri(1, 5), ri(1, 5)  # n_right: batch of right matrices per left one
            left, right = ints(rng, (n_left, rows, cols), dtype), ints(rng, (n_left * n_right, rows, cols), dtype)
            exp = np.stack([oracle.one_to_one(left[i % n_left], right[i], threads=4) for i in range(n_left * n_right)])
        elif fam in ("warp_per_overlap", "block_per_overlap", "shuffle", "split_row", "grouped_overlap"):
            left, right = ints(rng, (rows, cols), dtype), ints(rng, (rows, cols), dtype)
            exp = oracle.one_to_one(left, right, threads=4)[None]
            if fam == "warp_per_overlap":
                kw = dict(warp_per_overlap_variant=ri(0, 3), shifts_per_thread_block=ri(0, 33))
                if kw["warp_per_overlap_variant"] == 2:
                    kw.update(rows_per_thread=ri(1, rows + 4), distribution_type=ri(0, 4))
            elif fam == "block_per_overlap":
                kw = dict(block_size=int(rng.choice([0, 64, 128, 192, 256, 512, 1024])))
            elif fam == "shuffle":
                kw = dict(warps_per_thread_block=ri(0, 33))
            elif fam == "split_row":
                kw = dict(warps_per_thread_block=ri(0, 33), rows_per_thread=ri(0, rows + 4), distribution_type=ri(0, 4))
            else:
                kw = dict(shifts_per_thread=ri(0, 9), rows_per_thread=ri(0, rows + 4), left_rows_per_iteration=ri(0, 9),
                          distribution_type=ri(0, 4), column_chunks=ri(0, 5))
        elif fam in ("warp_per_overlap_lds", "multimat_right"):
            n_right = ri(1, 14)
            left, right = ints(rng, (1, rows, cols), dtype), ints(rng, (n_right, rows, cols), dtype)
            exp = oracle.one_to_many(left, right, threads=4)
            if fam == "warp_per_overlap_lds":
                spb = ri(0, 33)
                kw = dict(shifts_per_thread_block=spb, right_matrices_per_block=ri(0, 9), strided_load=ri(0, 2),
                          column_group_per_block=ri(0, 2), shared_mem_row_size=int(rng.choice([0, 32, 64, 128])))
                if rng.random() < 0.5:
                    kw["shared_mem_rows"] = min(max(spb, 1), 16) + ri(0, 20)
            else:
                kw = dict(warps_per_thread_block=ri(0, 33), right_matrices_per_thread=ri(0, 9))
                if rng.random() < 0.5:
                    kw.update(rows_per_thread=ri(1, rows + 4), distribution_type=ri(0, 4))
        else:
            n_left, n_right = ri(1, 6), ri(1, 10)
            left = ints(rng, (n_left, rows, cols), dtype)
            if fam == "multimat_right_grouped":  # n_to_mn: n_right right matrices per left one, grouped by left matrix
                right = ints(rng, (n_left * n_right, rows, cols), dtype)
                exp = np.concatenate([oracle.one_to_many(left[l:l + 1], right[l * n_right:(l + 1) * n_right], threads=4)
                                      for l in range(n_left)])
                kw = dict(shifts_per_thread_right_matrix=ri(0, 5), right_matrices_per_thread=ri(0, 5),
                          left_rows_per_iteration=ri(0, 5), rows_per_thread=ri(0, rows + 4), distribution_type=ri(0, 4))
            else:
                right = ints(rng, (n_right, rows, cols), dtype)
                exp = oracle.n_to_m(left, right, threads=4)
                if fam == "multimat_both":
                    kw = dict(warps_per_thread_block=ri(0, 33), left_matrices_per_thread=ri(0, 9), right_matrices_per_thread=ri(0, 9),
                              rows_per_thread=ri(0, rows + 4), distribution_type=ri(0, 4))
                else:
                    kw = dict(shifts_per_thread_right_matrix=ri(0, 5), left_matrices_per_thread=ri(0, 5),
                              right_matrices_per_thread=ri(0, 5), rows_per_thread=ri(0, rows + 4), distribution_type=ri(0, 4))
        print("case", case, fam, np.dtype(dtype).name, rows, cols, n_left, n_right, kw, flush=True)
        try:
            got = xc.run(fam, left, right, exp.shape[0], n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
        except xc.XcorrError as e:
            assert e.code == 1, (case, fam, kw, e.message)  # XCORR_ERR_INVALID_ARGUMENT
            rejected += 1
            continue
        assert np.array_equal(got.reshape(exp.shape), exp), (case, fam, rows, cols, kw, xc.last_launch()["kernel"])
    assert rejected <= 8
