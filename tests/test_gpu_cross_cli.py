"""GPU tests of the `cross` binary: every algorithm name runs end to end (CSV in, kernels
through the C ABI, CSV out), validates against the binary's own host computation and against
the oracle, and writes the reference's measurement CSV."""
import numpy as np
import pytest

from cross_cli import read_matrices, run_cross, write_args, write_matrices

pytestmark = pytest.mark.gpu

MODE_SHAPES = {
    "one_to_one": (1, 1),
    "one_to_many": (1, 5),
    "n_to_mn": (3, 6),
    "n_to_m": (3, 4),
}


def mode_of(name):
    for m in ("one_to_one", "one_to_many", "n_to_mn", "n_to_m"):
        if name.endswith(m):
            return m
    raise AssertionError(name)


def expected(oracle, mode, left, right):
    return getattr(oracle, mode)(left, right)


def gpu_names():
    import subprocess

    from cross_cli import cross_path

    out = subprocess.run([cross_path(), "list"], capture_output=True, text=True).stdout.split()
    return [n for n in out if not n.startswith(("cpu_", "fft_"))]


@pytest.mark.parametrize("dtype", ["single", "double"])
def test_every_algorithm_name(tmp_path, oracle, dtype):
    rng = np.random.default_rng(42)
    np_dtype = np.float32 if dtype == "single" else np.float64
    inputs = {}
    for mode, (n_left, n_right) in MODE_SHAPES.items():
        left = rng.integers(-4, 5, size=(n_left, 21, 18)).astype(np_dtype)
        right = rng.integers(-4, 5, size=(n_right, 21, 18)).astype(np_dtype)
        inputs[mode] = (left, right, write_matrices(tmp_path / f"l_{mode}.csv", left), write_matrices(tmp_path / f"r_{mode}.csv", right))
    names = gpu_names()
    assert len(names) == 31
    for name in names:
        print("cross run", dtype, name, flush=True)
        mode = mode_of(name)
        left, right, lp, rp = inputs[mode]
        out_path = tmp_path / f"{name}.csv"
        rc, out, err = run_cross("run", "-d", dtype, "--out", out_path, "--validate", "--no_progress", "-b", "Algorithm", "-m", "0.0001",
                                 "-t", tmp_path / f"{name}_t.csv", name, lp, rp, cwd=tmp_path)
        assert rc == 0, (name, err)
        lines = out.strip().splitlines()
        assert lines[0] == "Max,Mean,Stddev", (name, out)
        assert float(lines[1].split(",")[0]) == 0.0, (name, out)  # integer-valued inputs: exact
        # output file is in the inputs' file order whatever the device layout was
        np.testing.assert_array_equal(read_matrices(out_path), expected(oracle, mode, left, right), err_msg=name)
        header, row = (tmp_path / f"{name}_t.csv").read_text().strip().splitlines()
        assert header.split(",")[:2] == ["Kernel", "Kernel_iterations"], name
        assert int(row.split(",")[0]) > 0 and int(row.split(",")[1]) >= 1, (name, row)
        assert len(header.split(",")) == len(row.split(",")), name


def test_json_arguments_and_properties(tmp_path, oracle):
    rng = np.random.default_rng(43)
    left = rng.random((1, 40, 33), dtype=np.float32)
    right = rng.random((7, 40, 33), dtype=np.float32)
    lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
    args = write_args(tmp_path / "a.json", warps_per_thread_block=4, shifts_per_thread_right_matrix=2, right_matrices_per_thread=2,
                      left_rows_per_iteration=1)
    rc, out, err = run_cross("run", "--args_path", args, "--validate", "--no_progress", "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "t.csv",
                             "--out", tmp_path / "o.csv", "nai_shuffle_multirow_both_multimat_right_one_to_many", lp, rp, cwd=tmp_path)
    assert rc == 0, err
    assert float(out.strip().splitlines()[1].split(",")[0]) < 1e-5
    header, row = (tmp_path / "t.csv").read_text().strip().splitlines()
    assert header == "Kernel,Kernel_iterations,warps_per_thread_block,shifts_per_thread_right_matrix,right_matrices_per_thread,left_rows_per_iteration"
    # the tile-selecting integers are exact requests, answered by the nearest compiled tile at or above them, and the
    # measurement file reports what ran: 2 y shifts -> the 4-shift tile, 2 right matrices -> 4 (one per lane, four lanes)
    assert row.split(",")[2:] == ["4", "4", "4", "1"]
    got = read_matrices(tmp_path / "o.csv")
    exp = oracle.one_to_many(left, right)
    assert np.abs(got - exp).max() <= 1e-3 * np.abs(exp).max()
    # a tuning value above the reference's limit fails inside the computation phase: exit code 3
    args = write_args(tmp_path / "b.json", shifts_per_thread=9)
    rc, _, err = run_cross("run", "--args_path", args, "nai_shuffle_multirow_both_one_to_one", lp, lp, cwd=tmp_path)
    assert rc == 3 and "Exception occured durign computation step: Too many shifts per thread: 9 (max 8)" in err
    assert "Last kernel launch arguments:" in err
    # distribution names and the split-row properties
    args = write_args(tmp_path / "c.json", rows_per_thread=4, distribution_type="triangle")
    rc, _, err = run_cross("run", "--args_path", args, "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "t2.csv", "--validate", "--no_progress",
                           "nai_shuffle_work_distribution_one_to_one", lp, lp, cwd=tmp_path)
    assert rc == 0, err
    header, row = (tmp_path / "t2.csv").read_text().strip().splitlines()
    assert header.endswith("warps_per_thread_block,rows_per_thread,distribution_type") and row.endswith("8,4,triangle")
    # without rows_per_thread in the file the library picks the chunk (not the reference's 10) and the measurement file
    # reports it: a pair this small runs whole in LDS without any split (and the binary, which asks first, does not clear
    # the output) ...
    args = write_args(tmp_path / "d.json", distribution_type="rectangle")
    rc, _, err = run_cross("run", "--args_path", args, "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "t3.csv", "--validate", "--no_progress",
                           "nai_shuffle_work_distribution_one_to_one", lp, lp, cwd=tmp_path)
    assert rc == 0, err
    header, row = (tmp_path / "t3.csv").read_text().strip().splitlines()
    warps, chunk, dist = row.split(",")[-3:]
    assert (warps, chunk, dist) == ("8", "40", "none"), row
    # ... a larger one is cut into chunks of rows
    big = write_matrices(tmp_path / "big.csv", rng.random((1, 150, 140), dtype=np.float32))
    rc, out, err = run_cross("run", "--args_path", args, "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "t4.csv", "--validate", "--no_progress",
                             "nai_shuffle_work_distribution_one_to_one", big, big, cwd=tmp_path)
    assert rc == 0, err
    assert float(out.strip().splitlines()[1].split(",")[0]) < 1e-5
    header, row = (tmp_path / "t4.csv").read_text().strip().splitlines()
    warps, chunk, dist = row.split(",")[-3:]
    assert warps == "8" and dist in ("rectangle", "triangle") and 1 <= int(chunk) < 150, row


def test_tuning_integers_select_tiles(tmp_path, oracle):
    """shifts_per_thread 4 / 8 in the arguments file run the 4- / 8-shift tiles (reported in the measurement file);
    without the key the library chooses by itself; results are the same."""
    rng = np.random.default_rng(45)
    left = rng.integers(-3, 4, (1, 150, 140)).astype(np.float32)
    right = rng.integers(-3, 4, (1, 150, 140)).astype(np.float32)
    lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
    exp = oracle.one_to_one(left[0], right[0])
    seen = {}
    for label, kw in [("none", {}), ("four", dict(shifts_per_thread=4)), ("eight", dict(shifts_per_thread=8)), ("three", dict(shifts_per_thread=3)),
                      ("five", dict(shifts_per_thread=5))]:
        args = write_args(tmp_path / f"{label}.json", **kw)
        rc, out, err = run_cross("run", "--args_path", args, "--no_progress", "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / f"{label}_t.csv",
                                 "--out", tmp_path / f"{label}_o.csv", "nai_shuffle_multirow_both_one_to_one", lp, rp, cwd=tmp_path)
        assert rc == 0, err
        header, row = (tmp_path / f"{label}_t.csv").read_text().strip().splitlines()
        seen[label] = dict(zip(header.split(","), row.split(",")))["shifts_per_thread"]
        np.testing.assert_array_equal(read_matrices(tmp_path / f"{label}_o.csv")[0], exp[0], err_msg=label)
    assert seen["four"] == "4" and seen["three"] == "4" and seen["eight"] == "8" and seen["five"] == "8", seen
    assert seen["none"] in ("4", "8", "16")  # 16: the matrix-core tile, a lane holds 16 y shifts of its 32 x 32 result tile
    # n_to_m: matrices per thread pick the lanes-over-matrices tiles
    left = rng.integers(-3, 4, (8, 30, 30)).astype(np.float32)
    right = rng.integers(-3, 4, (8, 30, 30)).astype(np.float32)
    lp, rp = write_matrices(tmp_path / "l8.csv", left), write_matrices(tmp_path / "r8.csv", right)
    exp = oracle.n_to_m(left, right)
    for lm, rm in [(1, 1), (4, 4), (2, 3)]:
        args = write_args(tmp_path / "m.json", left_matrices_per_thread=lm, right_matrices_per_thread=rm)
        rc, out, err = run_cross("run", "--args_path", args, "--no_progress", "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "m_t.csv",
                                 "--out", tmp_path / "m_o.csv", "nai_shuffle_multirow_both_multimat_both_n_to_m", lp, rp, cwd=tmp_path)
        assert rc == 0, err
        header, row = (tmp_path / "m_t.csv").read_text().strip().splitlines()
        props = dict(zip(header.split(","), row.split(",")))
        assert int(props["left_matrices_per_thread"]) >= lm and int(props["right_matrices_per_thread"]) >= rm, props
        if (lm, rm) == (1, 1):
            assert props["left_matrices_per_thread"] == "1" and props["right_matrices_per_thread"] == "1", props
        if (lm, rm) == (4, 4):
            assert props["left_matrices_per_thread"] == "4" and props["right_matrices_per_thread"] == "4", props
        np.testing.assert_array_equal(read_matrices(tmp_path / "m_o.csv"), exp)


def test_fft_algorithm_repeated_by_min_time_still_validates(tmp_path, oracle):
    """An fft_* algorithm measured with a min_time that forces many repetitions: the in-place hadamard and the
    input-consuming inverse transform are repeated, and the stored / validated result must still be that of one pass."""
    rng = np.random.default_rng(46)
    left = rng.random((1, 32, 32), dtype=np.float32)
    right = rng.random((1, 32, 32), dtype=np.float32)
    lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
    rc, out, err = run_cross("run", "--validate", "--normalize", "--no_progress", "-b", "Algorithm", "-m", "0.02", "-t", tmp_path / "t.csv",
                             "--out", tmp_path / "o.csv", "fft_orig_one_to_one", lp, rp, cwd=tmp_path)
    assert rc == 0, err
    header, row = (tmp_path / "t.csv").read_text().strip().splitlines()
    cols = dict(zip(header.split(","), row.split(",")))
    assert int(cols["Hadamard_iterations"]) > 1 and int(cols["Inverse FFT_iterations"]) > 1, cols
    exp = oracle.one_to_one(left[0], right[0])
    assert float(out.strip().splitlines()[1].split(",")[0]) <= 1e-3 * np.abs(exp).max(), out
    got = read_matrices(tmp_path / "o.csv")
    assert np.abs(got - exp).max() <= 1e-4 * np.abs(exp).max()


def test_common_steps_and_streams(tmp_path, oracle):
    rng = np.random.default_rng(44)
    left = rng.random((4, 24, 24), dtype=np.float32)
    right = rng.random((8, 24, 24), dtype=np.float32)
    lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
    for streams in (1, 3, 20):
        args = write_args(tmp_path / "s.json", num_cuda_streams=streams)
        rc, out, err = run_cross("run", "--args_path", args, "--validate", "--no_progress", "-b", "CommonSteps", "-m", "0.001", "-t", tmp_path / "t.csv",
                                 "--out", tmp_path / "o.csv", "nai_shuffle_multirow_both_multimat_right_n_to_mn", lp, rp, cwd=tmp_path)
        assert rc == 0, err
        assert float(out.strip().splitlines()[1].split(",")[0]) < 1e-5
        header, row = (tmp_path / "t.csv").read_text().strip().splitlines()
        assert header.startswith("Load,Load_iterations,Prepare,Prepare_iterations,Transfer,") and header.endswith(",num_cuda_streams")
        assert row.endswith("," + str(streams))
        got = read_matrices(tmp_path / "o.csv")
        exp = oracle.n_to_mn(left, right)
        assert np.abs(got - exp).max() <= 1e-3 * np.abs(exp).max()
    # without the key: one launch over all left matrices, device-event timing, the default is still reported
    rc, out, err = run_cross("run", "--validate", "--no_progress", "-b", "Algorithm", "-m", "0.001", "-t", tmp_path / "t1.csv",
                             "--out", tmp_path / "o1.csv", "nai_shuffle_multirow_both_multimat_right_n_to_mn", lp, rp, cwd=tmp_path)
    assert rc == 0, err
    header, row = (tmp_path / "t1.csv").read_text().strip().splitlines()
    assert header.endswith(",num_cuda_streams") and row.endswith(",8")
    got = read_matrices(tmp_path / "o1.csv")
    assert np.abs(got - exp).max() <= 1e-3 * np.abs(exp).max()
