"""GPU tests of the FFT comparison path: the C ABI of libxcorr_fft.so (hipFFT plans, hadamard and
scatter kernels) through ctypes, and the seven fft_* algorithm names of the `cross` binary.

Tolerances: an FFT-based correlation is not bit-exact even for integer inputs. With values of
magnitude <= 4 and up to 48x40 overlaps the result magnitudes are ~1e3; hipFFT's rounding error is
a few ulp of the largest spectrum value, so the bound is relative to the LARGEST element of the
expected result: 2e-5 in fp32, 1e-12 in fp64."""
import importlib

import numpy as np
import pytest

from conftest import load_package
from cross_cli import read_matrices, run_cross, write_args, write_matrices

pytestmark = pytest.mark.gpu

TOL = {np.float32: 2e-5, np.float64: 1e-12}
SHAPES = {"one_to_one": (1, 1), "one_to_many": (1, 5), "n_to_mn": (3, 6), "n_to_m": (3, 4)}


def fft_module():
    return importlib.import_module(load_package().__name__ + ".fft")


def close(got, exp, dtype, file_rounding=0.0):
    return np.abs(got.astype(np.float64) - exp).max() <= TOL[dtype] * np.abs(exp).max() + file_rounding


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rows,cols", [(16, 16), (21, 18), (5, 48), (1, 9)])
def test_c_abi_path_against_oracle(oracle, dtype, rows, cols):
    fft = fft_module()
    rng = np.random.default_rng(rows * 100 + cols)
    cases = [("one_to_one", "original"), ("one_to_one", "reduced_transfer"), ("one_to_many", "original"),
             ("one_to_many", "reduced_transfer"), ("n_to_mn", "original"), ("n_to_mn", "reduced_transfer"),
             ("n_to_m", "over_output"), ("n_to_m", "over_right")]
    for mode, variant in cases:
        print("fft", mode, variant, np.dtype(dtype).name, rows, cols, flush=True)
        n_left, n_right = SHAPES[mode]
        left = rng.integers(-4, 5, size=(n_left, rows, cols)).astype(dtype)
        right = rng.integers(-4, 5, size=(n_right, rows, cols)).astype(dtype)
        for threads, items in [(256, 10), (64, 1), (1024, 3)]:
            raw = fft.cross_correlate(left, right, mode, variant, threads=threads, items=items)
            assert raw.shape == (SHAPES[mode][1] if mode != "n_to_m" else n_left * n_right, 2 * rows, 2 * cols)
            got = fft.normalize(raw)
            exp = getattr(oracle, mode)(left.astype(np.float64), right.astype(np.float64))
            assert close(got, exp, dtype), (mode, variant, threads, items, np.abs(got - exp).max())
            # the dropped middle row and column of the circular result hold no overlap
            assert np.abs(raw[:, rows, :]).max() <= TOL[dtype] * np.abs(exp).max() * raw[0].size
            assert np.abs(raw[:, :, cols]).max() <= TOL[dtype] * np.abs(exp).max() * raw[0].size


def fft_names():
    import subprocess

    from cross_cli import cross_path

    out = subprocess.run([cross_path(), "list"], capture_output=True, text=True).stdout.split()
    return [n for n in out if n.startswith("fft_")]


@pytest.mark.parametrize("dtype", ["single", "double"])
def test_every_fft_algorithm_name(tmp_path, oracle, dtype):
    np_dtype = np.float32 if dtype == "single" else np.float64
    rng = np.random.default_rng(46)
    names = fft_names()
    assert len(names) == 7
    for name in names:
        mode = next(m for m in ("one_to_one", "one_to_many", "n_to_mn", "n_to_m") if name.endswith(m))
        n_left, n_right = SHAPES[mode]
        # positive values: no result element cancels to zero, where the binary's relative difference
        # (|a-b| / max(|a|,|b|), validate.hpp:134-188) of an FFT result would read 1
        left = rng.random((n_left, 21, 18)).astype(np_dtype)
        right = rng.random((n_right, 21, 18)).astype(np_dtype)
        lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
        exp = getattr(oracle, mode)(left.astype(np.float64), right.astype(np.float64))
        print("cross run", dtype, name, flush=True)
        # Algorithm measurements with a minimum time: the adaptive loop repeats the phases that consume
        # their inputs, the stored result must still be that of one pass
        rc, out, err = run_cross("run", "-d", dtype, "--out", tmp_path / "raw.csv", "--validate", "--no_progress", "-b", "Algorithm",
                                 "-m", "0.0001", "-t", tmp_path / "t.csv", name, lp, rp, cwd=tmp_path)
        assert rc == 0, (name, err)
        lines = out.strip().splitlines()
        # per-element relative difference: corner elements (one-element overlaps, ~1e-3) carry the absolute
        # error of the whole transform, hence the loose maximum and the tight mean in single precision
        mx, mean = (float(x) for x in lines[1].split(",")[:2])
        assert lines[0] == "Max,Mean,Stddev" and mx < (5e-2 if dtype == "single" else 1e-9) and mean < (1e-4 if dtype == "single" else 1e-12), (name, out)
        raw = read_matrices(tmp_path / "raw.csv")
        assert raw.shape == (exp.shape[0], 42, 36), name  # raw circular result of the padded size
        header, row = (tmp_path / "t.csv").read_text().strip().splitlines()
        labels = header.split(",")
        if "reduced_transfer" in name:
            assert labels[:14:2] == ["Forward FFT", "Hadamard", "Inverse FFT", "ToDevice", "Scatter", "Allocation", "Plan"], name
            assert labels[14:] == ["scatter_threads_per_block", "scatter_items_per_thread", "hadamard_threads_per_block"], name
        else:
            assert labels[:10:2] == ["Forward FFT", "Hadamard", "Inverse FFT", "Allocation", "Plan"], name
            assert labels[10:] == ["hadamard_threads_per_block"] + (["hadamard_items_per_thread"] if "better" in name else []), name
        assert len(labels) == len(row.split(",")), name
        # --normalize stores the definition's layout; `cross validate --normalize` does the same to a raw file
        args = write_args(tmp_path / "a.json", hadamard_threads_per_block=128, hadamard_items_per_thread=3, scatter_threads_per_block=64,
                          scatter_items_per_thread=2)
        rc, out, err = run_cross("run", "-d", dtype, "--args_path", args, "--normalize", "--out", tmp_path / "norm.csv", "--no_progress",
                                 name, lp, rp, cwd=tmp_path)
        assert rc == 0, (name, err)
        got = read_matrices(tmp_path / "norm.csv")
        # CSV files keep six decimals
        assert got.shape == exp.shape and close(got, exp, np_dtype, 5.1e-7), (name, np.abs(got - exp).max())
        vp = write_matrices(tmp_path / "valid.csv", exp)
        rc, out, err = run_cross("validate", "--csv", "--normalize", vp, tmp_path / "raw.csv")
        assert rc == 0 and float(out.strip().splitlines()[-1].split(",")[1]) < 1e-4, (name, out, err)  # mean


def test_fft_common_steps_and_input_errors(tmp_path):
    rng = np.random.default_rng(47)
    left = rng.random((2, 32, 32), dtype=np.float32)
    right = rng.random((4, 32, 32), dtype=np.float32)
    lp, rp = write_matrices(tmp_path / "l.csv", left), write_matrices(tmp_path / "r.csv", right)
    rc, out, err = run_cross("run", "--validate", "--no_progress", "-b", "CommonSteps", "-m", "0.001", "-t", tmp_path / "t.csv",
                             "fft_reduced_transfer_n_to_mn", lp, rp, cwd=tmp_path)
    assert rc == 0, err
    assert float(out.strip().splitlines()[1].split(",")[1]) < 1e-4  # mean relative difference
    header = (tmp_path / "t.csv").read_text().splitlines()[0]
    assert header.startswith("Load,Load_iterations,Prepare,") and header.endswith("hadamard_threads_per_block")
    rc, _, err = run_cross("run", "fft_orig_one_to_one", lp, rp, cwd=tmp_path)
    assert rc == 3 and "expected one left matrix" in err
    rc, _, err = run_cross("run", "fft_orig_n_to_mn", rp, lp, cwd=tmp_path)
    assert rc == 3 and "not divisible" in err


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_fft_path_agrees_with_definition_kernels_at_256(dtype):
    """Two independent device paths on the same inputs at a size the CPU oracle needs minutes for: one-to-many
    1 x 8 matrices of 256x256, hipFFT path against the grouped definition-based kernels. Relative to the largest
    result element: 2e-5 in fp32 (both paths round differently), 1e-11 in fp64."""
    xc = load_package()
    fft = fft_module()
    rng = np.random.default_rng(48)
    left = rng.random((1, 256, 256)).astype(dtype)
    right = rng.random((8, 256, 256)).astype(dtype)
    by_definition = xc.run("multimat_right_grouped", left, right, 8, n_left=1, n_right=8).astype(np.float64)
    by_fft = fft.normalize(fft.cross_correlate(left, right, "one_to_many", "original")).astype(np.float64)
    assert by_fft.shape == by_definition.shape == (8, 511, 511)
    bound = (2e-5 if dtype == np.float32 else 1e-11) * np.abs(by_definition).max()
    assert np.abs(by_fft - by_definition).max() <= bound, np.abs(by_fft - by_definition).max() / np.abs(by_definition).max()
