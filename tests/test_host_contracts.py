"""Small contracts of the host program that the end-to-end CLI tests only touch in passing (CPU only):
the adaptive repetition rule of the timing harness, and the exact command line the reference's benchmark
driver issues."""
import math
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT
from cross_cli import cross_path, read_matrices, run_cross, write_args, write_matrices


@pytest.fixture(scope="module")
def next_count(tmp_path_factory):
    """get_next_iteration_count of host/stopwatch.hpp, through a tiny program compiled from the header."""
    exe = tmp_path_factory.mktemp("sw") / "stopwatch_check"
    host = os.path.join(ROOT, "jpdc23-artifact_amd", "host")
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", host, "-o", str(exe), os.path.join(ROOT, "tests", "host_stopwatch_check.cpp")],
                   check=True, capture_output=True)

    def call(*triples):
        args = [str(v) for t in triples for v in t]
        out = subprocess.run([str(exe), *args], check=True, capture_output=True, text=True).stdout.split()
        return [int(x) for x in out]

    return call


def test_next_iteration_count_rule(next_count):
    """Reference stopwatch.hpp:57-71: no further round once the measured total has reached min_time;
    otherwise iterations * clamp(1.5 * min_time / total, 1.5, 100), rounded up. Hand-computed cases."""
    ms = 1_000_000
    cases = [
        # (min_time, total, iterations) -> next
        ((10 * ms, 10 * ms, 1), 0),        # total == min_time: done
        ((10 * ms, 25 * ms, 7), 0),        # total > min_time: done
        ((10 * ms, 5 * ms, 1), 3),         # ratio 2 * 1.5 = 3
        ((10 * ms, 5 * ms, 4), 12),        # scales with the iterations already done
        ((10 * ms, 9 * ms, 10), 17),       # 1.5 * 10 / 9 = 1.667 -> ceil(16.67)
        ((10 * ms, 9_999_999, 2), 4),      # just short: factor 1.5000002 -> ceil(3.0000003) = 4
        ((10 * ms, 8 * ms, 3), 6),         # 1.875 -> ceil(5.625)
        ((10 * ms, 100_000, 1), 100),      # ratio 100 * 1.5 clamped to 100
        ((10 * ms, 1, 1), 100),            # tiny total: still 100, not more
        ((10 * ms, 100_000, 3), 300),
        ((1000 * ms, 20 * ms, 5), 375),    # 50 * 1.5 = 75
        ((10 * ms, 7_500_000, 2), 4),      # 1.5 * 4/3 = 2.0 exactly
        ((0, 5, 3), 0),                    # min_time 0: one round is enough
    ]
    got = next_count(*[c[0] for c in cases])
    assert got == [c[1] for c in cases]
    # the rule, once more in its own words, on a sweep (guards the clamp boundaries)
    triples = [(10 * ms, t, n) for t in (1, 1000, 99_999, 150_000, 150_001, 3 * ms, 9_999_999) for n in (1, 2, 13)]
    expect = [math.ceil(n * max(min(10 * ms / t * 1.5, 100.0), 1.5)) for (_, t, n) in triples]
    assert next_count(*triples) == expect


@pytest.mark.parametrize("bench", ["Algorithm", "Compute"])
@pytest.mark.parametrize("with_out,with_validate,append", [(False, False, False), (True, False, False), (True, True, False), (True, True, True)])
def test_reference_driver_command_line(tmp_path, oracle, with_out, with_validate, append, bench):
    """The literal argv of the reference's benchmark driver (benchmark/external/executable.py:117-145):
    run [--out P] [--validate P] [--append] --times P --no_progress --args_path P --data_type single
    --benchmark_type Algorithm --outer_loops N --min_time S <alg> <left> <right>, against cpu_one_to_one (whose
    Algorithm-level measurement has no labels, like the reference's: the file then holds one empty line per
    header and row; with Compute it has the one label Computation)."""
    rng = np.random.default_rng(3)
    left, right = rng.random((6, 9)), rng.random((6, 9))
    lp, rp = write_matrices(tmp_path / "left.csv", left), write_matrices(tmp_path / "right.csv", right)
    expected = oracle.one_to_one(left.astype(np.float32), right.astype(np.float32))
    valid = write_matrices(tmp_path / "valid.csv", expected)
    times, out = tmp_path / "times.csv", tmp_path / "out.csv"
    args_path = write_args(tmp_path / "args.json", warps_per_thread_block=4)
    # adaptive measurements report <label>,<label>_iterations (measurement.hpp of the reference)
    header = "Computation,Computation_iterations" if bench == "Compute" else ""
    if append:
        times.write_text(header + "\n" + ("6,1" if header else "") + "\n")
    optional = (["--out", out] if with_out else []) + (["--validate", valid] if with_validate else []) + (["--append"] if append else [])
    default = ["--times", times, "--no_progress", "--args_path", args_path, "--data_type", "single", "--benchmark_type", bench,
               "--outer_loops", 2, "--min_time", 0.001]
    code, stdout, stderr = run_cross("run", *optional, *default, "cpu_one_to_one", lp, rp)
    assert code == 0, stderr
    text = times.read_text()
    assert text.endswith("\n")
    lines = text[:-1].split("\n")
    # header + one row per outer loop; with --append the old header and row are kept and no second header is written
    assert len(lines) == (4 if append else 3), text
    assert lines[0] == header
    if append:
        assert lines[1] == ("6,1" if header else "")
    for row in lines[-2:]:
        if header:
            nanoseconds, iterations = (int(x) for x in row.split(","))
            assert nanoseconds > 0 and iterations >= 1
        else:
            assert row == ""
    if with_out:
        # outer_loops > 1: one result file per loop (out_0.csv, out_1.csv next to the given name)
        outs = sorted(p for p in tmp_path.iterdir() if p.name.startswith("out"))
        assert len(outs) == 2, [p.name for p in outs]
        for p in outs:
            np.testing.assert_allclose(read_matrices(p), expected, rtol=0, atol=1e-5)
    if with_validate:
        rows = [l for l in stdout.splitlines() if l.strip() and (l[0].isdigit() or l[0] == "-" or l.lower().startswith("max"))]
        assert rows, stdout
    else:
        assert "Difference" not in stdout
