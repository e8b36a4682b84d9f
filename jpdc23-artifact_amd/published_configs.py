#!/usr/bin/env python3
"""Runs the `cross` binary on the configurations for which the reference publishes kernel times
(results/ampere/*/*.csv of the artifact, A100 PCIe 80 GB; column `Kernel` of `-b Algorithm` runs) with the
same algorithm names and the reference's default arguments, and prints a table with both times.

  python published_configs.py [--min-time SECONDS] [--out table.md] [--skip-large]

Inputs are seeded uniform [0, 1) fp32 matrices in this build's binary matrix format. The A100 figures
are the best of the reference's argument sweeps; here nothing is swept (one row names its arguments).
"""
import argparse
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import matrix_io  # noqa: E402

CROSS = os.path.join(HERE, "bin", "cross")

# (label, algorithm, n_left, n_right, size, A100 time in microseconds, source file under results/ampere/[, JSON arguments])
CONFIGS = [
    ("1-1 64x64 overlap-wise", "nai_orig_one_to_one", 1, 1, 64, 120.1, "one_to_one/original.csv"),
    ("1-1 64x64 split-row", "nai_shuffle_work_distribution_one_to_one", 1, 1, 64, 19.4, "one_to_one/work_distribution.csv"),
    ("1-1 64x64 split-row, rows_per_thread 5, triangle", "nai_shuffle_work_distribution_one_to_one", 1, 1, 64, 19.4, "one_to_one/work_distribution.csv",
     {"rows_per_thread": 5, "distribution_type": "triangle"}),
    ("1-1 64x64 warp-per-overlap", "nai_warp_per_shift_one_to_one", 1, 1, 64, 19.8, "one_to_one/warp-per-shift.csv"),
    ("1-1 64x64 warp-per-overlap, shared memory", "nai_warp_per_shift_shared_mem_one_to_one", 1, 1, 64, 18.2, "one_to_one/warp-per-shift-shared-memory.csv"),
    ("1-1 64x64 grouped-overlap", "nai_shuffle_multirow_both_one_to_one", 1, 1, 64, 52.9, "one_to_one/multirow_both.csv"),
    ("1-1 128x128 split-row", "nai_shuffle_work_distribution_one_to_one", 1, 1, 128, 199.4, "one_to_one/work_distribution.csv"),
    ("1-1 128x128 grouped-overlap", "nai_shuffle_multirow_both_one_to_one", 1, 1, 128, 205.3, "one_to_one/multirow_both.csv"),
    ("1-1 256x256 overlap-wise", "nai_orig_one_to_one", 1, 1, 256, 3239.0, "one_to_one/original.csv"),
    ("1-1 256x256 split-row", "nai_shuffle_work_distribution_one_to_one", 1, 1, 256, 2718.0, "one_to_one/work_distribution.csv"),
    ("1-1 256x256 grouped-overlap", "nai_shuffle_multirow_both_one_to_one", 1, 1, 256, 1053.5, "one_to_one/multirow_both.csv"),
    ("1-many 1x32 256x256 overlap-wise", "nai_orig_one_to_many", 1, 32, 256, 119600.0, "one_to_many/original.csv"),
    ("1-many 1x32 256x256 multimat-right", "nai_shuffle_multimat_right_one_to_many", 1, 32, 256, 38100.0, "one_to_many/multimat-right.csv"),
    ("1-many 1x32 256x256 multimat-right x grouped-overlap", "nai_shuffle_multirow_both_multimat_right_one_to_many", 1, 32, 256, 19410.0,
     "one_to_many/multimat-right-multirow-both.csv"),
    ("1-many 1x4000 256x256 (saturated) multimat-right x grouped-overlap", "nai_shuffle_multirow_both_multimat_right_one_to_many", 1, 4000, 256,
     2383000.0, "one_to_many_saturated/multimat-right-multirow-both.csv"),
    ("n-mn 8x32 128x128 overlap-wise", "nai_orig_n_to_mn", 8, 32, 128, 5803.0, "n_to_mn/original.csv"),
    ("n-mn 8x32 128x128 multimat-right x grouped-overlap", "nai_shuffle_multirow_both_multimat_right_n_to_mn", 8, 32, 128, 3020.0,
     "n_to_mn/multimat-right-multirow-both.csv"),
    ("n-mn 8x32 256x256 multimat-right x grouped-overlap", "nai_shuffle_multirow_both_multimat_right_n_to_mn", 8, 32, 256, 30780.0,
     "n_to_mn/multimat-right-multirow-both.csv"),
    ("n-m 32x32 64x64 overlap-wise", "nai_orig_n_to_m", 32, 32, 64, 17260.0, "n_to_m/original.csv"),
    ("n-m 32x32 64x64 multimat-both (split-row)", "nai_shuffle_multimat_both_work_distribution_n_to_m", 32, 32, 64, 4877.0, "n_to_m/multimat-both.csv"),
    ("n-m 32x32 64x64 multimat-both x grouped-overlap", "nai_shuffle_multirow_both_multimat_both_n_to_m", 32, 32, 64, 2565.0,
     "n_to_m/multimat-both-multirow-both.csv"),
    ("n-m 128x128 64x64 (saturated) multimat-both x grouped-overlap", "nai_shuffle_multirow_both_multimat_both_n_to_m", 128, 128, 64, 41800.0,
     "n_to_m_saturated/multimat-both-multirow-both.csv"),
    ("n-m 128x128 128x128 (saturated) multimat-both x grouped-overlap", "nai_shuffle_multirow_both_multimat_both_n_to_m", 128, 128, 128, 462900.0,
     "n_to_m_saturated/multimat-both-multirow-both.csv"),
]
LARGE = 1000  # result matrices above which a configuration counts as large (--skip-large)


def kernel_seconds(alg, min_time, left, right, workdir, json_args=None):
    times = os.path.join(workdir, "t.csv")
    extra = []
    if json_args:
        import json

        with open(os.path.join(workdir, "args.json"), "w") as fh:
            json.dump(json_args, fh)
        extra = ["--args_path", os.path.join(workdir, "args.json")]
    proc = subprocess.run([CROSS, "run", "-d", "single", "-b", "Algorithm", "-m", str(min_time), "-t", times, "--no_progress", *extra, alg, left, right],
                          capture_output=True, text=True, cwd=workdir)
    if proc.returncode != 0:
        raise RuntimeError(f"{alg}: {proc.stderr.strip()}")
    header, row = open(times).read().strip().splitlines()[:2]
    return int(dict(zip(header.split(","), row.split(",")))["Kernel"]) * 1e-9


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--min-time", type=float, default=0.05)
    ap.add_argument("--out", default=None)
    ap.add_argument("--skip-large", action="store_true")
    a = ap.parse_args()
    lines = ["| configuration | algorithm | A100 (reference, best of its sweep) | MI355X (this build, default arguments) | TFLOP/s here | speed-up |",
             "|---|---|---|---|---|---|"]
    rng = np.random.default_rng(2023)
    cache = {}
    with tempfile.TemporaryDirectory() as tmp:
        for label, alg, n_left, n_right, size, a100_us, src, *json_args in CONFIGS:
            n_out = n_left * n_right if alg.endswith("n_to_m") else n_right
            if a.skip_large and n_out > LARGE:
                continue
            key = (n_left, n_right, size)
            if key not in cache:
                paths = (os.path.join(tmp, f"l_{n_left}_{size}.bin"), os.path.join(tmp, f"r_{n_right}_{size}.bin"))
                matrix_io.write(paths[0], rng.random((n_left, size, size), dtype=np.float32))
                matrix_io.write(paths[1], rng.random((n_right, size, size), dtype=np.float32))
                cache[key] = paths
            t = kernel_seconds(alg, a.min_time, *cache[key], tmp, json_args[0] if json_args else None)
            tflops = 2.0 * n_out * float(size) ** 4 / t / 1e12
            us = t * 1e6
            line = (f"| {label} | `{alg}` | {a100_us:,.1f} us (`{src}`) | {us:,.1f} us | {tflops:.1f} | {a100_us / us:.1f}x |")
            print(line, flush=True)
            lines.append(line)
    if a.out:
        with open(a.out, "w") as fh:
            fh.write("\n".join(lines) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
