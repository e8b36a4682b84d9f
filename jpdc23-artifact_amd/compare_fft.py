#!/usr/bin/env python3
"""Definition-based kernels against the FFT path on the same inputs: the comparison behind the
reference's definition-vs-FFT plots (benchmark.yml groups one_to_one, one_to_many, n_to_mn, n_to_m with
their fft_* runs), through the `cross` binary.

  python compare_fft.py [--dtype single|double] [--min-time SECONDS] [--out table.md]

For every shape both algorithms run with `-b Algorithm`, i.e. with their own measurement labels:
the definition-based time is the `Kernel` label, the FFT time is Forward FFT + Hadamard + Inverse FFT
(plans and allocations excluded, as in the reference's fft.csv files). Inputs are seeded uniform
[0, 1) matrices in this build's binary matrix format.
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

# mode -> (definition-based algorithm, FFT algorithm, (n_left, n_right), sizes)
SWEEPS = {
    "one_to_one": ("nai_shuffle_multirow_both_one_to_one", "fft_orig_one_to_one", (1, 1), [16, 32, 64, 128, 256, 512, 1024]),
    "one_to_many": ("nai_shuffle_multirow_both_multimat_right_one_to_many", "fft_orig_one_to_many", (1, 32), [16, 32, 64, 128, 256]),
    "n_to_mn": ("nai_shuffle_multirow_both_multimat_right_n_to_mn", "fft_orig_n_to_mn", (8, 32), [16, 32, 64, 128, 256]),
    "n_to_m": ("nai_shuffle_multirow_both_multimat_both_n_to_m", "fft_better_n_to_m", (32, 32), [16, 32, 64, 128]),
}


def run(alg, dtype, min_time, left, right, workdir):
    times = os.path.join(workdir, "t.csv")
    proc = subprocess.run([CROSS, "run", "-d", dtype, "-b", "Algorithm", "-m", str(min_time), "-t", times, "--no_progress", alg, left, right],
                          capture_output=True, text=True, cwd=workdir)
    if proc.returncode != 0:
        raise RuntimeError(f"{alg}: {proc.stderr.strip()}")
    header, row = open(times).read().strip().splitlines()[:2]
    values = dict(zip(header.split(","), row.split(",")))
    return {k: int(v) * 1e-9 for k, v in values.items() if k in ("Kernel", "Forward FFT", "Hadamard", "Inverse FFT")}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--dtype", default="single", choices=["single", "double"])
    ap.add_argument("--min-time", type=float, default=0.05, help="minimum measured time per label in seconds (adaptive repetition)")
    ap.add_argument("--out", default=None)
    ap.add_argument("--modes", default=",".join(SWEEPS))
    a = ap.parse_args()
    np_dtype = np.float32 if a.dtype == "single" else np.float64
    lines = [f"| mode | matrices | size | definition-based kernel | FFT (forward + hadamard + inverse) | forward / hadamard / inverse | FFT faster by |",
             "|---|---|---|---|---|---|---|"]
    rng = np.random.default_rng(2023)
    with tempfile.TemporaryDirectory() as tmp:
        for mode in a.modes.split(","):
            definition, fft, (n_left, n_right), sizes = SWEEPS[mode]
            for size in sizes:
                left = os.path.join(tmp, "left.bin")
                right = os.path.join(tmp, "right.bin")
                matrix_io.write(left, rng.random((n_left, size, size)).astype(np_dtype))
                matrix_io.write(right, rng.random((n_right, size, size)).astype(np_dtype))
                d = run(definition, a.dtype, a.min_time, left, right, tmp)["Kernel"]
                f = run(fft, a.dtype, a.min_time, left, right, tmp)
                total = f["Forward FFT"] + f["Hadamard"] + f["Inverse FFT"]
                line = (f"| {mode} | {n_left} x {n_right} | {size} x {size} | {d * 1e6:.1f} us | {total * 1e6:.1f} us | "
                        f"{f['Forward FFT'] * 1e6:.1f} / {f['Hadamard'] * 1e6:.1f} / {f['Inverse FFT'] * 1e6:.1f} us | {d / total:.2f}x |")
                print(line, flush=True)
                lines.append(line)
    if a.out:
        with open(a.out, "w") as fh:
            fh.write("\n".join(lines) + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
