#!/usr/bin/env python3
"""Writes seeded inputs as the two matrix files the `cross` binary reads (format of the reference's
benchmark/input_generator.py:21-28: numpy.savetxt with header 'rows,cols,n', i.e. first line '# rows,cols,n',
values as %.18e).

  python generate_inputs.py C3 out_dir            -> out_dir/C3_left.csv, out_dir/C3_right.csv (a benchmark configuration)
  python generate_inputs.py C3 out_dir --binary   -> out_dir/C3_left.bin, out_dir/C3_right.bin (this build's binary
                                                     matrix format, see matrix_io.py; loads in milliseconds)
  python generate_inputs.py --shape N_LEFT N_RIGHT ROWS COLS [--dtype single|double] [--seed S] [--binary] NAME out_dir
                                                  -> out_dir/NAME_left.*, out_dir/NAME_right.*: uniform [0, 1) values like the
                                                     reference's generator (benchmark/input_generator.py:31-33), seeded
"""
import argparse
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import matrix_io  # noqa: E402
import workloads  # noqa: E402


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("name", help="a benchmark configuration (" + ", ".join(workloads.CONFIGS) + ") or, with --shape, the stem of the file names")
    ap.add_argument("out_dir")
    ap.add_argument("--binary", action="store_true")
    ap.add_argument("--shape", nargs=4, type=int, metavar=("N_LEFT", "N_RIGHT", "ROWS", "COLS"))
    ap.add_argument("--dtype", choices=["single", "double"], default="single")
    ap.add_argument("--seed", type=int, default=2023)
    a = ap.parse_args()
    if a.shape:
        n_left, n_right, rows, cols = a.shape
        rng = np.random.default_rng(a.seed)
        dtype = np.float32 if a.dtype == "single" else np.float64
        left = rng.random((n_left, rows, cols)).astype(dtype)
        right = rng.random((n_right, rows, cols)).astype(dtype)
    elif a.name in workloads.CONFIGS:
        left, right = workloads.generate(workloads.CONFIGS[a.name])
    else:
        ap.error("unknown configuration " + a.name + " (give --shape for other inputs)")
    os.makedirs(a.out_dir, exist_ok=True)
    ext = "bin" if a.binary else "csv"
    paths = [os.path.join(a.out_dir, f"{a.name}_{side}.{ext}") for side in ("left", "right")]
    matrix_io.write(paths[0], left)
    matrix_io.write(paths[1], right)
    print(*paths)
    return 0


if __name__ == "__main__":
    sys.exit(main())
