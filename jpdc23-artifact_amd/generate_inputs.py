#!/usr/bin/env python3
"""Writes the seeded inputs of a benchmark configuration as the two CSV files the `cross`
binary reads (format of the reference's benchmark/input_generator.py:21-28: numpy.savetxt with
header 'rows,cols,n', i.e. first line '# rows,cols,n', values as %.18e).

  python generate_inputs.py C3 out_dir        -> out_dir/C3_left.csv, out_dir/C3_right.csv
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import workloads  # noqa: E402


def write(path, a):
    n, rows, cols = a.shape
    np.savetxt(path, a.reshape(n * rows, cols), delimiter=",", header=f"{rows},{cols},{n}")


def main():
    if len(sys.argv) != 3 or sys.argv[1] not in workloads.CONFIGS:
        print(__doc__)
        print("configurations:", ", ".join(workloads.CONFIGS))
        return 1
    name, out_dir = sys.argv[1], sys.argv[2]
    os.makedirs(out_dir, exist_ok=True)
    left, right = workloads.generate(workloads.CONFIGS[name])
    write(os.path.join(out_dir, f"{name}_left.csv"), left)
    write(os.path.join(out_dir, f"{name}_right.csv"), right)
    print(os.path.join(out_dir, f"{name}_left.csv"), os.path.join(out_dir, f"{name}_right.csv"))
    return 0


if __name__ == "__main__":
    sys.exit(main())
