#!/usr/bin/env python3
"""Writes the seeded inputs of a benchmark configuration as the two CSV files the `cross`
binary reads (format of the reference's benchmark/input_generator.py:21-28: numpy.savetxt with
header 'rows,cols,n', i.e. first line '# rows,cols,n', values as %.18e).

  python generate_inputs.py C3 out_dir            -> out_dir/C3_left.csv, out_dir/C3_right.csv
  python generate_inputs.py C3 out_dir --binary   -> out_dir/C3_left.bin, out_dir/C3_right.bin (this build's
                                                     binary matrix format, see matrix_io.py; loads in milliseconds)
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import matrix_io  # noqa: E402
import workloads  # noqa: E402


def main():
    binary = "--binary" in sys.argv
    if binary:
        sys.argv.remove("--binary")
    if len(sys.argv) != 3 or sys.argv[1] not in workloads.CONFIGS:
        print(__doc__)
        print("configurations:", ", ".join(workloads.CONFIGS))
        return 1
    name, out_dir = sys.argv[1], sys.argv[2]
    os.makedirs(out_dir, exist_ok=True)
    left, right = workloads.generate(workloads.CONFIGS[name])
    ext = "bin" if binary else "csv"
    paths = [os.path.join(out_dir, f"{name}_{side}.{ext}") for side in ("left", "right")]
    matrix_io.write(paths[0], left)
    matrix_io.write(paths[1], right)
    print(*paths)
    return 0


if __name__ == "__main__":
    sys.exit(main())
