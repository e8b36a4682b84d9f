"""Helpers shared by the CLI tests: write matrices in the reference's CSV input format
(benchmark/input_generator.py:21-28: numpy.savetxt, delimiter ',', header 'rows,cols,n'
which numpy prefixes with '# ') and run the `cross` binary."""
import json
import os
import subprocess

import numpy as np

from conftest import load_package


def cross_path():
    return load_package().CROSS_PATH


def write_matrices(path, a):
    a = np.asarray(a)
    if a.ndim == 2:
        a = a[None]
    n, rows, cols = a.shape
    np.savetxt(path, a.reshape(n * rows, cols), delimiter=",", header=f"{rows},{cols},{n}")
    return path


def read_matrices(path):
    with open(path) as f:
        header = f.readline()
    assert header.startswith("# ")
    rows, cols, n = (int(x) for x in header[2:].split(","))
    data = np.loadtxt(path, delimiter=",", ndmin=2)
    return data.reshape(n, rows, cols)


def run_cross(*args, cwd=None, timeout=300):
    proc = subprocess.run([cross_path(), *[str(a) for a in args]], capture_output=True, text=True, cwd=cwd, timeout=timeout)
    return proc.returncode, proc.stdout, proc.stderr


def write_args(path, **kw):
    with open(path, "w") as f:
        json.dump(kw, f)
    return path
