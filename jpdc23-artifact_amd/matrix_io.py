"""Matrix files of the `cross` binary, read and written from Python.

Text: the reference's CSV format (matrix.hpp:94-185; what benchmark/input_generator.py:21-28
writes with numpy.savetxt): first line '# rows,cols,n', then rows*n lines of cols values.
Binary (this build only; the reference has a commented-out stub, matrix.hpp:49-91): 32-byte
little-endian header b'XCORRMAT', version 1, bytes per element (4 or 8), rows, cols, n, 0,
followed by the n matrices row-major. `cross` recognises it by the magic when reading and writes
it for output paths ending in '.bin'.
"""
import struct

import numpy as np

MAGIC = b"XCORRMAT"


def _as3d(a):
    a = np.asarray(a)
    return a[None] if a.ndim == 2 else a


def write_csv(path, a):
    a = _as3d(a)
    n, rows, cols = a.shape
    np.savetxt(path, a.reshape(n * rows, cols), delimiter=",", header=f"{rows},{cols},{n}")
    return path


def read_csv(path):
    with open(path) as f:
        header = f.readline()
    if not header.startswith("# "):
        raise ValueError("Invalid file header format")
    parts = [int(x) for x in header[2:].split(",")]
    rows, cols = parts[0], parts[1]
    n = parts[2] if len(parts) > 2 else 1
    return np.loadtxt(path, delimiter=",", ndmin=2).reshape(n, rows, cols)


def write_binary(path, a):
    a = _as3d(a)
    if a.dtype not in (np.float32, np.float64):
        a = a.astype(np.float64)
    n, rows, cols = a.shape
    with open(path, "wb") as f:
        f.write(MAGIC + struct.pack("<6I", 1, a.dtype.itemsize, rows, cols, n, 0))
        f.write(np.ascontiguousarray(a).astype(a.dtype.newbyteorder("<"), copy=False).tobytes())
    return path


def read_binary(path):
    with open(path, "rb") as f:
        head = f.read(32)
        if len(head) != 32 or head[:8] != MAGIC:
            raise ValueError("Invalid binary matrix file header")
        version, elem, rows, cols, n, _ = struct.unpack("<6I", head[8:])
        if version != 1 or elem not in (4, 8):
            raise ValueError("Unsupported binary matrix file version or element size")
        data = np.frombuffer(f.read(), dtype="<f4" if elem == 4 else "<f8", count=n * rows * cols)
    return data.reshape(n, rows, cols)


def write(path, a):
    return write_binary(path, a) if str(path).endswith(".bin") else write_csv(path, a)


def read(path):
    with open(path, "rb") as f:
        binary = f.read(8) == MAGIC
    return read_binary(path) if binary else read_csv(path)
