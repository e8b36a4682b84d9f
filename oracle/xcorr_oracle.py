"""numpy front end of the CPU oracle (``libxcorr_oracle.so``).

Test infrastructure only: the library restates the reference's host
cross-correlation (repo/cross-corr/src/validate.hpp) and is the checker the HIP
path is compared against. Nothing that ships may import this module; tests, the
smoke check and the benchmark's CPU-baseline leg do.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libxcorr_oracle.so")


def build(force=False):
    """Compile the oracle with the recipe next to it (gcc, no dependencies)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libxcorr_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


class Validation(ctypes.Structure):
    _fields_ = [
        ("diff_max", ctypes.c_double),
        ("diff_mean", ctypes.c_double),
        ("diff_stddev", ctypes.c_double),
        ("at_max_result", ctypes.c_double),
        ("at_max_valid", ctypes.c_double),
    ]


class Errors(ctypes.Structure):
    _fields_ = [
        ("rel_frobenius", ctypes.c_double),
        ("max_abs", ctypes.c_double),
        ("max_rel", ctypes.c_double),
    ]


class AssignedWork(ctypes.Structure):
    _fields_ = [
        ("output_row", ctypes.c_uint),
        ("worker_idx", ctypes.c_uint),
        ("workers_for_row", ctypes.c_uint),
    ]


ERROR_NAMES = {
    1: "Invalid result matrix size",
    2: "Invalid number of result matrices",
    3: "Invalid ref and target data counts, not divisible",
    4: "Cannot validate matrices of different sizes",
}

DISTRIBUTIONS = {"none": 0, "rectangle": 1, "triangle": 2}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.xo_hadamard_and_sum_f32.restype = ctypes.c_float
        _lib.xo_hadamard_and_sum_f64.restype = ctypes.c_double
        _lib.xo_hadamard_and_sum_f32_acc64.restype = ctypes.c_double
        _lib.xo_interleave_index.restype = ctypes.c_uint
        _lib.xo_dist_num_workers.restype = ctypes.c_uint
        _lib.xo_dist_distribute_rows.restype = AssignedWork
        _lib.xo_dist_distribute_rows.argtypes = [ctypes.c_int] + [ctypes.c_uint] * 4
        _lib.xo_dist_num_workers.argtypes = [ctypes.c_int] + [ctypes.c_uint] * 3
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _suffix(dtype):
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"unsupported dtype {dtype}")


def _as_matrices(a, dtype=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    if a.ndim == 2:
        a = a[None]
    if a.ndim != 3:
        raise ValueError("expected (rows, cols) or (n, rows, cols)")
    return a


def hadamard_and_sum(ref, target, offset_x, offset_y, acc64=False):
    ref = np.ascontiguousarray(ref)
    target = np.ascontiguousarray(target, dtype=ref.dtype)
    rows, cols = ref.shape
    name = "xo_hadamard_and_sum_" + _suffix(ref.dtype) + ("_acc64" if acc64 else "")
    return getattr(lib(), name)(_ptr(ref), _ptr(target), cols, rows, int(offset_x), int(offset_y))


def cross_corr(ref, target, threads=1, row_begin=None, row_end=None, acc64=False, out=None):
    """Full cross-correlation of two equally sized matrices; result (2r-1, 2c-1).

    With row_begin/row_end only that band of output rows is written (the rest of
    ``out`` is left untouched)."""
    ref = np.ascontiguousarray(ref)
    target = np.ascontiguousarray(target, dtype=ref.dtype)
    if ref.shape != target.shape or ref.ndim != 2:
        raise ValueError("ref and target must be 2-D and of equal shape")
    rows, cols = ref.shape
    out_dtype = np.float64 if acc64 else ref.dtype
    if out is None:
        out = np.zeros((2 * rows - 1, 2 * cols - 1), dtype=out_dtype)
    name = "xo_cross_corr_rows_" + _suffix(ref.dtype) + ("_acc64" if acc64 else "")
    rb = 0 if row_begin is None else int(row_begin)
    re = 2 * rows - 1 if row_end is None else int(row_end)
    getattr(lib(), name)(_ptr(ref), _ptr(target), _ptr(out), cols, rows, rb, re, int(threads))
    return out


def _mode(name, ref, target, n_results, threads, with_counts, result_shape=None):
    ref = _as_matrices(ref)
    target = _as_matrices(target, dtype=ref.dtype)
    rows, cols = ref.shape[1:]
    if target.shape[1:] != (rows, cols):
        raise ValueError("ref and target matrices must be of equal size")
    if result_shape is None:
        result_shape = (n_results, 2 * rows - 1, 2 * cols - 1)
    res = np.zeros(result_shape, dtype=ref.dtype)
    fn = getattr(lib(), f"xo_{name}_{_suffix(ref.dtype)}")
    args = [_ptr(ref), _ptr(target), _ptr(res), cols, rows] + with_counts(ref, target)
    args += [result_shape[2], result_shape[1], result_shape[0], int(threads)]
    err = fn(*args)
    if err:
        raise RuntimeError(ERROR_NAMES[err])
    return res


def one_to_one(ref, target, threads=1, result_shape=None):
    return _mode("one_to_one", ref, target, 1, threads, lambda r, t: [], result_shape)


def one_to_many(ref, target, threads=1, result_shape=None):
    t = _as_matrices(target)
    return _mode("one_to_many", ref, t, t.shape[0], threads, lambda r, t: [t.shape[0]], result_shape)


def n_to_mn(ref, target, threads=1, result_shape=None):
    t = _as_matrices(target)
    return _mode("n_to_mn", ref, t, t.shape[0], threads, lambda r, t: [r.shape[0], t.shape[0]], result_shape)


def n_to_m(ref, target, threads=1, result_shape=None):
    r = _as_matrices(ref)
    t = _as_matrices(target)
    return _mode("n_to_m", r, t, r.shape[0] * t.shape[0], threads,
                 lambda r, t: [r.shape[0], t.shape[0]], result_shape)


def validate_result(result, valid):
    result = np.ascontiguousarray(result)
    valid = np.ascontiguousarray(valid, dtype=result.dtype)
    if result.shape != valid.shape:
        raise RuntimeError(ERROR_NAMES[4])
    out = Validation()
    fn = getattr(lib(), "xo_validate_result_" + _suffix(result.dtype))
    fn(_ptr(result), _ptr(valid), ctypes.c_size_t(result.size), ctypes.byref(out))
    return out


def errors(a, b):
    """Relative Frobenius error, max abs and max relative element error of a against b."""
    a = np.ascontiguousarray(a)
    out = Errors()
    if a.dtype == np.float32 and np.asarray(b).dtype == np.float64:
        b = np.ascontiguousarray(b)
        lib().xo_errors_f32_vs_f64(_ptr(a), _ptr(b), ctypes.c_size_t(a.size), ctypes.byref(out))
    else:
        b = np.ascontiguousarray(b, dtype=a.dtype)
        getattr(lib(), "xo_errors_" + _suffix(a.dtype))(_ptr(a), _ptr(b), ctypes.c_size_t(a.size), ctypes.byref(out))
    if a.shape != np.asarray(b).shape:
        raise ValueError("shape mismatch")
    return out


def interleave_index(idx, num_matrices, group_size):
    return lib().xo_interleave_index(int(idx), int(num_matrices), int(group_size))


def dist_num_workers(dist, max_rows_per_worker, matrix_rows, search_rows):
    return lib().xo_dist_num_workers(DISTRIBUTIONS[dist], max_rows_per_worker, matrix_rows, search_rows)


def dist_distribute_rows(dist, worker_y_index, max_rows_per_worker, matrix_rows, search_rows):
    w = lib().xo_dist_distribute_rows(DISTRIBUTIONS[dist], worker_y_index, max_rows_per_worker, matrix_rows, search_rows)
    return w.output_row, w.worker_idx, w.workers_for_row
