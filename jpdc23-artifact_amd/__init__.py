"""Python plumbing around libxcorr_hip.so (ctypes): build helper, struct mirrors of
include/xcorr_hip.h and a thin numpy-in / numpy-out convenience layer used by the
tests and the benchmark. The product is the C ABI library and the `cross` host
binary; nothing here computes a cross-correlation on the CPU, and every call
raises if the library is missing or a launch fails.
"""
import ctypes
import os
import subprocess

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "lib", "libxcorr_hip.so")
CROSS_PATH = os.path.join(PKG_DIR, "bin", "cross")
HEADER_PATH = os.path.join(ROOT, "include", "xcorr_hip.h")

DIST = {"default": 0, "none": 1, "rectangle": 2, "triangle": 3}
DIST_NAMES = {v: k for k, v in DIST.items()}
WPO_VARIANT = {"base": 0, "simple_indexing": 1, "work_distribution": 2}


class XcorrError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"xcorr error {code}: {message}")
        self.code = code
        self.message = message


class Params(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint),
        ("warps_per_thread_block", ctypes.c_uint),
        ("shifts_per_thread_block", ctypes.c_uint),
        ("rows_per_thread", ctypes.c_uint),
        ("distribution_type", ctypes.c_uint),
        ("shifts_per_thread", ctypes.c_uint),
        ("left_rows_per_iteration", ctypes.c_uint),
        ("right_matrices_per_thread", ctypes.c_uint),
        ("left_matrices_per_thread", ctypes.c_uint),
        ("shifts_per_thread_right_matrix", ctypes.c_uint),
        ("warp_per_overlap_variant", ctypes.c_uint),
        ("x_shifts_per_thread", ctypes.c_uint),
        ("lanes_x", ctypes.c_uint),
        ("lanes_y", ctypes.c_uint),
        ("specialisation", ctypes.c_uint),
        ("shared_mem_row_size", ctypes.c_uint),
        ("shared_mem_rows", ctypes.c_uint),
        ("right_matrices_per_block", ctypes.c_uint),
        ("strided_load", ctypes.c_uint),
        ("column_group_per_block", ctypes.c_uint),
        ("block_size", ctypes.c_uint),
        ("column_chunks", ctypes.c_uint),
        ("whole_pair_in_lds", ctypes.c_uint),
        ("matrix_cores", ctypes.c_uint),
    ]


class LaunchRecord(ctypes.Structure):
    _fields_ = [
        ("kernel", ctypes.c_char * 64),
        ("block", ctypes.c_uint * 3),
        ("grid", ctypes.c_uint * 3),
        ("shared_mem_bytes", ctypes.c_uint),
        ("y_shifts_per_thread", ctypes.c_uint),
        ("x_shifts_per_thread", ctypes.c_uint),
        ("left_matrices_per_thread", ctypes.c_uint),
        ("right_matrices_per_thread", ctypes.c_uint),
        ("lanes_x", ctypes.c_uint),
        ("lanes_y", ctypes.c_uint),
        ("lanes_left", ctypes.c_uint),
        ("lanes_right", ctypes.c_uint),
        ("waves_x", ctypes.c_uint),
        ("waves_y", ctypes.c_uint),
        ("rows_per_worker", ctypes.c_uint),
        ("distribution_type", ctypes.c_uint),
        ("uses_atomics", ctypes.c_uint),
        ("blocks_per_cu", ctypes.c_uint),
        ("column_chunks", ctypes.c_uint),
        ("matrix_cores", ctypes.c_uint),
        ("predicted_us", ctypes.c_float),
    ]

    def as_dict(self):
        d = {}
        for name, _ in self._fields_:
            v = getattr(self, name)
            if name == "kernel":
                v = v.decode()
            elif name in ("block", "grid"):
                v = list(v)
            d[name] = v
        return d


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 128),
        ("arch", ctypes.c_char * 32),
        ("compute_units", ctypes.c_int),
        ("clock_khz", ctypes.c_int),
        ("memory_clock_khz", ctypes.c_int),
        ("memory_bus_bits", ctypes.c_int),
        ("lds_bytes_per_block", ctypes.c_int),
        ("global_mem_bytes", ctypes.c_size_t),
        ("fp32_vector_peak_tflops", ctypes.c_double),
        ("fp64_vector_peak_tflops", ctypes.c_double),
    ]


def build(verbose=False):
    """Compile libxcorr_hip.so and the cross binary for gfx950 (make in the package dir)."""
    proc = subprocess.run(["make", "-C", PKG_DIR, "-j8", "all"], capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout[-4000:])
        print(proc.stderr[-4000:])
    if proc.returncode != 0:
        raise RuntimeError("building libxcorr_hip.so failed")
    return LIB_PATH


_lib = None


def lib():
    """The loaded C ABI library. Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C {PKG_DIR}` (hipcc, gfx950)")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.xcorr_last_error.restype = ctypes.c_char_p
        _lib.xcorr_version.restype = ctypes.c_char_p
    return _lib


def _check(code):
    if code != 0:
        raise XcorrError(code, lib().xcorr_last_error().decode())


def last_launch():
    rec = LaunchRecord()
    _check(lib().xcorr_last_launch(ctypes.byref(rec)))
    return rec.as_dict()


def device_info():
    info = DeviceInfo()
    _check(lib().xcorr_device_info_get(ctypes.byref(info)))
    return info


class DeviceBuffer:
    """Device memory owned through the C ABI shims (xcorr_malloc / xcorr_free)."""

    def __init__(self, nbytes):
        self.ptr = ctypes.c_void_p()
        self.nbytes = int(nbytes)
        _check(lib().xcorr_malloc(ctypes.byref(self.ptr), ctypes.c_size_t(max(self.nbytes, 1))))

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        _check(lib().xcorr_memcpy_h2d(buf.ptr, a.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(a.nbytes)))
        return buf

    def to_numpy(self, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _check(lib().xcorr_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), self.ptr, ctypes.c_size_t(out.nbytes)))
        return out

    def zero(self, stream=None):
        _check(lib().xcorr_memset_async(self.ptr, 0, ctypes.c_size_t(self.nbytes), stream))

    def fill_bytes(self, value):
        _check(lib().xcorr_memset_async(self.ptr, int(value), ctypes.c_size_t(self.nbytes), None))

    def free(self):
        if self.ptr:
            lib().xcorr_free(self.ptr)
            self.ptr = ctypes.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sync():
    _check(lib().xcorr_device_sync())


class Event:
    def __init__(self):
        self.ptr = ctypes.c_void_p()
        _check(lib().xcorr_event_create(ctypes.byref(self.ptr)))

    def record(self, stream=None):
        _check(lib().xcorr_event_record(self.ptr, stream))

    def sync(self):
        _check(lib().xcorr_event_sync(self.ptr))

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        _check(lib().xcorr_event_elapsed_ms(self.ptr, stop.ptr, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().xcorr_event_destroy(self.ptr)
        except Exception:
            pass


class Stream:
    """A HIP stream of default priority, owned through the C ABI."""

    def __init__(self):
        self.ptr = ctypes.c_void_p()
        _check(lib().xcorr_stream_create(ctypes.byref(self.ptr)))

    def sync(self):
        _check(lib().xcorr_stream_sync(self.ptr))

    def destroy(self):
        if self.ptr:
            lib().xcorr_stream_destroy(self.ptr)
            self.ptr = ctypes.c_void_p()


class Graph:
    """Launches captured from a stream between begin() and end(), replayed with launch()."""

    def __init__(self, stream):
        self.stream = stream
        self.exec = ctypes.c_void_p()

    def begin(self):
        _check(lib().xcorr_graph_capture_begin(self.stream.ptr))

    def end(self):
        _check(lib().xcorr_graph_capture_end(self.stream.ptr, ctypes.byref(self.exec)))

    def launch(self, stream=None):
        _check(lib().xcorr_graph_launch(self.exec, (stream or self.stream).ptr))

    def destroy(self):
        if self.exec:
            lib().xcorr_graph_destroy(self.exec)
            self.exec = ctypes.c_void_p()


def make_params(**kw):
    p = Params()
    p.struct_size = ctypes.sizeof(Params)
    for k, v in kw.items():
        if k == "distribution_type" and isinstance(v, str):
            v = DIST[v]
        if k == "warp_per_overlap_variant" and isinstance(v, str):
            v = WPO_VARIANT[v]
        if not hasattr(p, k):
            raise KeyError(k)
        setattr(p, k, int(v))
    return p


# family -> (entry point stem, kind of matrix-count arguments, caller must zero the output)
FAMILIES = {
    "overlap_wise": ("xcorr_overlap_wise", "batch", False),
    "overlap_wise_all_pairs": ("xcorr_overlap_wise_all_pairs", "batch", False),
    "warp_per_overlap": ("xcorr_warp_per_overlap", "pair", None),
    "warp_per_overlap_lds": ("xcorr_warp_per_overlap_lds", "right", None),
    "block_per_overlap": ("xcorr_block_per_overlap", "pair", False),
    "shuffle": ("xcorr_shuffle", "pair", False),
    "split_row": ("xcorr_split_row", "pair", True),
    "grouped_overlap": ("xcorr_grouped_overlap", "pair", False),
    "grouped_overlap_ordered": ("xcorr_grouped_overlap_ordered", "pair", False),  # fp32 only
    "multimat_right": ("xcorr_multimat_right", "right", None),
    "multimat_right_groups": ("xcorr_multimat_right_groups", "both", None),
    "multimat_right_grouped": ("xcorr_multimat_right_grouped", "both", False),
    "multimat_both": ("xcorr_multimat_both", "both", True),
    "multimat_both_grouped": ("xcorr_multimat_both_grouped", "both", False),
}


def _suffix(dtype):
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"unsupported dtype {dtype}")


def launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, dtype, params=None, stream=None):
    """Asynchronous launch on raw device buffers. Matrix-count meaning per family:
    overlap_wise: (n_left, batch); pair families: ignored; multimat_right: n_right;
    the others: (n_left, n_right) as documented in include/xcorr_hip.h."""
    stem, kind, _ = FAMILIES[family]
    fn = getattr(lib(), f"{stem}_{_suffix(np.dtype(dtype))}")
    p = ctypes.byref(params) if params is not None else None
    if kind == "batch":
        code = fn(d_left.ptr, d_right.ptr, d_out.ptr, cols, rows, n_left, n_right, stream)
    elif kind == "pair":
        code = fn(d_left.ptr, d_right.ptr, d_out.ptr, cols, rows, p, stream)
    elif kind == "right":
        code = fn(d_left.ptr, d_right.ptr, d_out.ptr, cols, rows, n_right, p, stream)
    else:
        code = fn(d_left.ptr, d_right.ptr, d_out.ptr, cols, rows, n_left, n_right, p, stream)
    _check(code)


def needs_zeroed_output(family, params):
    zero = FAMILIES[family][2]
    if zero is not None:
        return zero
    if family == "warp_per_overlap":
        return params is not None and params.warp_per_overlap_variant == 2
    if family in ("multimat_right", "multimat_right_groups"):
        return params is not None and (params.rows_per_thread > 0 or params.distribution_type in (2, 3))
    if family == "warp_per_overlap_lds":
        return params is not None and params.column_group_per_block != 0
    return False


def run(family, left, right, n_results, n_left=1, n_right=1, params=None, poison=True):
    """numpy in, numpy out: copies the inputs to the device, launches `family`, copies the
    result back. The output buffer is first filled with a NaN byte pattern (or zeroed where
    the family's contract says the caller zeroes it) so unwritten elements show up."""
    left = np.ascontiguousarray(left)
    right = np.ascontiguousarray(right, dtype=left.dtype)
    rows, cols = left.shape[-2:]
    out_shape = (n_results, 2 * rows - 1, 2 * cols - 1)
    d_left = DeviceBuffer.from_numpy(left)
    d_right = DeviceBuffer.from_numpy(right)
    d_out = DeviceBuffer(int(np.prod(out_shape)) * left.dtype.itemsize)
    try:
        if needs_zeroed_output(family, params):
            d_out.zero()
        elif poison:
            d_out.fill_bytes(0xFF)
        launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, left.dtype, params)
        sync()
        return d_out.to_numpy(out_shape, left.dtype)
    finally:
        d_left.free()
        d_right.free()
        d_out.free()
