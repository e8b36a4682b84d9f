"""ctypes mirror of include/xcorr_fft.h: the FFT-based comparison path (hipFFT plans and the
hadamard / scatter kernels of libxcorr_fft.so) on device buffers owned through the main library.

The reference's FFT algorithms (one_to_one.hpp:888-1150, n_to_mn.hpp:720-1000, n_to_m.hpp:647-790)
zero-pad both inputs to twice their size, transform, multiply left spectra with conjugated right
spectra and transform back; `normalize` below is fft_helpers.hpp:193-262 in numpy."""
import ctypes
import os

import numpy as np

from . import PKG_DIR, DeviceBuffer, XcorrError, sync

FFT_LIB_PATH = os.path.join(PKG_DIR, "lib", "libxcorr_fft.so")
FFT_HEADER_PATH = os.path.join(os.path.dirname(PKG_DIR), "include", "xcorr_fft.h")

_lib = None


def lib():
    """The loaded FFT library. Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(FFT_LIB_PATH):
            raise RuntimeError(f"{FFT_LIB_PATH} is missing: build it with `make -C {PKG_DIR}` (hipcc, gfx950)")
        _lib = ctypes.CDLL(FFT_LIB_PATH)
        _lib.xcorr_fft_last_error.restype = ctypes.c_char_p
    return _lib


def _check(code):
    if code != 0:
        raise XcorrError(code, lib().xcorr_fft_last_error().decode())


class Plan:
    def __init__(self, direction, rows, cols, batch, dtype):
        self.ptr = ctypes.c_void_p()
        make = lib().xcorr_fft_plan_forward if direction == "forward" else lib().xcorr_fft_plan_inverse
        self.direction = direction
        _check(make(ctypes.byref(self.ptr), rows, cols, batch, np.dtype(dtype).itemsize))

    def execute(self, src, dst):
        fn = lib().xcorr_fft_exec_forward if self.direction == "forward" else lib().xcorr_fft_exec_inverse
        _check(fn(self.ptr, src.ptr, dst.ptr))

    def destroy(self):
        if self.ptr:
            _check(lib().xcorr_fft_plan_destroy(self.ptr))
            self.ptr = ctypes.c_void_p()


def normalize(raw):
    """fft_helpers.hpp:193-262: quadrant swap around the empty middle row and column of the circular
    result, which are dropped, and division by the number of elements. raw: (n, 2*rows, 2*cols)."""
    raw = np.asarray(raw)
    _, pr, pc = raw.shape
    # output row oy holds the shift oy - (rows - 1), which the circular result keeps at that shift mod 2*rows
    ys = (np.arange(pr - 1) - (pr // 2 - 1)) % pr
    xs = (np.arange(pc - 1) - (pc // 2 - 1)) % pc
    return raw[:, ys][:, :, xs] / (pr * pc)


def cross_correlate(left, right, mode, variant="original", threads=256, items=10):
    """The whole FFT path on the device for (n_left, rows, cols) and (n_right, rows, cols) arrays:
    returns the RAW circular result (n_out, 2*rows, 2*cols) as the `cross` binary stores it without
    --normalize. mode: one_to_one / one_to_many / n_to_mn (variant original or reduced_transfer) or
    n_to_m (variant over_output or over_right)."""
    left, right = np.ascontiguousarray(left), np.ascontiguousarray(right)
    dtype = left.dtype
    sfx = "f32" if dtype == np.float32 else "f64"
    n_left, rows, cols = left.shape
    n_right = right.shape[0]
    pr, pc = 2 * rows, 2 * cols
    fc = pc // 2 + 1
    n_in = n_left + n_right
    n_out = n_left * n_right if mode == "n_to_m" else n_right
    if mode != "n_to_m" and n_right % n_left:
        raise ValueError("right count must be a multiple of the left count")
    both = np.concatenate([left, right])
    if variant == "reduced_transfer":
        d_in = DeviceBuffer.from_numpy(both)
        d_pad = DeviceBuffer(n_in * pr * pc * dtype.itemsize)
        d_pad.zero()
        _check(getattr(lib(), f"xcorr_scatter_{sfx}")(d_in.ptr, d_pad.ptr, cols, rows, n_in, pc, pr, 0, 0, threads, items, None))
    else:
        padded = np.zeros((n_in, pr, pc), dtype)
        padded[:, :rows, :cols] = both
        d_pad = DeviceBuffer.from_numpy(padded)
    d_spec = DeviceBuffer(n_in * pr * fc * 2 * dtype.itemsize)
    d_out = DeviceBuffer(n_out * pr * pc * dtype.itemsize)
    fwd, inv = Plan("forward", pr, pc, n_in, dtype), Plan("inverse", pr, pc, n_out, dtype)
    fwd.execute(d_pad, d_spec)
    spec_bytes = pr * fc * 2 * dtype.itemsize
    d_left = ctypes.c_void_p(d_spec.ptr.value)
    d_right = ctypes.c_void_p(d_spec.ptr.value + n_left * spec_bytes)
    if mode == "n_to_m":
        d_prod = DeviceBuffer(n_out * spec_bytes)
        fn = getattr(lib(), f"xcorr_hadamard_n_to_m_{variant}_{sfx}")
        _check(fn(d_left, d_right, d_prod.ptr, fc, pr, n_left, n_right, threads, items, None))
        src = d_prod
    else:
        fn = getattr(lib(), f"xcorr_hadamard_original_{sfx}")
        _check(fn(d_left, d_right, fc, pr, n_left, n_right // n_left, threads, None))
        src = type("View", (), {"ptr": d_right})()
    inv.execute(src, d_out)
    sync()
    out = d_out.to_numpy((n_out, pr, pc), dtype)
    fwd.destroy()
    inv.destroy()
    return out
