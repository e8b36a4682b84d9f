"""Run-to-run behaviour of the launches (reference: the grouped-overlap kernels write every output once, no atomics,
naive_shuffle_multirow_both.cu:396-482; validate.hpp:102-111 fixes the summation order of the host loop).
Launches that report uses_atomics = 0 must give the same bits every run; the default launches, which may add partial sums
atomically in any order, must agree with themselves to the last bits (relative Frobenius distance between two runs <= 1e-6)."""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def run_twice(xc, family, left, right, n_results, n_left, n_right, **kw):
    a = xc.run(family, left, right, n_results, n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
    rec = xc.last_launch()
    b = xc.run(family, left, right, n_results, n_left=n_left, n_right=n_right, params=xc.make_params(**kw))
    return a, b, rec


def distance(a, b):
    return float(np.linalg.norm((a.astype(np.float64) - b).ravel()) / np.linalg.norm(a.astype(np.float64).ravel()))


def test_launches_without_atomics_repeat_bit_for_bit():
    xc = load_package()
    rng = np.random.default_rng(77)
    left, right = rng.random((1024, 1024), dtype=np.float32), rng.random((1024, 1024), dtype=np.float32)
    a, b, rec = run_twice(xc, "grouped_overlap", left, right, 1, 1, 1, rows_per_thread=1024, column_chunks=1)
    print("no atomics:", rec["kernel"], rec["uses_atomics"], flush=True)
    assert rec["uses_atomics"] == 0 and np.array_equal(a, b)
    a, b, rec = run_twice(xc, "shuffle", left, right, 1, 1, 1, distribution_type="none")
    print("one pass over the rows:", rec["kernel"], rec["uses_atomics"], flush=True)
    assert rec["uses_atomics"] == 0 and rec["matrix_cores"] == 0 and np.array_equal(a, b)
    # several matrices: one_to_many, n_to_mn in one launch, n_to_m; fp32 and fp64
    for dtype in (np.float32, np.float64):
        l3, r12 = rng.standard_normal((3, 96, 80)).astype(dtype), rng.standard_normal((12, 96, 80)).astype(dtype)
        for family, n_res, nl, nr in [("multimat_right_grouped", 12, 1, 12), ("multimat_right_grouped", 12, 3, 4), ("multimat_both_grouped", 36, 3, 12)]:
            a, b, rec = run_twice(xc, family, l3[:nl] if family != "multimat_both_grouped" else l3, r12, n_res, nl, nr, rows_per_thread=96, column_chunks=1)
            print(family, np.dtype(dtype).name, rec["kernel"], flush=True)
            assert rec["uses_atomics"] == 0 and np.array_equal(a, b), (family, dtype, rec["kernel"])
        a, b, rec = run_twice(xc, "multimat_right", l3[:1], r12, 12, 1, 12, distribution_type="none")
        assert rec["uses_atomics"] == 0 and np.array_equal(a, b), rec["kernel"]


def test_default_launches_agree_with_themselves_to_the_last_bits():
    xc = load_package()
    rng = np.random.default_rng(78)
    left, right = rng.random((1024, 1024), dtype=np.float32), rng.random((1024, 1024), dtype=np.float32)
    a, b, rec = run_twice(xc, "grouped_overlap", left, right, 1, 1, 1)
    d = distance(a, b)
    print("default C2-sized launch:", rec["kernel"], "atomics", rec["uses_atomics"], "distance between two runs %.3e" % d, flush=True)
    assert d <= 1e-6
    l4, r8 = rng.standard_normal((4, 128, 128)), rng.standard_normal((8, 128, 128))
    a, b, rec = run_twice(xc, "multimat_both_grouped", l4, r8, 32, 4, 8)
    d = distance(a, b)
    print("default n_to_m fp64:", rec["kernel"], "atomics", rec["uses_atomics"], "distance %.3e" % d, flush=True)
    assert d <= 1e-12
    a, b, rec = run_twice(xc, "split_row", left[:256, :256], right[:256, :256], 1, 1, 1)
    assert rec["uses_atomics"] == 1 and distance(a, b) <= 1e-6


def test_output_in_pinned_host_memory(oracle):
    """The float atomic add is not defined on host-mapped memory (it is dropped without an error): a launch into such an
    output that names no chunk is replanned with whole reductions and plain stores and gives the right result; one whose
    chunk the caller fixed is refused (XCORR_ERR_UNSUPPORTED) before anything is launched."""
    import ctypes

    xc = load_package()
    lib = xc.lib()
    rng = np.random.default_rng(79)
    rows = cols = 200
    left = rng.integers(-3, 4, (rows, cols)).astype(np.float32)
    right = rng.integers(-3, 4, (rows, cols)).astype(np.float32)
    out_shape = (2 * rows - 1, 2 * cols - 1)
    exp = oracle.one_to_one(left, right).reshape(out_shape)
    nbytes = int(np.prod(out_shape)) * 4
    d_left, d_right = xc.DeviceBuffer.from_numpy(left), xc.DeviceBuffer.from_numpy(right)
    host = ctypes.c_void_p()
    assert lib.xcorr_host_alloc_pinned(ctypes.byref(host), ctypes.c_size_t(nbytes)) == 0
    try:
        view = np.ctypeslib.as_array(ctypes.cast(host, ctypes.POINTER(ctypes.c_float)), shape=out_shape)
        for family, fn in (("grouped_overlap", lib.xcorr_grouped_overlap_f32), ("split_row", lib.xcorr_split_row_f32)):
            # on device memory this launch splits and adds atomically ...
            lib.xcorr_plan_only(1)
            p = xc.make_params()
            assert fn(d_left.ptr, d_right.ptr, d_left.ptr, cols, rows, ctypes.byref(p), None) == 0
            planned = xc.last_launch()
            lib.xcorr_plan_only(0)
            assert planned["uses_atomics"] == 1, planned
            # ... into pinned host memory it does not
            view[:] = np.nan
            code = fn(d_left.ptr, d_right.ptr, host, cols, rows, ctypes.byref(p), None)
            assert code == 0, lib.xcorr_last_error()
            xc.sync()
            rec = xc.last_launch()
            print(family, "into pinned host memory:", rec["kernel"], "atomics", rec["uses_atomics"], flush=True)
            assert rec["uses_atomics"] == 0 and rec["rows_per_worker"] == rows
            assert np.array_equal(view, exp), family
            p = xc.make_params(rows_per_thread=32)
            assert fn(d_left.ptr, d_right.ptr, host, cols, rows, ctypes.byref(p), None) == 3
            assert b"atomics" in lib.xcorr_last_error()
    finally:
        xc.sync()
        lib.xcorr_host_free(host)
        d_left.free()
        d_right.free()
