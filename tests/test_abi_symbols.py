"""CPU-only: the C ABI library loads without a GPU and exports every symbol that
include/xcorr_hip.h declares; argument validation that needs no device works."""
import ctypes
import os
import re

import numpy as np
import pytest

from conftest import load_package


def declared_symbols():
    xc = load_package()
    text = open(xc.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xcorr_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for family in ["overlap_wise", "overlap_wise_all_pairs", "warp_per_overlap", "warp_per_overlap_lds", "block_per_overlap", "shuffle", "split_row", "grouped_overlap", "multimat_right",
                   "multimat_right_groups", "multimat_right_grouped", "multimat_both", "multimat_both_grouped"]:
        assert f"xcorr_{family}_f32" in names and f"xcorr_{family}_f64" in names
    assert len(names) >= 40


def test_library_exports_every_declared_symbol():
    xc = load_package()
    if not os.path.exists(xc.LIB_PATH):
        pytest.fail(f"{xc.LIB_PATH} not built")
    lib = xc.lib()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_python_struct_mirrors_match_header_field_order():
    xc = load_package()
    text = open(xc.HEADER_PATH).read()
    body = re.search(r"typedef struct xcorr_params \{(.*?)\} xcorr_params;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"unsigned\s+([a-z_]+)(?:\[\d+\])?;", body)
    assert fields == [f[0] for f in xc.Params._fields_]


def test_argument_errors_without_a_device():
    xc = load_package()
    lib = xc.lib()
    p = xc.make_params(shifts_per_thread=9)
    dummy = ctypes.c_void_p(16)
    rc = lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 8, 8, ctypes.byref(p), None)
    assert rc == 1
    assert b"Too many shifts per thread: 9 (max 8)" in lib.xcorr_last_error()
    p = xc.make_params(warps_per_thread_block=33)
    assert lib.xcorr_shuffle_f32(dummy, dummy, dummy, 8, 8, ctypes.byref(p), None) == 1
    assert b"Too many warps per thread block: 33 (max 32)" in lib.xcorr_last_error()
    assert lib.xcorr_grouped_overlap_f32(None, dummy, dummy, 8, 8, None, None) == 1
    assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 0, 8, None, None) == 1
    p = xc.make_params(distribution_type=7)
    assert lib.xcorr_split_row_f64(dummy, dummy, dummy, 8, 8, ctypes.byref(p), None) == 1
    assert b"Unknown distribution" in lib.xcorr_last_error()
    p = xc.make_params(right_matrices_per_thread=5)
    assert lib.xcorr_multimat_both_grouped_f32(dummy, dummy, dummy, 8, 8, 2, 2, ctypes.byref(p), None) == 1
    p = xc.make_params(shifts_per_thread_block=33)
    assert lib.xcorr_warp_per_overlap_lds_f32(dummy, dummy, dummy, 8, 8, 1, ctypes.byref(p), None) == 1
    assert b"Too many shifts per block: 33 (max 32)" in lib.xcorr_last_error()
    p = xc.make_params(right_matrices_per_block=9)
    assert lib.xcorr_warp_per_overlap_lds_f32(dummy, dummy, dummy, 8, 8, 1, ctypes.byref(p), None) == 1
    assert b"Invalid number of right matrices per block: 9 [1-8]" in lib.xcorr_last_error()
    p = xc.make_params(shifts_per_thread_block=8, shared_mem_rows=4)
    assert lib.xcorr_warp_per_overlap_lds_f64(dummy, dummy, dummy, 8, 8, 1, ctypes.byref(p), None) == 1
    assert b"Invalid number of shared memory rows [4]" in lib.xcorr_last_error()
    p = xc.make_params(block_size=2048)
    assert lib.xcorr_block_per_overlap_f32(dummy, dummy, dummy, 8, 8, ctypes.byref(p), None) == 1
    assert b"Thread block too large: 2048 (max 1024)" in lib.xcorr_last_error()
    assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 16385, 8, None, None) == 1
    assert b"matrix too large: 8 x 16385 (max 16384)" in lib.xcorr_last_error()
    # matrix counts whose product leaves the 31-bit range of the work-item arithmetic
    assert lib.xcorr_multimat_both_grouped_f32(dummy, dummy, dummy, 8, 8, 1 << 16, 1 << 16, None, None) == 1
    assert b"too many matrices: 65536 left, 65536 right" in lib.xcorr_last_error()
    assert lib.xcorr_multimat_right_grouped_f64(dummy, dummy, dummy, 8, 8, 3, 0xC0000000, None, None) == 1
    assert b"too many matrices" in lib.xcorr_last_error()
    assert lib.xcorr_multimat_right_f32(dummy, dummy, dummy, 8, 8, 0, None, None) == 1
    assert b"no matrices" in lib.xcorr_last_error()
    assert lib.xcorr_overlap_wise_f32(dummy, dummy, dummy, 8, 8, 1, 0x80000000, None) == 1
    assert b"too many matrices" in lib.xcorr_last_error()
    rec = xc.LaunchRecord()
    assert lib.xcorr_last_launch(ctypes.byref(rec)) == 1
    assert b"No kernel launch" in lib.xcorr_last_error()


def fft_module():
    import importlib
    return importlib.import_module(load_package().__name__ + ".fft")


def test_fft_library_exports_every_declared_symbol():
    fft = fft_module()
    text = re.sub(r"/\*.*?\*/", "", open(fft.FFT_HEADER_PATH).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(xcorr_[a-z0-9_]+)\s*\(", text)))
    assert len(names) == 15 and "xcorr_fft_plan_forward" in names and "xcorr_scatter_f64" in names
    if not os.path.exists(fft.FFT_LIB_PATH):
        pytest.fail(f"{fft.FFT_LIB_PATH} not built")
    for name in names:
        assert hasattr(fft.lib(), name), name


def test_fft_argument_errors_without_a_device():
    fft = fft_module()
    lib = fft.lib()
    plan = ctypes.c_void_p()
    assert lib.xcorr_fft_plan_forward(ctypes.byref(plan), 8, 8, 1, 2) == 1
    assert b"elem" in lib.xcorr_fft_last_error()
    assert lib.xcorr_fft_plan_forward(None, 8, 8, 1, 4) == 1
    assert lib.xcorr_fft_plan_inverse(ctypes.byref(plan), 0, 8, 1, 4) == 1
    dummy = ctypes.c_void_p(16)
    assert lib.xcorr_hadamard_original_f32(dummy, dummy, 5, 8, 1, 1, 0, None) == 1
    assert lib.xcorr_hadamard_n_to_m_over_output_f64(dummy, None, dummy, 5, 8, 1, 1, 256, 10, None) == 1
    assert lib.xcorr_scatter_f32(dummy, dummy, 8, 8, 1, 4, 16, 0, 0, 256, 10, None) == 1  # does not fit
    assert lib.xcorr_fft_exec_forward(None, dummy, dummy) == 1


def test_fft_normalize_matches_the_definition():
    """numpy mirror of fft_helpers.hpp:193-262 against scipy's full correlation."""
    from scipy.signal import correlate2d
    fft = fft_module()
    rng = np.random.default_rng(5)
    for rows, cols in [(1, 1), (4, 4), (3, 5), (6, 2), (1, 7)]:
        a, b = rng.random((rows, cols)), rng.random((rows, cols))
        s = (2 * rows, 2 * cols)
        raw = np.fft.irfft2(np.fft.rfft2(a, s=s) * np.conj(np.fft.rfft2(b, s=s)), s=s) * (4 * rows * cols)
        assert np.allclose(fft.normalize(raw[None])[0], correlate2d(a, b, mode="full"), atol=1e-12)


def test_params_struct_size_rules():
    """xcorr_params.struct_size: 0 (a struct laid out before the field existed) is refused; a smaller size than this build's
    (a caller built against an older header) is read that far and the rest taken as 0, whatever lies behind it."""
    xc = load_package()
    lib = xc.lib()
    assert b"0.2" in lib.xcorr_version()
    dummy = ctypes.c_void_p(16)
    assert lib.xcorr_plan_only(1) == 0
    try:
        p = xc.Params()  # struct_size 0
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 1
        assert b"struct_size" in lib.xcorr_last_error()
        p = xc.make_params()
        assert p.struct_size == ctypes.sizeof(xc.Params)
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 0
        whole = xc.last_launch()
        # an older caller: its struct ends before matrix_cores, and what follows in memory is not the library's to read
        p = xc.make_params(matrix_cores=7)
        p.struct_size = xc.Params.matrix_cores.offset
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 0, lib.xcorr_last_error()
        assert xc.last_launch() == whole
        p.struct_size = ctypes.sizeof(xc.Params)
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 1
        assert b"matrix_cores" in lib.xcorr_last_error()
        # a larger struct than this build knows (a newer caller): the known part is read
        p = xc.make_params(shifts_per_thread=4)
        p.struct_size = ctypes.sizeof(xc.Params) + 16
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 0
        assert xc.last_launch()["y_shifts_per_thread"] == 4
        p.struct_size = 6
        assert lib.xcorr_grouped_overlap_f32(dummy, dummy, dummy, 200, 200, ctypes.byref(p), None) == 1
    finally:
        lib.xcorr_plan_only(0)


def test_split_plans_need_ordinary_device_memory():
    """Plan-only mode 2 plans for an output the float atomic add is not defined on (host-mapped, managed): the launcher's own
    split is given up for the whole reduction per work item, a named chunk (which needs the atomic adds) is refused."""
    xc = load_package()
    lib = xc.lib()
    dummy = ctypes.c_void_p(16)

    def ask(fn, mode, *args, **kw):
        assert lib.xcorr_plan_only(mode) == 0
        try:
            p = xc.make_params(**kw)
            code = getattr(lib, fn)(dummy, dummy, dummy, *args, ctypes.byref(p), None)
            return code, (xc.last_launch() if code == 0 else lib.xcorr_last_error())
        finally:
            lib.xcorr_plan_only(0)

    code, rec = ask("xcorr_grouped_overlap_f32", 1, 512, 512)
    assert code == 0 and rec["uses_atomics"] == 1
    code, rec = ask("xcorr_grouped_overlap_f32", 2, 512, 512)
    assert code == 0 and rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 512
    code, rec = ask("xcorr_shuffle_f32", 2, 64, 64, matrix_cores=2)
    assert code == 0 and rec["uses_atomics"] == 0
    # a small pair runs whole in LDS whatever the memory; a large one of a zeroed-output family is replanned with whole rows
    code, rec = ask("xcorr_split_row_f32", 2, 64, 64)
    assert code == 0 and rec["uses_atomics"] == 0 and "pair_in_lds" in rec["kernel"]
    code, rec = ask("xcorr_split_row_f32", 1, 512, 512)
    assert code == 0 and rec["uses_atomics"] == 1
    code, rec = ask("xcorr_split_row_f32", 2, 512, 512)
    assert code == 0 and rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 512 and rec["column_chunks"] == 1
    code, msg = ask("xcorr_split_row_f32", 2, 512, 512, rows_per_thread=32)
    assert code == 3 and b"atomics" in msg
    code, msg = ask("xcorr_grouped_overlap_f32", 2, 512, 512, rows_per_thread=32)
    assert code == 3
    code, rec = ask("xcorr_multimat_both_f64", 2, 64, 64, 4, 4, rows_per_thread=16)
    assert code == 3
    code, rec = ask("xcorr_multimat_both_f64", 2, 64, 64, 4, 4)
    assert code == 0 and rec["uses_atomics"] == 0
    assert lib.xcorr_plan_only(3) == 1


def test_callers_are_told_when_to_zero_the_output():
    """xcorr_multimat_right with a distribution but no chunk runs under the work-distribution contract (the caller zeroes
    `out`): the package's own wrapper zeroes in exactly the cases the header names."""
    xc = load_package()
    assert not xc.needs_zeroed_output("multimat_right", xc.make_params())
    assert not xc.needs_zeroed_output("multimat_right", xc.make_params(distribution_type="none"))
    assert xc.needs_zeroed_output("multimat_right", xc.make_params(distribution_type="rectangle"))
    assert xc.needs_zeroed_output("multimat_right", xc.make_params(distribution_type="triangle"))
    assert xc.needs_zeroed_output("multimat_right", xc.make_params(rows_per_thread=4))
    assert xc.needs_zeroed_output("multimat_right_groups", xc.make_params(rows_per_thread=4))
    assert xc.needs_zeroed_output("split_row", None) and xc.needs_zeroed_output("multimat_both", None)
    assert not xc.needs_zeroed_output("grouped_overlap", None) and not xc.needs_zeroed_output("multimat_right_grouped", None)
