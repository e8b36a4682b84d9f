"""CPU-only: what the launcher of the sliding-window engine would run, asked through xcorr_plan_only (the entry
points validate, plan and fill the launch record without launching; without a GPU the planner assumes 256 CUs).
Only rules that do not depend on the occupancy the runtime reports for a kernel are pinned here: the tile class a
family and its tuning integers select, the chunk rule of the one-output-row families, when plain launchers split,
column chunks, the whole-pair route, and the error paths."""
import ctypes

import numpy as np
import pytest

from conftest import load_package


class _Dummy:
    ptr = ctypes.c_void_p(64)  # never read in plan-only mode


@pytest.fixture()
def plan():
    xc = load_package()
    lib = xc.lib()
    assert lib.xcorr_plan_only(1) == 0

    def ask(family, cols, rows, n_left=1, n_right=1, dtype=np.float32, **kw):
        xc.launch(family, _Dummy, _Dummy, _Dummy, cols, rows, n_left, n_right, dtype, xc.make_params(**kw))
        return xc.last_launch()

    try:
        yield ask
    finally:
        lib.xcorr_plan_only(0)


def register_tiles(plan):
    """The same planner with the matrix-core tiles excluded: the rules of the one-output-row tiles."""
    return lambda *a, **kw: plan(*a, matrix_cores=2, **kw)


def test_plain_one_row_launcher_splits_only_when_it_pays(plan):
    plan = register_tiles(plan)
    rec = plan("shuffle", 64, 64)
    assert rec["kernel"] == "shuffle/f32_a1b4" and rec["uses_atomics"] == 1 and 3 <= rec["rows_per_worker"] <= 8
    rec = plan("shuffle", 64, 64, distribution_type="none")
    assert rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 64 and rec["distribution_type"] == 1
    # a large pair: wide tile; "none" keeps it whole whatever the planner would gain
    rec = plan("shuffle", 1024, 1024, distribution_type="none")
    assert rec["kernel"] == "shuffle/f32_a1b8" and rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 1024
    assert plan("shuffle", 512, 512)["kernel"] == "shuffle/f32_a1b8"
    assert plan("shuffle", 256, 256)["kernel"] == "shuffle/f32_a1b4"
    assert plan("shuffle", 64, 64, dtype=np.float64)["kernel"] == "shuffle/f64_a1b4"


def test_split_row_chunk(plan):
    plan = register_tiles(plan)
    # the caller's chunk and distribution are taken as given
    rec = plan("split_row", 100, 90, rows_per_thread=7, distribution_type="triangle")
    assert rec["rows_per_worker"] == 7 and rec["distribution_type"] == 3 and rec["uses_atomics"] == 1
    rec = plan("split_row", 100, 90, rows_per_thread=10)
    assert rec["rows_per_worker"] == 10 and rec["distribution_type"] == 2  # the reference's default: rectangle
    # none given: short chunks for one small pair, longer ones as the matrices grow
    small, medium, large = (plan("split_row", n, n)["rows_per_worker"] for n in (32, 128, 512))
    assert small <= 5 and 8 <= medium <= 16 and 16 <= large <= 64
    # rows explicitly whole and few work items: the columns are cut instead
    rec = plan("split_row", 64, 64, distribution_type="none")
    assert rec["rows_per_worker"] == 64 and rec["column_chunks"] > 1 and rec["uses_atomics"] == 1
    rec = plan("split_row", 64, 64, distribution_type="none", column_chunks=1)
    assert rec["column_chunks"] == 1


def test_matrices_per_lane(plan):
    plan = register_tiles(plan)
    # small launches: one matrix per lane; a request for matrices per thread overrides; large launches reuse
    assert plan("multimat_both", 16, 16, 2, 2)["kernel"] == "multimat_both/f32_a1b4"
    assert plan("multimat_both", 16, 16, 2, 2, right_matrices_per_thread=4)["kernel"] == "multimat_both/f32_a1b4_r4"
    assert plan("multimat_both", 16, 16, 2, 2, left_matrices_per_thread=2, right_matrices_per_thread=2)["kernel"] == "multimat_both/f32_a1b4_l2r2"
    rec = plan("multimat_both", 128, 128, 32, 32)
    assert rec["left_matrices_per_thread"] * rec["right_matrices_per_thread"] > 1
    assert rec["rows_per_worker"] == 128  # the pairs alone fill the device: whole matrices
    assert plan("multimat_right", 32, 32, 1, 8)["kernel"] == "multimat_right/f32_a1b4"
    rec = plan("multimat_right", 256, 256, 1, 32)
    assert rec["right_matrices_per_thread"] == 4


def test_multimat_right_contracts(plan):
    # plain launcher: may split (then clears the output itself); a distribution or a chunk: the work-distribution contract
    xc = load_package()
    assert not xc.needs_zeroed_output("multimat_right", xc.make_params())
    assert xc.needs_zeroed_output("multimat_right", xc.make_params(distribution_type="triangle"))
    assert xc.needs_zeroed_output("multimat_right", xc.make_params(rows_per_thread=3))
    assert not xc.needs_zeroed_output("multimat_right", xc.make_params(distribution_type="none"))
    rec = plan("multimat_right", 64, 64, 1, 8, distribution_type="triangle")
    assert rec["uses_atomics"] == 1 and rec["distribution_type"] == 3 and 1 <= rec["rows_per_worker"] < 64
    rec = plan("multimat_right", 64, 64, 1, 8, distribution_type="none")
    assert rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 64
    # the groups entry point plans like the single-left one, over all left matrices
    one = plan("multimat_right", 64, 64, 1, 4, rows_per_thread=8, distribution_type="rectangle")
    many = plan("multimat_right_groups", 64, 64, 5, 4, rows_per_thread=8, distribution_type="rectangle")
    assert many["kernel"] == one["kernel"] and many["grid"][0] == 5 * one["grid"][0]


def test_grouped_requests_and_whole_pair_route(plan):
    assert "pair_in_lds" in plan("grouped_overlap", 64, 64)["kernel"]
    assert "pair_in_lds" not in plan("grouped_overlap", 64, 64, whole_pair_in_lds=2)["kernel"]
    assert "pair_in_lds" not in plan("grouped_overlap", 64, 64, shifts_per_thread=8)["kernel"]
    assert "pair_in_lds" not in plan("grouped_overlap", 300, 300)["kernel"]
    for asked, got in [(1, 4), (3, 4), (4, 4), (5, 8), (8, 8)]:
        assert plan("grouped_overlap", 300, 300, shifts_per_thread=asked)["y_shifts_per_thread"] == got
    rec = plan("multimat_both_grouped", 30, 30, 8, 8, left_matrices_per_thread=4, right_matrices_per_thread=4)
    assert rec["left_matrices_per_thread"] * rec["lanes_left"] == 4 and rec["right_matrices_per_thread"] * rec["lanes_right"] == 4
    rec = plan("multimat_right_grouped", 40, 33, 1, 7, shifts_per_thread_right_matrix=2, right_matrices_per_thread=2)
    assert rec["y_shifts_per_thread"] == 4 and rec["right_matrices_per_thread"] * rec["lanes_right"] == 4


def test_matrix_core_tiles(plan):
    # a large pair runs on the matrix cores by default; matrix_cores = 2 keeps the register tiles, 1 excludes them
    rec = plan("grouped_overlap", 1024, 1024)
    assert rec["matrix_cores"] == 1 and rec["kernel"].startswith("grouped_overlap/f32_m") and rec["predicted_us"] > 0
    assert rec["lanes_x"] * rec["lanes_y"] * rec["lanes_left"] * rec["lanes_right"] == 64
    rec = plan("grouped_overlap", 1024, 1024, matrix_cores=2)
    assert rec["matrix_cores"] == 0 and rec["kernel"] == "grouped_overlap/f32_a8b4"
    rec = plan("grouped_overlap", 512, 512, dtype=np.float64, matrix_cores=1)
    assert rec["matrix_cores"] == 1 and "f64_m32x" in rec["kernel"]
    # one left matrix with its own right matrices: only tiles with a single left matrix; all pairs: any
    rec = plan("multimat_right_grouped", 128, 128, 8, 16, matrix_cores=1)
    assert rec["matrix_cores"] == 1 and rec["left_matrices_per_thread"] * rec["lanes_left"] == 1
    rec = plan("multimat_both_grouped", 64, 64, 16, 32, matrix_cores=1)
    assert rec["matrix_cores"] == 1
    # the reference's tuning integers still restrict the choice: eight y shifts per thread exist among the register tiles only
    rec = plan("grouped_overlap", 300, 300, shifts_per_thread=8)
    assert rec["matrix_cores"] == 0 and rec["y_shifts_per_thread"] == 8
    xc = load_package()
    with pytest.raises(xc.XcorrError, match="matrix_cores must be 0, 1 or 2"):
        plan("grouped_overlap", 300, 300, matrix_cores=3)


def test_one_row_families_on_matrix_core_tiles(plan):
    """The one-output-row families are contracts: large enough launches that name no tile run a matrix-core tile under them."""
    rec = plan("split_row", 256, 256)
    assert rec["matrix_cores"] == 1 and rec["kernel"].startswith("split_row/f32_m") and rec["uses_atomics"] == 1 and rec["distribution_type"] == 3
    # (a matrix-core tile deals its work items tile by tile whatever distribution is named; the record tells)
    rec = plan("split_row", 256, 256, rows_per_thread=32, distribution_type="rectangle")
    assert rec["matrix_cores"] == 1 and rec["rows_per_worker"] == 32 and rec["distribution_type"] == 3
    rec = plan("split_row", 256, 256, distribution_type="none")
    # (one work item per result tile: plain stores, and the record says that nothing is added into the output)
    assert rec["matrix_cores"] == 1 and rec["rows_per_worker"] == 256 and rec["uses_atomics"] == 0
    # short chunks of rows fixed by the caller, a tile request, small launches, matrix_cores = 2: the one-row tiles
    assert plan("split_row", 256, 256, rows_per_thread=7)["matrix_cores"] == 0
    assert plan("multimat_right", 128, 128, 1, 32, right_matrices_per_thread=4)["matrix_cores"] == 0
    # (whole_pair_in_lds = 2: not the kernel that keeps small pairs whole in LDS, which comes before the engine's tiles)
    assert plan("shuffle", 32, 32, whole_pair_in_lds=2)["matrix_cores"] == 0 and plan("shuffle", 64, 64, whole_pair_in_lds=2)["matrix_cores"] == 1
    assert plan("multimat_both", 32, 32, 2, 2, whole_pair_in_lds=2)["matrix_cores"] == 0
    assert plan("multimat_both", 32, 32, 8, 8, whole_pair_in_lds=2)["matrix_cores"] == 1
    assert plan("multimat_right", 32, 32, 1, 2, whole_pair_in_lds=2)["matrix_cores"] == 0
    assert plan("multimat_right", 32, 32, 1, 32, whole_pair_in_lds=2)["matrix_cores"] == 1
    # few small pairs and nothing named: every pair whole in LDS, plain stores under any of the contracts
    for family, shape in (("shuffle", (64, 64)), ("split_row", (96, 96)), ("multimat_right", (32, 32, 1, 16)), ("multimat_right_groups", (16, 16, 4, 4)),
                          ("multimat_both", (16, 16, 8, 8)), ("warp_per_overlap_lds", (32, 32, 1, 8))):
        rec = plan(family, *shape)
        assert "pair_in_lds" in rec["kernel"] and rec["uses_atomics"] == 0, (family, rec)
    assert "pair_in_lds" not in plan("multimat_both", 16, 16, 9, 8)["kernel"] and "pair_in_lds" not in plan("multimat_both", 32, 32, 8, 8)["kernel"]
    assert "pair_in_lds" not in plan("warp_per_overlap_lds", 32, 32, 1, 8, right_matrices_per_block=2)["kernel"] and "pair_in_lds" not in plan("split_row", 128, 128)["kernel"]
    assert "pair_in_lds" not in plan("multimat_both", 32, 32, 2, 2, rows_per_thread=8)["kernel"]
    assert plan("multimat_right", 256, 256, 1, 32, matrix_cores=2)["matrix_cores"] == 0
    # the plain launcher told to keep the rows whole keeps the summation order of one pass over the rows: a one-row tile
    rec = plan("shuffle", 256, 256, distribution_type="none")
    assert rec["matrix_cores"] == 0 and rec["uses_atomics"] == 0 and rec["rows_per_worker"] == 256
    # matrix_cores = 1 forces the route also for small launches
    assert plan("shuffle", 16, 16, matrix_cores=1)["matrix_cores"] == 1


def test_largest_matrices(plan):
    # 16384 x 16384: chunk sizes whose work items do not fit the launch arithmetic are passed over, not reported
    rec = plan("grouped_overlap", 16384, 16384)
    assert rec["grid"][0] > 0 and rec["matrix_cores"] == 1
    # (every band of a matrix-core tile has a 64-bit base of its own: tiles of several matrices serve these sizes too)
    rec = plan("multimat_right_grouped", 16384, 16384, 1, 8)
    assert rec["grid"][0] > 0


def test_errors_in_plan_only_mode(plan):
    xc = load_package()
    with pytest.raises(xc.XcorrError, match="Too many shifts per thread: 9"):
        plan("grouped_overlap", 64, 64, shifts_per_thread=9)
    with pytest.raises(xc.XcorrError, match="does not exist"):
        plan("grouped_overlap", 64, 64, specialisation=999)
    with pytest.raises(xc.XcorrError, match="does not fit the LDS"):
        plan("grouped_overlap", 300, 300, whole_pair_in_lds=1)
    with pytest.raises(xc.XcorrError):
        plan("multimat_right_groups", 16, 16, 3, 0)


FIVE_CONFIGURATIONS = [
    # family, cols, rows, n_left, n_right (per left matrix for n_to_mn), dtype, kernel of the default launch on an MI355X
    ("grouped_overlap", 64, 64, 1, 1, np.float32, "grouped_overlap/pair_in_lds_f32_a1"),
    ("grouped_overlap", 1024, 1024, 1, 1, np.float32, "grouped_overlap/f32_m32x32"),
    ("multimat_right_grouped", 256, 256, 1, 64, np.float32, "multimat_right_grouped/f32_m16x16_r4_s4"),
    ("multimat_right_grouped", 128, 128, 8, 16, np.float32, "multimat_right_grouped/f32_m16x16_r4_s4"),
    ("multimat_both_grouped", 64, 64, 16, 32, np.float64, "multimat_both_grouped/f64_m8x8_l4r4"),
]


def test_the_five_benchmark_configurations_plan_as_on_the_device(plan):
    """Without a GPU the planner assumes an MI355X: 256 CUs and that device's blocks per CU for every compiled kernel (a table
    that a GPU test compares with the runtime's answers). The kernels named here are the ones bench.py reports there."""
    for family, cols, rows, n_left, n_right, dtype, kernel in FIVE_CONFIGURATIONS:
        rec = plan(family, cols, rows, n_left, n_right, dtype=dtype)
        assert rec["kernel"] == kernel, (family, cols, rec["kernel"])
        assert rec["blocks_per_cu"] >= 1
    rec = plan("grouped_overlap", 1024, 1024)
    assert rec["rows_per_worker"] == 32 and rec["uses_atomics"] == 1 and rec["blocks_per_cu"] == 5
