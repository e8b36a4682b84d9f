"""The entry point that allocates nothing and adds the chunks of a split reduction in order
(xcorr_grouped_overlap_ordered_f32: tickets in a fixed device array of the library) against the existing entry point
xcorr_grouped_overlap_f32, through the C ABI: bit for bit on integer-valued inputs, to 1e-5 (relative Frobenius) on real ones;
two calls in a row, the second with a smaller input; the same bits every run."""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def rel_frob(a, b):
    return float(np.linalg.norm((a.astype(np.float64) - b).ravel()) / np.linalg.norm(b.astype(np.float64).ravel()))


def test_ordered_entry_point_matches_the_existing_one():
    xc = load_package()
    rng = np.random.default_rng(2026)
    # first call: a pair whose reduction the launcher splits; second call: a smaller one (fewer tiles, fewer chunks)
    for shape in [(700, 520), (300, 260), (64, 64), (130, 150)]:
        left = rng.integers(-4, 5, shape).astype(np.float32)
        right = rng.integers(-4, 5, shape).astype(np.float32)
        print("ordered, integer-valued", shape, flush=True)
        want = xc.run("grouped_overlap", left, right, 1)
        rec_existing = xc.last_launch()
        got = xc.run("grouped_overlap_ordered", left, right, 1)
        rec = xc.last_launch()
        print("   existing:", rec_existing["kernel"], "atomics", rec_existing["uses_atomics"], "| ordered:", rec["kernel"], "atomics", rec["uses_atomics"],
              "rows per chunk", rec["rows_per_worker"], flush=True)
        assert rec["uses_atomics"] == 0
        assert np.array_equal(got, want), (shape, np.argwhere(got != want)[:3].tolist())
    # real-valued: within the bar of the existing entry point, and the same bits on every call
    for shape in [(1024, 1024), (512, 384)]:
        left, right = rng.random(shape, dtype=np.float32), rng.random(shape, dtype=np.float32)
        print("ordered, uniform data", shape, flush=True)
        want = xc.run("grouped_overlap", left, right, 1)
        a = xc.run("grouped_overlap_ordered", left, right, 1)
        rec = xc.last_launch()
        b = xc.run("grouped_overlap_ordered", left, right, 1)
        e = rel_frob(a, want)
        print("   ", rec["kernel"], "rows per chunk", rec["rows_per_worker"], "atomics", rec["uses_atomics"], "distance from the existing entry point %.3e" % e, flush=True)
        assert rec["uses_atomics"] == 0 and rec["rows_per_worker"] < shape[0]
        assert e <= 1e-5
        assert np.array_equal(a, b)


def test_ordered_entry_point_limits():
    xc = load_package()
    left = np.ones((200, 200), np.float32)
    with pytest.raises(xc.XcorrError, match="matrix-core"):
        xc.run("grouped_overlap_ordered", left, left, 1, params=xc.make_params(matrix_cores=2))
    with pytest.raises(xc.XcorrError, match="column_chunks"):
        xc.run("grouped_overlap_ordered", left, left, 1, params=xc.make_params(column_chunks=2))
    # forced chunks: every tile's chunks in order, also where a tile has a single chunk
    rng = np.random.default_rng(3)
    a, b = rng.integers(-3, 4, (150, 90)).astype(np.float32), rng.integers(-3, 4, (150, 90)).astype(np.float32)
    want = xc.run("grouped_overlap", a, b, 1, params=xc.make_params(rows_per_thread=150, column_chunks=1))
    for rows in (8, 24, 40, 149):
        got = xc.run("grouped_overlap_ordered", a, b, 1, params=xc.make_params(rows_per_thread=rows))
        rec = xc.last_launch()
        assert rec["uses_atomics"] == 0 and rec["rows_per_worker"] == rows, rec
        assert np.array_equal(got, want), rows
