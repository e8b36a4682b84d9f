"""Launches on many streams at once (reference: the n_to_mn / n_to_m algorithms launch one kernel per left matrix round-robin
on `num_cuda_streams` streams, n_to_mn.hpp:553-571). The matrix-core kernel runs persistent blocks that draw their work
items from counters the library keeps per stream (64 streams; further ones run one block per work item): launches that are
in flight together on different streams must not see each other's counters, a stream's counters must be back at zero when
its kernel ends, and a stream beyond the 64th must still get the right result."""
import ctypes

import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def test_seventy_streams_in_flight(oracle):
    xc = load_package()
    rng = np.random.default_rng(31)
    size, n_streams, rounds = 256, 70, 3
    out_shape = (1, 2 * size - 1, 2 * size - 1)
    # eight distinct pairs shared by the streams (integers: every launch must be bit-exact, in any order of atomic adds)
    pairs = []
    for _ in range(8):
        left, right = rng.integers(-2, 3, (size, size)).astype(np.float32), rng.integers(-2, 3, (size, size)).astype(np.float32)
        pairs.append((xc.DeviceBuffer.from_numpy(left), xc.DeviceBuffer.from_numpy(right), oracle.one_to_one(left, right).reshape(out_shape)))
    streams = [xc.Stream() for _ in range(n_streams)]
    outs = [xc.DeviceBuffer(int(np.prod(out_shape)) * 4) for _ in range(n_streams)]
    try:
        # what runs: a launch with more work items than the device holds blocks, i.e. persistent blocks with a queue
        xc.lib().xcorr_plan_only(1)
        xc.launch("grouped_overlap", pairs[0][0], pairs[0][1], outs[0], size, size, 1, 1, np.float32, None, None)
        rec = xc.last_launch()
        xc.lib().xcorr_plan_only(0)
        print("kernel", rec["kernel"], "work items", rec["grid"][0], "blocks per CU", rec["blocks_per_cu"], flush=True)
        assert rec["matrix_cores"] == 1 and rec["grid"][0] > 256 * rec["blocks_per_cu"]
        for r in range(rounds):  # (a stream's second launch finds the counters its first one left)
            for i, s in enumerate(streams):
                d_left, d_right, _ = pairs[(i + r) % len(pairs)]
                for b in (outs[i],):
                    assert xc.lib().xcorr_memset_async(b.ptr, 0xFF, ctypes.c_size_t(b.nbytes), s.ptr) == 0
                xc.launch("grouped_overlap", d_left, d_right, outs[i], size, size, 1, 1, np.float32, None, s.ptr)
            xc.sync()
            for i in range(n_streams):
                got = outs[i].to_numpy(out_shape, np.float32)
                assert np.array_equal(got, pairs[(i + r) % len(pairs)][2]), (r, i)
        # the default stream after all that
        d_left, d_right, exp = pairs[3]
        xc.launch("grouped_overlap", d_left, d_right, outs[0], size, size, 1, 1, np.float32, None, None)
        xc.sync()
        assert np.array_equal(outs[0].to_numpy(out_shape, np.float32), exp)
    finally:
        xc.sync()
        for s in streams:
            s.destroy()
        for b in outs:
            b.free()
        for d_left, d_right, _ in pairs:
            d_left.free()
            d_right.free()
