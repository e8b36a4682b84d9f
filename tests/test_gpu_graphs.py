"""HIP graph capture of the C ABI's launches: a captured sequence (clear kernel, split-row family with atomics, the
grouped family with its own clear and row split on register and on matrix-core tiles, the overlap-wise kernel) is replayed several times with eager work and
synchronisations between the replays and with fresh inputs each time; every replay must equal the oracle exactly."""
import ctypes

import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def ints(rng, shape, dtype):
    return rng.integers(-4, 5, size=shape).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_captured_sequence_replays_with_fresh_inputs(oracle, dtype):
    xc = load_package()
    lib = xc.lib()
    rng = np.random.default_rng(1000)
    shape = (48, 40)
    out_elems = 95 * 79
    item = np.dtype(dtype).itemsize
    d_left, d_right = xc.DeviceBuffer(48 * 40 * item), xc.DeviceBuffer(48 * 40 * item)
    d_many = xc.DeviceBuffer(6 * 48 * 40 * item)
    outs = {k: xc.DeviceBuffer(n * out_elems * item) for k, n in [("split_row", 1), ("grouped", 1), ("overlap_wise", 1), ("many", 6), ("cores", 1), ("many_cores", 6)]}

    def upload(buf, a):
        a = np.ascontiguousarray(a)
        assert lib.xcorr_memcpy_h2d(buf.ptr, a.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(a.nbytes)) == 0

    def sequence(stream):
        assert lib.xcorr_clear_async(outs["split_row"].ptr, ctypes.c_size_t(outs["split_row"].nbytes), stream) == 0
        xc.launch("split_row", d_left, d_right, outs["split_row"], 40, 48, 1, 1, dtype, xc.make_params(rows_per_thread=7), stream)
        xc.launch("grouped_overlap", d_left, d_right, outs["grouped"], 40, 48, 1, 1, dtype, None, stream)
        xc.launch("overlap_wise", d_left, d_right, outs["overlap_wise"], 40, 48, 1, 1, dtype, None, stream)
        xc.launch("grouped_overlap", d_left, d_right, outs["cores"], 40, 48, 1, 1, dtype, xc.make_params(matrix_cores=1, rows_per_thread=16), stream)
        assert xc.last_launch()["matrix_cores"] == 1 and xc.last_launch()["uses_atomics"] == 1
        xc.launch("multimat_right_grouped", d_left, d_many, outs["many_cores"], 40, 48, 1, 6, dtype, xc.make_params(matrix_cores=1), stream)
        assert xc.last_launch()["matrix_cores"] == 1
        xc.launch("multimat_right_grouped", d_left, d_many, outs["many"], 40, 48, 1, 6, dtype, xc.make_params(matrix_cores=2, rows_per_thread=18), stream)

    def check(left, right, many, what):
        exp = oracle.one_to_one(left, right)[0]
        for k in ("split_row", "grouped", "overlap_wise", "cores"):
            got = outs[k].to_numpy((95, 79), dtype)
            np.testing.assert_array_equal(got, exp, err_msg=f"{what} {k}")
        got = outs["many"].to_numpy((6, 95, 79), dtype)
        np.testing.assert_array_equal(got, oracle.one_to_many(left, many), err_msg=f"{what} many")
        got = outs["many_cores"].to_numpy((6, 95, 79), dtype)
        np.testing.assert_array_equal(got, oracle.one_to_many(left, many), err_msg=f"{what} many, matrix cores")

    left, right, many = ints(rng, shape, dtype), ints(rng, shape, dtype), ints(rng, (6,) + shape, dtype)
    upload(d_left, left), upload(d_right, right), upload(d_many, many)
    stream = xc.Stream()
    sequence(stream.ptr)  # eager first: one-time set-up happens outside the capture
    stream.sync()
    check(left, right, many, "eager")
    assert xc.last_launch()["uses_atomics"] == 1  # the last launch of the sequence is a row-split plan with its own clear kernel

    graph = xc.Graph(stream)
    graph.begin()
    sequence(stream.ptr)
    graph.end()
    for replay in range(4):
        left, right, many = ints(rng, shape, dtype), ints(rng, shape, dtype), ints(rng, (6,) + shape, dtype)
        upload(d_left, left), upload(d_right, right), upload(d_many, many)
        for o in outs.values():
            o.fill_bytes(0x7F)  # stale results cannot pass
        xc.sync()
        graph.launch()
        stream.sync()
        check(left, right, many, f"replay {replay}")
        # eager work between the replays, on the same buffers
        sequence(stream.ptr)
        stream.sync()
        check(left, right, many, f"eager after replay {replay}")
    graph.destroy()
    stream.destroy()
    with pytest.raises(xc.XcorrError, match="NULL stream"):
        xc._check(lib.xcorr_graph_capture_begin(None))
