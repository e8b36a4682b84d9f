#!/usr/bin/env python3
"""Benchmark of the definition-based 2D cross-correlation hot path on one MI355X.

A step is one pass of the hot path (one C-ABI launch: the engine kernel, preceded by
the output clear when the launcher splits the reduction) over one batch of synthetic
input that is already resident in HBM. Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_oracle, load_package  # noqa: E402

# MI355X published vector peaks (TFLOP/s)
PEAK_TFLOPS = {"float32": 157.3, "float64": 78.6}
# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs scaled
# by the library's copy kernel (figures and commands: profiles/engine_f32_a8b4_one_to_one_1024.md, profiles/engine_other_workloads.md).
# Measured for the default parameters of each workload only (fetched + written).
MEASURED_TRAFFIC_BYTES = {"C2": 2.232e9 + 0.636e9, "C3": 0.0253e9 + 0.143e9, "C4": 0.0114e9 + 0.062e9, "C5": 0.006e9 + 0.108e9}


def cpu_baseline(oracle, cfg, left, right, budget_s=15.0):
    """The oracle (a port of the reference's single-threaded host loop, validate.hpp:94-132,
    here split over output rows with OpenMP, bit-identical per element) timed on a bounded
    sample of the same workload: a band of central output rows of the first pair."""
    threads = max(1, min(16, os.cpu_count() or 1))
    rows, cols = cfg["rows"], cfg["cols"]
    l0, r0 = left[0], right[0]
    centre = rows - 1

    def band_fmas(lo, hi):  # output row oy costs (rows - |oy - centre|) * cols^2 FMAs
        return sum((rows - abs(oy - centre)) * cols * cols for oy in range(lo, hi))

    def timed(n_rows):
        lo = max(0, centre - n_rows // 2)
        hi = min(2 * rows - 1, lo + n_rows)
        t0 = time.perf_counter()
        out = oracle.cross_corr(l0, r0, threads=threads, row_begin=lo, row_end=hi)
        return time.perf_counter() - t0, lo, hi, out

    probe_rows = min(2 * rows - 1, threads)
    dt, lo, hi, out = timed(probe_rows)
    rate = band_fmas(lo, hi) / max(dt, 1e-6)
    want = int(budget_s * rate / (rows * cols * cols))
    want = max(probe_rows, min(2 * rows - 1, want))
    if want > probe_rows:
        dt, lo, hi, out = timed(want)
    t_total, fmas = dt, band_fmas(lo, hi)
    gflops = 2.0 * fmas / t_total / 1e9
    return {
        "value": round(gflops, 3),
        "unit": "GFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"output rows [{lo},{hi}) of pair 0 of {cfg['name']} ({fmas:.3e} FMAs, {t_total:.2f} s), OpenMP over output rows",
        "time_per_instance_us_extrapolated": round(2.0 * (rows * cols) ** 2 / (gflops * 1e9) * 1e6, 1),
    }, (lo, hi, out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="C2")
    ap.add_argument("--family", default=None)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--params", default="{}", help="JSON object of xcorr_params fields")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the library's plain copy kernel on 256 MiB so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "readings of the same run can be scaled to bytes")
    ap.add_argument("--data", choices=["config", "integers", "zeros"], default="config",
                    help="input values: the configuration's seeded distribution (default; what the figures are quoted on), "
                         "small integers, or zeros. The kernels execute the same instructions for any values, but the shader "
                         "clock of the GPU is power-managed and runs 10-15 %% higher when few operand bits toggle")
    ap.add_argument("--graph-replay", type=int, default=0, metavar="N",
                    help="additionally capture N steps into one HIP graph and time its replays (reported under \"graph_replay\")")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every output element is an independent reduction; "
              "no multi-GPU path is built). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    xc = load_package()
    from jpdc23_artifact_amd import workloads

    cfg = dict(workloads.CONFIGS[args.config], name=args.config)
    family = args.family or cfg["family"]
    dtype = np.dtype(cfg["dtype"])
    left, right = workloads.generate(cfg, integer_valued=args.data != "config")
    if args.data == "zeros":
        left, right = np.zeros_like(left), np.zeros_like(right)
    rows, cols = cfg["rows"], cfg["cols"]
    pairs = workloads.num_pairs(cfg)
    n_left = cfg["n_left"]
    n_right = cfg["n_right"] // n_left if cfg["mode"] == "n_to_mn" else cfg["n_right"]
    if cfg["mode"] == "n_to_mn":
        # device order: left l owns the contiguous group [l*m, (l+1)*m) (file matrix t*n + l)
        n, m = n_left, n_right
        right_dev = np.ascontiguousarray(right.reshape(m, n, rows, cols).transpose(1, 0, 2, 3)).reshape(n * m, rows, cols)
    else:
        right_dev = right
    params = xc.make_params(**dict(cfg.get("params", {}) if args.family is None else {}, **json.loads(args.params)))

    d_left = xc.DeviceBuffer.from_numpy(left)
    d_right = xc.DeviceBuffer.from_numpy(right_dev)
    out_shape = (pairs, 2 * rows - 1, 2 * cols - 1)
    d_out = xc.DeviceBuffer(int(np.prod(out_shape)) * dtype.itemsize)
    zero_first = xc.needs_zeroed_output(family, params)

    def step():
        if zero_first:
            d_out.zero()
        xc.launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, dtype, params)

    if args.calibrate_copy:
        import ctypes

        nbytes = 256 * 1024 * 1024
        src, dst = xc.DeviceBuffer(nbytes), xc.DeviceBuffer(nbytes)
        src.zero()
        for _ in range(3):  # each launch reads 256 MiB and writes 256 MiB
            code = xc.lib().xcorr_copy_kernel(dst.ptr, src.ptr, ctypes.c_size_t(nbytes), None)
            assert code == 0, xc.lib().xcorr_last_error()
        xc.sync()
        src.free()
        dst.free()

    # the shader clock of an idle MI355X needs some tens of milliseconds of load to reach its
    # operating point (measured: 2.0 GHz in the first 5 ms, 2.4 GHz after ~100 ms), so short
    # workloads get an untimed pre-warm of at least 0.3 s before the W warmup steps
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < 0.3:
        for _ in range(4):
            step()
        xc.sync()
    for _ in range(args.warmup):
        step()
    xc.sync()
    start, stop = xc.Event(), xc.Event()
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    xc.sync()
    wall = time.perf_counter() - t0
    ev_ms = start.elapsed_ms(stop)
    rec = xc.last_launch()

    graph_replay = None
    if args.graph_replay > 0:
        # launch-bound workloads: N steps recorded once, replayed as one submission
        import ctypes

        stream = xc.Stream()

        def step_on(s):
            if zero_first:
                code = xc.lib().xcorr_clear_async(d_out.ptr, ctypes.c_size_t(d_out.nbytes), s)
                assert code == 0, xc.lib().xcorr_last_error()
            xc.launch(family, d_left, d_right, d_out, cols, rows, n_left, n_right, dtype, params, s)

        step_on(stream.ptr)
        stream.sync()
        graph = xc.Graph(stream)
        graph.begin()
        for _ in range(args.graph_replay):
            step_on(stream.ptr)
        graph.end()
        for _ in range(3):
            graph.launch()
        stream.sync()
        replays = max(1, args.steps // 2)
        g0 = time.perf_counter()
        for _ in range(replays):
            graph.launch()
        stream.sync()
        g_wall = time.perf_counter() - g0
        graph_replay = {"steps_per_graph": args.graph_replay, "replays": replays,
                        "us_per_step": round(g_wall * 1e6 / (replays * args.graph_replay), 3)}
        graph.destroy()
        stream.destroy()

    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = ev_ms / args.steps
    fmas = workloads.fma_count(cfg)
    flop = 2.0 * fmas
    gflops = flop / (ms_per_step * 1e-3) / 1e9
    achieved_tflops = flop / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[cfg["dtype"]]

    result = {
        "metric": "xcorr GFLOP/s (2 FLOP per overlapping element pair); time/instance in time_per_instance_us",
        "value": round(gflops, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "time_per_instance_us": round(ms_per_step * 1e3 / pairs, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if dtype == np.float32 else "f64",
        "data": "synthetic" if args.data == "config" else f"synthetic ({args.data})",
        "config": {
            "workload": f"{args.config}: {cfg['mode']} {cfg['n_left']}x{cfg['n_right']} matrices of {rows}x{cols} {cfg['dtype']}, "
                        f"{cfg['dist']} seed {cfg['seed']}, family {family}",
            "kernel": rec["kernel"],
            "grid": rec["grid"][0],
            "block": rec["block"][0],
            "rows_per_worker": rec["rows_per_worker"],
            "uses_atomics": rec["uses_atomics"],
        },
        "roofline": {
            "bound": "valu",
            "achieved": round(achieved_tflops, 3),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(achieved_tflops / peak, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.config) if (args.family is None and args.params == "{}") else None,
            "algorithmic_bytes": workloads.algorithmic_bytes(cfg),
            "kernel_ms": round(kernel_ms, 4),
            "note": "vector-FMA roofline (MFMA is not used); the kernel issues plain v_fmac_f32, which measures "
                    "0.97 of this peak in a register-only loop on MI355X; the peak assumes 2.4 GHz, the power-managed "
                    "shader clock under this kernel is 2.0-2.1 GHz on random data (2.37 GHz with --data integers)" if dtype == np.float32 else
                    "vector-FMA roofline, v_fma_f64",
        },
    }

    if graph_replay:
        result["graph_replay"] = graph_replay
    if not args.no_cpu:
        oracle = load_oracle()
        base, (lo, hi, band) = cpu_baseline(oracle, cfg, left, right)
        result["cpu_baseline"] = base
        got = d_out.to_numpy(out_shape, dtype)
        e = oracle.errors(got[0][lo:hi], band[lo:hi])
        result["parity"] = {
            "against": f"oracle rows [{lo},{hi}) of pair 0",
            "rel_frobenius": float(f"{e.rel_frobenius:.3e}"),
            "max_abs": float(f"{e.max_abs:.3e}"),
            "max_rel": float(f"{e.max_rel:.3e}"),
        }
        if dtype == np.float32:
            # the host loop adds every overlap one product at a time in fp32 and drifts from the exact
            # sum on long overlaps; the same loop with an fp64 accumulator tells the two apart
            mid = (lo + hi) // 2
            lo64, hi64 = max(lo, mid - 8), min(hi, mid + 8)
            exact = oracle.cross_corr(left[0], right[0], threads=base["cores"], row_begin=lo64, row_end=hi64, acc64=True)
            e64 = oracle.errors(got[0][lo64:hi64], exact[lo64:hi64])
            o64 = oracle.errors(band[lo64:hi64], exact[lo64:hi64])
            result["parity"]["rows_checked_with_fp64_accumulator"] = [lo64, hi64]
            result["parity"]["rel_frobenius_vs_fp64_accumulated"] = float(f"{e64.rel_frobenius:.3e}")
            result["parity"]["oracle_fp32_vs_fp64_accumulated"] = float(f"{o64.rel_frobenius:.3e}")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
