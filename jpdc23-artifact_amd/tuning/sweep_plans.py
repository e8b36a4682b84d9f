#!/usr/bin/env python3
"""Measures every compiled grouped tile with every chunking of the reduction on a list of problem shapes,
next to the plan the library's planner picks: the data the constants of the planner's run-time model
(csrc/engine_plan.hip, predict_us) were fitted to, and the check that its picks are close to the best plan.

  python sweep_plans.py [--dtype float32|float64] [--shapes mode:n_left:n_right:size,...] [--planner-only] > sweep.log
  python fit_planner_model.py sweep.log          # re-fit the constants, report the regret of the model's picks

One line per measured plan:
  <shape> spec=<1-based tile index, 0 = planner> <kernel> rc=<rows per work item> grid=<blocks> lds=<bytes> occ=<blocks per CU>
  xc=<column chunks> <microseconds> us <TFLOP/s> TF
Every plan is launched through the C ABI with `specialisation` / `rows_per_thread` forced (HIP events around 20
back-to-back launches after 50 ms of warm-up).
"""
import argparse
import os
import sys
import time

import numpy as np

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(PKG))
from __graft_entry__ import load_package  # noqa: E402

FAMILY = {"one_to_one": "grouped_overlap", "one_to_many": "multimat_right_grouped", "n_to_mn": "multimat_right_grouped",
          "n_to_m": "multimat_both_grouped"}


def default_shapes():
    shapes = [f"one_to_one:1:1:{s}" for s in (16, 32, 64, 128, 256, 512)]
    for s in (16, 32, 64, 128, 256):
        shapes += [f"one_to_many:1:8:{s}", f"one_to_many:1:32:{s}", f"n_to_mn:8:32:{s}", f"n_to_m:4:8:{s}"]
    for s in (16, 32, 64, 128):
        shapes += [f"n_to_m:32:32:{s}", f"one_to_many:1:128:{s}"]
    return shapes


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--dtype", default="float32", choices=["float32", "float64"])
    ap.add_argument("--shapes", default=",".join(default_shapes()))
    ap.add_argument("--planner-only", action="store_true", help="measure the planner's own pick only")
    a = ap.parse_args()
    xc = load_package()
    dtype = np.dtype(a.dtype)
    for shape in a.shapes.split(","):
        mode, n_left, n_right, size = shape.split(":")
        n_left, n_right, size = int(n_left), int(n_right), int(size)
        rng = np.random.default_rng(1)
        d_left = xc.DeviceBuffer.from_numpy(rng.random((n_left, size, size)).astype(dtype))
        d_right = xc.DeviceBuffer.from_numpy(rng.random((n_right, size, size)).astype(dtype))
        pairs = n_left * n_right if mode == "n_to_m" else n_right
        per_left = n_right // n_left if mode == "n_to_mn" else n_right
        d_out = xc.DeviceBuffer(pairs * (2 * size - 1) ** 2 * dtype.itemsize)
        flop = 2.0 * pairs * float(size) ** 4
        label = f"{shape}:{a.dtype}"

        def measure(spec, rows):
            # forced plans are not cut over columns (the model covers row chunks only); the planner's pick may be
            params = xc.make_params(specialisation=spec, rows_per_thread=rows, column_chunks=1 if spec else 0)

            def go():
                xc.launch(FAMILY[mode], d_left, d_right, d_out, size, size, n_left, per_left, dtype, params)

            go()
            xc.sync()
            rec = xc.last_launch()
            t = time.perf_counter()
            while time.perf_counter() - t < 0.05:
                go()
                xc.sync()
            start, stop = xc.Event(), xc.Event()
            start.record()
            for _ in range(20):
                go()
            stop.record()
            xc.sync()
            us = start.elapsed_ms(stop) / 20 * 1e3
            print(f"{label:34s} spec={spec:2d} {rec['kernel']:28s} rc={rec['rows_per_worker']:4d} grid={rec['grid'][0]:6d} "
                  f"lds={rec['shared_mem_bytes']:6d} occ={rec['blocks_per_cu']:2d} xc={rec['column_chunks']:2d} {us:10.1f} us {flop / us / 1e6:8.2f} TF",
                  flush=True)
            return rec

        measure(0, 0)
        if a.planner_only:
            continue
        spec = 1
        while True:
            try:
                rec = measure(spec, size)  # rows_per_thread >= rows: the reduction is not cut
            except xc.XcorrError as e:
                if "does not exist" in e.message:
                    break
                print(label, spec, "skipped:", e.message[:90], flush=True)
                spec += 1
                continue
            if rec["y_shifts_per_thread"] > 1:  # grouped tile: chunks of whole row groups
                group = rec["y_shifts_per_thread"] + 1
                for k in (2, 3, 4, 6, 8, 12, 16):
                    if k * group < size:
                        measure(spec, k * group)
            spec += 1
        d_out.free()


if __name__ == "__main__":
    main()
