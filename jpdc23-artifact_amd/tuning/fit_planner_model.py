#!/usr/bin/env python3
"""Fits the constants of the planner's run-time model (csrc/engine_plan.hip, predict_us) to logs of sweep_plans.py
and reports how far the model's pick is from the best measured plan of every shape.

  python fit_planner_model.py sweep_f32.log [more logs of the same element type ...] [--fix-global '...']
  python fit_planner_model.py sweep_f32.log --installed     # no fit: the constants in the sources against these logs

The model below mirrors predict_us term by term. Fitted by weighted least squares on log(time): plans close
to the best of their shape weigh most, so that the ranking near the optimum is what the fit gets right.
Printed: the global constants, `issue_factor` and `stage_factor` per tile (the two numbers after the tile name in
csrc/engine_f32.hip / engine_f64.hip), and the regret table. For fp64 the constants shared with fp32 (block cost,
issue efficiency curve, stage cost, tail share) are kept at the values given with --fix-global (a line
`t_block tau e_full t_stage k_tail`), as the planner uses one set for both element types.
The tile geometry is read from the `using <Name> = EngineCfg<...>` lines of the two source files.
"""
import argparse
import math
import os
import re
import sys

import numpy as np
from scipy.optimize import least_squares

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
CUS = 256            # compute units of an MI355X
CLOCK_MHZ = 2100.0   # shader clock under the engine's FMA + LDS mix


def tile_table():
    """kernel name -> (A, B, K, LX, LY, LV, LU, RL, KBX, WZ) for the grouped tiles of both element types"""
    tiles = {}
    for path in ("engine_f32.hip", "engine_f64.hip"):
        text = open(os.path.join(CSRC, path)).read()
        cfg = {m.group(1): [x.strip() for x in m.group(2).split(",")] for m in re.finditer(r"using (\w+) = EngineCfg<([^>]*)>;", text)}
        for m in re.finditer(r'make_spec<(\w+)>\("(\w+)"', text):
            p = cfg[m.group(1)]
            a, b, k, lx, ly, lv, lu, rl, kbx = (int(p[i]) for i in (1, 2, 3, 6, 7, 8, 9, 12, 13))
            wz = int(p[15]) if len(p) > 15 else 1
            if a > 1:
                tiles[m.group(2)] = (a, b, k, lx, ly, lv, lu, rl, kbx, wz)
    return tiles


LINE = re.compile(r"(\S+)\s+spec=\s*(\d+)\s+\S+/(\S+)\s+rc=\s*(\d+) grid=\s*(\d+) lds=\s*\d+ occ=\s*(\d+)(?: xc=\s*(\d+))?\s+([\d.]+) us")


def read_logs(paths, tiles):
    rows = []
    for path in paths:
        for line in open(path):
            m = LINE.match(line)
            if not m or int(m.group(2)) == 0 or m.group(3) not in tiles or int(m.group(7) or 1) != 1:
                continue
            mode, n_left, n_right, size, dtype = m.group(1).split(":")
            rows.append(dict(shape=m.group(1), W=int(size), H=int(size), name=m.group(3), rc=int(m.group(4)), grid=int(m.group(5)),
                             occ=int(m.group(6)), us=float(m.group(8)), f64=dtype == "float64"))
    return rows


def predict(x, names, tiles, r):
    t_block, tau, e_full, t_stage, k_tail, t_clear, t_atomic, atomic_plain, atomic_lanes = x[:9]
    issue = x[9 + names.index(r["name"])]
    stage = x[9 + len(names) + names.index(r["name"])]
    A, B, K, LX, LY, LV, LU, RL, KBX, WZ = tiles[r["name"]]
    W, H, rc = r["W"], r["H"], r["rc"]
    lanes_over_matrices = LV * LU > 1
    cyc = (4.0 if r["f64"] else 2.0) / CLOCK_MHZ
    TXW, TYW = LX * B, LY * A
    ntx, nty = -(-(2 * W - 1) // TXW), -(-(2 * H - 1) // TYW)
    split = rc < H
    cols_avg = min(W, W * (W + TXW) / (ntx * TXW))
    rows_tile = min(H, H * (H + TYW) / (nty * TYW))
    rows_avg = (min(rc, rows_tile) if split else rows_tile) + A - 1
    rows_max = (rc if split else H) + A - 1
    per_element = A * B / WZ * issue
    inst_avg, inst_max = per_element * rows_avg * cols_avg, per_element * rows_max * W
    stages_avg = math.ceil(rows_avg / RL) * math.ceil((cols_avg + TXW) / KBX) * stage
    stages_max = math.ceil(rows_max / RL) * math.ceil((W + TXW) / KBX) * stage
    items = r["grid"]
    n1 = min(r["occ"], -(-items // CUS))
    fixed = t_block + (t_atomic * A * B if split and not lanes_over_matrices else 0.0)
    # n1 blocks per CU (one wavefront each per SIMD) issue at e_full * (1 - exp(-n1 / tau)) of the FMA rate together
    crit = fixed + t_stage * stages_max + n1 * inst_max * cyc / (e_full * (1.0 - math.exp(-n1 / tau)))
    per_block = (fixed + t_stage * stages_avg) / n1 + inst_avg * cyc / e_full
    t = max(items * per_block / CUS + k_tail * crit, crit)
    if split:
        t += t_clear + items * 64.0 * A * B * (atomic_lanes if lanes_over_matrices else atomic_plain)
    return t


def installed_constants(names, f64):
    """the constants of predict_us and the per-tile factors as they stand in the sources"""
    text = open(os.path.join(CSRC, "engine_plan.hip")).read()
    body = text[text.index("static double predict_us"):]

    def pair(name):  # 'name = f32 ? a : b' or 'name = a'
        m = re.search(name + r" = (?:f32 \? )?([\d.e-]+)(?: : ([\d.e-]+))?", body)
        return float(m.group(2) if f64 and m.group(2) else m.group(1))

    m = re.search(r"us_per_atomic = lanes_over_matrices \? \(f32 \? ([\d.e-]+) : ([\d.e-]+)\) : \(f32 \? ([\d.e-]+) : ([\d.e-]+)\)", body)
    lanes, plain = (float(m.group(2)), float(m.group(4))) if f64 else (float(m.group(1)), float(m.group(3)))
    x = [pair("t_block"), pair("tau"), pair("e_full"), pair("t_stage"), pair("k_tail"), pair("t_clear"), pair("t_atomic"), plain, lanes]
    tile_text = open(os.path.join(CSRC, "engine_f64.hip" if f64 else "engine_f32.hip")).read()
    factors = {m.group(1): (float(m.group(2)), float(m.group(3))) for m in re.finditer(r'make_spec<\w+>\("(\w+)", ([\d.]+), ([\d.]+)\)', tile_text)}
    return x + [factors[n][0] for n in names] + [factors[n][1] for n in names]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("logs", nargs="+")
    ap.add_argument("--installed", action="store_true", help="do not fit: evaluate the constants that stand in the sources")
    ap.add_argument("--fix-global", default=None, metavar="'t_block tau e_full t_stage k_tail'")
    a = ap.parse_args()
    tiles = tile_table()
    rows = read_logs(a.logs, tiles)
    names = sorted({r["name"] for r in rows})
    best = {}
    for r in rows:
        best[r["shape"]] = min(best.get(r["shape"], 1e30), r["us"])
    x0 = [4.0, 1.5, 0.9, 0.1, 0.4, 1.0, 0.03, 3e-6, 5e-6] + [0.9] * len(names) + [1.0] * len(names)
    lo = [0.0, 0.2, 0.3, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0] + [0.5] * len(names) + [0.0] * len(names)
    hi = [20.0, 8.0, 1.0, 10.0, 2.0, 10.0, 1.0, 1e-2, 1e-2] + [4.0] * len(names) + [20.0] * len(names)
    if a.fix_global:
        for i, v in enumerate(float(t) for t in a.fix_global.split()):
            x0[i], lo[i], hi[i] = v, v - 1e-9, v + 1e-9

    def residuals(x):
        return [math.log(predict(x, names, tiles, r) / r["us"]) * (best[r["shape"]] / r["us"]) ** 1.5 for r in rows]

    if a.installed:
        x = np.array(installed_constants(names, rows[0]["f64"]))
        print(f"{len(rows)} measurements, constants of the sources, weighted rms of log(model / measured) = {np.sqrt(np.mean(np.square(residuals(x)))):.3f}")
    else:
        sol = least_squares(residuals, x0, bounds=(lo, hi))
        x = sol.x
        print(f"{len(rows)} measurements, weighted rms of log(model / measured) = {np.sqrt(np.mean(np.square(sol.fun))):.3f}")
    print("t_block tau e_full t_stage k_tail =", " ".join(f"{v:.4g}" for v in x[:5]))
    print("t_clear t_atomic us_per_atomic(plain) us_per_atomic(lanes over matrices) =", " ".join(f"{v:.4g}" for v in x[5:9]))
    for i, n in enumerate(names):
        print(f"  {n:20s} issue_factor {x[9 + i]:.3f}  stage_factor {x[9 + len(names) + i]:.3f}")
    by_shape = {}
    for r in rows:
        by_shape.setdefault(r["shape"], []).append(r)
    regrets = []
    for shape, rs in by_shape.items():
        # the planner does not cut tiles with lanes over matrices into chunks shorter than 36 rows or matrices below 72 rows
        allowed = [r for r in rs if not (tiles[r["name"]][5] * tiles[r["name"]][6] > 1 and r["rc"] < r["H"] and (r["rc"] < 36 or r["H"] < 72))]
        pick = min(allowed, key=lambda r: predict(x, names, tiles, r))
        top = min(rs, key=lambda r: r["us"])
        regrets.append(pick["us"] / top["us"])
        print(f"{shape:34s} model picks {pick['name']:18s} rc={pick['rc']:4d} {pick['us']:9.1f} us (predicted {predict(x, names, tiles, pick):9.1f}) | "
              f"best {top['name']:18s} rc={top['rc']:4d} {top['us']:9.1f} us | {pick['us'] / top['us']:.2f}")
    print(f"pick / best: mean {np.mean(regrets):.3f}, worst {np.max(regrets):.2f}")


if __name__ == "__main__":
    sys.exit(main())
