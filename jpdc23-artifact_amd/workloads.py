"""The five benchmark configurations and their seeded synthetic inputs.

The reference's input generator is unseeded (benchmark/input_generator.py:31-33:
numpy default_rng().random(), uniform [0,1)); here every configuration has a fixed
seed (1234 + configuration number) and one generator, numpy's PCG64
``default_rng(seed)``: the left array is drawn first, then the right array, row-major,
matrix after matrix, directly in the configuration's dtype.
"""
import numpy as np

CONFIGS = {
    "C1": dict(mode="one_to_one", dtype="float32", rows=64, cols=64, n_left=1, n_right=1, dist="uniform", seed=1235,
               family="grouped_overlap"),
    "C2": dict(mode="one_to_one", dtype="float32", rows=1024, cols=1024, n_left=1, n_right=1, dist="uniform", seed=1236,
               family="grouped_overlap"),
    "C3": dict(mode="one_to_many", dtype="float32", rows=256, cols=256, n_left=1, n_right=64, dist="uniform", seed=1237,
               family="multimat_right_grouped"),
    "C4": dict(mode="n_to_mn", dtype="float32", rows=128, cols=128, n_left=8, n_right=128, dist="normal", seed=1238,
               family="multimat_right_grouped"),
    "C5": dict(mode="n_to_m", dtype="float64", rows=64, cols=64, n_left=16, n_right=32, dist="normal", seed=1239,
               family="multimat_both_grouped"),
}


def num_pairs(cfg):
    if cfg["mode"] == "n_to_m":
        return cfg["n_left"] * cfg["n_right"]
    return cfg["n_right"]


def fma_count(cfg):
    """FMAs of the definition: (rows*cols)^2 per pair (sum over shifts of the overlap area)."""
    return num_pairs(cfg) * (cfg["rows"] * cfg["cols"]) ** 2


def algorithmic_bytes(cfg):
    """Inputs read once plus outputs written once."""
    item = np.dtype(cfg["dtype"]).itemsize
    area = cfg["rows"] * cfg["cols"]
    out_area = (2 * cfg["rows"] - 1) * (2 * cfg["cols"] - 1)
    return item * ((cfg["n_left"] + cfg["n_right"]) * area + num_pairs(cfg) * out_area)


def generate(cfg, integer_valued=False):
    """(left, right) arrays of shape (n, rows, cols). integer_valued draws small integers
    instead, so that every sum is exact in the configuration's dtype."""
    rng = np.random.default_rng(cfg["seed"])
    dtype = np.dtype(cfg["dtype"])
    shape_l = (cfg["n_left"], cfg["rows"], cfg["cols"])
    shape_r = (cfg["n_right"], cfg["rows"], cfg["cols"])
    if integer_valued:
        terms = cfg["rows"] * cfg["cols"]
        # keep |sum| < 2^24 (fp32) with room to spare
        amp = 1 if terms > 2 ** 18 else 3 if terms > 2 ** 14 else 8
        return (rng.integers(-amp, amp + 1, size=shape_l).astype(dtype),
                rng.integers(-amp, amp + 1, size=shape_r).astype(dtype))
    if cfg["dist"] == "uniform":
        return rng.random(shape_l, dtype=dtype), rng.random(shape_r, dtype=dtype)
    return rng.standard_normal(shape_l, dtype=dtype), rng.standard_normal(shape_r, dtype=dtype)


def pair_list(cfg):
    """(left index, right index, result index) of every pair, in the reference's order
    (validate.hpp:236-239, 264-269, 285-289). n_to_mn inputs are in file order here."""
    n, m = cfg["n_left"], cfg["n_right"]
    if cfg["mode"] == "one_to_one":
        return [(0, 0, 0)]
    if cfg["mode"] == "one_to_many":
        return [(0, i, i) for i in range(m)]
    if cfg["mode"] == "n_to_mn":
        return [(i % n, i, i) for i in range(m)]
    return [(l, r, l * m + r) for l in range(n) for r in range(m)]
