"""The five benchmark configurations at their full sizes, through the C ABI.

C1, C4 and C5 completely, and four of the 64 right matrices of C3, are compared with the CPU
oracle itself on the seeded inputs (a few seconds of its loop on 16 threads each); C2 on a band of
central output rows. Besides that, parity is established through properties that do not
depend on size:
  * integer-valued inputs: every product and partial sum is an exactly representable integer,
    so the result is independent of the summation order and must equal, bit for bit, the
    correlation computed with double-precision FFTs and rounded to the nearest integer (the FFT
    identity itself is checked against the oracle at a small size first);
  * real-valued seeded inputs: relative Frobenius error against the double-precision FFT
    result at most 1e-5 (fp32) / 1e-12 (fp64), the tolerances of the build's brief; the max
    element error is printed;
  * the all-ones closed form at the largest size;
  * a band of central output rows of the largest configuration against the oracle itself.
"""
import numpy as np
import pytest

from conftest import load_package

pytestmark = pytest.mark.gpu


def fft_xcorr(left, right):
    """Full cross-correlation of two equally sized matrices in double precision via FFT."""
    rows, cols = left.shape
    shape = (2 * rows - 1, 2 * cols - 1)
    f = np.fft.rfft2(left.astype(np.float64), shape) * np.fft.rfft2(right.astype(np.float64)[::-1, ::-1], shape)
    return np.fft.irfft2(f, shape)


def fft_reference(cfg, left, right, workloads):
    out = []
    for l, r, _ in workloads.pair_list(cfg):
        out.append(fft_xcorr(left[l], right[r]))
    return np.stack(out)


def device_order(cfg, right):
    """n_to_mn inputs are generated in file order; the one-launch entry point takes the right
    matrices grouped per left matrix."""
    if cfg["mode"] != "n_to_mn":
        return right, None
    n = cfg["n_left"]
    m = cfg["n_right"] // n
    slot = np.array([(i % n) * m + i // n for i in range(n * m)])
    grouped = np.empty_like(right)
    grouped[slot] = right
    return grouped, slot


def run_config(xc, cfg, left, right, family=None, params=None):
    n_left = cfg["n_left"]
    n_right = cfg["n_right"] // n_left if cfg["mode"] == "n_to_mn" else cfg["n_right"]
    right_dev, slot = device_order(cfg, right)
    pairs = cfg["n_left"] * cfg["n_right"] if cfg["mode"] == "n_to_m" else cfg["n_right"]
    got = xc.run(family or cfg["family"], left, right_dev, pairs, n_left=n_left, n_right=n_right,
                 params=xc.make_params(**(params if params is not None else cfg.get("params", {}))))
    return got if slot is None else got[slot]


def test_fft_identity_matches_oracle(oracle):
    rng = np.random.default_rng(0)
    a = rng.integers(-5, 6, size=(9, 14)).astype(np.float64)
    b = rng.integers(-5, 6, size=(9, 14)).astype(np.float64)
    np.testing.assert_array_equal(np.rint(fft_xcorr(a, b)), oracle.cross_corr(a, b))


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_integer_inputs_bit_exact_at_full_size(name):
    xc = load_package()
    from jpdc23_artifact_amd import workloads

    cfg = dict(workloads.CONFIGS[name])
    left, right = workloads.generate(cfg, integer_valued=True)
    print(name, cfg["mode"], left.shape, right.shape, flush=True)
    got = run_config(xc, cfg, left, right)
    exp = np.rint(fft_reference(cfg, left, right, workloads))
    assert np.abs(exp).max() < 2 ** 24
    print(name, xc.last_launch()["kernel"], "max |value|", np.abs(exp).max(), flush=True)
    np.testing.assert_array_equal(got, exp.astype(got.dtype))


@pytest.mark.parametrize("name,family", [
    ("C1", None), ("C1", "grouped_overlap"), ("C1", "split_row"), ("C2", None), ("C2", "split_row"),
    ("C3", None), ("C3", "multimat_right"), ("C4", None), ("C5", None), ("C5", "multimat_both"),
])
def test_seeded_inputs_within_tolerance_at_full_size(name, family):
    xc = load_package()
    from jpdc23_artifact_amd import workloads

    cfg = dict(workloads.CONFIGS[name])
    left, right = workloads.generate(cfg)
    if family in ("multimat_right", "multimat_both", "split_row"):
        params = dict(rows_per_thread=64, distribution_type="triangle")
    else:
        params = None if family is None else {}
    got = run_config(xc, cfg, left, right, family=family, params=params)
    exp = fft_reference(cfg, left, right, workloads)
    err = np.linalg.norm(got.astype(np.float64).ravel() - exp.ravel()) / np.linalg.norm(exp.ravel())
    max_abs = np.abs(got - exp).max()
    tol = 1e-5 if cfg["dtype"] == "float32" else 1e-12
    print(f"{name} {xc.last_launch()['kernel']}: rel_frobenius={err:.3e} max_abs={max_abs:.3e} max|ref|={np.abs(exp).max():.3e}", flush=True)
    assert np.isfinite(got).all()
    assert err <= tol


def oracle_full(oracle, cfg, left, right, threads=16):
    """The oracle's mode driver for a configuration (inputs and results in file order)."""
    fn = {"one_to_one": oracle.one_to_one, "one_to_many": oracle.one_to_many, "n_to_mn": oracle.n_to_mn, "n_to_m": oracle.n_to_m}[cfg["mode"]]
    return fn(left if cfg["mode"] not in ("one_to_one", "one_to_many") else left[0], right if cfg["mode"] != "one_to_one" else right[0],
              threads=threads)


@pytest.mark.parametrize("name,subset", [("C1", None), ("C3", 4), ("C4", None), ("C5", None)])
def test_seeded_inputs_against_the_oracle_at_full_size(oracle, name, subset):
    """The default launch of a configuration against the oracle's own loop on the same seeded inputs
    (the reference's host result, validate.hpp:94-132 and its mode drivers :216-298): relative Frobenius
    error at most 1e-5 (fp32) / 1e-12 (fp64) over ALL results, max element error printed. C3 costs the
    oracle 2.7e11 FMAs, so the GPU runs all 64 right matrices and four of them (first, two in the
    middle, last) are compared."""
    xc = load_package()
    from jpdc23_artifact_amd import workloads

    cfg = dict(workloads.CONFIGS[name])
    left, right = workloads.generate(cfg)
    print(name, cfg["mode"], left.shape, right.shape, flush=True)
    got = run_config(xc, cfg, left, right)
    kernel = xc.last_launch()["kernel"]
    if subset:
        picks = sorted({0, cfg["n_right"] // 3, (2 * cfg["n_right"]) // 3, cfg["n_right"] - 1})[:subset]
        exp = oracle.one_to_many(left[0], right[picks], threads=16)
        got = got[picks]
    else:
        exp = oracle_full(oracle, cfg, left, right)
    assert got.shape == exp.shape
    e = oracle.errors(got, exp)
    tol = 1e-5 if cfg["dtype"] == "float32" else 1e-12
    print(f"{name} {kernel} vs oracle: rel_frobenius={e.rel_frobenius:.3e} max_abs={e.max_abs:.3e} max_rel={e.max_rel:.3e} "
          f"max|ref|={np.abs(exp).max():.3e} ({exp.shape[0]} results)", flush=True)
    assert np.isfinite(got).all()
    assert e.rel_frobenius <= tol


def test_all_ones_closed_form_1024():
    xc = load_package()
    n = 1024
    ones = np.ones((n, n), dtype=np.float32)
    got = xc.run("grouped_overlap", ones, ones, 1)[0]
    o = np.arange(2 * n - 1)
    exp = np.outer(n - np.abs(o - (n - 1)), n - np.abs(o - (n - 1))).astype(np.float32)
    np.testing.assert_array_equal(got, exp)


def test_c2_band_against_oracle(oracle):
    """Sixteen central output rows of the 1024x1024 pair against the oracle.

    The reference's host loop adds ~10^6 positive products one by one in fp32; at the centre of
    this configuration that loses about 1.2e-4 relative to the exact sum (the fp64-accumulating
    variant of the same loop shows it). Three things are asserted:
      * the default launch, which splits the reduction into chunks of a few dozen left rows and
        therefore rounds less, is within 1e-5 of the exactly accumulated result;
      * the same entry point asked not to split into chunks (rows_per_thread >= rows) still adds
        the partial sums of its four row-sharing wavefronts, and stays within 2e-5 of the exact
        result;
      * the one-accumulator-per-output-element family (`shuffle`: every accumulator runs over the
        whole overlap like a thread of the reference's kernel does) reproduces the fp32 host loop
        itself to 1e-5.
    The default launch therefore MISSES the 1e-5 bar against the fp32 host loop on this configuration
    (about 1.0e-4); what is asserted about that distance is that it is explained by the host loop's own
    rounding: no larger than the loop's distance from the exact sum plus 1e-5.
    All pairwise differences are printed with their max element error."""
    xc = load_package()
    from jpdc23_artifact_amd import workloads

    cfg = dict(workloads.CONFIGS["C2"])
    left, right = workloads.generate(cfg)
    lo, hi = 1015, 1031
    ref32 = oracle.cross_corr(left[0], right[0], threads=16, row_begin=lo, row_end=hi)[lo:hi]
    ref64 = oracle.cross_corr(left[0], right[0], threads=16, row_begin=lo, row_end=hi, acc64=True)[lo:hi]
    o64 = oracle.errors(ref32, ref64)
    print(f"fp32 host loop vs fp64-accumulated: rel_frobenius={o64.rel_frobenius:.3e} max_abs={o64.max_abs:.3e}", flush=True)

    got = xc.run("grouped_overlap", left, right, 1)[0]
    rec = xc.last_launch()
    e32 = oracle.errors(got[lo:hi], ref32)
    e64 = oracle.errors(got[lo:hi], ref64)
    print(f"default ({rec['kernel']}, {rec['rows_per_worker']} rows per worker) vs fp32 host loop: "
          f"rel_frobenius={e32.rel_frobenius:.3e} max_abs={e32.max_abs:.3e} max_rel={e32.max_rel:.3e}", flush=True)
    print(f"default vs fp64-accumulated: rel_frobenius={e64.rel_frobenius:.3e} max_abs={e64.max_abs:.3e}", flush=True)
    assert e64.rel_frobenius <= 1e-5
    assert e32.rel_frobenius <= o64.rel_frobenius + 1e-5

    got = xc.run("grouped_overlap", left, right, 1, params=xc.make_params(rows_per_thread=1024))[0]
    rec = xc.last_launch()
    assert rec["uses_atomics"] == 0
    u32 = oracle.errors(got[lo:hi], ref32)
    u64 = oracle.errors(got[lo:hi], ref64)
    print(f"unsplit ({rec['kernel']}) vs fp32 host loop: rel_frobenius={u32.rel_frobenius:.3e} max_abs={u32.max_abs:.3e} "
          f"max_rel={u32.max_rel:.3e}", flush=True)
    print(f"unsplit vs fp64-accumulated: rel_frobenius={u64.rel_frobenius:.3e} max_abs={u64.max_abs:.3e}", flush=True)
    assert u64.rel_frobenius <= 2e-5

    got = xc.run("shuffle", left, right, 1, params=xc.make_params(distribution_type="none"))[0]  # "none": never split
    rec = xc.last_launch()
    assert rec["uses_atomics"] == 0
    s32 = oracle.errors(got[lo:hi], ref32)
    s64 = oracle.errors(got[lo:hi], ref64)
    print(f"one accumulator per element ({rec['kernel']}) vs fp32 host loop: rel_frobenius={s32.rel_frobenius:.3e} "
          f"max_abs={s32.max_abs:.3e} max_rel={s32.max_rel:.3e}", flush=True)
    print(f"one accumulator per element vs fp64-accumulated: rel_frobenius={s64.rel_frobenius:.3e} max_abs={s64.max_abs:.3e}", flush=True)
    assert s32.rel_frobenius <= 1e-5


def test_output_larger_than_2_32_elements(oracle):
    """n_to_m 130 x 128 matrices of 256x256 fp32: 16 640 results of 511x511 = 4.345e9 elements (17.4 GB), more than
    32-bit element indices reach (the reference's dsize_t is uint32, types.cuh:12; its largest published run, 128 x 128,
    stays 0.4 % below 2^32). Integer-valued inputs; the first, a middle and the last pairs - the last ones lie wholly
    beyond element 2^32 - must match the oracle exactly, and the centre element of every 1000th result must equal
    the plain dot product."""
    import ctypes

    xc = load_package()
    rng = np.random.default_rng(77)
    n_left, n, size = 130, 128, 256
    left = rng.integers(-2, 3, size=(n_left, size, size)).astype(np.float32)
    right = rng.integers(-2, 3, size=(n, size, size)).astype(np.float32)
    per = (2 * size - 1) ** 2
    total = n_left * n * per
    assert total > 2 ** 32
    d_left, d_right = xc.DeviceBuffer.from_numpy(left), xc.DeviceBuffer.from_numpy(right)
    d_out = xc.DeviceBuffer(total * 4)
    d_out.fill_bytes(0x7F)
    print("n_to_m 130x128 256x256 fp32, output bytes", total * 4, flush=True)
    xc.launch("multimat_both_grouped", d_left, d_right, d_out, size, size, n_left, n, np.float32, None)
    xc.sync()
    print(xc.last_launch(), flush=True)

    def fetch(pair):
        host = np.empty((2 * size - 1, 2 * size - 1), np.float32)
        src = ctypes.c_void_p(d_out.ptr.value + pair * per * 4)
        assert xc.lib().xcorr_memcpy_d2h(host.ctypes.data_as(ctypes.c_void_p), src, ctypes.c_size_t(host.nbytes)) == 0
        return host

    for l, r in [(0, 0), (61, 77), (128, 64), (128, 70), (129, 127)]:
        pair = l * n + r
        assert l < 128 or r == 64 or pair * per > 2 ** 32  # pair (128, 64) straddles element 2^32
        got = fetch(pair)
        exp = oracle.one_to_one(left[l], right[r], threads=8)[0]
        np.testing.assert_array_equal(got, exp, err_msg=f"pair {l},{r}")
    for pair in range(0, n_left * n, 1000):
        l, r = divmod(pair, n)
        centre = fetch(pair)[size - 1, size - 1]
        assert centre == float(np.sum(left[l].astype(np.float64) * right[r])), pair
    d_out.free()


@pytest.mark.parametrize("rows,cols,dtype,family", [(3000, 2500, np.float32, "grouped_overlap"),
                                                    (1537, 4099, np.float64, "grouped_overlap"),
                                                    (2049, 1023, np.float32, "split_row"),
                                                    (700, 9000, np.float32, "grouped_overlap")])
def test_large_non_square_pair_spot_checked(rows, cols, dtype, family):
    """Single pairs beyond the benchmark sizes (up to 7.5e6 elements per matrix, ragged against every tile and
    staging width): too large for the oracle's loop, so the corners, the centre and 300 random result elements
    are compared with the definition evaluated for that element alone (values in {-1, 0, 1}: every sum is exact)."""
    xc = load_package()
    rng = np.random.default_rng(5)
    left = rng.integers(-1, 2, (rows, cols)).astype(dtype)
    right = rng.integers(-1, 2, (rows, cols)).astype(dtype)
    print("case", family, rows, cols, np.dtype(dtype).name, flush=True)
    got = xc.run(family, left, right, 1)[0]
    points = [(0, 0), (2 * rows - 2, 2 * cols - 2), (rows - 1, cols - 1), (0, 2 * cols - 2), (2 * rows - 2, 0)]
    points += [(int(rng.integers(0, 2 * rows - 1)), int(rng.integers(0, 2 * cols - 1))) for _ in range(300)]
    for oy, ox in points:
        sy, sx = oy - (rows - 1), ox - (cols - 1)
        y0, y1 = max(0, -sy), min(rows, rows - sy)
        x0, x1 = max(0, -sx), min(cols, cols - sx)
        exp = float(np.sum(left[y0 + sy:y1 + sy, x0 + sx:x1 + sx].astype(np.float64) * right[y0:y1, x0:x1].astype(np.float64)))
        assert got[oy, ox] == exp, (oy, ox, got[oy, ox], exp, xc.last_launch()["kernel"])
