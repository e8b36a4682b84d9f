// Host-side planner and launcher of the sliding-window engine: picks a compiled
// specialisation for a request, decides how the reduction over left rows is split
// into work items, clears the output when it splits on its own, launches and
// records the geometry.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "engine_registry.hpp"

namespace xcorr {

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Workgroups per CU of every compiled kernel on an MI355X (256 CUs, 160 KB of LDS and 512 registers per lane and SIMD), as
// hipOccupancyMaxActiveBlocksPerMultiprocessor reports them there: what the planner assumes where it cannot ask a device
// (xcorr_plan_only without a GPU), so that it names the kernels an MI355X would run. A GPU test compares the table with the
// runtime's answers.
static const struct {
    const char *name;
    int blocks;
} occupancy_mi355x[] = {
    {"f32_a1b8", 6},
    {"f32_a1b8_r4", 4},
    {"f32_a1b8_l2r2", 4},
    {"f32_a8b4", 4},
    {"f32_a8b8", 4},
    {"f32_a4b4", 5},
    {"f32_a8b4_lr4", 4},
    {"f32_a8b8_lr4", 4},
    {"f32_a8b4_lr16", 3},
    {"f32_a8b8_lr16", 3},
    {"f32_a8b4_ll4lr4", 4},
    {"f32_a8b8_ll4lr4", 4},
    {"f32_a8b8_ll8lr8", 4},
    {"f32_a8b4_lr8", 3},
    {"f32_a8b4_ll4lr8", 3},
    {"f32_a4b4_lr4", 4},
    {"f32_a4b4_lr8", 4},
    {"f32_a1b4", 16},
    {"f32_a1b4_r4", 8},
    {"f32_a1b4_l2r2", 8},
    {"f32_a8b4_pairs8", 3},
    {"f32_m32x32", 5},
    {"f32_m64x32", 4},
    {"f32_m32x8_r4", 4},
    {"f32_m32x8_r8", 5},
    {"f32_m8x8_l4r4", 6},
    {"f32_m16x16_r4", 4},
    {"f32_m16x16_r8", 4},
    {"f32_m8x8_l4r8", 4},
    {"f32_m32x32_s16", 7},
    {"f32_m64x64_s16", 5},
    {"f32_m16x16_r4_s4", 6},
    {"f64_a1b8", 5},
    {"f64_a1b4_l2r2", 4},
    {"f64_a8b8", 2},
    {"f64_a4b4", 4},
    {"f64_a8b8_lr4", 2},
    {"f64_a8b8_lr16", 2},
    {"f64_a8b8_ll4lr4", 2},
    {"f64_a8b8_ll8lr8", 2},
    {"f64_a8b4_lr4", 3},
    {"f64_a8b4", 3},
    {"f64_a8b4_ll4lr4", 3},
    {"f64_a8b4_ll4lr8", 3},
    {"f64_a4b4_lr4", 4},
    {"f64_a4b4_lr8", 4},
    {"f64_a1b4", 14},
    {"f64_a1b4_l2r2_narrow", 8},
    {"f64_m32x32", 4},
    {"f64_m32x16", 4},
    {"f64_m32x8_r4", 4},
    {"f64_m8x8_l4r4", 4},
    {"f64_m32x32_s16", 4},
    {"f64_m16x16_r4_s4", 3},
};

int EngineSpec::resident_blocks() const {
    const int n = resident_blocks_of_device();
    if (n > 0) return n;
    for (const auto &e : occupancy_mi355x)
        if (strcmp(e.name, name) == 0) return e.blocks;
    return 1;
}

// Relative cost of running a request of the one-output-row families on one of their tiles
// (their wavefronts tile 2x2 or 1x2 over the shifts):
//   * work issued for partial overlaps at tile edges: a wavefront skips what cannot overlap its
//     own tile, but the wavefronts of a block wait for each other after every staged band, so both
//     the wavefront tile and the block tile count;
//   * lanes idling over matrices that do not exist;
//   * issue slots lost to LDS reads (a read plus the wait that guards it displace about four fp32
//     FMA slots, half as many fp64 ones: with that weight the tiles of 32 x shifts per wavefront win up
//     to 256x256 matrices and the ones of 64 from 512x512 on, as measured);
//   * several matrices per lane: the register ring of right rows grows, some spills.
static double spec_cost(const EngineSpec &s, const EngineRequest &rq) {
    double waste_x = std::sqrt((double)(rq.W + s.TXW()) * (rq.W + s.TXB())) / rq.W;
    double waste_y = std::sqrt((double)(rq.H + s.TYW()) * (rq.H + s.TYB())) / rq.H;
    int nu = rq.group_m > 0 ? rq.group_m : rq.nU;
    double util_v = (double)rq.nV / ((double)ceil_div(rq.nV, s.NVB()) * s.NVB());
    double util_u = (double)nu / ((double)ceil_div(nu, s.NUB()) * s.NUB());
    double cost = waste_x * waste_y / (util_v * util_u);
    int vk = 16 / s.elem_bytes;
    double reads = s.NV * ceil_div(s.B + s.K - 1, vk) + s.NU * (s.K / vk);
    double fmas = (double)s.NV * s.NU * s.A * s.B * s.K;
    cost *= 1.0 + (s.elem_bytes == 4 ? 4.0 : 2.0) * reads / fmas;
    if (s.NV * s.NU > 1) cost *= 1.15;
    return cost;
}

// How far a tile's value x is from a requested tuning integer r (0: not requested): nothing when it matches, the number
// of doublings above the request when the tile has more, and a large penalty when it has fewer (the nearest compiled
// value at or above the request is wanted; if none exists the largest below it).
static double request_distance(int x, unsigned r) {
    if (r == 0) return 0.0;
    return x >= (int)r ? std::log2((double)x / r) : 16.0 + std::log2((double)r / x);
}

// The reference's tuning integers, when given (non-zero), are exact requests: the tile must come as close as the compiled
// list allows to `y_shifts` adjacent y shifts per lane and to `right_mats` / `left_mats` matrices per lane position
// (matrices per lane x lanes laid over matrices). The distances add up; the sum is compared before any cost or run time.
struct RequestMatch {
    double d;
    bool better_than(const RequestMatch &o) const { return d < o.d; }
    bool same_as(const RequestMatch &o) const { return d == o.d; }
};
static RequestMatch match_request(const EngineSpec &s, const EngineRequest &rq) {
    // (the lanes a paired-groups tile lays over left matrices serve different pairs, not several left matrices per thread)
    return RequestMatch{(s.A > 1 ? request_distance(s.A, rq.y_shifts > 1 ? rq.y_shifts : 0) : 0.0) + request_distance(s.NUB(), rq.right_mats) +
                        (s.PG ? 0.0 : request_distance(s.NVB(), rq.left_mats))};
}

// Number of (y tile, chunk) workers when every y tile's rows are cut into chunks of rc rows.
static long count_chunks(const EngineSpec &s, int H, int nty, int rc, int *max_chunks) {
    long total = 0;
    int most = 0;
    for (int ty = 0; ty < nty; ++ty) {
        int syb = -(H - 1) + ty * s.TYB();
        int lo = syb > 0 ? syb : 0;
        int hi = syb + s.TYB() - 1 + H;
        if (hi > H) hi = H;
        int n = ceil_div(hi - lo, rc);
        if (n > most) most = n;
        total += n;
    }
    if (max_chunks) *max_chunks = most;
    return total;
}

// Fills the geometry of `plan` for specialisation `s` with the reduction over left rows cut into
// chunks of `rc` rows (rc <= 0 or rc >= H: not cut) and the reduction over right columns into `xc`
// chunks (whole shares of the block's wavefronts; ignored where the plan may not add atomically).
static int shape_plan(const EngineSpec &s, const EngineRequest &rq, int rc, int xc, EnginePlan &plan) {
    plan.spec = &s;
    plan.predicted_us = 0;
    plan.ordered = false;
    plan.x_chunks = 1;
    plan.x_chunk_cols = rq.W;
    if (xc > 1 && (rq.may_split || rq.caller_zeroes)) {
        const int granule = s.K * s.WZ;
        const int cw = ceil_div(ceil_div(rq.W, xc), granule) * granule;
        plan.x_chunks = ceil_div(rq.W, cw);
        plan.x_chunk_cols = cw;
    }
    const int Sx = 2 * rq.W - 1, Sy = 2 * rq.H - 1;
    plan.ntx = ceil_div(Sx, s.TXB());
    plan.nty = ceil_div(Sy, s.TYB());
    plan.nvg = ceil_div(rq.nV, s.NVB());
    plan.nug = ceil_div(rq.group_m > 0 ? rq.group_m : rq.nU, s.NUB());
    int dist = rq.dist == XCORR_DIST_NONE ? 0 : rq.dist == XCORR_DIST_RECTANGLE ? 1 : rq.dist == XCORR_DIST_TRIANGLE ? 2 : -1;
    if (rq.caller_zeroes) {
        // split-row contract (reference one_to_one.hpp:276-288): zeroed output, atomics
        if (dist < 0) dist = 1; // the reference's default is "rectangle" (one_to_one.hpp:232)
        if (rc <= 0) rc = s.RL;
        if (dist == 0) rc = rq.H;
        plan.atomic = 1;
        plan.zero_fill = false;
        if (rc >= rq.H && plan.x_chunks == 1) {
            // one work item per result tile: plain stores leave in a zeroed output what the atomic adds would (and need no
            // zeroed output: a caller that looks at the record of a planning call first may skip its clear)
            dist = 0;
            plan.atomic = 0;
        }
    } else if ((rc <= 0 || rc >= rq.H || !rq.may_split) && plan.x_chunks == 1) {
        rc = rq.H;
        dist = 0;
        plan.atomic = 0;
        plan.zero_fill = false;
    } else if (rc <= 0 || rc >= rq.H) {
        rc = rq.H;
        dist = 0;
        plan.atomic = 1;
        plan.zero_fill = true;
    } else if (rq.ordered && plan.x_chunks == 1) {
        dist = 3;
        plan.atomic = 0;
        plan.zero_fill = false;
        plan.ordered = true;
    } else {
        if (dist <= 0) dist = 2;
        plan.atomic = 1;
        plan.zero_fill = true;
    }
    if (rc > rq.H) rc = rq.H;
    plan.rows_per_chunk = rc;
    plan.dist = dist;

    // workers along y: (y tile, chunk) pairs
    int max_chunks = 0;
    long total_chunks = count_chunks(s, rq.H, plan.nty, rc, &max_chunks);
    if (dist == 0)
        plan.nworkers_y = plan.nty;
    else if (dist == 1)
        plan.nworkers_y = plan.nty * max_chunks;
    else
        plan.nworkers_y = (int)total_chunks;
    long items = (long)plan.nvg * plan.nug * plan.nworkers_y * plan.ntx * plan.x_chunks;
    if (items <= 0 || items > 0x7fffffffL) return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: %ld work items are out of range", rq.family, items);
    plan.total_items = (int)items;
    plan.grid = (unsigned)items;
    return XCORR_OK;
}

// Predicted run time in microseconds of a grouped-tile plan. The launch is seen as `items` blocks
// of four wavefronts (one per SIMD) of which a CU holds `occ` at a time:
//   * a block issues A*B FMAs per lane for every (right row, right column) its shift tile overlaps;
//     a chunk of rc left rows meets rc + A - 1 right rows, so short chunks pay for the window;
//   * with many blocks the run is bound by the issue rate of the CUs (average block), with few by
//     the largest block (the centre tile, all rows and columns) at the issue rate the few wavefronts
//     of a SIMD reach together (one alone: 0.6 of what four reach);
//     the two regimes blend: issue-bound time of all blocks plus a share of the largest block's time;
//   * every block costs a fixed prologue / epilogue and every staged band a little; a split plan
//     pays the clear kernel and the atomic adds of all blocks at the rate the memory system takes
//     them (lower when the lanes of a wavefront write to different result matrices).
// The constants were fitted to sweeps of all grouped tiles and chunk sizes over 16x16 ... 1024x1024
// matrices and 1 ... 1024 pairs on MI355X (weighted least squares on the logarithm of the run time);
// `issue_factor` and `stage_factor` are per tile.
static double predict_us(const EngineSpec &s, const EngineRequest &rq, const EnginePlan &plan) {
    // (a matrix-core tile lays matrices over the rows and columns of its result tiles: its atomic adds scatter like those of
    // lanes over matrices; it has no window of A right rows to fill before a chunk's first row)
    const bool f32 = s.elem_bytes == 4, lanes_over_matrices = s.MFMA ? s.NVB() * s.NUB() > 1 : s.LV * s.LU > 1;
    const int window = s.MFMA ? 0 : s.A - 1;
    // A matrix-core tile whose columns hold copies of the x shifts some rows apart (TYB > TYW) sweeps the left rows of its first copy,
    // from `copies` rows before a chunk's first row on: as many as its shifts overlap when whole (up to `copies` more for the tiles
    // around y shift 0), `copies` more than the chunk when cut.
    const int copies = s.MFMA ? s.TYB() - s.TYW() : 0;
    // (two sets of constants: the register-tile kernel, one block per work item, and the matrix-core kernel, whose persistent blocks
    // overlap the atomic adds and stores of one item with the next: fitted to 3 000 launches of its tiles - every chunk size of the
    // ladder on 85 shapes of 16x16 ... 1024x1024 matrices, 1 ... 40 000 pairs, both element types - to 8 % (rms of the logarithm);
    // the plan it picks is within 3 % of the best measured one on average, 16 % at worst)
    const bool mm = s.MFMA != 0;
    const double t_block = mm ? 5.46 : 4.41, tau = mm ? 0.686 : 1.07, e_full = 0.954, t_stage = mm ? 0.0 : 0.209, k_tail = mm ? 0.50 : 0.281;
    const double t_clear = f32 ? (mm ? 1.42 : 1.49) : 0.0, t_atomic = f32 ? (mm ? 0.0094 : 0.0462) : (mm ? 0.194 : 0.0811);
    const double us_per_atomic = mm ? (lanes_over_matrices ? (f32 ? 1.98e-6 : 3.06e-6) : (f32 ? 2.37e-6 : 1.51e-6))
                                    : lanes_over_matrices ? (f32 ? 4.5e-6 : 3.0e-6) : (f32 ? 1.6e-6 : 4.4e-6);
    const double cyc = (f32 ? 2.0 : 4.0) / 2100.0; // microseconds per FMA instruction of a wavefront
    // (a tile-by-tile sweep pays the edge zeros of one result tile, not of the block tile)
    const double W = rq.W, H = rq.H, TXW = s.fine_x ? s.fine_x : s.TXB(), TYW = s.fine_y ? s.fine_y : s.TYB();
    const double ntx = (double)plan.ntx * s.TXB() / TXW, nty = (double)plan.nty * s.TYB() / TYW;
    const bool split = plan.atomic != 0 || plan.ordered;
    const double rc = plan.rows_per_chunk;
    // a tile overlaps cols_tile right columns on average; cut into chunks, ceil(cols_tile / chunk) of its
    // x_chunks work items find columns, the others return at once
    const double cols_tile = std::fmin(W, W * (W + TXW) / (ntx * TXW));
    const double live = plan.x_chunks > 1 ? std::fmin(plan.x_chunks, std::ceil(cols_tile / plan.x_chunk_cols)) : 1.0;
    const double cols_avg = cols_tile / live, cols_max = plan.x_chunks > 1 ? std::fmin(W, plan.x_chunk_cols) : W;
    const double rows_tile = std::fmin(H, H * (H + TYW) / (nty * TYW));
    const double rows_avg = (split && rc < rows_tile ? rc + copies : rows_tile) + window;
    const double rows_max = (split && rc < H ? rc + copies : H + 0.5 * copies) + window;
    const double per_element = (double)s.NV * s.NU * s.A * s.B / s.WZ * s.issue_factor;
    const double inst_avg = per_element * rows_avg * cols_avg, inst_max = per_element * rows_max * cols_max;
    const double stages_avg = std::ceil(rows_avg / s.RL) * std::ceil((cols_avg + TXW) / s.KBX) * s.stage_factor;
    const double stages_max = std::ceil(rows_max / s.RL) * std::ceil((cols_max + TXW) / s.KBX) * s.stage_factor;
    const double items = plan.total_items * live / plan.x_chunks;
    const int cus = device_cus(), occ = s.resident_blocks();
    double n1 = std::ceil(items / cus);
    if (n1 > occ) n1 = occ;
    const double fixed = t_block + (split && !lanes_over_matrices ? t_atomic * s.NV * s.NU * s.A * s.B : 0.0);
    // n1 blocks on a CU (one wavefront each per SIMD) issue together at e_full * (1 - exp(-n1 / tau)) of the FMA rate
    const double crit = fixed + t_stage * stages_max + n1 * inst_max * cyc / (e_full * (1.0 - std::exp(-n1 / tau)));
    const double per_block = (fixed + t_stage * stages_avg) / n1 + inst_avg * cyc / e_full;
    const double tail = k_tail * crit;
    double t = std::fmax(items * per_block / cus + tail, crit);
    if (s.MFMA) {
        // The matrix-core kernel runs `slots` persistent blocks that take the items in launch order, heaviest first: the launch
        // is a number of full rounds of items that share their CU with occ - 1 others, a last, partly filled round of small items
        // with fewer neighbours, and the difference between the first round's items and the average ones.
        const double k_last = 0.82;
        auto item_time = [&](double inst, double stages, double n) {
            return fixed + t_stage * stages + n * inst * cyc / (e_full * (1.0 - std::exp(-n / tau)));
        };
        const double slots = (double)cus * occ;
        if (items <= slots) {
            t = item_time(inst_max, stages_max, n1);
        } else {
            const double full = std::floor(items / slots), rest = items - full * slots;
            const double n_last = std::fmax(1.0, std::fmin((double)occ, std::ceil(rest / cus)));
            t = full * item_time(inst_avg, stages_avg, occ) + (rest > 0 ? item_time(inst_avg * k_last, stages_avg, n_last) : 0.0) +
                k_tail * (item_time(inst_max, stages_max, occ) - item_time(inst_avg, stages_avg, occ));
        }
    }
    // (chunks that add themselves in order: a read and a write of the tile through to memory per item, as an atomic add is)
    if (split) t += (plan.ordered ? 0.0 : t_clear) + items * 64.0 * s.NV * s.NU * s.A * s.B * us_per_atomic;
    // Sustained vector-FMA load pulls the power-managed shader clock from 2.35 to 2.0-2.1 GHz within the first milliseconds
    // of a launch (random operands); the matrix cores hold 2.35 GHz on the same data. Measured / predicted run time of the
    // register tiles is 1.0 below half a millisecond and 1.3 from five milliseconds on, of the matrix-core tiles 1.1
    // throughout: the register tiles pay the difference, phased in over a decade of run time.
    if (!s.MFMA && t > 500.0) t *= 1.0 + 0.18 * std::fmin(1.0, std::log10(t / 500.0));
    {
        // No launch is faster than its multiply instructions. A wavefront of a matrix-core block owns one SIMD's matrix pipeline, 2 (fp64: 4)
        // cycles per accumulator element and multiplied element pair, the clock holds 2.35 GHz under that kernel and the pipelines measured busy
        // 0.94 of the time at best (0.92 with the 32-cycle instruction of the tile-by-tile sweeps); the vector-FMA tiles issue in 0.86-0.89 of the
        // cycles at the 2.0-2.1 GHz their load pulls the clock to: 0.75 of the rate at 2.4 GHz for the A8xB4 tile, the others in proportion to
        // their issue factors. The fitted terms above are up to 20 % below this bound where many equal items keep every CU in its sweep (C2,
        // thousands of pairs from 128x128 on, pairs of 4096x4096 and more).
        const double best_rate = s.MFMA ? (s.fine_x ? 0.93 : 0.95) * 2350.0 / 2400.0 : 0.75 * (f32 ? 0.713 : 0.676) / s.issue_factor;
        const double multiplies = (double)s.NV * s.NU * s.A * s.B / s.WZ * (rows_avg - window) * cols_avg; // per wavefront of an average item
        // (plans at the bound still differ by what the fitted terms see - chunk sizes, atomic adds -: a small share of them keeps their order)
        const double bound = items * multiplies * (f32 ? 2.0 : 4.0) / 2400.0 / cus / best_rate + (split ? (plan.ordered ? 0.0 : t_clear) : 0.0);
        if (bound > t) t = bound + 0.03 * t;
    }
    return t;
}

// Grouped families: every compatible tile is tried with the reduction uncut and cut into 2, 3, 4, 6 ...
// groups of G = A + 1 rows (the granule of the inner loop); the plan with the shortest predicted
// run time wins among the tiles that match the reference's tuning integers best (match_request; all tiles when none is given).
static int plan_grouped(const EngineRequest &rq, const EngineSpec *specs, int count, EnginePlan &plan) {
    static const int ladder[] = {0, 2, 3, 4, 6, 8, 12, 16, 24, 32};
    bool found = false;
    double best = 0;
    int candidate_error = XCORR_OK;
    RequestMatch best_match = {};
    for (int i = 0; i < count; ++i) {
        const EngineSpec &s = specs[i];
        if (rq.spec_index > 0 ? i != (int)rq.spec_index - 1 : s.A == 1) continue;
        if (rq.group_m > 0 ? (s.NVB() != 1 && !s.PG) : s.PG != 0) continue; // lanes over left matrices: all pairs, or paired groups
        if (rq.ordered && !s.MFMA) continue;
        if (rq.spec_index == 0) {
            if (rq.matrix_cores == 1 ? !s.MFMA : rq.matrix_cores == 2 ? s.MFMA != 0 : false) continue;
            // The tiles whose columns hold copies of the x shifts win up to about 256x256 matrices (2-7 % over their 32 x 8
            // counterparts) and measured level at 300x300, 3-14 % behind at 384x384 ... 1024x1024, which the model does not show.
            if (s.MFMA && s.TYB() != s.TYW() && (double)rq.W * rq.H > 300.0 * 300.0) continue;
            // The tile-by-tile sweep is the launcher's own choice (a request for y shifts per thread means the tiles that had them
            // before), for matrices of 17 ... 300 rows and columns: on 16x16 the four-shift register tile is ahead (30 against 36 us
            // for 4000 pairs), one pair of 512x512 runs 8 % slower than on the 32 x 32 tile (its edge is a small share there, and
            // the smaller instruction issues twice as often), 1024x1024 level.
            if (s.fine_y && (rq.y_shifts > 1 || (rq.W <= 16 && rq.H <= 16) || (double)rq.W * rq.H > 300.0 * 300.0)) continue;
            if (rq.x_shifts && (unsigned)s.B != rq.x_shifts) continue;
            if (rq.lanes_x && (unsigned)s.LX != rq.lanes_x) continue;
            if (rq.lanes_y && (unsigned)s.LY != rq.lanes_y) continue;
        }
        // Tiny matrices: the run-time model was fitted from 16x16 up but ranks the eight-shift tiles too well at its
        // lower end; measured on 4000 ... 16384 pairs, the four-shift tiles are 1.25-1.7x faster on 16x16 matrices and,
        // where one left matrix meets many right ones, 1.1x on 32x32.
        const int longest = rq.W > rq.H ? rq.W : rq.H;
        const bool no_request = rq.spec_index == 0 && rq.y_shifts == 0 && rq.left_mats <= 1 && rq.right_mats == 0 && rq.x_shifts == 0 &&
                                rq.lanes_x == 0 && rq.lanes_y == 0;
        if (no_request && s.A > 4 && !s.fine_x && (longest <= (s.PG ? 16 : 24) || (longest <= 32 && !s.PG && (rq.group_m > 0 || rq.nV == 1)))) continue;
        const RequestMatch match = match_request(s, rq);
        if (found && best_match.better_than(match)) continue;
        const int G = s.MFMA ? 8 : s.A + 1; // granule of the chunk sizes tried
        const bool matrices_in_tile = s.MFMA ? s.NVB() * s.NUB() > 1 : s.LV * s.LU > 1;
        for (int k : ladder) {
            // (chunks of rows leave the trimming of a tile's rows nothing to save: one pair of 256x256 in chunks of 32 rows measured 8 %
            // slower than on the 32 x 32 tile)
            if (k != 0 && s.fine_y && rq.rows_per_worker == 0) break;
            int rc = k * G;
            if (rq.rows_per_worker > 0) {
                if (k != 0) break;
                rc = (int)rq.rows_per_worker;
            } else if (rq.caller_zeroes) {
                // zeroed output, atomic adds, no chunk named: whole rows (k = 0) or any chunk of the ladder
                if (k == 0) rc = rq.H;
                if (k != 0 && (rc >= rq.H || rq.dist == XCORR_DIST_NONE)) break;
            } else if (k != 0 && (!rq.may_split || rc >= rq.H)) {
                break;
            } else if (k != 0 && !s.MFMA && matrices_in_tile && (rc < 36 || rq.H < 72)) {
                continue; // measured: short chunks of register tiles whose lanes lie over matrices lose to their scattered atomic adds
            }
            EnginePlan cand;
            if (int e = shape_plan(s, rq, rc, (int)rq.column_chunks, cand)) {
                // (more work items than the launch arithmetic holds, e.g. short chunks of a 16384x16384 pair: another candidate will do)
                candidate_error = e;
                continue;
            }
            const double t = predict_us(s, rq, cand);
            if (!found || match.better_than(best_match) || t < best) {
                found = true;
                best = t;
                best_match = match;
                plan = cand;
                plan.predicted_us = t;
            }
        }
    }
    if (!found && candidate_error != XCORR_OK) return candidate_error; // (its message is the last error text)
    if (!found)
        return fail(XCORR_ERR_UNSUPPORTED, "%s: no compiled specialisation matches x_shifts_per_thread=%u lanes_x=%u lanes_y=%u",
                    rq.family, rq.x_shifts, rq.lanes_x, rq.lanes_y);
    // A split plan that still leaves CUs without a block (a single pair of 32x32 ... 64x64 matrices) also cuts the
    // reduction over right columns in two: measured 12-20 % faster there, slower as soon as every CU has a block
    // (the model above was not fitted for column chunks and is not asked).
    if (rq.column_chunks == 0 && plan.zero_fill && plan.spec->LV * plan.spec->LU == 1 && !plan.spec->MFMA && plan.total_items < device_cus() && rq.W >= 32) {
        EnginePlan cut;
        if (int e = shape_plan(*plan.spec, rq, plan.rows_per_chunk, 2, cut)) return e;
        plan = cut;
    }
    return XCORR_OK;
}

int plan_engine(const EngineRequest &rq, EnginePlan &plan) {
    int count = 0;
    const EngineSpec *specs = rq.elem_bytes == 4 ? engine_specs_f32(&count) : engine_specs_f64(&count);
    if (rq.matrix_cores > 2) return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: matrix_cores must be 0, 1 or 2, not %u", rq.family, rq.matrix_cores);
    if (rq.spec_index > (unsigned)count)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: specialisation %u does not exist (%d compiled)", rq.family, rq.spec_index, count);
    if (rq.spec_index > 0 && rq.group_m <= 0 && specs[rq.spec_index - 1].PG)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: specialisation %s pairs every left matrix with its own group only", rq.family,
                    specs[rq.spec_index - 1].name);
    if (rq.spec_index > 0 && rq.group_m > 0 && specs[rq.spec_index - 1].NVB() != 1 && !specs[rq.spec_index - 1].PG)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: specialisation %s cannot pair one left matrix with a group", rq.family,
                    specs[rq.spec_index - 1].name);
    const bool grouped = rq.spec_index > 0 ? specs[rq.spec_index - 1].A > 1 : rq.y_shifts != 1;
    if (grouped) return plan_grouped(rq, specs, count, plan);

    // The one-output-row families are contracts (who clears the output, how the rows are dealt to workers), not kernels:
    // where the caller names no tile geometry, a matrix-core tile serves them under the same contract (its work items
    // take the caller's rows per worker and distribution like any other tile's). Measured against the one-row tiles
    // (fp32, 16x16 ... 1024x1024, 1 ... 1024 pairs): 1.2-4.9x faster from 64x64 on and from eight pairs of 32x32 on,
    // 0.8-1.0x below; taken from 8192 elements per launch on (pairs x rows x columns), for a single pair from 64x64 on
    // (fp64: from 32x32 matrices on).
    const bool no_tile_asked = rq.spec_index == 0 && rq.x_shifts == 0 && rq.lanes_x == 0 && rq.lanes_y == 0 && rq.left_mats <= 1 && rq.right_mats <= 1;
    const double pair_count = rq.group_m > 0 ? (double)rq.nU : (double)rq.nV * rq.nU;
    const double elements = pair_count * rq.W * rq.H;
    const double area = (double)rq.W * rq.H;
    // (fp64: measured 1.1-1.5x faster already on 32x32 matrices, 1.5-5.4x beyond)
    const bool large_enough = rq.elem_bytes == 8 ? area >= 1024.0 : pair_count >= 2.0 ? elements >= 8192.0 : area >= 4096.0;
    // (a caller who fixes short chunks of rows wants the reference's work distribution: left to the one-row tiles)
    const bool chunk_fits = rq.rows_per_worker == 0 || rq.rows_per_worker >= 16 || rq.dist == XCORR_DIST_NONE; // ("none": the chunk is not used)
    // (a plain launcher told to keep the rows whole promises the summation order of one pass over the rows, which is what
    // brings the large fp32 pair within 1e-5 of the reference's fp32 host loop: the one-row tiles keep it)
    const bool order_free = rq.may_split || rq.caller_zeroes;
    if (no_tile_asked && (rq.matrix_cores == 1 || (rq.matrix_cores == 0 && large_enough && chunk_fits && order_free))) {
        EngineRequest q = rq;
        q.y_shifts = q.left_mats = q.right_mats = 0;
        q.matrix_cores = 1;
        // The work items of a matrix-core tile are always dealt tile by tile ("triangle"): the "rectangle" of the reference -
        // as many workers per tile as the tallest tile needs, the surplus idle - measured 1.6-1.9x slower with these tiles
        // (512x512 split-row: 2061 against 1128 us) in either enumeration order. Like the tuning integers, the name is a
        // request that is mapped onto what exists; the launch record tells.
        if (q.caller_zeroes && q.dist != XCORR_DIST_NONE) q.dist = XCORR_DIST_TRIANGLE;
        return plan_grouped(q, specs, count, plan);
    }

    // one-output-row families: relative cost of the tile, then the split rule below
    const EngineSpec *best = rq.spec_index > 0 ? &specs[rq.spec_index - 1] : nullptr;
    double best_cost = 0;
    RequestMatch best_match = {};
    // Several matrices per lane reuse every staged left value, but make a quarter as many work items four times as long:
    // measured (fp32, 1 x 8 ... 1 x 256 and 2 x 2 ... 32 x 32 matrices of 16x16 ... 256x256) the one-matrix tiles win up to
    // about 3e9 multiply-adds per launch (by 1.2-1.5x on the smallest), the others beyond; a request for matrices per
    // thread overrides this.
    const double pairs = pair_count;
    const bool one_matrix_per_lane = rq.left_mats <= 1 && rq.right_mats == 0 && pairs * area * area < 3e9;
    for (int i = 0; i < count && rq.spec_index == 0; ++i) {
        const EngineSpec &s = specs[i];
        if (s.A != 1) continue;
        if (one_matrix_per_lane && s.NV * s.NU > 1) continue;
        if (rq.group_m > 0 ? (s.NVB() != 1 && !s.PG) : s.PG != 0) continue; // lanes over left matrices: all pairs, or paired groups
        if (rq.x_shifts && (unsigned)s.B != rq.x_shifts) continue;
        if (rq.lanes_x && (unsigned)s.LX != rq.lanes_x) continue;
        if (rq.lanes_y && (unsigned)s.LY != rq.lanes_y) continue;
        const double c = spec_cost(s, rq);
        const RequestMatch match = match_request(s, rq);
        if (!best || match.better_than(best_match) || (match.same_as(best_match) && c < best_cost)) {
            best = &s;
            best_cost = c;
            best_match = match;
        }
    }
    if (!best)
        return fail(XCORR_ERR_UNSUPPORTED, "%s: no compiled specialisation matches x_shifts_per_thread=%u lanes_x=%u lanes_y=%u",
                    rq.family, rq.x_shifts, rq.lanes_x, rq.lanes_y);
    int rc = (int)rq.rows_per_worker;
    const bool split_by_default = rq.caller_zeroes ? rq.dist != XCORR_DIST_NONE : rq.may_split;
    if (rc <= 0 && split_by_default) {
        // No chunk size from the caller: the chunk with the lowest relative cost
        //     (1 + 1300 / (average rows of a work item x columns)) x (1 + 6.7 x CUs / work items).
        // The first factor is what a work item pays around its sweep (ring start-up, atomic adds of its tile), the second
        // how badly few items balance over the device; together they put the best number of work items near
        // sqrt(1.3 x CUs x rows of all tiles x columns). Fitted to measured split-row, multimat-right and multimat-both
        // launches of 16x16 ... 512x512 fp32 matrices, 1 ... 1024 pairs (3-5 rows for a single pair up to 96x96, 8-16 rows
        // around 128x128 ... 512x512, whole matrices when the pairs alone fill the device).
        EnginePlan whole;
        if (int e = shape_plan(*best, rq, 0, 1, whole)) return e;
        const double per_tile_column = (double)whole.ntx * whole.nvg * whole.nug;
        const double rows_of_all_tiles = per_tile_column * count_chunks(*best, rq.H, whole.nty, 1, nullptr);
        auto chunk_cost = [&](int c) {
            const double items = per_tile_column * count_chunks(*best, rq.H, whole.nty, c, nullptr);
            return (1.0 + 1300.0 / (rows_of_all_tiles / items * rq.W)) * (1.0 + 6.7 * device_cus() / items);
        };
        const int candidates[] = {3, 5, 8, 16, 32, 64, rq.H};
        double best_chunk_cost = 0;
        for (int c : candidates) {
            if (c > rq.H) continue;
            const double cost = chunk_cost(c);
            if (rc <= 0 || cost < best_chunk_cost) {
                rc = c;
                best_chunk_cost = cost;
            }
        }
        // A launcher whose contract is a plain store (no zeroed output, the same bits every run, the summation order of
        // one pass over the rows) and whose whole tiles already give every CU two work items only gives that up for a
        // predicted gain of 1.4 x or more.
        if (!rq.caller_zeroes && whole.total_items >= 2L * device_cus() && best_chunk_cost > 0.7 * chunk_cost(rq.H)) rc = rq.H;
    }
    int xc = (int)rq.column_chunks;
    if (xc == 0 && rq.caller_zeroes && rq.dist == XCORR_DIST_NONE) {
        // The split-row contract (zeroed output, atomic adds) with the rows explicitly left whole: when that gives the
        // device less than two work items per CU the reduction over right columns is cut instead, into chunks of at
        // least 16 columns.
        EnginePlan whole;
        if (int e = shape_plan(*best, rq, rc, 1, whole)) return e;
        if (whole.total_items < 2L * device_cus()) {
            xc = ceil_div(2 * device_cus(), whole.total_items);
            if (xc > rq.W / 16) xc = rq.W / 16;
        }
    }
    return shape_plan(*best, rq, rc, xc > 1 ? xc : 1, plan);
}

// ---- scratch of the launches that add the chunks of a split reduction in order ----
// One ticket (32 bits) per result tile of the launch, in a fixed array that belongs to the library's code object: nothing is
// allocated. Every device that runs the library holds its own copy until the process ends; its address there is asked of the
// runtime once per device (the array's name is a host-side stand-in, not a device address). All launches on a device share the
// array: ordered launches that overlap in time on one device race for it.
constexpr size_t SCRATCH_WORDS = 1u << 20; // 4 MiB: a single pair of up to 16384 x 16384 elements in tiles of 32 x 32 shifts
static __device__ __align__(256) unsigned scratch[SCRATCH_WORDS];

static unsigned *scratch_of_device() {
    static unsigned *address[MAX_DEVICES] = {};
    static std::mutex lock;
    std::lock_guard<std::mutex> guard(lock);
    const int dev = current_device();
    if (address[dev] == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        address[dev] = static_cast<unsigned *>(p);
    }
    return address[dev];
}
size_t ordered_scratch_tiles() { return SCRATCH_WORDS; }

// ---- work queues of persistent launches ----
// A persistent launch (matrix-core sweep, more work items than the device holds blocks) hands out its work items through a
// counter in device memory. Launches on one stream run one after the other, so every stream gets a counter pair of its own, in
// a fixed array that belongs to the library's code object (nothing is allocated); a kernel leaves its pair zeroed. Streams
// that cannot be told apart by their handle (the per-thread default stream) or that are being captured into a graph - whose
// replays may run beside anything - get no queue: such launches run one block per work item.
constexpr int QUEUE_SLOTS = 64, QUEUES = 8, QUEUE_STRIDE = 32 * QUEUES; // per stream: eight counter pairs, 128 bytes apart
static __device__ __align__(256) unsigned launch_queues[QUEUE_SLOTS * QUEUE_STRIDE];

struct QueueTable {
    std::mutex lock;
    unsigned *base[MAX_DEVICES] = {};
    hipStream_t owner[MAX_DEVICES][QUEUE_SLOTS] = {};
    int used[MAX_DEVICES] = {};
};
static QueueTable &queue_table() {
    static QueueTable t;
    return t;
}

// The queue of `stream` on the current device, or nullptr if it can have none. Call with the table locked, and keep it locked
// until the launch that uses the queue has been enqueued (an idle stream's slot may be given to another stream).
static unsigned *queue_for(hipStream_t stream) {
    if (stream == hipStreamPerThread) return nullptr;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    QueueTable &t = queue_table();
    const int dev = current_device();
    if (t.base[dev] == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(launch_queues)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        t.base[dev] = static_cast<unsigned *>(p);
    }
    for (int i = 0; i < t.used[dev]; ++i)
        if (t.owner[dev][i] == stream) return t.base[dev] + (size_t)i * QUEUE_STRIDE;
    if (t.used[dev] < QUEUE_SLOTS) {
        t.owner[dev][t.used[dev]] = stream;
        return t.base[dev] + (size_t)(t.used[dev]++) * QUEUE_STRIDE;
    }
    // all slots taken: one whose stream has no work in flight (or no longer exists) can change hands
    for (int i = 0; i < QUEUE_SLOTS; ++i)
        if (hipStreamQuery(t.owner[dev][i]) != hipErrorNotReady) {
            (void)hipGetLastError();
            t.owner[dev][i] = stream;
            return t.base[dev] + (size_t)i * QUEUE_STRIDE;
        }
    return nullptr;
}

template <typename T>
static int launch_typed(const EngineRequest &rq, const EnginePlan &plan, hipStream_t stream) {
    EngineArgs<T> a;
    a.V = static_cast<const T *>(rq.V);
    a.U = static_cast<const T *>(rq.U);
    a.out = static_cast<T *>(rq.out);
    a.W = rq.W;
    a.H = rq.H;
    a.nV = rq.nV;
    a.nU = rq.nU;
    a.group_m = rq.group_m;
    a.rows_per_chunk = plan.rows_per_chunk;
    a.dist = plan.dist;
    a.atomic = plan.atomic;
    a.ntx = plan.ntx;
    a.nty = plan.nty;
    a.nworkers_y = plan.nworkers_y;
    a.nvg = plan.nvg;
    a.nug = plan.nug;
    a.total_items = plan.total_items;
    a.x_chunks = plan.x_chunks;
    a.x_chunk_cols = plan.x_chunk_cols;
    a.queue = nullptr;
    a.queues = 1;
    a.tickets = nullptr;
    if (plan.ordered) {
        const size_t tiles = (size_t)plan.nvg * plan.nug * plan.ntx * plan.nty;
        unsigned *tickets = scratch_of_device();
        if (tickets == nullptr) return fail(XCORR_ERR_RUNTIME, "%s: the library's scratch array is not reachable on this device", rq.family);
        if (tiles > SCRATCH_WORDS) return fail(XCORR_ERR_UNSUPPORTED, "%s: %zu result tiles need more tickets than the scratch array holds (%zu)", rq.family, tiles, SCRATCH_WORDS);
        // (a kernel, not a memset: the launch may be captured into a graph)
        zero_fill_kernel<unsigned><<<dim3((unsigned)((tiles + 255) / 256)), dim3(256), 0, stream>>>(tickets, tiles);
        XCORR_HIP(hipGetLastError());
        a.tickets = tickets;
    }
    if (plan.zero_fill) {
        size_t n = (size_t)(2 * rq.W - 1) * (2 * rq.H - 1) * (rq.group_m > 0 ? (size_t)rq.nU : (size_t)rq.nV * rq.nU);
        size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
        if (blocks > 65536) blocks = 65536;
        zero_fill_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a.out, n);
        XCORR_HIP(hipGetLastError());
    }
    // more work items than the device holds blocks of this kernel: as many blocks as it holds, fed from the stream's queue
    const long slots = (long)device_cus() * plan.spec->resident_blocks();
    if (plan.spec->MFMA && plan.total_items > slots) {
        std::lock_guard<std::mutex> guard(queue_table().lock);
        a.queue = queue_for(stream);
        a.queues = slots % QUEUES == 0 ? QUEUES : 1;
        XCORR_HIP(plan.spec->launch(&a, a.queue ? (unsigned)slots : plan.grid, stream));
        return XCORR_OK;
    }
    XCORR_HIP(plan.spec->launch(&a, plan.grid, stream));
    return XCORR_OK;
}

// Planning costs 4-40 microseconds of host time, as much as a small kernel runs: the last few plans are kept per
// thread and reused when a request differs in its pointers only.
static bool same_shape(const EngineRequest &a, const EngineRequest &b) {
    return strcmp(a.family, b.family) == 0 && a.elem_bytes == b.elem_bytes && a.W == b.W && a.H == b.H && a.nV == b.nV && a.nU == b.nU &&
           a.group_m == b.group_m && a.y_shifts == b.y_shifts && a.x_shifts == b.x_shifts && a.left_mats == b.left_mats &&
           a.right_mats == b.right_mats && a.lanes_x == b.lanes_x && a.lanes_y == b.lanes_y && a.waves == b.waves &&
           a.spec_index == b.spec_index && a.rows_per_worker == b.rows_per_worker && a.column_chunks == b.column_chunks && a.matrix_cores == b.matrix_cores &&
           a.dist == b.dist && a.caller_zeroes == b.caller_zeroes && a.may_split == b.may_split && a.ordered == b.ordered;
}

static int cached_plan(const EngineRequest &rq, EnginePlan &plan) {
    struct Entry {
        bool used;
        int dev; // plans depend on the device's CU count and occupancy
        EngineRequest rq;
        EnginePlan plan;
    };
    constexpr int N = 8;
    thread_local Entry cache[N] = {};
    thread_local int next = 0;
    const int dev = current_device();
    for (int i = 0; i < N; ++i)
        if (cache[i].used && cache[i].dev == dev && same_shape(cache[i].rq, rq)) {
            plan = cache[i].plan;
            return XCORR_OK;
        }
    int rc = plan_engine(rq, plan);
    if (rc != XCORR_OK) return rc;
    cache[next] = Entry{true, dev, rq, plan};
    next = (next + 1) % N;
    return XCORR_OK;
}

// The hardware's floating-point atomic add is only defined on ordinary (coarse-grained) device memory; on host-mapped or managed
// allocations it is dropped without an error. True if `out` is memory a split plan may accumulate into. The answer for the
// last pointer asked about is kept per thread (a query costs about a microsecond).
static bool atomics_defined_on(const void *out) {
    if (plan_only()) return plan_only_mode() != 2;
    thread_local const void *last = nullptr;
    thread_local bool last_ok = false;
    if (out == last && out != nullptr) return last_ok;
    hipPointerAttribute_t attr;
    bool ok = hipPointerGetAttributes(&attr, out) == hipSuccess && attr.type == hipMemoryTypeDevice && !attr.isManaged;
    (void)hipGetLastError();
    last = out;
    last_ok = ok;
    return ok;
}

int run_engine(const EngineRequest &request, hipStream_t stream) {
    EngineRequest rq = request;
    EnginePlan plan;
    int rc = cached_plan(rq, plan);
    if (rc != XCORR_OK) return rc;
    if (plan.atomic && !atomics_defined_on(rq.out)) {
        if (rq.rows_per_worker != 0 || rq.column_chunks > 1)
            return fail(XCORR_ERR_UNSUPPORTED,
                        "%s: this launch adds partial sums with floating-point atomics, which are only defined on ordinary device memory "
                        "(hipMalloc); `out` is host-mapped, managed or unknown memory", rq.family);
        // no chunk named, the split is the launcher's own choice: the whole reduction per work item instead, plain stores
        if (rq.caller_zeroes)
            rq.dist = XCORR_DIST_NONE;
        else
            rq.may_split = false;
        rq.column_chunks = 1;
        if ((rc = cached_plan(rq, plan)) != XCORR_OK) return rc;
    }
    if (!plan_only()) {
        rc = rq.elem_bytes == 4 ? launch_typed<float>(rq, plan, stream) : launch_typed<double>(rq, plan, stream);
        if (rc != XCORR_OK) return rc;
    }
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "%s/%s", rq.family, plan.spec->name);
    rec.block[0] = plan.spec->threads;
    rec.block[1] = rec.block[2] = 1;
    rec.grid[0] = plan.grid;
    rec.grid[1] = rec.grid[2] = 1;
    rec.shared_mem_bytes = plan.spec->lds_bytes;
    rec.y_shifts_per_thread = plan.spec->A;
    rec.x_shifts_per_thread = plan.spec->B;
    rec.left_matrices_per_thread = plan.spec->NV;
    rec.right_matrices_per_thread = plan.spec->NU;
    rec.lanes_x = plan.spec->LX;
    rec.lanes_y = plan.spec->LY;
    rec.lanes_left = plan.spec->LV;
    rec.lanes_right = plan.spec->LU;
    rec.waves_x = plan.spec->WX;
    rec.waves_y = plan.spec->WY;
    rec.rows_per_worker = plan.rows_per_chunk;
    rec.distribution_type = plan.dist == 0 ? XCORR_DIST_NONE : plan.dist == 1 ? XCORR_DIST_RECTANGLE : XCORR_DIST_TRIANGLE; // (3, by levels: triangle)
    rec.uses_atomics = plan.atomic;
    rec.blocks_per_cu = plan.spec->resident_blocks();
    rec.column_chunks = plan.x_chunks;
    rec.matrix_cores = plan.spec->MFMA;
    rec.predicted_us = (float)plan.predicted_us;
    have_last_launch() = true;
    return XCORR_OK;
}

} // namespace xcorr
