// Host-side planner and launcher of the sliding-window engine: picks a compiled
// specialisation for a request, decides how the reduction over left rows is split
// into work items, clears the output when it splits on its own, launches and
// records the geometry.
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "engine_registry.hpp"

namespace xcorr {

static int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
            cus = prop.multiProcessorCount;
        else
            cus = 256;
    }
    return cus;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

static double log2_ratio(double a, double b) { return std::fabs(std::log2(a / b)); }

// Relative cost of running the request on a specialisation, calibrated on MI355X sweeps of
// 64x64 ... 1024x1024 matrices in all four modes:
//   * work issued for partial overlaps at tile edges: a wavefront skips what cannot overlap its
//     own tile, but wavefronts that own different shift tiles of one block wait for each other
//     after every staged band, so for those both the wavefront tile and the block tile count;
//   * lanes idling over matrices that do not exist;
//   * the issue rate of the tile: one-row tiles lose issue slots to LDS reads (a read plus the
//     wait that guards it displace about nine fp32 FMA slots, half as many fp64 ones); among
//     the grouped tiles 8x4 measured fastest, 4x4 and 8x8 (which spills a little) about 8 % slower (fp64: 8x8 5 % slower);
//   * lanes laid over matrices stage one band per matrix, and a right band carries a halo of
//     TYW-1 rows: +2.8 % per extra right matrix, +2 % per extra left matrix.
// Hints scale the cost a little so that the nearest of equally good specialisations wins.
static double spec_cost(const EngineSpec &s, const EngineRequest &rq) {
    double waste_x = std::sqrt((double)(rq.W + s.TXW()) * (rq.W + s.TXB())) / rq.W;
    double waste_y = std::sqrt((double)(rq.H + s.TYW()) * (rq.H + s.TYB())) / rq.H;
    int nu = rq.group_m > 0 ? rq.group_m : rq.nU;
    double util_v = (double)rq.nV / ((double)ceil_div(rq.nV, s.NVB()) * s.NVB());
    double util_u = (double)nu / ((double)ceil_div(nu, s.NUB()) * s.NUB());
    double cost = waste_x * waste_y / (util_v * util_u);
    if (s.A == 1) {
        int vk = 16 / s.elem_bytes;
        double reads = s.NV * ceil_div(s.B + s.K - 1, vk) + s.NU * (s.K / vk);
        double fmas = (double)s.NV * s.NU * s.A * s.B * s.K;
        cost *= 1.0 + (s.elem_bytes == 4 ? 9.0 : 4.5) * reads / fmas;
    } else if (s.A == 8 && s.B == 8) {
        cost *= s.elem_bytes == 4 ? 1.08 : 1.05;
    } else if (s.A == 4 && s.B == 4) {
        cost *= s.elem_bytes == 4 ? 1.08 : 1.0;
    }
    cost *= 1.0 + 0.028 * (s.LU - 1) + 0.02 * (s.LV - 1);
    if (s.NV * s.NU > 1) cost *= 1.15; // several matrices per lane: the register ring of right rows grows, some spills
    if (s.WX * s.WY * s.WZ < 4) cost *= 1.25; // fewer than one wavefront per SIMD per block: uneven SIMD load
    if (s.A > 1 && s.WZ == 1) cost *= 1.1; // shift-tiled blocks wait at the barriers of partial stages
    // the reference's tuning integers were found for its own kernels on other hardware: they only
    // break ties here (2 % per doubling away from the request)
    if (rq.y_shifts > 1) cost *= 1.0 + 0.02 * log2_ratio(s.A, rq.y_shifts);
    if (rq.left_mats) cost *= 1.0 + 0.02 * log2_ratio(s.NV * s.LV, rq.left_mats);
    if (rq.right_mats) cost *= 1.0 + 0.02 * log2_ratio(s.NU * s.LU, rq.right_mats);
    if (rq.waves) cost *= 1.0 + 0.01 * log2_ratio(s.WX * s.WY * s.WZ, rq.waves);
    return cost;
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

int plan_engine(const EngineRequest &rq, EnginePlan &plan) {
    int count = 0;
    const EngineSpec *specs = rq.elem_bytes == 4 ? engine_specs_f32(&count) : engine_specs_f64(&count);
    const EngineSpec *best = nullptr;
    double best_cost = 0;
    if (rq.spec_index > 0) {
        if ((int)rq.spec_index > count)
            return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: specialisation %u does not exist (%d compiled)", rq.family, rq.spec_index, count);
        const EngineSpec &s = specs[rq.spec_index - 1];
        if (rq.group_m > 0 && s.NVB() != 1)
            return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: specialisation %s cannot pair one left matrix with a group", rq.family, s.name);
        best = &s;
    }
    for (int i = 0; i < count && rq.spec_index == 0; ++i) {
        const EngineSpec &s = specs[i];
        if ((rq.y_shifts == 1) != (s.A == 1)) continue; // one-output-row families vs grouped families
        if (rq.group_m > 0 && s.NVB() != 1) continue;
        if (rq.x_shifts && (unsigned)s.B != rq.x_shifts) continue;
        if (rq.lanes_x && (unsigned)s.LX != rq.lanes_x) continue;
        if (rq.lanes_y && (unsigned)s.LY != rq.lanes_y) continue;
        double c = spec_cost(s, rq);
        if (!best || c < best_cost) {
            best = &s;
            best_cost = c;
        }
    }
    if (!best)
        return fail(XCORR_ERR_UNSUPPORTED, "%s: no compiled specialisation matches x_shifts_per_thread=%u lanes_x=%u lanes_y=%u",
                    rq.family, rq.x_shifts, rq.lanes_x, rq.lanes_y);
    plan.spec = best;
    const int Sx = 2 * rq.W - 1, Sy = 2 * rq.H - 1;
    plan.ntx = ceil_div(Sx, best->TXB());
    plan.nty = ceil_div(Sy, best->TYB());
    plan.nvg = ceil_div(rq.nV, best->NVB());
    plan.nug = ceil_div(rq.group_m > 0 ? rq.group_m : rq.nU, best->NUB());
    const long tiles = (long)plan.ntx * plan.nty * plan.nvg * plan.nug;

    int dist = rq.dist == XCORR_DIST_NONE ? 0 : rq.dist == XCORR_DIST_RECTANGLE ? 1 : rq.dist == XCORR_DIST_TRIANGLE ? 2 : -1;
    int rc = (int)rq.rows_per_worker;
    if (rq.caller_zeroes) {
        // split-row contract (reference one_to_one.hpp:276-288): zeroed output, atomics
        if (dist < 0) dist = 1; // the reference's default is "rectangle" (one_to_one.hpp:232)
        if (rc <= 0) rc = best->RL;
        if (dist == 0) rc = rq.H;
        plan.atomic = 1;
        plan.zero_fill = false;
    } else {
        // Few tiles, or long ones: cut the reduction over left rows into chunks (whole groups of
        // G = A+1 rows, the granule of the inner loop) until the launch has about 128 work items
        // per CU. Finer items even out the last wave of blocks and cost little, because the four
        // wavefronts of a block add their partial tiles in LDS before the atomic adds (1024x1024:
        // flat between 18 and 54 rows, 3 % slower at 72, 6 % at 144; 2048x2048 unsplit 20 % slower).
        // Items shorter than 20 rows only pay for tiny problems that would otherwise leave CUs
        // without work. Lanes laid over matrices write one result matrix per lane: their
        // atomics would not coalesce, so such tiles are never split by the planner itself.
        const bool split_ok = rq.may_split && best->LV * best->LU == 1;
        const int G = best->A + 1;
        const int rc_most = 4 * best->RL;
        if (rc <= 0 && split_ok && (tiles < 48L * device_cus() || rq.H > rc_most)) {
            const long target = 128L * device_cus();
            const long per_tile_column = (long)plan.ntx * plan.nvg * plan.nug;
            // shortest item: 20 rows, or 9 when that leaves CUs without work (rounded up to whole groups)
            const int k_normal = ceil_div(20, G), k_tiny = ceil_div(9, G);
            const int k_min = per_tile_column * count_chunks(*best, rq.H, plan.nty, k_normal * G, nullptr) < 2L * device_cus() ? k_tiny : k_normal;
            int k = (rq.H < rc_most ? rq.H : rc_most) / G;
            for (; k >= k_min; --k) {
                rc = k * G;
                if (per_tile_column * count_chunks(*best, rq.H, plan.nty, rc, nullptr) >= target) break;
            }
            if (rc <= 0) rc = rq.H;
        }
        if (rc <= 0 || rc >= rq.H || !rq.may_split) {
            rc = rq.H;
            dist = 0;
            plan.atomic = 0;
            plan.zero_fill = false;
        } else {
            if (dist <= 0) dist = 2;
            plan.atomic = 1;
            plan.zero_fill = true;
        }
    }
    if (rc > rq.H) rc = rq.H;
    plan.rows_per_chunk = rc;
    plan.dist = dist;

    // workers along y: (y tile, chunk) pairs
    int max_chunks = 0;
    long total_chunks = count_chunks(*best, rq.H, plan.nty, rc, &max_chunks);
    if (dist == 0)
        plan.nworkers_y = plan.nty;
    else if (dist == 1)
        plan.nworkers_y = plan.nty * max_chunks;
    else
        plan.nworkers_y = (int)total_chunks;
    long items = (long)plan.nvg * plan.nug * plan.nworkers_y * plan.ntx;
    if (items <= 0 || items > 0x7fffffffL) return fail(XCORR_ERR_INVALID_ARGUMENT, "%s: %ld work items are out of range", rq.family, items);
    plan.total_items = (int)items;
    plan.grid = (unsigned)items;
    return XCORR_OK;
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
    if (plan.zero_fill) {
        size_t n = (size_t)(2 * rq.W - 1) * (2 * rq.H - 1) * (rq.group_m > 0 ? (size_t)rq.nU : (size_t)rq.nV * rq.nU);
        size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
        if (blocks > 65536) blocks = 65536;
        zero_fill_kernel<T><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a.out, n);
        XCORR_HIP(hipGetLastError());
    }
    XCORR_HIP(plan.spec->launch(&a, plan.grid, stream));
    return XCORR_OK;
}

int run_engine(const EngineRequest &rq, hipStream_t stream) {
    EnginePlan plan;
    int rc = plan_engine(rq, plan);
    if (rc != XCORR_OK) return rc;
    rc = rq.elem_bytes == 4 ? launch_typed<float>(rq, plan, stream) : launch_typed<double>(rq, plan, stream);
    if (rc != XCORR_OK) return rc;
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
    rec.distribution_type = plan.dist == 0 ? XCORR_DIST_NONE : plan.dist == 1 ? XCORR_DIST_RECTANGLE : XCORR_DIST_TRIANGLE;
    rec.uses_atomics = plan.atomic;
    have_last_launch() = true;
    return XCORR_OK;
}

} // namespace xcorr
