// Overlap-wise and warp-per-overlap kernel families for gfx950 wavefronts.
//
// overlap-wise      : one thread per shift, serial loop over the overlap straight from
//                     global memory (the definition; the reference's starting point,
//                     naive_original.cu:36-102).
// warp-per-overlap  : one 64-lane wavefront per shift; lanes stride the overlap and the
//                     partial sums are combined with DPP row operations (no LDS, no
//                     ds_bpermute), replacing the 32-lane cg::reduce of
//                     naive_warp_per_shift.cu:21-244.
// warp-per-overlap, LDS : the wavefronts of a block own consecutive y shifts of one x shift
//                     and share row chunks of the right matrices and of the left matrix
//                     staged in LDS (naive_warp_per_shift_shared_mem.cu:160-420).
// block-per-overlap : all wavefronts of a block reduce one shift together
//                     (naive_block_per_shift.cu:17-97).
#pragma once

#include <hip/hip_runtime.h>

#include "engine.hpp" // vec128
#include "xcorr_common.hpp"

namespace xcorr {

// ------------------------------------------------------------------ DPP wave reduction
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double v) {
    unsigned long long bits = __builtin_bit_cast(unsigned long long, v);
    int lo = (int)(unsigned)bits, hi = (int)(unsigned)(bits >> 32);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(double, ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// Sum over the 64 lanes of a wavefront; the total is valid in lane 63.
template <typename T>
__device__ __forceinline__ T wave_sum_to_lane63(T v) {
    v += dpp_move<0xB1, 0xf>(v);  // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xf>(v);  // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xf>(v); // row_half_mirror
    v += dpp_move<0x140, 0xf>(v); // row_mirror: every lane of a 16-lane row holds the row sum
    v += dpp_move<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v += dpp_move<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ void atomic_add_simple(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add_simple(double *p, double v) { unsafeAtomicAdd(p, v); }

// ------------------------------------------------------------------ overlap-wise
// Thread (x, y) of the strip of n_left result matrices laid side by side computes one
// shift; blockIdx.z walks the `batch` right matrices paired with its left matrix. The products
// are added in the order of the definition (row by row, left to right, one accumulator), so a
// result equals the host loop's bit for bit when that is compiled with the same contraction;
// eight element pairs are loaded ahead of the eight dependent FMAs so that the loads overlap.
// ALL_PAIRS: every right matrix is correlated with every left matrix, result index = left * batch + right; the strip
// holds `strip_lefts` result matrices and blockIdx.z walks (group of strip_lefts left matrices, right matrix).
// STAGE (one left matrix, small matrices): the block first copies the left matrix and, per right matrix, that matrix into
// LDS and the threads read their elements from there - same products, same order, less latency per load (the kernel is one
// dependent chain of loads and FMAs per thread; a 24x24 pair: 22.0 -> 18.1 us, and 16.2 us with WIDE_TAIL; 16x16: 13.8 -> 8.9 us).
// WIDE_TAIL: the last one to seven products of a row are loaded together like a whole group instead of one by one - shorter chains for
// launches of few blocks (16x16, 2 x 2 matrices: 13.6 -> 11.2 us), more load instructions for launches that fill the device (16x16,
// 32 x 32 matrices: 63 -> 93 us): the launcher sets it for launches of at most one block per CU.
template <typename T, bool ALL_PAIRS, bool STAGE, bool WIDE_TAIL>
__global__ __launch_bounds__(256) void overlap_wise_kernel(const T *__restrict__ left, const T *__restrict__ right,
                                                            T *__restrict__ out, int W, int H, int n_left, int batch, int strip_lefts) {
    extern __shared__ __attribute__((aligned(16))) unsigned char overlap_smem[];
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const int strip_x = blockIdx.x * blockDim.x + threadIdx.x;
    const int oy = blockIdx.y * blockDim.y + threadIdx.y;
    const int in_strip = strip_x / Sx;
    const bool active = in_strip < strip_lefts && oy < Sy;
    if (!STAGE && !active) return;
    const int ox = strip_x - in_strip * Sx;
    const int sx = ox - (W - 1), sy = oy - (H - 1);
    const int xl_lo = sx > 0 ? sx : 0, xl_hi = W + sx < W ? W + sx : W;
    const int yl_lo = sy > 0 ? sy : 0, yl_hi = H + sy < H ? H + sy : H;
    const size_t in_area = (size_t)W * H, out_area = (size_t)Sx * Sy;
    const int steps = ALL_PAIRS ? (n_left / strip_lefts) * batch : batch;
    const int tid = threadIdx.y * blockDim.x + threadIdx.x, nthreads = blockDim.x * blockDim.y;
    T *Ls = reinterpret_cast<T *>(overlap_smem), *Rs = Ls + in_area;
    if (STAGE)
        for (int i = tid; i < (int)in_area; i += nthreads) Ls[i] = left[i];
    for (int z = blockIdx.z; z < steps; z += gridDim.z) {
        const int b = ALL_PAIRS ? z % batch : z;
        const int region = ALL_PAIRS ? (z / batch) * strip_lefts + in_strip : in_strip;
        const size_t mat = ALL_PAIRS ? (size_t)region * batch + b : (size_t)b * n_left + region;
        const T *l = left + region * in_area;
        const T *r = right + (ALL_PAIRS ? (size_t)b : mat) * in_area;
        if (STAGE) { // (n_left == 1: region 0, right matrix b for every thread of the block)
            __syncthreads(); // the previous right matrix is no longer read
            const T *rz = right + (size_t)b * in_area;
            for (int i = tid; i < (int)in_area; i += nthreads) Rs[i] = rz[i];
            __syncthreads();
            if (!active) continue;
            l = Ls;
            r = Rs;
        }
        T sum = T(0);
        for (int yl = yl_lo; yl < yl_hi; ++yl) {
            const T *lrow = l + (size_t)yl * W;
            const T *rrow = r + (size_t)(yl - sy) * W - sx;
            int xl = xl_lo;
            for (; xl + 8 <= xl_hi; xl += 8) {
                T a[8], c[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a[i] = rrow[xl + i];
                    c[i] = lrow[xl + i];
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) sum += a[i] * c[i];
            }
            if (!WIDE_TAIL) {
                for (; xl < xl_hi; ++xl) sum += rrow[xl] * lrow[xl];
            } else if (xl < xl_hi) { // the last one to seven products: loaded together (from addresses inside the row), added in order
                T a[8], c[8];
#pragma unroll
                for (int i = 0; i < 7; ++i) {
                    const int x = xl + i < xl_hi ? xl + i : xl;
                    a[i] = rrow[x];
                    c[i] = lrow[x];
                }
#pragma unroll
                for (int i = 0; i < 7; ++i)
                    if (xl + i < xl_hi) sum += a[i] * c[i];
            }
        }
        out[mat * out_area + (size_t)oy * Sx + ox] = sum;
    }
}

template <typename T>
int run_overlap_wise(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_left,
                     unsigned batch, bool all_pairs, hipStream_t stream) {
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if (n_left == 0 || batch == 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "no matrices");
    if (batch > 0x7fffffffu) return fail(XCORR_ERR_INVALID_ARGUMENT, "too many matrices: batch of %u", batch);
    const unsigned Sx = 2 * cols - 1, Sy = 2 * rows - 1;
    dim3 block(64, 4);
    // (all left matrices side by side in the strip: measured faster than one result matrix per strip, which reads the
    // right matrix of a pair once per left matrix instead of once)
    const unsigned strip_lefts = n_left;
    unsigned long long strip = (unsigned long long)Sx * strip_lefts;
    if (strip > 0x7fffffffULL) return fail(XCORR_ERR_INVALID_ARGUMENT, "strip of %u result matrices is too wide", n_left);
    unsigned long long steps = batch;
    if (all_pairs) {
        steps = (unsigned long long)(n_left / strip_lefts) * batch;
        if ((unsigned long long)n_left * batch > 0x7fffffffULL) return fail(XCORR_ERR_INVALID_ARGUMENT, "too many matrices: %u left, %u right", n_left, batch);
    }
    dim3 grid((unsigned)((strip + block.x - 1) / block.x), (Sy + block.y - 1) / block.y, (unsigned)(steps < 65535 ? steps : 65535));
    // One left matrix and a pair that fits 64 KB of LDS: staged - always up to 32x32 fp32 (1 x 4000 of 32x32: 4.1 -> 2.7 ms), larger pairs
    // while the launch has at most sixteen blocks per CU (1 x 32 of 64x64: 491 -> 398 us; 1 x 4000 of 64x64, where the 32 KB per block cost
    // more occupancy than the shorter loads give back: 32.8 -> 35.7 ms, so not there).
    const unsigned long long blocks = (unsigned long long)grid.x * grid.y * grid.z;
    const size_t pair_bytes = 2 * (size_t)cols * rows * sizeof(T);
    const bool stage = n_left == 1 && pair_bytes <= 64 * 1024 && (pair_bytes <= 8 * 1024 || blocks <= 16ull * (unsigned)device_cus());
    const bool few_blocks = blocks <= (unsigned long long)device_cus();
    const int W = (int)cols, H = (int)rows, nl = (int)n_left, nb = (int)batch, sl = (int)strip_lefts;
    if (stage && few_blocks)
        overlap_wise_kernel<T, false, true, true><<<grid, block, pair_bytes, stream>>>(left, right, out, W, H, 1, nb, 1);
    else if (stage)
        overlap_wise_kernel<T, false, true, false><<<grid, block, pair_bytes, stream>>>(left, right, out, W, H, 1, nb, 1);
    else if (all_pairs && few_blocks)
        overlap_wise_kernel<T, true, false, true><<<grid, block, 0, stream>>>(left, right, out, W, H, nl, nb, sl);
    else if (all_pairs)
        overlap_wise_kernel<T, true, false, false><<<grid, block, 0, stream>>>(left, right, out, W, H, nl, nb, sl);
    else if (few_blocks)
        overlap_wise_kernel<T, false, false, true><<<grid, block, 0, stream>>>(left, right, out, W, H, nl, nb, sl);
    else
        overlap_wise_kernel<T, false, false, false><<<grid, block, 0, stream>>>(left, right, out, W, H, nl, nb, sl);
    XCORR_HIP(hipGetLastError());
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "overlap_wise/%s%s", sizeof(T) == 4 ? "f32" : "f64", all_pairs ? "_all_pairs" : "");
    rec.block[0] = block.x, rec.block[1] = block.y, rec.block[2] = 1;
    rec.grid[0] = grid.x, rec.grid[1] = grid.y, rec.grid[2] = grid.z;
    rec.y_shifts_per_thread = rec.x_shifts_per_thread = 1;
    rec.left_matrices_per_thread = 1;
    rec.right_matrices_per_thread = batch;
    rec.distribution_type = XCORR_DIST_NONE;
    have_last_launch() = true;
    return XCORR_OK;
}

// ------------------------------------------------------------------ warp-per-overlap
// Dense ("triangle") packing of split-row workers: output row r has
// ceil(overlap_rows(r) / max_rows) workers, numbered consecutively over rows.
__host__ __device__ inline unsigned wpo_overlap_rows(unsigned row, unsigned H) { return row < H ? row + 1 : 2 * H - 1 - row; }
__host__ __device__ inline unsigned wpo_workers(unsigned row, unsigned H, unsigned max_rows) {
    return (wpo_overlap_rows(row, H) + max_rows - 1) / max_rows;
}
// number of workers of output rows [0, n) for n <= H (ascending half)
__host__ __device__ inline unsigned long long wpo_prefix_ascending(unsigned n, unsigned R) {
    unsigned long long q = n / R, rem = n % R;
    return (unsigned long long)R * q * (q + 1) / 2 + rem * (q + 1);
}
// number of workers of output rows [0, n), 0 <= n <= 2H-1
__host__ __device__ inline unsigned long long wpo_prefix(unsigned n, unsigned H, unsigned R) {
    if (n <= H) return wpo_prefix_ascending(n, R);
    // rows H .. n-1 mirror rows H-2 .. 2H-1-n
    unsigned m = n - H; // count of descending rows taken
    return wpo_prefix_ascending(H, R) + (wpo_prefix_ascending(H - 1, R) - wpo_prefix_ascending(H - 1 - m, R));
}

struct WpoWork {
    unsigned row, idx, per_row;
};

template <int DIST>
__device__ __forceinline__ WpoWork wpo_distribute(unsigned worker, unsigned max_rows, unsigned H) {
    const unsigned Sy = 2 * H - 1;
    WpoWork w;
    if (DIST == 0) {
        w.row = worker;
        w.idx = 0;
        w.per_row = worker < Sy ? 1u : 0u;
    } else if (DIST == 1) {
        w.row = worker % Sy;
        w.idx = worker / Sy;
        w.per_row = wpo_workers(w.row, H, max_rows);
    } else {
        // largest row whose prefix is <= worker
        unsigned lo = 0, hi = Sy; // prefix(lo) <= worker < prefix(hi) unless worker is surplus
        if (worker >= wpo_prefix(Sy, H, max_rows)) {
            w.row = Sy;
            w.idx = 0;
            w.per_row = 0;
            return w;
        }
        while (hi - lo > 1) {
            unsigned mid = (lo + hi) / 2;
            if (wpo_prefix(mid, H, max_rows) <= worker)
                lo = mid;
            else
                hi = mid;
        }
        w.row = lo;
        w.idx = worker - (unsigned)wpo_prefix(lo, H, max_rows);
        w.per_row = wpo_workers(lo, H, max_rows);
    }
    return w;
}

// VARIANT 0: lanes stride the flattened overlap; 1: row loop, lanes stride the columns;
// 2: the rows of a shift are split over workers (DIST) and added atomically (the reference's kernel strides the
// flattened part like 0, naive_warp_per_shift.cu:160-175; here the row loop of 1, which is faster and whose
// summation order is free anyway once parts are added atomically).
template <typename T, int VARIANT, int DIST>
__global__ __launch_bounds__(1024) void warp_per_overlap_kernel(const T *__restrict__ left, const T *__restrict__ right,
                                                                 T *__restrict__ out, int W, int H, unsigned max_rows) {
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const int lane = threadIdx.x;
    const int ox = blockIdx.x * blockDim.y + threadIdx.y;
    int oy = blockIdx.y;
    unsigned part = 0, parts = 1;
    if (VARIANT == 2) {
        WpoWork w = wpo_distribute<DIST>(blockIdx.y, max_rows, (unsigned)H);
        if (w.idx >= w.per_row) return;
        oy = (int)w.row;
        part = w.idx;
        parts = w.per_row;
    }
    if (ox >= Sx || oy >= Sy) return;
    const int sx = ox - (W - 1), sy = oy - (H - 1);
    // overlap in right-matrix coordinates
    const int xr_lo = sx < 0 ? -sx : 0, xr_hi = W - sx < W ? W - sx : W;
    int yr_lo = sy < 0 ? -sy : 0, yr_hi = H - sy < H ? H - sy : H;
    if (VARIANT == 2) {
        const int rows_all = yr_hi - yr_lo;
        const int per = (rows_all + (int)parts - 1) / (int)parts;
        yr_lo += (int)part * per;
        if (yr_lo + per < yr_hi) yr_hi = yr_lo + per;
    }
    const int ow = xr_hi - xr_lo, oh = yr_hi - yr_lo;
    T sum = T(0);
    if (VARIANT != 0) {
        // columns outer (one pass up to 64 columns), rows inner and unrolled eight times with
        // independent partial sums: sixteen loads are in flight per lane instead of two, which is
        // what a wavefront that owns a single short reduction needs to hide the cache latency
        T part_sum[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) part_sum[r] = T(0);
        for (int xr = xr_lo + lane; xr < xr_hi; xr += 64) {
            const T *rp = right + (size_t)yr_lo * W + xr;
            const T *lp = left + (size_t)(yr_lo + sy) * W + (sx + xr);
            int yr = yr_lo;
            for (; yr + 8 <= yr_hi; yr += 8) {
#pragma unroll
                for (int r = 0; r < 8; ++r) part_sum[r] += lp[(size_t)r * W] * rp[(size_t)r * W];
                lp += (size_t)8 * W;
                rp += (size_t)8 * W;
            }
            for (; yr < yr_hi; ++yr) {
                part_sum[0] += lp[0] * rp[0];
                lp += W;
                rp += W;
            }
        }
        sum = ((part_sum[0] + part_sum[1]) + (part_sum[2] + part_sum[3])) + ((part_sum[4] + part_sum[5]) + (part_sum[6] + part_sum[7]));
    } else if (oh > 0 && ow > 0) {
        // lanes stride the flattened overlap. Four strides are in flight with a partial sum each, and a
        // position's (row, column) advances by 256 elements with one compare instead of a division.
        const unsigned uow = (unsigned)ow, total = uow * (unsigned)oh;
        const unsigned step_rows = 256u / uow, step_cols = 256u % uow;
        T part_sum[4];
        unsigned row[4], col[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            part_sum[k] = T(0);
            row[k] = ((unsigned)lane + 64u * k) / uow;
            col[k] = ((unsigned)lane + 64u * k) - row[k] * uow;
        }
        auto product = [&](int k) {
            const int yr = yr_lo + (int)row[k], xr = xr_lo + (int)col[k];
            return left[(size_t)(yr + sy) * W + (xr + sx)] * right[(size_t)yr * W + xr];
        };
        unsigned i = (unsigned)lane;
        for (; i + 192u < total; i += 256u) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                part_sum[k] += product(k);
                row[k] += step_rows;
                col[k] += step_cols;
                if (col[k] >= uow) {
                    col[k] -= uow;
                    ++row[k];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < 3; ++k)
            if (i + 64u * k < total) part_sum[k] += product(k);
        sum = (part_sum[0] + part_sum[1]) + (part_sum[2] + part_sum[3]);
    }
    sum = wave_sum_to_lane63(sum);
    if (lane == 63) {
        T *p = out + (size_t)oy * Sx + ox;
        if (VARIANT == 2)
            atomic_add_simple(p, sum);
        else
            *p = sum;
    }
}

template <typename T>
int run_warp_per_overlap(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params &p,
                         hipStream_t stream) {
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    // reference limit: naive_warp_per_shift.cu:316-318 (32 warps of 32 lanes per block)
    if ((rc = check_limit("shifts per thread block", p.shifts_per_thread_block, 32))) return rc;
    if (p.warp_per_overlap_variant > XCORR_WPO_WORK_DISTRIBUTION)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "Unknown warp-per-overlap variant %u", p.warp_per_overlap_variant);
    if (p.distribution_type > XCORR_DIST_TRIANGLE) return fail(XCORR_ERR_INVALID_ARGUMENT, "Unknown distribution %u", p.distribution_type);
    unsigned spb = p.shifts_per_thread_block ? p.shifts_per_thread_block : 8; // reference default one_to_one.hpp:415
    if (spb > 16) spb = 16; // a block holds at most 16 wavefronts of 64 lanes
    const unsigned Sx = 2 * cols - 1, Sy = 2 * rows - 1;
    dim3 block(64, spb);
    unsigned grid_y = Sy;
    // rows per worker of the work-distribution variant. The reference's default is 3 (rows_per_warp, one_to_one.hpp:458);
    // here 0 keeps every shift whole: measured on 16x16 ... 256x256 pairs, any split was slower than none (a worker's
    // wavefront-wide sum and atomic add cost more than the few rows it saves)
    unsigned max_rows = p.rows_per_thread ? p.rows_per_thread : rows;
    unsigned dist = p.distribution_type == XCORR_DIST_DEFAULT ? XCORR_DIST_RECTANGLE : p.distribution_type;
    const int variant = (int)p.warp_per_overlap_variant;
    if (variant == 2) {
        if (dist == XCORR_DIST_NONE)
            grid_y = Sy;
        else if (dist == XCORR_DIST_RECTANGLE)
            grid_y = Sy * ((rows + max_rows - 1) / max_rows);
        else
            grid_y = (unsigned)wpo_prefix(Sy, rows, max_rows);
    }
    dim3 grid((Sx + spb - 1) / spb, grid_y);
    const int W = (int)cols, H = (int)rows;
    if (plan_only())
        ; // (planning only: the record below is what a launch would report)
    else if (variant == 0)
        warp_per_overlap_kernel<T, 0, 0><<<grid, block, 0, stream>>>(left, right, out, W, H, max_rows);
    else if (variant == 1)
        warp_per_overlap_kernel<T, 1, 0><<<grid, block, 0, stream>>>(left, right, out, W, H, max_rows);
    else if (dist == XCORR_DIST_NONE)
        warp_per_overlap_kernel<T, 2, 0><<<grid, block, 0, stream>>>(left, right, out, W, H, max_rows);
    else if (dist == XCORR_DIST_RECTANGLE)
        warp_per_overlap_kernel<T, 2, 1><<<grid, block, 0, stream>>>(left, right, out, W, H, max_rows);
    else
        warp_per_overlap_kernel<T, 2, 2><<<grid, block, 0, stream>>>(left, right, out, W, H, max_rows);
    if (!plan_only()) XCORR_HIP(hipGetLastError());
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "warp_per_overlap/%s_v%d", sizeof(T) == 4 ? "f32" : "f64", variant);
    rec.block[0] = block.x, rec.block[1] = block.y, rec.block[2] = 1;
    rec.grid[0] = grid.x, rec.grid[1] = grid.y, rec.grid[2] = 1;
    rec.y_shifts_per_thread = rec.x_shifts_per_thread = 1;
    rec.left_matrices_per_thread = rec.right_matrices_per_thread = 1;
    rec.rows_per_worker = variant == 2 ? max_rows : rows;
    rec.distribution_type = variant == 2 ? dist : XCORR_DIST_NONE;
    rec.uses_atomics = variant == 2;
    have_last_launch() = true;
    return XCORR_OK;
}

// ------------------------------------------------------------------ whole pair in LDS
// One small pair (both matrices fit the LDS of a CU together): every block first copies BOTH matrices
// into LDS - the left one with B zero columns on either side of every row and a few zero rows above and
// below, the right one with zero rows below - and then its wavefronts work through tasks of A adjacent
// y shifts x B adjacent x shifts: lane = right column; per overlapping right row one LDS read of the right
// element and B reads of ONE new left row (the A left rows a step pairs with that right row slide down by
// one row per step and are kept in registers) for A * B FMAs; the 64 partial sums of every shift are
// combined by DPP row operations. One launch, no atomics, no clearing of the output, nothing but LDS
// traffic after the first 2 * rows * cols * sizeof(T) bytes per block; a 64x64 fp32 pair is 4064 tasks of one
// y shift, one per wavefront of 256 blocks of 16. This is what the reference's shared-memory
// warp-per-shift kernel (naive_warp_per_shift_shared_mem.cu:160-420, its fastest at 64x64) reaches for with
// its row slabs. Tasks are dealt so that the wavefronts of a block get output rows far apart (a mix of
// long and short overlaps on every CU).
// (Indices are split into row and column by multiplication with a rounded-up reciprocal that the host passes in:
// the integer divisions the compiler would emit for run-time pitches cost about forty instructions each, and the
// copy into LDS was bound by them.)
struct PairGeometry {
    int W, H, pitch_l, pitch_r, tasks_x, total_tasks;
    unsigned magic_pl, magic_pr, magic_tx; // floor(2^32 / d) + 1 for d = pieces per left row, per right row, tasks per output row
    // several pairs in one launch: blocks_per_pair consecutive blocks share a pair; pair p is left matrix p / left_div with right
    // matrix p % right_mod (right_mod 0: right matrix p) and writes result p
    int blocks_per_pair, left_div, right_mod;
};
__device__ __forceinline__ int div_by(int n, int d, unsigned magic) { return d == 1 ? n : (int)__umulhi((unsigned)n, magic); }

// COLS != 0 compiles the kernel for matrices of exactly that many columns: the row pitches of the LDS images are then
// constants and every LDS read of a round is the round's base address plus an immediate offset (with run-time pitches
// one address addition per read, two thirds as many instructions again as the FMAs).
template <typename T, int A, int B, int U, int COLS>
__global__ __launch_bounds__(1024) void pair_in_lds_kernel(const T *__restrict__ left_all, const T *__restrict__ right_all, T *__restrict__ out_all,
                                                           const PairGeometry geo) {
    const int W = COLS ? COLS : geo.W, H = geo.H, tasks_x = geo.tasks_x, total_tasks = geo.total_tasks;
    // (one pair: no divisions - they would be a twentieth of this kernel's run time on a 16x16 pair)
    int block_of_pair = (int)blockIdx.x;
    const T *left = left_all, *right = right_all;
    T *out = out_all;
    if ((int)gridDim.x != geo.blocks_per_pair) {
        const int pair = (int)blockIdx.x / geo.blocks_per_pair;
        block_of_pair = (int)blockIdx.x - pair * geo.blocks_per_pair;
        left += (size_t)(pair / geo.left_div) * W * H;
        right += (size_t)(geo.right_mod ? pair % geo.right_mod : pair) * W * H;
        out += (size_t)pair * (2 * W - 1) * (2 * H - 1);
    }
    const int pitch_l = COLS ? COLS + 2 * (B < 16 / (int)sizeof(T) ? 16 / (int)sizeof(T) : B) : geo.pitch_l, pitch_r = COLS ? COLS : geo.pitch_r;
    using vec = typename vec128<T>::type;
    constexpr int VK = 16 / (int)sizeof(T);
    constexpr int PAD = B < VK ? VK : B;          // zero columns on either side of a left row (keeps 128-bit pieces aligned)
    constexpr int TOP = A - 1, BOT = U + A - 2;   // zero rows above / below the left matrix; the right one has U - 1 below
    extern __shared__ __attribute__((aligned(16))) unsigned char pair_smem[];
    T *Ls = reinterpret_cast<T *>(pair_smem);
    const int rows_l = H + TOP + BOT, rows_r = H + U - 1;
    T *Rs = Ls + (size_t)rows_l * pitch_l;
    const int tid = (int)threadIdx.x, nt = (int)blockDim.x;
    // ---- both matrices into LDS, 128-bit pieces; the loads of four pieces per thread are in flight together ----
    {
        const int pl = pitch_l / VK, pr = pitch_r / VK;
        const int total_l = rows_l * pl, total = total_l + rows_r * pr; // the right image follows the left one
        constexpr int NB = 4;
        for (int p0 = tid; p0 < total; p0 += nt * NB) {
            vec v[NB];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int p = p0 + j * nt;
#pragma unroll
                for (int e = 0; e < VK; ++e) v[j][e] = T(0);
                if (p >= total) continue;
                const bool is_left = p < total_l;
                const int q = is_left ? p : p - total_l, pp = is_left ? pl : pr;
                const int qrow = div_by(q, pp, is_left ? geo.magic_pl : geo.magic_pr);
                const int row = qrow - (is_left ? TOP : 0), col = (q - qrow * pp) * VK - (is_left ? PAD : 0); // matrix row, first column
                if (row < 0 || row >= H) continue;
                const T *src = (is_left ? left : right) + (size_t)row * W + col;
                if (col >= 0 && col + VK <= W) {
                    __builtin_memcpy(&v[j], src, sizeof(vec)); // element-aligned only
                } else {
#pragma unroll
                    for (int e = 0; e < VK; ++e)
                        if (col + e >= 0 && col + e < W) v[j][e] = src[e];
                }
            }
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int p = p0 + j * nt;
                if (p < total) *reinterpret_cast<vec *>(Ls + (size_t)p * VK) = v[j];
            }
        }
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    // task (wave w of block b of the pair's blocks, round i) = w * blocks + b + i * blocks * nw
    for (int t = wave * geo.blocks_per_pair + block_of_pair; t < total_tasks; t += geo.blocks_per_pair * nw) {
        const int ty = div_by(t, tasks_x, geo.magic_tx);
        const int oy0 = ty * A, ox0 = (t - ty * tasks_x) * B;
        const int sy0 = oy0 - (H - 1), sx0 = ox0 - (W - 1);
        // right rows / columns that overlap any of the A x B shifts
        int y_lo = -(sy0 + A - 1), y_hi = H - sy0, x_lo = -(sx0 + B - 1), x_hi = W - sx0;
        if (y_lo < 0) y_lo = 0;
        if (y_hi > H) y_hi = H;
        if (x_lo < 0) x_lo = 0;
        if (x_hi > W) x_hi = W;
        const int rounds = (y_hi - y_lo + U - 1) / U; // whole rounds of U rows: the last one may run into the zero rows
        T acc[A][B];
#pragma unroll
        for (int a = 0; a < A; ++a)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[a][b] = T(0);
        for (int c0 = x_lo; c0 < x_hi; c0 += 64) {
            const int xr = c0 + lane;
            if (xr < x_hi) {
                const T *rp = Rs + (size_t)y_lo * pitch_r + xr;
                const T *lp = Ls + (size_t)(y_lo + sy0 + TOP) * pitch_l + PAD + xr + sx0; // left row that pairs with y_lo for shift sy0
                // left rows y + sy0 .. y + sy0 + U + A - 2 of a round that starts at right row y; the last A - 1 of them
                // are the first A - 1 of the next round
                T win[U + A - 1][B];
#pragma unroll
                for (int a = 0; a < A - 1; ++a)
#pragma unroll
                    for (int b = 0; b < B; ++b) win[a][b] = lp[a * pitch_l + b];
                for (int g = 0; g < rounds; ++g) {
                    T r[U];
#pragma unroll
                    for (int j = 0; j < U; ++j) { // U * (B + 1) reads in flight ahead of the FMAs
                        r[j] = rp[j * pitch_r];
#pragma unroll
                        for (int b = 0; b < B; ++b) win[A - 1 + j][b] = lp[(A - 1 + j) * pitch_l + b];
                    }
#pragma unroll
                    for (int j = 0; j < U; ++j)
#pragma unroll
                        for (int a = 0; a < A; ++a)
#pragma unroll
                            for (int b = 0; b < B; ++b) acc[a][b] += win[j + a][b] * r[j];
#pragma unroll
                    for (int a = 0; a < A - 1; ++a)
#pragma unroll
                        for (int b = 0; b < B; ++b) win[a][b] = win[U + a][b];
                    rp += U * pitch_r;
                    lp += U * pitch_l;
                }
            }
        }
#pragma unroll
        for (int a = 0; a < A; ++a)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[a][b] = wave_sum_to_lane63(acc[a][b]);
        if (lane == 63) {
#pragma unroll
            for (int a = 0; a < A; ++a)
#pragma unroll
                for (int b = 0; b < B; ++b)
                    if (oy0 + a < Sy && ox0 + b < Sx) out[(size_t)(oy0 + a) * Sx + ox0 + b] = acc[a][b];
        }
    }
}

constexpr int PAIR_B = 4; // x shifts per task of the whole-pair kernel

// Bytes of LDS the whole-pair kernel needs for a rows x cols pair with A y shifts per task and U rows per round.
template <typename T>
inline size_t pair_in_lds_bytes(unsigned cols, unsigned rows, unsigned A, unsigned U) {
    constexpr unsigned VK = 16 / sizeof(T), PAD = PAIR_B < VK ? VK : PAIR_B;
    const size_t pitch_l = (cols + 2 * PAD + VK - 1) / VK * VK, pitch_r = (cols + VK - 1) / VK * VK;
    return ((size_t)(rows + U + 2 * A - 3) * pitch_l + (size_t)(rows + U - 1) * pitch_r) * sizeof(T);
}
// whether the whole-pair kernel can run a rows x cols pair at all (its smallest variant)
template <typename T>
inline bool pair_fits_lds(unsigned cols, unsigned rows) {
    return pair_in_lds_bytes<T>(cols, rows, 2, 4) <= 160 * 1024;
}

// What the pairs of a launch are: n_pairs results; pair p = left p / left_div x right p % right_mod (0: right p).
struct PairList {
    unsigned n_pairs = 1, left_div = 1, right_mod = 0;
};

template <typename T, int A, int U, int COLS>
int launch_pair_in_lds(const T *left, const T *right, T *out, unsigned cols, unsigned rows, size_t bytes, const PairList &pairs, unsigned *grid_out,
                       unsigned *waves_out, hipStream_t stream) {
    constexpr unsigned VK = 16 / sizeof(T), B = PAIR_B, PAD = B < VK ? VK : B;
    const int pitch_l = (int)((cols + 2 * PAD + VK - 1) / VK * VK), pitch_r = (int)((cols + VK - 1) / VK * VK);
    static bool attr_set[64] = {};
    int dev = 0;
    if (!plan_only()) XCORR_HIP(hipGetDevice(&dev));
    if (!plan_only() && bytes > 64 * 1024 && !(dev >= 0 && dev < 64 && attr_set[dev])) {
        XCORR_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&pair_in_lds_kernel<T, A, B, U, COLS>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      160 * 1024));
        if (dev >= 0 && dev < 64) attr_set[dev] = true;
    }
    const unsigned Sx = 2 * cols - 1, Sy = 2 * rows - 1;
    const unsigned tasks_x = (Sx + B - 1) / B, total = tasks_x * ((Sy + A - 1) / A);
    const int cus = device_cus();
    // eight wavefronts per block while that still gives every task a wavefront of its own, else sixteen
    const unsigned waves = (size_t)total * pairs.n_pairs <= 8u * (size_t)cus ? 8 : 16;
    unsigned grid = (total + waves - 1) / waves;
    // one block per CU: every block pays for its own copy of the pair (several pairs: the CUs are dealt to them, two blocks
    // per CU where two fit)
    const unsigned slots = (unsigned)cus * (pairs.n_pairs > 1 && bytes <= 64 * 1024 ? 2u : 1u);
    const unsigned share = slots / pairs.n_pairs > 0 ? slots / pairs.n_pairs : 1;
    if (grid > share) grid = share;
    auto magic = [](unsigned d) { return (unsigned)((1ull << 32) / d) + 1u; }; // exact for n * d < 2^32, far above any index here
    const PairGeometry geo = {(int)cols,         (int)rows,          pitch_l,       pitch_r, (int)tasks_x, (int)total,
                              magic(pitch_l / VK), magic(pitch_r / VK), magic(tasks_x), (int)grid, (int)pairs.left_div, (int)pairs.right_mod};
    grid *= pairs.n_pairs;
    if (!plan_only()) {
        pair_in_lds_kernel<T, A, B, U, COLS><<<dim3(grid), dim3(64 * waves), bytes, stream>>>(left, right, out, geo);
        XCORR_HIP(hipGetLastError());
    }
    *grid_out = grid;
    *waves_out = waves;
    return XCORR_OK;
}

template <typename T>
int run_pair_in_lds(const char *family, const T *left, const T *right, T *out, unsigned cols, unsigned rows, hipStream_t stream,
                    const PairList &pairs = PairList()) {
    if (!pair_fits_lds<T>(cols, rows)) return fail(XCORR_ERR_UNSUPPORTED, "%s: a %u x %u pair does not fit the LDS of a CU", family, rows, cols);
    // One y shift per task while the tasks are few (at 64x64 fp32 every wavefront slot of the device gets one task: the
    // kernel is bound by the latency of a task, not by LDS throughput), two beyond. Measured, microseconds per launch with
    // one / two y shifts per task: fp32 64x64 6.0 / 6.8, 96x96 17.0 / 14.1, 128x128 46 / 29; fp64 32x32 4.4 / 5.0,
    // 64x64 9.0 / 8.6, 96x96 27 / 19. Eight rows per round instead of four changed nothing.
    constexpr unsigned U = 4;
    const unsigned A = (size_t)cols * rows <= (sizeof(T) == 4 ? 88u * 88u : 40u * 40u) ? 1 : 2;
    const size_t bytes = pair_in_lds_bytes<T>(cols, rows, A, U);
    unsigned grid = 0, waves = 0;
    int rc;
    // the column counts the reference's benchmarks use are compiled in (multiples of 16 whose pitches need no rounding)
    if (A == 1 && cols == 64)
        rc = launch_pair_in_lds<T, 1, U, 64>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else if (A == 1 && cols == 32)
        rc = launch_pair_in_lds<T, 1, U, 32>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else if (A == 1 && cols == 16)
        rc = launch_pair_in_lds<T, 1, U, 16>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else if (A == 1)
        rc = launch_pair_in_lds<T, 1, U, 0>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else if (cols == 64)
        rc = launch_pair_in_lds<T, 2, U, 64>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else if (cols == 96)
        rc = launch_pair_in_lds<T, 2, U, 96>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    else
        rc = launch_pair_in_lds<T, 2, U, 0>(left, right, out, cols, rows, bytes, pairs, &grid, &waves, stream);
    if (rc != XCORR_OK) return rc;
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "%s/pair_in_lds_%s_a%u", family, sizeof(T) == 4 ? "f32" : "f64", A);
    rec.block[0] = 64 * waves, rec.block[1] = rec.block[2] = 1;
    rec.grid[0] = grid, rec.grid[1] = rec.grid[2] = 1;
    rec.shared_mem_bytes = (unsigned)bytes;
    rec.y_shifts_per_thread = A;
    rec.x_shifts_per_thread = PAIR_B;
    rec.left_matrices_per_thread = rec.right_matrices_per_thread = 1;
    rec.lanes_x = rec.lanes_y = 1;
    rec.rows_per_worker = rows;
    rec.distribution_type = XCORR_DIST_NONE;
    rec.blocks_per_cu = 1;
    rec.column_chunks = 1;
    have_last_launch() = true;
    return XCORR_OK;
}

// ------------------------------------------------------------------ warp-per-overlap through LDS
// Block = NW wavefronts; wavefront w owns shift (sx, sy0 + w) for NR right matrices of one
// group. Per pass the block stages `SR` rows x 64 columns of each right matrix and the
// SR + NW - 1 left rows those shifts pair them with (zero outside the matrices, so the sweep
// has no bounds checks), then every wavefront multiplies its own diagonal of row pairs:
// lane = column, one LDS read of the left row and NR reads of right rows per NR FMAs.
// gridDim.z > 1: block z owns the 64-column group z only and adds its sums atomically.
template <typename T, int NR>
__global__ __launch_bounds__(1024) void warp_per_overlap_lds_kernel(const T *__restrict__ left, const T *__restrict__ right,
                                                                     T *__restrict__ out, int W, int H, int n_right, int SR) {
    extern __shared__ __attribute__((aligned(16))) unsigned char wpo_smem[];
    T *Ls = reinterpret_cast<T *>(wpo_smem);                      // [SR + NW - 1][64]
    const int NW = blockDim.y;
    T *Rs = Ls + (size_t)(SR + NW - 1) * 64;                       // [NR][SR][64]
    const int Sx = 2 * W - 1, Sy = 2 * H - 1;
    const int lane = threadIdx.x, w = threadIdx.y;
    const int tid = w * 64 + lane, nthreads = NW * 64;
    const int ox = blockIdx.x % Sx, group = blockIdx.x / Sx;
    const int sx = ox - (W - 1);
    const int sy0 = (int)blockIdx.y * NW - (H - 1);
    const int oy = (int)blockIdx.y * NW + w;
    const int m0 = group * NR;
    const int nr = n_right - m0 < NR ? n_right - m0 : NR;
    // overlap of the block in right-matrix coordinates: columns of this x shift, rows of any of its y shifts
    int xr_lo = sx < 0 ? -sx : 0, xr_hi = W - sx < W ? W - sx : W;
    if (gridDim.z > 1) {
        xr_lo += (int)blockIdx.z * 64;
        if (xr_lo + 64 < xr_hi) xr_hi = xr_lo + 64;
        if (xr_lo >= xr_hi) return;
    }
    const int sy_max = sy0 + NW - 1;
    const int yr_lo = sy_max < 0 ? -sy_max : 0;
    const int yr_hi = H - sy0 < H ? H - sy0 : H;
    T sum[NR];
#pragma unroll
    for (int m = 0; m < NR; ++m) sum[m] = T(0);
    const size_t HW = (size_t)W * H;
    for (int c0 = xr_lo; c0 < xr_hi; c0 += 64) {
        for (int yr0 = yr_lo; yr0 < yr_hi; yr0 += SR) {
            __syncthreads(); // the previous pass is no longer read
            for (int i = tid; i < (SR + NW - 1) * 64; i += nthreads) {
                const int r = i >> 6, c = i & 63;
                const int yl = yr0 + sy0 + r, xr = c0 + c;
                T v = T(0);
                if (yl >= 0 && yl < H && xr < xr_hi) v = left[(size_t)yl * W + (xr + sx)];
                Ls[i] = v;
            }
            for (int i = tid; i < NR * SR * 64; i += nthreads) {
                const int c = i & 63, r = (i >> 6) % SR, m = (i >> 6) / SR;
                const int yr = yr0 + r, xr = c0 + c;
                T v = T(0);
                if (m < nr && yr < yr_hi && xr < xr_hi) v = right[(size_t)(m0 + m) * HW + (size_t)yr * W + xr];
                Rs[i] = v;
            }
            __syncthreads();
            const T *lp = Ls + w * 64 + lane;
            const T *rp = Rs + lane;
#pragma unroll 4
            for (int r = 0; r < SR; ++r) {
                const T l = lp[r * 64];
#pragma unroll
                for (int m = 0; m < NR; ++m) sum[m] += l * rp[(m * SR + r) * 64];
            }
        }
    }
    if (oy >= Sy) return;
#pragma unroll
    for (int m = 0; m < NR; ++m) {
        const T total = wave_sum_to_lane63(sum[m]);
        if (lane == 63 && m < nr) {
            T *p = out + (size_t)(m0 + m) * Sx * Sy + (size_t)oy * Sx + ox;
            if (gridDim.z > 1)
                atomic_add_simple(p, total);
            else
                *p = total;
        }
    }
}

template <typename T, int NR>
static void launch_wpo_lds(const T *left, const T *right, T *out, int W, int H, int n_right, int SR, dim3 grid, dim3 block,
                           size_t lds, hipStream_t stream) {
    warp_per_overlap_lds_kernel<T, NR><<<grid, block, lds, stream>>>(left, right, out, W, H, n_right, SR);
}

// One left matrix against n_right right matrices (reference run_ccn_warp_per_shift_shared_mem,
// naive_warp_per_shift_shared_mem.cu:610-700).
template <typename T>
int run_warp_per_overlap_lds(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_right,
                             const xcorr_params &p, hipStream_t stream) {
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if (n_right == 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "warp_per_overlap_lds: no right matrices");
    // reference limits: naive_warp_per_shift_shared_mem.cu:681-693
    if (p.shifts_per_thread_block > 32)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "Too many shifts per block: %u (max 32)", p.shifts_per_thread_block);
    unsigned nr = p.right_matrices_per_block ? p.right_matrices_per_block : 8; // (the reference's default, one_to_many.hpp:415)
    if (nr > 8) return fail(XCORR_ERR_INVALID_ARGUMENT, "Invalid number of right matrices per block: %u [1-8]", nr);
    if (nr > n_right) nr = n_right; // no bands and FMAs for matrices that do not exist
    unsigned nw = p.shifts_per_thread_block ? p.shifts_per_thread_block : 16;
    if (nw > 16) nw = 16; // a block holds at most 16 wavefronts of 64 lanes
    unsigned sr = p.shared_mem_rows ? p.shared_mem_rows : nw;
    if (sr < nw) return fail(XCORR_ERR_INVALID_ARGUMENT, "Invalid number of shared memory rows [%u], must be greater than shifts per block [%u]", sr, nw);
    // columns are staged 64 at a time (one per lane), whatever shared_mem_row_size asks for; the
    // rows per pass are cut down until the bands fit 64 KB of LDS (the kernel itself works with
    // any number of rows per pass; the rule above is the reference's)
    auto lds_bytes = [&](unsigned r) { return ((size_t)(nr + 1) * r + nw - 1) * 64 * sizeof(T); };
    while (sr > 1 && lds_bytes(sr) > 64 * 1024) sr /= 2;
    const size_t lds = lds_bytes(sr);
    if (lds > 64 * 1024) return fail(XCORR_ERR_UNSUPPORTED, "warp_per_overlap_lds: %zu bytes of LDS needed (max 65536)", lds);
    const unsigned Sx = 2 * cols - 1, Sy = 2 * rows - 1;
    const unsigned groups = (n_right + nr - 1) / nr;
    const unsigned column_groups = p.column_group_per_block ? (cols + 63) / 64 : 1;
    dim3 block(64, nw), grid(Sx * groups, (Sy + nw - 1) / nw, column_groups);
    const int W = (int)cols, H = (int)rows;
    switch (plan_only() ? 0u : nr) {
    case 0: break; // (planning only: the record below is what a launch would report)
    case 1: launch_wpo_lds<T, 1>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 2: launch_wpo_lds<T, 2>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 3: launch_wpo_lds<T, 3>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 4: launch_wpo_lds<T, 4>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 5: launch_wpo_lds<T, 5>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 6: launch_wpo_lds<T, 6>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    case 7: launch_wpo_lds<T, 7>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    default: launch_wpo_lds<T, 8>(left, right, out, W, H, (int)n_right, (int)sr, grid, block, lds, stream); break;
    }
    if (!plan_only()) XCORR_HIP(hipGetLastError());
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "warp_per_overlap_lds/%s_r%u", sizeof(T) == 4 ? "f32" : "f64", nr);
    rec.block[0] = block.x, rec.block[1] = block.y, rec.block[2] = 1;
    rec.grid[0] = grid.x, rec.grid[1] = grid.y, rec.grid[2] = grid.z;
    rec.shared_mem_bytes = (unsigned)lds;
    rec.y_shifts_per_thread = rec.x_shifts_per_thread = 1;
    rec.left_matrices_per_thread = 1;
    rec.right_matrices_per_thread = nr;
    rec.rows_per_worker = sr;
    rec.distribution_type = XCORR_DIST_NONE;
    rec.uses_atomics = column_groups > 1;
    have_last_launch() = true;
    return XCORR_OK;
}

// ------------------------------------------------------------------ block-per-overlap
// One block per shift: wavefront w takes the overlap rows w, w + NW, ..., lanes stride the
// columns; wavefront sums meet in LDS and wavefront 0 adds them in order.
template <typename T>
__global__ __launch_bounds__(1024) void block_per_overlap_kernel(const T *__restrict__ left, const T *__restrict__ right,
                                                                  T *__restrict__ out, int W, int H) {
    __shared__ T partial[16];
    const int Sx = 2 * W - 1;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int ox = blockIdx.x, oy = blockIdx.y;
    const int sx = ox - (W - 1), sy = oy - (H - 1);
    const int xr_lo = sx < 0 ? -sx : 0, xr_hi = W - sx < W ? W - sx : W;
    const int yr_lo = sy < 0 ? -sy : 0, yr_hi = H - sy < H ? H - sy : H;
    T part_sum[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) part_sum[r] = T(0);
    for (int xr = xr_lo + lane; xr < xr_hi; xr += 64) {
        int yr = yr_lo + w;
        for (; yr + 3 * nw < yr_hi; yr += 4 * nw) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                part_sum[r] += left[(size_t)(yr + r * nw + sy) * W + (xr + sx)] * right[(size_t)(yr + r * nw) * W + xr];
        }
        for (; yr < yr_hi; yr += nw) part_sum[0] += left[(size_t)(yr + sy) * W + (xr + sx)] * right[(size_t)yr * W + xr];
    }
    T sum = wave_sum_to_lane63((part_sum[0] + part_sum[1]) + (part_sum[2] + part_sum[3]));
    if (lane == 63) partial[w] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        T total = partial[0];
        for (int i = 1; i < nw; ++i) total += partial[i];
        out[(size_t)oy * Sx + ox] = total;
    }
}

// reference run_ccn_block_per_shift, naive_block_per_shift.cu:127-160
template <typename T>
int run_block_per_overlap(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params &p,
                          hipStream_t stream) {
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    const unsigned asked = p.block_size ? p.block_size : 128; // reference default one_to_one.hpp:649
    if (asked > 1024) return fail(XCORR_ERR_INVALID_ARGUMENT, "Thread block too large: %u (max 1024)", asked);
    unsigned threads = asked / 64 * 64; // whole wavefronts
    if (threads == 0) threads = 64;
    dim3 block(threads), grid(2 * cols - 1, 2 * rows - 1);
    block_per_overlap_kernel<T><<<grid, block, 0, stream>>>(left, right, out, (int)cols, (int)rows);
    XCORR_HIP(hipGetLastError());
    xcorr_launch_record &rec = last_launch();
    memset(&rec, 0, sizeof(rec));
    snprintf(rec.kernel, sizeof(rec.kernel), "block_per_overlap/%s", sizeof(T) == 4 ? "f32" : "f64");
    rec.block[0] = block.x, rec.block[1] = rec.block[2] = 1;
    rec.grid[0] = grid.x, rec.grid[1] = grid.y, rec.grid[2] = 1;
    rec.shared_mem_bytes = 16 * sizeof(T);
    rec.y_shifts_per_thread = rec.x_shifts_per_thread = 1;
    rec.left_matrices_per_thread = rec.right_matrices_per_thread = 1;
    rec.rows_per_worker = rows;
    rec.distribution_type = XCORR_DIST_NONE;
    have_last_launch() = true;
    return XCORR_OK;
}

} // namespace xcorr
