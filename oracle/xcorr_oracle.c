/*
 * CPU oracle for definition-based 2D cross-correlation: test infrastructure only,
 * see xcorr_oracle.h for what it restates and how each function is pinned.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (no -ffast-math: the
 * sequential accumulation order is part of what is restated).
 */
#include "xcorr_oracle.h"

#include <math.h>
#include <stdlib.h>

static inline int imax(int a, int b) { return a > b ? a : b; }
static inline int imin(int a, int b) { return a < b ? a : b; }

/* validate.hpp:94-114: rows outer, columns inner, accumulator of the element type
 * starting at zero, product written target * ref. */
#define DEFINE_HADAMARD(NAME, IN_T, ACC_T)                                                              \
    ACC_T NAME(const IN_T *ref, const IN_T *target, int cols, int rows, int offset_x, int offset_y) {   \
        int x_ref_start = imax(offset_x, 0);                                                            \
        int x_ref_end = imin(cols + offset_x, cols);                                                    \
        int y_ref_start = imax(offset_y, 0);                                                            \
        int y_ref_end = imin(rows + offset_y, rows);                                                    \
        ACC_T sum = 0;                                                                                  \
        for (int y_ref = y_ref_start; y_ref < y_ref_end; ++y_ref) {                                     \
            const IN_T *ref_row = ref + (size_t)y_ref * cols;                                           \
            const IN_T *target_row = target + (size_t)(y_ref - offset_y) * cols;                        \
            for (int x_ref = x_ref_start; x_ref < x_ref_end; ++x_ref) {                                 \
                sum += (ACC_T)target_row[x_ref - offset_x] * (ACC_T)ref_row[x_ref];                     \
            }                                                                                           \
        }                                                                                               \
        return sum;                                                                                     \
    }

DEFINE_HADAMARD(xo_hadamard_and_sum_f32, float, float)
DEFINE_HADAMARD(xo_hadamard_and_sum_f64, double, double)
DEFINE_HADAMARD(xo_hadamard_and_sum_f32_acc64, float, double)

/* validate.hpp:117-132: shifts y in [-hy, hy], x in [-hx, hx], h = (search - 1) / 2,
 * result element (y + hy) * search_x + (x + hx). Restricted to a band of output rows;
 * OpenMP splits output rows only, never a reduction. */
#define DEFINE_ROWS(NAME, HADAMARD, IN_T, OUT_T)                                                        \
    void NAME(const IN_T *ref, const IN_T *target, OUT_T *res, int cols, int rows, int row_begin,       \
              int row_end, int threads) {                                                               \
        int search_x = 2 * cols - 1;                                                                    \
        int search_y = 2 * rows - 1;                                                                    \
        int half_x = (search_x - 1) / 2;                                                                \
        int half_y = (search_y - 1) / 2;                                                                \
        if (row_begin < 0) row_begin = 0;                                                               \
        if (row_end > search_y) row_end = search_y;                                                     \
        if (threads < 1) threads = 1;                                                                   \
        _Pragma("omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)")          \
        for (int oy = row_begin; oy < row_end; ++oy) {                                                  \
            int y = oy - half_y;                                                                        \
            for (int x = -half_x; x <= half_x; ++x) {                                                   \
                res[(size_t)oy * search_x + (size_t)(x + half_x)] = HADAMARD(ref, target, cols, rows, x, y); \
            }                                                                                           \
        }                                                                                               \
    }

DEFINE_ROWS(xo_cross_corr_rows_f32, xo_hadamard_and_sum_f32, float, float)
DEFINE_ROWS(xo_cross_corr_rows_f64, xo_hadamard_and_sum_f64, double, double)
DEFINE_ROWS(xo_cross_corr_rows_f32_acc64, xo_hadamard_and_sum_f32_acc64, float, double)

void xo_naive_cross_corr_f32(const float *ref, const float *target, float *res, int cols, int rows) {
    xo_cross_corr_rows_f32(ref, target, res, cols, rows, 0, 2 * rows - 1, 1);
}
void xo_naive_cross_corr_f64(const double *ref, const double *target, double *res, int cols, int rows) {
    xo_cross_corr_rows_f64(ref, target, res, cols, rows, 0, 2 * rows - 1, 1);
}
void xo_naive_cross_corr_f32_acc64(const float *ref, const float *target, double *res, int cols, int rows) {
    xo_cross_corr_rows_f32_acc64(ref, target, res, cols, rows, 0, 2 * rows - 1, 1);
}

/* validate.hpp:190-214 */
static int check_result(int cols, int rows, int res_cols, int res_rows, int res_count, int expected_count) {
    if (res_cols != 2 * cols - 1 || res_rows != 2 * rows - 1) return XO_ERR_RESULT_SIZE;
    if (res_count != expected_count) return XO_ERR_RESULT_COUNT;
    return XO_OK;
}

#define DEFINE_MODES(SUFFIX, T)                                                                         \
    /* validate.hpp:216-222 */                                                                          \
    int xo_one_to_one_##SUFFIX(const T *ref, const T *target, T *res, int cols, int rows, int res_cols, \
                               int res_rows, int res_count, int threads) {                              \
        int err = check_result(cols, rows, res_cols, res_rows, res_count, 1);                           \
        if (err) return err;                                                                            \
        xo_cross_corr_rows_##SUFFIX(ref, target, res, cols, rows, 0, res_rows, threads);                \
        return XO_OK;                                                                                   \
    }                                                                                                   \
    /* validate.hpp:231-240: result i = ref 0 x target i */                                             \
    int xo_one_to_many_##SUFFIX(const T *ref, const T *target, T *res, int cols, int rows, int n_target, \
                                int res_cols, int res_rows, int res_count, int threads) {               \
        int err = check_result(cols, rows, res_cols, res_rows, res_count, n_target);                    \
        if (err) return err;                                                                            \
        size_t in_area = (size_t)cols * rows, out_area = (size_t)res_cols * res_rows;                   \
        for (int i = 0; i < n_target; ++i)                                                              \
            xo_cross_corr_rows_##SUFFIX(ref, target + i * in_area, res + i * out_area, cols, rows, 0,   \
                                        res_rows, threads);                                             \
        return XO_OK;                                                                                   \
    }                                                                                                   \
    /* validate.hpp:249-270: target t*n + r pairs with ref r, result at the target's index */           \
    int xo_n_to_mn_##SUFFIX(const T *ref, const T *target, T *res, int cols, int rows, int n_ref,       \
                            int n_target, int res_cols, int res_rows, int res_count, int threads) {     \
        int err = check_result(cols, rows, res_cols, res_rows, res_count, n_target);                    \
        if (err) return err;                                                                            \
        if (n_ref <= 0 || n_target % n_ref != 0) return XO_ERR_NOT_DIVISIBLE;                           \
        size_t in_area = (size_t)cols * rows, out_area = (size_t)res_cols * res_rows;                   \
        for (int r = 0; r < n_ref; ++r) {                                                               \
            for (int t = 0; t < n_target / n_ref; ++t) {                                                \
                int t_index = t * n_ref + r;                                                            \
                xo_cross_corr_rows_##SUFFIX(ref + r * in_area, target + t_index * in_area,              \
                                            res + t_index * out_area, cols, rows, 0, res_rows, threads); \
            }                                                                                           \
        }                                                                                               \
        return XO_OK;                                                                                   \
    }                                                                                                   \
    /* validate.hpp:279-290: result r * n_target + t = ref r x target t */                              \
    int xo_n_to_m_##SUFFIX(const T *ref, const T *target, T *res, int cols, int rows, int n_ref,        \
                           int n_target, int res_cols, int res_rows, int res_count, int threads) {      \
        int err = check_result(cols, rows, res_cols, res_rows, res_count, n_ref * n_target);            \
        if (err) return err;                                                                            \
        size_t in_area = (size_t)cols * rows, out_area = (size_t)res_cols * res_rows;                   \
        for (int r = 0; r < n_ref; ++r) {                                                               \
            for (int t = 0; t < n_target; ++t) {                                                        \
                size_t index = (size_t)r * n_target + t;                                                \
                xo_cross_corr_rows_##SUFFIX(ref + r * in_area, target + t * in_area,                    \
                                            res + index * out_area, cols, rows, 0, res_rows, threads);  \
            }                                                                                           \
        }                                                                                               \
        return XO_OK;                                                                                   \
    }

DEFINE_MODES(f32, float)
DEFINE_MODES(f64, double)

/* validate.hpp:134-188. The per-element difference is computed in the element type of
 * `result`; |a| and |b| both <= 1e-5 counts as 0. Max, mean and the square root of the
 * population variance (boost's lazy variance: mean of squares minus squared mean) are
 * taken in double. The reported pair is the first element whose difference equals max. */
#define DEFINE_VALIDATE(NAME, T, FABS)                                                                  \
    int NAME(const T *result, const T *valid, size_t n, xo_validation *out) {                           \
        const T epsilon = (T)1e-5;                                                                      \
        double max = 0.0, sum = 0.0, sum_sq = 0.0;                                                      \
        size_t max_at = 0;                                                                              \
        int have_max = 0;                                                                               \
        for (size_t i = 0; i < n; ++i) {                                                                \
            T a = result[i], b = valid[i], d;                                                           \
            if (FABS(a) <= epsilon && FABS(b) <= epsilon) {                                             \
                d = (T)0;                                                                               \
            } else {                                                                                    \
                T m = FABS(a) > FABS(b) ? FABS(a) : FABS(b);                                            \
                d = FABS(a - b) / m;                                                                    \
            }                                                                                           \
            double dd = (double)d;                                                                      \
            if (!have_max || dd > max) {                                                                \
                max = dd;                                                                               \
                max_at = i;                                                                             \
                have_max = 1;                                                                           \
            }                                                                                           \
            sum += dd;                                                                                  \
            sum_sq += dd * dd;                                                                          \
        }                                                                                               \
        if (n == 0) {                                                                                   \
            out->diff_max = out->diff_mean = out->diff_stddev = NAN;                                    \
            out->at_max_result = out->at_max_valid = NAN;                                               \
            return XO_OK;                                                                               \
        }                                                                                               \
        double mean = sum / (double)n;                                                                  \
        double var = sum_sq / (double)n - mean * mean;                                                  \
        out->diff_max = max;                                                                            \
        out->diff_mean = mean;                                                                          \
        out->diff_stddev = sqrt(var);                                                                   \
        out->at_max_result = (double)result[max_at];                                                    \
        out->at_max_valid = (double)valid[max_at];                                                      \
        return XO_OK;                                                                                   \
    }

DEFINE_VALIDATE(xo_validate_result_f32, float, fabsf)
DEFINE_VALIDATE(xo_validate_result_f64, double, fabs)

#define DEFINE_ERRORS(NAME, A_T, B_T)                                                                   \
    void NAME(const A_T *a, const B_T *b, size_t n, xo_errors *out) {                                   \
        double num = 0.0, den = 0.0, max_abs = 0.0, max_rel = 0.0;                                      \
        for (size_t i = 0; i < n; ++i) {                                                                \
            double x = (double)a[i], y = (double)b[i], d = fabs(x - y);                                 \
            num += d * d;                                                                               \
            den += y * y;                                                                               \
            if (d > max_abs) max_abs = d;                                                               \
            double m = fabs(x) > fabs(y) ? fabs(x) : fabs(y);                                           \
            if (m > 1e-5 && d / m > max_rel) max_rel = d / m;                                           \
        }                                                                                               \
        out->rel_frobenius = den > 0.0 ? sqrt(num / den) : sqrt(num);                                   \
        out->max_abs = max_abs;                                                                         \
        out->max_rel = max_rel;                                                                         \
    }

DEFINE_ERRORS(xo_errors_f32, float, float)
DEFINE_ERRORS(xo_errors_f64, double, double)
DEFINE_ERRORS(xo_errors_f32_vs_f64, float, double)

/* matrix.hpp:614-618 */
unsigned xo_interleave_index(unsigned idx, unsigned num_matrices, unsigned group_size) {
    unsigned group_offset = idx % group_size;
    unsigned group_start = num_matrices / group_size;
    return group_offset * group_start + idx / group_size;
}

/* ---- row_distribution.cuh ---- */

static unsigned div_up(unsigned a, unsigned b) { return (a + b - 1) / b; }

/* row_distribution.cuh:26-33, instantiated with int */
static int quadratic_i(int a, int b, int c, int x) { return a * x * x + b * x + c; }

/* row_distribution.cuh:38-83 */
static unsigned tri_top_row(unsigned r, unsigned search_rows) { return search_rows % (2 * r); }
static unsigned tri_total_rows(unsigned r, unsigned matrix_rows) { return div_up(matrix_rows, r); }
static unsigned tri_first_worker_on_row(int r, int t, int worker_row) {
    return (unsigned)quadratic_i(r, -(3 * r - t), 2 * r - t, worker_row);
}

unsigned xo_dist_num_workers(int dist, unsigned max_rows_per_worker, unsigned matrix_rows, unsigned search_rows) {
    switch (dist) {
    case 0: /* row_distribution.cuh:264-270 */
        return search_rows;
    case 1: /* row_distribution.cuh:222-228 */
        return search_rows * div_up(matrix_rows, max_rows_per_worker);
    default: { /* row_distribution.cuh:71-83 */
        unsigned t = tri_top_row(max_rows_per_worker, search_rows);
        unsigned total = tri_total_rows(max_rows_per_worker, matrix_rows);
        return tri_first_worker_on_row((int)max_rows_per_worker, (int)t, (int)total + 1);
    }
    }
}

xo_assigned_work xo_dist_distribute_rows(int dist, unsigned worker_y_index, unsigned max_rows_per_worker,
                                         unsigned matrix_rows, unsigned search_rows) {
    xo_assigned_work w;
    if (dist == 0) { /* row_distribution.cuh:272-283 */
        w.output_row = worker_y_index;
        w.worker_idx = 0;
        w.workers_for_row = worker_y_index < search_rows ? 1u : 0u;
        return w;
    }
    if (dist == 1) { /* row_distribution.cuh:230-246 */
        unsigned center_row = search_rows / 2;
        unsigned output_row = worker_y_index % search_rows;
        unsigned dist_from_center = (unsigned)abs((int)output_row - (int)center_row);
        w.output_row = output_row;
        w.worker_idx = worker_y_index / search_rows;
        w.workers_for_row = div_up(matrix_rows - dist_from_center, max_rows_per_worker);
        return w;
    }
    /* row_distribution.cuh:93-204: unsigned 32-bit arithmetic and single-precision
     * square root exactly as written there */
    uint32_t r = max_rows_per_worker;
    uint32_t t = tri_top_row(r, search_rows);
    uint32_t total_worker_rows = tri_total_rows(r, matrix_rows);
    uint32_t i = worker_y_index;
    uint32_t tmp3r_t = 3 * r - t;
    uint32_t disc = tmp3r_t * tmp3r_t - 4 * r * (2 * r - t - i);
    float numerator = (float)tmp3r_t + sqrtf((float)disc);
    uint32_t worker_row = (uint32_t)floorf(numerator / (float)(2 * r));
    if (worker_row > total_worker_rows) {
        w.output_row = search_rows;
        w.worker_idx = 0;
        w.workers_for_row = 0;
        return w;
    }
    uint32_t first = (uint32_t)quadratic_i((int)r, (int)(0u - tmp3r_t), (int)(2 * r - t), (int)worker_row);
    uint32_t in_worker_row_offset = worker_y_index - first;
    uint32_t worker_row_row_offset = (total_worker_rows - worker_row) * r;
    uint32_t worker_output_row = worker_row_row_offset + in_worker_row_offset;
    uint32_t center_row = search_rows / 2;
    uint32_t dist_from_center = (uint32_t)abs((int)worker_output_row - (int)center_row);
    w.output_row = worker_output_row;
    w.worker_idx = total_worker_rows - worker_row;
    w.workers_for_row = div_up(matrix_rows - dist_from_center, r);
    return w;
}
