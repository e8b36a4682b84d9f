/*
 * CPU oracle for definition-based 2D cross-correlation.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker the HIP path is compared
 * against; nothing that ships (the C-ABI library, the `cross` host binary's GPU
 * algorithms) may call it. Only tests, the smoke check and the benchmark's CPU
 * baseline leg load it.
 *
 * It restates, in plain C, the host cross-correlation of the reference
 * (repo/cross-corr/src/validate.hpp) with the same accumulation order and
 * accumulator type, the reference's result-matrix index maps for the four input
 * modes, its element-wise validation statistic, the n_to_mn interleave index map
 * (matrix.hpp:614-618) and the split-row worker maps (row_distribution.cuh).
 *
 * How each function is pinned (no reference test, golden vector or fixture exists
 * for this path, and the reference headers cannot be compiled here: they need
 * Boost and the CUDA runtime headers):
 *   xo_hadamard_and_sum_*, xo_naive_cross_corr_* : closed forms (all-ones, delta,
 *       corner and centre elements), identity with scipy.signal.correlate2d on
 *       committed fixtures, a 4-loop brute force written from the textbook
 *       definition, the flip symmetry xcorr(a,b)[y][x] == xcorr(b,a)[Sy-1-y][Sx-1-x]
 *       and linearity.
 *   xo_one_to_one_* .. xo_n_to_m_* : constant-valued matrices that identify the
 *       (left, right) pair of every result matrix; the n_to_mn file order
 *       t*n + r is fixed by the reference's source text only (validate.hpp:264-269).
 *   xo_validate_result_* : hand-computed cases incl. the 1e-5 double-zero rule.
 *   xo_dist_* : brute-force coverage property (every overlap row of every output
 *       row is assigned to exactly one active worker).
 *   xo_interleave_index : permutation property and the explicit n=2, m=3 table.
 * Accumulation ORDER and TYPE (y outer, x inner, T accumulator, target*ref) are
 * fixed by validate.hpp:102-111 read as text; no executable check can pin the
 * low-order bits that follow from them.
 */
#ifndef XCORR_ORACLE_H
#define XCORR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes of the mode drivers (the reference throws std::runtime_error) */
#define XO_OK 0
#define XO_ERR_RESULT_SIZE 1   /* validate.hpp:194-203 */
#define XO_ERR_RESULT_COUNT 2  /* validate.hpp:205-214 */
#define XO_ERR_NOT_DIVISIBLE 3 /* validate.hpp:254-261 */
#define XO_ERR_SIZE_MISMATCH 4 /* validate.hpp:135-137 */

/* validate.hpp:94-114. ref/target are rows x cols row-major, offsets are shifts. */
float xo_hadamard_and_sum_f32(const float *ref, const float *target, int cols, int rows, int offset_x, int offset_y);
double xo_hadamard_and_sum_f64(const double *ref, const double *target, int cols, int rows, int offset_x, int offset_y);
/* same products, accumulated in double (rounding-free yardstick for fp32 inputs; not in the reference) */
double xo_hadamard_and_sum_f32_acc64(const float *ref, const float *target, int cols, int rows, int offset_x, int offset_y);

/* validate.hpp:117-132. res is (2*rows-1) x (2*cols-1). */
void xo_naive_cross_corr_f32(const float *ref, const float *target, float *res, int cols, int rows);
void xo_naive_cross_corr_f64(const double *ref, const double *target, double *res, int cols, int rows);
void xo_naive_cross_corr_f32_acc64(const float *ref, const float *target, double *res, int cols, int rows);

/* Output rows [row_begin, row_end) of the same result only (res still points at the
 * full result matrix). threads > 1 splits the output rows over OpenMP threads; every
 * element keeps the sequential accumulation order, so results are bit-identical. */
void xo_cross_corr_rows_f32(const float *ref, const float *target, float *res, int cols, int rows, int row_begin, int row_end, int threads);
void xo_cross_corr_rows_f64(const double *ref, const double *target, double *res, int cols, int rows, int row_begin, int row_end, int threads);
void xo_cross_corr_rows_f32_acc64(const float *ref, const float *target, double *res, int cols, int rows, int row_begin, int row_end, int threads);

/* validate.hpp:216-298. Matrices of an array are contiguous. res_* describe the
 * caller's result array so that the reference's size/count checks can be restated.
 * threads parallelises over output rows inside each pair (bit-identical). */
int xo_one_to_one_f32(const float *ref, const float *target, float *res, int cols, int rows, int res_cols, int res_rows, int res_count, int threads);
int xo_one_to_many_f32(const float *ref, const float *target, float *res, int cols, int rows, int n_target, int res_cols, int res_rows, int res_count, int threads);
int xo_n_to_mn_f32(const float *ref, const float *target, float *res, int cols, int rows, int n_ref, int n_target, int res_cols, int res_rows, int res_count, int threads);
int xo_n_to_m_f32(const float *ref, const float *target, float *res, int cols, int rows, int n_ref, int n_target, int res_cols, int res_rows, int res_count, int threads);
int xo_one_to_one_f64(const double *ref, const double *target, double *res, int cols, int rows, int res_cols, int res_rows, int res_count, int threads);
int xo_one_to_many_f64(const double *ref, const double *target, double *res, int cols, int rows, int n_target, int res_cols, int res_rows, int res_count, int threads);
int xo_n_to_mn_f64(const double *ref, const double *target, double *res, int cols, int rows, int n_ref, int n_target, int res_cols, int res_rows, int res_count, int threads);
int xo_n_to_m_f64(const double *ref, const double *target, double *res, int cols, int rows, int n_ref, int n_target, int res_cols, int res_rows, int res_count, int threads);

/* validate.hpp:134-188: element-wise relative difference statistic. */
typedef struct xo_validation {
    double diff_max;
    double diff_mean;
    double diff_stddev;
    double at_max_result; /* element of `result` where the max difference occurs */
    double at_max_valid;  /* element of `valid` at the same position */
} xo_validation;
int xo_validate_result_f32(const float *result, const float *valid, size_t n, xo_validation *out);
int xo_validate_result_f64(const double *result, const double *valid, size_t n, xo_validation *out);

/* error measures the build reports next to the reference's statistic */
typedef struct xo_errors {
    double rel_frobenius; /* ||a-b||_F / ||b||_F */
    double max_abs;
    double max_rel;       /* max |a-b| / max(|a|,|b|) over elements that are not both tiny */
} xo_errors;
void xo_errors_f32(const float *a, const float *b, size_t n, xo_errors *out);
void xo_errors_f64(const double *a, const double *b, size_t n, xo_errors *out);
void xo_errors_f32_vs_f64(const float *a, const double *b, size_t n, xo_errors *out);

/* matrix.hpp:614-618: slot of file matrix idx after de-interleaving groups of group_size */
unsigned xo_interleave_index(unsigned idx, unsigned num_matrices, unsigned group_size);

/* row_distribution.cuh: split-row worker maps. dist: 0 none, 1 rectangle, 2 triangle */
typedef struct xo_assigned_work {
    unsigned output_row;
    unsigned worker_idx;
    unsigned workers_for_row;
} xo_assigned_work;
unsigned xo_dist_num_workers(int dist, unsigned max_rows_per_worker, unsigned matrix_rows, unsigned search_rows);
xo_assigned_work xo_dist_distribute_rows(int dist, unsigned worker_y_index, unsigned max_rows_per_worker, unsigned matrix_rows, unsigned search_rows);

#ifdef __cplusplus
}
#endif
#endif
