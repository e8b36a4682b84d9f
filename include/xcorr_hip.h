/*
 * xcorr_hip.h - C ABI of libxcorr_hip.so: definition-based 2D cross-correlation
 * on AMD MI355X (gfx950), hand-written HIP kernels.
 *
 * The entry points replace the launcher functions of the reference's
 * repo/cross-corr/src/kernels.cuh (the `run_*` templates, lines 41-283) one for
 * one: plain pointers to caller-owned device memory, sizes, tuning integers and a
 * stream. Like the reference launchers they neither allocate nor copy nor
 * synchronise; the launch is asynchronous on `stream` (NULL = the default stream).
 *
 * Conventions shared by every compute entry point
 *   - matrices are dense row-major `rows x cols`; the matrices of an array are
 *     contiguous (reference matrix.hpp:590-595); left and right matrices have the
 *     same size (validate.hpp:94-101 assumes it);
 *   - every result matrix is `(2*rows-1) x (2*cols-1)`; element (oy, ox) is the
 *     shift (oy-(rows-1), ox-(cols-1)):
 *         out[oy][ox] = sum over (y, x) of left[y+sy][x+sx] * right[y][x]
 *     which equals the reference host result validate.hpp:117-132 with
 *     ref = left, target = right;
 *   - return value: XCORR_OK or an error code; the message is available from
 *     xcorr_last_error(). Where the reference launcher throws
 *     std::runtime_error for a tuning value (e.g.
 *     naive_shuffle_multirow_both.cu:645-665) the entry point returns
 *     XCORR_ERR_INVALID_ARGUMENT with an equivalent message. Nothing throws
 *     across this boundary;
 *   - a tuning field of xcorr_params set to 0 selects the library's tuned default;
 *   - after a successful launch the geometry actually used is available from
 *     xcorr_last_launch() (reference kernel_args.hpp:9-33, one record per process
 *     there; here one per host thread, like the error message);
 *   - `left`, `right` and `out` are ordinary device allocations (hipMalloc /
 *     xcorr_malloc: coarse-grained memory of the current device). Launches that
 *     split a reduction add partial sums with the hardware's floating-point
 *     atomic add (xcorr_last_launch().uses_atomics == 1: the split-row families
 *     always; the grouped families, xcorr_shuffle and the plain xcorr_multimat_right
 *     when the launcher cuts the reduction to fill the device, clearing `out` itself). That instruction is only defined on coarse-grained memory -
 *     on fine-grained, host-mapped or managed allocations it is silently dropped -
 *     and the order of the additions, hence the last bits of such a result, varies
 *     from run to run. rows_per_thread >= rows together with column_chunks = 1
 *     asks a grouped family for the launch without atomics, distribution_type =
 *     XCORR_DIST_NONE asks xcorr_shuffle / the plain xcorr_multimat_right for it;
 *     its result is the same bits every run;
 *   - host threads may launch side by side (error text, launch record and plan cache
 *     are per thread); the library keeps per-device facts for up to 64 devices and
 *     always works on the calling thread's current device.
 */
#ifndef XCORR_HIP_H
#define XCORR_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XCORR_OK 0
#define XCORR_ERR_INVALID_ARGUMENT 1 /* bad tuning value or shape (reference: std::runtime_error) */
#define XCORR_ERR_RUNTIME 2          /* a HIP runtime call failed (reference: CUCH, cuda_helpers.cuh:13-24) */
#define XCORR_ERR_UNSUPPORTED 3      /* combination this build has no kernel for */

/* reference row_distribution.cuh:9-13 */
#define XCORR_DIST_DEFAULT 0
#define XCORR_DIST_NONE 1
#define XCORR_DIST_RECTANGLE 2
#define XCORR_DIST_TRIANGLE 3

/* variants of the warp-per-overlap family (reference naive_warp_per_shift.cu) */
#define XCORR_WPO_BASE 0              /* run_ccn_warp_per_shift, kernels.cuh:99-107 */
#define XCORR_WPO_SIMPLE_INDEXING 1   /* run_ccn_warp_per_shift_simple_indexing, kernels.cuh:109-117 */
#define XCORR_WPO_WORK_DISTRIBUTION 2 /* run_ccn_warp_per_shift_work_distribution, kernels.cuh:119-128 */

/*
 * Tuning integers, named after the reference's per-algorithm JSON keys
 * (one_to_one.hpp:739-741, n_to_m.hpp:321-325, n_to_m.hpp:475-479, ...). The
 * reference counts 32-lane warps and instantiates one kernel per value; this
 * library runs a short list of gfx950 tiles on 64-lane wavefronts. All integers are
 * checked against the reference's release limits (CMakeLists.txt:16-46; larger
 * values are rejected as there). 0 leaves a choice to the library's cost model.
 * A non-zero shifts_per_thread / shifts_per_thread_right_matrix,
 * right_matrices_per_thread or left_matrices_per_thread is an exact request: the
 * launch uses the compiled tile with the nearest value at or above it (y shifts per
 * lane: 4 or 8; matrices per lane position = matrices per lane x lanes laid over
 * matrices: 1, 4, 8, 16; the distances of the three requests add up), and among
 * equally near tiles the one the cost model rates fastest. left_rows_per_iteration and
 * warps_per_thread_block have no counterpart in these kernels (every tile stages its
 * own band height and runs four wavefronts per block) and are only validated.
 * The tile actually used is reported by xcorr_last_launch(). The geometry fields
 * further down select a tile exactly.
 */
typedef struct xcorr_params {
    unsigned struct_size;                    /* sizeof(xcorr_params) as the CALLER's header declares it (XCORR_PARAMS_INIT sets it).
                                                The library reads that many bytes and takes fields it knows beyond them as 0, so a
                                                caller built against an older header keeps working when fields are appended; 0 is
                                                rejected (a struct laid out before this field existed starts with
                                                warps_per_thread_block, usually 0) */
    unsigned warps_per_thread_block;         /* <= 32 */
    unsigned shifts_per_thread_block;        /* <= 32, warp-per-overlap family */
    unsigned rows_per_thread;                /* split-row contract: max overlap rows per worker (JSON rows_per_thread / rows_per_warp);
                                                0: the library picks the chunk */
    unsigned distribution_type;              /* XCORR_DIST_* */
    unsigned shifts_per_thread;              /* grouped-overlap, <= 8 */
    unsigned left_rows_per_iteration;        /* grouped-overlap <= 8, combined kernels <= 4 */
    unsigned right_matrices_per_thread;      /* <= 8, combined kernels <= 4 */
    unsigned left_matrices_per_thread;       /* <= 8, combined kernels <= 4 */
    unsigned shifts_per_thread_right_matrix; /* combined kernels, <= 4 */
    unsigned warp_per_overlap_variant;       /* XCORR_WPO_* */
    /* gfx950 tile geometry, no counterpart in the reference; 0 = tuned default */
    unsigned x_shifts_per_thread;            /* adjacent x shifts one lane accumulates: 4 or 8 */
    unsigned lanes_x;                        /* lanes of a wavefront laid along x shifts (power of two) */
    unsigned lanes_y;                        /* lanes laid along y shifts; the rest are laid over matrices */
    unsigned specialisation;                 /* 1-based index into the compiled tile list of the dtype (tuning sweeps) */
    /* warp-per-overlap through LDS (one_to_one.hpp:568-572) and block-per-overlap (one_to_one.hpp:649) */
    unsigned shared_mem_row_size;            /* columns staged per pass; this build always stages 64 (one per lane) */
    unsigned shared_mem_rows;                /* right rows staged per pass; 0 = shifts_per_thread_block, smaller is an error */
    unsigned right_matrices_per_block;       /* 0 = 8 (never more than there are); <= 8 */
    unsigned strided_load;                   /* load pattern of the reference's staging; no effect here */
    unsigned column_group_per_block;         /* 1: one block per group of 64 columns, sums added atomically (caller zeroes `out`) */
    unsigned block_size;                     /* block-per-overlap: threads per block, 0 = 128, <= 1024 */
    unsigned column_chunks;                  /* engine families: cut the reduction over right columns into this many chunks
                                                (atomic adds, like rows_per_thread for rows); 0 = planner decides, no counterpart in the reference */
    unsigned whole_pair_in_lds;              /* few small matrices (see "Few small matrices" below): 0 = the launcher decides, 1 = always
                                                run the kernel that keeps both matrices of a pair in LDS (an error if they do not
                                                fit), 2 = never; no counterpart in the reference */
    unsigned matrix_cores;                   /* engine families: 0 = the launcher decides between its register tiles (vector FMA) and
                                                its matrix-core tiles (v_mfma), 1 = matrix-core tiles only, 2 = never; the one-output-row
                                                launchers (shuffle, split_row, multimat_right, multimat_both) take a matrix-core tile
                                                under their own contract when no tile geometry and no chunk below 16 rows is named
                                                and the launch is large enough; no counterpart in the reference */
} xcorr_params;
/* xcorr_params p = XCORR_PARAMS_INIT;  - every tuning field 0 (the library's choice), struct_size set */
#define XCORR_PARAMS_INIT {sizeof(xcorr_params)}

/* Geometry of the most recent launch (reference kernel_args.hpp:9-33 plus the
 * template parameters each launcher records, e.g. naive_shuffle_multirow_both.cu:488-522). */
typedef struct xcorr_launch_record {
    char kernel[64];
    unsigned block[3];
    unsigned grid[3];
    unsigned shared_mem_bytes;
    unsigned y_shifts_per_thread;
    unsigned x_shifts_per_thread;
    unsigned left_matrices_per_thread;
    unsigned right_matrices_per_thread;
    unsigned lanes_x, lanes_y, lanes_left, lanes_right; /* how the 64 lanes are laid out */
    unsigned waves_x, waves_y;
    unsigned rows_per_worker;  /* left rows one work item reduces over */
    unsigned distribution_type;
    unsigned uses_atomics;     /* 1: partial sums are added with float atomics into a zeroed output */
    unsigned blocks_per_cu;    /* workgroups of this kernel one CU holds at a time (0: not recorded) */
    unsigned column_chunks;    /* chunks the reduction over right columns is cut into (1: not cut) */
    unsigned matrix_cores;     /* 1: the kernel multiplies on the matrix cores (v_mfma), 0: vector FMAs */
    float predicted_us;        /* run time the launcher's model expected for the plan it chose (grouped engine families; 0: none) */
} xcorr_launch_record;

typedef struct xcorr_device_info {
    char name[128];
    char arch[32];
    int compute_units;
    int clock_khz;        /* engine clock */
    int memory_clock_khz;
    int memory_bus_bits;
    int lds_bytes_per_block;
    size_t global_mem_bytes;
    double fp32_vector_peak_tflops; /* CUs x 4 SIMD x 16 lanes x 2 (packed) x 2 FLOP x clock */
    double fp64_vector_peak_tflops; /* CUs x 4 SIMD x 16 lanes x 2 FLOP x clock */
} xcorr_device_info;

/* ---- status ---- */
const char *xcorr_last_error(void);
int xcorr_last_launch(xcorr_launch_record *out);
int xcorr_device_info_get(xcorr_device_info *out);
const char *xcorr_version(void);
/* Planning without launching (per host thread; no counterpart in the reference): while on, the entry points of the
 * sliding-window engine (xcorr_shuffle ... xcorr_multimat_both_grouped) validate their arguments, choose kernel and
 * geometry, fill the launch record and return without launching or reading the pointers. Works without a GPU (256
 * CUs and the occupancies of an MI355X are assumed then); for tools and tests that ask what a call would run.
 * on = 2 plans as if `out` were memory the floating-point atomic add is not defined on (host-mapped, managed): a launch
 * that names no chunk stays whole (plain stores), one whose chunk the caller fixed is refused. */
int xcorr_plan_only(int on);

/* ---- memory / queue shims: the C++ host never includes the HIP headers.
 * They stand in for the reference's cuda_helpers.cuh:26-97 (cuda_malloc,
 * cuda_memcpy_to_device, cuda_memcpy_from_device, cuda_memset, cuda_free),
 * allocator.cuh:16-86 (pinned host memory) and stopwatch.hpp:236-301 (events). ---- */
int xcorr_malloc(void **dev_ptr, size_t bytes);
int xcorr_free(void *dev_ptr);
int xcorr_memset_async(void *dev_ptr, int value, size_t bytes, void *stream);
/* plain device-to-device copy KERNEL (16 bytes per lane), no reference counterpart: a launch of
 * known read and write size against which memory-traffic counters are calibrated */
int xcorr_copy_kernel(void *dev_dst, const void *dev_src, size_t bytes, void *stream);
int xcorr_memcpy_h2d(void *dev_dst, const void *host_src, size_t bytes);
int xcorr_memcpy_d2h(void *host_dst, const void *dev_src, size_t bytes);
int xcorr_memcpy_h2d_async(void *dev_dst, const void *host_src, size_t bytes, void *stream);
int xcorr_memcpy_d2h_async(void *host_dst, const void *dev_src, size_t bytes, void *stream);
int xcorr_host_alloc_pinned(void **host_ptr, size_t bytes);
int xcorr_host_free(void *host_ptr);
int xcorr_stream_create(void **stream);
int xcorr_stream_destroy(void *stream);
int xcorr_stream_sync(void *stream);
int xcorr_device_sync(void);
/* ---- HIP graphs: launch-bound sequences (many small instances) are captured once and replayed.
 * No counterpart in the reference. Every entry point above may be called on a capturing stream
 * (after one eager call of the same family and element type, so that one-time set-up is not
 * captured); clear buffers with xcorr_clear_async (a kernel), not xcorr_memset_async, inside a
 * capture. The stream must not be the NULL stream. ---- */
int xcorr_clear_async(void *dev_ptr, size_t bytes, void *stream); /* bytes: multiple of 4 */
int xcorr_graph_capture_begin(void *stream);
int xcorr_graph_capture_end(void *stream, void **graph_exec);
int xcorr_graph_launch(void *graph_exec, void *stream);
int xcorr_graph_destroy(void *graph_exec);

int xcorr_event_create(void **event);
int xcorr_event_record(void *event, void *stream);
int xcorr_event_sync(void *event);
int xcorr_event_elapsed_ms(void *start, void *stop, float *ms);
int xcorr_event_destroy(void *event);

/* ---- compute entry points ---- */

/* Overlap-wise: one thread per shift, serial loop over the overlap.
 * Replaces run_cross_corr_naive_original (kernels.cuh:41-51, naive_original.cu:130-161):
 * `n_left` = subregions_per_pic, `batch` = batch_size. Right matrix b*n_left + i is
 * correlated with left matrix i; the result has the right matrix's index. */
int xcorr_overlap_wise_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                           unsigned n_left, unsigned batch, void *stream);
int xcorr_overlap_wise_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                           unsigned n_left, unsigned batch, void *stream);
/* The same kernel over all pairs in one launch: every right matrix with every left matrix,
 * result index = left * n_right + right (the n_to_m mode). The reference's host reaches
 * that with one launch per left matrix on num_cuda_streams streams (n_to_m.hpp:198-212);
 * it has no such launcher. */
int xcorr_overlap_wise_all_pairs_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                     unsigned n_left, unsigned n_right, void *stream);
int xcorr_overlap_wise_all_pairs_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                     unsigned n_left, unsigned n_right, void *stream);

/* Warp-per-overlap: one wavefront per shift, lanes stride the overlap, DPP reduction.
 * Replaces run_ccn_warp_per_shift, run_ccn_warp_per_shift_simple_indexing and
 * run_ccn_warp_per_shift_work_distribution (kernels.cuh:99-128). One pair.
 * Uses p->shifts_per_thread_block, p->warp_per_overlap_variant and, for the
 * work-distribution variant (caller zeroes `out` first, as one_to_one.hpp:476-489),
 * p->rows_per_thread and p->distribution_type. */
int xcorr_warp_per_overlap_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                               const xcorr_params *p, void *stream);
int xcorr_warp_per_overlap_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                               const xcorr_params *p, void *stream);

/* Warp-per-overlap through LDS: the wavefronts of a block own consecutive y shifts of
 * one x shift and share staged row chunks of the left matrix and of up to eight right
 * matrices. Replaces run_ccn_warp_per_shift_shared_mem (kernels.cuh:144-161). One left
 * matrix against `n_right` right matrices, result i belongs to right matrix i. Uses
 * p->shifts_per_thread_block (<= 32; at most 16 wavefronts fit a block),
 * p->shared_mem_rows, p->right_matrices_per_block and p->column_group_per_block
 * (then the caller zeroes `out` first, as one_to_one.hpp:600-605). */
int xcorr_warp_per_overlap_lds_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                   unsigned n_right, const xcorr_params *p, void *stream);
int xcorr_warp_per_overlap_lds_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                   unsigned n_right, const xcorr_params *p, void *stream);

/* Block-per-overlap: all wavefronts of a block reduce one shift together.
 * Replaces run_ccn_block_per_shift (kernels.cuh:197-205). One pair. Uses p->block_size. */
int xcorr_block_per_overlap_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                const xcorr_params *p, void *stream);
int xcorr_block_per_overlap_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                const xcorr_params *p, void *stream);

/* Few small matrices. A launch is short of work for 256 CUs when its matrices are few and small, and what it costs then is
 * the number of kernels it takes and the latency of one block. xcorr_shuffle, xcorr_split_row, xcorr_multimat_right(_groups),
 * xcorr_multimat_both, xcorr_grouped_overlap, xcorr_multimat_right_grouped, xcorr_multimat_both_grouped, the work-distribution
 * variant of xcorr_warp_per_overlap and xcorr_warp_per_overlap_lds therefore hand such a launch to one kernel of another kind when the call names no tile, no
 * chunk of rows or columns and none of the LDS family's staging sizes: every block keeps both matrices of ITS pair whole in
 * LDS and its wavefronts reduce groups of four adjacent x shifts over all rows (the role of run_ccn_warp_per_shift_shared_mem,
 * kernels.cuh:144-161, at such sizes). One launch, plain stores, the same bits every run: `out` need not be zeroed whatever
 * the family's contract says (xcorr_last_launch().uses_atomics == 0; a caller that plans first - xcorr_plan_only - may skip
 * its clear, the `cross` binary does). Taken for one pair up to 96 x 96 fp32 / 64 x 64 fp64, and for at most 64 pairs of up to
 * 32 x 32 with at most 2^24 multiply-adds in all; p->whole_pair_in_lds = 1 forces it (any number of pairs that fit), 2 keeps the
 * family's own kernels. */

/* Sliding-window base: every lane owns adjacent x shifts of one output row.
 * Replaces run_ccn_shuffle (kernels.cuh:65-73). One pair. Uses p->warps_per_thread_block. */
int xcorr_shuffle_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                      const xcorr_params *p, void *stream);
int xcorr_shuffle_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                      const xcorr_params *p, void *stream);

/* Split-row: the overlap rows of an output row are split over several workers of at
 * most p->rows_per_thread rows each, partial sums are added atomically.
 * Replaces run_ccn_shuffle_work_distribution<DIST> (kernels.cuh:75-85). One pair.
 * THE CALLER ZEROES `out` FIRST (reference one_to_one.hpp:276-277). A launch that ends up with one work item per result tile
 * (rows left whole, columns not cut) stores instead of adding: xcorr_last_launch().uses_atomics tells, also from a planning call. */
int xcorr_split_row_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                        const xcorr_params *p, void *stream);
int xcorr_split_row_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                        const xcorr_params *p, void *stream);

/* Grouped-overlap: every lane accumulates p->shifts_per_thread adjacent y shifts.
 * Replaces run_ccn_shuffle_multirow_both (kernels.cuh:185-195). One pair.
 * `out` need not be zeroed: when the launcher splits the reduction to fill the
 * device it clears `out` itself on `stream` first. A small pair given no tile
 * selection runs whole in LDS ("Few small matrices" above). */
int xcorr_grouped_overlap_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                              const xcorr_params *p, void *stream);
int xcorr_grouped_overlap_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                              const xcorr_params *p, void *stream);

/* The same launcher with the chunks of a split reduction added IN ORDER instead of atomically. No counterpart in the
 * reference; for callers that can neither allocate nor tolerate run-to-run differences: code under HIP graph capture,
 * serving loops, harnesses that compare bits. Arguments and results as xcorr_grouped_overlap_f32 (same tiles, same
 * choice of chunk; `out` need not be zeroed and is not cleared), but
 *   - the launch never uses atomic adds (xcorr_last_launch().uses_atomics == 0): chunk 0 of a result tile stores, every
 *     later chunk waits for its predecessor's ticket and adds itself on top, so every output is summed in the same order
 *     every run: the same bits every run, at the speed of the split launch (a pair of 1024 x 1024: about 1 % slower);
 *   - the tickets (32 bits per result tile of the launch) live in a fixed 4 MiB array inside the library's code object,
 *     one copy per device, held until the process ends. The entry point allocates nothing and frees nothing. Launches
 *     whose tiles outnumber the array (1 048 576: beyond any single pair of 16384 x 16384) return XCORR_ERR_UNSUPPORTED;
 *   - all calls on one device share that array, which is cleared (by a kernel on `stream`) at the start of every call:
 *     calls of this entry point that overlap in time on one device - different streams, different host threads - race
 *     and give wrong results; calls on one stream, or otherwise ordered one after the other, are safe;
 *   - `out` must be ordinary device memory that every compute unit reads and writes coherently through memory
 *     (hipMalloc); only the matrix-core tiles run this way (matrix_cores = 2 is refused, column_chunks must be 0 or 1).
 * A small pair that the launcher serves with the whole-pair-in-LDS kernel, and launches that do not split, run exactly as
 * under xcorr_grouped_overlap_f32 (they never used atomics). */
int xcorr_grouped_overlap_ordered_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                      const xcorr_params *p, void *stream);

/* Multi-matrix-right: one left matrix against n_right right matrices, each lane
 * reuses a left value for p->right_matrices_per_thread right matrices.
 * Replaces run_ccn_shuffle_multimat_right_work_distribution<DIST> (kernels.cuh:130-142;
 * THE CALLER ZEROES `out`) when p->rows_per_thread > 0 or p->distribution_type is
 * rectangle or triangle (rows_per_thread 0 then leaves the chunk to the library), and
 * run_ccn_shuffle_multimat_right (kernels.cuh:87-97; `out` need not be zeroed)
 * otherwise. Result i = left x right i. */
int xcorr_multimat_right_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                             unsigned n_right, const xcorr_params *p, void *stream);
int xcorr_multimat_right_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                             unsigned n_right, const xcorr_params *p, void *stream);

/* Multi-matrix-right over n_left groups in one launch: left l against the right matrices
 * [l*n_right, (l+1)*n_right) (the de-interleaved order of n_to_mn.hpp:165-172), result
 * index = right index; the same results as n_left calls of xcorr_multimat_right on the
 * consecutive groups, with the same meaning of p (p->rows_per_thread > 0: caller zeroes
 * `out`). The reference has no such launcher: its host issues one launch per left
 * matrix on num_cuda_streams streams (n_to_mn.hpp:228-300); on this device the launch
 * overhead of that loop dominates small matrices. */
int xcorr_multimat_right_groups_f32(const float *left, const float *right, float *out, unsigned cols,
                                    unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                    void *stream);
int xcorr_multimat_right_groups_f64(const double *left, const double *right, double *out, unsigned cols,
                                    unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                    void *stream);

/* Multi-matrix-right x grouped-overlap.
 * Replaces run_ccn_shuffle_one_to_many_multirow_both_multimat_right (kernels.cuh:221-234).
 * Extension: n_left > 1 runs the n_to_mn mode in one launch, left l against the
 * right matrices [l*n_right, (l+1)*n_right) (the de-interleaved order of
 * n_to_mn.hpp:165-172), result index = right index. `out` need not be zeroed. */
int xcorr_multimat_right_grouped_f32(const float *left, const float *right, float *out, unsigned cols,
                                     unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                     void *stream);
int xcorr_multimat_right_grouped_f64(const double *left, const double *right, double *out, unsigned cols,
                                     unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                     void *stream);

/* Multi-matrix-both: all n_left x n_right pairs, result index l*n_right + r, split-row.
 * Replaces run_ccn_shuffle_n_to_m_multimat_both_work_distribution<DIST>
 * (kernels.cuh:163-176). THE CALLER ZEROES `out` FIRST (n_to_m.hpp:341). */
int xcorr_multimat_both_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                            unsigned n_left, unsigned n_right, const xcorr_params *p, void *stream);
int xcorr_multimat_both_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                            unsigned n_left, unsigned n_right, const xcorr_params *p, void *stream);

/* Multi-matrix-both x grouped-overlap.
 * Replaces run_ccn_n_to_m_shuffle_multirow_both_multimat_both (kernels.cuh:236-250).
 * `out` need not be zeroed. */
int xcorr_multimat_both_grouped_f32(const float *left, const float *right, float *out, unsigned cols,
                                    unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                    void *stream);
int xcorr_multimat_both_grouped_f64(const double *left, const double *right, double *out, unsigned cols,
                                    unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params *p,
                                    void *stream);

#ifdef __cplusplus
}
#endif
#endif
