// extern "C" surface of libxcorr_hip.so: status, memory / queue shims and the
// compute entry points that stand in for the reference launchers (kernels.cuh:41-283).
#include "engine_registry.hpp"
#include "simple_kernels.hpp"
#include "xcorr_common.hpp"

using namespace xcorr;

static hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

__global__ void xcorr_plain_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

extern "C" {

// ------------------------------------------------------------------ status
const char *xcorr_last_error(void) { return error_buffer(); }

const char *xcorr_version(void) { return "xcorr_hip 0.2 (gfx950)"; }

int xcorr_last_launch(xcorr_launch_record *out) {
    if (!out) return fail(XCORR_ERR_INVALID_ARGUMENT, "null record pointer");
    if (!have_last_launch()) return fail(XCORR_ERR_INVALID_ARGUMENT, "No kernel launch");
    *out = last_launch();
    return XCORR_OK;
}

int xcorr_plan_only(int on) {
    if (on < 0 || on > 2) return fail(XCORR_ERR_INVALID_ARGUMENT, "xcorr_plan_only: %d is not 0, 1 or 2", on);
    plan_only() = on != 0;
    plan_only_mode() = on;
    return XCORR_OK;
}

int xcorr_device_info_get(xcorr_device_info *out) {
    if (!out) return fail(XCORR_ERR_INVALID_ARGUMENT, "null info pointer");
    int dev = 0;
    XCORR_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    XCORR_HIP(hipGetDeviceProperties(&prop, dev));
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", prop.name);
    snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
    out->compute_units = prop.multiProcessorCount;
    out->clock_khz = prop.clockRate;
    out->memory_clock_khz = prop.memoryClockRate;
    out->memory_bus_bits = prop.memoryBusWidth;
    out->lds_bytes_per_block = (int)prop.sharedMemPerBlock;
    out->global_mem_bytes = prop.totalGlobalMem;
    double lanes_per_s = (double)prop.multiProcessorCount * 4.0 * 16.0 * (double)prop.clockRate * 1e3;
    out->fp32_vector_peak_tflops = lanes_per_s * 2.0 * 2.0 / 1e12;
    out->fp64_vector_peak_tflops = lanes_per_s * 2.0 / 1e12;
    return XCORR_OK;
}

// ------------------------------------------------------------------ shims
int xcorr_malloc(void **dev_ptr, size_t bytes) {
    if (!dev_ptr) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    XCORR_HIP(hipMalloc(dev_ptr, bytes));
    return XCORR_OK;
}
int xcorr_free(void *dev_ptr) {
    XCORR_HIP(hipFree(dev_ptr));
    return XCORR_OK;
}
int xcorr_memset_async(void *dev_ptr, int value, size_t bytes, void *stream) {
    XCORR_HIP(hipMemsetAsync(dev_ptr, value, bytes, as_stream(stream)));
    return XCORR_OK;
}
int xcorr_copy_kernel(void *dev_dst, const void *dev_src, size_t bytes, void *stream) {
    if (!dev_dst || !dev_src) return fail(XCORR_ERR_INVALID_ARGUMENT, "null device pointer");
    if (bytes % 16 != 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "copy size %zu is not a multiple of 16 bytes", bytes);
    if (bytes == 0) return XCORR_OK;
    size_t n = bytes / 16;
    size_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    xcorr_plain_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(static_cast<uint4 *>(dev_dst),
                                                                                       static_cast<const uint4 *>(dev_src), n);
    XCORR_HIP(hipGetLastError());
    return XCORR_OK;
}
int xcorr_memcpy_h2d(void *dev_dst, const void *host_src, size_t bytes) {
    XCORR_HIP(hipMemcpy(dev_dst, host_src, bytes, hipMemcpyHostToDevice));
    return XCORR_OK;
}
int xcorr_memcpy_d2h(void *host_dst, const void *dev_src, size_t bytes) {
    XCORR_HIP(hipMemcpy(host_dst, dev_src, bytes, hipMemcpyDeviceToHost));
    return XCORR_OK;
}
int xcorr_memcpy_h2d_async(void *dev_dst, const void *host_src, size_t bytes, void *stream) {
    XCORR_HIP(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return XCORR_OK;
}
int xcorr_memcpy_d2h_async(void *host_dst, const void *dev_src, size_t bytes, void *stream) {
    XCORR_HIP(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return XCORR_OK;
}
int xcorr_host_alloc_pinned(void **host_ptr, size_t bytes) {
    if (!host_ptr) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    XCORR_HIP(hipHostMalloc(host_ptr, bytes, hipHostMallocDefault));
    return XCORR_OK;
}
int xcorr_host_free(void *host_ptr) {
    XCORR_HIP(hipHostFree(host_ptr));
    return XCORR_OK;
}
int xcorr_stream_create(void **stream) {
    if (!stream) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    hipStream_t s;
    XCORR_HIP(hipStreamCreate(&s)); // default priority only
    *stream = s;
    return XCORR_OK;
}
int xcorr_stream_destroy(void *stream) {
    XCORR_HIP(hipStreamDestroy(as_stream(stream)));
    return XCORR_OK;
}
int xcorr_stream_sync(void *stream) {
    XCORR_HIP(hipStreamSynchronize(as_stream(stream)));
    return XCORR_OK;
}
int xcorr_clear_async(void *dev_ptr, size_t bytes, void *stream) {
    if (!dev_ptr) return fail(XCORR_ERR_INVALID_ARGUMENT, "null device pointer");
    if (bytes % 4 != 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "xcorr_clear_async: %zu bytes are not a multiple of 4", bytes);
    const size_t n = bytes / 4;
    if (n == 0) return XCORR_OK;
    size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
    if (blocks > 65536) blocks = 65536;
    zero_fill_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(static_cast<float *>(dev_ptr), n);
    XCORR_HIP(hipGetLastError());
    return XCORR_OK;
}
int xcorr_graph_capture_begin(void *stream) {
    if (!stream) return fail(XCORR_ERR_INVALID_ARGUMENT, "the NULL stream cannot be captured");
    // relaxed: one-time set-up calls of a first launch (function attributes, occupancy queries) do not break the capture
    XCORR_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
    return XCORR_OK;
}
int xcorr_graph_capture_end(void *stream, void **graph_exec) {
    if (!stream || !graph_exec) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    hipGraph_t graph = nullptr;
    XCORR_HIP(hipStreamEndCapture(as_stream(stream), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    XCORR_HIP(e);
    *graph_exec = exec;
    return XCORR_OK;
}
int xcorr_graph_launch(void *graph_exec, void *stream) {
    if (!graph_exec) return fail(XCORR_ERR_INVALID_ARGUMENT, "null graph");
    XCORR_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
    return XCORR_OK;
}
int xcorr_graph_destroy(void *graph_exec) {
    if (!graph_exec) return XCORR_OK;
    XCORR_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return XCORR_OK;
}
int xcorr_device_sync(void) {
    XCORR_HIP(hipDeviceSynchronize());
    XCORR_HIP(hipGetLastError());
    return XCORR_OK;
}
int xcorr_event_create(void **event) {
    if (!event) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    hipEvent_t e;
    XCORR_HIP(hipEventCreate(&e));
    *event = e;
    return XCORR_OK;
}
int xcorr_event_record(void *event, void *stream) {
    XCORR_HIP(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return XCORR_OK;
}
int xcorr_event_sync(void *event) {
    XCORR_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return XCORR_OK;
}
int xcorr_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!ms) return fail(XCORR_ERR_INVALID_ARGUMENT, "null pointer");
    XCORR_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return XCORR_OK;
}
int xcorr_event_destroy(void *event) {
    XCORR_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return XCORR_OK;
}

} // extern "C"

// ------------------------------------------------------------------ compute
namespace {

// The caller's parameter block, as much of it as the caller's header declares (struct_size), in the layout of this build;
// a null pointer stands for all defaults.
struct LoadedParams {
    xcorr_params p = {};
    int error = XCORR_OK;
    explicit LoadedParams(const xcorr_params *from) {
        p.struct_size = sizeof(xcorr_params);
        if (!from) return;
        const unsigned n = from->struct_size;
        if (n < 2 * sizeof(unsigned) || n % sizeof(unsigned) != 0) {
            error = fail(XCORR_ERR_INVALID_ARGUMENT,
                         "xcorr_params.struct_size is %u: set it to sizeof(xcorr_params) (XCORR_PARAMS_INIT; the field leads the struct since version 0.2)", n);
            return;
        }
        memcpy(&p, from, n < sizeof(xcorr_params) ? n : sizeof(xcorr_params));
        p.struct_size = sizeof(xcorr_params);
    }
};

int check_dist(unsigned d) {
    if (d > XCORR_DIST_TRIANGLE) return fail(XCORR_ERR_INVALID_ARGUMENT, "Unknown distribution %u", d);
    return XCORR_OK;
}

// warps of the reference are 32 lanes wide; a wavefront holds two of them
unsigned waves_from_warps(unsigned warps) { return warps == 0 ? 0 : (warps + 1) / 2; }

EngineRequest base_request(const char *family, int elem_bytes, const void *left, const void *right, void *out,
                           unsigned cols, unsigned rows, unsigned n_left, unsigned n_right, const xcorr_params &p) {
    EngineRequest rq = {};
    rq.family = family;
    rq.elem_bytes = elem_bytes;
    rq.V = left;
    rq.U = right;
    rq.out = out;
    rq.W = (int)cols;
    rq.H = (int)rows;
    rq.nV = (int)n_left;
    rq.nU = (int)n_right;
    rq.x_shifts = p.x_shifts_per_thread;
    rq.lanes_x = p.lanes_x;
    rq.lanes_y = p.lanes_y;
    rq.spec_index = p.specialisation;
    rq.column_chunks = p.column_chunks;
    rq.matrix_cores = p.matrix_cores;
    rq.waves = waves_from_warps(p.warps_per_thread_block);
    rq.dist = p.distribution_type;
    return rq;
}

// Few small matrices and a call that names no tile or chunk: every pair whole in the LDS of its share of the
// CUs (pair_in_lds_kernel), one launch, plain stores - whatever the family's contract says about a zeroed output (stores into
// a zeroed output are what the atomic adds of one work item per tile would leave there). The launch record then says
// uses_atomics = 0, and a caller that asks first (xcorr_plan_only) may skip its clear. Measured against the engine's launches
// (with the clear kernel where the contract has one) through the `cross` binary, microseconds per launch: one pair up to
// 96x96 fp32 / 64x64 fp64 as for xcorr_grouped_overlap; at most 64 pairs of up to 32x32 and 2^24 multiply-adds in all.
// Whether a call of the sliding-window families names a tile or a chunk. (A distribution alone names neither: it says how a
// split launch would cut the rows. With one pair the matrices per thread say nothing either.)
bool names_tile_or_chunk(const xcorr_params &p, size_t n_pairs) {
    return p.specialisation || p.x_shifts_per_thread || p.lanes_x || p.lanes_y || p.rows_per_thread || p.column_chunks || p.matrix_cores ||
           p.shifts_per_thread || p.shifts_per_thread_right_matrix || p.shifts_per_thread_block ||
           (n_pairs > 1 && (p.right_matrices_per_thread || p.left_matrices_per_thread));
}

template <typename T>
bool small_pairs_in_lds(const xcorr_params &p, bool named, unsigned cols, unsigned rows, size_t n_pairs, int *error) {
    *error = XCORR_OK;
    if (p.whole_pair_in_lds > 2) {
        *error = fail(XCORR_ERR_INVALID_ARGUMENT, "whole_pair_in_lds must be 0, 1 or 2, not %u", p.whole_pair_in_lds);
        return false;
    }
    if (p.whole_pair_in_lds == 2) return false;
    if (p.whole_pair_in_lds == 1) return true; // (an error from the launcher if the pair does not fit)
    if (named || !pair_fits_lds<T>(cols, rows)) return false;
    const size_t elems = (size_t)cols * rows;
    if (n_pairs == 1) return cols <= 128 && elems <= (sizeof(T) == 4 ? 96u * 96u : 64u * 64u);
    // (pairs of 32x32: 4.0 us for 2, 5.8 for 8, 8.8 for 16, 15.1 for 32 - where the engine's tiles take 9.4)
    return cols <= 32 && rows <= 32 && n_pairs <= 64 && n_pairs * elems * elems <= (1u << 24);
}

template <typename T>
int shuffle_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params *pp,
                 void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, 1), cols, rows, 1, &rc)) return run_pair_in_lds<T>("shuffle", left, right, out, cols, rows, as_stream(stream));
    if (rc) return rc;
    EngineRequest rq = base_request("shuffle", sizeof(T), left, right, out, cols, rows, 1, 1, p);
    rq.y_shifts = 1;
    rq.left_mats = rq.right_mats = 1;
    // The reference's launcher never splits the reduction. Here the planner may (clearing the output itself and adding
    // partial sums atomically) when the launch would otherwise leave most of the device idle; distribution_type "none"
    // asks for the unsplit launch.
    rq.may_split = p.distribution_type != XCORR_DIST_NONE;
    rq.dist = rq.may_split ? XCORR_DIST_DEFAULT : XCORR_DIST_NONE;
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int split_row_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params *pp,
                   void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, 1), cols, rows, 1, &rc)) return run_pair_in_lds<T>("split_row", left, right, out, cols, rows, as_stream(stream));
    if (rc) return rc;
    EngineRequest rq = base_request("split_row", sizeof(T), left, right, out, cols, rows, 1, 1, p);
    rq.y_shifts = 1;
    rq.left_mats = rq.right_mats = 1;
    rq.rows_per_worker = p.rows_per_thread;
    rq.caller_zeroes = true;
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int grouped_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params *pp,
                 void *stream, bool ordered = false) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_limit("shifts per thread", p.shifts_per_thread, Limits::shifts_per_thread))) return rc;
    if ((rc = check_limit("left rows per iteration", p.left_rows_per_iteration, Limits::left_rows))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (p.whole_pair_in_lds > 2) return fail(XCORR_ERR_INVALID_ARGUMENT, "whole_pair_in_lds must be 0, 1 or 2, not %u", p.whole_pair_in_lds);
    // A small pair with no tile asked for: both matrices in the LDS of every block, one launch, no atomics. Measured
    // against the engine's best plan on square pairs (microseconds per launch, whole-pair kernel / engine, which runs a
    // matrix-core tile from about 100x100 on): fp32 16: 3.9 / 5.3, 32: 4.1 / 7.3, 64: 5.5 / 10.3, 80: 11.9 / 12.3, 96: 12.5 / 13.7,
    // 104: 15.4 / 14.1, 112: 18.4 / 14.8, 128: 28.4 / 17.3; fp64 32: 4.2 / 7.8, 64: 7.9 / 11.7, 72: 16.4 / 13.4, 96: 17.4 / 15.0.
    // Beyond the sizes below the engine wins.
    const bool tile_asked = p.specialisation || p.x_shifts_per_thread || p.lanes_x || p.lanes_y || p.rows_per_thread || p.column_chunks ||
                            p.shifts_per_thread || p.matrix_cores || p.distribution_type != XCORR_DIST_DEFAULT;
    const size_t elems = (size_t)cols * rows;
    const bool small = pair_fits_lds<T>(cols, rows) && cols <= 128 && elems <= (sizeof(T) == 4 ? 96u * 96u : 64u * 64u);
    if (p.whole_pair_in_lds == 1 || (p.whole_pair_in_lds == 0 && !tile_asked && small))
        return run_pair_in_lds<T>("grouped_overlap", left, right, out, cols, rows, as_stream(stream));
    EngineRequest rq = base_request(ordered ? "grouped_overlap_ordered" : "grouped_overlap", sizeof(T), left, right, out, cols, rows, 1, 1, p);
    rq.y_shifts = p.shifts_per_thread == 1 ? 2 : p.shifts_per_thread; // 0 = planner's choice among the grouped tiles
    rq.rows_per_worker = p.rows_per_thread;
    rq.may_split = true;
    rq.ordered = ordered;
    if (ordered) {
        if (p.column_chunks > 1) return fail(XCORR_ERR_INVALID_ARGUMENT, "grouped_overlap_ordered: the columns of a reduction are not cut (column_chunks %u)", p.column_chunks);
        if (p.matrix_cores == 2) return fail(XCORR_ERR_UNSUPPORTED, "grouped_overlap_ordered: only the matrix-core tiles add their chunks in order");
        rq.column_chunks = 1;
    }
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int multimat_right_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_left, unsigned n_right,
                        const xcorr_params *pp, void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_counts(n_left, n_right, n_left > 1))) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_limit("right matrices per thread", p.right_matrices_per_thread, Limits::right_matrices))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, (size_t)n_left * n_right), cols, rows, (size_t)n_left * n_right, &rc)) {
        PairList pairs;
        pairs.n_pairs = n_left * n_right;
        pairs.left_div = n_right; // left l meets the right matrices [l * n_right, (l + 1) * n_right)
        return run_pair_in_lds<T>("multimat_right", left, right, out, cols, rows, as_stream(stream), pairs);
    }
    if (rc) return rc;
    EngineRequest rq = base_request("multimat_right", sizeof(T), left, right, out, cols, rows, n_left, n_left * n_right, p);
    rq.group_m = n_left > 1 ? (int)n_right : 0; // left l against its own group of n_right right matrices
    rq.y_shifts = 1;
    rq.left_mats = 1;
    rq.right_mats = p.right_matrices_per_thread;
    if (p.rows_per_thread > 0 || p.distribution_type == XCORR_DIST_RECTANGLE || p.distribution_type == XCORR_DIST_TRIANGLE) {
        // the work-distribution launcher (rows_per_thread 0 with a distribution: the planner picks the chunk)
        rq.rows_per_worker = p.rows_per_thread;
        rq.caller_zeroes = true;
    } else { // the plain launcher: split only by the planner's own choice, never with distribution_type "none"
        rq.may_split = p.distribution_type != XCORR_DIST_NONE;
        rq.dist = rq.may_split ? XCORR_DIST_DEFAULT : XCORR_DIST_NONE;
    }
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int multimat_right_grouped_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_left,
                                unsigned n_right, const xcorr_params *pp, void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_counts(n_left, n_right, true))) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_limit("shifts per thread per right matrix", p.shifts_per_thread_right_matrix, Limits::combined))) return rc;
    if ((rc = check_limit("right matrices per thread", p.right_matrices_per_thread, Limits::combined))) return rc;
    if ((rc = check_limit("left rows per iteration", p.left_rows_per_iteration, Limits::combined))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, (size_t)n_left * n_right), cols, rows, (size_t)n_left * n_right, &rc)) {
        PairList pairs;
        pairs.n_pairs = n_left * n_right;
        pairs.left_div = n_right; // left l meets the right matrices [l * n_right, (l + 1) * n_right)
        return run_pair_in_lds<T>("multimat_right_grouped", left, right, out, cols, rows, as_stream(stream), pairs);
    }
    if (rc) return rc;
    EngineRequest rq = base_request("multimat_right_grouped", sizeof(T), left, right, out, cols, rows, n_left,
                                    n_left * n_right, p);
    rq.group_m = n_left > 1 ? (int)n_right : 0;
    if (n_left == 1) rq.nU = (int)n_right;
    rq.y_shifts = p.shifts_per_thread_right_matrix == 1 ? 2 : p.shifts_per_thread_right_matrix;
    rq.left_mats = 1;
    rq.right_mats = p.right_matrices_per_thread;
    rq.rows_per_worker = p.rows_per_thread;
    rq.may_split = true;
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int multimat_both_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_left,
                       unsigned n_right, const xcorr_params *pp, void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_counts(n_left, n_right, true))) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_limit("left matrices per thread", p.left_matrices_per_thread, Limits::left_matrices))) return rc;
    if ((rc = check_limit("right matrices per thread", p.right_matrices_per_thread, Limits::right_matrices))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, (size_t)n_left * n_right), cols, rows, (size_t)n_left * n_right, &rc)) {
        PairList pairs;
        pairs.n_pairs = n_left * n_right;
        pairs.left_div = n_right; // result l * n_right + r
        pairs.right_mod = n_right;
        return run_pair_in_lds<T>("multimat_both", left, right, out, cols, rows, as_stream(stream), pairs);
    }
    if (rc) return rc;
    EngineRequest rq = base_request("multimat_both", sizeof(T), left, right, out, cols, rows, n_left, n_right, p);
    rq.y_shifts = 1;
    rq.left_mats = p.left_matrices_per_thread;
    rq.right_mats = p.right_matrices_per_thread;
    rq.rows_per_worker = p.rows_per_thread;
    if (rq.dist == XCORR_DIST_DEFAULT) rq.dist = XCORR_DIST_TRIANGLE; // reference default, n_to_m.hpp:325
    rq.caller_zeroes = true;
    return run_engine(rq, as_stream(stream));
}

template <typename T>
int multimat_both_grouped_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_left,
                               unsigned n_right, const xcorr_params *pp, void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_counts(n_left, n_right, true))) return rc;
    if ((rc = check_limit("warps per thread block", p.warps_per_thread_block, Limits::warps_per_block))) return rc;
    if ((rc = check_limit("shifts per thread per right matrix", p.shifts_per_thread_right_matrix, Limits::combined))) return rc;
    if ((rc = check_limit("left matrices per thread", p.left_matrices_per_thread, Limits::combined))) return rc;
    if ((rc = check_limit("right matrices per thread", p.right_matrices_per_thread, Limits::combined))) return rc;
    if ((rc = check_limit("left rows per iteration", p.left_rows_per_iteration, Limits::combined))) return rc;
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (small_pairs_in_lds<T>(p, names_tile_or_chunk(p, (size_t)n_left * n_right), cols, rows, (size_t)n_left * n_right, &rc)) {
        PairList pairs;
        pairs.n_pairs = n_left * n_right;
        pairs.left_div = n_right; // result l * n_right + r
        pairs.right_mod = n_right;
        return run_pair_in_lds<T>("multimat_both_grouped", left, right, out, cols, rows, as_stream(stream), pairs);
    }
    if (rc) return rc;
    EngineRequest rq = base_request("multimat_both_grouped", sizeof(T), left, right, out, cols, rows, n_left, n_right, p);
    rq.y_shifts = p.shifts_per_thread_right_matrix == 1 ? 2 : p.shifts_per_thread_right_matrix;
    rq.left_mats = p.left_matrices_per_thread;
    rq.right_mats = p.right_matrices_per_thread;
    rq.rows_per_worker = p.rows_per_thread;
    rq.may_split = true;
    return run_engine(rq, as_stream(stream));
}

// The work-distribution variant (zeroed output, atomic adds of row chunks) on a small pair with no chunk named: the whole pair in LDS
// instead, one launch, plain stores (small_pairs_in_lds); the other variants are the kernels their names say.
template <typename T>
int warp_per_overlap_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, const xcorr_params *pp, void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    if ((rc = check_limit("shifts per thread block", p.shifts_per_thread_block, 32))) return rc; // naive_warp_per_shift.cu:316-318
    if ((rc = check_dist(p.distribution_type))) return rc;
    if (p.warp_per_overlap_variant == XCORR_WPO_WORK_DISTRIBUTION) {
        xcorr_params q = p;
        q.shifts_per_thread_block = 0; // (the shape of a block, not a chunk of the work)
        if (small_pairs_in_lds<T>(q, names_tile_or_chunk(q, 1), cols, rows, 1, &rc)) return run_pair_in_lds<T>("warp_per_overlap", left, right, out, cols, rows, as_stream(stream));
        if (rc) return rc;
    }
    return run_warp_per_overlap<T>(left, right, out, cols, rows, p, as_stream(stream));
}

// The LDS-staged wavefront-per-overlap family on few small matrices with none of its staging parameters named: the kernel that
// keeps every pair whole in LDS does the same work (a wavefront per group of overlaps, both matrices in LDS) in one pass.
template <typename T>
int warp_per_overlap_lds_impl(const T *left, const T *right, T *out, unsigned cols, unsigned rows, unsigned n_right, const xcorr_params *pp,
                              void *stream) {
    const LoadedParams loaded(pp);
    if (loaded.error) return loaded.error;
    const xcorr_params &p = loaded.p;
    int rc = check_shape(left, right, out, cols, rows);
    if (rc) return rc;
    const bool named = p.shifts_per_thread_block || p.shared_mem_rows || p.shared_mem_row_size || p.right_matrices_per_block || p.column_group_per_block;
    if (n_right > 0 && small_pairs_in_lds<T>(p, named, cols, rows, n_right, &rc)) {
        PairList pairs;
        pairs.n_pairs = pairs.left_div = n_right;
        return run_pair_in_lds<T>("warp_per_overlap_lds", left, right, out, cols, rows, as_stream(stream), pairs);
    }
    if (rc) return rc;
    return run_warp_per_overlap_lds<T>(left, right, out, cols, rows, n_right, p, as_stream(stream));
}

} // namespace

extern "C" {

int xcorr_overlap_wise_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                           unsigned n_left, unsigned batch, void *stream) {
    return run_overlap_wise<float>(left, right, out, cols, rows, n_left, batch, false, as_stream(stream));
}
int xcorr_overlap_wise_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                           unsigned n_left, unsigned batch, void *stream) {
    return run_overlap_wise<double>(left, right, out, cols, rows, n_left, batch, false, as_stream(stream));
}
int xcorr_overlap_wise_all_pairs_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                     unsigned n_left, unsigned n_right, void *stream) {
    return run_overlap_wise<float>(left, right, out, cols, rows, n_left, n_right, true, as_stream(stream));
}
int xcorr_overlap_wise_all_pairs_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                     unsigned n_left, unsigned n_right, void *stream) {
    return run_overlap_wise<double>(left, right, out, cols, rows, n_left, n_right, true, as_stream(stream));
}

int xcorr_warp_per_overlap_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                               const xcorr_params *p, void *stream) {
    return warp_per_overlap_impl<float>(left, right, out, cols, rows, p, stream);
}
int xcorr_warp_per_overlap_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                               const xcorr_params *p, void *stream) {
    return warp_per_overlap_impl<double>(left, right, out, cols, rows, p, stream);
}

int xcorr_warp_per_overlap_lds_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                   unsigned n_right, const xcorr_params *p, void *stream) {
    return warp_per_overlap_lds_impl<float>(left, right, out, cols, rows, n_right, p, stream);
}
int xcorr_warp_per_overlap_lds_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                   unsigned n_right, const xcorr_params *p, void *stream) {
    return warp_per_overlap_lds_impl<double>(left, right, out, cols, rows, n_right, p, stream);
}

int xcorr_block_per_overlap_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                const xcorr_params *p, void *stream) {
    const LoadedParams loaded(p);
    if (loaded.error) return loaded.error;
    return run_block_per_overlap<float>(left, right, out, cols, rows, loaded.p, as_stream(stream));
}
int xcorr_block_per_overlap_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                                const xcorr_params *p, void *stream) {
    const LoadedParams loaded(p);
    if (loaded.error) return loaded.error;
    return run_block_per_overlap<double>(left, right, out, cols, rows, loaded.p, as_stream(stream));
}

#define XCORR_PAIR_ENTRY(NAME, IMPL)                                                                              \
    int NAME##_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,               \
                   const xcorr_params *p, void *stream) {                                                         \
        return IMPL<float>(left, right, out, cols, rows, p, stream);                                              \
    }                                                                                                             \
    int NAME##_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,            \
                   const xcorr_params *p, void *stream) {                                                         \
        return IMPL<double>(left, right, out, cols, rows, p, stream);                                             \
    }

XCORR_PAIR_ENTRY(xcorr_shuffle, shuffle_impl)
XCORR_PAIR_ENTRY(xcorr_split_row, split_row_impl)
XCORR_PAIR_ENTRY(xcorr_grouped_overlap, grouped_impl)

int xcorr_grouped_overlap_ordered_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                                      const xcorr_params *p, void *stream) {
    return grouped_impl<float>(left, right, out, cols, rows, p, stream, true);
}

int xcorr_multimat_right_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,
                             unsigned n_right, const xcorr_params *p, void *stream) {
    return multimat_right_impl<float>(left, right, out, cols, rows, 1, n_right, p, stream);
}
int xcorr_multimat_right_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,
                             unsigned n_right, const xcorr_params *p, void *stream) {
    return multimat_right_impl<double>(left, right, out, cols, rows, 1, n_right, p, stream);
}

#define XCORR_NM_ENTRY(NAME, IMPL)                                                                                \
    int NAME##_f32(const float *left, const float *right, float *out, unsigned cols, unsigned rows,               \
                   unsigned n_left, unsigned n_right, const xcorr_params *p, void *stream) {                      \
        return IMPL<float>(left, right, out, cols, rows, n_left, n_right, p, stream);                             \
    }                                                                                                             \
    int NAME##_f64(const double *left, const double *right, double *out, unsigned cols, unsigned rows,            \
                   unsigned n_left, unsigned n_right, const xcorr_params *p, void *stream) {                      \
        return IMPL<double>(left, right, out, cols, rows, n_left, n_right, p, stream);                            \
    }

XCORR_NM_ENTRY(xcorr_multimat_right_groups, multimat_right_impl)
XCORR_NM_ENTRY(xcorr_multimat_right_grouped, multimat_right_grouped_impl)
XCORR_NM_ENTRY(xcorr_multimat_both, multimat_both_impl)
XCORR_NM_ENTRY(xcorr_multimat_both_grouped, multimat_both_grouped_impl)

} // extern "C"
