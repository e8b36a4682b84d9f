// Shared host-side pieces of libxcorr_hip.so: error state, last-launch record,
// parameter validation against the reference's limits.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>

#include "../../include/xcorr_hip.h"

namespace xcorr {

// ---- error state (one message per thread) ----
inline char *error_buffer() {
    static thread_local char buf[512] = "";
    return buf;
}

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int hip_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return XCORR_OK;
    // same information as the reference's CUCH macro (cuda_helpers.cuh:13-24)
    return fail(XCORR_ERR_RUNTIME, "HIP error %d (%s: %s) in %s", (int)e, hipGetErrorName(e), hipGetErrorString(e), what);
}

#define XCORR_HIP(call)                                  \
    do {                                                 \
        int _rc = ::xcorr::hip_check((call), #call);     \
        if (_rc != XCORR_OK) return _rc;                 \
    } while (0)

// ---- last launch record (reference kernel_args.cpp:7-19 keeps one per process; here one per host thread, like the
// error text, so that threads launching side by side do not overwrite each other's record) ----
inline xcorr_launch_record &last_launch() {
    static thread_local xcorr_launch_record rec;
    return rec;
}
// Per host thread: plan and record, but do not launch (xcorr_plan_only).
inline bool &plan_only() {
    static thread_local bool on = false;
    return on;
}
// 1: plan as for ordinary device memory; 2: plan as for an output the hardware's float atomics are not defined on
inline int &plan_only_mode() {
    static thread_local int mode = 0;
    return mode;
}
inline bool &have_last_launch() {
    static thread_local bool have = false;
    return have;
}

// ---- per-device facts that are asked of the runtime once ----
constexpr int MAX_DEVICES = 64;
inline int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 0;
    return dev;
}
inline int device_cus() {
    static int cus[MAX_DEVICES] = {};
    const int dev = current_device();
    if (cus[dev] == 0) {
        hipDeviceProp_t prop;
        cus[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    return cus[dev];
}

// Release limits of the reference build (CMakeLists.txt:16-46).
struct Limits {
    static constexpr unsigned warps_per_block = 32;             // every launcher, e.g. naive_shuffle_multirow_both.cu:645
    static constexpr unsigned shifts_per_thread = 8;            // SHUFFLE_MULTIROW_BOTH_SHIFTS_PER_THREAD_LIMIT
    static constexpr unsigned left_rows = 8;                    // SHUFFLE_MULTIROW_BOTH_LEFT_ROWS_LIMIT
    static constexpr unsigned right_matrices = 8;               // SHUFFLE_MULTIMAT_RIGHT_RIGHT_MATRICES_PER_THREAD_LIMIT
    static constexpr unsigned left_matrices = 8;                // SHUFFLE_N_TO_M_MULTIMAT_BOTH_LEFT_MATRICES_PER_THREAD_LIMIT
    static constexpr unsigned combined = 4;                     // the 4/4/4(/4) limits of the combined kernels
};

inline int check_limit(const char *what, unsigned value, unsigned limit) {
    if (value > limit) return fail(XCORR_ERR_INVALID_ARGUMENT, "Too many %s: %u (max %u)", what, value, limit);
    return XCORR_OK;
}

inline int check_shape(const void *left, const void *right, const void *out, unsigned cols, unsigned rows) {
    if (!left || !right || !out) return fail(XCORR_ERR_INVALID_ARGUMENT, "null device pointer");
    if (cols == 0 || rows == 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "empty matrix: %u x %u", rows, cols);
    // result indices are 32-bit in the kernels' per-matrix arithmetic
    if (cols > 16384 || rows > 16384) return fail(XCORR_ERR_INVALID_ARGUMENT, "matrix too large: %u x %u (max 16384)", rows, cols);
    return XCORR_OK;
}

// matrix counts and the number of result matrices are 32-bit signed in the planner and the kernels
inline int check_counts(unsigned n_left, unsigned n_right, bool all_pairs) {
    if (n_left == 0 || n_right == 0) return fail(XCORR_ERR_INVALID_ARGUMENT, "no matrices");
    const unsigned long long results = all_pairs ? (unsigned long long)n_left * n_right : n_right;
    if (n_left > 0x7fffffffu || n_right > 0x7fffffffu || results > 0x7fffffffull)
        return fail(XCORR_ERR_INVALID_ARGUMENT, "too many matrices: %u left, %u right", n_left, n_right);
    return XCORR_OK;
}

} // namespace xcorr
