// C++ convenience layer over the C ABI of libxcorr_hip.so. The host program includes
// no HIP header: device memory, streams and events are reached through the ABI's shims
// (the reference's host side uses cuda_helpers.cuh:13-97 and allocator.cuh:16-86 here).
#pragma once

#include <cstddef>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/xcorr_hip.h"

namespace cross {

// status -> exception, like the reference's CUCH macro (cuda_helpers.cuh:13-24)
inline void xcheck(int rc) {
    if (rc != XCORR_OK) throw std::runtime_error(xcorr_last_error());
}

// Thrown for bad per-algorithm JSON values (reference argument_error.hpp:10-20): exit code 1.
class argument_error : public std::runtime_error {
public:
    argument_error(const std::string &msg, std::string arg_name)
        : std::runtime_error(msg), arg_name_(std::move(arg_name)) {}
    const std::string &arg_name() const { return arg_name_; }

private:
    std::string arg_name_;
};

// Pinned host memory for the arrays that are copied to and from the device
// (reference pinned_allocator, allocator.cuh:16-86). Falls back to the C++ heap when
// no device is present so that the CPU algorithms run anywhere.
template <typename T>
struct pinned_allocator {
    using value_type = T;
    pinned_allocator() = default;
    template <typename U>
    pinned_allocator(const pinned_allocator<U> &) {}
    T *allocate(std::size_t n) {
        void *p = nullptr;
        if (n == 0) n = 1;
        if (xcorr_host_alloc_pinned(&p, n * sizeof(T)) != XCORR_OK) throw std::bad_alloc();
        return static_cast<T *>(p);
    }
    void deallocate(T *p, std::size_t) { xcorr_host_free(p); }
    template <typename U>
    bool operator==(const pinned_allocator<U> &) const { return true; }
    template <typename U>
    bool operator!=(const pinned_allocator<U> &) const { return false; }
};

inline std::string last_kernel_launch_args_string() {
    // same layout as reference kernel_args.cpp:32-43
    xcorr_launch_record r;
    if (xcorr_last_launch(&r) != XCORR_OK) return "No kernel launch";
    std::string s;
    s += "Block size: [" + std::to_string(r.block[0]) + ", " + std::to_string(r.block[1]) + ", " + std::to_string(r.block[2]) + "]";
    s += "\nGrid size: [" + std::to_string(r.grid[0]) + ", " + std::to_string(r.grid[1]) + ", " + std::to_string(r.grid[2]) + "]";
    s += "\nShared memory: " + std::to_string(r.shared_mem_bytes) + "B\n";
    s += std::string("kernel: ") + r.kernel + "\n";
    s += "y_shifts_per_thread: " + std::to_string(r.y_shifts_per_thread) + "\n";
    s += "x_shifts_per_thread: " + std::to_string(r.x_shifts_per_thread) + "\n";
    s += "left_matrices_per_thread: " + std::to_string(r.left_matrices_per_thread) + "\n";
    s += "right_matrices_per_thread: " + std::to_string(r.right_matrices_per_thread) + "\n";
    s += "rows_per_worker: " + std::to_string(r.rows_per_worker) + "\n";
    return s;
}

} // namespace cross
