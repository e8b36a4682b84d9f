// Timing harness: wall-clock and device-event measurements with the reference's adaptive
// repetition (stopwatch.hpp:57-71: repeat a block with a growing iteration count until the
// measured total reaches min_time, report total / iterations). Device events go through
// the C ABI; kernel time, transfers and file I/O are reported under separate labels.
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <stdexcept>
#include <vector>

#include "xcorr_api.hpp"

namespace cross {

using sw_clock = std::chrono::high_resolution_clock;

class measurement_result {
public:
    using duration = sw_clock::duration;
    measurement_result() : total_time_(duration::zero()), iterations_(0) {}
    measurement_result(duration total_time, std::size_t iterations) : total_time_(total_time), iterations_(iterations) {}
    duration get_iteration_time() const {
        if (total_time_ == duration::zero()) return duration::zero();
        if (iterations_ == 0) throw std::runtime_error("Zero iterations with non-zero total time");
        return total_time_ / iterations_;
    }
    duration get_total_time() const { return total_time_; }
    std::size_t get_iterations() const { return iterations_; }

private:
    duration total_time_;
    std::size_t iterations_;
};

// iterations * clamp(1.5 * min_time / total, 1.5, 100), 0 when the total is long enough
inline std::size_t get_next_iteration_count(std::chrono::nanoseconds min_time, const measurement_result &res) {
    auto total = std::chrono::duration_cast<std::chrono::nanoseconds>(res.get_total_time());
    if (total >= min_time) return 0;
    double ratio = static_cast<double>(min_time.count()) / static_cast<double>(std::max<long long>(total.count(), 1));
    double next = std::ceil(res.get_iterations() * std::max(std::min(ratio * 1.5, 100.0), 1.5));
    return static_cast<std::size_t>(next);
}

class stopwatch {
public:
    stopwatch(std::size_t num_measurements, std::chrono::nanoseconds min_time)
        : measurements_(num_measurements), min_time_(min_time), events_(num_measurements) {}
    ~stopwatch() {
        for (auto &e : events_) {
            if (e.start) xcorr_event_destroy(e.start);
            if (e.stop) xcorr_event_destroy(e.stop);
        }
    }
    stopwatch(const stopwatch &) = delete;
    stopwatch &operator=(const stopwatch &) = delete;

    std::chrono::nanoseconds get_min_time() const { return min_time_; }
    const std::vector<measurement_result> &results() const { return measurements_; }
    void reset() { std::fill(measurements_.begin(), measurements_.end(), measurement_result()); }
    void resize(std::size_t n) {
        measurements_.assign(n, measurement_result());
        events_.resize(n);
    }

    // CPU_MEASURE (stopwatch.hpp:143-157)
    template <typename F>
    void cpu_measure(std::size_t label, bool enable, bool gpu_sync, F &&block) {
        if (!enable) {
            block();
            return;
        }
        auto start = sw_clock::now();
        block();
        if (gpu_sync) xcheck(xcorr_device_sync());
        measurements_[label] = measurement_result(sw_clock::now() - start, 1);
    }

    // CPU_ADAPTIVE_MEASURE (stopwatch.hpp:179-200)
    template <typename F>
    void cpu_adaptive_measure(std::size_t label, bool enable, bool gpu_sync, F &&block) {
        if (!enable) {
            block();
            return;
        }
        std::size_t iterations = 1;
        do {
            auto start = sw_clock::now();
            for (std::size_t i = 0; i < iterations; ++i) {
                block();
                if (gpu_sync) xcheck(xcorr_device_sync());
            }
            measurements_[label] = measurement_result(sw_clock::now() - start, iterations);
            iterations = get_next_iteration_count(min_time_, measurements_[label]);
        } while (iterations != 0);
    }

    // CUDA_ADAPTIVE_MEASURE (stopwatch.hpp:125-141): an event pair around `iterations`
    // back-to-back launches on the default stream
    template <typename F>
    void device_adaptive_measure(std::size_t label, bool enable, F &&block) {
        if (!enable) {
            block();
            return;
        }
        event_pair &ev = events_[label];
        if (!ev.start) {
            xcheck(xcorr_event_create(&ev.start));
            xcheck(xcorr_event_create(&ev.stop));
        }
        std::size_t iterations = 1;
        do {
            xcheck(xcorr_event_record(ev.start, nullptr));
            for (std::size_t i = 0; i < iterations; ++i) block();
            xcheck(xcorr_event_record(ev.stop, nullptr));
            xcheck(xcorr_event_sync(ev.stop));
            float ms = 0;
            xcheck(xcorr_event_elapsed_ms(ev.start, ev.stop, &ms));
            auto t = std::chrono::duration_cast<sw_clock::duration>(std::chrono::duration<double, std::milli>(ms));
            measurements_[label] = measurement_result(t, iterations);
            iterations = get_next_iteration_count(min_time_, measurements_[label]);
        } while (iterations != 0);
    }

private:
    struct event_pair {
        void *start = nullptr;
        void *stop = nullptr;
    };
    std::vector<measurement_result> measurements_;
    std::chrono::nanoseconds min_time_;
    std::vector<event_pair> events_;
};

} // namespace cross
