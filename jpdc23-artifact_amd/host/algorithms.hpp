// Algorithm classes of the `cross` binary: one object per (algorithm name, data type) that
// owns the host arrays, the device buffers and the tuning arguments and runs the phases
// load -> prepare -> transfer -> run -> finalize -> free -> store, each under its own
// measurement label (reference cross_corr.hpp:21-189 and the per-mode headers
// one_to_one.hpp, one_to_many.hpp, n_to_mn.hpp, n_to_m.hpp).
//
// The reference has one class per algorithm name; here the names are rows of a table
// (algorithm_registry.cpp) that say which kernel family of libxcorr_hip.so they launch,
// which JSON keys they read with which defaults, and how they are measured.
#pragma once

#include <chrono>
#include <filesystem>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "cpu_xcorr.hpp"
#include "json_lite.hpp"
#include "matrix.hpp"
#include "stopwatch.hpp"
#include "xcorr_api.hpp"

namespace cross {

enum class BenchmarkType { Unknown, None, Compute, CommonSteps, Algorithm };
enum class Mode { one_to_one, one_to_many, n_to_mn, n_to_m };

inline const char *mode_name(Mode m) {
    switch (m) {
    case Mode::one_to_one: return "one_to_one";
    case Mode::one_to_many: return "one_to_many";
    case Mode::n_to_mn: return "n_to_mn";
    default: return "n_to_m";
    }
}

// reference one_to_one.hpp:20-22, one_to_many.hpp:15-17, n_to_mn.hpp:23-25, n_to_m.hpp:19-21
inline bool validate_input_size(Mode mode, dsize_t rows, dsize_t cols, dsize_t left, dsize_t right) {
    switch (mode) {
    case Mode::one_to_one: return rows > 0 && cols > 0 && left == 1 && right == 1;
    case Mode::one_to_many: return rows > 0 && cols > 0 && left == 1 && right > 0;
    case Mode::n_to_mn: return rows > 0 && cols > 0 && left > 0 && right > 0 && right % left == 0;
    default: return rows > 0 && cols > 0 && left > 0 && right > 0;
    }
}

using properties = std::vector<std::pair<std::string, std::string>>;

// Interface the phase runner in main.cpp drives.
class algorithm {
public:
    algorithm(BenchmarkType bench, std::size_t num_alg_measurements, std::chrono::nanoseconds min_time)
        : bench_(bench), sw_(bench == BenchmarkType::CommonSteps ? 7 : (bench == BenchmarkType::Algorithm ? num_alg_measurements : 0), min_time) {}
    virtual ~algorithm() = default;

    // phases with the CommonSteps labels (cross_corr.hpp:168-176)
    void load(const std::filesystem::path &ref, const std::filesystem::path &target) {
        sw_.cpu_measure(0, measure_common(), false, [&] { load_impl(ref, target); });
    }
    void prepare() { sw_.cpu_measure(1, measure_common(), false, [&] { prepare_impl(); }); }
    void transfer() { sw_.cpu_measure(2, measure_common(), uses_device(), [&] { transfer_impl(); }); }
    void run() { sw_.cpu_adaptive_measure(3, measure_common(), uses_device(), [&] { run_impl(); }); }
    void finalize() { sw_.cpu_measure(4, measure_common(), uses_device(), [&] { finalize_impl(); }); }
    void free() { sw_.cpu_measure(5, measure_common(), false, [&] { free_impl(); }); }
    void store_results(const std::filesystem::path &out) {
        sw_.cpu_measure(6, measure_common(), false, [&] { store_results_impl(out); });
    }

    void collect_measurements() {} // device measurements are synchronous here
    void reset_measurements() { sw_.reset(); }

    std::vector<std::string> measurement_labels() const {
        if (measure_common()) return {"Load", "Prepare", "Transfer", "Run", "Finalize", "Free", "Store"};
        return measure_alg() ? measurement_labels_impl() : std::vector<std::string>{};
    }
    const std::vector<measurement_result> &measurements() const { return sw_.results(); }
    virtual properties additional_properties() const { return {}; }
    virtual validation_results validate(const std::optional<std::filesystem::path> &valid_path) const = 0;
    virtual bool uses_device() const = 0;
    virtual bool is_fft() const { return false; }
    // --normalize: FFT algorithms store their results in the definition's layout (fft_alg.hpp:13-20)
    void set_normalize(bool on) { normalize_ = on; }

protected:
    bool normalize_ = false;
    BenchmarkType bench_;
    stopwatch sw_;
    bool measure_common() const { return bench_ == BenchmarkType::CommonSteps; }
    bool measure_alg() const { return bench_ == BenchmarkType::Algorithm; }

    virtual void load_impl(const std::filesystem::path &ref, const std::filesystem::path &target) = 0;
    virtual void prepare_impl() {}
    virtual void transfer_impl() {}
    virtual void run_impl() = 0;
    virtual void finalize_impl() {}
    virtual void free_impl() {}
    virtual void store_results_impl(const std::filesystem::path &out) const = 0;
    virtual std::vector<std::string> measurement_labels_impl() const { return {}; }
};

template <typename REFS, typename TARGETS>
void check_matrices_same_size(const REFS &ref, const TARGETS &target) {
    if (ref.matrix_size() != target.matrix_size())
        throw std::runtime_error("Invalid input matrix sizes, expected ref and target to be the same size: ref = " +
                                 to_string(ref.matrix_size()) + " target = " + to_string(target.matrix_size()));
}

inline void check_input_counts(Mode mode, dsize_t refs, dsize_t targets) {
    // the reference's per-mode loaders read one matrix (load_matrix_from_csv) or an array; a
    // count that does not fit the mode fails here with the same wording as n_to_mn.hpp:58-67
    if (mode == Mode::n_to_mn && (refs == 0 || targets % refs != 0))
        throw std::runtime_error("Invalid input data counts, " + std::to_string(targets) + " is not divisible by " + std::to_string(refs));
    if ((mode == Mode::one_to_one || mode == Mode::one_to_many) && refs != 1)
        throw std::runtime_error("Invalid input data counts, expected one left matrix, got " + std::to_string(refs));
    if (mode == Mode::one_to_one && targets != 1)
        throw std::runtime_error("Invalid input data counts, expected one right matrix, got " + std::to_string(targets));
}

inline dsize_t num_results(Mode mode, dsize_t refs, dsize_t targets) {
    return mode == Mode::n_to_m ? refs * targets : targets;
}

// host cross-correlation of a whole input in the mode's pairing, inputs in FILE order
template <typename T, typename A1, typename A2>
data_array<T> cpu_cross_corr(Mode mode, const data_array<T, A1> &refs, const data_array<T, A2> &targets) {
    // (the reference's by-value n_to_mn overload sizes its result with the number of LEFT
    // matrices, validate.hpp:274, and therefore throws for m > 1; the right count is used here)
    data_array<T> result{result_matrix_size(refs.matrix_size(), targets.matrix_size()),
                         num_results(mode, refs.num_matrices(), targets.num_matrices())};
    switch (mode) {
    case Mode::one_to_one: cpu_cross_corr_one_to_one(refs, targets, result); break;
    case Mode::one_to_many: cpu_cross_corr_one_to_many(refs, targets, result); break;
    case Mode::n_to_mn: cpu_cross_corr_n_to_mn(refs, targets, result); break;
    default: cpu_cross_corr_n_to_m(refs, targets, result); break;
    }
    return result;
}

// ---------------------------------------------------------------- CPU algorithms
// cpu_one_to_one, cpu_one_to_many, cpu_n_to_mn, cpu_n_to_m (one_to_one.hpp:41-84, ...)
template <typename T>
class cpu_algorithm : public algorithm {
public:
    cpu_algorithm(Mode mode, BenchmarkType bench, std::chrono::nanoseconds min_time) : algorithm(bench, 0, min_time), mode_(mode) {}
    bool uses_device() const override { return false; }
    validation_results validate(const std::optional<std::filesystem::path> &valid_path) const override {
        if (valid_path) return validate_result(results_, load_matrix_array_from_csv<T>(*valid_path));
        return validate_result(results_, cpu_cross_corr(mode_, refs_, targets_));
    }

protected:
    void load_impl(const std::filesystem::path &ref, const std::filesystem::path &target) override {
        refs_ = load_matrix_array_from_csv<T>(ref);
        targets_ = load_matrix_array_from_csv<T>(target);
        check_input_counts(mode_, refs_.num_matrices(), targets_.num_matrices());
        check_matrices_same_size(refs_, targets_);
    }
    void prepare_impl() override {
        results_ = data_array<T>{result_matrix_size(refs_.matrix_size(), targets_.matrix_size()),
                                 num_results(mode_, refs_.num_matrices(), targets_.num_matrices())};
    }
    void run_impl() override {
        switch (mode_) {
        case Mode::one_to_one: cpu_cross_corr_one_to_one(refs_, targets_, results_); break;
        case Mode::one_to_many: cpu_cross_corr_one_to_many(refs_, targets_, results_); break;
        case Mode::n_to_mn: cpu_cross_corr_n_to_mn(refs_, targets_, results_); break;
        default: cpu_cross_corr_n_to_m(refs_, targets_, results_); break;
        }
    }
    void store_results_impl(const std::filesystem::path &out) const override { results_.store(out); }

private:
    Mode mode_;
    data_array<T> refs_, targets_, results_;
};

// ---------------------------------------------------------------- GPU algorithms
enum class Family {
    overlap_wise,
    warp_per_overlap,
    warp_per_overlap_lds,
    block_per_overlap,
    shuffle,
    split_row,
    grouped_overlap,
    multimat_right,
    multimat_right_grouped,
    multimat_both,
    multimat_both_grouped
};

// One JSON key of an algorithm: its default, the xcorr_params field it feeds (may be none for
// keys that only exist for drop-in compatibility) and whether it is a fixed value that is
// reported but not read.
// The integers that pick a compiled tile in the library (shifts / matrices per thread) are exact requests there: they
// are passed only when the arguments file holds the key, 0 (the library's own choice) otherwise, and the measurement
// file reports the values the launch really used.
struct arg_spec {
    enum class type { uint, boolean, distribution };
    const char *key;
    type t;
    long long def;
    unsigned xcorr_params::*field;
    bool report = true;
};

struct algorithm_def {
    std::string name;
    Mode mode;
    Family family;
    std::vector<arg_spec> args;
    bool per_left_streams = false; // one launch per left matrix, round robin over num_cuda_streams
    bool per_left_streams_if_asked = false; // the same, but only when the arguments file holds num_cuda_streams
    bool deinterleave = false;     // n_to_mn: right matrices grouped per left matrix on the device
    bool zero_output = false;      // split-row contract: clear the output inside the measured block
    unsigned wpo_variant = 0;
    bool fixed_one_right_per_thread = false; // *_one_to_one flavours of the multi-matrix kernels
    bool shared_mem_rows_rule = false;       // argument_error rule of the shared-memory variants
};

const std::vector<algorithm_def> &gpu_algorithm_defs();

template <typename T>
struct device_entry_points;

template <typename T>
class gpu_algorithm : public algorithm {
public:
    using host_array = data_array<T, pinned_allocator<T>>;

    gpu_algorithm(const algorithm_def &def, const json_args &args, BenchmarkType bench, std::chrono::nanoseconds min_time);
    ~gpu_algorithm() override;

    bool uses_device() const override { return true; }
    properties additional_properties() const override { return props_; }
    validation_results validate(const std::optional<std::filesystem::path> &valid_path) const override;

protected:
    void load_impl(const std::filesystem::path &ref, const std::filesystem::path &target) override;
    void prepare_impl() override;
    void transfer_impl() override;
    void run_impl() override;
    void finalize_impl() override;
    void free_impl() override;
    void store_results_impl(const std::filesystem::path &out) const override;
    std::vector<std::string> measurement_labels_impl() const override { return {"Kernel"}; }

private:
    algorithm_def def_;
    xcorr_params params_ = [] { xcorr_params p{}; p.struct_size = sizeof(xcorr_params); return p; }(); // (XCORR_PARAMS_INIT, without -Wextra's remarks)
    bool zero_output_ = false; // clear the output inside the measured block (split-row contract, column groups)
    bool clear_before_launch_ = false; // ... and the launches of this instance do add into it
    properties props_;
    unsigned num_streams_ = 0;
    host_array refs_, targets_, results_;
    T *d_refs_ = nullptr, *d_targets_ = nullptr, *d_results_ = nullptr;
    std::vector<void *> streams_;

    void launch_all();
    void launch_kernels();
    bool launches_add_into_output();
    void report_effective_arguments();
    void release() noexcept;
    void launch(const T *left, const T *right, T *out, dsize_t n_left, dsize_t n_right, void *stream);
};

std::unique_ptr<algorithm> make_algorithm(const std::string &name, const std::string &data_type, const json_args &args,
                                          BenchmarkType bench, std::chrono::nanoseconds min_time);
std::vector<std::string> algorithm_names();
bool is_algorithm(const std::string &name);
std::optional<Mode> parse_mode(const std::string &name);

} // namespace cross
