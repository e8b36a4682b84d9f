#include "fft_algorithms.hpp"

namespace cross {

const std::vector<fft_algorithm_def> &fft_algorithm_defs() {
    // reference main.cpp:403-409
    static const std::vector<fft_algorithm_def> defs{
        {"fft_orig_one_to_one", Mode::one_to_one, FftVariant::original},
        {"fft_reduced_transfer_one_to_one", Mode::one_to_one, FftVariant::reduced_transfer},
        {"fft_orig_one_to_many", Mode::one_to_many, FftVariant::original},
        {"fft_reduced_transfer_one_to_many", Mode::one_to_many, FftVariant::reduced_transfer},
        {"fft_orig_n_to_mn", Mode::n_to_mn, FftVariant::original},
        {"fft_reduced_transfer_n_to_mn", Mode::n_to_mn, FftVariant::reduced_transfer},
        {"fft_better_n_to_m", Mode::n_to_m, FftVariant::better_hadamard},
    };
    return defs;
}

template <typename T>
fft_algorithm<T>::fft_algorithm(const fft_algorithm_def &def, const json_args &args, BenchmarkType bench, std::chrono::nanoseconds min_time)
    : algorithm(bench, def.variant == FftVariant::reduced_transfer ? 7 : 5, min_time), def_(def) {
    // JSON keys and defaults: one_to_one.hpp:895,1029-1031, n_to_m.hpp:654-655
    if (reduced()) {
        scatter_threads_ = args.value("scatter_threads_per_block", 256u);
        scatter_items_ = args.value("scatter_items_per_thread", 10u);
        props_.emplace_back("scatter_threads_per_block", std::to_string(scatter_threads_));
        props_.emplace_back("scatter_items_per_thread", std::to_string(scatter_items_));
    }
    hadamard_threads_ = args.value("hadamard_threads_per_block", 256u);
    props_.emplace_back("hadamard_threads_per_block", std::to_string(hadamard_threads_));
    if (def.variant == FftVariant::better_hadamard) {
        hadamard_items_ = args.value("hadamard_items_per_thread", 10u);
        props_.emplace_back("hadamard_items_per_thread", std::to_string(hadamard_items_));
    }
}

template <typename T>
std::vector<std::string> fft_algorithm<T>::measurement_labels_impl() const {
    if (reduced()) return {"Forward FFT", "Hadamard", "Inverse FFT", "ToDevice", "Scatter", "Allocation", "Plan"};
    return {"Forward FFT", "Hadamard", "Inverse FFT", "Allocation", "Plan"};
}

template <typename T>
void fft_algorithm<T>::load_impl(const std::filesystem::path &ref, const std::filesystem::path &target) {
    // The reference pads on the host while loading (relative_zero_padding<2>) except in the
    // reduced-transfer variants; here the files are always loaded as they are and the padding is
    // done where the variant does it: on the host in transfer (original, better) or by the
    // scatter kernel on the device (reduced transfer).
    refs_ = load_matrix_array_from_csv<T, pinned_allocator<T>>(ref);
    targets_ = load_matrix_array_from_csv<T, pinned_allocator<T>>(target);
    check_input_counts(def_.mode, refs_.num_matrices(), targets_.num_matrices());
    check_matrices_same_size(refs_, targets_);
}

template <typename T>
void fft_algorithm<T>::prepare_impl() {
    const dsize2_t in = refs_.matrix_size();
    padded_ = dsize2_t{2 * in.x, 2 * in.y};
    spectrum_ = (std::size_t)padded_.y * (padded_.x / 2 + 1);
    const dsize_t n_in = refs_.num_matrices() + targets_.num_matrices();
    const dsize_t n_out = num_results(def_.mode, refs_.num_matrices(), targets_.num_matrices());
    results_ = host_array{padded_, n_out};
    sw_.cpu_measure(slot_allocation(), measure_alg(), false, [&] {
        if (reduced()) xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_inputs_), (refs_.size() + targets_.size()) * sizeof(T)));
        xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_padded_), (std::size_t)n_in * padded_.area() * sizeof(T)));
        xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_results_), results_.size() * sizeof(T)));
        xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_spectra_), (std::size_t)n_in * spectrum_ * 2 * sizeof(T)));
        if (def_.variant == FftVariant::better_hadamard)
            xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_products_), (std::size_t)n_out * spectrum_ * 2 * sizeof(T)));
    });
    sw_.cpu_measure(slot_plan(), measure_alg(), false, [&] {
        fcheck(xcorr_fft_plan_forward(&plan_forward_, padded_.y, padded_.x, n_in, sizeof(T)));
        fcheck(xcorr_fft_plan_inverse(&plan_inverse_, padded_.y, padded_.x, n_out, sizeof(T)));
    });
}

template <typename T>
void fft_algorithm<T>::transfer_impl() {
    const dsize2_t in = refs_.matrix_size();
    const dsize_t n_in = refs_.num_matrices() + targets_.num_matrices();
    if (reduced()) {
        // unpadded inputs cross the bus, the device pads (one_to_one.hpp:1075-1093)
        sw_.cpu_measure(slot_to_device(), measure_alg(), false, [&] {
            xcheck(xcorr_memcpy_h2d(d_inputs_, refs_.data(), refs_.size() * sizeof(T)));
            xcheck(xcorr_memcpy_h2d(d_inputs_ + refs_.size(), targets_.data(), targets_.size() * sizeof(T)));
        });
        xcheck(xcorr_memset_async(d_padded_, 0, (std::size_t)n_in * padded_.area() * sizeof(T), nullptr));
        sw_.device_adaptive_measure(slot_scatter(), measure_alg(), [&] {
            if constexpr (sizeof(T) == 4)
                fcheck(xcorr_scatter_f32(d_inputs_, d_padded_, in.x, in.y, n_in, padded_.x, padded_.y, 0, 0, scatter_threads_, scatter_items_, nullptr));
            else
                fcheck(xcorr_scatter_f64(d_inputs_, d_padded_, in.x, in.y, n_in, padded_.x, padded_.y, 0, 0, scatter_threads_, scatter_items_, nullptr));
        });
        return;
    }
    // padded on the host, the padded matrices cross the bus (what loading with
    // relative_zero_padding<2> amounts to in the reference)
    host_array padded{padded_, n_in};
    std::fill(padded.data(), padded.data() + padded.size(), T(0));
    for (dsize_t m = 0; m < n_in; ++m) {
        const T *src = m < refs_.num_matrices() ? refs_.matrix(m) : targets_.matrix(m - refs_.num_matrices());
        T *dst = padded.matrix(m);
        for (dsize_t y = 0; y < in.y; ++y) std::copy(src + (std::size_t)y * in.x, src + (std::size_t)(y + 1) * in.x, dst + (std::size_t)y * padded_.x);
    }
    xcheck(xcorr_memcpy_h2d(d_padded_, padded.data(), padded.size() * sizeof(T)));
}

template <typename T>
void fft_algorithm<T>::run_impl() {
    const dsize_t n_left = refs_.num_matrices(), n_right = targets_.num_matrices();
    T *left_spectra = d_spectra_, *right_spectra = d_spectra_ + (std::size_t)n_left * spectrum_ * 2;
    const unsigned fft_cols = padded_.x / 2 + 1, fft_rows = padded_.y;
    // library calls are asynchronous: wall clock with a device synchronisation, like the reference's
    // CPU_ADAPTIVE_MEASURE around cuFFT (one_to_one.hpp:950-967); the hadamard kernel uses events
    sw_.cpu_adaptive_measure(0, measure_alg(), true, [&] { fcheck(xcorr_fft_exec_forward(plan_forward_, d_padded_, d_spectra_)); });
    T *products = def_.variant == FftVariant::better_hadamard ? d_products_ : right_spectra;
    auto hadamard = [&] {
        if (def_.variant == FftVariant::better_hadamard) {
            if constexpr (sizeof(T) == 4)
                fcheck(xcorr_hadamard_n_to_m_over_output_f32(left_spectra, right_spectra, d_products_, fft_cols, fft_rows, n_left, n_right,
                                                             hadamard_threads_, hadamard_items_, nullptr));
            else
                fcheck(xcorr_hadamard_n_to_m_over_output_f64(left_spectra, right_spectra, d_products_, fft_cols, fft_rows, n_left, n_right,
                                                             hadamard_threads_, hadamard_items_, nullptr));
        } else {
            // in place over the right spectra; n_to_mn: file order, right t*n + r pairs with left r
            const unsigned per_pic = n_left, batch = n_right / n_left;
            if constexpr (sizeof(T) == 4)
                fcheck(xcorr_hadamard_original_f32(left_spectra, right_spectra, fft_cols, fft_rows, per_pic, batch, hadamard_threads_, nullptr));
            else
                fcheck(xcorr_hadamard_original_f64(left_spectra, right_spectra, fft_cols, fft_rows, per_pic, batch, hadamard_threads_, nullptr));
        }
    };
    sw_.device_adaptive_measure(1, measure_alg(), hadamard);
    sw_.cpu_adaptive_measure(2, measure_alg(), true, [&] { fcheck(xcorr_fft_exec_inverse(plan_inverse_, products, d_results_)); });
    // The in-place hadamard product and the inverse transform consume their inputs: when the adaptive
    // measurement repeated one of them, compute the result once more from the padded inputs.
    if (measure_alg() && (sw_.results()[1].get_iterations() > 1 || sw_.results()[2].get_iterations() > 1)) {
        fcheck(xcorr_fft_exec_forward(plan_forward_, d_padded_, d_spectra_));
        hadamard();
        fcheck(xcorr_fft_exec_inverse(plan_inverse_, products, d_results_));
    }
}

template <typename T>
void fft_algorithm<T>::finalize_impl() {
    xcheck(xcorr_memcpy_d2h(results_.data(), d_results_, results_.size() * sizeof(T)));
}

template <typename T>
void fft_algorithm<T>::free_impl() {
    fcheck(xcorr_fft_plan_destroy(plan_inverse_));
    fcheck(xcorr_fft_plan_destroy(plan_forward_));
    plan_inverse_ = plan_forward_ = nullptr;
    for (T **p : {&d_products_, &d_spectra_, &d_results_, &d_padded_, &d_inputs_}) {
        if (*p) xcheck(xcorr_free(*p));
        *p = nullptr;
    }
}

template <typename T>
void fft_algorithm<T>::store_results_impl(const std::filesystem::path &out) const {
    // reference fft_alg.hpp:13-20
    if (normalize_)
        normalize_fft_results(results_).store(out);
    else
        results_.store(out);
}

template <typename T>
validation_results fft_algorithm<T>::validate(const std::optional<std::filesystem::path> &valid_path) const {
    // cross_corr.hpp:90-97. Without a file the valid results are computed from the inputs as loaded
    // (the reference computes them from its host-padded copies, which have a different size).
    auto norm = normalize_fft_results(results_);
    if (valid_path) return validate_result(norm, load_matrix_array_from_csv<T>(*valid_path));
    return validate_result(norm, cpu_cross_corr<T>(def_.mode, refs_, targets_));
}

template class fft_algorithm<float>;
template class fft_algorithm<double>;

} // namespace cross
