// FFT-based cross-correlation algorithms of the `cross` binary: the reference's comparison
// baseline (fft_original_alg_*, fft_reduced_transfer_*, fft_better_hadamard_alg_n_to_m in
// one_to_one.hpp:888-1150, one_to_many.hpp:502-780, n_to_mn.hpp:720-1000, n_to_m.hpp:647-790)
// on hipFFT through libxcorr_fft.so. Zero-padded inputs of twice the size are transformed,
// the left spectra are multiplied with the conjugated right spectra and transformed back; the
// raw result is the un-normalised CIRCULAR correlation of the padded size, which
// normalize_fft_results() turns into the (2 rows - 1) x (2 cols - 1) layout of the definition.
#pragma once

#include "algorithms.hpp"
#include "../../include/xcorr_fft.h"

namespace cross {

inline void fcheck(int code) {
    if (code != XCORR_OK) throw std::runtime_error(xcorr_fft_last_error());
}

// reference fft_helpers.hpp:193-262: swap the quadrants of the circular result around the
// (empty) middle row and column, drop those, divide by the number of elements
template <typename T, typename ALLOC>
data_array<T> normalize_fft_results(const data_array<T, ALLOC> &res) {
    const dsize2_t rs = res.matrix_size();
    data_array<T> norm{dsize2_t{rs.x - 1, rs.y - 1}, res.num_matrices()};
    const dsize2_t ns = norm.matrix_size();
    const dsize_t empty_x = rs.x / 2, empty_y = rs.y / 2;
    const T area = static_cast<T>(rs.area());
    for (dsize_t m = 0; m < res.num_matrices(); ++m) {
        const T *src = res.matrix(m);
        T *dst = norm.matrix(m);
        auto copy = [&](dsize_t sx, dsize_t sy, dsize_t w, dsize_t h, dsize_t tx, dsize_t ty) {
            for (dsize_t y = 0; y < h; ++y)
                for (dsize_t x = 0; x < w; ++x) dst[(std::size_t)(ty + y) * ns.x + tx + x] = src[(std::size_t)(sy + y) * rs.x + sx + x] / area;
        };
        copy(0, 0, empty_x, empty_y, ns.x / 2, ns.y / 2);                                  // top left -> bottom right
        copy(empty_x + 1, 0, rs.x - empty_x - 1, empty_y, 0, ns.y / 2);                   // top right -> bottom left
        copy(0, empty_y + 1, empty_x, rs.y - empty_y - 1, ns.x / 2, 0);                   // bottom left -> top right
        copy(empty_x + 1, empty_y + 1, rs.x - empty_x - 1, rs.y - empty_y - 1, 0, 0);     // bottom right -> top left
    }
    return norm;
}

enum class FftVariant { original, reduced_transfer, better_hadamard };

struct fft_algorithm_def {
    const char *name;
    Mode mode;
    FftVariant variant;
};

const std::vector<fft_algorithm_def> &fft_algorithm_defs();

template <typename T>
class fft_algorithm : public algorithm {
public:
    using host_array = data_array<T, pinned_allocator<T>>;

    fft_algorithm(const fft_algorithm_def &def, const json_args &args, BenchmarkType bench, std::chrono::nanoseconds min_time);

    bool uses_device() const override { return true; }
    bool is_fft() const override { return true; }
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
    std::vector<std::string> measurement_labels_impl() const override;

private:
    fft_algorithm_def def_;
    properties props_;
    unsigned hadamard_threads_ = 256, hadamard_items_ = 10, scatter_threads_ = 256, scatter_items_ = 10;
    host_array refs_, targets_, results_; // unpadded inputs, raw (padded-size, circular) results
    dsize2_t padded_{};
    std::size_t spectrum_ = 0;            // complex elements of one transformed matrix
    T *d_inputs_ = nullptr, *d_padded_ = nullptr, *d_results_ = nullptr;
    T *d_spectra_ = nullptr, *d_products_ = nullptr; // interleaved complex
    void *plan_forward_ = nullptr, *plan_inverse_ = nullptr;

    bool reduced() const { return def_.variant == FftVariant::reduced_transfer; }
    // measurement slots (labels of the reference's classes)
    std::size_t slot_to_device() const { return 3; }
    std::size_t slot_scatter() const { return 4; }
    std::size_t slot_allocation() const { return reduced() ? 5 : 3; }
    std::size_t slot_plan() const { return reduced() ? 6 : 4; }
};

} // namespace cross
