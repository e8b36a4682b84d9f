// The reference's CPU path: the definition-based cross-correlation on the host
// (validate.hpp:94-132), its drivers for the four input modes (validate.hpp:216-298),
// the element-wise validation statistic (validate.hpp:134-188) and how it is printed
// (validate.hpp:24-92). It backs the cpu_* algorithms and `--validate` without a file;
// the GPU algorithms never compute through it.
#pragma once

#include <algorithm>
#include <cmath>
#include <limits>
#include <ostream>
#include <sstream>
#include <stdexcept>
#include <string>

#include "matrix.hpp"

namespace cross {

class validation_results {
public:
    validation_results() : empty_(true) {}
    validation_results(double diff_max, double diff_mean, double diff_std_dev, double at_max_result, double at_max_valid)
        : empty_(false), diff_max_(diff_max), diff_mean_(diff_mean), diff_std_dev_(diff_std_dev),
          at_max_result_(at_max_result), at_max_valid_(at_max_valid) {}
    bool empty() const { return empty_; }
    double get_diff_max() const { return diff_max_; }
    double get_diff_mean() const { return diff_mean_; }
    double get_diff_std_dev() const { return diff_std_dev_; }
    double at_max_result() const { return at_max_result_; }
    double at_max_valid() const { return at_max_valid_; }
    std::string csv_header() const { return "Max,Mean,Stddev"; }
    std::string csv_data() const {
        std::stringstream ss;
        ss << std::scientific << diff_max_ << "," << diff_mean_ << "," << diff_std_dev_;
        return ss.str();
    }

private:
    bool empty_;
    double diff_max_ = 0, diff_mean_ = 0, diff_std_dev_ = 0, at_max_result_ = 0, at_max_valid_ = 0;
};

// reference validate.hpp:78-92: "Max: <max> (<actual> instead of <valid>)"
inline std::ostream &operator<<(std::ostream &out, const validation_results &res) {
    if (res.empty()) {
        out << "No validation\n";
    } else {
        out << "Difference from valid values:\n";
        out << "Max: " << res.get_diff_max() << " (" << std::fixed << res.at_max_result() << " instead of " << res.at_max_valid() << ")\n";
        out.unsetf(std::ios_base::fixed);
        out << std::scientific;
        out << "Mean: " << res.get_diff_mean() << "\n";
        out << "Stddev: " << res.get_diff_std_dev() << "\n";
        out.unsetf(std::ios_base::scientific);
    }
    return out;
}

// validate.hpp:94-114: rows outer, columns inner, accumulator of the element type
template <typename T>
T hadamard_and_sum(const T *ref, const T *target, dsize2_t size, int offset_x, int offset_y) {
    int x_start = std::max(offset_x, 0), x_end = std::min((int)size.x + offset_x, (int)size.x);
    int y_start = std::max(offset_y, 0), y_end = std::min((int)size.y + offset_y, (int)size.y);
    T sum = T{};
    for (int y = y_start; y < y_end; ++y) {
        const T *ref_row = ref + (std::size_t)y * size.x;
        const T *target_row = target + (std::size_t)(y - offset_y) * size.x;
        for (int x = x_start; x < x_end; ++x) sum += target_row[x - offset_x] * ref_row[x];
    }
    return sum;
}

// validate.hpp:117-132
template <typename T>
void naive_cpu_cross_corr(const T *ref, const T *target, T *res, dsize2_t size) {
    dsize2_t search = result_matrix_size(size, size);
    int half_x = ((int)search.x - 1) / 2, half_y = ((int)search.y - 1) / 2;
    for (int y = -half_y; y <= half_y; ++y)
        for (int x = -half_x; x <= half_x; ++x)
            res[(std::size_t)(y + half_y) * search.x + (x + half_x)] = hadamard_and_sum(ref, target, size, x, y);
}

inline void check_matrix_size(dsize2_t ref, dsize2_t target, dsize2_t result) {
    if (result != result_matrix_size(ref, target))
        throw std::runtime_error("Invalid result matrix size " + to_string(result) + ", expected " + to_string(result_matrix_size(ref, target)));
}
inline void check_num_result_matrices(dsize_t actual, dsize_t expected) {
    if (actual != expected)
        throw std::runtime_error("Invalid number of result matrices " + std::to_string(actual) + ", expected " + std::to_string(expected));
}

template <typename REF, typename TARGET, typename RESULT>
void cpu_cross_corr_one_to_one(const REF &ref, const TARGET &target, RESULT &result) {
    check_matrix_size(ref.matrix_size(), target.matrix_size(), result.matrix_size());
    check_num_result_matrices(result.num_matrices(), 1);
    naive_cpu_cross_corr(ref.matrix(0), target.matrix(0), result.matrix(0), ref.matrix_size());
}

template <typename REF, typename TARGET, typename RESULT>
void cpu_cross_corr_one_to_many(const REF &ref, const TARGET &target, RESULT &result) {
    check_matrix_size(ref.matrix_size(), target.matrix_size(), result.matrix_size());
    check_num_result_matrices(result.num_matrices(), target.num_matrices());
    for (dsize_t i = 0; i < target.num_matrices(); ++i)
        naive_cpu_cross_corr(ref.matrix(0), target.matrix(i), result.matrix(i), ref.matrix_size());
}

template <typename REF, typename TARGET, typename RESULT>
void cpu_cross_corr_n_to_mn(const REF &ref, const TARGET &target, RESULT &result) {
    check_matrix_size(ref.matrix_size(), target.matrix_size(), result.matrix_size());
    check_num_result_matrices(result.num_matrices(), target.num_matrices());
    if (ref.num_matrices() == 0 || target.num_matrices() % ref.num_matrices() != 0)
        throw std::runtime_error("Invalid ref and target data counts, " + std::to_string(target.num_matrices()) +
                                 " is not divisible by " + std::to_string(ref.num_matrices()));
    for (dsize_t r = 0; r < ref.num_matrices(); ++r)
        for (dsize_t t = 0; t < target.num_matrices() / ref.num_matrices(); ++t) {
            dsize_t index = t * ref.num_matrices() + r;
            naive_cpu_cross_corr(ref.matrix(r), target.matrix(index), result.matrix(index), ref.matrix_size());
        }
}

template <typename REF, typename TARGET, typename RESULT>
void cpu_cross_corr_n_to_m(const REF &ref, const TARGET &target, RESULT &result) {
    check_matrix_size(ref.matrix_size(), target.matrix_size(), result.matrix_size());
    check_num_result_matrices(result.num_matrices(), ref.num_matrices() * target.num_matrices());
    for (dsize_t r = 0; r < ref.num_matrices(); ++r)
        for (dsize_t t = 0; t < target.num_matrices(); ++t)
            naive_cpu_cross_corr(ref.matrix(r), target.matrix(t), result.matrix(r * target.num_matrices() + t), ref.matrix_size());
}

// validate.hpp:134-188: per element |a-b| / max(|a|,|b|) in the result's element type, 0 when
// both are at most 1e-5 in magnitude; max, mean and population standard deviation in double;
// the reported pair is the first element that attains the maximum.
template <typename MAT1, typename MAT2>
validation_results validate_result(const MAT1 &result, const MAT2 &valid) {
    if (result.size() != valid.size()) throw std::runtime_error("Cannot validate matrices of different sizes");
    using T = typename MAT1::value_type;
    const T epsilon = static_cast<T>(1e-5);
    double max = -std::numeric_limits<double>::infinity(), sum = 0, sum_sq = 0;
    std::size_t at = 0, n = result.size();
    const auto *a = result.begin();
    const auto *b = valid.begin();
    for (std::size_t i = 0; i < n; ++i) {
        T x = a[i], y = static_cast<T>(b[i]);
        T d = (std::abs(x) <= epsilon && std::abs(y) <= epsilon) ? T{0} : std::abs(x - y) / std::max(std::abs(x), std::abs(y));
        double dd = static_cast<double>(d);
        if (dd > max) {
            max = dd;
            at = i;
        }
        sum += dd;
        sum_sq += dd * dd;
    }
    if (n == 0) {
        double nan = std::numeric_limits<double>::quiet_NaN();
        return validation_results{nan, nan, nan, nan, nan};
    }
    double mean = sum / (double)n;
    return validation_results{max, mean, std::sqrt(sum_sq / (double)n - mean * mean), (double)a[at], (double)b[at]};
}

} // namespace cross
