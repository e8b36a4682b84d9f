// Matrix array container and the CSV matrix format of the reference
// (matrix.hpp:94-185 reader/writer, :410-619 data_array): line 1 is
// "# <rows>,<cols>[,<num_matrices>]", then rows * num_matrices lines of cols
// comma-separated reals; matrices follow each other without separators.
#pragma once

#include <cstdlib>
#include <fstream>
#include <filesystem>
#include <istream>
#include <ostream>
#include <stdexcept>
#include <string>
#include <vector>

namespace cross {

using dsize_t = unsigned int;

struct dsize2_t {
    dsize_t x = 0, y = 0; // x = columns, y = rows (reference types.cuh:18-135)
    dsize_t area() const { return x * y; }
    bool operator==(const dsize2_t &o) const { return x == o.x && y == o.y; }
    bool operator!=(const dsize2_t &o) const { return !(*this == o); }
};
inline std::string to_string(const dsize2_t &v) { return "[" + std::to_string(v.x) + "," + std::to_string(v.y) + "]"; }
inline dsize2_t result_matrix_size(dsize2_t a, dsize2_t b) { return dsize2_t{a.x + b.x - 1, a.y + b.y - 1}; }

// reference matrix.hpp:614-618
inline dsize_t get_interleaved_index(dsize_t idx, dsize_t group_size, dsize_t num_groups) {
    return (idx % group_size) * num_groups + idx / group_size;
}

template <typename T>
inline T from_string(const std::string &in);
// std::stof / std::stod semantics (host_helpers.hpp:12-24): leading blanks allowed, trailing
// characters ignored, no digits at all is an error
template <>
inline float from_string<float>(const std::string &in) { return std::stof(in); }
template <>
inline double from_string<double>(const std::string &in) { return std::stod(in); }

namespace csv {

// Fields of one line, comma separated; double quotes group a field and a backslash
// escapes the next character (what boost's escaped_list_separator, used by the
// reference, accepts).
inline void split_line(const std::string &line, std::vector<std::string> &out) {
    out.clear();
    std::string field;
    bool quoted = false;
    for (std::size_t i = 0; i < line.size(); ++i) {
        char c = line[i];
        if (c == '\\' && i + 1 < line.size()) {
            char n = line[++i];
            field += n == 'n' ? '\n' : n;
        } else if (c == '"') {
            quoted = !quoted;
        } else if (c == ',' && !quoted) {
            out.push_back(field);
            field.clear();
        } else if (c != '\r') {
            field += c;
        }
    }
    out.push_back(field);
}

inline void read_header(std::istream &in, dsize2_t &size, dsize_t &num_matrices) {
    std::string line;
    if (!std::getline(in, line)) throw std::runtime_error{"Could not read file header"};
    if (line.compare(0, 2, "# ") != 0) throw std::runtime_error{"Invalid file header format"};
    std::vector<std::string> tok;
    split_line(line.substr(2), tok);
    if (tok.empty() || (tok.size() == 1 && tok[0].empty())) throw std::runtime_error{"Missing matrix header"};
    dsize_t rows = static_cast<dsize_t>(std::stoi(tok[0]));
    if (tok.size() < 2) throw std::runtime_error("Missing number of columns");
    dsize_t cols = static_cast<dsize_t>(std::stoi(tok[1]));
    num_matrices = 1;
    if (tok.size() >= 3) {
        num_matrices = static_cast<dsize_t>(std::stoi(tok[2]));
        if (tok.size() > 3) throw std::runtime_error("Invalid matrix header format, too many tokens");
    }
    size = dsize2_t{cols, rows};
}

template <typename T>
void read_data(std::istream &in, dsize2_t matrix_size, T *out) {
    std::string line;
    std::vector<std::string> tok;
    for (dsize_t y = 0; y < matrix_size.y; ++y) {
        if (!std::getline(in, line)) throw std::runtime_error{"Failed to read line " + std::to_string(y) + " from csv file"};
        split_line(line, tok);
        if (tok.size() > matrix_size.x)
            throw std::runtime_error{"Line " + std::to_string(y) + " is too long, expected " + std::to_string(matrix_size.x) + "values"};
        if (tok.size() < matrix_size.x)
            throw std::runtime_error{"Line" + std::to_string(y) + " is too short, expected " + std::to_string(matrix_size.x) +
                                     ", got " + std::to_string(tok.size()) + " values"};
        for (dsize_t x = 0; x < matrix_size.x; ++x) out[(std::size_t)y * matrix_size.x + x] = from_string<T>(tok[x]);
    }
}

inline void write_header(std::ostream &out, dsize2_t size, dsize_t num_matrices) {
    out << "# " << size.y << "," << size.x << "," << num_matrices << "\n";
}

// std::fixed with the default precision of 6 (reference matrix.hpp:176). The reference
// indexes rows with the row COUNT as pitch (matrix.hpp:180), which is only right for
// square matrices; the column count is used here.
template <typename T>
void write_data(std::ostream &out, dsize2_t matrix_size, const T *data) {
    out << std::fixed;
    for (dsize_t y = 0; y < matrix_size.y; ++y) {
        const char *sep = "";
        for (dsize_t x = 0; x < matrix_size.x; ++x) {
            out << sep << data[(std::size_t)y * matrix_size.x + x];
            sep = ",";
        }
        out << "\n";
    }
}

} // namespace csv

template <typename T, typename ALLOC = std::allocator<T>>
class data_array {
public:
    using value_type = T;

    data_array() = default;
    explicit data_array(dsize2_t matrix_size, dsize_t num_matrices = 1)
        : num_matrices_(num_matrices), matrix_size_(matrix_size), data_((std::size_t)matrix_size.area() * num_matrices) {}

    static data_array load_from_csv(std::istream &in) {
        dsize2_t size;
        dsize_t n;
        csv::read_header(in, size, n);
        data_array a{size, n};
        for (dsize_t i = 0; i < n; ++i) csv::read_data<T>(in, size, a.data() + (std::size_t)size.area() * i);
        return a;
    }

    // File matrix i is placed at slot (i % group_size) * num_groups + i / group_size, so that the
    // right matrices of left matrix l become contiguous (reference matrix.hpp:462-503).
    static data_array load_interleaved_from_csv(std::istream &in, dsize_t group_size) {
        dsize2_t size;
        dsize_t n;
        csv::read_header(in, size, n);
        if (group_size == 0 || n % group_size != 0)
            throw std::runtime_error{"Data array cannot be interleaved, as number of matrices is not divisible by group size"};
        dsize_t num_groups = n / group_size;
        data_array a{size, n};
        for (dsize_t i = 0; i < n; ++i)
            csv::read_data<T>(in, size, a.data() + (std::size_t)size.area() * get_interleaved_index(i, group_size, num_groups));
        return a;
    }

    void store_to_csv(std::ostream &out) const {
        csv::write_header(out, matrix_size_, num_matrices_);
        for (dsize_t i = 0; i < num_matrices_; ++i) csv::write_data(out, matrix_size_, data() + (std::size_t)matrix_size_.area() * i);
    }

    // inverse of load_interleaved_from_csv; num_groups is the group count of the original input
    void store_interleaved_to_csv(std::ostream &out, dsize_t num_groups) const {
        if (num_groups == 0 || num_matrices_ % num_groups != 0)
            throw std::runtime_error{"Data array cannot be interleaved, as number of matrices is not divisible by group size"};
        csv::write_header(out, matrix_size_, num_matrices_);
        dsize_t group_size = num_matrices_ / num_groups;
        for (dsize_t i = 0; i < num_matrices_; ++i)
            csv::write_data(out, matrix_size_, data() + (std::size_t)matrix_size_.area() * get_interleaved_index(i, group_size, num_groups));
    }

    template <typename OUT_ALLOC = ALLOC>
    data_array<T, OUT_ALLOC> interleave(dsize_t group_size) const {
        data_array<T, OUT_ALLOC> out{matrix_size_, num_matrices_};
        dsize_t num_groups = num_matrices_ / group_size;
        std::size_t area = matrix_size_.area();
        for (dsize_t i = 0; i < num_matrices_; ++i) {
            const T *src = data() + area * i;
            T *dst = out.data() + area * get_interleaved_index(i, group_size, num_groups);
            for (std::size_t k = 0; k < area; ++k) dst[k] = src[k];
        }
        return out;
    }

    std::size_t size() const { return data_.size(); }
    dsize_t num_matrices() const { return num_matrices_; }
    dsize2_t matrix_size() const { return matrix_size_; }
    T *data() { return data_.data(); }
    const T *data() const { return data_.data(); }
    T *matrix(dsize_t i) { return data() + (std::size_t)matrix_size_.area() * i; }
    const T *matrix(dsize_t i) const { return data() + (std::size_t)matrix_size_.area() * i; }
    const T *begin() const { return data(); }
    const T *end() const { return data() + size(); }

private:
    dsize_t num_matrices_ = 0;
    dsize2_t matrix_size_{};
    std::vector<T, ALLOC> data_;
};

template <typename T, typename ALLOC = std::allocator<T>>
data_array<T, ALLOC> load_matrix_array_from_csv(const std::filesystem::path &path) {
    std::ifstream file(path);
    if (!file) throw std::runtime_error("Could not open " + path.string());
    return data_array<T, ALLOC>::load_from_csv(file);
}

template <typename T, typename ALLOC = std::allocator<T>>
data_array<T, ALLOC> load_interleaved_matrix_array_from_csv(const std::filesystem::path &path, dsize_t group_size) {
    std::ifstream file(path);
    if (!file) throw std::runtime_error("Could not open " + path.string());
    return data_array<T, ALLOC>::load_interleaved_from_csv(file, group_size);
}

} // namespace cross
