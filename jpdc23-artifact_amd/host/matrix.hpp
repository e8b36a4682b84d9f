// Matrix array container and the CSV matrix format of the reference
// (matrix.hpp:94-185 reader/writer, :410-619 data_array): line 1 is
// "# <rows>,<cols>[,<num_matrices>]", then rows * num_matrices lines of cols
// comma-separated reals; matrices follow each other without separators.
//
// Besides the text format there is a binary one (the reference only has a commented-out
// stub for it, matrix.hpp:49-91): a 32-byte little-endian header - "XCORRMAT", version 1,
// bytes per element (4 or 8), rows, cols, number of matrices, 0 - followed by the matrices,
// row-major. Readers recognise it by the magic; writers use it for paths that end in ".bin".
#pragma once

#include <cerrno>
#include <charconv>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
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

// strtof / strtod at the start of a field, with the error behaviour of std::stof / std::stod
// (which call them): no digits -> invalid_argument, ERANGE -> out_of_range
inline float parse_at(const char *p, char **end, float) { return std::strtof(p, end); }
inline double parse_at(const char *p, char **end, double) { return std::strtod(p, end); }

template <typename T>
void read_data(std::istream &in, dsize2_t matrix_size, T *out) {
    std::string line;
    std::vector<std::string> tok;
    for (dsize_t y = 0; y < matrix_size.y; ++y) {
        if (!std::getline(in, line)) throw std::runtime_error{"Failed to read line " + std::to_string(y) + " from csv file"};
        T *row = out + (std::size_t)y * matrix_size.x;
        if (line.find_first_of("\"\\") == std::string::npos) {
            // plain line (what numpy.savetxt and the writer below produce): numbers are parsed in
            // place, no per-field strings. A number cannot contain a comma, so parsing from the
            // start of a field gives what std::stof of the field gives.
            dsize_t fields = 1;
            for (char c : line) fields += c == ',';
            if (fields > matrix_size.x)
                throw std::runtime_error{"Line " + std::to_string(y) + " is too long, expected " + std::to_string(matrix_size.x) + "values"};
            if (fields < matrix_size.x)
                throw std::runtime_error{"Line" + std::to_string(y) + " is too short, expected " + std::to_string(matrix_size.x) +
                                         ", got " + std::to_string(fields) + " values"};
            const char *p = line.c_str(), *line_end = p + line.size();
            for (dsize_t x = 0; x < matrix_size.x; ++x) {
                // std::from_chars is several times faster than strtod and equally exact; whatever
                // it does not take whole (leading blank, '+', hex, trailing characters, out of
                // range) goes to strtod, whose verdict is std::stof's
                T v;
                auto r = std::from_chars(p, line_end, v);
                if (r.ec == std::errc() && (r.ptr == line_end || *r.ptr == ',')) {
                    row[x] = v;
                    p = r.ptr;
                } else {
                    char *end = nullptr;
                    errno = 0;
                    row[x] = parse_at(p, &end, T{});
                    if (end == p) throw std::invalid_argument(sizeof(T) == 4 ? "stof" : "stod");
                    if (errno == ERANGE) throw std::out_of_range(sizeof(T) == 4 ? "stof" : "stod");
                    p = std::strchr(end, ',');
                    if (!p) p = line_end;
                }
                if (p != line_end) ++p; // past the comma
            }
            continue;
        }
        split_line(line, tok);
        if (tok.size() > matrix_size.x)
            throw std::runtime_error{"Line " + std::to_string(y) + " is too long, expected " + std::to_string(matrix_size.x) + "values"};
        if (tok.size() < matrix_size.x)
            throw std::runtime_error{"Line" + std::to_string(y) + " is too short, expected " + std::to_string(matrix_size.x) +
                                     ", got " + std::to_string(tok.size()) + " values"};
        for (dsize_t x = 0; x < matrix_size.x; ++x) row[x] = from_string<T>(tok[x]);
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
    // "%f" of the value widened to double is what `out << std::fixed << value` prints; a row is
    // formatted into one buffer and written at once
    std::string buf;
    char num[352]; // longest "%f" of a double: 309 integer digits, sign, point, 6 decimals
    for (dsize_t y = 0; y < matrix_size.y; ++y) {
        buf.clear();
        for (dsize_t x = 0; x < matrix_size.x; ++x) {
            if (x) buf += ',';
            int n = std::snprintf(num, sizeof(num), "%f", (double)data[(std::size_t)y * matrix_size.x + x]);
            buf.append(num, n > 0 ? (std::size_t)n : 0);
        }
        buf += '\n';
        out.write(buf.data(), (std::streamsize)buf.size());
    }
}

} // namespace csv

namespace binary {

constexpr char MAGIC[8] = {'X', 'C', 'O', 'R', 'R', 'M', 'A', 'T'};

struct header {
    char magic[8];
    std::uint32_t version, elem_bytes, rows, cols, num_matrices, reserved;
};
static_assert(sizeof(header) == 32, "binary matrix file header");

inline bool has_magic(std::istream &in) {
    char m[8] = {};
    auto pos = in.tellg();
    in.read(m, 8);
    bool ok = in.gcount() == 8 && std::memcmp(m, MAGIC, 8) == 0;
    in.clear();
    in.seekg(pos);
    return ok;
}

inline header read_header(std::istream &in) {
    header h{};
    if (!in.read(reinterpret_cast<char *>(&h), sizeof(h)) || std::memcmp(h.magic, MAGIC, 8) != 0)
        throw std::runtime_error{"Invalid binary matrix file header"};
    if (h.version != 1 || (h.elem_bytes != 4 && h.elem_bytes != 8))
        throw std::runtime_error{"Unsupported binary matrix file version or element size"};
    return h;
}

// one matrix of `count` elements stored with `elem_bytes` per element, converted to T
template <typename T>
void read_matrix(std::istream &in, std::uint32_t elem_bytes, std::size_t count, T *out) {
    if (elem_bytes == sizeof(T)) {
        if (!in.read(reinterpret_cast<char *>(out), (std::streamsize)(count * sizeof(T)))) throw std::runtime_error{"Binary matrix file is too short"};
        return;
    }
    std::vector<char> raw(count * elem_bytes);
    if (!in.read(raw.data(), (std::streamsize)raw.size())) throw std::runtime_error{"Binary matrix file is too short"};
    for (std::size_t i = 0; i < count; ++i) {
        if (elem_bytes == 4) {
            float v;
            std::memcpy(&v, raw.data() + i * 4, 4);
            out[i] = static_cast<T>(v);
        } else {
            double v;
            std::memcpy(&v, raw.data() + i * 8, 8);
            out[i] = static_cast<T>(v);
        }
    }
}

template <typename T>
void write_header(std::ostream &out, dsize2_t size, dsize_t num_matrices) {
    header h{};
    std::memcpy(h.magic, MAGIC, 8);
    h.version = 1;
    h.elem_bytes = sizeof(T);
    h.rows = size.y;
    h.cols = size.x;
    h.num_matrices = num_matrices;
    out.write(reinterpret_cast<const char *>(&h), sizeof(h));
}

inline bool path_is_binary(const std::filesystem::path &p) { return p.extension() == ".bin"; }

} // namespace binary

template <typename T, typename ALLOC = std::allocator<T>>
class data_array {
public:
    using value_type = T;

    data_array() = default;
    explicit data_array(dsize2_t matrix_size, dsize_t num_matrices = 1)
        : num_matrices_(num_matrices), matrix_size_(matrix_size), data_((std::size_t)matrix_size.area() * num_matrices) {}

    // (either format; the name is the reference's)
    static data_array load_from_csv(std::istream &in) {
        if (binary::has_magic(in)) {
            binary::header h = binary::read_header(in);
            data_array a{dsize2_t{h.cols, h.rows}, h.num_matrices};
            for (dsize_t i = 0; i < h.num_matrices; ++i) binary::read_matrix<T>(in, h.elem_bytes, a.matrix_size().area(), a.matrix(i));
            return a;
        }
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
        const bool bin = binary::has_magic(in);
        binary::header h{};
        dsize2_t size;
        dsize_t n;
        if (bin) {
            h = binary::read_header(in);
            size = dsize2_t{h.cols, h.rows};
            n = h.num_matrices;
        } else {
            csv::read_header(in, size, n);
        }
        if (group_size == 0 || n % group_size != 0)
            throw std::runtime_error{"Data array cannot be interleaved, as number of matrices is not divisible by group size"};
        dsize_t num_groups = n / group_size;
        data_array a{size, n};
        for (dsize_t i = 0; i < n; ++i) {
            T *dst = a.data() + (std::size_t)size.area() * get_interleaved_index(i, group_size, num_groups);
            if (bin)
                binary::read_matrix<T>(in, h.elem_bytes, size.area(), dst);
            else
                csv::read_data<T>(in, size, dst);
        }
        return a;
    }

    void store_to_binary(std::ostream &out) const {
        binary::write_header<T>(out, matrix_size_, num_matrices_);
        out.write(reinterpret_cast<const char *>(data()), (std::streamsize)(size() * sizeof(T)));
    }

    void store_interleaved_to_binary(std::ostream &out, dsize_t num_groups) const {
        if (num_groups == 0 || num_matrices_ % num_groups != 0)
            throw std::runtime_error{"Data array cannot be interleaved, as number of matrices is not divisible by group size"};
        binary::write_header<T>(out, matrix_size_, num_matrices_);
        dsize_t group_size = num_matrices_ / num_groups;
        for (dsize_t i = 0; i < num_matrices_; ++i)
            out.write(reinterpret_cast<const char *>(matrix(get_interleaved_index(i, group_size, num_groups))),
                      (std::streamsize)(matrix_size_.area() * sizeof(T)));
    }

    // text or binary by the extension of `path`
    void store(const std::filesystem::path &path) const {
        const bool bin = binary::path_is_binary(path);
        std::ofstream file(path, bin ? std::ios::binary : std::ios::out);
        if (!file) throw std::runtime_error("Could not open " + path.string());
        if (bin)
            store_to_binary(file);
        else
            store_to_csv(file);
    }
    void store_interleaved(const std::filesystem::path &path, dsize_t num_groups) const {
        const bool bin = binary::path_is_binary(path);
        std::ofstream file(path, bin ? std::ios::binary : std::ios::out);
        if (!file) throw std::runtime_error("Could not open " + path.string());
        if (bin)
            store_interleaved_to_binary(file, num_groups);
        else
            store_interleaved_to_csv(file, num_groups);
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
    std::ifstream file(path, std::ios::binary);
    if (!file) throw std::runtime_error("Could not open " + path.string());
    return data_array<T, ALLOC>::load_from_csv(file);
}

template <typename T, typename ALLOC = std::allocator<T>>
data_array<T, ALLOC> load_interleaved_matrix_array_from_csv(const std::filesystem::path &path, dsize_t group_size) {
    std::ifstream file(path, std::ios::binary);
    if (!file) throw std::runtime_error("Could not open " + path.string());
    return data_array<T, ALLOC>::load_interleaved_from_csv(file, group_size);
}

} // namespace cross
