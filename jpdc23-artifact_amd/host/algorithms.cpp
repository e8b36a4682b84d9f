// Algorithm registry (the reference's main.cpp:361-411) and the generic GPU algorithm.
#include "algorithms.hpp"
#include "fft_algorithms.hpp"

#include <algorithm>

namespace cross {

namespace {

using P = xcorr_params;
using A = arg_spec;
constexpr auto U = arg_spec::type::uint;
constexpr auto B = arg_spec::type::boolean;
constexpr auto D = arg_spec::type::distribution;

// distribution names (row_distribution.cpp:8-12); the integer is the JSON default's index here
constexpr long long DIST_RECTANGLE = XCORR_DIST_RECTANGLE, DIST_TRIANGLE = XCORR_DIST_TRIANGLE;

A warps() { return {"warps_per_thread_block", U, 8, &P::warps_per_thread_block}; }
A streams() { return {"num_cuda_streams", U, 8, nullptr}; }

std::vector<A> shared_mem_args(long long shifts_default, bool with_right_mats, bool with_streams) {
    std::vector<A> v{{"shifts_per_thread_block", U, shifts_default, &P::shifts_per_thread_block},
                     {"shared_mem_row_size", U, 32, &P::shared_mem_row_size},
                     {"shared_mem_rows", U, -1, &P::shared_mem_rows}, // default: shifts_per_thread_block
                     {"strided_load", B, 1, &P::strided_load},
                     {"column_group_per_block", B, 0, &P::column_group_per_block}};
    if (with_right_mats) v.push_back({"right_matrices_per_block", U, 8, &P::right_matrices_per_block});
    if (with_streams) v.push_back(streams());
    return v;
}

std::vector<algorithm_def> build_defs() {
    std::vector<algorithm_def> d;
    auto add = [&](const char *name, Mode mode, Family family, std::vector<A> args) -> algorithm_def & {
        algorithm_def a;
        a.name = name;
        a.mode = mode;
        a.family = family;
        a.args = std::move(args);
        d.push_back(a);
        return d.back();
    };
    // overlap-wise (one_to_one.hpp:145, one_to_many.hpp:142, n_to_mn.hpp:189, n_to_m.hpp:146)
    add("nai_orig_one_to_one", Mode::one_to_one, Family::overlap_wise, {});
    add("nai_orig_one_to_many", Mode::one_to_many, Family::overlap_wise, {});
    add("nai_orig_n_to_mn", Mode::n_to_mn, Family::overlap_wise, {});
    // (one launch over all pairs unless the arguments file holds num_cuda_streams; then one launch per left matrix on that
    // many streams like the reference, n_to_m.hpp:198-212)
    add("nai_orig_n_to_m", Mode::n_to_m, Family::overlap_wise, {streams()}).per_left_streams_if_asked = true;
    // sliding-window base and split-row (one_to_one.hpp:180, :224)
    add("nai_shuffle_one_to_one", Mode::one_to_one, Family::shuffle, {warps()});
    add("nai_shuffle_work_distribution_one_to_one", Mode::one_to_one, Family::split_row,
        {warps(), {"rows_per_thread", U, 10, &P::rows_per_thread}, {"distribution_type", D, DIST_RECTANGLE, &P::distribution_type}})
        .zero_output = true;
    // multi-matrix-right (one_to_one.hpp:293,:339, one_to_many.hpp:179,:228, n_to_mn.hpp:228, n_to_m.hpp:216)
    add("nai_shuffle_multimat_right_one_to_one", Mode::one_to_one, Family::multimat_right, {warps()}).fixed_one_right_per_thread = true;
    add("nai_shuffle_multimat_right_one_to_many", Mode::one_to_many, Family::multimat_right,
        {warps(), {"right_matrices_per_thread", U, 2, &P::right_matrices_per_thread}});
    {
        auto &a = add("nai_shuffle_multimat_right_work_distribution_one_to_one", Mode::one_to_one, Family::multimat_right,
                      {warps(), {"rows_per_thread", U, 10, &P::rows_per_thread}, {"distribution_type", D, DIST_RECTANGLE, &P::distribution_type}});
        a.zero_output = true;
        a.fixed_one_right_per_thread = true;
    }
    std::vector<A> mmr_wd{warps(),
                          {"right_matrices_per_thread", U, 2, &P::right_matrices_per_thread},
                          {"rows_per_thread", U, 10, &P::rows_per_thread},
                          {"distribution_type", D, DIST_RECTANGLE, &P::distribution_type}};
    add("nai_shuffle_multimat_right_work_distribution_one_to_many", Mode::one_to_many, Family::multimat_right, mmr_wd).zero_output = true;
    std::vector<A> mmr_wd_streams = mmr_wd;
    mmr_wd_streams.push_back(streams());
    {
        auto &a = add("nai_shuffle_multimat_right_work_distribution_n_to_mn", Mode::n_to_mn, Family::multimat_right, mmr_wd_streams);
        // one launch over all left matrices unless the arguments file holds num_cuda_streams (then one launch per left
        // matrix on that many streams like the reference, n_to_mn.hpp:286-300)
        a.zero_output = a.per_left_streams_if_asked = a.deinterleave = true;
    }
    {
        auto &a = add("nai_shuffle_multimat_right_work_distribution_n_to_m", Mode::n_to_m, Family::multimat_right, mmr_wd_streams);
        a.zero_output = a.per_left_streams = true;
    }
    // multi-matrix-both (n_to_m.hpp:316, :393; the local_mem twin only differs in how nvcc spills)
    std::vector<A> mmb{warps(),
                       {"left_matrices_per_thread", U, 2, &P::left_matrices_per_thread},
                       {"right_matrices_per_thread", U, 2, &P::right_matrices_per_thread},
                       {"rows_per_thread", U, 10, &P::rows_per_thread},
                       {"distribution_type", D, DIST_TRIANGLE, &P::distribution_type}};
    add("nai_shuffle_multimat_both_work_distribution_n_to_m", Mode::n_to_m, Family::multimat_both, mmb).zero_output = true;
    add("nai_shuffle_multimat_both_work_distribution_local_mem_n_to_m", Mode::n_to_m, Family::multimat_both, mmb).zero_output = true;
    // grouped-overlap (one_to_one.hpp:734, :785)
    std::vector<A> go{warps(), {"shifts_per_thread", U, 4, &P::shifts_per_thread}, {"left_rows_per_iteration", U, 3, &P::left_rows_per_iteration}};
    add("nai_shuffle_multirow_both_one_to_one", Mode::one_to_one, Family::grouped_overlap, go);
    add("nai_shuffle_multirow_both_local_mem_one_to_one", Mode::one_to_one, Family::grouped_overlap, go);
    // multi-matrix-right x grouped-overlap (one_to_many.hpp:357, n_to_mn.hpp:462)
    std::vector<A> mrg{warps(),
                       {"shifts_per_thread_right_matrix", U, 4, &P::shifts_per_thread_right_matrix},
                       {"right_matrices_per_thread", U, 4, &P::right_matrices_per_thread},
                       {"left_rows_per_iteration", U, 4, &P::left_rows_per_iteration}};
    add("nai_shuffle_multirow_both_multimat_right_one_to_many", Mode::one_to_many, Family::multimat_right_grouped, mrg);
    {
        std::vector<A> v = mrg;
        v.push_back(streams());
        auto &a = add("nai_shuffle_multirow_both_multimat_right_n_to_mn", Mode::n_to_mn, Family::multimat_right_grouped, v);
        // one launch over all left matrices by default; when the arguments file holds num_cuda_streams, one launch per
        // left matrix on that many streams like the reference (n_to_mn.hpp:553-571)
        a.deinterleave = true;
        a.per_left_streams_if_asked = true;
    }
    // multi-matrix-both x grouped-overlap (n_to_m.hpp:470)
    add("nai_shuffle_multirow_both_multimat_both_n_to_m", Mode::n_to_m, Family::multimat_both_grouped,
        {warps(),
         {"shifts_per_thread_right_matrix", U, 2, &P::shifts_per_thread_right_matrix},
         {"left_matrices_per_thread", U, 2, &P::left_matrices_per_thread},
         {"right_matrices_per_thread", U, 2, &P::right_matrices_per_thread},
         {"left_rows_per_iteration", U, 2, &P::left_rows_per_iteration}});
    // unpublished variants, mapped onto the families above: "multirow_right" is grouped-overlap
    // with one left row per iteration (one_to_one.hpp:687,:837, one_to_many.hpp:307, n_to_mn.hpp:352)
    add("nai_shuffle_multirow_right_one_to_one", Mode::one_to_one, Family::grouped_overlap,
        {warps(), {"right_rows_per_thread", U, 4, &P::shifts_per_thread}});
    add("nai_shuffle_multirow_right_multimat_right_one_to_one", Mode::one_to_one, Family::multimat_right_grouped,
        {warps(), {"right_rows_per_thread", U, 4, &P::shifts_per_thread_right_matrix}})
        .fixed_one_right_per_thread = true;
    std::vector<A> mrr{warps(),
                       {"right_rows_per_thread", U, 4, &P::shifts_per_thread_right_matrix},
                       {"right_matrices_per_thread", U, 4, &P::right_matrices_per_thread}};
    add("nai_shuffle_multirow_right_multimat_right_one_to_many", Mode::one_to_many, Family::multimat_right_grouped, mrr);
    {
        std::vector<A> v = mrr;
        v.push_back(streams());
        auto &a = add("nai_shuffle_multirow_right_multimat_right_n_to_mn", Mode::n_to_mn, Family::multimat_right_grouped, v);
        a.deinterleave = true; // one launch unless num_cuda_streams is given, as above
        a.per_left_streams_if_asked = true;
    }
    // warp-per-overlap (one_to_one.hpp:410, :519, :452)
    add("nai_warp_per_shift_one_to_one", Mode::one_to_one, Family::warp_per_overlap,
        {{"shifts_per_thread_block", U, 8, &P::shifts_per_thread_block}});
    add("nai_warp_per_shift_simple_indexing_one_to_one", Mode::one_to_one, Family::warp_per_overlap,
        {{"shifts_per_thread_block", U, 8, &P::shifts_per_thread_block}})
        .wpo_variant = XCORR_WPO_SIMPLE_INDEXING;
    {
        auto &a = add("nai_warp_per_shift_work_distribution_one_to_one", Mode::one_to_one, Family::warp_per_overlap,
                      {{"shifts_per_thread_block", U, 8, &P::shifts_per_thread_block},
                       {"rows_per_warp", U, 3, &P::rows_per_thread},
                       {"distribution_type", D, DIST_RECTANGLE, &P::distribution_type}});
        a.wpo_variant = XCORR_WPO_WORK_DISTRIBUTION;
        a.zero_output = true;
    }
    // shared-memory warp-per-shift (one_to_one.hpp:561, one_to_many.hpp:411, n_to_mn.hpp:575,
    // n_to_m.hpp:529): the LDS-staged engine families stand in for it
    add("nai_warp_per_shift_shared_mem_one_to_one", Mode::one_to_one, Family::warp_per_overlap_lds, shared_mem_args(32, false, false))
        .shared_mem_rows_rule = true;
    add("nai_warp_per_shift_shared_mem_one_to_many", Mode::one_to_many, Family::warp_per_overlap_lds, shared_mem_args(16, true, false))
        .shared_mem_rows_rule = true;
    {
        auto &a = add("nai_warp_per_shift_shared_mem_n_to_mn", Mode::n_to_mn, Family::warp_per_overlap_lds, shared_mem_args(16, true, true));
        a.shared_mem_rows_rule = a.per_left_streams = a.deinterleave = true;
    }
    {
        auto &a = add("nai_warp_per_shift_shared_mem_n_to_m", Mode::n_to_m, Family::warp_per_overlap_lds, shared_mem_args(16, true, true));
        a.shared_mem_rows_rule = a.per_left_streams = true;
    }
    // block-per-shift (one_to_one.hpp:644)
    add("nai_block_per_shift_one_to_one", Mode::one_to_one, Family::block_per_overlap, {{"block_size", U, 128, &P::block_size}});
    return d;
}

template <typename T>
struct entry;
template <>
struct entry<float> {
    static constexpr auto overlap_wise = xcorr_overlap_wise_f32;
    static constexpr auto overlap_wise_all_pairs = xcorr_overlap_wise_all_pairs_f32;
    static constexpr auto warp_per_overlap = xcorr_warp_per_overlap_f32;
    static constexpr auto warp_per_overlap_lds = xcorr_warp_per_overlap_lds_f32;
    static constexpr auto block_per_overlap = xcorr_block_per_overlap_f32;
    static constexpr auto shuffle = xcorr_shuffle_f32;
    static constexpr auto split_row = xcorr_split_row_f32;
    static constexpr auto grouped_overlap = xcorr_grouped_overlap_f32;
    static constexpr auto multimat_right = xcorr_multimat_right_f32;
    static constexpr auto multimat_right_groups = xcorr_multimat_right_groups_f32;
    static constexpr auto multimat_right_grouped = xcorr_multimat_right_grouped_f32;
    static constexpr auto multimat_both = xcorr_multimat_both_f32;
    static constexpr auto multimat_both_grouped = xcorr_multimat_both_grouped_f32;
};
template <>
struct entry<double> {
    static constexpr auto overlap_wise = xcorr_overlap_wise_f64;
    static constexpr auto overlap_wise_all_pairs = xcorr_overlap_wise_all_pairs_f64;
    static constexpr auto warp_per_overlap = xcorr_warp_per_overlap_f64;
    static constexpr auto warp_per_overlap_lds = xcorr_warp_per_overlap_lds_f64;
    static constexpr auto block_per_overlap = xcorr_block_per_overlap_f64;
    static constexpr auto shuffle = xcorr_shuffle_f64;
    static constexpr auto split_row = xcorr_split_row_f64;
    static constexpr auto grouped_overlap = xcorr_grouped_overlap_f64;
    static constexpr auto multimat_right = xcorr_multimat_right_f64;
    static constexpr auto multimat_right_groups = xcorr_multimat_right_groups_f64;
    static constexpr auto multimat_right_grouped = xcorr_multimat_right_grouped_f64;
    static constexpr auto multimat_both = xcorr_multimat_both_f64;
    static constexpr auto multimat_both_grouped = xcorr_multimat_both_grouped_f64;
};

unsigned distribution_from_string(const std::string &s) {
    if (s == "none") return XCORR_DIST_NONE;
    if (s == "rectangle") return XCORR_DIST_RECTANGLE;
    if (s == "triangle") return XCORR_DIST_TRIANGLE;
    throw std::runtime_error("Unknown distribution " + s); // row_distribution.cpp:17-19
}
const char *distribution_to_string(unsigned d) {
    return d == XCORR_DIST_NONE ? "none" : d == XCORR_DIST_RECTANGLE ? "rectangle" : "triangle";
}

} // namespace

const std::vector<algorithm_def> &gpu_algorithm_defs() {
    static const std::vector<algorithm_def> defs = build_defs();
    return defs;
}

std::vector<std::string> algorithm_names() {
    std::vector<std::string> names{"cpu_one_to_one", "cpu_one_to_many", "cpu_n_to_mn", "cpu_n_to_m"};
    for (auto &d : gpu_algorithm_defs()) names.push_back(d.name);
    for (auto &d : fft_algorithm_defs()) names.push_back(d.name);
    std::sort(names.begin(), names.end());
    return names;
}

bool is_algorithm(const std::string &name) {
    auto names = algorithm_names();
    return std::find(names.begin(), names.end(), name) != names.end();
}

std::optional<Mode> parse_mode(const std::string &name) {
    for (Mode m : {Mode::one_to_one, Mode::one_to_many, Mode::n_to_mn, Mode::n_to_m})
        if (name == mode_name(m)) return m;
    return std::nullopt;
}

// ---------------------------------------------------------------- gpu_algorithm
namespace {
// keys whose value picks a compiled tile in the library: an exact request there, so only passed when the file holds them
bool selects_tile(const std::string &key) {
    return key == "shifts_per_thread" || key == "shifts_per_thread_right_matrix" || key == "right_rows_per_thread" ||
           key == "right_matrices_per_thread" || key == "left_matrices_per_thread";
}
} // namespace

template <typename T>
gpu_algorithm<T>::gpu_algorithm(const algorithm_def &def, const json_args &args, BenchmarkType bench, std::chrono::nanoseconds min_time)
    : algorithm(bench, 1, min_time), def_(def) {
    params_.warp_per_overlap_variant = def.wpo_variant;
    unsigned shifts_per_thread_block = 0, shared_mem_rows = 0;
    for (const arg_spec &a : def.args) {
        std::string shown;
        unsigned value = 0;
        if (a.t == arg_spec::type::distribution) {
            value = distribution_from_string(args.value(a.key, distribution_to_string((unsigned)a.def)));
            shown = distribution_to_string(value);
        } else if (a.t == arg_spec::type::boolean) {
            value = args.value(a.key, a.def != 0) ? 1u : 0u;
            shown = std::to_string(value);
        } else {
            long long def_value = a.def;
            if (std::string(a.key) == "shared_mem_rows") def_value = shifts_per_thread_block;
            value = args.value(a.key, static_cast<unsigned>(def_value));
            if (std::string(a.key) == "shifts_per_thread_block") shifts_per_thread_block = value;
            if (std::string(a.key) == "shared_mem_rows") {
                if (value == 0) value = shifts_per_thread_block;
                shared_mem_rows = value;
            }
            if (std::string(a.key) == "num_cuda_streams") num_streams_ = value;
            shown = std::to_string(value);
        }
        // (the split-row launchers of the sliding-window engine also take their chunk of rows from the library unless the file
        // names one: the reference's default of 10 rows leaves most of the GPU idle on small inputs and cuts large ones too short)
        const bool engine_split_row = def.family == Family::split_row || def.family == Family::multimat_right || def.family == Family::multimat_both;
        // (and the staging parameters of the LDS wavefront-per-overlap family, whose defaults in the library are the reference's:
        // with none of them named the library may keep few small matrices whole in LDS instead)
        const bool lds_staging = def.family == Family::warp_per_overlap_lds && a.t == arg_spec::type::uint && a.field != nullptr;
        const bool library_default = !args.contains(a.key) && (selects_tile(a.key) || (engine_split_row && std::string(a.key) == "rows_per_thread") ||
                                                               (def.family == Family::warp_per_overlap && std::string(a.key) == "rows_per_warp") || lds_staging);
        if (a.field) params_.*(a.field) = library_default ? 0u : value;
        if (a.report) props_.emplace_back(a.key, shown);
    }
    if (def.shared_mem_rows_rule && shared_mem_rows < shifts_per_thread_block) {
        // one_to_many.hpp:427-436
        throw argument_error("Invalid number of shared memory rows [" + std::to_string(shared_mem_rows) +
                                 "], must be greater than shifts per block [" + std::to_string(shifts_per_thread_block) + "]",
                             "shared_mem_rows");
    }
    // (the shifts-per-block and block-size limits are the launchers': they fail in the first launch, exit code 3)
    zero_output_ = def.zero_output || (def.family == Family::warp_per_overlap_lds && params_.column_group_per_block);
    if (def.fixed_one_right_per_thread) params_.right_matrices_per_thread = 1;
    if (def.per_left_streams_if_asked && args.contains("num_cuda_streams")) def_.per_left_streams = true;
    if (def_.per_left_streams && num_streams_ == 0) num_streams_ = 1;
    // the unpublished "multirow_right" kernels allow up to 8 rows, the combined engine tiles 4
    if (def.family == Family::multimat_right_grouped && params_.shifts_per_thread_right_matrix > 4 &&
        def.name.find("multirow_right") != std::string::npos)
        params_.shifts_per_thread_right_matrix = 4;
}

template <typename T>
void gpu_algorithm<T>::release() noexcept {
    for (auto &s : streams_)
        if (s) xcorr_stream_destroy(s);
    streams_.clear();
    if (d_results_) xcorr_free(d_results_);
    if (d_targets_) xcorr_free(d_targets_);
    if (d_refs_) xcorr_free(d_refs_);
    d_results_ = d_targets_ = d_refs_ = nullptr;
}

template <typename T>
gpu_algorithm<T>::~gpu_algorithm() {
    release(); // whatever a phase that threw left behind (free() has released everything after a normal run)
}

template <typename T>
void gpu_algorithm<T>::load_impl(const std::filesystem::path &ref, const std::filesystem::path &target) {
    refs_ = load_matrix_array_from_csv<T, pinned_allocator<T>>(ref);
    if (def_.deinterleave) {
        // n_to_mn.hpp:165-172: group the right matrices of each left matrix together
        targets_ = load_interleaved_matrix_array_from_csv<T, pinned_allocator<T>>(target, refs_.num_matrices());
    } else {
        targets_ = load_matrix_array_from_csv<T, pinned_allocator<T>>(target);
    }
    check_input_counts(def_.mode, refs_.num_matrices(), targets_.num_matrices());
    check_matrices_same_size(refs_, targets_);
}

template <typename T>
void gpu_algorithm<T>::prepare_impl() {
    results_ = host_array{result_matrix_size(refs_.matrix_size(), targets_.matrix_size()),
                          num_results(def_.mode, refs_.num_matrices(), targets_.num_matrices())};
    xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_refs_), refs_.size() * sizeof(T)));
    xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_targets_), targets_.size() * sizeof(T)));
    xcheck(xcorr_malloc(reinterpret_cast<void **>(&d_results_), results_.size() * sizeof(T)));
    if (def_.family == Family::overlap_wise && def_.mode == Mode::n_to_m && !def_.per_left_streams) {
        // One launch over all pairs wins while the launches per left matrix would be short (16x16, 8 x 8 matrices:
        // 106 -> 14 us); from about 4e8 multiply-adds per left matrix on, the reference's one launch per left matrix on
        // eight streams is 10-30 % faster (128x128, 32 x 32: 90 against 126 ms).
        const double area = (double)refs_.matrix_size().area();
        if (refs_.num_matrices() >= 4 && (double)targets_.num_matrices() * area * area >= 4e8) {
            def_.per_left_streams = true;
            if (num_streams_ == 0) num_streams_ = 8;
        }
    }
    if (def_.per_left_streams) {
        streams_.assign(num_streams_, nullptr);
        for (auto &s : streams_) xcheck(xcorr_stream_create(&s));
    }
}

template <typename T>
void gpu_algorithm<T>::transfer_impl() {
    xcheck(xcorr_memcpy_h2d(d_refs_, refs_.data(), refs_.size() * sizeof(T)));
    xcheck(xcorr_memcpy_h2d(d_targets_, targets_.data(), targets_.size() * sizeof(T)));
}

template <typename T>
void gpu_algorithm<T>::launch(const T *left, const T *right, T *out, dsize_t n_left, dsize_t n_right, void *stream) {
    const dsize_t cols = refs_.matrix_size().x, rows = refs_.matrix_size().y;
    using E = entry<T>;
    switch (def_.family) {
    case Family::overlap_wise:
        if (def_.mode == Mode::n_to_m && n_left > 1)
            xcheck(E::overlap_wise_all_pairs(left, right, out, cols, rows, n_left, n_right, stream));
        else
            xcheck(E::overlap_wise(left, right, out, cols, rows, n_left, n_right, stream));
        break;
    case Family::warp_per_overlap: xcheck(E::warp_per_overlap(left, right, out, cols, rows, &params_, stream)); break;
    case Family::warp_per_overlap_lds: xcheck(E::warp_per_overlap_lds(left, right, out, cols, rows, n_right, &params_, stream)); break;
    case Family::block_per_overlap: xcheck(E::block_per_overlap(left, right, out, cols, rows, &params_, stream)); break;
    case Family::shuffle: xcheck(E::shuffle(left, right, out, cols, rows, &params_, stream)); break;
    case Family::split_row: xcheck(E::split_row(left, right, out, cols, rows, &params_, stream)); break;
    case Family::grouped_overlap: xcheck(E::grouped_overlap(left, right, out, cols, rows, &params_, stream)); break;
    case Family::multimat_right:
        if (n_left > 1)
            xcheck(E::multimat_right_groups(left, right, out, cols, rows, n_left, n_right, &params_, stream));
        else
            xcheck(E::multimat_right(left, right, out, cols, rows, n_right, &params_, stream));
        break;
    case Family::multimat_right_grouped:
        xcheck(E::multimat_right_grouped(left, right, out, cols, rows, n_left, n_right, &params_, stream));
        break;
    case Family::multimat_both: xcheck(E::multimat_both(left, right, out, cols, rows, n_left, n_right, &params_, stream)); break;
    case Family::multimat_both_grouped:
        xcheck(E::multimat_both_grouped(left, right, out, cols, rows, n_left, n_right, &params_, stream));
        break;
    }
}

template <typename T>
void gpu_algorithm<T>::launch_all() {
    // (the clear is a small fill kernel: shorter than a memset command for the outputs of small instances, and it may be captured)
    if (clear_before_launch_) xcheck(xcorr_clear_async(d_results_, results_.size() * sizeof(T), nullptr));
    launch_kernels();
}

// The families whose contract is a zeroed output are asked first what they would run on this instance (a planning call:
// nothing is launched): a launch that adds nothing into the output - one work item per result tile, or a small instance
// whose pairs run whole in LDS - stores every element, and the clear kernel in front of it would only cost time.
template <typename T>
bool gpu_algorithm<T>::launches_add_into_output() {
    const bool plans = def_.family == Family::split_row || def_.family == Family::multimat_right || def_.family == Family::multimat_both ||
                       def_.family == Family::warp_per_overlap || def_.family == Family::warp_per_overlap_lds;
    if (!plans) return true;
    xcorr_plan_only(1);
    try {
        launch_kernels();
    } catch (...) {
        xcorr_plan_only(0);
        throw;
    }
    xcorr_plan_only(0);
    xcorr_launch_record rec; // (the launches of one run all have the same shape: the last record speaks for them)
    return xcorr_last_launch(&rec) != XCORR_OK || rec.uses_atomics != 0;
}

template <typename T>
void gpu_algorithm<T>::launch_kernels() {
    const dsize_t n = refs_.num_matrices(), total_right = targets_.num_matrices();
    const std::size_t in_area = refs_.matrix_size().area(), out_area = results_.matrix_size().area();
    if (def_.per_left_streams) {
        if (clear_before_launch_) xcheck(xcorr_device_sync()); // the clear runs on the default stream
        // one launch per left matrix, left r on stream r mod k (n_to_mn.hpp:553-571, n_to_m.hpp:198-212)
        const bool all_pairs = def_.mode == Mode::n_to_m;
        const dsize_t per_left = all_pairs ? total_right : total_right / n;
        for (dsize_t r = 0; r < n; ++r) {
            const T *right = all_pairs ? d_targets_ : d_targets_ + (std::size_t)r * per_left * in_area;
            T *out = d_results_ + (std::size_t)r * per_left * out_area;
            launch(d_refs_ + r * in_area, right, out, 1, per_left, streams_[r % streams_.size()]);
        }
        return;
    }
    switch (def_.mode) {
    case Mode::one_to_one: launch(d_refs_, d_targets_, d_results_, 1, 1, nullptr); break;
    case Mode::one_to_many: launch(d_refs_, d_targets_, d_results_, 1, total_right, nullptr); break;
    case Mode::n_to_mn:
        // overlap-wise: file order, (subregions_per_pic, batch_size) = (n, m) (n_to_mn.hpp:201-212)
        launch(d_refs_, d_targets_, d_results_, n, total_right / n, nullptr);
        break;
    case Mode::n_to_m: launch(d_refs_, d_targets_, d_results_, n, total_right, nullptr); break;
    }
}

template <typename T>
void gpu_algorithm<T>::run_impl() {
    clear_before_launch_ = zero_output_ && launches_add_into_output();
    if (def_.per_left_streams) {
        // several streams: wall clock around launch + device synchronisation (n_to_mn.hpp:500-505)
        sw_.cpu_adaptive_measure(0, measure_alg(), true, [&] { launch_all(); });
    } else {
        sw_.device_adaptive_measure(0, measure_alg(), [&] { launch_all(); });
    }
    report_effective_arguments();
}

// The measurement file reports what the launch used, not what was asked: the library maps the reference's integers onto
// its compiled tiles (xcorr_last_launch).
template <typename T>
void gpu_algorithm<T>::report_effective_arguments() {
    xcorr_launch_record rec;
    if (xcorr_last_launch(&rec) != XCORR_OK) return;
    for (auto &[key, value] : props_) {
        if (key == "shifts_per_thread" || key == "shifts_per_thread_right_matrix" || key == "right_rows_per_thread")
            value = std::to_string(rec.y_shifts_per_thread);
        else if (key == "right_matrices_per_thread")
            value = std::to_string(rec.right_matrices_per_thread * (rec.lanes_right ? rec.lanes_right : 1u));
        else if (key == "left_matrices_per_thread")
            value = std::to_string(rec.left_matrices_per_thread * (rec.lanes_left ? rec.lanes_left : 1u));
        else if (key == "rows_per_warp" && def_.family == Family::warp_per_overlap)
            value = std::to_string(rec.rows_per_worker);
        else if (key == "rows_per_thread" && (def_.family == Family::split_row || def_.family == Family::multimat_right || def_.family == Family::multimat_both))
            value = std::to_string(rec.rows_per_worker);
        else if (key == "distribution_type" && (def_.family == Family::split_row || def_.family == Family::multimat_right || def_.family == Family::multimat_both))
            value = distribution_to_string(rec.distribution_type); // (a matrix-core tile maps "rectangle" onto "triangle")
    }
}

template <typename T>
void gpu_algorithm<T>::finalize_impl() {
    xcheck(xcorr_memcpy_d2h(results_.data(), d_results_, results_.size() * sizeof(T)));
}

template <typename T>
void gpu_algorithm<T>::free_impl() {
    for (auto &s : streams_) {
        void *stream = s;
        s = nullptr;
        xcheck(xcorr_stream_destroy(stream));
    }
    streams_.clear();
    T *buffers[3] = {d_results_, d_targets_, d_refs_};
    d_results_ = d_targets_ = d_refs_ = nullptr;
    for (T *b : buffers) xcheck(xcorr_free(b));
}

template <typename T>
void gpu_algorithm<T>::store_results_impl(const std::filesystem::path &out) const {
    if (def_.deinterleave) // back to the file order of the inputs (n_to_mn.hpp:515-519)
        results_.store_interleaved(out, targets_.num_matrices() / refs_.num_matrices());
    else
        results_.store(out);
}

template <typename T>
validation_results gpu_algorithm<T>::validate(const std::optional<std::filesystem::path> &valid_path) const {
    if (valid_path) {
        if (def_.deinterleave) // n_to_mn.hpp:527-530
            return validate_result(results_, load_interleaved_matrix_array_from_csv<T>(*valid_path, refs_.num_matrices()));
        return validate_result(results_, load_matrix_array_from_csv<T>(*valid_path));
    }
    if (def_.deinterleave) {
        // n_to_mn.hpp:532-540: back to file order for the host computation, then group its result again
        dsize_t num_groups = targets_.num_matrices() / refs_.num_matrices();
        auto file_order_targets = targets_.template interleave<std::allocator<T>>(num_groups);
        return validate_result(results_, cpu_cross_corr(def_.mode, refs_, file_order_targets).interleave(refs_.num_matrices()));
    }
    return validate_result(results_, cpu_cross_corr(def_.mode, refs_, targets_));
}

template class gpu_algorithm<float>;
template class gpu_algorithm<double>;

std::unique_ptr<algorithm> make_algorithm(const std::string &name, const std::string &data_type, const json_args &args,
                                          BenchmarkType bench, std::chrono::nanoseconds min_time) {
    const bool is_double = data_type == "double";
    if (name.rfind("cpu_", 0) == 0) {
        auto mode = parse_mode(name.substr(4));
        if (!mode) throw std::runtime_error("Invalid algorithm specified \"" + name + "\"");
        if (is_double) return std::make_unique<cpu_algorithm<double>>(*mode, bench, min_time);
        return std::make_unique<cpu_algorithm<float>>(*mode, bench, min_time);
    }
    for (auto &d : gpu_algorithm_defs()) {
        if (d.name != name) continue;
        if (is_double) return std::make_unique<gpu_algorithm<double>>(d, args, bench, min_time);
        return std::make_unique<gpu_algorithm<float>>(d, args, bench, min_time);
    }
    for (auto &d : fft_algorithm_defs()) {
        if (d.name != name) continue;
        if (is_double) return std::make_unique<fft_algorithm<double>>(d, args, bench, min_time);
        return std::make_unique<fft_algorithm<float>>(d, args, bench, min_time);
    }
    throw std::runtime_error("Invalid algorithm specified \"" + name + "\"");
}

} // namespace cross
