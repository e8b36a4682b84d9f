// `cross`: command-line front end with the reference's surface (main.cpp:465-683):
//   cross list
//   cross run [run options] <alg> <ref_path> <target_path>
//   cross validate [validate options] <template_data_path> <validate_data_path>...
//   cross input <alg_type> <rows> <columns> <left_matrices> <right_matrices>
// Exit codes: 0 ok, 1 bad command line / unknown algorithm / bad algorithm argument,
// 2 any other exception, 3 a failure inside a computation phase.
#include <algorithm>
#include <cctype>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <iostream>
#include <optional>
#include <string>
#include <vector>

#include "algorithms.hpp"
#include "fft_algorithms.hpp"

using namespace cross;
namespace fs = std::filesystem;

namespace {

struct cli_error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ---------------------------------------------------------------- option parsing
struct option_def {
    const char *long_name;
    char short_name;
    enum { flag, value, optional_value } kind;
};

struct parsed_options {
    std::map<std::string, std::string> values;
    std::vector<std::string> positional;
    bool has(const std::string &k) const { return values.count(k) != 0; }
    std::string get(const std::string &k, const std::string &def) const {
        auto it = values.find(k);
        return it == values.end() ? def : it->second;
    }
};

// Long options as "--name value" or "--name=value", short options as "-x value" or "-xvalue",
// switches without a value, and options with an optional value (--validate [path]) that take
// the next token only if it does not look like an option (what boost::program_options does
// with implicit_value, which is why the reference's driver never puts --validate last).
parsed_options parse_options(const std::vector<std::string> &args, const std::vector<option_def> &defs) {
    parsed_options out;
    auto find_long = [&](const std::string &n) -> const option_def * {
        for (auto &d : defs)
            if (n == d.long_name) return &d;
        return nullptr;
    };
    auto find_short = [&](char c) -> const option_def * {
        for (auto &d : defs)
            if (d.short_name && c == d.short_name) return &d;
        return nullptr;
    };
    for (std::size_t i = 0; i < args.size(); ++i) {
        const std::string &a = args[i];
        const option_def *d = nullptr;
        std::optional<std::string> attached;
        if (a.size() > 2 && a[0] == '-' && a[1] == '-') {
            auto eq = a.find('=');
            std::string name = a.substr(2, eq == std::string::npos ? std::string::npos : eq - 2);
            d = find_long(name);
            if (!d) throw cli_error("unrecognised option '" + a + "'");
            if (eq != std::string::npos) attached = a.substr(eq + 1);
        } else if (a.size() >= 2 && a[0] == '-' && !std::isdigit(static_cast<unsigned char>(a[1])) && a[1] != '.') {
            d = find_short(a[1]);
            if (!d) throw cli_error("unrecognised option '" + a + "'");
            if (a.size() > 2) attached = a.substr(2);
        } else {
            out.positional.push_back(a);
            continue;
        }
        if (d->kind == option_def::flag) {
            if (attached) throw cli_error(std::string("option '--") + d->long_name + "' does not take any arguments");
            out.values[d->long_name] = "1";
        } else if (d->kind == option_def::value) {
            if (attached) {
                out.values[d->long_name] = *attached;
            } else {
                if (i + 1 >= args.size()) throw cli_error(std::string("the required argument for option '--") + d->long_name + "' is missing");
                out.values[d->long_name] = args[++i];
            }
        } else {
            if (attached)
                out.values[d->long_name] = *attached;
            else if (i + 1 < args.size() && (args[i + 1].empty() || args[i + 1][0] != '-'))
                out.values[d->long_name] = args[++i];
            else
                out.values[d->long_name] = "";
        }
    }
    return out;
}

const std::vector<option_def> run_option_defs{
    {"data_type", 'd', option_def::value},      {"out", 'o', option_def::value},         {"times", 't', option_def::value},
    {"validate", 'v', option_def::optional_value}, {"normalize", 'n', option_def::flag}, {"append", 'a', option_def::flag},
    {"no_progress", 'p', option_def::flag},     {"benchmark_type", 'b', option_def::value}, {"outer_loops", 'l', option_def::value},
    {"min_time", 'm', option_def::value},       {"args_path", 0, option_def::value},     {"help", 'h', option_def::flag}};
const std::vector<option_def> validate_option_defs{
    {"normalize", 'n', option_def::flag}, {"csv", 'c', option_def::flag}, {"print_header", 'p', option_def::flag}, {"help", 'h', option_def::flag}};
const std::vector<option_def> no_option_defs{{"help", 'h', option_def::flag}};

void print_help(std::ostream &out, const std::string &name) {
    out << "Usage: " << name << " [global options] command [command options]\n";
    out << "Commands: \n";
    out << "\t" << name << " [global options] list\n";
    out << "\t" << name << " [global options] run [run options] <alg> <ref_path> <target_path>\n";
    out << "\t" << name << " [global options] validate [validate options] <validate_data_path> <template_data_path>\n";
    out << "\t" << name << " [global options] input [input options] <alg_type> <rows> <columns> <left_matrices> <right_matrices>\n";
    out << "\t" << name << " [global options] convert <in_path> <out_path>   (text <-> binary matrix file; \".bin\" selects binary)\n";
    out << "Global options:\n  -h [ --help ]                         display this help and exit\n";
    out << "Validate options:\n"
           "  -n [ --normalize ]                    Normalize the data to be validated as they are denormalized fft output\n"
           "  -c [ --csv ]                          CSV output\n"
           "  -p [ --print_header ]                 Print header\n";
    out << "Run options:\n"
           "  -d [ --data_type ] arg (=single)      Data type to use for computation (single, double)\n"
           "  -o [ --out ] arg                      Path of the output file to be created\n"
           "  -t [ --times ] arg (=measurements.csv) File to store the measured times in\n"
           "  -v [ --validate ] [=arg(=)]           If validation of the results should be done and optionally path to a file "
           "containing the valid results\n"
           "  -n [ --normalize ]                    If algorithm is fft, normalize the results\n"
           "  -a [ --append ]                       Append time measurements without the header if the times file already exists\n"
           "  -p [ --no_progress ]                  Do not print human readable progress, messages to stdout are formated for "
           "machine processing\n"
           "  -b [ --benchmark_type ] arg (=None)   Which part should be measured: Compute, CommonSteps, Algorithm\n"
           "  -l [ --outer_loops ] arg (=1)         How many measurements of the computation loop should be done with the loaded data\n"
           "  -m [ --min_time ] arg (=1)            The minimum time to consider measurement statistically relevant, in seconds\n"
           "  --args_path arg                       Path to the JSON file containing arguments for the algorithm\n";
}

bool iequals(const std::string &a, const char *b) {
    if (a.size() != std::strlen(b)) return false;
    for (std::size_t i = 0; i < a.size(); ++i)
        if (std::tolower(static_cast<unsigned char>(a[i])) != std::tolower(static_cast<unsigned char>(b[i]))) return false;
    return true;
}

// run_args.cpp:17-32
BenchmarkType parse_benchmark_type(const std::string &token) {
    if (iequals(token, "Compute")) return BenchmarkType::Compute;
    if (iequals(token, "CommonSteps")) return BenchmarkType::CommonSteps;
    if (iequals(token, "Algorithm")) return BenchmarkType::Algorithm;
    if (iequals(token, "None")) return BenchmarkType::None;
    return BenchmarkType::Unknown;
}

std::string join(const std::vector<std::string> &v) {
    std::string s;
    for (auto &e : v) s += (s.empty() ? "" : ", ") + e;
    return s;
}

// ---------------------------------------------------------------- logging (simple_logger.hpp:16-45)
class simple_logger {
public:
    simple_logger(bool print_progress, bool append_result_stats) : print_progress_(print_progress), append_result_stats_(append_result_stats) {}
    void log(const std::string &message) const {
        if (print_progress_) std::cout << message << std::endl;
    }
    void result_stats(const validation_results &results, std::optional<bool> print_header_override = std::nullopt) const {
        if (print_progress_) {
            std::cout << results;
        } else {
            if ((print_header_override.has_value() && *print_header_override) || (!print_header_override.has_value() && !append_result_stats_))
                std::cout << results.csv_header() << "\n";
            std::cout << results.csv_data() << "\n";
        }
    }

private:
    bool print_progress_, append_result_stats_;
};

struct run_args {
    BenchmarkType benchmark_type = BenchmarkType::None;
    std::string data_type = "single";
    std::string alg_name;
    std::optional<fs::path> alg_args_path;
    fs::path ref_path, target_path;
    std::optional<fs::path> out_path;
    fs::path measurements_path = "measurements.csv";
    std::optional<std::string> validate; // nullopt: no validation; "": compute valid results; else path
    std::size_t outer_loops = 1;
    bool normalize = false, append_measurements = false, print_progress = true;
    std::chrono::nanoseconds min_time{1000000000};

    // run_args.cpp:142-150
    std::optional<fs::path> get_loop_out_path(std::size_t loop) const {
        if (!out_path) return out_path;
        fs::path p = *out_path;
        return p.replace_filename(out_path->stem().string() + "_" + std::to_string(loop) + out_path->extension().string());
    }
};

// ---------------------------------------------------------------- measurements CSV (main.cpp:81-121, csv.hpp:35-47)
void output_measurements(const fs::path &path, const std::vector<std::string> &labels, const std::vector<measurement_result> &measurements,
                         const properties &props, bool append) {
    std::ofstream file;
    if (append) {
        file.open(path, std::ios_base::app);
    } else {
        file.open(path);
        const char *sep = "";
        for (auto &l : labels) {
            file << sep << l << "," << l << "_iterations";
            sep = ",";
        }
        if (!props.empty()) {
            if (!labels.empty()) file << ",";
            sep = "";
            for (auto &p : props) {
                file << sep << p.first;
                sep = ",";
            }
        }
        file << "\n";
    }
    const char *sep = "";
    for (auto &m : measurements) {
        file << sep << std::chrono::duration_cast<std::chrono::nanoseconds>(m.get_iteration_time()).count() << "," << m.get_iterations();
        sep = ",";
    }
    if (!props.empty()) {
        if (!measurements.empty()) file << ",";
        sep = "";
        for (auto &p : props) {
            file << sep << p.second;
            sep = ",";
        }
    }
    file << "\n";
}

// main.cpp:123-174
int run_computation_steps(algorithm &alg, const simple_logger &logger) {
    struct step {
        const char *message;
        const char *name;
        void (algorithm::*fn)();
    };
    const step steps[] = {{"Allocating", "allocation", &algorithm::prepare},
                          {"Transfering data", "data transfer", &algorithm::transfer},
                          {"Running test alg", "computation", &algorithm::run},
                          {"Copying output data to host", "finalization", &algorithm::finalize},
                          {"Free resources", "free", &algorithm::free}};
    for (auto &s : steps) {
        try {
            logger.log(s.message);
            (alg.*(s.fn))();
        } catch (std::exception &e) {
            std::cerr << "Exception occured durign " << s.name << " step: " << e.what() << "\nLast kernel launch arguments:\n"
                      << last_kernel_launch_args_string() << std::endl;
            return 3;
        }
    }
    return 0;
}

// main.cpp:230-326
int run_measurement(const run_args &ra) {
    const bool do_compute_measurement = ra.benchmark_type == BenchmarkType::Compute;
    simple_logger logger{ra.print_progress && !do_compute_measurement, ra.append_measurements};
    std::vector<std::string> compute_labels{"Computation"};
    stopwatch sw{compute_labels.size(), ra.min_time};

    json_args alg_args;
    if (ra.alg_args_path) {
        std::ifstream args_file{*ra.alg_args_path};
        if (!args_file) throw std::runtime_error("Could not open " + ra.alg_args_path->string());
        alg_args = json_args::parse(args_file);
    }
    auto alg = make_algorithm(ra.alg_name, ra.data_type, alg_args, ra.benchmark_type, ra.min_time);
    alg->set_normalize(ra.normalize); // main.cpp:176-187

    try {
        logger.log("Loading inputs");
        alg->load(ra.ref_path, ra.target_path);
    } catch (std::exception &e) {
        std::cerr << "Exception occured durign data loading step: " << e.what() << std::endl;
        return 3;
    }

    for (std::size_t loop = 0; loop < ra.outer_loops; ++loop) {
        int ret = 0;
        sw.cpu_adaptive_measure(0, do_compute_measurement, alg->uses_device(), [&] {
            if (ret == 0) ret = run_computation_steps(*alg, logger);
        });
        if (ret != 0) return ret;
        if (alg->uses_device()) {
            if (xcorr_device_sync() != XCORR_OK) {
                std::cerr << "Exception somewhere in HIP code: " << xcorr_last_error() << "\nLast kernel launch arguments:\n"
                          << last_kernel_launch_args_string() << std::endl;
                return 3;
            }
        }
        if (ra.benchmark_type != BenchmarkType::None) {
            if (!do_compute_measurement) {
                logger.log("Collect measurements");
                alg->collect_measurements();
            }
            output_measurements(ra.measurements_path, do_compute_measurement ? compute_labels : alg->measurement_labels(),
                                do_compute_measurement ? sw.results() : alg->measurements(), alg->additional_properties(),
                                ra.append_measurements || loop > 0);
            if (!do_compute_measurement) {
                logger.log("Reset measurement");
                alg->reset_measurements();
            }
        }
        auto out_path = ra.outer_loops > 1 ? ra.get_loop_out_path(loop) : ra.out_path;
        if (out_path) {
            logger.log("Storing results");
            alg->store_results(*out_path);
        }
        const bool print_header = !ra.append_measurements && loop == 0;
        if (!ra.validate) {
            logger.log("No validation");
        } else if (!ra.validate->empty()) {
            logger.log("Validating results against " + *ra.validate);
            logger.result_stats(alg->validate(fs::path(*ra.validate)), print_header);
        } else {
            logger.log("Computing valid results and validating");
            logger.result_stats(alg->validate(std::nullopt), print_header);
        }
    }
    return 0;
}

int cmd_run(const std::vector<std::string> &args, const std::string &prog) {
    parsed_options o = parse_options(args, run_option_defs);
    if (o.positional.size() < 3) {
        static const char *names[] = {"alg", "ref_path", "target_path"};
        throw cli_error(std::string("the option '--") + names[o.positional.size()] + "' is required but missing");
    }
    if (o.positional.size() > 3) throw cli_error("too many positional options have been specified on the command line");
    run_args ra;
    ra.alg_name = o.positional[0];
    ra.ref_path = o.positional[1];
    ra.target_path = o.positional[2];
    ra.benchmark_type = parse_benchmark_type(o.get("benchmark_type", "None"));
    ra.data_type = o.get("data_type", "single");
    if (o.has("args_path")) ra.alg_args_path = fs::path(o.get("args_path", ""));
    if (!o.get("out", "").empty()) ra.out_path = fs::path(o.get("out", ""));
    ra.measurements_path = o.get("times", "measurements.csv");
    if (o.has("validate")) ra.validate = o.get("validate", "");
    try {
        ra.outer_loops = static_cast<std::size_t>(std::stoull(o.get("outer_loops", "1")));
        ra.min_time = std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::duration<double>(std::stod(o.get("min_time", "1"))));
    } catch (std::exception &) {
        throw cli_error("the argument for option '--outer_loops' or '--min_time' is invalid");
    }
    ra.normalize = o.has("normalize");
    ra.append_measurements = o.has("append");
    ra.print_progress = !o.has("no_progress");

    if (!is_algorithm(ra.alg_name)) { // run_args.cpp:108-111
        std::cerr << "Unknown algorithm \"" << ra.alg_name << "\", expected one of " << join(algorithm_names()) << std::endl;
        print_help(std::cerr, prog);
        return 1;
    }
    if (ra.benchmark_type == BenchmarkType::Unknown) {
        std::cerr << "Unknown benchmark type" << std::endl;
        print_help(std::cerr, prog);
        return 1;
    }
    if (ra.data_type != "single" && ra.data_type != "double") { // main.cpp:431-438 (single only there)
        std::cerr << "Unknown data type " << ra.data_type << "\n";
        print_help(std::cerr, prog);
        return 1;
    }
    return run_measurement(ra);
}

// main.cpp:56-79
int cmd_validate(const std::vector<std::string> &args) {
    parsed_options o = parse_options(args, validate_option_defs);
    if (o.positional.empty()) throw cli_error("the option '--template_data_path' is required but missing");
    if (o.positional.size() < 2) throw cli_error("the option '--validate_data_path' is required but missing");
    const bool normalize = o.has("normalize");
    const bool csv = o.has("csv"), print_header = o.has("print_header");
    simple_logger logger{!csv, true};
    auto valid = load_matrix_array_from_csv<double>(o.positional[0]);
    for (std::size_t i = 1; i < o.positional.size(); ++i) {
        logger.log("Validating " + o.positional[i]);
        auto target = load_matrix_array_from_csv<double>(o.positional[i]);
        if (normalize) target = normalize_fft_results(target); // main.cpp:74-76
        logger.result_stats(validate_result(target, valid), i == 1 && print_header);
    }
    return 0;
}

// Not in the reference: rewrites a matrix file in the other format (the extension of the output
// path decides), so large inputs are parsed from text only once.
int cmd_convert(const std::vector<std::string> &args) {
    parsed_options o = parse_options(args, no_option_defs);
    if (o.positional.size() != 2) throw cli_error("convert expects <in_path> <out_path>");
    load_matrix_array_from_csv<double>(o.positional[0]).store(o.positional[1]);
    return 0;
}

// main.cpp:328-359
int cmd_input(const std::vector<std::string> &args, const std::string &prog) {
    parsed_options o = parse_options(args, no_option_defs);
    static const char *names[] = {"alg_type", "rows", "columns", "left_matrices", "right_matrices"};
    if (o.positional.size() < 5) throw cli_error(std::string("the option '--") + names[o.positional.size()] + "' is required but missing");
    if (o.positional.size() > 5) throw cli_error("too many positional options have been specified on the command line");
    dsize_t v[4];
    for (int i = 0; i < 4; ++i) {
        try {
            std::size_t pos = 0;
            long long x = std::stoll(o.positional[i + 1], &pos);
            if (pos != o.positional[i + 1].size() || x < 0) throw std::invalid_argument("");
            v[i] = static_cast<dsize_t>(x);
        } catch (std::exception &) {
            throw cli_error(std::string("the argument ('") + o.positional[i + 1] + "') for option '--" + names[i + 1] + "' is invalid");
        }
    }
    auto mode = parse_mode(o.positional[0]);
    if (!mode) {
        std::cerr << "Unknown algorithm type \"" << o.positional[0] << "\", expected one of n_to_m, n_to_mn, one_to_many, one_to_one" << std::endl;
        print_help(std::cerr, prog);
        return 1;
    }
    std::cout << (validate_input_size(*mode, v[0], v[1], v[2], v[3]) ? "Valid\n" : "Invalid\n");
    return 0;
}

} // namespace

int main(int argc, char **argv) {
    const std::string prog = argc > 0 ? argv[0] : "cross";
    try {
        std::vector<std::string> args(argv + 1, argv + argc);
        // global options come before the command
        std::size_t i = 0;
        bool help = false;
        for (; i < args.size() && !args[i].empty() && args[i][0] == '-'; ++i) {
            if (args[i] == "-h" || args[i] == "--help")
                help = true;
            else
                throw cli_error("unrecognised option '" + args[i] + "'");
        }
        if (help || i >= args.size()) {
            print_help(std::cout, prog);
            return 0;
        }
        const std::string cmd = args[i];
        std::vector<std::string> sub(args.begin() + i + 1, args.end());
        if (std::find(sub.begin(), sub.end(), "--help") != sub.end() || std::find(sub.begin(), sub.end(), "-h") != sub.end()) {
            print_help(std::cout, prog);
            return 0;
        }
        if (cmd == "run") {
            int ret = cmd_run(sub, prog);
            return ret;
        } else if (cmd == "validate") {
            return cmd_validate(sub);
        } else if (cmd == "list") {
            for (auto &name : algorithm_names()) std::cout << name << "\n";
            return 0;
        } else if (cmd == "input") {
            return cmd_input(sub, prog);
        } else if (cmd == "convert") {
            return cmd_convert(sub);
        }
        std::cerr << "Unknown command " << cmd << "\n";
        print_help(std::cerr, prog);
        return 1;
    } catch (cli_error &e) {
        std::cerr << "Invalid commandline options: " << e.what() << std::endl;
        return 1;
    } catch (argument_error &e) {
        std::cerr << "Invalid algorithm argument value: " << e.what() << std::endl;
        return 1;
    } catch (std::exception &e) {
        std::cerr << "Exception occured: " << e.what() << std::endl;
        return 2;
    }
}
