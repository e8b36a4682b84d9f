// Prints get_next_iteration_count (host/stopwatch.hpp, restating the reference's stopwatch.hpp:57-71) for the
// (min_time ns, total ns, iterations) triples given on the command line, one result per line.
#include <cstdio>
#include <cstdlib>

#include "stopwatch.hpp"

int main(int argc, char **argv) {
    for (int i = 1; i + 2 < argc; i += 3) {
        const long long min_ns = std::atoll(argv[i]), total_ns = std::atoll(argv[i + 1]);
        const std::size_t iterations = (std::size_t)std::atoll(argv[i + 2]);
        cross::measurement_result res(std::chrono::duration_cast<cross::sw_clock::duration>(std::chrono::nanoseconds(total_ns)), iterations);
        std::printf("%zu\n", cross::get_next_iteration_count(std::chrono::nanoseconds(min_ns), res));
    }
    return 0;
}
