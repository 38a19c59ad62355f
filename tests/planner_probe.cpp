// The planner compiled on its own with a host compiler (no HIP, no device): prints the plan of every shape given
// on the command line as "n_samples l_max mode is_f64 normalized" quintuples, one line each, as the library's
// sphx_describe_plan words it for an MI355X (160 KB of LDS per workgroup, 256 CUs).
#include <cstdio>
#include <cstdlib>

#include "../sphericart_amd/csrc/sphx_plan.hpp"

int main(int argc, char** argv) {
    for (int i = 1; i + 4 < argc; i += 5) {
        const size_t n = static_cast<size_t>(std::atoll(argv[i]));
        const int l_max = std::atoi(argv[i + 1]), mode = std::atoi(argv[i + 2]);
        const bool is_f64 = std::atoi(argv[i + 3]) != 0, normalized = std::atoi(argv[i + 4]) != 0;
        sphx::Plan plan;
        (void)sphx::refresh_switches();
        const int status = sphx::make_plan(n, l_max, mode, is_f64 ? 8 : 4, 160 * 1024, 256, &plan, true, normalized);
        if (status != 0) {
            std::printf("status %d: %s\n", status, sphx::t_error.c_str());
        } else {
            std::printf("%s\n", sphx::describe(plan, l_max, mode, is_f64, normalized).c_str());
        }
    }
    return 0;
}
