#include <cstring>

#include "axiom/graph/graph_registry.hpp"
#include "test_framework.hpp"

int main(int argc, char **argv) {
    bool only_cpu = false, only_gpu = false, list = false;
    std::string filter;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--cpu")) only_cpu = true;
        else if (!std::strcmp(argv[i], "--gpu")) only_gpu = true;
        else if (!std::strcmp(argv[i], "--list")) list = true;
        else filter = argv[i];
    }
    axiom::graph::record_gpu_plan_kernels(true); // several cases assert which kernels a graph ran on
    int ran = 0, failed = 0, skipped = 0;
    for (const auto &c : axtest::registry()) {
        const std::string full = c.suite + "." + c.name;
        if (only_cpu && c.needs_gpu) continue;
        if (only_gpu && !c.needs_gpu) continue;
        if (!filter.empty() && full.find(filter) == std::string::npos) continue;
        if (list) {
            std::printf("%s%s\n", full.c_str(), c.needs_gpu ? " [gpu]" : "");
            continue;
        }
        std::printf("[ RUN      ] %s\n", full.c_str());
        std::fflush(stdout);
        const int before = axtest::soft_failures();
        bool skip = false;
        try {
            if (c.needs_gpu && !axiom::system::should_run_gpu_tests()) throw axtest::Skip("no GPU");
            c.fn();
        } catch (const axtest::Skip &) {
            skip = true;
        } catch (const axtest::Failure &) {
        } catch (const std::exception &e) {
            std::fprintf(stderr, "  unexpected exception: %s\n", e.what());
            ++axtest::soft_failures();
        }
        if (skip) {
            ++skipped;
            std::printf("[  SKIPPED ] %s\n", full.c_str());
        } else if (axtest::soft_failures() != before) {
            ++failed;
            ++ran;
            std::printf("[  FAILED  ] %s\n", full.c_str());
        } else {
            ++ran;
            std::printf("[       OK ] %s\n", full.c_str());
        }
        std::fflush(stdout);
    }
    if (!list) std::printf("%d ran, %d failed, %d skipped\n", ran, failed, skipped);
    return failed ? 1 : 0;
}
