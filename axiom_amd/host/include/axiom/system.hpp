// Availability probes (src/tensor/system.cpp:11-29).
#pragma once

namespace axiom::system {
bool is_gpu_available();
// false when AXIOM_SKIP_GPU_TESTS=1 or no device is present
bool should_run_gpu_tests();
} // namespace axiom::system
