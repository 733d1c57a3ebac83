// GPU execution of fused steps that a CPU-side plan hands over
// (include/axiom/graph/gpu_fusion.hpp:14-22; Metal implementation
// src/backends/metal/mpsgraph_fused.mm:409-567, 573-772).  Both rebuild the step as a lazy
// GPU graph and materialise it, so the step runs as one fused launch of libaxhip.
// Return false when the chain holds an op without a GPU kernel: the caller then runs it op by op.
#pragma once

#include <vector>

#include "axiom/graph/compiled_graph.hpp"
#include "axiom/tensor.hpp"

namespace axiom::graph {

bool execute_gpu_fused_chain(const StepBase &step, const std::vector<ops::OpType> &op_chain, std::vector<Tensor> &buffers);
bool execute_gpu_fused_reduction(const FusedReductionStep &step, std::vector<Tensor> &buffers);

} // namespace axiom::graph
