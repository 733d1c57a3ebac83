// Step descriptions of a CPU-planned graph that the GPU fusion hooks receive
// (include/axiom/graph/compiled_graph.hpp:41-70; the fields those hooks read).
#pragma once

#include <vector>

#include "axiom/graph/graph_node.hpp"

namespace axiom::graph {

struct StepBase {
    int output_slot = -1;
    size_t total_elements = 0;
    Shape output_shape;
    DType output_dtype{};
    Device device = Device::CPU;
    // per op of the chain: the buffer slots of its inputs; -1 = the previous op's result
    std::vector<std::vector<int>> input_slot_indices;
};

struct FusedGenericStep : StepBase {
    std::vector<ops::OpType> op_chain;
};

struct FusedReductionStep : StepBase {
    ops::OpType reduction_op{};
    DType chain_dtype{};
    OpParams params; // ReductionParams
    std::vector<ops::OpType> op_chain;
};

} // namespace axiom::graph
