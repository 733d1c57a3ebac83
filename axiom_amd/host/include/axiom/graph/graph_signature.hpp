// Structural signature of a lazy graph: FNV-1a over node count and, per node in
// topological order, op, shape, dtype, device, constant flag (+ constant
// strides), input edges and parameters -- never the data
// (src/graph/graph_signature.cpp:96-211).
#pragma once

#include <cstdint>
#include <functional>

#include "axiom/graph/graph_node.hpp"

namespace axiom::graph {

struct GraphSignature {
    uint64_t hash = 0;
    bool operator==(const GraphSignature &o) const { return hash == o.hash; }
    bool operator!=(const GraphSignature &o) const { return hash != o.hash; }
};

struct GraphSignatureHash {
    size_t operator()(const GraphSignature &s) const { return static_cast<size_t>(s.hash); }
};

// nodes below `root` in dependency order (inputs first); stops at constants and materialised nodes
std::vector<const GraphNode *> topo_sort(const GraphNode *root);
GraphSignature compute_signature(const GraphNode *root);

} // namespace axiom::graph
