// Cache of compiled GPU plans keyed by graph signature; the role of Axiom's
// GraphCache (include/axiom/graph/graph_cache.hpp:19-35) and of the Metal
// backend's g_gpu_graph_cache (src/backends/metal/mpsgraph_graph_compiler.mm:
// 696-698, 128 entries, cleared whole when full).
#pragma once

#include <cstddef>

namespace axiom::graph {

class GraphCache {
  public:
    static GraphCache &instance();
    void clear();
    size_t size() const;
    size_t hits() const;
    size_t misses() const;
    static constexpr size_t max_entries = 128;
};

} // namespace axiom::graph
