// Umbrella header of the gfx950 host layer.
#pragma once

#include "axiom/backends/hip/hip_operations.hpp"
#include "axiom/dtype.hpp"
#include "axiom/error.hpp"
#include "axiom/graph/compiled_graph.hpp"
#include "axiom/graph/gpu_fusion.hpp"
#include "axiom/graph/graph_cache.hpp"
#include "axiom/graph/graph_node.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/graph/graph_signature.hpp"
#include "axiom/nn.hpp"
#include "axiom/operations.hpp"
#include "axiom/random.hpp"
#include "axiom/shape.hpp"
#include "axiom/storage.hpp"
#include "axiom/system.hpp"
#include "axiom/tensor.hpp"
