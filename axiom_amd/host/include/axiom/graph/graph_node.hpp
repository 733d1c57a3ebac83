// Deferred-computation node of the lazy graph
// (include/axiom/graph/graph_node.hpp:25-138).
#pragma once

#include <atomic>
#include <memory>
#include <utility>
#include <variant>
#include <vector>

#include "axiom/dtype.hpp"
#include "axiom/operations.hpp"
#include "axiom/shape.hpp"
#include "axiom/storage.hpp"

namespace axiom::graph {

struct NoParams {};
struct ReductionParams {
    std::vector<int> axes;
    bool keep_dims = false;
};
struct MatMulParams {
    bool transpose_a = false;
    bool transpose_b = false;
};
struct ActivationParams {
    float alpha = 0.01f;
    int axis = -1;
};
struct ReshapeParams {
    Shape new_shape;
};
struct NormParams {
    int axis = -1;
    float eps = 1e-5f;
};
struct TransposeParams {
    std::vector<int> axes;
};

struct SliceParams { // per dimension; steps are positive
    std::vector<int64_t> starts, ends, steps;
};
struct PadParams {
    std::vector<std::pair<size_t, size_t>> pad_widths;
    double value = 0.0;
    int mode = 0; // AXHIP_PAD_*: constant, reflect, replicate, circular
};
struct MaskedFillParams {
    float value = 0.0f;
};
struct UnfoldParams { // windows of `kernel` taps along the last dimension (and `kernel_h` along the one before it, for 2-D)
    int kernel = 1, stride = 1, dilation = 1;
    int kernel_h = 1, stride_h = 1, dilation_h = 1;
    int groups = 1; // > 1: the channels are cut into groups, which lead the window view: (G, N, ..., C_in / G, K...)
};

using OpParams = std::variant<NoParams, ReductionParams, MatMulParams, ActivationParams, ReshapeParams, NormParams, TransposeParams, SliceParams,
                              PadParams, MaskedFillParams, UnfoldParams>;

template <typename T> const T &get_params(const OpParams &p) { return std::get<T>(p); }

struct GraphNode {
    uint64_t id;
    ops::OpType op_type{};
    std::vector<std::shared_ptr<GraphNode>> inputs;

    Shape output_shape;
    DType output_dtype{};
    Device target_device = Device::CPU;
    OpParams params;

    // an eager tensor fed into a lazy op
    std::shared_ptr<Storage> constant_storage;
    Strides constant_strides;
    size_t constant_offset = 0;
    bool is_constant = false;

    std::atomic<size_t> ref_count{0}; // how many other nodes consume this one

    mutable std::shared_ptr<Storage> cached_result_;
    mutable Shape cached_shape_;
    mutable Strides cached_strides_;
    mutable size_t cached_offset_ = 0;
    mutable bool is_materialized_ = false;

    GraphNode() : id(next_id()) {}
    // a node that goes away stops consuming its inputs
    ~GraphNode() {
        for (auto &in : inputs)
            if (in && !in->is_constant && in->ref_count.load() > 0) in->ref_count.fetch_sub(1);
    }
    size_t byte_size() const { return ShapeUtils::size(output_shape) * dtype_size(output_dtype); }

  private:
    static uint64_t next_id() {
        static std::atomic<uint64_t> counter{0};
        return counter.fetch_add(1);
    }
};

} // namespace axiom::graph
