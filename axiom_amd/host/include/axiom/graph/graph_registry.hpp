// Lazy tensor creation and materialisation
// (include/axiom/graph/graph_registry.hpp:23-154).
#pragma once

#include <array>

#include <memory>
#include <string>
#include <vector>

#include "axiom/graph/graph_node.hpp"

namespace axiom {
class Tensor;

namespace graph {

bool is_eager_mode_enabled(); // AXIOM_EAGER_MODE=1 or an active EagerModeScope
size_t get_max_pending_nodes();
void set_max_pending_nodes(size_t max_nodes);

Shape infer_binary_shape(const Shape &lhs, const Shape &rhs);
Shape infer_reduction_shape(const Shape &input, const std::vector<int> &axes, bool keep_dims);
Shape infer_matmul_shape(const Shape &a, const Shape &b, bool transpose_a, bool transpose_b);
DType infer_binary_dtype(DType lhs, DType rhs);
DType infer_unary_dtype(ops::OpType op, DType input);
DType infer_reduction_dtype(ops::OpType op, DType input); // Mean of a non-f64 dtype is Float32

class GraphRegistry {
  public:
    static Tensor create_lazy_unary(ops::OpType op, const Tensor &input, const OpParams &params = NoParams{});
    static Tensor create_lazy_binary(ops::OpType op, const Tensor &lhs, const Tensor &rhs, const OpParams &params = NoParams{});
    static Tensor create_lazy_where(const Tensor &condition, const Tensor &a, const Tensor &b);
    static Tensor create_lazy_cast(const Tensor &input, DType target);
    static Tensor create_lazy_reduction(ops::OpType op, const Tensor &input, const std::vector<int> &axes, bool keep_dims);
    static Tensor create_lazy_matmul(const Tensor &a, const Tensor &b, bool transpose_a, bool transpose_b);
    static Tensor create_lazy_softmax(ops::OpType op, const Tensor &input, int axis);
    static Tensor create_lazy_layernorm(const Tensor &input, const Tensor &weight, const Tensor &bias, int axis, float eps);
    // RMS norm is captured lazily too, so that rms_norm + activation is one kernel
    static Tensor create_lazy_rmsnorm(const Tensor &input, const Tensor &weight, int axis, float eps);
    static Tensor create_lazy_reshape(const Tensor &input, const Shape &new_shape);
    static Tensor create_lazy_transpose(const Tensor &input, const std::vector<int> &axes);
    // the remaining node kinds of whole forward passes (include/axiom/graph/graph_registry.hpp:70-122)
    static Tensor create_lazy_slice(const Tensor &input, const std::vector<int64_t> &starts, const std::vector<int64_t> &ends,
                                    const std::vector<int64_t> &steps, const Shape &output_shape);
    static Tensor create_lazy_pad(const Tensor &input, const std::vector<std::pair<size_t, size_t>> &pad_widths, double value, const Shape &output_shape,
                                  int mode = 0);
    static Tensor create_lazy_masked_fill(const Tensor &input, const Tensor &mask, float value);
    static Tensor create_lazy_glu(const Tensor &input, int dim, const Shape &output_shape);
    static Tensor create_lazy_batchnorm(const Tensor &input, const Tensor &weight, const Tensor &bias, const Tensor &running_mean,
                                        const Tensor &running_var, float eps);
    static Tensor create_lazy_conv1d(const Tensor &input, const Tensor &weight, const Tensor &bias, int stride, int padding, int dilation, int groups = 1);
    static Tensor create_lazy_conv2d(const Tensor &input, const Tensor &weight, const Tensor &bias, std::array<int, 2> stride,
                                     std::array<int, 2> padding, std::array<int, 2> dilation, int groups = 1);
    static Tensor create_lazy_embedding(const Tensor &weight, const Tensor &indices);

    // signature -> plan cache -> compile -> execute; GPU graphs go to materialize_gpu_graph
    static void materialize(GraphNode *node);
    static size_t pending_node_count();
    static void materialize_all();
    static Tensor finalize_lazy_node(std::shared_ptr<GraphNode> node);

  private:
    static thread_local std::vector<std::weak_ptr<GraphNode>> pending_nodes_;
};

class EagerModeScope {
  public:
    EagerModeScope();
    ~EagerModeScope();
    EagerModeScope(const EagerModeScope &) = delete;
    EagerModeScope &operator=(const EagerModeScope &) = delete;

  private:
    bool previous_mode_;
};

// The GPU hook of GraphRegistry::materialize (src/graph/graph_registry.cpp:834-850;
// Metal counterpart src/backends/metal/mpsgraph_graph_compiler.mm:706-944): turns the DAG
// under `root` into fused row programs, GEMMs and copies of libaxhip, runs them on the
// backend stream and leaves the result in root->cached_result_ / cached_shape_ /
// cached_strides_ with is_materialized_ set.
void materialize_gpu_graph(GraphNode *root);

// kernels launched by the last materialize_gpu_graph on this thread, in order
// (e.g. "rows_static_relu_adds_mulf_softmax_sum_f32_g256_it8"); for tests and AXIOM_DEBUG_FUSION
const std::vector<std::string> &last_gpu_plan_kernels();
// The names are collected only while this is on (or AXIOM_DEBUG_FUSION is set): asking the backend for a kernel's
// name costs about as much as launching it.
void record_gpu_plan_kernels(bool on);

} // namespace graph
} // namespace axiom
