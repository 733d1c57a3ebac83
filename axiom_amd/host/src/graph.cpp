// Lazy graph: node construction with shape / dtype inference, eager-mode switches,
// the pending list, the structural signature and GraphRegistry::materialize
// (behaviour of src/graph/graph_registry.cpp and graph_signature.cpp for the hot-path ops).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <unordered_map>
#include <unordered_set>

#include "axiom/error.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/graph/graph_signature.hpp"
#include "axiom/tensor.hpp"

namespace axiom::graph {

// ------------------------------------------------------------ eager switches
namespace {
thread_local bool tl_eager_scope = false;
size_t g_max_pending = 10000; // src/graph/graph_registry.cpp:30-35

bool env_eager() {
    static const bool v = [] {
        const char *e = std::getenv("AXIOM_EAGER_MODE");
        return e && std::string(e) == "1";
    }();
    return v;
}
} // namespace

bool is_eager_mode_enabled() { return tl_eager_scope || env_eager(); }
size_t get_max_pending_nodes() { return g_max_pending; }
void set_max_pending_nodes(size_t n) { g_max_pending = n; }

EagerModeScope::EagerModeScope() : previous_mode_(tl_eager_scope) { tl_eager_scope = true; }
EagerModeScope::~EagerModeScope() { tl_eager_scope = previous_mode_; }

// ----------------------------------------------------------------- inference
Shape infer_binary_shape(const Shape &lhs, const Shape &rhs) { return ShapeUtils::broadcast(lhs, rhs); }

// a full reduction without keep_dims yields shape {1} (src/graph/graph_registry.cpp:102-111)
Shape infer_reduction_shape(const Shape &input, const std::vector<int> &axes, bool keep_dims) {
    const int nd = static_cast<int>(input.size());
    std::vector<bool> red(nd, axes.empty());
    for (int a : axes) red[ShapeUtils::normalize_axis(a, nd)] = true;
    Shape out;
    for (int i = 0; i < nd; ++i) {
        if (!red[i]) out.push_back(input[i]);
        else if (keep_dims) out.push_back(1);
    }
    if (out.empty()) out.push_back(1);
    return out;
}

Shape infer_matmul_shape(const Shape &a, const Shape &b, bool ta, bool tb) {
    if (a.size() < 2 || b.size() < 2) throw ShapeError("matmul needs operands with at least 2 dimensions");
    const size_t m = ta ? a[a.size() - 1] : a[a.size() - 2], ka = ta ? a[a.size() - 2] : a[a.size() - 1];
    const size_t kb = tb ? b[b.size() - 1] : b[b.size() - 2], n = tb ? b[b.size() - 2] : b[b.size() - 1];
    if (ka != kb) throw ShapeError("matmul: inner dimensions differ (" + std::to_string(ka) + " vs " + std::to_string(kb) + ")");
    Shape out = ShapeUtils::broadcast(Shape(a.begin(), a.end() - 2), Shape(b.begin(), b.end() - 2));
    out.push_back(m);
    out.push_back(n);
    return out;
}

DType infer_binary_dtype(DType lhs, DType rhs) { return ops::promote_types(lhs, rhs); }
// comparisons and logical operations give Bool (src/graph/graph_registry.cpp:231-263)
DType infer_binary_output_dtype(ops::OpType op, DType lhs, DType rhs) {
    using ops::OpType;
    switch (op) {
    case OpType::Equal: case OpType::NotEqual: case OpType::Less: case OpType::LessEqual: case OpType::Greater: case OpType::GreaterEqual:
    case OpType::LogicalAnd: case OpType::LogicalOr: case OpType::LogicalXor:
        return DType::Bool;
    default: return ops::promote_types(lhs, rhs);
    }
}
DType infer_unary_dtype(ops::OpType op, DType input) {
    using ops::OpType;
    switch (op) {
    case OpType::IsNaN: case OpType::IsInf: case OpType::IsFinite: case OpType::LogicalNot: return DType::Bool;
    default: return input;
    }
}
DType infer_reduction_dtype(ops::OpType op, DType input) {
    if (op == ops::OpType::Mean) return input == DType::Float64 ? input : DType::Float32; // src/graph/graph_registry.cpp:278-287
    return input;
}

// ------------------------------------------------------------------ registry
thread_local std::vector<std::weak_ptr<GraphNode>> GraphRegistry::pending_nodes_;

namespace {

// Wraps an input tensor as a graph node: a lazy tensor contributes its node (ref_count++),
// an eager one a constant node over its storage, strides and offset
// (src/graph/graph_registry.cpp:297-311).
std::shared_ptr<GraphNode> input_node(const Tensor &t) {
    if (t.is_lazy() && !t.lazy_node()->is_materialized_) {
        auto n = t.lazy_node();
        n->ref_count.fetch_add(1);
        return n;
    }
    auto n = std::make_shared<GraphNode>();
    n->is_constant = true;
    n->output_shape = t.shape();
    n->output_dtype = t.dtype();
    n->target_device = t.device();
    n->constant_storage = t.storage();
    n->constant_strides = t.strides();
    n->constant_offset = t.offset();
    return n;
}

Device pick_device(std::initializer_list<const Tensor *> ts) {
    for (const Tensor *t : ts)
        if (!t->empty() && t->device() == Device::GPU) return Device::GPU;
    return Device::CPU;
}

void require_gpu(Device d, ops::OpType op) {
    if (d != Device::GPU)
        throw RuntimeError(std::string("ops::") + ops::op_name(op) + " on CPU tensors: this library is the gfx950 GPU backend only; move the operands with .gpu()");
}

// operands of a GPU op living on the host are moved over (src/tensor/operations.cpp:4018-4029)
Tensor on_gpu(const Tensor &t) { return t.empty() || t.device() == Device::GPU ? t : t.to(Device::GPU); }

} // namespace

Tensor GraphRegistry::finalize_lazy_node(std::shared_ptr<GraphNode> node) {
    if (is_eager_mode_enabled()) { // every op is its own graph
        Tensor t(node);
        t.sync();
        return t;
    }
    auto &pend = pending_nodes_;
    pend.push_back(node);
    if (pend.size() >= g_max_pending) { // src/graph/graph_registry.cpp:379-382
        Tensor t(node);
        materialize_all();
        return t;
    }
    return Tensor(std::move(node));
}

Tensor GraphRegistry::create_lazy_unary(ops::OpType op, const Tensor &input, const OpParams &params) {
    require_gpu(pick_device({&input}), op);
    // f(transpose(x)) == transpose(f(x)) for an elementwise f: apply it below a pending transpose, where it
    // can still fuse into whatever produces x (a GEMM epilogue, a row kernel) instead of forcing a gather
    // (the same holds for a pending reshape, which a convolution's result passes through)
    // `sinking` > 0: this call comes from the rewrite one level up, whose view node is the one consumer allowed
    static thread_local int sinking = 0;
    if (input.is_lazy() && !input.lazy_node()->is_materialized_ &&
        (input.lazy_node()->op_type == ops::OpType::Transpose || input.lazy_node()->op_type == ops::OpType::Reshape) &&
        input.lazy_node()->ref_count.load() == (sinking > 0 ? 1u : 0u) && !is_eager_mode_enabled()) {
        const auto tn = input.lazy_node();
        const Tensor inner = tn->inputs[0]->is_constant
                                 ? Tensor(tn->inputs[0]->constant_storage, tn->inputs[0]->output_shape, tn->inputs[0]->constant_strides,
                                          tn->inputs[0]->output_dtype, tn->inputs[0]->constant_offset)
                                 : Tensor(tn->inputs[0]);
        ++sinking;
        Tensor below;
        try {
            below = create_lazy_unary(op, inner, params);
        } catch (...) {
            --sinking;
            throw;
        }
        --sinking;
        if (tn->op_type == ops::OpType::Transpose) return create_lazy_transpose(below, get_params<TransposeParams>(tn->params).axes);
        return create_lazy_reshape(below, get_params<ReshapeParams>(tn->params).new_shape);
    }
    auto n = std::make_shared<GraphNode>();
    n->op_type = op;
    n->inputs = {input_node(input)};
    n->output_shape = input.shape();
    n->output_dtype = infer_unary_dtype(op, input.dtype());
    n->target_device = Device::GPU;
    n->params = params;
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_binary(ops::OpType op, const Tensor &lhs, const Tensor &rhs, const OpParams &params) {
    require_gpu(pick_device({&lhs, &rhs}), op);
    const Shape out = infer_binary_shape(lhs.shape(), rhs.shape());
    auto n = std::make_shared<GraphNode>();
    n->op_type = op;
    n->inputs = {input_node(on_gpu(lhs)), input_node(on_gpu(rhs))};
    n->output_shape = out;
    n->output_dtype = infer_binary_output_dtype(op, lhs.dtype(), rhs.dtype());
    n->target_device = Device::GPU;
    n->params = params;
    return finalize_lazy_node(std::move(n));
}

// where(condition, a, b): the three broadcast together; promote_types(a, b) is the result type
Tensor GraphRegistry::create_lazy_where(const Tensor &condition, const Tensor &a, const Tensor &b) {
    require_gpu(pick_device({&condition, &a, &b}), ops::OpType::Where);
    const Shape out = infer_binary_shape(infer_binary_shape(condition.shape(), a.shape()), b.shape());
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Where;
    n->inputs = {input_node(on_gpu(condition)), input_node(on_gpu(a)), input_node(on_gpu(b))};
    n->output_shape = out;
    n->output_dtype = infer_binary_dtype(a.dtype(), b.dtype());
    n->target_device = Device::GPU;
    return finalize_lazy_node(std::move(n));
}

// the GPU Cast as a node: the planner folds it into the kernel that produces or consumes the value
Tensor GraphRegistry::create_lazy_cast(const Tensor &input, DType target) {
    require_gpu(pick_device({&input}), ops::OpType::Cast);
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Cast;
    n->inputs = {input_node(input)};
    n->output_shape = input.shape();
    n->output_dtype = target;
    n->target_device = Device::GPU;
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_reduction(ops::OpType op, const Tensor &input, const std::vector<int> &axes, bool keep_dims) {
    require_gpu(pick_device({&input}), op);
    // Nothing to read: an empty result stays empty; a reduction over an empty extent gives the operation's identity
    // (sum 0, product 1, mean 0/0), and there is no largest or smallest element of nothing.
    if (ShapeUtils::size(input.shape()) == 0) {
        const Shape wanted = infer_reduction_shape(input.shape(), axes, keep_dims);
        const DType rd = infer_reduction_dtype(op, input.dtype());
        if (ShapeUtils::size(wanted) == 0) return Tensor(wanted, rd, Device::GPU);
        if (op == ops::OpType::Max || op == ops::OpType::Min) throw ValueError(std::string("ops::") + ops::op_name(op) + " over an empty axis");
        const double identity = op == ops::OpType::Prod ? 1.0 : op == ops::OpType::Mean ? std::nan("") : 0.0;
        return Tensor::full(wanted, static_cast<float>(identity), Device::CPU).astype(rd).to(Device::GPU);
    }
    // The device reduces over the last axis or over everything.  Any other set of axes is brought there first: the
    // kept axes in front, the reduced ones behind them and folded into one (a transposed view that the planner
    // gathers into a contiguous array), then the result takes the shape the caller asked for.
    {
        const int nd = static_cast<int>(input.ndim());
        const Shape wanted = infer_reduction_shape(input.shape(), axes, keep_dims); // validates the axes
        std::vector<bool> red(static_cast<size_t>(nd), axes.empty());
        for (int a : axes) red[static_cast<size_t>(ShapeUtils::normalize_axis(a, nd))] = true;
        std::vector<int> kept_axes, red_axes;
        size_t kept = 1, folded = 1;
        for (int i = 0; i < nd; ++i) {
            (red[static_cast<size_t>(i)] ? red_axes : kept_axes).push_back(i);
            (red[static_cast<size_t>(i)] ? folded : kept) *= input.shape()[static_cast<size_t>(i)];
        }
        const bool all = kept_axes.empty() || kept == 1;
        const bool last_only = red_axes.size() == 1 && red_axes[0] == nd - 1;
        // (one run of neighbouring axes that ends before the last one is reduced where it lies: the planner has a
        // kernel for the middle extent of an (outer, axis, inner) array)
        const bool inner_run = !red_axes.empty() && red_axes.back() != nd - 1 && red_axes.back() - red_axes.front() + 1 == static_cast<int>(red_axes.size()) &&
                               [&] { size_t in = 1; for (int i = red_axes.back() + 1; i < nd; ++i) in *= input.shape()[static_cast<size_t>(i)]; return in > 1; }();
        if (!all && !last_only && !inner_run && !red_axes.empty() && kept * folded > 0) {
            std::vector<int> order = kept_axes;
            order.insert(order.end(), red_axes.begin(), red_axes.end());
            bool identity = true;
            for (int i = 0; i < nd; ++i) identity = identity && order[static_cast<size_t>(i)] == i;
            const Tensor moved = identity ? input : create_lazy_transpose(input, order);
            const Tensor rows = create_lazy_reshape(moved, Shape{kept, folded});
            return create_lazy_reshape(create_lazy_reduction(op, rows, {1}, false), wanted);
        }
    }
    auto n = std::make_shared<GraphNode>();
    n->op_type = op;
    n->output_shape = infer_reduction_shape(input.shape(), axes, keep_dims); // validates the axes
    n->inputs = {input_node(input)};
    n->output_dtype = infer_reduction_dtype(op, input.dtype());
    n->target_device = Device::GPU;
    n->params = ReductionParams{axes, keep_dims};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_matmul(const Tensor &a, const Tensor &b, bool ta, bool tb) {
    require_gpu(pick_device({&a, &b}), ops::OpType::MatMul);
    const Shape out = infer_matmul_shape(a.shape(), b.shape(), ta, tb);
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::MatMul;
    n->inputs = {input_node(on_gpu(a)), input_node(on_gpu(b))};
    n->output_shape = out;
    n->output_dtype = infer_binary_dtype(a.dtype(), b.dtype());
    n->target_device = Device::GPU;
    n->params = MatMulParams{ta, tb};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_softmax(ops::OpType op, const Tensor &input, int axis) {
    require_gpu(pick_device({&input}), op);
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(input.ndim()));
    // (over another axis than the last: the planner has a kernel for the middle extent of an (outer, axis, inner) array)
    auto n = std::make_shared<GraphNode>();
    n->op_type = op;
    n->inputs = {input_node(input)};
    n->output_shape = input.shape();
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    ActivationParams p;
    p.axis = a;
    n->params = p;
    return finalize_lazy_node(std::move(n));
}

// the norm output keeps the input dtype on GPU (src/graph/graph_registry.cpp:622-627)
Tensor GraphRegistry::create_lazy_layernorm(const Tensor &input, const Tensor &weight, const Tensor &bias, int axis, float eps) {
    require_gpu(pick_device({&input}), ops::OpType::LayerNorm);
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(input.ndim()));
    // over another axis than the last (per-channel statistics of a channels-first array): that axis and the last one
    // change places, before and after the row kernel
    if (a != static_cast<int>(input.ndim()) - 1) {
        std::vector<int> swap(input.ndim());
        for (size_t i = 0; i < swap.size(); ++i) swap[i] = static_cast<int>(i);
        std::swap(swap[static_cast<size_t>(a)], swap.back());
        return create_lazy_transpose(create_lazy_layernorm(create_lazy_transpose(input, swap), weight, bias, -1, eps), swap);
    }
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::LayerNorm;
    n->inputs = {input_node(input)};
    if (!weight.empty()) n->inputs.push_back(input_node(on_gpu(weight)));
    if (!bias.empty()) {
        if (weight.empty()) throw ValueError("layer_norm: bias without weight");
        n->inputs.push_back(input_node(on_gpu(bias)));
    }
    n->output_shape = input.shape();
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = NormParams{a, eps};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_rmsnorm(const Tensor &input, const Tensor &weight, int axis, float eps) {
    require_gpu(pick_device({&input}), ops::OpType::RMSNorm);
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(input.ndim()));
    if (a != static_cast<int>(input.ndim()) - 1) { // as for layer_norm
        std::vector<int> swap(input.ndim());
        for (size_t i = 0; i < swap.size(); ++i) swap[i] = static_cast<int>(i);
        std::swap(swap[static_cast<size_t>(a)], swap.back());
        return create_lazy_transpose(create_lazy_rmsnorm(create_lazy_transpose(input, swap), weight, -1, eps), swap);
    }
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::RMSNorm;
    n->inputs = {input_node(input)};
    if (!weight.empty()) n->inputs.push_back(input_node(on_gpu(weight)));
    n->output_shape = input.shape();
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = NormParams{a, eps};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_reshape(const Tensor &input, const Shape &new_shape) {
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Reshape;
    n->inputs = {input_node(input)};
    n->output_shape = new_shape;
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = ReshapeParams{new_shape};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_transpose(const Tensor &input, const std::vector<int> &axes) {
    // transpose(transpose(x, p), q) == transpose(x, p o q); the identity gives x back
    if (input.is_lazy() && !input.lazy_node()->is_materialized_ && input.lazy_node()->op_type == ops::OpType::Transpose &&
        !input.lazy_node()->inputs[0]->is_constant) {
        const auto tn = input.lazy_node();
        const auto &inner_axes = get_params<TransposeParams>(tn->params).axes;
        std::vector<int> composed(axes.size());
        bool identity = true;
        for (size_t i = 0; i < axes.size(); ++i) {
            composed[i] = inner_axes[axes[i]];
            identity = identity && composed[i] == static_cast<int>(i);
        }
        const Tensor inner(tn->inputs[0]);
        return identity ? inner : create_lazy_transpose(inner, composed);
    }
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Transpose;
    n->inputs = {input_node(input)};
    const Shape &in = input.shape();
    Shape out(in.size());
    for (size_t i = 0; i < axes.size(); ++i) out[i] = in[axes[i]];
    n->output_shape = out;
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = TransposeParams{axes};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_slice(const Tensor &input, const std::vector<int64_t> &starts, const std::vector<int64_t> &ends,
                                        const std::vector<int64_t> &steps, const Shape &output_shape) {
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Slice;
    n->inputs = {input_node(input)};
    n->output_shape = output_shape;
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = SliceParams{starts, ends, steps};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_pad(const Tensor &input, const std::vector<std::pair<size_t, size_t>> &pad_widths, double value,
                                      const Shape &output_shape, int mode) {
    require_gpu(pick_device({&input}), ops::OpType::Pad);
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Pad;
    n->inputs = {input_node(input)};
    n->output_shape = output_shape;
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = PadParams{pad_widths, value, mode};
    return finalize_lazy_node(std::move(n));
}

Tensor GraphRegistry::create_lazy_masked_fill(const Tensor &input, const Tensor &mask, float value) {
    require_gpu(pick_device({&input, &mask}), ops::OpType::MaskedFill);
    if (dtype_size(mask.dtype()) != 1) throw TypeError("masked_fill: the mask must be Bool (or a one-byte integer type)");
    const Shape out = infer_binary_shape(input.shape(), mask.shape());
    if (out != input.shape()) throw ShapeError("masked_fill: the mask must broadcast to the input's shape");
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::MaskedFill;
    n->inputs = {input_node(on_gpu(input)), input_node(on_gpu(mask))};
    n->output_shape = input.shape();
    n->output_dtype = input.dtype();
    n->target_device = Device::GPU;
    n->params = MaskedFillParams{value};
    return finalize_lazy_node(std::move(n));
}

// a * sigmoid(b) over the halves of `dim`: two Slice views (gathered when the cut leaves them strided),
// then Sigmoid and Multiply in one row kernel
Tensor GraphRegistry::create_lazy_glu(const Tensor &input, int dim, const Shape &output_shape) {
    require_gpu(pick_device({&input}), ops::OpType::GLU);
    const size_t nd = input.ndim(), half = output_shape[dim];
    std::vector<int64_t> lo(nd, 0), hi(input.shape().begin(), input.shape().end()), st(nd, 1);
    auto a_hi = hi, b_lo = lo;
    a_hi[dim] = static_cast<int64_t>(half);
    b_lo[dim] = static_cast<int64_t>(half);
    const Tensor a = create_lazy_slice(input, lo, a_hi, st, output_shape), b = create_lazy_slice(input, b_lo, hi, st, output_shape);
    return create_lazy_binary(ops::OpType::Multiply, a, create_lazy_unary(ops::OpType::Sigmoid, b));
}

// (x - mean) / sqrt(var + eps) * w + b per channel (dim 1), lowered to x * scale + shift with the two
// per-channel vectors computed by tiny elementwise graphs of their own
Tensor GraphRegistry::create_lazy_batchnorm(const Tensor &input, const Tensor &weight, const Tensor &bias, const Tensor &running_mean,
                                            const Tensor &running_var, float eps) {
    require_gpu(pick_device({&input}), ops::OpType::BatchNorm1D);
    if (input.ndim() != 2 && input.ndim() != 3) throw ShapeError("batch_norm1d expects (N, C) or (N, C, L), got " + std::to_string(input.ndim()) + " dimensions");
    const size_t C = input.shape()[1];
    for (const Tensor *t : {&running_mean, &running_var})
        if (t->ndim() != 1 || t->shape()[0] != C) throw ShapeError("batch_norm1d: running statistics must have shape (C)");
    const Tensor var = on_gpu(running_var), mean = on_gpu(running_mean);
    Tensor scale = create_lazy_unary(ops::OpType::Reciprocal, create_lazy_unary(ops::OpType::Sqrt, var + eps));
    if (!weight.empty()) scale = create_lazy_binary(ops::OpType::Multiply, scale, on_gpu(weight));
    Tensor shift = create_lazy_unary(ops::OpType::Negate, create_lazy_binary(ops::OpType::Multiply, mean, scale));
    if (!bias.empty()) shift = create_lazy_binary(ops::OpType::Add, shift, on_gpu(bias));
    if (input.ndim() == 3) {
        scale = scale.reshape({C, 1});
        shift = shift.reshape({C, 1});
    }
    return create_lazy_binary(ops::OpType::Add, create_lazy_binary(ops::OpType::Multiply, input, scale), shift);
}

// Convolution as a GEMM: constant padding, the (N, L_out, C_in, K) window view of the padded signal, its
// gather to (N, L_out, C_in K), a product with the (C_out, C_in K) filter matrix (bias and a following
// activation ride in the GEMM epilogue), and the (N, C_out, L_out) view of the result.
Tensor GraphRegistry::create_lazy_conv1d(const Tensor &input, const Tensor &weight, const Tensor &bias, int stride, int padding, int dilation, int groups) {
    require_gpu(pick_device({&input}), ops::OpType::Conv1D);
    const size_t N = input.shape()[0], Cin = input.shape()[1], L = input.shape()[2];
    const size_t Cout = weight.shape()[0], K = weight.shape()[2];
    const size_t Lp = L + 2 * static_cast<size_t>(padding), span = static_cast<size_t>(dilation) * (K - 1) + 1;
    if (Lp < span) throw ShapeError("conv1d: the kernel does not fit the padded input");
    const size_t Lout = (Lp - span) / static_cast<size_t>(stride) + 1;
    Tensor x = on_gpu(input);
    if (padding > 0) x = create_lazy_pad(x, {{0, 0}, {0, 0}, {static_cast<size_t>(padding), static_cast<size_t>(padding)}}, 0.0, Shape{N, Cin, Lp});
    auto un = std::make_shared<GraphNode>();
    un->op_type = ops::OpType::Unfold1D;
    un->inputs = {input_node(x)};
    un->output_shape = Shape{N, Lout, Cin, K};
    un->output_dtype = x.dtype();
    un->target_device = Device::GPU;
    UnfoldParams up{static_cast<int>(K), stride, dilation};
    up.groups = groups;
    un->params = up;
    if (groups > 1) {
        // Grouped: the windows lead with the group, (G, N, L_out, C_in / G, K), one batched product against the
        // (G, C_out / G, C_in / G * K) filters gives (G, N L_out, C_out / G), which is brought to (N, C_out, L_out).
        const size_t G = static_cast<size_t>(groups), Cg = Cin / G, Og = Cout / G;
        un->output_shape = Shape{G, N, Lout, Cg, K};
        const Tensor cols = create_lazy_reshape(finalize_lazy_node(std::move(un)), Shape{G, N * Lout, Cg * K});
        const Tensor w3 = on_gpu(weight).reshape({G, Og, Cg * K});
        Tensor y = create_lazy_matmul(cols, w3, false, true); // (G, N L_out, O_g)
        if (!bias.empty()) y = create_lazy_binary(ops::OpType::Add, y, on_gpu(bias).reshape({G, 1, Og}));
        const Tensor moved = create_lazy_transpose(create_lazy_reshape(y, Shape{G, N, Lout, Og}), {1, 0, 3, 2}); // (N, G, O_g, L_out)
        return create_lazy_reshape(moved, Shape{N, Cout, Lout});
    }
    const Tensor cols = create_lazy_reshape(finalize_lazy_node(std::move(un)), Shape{N, Lout, Cin * K});
    const Tensor w2 = on_gpu(weight).reshape({Cout, Cin * K});
    Tensor y = create_lazy_matmul(cols, w2, false, true);
    if (!bias.empty()) y = create_lazy_binary(ops::OpType::Add, y, on_gpu(bias));
    return create_lazy_transpose(y, {0, 2, 1});
}

// The same lowering in two dimensions: windows (N, H_out, W_out, C_in, KH, KW), product with the (C_out, C_in KH KW)
// filter matrix, result laid out (N, H_out, W_out, C_out) and returned as its (N, C_out, H_out, W_out) view.
Tensor GraphRegistry::create_lazy_conv2d(const Tensor &input, const Tensor &weight, const Tensor &bias, std::array<int, 2> stride,
                                         std::array<int, 2> padding, std::array<int, 2> dilation, int groups) {
    require_gpu(pick_device({&input}), ops::OpType::Conv2D);
    const size_t N = input.shape()[0], Cin = input.shape()[1], Hin = input.shape()[2], Win = input.shape()[3];
    const size_t Cout = weight.shape()[0], KH = weight.shape()[2], KW = weight.shape()[3];
    const size_t Hp = Hin + 2 * static_cast<size_t>(padding[0]), Wp = Win + 2 * static_cast<size_t>(padding[1]);
    const size_t span_h = static_cast<size_t>(dilation[0]) * (KH - 1) + 1, span_w = static_cast<size_t>(dilation[1]) * (KW - 1) + 1;
    if (Hp < span_h || Wp < span_w) throw ShapeError("conv2d: the kernel does not fit the padded input");
    const size_t Hout = (Hp - span_h) / static_cast<size_t>(stride[0]) + 1, Wout = (Wp - span_w) / static_cast<size_t>(stride[1]) + 1;
    Tensor x = on_gpu(input);
    if (padding[0] > 0 || padding[1] > 0)
        x = create_lazy_pad(x, {{0, 0}, {0, 0}, {static_cast<size_t>(padding[0]), static_cast<size_t>(padding[0])}, {static_cast<size_t>(padding[1]), static_cast<size_t>(padding[1])}},
                            0.0, Shape{N, Cin, Hp, Wp});
    auto un = std::make_shared<GraphNode>();
    un->op_type = ops::OpType::Unfold2D;
    un->inputs = {input_node(x)};
    un->output_shape = Shape{N, Hout, Wout, Cin, KH, KW};
    un->output_dtype = x.dtype();
    un->target_device = Device::GPU;
    UnfoldParams up;
    up.kernel = static_cast<int>(KW);
    up.stride = stride[1];
    up.dilation = dilation[1];
    up.kernel_h = static_cast<int>(KH);
    up.stride_h = stride[0];
    up.dilation_h = dilation[0];
    up.groups = groups;
    un->params = up;
    if (groups > 1) { // as for conv1d: (G, N, H_out, W_out, C_in / G, KH, KW) windows, one batched product
        const size_t G = static_cast<size_t>(groups), Cg = Cin / G, Og = Cout / G;
        un->output_shape = Shape{G, N, Hout, Wout, Cg, KH, KW};
        const Tensor cols = create_lazy_reshape(finalize_lazy_node(std::move(un)), Shape{G, N * Hout * Wout, Cg * KH * KW});
        const Tensor w3 = on_gpu(weight).reshape({G, Og, Cg * KH * KW});
        Tensor y = create_lazy_matmul(cols, w3, false, true); // (G, N H_out W_out, O_g)
        if (!bias.empty()) y = create_lazy_binary(ops::OpType::Add, y, on_gpu(bias).reshape({G, 1, Og}));
        const Tensor moved = create_lazy_transpose(create_lazy_reshape(y, Shape{G, N, Hout * Wout, Og}), {1, 0, 3, 2}); // (N, G, O_g, H_out W_out)
        return create_lazy_reshape(moved, Shape{N, Cout, Hout, Wout});
    }
    const Tensor cols = create_lazy_reshape(finalize_lazy_node(std::move(un)), Shape{N, Hout * Wout, Cin * KH * KW});
    const Tensor w2 = on_gpu(weight).reshape({Cout, Cin * KH * KW});
    Tensor y = create_lazy_matmul(cols, w2, false, true);
    if (!bias.empty()) y = create_lazy_binary(ops::OpType::Add, y, on_gpu(bias));
    return create_lazy_transpose(create_lazy_reshape(y, Shape{N, Hout, Wout, Cout}), {0, 3, 1, 2});
}

Tensor GraphRegistry::create_lazy_embedding(const Tensor &weight, const Tensor &indices) {
    require_gpu(pick_device({&weight, &indices}), ops::OpType::Gather);
    auto n = std::make_shared<GraphNode>();
    n->op_type = ops::OpType::Gather;
    n->inputs = {input_node(on_gpu(weight)), input_node(on_gpu(indices))};
    Shape out = indices.shape();
    out.push_back(weight.shape()[1]);
    n->output_shape = out;
    n->output_dtype = weight.dtype();
    n->target_device = Device::GPU;
    return finalize_lazy_node(std::move(n));
}

// src/graph/graph_registry.cpp:830-927; GPU graphs bypass the CPU compiler (:834-850)
void GraphRegistry::materialize(GraphNode *node) {
    if (!node || node->is_materialized_) return;
    if (node->target_device != Device::GPU)
        throw RuntimeError("lazy CPU graphs cannot be materialised: this library is the gfx950 GPU backend only");
    materialize_gpu_graph(node);
}

size_t GraphRegistry::pending_node_count() {
    auto &p = pending_nodes_;
    p.erase(std::remove_if(p.begin(), p.end(), [](const std::weak_ptr<GraphNode> &w) {
                auto s = w.lock();
                return !s || s->is_materialized_;
            }),
            p.end());
    return p.size();
}

void GraphRegistry::materialize_all() {
    auto pending = std::move(pending_nodes_);
    pending_nodes_.clear();
    // newest first: a root materialises its whole subgraph, older entries are then done
    for (auto it = pending.rbegin(); it != pending.rend(); ++it)
        if (auto n = it->lock())
            if (!n->is_materialized_) materialize(n.get());
}

// ----------------------------------------------------------------- signature
std::vector<const GraphNode *> topo_sort(const GraphNode *root) {
    std::vector<const GraphNode *> order;
    std::unordered_set<const GraphNode *> seen;
    struct Frame {
        const GraphNode *n;
        size_t next;
    };
    std::vector<Frame> stack{{root, 0}};
    seen.insert(root);
    while (!stack.empty()) {
        Frame &f = stack.back();
        const bool leaf = f.n->is_constant || (f.n->is_materialized_ && f.n != root);
        if (!leaf && f.next < f.n->inputs.size()) {
            const GraphNode *c = f.n->inputs[f.next++].get();
            if (seen.insert(c).second) stack.push_back({c, 0});
        } else {
            order.push_back(f.n);
            stack.pop_back();
        }
    }
    return order;
}

namespace {
// FNV-1a over the bytes of everything that decides what a graph computes.  A value is fed in the width named by the
// call (sizes and indices as 64 bits, axes and window sizes as 32, floats by their bit pattern, flags as one byte).
class Fnv1a {
  public:
    void bytes(const void *p, size_t n) {
        const unsigned char *b = static_cast<const unsigned char *>(p);
        for (size_t i = 0; i < n; ++i) state_ = (state_ ^ b[i]) * 1099511628211ULL;
    }
    void u64(uint64_t v) { bytes(&v, 8); }
    void i32(int32_t v) { bytes(&v, 4); }
    void f32(float v) { bytes(&v, 4); }
    void flag(bool v) {
        const unsigned char b = v ? 1 : 0;
        bytes(&b, 1);
    }
    template <typename T, typename F> void list(const std::vector<T> &v, F &&each) {
        u64(v.size());
        for (const T &x : v) each(x);
    }
    uint64_t value() const { return state_; }

  private:
    uint64_t state_ = 14695981039346656037ULL;
};

// what each kind of node parameters contributes (nodes without parameters: nothing beyond the variant's index)
void feed(Fnv1a &h, const NoParams &) { (void)h; }
void feed(Fnv1a &h, const ReductionParams &p) {
    h.list(p.axes, [&](int a) { h.i32(a); });
    h.flag(p.keep_dims);
}
void feed(Fnv1a &h, const MatMulParams &p) {
    h.flag(p.transpose_a);
    h.flag(p.transpose_b);
}
void feed(Fnv1a &h, const ActivationParams &p) {
    h.f32(p.alpha);
    h.i32(p.axis);
}
void feed(Fnv1a &h, const ReshapeParams &p) {
    h.list(p.new_shape, [&](size_t d) { h.u64(d); });
}
void feed(Fnv1a &h, const NormParams &p) {
    h.i32(p.axis);
    h.f32(p.eps);
}
void feed(Fnv1a &h, const TransposeParams &p) {
    h.list(p.axes, [&](int a) { h.i32(a); });
}
void feed(Fnv1a &h, const SliceParams &p) {
    h.u64(p.starts.size());
    for (size_t i = 0; i < p.starts.size(); ++i) {
        h.u64(static_cast<uint64_t>(p.starts[i]));
        h.u64(static_cast<uint64_t>(p.ends[i]));
        h.u64(static_cast<uint64_t>(p.steps[i]));
    }
}
void feed(Fnv1a &h, const PadParams &p) {
    h.list(p.pad_widths, [&](const auto &w) {
        h.u64(w.first);
        h.u64(w.second);
    });
    h.bytes(&p.value, sizeof(p.value));
    h.i32(p.mode);
}
void feed(Fnv1a &h, const MaskedFillParams &p) { h.f32(p.value); }
void feed(Fnv1a &h, const UnfoldParams &p) {
    for (int v : {p.kernel, p.stride, p.dilation, p.kernel_h, p.stride_h, p.dilation_h, p.groups}) h.i32(v);
}

// one node: operation, result, where it sits in the order, what it reads
void feed_node(Fnv1a &h, const GraphNode *n, const GraphNode *root, const std::unordered_map<const GraphNode *, uint32_t> &position) {
    h.u64(static_cast<uint64_t>(n->op_type));
    h.list(n->output_shape, [&](size_t d) { h.u64(d); });
    h.u64(static_cast<uint64_t>(n->output_dtype));
    h.u64(static_cast<uint64_t>(n->target_device));
    h.flag(n->is_constant);
    if (n->is_constant) h.list(n->constant_strides, [&](int64_t s) { h.u64(static_cast<uint64_t>(s)); });
    // a constant, and a node that already holds its result, are inputs of the plan: what produced them is not part of it
    const bool leaf = n->is_constant || (n->is_materialized_ && n != root);
    if (leaf) {
        h.u64(0);
    } else {
        h.list(n->inputs, [&](const std::shared_ptr<GraphNode> &in) {
            const auto it = position.find(in.get());
            h.u64(it != position.end() ? it->second : UINT64_MAX);
        });
    }
    h.u64(n->params.index());
    std::visit([&](const auto &p) { feed(h, p); }, n->params);
}
} // namespace

GraphSignature compute_signature(const GraphNode *root) {
    const auto order = topo_sort(root);
    std::unordered_map<const GraphNode *, uint32_t> position;
    position.reserve(order.size());
    for (uint32_t i = 0; i < order.size(); ++i) position.emplace(order[i], i);
    Fnv1a h;
    h.u64(order.size());
    for (const GraphNode *n : order) feed_node(h, n, root, position);
    return GraphSignature{h.value()};
}

} // namespace axiom::graph
