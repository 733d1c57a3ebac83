// ops:: entry points: validation, device unification and routing into the lazy graph
// or the eager attention call (behaviour of src/tensor/operations.cpp for the hot-path ops).
#include "axiom/operations.hpp"

#include <cmath>
#include <map>

#include "axiom/error.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/tensor.hpp"
#include "hip_call.hpp"

namespace axiom::ops {

const char *op_name(OpType op) {
    switch (op) {
    case OpType::Add: return "add";
    case OpType::Subtract: return "subtract";
    case OpType::Multiply: return "multiply";
    case OpType::Divide: return "divide";
    case OpType::Maximum: return "maximum";
    case OpType::Minimum: return "minimum";
    case OpType::Power: return "power";
    case OpType::Modulo: return "modulo";
    case OpType::Atan2: return "atan2";
    case OpType::Hypot: return "hypot";
    case OpType::Equal: return "equal";
    case OpType::NotEqual: return "not_equal";
    case OpType::Less: return "less";
    case OpType::LessEqual: return "less_equal";
    case OpType::Greater: return "greater";
    case OpType::GreaterEqual: return "greater_equal";
    case OpType::LogicalAnd: return "logical_and";
    case OpType::LogicalOr: return "logical_or";
    case OpType::LogicalXor: return "logical_xor";
    case OpType::LogicalNot: return "logical_not";
    case OpType::Sin: return "sin";
    case OpType::Cos: return "cos";
    case OpType::Tan: return "tan";
    case OpType::Erf: return "erf";
    case OpType::Sign: return "sign";
    case OpType::Floor: return "floor";
    case OpType::Ceil: return "ceil";
    case OpType::Trunc: return "trunc";
    case OpType::Round: return "round";
    case OpType::Cbrt: return "cbrt";
    case OpType::IsNaN: return "isnan";
    case OpType::IsInf: return "isinf";
    case OpType::IsFinite: return "isfinite";
    case OpType::LeakyReLU: return "leaky_relu";
    case OpType::Where: return "where";
    case OpType::Cast: return "cast";
    case OpType::Prod: return "prod";
    case OpType::Any: return "any";
    case OpType::All: return "all";
    case OpType::Negate: return "negate";
    case OpType::Abs: return "abs";
    case OpType::Sqrt: return "sqrt";
    case OpType::Exp: return "exp";
    case OpType::Log: return "log";
    case OpType::Reciprocal: return "reciprocal";
    case OpType::Square: return "square";
    case OpType::ReLU: return "relu";
    case OpType::SiLU: return "silu";
    case OpType::Sigmoid: return "sigmoid";
    case OpType::Tanh: return "tanh";
    case OpType::GELU: return "gelu";
    case OpType::Softmax: return "softmax";
    case OpType::LogSoftmax: return "log_softmax";
    case OpType::Sum: return "sum";
    case OpType::Mean: return "mean";
    case OpType::Max: return "max";
    case OpType::Min: return "min";
    case OpType::MatMul: return "matmul";
    case OpType::LayerNorm: return "layer_norm";
    case OpType::RMSNorm: return "rms_norm";
    case OpType::Reshape: return "reshape";
    case OpType::Transpose: return "transpose";
    case OpType::Slice: return "slice";
    case OpType::Pad: return "pad";
    case OpType::MaskedFill: return "masked_fill";
    case OpType::GLU: return "glu";
    case OpType::Gather: return "embedding";
    case OpType::Conv1D: return "conv1d";
    case OpType::BatchNorm1D: return "batch_norm1d";
    case OpType::Unfold1D: return "unfold1d";
    case OpType::Unfold2D: return "unfold2d";
    case OpType::Conv2D: return "conv2d";
    case OpType::ScaledDotProductAttention: return "scaled_dot_product_attention";
    default: return "op";
    }
}

// src/tensor/operations.cpp:346-397: the higher rank wins among floats; mixed-sign
// integers of equal width widen
DType promote_types(DType lhs, DType rhs) {
    if (lhs == rhs) return lhs;
    static const std::map<DType, int> rank = {
        {DType::Bool, 0}, {DType::Int8, 1}, {DType::UInt8, 2}, {DType::Int16, 3}, {DType::UInt16, 4},
        {DType::Int32, 5}, {DType::UInt32, 6}, {DType::Int64, 7}, {DType::UInt64, 8}, {DType::Float16, 9},
        {DType::BFloat16, 10}, {DType::Float32, 11}, {DType::Float64, 12}, {DType::Complex64, 13}, {DType::Complex128, 14}};
    const bool l_hi = rank.at(lhs) > rank.at(rhs);
    const DType t1 = l_hi ? lhs : rhs, t2 = l_hi ? rhs : lhs;
    if (is_complex_dtype(t1) || is_floating_dtype(t1)) return t1;
    auto is_signed = [](DType d) { return d == DType::Int8 || d == DType::Int16 || d == DType::Int32 || d == DType::Int64; };
    const bool s1 = is_signed(t1), s2 = is_signed(t2);
    const size_t z1 = dtype_size(t1), z2 = dtype_size(t2);
    if (s1 == s2 || z1 > z2) return t1;
    switch (std::max(z1, z2)) {
    case 1: return DType::Int16;
    case 2: return DType::Int32;
    case 4: return DType::Int64;
    default: return DType::Float64;
    }
}

using graph::GraphRegistry;

Tensor add(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Add, a, b); }
Tensor subtract(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Subtract, a, b); }
Tensor multiply(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Multiply, a, b); }
Tensor divide(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Divide, a, b); }
Tensor maximum(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Maximum, a, b); }
Tensor minimum(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Minimum, a, b); }

Tensor power(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Power, a, b); }
Tensor modulo(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Modulo, a, b); }
Tensor atan2(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Atan2, a, b); }
Tensor hypot(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Hypot, a, b); }
Tensor equal(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Equal, a, b); }
Tensor not_equal(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::NotEqual, a, b); }
Tensor less(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Less, a, b); }
Tensor less_equal(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::LessEqual, a, b); }
Tensor greater(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::Greater, a, b); }
Tensor greater_equal(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::GreaterEqual, a, b); }
Tensor logical_and(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::LogicalAnd, a, b); }
Tensor logical_or(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::LogicalOr, a, b); }
Tensor logical_xor(const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_binary(OpType::LogicalXor, a, b); }
Tensor logical_not(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::LogicalNot, x); }

Tensor sin(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Sin, x); }
Tensor cos(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Cos, x); }
Tensor tan(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Tan, x); }
Tensor erf(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Erf, x); }
Tensor sign(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Sign, x); }
Tensor floor(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Floor, x); }
Tensor ceil(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Ceil, x); }
Tensor trunc(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Trunc, x); }
Tensor round(const Tensor &x, int decimals) {
    if (decimals == 0) return GraphRegistry::create_lazy_unary(OpType::Round, x);
    const double scale = std::pow(10.0, decimals); // src/tensor/operations.cpp:1334-1340
    return GraphRegistry::create_lazy_unary(OpType::Round, x * static_cast<float>(scale)) * static_cast<float>(1.0 / scale);
}
Tensor cbrt(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Cbrt, x); }
Tensor isnan(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::IsNaN, x); }
Tensor isinf(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::IsInf, x); }
Tensor isfinite(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::IsFinite, x); }
Tensor clip(const Tensor &x, const Tensor &lo, const Tensor &hi) { return maximum(minimum(x, hi), lo); }
// one node with the slope as its parameter (the reference builds other slopes than 0.01 from two ReLUs,
// src/tensor/operations.cpp:1391-1403: the same function)
Tensor leaky_relu(const Tensor &x, float negative_slope) {
    graph::ActivationParams p;
    p.alpha = negative_slope;
    return GraphRegistry::create_lazy_unary(OpType::LeakyReLU, x, p);
}
Tensor where(const Tensor &condition, const Tensor &a, const Tensor &b) { return GraphRegistry::create_lazy_where(condition, a, b); }
Tensor cast(const Tensor &x, DType target) {
    if (x.dtype() == target) return x;
    auto ok = [](DType d) { return d == DType::Float32 || d == DType::Float16 || d == DType::BFloat16 || d == DType::Bool; };
    if (!ok(x.dtype()) || !ok(target)) throw TypeError("ops::cast on the GPU: Float32, Float16, BFloat16 and Bool; got " + dtype_name(x.dtype()) + " -> " + dtype_name(target));
    return GraphRegistry::create_lazy_cast(x, target);
}

Tensor negate(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Negate, x); }
Tensor abs(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Abs, x); }
Tensor sqrt(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Sqrt, x); }
Tensor exp(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Exp, x); }
Tensor log(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Log, x); }
Tensor reciprocal(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Reciprocal, x); }
Tensor square(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Square, x); }
Tensor relu(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::ReLU, x); }
Tensor silu(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::SiLU, x); }
Tensor sigmoid(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Sigmoid, x); }
Tensor tanh(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::Tanh, x); }
Tensor gelu(const Tensor &x) { return GraphRegistry::create_lazy_unary(OpType::GELU, x); }

// on GPU softmax and the norms are captured lazily (src/tensor/operations.cpp:1420-1425, 1791-1795)
Tensor softmax(const Tensor &x, int axis) { return GraphRegistry::create_lazy_softmax(OpType::Softmax, x, axis); }
Tensor log_softmax(const Tensor &x, int axis) { return GraphRegistry::create_lazy_softmax(OpType::LogSoftmax, x, axis); }

Tensor sum(const Tensor &x, const std::vector<int> &axes, bool keep) { return GraphRegistry::create_lazy_reduction(OpType::Sum, x, axes, keep); }
Tensor mean(const Tensor &x, const std::vector<int> &axes, bool keep) { return GraphRegistry::create_lazy_reduction(OpType::Mean, x, axes, keep); }
Tensor max(const Tensor &x, const std::vector<int> &axes, bool keep) { return GraphRegistry::create_lazy_reduction(OpType::Max, x, axes, keep); }
Tensor min(const Tensor &x, const std::vector<int> &axes, bool keep) { return GraphRegistry::create_lazy_reduction(OpType::Min, x, axes, keep); }
Tensor prod(const Tensor &x, const std::vector<int> &axes, bool keep) { return GraphRegistry::create_lazy_reduction(OpType::Prod, x, axes, keep); }
// Bool results (src/graph/graph_registry.cpp:273-276): the largest / smallest truth value of x != 0
namespace {
// any / all over nothing: false / true wherever the result has elements
Tensor empty_truth(const Tensor &x, const std::vector<int> &axes, bool keep, bool value) {
    const Tensor shape_only = GraphRegistry::create_lazy_reduction(OpType::Sum, x, axes, keep); // (validates the axes, gives the shape)
    Tensor out(shape_only.shape(), DType::Bool, Device::CPU);
    for (size_t i = 0; i < out.size(); ++i) static_cast<uint8_t *>(out.data())[i] = value ? 1 : 0;
    return out.to(Device::GPU);
}
} // namespace
Tensor any(const Tensor &x, const std::vector<int> &axes, bool keep) {
    if (x.size() == 0) return empty_truth(x, axes, keep, false);
    const Tensor truth = x.dtype() == DType::Bool ? x : cast(x, DType::Bool);
    return GraphRegistry::create_lazy_reduction(OpType::Max, truth, axes, keep);
}
Tensor all(const Tensor &x, const std::vector<int> &axes, bool keep) {
    if (x.size() == 0) return empty_truth(x, axes, keep, true);
    const Tensor truth = x.dtype() == DType::Bool ? x : cast(x, DType::Bool);
    return GraphRegistry::create_lazy_reduction(OpType::Min, truth, axes, keep);
}

namespace {
// src/backends/cpu/cpu_operations.cpp:2157-2229 (shape rules) on the device kernel; the input is made contiguous
// first, as the CPU path does (:2161)
Tensor arg_reduce(const Tensor &x, int axis, bool keep_dims, bool want_min) {
    const int nd = static_cast<int>(x.ndim());
    if (nd == 0) throw ShapeError("argmax / argmin of a rank-0 tensor");
    if (axis < 0) axis += nd;
    if (axis < 0 || axis >= nd) throw ShapeError("argmax / argmin: axis out of range");
    if (x.device() != Device::GPU)
        throw RuntimeError("ops::argmax / argmin on CPU tensors: this library is the gfx950 GPU backend only; move the operand with .gpu()");
    if (x.dtype() != DType::Float32 && x.dtype() != DType::Float16 && x.dtype() != DType::BFloat16)
        throw TypeError("argmax / argmin: Float32, Float16 or BFloat16 input");
    const Tensor src = x.ascontiguousarray(); // materialises a lazy input
    const Shape &sh = src.shape();
    size_t outer = 1, inner = 1;
    Shape out_shape;
    for (int d = 0; d < nd; ++d) {
        if (d < axis) outer *= sh[d];
        if (d > axis) inner *= sh[d];
        if (d != axis) out_shape.push_back(sh[d]);
        else if (keep_dims) out_shape.push_back(1);
    }
    if (sh[axis] == 0) throw ShapeError("argmax / argmin along an empty axis");
    Tensor out(out_shape, DType::Int64, Device::GPU);
    // temporary memory (few results over a long axis) comes from this layer's block cache, not from the library
    const char *src_ptr = static_cast<const char *>(src.storage()->raw()) + src.offset();
    const int32_t dt = ::axiom::detail::to_axhip_dtype(src.dtype());
    const size_t ws_bytes = axhip_argreduce_workspace_bytes(src_ptr, dt, static_cast<int64_t>(outer), static_cast<int64_t>(sh[axis]), static_cast<int64_t>(inner));
    const std::unique_ptr<Storage> ws = ws_bytes ? make_storage(ws_bytes, Device::GPU) : nullptr;
    AXHIP_CALL(axhip_argreduce_ws(src_ptr, dt, static_cast<int64_t>(outer), static_cast<int64_t>(sh[axis]), static_cast<int64_t>(inner), want_min ? 1 : 0,
                                  static_cast<int64_t *>(out.storage()->raw()), ws ? ws->raw() : nullptr, ws_bytes, nullptr));
    return out; // asynchronous; .cpu() / item() synchronise
}
} // namespace

Tensor argmax(const Tensor &x, int axis, bool keep_dims) { return arg_reduce(x, axis, keep_dims, false); }
Tensor argmin(const Tensor &x, int axis, bool keep_dims) { return arg_reduce(x, axis, keep_dims, true); }

Tensor layer_norm(const Tensor &x, const Tensor &weight, const Tensor &bias, int axis, float eps) {
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(x.ndim()));
    for (const Tensor *p : {&weight, &bias})
        if (!p->empty() && (p->ndim() != 1 || p->shape()[0] != x.shape()[a]))
            throw ShapeError("layer_norm: weight / bias must have shape [" + std::to_string(x.shape()[a]) + "]");
    return GraphRegistry::create_lazy_layernorm(x, weight, bias, axis, eps);
}

Tensor rms_norm(const Tensor &x, const Tensor &weight, int axis, float eps) {
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(x.ndim()));
    if (!weight.empty() && (weight.ndim() != 1 || weight.shape()[0] != x.shape()[a]))
        throw ShapeError("rms_norm: weight must have shape [" + std::to_string(x.shape()[a]) + "]");
    return GraphRegistry::create_lazy_rmsnorm(x, weight, axis, eps);
}

Tensor matmul(const Tensor &a, const Tensor &b, bool ta, bool tb) { return GraphRegistry::create_lazy_matmul(a, b, ta, tb); }

// src/tensor/operations.cpp:1451-1476
Tensor glu(const Tensor &x, int dim) {
    const int nd = static_cast<int>(x.ndim());
    const int d = dim < 0 ? dim + nd : dim;
    if (d < 0 || d >= nd) throw ValueError("glu: dim " + std::to_string(dim) + " out of range for tensor with " + std::to_string(nd) + " dimensions");
    if (x.shape()[d] % 2 != 0)
        throw ValueError("glu: dimension " + std::to_string(d) + " size (" + std::to_string(x.shape()[d]) + ") must be divisible by 2");
    Shape out = x.shape();
    out[d] /= 2;
    return GraphRegistry::create_lazy_glu(x, d, out);
}

Tensor masked_fill(const Tensor &x, const Tensor &mask, float value) { return GraphRegistry::create_lazy_masked_fill(x, mask, value); }
Tensor masked_fill(const Tensor &x, const Tensor &mask, double value) { return masked_fill(x, mask, static_cast<float>(value)); }

Tensor pad(const Tensor &x, const std::vector<std::pair<size_t, size_t>> &pad_width, const std::string &mode, double value) {
    // src/tensor/operations.cpp:2178-2184 (the reference's GPU path leaves "circular" to the CPU; here it has a kernel)
    const int m = mode == "constant" ? AXHIP_PAD_CONSTANT : mode == "reflect" ? AXHIP_PAD_REFLECT : mode == "replicate" ? AXHIP_PAD_REPLICATE
                  : mode == "circular" ? AXHIP_PAD_CIRCULAR : -1;
    if (m < 0) throw ValueError("pad: mode must be 'constant', 'reflect', 'replicate', or 'circular', got '" + mode + "'");
    if (pad_width.size() != x.ndim()) throw ShapeError("pad: pad_width must have one (before, after) pair per dimension");
    Shape out = x.shape();
    for (size_t d = 0; d < out.size(); ++d) {
        const size_t widest = std::max(pad_width[d].first, pad_width[d].second);
        if (m == AXHIP_PAD_REFLECT && widest > 0 && widest >= x.shape()[d])
            throw ValueError("pad: a reflected pad must be shorter than the dimension it reflects");
        if (m != AXHIP_PAD_CONSTANT && widest > 0 && x.shape()[d] == 0) throw ValueError("pad: nothing to repeat along an empty dimension");
        out[d] += pad_width[d].first + pad_width[d].second;
    }
    return GraphRegistry::create_lazy_pad(x, pad_width, value, out, m);
}

Tensor embedding(const Tensor &weight, const Tensor &indices) {
    if (weight.ndim() != 2) throw ShapeError("embedding: weight must be (vocab_size, embed_dim)");
    if (indices.dtype() != DType::Int64 && indices.dtype() != DType::Int32) throw TypeError("embedding: indices must be Int32 or Int64");
    return GraphRegistry::create_lazy_embedding(weight, indices);
}

Tensor conv1d(const Tensor &input, const Tensor &weight, const Tensor &bias, int stride, int padding, int dilation, int groups) {
    if (groups <= 0) throw ValueError("conv1d: groups must be > 0, got " + std::to_string(groups)); // src/tensor/operations.cpp:2982-3016
    if (stride < 1 || dilation < 1 || padding < 0) throw ValueError("conv1d: stride and dilation must be positive, padding non-negative");
    if (input.ndim() == 2) { // unbatched (C_in, L)
        const Tensor y = conv1d(input.unsqueeze(0), weight, bias, stride, padding, dilation, groups);
        return y.squeeze(0);
    }
    if (input.ndim() != 3 || weight.ndim() != 3) throw ShapeError("conv1d expects input (N, C_in, L) and weight (C_out, C_in / groups, K)");
    if (input.shape()[1] != weight.shape()[1] * static_cast<size_t>(groups))
        throw ShapeError("conv1d: input has " + std::to_string(input.shape()[1]) + " channels, weight expects " + std::to_string(weight.shape()[1]) +
                         " per group times " + std::to_string(groups) + " groups");
    if (weight.shape()[0] % static_cast<size_t>(groups) != 0) throw ShapeError("conv1d: C_out must be divisible by groups");
    if (!bias.empty() && (bias.ndim() != 1 || bias.shape()[0] != weight.shape()[0])) throw ShapeError("conv1d: bias must have shape (C_out)");
    return GraphRegistry::create_lazy_conv1d(input, weight, bias, stride, padding, dilation, groups);
}

Tensor conv1d(const Tensor &input, const Tensor &weight) { return conv1d(input, weight, Tensor(), 1, 0, 1, 1); }

Tensor conv2d(const Tensor &input, const Tensor &weight, const Tensor &bias, std::array<int, 2> stride, std::array<int, 2> padding,
              std::array<int, 2> dilation, int groups) {
    if (groups <= 0) throw ValueError("conv2d: groups must be > 0, got " + std::to_string(groups)); // src/tensor/operations.cpp:3153-3189
    for (int i = 0; i < 2; ++i)
        if (stride[i] < 1 || dilation[i] < 1 || padding[i] < 0) throw ValueError("conv2d: stride and dilation must be positive, padding non-negative");
    if (input.ndim() == 3) return conv2d(input.unsqueeze(0), weight, bias, stride, padding, dilation, groups).squeeze(0); // unbatched (C_in, H, W)
    if (input.ndim() != 4 || weight.ndim() != 4) throw ShapeError("conv2d expects input (N, C_in, H, W) and weight (C_out, C_in / groups, KH, KW)");
    if (input.shape()[1] != weight.shape()[1] * static_cast<size_t>(groups))
        throw ShapeError("conv2d: input has " + std::to_string(input.shape()[1]) + " channels, weight expects " + std::to_string(weight.shape()[1]) +
                         " per group times " + std::to_string(groups) + " groups");
    if (weight.shape()[0] % static_cast<size_t>(groups) != 0) throw ShapeError("conv2d: C_out must be divisible by groups");
    if (!bias.empty() && (bias.ndim() != 1 || bias.shape()[0] != weight.shape()[0])) throw ShapeError("conv2d: bias must have shape (C_out)");
    return GraphRegistry::create_lazy_conv2d(input, weight, bias, stride, padding, dilation, groups);
}
Tensor conv2d(const Tensor &input, const Tensor &weight) { return conv2d(input, weight, Tensor(), {1, 1}, {0, 0}, {1, 1}, 1); }

Tensor batch_norm1d(const Tensor &x, const Tensor &weight, const Tensor &bias, const Tensor &running_mean, const Tensor &running_var, float eps) {
    return GraphRegistry::create_lazy_batchnorm(x, weight, bias, running_mean, running_var, eps);
}

// ---------------------------------------------------------------- attention
namespace {
thread_local std::string tl_sdpa_kernel = "";

// last dimension contiguous, non-negative strides: what axhip_sdpa_fwd addresses directly
Tensor sdpa_operand(const Tensor &t) {
    Tensor g = t.device() == Device::GPU ? t : t.to(Device::GPU);
    const Strides &st = g.strides(); // materialises a lazy operand
    bool ok = st.back() == static_cast<int64_t>(g.itemsize()) || g.shape().back() == 1;
    for (int64_t s : st) ok = ok && s >= 0 && s % static_cast<int64_t>(g.itemsize()) == 0;
    return ok ? g : g.ascontiguousarray();
}

// src/backends/metal/flash_attention_dispatch.mm:125-162: S = Q K^T * scale, masked entries set to -1e9, softmax, P V
Tensor decomposed_sdpa(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor &mask, float scale, bool is_causal) {
    Tensor scores = ops::matmul(q, k, false, true);
    scores = ops::multiply(scores, Tensor::full({1}, scale, Device::GPU).astype(scores.dtype()));
    if (is_causal) {
        const size_t sq = q.shape()[2], skv = k.shape()[2];
        Tensor above = Tensor::zeros({sq, skv}, DType::Bool, Device::CPU);
        uint8_t *a = above.typed_data<uint8_t>();
        for (size_t i = 0; i < sq; ++i)
            for (size_t j = i + 1; j < skv; ++j) a[i * skv + j] = 1;
        scores = ops::masked_fill(scores, above.to(Device::GPU), -1e9f);
    }
    if (!mask.empty()) scores = ops::masked_fill(scores, mask, -1e9f);
    return ops::matmul(ops::softmax(scores, -1), v);
}
} // namespace

const char *last_sdpa_kernel() { return tl_sdpa_kernel.c_str(); }

Tensor scaled_dot_product_attention(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask, float scale, bool is_causal) {
    return detail::sdpa(query, key, value, mask, scale, is_causal, false);
}

// src/tensor/operations.cpp:3979-4044
Tensor detail::sdpa(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask, float scale, bool is_causal, bool out_bshd) {
    if (query.ndim() != 4 || key.ndim() != 4 || value.ndim() != 4)
        throw ShapeError("scaled_dot_product_attention expects 4-D (batch, heads, seq, head_dim) tensors");
    const Shape &qs = query.shape(), &ks = key.shape(), &vs = value.shape();
    if (qs[0] != ks[0] || qs[0] != vs[0]) throw ShapeError("scaled_dot_product_attention: batch sizes differ");
    if (qs[1] != ks[1] || qs[1] != vs[1]) throw ShapeError("scaled_dot_product_attention: head counts differ");
    if (ks[2] != vs[2]) throw ShapeError("scaled_dot_product_attention: key and value sequence lengths differ");
    if (qs[3] != ks[3] || qs[3] != vs[3]) throw ShapeError("scaled_dot_product_attention: head dimensions differ");
    if (query.dtype() != key.dtype() || query.dtype() != value.dtype()) throw TypeError("scaled_dot_product_attention: q, k, v dtypes differ");
    const size_t B = qs[0], H = qs[1], Sq = qs[2], Skv = ks[2], D = qs[3];

    if (query.device() != Device::GPU && key.device() != Device::GPU && value.device() != Device::GPU)
        throw RuntimeError("ops::scaled_dot_product_attention on CPU tensors: this library is the gfx950 GPU backend only; move the operands with .gpu()");
    // Head sizes between the matrix-core kernels' 32 / 64 / 128 are padded with zero dims up to the next one (zeros
    // change neither Q K^T nor the wanted part of P V) once the problem is large enough for three pad passes and an
    // output slice to be small change against the FMA kernel they avoid (two orders of magnitude slower); this is
    // where the reference's decomposed fallback for such sizes (flash_attention_dispatch.mm:180-196) ends up.
    // (16-bit head sizes that are multiples of 8 above 32 need none of this: the kernels take them as they are)
    // 16-bit head sizes between 128 and 256 go to the head_dim-256 kernel the same way.
    const bool half = query.dtype() == DType::Float16 || query.dtype() == DType::BFloat16;
    const bool kernel_takes_it = (half && D <= 256 && D % 8 == 0) || (query.dtype() == DType::Float32 && D <= 128 && D % 4 == 0);
    const bool below_a_kernel = (D > 0 && D < 128 && D != 32 && D != 64) || (half && D > 128 && D < 256);
    if (below_a_kernel && !kernel_takes_it && static_cast<double>(B) * H * Sq * Skv * D >= double(1 << 24) &&
        (query.dtype() == DType::Float32 || half)) {
        const size_t Dp = D < 32 ? 32 : D < 64 ? 64 : D < 128 ? 128 : 256;
        const std::vector<std::pair<size_t, size_t>> widen{{0, 0}, {0, 0}, {0, 0}, {0, Dp - D}};
        auto on_gpu = [](const Tensor &t) { return t.device() == Device::GPU ? t : t.to(Device::GPU); };
        const float sc = scale > 0.0f ? scale : 1.0f / std::sqrt(static_cast<float>(D));
        Tensor wide = detail::sdpa(ops::pad(on_gpu(query), widen), ops::pad(on_gpu(key), widen), ops::pad(on_gpu(value), widen), mask, sc, is_causal, out_bshd);
        return wide.slice({Slice(), Slice(), Slice(), Slice(0, static_cast<int64_t>(D))});
    }
    const Tensor q = sdpa_operand(query), k = sdpa_operand(key), v = sdpa_operand(value);

    AxhipSdpaParams p{};
    p.dtype = ::axiom::detail::to_axhip_dtype(q.dtype());
    p.batch = static_cast<int32_t>(B);
    p.heads = static_cast<int32_t>(H);
    p.seq_q = static_cast<int32_t>(Sq);
    p.seq_kv = static_cast<int32_t>(Skv);
    p.head_dim = static_cast<int32_t>(D);
    p.scale = scale; // <= 0: the library uses 1/sqrt(D) (operations.cpp:4013-4015)
    p.is_causal = is_causal ? 1 : 0;
    const int64_t isz = static_cast<int64_t>(q.itemsize());
    for (int i = 0; i < 3; ++i) {
        p.q_strides[i] = q.strides()[i] / isz;
        p.k_strides[i] = k.strides()[i] / isz;
        p.v_strides[i] = v.strides()[i] / isz;
    }
    // out_bshd: the result is laid out (B, Sq, H, D) in memory and returned as its (B, H, Sq, D) view
    Tensor out = out_bshd ? Tensor(Shape{B, Sq, H, D}, q.dtype(), Device::GPU).transpose({0, 2, 1, 3}) : Tensor(Shape{B, H, Sq, D}, q.dtype(), Device::GPU);
    for (int i = 0; i < 3; ++i) p.o_strides[i] = out.strides()[i] / isz;

    Tensor m;
    const uint8_t *mask_ptr = nullptr;
    if (!mask.empty()) {
        if (mask.dtype() != DType::Bool && mask.dtype() != DType::UInt8) throw TypeError("scaled_dot_product_attention: mask must be Bool");
        const Shape &ms = mask.shape();
        const bool two_d = ms.size() == 2 && ms[0] == Sq && ms[1] == Skv;
        const bool four_d = ms.size() == 4 && ms[2] == Sq && ms[3] == Skv && (ms[0] == B || ms[0] == 1) && (ms[1] == H || ms[1] == 1);
        if (!two_d && !four_d) throw ShapeError("scaled_dot_product_attention: mask must be (Sq, Skv) or (B|1, H|1, Sq, Skv)");
        m = (mask.device() == Device::GPU ? mask : mask.to(Device::GPU)).ascontiguousarray();
        mask_ptr = static_cast<const uint8_t *>(m.storage()->raw()) + m.offset();
        if (four_d) { // size-1 dims broadcast with stride 0
            p.mask_strides[0] = ms[0] == 1 ? 0 : static_cast<int64_t>(ms[1] * Sq * Skv);
            p.mask_strides[1] = ms[1] == 1 ? 0 : static_cast<int64_t>(Sq * Skv);
        }
    }
    auto ptr = [](const Tensor &t) { return static_cast<const char *>(t.storage()->raw()) + t.offset(); };
    tl_sdpa_kernel = axhip_sdpa_kernel_name(&p);
    // Shapes no attention kernel takes (head sizes above 256; 65 536 or more (batch, head) slices on the FMA kernel)
    // are composed from the matrix product, masking and softmax kernels, as the reference composes what its own
    // kernels do not take (src/backends/metal/flash_attention_dispatch.mm:125-162, 180-196).
    // fp32 head sizes between 129 and 256 have the FMA kernel only (a few TFLOP/s): once the problem is large enough to
    // notice, and its score matrix small enough to hold (32 GiB), the composed form on the matrix-core GEMM is two
    // orders of magnitude faster.  (16-bit: 256 has a matrix-core kernel, the sizes below it were padded to it above.)
    const double work = static_cast<double>(B) * H * Sq * Skv * D, score_bytes = static_cast<double>(B) * H * Sq * Skv * static_cast<double>(q.itemsize());
    const bool wide_head = D > 128 && work >= double(1 << 24) && score_bytes <= 32.0 * double(1 << 30);
    if (tl_sdpa_kernel == "invalid" || (tl_sdpa_kernel == "generic" && (B * H >= 65536 || wide_head))) {
        tl_sdpa_kernel = "decomposed";
        Tensor o = decomposed_sdpa(q, k, v, m, scale > 0.0f ? scale : 1.0f / std::sqrt(static_cast<float>(D)), is_causal);
        if (!out_bshd) return o;
        return o.transpose({0, 2, 1, 3}).ascontiguousarray().transpose({0, 2, 1, 3});
    }
    // (a decoding step's partial results live in a block of this layer's cache: the block goes back when this
    // function returns and is handed out again in stream order)
    const size_t ws_bytes = axhip_sdpa_workspace_bytes(&p, mask_ptr != nullptr);
    const std::unique_ptr<Storage> ws = ws_bytes ? make_storage(ws_bytes, Device::GPU) : nullptr;
    AXHIP_CALL(axhip_sdpa_fwd_ws(ptr(q), ptr(k), ptr(v), out.storage()->raw(), mask_ptr, &p, ws ? ws->raw() : nullptr, ws_bytes, nullptr));
    return out; // asynchronous; .cpu() / item() synchronise
}

} // namespace axiom::ops
