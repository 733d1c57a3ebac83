// materialize_gpu_graph: the GPU hook of the lazy graph.  Cuts the DAG under a root
// into launches of libaxhip -- fused row programs, full reductions, GEMMs with epilogue,
// strided gathers -- and caches the resulting plan by graph signature.
//
// Contract (src/graph/graph_registry.cpp:834-850 and the Metal implementation
// src/backends/metal/mpsgraph_graph_compiler.mm:706-944): on return the root holds its
// result (cached_result_, cached_shape_, cached_strides_, is_materialized_), nodes that
// other consumers share were materialised on the way, and the inputs of every
// materialised node lost one reference.
//
// Fusion rule: walking down from a node through inputs that nobody else consumes,
//     [row reduction] <- [elementwise chain] <- [softmax | log-softmax | layer norm | rms norm]
//                     <- [elementwise chain] <- input
// becomes ONE axhip_fused_rows launch; [full reduction] <- [elementwise chain] one
// axhip_fused_full_reduce; [activation] <- [+ residual] <- [+ bias] <- matmul one
// axhip_gemm.  Reshape and transpose are views; a view that a kernel cannot address
// directly is gathered with axhip_strided_copy first.
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <unordered_set>

#include "axiom/error.hpp"
#include "axiom/graph/graph_cache.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/graph/graph_signature.hpp"
#include "hip_call.hpp"

namespace axiom::graph {

namespace {

using ops::OpType;

// ---------------------------------------------------------------- plan types
struct ValueSpec {
    bool is_leaf = false;
    int index = 0; // leaf index or temp index
    Shape shape;
    Strides strides; // bytes
    DType dtype = DType::Float32;
    size_t offset = 0; // bytes past the start of the leaf's data / the temporary (views cut by Slice)
};

struct RowsStep {
    AxhipRowsProgram prog{}; // pointers filled at run time
    int input = -1, output = -1;
    int operand_value[AXHIP_MAX_OPERANDS] = {};
    bool full_reduce = false;
    int workspace = -1; // temp index of the full-reduce scratch
};

struct GemmStep {
    AxhipGemmParams p{};
    int a = -1, b = -1, c = -1, bias = -1, residual = -1;
};

struct CopyStep {
    int src = -1, dst = -1;
    Shape shape;         // iteration space
    Strides src_strides; // bytes; 0 on broadcast dims
};

struct PadStep {
    int src = -1, dst = -1;
    std::vector<int64_t> before, after;
    double value = 0.0;
    int mode = 0;
};

struct MaskedFillStep {
    int src = -1, mask = -1, dst = -1;
    Strides mask_strides; // bytes == elements for the one-byte mask; 0 on broadcast dims
    float value = 0.0f;
};

struct GatherStep {
    int table = -1, indices = -1, dst = -1;
};

struct WhereStep { // dst = cond ? a : b over dst's shape; strides in bytes, 0 on broadcast dims
    int cond = -1, a = -1, b = -1, dst = -1;
    Strides cond_strides, a_strides, b_strides;
};

struct AxisReduceStep { // a reduction, or a softmax, along the middle extent of a contiguous (outer, axis, inner) value
    int src = -1, dst = -1;
    int64_t outer = 1, axis = 1, inner = 1;
    int reduce = 0;  // AXHIP_RED_*; for AXIS_SOFTMAX: 1 = log-softmax
};

struct Step {
    enum Kind { ROWS, GEMM, COPY, PAD, MASKED_FILL, GATHER, AXIS_REDUCE, AXIS_SOFTMAX, WHERE } kind;
    RowsStep rows;
    GemmStep gemm;
    CopyStep copy;
    PadStep pad;
    MaskedFillStep mfill;
    GatherStep gather;
    AxisReduceStep axred;
    WhereStep where;
};

struct Plan {
    std::vector<ValueSpec> values;
    std::vector<size_t> temp_bytes;
    std::vector<Step> steps;
    std::vector<std::pair<int, int>> node_results; // (topological index of a node, value holding its result)
    size_t n_leaves = 0;
    // what the plan was built for, compared on every cache hit: the cache is keyed by a 64-bit hash, and a plan bound
    // to a graph of other extents would launch kernels past the caller's buffers
    std::vector<int64_t> fingerprint;
};

bool is_leaf(const GraphNode *n, const GraphNode *root) { return n->is_constant || (n->is_materialized_ && n != root); }

bool is_unary_ew(OpType op) {
    switch (op) {
    case OpType::Negate: case OpType::Abs: case OpType::Sqrt: case OpType::Exp: case OpType::Log: case OpType::Reciprocal:
    case OpType::Square: case OpType::ReLU: case OpType::SiLU: case OpType::Sigmoid: case OpType::Tanh: case OpType::GELU:
    case OpType::Sin: case OpType::Cos: case OpType::Tan: case OpType::Erf: case OpType::Sign: case OpType::Floor: case OpType::Ceil:
    case OpType::Trunc: case OpType::Round: case OpType::Cbrt: case OpType::IsNaN: case OpType::IsInf: case OpType::IsFinite:
    case OpType::LogicalNot: case OpType::LeakyReLU: case OpType::Cast:
        return true;
    default: return false;
    }
}
bool is_binary_ew(OpType op) {
    switch (op) {
    case OpType::Add: case OpType::Subtract: case OpType::Multiply: case OpType::Divide: case OpType::Maximum: case OpType::Minimum:
    case OpType::Power: case OpType::Modulo: case OpType::Atan2: case OpType::Hypot: case OpType::Equal: case OpType::NotEqual:
    case OpType::Less: case OpType::LessEqual: case OpType::Greater: case OpType::GreaterEqual: case OpType::LogicalAnd:
    case OpType::LogicalOr: case OpType::LogicalXor:
        return true;
    default: return false;
    }
}
bool is_elementwise(OpType op) { return is_unary_ew(op) || is_binary_ew(op); }
bool is_row_op(OpType op) { return op == OpType::Softmax || op == OpType::LogSoftmax || op == OpType::LayerNorm || op == OpType::RMSNorm; }
bool is_reduction(OpType op) { return op == OpType::Sum || op == OpType::Mean || op == OpType::Max || op == OpType::Min || op == OpType::Prod; }
int reduce_code(OpType op) {
    return op == OpType::Sum ? AXHIP_RED_SUM : op == OpType::Mean ? AXHIP_RED_MEAN : op == OpType::Max ? AXHIP_RED_MAX : op == OpType::Min ? AXHIP_RED_MIN : AXHIP_RED_PROD;
}
// a Cast that loses precision in the middle of a chain would need a rounding step of its own: such a node ends the
// chain below it (on top of a chain it is the kernel's output type).  Widening casts and casts from Bool change no
// value; a cast to Bool is "!= 0".
bool narrowing_cast(const GraphNode *n) {
    if (n->op_type != OpType::Cast) return false;
    const DType from = n->inputs[0]->output_dtype, to = n->output_dtype;
    if (to == DType::Bool || from == DType::Bool || from == to) return false;
    return !(to == DType::Float32);
}

int unary_code(OpType op) {
    switch (op) {
    case OpType::Negate: return AXHIP_OP_NEG;
    case OpType::Abs: return AXHIP_OP_ABS;
    case OpType::Sqrt: return AXHIP_OP_SQRT;
    case OpType::Exp: return AXHIP_OP_EXP;
    case OpType::Log: return AXHIP_OP_LOG;
    case OpType::Reciprocal: return AXHIP_OP_RECIP;
    case OpType::Square: return AXHIP_OP_SQUARE;
    case OpType::ReLU: return AXHIP_OP_RELU;
    case OpType::SiLU: return AXHIP_OP_SILU;
    case OpType::Sigmoid: return AXHIP_OP_SIGMOID;
    case OpType::Tanh: return AXHIP_OP_TANH;
    case OpType::GELU: return AXHIP_OP_GELU;
    case OpType::Sin: return AXHIP_OP_SIN;
    case OpType::Cos: return AXHIP_OP_COS;
    case OpType::Tan: return AXHIP_OP_TAN;
    case OpType::Erf: return AXHIP_OP_ERF;
    case OpType::Sign: return AXHIP_OP_SIGN;
    case OpType::Floor: return AXHIP_OP_FLOOR;
    case OpType::Ceil: return AXHIP_OP_CEIL;
    case OpType::Trunc: return AXHIP_OP_TRUNC;
    case OpType::Round: return AXHIP_OP_ROUND;
    case OpType::Cbrt: return AXHIP_OP_CBRT;
    case OpType::IsNaN: return AXHIP_OP_ISNAN;
    case OpType::IsInf: return AXHIP_OP_ISINF;
    case OpType::IsFinite: return AXHIP_OP_ISFINITE;
    case OpType::LogicalNot: return AXHIP_OP_NOT;
    default: return 0;
    }
}
// chain_is_rhs: the running value is the op's second operand
int binary_code(OpType op, bool chain_is_rhs) {
    switch (op) {
    case OpType::Add: return AXHIP_OP_ADD;
    case OpType::Multiply: return AXHIP_OP_MUL;
    case OpType::Maximum: return AXHIP_OP_MAX;
    case OpType::Minimum: return AXHIP_OP_MIN;
    case OpType::Subtract: return chain_is_rhs ? AXHIP_OP_RSUB : AXHIP_OP_SUB;
    case OpType::Divide: return chain_is_rhs ? AXHIP_OP_RDIV : AXHIP_OP_DIV;
    case OpType::Power: return chain_is_rhs ? AXHIP_OP_RPOW : AXHIP_OP_POW;
    case OpType::Modulo: return chain_is_rhs ? AXHIP_OP_RMOD : AXHIP_OP_MOD;
    case OpType::Atan2: return chain_is_rhs ? AXHIP_OP_RATAN2 : AXHIP_OP_ATAN2;
    case OpType::Hypot: return AXHIP_OP_HYPOT;
    case OpType::Equal: return AXHIP_OP_EQ;
    case OpType::NotEqual: return AXHIP_OP_NE;
    case OpType::Less: return chain_is_rhs ? AXHIP_OP_GT : AXHIP_OP_LT; // a < v  <=>  v > a
    case OpType::LessEqual: return chain_is_rhs ? AXHIP_OP_GE : AXHIP_OP_LE;
    case OpType::Greater: return chain_is_rhs ? AXHIP_OP_LT : AXHIP_OP_GT;
    case OpType::GreaterEqual: return chain_is_rhs ? AXHIP_OP_LE : AXHIP_OP_GE;
    case OpType::LogicalAnd: return AXHIP_OP_AND;
    case OpType::LogicalOr: return AXHIP_OP_OR;
    case OpType::LogicalXor: return AXHIP_OP_XOR;
    default: return 0;
    }
}

// Interior nodes whose result must exist on its own after the graph has run: those with more than one
// consumer in the graph, and those a live Tensor handle still refers to (the handle may feed a later graph,
// e.g. the residual stream kept across an attention call) when recomputing them would repeat a GEMM.  Cheap
// elementwise / row work held by a handle stays fused and is recomputed if it is ever asked for, which is
// what keeps softmax(...).sum() one kernel when the softmax has a name in user code.
using SharedSet = std::unordered_set<const GraphNode *>;
SharedSet shared_nodes(const GraphNode *root, const std::vector<const GraphNode *> &topo) {
    std::unordered_map<const GraphNode *, long> holders; // shared_ptr owners: graph edges + Tensor handles
    std::unordered_map<const GraphNode *, bool> heavy;   // a MatMul at or below the node, above the leaves
    SharedSet out;
    for (const GraphNode *n : topo) { // inputs precede their consumers
        if (is_leaf(n, root)) continue;
        bool h = n->op_type == OpType::MatMul;
        for (const auto &in : n->inputs) {
            holders[in.get()] = in.use_count();
            auto it = heavy.find(in.get());
            h = h || (it != heavy.end() && it->second);
        }
        heavy[n] = h;
    }
    for (const GraphNode *n : topo) {
        if (is_leaf(n, root) || n == root) continue;
        const long refs = static_cast<long>(n->ref_count.load());
        if (refs > 1 || (heavy[n] && holders[n] > refs)) out.insert(n);
    }
    return out;
}

// ------------------------------------------------------------------ builder
class PlanBuilder {
  public:
    PlanBuilder(const GraphNode *root, const std::vector<const GraphNode *> &topo, const SharedSet &shared) : root_(root), shared_(shared) {
        for (size_t i = 0; i < topo.size(); ++i) {
            topo_index_[topo[i]] = static_cast<int>(i);
            if (is_leaf(topo[i], root)) {
                ValueSpec v;
                v.is_leaf = true;
                v.index = static_cast<int>(plan_.n_leaves++);
                const GraphNode *n = topo[i];
                v.shape = n->is_constant ? n->output_shape : n->cached_shape_;
                v.strides = n->is_constant ? n->constant_strides : n->cached_strides_;
                v.dtype = n->output_dtype;
                memo_[n] = add_value(v);
            }
        }
    }

    Plan build() {
        eval(root_);
        return std::move(plan_);
    }

  private:
    int add_value(const ValueSpec &v) {
        plan_.values.push_back(v);
        return static_cast<int>(plan_.values.size()) - 1;
    }
    int new_temp(const Shape &shape, DType dt) {
        ValueSpec v;
        v.index = static_cast<int>(plan_.temp_bytes.size());
        v.shape = shape;
        v.dtype = dt;
        v.strides = ShapeUtils::contiguous_strides(shape, dtype_size(dt));
        plan_.temp_bytes.push_back(std::max<size_t>(ShapeUtils::size(shape) * dtype_size(dt), 16));
        return add_value(v);
    }
    const ValueSpec &val(int v) const { return plan_.values[v]; }
    bool contiguous(int v) const { return ShapeUtils::is_contiguous(val(v).shape, val(v).strides, dtype_size(val(v).dtype)); }

    // a contiguous value with the same contents (gathered if necessary), optionally broadcast to `to`
    int make_contiguous(int v, const Shape *to = nullptr) {
        const Shape target = to ? *to : val(v).shape;
        if (target == val(v).shape && contiguous(v)) return v;
        detail::to_axhip_dtype_or_bool(val(v).dtype); // only kernel dtypes can be gathered on the device
        const ValueSpec src = val(v);
        const int out = new_temp(target, src.dtype);
        Step s{};
        s.kind = Step::COPY;
        s.copy.src = v;
        s.copy.dst = out;
        s.copy.shape = target;
        s.copy.src_strides.assign(target.size(), 0);
        const size_t lead = target.size() - src.shape.size();
        for (size_t i = 0; i < src.shape.size(); ++i) s.copy.src_strides[lead + i] = src.shape[i] == 1 ? 0 : src.strides[i];
        if (target.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU gather of more than 8 dimensions");
        for (int64_t st : s.copy.src_strides)
            if (st < 0) throw RuntimeError::not_implemented("negative strides (flipped views)");
        plan_.steps.push_back(s);
        return out;
    }

    // A reduction whose axes are one run of neighbours that stops short of the last axis: (outer, axis, inner) of the
    // input, with more than one kept element behind the run.  False for everything the row kernels take (the last
    // axis, all axes, a single kept element).
    static bool inner_axis_run(const GraphNode *n, int64_t *outer, int64_t *axis, int64_t *inner) {
        const auto &rp = get_params<ReductionParams>(n->params);
        const Shape &F = n->inputs[0]->output_shape;
        const int nd = static_cast<int>(F.size());
        if (rp.axes.empty() || nd < 2) return false;
        std::vector<bool> red(static_cast<size_t>(nd), false);
        for (int a : rp.axes) red[static_cast<size_t>(ShapeUtils::normalize_axis(a, nd))] = true;
        int first = -1, last = -1, count = 0;
        for (int i = 0; i < nd; ++i)
            if (red[static_cast<size_t>(i)]) {
                if (first < 0) first = i;
                last = i;
                ++count;
            }
        if (count != last - first + 1 || last == nd - 1) return false;
        int64_t o = 1, a = 1, in = 1;
        for (int i = 0; i < nd; ++i) (i < first ? o : i <= last ? a : in) *= static_cast<int64_t>(F[static_cast<size_t>(i)]);
        if (in <= 1 || a == 0 || o * in <= 1) return false;
        if (outer) *outer = o;
        if (axis) *axis = a;
        if (inner) *inner = in;
        return true;
    }

    // the row kernels take softmax and the norms over the last axis
    static bool row_axis_is_last(const GraphNode *n) {
        const int nd = static_cast<int>(n->output_shape.size());
        const int axis = n->op_type == OpType::Softmax || n->op_type == OpType::LogSoftmax ? get_params<ActivationParams>(n->params).axis
                                                                                           : get_params<NormParams>(n->params).axis;
        return nd == 0 || ShapeUtils::normalize_axis(axis, nd) == nd - 1;
    }

    // is the input of this Cast node a view (of a leaf or of a computed value) that is not contiguous
    bool strided_view_below(const GraphNode *n) {
        const GraphNode *in = n->inputs[0].get();
        const bool view = is_leaf(in, root_) || in->op_type == OpType::Transpose || in->op_type == OpType::Slice || in->op_type == OpType::Reshape ||
                          memo_.count(in) > 0;
        return view && !contiguous(eval(in));
    }

    bool consumable(const GraphNode *c, const GraphNode *entry) const {
        return !is_leaf(c, root_) && (c == entry || !shared_.count(c)) && !memo_.count(c);
    }

    int eval(const GraphNode *n) {
        auto it = memo_.find(n);
        if (it != memo_.end()) return it->second;
        const size_t arity = is_binary_ew(n->op_type) || n->op_type == OpType::MatMul ? 2 : 1;
        if (n->inputs.size() < arity) throw RuntimeError(std::string("malformed graph node '") + ops::op_name(n->op_type) + "': missing inputs");
        int v;
        const OpType op = n->op_type;
        if (op == OpType::Reshape) {
            const int in = make_contiguous(eval(n->inputs[0].get()));
            ValueSpec s = val(in);
            s.shape = n->output_shape;
            s.strides = ShapeUtils::contiguous_strides(s.shape, dtype_size(s.dtype));
            v = add_value(s);
        } else if (op == OpType::Transpose) {
            const int in = eval(n->inputs[0].get());
            const auto &axes = get_params<TransposeParams>(n->params).axes;
            ValueSpec s = val(in);
            for (size_t i = 0; i < axes.size(); ++i) {
                s.shape[i] = val(in).shape[axes[i]];
                s.strides[i] = val(in).strides[axes[i]];
            }
            v = add_value(s);
        } else if (op == OpType::Slice) {
            const int in = eval(n->inputs[0].get());
            const auto &sp = get_params<SliceParams>(n->params);
            ValueSpec s = val(in);
            for (size_t d = 0; d < s.shape.size(); ++d) {
                s.offset += static_cast<size_t>(sp.starts[d] * val(in).strides[d]);
                s.strides[d] = val(in).strides[d] * sp.steps[d];
            }
            s.shape = n->output_shape;
            v = add_value(s);
        } else if (op == OpType::Unfold1D) {
            // (N, C, L) -> windows (N, L_out, C, K): element (n, l, c, k) is input (n, c, l * stride + k * dilation)
            const int in = eval(n->inputs[0].get());
            const auto &up = get_params<UnfoldParams>(n->params);
            ValueSpec s = val(in);
            const Strides is = val(in).strides;
            s.shape = n->output_shape;
            s.strides = {is[0], is[2] * up.stride, is[1], is[2] * up.dilation};
            if (up.groups > 1) s.strides.insert(s.strides.begin(), is[1] * static_cast<int64_t>(n->output_shape[3])); // (G, N, L_out, C / G, K)
            v = add_value(s);
        } else if (op == OpType::Unfold2D) {
            // (N, C, H, W) -> windows (N, H_out, W_out, C, KH, KW): element (n, i, j, c, a, b) is input (n, c, i sh + a dh, j sw + b dw)
            const int in = eval(n->inputs[0].get());
            const auto &up = get_params<UnfoldParams>(n->params);
            ValueSpec s = val(in);
            const Strides is = val(in).strides;
            s.shape = n->output_shape;
            s.strides = {is[0], is[2] * up.stride_h, is[3] * up.stride, is[1], is[2] * up.dilation_h, is[3] * up.dilation};
            if (up.groups > 1) s.strides.insert(s.strides.begin(), is[1] * static_cast<int64_t>(n->output_shape[4])); // (G, N, H_out, W_out, C / G, KH, KW)
            v = add_value(s);
        } else if (op == OpType::Pad) {
            const int in = eval(n->inputs[0].get());
            detail::to_axhip_dtype(val(in).dtype);
            const auto &pp = get_params<PadParams>(n->params);
            if (val(in).shape.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU pad of more than 8 dimensions");
            Step st{};
            st.kind = Step::PAD;
            st.pad.src = in;
            st.pad.dst = v = new_temp(n->output_shape, n->output_dtype);
            for (const auto &w : pp.pad_widths) {
                st.pad.before.push_back(static_cast<int64_t>(w.first));
                st.pad.after.push_back(static_cast<int64_t>(w.second));
            }
            st.pad.value = pp.value;
            st.pad.mode = pp.mode;
            plan_.steps.push_back(st);
        } else if (op == OpType::MaskedFill) {
            if (n->inputs.size() < 2) throw RuntimeError("malformed graph node 'masked_fill': missing inputs");
            const int in = eval(n->inputs[0].get()), mk = eval(n->inputs[1].get());
            detail::to_axhip_dtype(val(in).dtype);
            const Shape F = val(in).shape, M = val(mk).shape; // copies: new_temp() below grows the value table
            const Strides mask_strides = val(mk).strides;
            if (F.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU masked_fill of more than 8 dimensions");
            Step st{};
            st.kind = Step::MASKED_FILL;
            st.mfill.src = in;
            st.mfill.mask = mk;
            st.mfill.dst = v = new_temp(F, n->output_dtype);
            st.mfill.value = get_params<MaskedFillParams>(n->params).value;
            st.mfill.mask_strides.assign(F.size(), 0);
            const size_t lead = F.size() - M.size();
            for (size_t i = 0; i < M.size(); ++i) st.mfill.mask_strides[lead + i] = M[i] == 1 ? 0 : mask_strides[i];
            plan_.steps.push_back(st);
        } else if (op == OpType::Where) {
            if (n->inputs.size() < 3) throw RuntimeError("malformed graph node 'where': missing inputs");
            const int c = eval(n->inputs[0].get()), a = eval(n->inputs[1].get()), b = eval(n->inputs[2].get());
            const Shape F = n->output_shape;
            if (F.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU where of more than 8 dimensions");
            Step st{};
            st.kind = Step::WHERE;
            st.where.cond = c;
            st.where.a = a;
            st.where.b = b;
            auto broadcast_strides = [&](int v) {
                detail::to_axhip_dtype_or_bool(val(v).dtype);
                const Shape S = val(v).shape;
                const Strides in = val(v).strides;
                Strides out(F.size(), 0);
                const size_t lead = F.size() - S.size();
                for (size_t i = 0; i < S.size(); ++i) {
                    if (in[i] < 0) throw RuntimeError::not_implemented("negative strides (flipped views)");
                    out[lead + i] = S[i] == 1 ? 0 : in[i];
                }
                return out;
            };
            st.where.cond_strides = broadcast_strides(c);
            st.where.a_strides = broadcast_strides(a);
            st.where.b_strides = broadcast_strides(b);
            st.where.dst = v = new_temp(F, n->output_dtype);
            detail::to_axhip_dtype_or_bool(n->output_dtype);
            plan_.steps.push_back(st);
        } else if (op == OpType::Gather) { // embedding rows
            if (n->inputs.size() < 2) throw RuntimeError("malformed graph node 'embedding': missing inputs");
            const int table = make_contiguous(eval(n->inputs[0].get())), idx = eval(n->inputs[1].get());
            if (!contiguous(idx)) throw RuntimeError::not_implemented("embedding with non-contiguous indices on the GPU");
            Step st{};
            st.kind = Step::GATHER;
            st.gather.table = table;
            st.gather.indices = idx;
            st.gather.dst = v = new_temp(n->output_shape, n->output_dtype);
            plan_.steps.push_back(st);
        } else if (op == OpType::MatMul) {
            v = emit_gemm(n, {}, -1, -1, 0);
        } else if (is_reduction(op) && inner_axis_run(n, nullptr, nullptr, nullptr)) {
            // one run of neighbouring axes that ends before the last one: reduced where the data lie, no transposing copy
            int64_t outer, axis, inner;
            inner_axis_run(n, &outer, &axis, &inner);
            Step st{};
            st.kind = Step::AXIS_REDUCE;
            st.axred.src = make_contiguous(eval(n->inputs[0].get()));
            st.axred.outer = outer;
            st.axred.axis = axis;
            st.axred.inner = inner;
            st.axred.reduce = reduce_code(op);
            detail::to_axhip_dtype_or_bool(val(st.axred.src).dtype);
            st.axred.dst = v = new_temp(n->output_shape, n->output_dtype);
            plan_.steps.push_back(st);
        } else if ((op == OpType::Softmax || op == OpType::LogSoftmax) && !row_axis_is_last(n)) {
            // softmax over an axis other than the last: where the data lie, no transposing copies
            const Shape &F = n->output_shape;
            const int ax = ShapeUtils::normalize_axis(get_params<ActivationParams>(n->params).axis, static_cast<int>(F.size()));
            Step st{};
            st.kind = Step::AXIS_SOFTMAX;
            st.axred.src = make_contiguous(eval(n->inputs[0].get()));
            for (int i = 0; i < static_cast<int>(F.size()); ++i)
                (i < ax ? st.axred.outer : i == ax ? st.axred.axis : st.axred.inner) *= static_cast<int64_t>(F[static_cast<size_t>(i)]);
            st.axred.reduce = op == OpType::LogSoftmax ? 1 : 0;
            detail::to_axhip_dtype(val(st.axred.src).dtype);
            st.axred.dst = v = new_temp(F, n->output_dtype);
            plan_.steps.push_back(st);
        } else if (op == OpType::Cast && strided_view_below(n)) {
            // a cast of a strided view: the gather converts on its way, one pass instead of a gather and a cast
            const int in = eval(n->inputs[0].get());
            const ValueSpec src = val(in);
            detail::to_axhip_dtype_or_bool(src.dtype);
            detail::to_axhip_dtype_or_bool(n->output_dtype);
            if (src.shape.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU gather of more than 8 dimensions");
            Step st{};
            st.kind = Step::COPY;
            st.copy.src = in;
            st.copy.dst = v = new_temp(src.shape, n->output_dtype);
            st.copy.shape = src.shape;
            st.copy.src_strides = src.strides;
            for (size_t i = 0; i < src.shape.size(); ++i)
                if (src.shape[i] == 1) st.copy.src_strides[i] = 0;
            for (int64_t sd : st.copy.src_strides)
                if (sd < 0) throw RuntimeError::not_implemented("negative strides (flipped views)");
            plan_.steps.push_back(st);
        } else if (is_elementwise(op) || is_row_op(op) || is_reduction(op)) {
            v = emit_rows(n);
        } else {
            throw RuntimeError::not_implemented(std::string("GPU lazy graph node '") + ops::op_name(op) + "'");
        }
        memo_[n] = v;
        if (n == root_ || shared_.count(n)) plan_.node_results.emplace_back(topo_index_.at(n), v);
        return v;
    }

    struct ChainItem {
        const GraphNode *node;
        int primary; // input index the chain continues through
    };

    // Collects elementwise nodes downwards from `c` while each is consumable and keeps the full shape F.
    void collect(const GraphNode *&c, const GraphNode *entry, const Shape &F, std::vector<ChainItem> &list, size_t limit, size_t &operands) {
        while (consumable(c, entry) && is_elementwise(c->op_type) && c->output_shape == F && list.size() < limit) {
            if (!list.empty() && narrowing_cast(c)) break; // rounds in mid-chain: a kernel of its own below this one
            int primary = 0;
            if (is_binary_ew(c->op_type)) {
                if (c->inputs.size() < 2) throw RuntimeError(std::string("malformed graph node '") + ops::op_name(c->op_type) + "': missing inputs");
                const GraphNode *l = c->inputs[0].get(), *r = c->inputs[1].get();
                const bool lf = l->output_shape == F, rf = r->output_shape == F;
                if (!lf && !rf) break; // both operands broadcast: evaluated on its own (see emit_rows)
                // continue through the operand that can still be fused; a leaf, a shared node or one that
                // already has a value is the better memory operand
                if (lf && rf) primary = (!consumable(l, nullptr) && consumable(r, nullptr)) ? 1 : 0;
                else primary = lf ? 0 : 1;
                if (operands + 1 > AXHIP_MAX_OPERANDS - 2) break; // keep room for norm weight / bias
                ++operands;
            }
            list.push_back({c, primary});
            c = c->inputs[primary].get();
        }
    }

    // classifies / prepares the memory operand of a binary op against the full shape F = [rows..., cols]
    void add_operand(RowsStep &rs, AxhipChainOp &cop, const GraphNode *operand, const Shape &F, bool chain_is_rhs, OpType op) {
        int v = eval(operand);
        const Shape S = val(v).shape;
        const size_t numel = ShapeUtils::size(S), cols = F.empty() ? 1 : F.back();
        int kind;
        Shape stripped = S;
        while (stripped.size() > 1 && stripped.front() == 1) stripped.erase(stripped.begin());
        bool colvec = S.size() == F.size() && !S.empty() && S.back() == 1 && F.back() != 1;
        for (size_t i = 0; colvec && i + 1 < S.size(); ++i) colvec = S[i] == F[i];
        Shape f_stripped = F;
        while (f_stripped.size() > 1 && f_stripped.front() == 1) f_stripped.erase(f_stripped.begin());
        if (numel == 1) kind = AXHIP_BK_SCALAR;
        else if (S == F || stripped == f_stripped) kind = AXHIP_BK_FULL; // leading unit dimensions change nothing in memory
        else if (stripped.size() == 1 && stripped[0] == cols) kind = AXHIP_BK_ROWVEC;
        else if (colvec) kind = AXHIP_BK_COLVEC;
        else {
            v = make_contiguous(v, &F); // general broadcast: expand once
            kind = AXHIP_BK_FULL;
        }
        v = make_contiguous(v);
        const int slot = rs.prog.n_operands++;
        rs.prog.operands[slot].dtype = detail::to_axhip_dtype_or_bool(val(v).dtype);
        rs.prog.operands[slot].kind = kind;
        rs.operand_value[slot] = v;
        cop.op = binary_code(op, chain_is_rhs);
        cop.operand = slot;
        cop.imm = 0.0f;
        cop.imm_kind = 0;
    }

    void fill_chain(RowsStep &rs, const std::vector<ChainItem> &bottom_up, AxhipChainOp *dst, int32_t &count, const Shape &F) {
        for (const ChainItem &it : bottom_up) {
            AxhipChainOp &cop = dst[count++];
            if (it.node->op_type == OpType::LeakyReLU) { // the slope rides along as an immediate operand
                cop.op = AXHIP_OP_LEAKY_RELU;
                cop.operand = -1;
                cop.imm = get_params<ActivationParams>(it.node->params).alpha;
                cop.imm_kind = AXHIP_BK_IMM;
            } else if (it.node->op_type == OpType::Cast) {
                if (it.node->output_dtype == DType::Bool && it.node->inputs[0]->output_dtype != DType::Bool) {
                    cop.op = AXHIP_OP_NE; // a truth value: != 0
                    cop.operand = -1;
                    cop.imm = 0.0f;
                    cop.imm_kind = AXHIP_BK_IMM;
                } else {
                    --count; // no arithmetic: the kernel converts on load and on store
                }
            } else if (is_unary_ew(it.node->op_type)) {
                cop.op = unary_code(it.node->op_type);
                cop.operand = -1;
                cop.imm = 0.0f;
                cop.imm_kind = 0;
            } else {
                add_operand(rs, cop, it.node->inputs[1 - it.primary].get(), F, it.primary == 1, it.node->op_type);
            }
        }
    }

    int emit_rows(const GraphNode *n) {
        RowsStep rs;
        rs.prog.norm_weight = rs.prog.norm_bias = -1;
        const GraphNode *cur = n;
        const GraphNode *entry = n;
        Shape F = n->output_shape;

        if (is_reduction(n->op_type)) {
            const auto &rp = get_params<ReductionParams>(n->params);
            const GraphNode *in = n->inputs[0].get();
            F = in->output_shape;
            const int nd = static_cast<int>(F.size());
            std::vector<bool> red(nd, rp.axes.empty());
            for (int a : rp.axes) red[ShapeUtils::normalize_axis(a, nd)] = true;
            size_t n_red = 0, kept_elems = 1;
            for (int i = 0; i < nd; ++i) {
                n_red += red[i];
                if (!red[i]) kept_elems *= F[i];
            }
            const bool all = n_red == static_cast<size_t>(nd) || kept_elems == 1;
            const bool last_only = !all && n_red == 1 && red[nd - 1];
            if (!all && !last_only) throw RuntimeError::not_implemented("GPU reduction over axes other than the last one (or all)");
            rs.full_reduce = all;
            rs.prog.reduce = reduce_code(n->op_type);
            cur = in;
            entry = nullptr; // below the reduction only unshared nodes fuse
        }

        size_t operands = 0;
        int gemm_input = -1; // value of a GEMM that absorbed the pre chain
        std::vector<ChainItem> upper, lower;
        collect(cur, entry, F, upper, AXHIP_MAX_CHAIN, operands);
        const GraphNode *rowop = nullptr;
        if (!rs.full_reduce && consumable(cur, entry) && is_row_op(cur->op_type) && cur->output_shape == F &&
            (row_axis_is_last(cur) || (cur->op_type != OpType::Softmax && cur->op_type != OpType::LogSoftmax))) { // (a softmax over another axis is a step of its own)
            const int axis = cur->op_type == OpType::Softmax || cur->op_type == OpType::LogSoftmax ? get_params<ActivationParams>(cur->params).axis
                                                                                                  : get_params<NormParams>(cur->params).axis;
            if (ShapeUtils::normalize_axis(axis, static_cast<int>(F.size())) != static_cast<int>(F.size()) - 1)
                throw RuntimeError::not_implemented("GPU softmax / norm over an axis other than the last one");
            rowop = cur;
            cur = cur->inputs[0].get();
            collect(cur, nullptr, F, lower, AXHIP_MAX_CHAIN, operands);
            // bias / residual / activation directly above a matmul ride in the GEMM epilogue, and the
            // row kernel reads the finished product (Linear -> + x -> LayerNorm is GEMM + one row kernel)
            if (!lower.empty() && consumable(cur, nullptr) && cur->op_type == OpType::MatMul) {
                const int g = try_gemm_epilogue(lower.front().node->output_dtype, F, cur, lower, F);
                if (g >= 0) {
                    lower.clear();
                    gemm_input = g;
                }
            }
        } else if (upper.empty() && !is_reduction(n->op_type)) {
            // an elementwise node whose two operands are both broadcast: expand the left one and chain through it
            if (!is_binary_ew(n->op_type)) throw RuntimeError::not_implemented(std::string("GPU lazy graph node '") + ops::op_name(n->op_type) + "'");
            upper.push_back({n, 0});
            cur = n->inputs[0].get();
        }

        // MatMul feeding a short epilogue chain: one GEMM launch
        if (!rowop && rs.prog.reduce == AXHIP_RED_NONE && consumable(cur, entry) && cur->op_type == OpType::MatMul && !upper.empty()) {
            const int g = try_gemm_epilogue(n->output_dtype, n->output_shape, cur, upper, F);
            if (g >= 0) return g;
        }

        // the pre chain runs bottom-up: reverse the collected (top-down) lists
        std::reverse(upper.begin(), upper.end());
        std::reverse(lower.begin(), lower.end());
        int in_v = gemm_input >= 0 ? gemm_input : eval(cur);
        if (val(in_v).shape != F) in_v = make_contiguous(in_v, &F);
        in_v = make_contiguous(in_v);
        rs.input = in_v;
        rs.prog.input_dtype = detail::to_axhip_dtype_or_bool(val(in_v).dtype);
        rs.prog.cols = F.empty() ? 1 : static_cast<int64_t>(F.back());
        rs.prog.rows = static_cast<int64_t>(ShapeUtils::size(F)) / std::max<int64_t>(rs.prog.cols, 1);
        if (ShapeUtils::size(F) == 0) rs.prog.rows = 0;

        if (rowop) {
            fill_chain(rs, lower, rs.prog.pre, rs.prog.n_pre, F);
            switch (rowop->op_type) {
            case OpType::Softmax: rs.prog.row_op = AXHIP_ROWOP_SOFTMAX; break;
            case OpType::LogSoftmax: rs.prog.row_op = AXHIP_ROWOP_LOGSOFTMAX; break;
            case OpType::LayerNorm: rs.prog.row_op = AXHIP_ROWOP_LAYERNORM; break;
            default: rs.prog.row_op = AXHIP_ROWOP_RMSNORM; break;
            }
            if (rowop->op_type == OpType::LayerNorm || rowop->op_type == OpType::RMSNorm) {
                rs.prog.eps = get_params<NormParams>(rowop->params).eps;
                for (size_t i = 1; i < rowop->inputs.size(); ++i) {
                    const int wv = make_contiguous(eval(rowop->inputs[i].get()));
                    const int slot = rs.prog.n_operands++;
                    rs.prog.operands[slot].dtype = detail::to_axhip_dtype(val(wv).dtype);
                    rs.prog.operands[slot].kind = AXHIP_BK_ROWVEC;
                    rs.operand_value[slot] = wv;
                    (i == 1 ? rs.prog.norm_weight : rs.prog.norm_bias) = slot;
                }
            }
            fill_chain(rs, upper, rs.prog.post, rs.prog.n_post, F);
        } else {
            fill_chain(rs, upper, rs.prog.pre, rs.prog.n_pre, F);
        }

        rs.output = new_temp(n->output_shape, n->output_dtype);
        rs.prog.output_dtype = detail::to_axhip_dtype_or_bool(n->output_dtype);
        if (rs.full_reduce) {
            rs.workspace = static_cast<int>(plan_.temp_bytes.size());
            plan_.temp_bytes.push_back(axhip_full_reduce_workspace_bytes());
        }
        Step s{};
        s.kind = Step::ROWS;
        s.rows = rs;
        plan_.steps.push_back(s);
        return rs.output;
    }

    // [activation] <- [+ residual FULL] <- [+ bias ROWVEC] <- matmul, all in the GEMM's dtype
    int try_gemm_epilogue(DType out_dtype, const Shape &out_shape, const GraphNode *mm, const std::vector<ChainItem> &top_down, const Shape &F) {
        std::vector<ChainItem> ops(top_down.rbegin(), top_down.rend()); // bottom-up
        size_t i = 0;
        const GraphNode *bias = nullptr, *residual = nullptr;
        int act = 0;
        const size_t N = F.back();
        auto other = [](const ChainItem &c) { return c.node->inputs[1 - c.primary].get(); };
        if (i < ops.size() && ops[i].node->op_type == OpType::Add) {
            const Shape &s = other(ops[i])->output_shape;
            Shape stripped = s;
            while (stripped.size() > 1 && stripped.front() == 1) stripped.erase(stripped.begin());
            if (stripped.size() == 1 && stripped[0] == N && other(ops[i])->output_dtype == mm->output_dtype) bias = other(ops[i++]);
        }
        if (i < ops.size() && ops[i].node->op_type == OpType::Add && other(ops[i])->output_shape == F && other(ops[i])->output_dtype == mm->output_dtype)
            residual = other(ops[i++]);
        if (i < ops.size() && is_unary_ew(ops[i].node->op_type)) {
            const OpType a = ops[i].node->op_type;
            if (a == OpType::ReLU || a == OpType::GELU || a == OpType::SiLU || a == OpType::Sigmoid || a == OpType::Tanh) act = unary_code(ops[i++].node->op_type);
        }
        if (i != ops.size() || out_dtype != mm->output_dtype) return -1;
        const int bias_v = bias ? make_contiguous(eval(bias)) : -1;
        const int res_v = residual ? make_contiguous(eval(residual)) : -1;
        return emit_gemm(mm, out_shape, bias_v, res_v, act);
    }

    int emit_gemm(const GraphNode *n, const Shape &out_shape_override, int bias_v, int res_v, int act) {
        const auto &mp = get_params<MatMulParams>(n->params);
        bool ta = mp.transpose_a, tb = mp.transpose_b;
        int a = eval(n->inputs[0].get()), b = eval(n->inputs[1].get());
        if (val(a).dtype != val(b).dtype) throw TypeError("GPU matmul needs operands of one dtype");
        // The matrix-core kernels want both operands contiguous along k: A stored [M, K], B stored [N, K].
        //  * an operand that is a transposed view of contiguous memory is taken as that memory with its flag flipped
        //    (matmul(x, w.transpose()) costs no copy);
        //  * an operand stored the other way round is transposed once by the gather kernel when the product is large
        //    enough for that pass to be small change against the FMA kernel it avoids.
        auto swapped = [&](int v) {
            ValueSpec t = val(v);
            const size_t r = t.shape.size();
            std::swap(t.shape[r - 1], t.shape[r - 2]);
            std::swap(t.strides[r - 1], t.strides[r - 2]);
            return add_value(t);
        };
        auto k_contiguous = [&](int v, bool &flag, bool wanted_flag, bool worth_a_copy) {
            if (val(v).shape.size() >= 2 && !contiguous(v)) {
                const int sw = swapped(v);
                if (contiguous(sw)) {
                    v = sw;
                    flag = !flag;
                }
            }
            v = make_contiguous(v);
            if (flag != wanted_flag && worth_a_copy && val(v).shape.size() >= 2) {
                v = make_contiguous(swapped(v));
                flag = wanted_flag;
            }
            return v;
        };
        {
            const Shape &as0 = val(a).shape, &bs0 = val(b).shape;
            const double m0 = static_cast<double>(ta ? as0.back() : as0[as0.size() - 2]), k0 = static_cast<double>(ta ? as0[as0.size() - 2] : as0.back());
            const double n0 = static_cast<double>(tb ? bs0[bs0.size() - 2] : bs0.back());
            const bool big = m0 * n0 * k0 >= double(1 << 22) && m0 >= 64 && n0 >= 64 && k0 >= 32;
            a = k_contiguous(a, ta, false, big);
            b = k_contiguous(b, tb, true, big);
            // A reduction length that leaves the rows off their 16-byte alignment (K = 1001) would send a large product
            // to the FMA kernel (two orders of magnitude slower): both operands get zero columns up to the next
            // aligned length instead -- two copy passes, and zeros add nothing to the products.
            const size_t align = val(a).dtype == DType::Float32 ? 4 : 8, k_now = val(a).shape.back();
            if (big && !ta && tb && k_now % align != 0 && val(a).shape.size() <= AXHIP_MAX_DIMS && val(b).shape.size() <= AXHIP_MAX_DIMS) {
                auto widen = [&](int v) {
                    Shape wide = val(v).shape;
                    wide.back() = (k_now + align - 1) / align * align;
                    Step st{};
                    st.kind = Step::PAD;
                    st.pad.src = v;
                    st.pad.dst = new_temp(wide, val(v).dtype);
                    st.pad.before.assign(wide.size(), 0);
                    st.pad.after.assign(wide.size(), 0);
                    st.pad.after.back() = static_cast<int64_t>(wide.back() - k_now);
                    st.pad.value = 0.0;
                    const int dst = st.pad.dst;
                    plan_.steps.push_back(st);
                    return dst;
                };
                a = widen(a);
                b = widen(b);
            }
        }
        // Batch dimensions that broadcast against each other in part ([B,1,M,K] x [1,H,K,N], or equal counts in
        // different shapes): both operands are expanded to the common batch shape once (a gather with zero strides);
        // a shared operand without batch dimensions, or with all of them 1, needs no copy (stride 0 below).
        {
            const Shape a_batch(val(a).shape.begin(), val(a).shape.end() - 2), b_batch(val(b).shape.begin(), val(b).shape.end() - 2);
            const size_t na = ShapeUtils::size(a_batch), nb = ShapeUtils::size(b_batch);
            if (na > 1 && nb > 1 && a_batch != b_batch) {
                const size_t nd = std::max(a_batch.size(), b_batch.size());
                Shape common(nd, 1);
                for (size_t i = 0; i < nd; ++i) {
                    const size_t da = i + a_batch.size() >= nd ? a_batch[i + a_batch.size() - nd] : 1;
                    const size_t db = i + b_batch.size() >= nd ? b_batch[i + b_batch.size() - nd] : 1;
                    if (da != db && da != 1 && db != 1) throw ShapeError("matmul: batch dimensions do not broadcast");
                    common[i] = std::max(da, db);
                }
                auto expanded = [&](int v) {
                    Shape target = common;
                    target.push_back(val(v).shape[val(v).shape.size() - 2]);
                    target.push_back(val(v).shape.back());
                    return make_contiguous(v, &target);
                };
                a = expanded(a);
                b = expanded(b);
            }
        }
        const Shape &as = val(a).shape, &bs = val(b).shape;
        GemmStep g;
        g.p.dtype = detail::to_axhip_dtype(val(a).dtype);
        g.p.trans_a = ta;
        g.p.trans_b = tb;
        const size_t ar = as[as.size() - 2], ac = as.back(), br = bs[bs.size() - 2], bc = bs.back();
        g.p.m = static_cast<int64_t>(ta ? ac : ar);
        g.p.k = static_cast<int64_t>(ta ? ar : ac);
        g.p.n = static_cast<int64_t>(tb ? br : bc);
        g.p.lda = static_cast<int64_t>(ac);
        g.p.ldb = static_cast<int64_t>(bc);
        g.p.ldc = g.p.n;
        const size_t batch_a = ShapeUtils::size(as) / (ar * ac), batch_b = ShapeUtils::size(bs) / (br * bc);
        if (batch_b == 1 && !ta) { // shared right operand (a Linear weight): fold the batch into M
            g.p.m *= static_cast<int64_t>(batch_a);
            g.p.batch = 1;
        } else if (batch_a == batch_b || batch_b == 1 || batch_a == 1) {
            if (batch_a == batch_b && batch_a > 1 && Shape(as.begin(), as.end() - 2) != Shape(bs.begin(), bs.end() - 2))
                throw RuntimeError::not_implemented("GPU matmul with differently shaped batch dimensions");
            g.p.batch = static_cast<int64_t>(std::max(batch_a, batch_b));
            g.p.stride_a = batch_a == 1 ? 0 : static_cast<int64_t>(ar * ac);
            g.p.stride_b = batch_b == 1 ? 0 : static_cast<int64_t>(br * bc);
            g.p.stride_c = g.p.m * g.p.n;
        } else {
            throw RuntimeError::not_implemented("GPU matmul with broadcast batch dimensions");
        }
        g.p.epilogue_op = act;
        g.a = a;
        g.b = b;
        g.bias = bias_v;
        g.residual = res_v;
        g.c = new_temp(out_shape_override.empty() ? n->output_shape : out_shape_override, n->output_dtype);
        Step s{};
        s.kind = Step::GEMM;
        s.gemm = g;
        plan_.steps.push_back(s);
        if (!out_shape_override.empty()) memo_[n] = g.c; // the bare product never exists
        return g.c;
    }

    const GraphNode *root_;
    const SharedSet &shared_;
    Plan plan_;
    std::unordered_map<const GraphNode *, int> memo_;
    std::unordered_map<const GraphNode *, int> topo_index_;
};

// ------------------------------------------------------------------- cache
struct CacheState {
    std::mutex mu;
    std::unordered_map<uint64_t, std::shared_ptr<const Plan>> plans;
    size_t hits = 0, misses = 0;
};
CacheState &cache() {
    static CacheState c;
    return c;
}

thread_local std::vector<std::string> tl_last_kernels;
std::atomic<bool> g_record_kernels{false};

uint64_t mix_u64(uint64_t h, uint64_t v) {
    for (int i = 0; i < 8; ++i) h = (h ^ ((v >> (8 * i)) & 0xFF)) * 1099511628211ULL;
    return h;
}

// The structural signature plus what else decides the plan: which interior nodes are
// shared (they are materialised on their own) and the layout of materialised leaves.
uint64_t plan_key(const GraphNode *root, const std::vector<const GraphNode *> &topo, const SharedSet &shared) {
    uint64_t h = compute_signature(root).hash;
    for (const GraphNode *n : topo) {
        if (is_leaf(n, root)) {
            if (!n->is_constant) {
                h = mix_u64(h, 0x6C656166); // materialised leaf: shape and strides
                for (size_t d : n->cached_shape_) h = mix_u64(h, d);
                for (int64_t s : n->cached_strides_) h = mix_u64(h, static_cast<uint64_t>(s));
            }
        } else {
            h = mix_u64(h, shared.count(n) ? 2 : 1);
        }
    }
    return h;
}

// node count, root shape and dtype, and per leaf its dtype, shape and strides
std::vector<int64_t> plan_fingerprint(const GraphNode *root, const std::vector<const GraphNode *> &topo) {
    std::vector<int64_t> f;
    f.reserve(16 + 8 * topo.size());
    f.push_back(static_cast<int64_t>(topo.size()));
    f.push_back(static_cast<int64_t>(root->output_dtype));
    f.push_back(static_cast<int64_t>(root->output_shape.size()));
    for (size_t d : root->output_shape) f.push_back(static_cast<int64_t>(d));
    for (const GraphNode *n : topo) {
        if (!is_leaf(n, root)) {
            f.push_back(-1 - static_cast<int64_t>(n->op_type));
            continue;
        }
        const Shape &shape = n->is_constant ? n->output_shape : n->cached_shape_;
        const Strides &strides = n->is_constant ? n->constant_strides : n->cached_strides_;
        f.push_back(static_cast<int64_t>(n->output_dtype));
        f.push_back(static_cast<int64_t>(shape.size()));
        for (size_t d : shape) f.push_back(static_cast<int64_t>(d));
        for (int64_t st : strides) f.push_back(st);
    }
    return f;
}

bool debug_fusion() {
    static const bool v = std::getenv("AXIOM_DEBUG_FUSION") != nullptr;
    return v;
}

} // namespace

GraphCache &GraphCache::instance() {
    static GraphCache g;
    return g;
}
void GraphCache::clear() {
    auto &c = cache();
    std::lock_guard<std::mutex> lk(c.mu);
    c.plans.clear();
    c.hits = c.misses = 0;
}
size_t GraphCache::size() const {
    auto &c = cache();
    std::lock_guard<std::mutex> lk(c.mu);
    return c.plans.size();
}
size_t GraphCache::hits() const { return cache().hits; }
size_t GraphCache::misses() const { return cache().misses; }

const std::vector<std::string> &last_gpu_plan_kernels() { return tl_last_kernels; }
void record_gpu_plan_kernels(bool on) { g_record_kernels.store(on); }

void materialize_gpu_graph(GraphNode *root) {
    if (!root || root->is_materialized_) return;
    const auto topo = topo_sort(root);

    // ---- plan: cached by signature
    const SharedSet shared = shared_nodes(root, topo);
    const uint64_t key = plan_key(root, topo, shared);
    std::shared_ptr<const Plan> plan;
    {
        auto &c = cache();
        std::lock_guard<std::mutex> lk(c.mu);
        auto it = c.plans.find(key);
        if (it != c.plans.end()) plan = it->second;
    }
    const std::vector<int64_t> fingerprint = plan_fingerprint(root, topo);
    if (plan && plan->fingerprint != fingerprint) plan.reset(); // two graphs under one hash: the newcomer replaces the entry
    {
        auto &c = cache();
        std::lock_guard<std::mutex> lk(c.mu);
        ++(plan ? c.hits : c.misses);
    }
    if (!plan) {
        Plan built = PlanBuilder(root, topo, shared).build();
        built.fingerprint = fingerprint;
        plan = std::make_shared<const Plan>(std::move(built));
        auto &c = cache();
        std::lock_guard<std::mutex> lk(c.mu);
        if (c.plans.size() >= GraphCache::max_entries) c.plans.clear(); // src/backends/metal/mpsgraph_graph_compiler.mm:899-900
        c.plans[key] = plan;
    }

    // ---- bind leaves (same order as the builder: topological order) and allocate temporaries
    struct Bound {
        std::shared_ptr<Storage> storage;
        size_t offset = 0;
    };
    std::vector<Bound> leaves;
    for (const GraphNode *n : topo)
        if (is_leaf(n, root)) {
            Bound b;
            b.storage = n->is_constant ? n->constant_storage : n->cached_result_;
            b.offset = n->is_constant ? n->constant_offset : n->cached_offset_;
            if (!b.storage || b.storage->device() != Device::GPU) throw DeviceError("GPU graph input is not resident on the GPU");
            leaves.push_back(std::move(b));
        }
    if (leaves.size() != plan->n_leaves) throw RuntimeError("GPU plan cache: leaf count mismatch");
    std::vector<std::shared_ptr<Storage>> temps(plan->temp_bytes.size());
    for (size_t i = 0; i < temps.size(); ++i) temps[i] = make_storage(plan->temp_bytes[i], Device::GPU);

    auto storage_of = [&](int v) -> std::shared_ptr<Storage> {
        const ValueSpec &s = plan->values[v];
        return s.is_leaf ? leaves[s.index].storage : temps[s.index];
    };
    auto ptr_of = [&](int v) -> void * {
        const ValueSpec &s = plan->values[v];
        char *base = static_cast<char *>(s.is_leaf ? leaves[s.index].storage->raw() : temps[s.index]->raw());
        return base + (s.is_leaf ? leaves[s.index].offset : 0) + s.offset;
    };

    // ---- run
    const bool record = g_record_kernels.load(std::memory_order_relaxed) || debug_fusion();
    tl_last_kernels.clear();
    for (const Step &st : plan->steps) {
        if (st.kind == Step::ROWS) {
            AxhipRowsProgram p = st.rows.prog;
            p.input = ptr_of(st.rows.input);
            p.output = ptr_of(st.rows.output);
            for (int i = 0; i < p.n_operands; ++i) p.operands[i].ptr = ptr_of(st.rows.operand_value[i]);
            if (st.rows.full_reduce) {
                if (record) tl_last_kernels.emplace_back("full_reduce");
                if (p.rows > 0 && p.cols > 0)
                    AXHIP_CALL(axhip_fused_full_reduce(&p, temps[st.rows.workspace]->raw(), temps[st.rows.workspace]->size_bytes(), nullptr));
            } else {
                if (record) tl_last_kernels.emplace_back(axhip_fused_rows_kernel_name(&p));
                AXHIP_CALL(axhip_fused_rows(&p, nullptr));
            }
        } else if (st.kind == Step::GEMM) {
            AxhipGemmParams p = st.gemm.p;
            p.bias = st.gemm.bias >= 0 ? ptr_of(st.gemm.bias) : nullptr;
            p.residual = st.gemm.residual >= 0 ? ptr_of(st.gemm.residual) : nullptr;
            if (record) tl_last_kernels.emplace_back("gemm");
            // (operands the library repacks go through a block of this layer's cache; steady-state graphs allocate nothing)
            const size_t ws_bytes = axhip_gemm_workspace_bytes(&p);
            const std::unique_ptr<Storage> ws = ws_bytes ? make_storage(ws_bytes, Device::GPU) : nullptr;
            AXHIP_CALL(axhip_gemm_ws(ptr_of(st.gemm.a), ptr_of(st.gemm.b), ptr_of(st.gemm.c), &p, ws ? ws->raw() : nullptr, ws_bytes, nullptr));
        } else if (st.kind == Step::PAD) {
            const ValueSpec &src = plan->values[st.pad.src];
            const int64_t isz = static_cast<int64_t>(dtype_size(src.dtype));
            std::vector<int64_t> shp(src.shape.begin(), src.shape.end()), est(src.strides.size());
            for (size_t i = 0; i < est.size(); ++i) est[i] = src.strides[i] / isz;
            if (record) tl_last_kernels.emplace_back("pad");
            AXHIP_CALL(axhip_pad_mode(ptr_of(st.pad.src), ptr_of(st.pad.dst), detail::to_axhip_dtype(src.dtype), static_cast<int32_t>(shp.size()), shp.data(),
                                      est.data(), st.pad.before.data(), st.pad.after.data(), st.pad.mode, st.pad.value, nullptr));
        } else if (st.kind == Step::MASKED_FILL) {
            const ValueSpec &src = plan->values[st.mfill.src];
            const int64_t isz = static_cast<int64_t>(dtype_size(src.dtype));
            std::vector<int64_t> shp(src.shape.begin(), src.shape.end()), est(src.strides.size()), mst(st.mfill.mask_strides.begin(), st.mfill.mask_strides.end());
            for (size_t i = 0; i < est.size(); ++i) est[i] = src.strides[i] / isz;
            if (record) tl_last_kernels.emplace_back("masked_fill");
            AXHIP_CALL(axhip_masked_fill(ptr_of(st.mfill.src), detail::to_axhip_dtype(src.dtype), static_cast<const uint8_t *>(ptr_of(st.mfill.mask)),
                                         ptr_of(st.mfill.dst), static_cast<int32_t>(shp.size()), shp.data(), est.data(), mst.data(), st.mfill.value, nullptr));
        } else if (st.kind == Step::AXIS_REDUCE) {
            const ValueSpec &src = plan->values[st.axred.src], &dst = plan->values[st.axred.dst];
            if (record) tl_last_kernels.emplace_back("reduce_axis");
            const int sdt = detail::to_axhip_dtype_or_bool(src.dtype);
            const size_t ws_bytes = axhip_reduce_axis_workspace_bytes(ptr_of(st.axred.src), sdt, st.axred.outer, st.axred.axis, st.axred.inner);
            const std::unique_ptr<Storage> ws = ws_bytes ? make_storage(ws_bytes, Device::GPU) : nullptr;
            AXHIP_CALL(axhip_reduce_axis_ws(ptr_of(st.axred.src), sdt, st.axred.outer, st.axred.axis, st.axred.inner, st.axred.reduce, ptr_of(st.axred.dst),
                                            detail::to_axhip_dtype_or_bool(dst.dtype), ws ? ws->raw() : nullptr, ws_bytes, nullptr));
        } else if (st.kind == Step::AXIS_SOFTMAX) {
            const ValueSpec &src = plan->values[st.axred.src];
            if (record) tl_last_kernels.emplace_back("softmax_axis");
            AXHIP_CALL(axhip_softmax_axis(ptr_of(st.axred.src), detail::to_axhip_dtype(src.dtype), st.axred.outer, st.axred.axis, st.axred.inner, st.axred.reduce,
                                          ptr_of(st.axred.dst), nullptr));
        } else if (st.kind == Step::WHERE) {
            const ValueSpec &c = plan->values[st.where.cond], &a = plan->values[st.where.a], &b = plan->values[st.where.b], &d = plan->values[st.where.dst];
            std::vector<int64_t> shp(d.shape.begin(), d.shape.end()), cst(shp.size()), ast(shp.size()), bst(shp.size());
            for (size_t i = 0; i < shp.size(); ++i) {
                cst[i] = st.where.cond_strides[i] / static_cast<int64_t>(dtype_size(c.dtype));
                ast[i] = st.where.a_strides[i] / static_cast<int64_t>(dtype_size(a.dtype));
                bst[i] = st.where.b_strides[i] / static_cast<int64_t>(dtype_size(b.dtype));
            }
            if (record) tl_last_kernels.emplace_back("where");
            AXHIP_CALL(axhip_where(ptr_of(st.where.cond), detail::to_axhip_dtype_or_bool(c.dtype), ptr_of(st.where.a), detail::to_axhip_dtype_or_bool(a.dtype),
                                   ptr_of(st.where.b), detail::to_axhip_dtype_or_bool(b.dtype), ptr_of(st.where.dst), detail::to_axhip_dtype_or_bool(d.dtype),
                                   static_cast<int32_t>(shp.size()), shp.data(), cst.data(), ast.data(), bst.data(), nullptr));
        } else if (st.kind == Step::GATHER) {
            const ValueSpec &tab = plan->values[st.gather.table], &idx = plan->values[st.gather.indices];
            if (record) tl_last_kernels.emplace_back("gather_rows");
            AXHIP_CALL(axhip_gather_rows(ptr_of(st.gather.table), detail::to_axhip_dtype(tab.dtype), static_cast<int64_t>(tab.shape[0]),
                                         static_cast<int64_t>(tab.shape[1]), ptr_of(st.gather.indices), static_cast<int32_t>(dtype_size(idx.dtype)),
                                         static_cast<int64_t>(ShapeUtils::size(idx.shape)), ptr_of(st.gather.dst), nullptr));
        } else {
            const ValueSpec &src = plan->values[st.copy.src];
            const int dt = detail::to_axhip_dtype_or_bool(src.dtype), ddt = detail::to_axhip_dtype_or_bool(plan->values[st.copy.dst].dtype);
            std::vector<int64_t> shp(st.copy.shape.begin(), st.copy.shape.end()), est(st.copy.src_strides.size());
            for (size_t i = 0; i < est.size(); ++i) est[i] = st.copy.src_strides[i] / static_cast<int64_t>(dtype_size(src.dtype));
            if (record) tl_last_kernels.emplace_back("strided_copy");
            AXHIP_CALL(axhip_strided_copy(ptr_of(st.copy.src), dt, ptr_of(st.copy.dst), ddt, static_cast<int32_t>(shp.size()), shp.data(),
                                          est.data(), nullptr));
        }
    }
    if (debug_fusion()) {
        std::string line = "[axiom gpu graph] " + std::to_string(topo.size()) + " nodes ->";
        for (const auto &k : tl_last_kernels) line += " " + k;
        fprintf(stderr, "%s\n", line.c_str());
    }

    // ---- publish results: the root and every shared node the plan materialised
    for (const auto &[idx, v] : plan->node_results) {
        GraphNode *n = const_cast<GraphNode *>(topo[idx]);
        const ValueSpec &s = plan->values[v];
        n->cached_result_ = storage_of(v);
        n->cached_shape_ = s.shape;
        n->cached_strides_ = s.strides;
        n->cached_offset_ = (s.is_leaf ? leaves[s.index].offset : 0) + s.offset;
        n->is_materialized_ = true;
    }
    // a materialised node no longer needs its inputs: drop the edges (src/backends/metal/
    // mpsgraph_graph_compiler.mm:931-942 decrements the same counts)
    for (const auto &[idx, v] : plan->node_results) {
        (void)v;
        GraphNode *n = const_cast<GraphNode *>(topo[idx]);
        for (auto &in : n->inputs)
            if (!in->is_constant && in->ref_count.load() > 0) in->ref_count.fetch_sub(1);
        n->inputs.clear();
    }
}

} // namespace axiom::graph
