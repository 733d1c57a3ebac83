// The remaining GPU hooks of Axiom's backend boundary: the per-op registry, the free gpu_*
// functions and the execution of CPU-planned fused steps.  All of them are thin: they build
// the same lazy nodes as ops:: and materialise at once.
#include <mutex>

#include "axiom/backends/hip/hip_operations.hpp"
#include "axiom/error.hpp"
#include "axiom/graph/gpu_fusion.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/operations.hpp"
#include "axiom/tensor.hpp"

namespace axiom {

// ------------------------------------------------------------ Operation base
namespace ops {

bool Operation::supports_binary(const Tensor &lhs, const Tensor &rhs) const { return lhs.shape() == rhs.shape(); }
Tensor Operation::execute_binary(const Tensor &, const Tensor &) const { throw RuntimeError::not_implemented(name() + "::execute_binary"); }
Tensor Operation::execute_unary(const Tensor &) const { throw RuntimeError::not_implemented(name() + "::execute_unary"); }
Tensor Operation::execute_reduction(const Tensor &, const std::vector<int> &, bool) const { throw RuntimeError::not_implemented(name() + "::execute_reduction"); }
Tensor Operation::execute_matmul(const Tensor &, const Tensor &, bool, bool) const { throw RuntimeError::not_implemented(name() + "::execute_matmul"); }
Tensor Operation::execute_cast(const Tensor &, DType) const { throw RuntimeError::not_implemented(name() + "::execute_cast"); }

namespace {
std::map<std::pair<OpType, Device>, std::unique_ptr<Operation>> &raw_registry() {
    static std::map<std::pair<OpType, Device>, std::unique_ptr<Operation>> r;
    return r;
}
std::mutex &registry_mutex() {
    static std::mutex m;
    return m;
}
std::once_flag g_builtin_once;
} // namespace

void OperationRegistry::register_operation(OpType op, Device device, std::unique_ptr<Operation> operation) {
    std::lock_guard<std::mutex> lk(registry_mutex());
    raw_registry()[{op, device}] = std::move(operation);
}

void OperationRegistry::initialize_builtin_operations() {
    std::call_once(g_builtin_once, [] { backends::hip::register_hip_operations(); });
}

const Operation *OperationRegistry::get_operation(OpType op, Device device) {
    initialize_builtin_operations();
    std::lock_guard<std::mutex> lk(registry_mutex());
    auto it = raw_registry().find({op, device});
    return it == raw_registry().end() ? nullptr : it->second.get();
}

bool OperationRegistry::is_operation_available(OpType op, Device device) { return get_operation(op, device) != nullptr; }

std::vector<Device> OperationRegistry::available_devices_for_operation(OpType op) {
    std::vector<Device> out;
    for (Device d : {Device::CPU, Device::GPU})
        if (is_operation_available(op, d)) out.push_back(d);
    return out;
}

} // namespace ops

// ------------------------------------------------------------- backend hooks
namespace backends::hip {

namespace {

using ops::OpType;

// one registry entry: routes the call into the lazy graph under an eager scope, so the op
// runs at once as its own (cached) plan -- the per-op graphs of src/backends/metal/
// mpsgraph_operations.mm:1056-1615
class HipOperation final : public ops::Operation {
  public:
    explicit HipOperation(OpType t) : type_(t) {}
    OpType type() const override { return type_; }
    std::string name() const override { return std::string("hip::") + ops::op_name(type_); }
    Device device() const override { return Device::GPU; }
    bool supports_binary(const Tensor &lhs, const Tensor &rhs) const override {
        try {
            ShapeUtils::broadcast(lhs.shape(), rhs.shape());
            return true;
        } catch (const ShapeError &) {
            return false;
        }
    }
    Tensor execute_binary(const Tensor &lhs, const Tensor &rhs) const override {
        if (!binary_type()) return Operation::execute_binary(lhs, rhs); // throws not_implemented
        graph::EagerModeScope eager;
        return graph::GraphRegistry::create_lazy_binary(type_, lhs, rhs);
    }
    Tensor execute_unary(const Tensor &input) const override {
        if (!unary_type()) return Operation::execute_unary(input);
        graph::EagerModeScope eager;
        if (type_ == OpType::Softmax || type_ == OpType::LogSoftmax) return graph::GraphRegistry::create_lazy_softmax(type_, input, -1);
        return graph::GraphRegistry::create_lazy_unary(type_, input);
    }
    Tensor execute_reduction(const Tensor &input, const std::vector<int> &axis, bool keep_dims) const override {
        if (!reduction_type()) return Operation::execute_reduction(input, axis, keep_dims);
        graph::EagerModeScope eager;
        if (type_ == OpType::Softmax || type_ == OpType::LogSoftmax) // softmax arrives through the reduction entry (operations.cpp:1427-1434)
            return graph::GraphRegistry::create_lazy_softmax(type_, input, axis.empty() ? -1 : axis[0]);
        return graph::GraphRegistry::create_lazy_reduction(type_, input, axis, keep_dims);
    }
    Tensor execute_matmul(const Tensor &a, const Tensor &b, bool ta, bool tb) const override {
        if (type_ != OpType::MatMul) return Operation::execute_matmul(a, b, ta, tb);
        graph::EagerModeScope eager;
        return graph::GraphRegistry::create_lazy_matmul(a, b, ta, tb);
    }
    Tensor execute_cast(const Tensor &input, DType target) const override { return input.astype(target); }

  private:
    bool binary_type() const {
        return type_ == OpType::Add || type_ == OpType::Subtract || type_ == OpType::Multiply || type_ == OpType::Divide ||
               type_ == OpType::Maximum || type_ == OpType::Minimum;
    }
    bool reduction_type() const {
        return type_ == OpType::Sum || type_ == OpType::Mean || type_ == OpType::Max || type_ == OpType::Min || type_ == OpType::Softmax ||
               type_ == OpType::LogSoftmax;
    }
    bool unary_type() const { return !binary_type() && type_ != OpType::MatMul && type_ != OpType::Cast && (!reduction_type() || type_ == OpType::Softmax || type_ == OpType::LogSoftmax); }
    OpType type_;
};

} // namespace

bool is_hip_available() { return is_available(); }

void register_hip_operations() {
    static const OpType supported[] = {OpType::Add, OpType::Subtract, OpType::Multiply, OpType::Divide, OpType::Maximum, OpType::Minimum,
                                       OpType::Negate, OpType::Abs, OpType::Sqrt, OpType::Exp, OpType::Log, OpType::Reciprocal, OpType::Square,
                                       OpType::ReLU, OpType::SiLU, OpType::Sigmoid, OpType::Tanh, OpType::GELU, OpType::Softmax,
                                       OpType::LogSoftmax, OpType::Sum, OpType::Mean, OpType::Max, OpType::Min, OpType::MatMul, OpType::Cast};
    for (OpType t : supported) ops::OperationRegistry::register_operation(t, Device::GPU, std::make_unique<HipOperation>(t));
}

Tensor gpu_layer_norm(const Tensor &input, const Tensor &weight, const Tensor &bias, int axis, float eps) {
    graph::EagerModeScope eager;
    return ops::layer_norm(input, weight, bias, axis, eps);
}
Tensor gpu_rms_norm(const Tensor &input, const Tensor &weight, int axis, float eps) {
    graph::EagerModeScope eager;
    return ops::rms_norm(input, weight, axis, eps);
}
Tensor gpu_scaled_dot_product_attention(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor &mask, float scale, bool is_causal) {
    return ops::scaled_dot_product_attention(q, k, v, mask, scale, is_causal);
}
Tensor gpu_fill_constant(const Shape &shape, DType dtype, double value) {
    Tensor t(shape, dtype, Device::CPU);
    t.fill(value);
    return t.to(Device::GPU);
}
Tensor gpu_make_contiguous(const Tensor &tensor) {
    tensor.sync();
    return tensor.ascontiguousarray();
}
// matmul(x, W, false, true) + bias built lazily and materialised at once: one GEMM with the bias in
// its epilogue (role of gpu_linear, src/backends/metal/mpsgraph_operations.mm:2409-2532)
Tensor gpu_linear(const Tensor &input, const Tensor &weight, const Tensor &bias, bool has_bias) {
    Tensor y = graph::GraphRegistry::create_lazy_matmul(input, weight, false, true);
    if (has_bias && !bias.empty()) y = ops::add(y, bias);
    y.sync();
    return y;
}

} // namespace backends::hip

// ------------------------------------------------ CPU-planned fused steps
namespace graph {

namespace {

bool is_unary(ops::OpType op) {
    using ops::OpType;
    switch (op) {
    case OpType::Negate: case OpType::Abs: case OpType::Sqrt: case OpType::Exp: case OpType::Log: case OpType::Reciprocal:
    case OpType::Square: case OpType::ReLU: case OpType::SiLU: case OpType::Sigmoid: case OpType::Tanh: case OpType::GELU:
        return true;
    default: return false;
    }
}
bool is_binary(ops::OpType op) {
    using ops::OpType;
    return op == OpType::Add || op == OpType::Subtract || op == OpType::Multiply || op == OpType::Divide || op == OpType::Maximum ||
           op == OpType::Minimum;
}

// threads the chain through lazy nodes; `ok` turns false on an op without a GPU kernel
Tensor build_chain(const StepBase &step, const std::vector<ops::OpType> &chain, std::vector<Tensor> &buffers, bool &ok) {
    Tensor prev;
    ok = !chain.empty() && step.input_slot_indices.size() >= chain.size();
    for (size_t i = 0; ok && i < chain.size(); ++i) {
        const auto &idx = step.input_slot_indices[i];
        auto resolve = [&](size_t k) -> Tensor {
            const int slot = k < idx.size() ? idx[k] : -1;
            if (slot == -1) return prev;
            if (slot < 0 || slot >= static_cast<int>(buffers.size())) {
                ok = false;
                return prev;
            }
            const Tensor &t = buffers[slot];
            return t.device() == Device::GPU ? t : t.to(Device::GPU);
        };
        if (is_unary(chain[i])) {
            Tensor in = resolve(0);
            if (ok && !in.empty()) prev = GraphRegistry::create_lazy_unary(chain[i], in);
            else ok = false;
        } else if (is_binary(chain[i])) {
            Tensor a = resolve(0), b = resolve(1);
            if (ok && !a.empty() && !b.empty()) prev = GraphRegistry::create_lazy_binary(chain[i], a, b);
            else ok = false;
        } else {
            ok = false;
        }
    }
    return prev;
}

} // namespace

bool execute_gpu_fused_chain(const StepBase &step, const std::vector<ops::OpType> &op_chain, std::vector<Tensor> &buffers) {
    const DType dt = step.output_dtype;
    if (dt != DType::Float32 && dt != DType::Float16 && dt != DType::BFloat16) return false;
    bool ok = true;
    Tensor out = build_chain(step, op_chain, buffers, ok);
    if (!ok) return false;
    if (out.dtype() != dt) out = out.astype(dt);
    out.sync(); // one fused launch (asynchronous on the backend stream)
    if (step.output_slot >= 0 && step.output_slot < static_cast<int>(buffers.size())) buffers[step.output_slot] = out;
    return true;
}

bool execute_gpu_fused_reduction(const FusedReductionStep &step, std::vector<Tensor> &buffers) {
    using ops::OpType;
    if (step.reduction_op != OpType::Sum && step.reduction_op != OpType::Mean && step.reduction_op != OpType::Max && step.reduction_op != OpType::Min)
        return false;
    const auto *rp = std::get_if<ReductionParams>(&step.params);
    bool ok = true;
    Tensor chain;
    if (step.op_chain.empty()) {
        if (step.input_slot_indices.empty() || step.input_slot_indices[0].empty()) return false;
        const int slot = step.input_slot_indices[0][0];
        if (slot < 0 || slot >= static_cast<int>(buffers.size())) return false;
        chain = buffers[slot].device() == Device::GPU ? buffers[slot] : buffers[slot].to(Device::GPU);
    } else {
        chain = build_chain(step, step.op_chain, buffers, ok);
        if (!ok) return false;
    }
    Tensor out = GraphRegistry::create_lazy_reduction(step.reduction_op, chain, rp ? rp->axes : std::vector<int>{}, rp ? rp->keep_dims : false);
    if (out.dtype() != step.output_dtype) out = out.astype(step.output_dtype);
    out.sync();
    if (step.output_slot >= 0 && step.output_slot < static_cast<int>(buffers.size())) buffers[step.output_slot] = out;
    return true;
}

} // namespace graph
} // namespace axiom
