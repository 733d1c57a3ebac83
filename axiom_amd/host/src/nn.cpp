// nn modules on the attention / norm path (behaviour of src/nn/{module,linear,
// normalization,attention,activation}.cpp).
#include <cstring>

#include "axiom/nn.hpp"

#include "axiom/operations.hpp"
#include "hip_call.hpp"

namespace axiom::nn {

Tensor Module::forward(const Tensor &) const { throw RuntimeError::not_implemented("forward(const Tensor&) for this module"); }

// A parameter is memory, never a deferred computation: a lazy tensor handed in as a weight (say
// (randn * 0.02).astype(bf16)) is run once here.  Left lazy, every forward would recompute it as a fused input
// of the product it feeds, and the stacked q/k/v projection could not take its address.
static void settle(Tensor &p) {
    if (!p.empty() && p.is_lazy()) p.sync();
}

Module &Module::to(Device device) {
    for (auto &[name, p] : params_)
        if (!p->empty()) {
            *p = p->to(device);
            settle(*p);
        }
    for (auto &[name, m] : submodules_) m->to(device);
    return *this;
}

Module &Module::to(DType dtype) {
    for (auto &[name, p] : params_)
        if (!p->empty()) {
            *p = p->astype(dtype);
            settle(*p);
        }
    for (auto &[name, m] : submodules_) m->to(dtype);
    return *this;
}

void Module::load_state_dict(const std::map<std::string, Tensor> &sd, const std::string &prefix, bool strict) {
    for (auto &[name, p] : params_) {
        auto it = sd.find(prefix + name);
        if (it != sd.end()) {
            *p = it->second;
            settle(*p);
        } else if (strict) throw ValueError("missing key '" + prefix + name + "' in state_dict");
    }
    for (auto &[name, m] : submodules_) m->load_state_dict(sd, prefix + name + ".", strict);
}

std::map<std::string, Tensor> Module::state_dict(const std::string &prefix) const {
    std::map<std::string, Tensor> out;
    for (auto &[name, p] : named_parameters(prefix)) out[name] = *p;
    return out;
}

std::vector<std::pair<std::string, Tensor *>> Module::named_parameters(const std::string &prefix) const {
    std::vector<std::pair<std::string, Tensor *>> out;
    for (auto &[name, p] : params_) out.emplace_back(prefix + name, p);
    for (auto &[name, m] : submodules_) {
        auto sub = m->named_parameters(prefix + name + ".");
        out.insert(out.end(), sub.begin(), sub.end());
    }
    return out;
}

std::vector<Tensor *> Module::parameters() const {
    std::vector<Tensor *> out;
    for (auto &[name, p] : named_parameters()) out.push_back(p);
    return out;
}

void Module::register_parameter(const std::string &name, Tensor &param) { params_.emplace_back(name, &param); }
void Module::register_module(const std::string &name, Module &sub) { submodules_.emplace_back(name, &sub); }

// ------------------------------------------------------------------ Linear
Linear::Linear(bool bias) : has_bias_(bias) {
    register_parameter("weight", weight_);
    if (bias) register_parameter("bias", bias_);
}

Tensor Linear::forward(const Tensor &input) const {
    if (weight_.empty()) throw RuntimeError("Linear: weight not initialized (load_state_dict first)");
    if (weight_.is_lazy()) weight_.sync(); // a lazy tensor assigned through parameters(): run it once, not per forward
    if (has_bias_ && bias_.is_lazy()) bias_.sync();
    Tensor y = ops::matmul(input, weight_, false, true);
    if (has_bias_ && !bias_.empty()) y = ops::add(y, bias_);
    return y;
}

// ------------------------------------------------------------------- norms
LayerNorm::LayerNorm(float eps) : eps_(eps) {
    register_parameter("weight", weight_);
    register_parameter("bias", bias_);
}
Tensor LayerNorm::forward(const Tensor &input) const {
    if (weight_.empty()) throw RuntimeError("LayerNorm: weight not initialized (load_state_dict first)");
    return ops::layer_norm(input, weight_, bias_, -1, eps_);
}

RMSNorm::RMSNorm(float eps) : eps_(eps) { register_parameter("weight", weight_); }
Tensor RMSNorm::forward(const Tensor &input) const {
    if (weight_.empty()) throw RuntimeError("RMSNorm: weight not initialized (load_state_dict first)");
    return ops::rms_norm(input, weight_, -1, eps_);
}

Tensor ReLU::forward(const Tensor &input) const { return ops::relu(input); }
Tensor GELU::forward(const Tensor &input) const { return ops::gelu(input); }

// ------------------------------------------- conv, embedding, batch norm
Conv1d::Conv1d(int stride, int padding, int dilation, int groups, bool bias)
    : stride_(stride), padding_(padding), dilation_(dilation), groups_(groups), has_bias_(bias) {
    register_parameter("weight", weight_);
    if (has_bias_) register_parameter("bias", bias_);
}
Tensor Conv1d::forward(const Tensor &input) const {
    if (weight_.empty()) throw RuntimeError("Conv1d: weight not initialized (load_state_dict first)");
    return ops::conv1d(input, weight_, has_bias_ ? bias_ : Tensor(), stride_, padding_, dilation_, groups_);
}

Conv2d::Conv2d(std::array<int, 2> stride, std::array<int, 2> padding, std::array<int, 2> dilation, int groups, bool bias)
    : stride_(stride), padding_(padding), dilation_(dilation), groups_(groups), has_bias_(bias) {
    register_parameter("weight", weight_);
    if (has_bias_) register_parameter("bias", bias_);
}
Tensor Conv2d::forward(const Tensor &input) const {
    if (weight_.empty()) throw RuntimeError("Conv2d: weight not initialized (load_state_dict first)");
    return ops::conv2d(input, weight_, has_bias_ ? bias_ : Tensor(), stride_, padding_, dilation_, groups_);
}

Embedding::Embedding() { register_parameter("weight", weight_); }
Tensor Embedding::forward(const Tensor &indices) const {
    if (weight_.empty()) throw RuntimeError("Embedding: weight not initialized (load_state_dict first)");
    return ops::embedding(weight_, indices);
}

BatchNorm1d::BatchNorm1d(float eps) : eps_(eps) {
    register_parameter("weight", weight_);
    register_parameter("bias", bias_);
    register_parameter("running_mean", running_mean_);
    register_parameter("running_var", running_var_);
}
Tensor BatchNorm1d::forward(const Tensor &input) const {
    if (running_mean_.empty() || running_var_.empty()) throw RuntimeError("BatchNorm1d: running statistics not initialized (load_state_dict first)");
    return ops::batch_norm1d(input, weight_, bias_, running_mean_, running_var_, eps_);
}

// ------------------------------------------------------- MultiHeadAttention
MultiHeadAttention::MultiHeadAttention(int num_heads, bool bias) : num_heads_(num_heads), q_proj_(bias), k_proj_(bias), v_proj_(bias), out_proj_(bias) {
    register_module("q_proj", q_proj_);
    register_module("k_proj", k_proj_);
    register_module("v_proj", v_proj_);
    register_module("out_proj", out_proj_);
}

// src/nn/attention.cpp:17-65.  The (B,S,H,Dh) -> (B,H,S,Dh) head split stays a strided view:
// the attention kernel takes the strides, nothing is copied.
Tensor MultiHeadAttention::forward(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask, bool is_causal) const {
    if (query.ndim() != 3 || key.ndim() != 3 || value.ndim() != 3)
        throw ShapeError("MultiHeadAttention expects (batch, seq, d_model) inputs");
    const size_t B = query.shape()[0], Sq = query.shape()[1], Dm = query.shape()[2], Skv = key.shape()[1];
    const size_t H = static_cast<size_t>(num_heads_);
    if (Dm % H != 0) throw ShapeError("MultiHeadAttention: d_model " + std::to_string(Dm) + " is not divisible by " + std::to_string(H) + " heads");
    const size_t Dh = Dm / H;
    Tensor q, k, v;
    if (!(&query == &key && &key == &value && fused_qkv(query, q, k, v))) {
        q = q_proj_.forward(query).reshape({B, Sq, H, Dh}).transpose({0, 2, 1, 3});
        k = k_proj_.forward(key).reshape({B, Skv, H, Dh}).transpose({0, 2, 1, 3});
        v = v_proj_.forward(value).reshape({B, Skv, H, Dh}).transpose({0, 2, 1, 3});
    }
    Tensor attn = ops::detail::sdpa(q, k, v, mask, -1.0f, is_causal, /*out_bshd=*/true);
    Tensor merged = attn.transpose({0, 2, 1, 3}).reshape({B, Sq, Dm});
    return out_proj_.forward(merged);
}

void MultiHeadAttention::drop_stacked_projection() {
    qkv_weight_ = qkv_bias_ = Tensor();
    for (auto &h : qkv_holders_) h.reset();
}
void MultiHeadAttention::load_state_dict(const std::map<std::string, Tensor> &sd, const std::string &prefix, bool strict) {
    drop_stacked_projection();
    Module::load_state_dict(sd, prefix, strict);
}
Module &MultiHeadAttention::to(Device device) {
    drop_stacked_projection();
    return Module::to(device);
}
Module &MultiHeadAttention::to(DType dtype) {
    drop_stacked_projection();
    return Module::to(dtype);
}

// q, k, v of self-attention as (B, H, S, Dh) views of one (B, S, 3 d_model) product.  False when the
// projections are not three same-typed contiguous GPU matrices (the caller then projects one by one).
bool MultiHeadAttention::fused_qkv(const Tensor &x, Tensor &q, Tensor &k, Tensor &v) const {
    const Linear *proj[3] = {&q_proj_, &k_proj_, &v_proj_};
    if (x.device() != Device::GPU) return false;
    const DType dt = x.dtype();
    const size_t B = x.shape()[0], S = x.shape()[1], Dm = x.shape()[2], H = static_cast<size_t>(num_heads_), Dh = Dm / H;
    bool any_bias = false;
    const void *sources[6];
    std::shared_ptr<Storage> holders[6];
    size_t offsets[6] = {};
    for (int i = 0; i < 3; ++i) {
        const Tensor &w = proj[i]->weight(), &b = proj[i]->bias();
        if (w.is_lazy()) w.sync();
        if (b.is_lazy()) b.sync();
        if (w.empty() || w.device() != Device::GPU || w.dtype() != dt || !w.is_contiguous() || w.ndim() != 2 || w.shape()[0] != Dm || w.shape()[1] != Dm)
            return false;
        const bool has_b = proj[i]->has_bias() && !b.empty();
        if (has_b && (b.device() != Device::GPU || b.dtype() != dt || !b.is_contiguous() || b.size() != Dm)) return false;
        any_bias = any_bias || has_b;
        sources[2 * i] = static_cast<const char *>(w.storage()->raw()) + w.offset();
        sources[2 * i + 1] = has_b ? static_cast<const char *>(b.storage()->raw()) + b.offset() : nullptr;
        holders[2 * i] = w.storage();
        offsets[2 * i] = w.offset();
        if (has_b) {
            holders[2 * i + 1] = b.storage();
            offsets[2 * i + 1] = b.offset();
        }
    }
    // The stacked copy is current while the six parameters are still the same storage objects at the same offsets.
    // The cache holds those storages, so a replaced parameter's block cannot be recycled into a new tensor at the old
    // address while it is compared (device addresses alone would match again after the allocator reuses the block).
    bool current = !qkv_weight_.empty() && qkv_weight_.dtype() == dt;
    for (int i = 0; i < 6 && current; ++i) current = holders[i] == qkv_holders_[i] && offsets[i] == qkv_offsets_[i];
    if (!current) {
        const size_t isz = dtype_size(dt);
        Tensor w3(Shape{3 * Dm, Dm}, dt, Device::GPU), b3;
        if (any_bias) b3 = Tensor(Shape{3 * Dm}, dt, Device::GPU);
        for (int i = 0; i < 3; ++i) {
            AXHIP_CALL(axhip_memcpy_d2d_async(static_cast<char *>(w3.storage()->raw()) + i * Dm * Dm * isz, sources[2 * i], Dm * Dm * isz, nullptr));
            if (!any_bias) continue;
            char *dst = static_cast<char *>(b3.storage()->raw()) + i * Dm * isz;
            if (sources[2 * i + 1]) AXHIP_CALL(axhip_memcpy_d2d_async(dst, sources[2 * i + 1], Dm * isz, nullptr));
            else AXHIP_CALL(axhip_fill(dst, detail::to_axhip_dtype(dt), 0.0, static_cast<int64_t>(Dm), nullptr));
        }
        qkv_weight_ = w3;
        qkv_bias_ = b3;
        for (int i = 0; i < 6; ++i) {
            qkv_holders_[i] = holders[i];
            qkv_offsets_[i] = offsets[i];
        }
    }
    Tensor qkv = ops::matmul(x, qkv_weight_, false, true);
    if (!qkv_bias_.empty()) qkv = ops::add(qkv, qkv_bias_);
    const auto st = qkv.storage(); // materialises: the attention kernel needs the memory anyway
    const int64_t e = static_cast<int64_t>(dtype_size(dt));
    const Strides strides{static_cast<int64_t>(S * 3 * Dm) * e, static_cast<int64_t>(Dh) * e, static_cast<int64_t>(3 * Dm) * e, e};
    const Shape shape{B, H, S, Dh};
    q = Tensor(st, shape, strides, dt, qkv.offset());
    k = Tensor(st, shape, strides, dt, qkv.offset() + Dm * static_cast<size_t>(e));
    v = Tensor(st, shape, strides, dt, qkv.offset() + 2 * Dm * static_cast<size_t>(e));
    return true;
}

} // namespace axiom::nn
