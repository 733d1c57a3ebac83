// nn modules on the attention / norm path (behaviour of src/nn/{module,linear,
// normalization,attention,activation}.cpp).
#include "axiom/nn.hpp"

#include "axiom/operations.hpp"

namespace axiom::nn {

Tensor Module::forward(const Tensor &) const { throw RuntimeError::not_implemented("forward(const Tensor&) for this module"); }

Module &Module::to(Device device) {
    for (auto &[name, p] : params_)
        if (!p->empty()) *p = p->to(device);
    for (auto &[name, m] : submodules_) m->to(device);
    return *this;
}

Module &Module::to(DType dtype) {
    for (auto &[name, p] : params_)
        if (!p->empty()) *p = p->astype(dtype);
    for (auto &[name, m] : submodules_) m->to(dtype);
    return *this;
}

void Module::load_state_dict(const std::map<std::string, Tensor> &sd, const std::string &prefix, bool strict) {
    for (auto &[name, p] : params_) {
        auto it = sd.find(prefix + name);
        if (it != sd.end()) *p = it->second;
        else if (strict) throw ValueError("missing key '" + prefix + name + "' in state_dict");
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
    Tensor q = q_proj_.forward(query).reshape({B, Sq, H, Dh}).transpose({0, 2, 1, 3});
    Tensor k = k_proj_.forward(key).reshape({B, Skv, H, Dh}).transpose({0, 2, 1, 3});
    Tensor v = v_proj_.forward(value).reshape({B, Skv, H, Dh}).transpose({0, 2, 1, 3});
    Tensor attn = ops::detail::sdpa(q, k, v, mask, -1.0f, is_causal, /*out_bshd=*/true);
    Tensor merged = attn.transpose({0, 2, 1, 3}).reshape({B, Sq, Dm});
    return out_proj_.forward(merged);
}

} // namespace axiom::nn
