// nn modules on the attention / norm path and around it (include/axiom/nn/{module,linear,
// normalization,attention,activation,conv,embedding,container}.hpp; src/nn/*.cpp).  Inference only.
#pragma once

#include <array>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "axiom/tensor.hpp"

namespace axiom::nn {

class Module {
  public:
    Module() = default;
    virtual ~Module() = default;
    Module(const Module &) = delete;
    Module &operator=(const Module &) = delete;

    virtual Tensor forward(const Tensor &input) const;
    Tensor operator()(const Tensor &input) const { return forward(input); }
    virtual Module &to(Device device);
    virtual Module &to(DType dtype);
    // parameters are looked up as prefix + name; submodules add "name." (src/nn/module.cpp:36-50)
    virtual void load_state_dict(const std::map<std::string, Tensor> &state_dict, const std::string &prefix = "", bool strict = true);
    std::map<std::string, Tensor> state_dict(const std::string &prefix = "") const;
    std::vector<std::pair<std::string, Tensor *>> named_parameters(const std::string &prefix = "") const; // insertion order
    std::vector<Tensor *> parameters() const;

  protected:
    void register_parameter(const std::string &name, Tensor &param);
    void register_module(const std::string &name, Module &submodule);

  private:
    std::vector<std::pair<std::string, Tensor *>> params_;
    std::vector<std::pair<std::string, Module *>> submodules_;
};

// y = x W^T + b, weight (out_features, in_features) (src/nn/linear.cpp:15-27)
class Linear : public Module {
  public:
    explicit Linear(bool bias = true);
    Tensor forward(const Tensor &input) const override;
    bool has_bias() const { return has_bias_; }
    const Tensor &weight() const { return weight_; }
    const Tensor &bias() const { return bias_; }

  private:
    Tensor weight_, bias_;
    bool has_bias_;
};

class LayerNorm : public Module {
  public:
    explicit LayerNorm(float eps = 1e-5f);
    Tensor forward(const Tensor &input) const override;

  private:
    Tensor weight_, bias_;
    float eps_;
};

class RMSNorm : public Module {
  public:
    explicit RMSNorm(float eps = 1e-5f);
    Tensor forward(const Tensor &input) const override;

  private:
    Tensor weight_;
    float eps_;
};

class ReLU : public Module {
  public:
    Tensor forward(const Tensor &input) const override;
};
class GELU : public Module {
  public:
    Tensor forward(const Tensor &input) const override;
};

// 1-D convolution, weight (C_out, C_in, K) (include/axiom/nn/conv.hpp:25-48)
class Conv1d : public Module {
  public:
    explicit Conv1d(int stride = 1, int padding = 0, int dilation = 1, int groups = 1, bool bias = true);
    Tensor forward(const Tensor &input) const override;
    const Tensor &weight() const { return weight_; }
    const Tensor &bias() const { return bias_; }

  private:
    Tensor weight_, bias_;
    int stride_, padding_, dilation_, groups_;
    bool has_bias_;
};

// 2-D convolution, weight (C_out, C_in, KH, KW) (include/axiom/nn/conv.hpp:50-75)
class Conv2d : public Module {
  public:
    explicit Conv2d(std::array<int, 2> stride = {1, 1}, std::array<int, 2> padding = {0, 0}, std::array<int, 2> dilation = {1, 1}, int groups = 1,
                    bool bias = true);
    Tensor forward(const Tensor &input) const override;

  private:
    Tensor weight_, bias_;
    std::array<int, 2> stride_, padding_, dilation_;
    int groups_;
    bool has_bias_;
};

// rows of weight (vocab, dim) by integer index (include/axiom/nn/embedding.hpp:7-16)
class Embedding : public Module {
  public:
    Embedding();
    Tensor forward(const Tensor &indices) const override;

  private:
    Tensor weight_;
};

// inference batch norm with running statistics (include/axiom/nn/normalization.hpp:37-58)
class BatchNorm1d : public Module {
  public:
    explicit BatchNorm1d(float eps = 1e-5f);
    Tensor forward(const Tensor &input) const override;

  private:
    Tensor weight_, bias_, running_mean_, running_var_;
    float eps_;
};

// owning list of submodules named "0", "1", ... (include/axiom/nn/container.hpp:11-35)
class ModuleList : public Module {
  public:
    template <typename T, typename... Args> T &emplace_back(Args &&...args) {
        auto ptr = std::make_unique<T>(std::forward<Args>(args)...);
        T &ref = *ptr;
        register_module(std::to_string(modules_.size()), ref);
        modules_.push_back(std::move(ptr));
        return ref;
    }
    Module &operator[](size_t index) { return *modules_.at(index); }
    const Module &operator[](size_t index) const { return *modules_.at(index); }
    size_t size() const { return modules_.size(); }

  private:
    std::vector<std::unique_ptr<Module>> modules_;
};

// q/k/v/out projections + scaled_dot_product_attention over num_heads heads
// (src/nn/attention.cpp:17-65).  Inputs (batch, seq, d_model).
class MultiHeadAttention : public Module {
  public:
    explicit MultiHeadAttention(int num_heads, bool bias = true);
    Tensor forward(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask = Tensor(), bool is_causal = false) const;
    int num_heads() const { return num_heads_; }
    // anything that replaces the parameters drops the stacked projection weight
    void load_state_dict(const std::map<std::string, Tensor> &state_dict, const std::string &prefix = "", bool strict = true) override;
    Module &to(Device device) override;
    Module &to(DType dtype) override;

  private:
    // self-attention on the GPU runs the three input projections as ONE product against the stacked
    // (3 d_model, d_model) weight; the stack is built on first use and rebuilt when a projection's weight changes
    bool fused_qkv(const Tensor &x, Tensor &q, Tensor &k, Tensor &v) const;

    int num_heads_;
    Linear q_proj_, k_proj_, v_proj_, out_proj_;
    mutable Tensor qkv_weight_, qkv_bias_;
    // the storages (and offsets) the stacked copy was made from; held so that their blocks cannot be recycled
    mutable std::shared_ptr<Storage> qkv_holders_[6];
    mutable size_t qkv_offsets_[6] = {0, 0, 0, 0, 0, 0};
    void drop_stacked_projection();
};

} // namespace axiom::nn
