// axiom::Tensor: value-semantic handle on (storage, shape, byte strides, dtype,
// byte offset) or on a lazy graph node (include/axiom/tensor.hpp:40-804; the
// hot-path subset of that surface).  shape()/dtype()/device() answer from the
// lazy node without materialising; strides()/storage()/data access materialise.
#pragma once

#include <initializer_list>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "axiom/dtype.hpp"
#include "axiom/error.hpp"
#include "axiom/shape.hpp"
#include "axiom/storage.hpp"

namespace axiom {

namespace graph {
struct GraphNode;
}

// start:stop:step along one dimension, Python semantics for negative and absent bounds
// (include/axiom/indexing.hpp:13-22); the step must be positive here
struct Slice {
    std::optional<int64_t> start, stop, step;
    Slice(std::optional<int64_t> start_val = std::nullopt, std::optional<int64_t> stop_val = std::nullopt,
          std::optional<int64_t> step_val = std::nullopt)
        : start(start_val), stop(stop_val), step(step_val) {}
};

class Tensor {
  public:
    Tensor();
    Tensor(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    Tensor(std::initializer_list<size_t> shape, DType dtype = DType::Float32, Device device = Device::CPU);
    Tensor(std::shared_ptr<Storage> storage, const Shape &shape, const Strides &strides, DType dtype, size_t offset = 0);
    explicit Tensor(std::shared_ptr<graph::GraphNode> lazy_node);

    // ---- metadata
    const Shape &shape() const;
    size_t ndim() const { return shape().size(); }
    size_t size() const { return ShapeUtils::size(shape()); }
    bool empty() const { return !storage_ && !lazy_node_; }
    DType dtype() const;
    Device device() const;
    size_t itemsize() const { return dtype_size(dtype()); }
    const Strides &strides() const; // materialises
    size_t offset() const;          // materialises
    bool is_contiguous() const;     // materialises
    std::shared_ptr<Storage> storage() const; // materialises

    bool is_lazy() const { return lazy_node_ != nullptr; }
    std::shared_ptr<graph::GraphNode> lazy_node() const { return lazy_node_; }
    void sync() const { materialize_if_needed(); }

    // ---- host data access (CPU tensors only: DeviceError::cpu_only on GPU)
    void *data();
    const void *data() const;
    template <typename T> T *typed_data() {
        check_typed(dtype_of<T>::value);
        return static_cast<T *>(data());
    }
    template <typename T> const T *typed_data() const {
        check_typed(dtype_of<T>::value);
        return static_cast<const T *>(data());
    }
    template <typename T> T item(const std::vector<size_t> &indices) const { return static_cast<T>(item_as_double(indices)); }
    // single-element tensors; a GPU tensor is brought to the host first
    template <typename T> T item() const {
        if (size() != 1) throw ValueError("item() requires tensor with exactly 1 element, got " + std::to_string(size()));
        return static_cast<T>(cpu().item_as_double(std::vector<size_t>(ndim(), 0)));
    }
    template <typename T> void set_item(const std::vector<size_t> &indices, const T &value) { set_item_double(indices, static_cast<double>(value)); }
    template <typename T> void fill(const T &value) { fill_double(static_cast<double>(value)); }

    // ---- views and layout
    Tensor ascontiguousarray() const; // a lazy GPU tensor is returned as is (src/tensor/tensor.cpp:503-508)
    Tensor contiguous() const { return ascontiguousarray(); }
    Tensor reshape(const Shape &new_shape) const;
    Tensor reshape(std::initializer_list<size_t> new_shape) const { return reshape(Shape(new_shape)); }
    Tensor transpose() const;
    Tensor transpose(const std::vector<int> &axes) const;
    Tensor permute(const std::vector<int> &axes) const { return transpose(axes); }
    Tensor squeeze(int axis = -1) const;
    Tensor unsqueeze(int axis) const;
    // one Slice per leading dimension; a view of materialised storage, a lazy Slice node on a lazy GPU tensor
    Tensor slice(const std::vector<Slice> &slice_args) const;
    std::vector<Tensor> chunk(size_t n_chunks, int axis = 0) const;

    // ---- device and dtype
    Tensor to(Device device) const;
    Tensor cpu() const { return to(Device::CPU); }
    Tensor gpu() const { return to(Device::GPU); }
    Tensor astype(DType new_dtype) const;
    Tensor half() const { return astype(DType::Float16); }
    Tensor bfloat16() const { return astype(DType::BFloat16); }
    Tensor to_float() const { return astype(DType::Float32); }

    // |a - b| <= atol + rtol * |b| elementwise (src/tensor/tensor.cpp:1761-1775)
    bool allclose(const Tensor &other, double rtol = 1e-5, double atol = 1e-8) const;

    // ---- reductions / activations as members
    Tensor sum(int axis = -1, bool keep_dims = false) const;
    Tensor sum(const std::vector<int> &axes, bool keep_dims = false) const;
    Tensor mean(int axis = -1, bool keep_dims = false) const;
    Tensor mean(const std::vector<int> &axes, bool keep_dims = false) const;
    Tensor max(int axis = -1, bool keep_dims = false) const;
    Tensor min(int axis = -1, bool keep_dims = false) const;
    Tensor argmax(int axis = -1, bool keep_dims = false) const;
    Tensor argmin(int axis = -1, bool keep_dims = false) const;
    Tensor softmax(int axis = -1) const;
    Tensor log_softmax(int axis = -1) const;
    Tensor relu() const;
    Tensor gelu() const;
    Tensor sigmoid() const;
    Tensor silu() const;
    Tensor tanh() const;
    Tensor glu(int dim = -1) const;
    // the NumPy-style members of include/axiom/tensor.hpp:330-437
    Tensor leaky_relu(float negative_slope = 0.01f) const;
    Tensor sign() const;
    Tensor floor() const;
    Tensor ceil() const;
    Tensor trunc() const;
    Tensor round(int decimals = 0) const;
    Tensor cbrt() const;
    Tensor isnan() const;
    Tensor isinf() const;
    Tensor isfinite() const;
    Tensor clip(double min_val, double max_val) const;
    Tensor where(const Tensor &condition, const Tensor &other) const; // condition ? *this : other
    Tensor prod(int axis = -1, bool keep_dims = false) const;
    Tensor prod(const std::vector<int> &axes, bool keep_dims = false) const;
    Tensor any(int axis = -1, bool keep_dims = false) const;
    Tensor any(const std::vector<int> &axes, bool keep_dims = false) const;
    Tensor all(int axis = -1, bool keep_dims = false) const;
    Tensor all(const std::vector<int> &axes, bool keep_dims = false) const;
    Tensor to_bool() const { return astype(DType::Bool); }
    Tensor masked_fill(const Tensor &mask, float value) const;
    Tensor masked_fill(const Tensor &mask, double value) const;
    Tensor matmul(const Tensor &other, bool transpose_self = false, bool transpose_other = false) const;

    // ---- factories: built on the host, then moved (src/tensor/tensor.cpp:1785-1935)
    static Tensor zeros(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor ones(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor empty(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor eye(size_t n, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor arange(int64_t start, int64_t end, int64_t step = 1, DType dtype = DType::Int64, Device device = Device::CPU);
    template <typename T> static Tensor full(const Shape &shape, const T &value, Device device = Device::CPU) {
        Tensor t(shape, dtype_of<T>::value, Device::CPU);
        t.fill_double(static_cast<double>(value));
        return device == Device::GPU ? t.to(device) : t;
    }
    static Tensor randn(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor rand(const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    static Tensor uniform(double low, double high, const Shape &shape, DType dtype = DType::Float32, Device device = Device::CPU);
    template <typename T> static Tensor from_data(const T *data, const Shape &shape, Device device = Device::CPU) {
        Tensor t(shape, dtype_of<T>::value, Device::CPU);
        t.copy_from_host(data, t.size() * sizeof(T));
        return device == Device::GPU ? t.to(device) : t;
    }
    static Tensor zeros_like(const Tensor &p) { return zeros(p.shape(), p.dtype(), p.device()); }
    static Tensor ones_like(const Tensor &p) { return ones(p.shape(), p.dtype(), p.device()); }
    static void manual_seed(uint64_t seed);

    // copies raw bytes into a contiguous CPU tensor's storage
    void copy_from_host(const void *src, size_t bytes);

  private:
    void materialize_if_needed() const;
    void check_typed(DType want) const;
    double item_as_double(const std::vector<size_t> &indices) const;
    void set_item_double(const std::vector<size_t> &indices, double v);
    void fill_double(double v);

    mutable std::shared_ptr<Storage> storage_;
    mutable Shape shape_;
    mutable Strides strides_;
    DType dtype_ = DType::Float32;
    mutable size_t offset_ = 0;
    mutable std::shared_ptr<graph::GraphNode> lazy_node_;
};

// arithmetic operators; a scalar becomes a {1}-shaped tensor of the tensor's dtype on its
// device (include/axiom/tensor_operators.hpp:196-235)
Tensor operator+(const Tensor &a, const Tensor &b);
Tensor operator-(const Tensor &a, const Tensor &b);
Tensor operator*(const Tensor &a, const Tensor &b);
Tensor operator/(const Tensor &a, const Tensor &b);
Tensor make_scalar_like(const Tensor &t, double value);
// comparisons give Bool tensors (include/axiom/tensor_operators.hpp)
Tensor operator<(const Tensor &a, const Tensor &b);
Tensor operator<=(const Tensor &a, const Tensor &b);
Tensor operator>(const Tensor &a, const Tensor &b);
Tensor operator>=(const Tensor &a, const Tensor &b);
Tensor operator==(const Tensor &a, const Tensor &b);
Tensor operator!=(const Tensor &a, const Tensor &b);
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator<(const Tensor &a, S s) { return a < make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator<=(const Tensor &a, S s) { return a <= make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator>(const Tensor &a, S s) { return a > make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator>=(const Tensor &a, S s) { return a >= make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator==(const Tensor &a, S s) { return a == make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator!=(const Tensor &a, S s) { return a != make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator<(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) < a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator<=(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) <= a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator>(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) > a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator>=(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) >= a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator+(const Tensor &a, S s) { return a + make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator-(const Tensor &a, S s) { return a - make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator*(const Tensor &a, S s) { return a * make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator/(const Tensor &a, S s) { return a / make_scalar_like(a, static_cast<double>(s)); }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator+(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) + a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator-(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) - a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator*(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) * a; }
template <typename S, typename = std::enable_if_t<std::is_arithmetic_v<S>>> Tensor operator/(S s, const Tensor &a) { return make_scalar_like(a, static_cast<double>(s)) / a; }

} // namespace axiom
