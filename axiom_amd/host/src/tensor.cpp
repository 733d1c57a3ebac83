// axiom::Tensor for the gfx950 host layer (behaviour of src/tensor/tensor.cpp for the
// hot-path subset: views, device moves, dtype casts, factories, allclose).
#include <map>
#include <mutex>
#include "axiom/tensor.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>

#include "axiom/graph/graph_node.hpp"
#include "axiom/graph/graph_registry.hpp"
#include "axiom/operations.hpp"
#include "axiom/random.hpp"
#include "hip_call.hpp"

namespace axiom {

Tensor::Tensor() = default;

Tensor::Tensor(const Shape &shape, DType dtype, Device device)
    : storage_(make_storage(ShapeUtils::size(shape) * dtype_size(dtype), device)), shape_(shape),
      strides_(ShapeUtils::contiguous_strides(shape, dtype_size(dtype))), dtype_(dtype) {}

Tensor::Tensor(std::initializer_list<size_t> shape, DType dtype, Device device) : Tensor(Shape(shape), dtype, device) {}

Tensor::Tensor(std::shared_ptr<Storage> storage, const Shape &shape, const Strides &strides, DType dtype, size_t offset)
    : storage_(std::move(storage)), shape_(shape), strides_(strides), dtype_(dtype), offset_(offset) {}

Tensor::Tensor(std::shared_ptr<graph::GraphNode> lazy_node) : dtype_(lazy_node->output_dtype), lazy_node_(std::move(lazy_node)) {}

// ---------------------------------------------------------------- metadata
const Shape &Tensor::shape() const { return lazy_node_ ? lazy_node_->output_shape : shape_; }
DType Tensor::dtype() const { return lazy_node_ ? lazy_node_->output_dtype : dtype_; }
Device Tensor::device() const {
    if (lazy_node_) return lazy_node_->target_device;
    return storage_ ? storage_->device() : Device::CPU;
}

// src/tensor/tensor.cpp:255-273: run the graph once, then behave like an eager tensor
void Tensor::materialize_if_needed() const {
    if (!lazy_node_) return;
    if (!lazy_node_->is_materialized_) graph::GraphRegistry::materialize(lazy_node_.get());
    storage_ = lazy_node_->cached_result_;
    shape_ = lazy_node_->cached_shape_;
    strides_ = lazy_node_->cached_strides_;
    offset_ = lazy_node_->cached_offset_;
    lazy_node_.reset();
}

const Strides &Tensor::strides() const {
    materialize_if_needed();
    return strides_;
}
size_t Tensor::offset() const {
    materialize_if_needed();
    return offset_;
}
bool Tensor::is_contiguous() const {
    materialize_if_needed();
    return ShapeUtils::is_contiguous(shape_, strides_, dtype_size(dtype_));
}
std::shared_ptr<Storage> Tensor::storage() const {
    materialize_if_needed();
    return storage_;
}

// ------------------------------------------------------------- host access
void *Tensor::data() {
    materialize_if_needed();
    if (!storage_) throw ValueError("tensor has no storage");
    if (storage_->device() != Device::CPU) throw DeviceError::cpu_only("data()");
    return static_cast<char *>(storage_->data()) + offset_;
}
const void *Tensor::data() const { return const_cast<Tensor *>(this)->data(); }

void Tensor::check_typed(DType want) const {
    if (device() != Device::CPU) throw DeviceError::cpu_only("typed_data()");
    if (want != dtype() && !(want == DType::UInt8 && dtype() == DType::Bool) && !(want == DType::Bool && dtype() == DType::UInt8))
        throw TypeError("typed_data<" + dtype_name(want) + ">() on a " + dtype_name(dtype()) + " tensor");
}

double Tensor::item_as_double(const std::vector<size_t> &indices) const {
    if (device() != Device::CPU) throw DeviceError::cpu_only("item()");
    materialize_if_needed();
    if (indices.size() != shape_.size()) throw IndexError("item(): expected " + std::to_string(shape_.size()) + " indices");
    int64_t off = static_cast<int64_t>(offset_);
    for (size_t i = 0; i < indices.size(); ++i) {
        if (indices[i] >= shape_[i]) throw IndexError("item(): index out of range");
        off += static_cast<int64_t>(indices[i]) * strides_[i];
    }
    return load_scalar(static_cast<const char *>(storage_->data()) + off, dtype_);
}

void Tensor::set_item_double(const std::vector<size_t> &indices, double v) {
    if (device() != Device::CPU) throw DeviceError::cpu_only("set_item()");
    materialize_if_needed();
    if (indices.size() != shape_.size()) throw IndexError("set_item(): expected " + std::to_string(shape_.size()) + " indices");
    int64_t off = static_cast<int64_t>(offset_);
    for (size_t i = 0; i < indices.size(); ++i) {
        if (indices[i] >= shape_[i]) throw IndexError("set_item(): index out of range");
        off += static_cast<int64_t>(indices[i]) * strides_[i];
    }
    store_scalar(static_cast<char *>(storage_->data()) + off, dtype_, v);
}

void Tensor::fill_double(double v) {
    if (device() != Device::CPU) {
        Tensor h(shape(), dtype(), Device::CPU);
        h.fill_double(v);
        *this = h.to(Device::GPU);
        return;
    }
    materialize_if_needed();
    if (!is_contiguous()) throw RuntimeError::not_implemented("fill() on a non-contiguous view");
    char *p = static_cast<char *>(data());
    const size_t n = size(), isz = dtype_size(dtype_);
    if (n == 0) return;
    store_scalar(p, dtype_, v);
    for (size_t i = 1; i < n; ++i) std::memcpy(p + i * isz, p, isz);
}

void Tensor::copy_from_host(const void *src, size_t bytes) {
    if (device() != Device::CPU || !is_contiguous()) throw DeviceError::cpu_only("copy_from_host()");
    if (bytes > size() * dtype_size(dtype_)) throw ValueError("copy_from_host(): source larger than the tensor");
    if (bytes) std::memcpy(data(), src, bytes);
}

// ------------------------------------------------------------------- views
namespace {

// visits every element of a strided view in row-major order
template <typename F> void for_each_offset(const Shape &shape, const Strides &strides, int64_t base, F f) {
    const size_t nd = shape.size();
    const size_t total = ShapeUtils::size(shape);
    std::vector<size_t> idx(nd, 0);
    int64_t off = base;
    for (size_t n = 0; n < total; ++n) {
        f(n, off);
        for (size_t d = nd; d-- > 0;) {
            off += strides[d];
            if (++idx[d] < shape[d]) break;
            off -= static_cast<int64_t>(shape[d]) * strides[d];
            idx[d] = 0;
        }
    }
}

// element strides for the C ABI; byte strides of a view are multiples of the item size
std::vector<int64_t> elem_strides(const Strides &st, size_t itemsize) {
    std::vector<int64_t> e(st.size());
    for (size_t i = 0; i < st.size(); ++i) e[i] = st[i] / static_cast<int64_t>(itemsize);
    return e;
}

bool gpu_kernel_dtype(DType d) { return d == DType::Float32 || d == DType::Float16 || d == DType::BFloat16; }

} // namespace

Tensor Tensor::ascontiguousarray() const {
    if (lazy_node_ && lazy_node_->target_device == Device::GPU && !lazy_node_->is_materialized_) return *this;
    materialize_if_needed();
    if (!storage_ || is_contiguous()) return *this;
    for (int64_t s : strides_)
        if (s < 0) throw RuntimeError::not_implemented("negative strides (flipped views)");
    Tensor out(shape_, dtype_, device());
    const size_t isz = dtype_size(dtype_);
    if (device() == Device::CPU) {
        const char *src = static_cast<const char *>(storage_->data());
        char *dst = static_cast<char *>(out.data());
        for_each_offset(shape_, strides_, static_cast<int64_t>(offset_), [&](size_t n, int64_t off) { std::memcpy(dst + n * isz, src + off, isz); });
        return out;
    }
    // the role of gpu_make_contiguous / gather_strided (src/backends/metal/kernels.metal:33-149)
    if (shape_.size() > AXHIP_MAX_DIMS) throw RuntimeError::not_implemented("GPU gather of more than 8 dimensions");
    std::vector<int64_t> shp(shape_.begin(), shape_.end()), est = elem_strides(strides_, isz);
    if (gpu_kernel_dtype(dtype_)) {
        const int dt = detail::to_axhip_dtype(dtype_);
        AXHIP_CALL(axhip_strided_copy(static_cast<const char *>(storage_->raw()) + offset_, dt, out.storage_->raw(), dt,
                                      static_cast<int32_t>(shp.size()), shp.data(), est.data(), nullptr));
        return out;
    }
    return cpu().ascontiguousarray().to(Device::GPU); // masks and integer tensors: small, via the host
}

Tensor Tensor::reshape(const Shape &new_shape) const {
    if (ShapeUtils::size(new_shape) != size()) throw ShapeError("cannot reshape tensor of size " + std::to_string(size()) + " to size " + std::to_string(ShapeUtils::size(new_shape)));
    if (lazy_node_ && lazy_node_->target_device == Device::GPU && !lazy_node_->is_materialized_)
        return graph::GraphRegistry::create_lazy_reshape(*this, new_shape); // src/tensor/tensor.cpp:623-629
    Tensor c = ascontiguousarray();
    return Tensor(c.storage_, new_shape, ShapeUtils::contiguous_strides(new_shape, dtype_size(c.dtype_)), c.dtype_, c.offset_);
}

Tensor Tensor::transpose() const {
    std::vector<int> axes(ndim());
    std::iota(axes.rbegin(), axes.rend(), 0);
    return transpose(axes);
}

Tensor Tensor::transpose(const std::vector<int> &axes) const {
    const int nd = static_cast<int>(ndim());
    if (static_cast<int>(axes.size()) != nd) throw ShapeError("transpose: axes must name every dimension");
    std::vector<int> norm(nd);
    std::vector<bool> seen(nd, false);
    for (int i = 0; i < nd; ++i) {
        norm[i] = ShapeUtils::normalize_axis(axes[i], nd);
        if (seen[norm[i]]) throw ShapeError("transpose: repeated axis");
        seen[norm[i]] = true;
    }
    if (lazy_node_ && lazy_node_->target_device == Device::GPU && !lazy_node_->is_materialized_)
        return graph::GraphRegistry::create_lazy_transpose(*this, norm); // src/tensor/tensor.cpp:716-730
    materialize_if_needed();
    Shape s(nd);
    Strides st(nd);
    for (int i = 0; i < nd; ++i) {
        s[i] = shape_[norm[i]];
        st[i] = strides_[norm[i]];
    }
    return Tensor(storage_, s, st, dtype_, offset_);
}

// Python slice semantics per dimension (src/tensor/tensor.cpp slice(); include/axiom/indexing.hpp:13-22)
Tensor Tensor::slice(const std::vector<Slice> &args) const {
    const Shape &in = shape();
    if (args.size() > in.size()) throw IndexError("slice: " + std::to_string(args.size()) + " slices for a tensor with " + std::to_string(in.size()) + " dimensions");
    const size_t nd = in.size();
    std::vector<int64_t> starts(nd, 0), ends(in.begin(), in.end()), steps(nd, 1);
    Shape out = in;
    for (size_t d = 0; d < args.size(); ++d) {
        const int64_t n = static_cast<int64_t>(in[d]), step = args[d].step.value_or(1);
        if (step <= 0) throw ValueError("slice: only positive steps are supported");
        int64_t b = args[d].start.value_or(0), e = args[d].stop.value_or(n);
        if (b < 0) b += n;
        if (e < 0) e += n;
        b = std::min(std::max<int64_t>(b, 0), n);
        e = std::min(std::max<int64_t>(e, b), n);
        starts[d] = b;
        ends[d] = e;
        steps[d] = step;
        out[d] = static_cast<size_t>((e - b + step - 1) / step);
    }
    if (lazy_node_ && lazy_node_->target_device == Device::GPU && !lazy_node_->is_materialized_)
        return graph::GraphRegistry::create_lazy_slice(*this, starts, ends, steps, out);
    materialize_if_needed();
    Strides st = strides_;
    size_t off = offset_;
    for (size_t d = 0; d < nd; ++d) {
        off += static_cast<size_t>(starts[d] * strides_[d]);
        st[d] = strides_[d] * steps[d];
    }
    return Tensor(storage_, out, st, dtype_, off);
}

std::vector<Tensor> Tensor::chunk(size_t n_chunks, int axis) const {
    if (n_chunks == 0) throw ValueError("chunk: the number of chunks must be positive");
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(ndim()));
    const size_t n = shape()[a], each = (n + n_chunks - 1) / n_chunks;
    std::vector<Tensor> out;
    for (size_t b = 0; b < n; b += each) {
        std::vector<Slice> args(a + 1);
        args[a] = Slice(static_cast<int64_t>(b), static_cast<int64_t>(std::min(n, b + each)));
        out.push_back(slice(args));
    }
    return out;
}

Tensor Tensor::squeeze(int axis) const {
    const int a = ShapeUtils::normalize_axis(axis, static_cast<int>(ndim()));
    if (shape()[a] != 1) throw ShapeError("squeeze: dimension " + std::to_string(a) + " has extent " + std::to_string(shape()[a]));
    Shape s = shape();
    s.erase(s.begin() + a);
    if (is_lazy() && device() == Device::GPU) return reshape(s);
    materialize_if_needed();
    Strides st = strides_;
    st.erase(st.begin() + a);
    return Tensor(storage_, s, st, dtype_, offset_);
}

Tensor Tensor::unsqueeze(int axis) const {
    const int nd = static_cast<int>(ndim()) + 1;
    const int a = ShapeUtils::normalize_axis(axis, nd);
    Shape s = shape();
    s.insert(s.begin() + a, 1);
    if (is_lazy() && device() == Device::GPU) return reshape(s);
    materialize_if_needed();
    Strides st = strides_;
    st.insert(st.begin() + a, a < static_cast<int>(st.size()) ? st[a] * static_cast<int64_t>(shape_[a]) : static_cast<int64_t>(dtype_size(dtype_)));
    return Tensor(storage_, s, st, dtype_, offset_);
}

// ------------------------------------------------------------ device, dtype
// src/tensor/tensor.cpp:1625-1638 (the discrete-memory branch; there is no shared-memory retag)
Tensor Tensor::to(Device target) const {
    if (empty()) return *this;
    if (device() == target) return *this;
    materialize_if_needed();
    Tensor src = ascontiguousarray();
    Tensor out(src.shape_, src.dtype_, target);
    const size_t bytes = src.size() * dtype_size(src.dtype_);
    if (bytes == 0) return out;
    if (target == Device::GPU) {
        AXHIP_CALL(axhip_memcpy_h2d_async(out.storage_->raw(), static_cast<const char *>(src.storage_->raw()) + src.offset_, bytes, nullptr));
        AXHIP_CALL(axhip_stream_sync(nullptr));
    } else { // waits for every kernel queued before it: the auto-synchronisation of .cpu()
        AXHIP_CALL(axhip_memcpy_d2h_async(out.storage_->raw(), static_cast<const char *>(src.storage_->raw()) + src.offset_, bytes, nullptr));
        AXHIP_CALL(axhip_stream_sync(nullptr));
    }
    return out;
}

Tensor Tensor::astype(DType nd) const {
    if (nd == dtype()) return *this;
    // among the kernel types and Bool the GPU Cast is a graph node: it folds into the kernel next to it
    if (device() == Device::GPU && !empty() && (gpu_kernel_dtype(dtype_) || dtype_ == DType::Bool) && (gpu_kernel_dtype(nd) || nd == DType::Bool))
        return ops::cast(*this, nd);
    materialize_if_needed();
    if (device() == Device::GPU) {
        if (gpu_kernel_dtype(dtype_) && gpu_kernel_dtype(nd)) { // the GPU Cast op (src/tensor/tensor.cpp:1665-1670)
            for (int64_t s : strides_)
                if (s < 0) throw RuntimeError::not_implemented("negative strides (flipped views)");
            Tensor out(shape_, nd, Device::GPU);
            std::vector<int64_t> shp(shape_.begin(), shape_.end()), est = elem_strides(strides_, dtype_size(dtype_));
            AXHIP_CALL(axhip_strided_copy(static_cast<const char *>(storage_->raw()) + offset_, detail::to_axhip_dtype(dtype_), out.storage_->raw(),
                                          detail::to_axhip_dtype(nd), static_cast<int32_t>(shp.size()), shp.data(), est.data(), nullptr));
            return out;
        }
        return cpu().astype(nd).to(Device::GPU);
    }
    Tensor out(shape_, nd, Device::CPU);
    const char *src = static_cast<const char *>(storage_->data());
    char *dst = static_cast<char *>(out.data());
    const size_t osz = dtype_size(nd);
    const DType sd = dtype_;
    for_each_offset(shape_, strides_, static_cast<int64_t>(offset_), [&](size_t n, int64_t off) { store_scalar(dst + n * osz, nd, load_scalar(src + off, sd)); });
    return out;
}

bool Tensor::allclose(const Tensor &other, double rtol, double atol) const {
    if (shape() != other.shape()) return false;
    Tensor a = cpu(), b = other.cpu();
    a.materialize_if_needed();
    b.materialize_if_needed();
    std::vector<double> av(a.size()), bv(b.size());
    const char *ap = static_cast<const char *>(a.storage_->data()), *bp = static_cast<const char *>(b.storage_->data());
    for_each_offset(a.shape_, a.strides_, static_cast<int64_t>(a.offset_), [&](size_t n, int64_t off) { av[n] = load_scalar(ap + off, a.dtype_); });
    for_each_offset(b.shape_, b.strides_, static_cast<int64_t>(b.offset_), [&](size_t n, int64_t off) { bv[n] = load_scalar(bp + off, b.dtype_); });
    for (size_t i = 0; i < av.size(); ++i) {
        if (std::isnan(av[i]) || std::isnan(bv[i])) return false;
        if (std::fabs(av[i] - bv[i]) > atol + rtol * std::fabs(bv[i])) return false;
    }
    return true;
}

// ---------------------------------------------------------------- members
Tensor Tensor::sum(int axis, bool keep_dims) const { return ops::sum(*this, {axis}, keep_dims); }
Tensor Tensor::sum(const std::vector<int> &axes, bool keep_dims) const { return ops::sum(*this, axes, keep_dims); }
Tensor Tensor::mean(int axis, bool keep_dims) const { return ops::mean(*this, {axis}, keep_dims); }
Tensor Tensor::mean(const std::vector<int> &axes, bool keep_dims) const { return ops::mean(*this, axes, keep_dims); }
Tensor Tensor::max(int axis, bool keep_dims) const { return ops::max(*this, {axis}, keep_dims); }
Tensor Tensor::min(int axis, bool keep_dims) const { return ops::min(*this, {axis}, keep_dims); }
Tensor Tensor::argmax(int axis, bool keep_dims) const { return ops::argmax(*this, axis, keep_dims); }
Tensor Tensor::argmin(int axis, bool keep_dims) const { return ops::argmin(*this, axis, keep_dims); }
Tensor Tensor::softmax(int axis) const { return ops::softmax(*this, axis); }
Tensor Tensor::log_softmax(int axis) const { return ops::log_softmax(*this, axis); }
Tensor Tensor::relu() const { return ops::relu(*this); }
Tensor Tensor::gelu() const { return ops::gelu(*this); }
Tensor Tensor::leaky_relu(float negative_slope) const { return ops::leaky_relu(*this, negative_slope); }
Tensor Tensor::sign() const { return ops::sign(*this); }
Tensor Tensor::floor() const { return ops::floor(*this); }
Tensor Tensor::ceil() const { return ops::ceil(*this); }
Tensor Tensor::trunc() const { return ops::trunc(*this); }
Tensor Tensor::round(int decimals) const { return ops::round(*this, decimals); }
Tensor Tensor::cbrt() const { return ops::cbrt(*this); }
Tensor Tensor::isnan() const { return ops::isnan(*this); }
Tensor Tensor::isinf() const { return ops::isinf(*this); }
Tensor Tensor::isfinite() const { return ops::isfinite(*this); }
Tensor Tensor::clip(double lo, double hi) const { return ops::clip(*this, make_scalar_like(*this, lo), make_scalar_like(*this, hi)); }
Tensor Tensor::where(const Tensor &condition, const Tensor &other) const { return ops::where(condition, *this, other); }
Tensor Tensor::prod(int axis, bool keep_dims) const { return ops::prod(*this, {axis}, keep_dims); }
Tensor Tensor::prod(const std::vector<int> &axes, bool keep_dims) const { return ops::prod(*this, axes, keep_dims); }
Tensor Tensor::any(int axis, bool keep_dims) const { return ops::any(*this, {axis}, keep_dims); }
Tensor Tensor::any(const std::vector<int> &axes, bool keep_dims) const { return ops::any(*this, axes, keep_dims); }
Tensor Tensor::all(int axis, bool keep_dims) const { return ops::all(*this, {axis}, keep_dims); }
Tensor Tensor::all(const std::vector<int> &axes, bool keep_dims) const { return ops::all(*this, axes, keep_dims); }
Tensor Tensor::sigmoid() const { return ops::sigmoid(*this); }
Tensor Tensor::silu() const { return ops::silu(*this); }
Tensor Tensor::tanh() const { return ops::tanh(*this); }
Tensor Tensor::glu(int dim) const { return ops::glu(*this, dim); }
Tensor Tensor::masked_fill(const Tensor &mask, float value) const { return ops::masked_fill(*this, mask, value); }
Tensor Tensor::masked_fill(const Tensor &mask, double value) const { return ops::masked_fill(*this, mask, value); }
Tensor Tensor::matmul(const Tensor &o, bool ta, bool tb) const { return ops::matmul(*this, o, ta, tb); }

// --------------------------------------------------------------- factories
Tensor Tensor::zeros(const Shape &shape, DType dtype, Device device) {
    Tensor t(shape, dtype, Device::CPU);
    if (t.size()) std::memset(t.data(), 0, t.size() * dtype_size(dtype));
    return device == Device::GPU ? t.to(device) : t;
}
Tensor Tensor::ones(const Shape &shape, DType dtype, Device device) {
    Tensor t(shape, dtype, Device::CPU);
    t.fill_double(1.0);
    return device == Device::GPU ? t.to(device) : t;
}
Tensor Tensor::empty(const Shape &shape, DType dtype, Device device) { return Tensor(shape, dtype, device); }
Tensor Tensor::eye(size_t n, DType dtype, Device device) {
    Tensor t = zeros({n, n}, dtype, Device::CPU);
    for (size_t i = 0; i < n; ++i) t.set_item_double({i, i}, 1.0);
    return device == Device::GPU ? t.to(device) : t;
}

Tensor Tensor::arange(int64_t start, int64_t end, int64_t step, DType dtype, Device device) {
    if (step == 0) throw ValueError("arange: step must not be zero");
    const int64_t n = step > 0 ? std::max<int64_t>(0, (end - start + step - 1) / step) : std::max<int64_t>(0, (start - end - step - 1) / -step);
    Tensor t(Shape{static_cast<size_t>(n)}, dtype, Device::CPU);
    for (int64_t i = 0; i < n; ++i) t.set_item_double({static_cast<size_t>(i)}, static_cast<double>(start + i * step));
    return device == Device::GPU ? t.to(device) : t;
}

// half types draw normal<float> and cast (src/tensor/tensor.cpp:1889-1899)
Tensor Tensor::randn(const Shape &shape, DType dtype, Device device) {
    if (!is_floating_dtype(dtype)) throw TypeError("randn needs a floating dtype");
    Tensor t(shape, dtype, Device::CPU);
    auto &rng = RandomGenerator::instance();
    char *p = static_cast<char *>(t.data());
    const size_t isz = dtype_size(dtype);
    for (size_t i = 0; i < t.size(); ++i) {
        const double v = dtype == DType::Float64 ? rng.normal<double>() : static_cast<double>(rng.normal<float>());
        store_scalar(p + i * isz, dtype, v);
    }
    return device == Device::GPU ? t.to(device) : t;
}
Tensor Tensor::uniform(double low, double high, const Shape &shape, DType dtype, Device device) {
    if (!is_floating_dtype(dtype)) throw TypeError("uniform needs a floating dtype");
    Tensor t(shape, dtype, Device::CPU);
    auto &rng = RandomGenerator::instance();
    char *p = static_cast<char *>(t.data());
    const size_t isz = dtype_size(dtype);
    for (size_t i = 0; i < t.size(); ++i) {
        const double v = dtype == DType::Float64 ? rng.uniform<double>(low, high) : static_cast<double>(rng.uniform<float>(static_cast<float>(low), static_cast<float>(high)));
        store_scalar(p + i * isz, dtype, v);
    }
    return device == Device::GPU ? t.to(device) : t;
}
Tensor Tensor::rand(const Shape &shape, DType dtype, Device device) { return uniform(0.0, 1.0, shape, dtype, device); }
void Tensor::manual_seed(uint64_t seed) { RandomGenerator::instance().seed(seed); }

// --------------------------------------------------------------- operators
// src/tensor/tensor_operators.hpp:196-235: a scalar operand becomes a {1} tensor of the tensor's dtype on its device.
// On the GPU that is an upload and a wait per expression (about 25 us, a third of the chain it feeds), so the device
// copies of recently used (value, dtype) pairs are kept: they are constants nothing writes to.
Tensor make_scalar_like(const Tensor &t, double value) {
    Tensor s(Shape{1}, t.dtype(), Device::CPU);
    s.set_item<double>({0}, value);
    if (t.device() != Device::GPU) return s;
    struct Key {
        uint64_t bits;
        int dtype;
        bool operator<(const Key &o) const { return bits != o.bits ? bits < o.bits : dtype < o.dtype; }
    };
    static std::mutex mu;
    static std::map<Key, Tensor> cache;
    Key key{0, static_cast<int>(t.dtype())};
    std::memcpy(&key.bits, &value, sizeof(value));
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = cache.find(key);
        if (it != cache.end()) return it->second;
    }
    Tensor d = s.to(Device::GPU);
    std::lock_guard<std::mutex> lock(mu);
    if (cache.size() >= 256) cache.clear();
    cache.emplace(key, d);
    return d;
}
Tensor operator+(const Tensor &a, const Tensor &b) { return ops::add(a, b); }
Tensor operator<(const Tensor &a, const Tensor &b) { return ops::less(a, b); }
Tensor operator<=(const Tensor &a, const Tensor &b) { return ops::less_equal(a, b); }
Tensor operator>(const Tensor &a, const Tensor &b) { return ops::greater(a, b); }
Tensor operator>=(const Tensor &a, const Tensor &b) { return ops::greater_equal(a, b); }
Tensor operator==(const Tensor &a, const Tensor &b) { return ops::equal(a, b); }
Tensor operator!=(const Tensor &a, const Tensor &b) { return ops::not_equal(a, b); }
Tensor operator-(const Tensor &a, const Tensor &b) { return ops::subtract(a, b); }
Tensor operator*(const Tensor &a, const Tensor &b) { return ops::multiply(a, b); }
Tensor operator/(const Tensor &a, const Tensor &b) { return ops::divide(a, b); }

} // namespace axiom
