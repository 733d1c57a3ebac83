// dtype, shape, storage, availability and RNG plumbing of the host layer.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <sstream>
#include <unordered_map>

#include "axhip.h"
#include "axiom/dtype.hpp"
#include "axiom/error.hpp"
#include "axiom/random.hpp"
#include "axiom/shape.hpp"
#include "axiom/storage.hpp"
#include "axiom/system.hpp"
#include "hip_call.hpp"

namespace axiom {

// ------------------------------------------------------------------ dtype
std::string dtype_name(DType d) {
    static const char *names[] = {"bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64",
                                  "float16", "bfloat16", "float32", "float64", "complex64", "complex128"};
    return names[static_cast<int>(d)];
}

// binary16 <-> binary32, round to nearest even, subnormals and infinities included
float16_t::float16_t(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag = x & 0x7FFFFFFFu;
    uint32_t h;
    if (mag > 0x7F800000u) {
        h = 0x7E00u; // NaN
    } else if (mag >= 0x47800000u) {
        h = 0x7C00u; // overflow -> inf (65520 and above round to inf)
    } else if (mag >= 0x38800000u) { // normal half
        const uint32_t m = mag - 0x38000000u; // rebias exponent by 112
        h = (m + 0xFFFu + ((m >> 13) & 1u)) >> 13;
    } else if (mag >= 0x33000000u) { // subnormal half
        const int e = static_cast<int>(mag >> 23);
        const uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;
        const int shift = 126 - e; // 14..24
        const uint32_t lsb = (man >> shift) & 1u;
        h = (man + (1u << (shift - 1)) - 1u + lsb) >> shift;
    } else {
        h = 0;
    }
    bits = static_cast<uint16_t>(sign | h);
}

float16_t::operator float() const {
    const uint32_t sign = (static_cast<uint32_t>(bits) & 0x8000u) << 16;
    const uint32_t e = (bits >> 10) & 0x1Fu, m = bits & 0x3FFu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else { // subnormal: normalise
            int k = 0;
            uint32_t mm = m;
            while (!(mm & 0x400u)) {
                mm <<= 1;
                ++k;
            }
            x = sign | ((113u - static_cast<uint32_t>(k)) << 23) | ((mm & 0x3FFu) << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7F800000u | (m << 13);
    } else {
        x = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

double load_scalar(const void *p, DType d) {
    switch (d) {
    case DType::Bool: return *static_cast<const uint8_t *>(p) != 0;
    case DType::Int8: return *static_cast<const int8_t *>(p);
    case DType::Int16: return *static_cast<const int16_t *>(p);
    case DType::Int32: return *static_cast<const int32_t *>(p);
    case DType::Int64: return static_cast<double>(*static_cast<const int64_t *>(p));
    case DType::UInt8: return *static_cast<const uint8_t *>(p);
    case DType::UInt16: return *static_cast<const uint16_t *>(p);
    case DType::UInt32: return *static_cast<const uint32_t *>(p);
    case DType::UInt64: return static_cast<double>(*static_cast<const uint64_t *>(p));
    case DType::Float16: return static_cast<float>(*static_cast<const float16_t *>(p));
    case DType::BFloat16: return static_cast<float>(*static_cast<const bfloat16_t *>(p));
    case DType::Float32: return *static_cast<const float *>(p);
    case DType::Float64: return *static_cast<const double *>(p);
    default: throw TypeError("complex dtypes are not supported by this backend");
    }
}

void store_scalar(void *p, DType d, double v) {
    switch (d) {
    case DType::Bool: *static_cast<uint8_t *>(p) = v != 0.0; break;
    case DType::Int8: *static_cast<int8_t *>(p) = static_cast<int8_t>(v); break;
    case DType::Int16: *static_cast<int16_t *>(p) = static_cast<int16_t>(v); break;
    case DType::Int32: *static_cast<int32_t *>(p) = static_cast<int32_t>(v); break;
    case DType::Int64: *static_cast<int64_t *>(p) = static_cast<int64_t>(v); break;
    case DType::UInt8: *static_cast<uint8_t *>(p) = static_cast<uint8_t>(v); break;
    case DType::UInt16: *static_cast<uint16_t *>(p) = static_cast<uint16_t>(v); break;
    case DType::UInt32: *static_cast<uint32_t *>(p) = static_cast<uint32_t>(v); break;
    case DType::UInt64: *static_cast<uint64_t *>(p) = static_cast<uint64_t>(v); break;
    // a double that came from a float converts back exactly, so half types round once
    case DType::Float16: *static_cast<float16_t *>(p) = float16_t(static_cast<float>(v)); break;
    case DType::BFloat16: *static_cast<bfloat16_t *>(p) = bfloat16_t(static_cast<float>(v)); break;
    case DType::Float32: *static_cast<float *>(p) = static_cast<float>(v); break;
    case DType::Float64: *static_cast<double *>(p) = v; break;
    default: throw TypeError("complex dtypes are not supported by this backend");
    }
}

// ------------------------------------------------------------------ shape
size_t ShapeUtils::size(const Shape &s) {
    size_t n = 1;
    for (size_t d : s) n *= d;
    return n;
}

Strides ShapeUtils::contiguous_strides(const Shape &s, size_t itemsize) {
    Strides st(s.size());
    int64_t acc = static_cast<int64_t>(itemsize);
    for (size_t i = s.size(); i-- > 0;) {
        st[i] = acc;
        acc *= static_cast<int64_t>(s[i]);
    }
    return st;
}

bool ShapeUtils::is_contiguous(const Shape &s, const Strides &st, size_t itemsize) {
    int64_t acc = static_cast<int64_t>(itemsize);
    for (size_t i = s.size(); i-- > 0;) {
        if (s[i] != 1 && st[i] != acc) return false;
        acc *= static_cast<int64_t>(s[i]);
    }
    return true;
}

Shape ShapeUtils::broadcast(const Shape &a, const Shape &b) {
    const size_t n = std::max(a.size(), b.size());
    Shape out(n);
    for (size_t i = 0; i < n; ++i) {
        const size_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
        const size_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
        if (da != db && da != 1 && db != 1)
            throw ShapeError("shapes are not broadcastable: " + to_string(a) + " vs " + to_string(b));
        out[i] = da == 1 ? db : da;
    }
    return out;
}

std::string ShapeUtils::to_string(const Shape &s) {
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < s.size(); ++i) o << (i ? ", " : "") << s[i];
    o << "]";
    return o.str();
}

int ShapeUtils::normalize_axis(int axis, int ndim) {
    const int a = axis < 0 ? axis + ndim : axis;
    if (a < 0 || a >= ndim)
        throw ShapeError("axis " + std::to_string(axis) + " out of bounds for tensor with " + std::to_string(ndim) + " dimensions");
    return a;
}

// ---------------------------------------------------------------- storage
namespace {

class CpuStorage final : public Storage {
  public:
    explicit CpuStorage(size_t bytes) : bytes_(bytes) {
        ptr_ = bytes ? std::aligned_alloc(64, (bytes + 63) / 64 * 64) : nullptr;
        if (bytes && !ptr_) throw MemoryError("cannot allocate " + std::to_string(bytes) + " bytes of host memory");
    }
    ~CpuStorage() override { std::free(ptr_); }
    void *data() override { return ptr_; }
    const void *data() const override { return ptr_; }
    void *raw() const override { return ptr_; }
    size_t size_bytes() const override { return bytes_; }
    Device device() const override { return Device::CPU; }
    void copy_to(Storage &other) const override { other.copy_from(*this); }
    void copy_from(const Storage &other) override {
        const size_t n = std::min(bytes_, other.size_bytes());
        if (other.device() == Device::CPU) {
            if (n) std::memcpy(ptr_, other.raw(), n);
        } else { // device -> host: everything queued before the copy has run when it returns
            AXHIP_CALL(axhip_memcpy_d2h_async(ptr_, other.raw(), n, nullptr));
            AXHIP_CALL(axhip_stream_sync(nullptr));
        }
    }
    std::unique_ptr<Storage> clone() const override {
        auto c = std::make_unique<CpuStorage>(bytes_);
        c->copy_from(*this);
        return c;
    }

  private:
    void *ptr_ = nullptr;
    size_t bytes_;
};

// Device allocations are recycled: a freed block goes to a size-keyed free list and serves the
// next request of the same (256-byte rounded) size.  Every kernel and copy of the host layer
// runs on the backend's one stream, so a block handed out again is only ever touched by work
// queued AFTER the work of its previous owner: no synchronisation on free, no hipMalloc /
// hipFree in steady state (each costs far more than a fused row kernel).
class HipPool {
  public:
    static HipPool &instance() {
        static HipPool *p = new HipPool; // never destroyed: the HIP runtime may be gone at static teardown
        return *p;
    }
    void *allocate(size_t bytes) {
        const size_t key = round_up(bytes);
        {
            std::lock_guard<std::mutex> lk(mu_);
            auto it = free_.find(key);
            if (it != free_.end()) {
                void *p = it->second;
                free_.erase(it);
                cached_ -= key;
                return p;
            }
        }
        void *p = nullptr;
        if (axhip_malloc(&p, key) != 0) { // out of memory: give the cached blocks back and retry
            release_all();
            AXHIP_CALL(axhip_malloc(&p, key));
        }
        return p;
    }
    void deallocate(void *p, size_t bytes) {
        const size_t key = round_up(bytes);
        std::lock_guard<std::mutex> lk(mu_);
        free_.emplace(key, p);
        cached_ += key;
    }
    void release_all() {
        std::unordered_multimap<size_t, void *> blocks;
        {
            std::lock_guard<std::mutex> lk(mu_);
            blocks.swap(free_);
            cached_ = 0;
        }
        if (blocks.empty()) return;
        axhip_stream_sync(nullptr); // work that still uses a cached block has been queued before this point
        for (auto &kv : blocks) axhip_free(kv.second);
    }
    size_t cached_bytes() {
        std::lock_guard<std::mutex> lk(mu_);
        return cached_;
    }

  private:
    static size_t round_up(size_t b) { return std::max<size_t>((b + 255) / 256 * 256, 256); }
    std::mutex mu_;
    std::unordered_multimap<size_t, void *> free_;
    size_t cached_ = 0;
};

// Device memory of the gfx950 backend; the role of MetalStorage
// (src/backends/metal/metal_storage.mm:54-142) with explicit copies in place of
// shared memory.
class HipStorage final : public Storage {
  public:
    explicit HipStorage(size_t bytes) : bytes_(bytes) {
        AXHIP_CALL(axhip_init(0));
        if (bytes) ptr_ = HipPool::instance().allocate(bytes);
    }
    ~HipStorage() override {
        if (ptr_) HipPool::instance().deallocate(ptr_, bytes_);
    }
    void *data() override { throw DeviceError("GPU storage has no host pointer; call .cpu() first"); }
    const void *data() const override { throw DeviceError("GPU storage has no host pointer; call .cpu() first"); }
    void *raw() const override { return ptr_; }
    size_t size_bytes() const override { return bytes_; }
    Device device() const override { return Device::GPU; }
    void copy_to(Storage &other) const override { other.copy_from(*this); }
    void copy_from(const Storage &other) override {
        const size_t n = std::min(bytes_, other.size_bytes());
        if (!n) return;
        if (other.device() == Device::CPU) {
            AXHIP_CALL(axhip_memcpy_h2d_async(ptr_, other.raw(), n, nullptr));
            AXHIP_CALL(axhip_stream_sync(nullptr)); // the host buffer may be released by the caller
        } else {
            AXHIP_CALL(axhip_memcpy_d2d_async(ptr_, other.raw(), n, nullptr));
        }
    }
    std::unique_ptr<Storage> clone() const override {
        auto c = std::make_unique<HipStorage>(bytes_);
        c->copy_from(*this);
        return c;
    }

  private:
    void *ptr_ = nullptr;
    size_t bytes_;
};

} // namespace

std::unique_ptr<Storage> make_storage(size_t size_bytes, Device device) {
    if (device == Device::CPU) return std::make_unique<CpuStorage>(size_bytes);
    if (!backends::hip::is_available()) throw DeviceError::not_available("GPU (gfx950) device");
    return std::make_unique<HipStorage>(size_bytes);
}

namespace backends::hip {
bool is_available() {
    int n = 0;
    return axhip_device_count(&n) == 0 && n > 0;
}
void synchronize() { AXHIP_CALL(axhip_stream_sync(nullptr)); }
void empty_cache() { HipPool::instance().release_all(); }
size_t cached_bytes() { return HipPool::instance().cached_bytes(); }
} // namespace backends::hip

namespace system {
bool is_gpu_available() { return backends::hip::is_available(); }
bool should_run_gpu_tests() {
    const char *skip = std::getenv("AXIOM_SKIP_GPU_TESTS");
    if (skip && std::string(skip) == "1") return false;
    return is_gpu_available();
}
} // namespace system

RandomGenerator &RandomGenerator::instance() {
    static thread_local RandomGenerator g;
    return g;
}

} // namespace axiom
