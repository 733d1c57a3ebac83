// Storage: owner of a tensor's bytes on one device
// (include/axiom/storage.hpp:8-32).  Device::GPU is a gfx950 device reached
// through the C ABI of libaxhip; host <-> device movement is an explicit copy.
#pragma once

#include <cstddef>
#include <memory>

namespace axiom {

enum class Device { CPU, GPU };

class Storage {
  public:
    virtual ~Storage() = default;
    virtual void *data() = 0;             // host pointer; GPU storage throws DeviceError
    virtual const void *data() const = 0;
    virtual size_t size_bytes() const = 0;
    virtual Device device() const = 0;
    virtual void copy_to(Storage &other) const = 0;
    virtual void copy_from(const Storage &other) = 0;
    virtual std::unique_ptr<Storage> clone() const = 0;
    // raw device address (GPU) or host address (CPU): what the C ABI takes
    virtual void *raw() const = 0;
};

// throws DeviceError::not_available when a GPU storage is asked for and no device exists
std::unique_ptr<Storage> make_storage(size_t size_bytes, Device device = Device::CPU);

namespace backends::hip {
// waits for every kernel and copy queued on the backend stream
void synchronize();
bool is_available();
// device blocks freed by tensors are kept for reuse; this returns them to the driver
void empty_cache();
size_t cached_bytes();
} // namespace backends::hip

} // namespace axiom
