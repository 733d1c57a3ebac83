// .safetensors weight files (include/axiom/io/safetensors.hpp:9-27, src/io/io_safetensors.cpp):
// 8-byte little-endian header length, a JSON header {name: {dtype, shape, data_offsets}, ...}
// (the "__metadata__" entry is skipped), then the raw little-endian tensor bytes.
#pragma once

#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "axiom/tensor.hpp"

namespace axiom::io {

// include/axiom/io/io.hpp:36-46
class SerializationError : public std::runtime_error {
  public:
    explicit SerializationError(const std::string &message) : std::runtime_error("Axiom serialization error: " + message) {}
};
class FileFormatError : public SerializationError {
  public:
    explicit FileFormatError(const std::string &message) : SerializationError("Invalid file format: " + message) {}
};

namespace safetensors {

bool is_safetensors_file(const std::string &filename); // by extension
// every tensor of the file; with Device::GPU each is uploaded after it is read
std::map<std::string, Tensor> load(const std::string &filename, Device device = Device::CPU);
std::vector<std::string> list_tensors(const std::string &filename); // names, without reading data
Tensor load_tensor(const std::string &filename, const std::string &tensor_name, Device device = Device::CPU);

} // namespace safetensors
} // namespace axiom::io
