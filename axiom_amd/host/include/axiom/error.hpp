// Error hierarchy of the host layer: same class names and meaning as Axiom's
// include/axiom/error.hpp:14-216, so tests can EXPECT_THROW the same types.
#pragma once

#include <exception>
#include <string>

namespace axiom {

class AxiomError : public std::exception {
  public:
    explicit AxiomError(std::string message) : message_(std::move(message)) {}
    const char *what() const noexcept override { return message_.c_str(); }
    const std::string &message() const { return message_; }

  protected:
    std::string message_;
};

#define AXIOM_DEFINE_ERROR(Name)                                                        \
    class Name : public AxiomError {                                                    \
      public:                                                                           \
        explicit Name(const std::string &message) : AxiomError(#Name ": " + message) {} \
    }

AXIOM_DEFINE_ERROR(ShapeError);
AXIOM_DEFINE_ERROR(TypeError);
AXIOM_DEFINE_ERROR(ValueError);
AXIOM_DEFINE_ERROR(IndexError);
AXIOM_DEFINE_ERROR(MemoryError);
#undef AXIOM_DEFINE_ERROR

class DeviceError : public AxiomError {
  public:
    explicit DeviceError(const std::string &message) : AxiomError("DeviceError: " + message) {}
    static DeviceError not_available(const std::string &what) { return DeviceError(what + " is not available"); }
    static DeviceError cpu_only(const std::string &what) { return DeviceError(what + " requires a CPU tensor; call .cpu() first"); }
};

class RuntimeError : public AxiomError {
  public:
    explicit RuntimeError(const std::string &message) : AxiomError("RuntimeError: " + message) {}
    static RuntimeError not_implemented(const std::string &what) { return RuntimeError(what + " is not implemented"); }
};

} // namespace axiom
