// Element types.  The enumeration keeps Axiom's order (include/axiom/dtype.hpp:171-191)
// so graph signatures hash the same values; the gfx950 kernels compute on
// Float32, Float16 and BFloat16 (Bool / UInt8 serve as attention masks).
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>

namespace axiom {

enum class DType : uint8_t {
    Bool, Int8, Int16, Int32, Int64, UInt8, UInt16, UInt32, UInt64,
    Float16, BFloat16, Float32, Float64, Complex64, Complex128
};

constexpr size_t dtype_size(DType d) {
    switch (d) {
    case DType::Bool: case DType::Int8: case DType::UInt8: return 1;
    case DType::Int16: case DType::UInt16: case DType::Float16: case DType::BFloat16: return 2;
    case DType::Int32: case DType::UInt32: case DType::Float32: return 4;
    case DType::Int64: case DType::UInt64: case DType::Float64: case DType::Complex64: return 8;
    case DType::Complex128: return 16;
    }
    return 0;
}

std::string dtype_name(DType d);
constexpr bool is_floating_dtype(DType d) { return d >= DType::Float16 && d <= DType::Float64; }
constexpr bool is_complex_dtype(DType d) { return d == DType::Complex64 || d == DType::Complex128; }

// bfloat16: round to nearest even, NaN -> 0x7FC0 (include/axiom/bfloat16.hpp:16-27)
struct bfloat16_t {
    uint16_t bits = 0;
    bfloat16_t() = default;
    bfloat16_t(float f) { // NOLINT: implicit like Axiom's
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if (f != f) bits = 0x7FC0;
        else bits = static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    }
    operator float() const { // NOLINT
        uint32_t u = static_cast<uint32_t>(bits) << 16;
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

// IEEE binary16, round to nearest even (include/axiom/float16.hpp:10-78)
struct float16_t {
    uint16_t bits = 0;
    float16_t() = default;
    float16_t(float f); // NOLINT
    operator float() const; // NOLINT
};

template <typename T> struct dtype_of;
template <> struct dtype_of<bool> { static constexpr DType value = DType::Bool; };
template <> struct dtype_of<int8_t> { static constexpr DType value = DType::Int8; };
template <> struct dtype_of<int16_t> { static constexpr DType value = DType::Int16; };
template <> struct dtype_of<int32_t> { static constexpr DType value = DType::Int32; };
template <> struct dtype_of<int64_t> { static constexpr DType value = DType::Int64; };
template <> struct dtype_of<uint8_t> { static constexpr DType value = DType::UInt8; };
template <> struct dtype_of<uint16_t> { static constexpr DType value = DType::UInt16; };
template <> struct dtype_of<uint32_t> { static constexpr DType value = DType::UInt32; };
template <> struct dtype_of<uint64_t> { static constexpr DType value = DType::UInt64; };
template <> struct dtype_of<float16_t> { static constexpr DType value = DType::Float16; };
template <> struct dtype_of<bfloat16_t> { static constexpr DType value = DType::BFloat16; };
template <> struct dtype_of<float> { static constexpr DType value = DType::Float32; };
template <> struct dtype_of<double> { static constexpr DType value = DType::Float64; };

// scalar load / store of any real dtype through double (host side only)
double load_scalar(const void *p, DType d);
void store_scalar(void *p, DType d, double v);

} // namespace axiom
