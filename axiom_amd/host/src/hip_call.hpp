// Turns a non-zero return of the C ABI into a DeviceError carrying the library's message.
#pragma once

#include <string>

#include "axhip.h"
#include "axiom/dtype.hpp"
#include "axiom/error.hpp"

#define AXHIP_CALL(expr)                                                                              \
    do {                                                                                              \
        const int axhip_rc_ = (expr);                                                                 \
        if (axhip_rc_ != 0)                                                                           \
            throw ::axiom::DeviceError(std::string(#expr) + " failed (" + std::to_string(axhip_rc_) + \
                                       "): " + axhip_last_error());                                   \
    } while (0)

namespace axiom::detail {
inline int to_axhip_dtype(DType d) {
    switch (d) {
    case DType::Float32: return AXHIP_DTYPE_F32;
    case DType::Float16: return AXHIP_DTYPE_F16;
    case DType::BFloat16: return AXHIP_DTYPE_BF16;
    default: throw TypeError("the gfx950 kernels compute on float32, float16 and bfloat16; got " + dtype_name(d));
    }
}
// the element types of the fused chains, the strided copy, where and the axis reductions: the above plus one-byte
// truth values (Bool; UInt8 is read the same way)
inline int to_axhip_dtype_or_bool(DType d) {
    if (d == DType::Bool || d == DType::UInt8) return AXHIP_DTYPE_U8;
    return to_axhip_dtype(d);
}
} // namespace axiom::detail
