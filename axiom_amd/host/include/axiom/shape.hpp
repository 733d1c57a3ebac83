// Shape and stride helpers.  Strides are in BYTES, as in Axiom
// (include/axiom/shape.hpp:11-17, src/tensor/tensor.cpp:109).
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace axiom {

using Shape = std::vector<size_t>;
using Strides = std::vector<int64_t>;

enum class MemoryOrder { RowMajor, ColMajor };

struct ShapeUtils {
    static size_t size(const Shape &s);
    static Strides contiguous_strides(const Shape &s, size_t itemsize);
    static bool is_contiguous(const Shape &s, const Strides &st, size_t itemsize);
    static Shape broadcast(const Shape &a, const Shape &b); // throws ShapeError
    static std::string to_string(const Shape &s);
    static int normalize_axis(int axis, int ndim); // throws ShapeError
};

} // namespace axiom
