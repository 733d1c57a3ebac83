// Free functions of the gfx950 backend with the shapes of the Metal backend's
// (src/backends/metal/metal_operations.hpp:15-68, the hot-path subset).  Each submits its
// work at once (no lazy node is left behind) and returns a GPU tensor.
#pragma once

#include "axiom/tensor.hpp"

namespace axiom::backends::hip {

bool is_hip_available();
// registers an Operation for every supported OpType under Device::GPU (role of
// register_metal_operations, src/backends/metal/metal_operations.mm:22-26)
void register_hip_operations();

Tensor gpu_layer_norm(const Tensor &input, const Tensor &weight, const Tensor &bias, int axis, float eps);
Tensor gpu_rms_norm(const Tensor &input, const Tensor &weight, int axis, float eps);
Tensor gpu_scaled_dot_product_attention(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask, float scale, bool is_causal);
Tensor gpu_fill_constant(const Shape &shape, DType dtype, double value);
Tensor gpu_make_contiguous(const Tensor &tensor);
Tensor gpu_linear(const Tensor &input, const Tensor &weight, const Tensor &bias, bool has_bias);

} // namespace axiom::backends::hip
