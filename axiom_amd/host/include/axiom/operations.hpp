// ops:: free functions for the GPU hot paths, same names and argument meaning
// as Axiom's include/axiom/operations.hpp.  Every function needs its tensors
// on Device::GPU: elementwise / softmax / norm / reduction / matmul calls build
// lazy graph nodes (src/tensor/operations.cpp:660-669, 857-869, 930-959,
// 1420-1435, 1775-1795); scaled_dot_product_attention runs eagerly
// (operations.cpp:3979-4044).  CPU tensors throw RuntimeError: this library
// carries no CPU compute path.
#pragma once

#include <array>
#include <map>
#include <memory>
#include <utility>
#include <string>
#include <vector>

#include "axiom/dtype.hpp"
#include "axiom/storage.hpp"

namespace axiom {
class Tensor;

namespace ops {

// Axiom's OpType (include/axiom/operations.hpp:55-208), same order and names.
enum class OpType {
    Add, Subtract, Multiply, Divide, Power, Modulo,
    Equal, NotEqual, Less, LessEqual, Greater, GreaterEqual,
    LogicalAnd, LogicalOr, LogicalXor, LogicalNot,
    BitwiseAnd, BitwiseOr, BitwiseXor, LeftShift, RightShift,
    Maximum, Minimum, Atan2, Hypot,
    Negate, Abs, Sqrt, Exp, Log, Sin, Cos, Tan, Erf,
    Sign, Floor, Ceil, Trunc, Round, Reciprocal, Square, Cbrt,
    IsNaN, IsInf, IsFinite,
    Conj, Real, Imag,
    ReLU, LeakyReLU, SiLU, Sigmoid, Tanh, GELU, Softmax, LogSoftmax,
    Sum, Mean, Max, Min, ArgMax, ArgMin, Any, All, Prod,
    MatMul, BatchMatMul,
    Where,
    MaskedFill, MaskedSelect,
    Gather, Scatter, IndexSelect, Take, TakeAlongAxis,
    LayerNorm, RMSNorm,
    Dropout,
    Cast,
    MaxPool1D, MaxPool2D, MaxPool3D, AvgPool1D, AvgPool2D, AvgPool3D, AdaptiveMaxPool2D, AdaptiveAvgPool2D,
    Conv1D, Conv2D, ConvTranspose1D, ConvTranspose2D,
    ScaledDotProductAttention,
    Reshape, Transpose, Pad, Slice, Unsqueeze, Concat,
    GLU, BatchNorm1D,
    Sort, Argsort, TopK,
    _Count,
    // internal to this backend's planner, after Axiom's own values: the (N, L_out, C_in, K) window view a
    // convolution is lowered through
    Unfold1D,
    Unfold2D // (N, H_out, W_out, C_in, KH, KW)
};

const char *op_name(OpType op);

// Per-device implementation of one OpType (include/axiom/operations.hpp:210-279).  The base
// implementations throw RuntimeError::not_implemented (src/tensor/operations.cpp:466-549).
class Operation {
  public:
    virtual ~Operation() = default;
    virtual OpType type() const = 0;
    virtual std::string name() const = 0;
    virtual Device device() const = 0;
    virtual bool supports_binary(const Tensor &lhs, const Tensor &rhs) const;
    virtual Tensor execute_binary(const Tensor &lhs, const Tensor &rhs) const;
    virtual Tensor execute_unary(const Tensor &input) const;
    virtual Tensor execute_reduction(const Tensor &input, const std::vector<int> &axis, bool keep_dims) const;
    virtual Tensor execute_matmul(const Tensor &a, const Tensor &b, bool transpose_a, bool transpose_b) const;
    virtual Tensor execute_cast(const Tensor &input, DType target_dtype) const;
};

// (OpType, Device) -> Operation (include/axiom/operations.hpp:285-302).  This library registers
// Device::GPU entries only; get_operation(op, Device::CPU) is null.
class OperationRegistry {
  public:
    static void register_operation(OpType op_type, Device device, std::unique_ptr<Operation> operation);
    static const Operation *get_operation(OpType op_type, Device device);
    static std::vector<Device> available_devices_for_operation(OpType op_type);
    static bool is_operation_available(OpType op_type, Device device);
    static void initialize_builtin_operations();
};
DType promote_types(DType lhs, DType rhs); // src/tensor/operations.cpp:346-397

Tensor add(const Tensor &a, const Tensor &b);
Tensor subtract(const Tensor &a, const Tensor &b);
Tensor multiply(const Tensor &a, const Tensor &b);
Tensor divide(const Tensor &a, const Tensor &b);
Tensor maximum(const Tensor &a, const Tensor &b);
Tensor minimum(const Tensor &a, const Tensor &b);
// include/axiom/operations.hpp:313-341.  power / modulo follow the CPU functors (std::pow; std::fmod, the sign of the
// dividend: src/backends/cpu/cpu_operations.hpp:214-235); comparisons and logical operations give Bool tensors, a
// logical operation reads any nonzero element as true
Tensor power(const Tensor &a, const Tensor &b);
Tensor modulo(const Tensor &a, const Tensor &b);
Tensor atan2(const Tensor &a, const Tensor &b);
Tensor hypot(const Tensor &a, const Tensor &b);
Tensor equal(const Tensor &a, const Tensor &b);
Tensor not_equal(const Tensor &a, const Tensor &b);
Tensor less(const Tensor &a, const Tensor &b);
Tensor less_equal(const Tensor &a, const Tensor &b);
Tensor greater(const Tensor &a, const Tensor &b);
Tensor greater_equal(const Tensor &a, const Tensor &b);
Tensor logical_and(const Tensor &a, const Tensor &b);
Tensor logical_or(const Tensor &a, const Tensor &b);
Tensor logical_xor(const Tensor &a, const Tensor &b);
Tensor logical_not(const Tensor &x);

Tensor negate(const Tensor &x);
Tensor abs(const Tensor &x);
Tensor sqrt(const Tensor &x);
Tensor exp(const Tensor &x);
Tensor log(const Tensor &x);
Tensor reciprocal(const Tensor &x);
Tensor square(const Tensor &x);
Tensor relu(const Tensor &x);
Tensor silu(const Tensor &x);
Tensor sigmoid(const Tensor &x);
Tensor tanh(const Tensor &x);
Tensor gelu(const Tensor &x);
// include/axiom/operations.hpp:349-380.  sign(NaN) is 0, round moves halves away from zero (std::round), the is* tests
// give Bool tensors (src/backends/cpu/cpu_operations.hpp:724-860); round with decimals != 0 is round(x 10^d) / 10^d
// (src/tensor/operations.cpp:1330-1341); clip is maximum(minimum(x, hi), lo) (:1369-1371)
Tensor sin(const Tensor &x);
Tensor cos(const Tensor &x);
Tensor tan(const Tensor &x);
Tensor erf(const Tensor &x);
Tensor sign(const Tensor &x);
Tensor floor(const Tensor &x);
Tensor ceil(const Tensor &x);
Tensor trunc(const Tensor &x);
Tensor round(const Tensor &x, int decimals = 0);
Tensor cbrt(const Tensor &x);
Tensor isnan(const Tensor &x);
Tensor isinf(const Tensor &x);
Tensor isfinite(const Tensor &x);
Tensor clip(const Tensor &x, const Tensor &min_val, const Tensor &max_val);
Tensor leaky_relu(const Tensor &x, float negative_slope = 0.01f);
// numpy.where(condition, a, b): the three broadcast together, the result has promote_types(a, b)
// (include/axiom/operations.hpp:425-429).  A lazy node here; the reference runs it when called.
Tensor where(const Tensor &condition, const Tensor &a, const Tensor &b);
// the GPU Cast (src/tensor/tensor.cpp:1665-1670) as a lazy node among Float32, Float16, BFloat16 and Bool
Tensor cast(const Tensor &x, DType target);

Tensor softmax(const Tensor &x, int axis = -1);
Tensor log_softmax(const Tensor &x, int axis = -1);

Tensor sum(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
Tensor mean(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
Tensor max(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
Tensor min(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
// include/axiom/operations.hpp:403-411: any / all give Bool tensors (an element counts when it is nonzero); they
// are built as max / min over not_equal(x, 0), which fuses into one kernel
Tensor any(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
Tensor all(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
Tensor prod(const Tensor &x, const std::vector<int> &axes = {}, bool keep_dims = false);
// Int64 index of the first occurrence of the extreme along one axis (include/axiom/operations.hpp:400-401); runs when
// called, like scaled_dot_product_attention, on the materialised input
Tensor argmax(const Tensor &x, int axis = -1, bool keep_dims = false);
Tensor argmin(const Tensor &x, int axis = -1, bool keep_dims = false);

// population variance, eps inside the square root; weight / bias may be empty tensors
Tensor layer_norm(const Tensor &x, const Tensor &weight, const Tensor &bias, int axis = -1, float eps = 1e-5f);
Tensor rms_norm(const Tensor &x, const Tensor &weight, int axis = -1, float eps = 1e-5f);

Tensor matmul(const Tensor &a, const Tensor &b, bool transpose_a = false, bool transpose_b = false);

// a * sigmoid(b) over the two halves of `dim` (src/tensor/operations.cpp:1451-1476); ValueError on an odd extent
Tensor glu(const Tensor &x, int dim = -1);
// where the Bool (or nonzero) mask, broadcast against x, is set the result holds `value`
// (include/axiom/operations.hpp:437-440)
Tensor masked_fill(const Tensor &x, const Tensor &mask, float value);
Tensor masked_fill(const Tensor &x, const Tensor &mask, double value);
// pad_width holds (before, after) per dimension; mode "constant", "reflect" (the border element is not repeated; each
// pad shorter than its dimension), "replicate" or "circular" (include/axiom/operations.hpp:519-526)
Tensor pad(const Tensor &x, const std::vector<std::pair<size_t, size_t>> &pad_width, const std::string &mode = "constant", double value = 0.0);
// rows of weight (vocab, dim) selected by integer indices of any shape -> (*indices.shape, dim)
// (include/axiom/operations.hpp:483-486).  On the GPU an index out of range gives a row of zeros.
Tensor embedding(const Tensor &weight, const Tensor &indices);
// PyTorch-compatible 1-D convolution: input (N, C_in, L) or (C_in, L), weight (C_out, C_in, K),
// output (N, C_out, L_out), L_out = (L + 2 padding - dilation (K-1) - 1) / stride + 1
// (include/axiom/operations.hpp:594-601).  groups > 1: weight (C_out, C_in / groups, K), one batched product over the groups.
Tensor conv1d(const Tensor &input, const Tensor &weight, const Tensor &bias, int stride = 1, int padding = 0, int dilation = 1, int groups = 1);
Tensor conv1d(const Tensor &input, const Tensor &weight); // no bias, stride 1, no padding
// 2-D convolution: input (N, C_in, H, W) or (C_in, H, W), weight (C_out, C_in, KH, KW), output (N, C_out, H_out, W_out)
// (include/axiom/operations.hpp:603-611).  groups as for conv1d.
Tensor conv2d(const Tensor &input, const Tensor &weight, const Tensor &bias, std::array<int, 2> stride = {1, 1}, std::array<int, 2> padding = {0, 0},
              std::array<int, 2> dilation = {1, 1}, int groups = 1);
Tensor conv2d(const Tensor &input, const Tensor &weight);
// inference batch norm over the channel dimension (dim 1) of (N, C) or (N, C, L):
// (x - running_mean) / sqrt(running_var + eps) * weight + bias
Tensor batch_norm1d(const Tensor &x, const Tensor &weight, const Tensor &bias, const Tensor &running_mean, const Tensor &running_var, float eps = 1e-5f);

// q (B,H,Sq,D), k/v (B,H,Skv,D); mask Bool (Sq,Skv) or (B,H,Sq,Skv), true = masked out;
// scale <= 0 means 1/sqrt(D).  ShapeError on bad ranks / mismatched batch, heads, Skv or D.
Tensor scaled_dot_product_attention(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask,
                                    float scale = -1.0f, bool is_causal = false);

namespace detail {
// as above; with out_bshd the output is written head-merged, (B, Sq, H, D) in memory, and
// returned as the (B, H, Sq, D) view of it, so MultiHeadAttention's merge needs no copy
Tensor sdpa(const Tensor &query, const Tensor &key, const Tensor &value, const Tensor &mask, float scale, bool is_causal, bool out_bshd);
} // namespace detail

// name of the gfx950 kernel the last scaled_dot_product_attention call on this thread launched
const char *last_sdpa_kernel();

} // namespace ops
} // namespace axiom
