// Compile-time-specialised fused-row kernels for the chain shapes that matter
// most (the counterpart of the known SIMD patterns in Axiom's
// src/graph/fused_patterns.cpp:12-71, next to the generic interpreter of
// rows.hip which plays the role of its FusedGenericStep).
//
// A program qualifies when
//   - input, full-size output and every vector operand share one dtype,
//   - cols holds at least one 16-byte vector (any other length, and pointers
//     that are only element-aligned, run the kernels' ragged variant: unaligned
//     16-byte accesses and an element-wise last chunk),
//   - a row fits in registers (cols <= 8192 fp32 / 16384 half elements),
//   - the pre chain is empty, [add FULL] (residual) or
//     [relu, add scalar, mul FULL]; the post chain is empty or one unary op,
//   - (pre, row_op, reduce) is one of the instantiated combinations.
// Everything else runs on the interpreter.
#pragma once

#include "common.hpp"

namespace axhip {

enum RowsPre { RP_NONE = 0, RP_ADDF = 1, RP_RELU_ADDS_MULF = 2, RP_MULS = 3, RP_MULS_ADDF = 4, RP_MULF = 5 }; // F: full-size operand, S: scalar

struct RowsStaticArgs {
    const void *x;      // [rows, cols]
    void *y;            // [rows, cols] or [rows]
    const void *f;      // FULL operand of the pre chain
    const void *s_ptr;  // device scalar of the pre chain, or NULL to use s_imm
    const void *w;      // norm weight [cols] or NULL
    const void *b;      // norm bias [cols] or NULL
    int64_t rows, cols;
    float s_imm;
    float eps;
    int32_t s_dtype;
    int32_t post_op;    // 0 or a unary AXHIP_OP_*
    int32_t red_mean;   // reduce == MEAN: scale the sum by 1/cols
    int32_t out_dtype;  // dtype of a reduced [rows] output
    int32_t stream_out; // full-size output written with non-temporal stores
    int32_t ragged;     // cols is not a multiple of the 16-byte vector, or a pointer is not 16-byte aligned
};

struct RowsStaticKey {
    int dtype, pre, row_op, reduce; // reduce: AXHIP_RED_NONE / SUM / MAX / MIN
    int group, it;
};

// (pre chain, row op, reduction) combinations that are instantiated, for each
// of the register plans below.
#define AXHIP_ROWS_STATIC_PATTERNS(X)                          \
    X(RP_NONE, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_NONE)            \
    X(RP_NONE, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_SUM)             \
    X(RP_NONE, AXHIP_ROWOP_LOGSOFTMAX, AXHIP_RED_NONE)         \
    X(RP_RELU_ADDS_MULF, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_NONE)  \
    X(RP_RELU_ADDS_MULF, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_SUM)   \
    X(RP_MULS, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_NONE)            \
    X(RP_ADDF, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_NONE)            \
    X(RP_MULS_ADDF, AXHIP_ROWOP_SOFTMAX, AXHIP_RED_NONE)       \
    X(RP_NONE, AXHIP_ROWOP_LAYERNORM, AXHIP_RED_NONE)          \
    X(RP_ADDF, AXHIP_ROWOP_LAYERNORM, AXHIP_RED_NONE)          \
    X(RP_NONE, AXHIP_ROWOP_RMSNORM, AXHIP_RED_NONE)            \
    X(RP_ADDF, AXHIP_ROWOP_RMSNORM, AXHIP_RED_NONE)            \
    X(RP_NONE, AXHIP_ROWOP_NONE, AXHIP_RED_SUM)                \
    X(RP_ADDF, AXHIP_ROWOP_NONE, AXHIP_RED_SUM)                \
    X(RP_MULF, AXHIP_ROWOP_NONE, AXHIP_RED_SUM)                \
    X(RP_NONE, AXHIP_ROWOP_NONE, AXHIP_RED_MAX)                \
    X(RP_NONE, AXHIP_ROWOP_NONE, AXHIP_RED_MIN)

// register plans: (threads sharing a row, 16-byte chunks per thread)
#define AXHIP_ROWS_STATIC_PLANS(X) X(64, 1) X(64, 2) X(64, 4) X(64, 8) X(256, 4) X(256, 8)

// Matches the program against the specialised kernels; fills `name` (when
// non-NULL) and launches when `launch` is set.  Returns false when the
// interpreter has to take the program.
bool rows_static_dispatch(const AxhipRowsProgram &P, hipStream_t s, bool launch, char *name, size_t name_len);

bool rows_static_launch_f32(const RowsStaticKey &k, const RowsStaticArgs &a, hipStream_t s);
bool rows_static_launch_f16(const RowsStaticKey &k, const RowsStaticArgs &a, hipStream_t s);
bool rows_static_launch_bf16(const RowsStaticKey &k, const RowsStaticArgs &a, hipStream_t s);

} // namespace axhip
