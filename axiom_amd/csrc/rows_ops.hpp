// Elementwise op kernels shared by the fused-row kernels: one switch per chain
// op (a wave-uniform scalar branch), each arm straight-line code over a
// thread's whole register tile.
#pragma once

#include "common.hpp"

namespace axhip {

constexpr float NEG_INF = -__builtin_huge_valf();
constexpr float POS_INF = __builtin_huge_valf();

// The long library routines of the wider operator table (powf, fmodf, atan2f, hypotf, erff, the trigonometric
// functions, cbrtf) as ONE function that the chain interpreters call per value: inlined into every arm of every
// interpreter kernel they multiplied the build time and the code size of this file by five.  A chain through this
// call runs at about 40 % of the HBM peak; comparisons, logical operations, rounding and the is* tests are inline
// arms like the first table's.  (The switch also lists those, for callers that come here with any extended code.)
// The compiled row programs have all of them inline.
__device__ __attribute__((noinline)) inline float extended_op(int op, float a, float b) {
    switch (op) {
    case AXHIP_OP_POW: return powf(a, b);
    case AXHIP_OP_RPOW: return powf(b, a);
    case AXHIP_OP_MOD: return fmodf(a, b);
    case AXHIP_OP_RMOD: return fmodf(b, a);
    case AXHIP_OP_ATAN2: return atan2f(a, b);
    case AXHIP_OP_RATAN2: return atan2f(b, a);
    case AXHIP_OP_HYPOT: return hypotf(a, b);
    case AXHIP_OP_EQ: return a == b ? 1.0f : 0.0f;
    case AXHIP_OP_NE: return a != b ? 1.0f : 0.0f;
    case AXHIP_OP_LT: return a < b ? 1.0f : 0.0f;
    case AXHIP_OP_LE: return a <= b ? 1.0f : 0.0f;
    case AXHIP_OP_GT: return a > b ? 1.0f : 0.0f;
    case AXHIP_OP_GE: return a >= b ? 1.0f : 0.0f;
    case AXHIP_OP_AND: return (a != 0.0f) && (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_OR: return (a != 0.0f) || (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_XOR: return (a != 0.0f) != (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_LEAKY_RELU: return a > 0.0f ? a : b * a;
    case AXHIP_OP_ERF: return erff(a);
    case AXHIP_OP_SIN: return sinf(a);
    case AXHIP_OP_COS: return cosf(a);
    case AXHIP_OP_TAN: return tanf(a);
    case AXHIP_OP_SIGN: return a > 0.0f ? 1.0f : a < 0.0f ? -1.0f : 0.0f;
    case AXHIP_OP_FLOOR: return floorf(a);
    case AXHIP_OP_CEIL: return ceilf(a);
    case AXHIP_OP_ROUND: return roundf(a);
    case AXHIP_OP_TRUNC: return truncf(a);
    case AXHIP_OP_CBRT: return cbrtf(a);
    case AXHIP_OP_ISNAN: return a != a ? 1.0f : 0.0f;
    case AXHIP_OP_ISINF: return fabsf(a) == POS_INF ? 1.0f : 0.0f;
    case AXHIP_OP_ISFINITE: return fabsf(a) < POS_INF ? 1.0f : 0.0f;
    case AXHIP_OP_NOT: return a == 0.0f ? 1.0f : 0.0f;
    default: return a;
    }
}

__device__ __forceinline__ float apply_unary(int op, float a) {
    switch (op) {
    case AXHIP_OP_RELU: return a > 0.0f ? a : 0.0f;
    case AXHIP_OP_GELU: return 0.5f * a * (1.0f + erff(a * 0.70710678118654752f));
    case AXHIP_OP_SQRT: return sqrtf(a);
    case AXHIP_OP_EXP: return expf(a);
    case AXHIP_OP_NEG: return -a;
    case AXHIP_OP_ABS: return fabsf(a);
    case AXHIP_OP_SIGMOID: {
        float e = expf(-fabsf(a)), d = 1.0f + e;
        return a >= 0.0f ? 1.0f / d : e / d;
    }
    case AXHIP_OP_TANH: return tanhf(a);
    case AXHIP_OP_SILU: return a / (1.0f + expf(-a));
    case AXHIP_OP_LOG: return logf(a);
    case AXHIP_OP_SQUARE: return a * a;
    case AXHIP_OP_RSQRT: return 1.0f / sqrtf(a);
    case AXHIP_OP_RECIP: return 1.0f / a;
    case AXHIP_OP_SIGN: return a > 0.0f ? 1.0f : a < 0.0f ? -1.0f : 0.0f;
    case AXHIP_OP_FLOOR: return floorf(a);
    case AXHIP_OP_CEIL: return ceilf(a);
    case AXHIP_OP_ROUND: return roundf(a);
    case AXHIP_OP_TRUNC: return truncf(a);
    case AXHIP_OP_ISNAN: return a != a ? 1.0f : 0.0f;
    case AXHIP_OP_ISINF: return fabsf(a) == POS_INF ? 1.0f : 0.0f;
    case AXHIP_OP_ISFINITE: return fabsf(a) < POS_INF ? 1.0f : 0.0f;
    case AXHIP_OP_NOT: return a == 0.0f ? 1.0f : 0.0f;
    default: return op >= AXHIP_OP_POW ? extended_op(op, a, 0.0f) : a;
    }
}

__device__ __forceinline__ float apply_binary(int op, float a, float b) {
    switch (op) {
    case AXHIP_OP_ADD: return a + b;
    case AXHIP_OP_SUB: return a - b;
    case AXHIP_OP_MUL: return a * b;
    case AXHIP_OP_DIV: return a / b;
    case AXHIP_OP_MAX: return fmaxf(a, b);
    case AXHIP_OP_MIN: return fminf(a, b);
    case AXHIP_OP_RSUB: return b - a;
    case AXHIP_OP_RDIV: return b / a;
    case AXHIP_OP_EQ: return a == b ? 1.0f : 0.0f;
    case AXHIP_OP_NE: return a != b ? 1.0f : 0.0f;
    case AXHIP_OP_LT: return a < b ? 1.0f : 0.0f;
    case AXHIP_OP_LE: return a <= b ? 1.0f : 0.0f;
    case AXHIP_OP_GT: return a > b ? 1.0f : 0.0f;
    case AXHIP_OP_GE: return a >= b ? 1.0f : 0.0f;
    case AXHIP_OP_AND: return (a != 0.0f) && (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_OR: return (a != 0.0f) || (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_XOR: return (a != 0.0f) != (b != 0.0f) ? 1.0f : 0.0f;
    case AXHIP_OP_LEAKY_RELU: return a > 0.0f ? a : b * a;
    default: return op >= AXHIP_OP_POW ? extended_op(op, a, b) : a;
    }
}

__host__ __device__ inline bool is_binary_op(int op) {
    return (op >= AXHIP_OP_ADD && op <= AXHIP_OP_RDIV) || (op >= AXHIP_OP_POW && op <= AXHIP_OP_LEAKY_RELU);
}
__host__ __device__ inline bool is_unary_op(int op) {
    return (op >= AXHIP_OP_RELU && op <= AXHIP_OP_RECIP) || (op >= AXHIP_OP_ERF && op <= AXHIP_OP_NOT);
}

// Apply one chain op to a thread's register tile.  The op code is a kernel
// argument, so the switch is a scalar (wave-uniform) branch taken once per op;
// each arm is straight-line vector code over the whole tile.
template <int IT, int E, typename F>
__device__ __forceinline__ void for_each_value(float (&v)[IT][E], F f) {
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
        for (int e = 0; e < E; ++e) v[it][e] = f(v[it][e], it, e);
}

// The same for the long-running functions (erff, expf, IEEE division ...): four values at a time, with a scheduling
// barrier between the groups.  Left to itself the scheduler interleaves all IT * E evaluations, and the
// temporaries of that one arm then set the register count of the whole kernel.  GROUPS = false (the 1024-thread
// kernels, whose register file share is fixed at 128 by the block size) keeps the free schedule.
template <int IT, int E, bool GROUPS, typename F>
__device__ __forceinline__ void for_each_value_in_groups(float (&v)[IT][E], F f) {
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
        for (int e = 0; e < E; ++e) {
            v[it][e] = f(v[it][e], it, e);
            if (GROUPS && (it * E + e) % 4 == 3) __builtin_amdgcn_sched_barrier(0);
        }
}

template <int IT, int E, bool GROUPS = true>
__device__ __forceinline__ void apply_unary_tile(int op, float (&v)[IT][E]) {
#define AXHIP_UNARY_CASE(code) \
    case code: for_each_value<IT, E>(v, [](float a, int, int) { return apply_unary(code, a); }); break
#define AXHIP_UNARY_LONG(code) \
    case code: for_each_value_in_groups<IT, E, GROUPS>(v, [](float a, int, int) { return apply_unary(code, a); }); break
    switch (op) {
        AXHIP_UNARY_CASE(AXHIP_OP_RELU);
        AXHIP_UNARY_LONG(AXHIP_OP_GELU);
        AXHIP_UNARY_LONG(AXHIP_OP_SQRT);
        AXHIP_UNARY_LONG(AXHIP_OP_EXP);
        AXHIP_UNARY_CASE(AXHIP_OP_NEG);
        AXHIP_UNARY_CASE(AXHIP_OP_ABS);
        AXHIP_UNARY_LONG(AXHIP_OP_SIGMOID);
        AXHIP_UNARY_LONG(AXHIP_OP_TANH);
        AXHIP_UNARY_LONG(AXHIP_OP_SILU);
        AXHIP_UNARY_LONG(AXHIP_OP_LOG);
        AXHIP_UNARY_CASE(AXHIP_OP_SQUARE);
        AXHIP_UNARY_LONG(AXHIP_OP_RSQRT);
        AXHIP_UNARY_LONG(AXHIP_OP_RECIP);
        AXHIP_UNARY_CASE(AXHIP_OP_SIGN);
        AXHIP_UNARY_CASE(AXHIP_OP_FLOOR);
        AXHIP_UNARY_CASE(AXHIP_OP_CEIL);
        AXHIP_UNARY_CASE(AXHIP_OP_ROUND);
        AXHIP_UNARY_CASE(AXHIP_OP_TRUNC);
        AXHIP_UNARY_CASE(AXHIP_OP_ISNAN);
        AXHIP_UNARY_CASE(AXHIP_OP_ISINF);
        AXHIP_UNARY_CASE(AXHIP_OP_ISFINITE);
        AXHIP_UNARY_CASE(AXHIP_OP_NOT);
    default: // the long library routines, through one call per value
        if (op >= AXHIP_OP_ERF) for_each_value<IT, E>(v, [op](float a, int, int) { return extended_op(op, a, 0.0f); });
        break;
    }
#undef AXHIP_UNARY_CASE
#undef AXHIP_UNARY_LONG
}

// w(it, e) yields the second operand of element (it, e)
template <int IT, int E, bool GROUPS = true, typename W>
__device__ __forceinline__ void apply_binary_tile(int op, float (&v)[IT][E], W w) {
#define AXHIP_BINARY_CASE(code) \
    case code: for_each_value<IT, E>(v, [&](float a, int it, int e) { return apply_binary(code, a, w(it, e)); }); break
#define AXHIP_BINARY_LONG(code) \
    case code: for_each_value_in_groups<IT, E, GROUPS>(v, [&](float a, int it, int e) { return apply_binary(code, a, w(it, e)); }); break
    switch (op) {
        AXHIP_BINARY_CASE(AXHIP_OP_ADD);
        AXHIP_BINARY_CASE(AXHIP_OP_SUB);
        AXHIP_BINARY_CASE(AXHIP_OP_MUL);
        AXHIP_BINARY_LONG(AXHIP_OP_DIV);
        AXHIP_BINARY_CASE(AXHIP_OP_MAX);
        AXHIP_BINARY_CASE(AXHIP_OP_MIN);
        AXHIP_BINARY_CASE(AXHIP_OP_RSUB);
        AXHIP_BINARY_LONG(AXHIP_OP_RDIV);
        AXHIP_BINARY_CASE(AXHIP_OP_EQ);
        AXHIP_BINARY_CASE(AXHIP_OP_NE);
        AXHIP_BINARY_CASE(AXHIP_OP_LT);
        AXHIP_BINARY_CASE(AXHIP_OP_LE);
        AXHIP_BINARY_CASE(AXHIP_OP_GT);
        AXHIP_BINARY_CASE(AXHIP_OP_GE);
        AXHIP_BINARY_CASE(AXHIP_OP_AND);
        AXHIP_BINARY_CASE(AXHIP_OP_OR);
        AXHIP_BINARY_CASE(AXHIP_OP_XOR);
        AXHIP_BINARY_CASE(AXHIP_OP_LEAKY_RELU);
    default: // the long library routines, through one call per value
        if (op >= AXHIP_OP_POW) for_each_value<IT, E>(v, [&](float a, int it, int e) { return extended_op(op, a, w(it, e)); });
        break;
    }
#undef AXHIP_BINARY_CASE
#undef AXHIP_BINARY_LONG
}

} // namespace axhip
