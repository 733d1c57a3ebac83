// Host-side matching of a row program against the compile-time-specialised
// kernels (rows_static.inc).
#include "rows_static.hpp"

#include <cstring>

namespace axhip {
namespace {

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

bool has_pattern(int pre, int row_op, int reduce) {
#define AXHIP_PATTERN_CASE(PRE, ROWOP, RED) \
    if (pre == PRE && row_op == ROWOP && reduce == RED) return true;
    AXHIP_ROWS_STATIC_PATTERNS(AXHIP_PATTERN_CASE)
#undef AXHIP_PATTERN_CASE
    return false;
}

const char *pre_name(int pre) {
    return pre == RP_NONE ? "" : pre == RP_ADDF ? "addf_" : pre == RP_MULS ? "muls_" : pre == RP_MULS_ADDF ? "muls_addf_" : pre == RP_MULF ? "mulf_" : "relu_adds_mulf_";
}
const char *rowop_name(int r) {
    switch (r) {
    case AXHIP_ROWOP_SOFTMAX: return "softmax";
    case AXHIP_ROWOP_LOGSOFTMAX: return "logsoftmax";
    case AXHIP_ROWOP_LAYERNORM: return "layernorm";
    case AXHIP_ROWOP_RMSNORM: return "rmsnorm";
    default: return "reduce";
    }
}
const char *red_name(int r) { return r == AXHIP_RED_SUM ? "_sum" : r == AXHIP_RED_MAX ? "_max" : r == AXHIP_RED_MIN ? "_min" : ""; }
const char *dtype_name(int dt) { return dt == AXHIP_DTYPE_F32 ? "f32" : dt == AXHIP_DTYPE_F16 ? "f16" : "bf16"; }

} // namespace

bool rows_static_dispatch(const AxhipRowsProgram &P, hipStream_t s, bool launch, char *name, size_t name_len) {
    if (P.rows <= 0 || P.cols <= 0) return false;
    const int dt = P.input_dtype;
    const int e = dt == AXHIP_DTYPE_F32 ? 4 : 8;
    if (P.cols < e) return false;
    if (P.reduce == AXHIP_RED_NONE && P.output_dtype != dt) return false;
    // anything that keeps a 16-byte access from being aligned selects the ragged variant of the kernel
    bool ragged = P.cols % e != 0 || !aligned16(P.input) || (P.reduce == AXHIP_RED_NONE && !aligned16(P.output));

    RowsStaticArgs a{};
    RowsStaticKey k{};
    k.dtype = dt;
    a.x = P.input;
    a.y = P.output;
    a.rows = P.rows;
    a.cols = P.cols;
    a.eps = P.eps;
    a.out_dtype = P.output_dtype;
    a.stream_out = P.reduce == AXHIP_RED_NONE && P.rows * P.cols * static_cast<int64_t>(dtype_size(P.output_dtype)) >= STREAMING_OUTPUT_BYTES;

    auto vector_operand = [&](int idx, int kind) -> const void * {
        if (idx < 0 || idx >= P.n_operands) return nullptr;
        const AxhipOperand &o = P.operands[idx];
        if (o.kind != kind || o.dtype != dt) return nullptr;
        if (!aligned16(o.ptr)) ragged = true;
        return o.ptr;
    };

    // a scalar of the pre chain: an immediate, or a one-element device operand
    auto scalar_of = [&](const AxhipChainOp &c) -> bool {
        if (c.imm_kind == AXHIP_BK_IMM) {
            a.s_imm = c.imm;
            return true;
        }
        const int idx = c.operand;
        if (idx < 0 || idx >= P.n_operands || P.operands[idx].kind != AXHIP_BK_SCALAR) return false;
        a.s_ptr = P.operands[idx].ptr;
        a.s_dtype = P.operands[idx].dtype;
        return true;
    };

    // pre chain
    bool pre_is_post = false;
    if (P.n_pre == 0) {
        k.pre = RP_NONE;
    } else if (P.n_pre == 1 && P.row_op == AXHIP_ROWOP_NONE && P.reduce != AXHIP_RED_NONE && P.n_post == 0 &&
               P.pre[0].op >= AXHIP_OP_RELU && P.pre[0].op <= AXHIP_OP_RECIP) {
        // one unary op, then a row reduction (sum(relu(x)), mean(x^2), max(abs(x))): with no row op in between the
        // op can run where the post op does, right before the accumulation
        k.pre = RP_NONE;
        pre_is_post = true;
    } else if (P.n_pre == 1 && P.pre[0].op == AXHIP_OP_ADD && P.pre[0].imm_kind != AXHIP_BK_IMM &&
               P.pre[0].operand >= 0 && P.pre[0].operand < P.n_operands && P.operands[P.pre[0].operand].kind == AXHIP_BK_FULL) {
        a.f = vector_operand(P.pre[0].operand, AXHIP_BK_FULL);
        if (!a.f) return false;
        k.pre = RP_ADDF;
    } else if (P.n_pre == 1 && P.pre[0].op == AXHIP_OP_MUL && P.pre[0].imm_kind != AXHIP_BK_IMM && P.pre[0].operand >= 0 &&
               P.pre[0].operand < P.n_operands && P.operands[P.pre[0].operand].kind == AXHIP_BK_FULL) { // x * y: the row dot product
        a.f = vector_operand(P.pre[0].operand, AXHIP_BK_FULL);
        if (!a.f) return false;
        k.pre = RP_MULF;
    } else if (P.n_pre == 1 && P.pre[0].op == AXHIP_OP_MUL) { // x * s: the scaled softmax
        if (!scalar_of(P.pre[0])) return false;
        k.pre = RP_MULS;
    } else if (P.n_pre == 2 && P.pre[0].op == AXHIP_OP_MUL && P.pre[1].op == AXHIP_OP_ADD && P.pre[1].imm_kind != AXHIP_BK_IMM) { // x * s + bias tensor
        if (!scalar_of(P.pre[0])) return false;
        a.f = vector_operand(P.pre[1].operand, AXHIP_BK_FULL);
        if (!a.f) return false;
        k.pre = RP_MULS_ADDF;
    } else if (P.n_pre == 3 && P.pre[0].op == AXHIP_OP_RELU && P.pre[1].op == AXHIP_OP_ADD && P.pre[2].op == AXHIP_OP_MUL &&
               P.pre[2].imm_kind != AXHIP_BK_IMM) {
        if (P.pre[1].imm_kind == AXHIP_BK_IMM) {
            a.s_imm = P.pre[1].imm;
        } else {
            const int idx = P.pre[1].operand;
            if (idx < 0 || idx >= P.n_operands || P.operands[idx].kind != AXHIP_BK_SCALAR) return false;
            a.s_ptr = P.operands[idx].ptr;
            a.s_dtype = P.operands[idx].dtype;
        }
        a.f = vector_operand(P.pre[2].operand, AXHIP_BK_FULL);
        if (!a.f) return false;
        k.pre = RP_RELU_ADDS_MULF;
    } else {
        return false;
    }

    // row op and its affine operands
    k.row_op = P.row_op;
    const bool is_norm = P.row_op == AXHIP_ROWOP_LAYERNORM || P.row_op == AXHIP_ROWOP_RMSNORM;
    if (P.norm_weight >= 0) {
        if (!is_norm) return false;
        a.w = vector_operand(P.norm_weight, AXHIP_BK_ROWVEC);
        if (!a.w) return false;
    }
    if (P.norm_bias >= 0) {
        if (P.row_op != AXHIP_ROWOP_LAYERNORM) return false;
        a.b = vector_operand(P.norm_bias, AXHIP_BK_ROWVEC);
        if (!a.b) return false;
    }

    // post chain: nothing or one unary op
    if (pre_is_post) a.post_op = P.pre[0].op;
    else if (P.n_post == 1 && P.post[0].op >= AXHIP_OP_RELU && P.post[0].op <= AXHIP_OP_RECIP) a.post_op = P.post[0].op;
    else if (P.n_post != 0) return false;

    k.reduce = P.reduce == AXHIP_RED_MEAN ? AXHIP_RED_SUM : P.reduce;
    a.red_mean = P.reduce == AXHIP_RED_MEAN;
    if (!has_pattern(k.pre, k.row_op, k.reduce)) return false;

    // register plan
    const int64_t chunks = (P.cols + e - 1) / e;
    a.ragged = ragged;
    if (ragged) a.stream_out = 0;
    if (chunks <= 512) {
        k.group = 64;
        k.it = chunks <= 64 ? 1 : chunks <= 128 ? 2 : chunks <= 256 ? 4 : 8;
    } else if (chunks <= 2048) {
        k.group = 256;
        k.it = chunks <= 1024 ? 4 : 8;
    } else {
        return false;
    }
    const int64_t rows_per_block = 256 / k.group;
    if ((P.rows + rows_per_block - 1) / rows_per_block >= (int64_t(1) << 31)) return false;

    if (name) {
        snprintf(name, name_len, "rows_static_%s%s%s_%s_g%d_it%d%s", pre_name(k.pre), rowop_name(k.row_op), red_name(k.reduce),
                 dtype_name(dt), k.group, k.it, ragged ? "_ragged" : "");
    }
    if (!launch) return true;
    return dt == AXHIP_DTYPE_F32 ? rows_static_launch_f32(k, a, s)
           : dt == AXHIP_DTYPE_F16 ? rows_static_launch_f16(k, a, s)
                                   : rows_static_launch_bf16(k, a, s);
}

} // namespace axhip
