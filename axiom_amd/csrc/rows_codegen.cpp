// Generator of the compiled fused-row programs (see rows_codegen.hpp).
#include "rows_codegen.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>

namespace axhip {

namespace {

int elem_size(int dt) { return dt == AXHIP_DTYPE_F32 ? 4 : dt == AXHIP_DTYPE_U8 ? 1 : 2; }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
const char *dt_name(int dt) { return dt == AXHIP_DTYPE_F32 ? "f32" : dt == AXHIP_DTYPE_F16 ? "f16" : dt == AXHIP_DTYPE_U8 ? "u8" : "bf16"; }
bool is_unary(int op) { return (op >= AXHIP_OP_RELU && op <= AXHIP_OP_RECIP) || (op >= AXHIP_OP_ERF && op <= AXHIP_OP_NOT); }
bool is_binary(int op) { return (op >= AXHIP_OP_ADD && op <= AXHIP_OP_RDIV) || (op >= AXHIP_OP_POW && op <= AXHIP_OP_LEAKY_RELU); }

const char *op_token(int op) {
    switch (op) {
    case AXHIP_OP_ADD: return "add";
    case AXHIP_OP_SUB: return "sub";
    case AXHIP_OP_MUL: return "mul";
    case AXHIP_OP_DIV: return "div";
    case AXHIP_OP_MAX: return "max";
    case AXHIP_OP_MIN: return "min";
    case AXHIP_OP_RSUB: return "rsub";
    case AXHIP_OP_RDIV: return "rdiv";
    case AXHIP_OP_RELU: return "relu";
    case AXHIP_OP_GELU: return "gelu";
    case AXHIP_OP_SQRT: return "sqrt";
    case AXHIP_OP_EXP: return "exp";
    case AXHIP_OP_NEG: return "neg";
    case AXHIP_OP_ABS: return "abs";
    case AXHIP_OP_SIGMOID: return "sigmoid";
    case AXHIP_OP_TANH: return "tanh";
    case AXHIP_OP_SILU: return "silu";
    case AXHIP_OP_LOG: return "log";
    case AXHIP_OP_SQUARE: return "square";
    case AXHIP_OP_RSQRT: return "rsqrt";
    case AXHIP_OP_RECIP: return "recip";
    case AXHIP_OP_POW: return "pow";
    case AXHIP_OP_RPOW: return "rpow";
    case AXHIP_OP_MOD: return "mod";
    case AXHIP_OP_RMOD: return "rmod";
    case AXHIP_OP_ATAN2: return "atan2";
    case AXHIP_OP_RATAN2: return "ratan2";
    case AXHIP_OP_HYPOT: return "hypot";
    case AXHIP_OP_EQ: return "eq";
    case AXHIP_OP_NE: return "ne";
    case AXHIP_OP_LT: return "lt";
    case AXHIP_OP_LE: return "le";
    case AXHIP_OP_GT: return "gt";
    case AXHIP_OP_GE: return "ge";
    case AXHIP_OP_AND: return "and";
    case AXHIP_OP_OR: return "or";
    case AXHIP_OP_XOR: return "xor";
    case AXHIP_OP_LEAKY_RELU: return "leaky";
    case AXHIP_OP_ERF: return "erf";
    case AXHIP_OP_SIN: return "sin";
    case AXHIP_OP_COS: return "cos";
    case AXHIP_OP_TAN: return "tan";
    case AXHIP_OP_SIGN: return "sign";
    case AXHIP_OP_FLOOR: return "floor";
    case AXHIP_OP_CEIL: return "ceil";
    case AXHIP_OP_ROUND: return "round";
    case AXHIP_OP_TRUNC: return "trunc";
    case AXHIP_OP_CBRT: return "cbrt";
    case AXHIP_OP_ISNAN: return "isnan";
    case AXHIP_OP_ISINF: return "isinf";
    case AXHIP_OP_ISFINITE: return "isfinite";
    case AXHIP_OP_NOT: return "not";
    default: return nullptr;
    }
}
const char *rowop_token(int r) {
    switch (r) {
    case AXHIP_ROWOP_SOFTMAX: return "softmax";
    case AXHIP_ROWOP_LOGSOFTMAX: return "logsoftmax";
    case AXHIP_ROWOP_LAYERNORM: return "layernorm";
    case AXHIP_ROWOP_RMSNORM: return "rmsnorm";
    default: return "reduce";
    }
}
const char *rowop_token(const AxhipRowsProgram &P) { return P.row_op == AXHIP_ROWOP_NONE && P.reduce == AXHIP_RED_NONE ? "map" : rowop_token(P.row_op); }

uint64_t fnv1a(const std::string &s, uint64_t h = 14695981039346656037ull) {
    for (unsigned char c : s) {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

// operands of the chains, by kind, in the order the chains first name them
struct OperandTables {
    int n[4] = {0, 0, 0, 0};      // per AXHIP_BK_FULL / ROWVEC / COLVEC / SCALAR
    int dt[4][8] = {};
    int slot[4][8] = {};
    int of_operand[AXHIP_MAX_OPERANDS]; // operand index -> position in its kind's table, or -1
    OperandTables() { for (int &v : of_operand) v = -1; }
};

struct Builder {
    const AxhipRowsProgram &P;
    RowsProgSpec &S;
    OperandTables T;
    int slot_of_operand[AXHIP_MAX_OPERANDS];
    bool post_full = false;
    bool ok = true;

    Builder(const AxhipRowsProgram &p, RowsProgSpec &s) : P(p), S(s) {
        for (int &v : slot_of_operand) v = -1;
    }

    int pointer_slot(int operand) {
        if (slot_of_operand[operand] < 0) {
            if (S.n_slots >= 8) {
                ok = false;
                return 0;
            }
            slot_of_operand[operand] = S.n_slots;
            S.slot_operand[S.n_slots++] = operand;
        }
        return slot_of_operand[operand];
    }

    // expression text of a binary op's second operand
    std::string operand_expr(const AxhipChainOp &c, bool post, int position, std::string *token) {
        char buf[64];
        if (c.imm_kind == AXHIP_BK_IMM) {
            if (S.n_imm >= 32) {
                ok = false;
                return "0.0f";
            }
            S.imm_ref[S.n_imm] = {post, position};
            snprintf(buf, sizeof(buf), "q.imm[%d]", S.n_imm++);
            *token += "s";
            return buf;
        }
        const int idx = c.operand;
        if (idx < 0 || idx >= P.n_operands) {
            ok = false;
            return "0.0f";
        }
        const AxhipOperand &o = P.operands[idx];
        if (o.kind < AXHIP_BK_FULL || o.kind > AXHIP_BK_SCALAR) {
            ok = false;
            return "0.0f";
        }
        if (T.of_operand[idx] < 0) {
            const int k = o.kind;
            if (T.n[k] >= 8) {
                ok = false;
                return "0.0f";
            }
            T.of_operand[idx] = T.n[k];
            T.dt[k][T.n[k]] = o.dtype;
            T.slot[k][T.n[k]] = pointer_slot(idx);
            ++T.n[k];
        }
        const int at = T.of_operand[idx];
        switch (o.kind) {
        case AXHIP_BK_FULL:
            if (post) post_full = true;
            snprintf(buf, sizeof(buf), "q.full[%d][e]", at);
            *token += "f";
            break;
        case AXHIP_BK_ROWVEC:
            snprintf(buf, sizeof(buf), "q.rowv[%d][e]", at);
            *token += "r";
            break;
        case AXHIP_BK_COLVEC:
            snprintf(buf, sizeof(buf), "q.colv[%d]", at);
            *token += "c";
            break;
        default:
            snprintf(buf, sizeof(buf), "q.scal[%d]", at);
            *token += "s";
            break;
        }
        return buf;
    }

    // one chain as statements on `t`; appends the chain's tokens to the label
    std::string chain_text(const AxhipChainOp *ops, int n, bool post, int fast, std::string *label) {
        std::ostringstream o;
        for (int i = 0; i < n; ++i) {
            const int op = ops[i].op;
            const char *tok = op_token(op);
            if (!tok) {
                ok = false;
                return "";
            }
            std::string token = tok;
            if (is_binary(op)) {
                const std::string b = operand_expr(ops[i], post, i, &token);
                switch (op) {
                case AXHIP_OP_ADD: o << "    t = t + " << b << ";\n"; break;
                case AXHIP_OP_SUB: o << "    t = t - " << b << ";\n"; break;
                case AXHIP_OP_MUL: o << "    t = t * " << b << ";\n"; break;
                case AXHIP_OP_DIV: o << "    t = t / " << b << ";\n"; break;
                case AXHIP_OP_MAX: o << "    t = fmaxf(t, " << b << ");\n"; break;
                case AXHIP_OP_MIN: o << "    t = fminf(t, " << b << ");\n"; break;
                case AXHIP_OP_RSUB: o << "    t = " << b << " - t;\n"; break;
                case AXHIP_OP_RDIV: o << "    t = " << b << " / t;\n"; break;
                case AXHIP_OP_POW: o << "    t = powf(t, " << b << ");\n"; break;
                case AXHIP_OP_RPOW: o << "    t = powf(" << b << ", t);\n"; break;
                case AXHIP_OP_MOD: o << "    t = fmodf(t, " << b << ");\n"; break;
                case AXHIP_OP_RMOD: o << "    t = fmodf(" << b << ", t);\n"; break;
                case AXHIP_OP_ATAN2: o << "    t = atan2f(t, " << b << ");\n"; break;
                case AXHIP_OP_RATAN2: o << "    t = atan2f(" << b << ", t);\n"; break;
                case AXHIP_OP_HYPOT: o << "    t = hypotf(t, " << b << ");\n"; break;
                case AXHIP_OP_EQ: o << "    t = t == " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_NE: o << "    t = t != " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_LT: o << "    t = t < " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_LE: o << "    t = t <= " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_GT: o << "    t = t > " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_GE: o << "    t = t >= " << b << " ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_AND: o << "    t = (t != 0.0f) && (" << b << " != 0.0f) ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_OR: o << "    t = (t != 0.0f) || (" << b << " != 0.0f) ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_XOR: o << "    t = (t != 0.0f) != (" << b << " != 0.0f) ? 1.0f : 0.0f;\n"; break;
                default: o << "    t = t > 0.0f ? t : " << b << " * t;\n"; break; // leaky ReLU
                }
            } else if (is_unary(op)) {
                switch (op) {
                case AXHIP_OP_RELU: o << "    t = t > 0.0f ? t : 0.0f;\n"; break;
                case AXHIP_OP_GELU: o << (fast == 2 ? "    t = gelu_fast_bf16(t);\n" : fast ? "    t = gelu_fast(t);\n" : "    t = gelu_erfc(t);\n"); break;
                case AXHIP_OP_SQRT: o << "    t = sqrtf(t);\n"; break;
                case AXHIP_OP_EXP: o << "    t = expf(t);\n"; break;
                case AXHIP_OP_NEG: o << "    t = -t;\n"; break;
                case AXHIP_OP_ABS: o << "    t = fabsf(t);\n"; break;
                case AXHIP_OP_SIGMOID: o << "    t = sigmoid_fast(t);\n"; break;
                case AXHIP_OP_TANH: o << (fast ? "    t = tanh_fast(t);\n" : "    t = tanhf(t);\n"); break;
                case AXHIP_OP_SILU: o << "    t = silu_fast(t);\n"; break;
                case AXHIP_OP_LOG: o << "    t = logf(t);\n"; break;
                case AXHIP_OP_SQUARE: o << "    t = t * t;\n"; break;
                case AXHIP_OP_RSQRT: o << "    t = 1.0f / sqrtf(t);\n"; break;
                case AXHIP_OP_RECIP: o << "    t = 1.0f / t;\n"; break;
                case AXHIP_OP_ERF: o << "    t = erff(t);\n"; break;
                case AXHIP_OP_SIN: o << "    t = sinf(t);\n"; break;
                case AXHIP_OP_COS: o << "    t = cosf(t);\n"; break;
                case AXHIP_OP_TAN: o << "    t = tanf(t);\n"; break;
                case AXHIP_OP_SIGN: o << "    t = t > 0.0f ? 1.0f : t < 0.0f ? -1.0f : 0.0f;\n"; break;
                case AXHIP_OP_FLOOR: o << "    t = floorf(t);\n"; break;
                case AXHIP_OP_CEIL: o << "    t = ceilf(t);\n"; break;
                case AXHIP_OP_ROUND: o << "    t = roundf(t);\n"; break;
                case AXHIP_OP_TRUNC: o << "    t = truncf(t);\n"; break;
                case AXHIP_OP_CBRT: o << "    t = cbrtf(t);\n"; break;
                case AXHIP_OP_ISNAN: o << "    t = t != t ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_ISINF: o << "    t = fabsf(t) == __builtin_huge_valf() ? 1.0f : 0.0f;\n"; break;
                case AXHIP_OP_ISFINITE: o << "    t = fabsf(t) < __builtin_huge_valf() ? 1.0f : 0.0f;\n"; break;
                default: o << "    t = t == 0.0f ? 1.0f : 0.0f;\n"; break; // logical not
                }
            } else {
                ok = false;
                return "";
            }
            *label += token + "_";
        }
        return o.str();
    }
};

std::string int_table(const char *name, const int *v, int n) {
    std::ostringstream o;
    o << "constexpr int " << name << "[" << (n > 0 ? n : 1) << "] = {";
    for (int i = 0; i < (n > 0 ? n : 1); ++i) o << (i ? ", " : "") << (i < n ? v[i] : 0);
    o << "};\n";
    return o.str();
}

} // namespace

namespace {
bool names_operand(const AxhipRowsProgram &P, int idx) {
    auto in = [&](const AxhipChainOp *ops, int n) {
        for (int i = 0; i < n; ++i)
            if (is_binary(ops[i].op) && ops[i].imm_kind != AXHIP_BK_IMM && ops[i].operand == idx) return true;
        return false;
    };
    return in(P.pre, P.n_pre) || in(P.post, P.n_post);
}
} // namespace

// Elements per chunk: 16 bytes of the widest full-size stream (the input, a full-size output, the full-size operands
// the chains name), so that every access of every stream is a contiguous run across the lanes of a wave: 4 as soon as
// one of them is fp32 (a 16-bit stream then moves 8 bytes per lane), else 8.
int rows_prog_chunk_elems(const AxhipRowsProgram &P) {
    bool wide = P.input_dtype == AXHIP_DTYPE_F32 || (P.reduce == AXHIP_RED_NONE && P.output_dtype == AXHIP_DTYPE_F32);
    for (int i = 0; i < P.n_operands; ++i)
        if (P.operands[i].kind == AXHIP_BK_FULL && P.operands[i].dtype == AXHIP_DTYPE_F32 && names_operand(P, i)) wide = true;
    return wide ? 4 : 8;
}

namespace {
// 32-bit words of raw input a thread holds per chunk: the input and every full-size operand the chains name
int raw_words_per_chunk(const AxhipRowsProgram &P) {
    const int e = rows_prog_chunk_elems(P);
    int words = e * elem_size(P.input_dtype) / 4;
    bool used[AXHIP_MAX_OPERANDS] = {};
    auto mark = [&](const AxhipChainOp *ops, int n) {
        for (int i = 0; i < n; ++i)
            if (is_binary(ops[i].op) && ops[i].imm_kind != AXHIP_BK_IMM && ops[i].operand >= 0 && ops[i].operand < P.n_operands) used[ops[i].operand] = true;
    };
    mark(P.pre, P.n_pre);
    mark(P.post, P.n_post);
    for (int i = 0; i < P.n_operands; ++i)
        if (used[i] && P.operands[i].kind == AXHIP_BK_FULL) words += e * elem_size(P.operands[i].dtype) / 4;
    return words;
}
// the same for the norm weight and bias of a row that spans several waves (a wavefront row reads them from LDS, a
// 1024-thread block requests them one chunk at a time)
int affine_words_per_chunk(const AxhipRowsProgram &P, int group) {
    if (group <= 64 || group == 1024) return 0;
    const int e = rows_prog_chunk_elems(P);
    int words = 0;
    for (int idx : {P.norm_weight, P.norm_bias})
        if (idx >= 0 && idx < P.n_operands) words += e * elem_size(P.operands[idx].dtype) / 4;
    return words;
}
} // namespace

bool rows_prog_grid_pays(const AxhipRowsProgram &P, int group, int it) {
    // Measured on rows of 1001 to 100 003 columns: chunks on memory's grid gain 2 to 25 % where every stream is
    // full-size; at two chunks per lane the extra chunk costs more than that.  A per-column operand ([cols] weights:
    // their position in the row no longer matches their address) costs 5 to 20 % on the grid in rows of up to 512
    // threads (wavefront rows stage it in LDS once per block when the chunks start at the row's first element) --
    // 1024-thread rows gain even so: their unaligned form spills (layer norm over 50 257 fp32 columns: 404 -> 172 us).
    if (group < 64) return true; // short rows: on the grid they share a wavefront, from their first element each takes one
    // AXHIP_ROWS_GRID=1 / 0 (read once): the grid wherever a plan exists for it / never beyond the short rows -- a
    // tuning switch for measurements
    static const int forced = [] {
        const char *e = getenv("AXHIP_ROWS_GRID");
        return e && *e ? atoi(e) : -1;
    }();
    if (forced == 1) return true;
    if (forced == 0) return false;
    if (group * it <= 128) return false;
    if (group > 512) return true;
    auto rowvec = [&](int idx) { return idx >= 0 && idx < P.n_operands && P.operands[idx].kind == AXHIP_BK_ROWVEC; };
    if (rowvec(P.norm_weight) || rowvec(P.norm_bias)) return false;
    for (int stage = 0; stage < 2; ++stage) {
        const AxhipChainOp *ops = stage ? P.post : P.pre;
        const int n = stage ? P.n_post : P.n_pre;
        for (int i = 0; i < n; ++i)
            if (is_binary(ops[i].op) && ops[i].imm_kind != AXHIP_BK_IMM && rowvec(ops[i].operand)) return false;
    }
    return true;
}

void rows_prog_plan_for(const AxhipRowsProgram &P, int group, int it, bool ragged, RowsProgPlan *plan, bool grid) {
    plan->group = group;
    plan->it = it;
    plan->ragged = ragged;
    plan->grid = ragged && grid;
    const bool heavy = ragged && !grid; // unaligned chunks carry an address and an element count each in registers
    // Pipelining keeps a second set of raw words alive: worth it while that set is at most 32 registers (a 16-bit
    // row of 4096 columns per wavefront, or a row with one operand at half that).  Ragged rows carry their chunk
    // bookkeeping in registers too and pipeline at half that.
    const int raw = raw_words_per_chunk(P), all = raw + affine_words_per_chunk(P, group);
    plan->pipe = all * it <= (heavy ? 16 : ragged ? 24 : 32); // (rows on the moving grid keep their end-of-row masks too)
    // Register allocation aims at 4 waves per SIMD (128 registers per thread).  The widest plans hold more than
    // that with their operands: they get the registers of 2 waves per SIMD instead of spilling.
    const bool resident_f32 = P.input_dtype == AXHIP_DTYPE_F32 || P.n_pre > 0 || P.row_op == AXHIP_ROWOP_SOFTMAX || P.row_op == AXHIP_ROWOP_LOGSOFTMAX;
    const int held = all * it + (resident_f32 && P.row_op != AXHIP_ROWOP_NONE ? rows_prog_chunk_elems(P) * it : 0);
    plan->min_waves = (held + (heavy ? 3 * it + 16 : 0) > 72 || it > 8) ? 2 : 4;
    // short rows on the grid: every row has a shift of its own, so a pipelined plan works out the next row's chunk
    // offsets on top of this row's (AXHIP_ROWS_PIPE_SHORT_GRID=0, read once: not pipelined; layer norm with weight
    // and bias over 170000 rows of 197 16-bit columns 63 against 79 us, softmax the same either way)
    static const bool pipe_short_grid = [] { const char *e = getenv("AXHIP_ROWS_PIPE_SHORT_GRID"); return !(e && e[0] == '0'); }();
    if (group < 64 && plan->grid && !pipe_short_grid) plan->pipe = false;
    // (AXHIP_ROWS_PIPE=0, read once: no plan is pipelined -- for measurements)
    static const bool pipe_off = [] { const char *v = getenv("AXHIP_ROWS_PIPE"); return v && v[0] == '0'; }();
    if (pipe_off) plan->pipe = false;
    // a 1024-thread block has 128 registers per thread whatever is asked for: no second set of raw words beyond that
    if (group == 1024 && held + (plan->pipe ? raw * it : 0) > 115) plan->pipe = false;
}

namespace {
bool plan_rows(const AxhipRowsProgram &P, bool tight, bool ragged, bool grid, RowsProgPlan *plan);
}

bool rows_prog_flat_large(const AxhipRowsProgram &P) {
    return P.rows >= 1024 && P.rows * P.cols * static_cast<int64_t>(elem_size(P.input_dtype)) >= (int64_t(8) << 20);
}

bool rows_prog_plan(const AxhipRowsProgram &P, bool tight, RowsProgPlan *plan) {
    if (P.cols <= 0) return false;
    // Flat elementwise chains have kernels of their own, which walk the chain's operations chunk by chunk; large ones
    // over aligned rows run here instead, as a row program without a row operation -- straight-line code, up to eight
    // chunks per lane requested together, the next row meanwhile: relu over bf16 [16384,4096] 68 -> 86 % of the HBM
    // peak back to back and 54 -> 71 % with the input from HBM, gelu 65 -> 80 % / 52 -> 69 %, x * y + z about the same.
    // AXHIP_ROWS_FLAT=0 (read once) keeps them all on the walking kernels.
    const bool flat = P.row_op == AXHIP_ROWOP_NONE && P.reduce == AXHIP_RED_NONE;
    if (flat) {
        static const bool flat_on = [] { const char *v = getenv("AXHIP_ROWS_FLAT"); return !(v && v[0] == '0'); }();
        if (!flat_on || !tight || !rows_prog_flat_large(P)) return false;
    }
    // products and one-byte streams (a Bool input, operand or full-size result) stay with the interpreter; a reduced
    // [rows] result may be a byte (any / all)
    // (an elementwise chain may leave truth values: a comparison's result, one byte per element)
    if (P.reduce > AXHIP_RED_MIN || P.input_dtype == AXHIP_DTYPE_U8 || (P.reduce == AXHIP_RED_NONE && P.output_dtype == AXHIP_DTYPE_U8 && P.row_op != AXHIP_ROWOP_NONE)) return false;
    for (int i = 0; i < P.n_operands; ++i)
        if (P.operands[i].dtype == AXHIP_DTYPE_U8) return false;
    const int dt = P.input_dtype;
    const int e = rows_prog_chunk_elems(P);
    bool ragged = P.cols % e != 0 || !aligned16(P.input) || (P.reduce == AXHIP_RED_NONE && !aligned16(P.output));
    bool same_size = P.reduce != AXHIP_RED_NONE || elem_size(P.output_dtype) == elem_size(dt);
    bool used[AXHIP_MAX_OPERANDS] = {};
    auto mark = [&](const AxhipChainOp *ops, int n) {
        for (int i = 0; i < n; ++i)
            if (is_binary(ops[i].op) && ops[i].imm_kind != AXHIP_BK_IMM && ops[i].operand >= 0 && ops[i].operand < P.n_operands) used[ops[i].operand] = true;
    };
    mark(P.pre, P.n_pre);
    mark(P.post, P.n_post);
    if (P.norm_weight >= 0 && P.norm_weight < P.n_operands) used[P.norm_weight] = true;
    if (P.norm_bias >= 0 && P.norm_bias < P.n_operands) used[P.norm_bias] = true;
    for (int i = 0; i < P.n_operands; ++i) {
        if (!used[i]) continue;
        const AxhipOperand &o = P.operands[i];
        if (o.kind == AXHIP_BK_FULL || o.kind == AXHIP_BK_ROWVEC) {
            if (!aligned16(o.ptr)) ragged = true;
            if (elem_size(o.dtype) != elem_size(dt)) same_size = false;
        }
    }
    // Short rows of odd length, many of them: a row per lane (or per 2, 4 or 8 lanes) out of a span staged in LDS
    // (every stream has its own geometry there, so the element sizes may differ).  All full-size streams must start
    // on a 16-byte boundary.  Tuning switches, read once: AXHIP_ROWS_LANE=0 switches the plan off,
    // AXHIP_ROWS_LANE_L=<1|2|4|8> sets the lanes per row, AXHIP_ROWS_LANE_VALS=<n> the values per lane from which a
    // row is spread over more lanes, AXHIP_ROWS_LANE_MAX=<n> the values per lane beyond which the plan is not taken.
    // Measured (16-bit softmax, % of the HBM peak with 1 / 2 / 4 / 8 lanes per row): 77 columns 71 / 73 / 61 / 54,
    // 197 columns 54 / 66 / 68 / 71, 250 columns 50 / 67 / 75 / 74, 513 columns - / - / 61 / 68 (a wavefront per row:
    // 50), 1001 columns - / - / 49 / 63 (a wavefront per row: 69).
    if (flat && (ragged || (P.cols + e - 1) / e > 2048)) return false; // (rows of odd length: the flat walk; longer rows: more rows of fewer columns would do)
    if (tight && !flat && P.cols % e != 0 && P.rows >= kRowsProgLaneMinRows) {
        static const bool lane_on = [] { const char *v = getenv("AXHIP_ROWS_LANE"); return !(v && v[0] == '0'); }();
        static const int lane_l = [] { const char *v = getenv("AXHIP_ROWS_LANE_L"); return v ? std::atoi(v) : 0; }();
        static const int lane_vals = [] { const char *v = getenv("AXHIP_ROWS_LANE_VALS"); return v ? std::atoi(v) : 64; }();
        static const int lane_most = [] { const char *v = getenv("AXHIP_ROWS_LANE_MAX"); return v ? std::atoi(v) : 96; }();
        bool ok = lane_on && aligned16(P.input) && (P.reduce != AXHIP_RED_NONE || aligned16(P.output));
        int widest = elem_size(dt), nreg = 1;
        if (P.reduce == AXHIP_RED_NONE) {
            widest = std::max(widest, static_cast<int>(elem_size(P.output_dtype)));
            if (elem_size(P.output_dtype) != elem_size(dt)) ++nreg;
        }
        for (int i = 0; i < P.n_operands; ++i)
            if (used[i] && P.operands[i].kind == AXHIP_BK_FULL) {
                ok = ok && aligned16(P.operands[i].ptr);
                widest = std::max(widest, static_cast<int>(elem_size(P.operands[i].dtype)));
                ++nreg;
            }
        const int64_t chunks = (P.cols + e - 1) / e;
        int lanes = (lane_l == 1 || lane_l == 2 || lane_l == 4 || lane_l == 8) ? lane_l : 1;
        // LDS bytes per wavefront and stream: the span, and room for a chunk that a lane reads past its end
        auto bytes_for = [&](int l) { return (64 / l * P.cols * widest + 32 + 16 * l + 1023) / 1024 * 1024; };
        if (lanes != lane_l)
            while (lanes < 8 && ((chunks + lanes - 1) / lanes * e > lane_vals || nreg * bytes_for(lanes) > 36864)) lanes *= 2;
        const int64_t it = (chunks + lanes - 1) / lanes;
        const int64_t lane_bytes = bytes_for(lanes);
        if (ok && it * e <= std::min(lane_most, 256) && nreg * lane_bytes <= 36864) {
            rows_prog_plan_for(P, 64, static_cast<int>(it), false, plan, false);
            plan->pipe = false;
            plan->min_waves = it * e > 160 ? 1 : it * e > 64 ? 2 : 4;
            plan->lane = true;
            plan->lane_l = lanes;
            plan->lane_bytes = static_cast<int>(lane_bytes);
            return true;
        }
    }
    // a ragged row is addressed in 16-byte chunks of every vector it touches: all of them must share the element size
    if (ragged && !same_size) return false;
    // When the input, the full-size operands and a full-size output sit at the same address modulo 16 (the usual case:
    // aligned allocations, a row length that is not a multiple of the chunk), the chunks follow memory's 16-byte grid:
    // every access aligned, a partial chunk at either end of a row, hence one chunk more than the row's own count.
    bool grid = ragged;
    if (grid) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(P.input) & 15u;
        if (P.reduce == AXHIP_RED_NONE && (reinterpret_cast<uintptr_t>(P.output) & 15u) != a) grid = false;
        for (int i = 0; i < P.n_operands; ++i)
            if (used[i] && P.operands[i].kind == AXHIP_BK_FULL && (reinterpret_cast<uintptr_t>(P.operands[i].ptr) & 15u) != a) grid = false;
    }
    if (grid && plan_rows(P, tight, ragged, true, plan) && rows_prog_grid_pays(P, plan->group, plan->it)) return true;
    if (P.cols < e) return false; // (rows shorter than a chunk: on the grid or not at all)
    return plan_rows(P, tight, ragged, false, plan);
}

namespace {
bool plan_rows(const AxhipRowsProgram &P, bool tight, bool ragged, bool grid, RowsProgPlan *plan) {
    *plan = RowsProgPlan{};
    const int dt = P.input_dtype;
    const int e = rows_prog_chunk_elems(P);
    const int64_t chunks = grid ? (P.cols + 2 * e - 2) / e : (P.cols + e - 1) / e;
    int group = 0, it = 0;
    // Short aligned rows (up to 32 chunks: 256 16-bit or 128 fp32 columns) share a wavefront: 4, 8, 16 or 32 lanes per
    // row, one chunk each, instead of a wavefront with most of its lanes idle (softmax over 64 16-bit columns ran at
    // 17 % of the HBM peak that way).  The build compiles these plans too.
    if ((!ragged || grid) && chunks <= 32) {
        const int g = chunks <= 4 ? 4 : chunks <= 8 ? 8 : chunks <= 16 ? 16 : 32;
        rows_prog_plan_for(P, g, 1, ragged, plan, grid);
        return true;
    }
    if (grid && P.cols < 2 * e) return false; // (longer plans on the grid count on a row's two ends lying in different chunks)
    if (!tight) {
        // the shapes the build compiles (rows_aot_gen.cpp): a wavefront per row with 1, 2, 3, 4, 5, 6 or 8 chunks per
        // lane, a 256-thread block per row with 3, 4 or 8 chunks per thread
        if (chunks <= 512) {
            group = 64;
            it = static_cast<int>((chunks + 63) / 64);
            if (it == 7) it = 8;
        } else if (chunks <= 2048) {
            group = 256;
            it = chunks <= 768 ? 3 : chunks <= 1024 ? 4 : 8;
        } else {
            return false;
        }
    } else {
        // the tightest fit among 64, 256, 512 and 1024 threads per row with up to 8 chunks each: fewest chunk slots (idle lanes
        // still issue their loads and arithmetic), then the smaller group
        static const int groups[4] = {64, 256, 512, 1024};
        // AXHIP_ROWS_GROUP (64, 256, 512, 1024; read once): take that many threads per row wherever the row fits them with up
        // to 8 chunks each -- a tuning switch for measurements, the default choice below is what the benchmarks ran
        static const int forced = [] {
            const char *e = std::getenv("AXHIP_ROWS_GROUP");
            return e ? std::atoi(e) : 0;
        }();
        int64_t best = 0;
        for (int i = 0; i < 4; ++i) {
            if (forced == groups[i] && (chunks + groups[i] - 1) / groups[i] <= (groups[i] == 64 ? 10 : 8) && chunks >= groups[i]) {
                group = groups[i];
                it = static_cast<int>((chunks + groups[i] - 1) / groups[i]);
                break;
            }
            const int64_t n = (chunks + groups[i] - 1) / groups[i];
            // up to 8 chunks per thread; a wavefront row may take 9 or 10 (a row just past 512 chunks would otherwise
            // leave a third of a 256-thread block idle) while the row fits the registers of 2 waves per SIMD (two 16-bit
            // streams of 4099 columns, held as fp32 as well: 144 registers, 72 against 95 us for the 256-thread plan)
            if (n > 8) {
                const bool resident_f32 = P.row_op != AXHIP_ROWOP_NONE && (dt == AXHIP_DTYPE_F32 || P.n_pre > 0 || P.row_op == AXHIP_ROWOP_SOFTMAX || P.row_op == AXHIP_ROWOP_LOGSOFTMAX);
                const int64_t held = (raw_words_per_chunk(P) + (resident_f32 ? rows_prog_chunk_elems(P) : 0)) * n;
                if (!(groups[i] == 64 && n <= 10 && held <= 160)) continue;
            }
            if (group == 0 || n * groups[i] < best) {
                group = groups[i];
                it = static_cast<int>(n);
                best = n * groups[i];
            }
        }
        bool rerun = false;
        if (group == 0) {
            // Longer rows: up to 16 chunks per thread of a 1024-thread block, held as the raw words they were loaded as
            // (at most 64 registers) instead of as fp32 -- still one read of the row, at the price of unpacking it and
            // running the pre chain once per pass.
            const int64_t n = (chunks + 1023) / 1024;
            if (n > 16 || raw_words_per_chunk(P) * n > 72) {
                // Longer still (aligned rows): a 1024-thread block walks the row in steps of 4 chunks per thread (2 when
                // the operands of a step would not fit 64 registers), once for the statistics and once for the output.
                if (ragged) return false;
                rows_prog_plan_for(P, 1024, raw_words_per_chunk(P) * 4 <= 64 ? 4 : 2, false, plan, false);
                plan->loop = true;
                plan->pipe = false;
                plan->min_waves = 4;
                return true;
            }
            group = 1024;
            it = static_cast<int>(n);
            rerun = true;
        }
        rows_prog_plan_for(P, group, it, ragged, plan, grid);
        // chunk c of a row on the grid lies inside the row for every shift when (c + 1) * e <= cols (and c > 0): true of
        // all chunks of a thread's first cols / e / group -- the last one or two per thread in a tight plan are in doubt
        if (plan->grid) plan->tail_from = static_cast<int>(std::min<int64_t>(std::max(it - 2, 0), P.cols / e / group));
        if (rerun) {
            plan->rerun = true;
            plan->pipe = false;
        }
        return true;
    }
    rows_prog_plan_for(P, group, it, ragged, plan, grid);
    return true;
}
} // namespace

bool rows_prog_spec(const AxhipRowsProgram &P, const RowsProgPlan &plan, RowsProgSpec *spec) {
    RowsProgSpec &S = *spec;
    S = RowsProgSpec{};
    Builder B(P, S);
    const int dt = P.input_dtype;
    // the result is rounded to 16 bits: fast activation forms, sized to the result's precision (8 bits for bf16, 11 for f16)
    const int fast = P.output_dtype == AXHIP_DTYPE_BF16 ? 2 : P.output_dtype == AXHIP_DTYPE_F16 ? 1 : 0;
    const bool is_norm = P.row_op == AXHIP_ROWOP_LAYERNORM || P.row_op == AXHIP_ROWOP_RMSNORM;

    int w_dt = -1, b_dt = -1, w_slot = -1, b_slot = -1;
    if (P.norm_weight >= 0) {
        if (!is_norm || P.norm_weight >= P.n_operands || P.operands[P.norm_weight].kind != AXHIP_BK_ROWVEC) return false;
        w_dt = P.operands[P.norm_weight].dtype;
        w_slot = B.pointer_slot(P.norm_weight);
    }
    if (P.norm_bias >= 0) {
        if (P.row_op != AXHIP_ROWOP_LAYERNORM || P.norm_bias >= P.n_operands || P.operands[P.norm_bias].kind != AXHIP_BK_ROWVEC) return false;
        b_dt = P.operands[P.norm_bias].dtype;
        b_slot = B.pointer_slot(P.norm_bias);
    }
    std::string pre_label, post_label;
    const std::string pre = B.chain_text(P.pre, P.n_pre, false, fast, &pre_label);
    const std::string post = B.chain_text(P.post, P.n_post, true, fast, &post_label);
    if (!B.ok) return false;
    bool pipe = plan.pipe;
    const bool resident = P.row_op != AXHIP_ROWOP_NONE && !(is_norm && dt != AXHIP_DTYPE_F32 && P.n_pre == 0);
    if (resident && B.post_full) pipe = false;

    const int red = P.reduce == AXHIP_RED_MEAN ? AXHIP_RED_SUM : P.reduce;
    std::ostringstream c;
    c << "constexpr int DT_IN = " << dt << ", DT_OUT = " << (P.reduce == AXHIP_RED_NONE ? P.output_dtype : dt) << ";\n";
    c << "constexpr int GROUP = " << plan.group << ", IT = " << (plan.lane ? 1 : plan.it) << ", E = " << rows_prog_chunk_elems(P) << ";\n";
    const bool rerun = plan.rerun && resident; // (a 16-bit norm without a pre chain never holds its row as fp32 anyway)
    if (rerun) pipe = false;
    c << "constexpr bool RAGGED = " << (plan.ragged ? "true" : "false") << ", PIPE = " << (pipe ? "true" : "false") << ", RERUN = " << (rerun ? "true" : "false")
      << ", GRID = " << (plan.ragged && plan.grid ? "true" : "false") << ";\n";
    c << "constexpr bool LOOP = " << (plan.loop ? "true" : "false") << ";\n";
    // looped rows with a row operation keep the raw words of their first steps: up to 48 registers per thread
    c << "constexpr int HOLD = " << (plan.loop && P.row_op != AXHIP_ROWOP_NONE ? 48 / (raw_words_per_chunk(P) * plan.it) : 0) << ";\n";
    c << "constexpr int TAIL_FROM = " << (plan.ragged && plan.grid ? plan.tail_from : 0) << ";\n";
    c << "constexpr int MIN_WAVES = " << plan.min_waves << ";\n";
    if (plan.lane) c << "constexpr int LANE_BYTES = " << plan.lane_bytes << ", LANE_IT = " << plan.it << ", LANE_L = " << plan.lane_l << ";\n";
    c << "constexpr int ROWOP = " << P.row_op << ", RED = " << red << ";\n";
    c << "constexpr int W_DT = " << w_dt << ", B_DT = " << b_dt << ", W_SLOT = " << w_slot << ", B_SLOT = " << b_slot << ";\n";
    static const char *kind_name[4] = {"FULL", "ROWV", "COLV", "SCAL"};
    for (int k = 0; k < 4; ++k) {
        c << "constexpr int N" << kind_name[k] << " = " << B.T.n[k] << ";\n";
        c << int_table((std::string(kind_name[k]) + "_DT").c_str(), B.T.dt[k], B.T.n[k]);
        c << int_table((std::string(kind_name[k]) + "_SLOT").c_str(), B.T.slot[k], B.T.n[k]);
    }
    c << "constexpr bool HAS_PRE = " << (P.n_pre > 0 ? "true" : "false") << ", POST_FULL = " << (B.post_full ? "true" : "false") << ";\n";
    S.config = c.str();

    std::ostringstream f;
    f << "__device__ __forceinline__ float pre_chain(float t, const Env &q, int e) {\n" << pre << "    return t;\n}\n";
    f << "__device__ __forceinline__ float post_chain(float t, const Env &q, int e) {\n" << post << "    return t;\n}\n";
    S.chains = f.str();

    char hash[24];
    snprintf(hash, sizeof(hash), "%016llx", static_cast<unsigned long long>(fnv1a(S.chains, fnv1a(S.config))));
    S.threads = plan.lane ? 64 : plan.group > 256 ? plan.group : 256;
    // bytes a block has requested and not yet used: its threads' chunks of every full-size input, twice when pipelined
    S.pipelined = pipe;
    S.post_ops = P.n_post;
    // (rows of odd length spend their time on instructions: they keep every wave slot)
    S.inflight_bytes = plan.lane || plan.ragged ? 0 : static_cast<int64_t>(S.threads) * plan.it * 4 * raw_words_per_chunk(P) * (pipe ? 2 : 1);
    S.rows_per_block = plan.lane ? 64 / plan.lane_l : S.threads / plan.group;
    S.lane = plan.lane;

    std::string label = pre_label + rowop_token(P) + "_" + post_label;
    if (w_dt >= 0) label += b_dt >= 0 ? "wb_" : "w_";
    else if (b_dt >= 0) label += "b_";
    if (red != AXHIP_RED_NONE) label += red == AXHIP_RED_SUM ? "sum_" : red == AXHIP_RED_MAX ? "max_" : "min_";
    char tail[64];
    const bool other_out = P.reduce == AXHIP_RED_NONE && P.output_dtype != dt;
    if (plan.lane) // (a row per lane; the LDS bytes per wavefront and stream in KiB)
        snprintf(tail, sizeof(tail), "%s%s%s_lane%d_%dk_it%d", dt_name(dt), other_out ? "_to_" : "", other_out ? dt_name(P.output_dtype) : "", plan.lane_l,
                 plan.lane_bytes / 1024, plan.it);
    else
    snprintf(tail, sizeof(tail), "%s%s%s_g%d_it%d%s", dt_name(dt), other_out ? "_to_" : "", other_out ? dt_name(P.output_dtype) : "", plan.group, plan.it,
             plan.loop ? "_loop" : !plan.ragged ? "" : plan.grid ? "_grid" : "_ragged"); // (grid: ragged rows addressed on memory's 16-byte grid)
    S.label = label + tail;
    // the kernel's symbol: the readable label (what a profiler lists) plus a hash of everything that shapes the code
    S.symbol = "axp_" + S.label + "_" + hash;
    return true;
}

void rows_prog_bind(const AxhipRowsProgram &P, const RowsProgSpec &S, RowsProgArgs *a) {
    *a = RowsProgArgs{};
    a->x = P.input;
    a->y = P.output;
    a->rows = P.rows;
    a->cols = P.cols;
    for (int i = 0; i < S.n_slots; ++i) a->ptr[i] = P.operands[S.slot_operand[i]].ptr;
    for (int i = 0; i < S.n_imm; ++i) a->imm[i] = S.imm_ref[i].post ? P.post[S.imm_ref[i].index].imm : P.pre[S.imm_ref[i].index].imm;
    a->eps = P.eps;
    // a full-size output far larger than the caches is written around them, so that it does not push the launch's own
    // inputs out of the last-level cache
    const int64_t out_bytes = P.rows * P.cols * static_cast<int64_t>(elem_size(P.output_dtype));
    // (AXHIP_ROWS_STREAM_OUT_MB=<n>, read once, moves the size.  A consumer that reads such an output next finds it in
    // HBM, not in the cache: relu -> softmax over bf16 [16384,4096] 50.0 + 50.6 us; with the output written through the
    // caches the producer takes 59.9 us and the consumer 46.4 us -- 5.7 us more for the pair.)
    static const int64_t stream_from = [] { const char *v = getenv("AXHIP_ROWS_STREAM_OUT_MB"); return (v ? atoll(v) : 64ll) << 20; }();
    a->stream_out = P.reduce == AXHIP_RED_NONE && out_bytes >= stream_from;
    a->red_scale = P.reduce == AXHIP_RED_MEAN ? 1.0f / static_cast<float>(P.cols) : 1.0f;
    a->red_dt = P.output_dtype;
}

std::string rows_prog_source(const RowsProgSpec &S, const std::string &body) {
    std::string ns = "ns_" + S.symbol;
    std::string src;
    src.reserve(body.size() + S.config.size() + S.chains.size() + 256);
    src += "#define AXP_NS " + ns + "\n#define AXP_KERNEL_NAME " + S.symbol + "\n";
    if (S.lane) src += "#define AXP_LANE 1\n";
    src += "namespace " + ns + " { namespace cfg {\n" + S.config + "} }\n";
    src += body;
    src += "\nnamespace " + ns + " {\n" + S.chains + "}\n";
    return src;
}

// ------------------------------------------------------------------ kernels built into the library
namespace {
std::map<std::string, const void *> &builtin_table() {
    static std::map<std::string, const void *> t;
    return t;
}
std::mutex &builtin_mutex() {
    static std::mutex m;
    return m;
}
} // namespace

RowsProgRegistrar::RowsProgRegistrar(const char *key, const void *kernel) {
    std::lock_guard<std::mutex> lock(builtin_mutex());
    builtin_table()[key] = kernel;
}

const void *rows_prog_find_builtin(const std::string &key) {
    std::lock_guard<std::mutex> lock(builtin_mutex());
    auto it = builtin_table().find(key);
    return it == builtin_table().end() ? nullptr : it->second;
}

} // namespace axhip
