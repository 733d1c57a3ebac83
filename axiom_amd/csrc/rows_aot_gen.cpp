// Build-time tool: writes the source files of the fused-row kernels that are compiled into the library.
//
//     rows_aot_gen <output directory> <number of files>
//
// A short list of program shapes (see shapes_of) for every register plan and both the aligned and the ragged row
// form.  Any other shape is compiled by the library at run time, from the same generator, and kept on disk.
#include <cstdio>
#include <cstring>
#include <fstream>
#include <set>
#include <string>
#include <vector>

#include "rows_codegen.hpp"

using namespace axhip;

namespace {

struct Shape {
    AxhipRowsProgram p;
};

void *fake(int i) { return reinterpret_cast<void *>(static_cast<uintptr_t>(0x1000 * (i + 1))); }

AxhipRowsProgram base(int dt) {
    AxhipRowsProgram p;
    memset(&p, 0, sizeof(p));
    p.rows = 1;
    p.cols = 8;
    p.input = fake(0);
    p.output = fake(1);
    p.input_dtype = p.output_dtype = dt;
    p.norm_weight = p.norm_bias = -1;
    return p;
}
int add_operand(AxhipRowsProgram &p, int dt, int kind) {
    p.operands[p.n_operands] = {fake(2 + p.n_operands), dt, kind};
    return p.n_operands++;
}
void push(AxhipChainOp *chain, int32_t &n, int op, int operand, bool imm) {
    chain[n].op = op;
    chain[n].operand = imm ? -1 : operand;
    chain[n].imm = 0.0f;
    chain[n].imm_kind = imm ? AXHIP_BK_IMM : 0;
    ++n;
}
// `s`: the chain's scalar as an immediate (true) or as a one-element device operand (false)
enum Pre { PRE_NONE, PRE_ADDF, PRE_MULF, PRE_MULS, PRE_MULS_ADDF, PRE_RELU_ADDS_MULF };
void add_pre(AxhipRowsProgram &p, int dt, Pre pre, bool imm) {
    const int s = (pre == PRE_MULS || pre == PRE_MULS_ADDF || pre == PRE_RELU_ADDS_MULF) && !imm ? add_operand(p, dt, AXHIP_BK_SCALAR) : -1;
    switch (pre) {
    case PRE_NONE: break;
    case PRE_ADDF: push(p.pre, p.n_pre, AXHIP_OP_ADD, add_operand(p, dt, AXHIP_BK_FULL), false); break;
    case PRE_MULF: push(p.pre, p.n_pre, AXHIP_OP_MUL, add_operand(p, dt, AXHIP_BK_FULL), false); break;
    case PRE_MULS: push(p.pre, p.n_pre, AXHIP_OP_MUL, s, imm); break;
    case PRE_MULS_ADDF:
        push(p.pre, p.n_pre, AXHIP_OP_MUL, s, imm);
        push(p.pre, p.n_pre, AXHIP_OP_ADD, add_operand(p, dt, AXHIP_BK_FULL), false);
        break;
    case PRE_RELU_ADDS_MULF:
        push(p.pre, p.n_pre, AXHIP_OP_RELU, -1, false);
        push(p.pre, p.n_pre, AXHIP_OP_ADD, s, imm);
        push(p.pre, p.n_pre, AXHIP_OP_MUL, add_operand(p, dt, AXHIP_BK_FULL), false);
        break;
    }
}

// The shapes compiled into the library: what BASELINE's configurations launch, the row forms of the reference's
// GPU builders (softmax / log-softmax / layer norm / RMS norm / row reductions,
// src/backends/metal/mpsgraph_graph_compiler.mm:287-330, :576-604) alone and behind the prefixes the reference's
// fused patterns put in front of them (src/graph/fused_patterns.cpp:12-71: x + y, x * s, x * y, relu / square / abs),
// and the row reductions that full reductions are folded onto.  Everything else is compiled when first launched and
// kept in the on-disk cache; a built-in and a run-time compiled kernel come out of the same generator.
std::vector<AxhipRowsProgram> shapes_of(int dt, int *n_primary) {
    std::vector<AxhipRowsProgram> out;
    auto softmax_like = [&](int rowop, Pre pre, bool imm) {
        AxhipRowsProgram p = base(dt);
        add_pre(p, dt, pre, imm);
        p.row_op = rowop;
        out.push_back(p);
    };
    auto norm = [&](int rowop, Pre pre, bool affine, int post) {
        AxhipRowsProgram p = base(dt);
        if (affine) {
            p.norm_weight = add_operand(p, dt, AXHIP_BK_ROWVEC);
            if (rowop == AXHIP_ROWOP_LAYERNORM) p.norm_bias = add_operand(p, dt, AXHIP_BK_ROWVEC);
        }
        add_pre(p, dt, pre, true);
        p.row_op = rowop;
        if (post) push(p.post, p.n_post, post, -1, false);
        out.push_back(p);
    };
    auto reduction = [&](int red, Pre pre, int unary) {
        AxhipRowsProgram p = base(dt);
        if (unary) push(p.pre, p.n_pre, unary, -1, false);
        add_pre(p, dt, pre, true);
        p.reduce = red;
        out.push_back(p);
    };
    // primary shapes (every register plan)
    softmax_like(AXHIP_ROWOP_SOFTMAX, PRE_NONE, true);
    norm(AXHIP_ROWOP_LAYERNORM, PRE_NONE, true, 0);
    norm(AXHIP_ROWOP_RMSNORM, PRE_NONE, true, 0);
    reduction(AXHIP_RED_SUM, PRE_NONE, 0);
    norm(AXHIP_ROWOP_LAYERNORM, PRE_NONE, true, AXHIP_OP_GELU);
    norm(AXHIP_ROWOP_RMSNORM, PRE_NONE, true, AXHIP_OP_GELU);
    *n_primary = static_cast<int>(out.size());
    // secondary shapes (the main plans only, and only for rows of whole, aligned vectors)
    softmax_like(AXHIP_ROWOP_LOGSOFTMAX, PRE_NONE, true);
    softmax_like(AXHIP_ROWOP_SOFTMAX, PRE_MULS, true);
    softmax_like(AXHIP_ROWOP_SOFTMAX, PRE_ADDF, true);
    norm(AXHIP_ROWOP_LAYERNORM, PRE_NONE, false, 0);
    norm(AXHIP_ROWOP_LAYERNORM, PRE_ADDF, true, 0);
    reduction(AXHIP_RED_MAX, PRE_NONE, 0);
    reduction(AXHIP_RED_SUM, PRE_ADDF, 0);
    reduction(AXHIP_RED_SUM, PRE_MULF, 0);
    reduction(AXHIP_RED_SUM, PRE_NONE, AXHIP_OP_SQUARE);
    reduction(AXHIP_RED_MAX, PRE_NONE, AXHIP_OP_ABS);
    if (dt == AXHIP_DTYPE_F32) // BASELINE configs[1]: softmax((relu(a) + 1) * b).sum(1), the 1 as an immediate or as a one-element operand
        for (bool imm : {true, false}) {
            AxhipRowsProgram q = base(dt);
            add_pre(q, dt, PRE_RELU_ADDS_MULF, imm);
            q.row_op = AXHIP_ROWOP_SOFTMAX;
            q.reduce = AXHIP_RED_SUM;
            out.push_back(q);
        }
    return out;
}

} // namespace

int main(int argc, char **argv) {
    if (argc < 3) {
        fprintf(stderr, "usage: %s <output directory> <number of files>\n", argv[0]);
        return 2;
    }
    const std::string dir = argv[1];
    const int n_files = atoi(argv[2]);
    if (n_files <= 0) return 2;
    // a wavefront per row up to 512 chunks (1, 2, 4, 8 chunks per lane, and 3 / 5 / 6 for the row lengths between the
    // powers of two: 1280, 1536, 2560, 3072 ... columns of 16-bit data), a 256-thread block per row beyond
    // (4 to 32 lanes per row: short aligned rows, several to a wavefront)
    // (the last five: primary shapes only)
    static const int plans[][2] = {{16, 1}, {32, 1}, {64, 1}, {64, 2}, {64, 4}, {64, 8}, {256, 4}, {256, 8}, {4, 1}, {8, 1}, {64, 3}, {64, 6}, {256, 3}};
    constexpr int n_main_plans = 8, n_plans = 13;
    std::vector<RowsProgSpec> specs;
    std::set<std::string> seen;
    // (fp32 is what the reference's GPU path computes in, bf16 what the benchmark configurations and Whisper run in; f16 shapes are compiled on first use)
    for (int dt : {AXHIP_DTYPE_F32, AXHIP_DTYPE_BF16}) {
        int n_primary = 0;
        const std::vector<AxhipRowsProgram> shapes = shapes_of(dt, &n_primary);
        for (size_t si = 0; si < shapes.size(); ++si) {
            const AxhipRowsProgram &p = shapes[si];
            for (int pi = 0; pi < (static_cast<int>(si) < n_primary ? n_plans : n_main_plans); ++pi) {
                const int *pl = plans[pi];
                for (bool ragged : {false, true}) {
                    if (ragged && static_cast<int>(si) >= n_primary) continue; // secondary shapes: whole-vector rows only
                    RowsProgPlan plan;
                    rows_prog_plan_for(p, pl[0], pl[1], ragged, &plan, /*the built-in ragged kernels are those for equally aligned streams*/ ragged && rows_prog_grid_pays(p, pl[0], pl[1]));
                    RowsProgSpec s;
                    if (!rows_prog_spec(p, plan, &s)) {
                        fprintf(stderr, "rows_aot_gen: a listed shape was refused by the generator\n");
                        return 1;
                    }
                    if (seen.insert(s.symbol).second) specs.push_back(s);
                }
            }
        }
    }
    std::vector<std::ofstream> files;
    for (int i = 0; i < n_files; ++i) {
        char name[64];
        snprintf(name, sizeof(name), "/rows_aot_%02d.hip", i);
        files.emplace_back(dir + name);
        files.back() << "// generated by rows_aot_gen: fused-row kernels built into the library\n"
                        "#include <hip/hip_runtime.h>\n#include \"rows_codegen.hpp\"\n";
    }
    for (size_t i = 0; i < specs.size(); ++i) {
        std::ofstream &f = files[i % n_files];
        const RowsProgSpec &s = specs[i];
        f << "\n// " << s.label << "\n" << rows_prog_source(s, "#include \"rows_prog.inc\"\n");
        f << "static const axhip::RowsProgRegistrar reg_" << s.symbol << "(R\"AXPKEY(" << s.config << s.chains << ")AXPKEY\", reinterpret_cast<const void *>(&"
          << s.symbol << "));\n";
    }
    printf("%zu kernels in %d files\n", specs.size(), n_files);
    return 0;
}
