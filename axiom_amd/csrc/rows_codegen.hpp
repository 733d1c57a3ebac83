// Compiled fused-row programs: from an AxhipRowsProgram to the source text of its kernel.
//
// Every row program (pre chain -> row op -> post chain -> optional row reduction) whose rows fit a register plan has
// one kernel of its own: rows_prog.inc compiled with a small configuration text in front (element types, plan, the
// two chains as straight-line code).  The same generator serves two users:
//   - the build, which writes the kernels of the common program shapes to source files that hipcc compiles into the
//     library (the counterpart of Axiom's known fused patterns, src/graph/fused_patterns.cpp:12-71), and
//   - the library at run time, which compiles any other shape through hipRTC the first time it is seen (the
//     counterpart of the reference's any-DAG-to-one-program graph compiler,
//     src/backends/metal/mpsgraph_graph_compiler.mm:706-944).
// Plain host C++: no HIP types, so that the build's generator tool compiles with g++.
#pragma once

#include <cstdint>
#include <string>

#include "axhip.h"

namespace axhip {

// kernel arguments; rows_prog.inc declares the same layout as axp::Args
struct RowsProgArgs {
    const void *x;
    void *y;
    int64_t rows, cols;
    const void *ptr[8];
    float imm[32];
    float eps;
    int32_t stream_out;
    float red_scale;  // 1, or 1/cols for a mean
    int32_t red_dt;   // element type of a reduced [rows] output
};

struct RowsProgPlan {
    int group = 0, it = 0; // threads per row, 16-byte input chunks per thread
    bool ragged = false;   // rows are not whole aligned vectors
    bool grid = false;     // ragged rows whose full-size streams share their address modulo 16: chunks on memory's 16-byte grid
    bool loop = false;     // rows beyond the registers of a block: every pass walks the row in steps of `it` chunks per thread
    int tail_from = 0;     // grid rows: a thread's chunks before this one are known to lie inside the row (0: nothing known)
    bool pipe = false;     // the next row is requested before the current one is computed
    bool rerun = false;    // the row stays in registers as raw words; every pass unpacks it and applies the pre chain again
    int min_waves = 4;     // waves per SIMD the kernel's register allocation aims for
    bool lane = false;     // short rows of odd length: a wavefront stages 64 / lane_l consecutive rows in LDS and lane_l lanes walk each
    int lane_l = 1;        // (lane) lanes per row; `it` chunks per lane, held as fp32 after the first pass
    int lane_bytes = 0;    // (lane) LDS bytes per wavefront and full-size stream
    int slots() const { return group * it; }
};

// everything that is compiled into one kernel
struct RowsProgSpec {
    std::string config;     // configuration text; doubles as the cache key
    std::string chains;     // definitions of the two chain functions (appended after the body)
    std::string label;      // human-readable kernel label, e.g. layernorm_gelu_bf16_g64_it8
    std::string symbol;     // extern "C" name of the kernel: axp_<hash of config and chains>
    int threads = 256;
    int rows_per_block = 4;
    bool lane = false;      // the row-per-lane body (its text is compiled only for these kernels)
    int64_t inflight_bytes = 0; // bytes of input a block keeps requested at a time (0: not counted)
    bool pipelined = false;     // the kernel requests a row while it computes the one before
    int post_ops = 0;           // operations behind the row operation (the output pass carries them)
    int n_slots = 0;
    int slot_operand[8] = {}; // pointer slot -> index into AxhipRowsProgram::operands
    int n_imm = 0;
    struct ImmRef { bool post; int index; } imm_ref[32] = {}; // immediate slot -> chain position
};

// Picks the register plan; false when the program does not qualify (no row op and no reduction, rows too long or
// too short, a vector operand whose element size keeps a ragged row from its 16-byte chunks): the interpreter takes it.
// tight = false: among the plan shapes the build compiles (64 or 256 threads per row, a few chunk counts per thread);
// tight = true: the plan with the fewest idle chunk slots for this row length (64, 256 or 512 threads per row, any chunk count up to 8).
// the row-per-lane plan is for arrays of at least this many rows (fewer rows want more than a wavefront per 64 of them)
constexpr int64_t kRowsProgLaneMinRows = 32768;
// an elementwise chain (no row operation, no reduction) takes a compiled kernel from this size on: 1024 rows, 8 MiB of input
bool rows_prog_flat_large(const AxhipRowsProgram &P);
int rows_prog_chunk_elems(const AxhipRowsProgram &P); // elements per chunk: 4 when a full-size stream is fp32, else 8
bool rows_prog_plan(const AxhipRowsProgram &P, bool tight, RowsProgPlan *plan);
// The plan with its shape given (the build's generator enumerates the shapes itself).
// whether ragged rows of this program are better served with chunks on memory's 16-byte grid (given equally aligned streams)
bool rows_prog_grid_pays(const AxhipRowsProgram &P, int group, int it);
void rows_prog_plan_for(const AxhipRowsProgram &P, int group, int it, bool ragged, RowsProgPlan *plan, bool grid = false);

// Builds the kernel's configuration for a program under a plan; false when the program names an operand kind or
// op code the generator does not know.
bool rows_prog_spec(const AxhipRowsProgram &P, const RowsProgPlan &plan, RowsProgSpec *spec);

// Fills the kernel arguments of one launch.
void rows_prog_bind(const AxhipRowsProgram &P, const RowsProgSpec &spec, RowsProgArgs *args);

// Full source text of the kernel: configuration, `body` (the text of rows_prog.inc), chain functions.
std::string rows_prog_source(const RowsProgSpec &spec, const std::string &body);

// ---- kernels compiled into the library register themselves here (static initialisers of the generated files)
struct RowsProgRegistrar {
    RowsProgRegistrar(const char *key, const void *kernel);
};
const void *rows_prog_find_builtin(const std::string &key);

} // namespace axhip
