// Fused row programs: elementwise chain -> row op (softmax / layer norm / RMS
// norm) -> elementwise chain -> optional row reduction, one launch, every input
// element read from HBM once, nothing intermediate written.
//
// Layout: a [rows, cols] row-major view.  A row is held in registers as fp32:
// each thread owns IT chunks of E consecutive elements (E*elem = 16 or 32 bytes,
// so every global access is a full-width vector), chunk c = it*GROUP + lane_in_group,
// which makes consecutive lanes touch consecutive 16/32-byte segments.
// Reductions are wave64 shuffles plus one LDS hop when a row spans several waves.
#include "rows_kernels.hpp"

#include <cstring>
#include <mutex>
#include <string>


// Partial sums of axhip_fused_full_reduce_noalloc: one float per stage-1 block or row (16640 at most, 65 KiB).  Every
// device the library runs on holds its own copy until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress; kernels and copies take the per-device address kept in g_scratch_ptr.
static __device__ __align__(256) float scratch[16640];

namespace axhip {

// Chain + reduction over every element: stage 1 leaves one partial per block (or, on the row kernels, per row) in
// the workspace, stage 2 (one block) folds the partials.
constexpr int FULL_RED_BLOCKS = 2048;      // blocks of the generic stage 1
constexpr int FULL_RED_ROWS = 16384;       // rows of a flat array handed to a row-reduction kernel
constexpr int FULL_RED_PARTIALS = FULL_RED_ROWS + 256; // capacity of the workspace, in floats (the rows plus the blocks of a remainder)
static_assert(sizeof(scratch) / sizeof(float) >= FULL_RED_PARTIALS, "the file-scope scratch array holds every partial of a full reduction");

template <int THREADS, int E>
__global__ __launch_bounds__(THREADS) void full_reduce_stage1(const AxhipRowsProgram P, float *partials) {
    __shared__ float lds[THREADS / WAVE];
    const int64_t cols = P.cols;
    const int64_t nchunk = P.rows * cols / E;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * THREADS;
    float acc = red_start(P.reduce);
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * THREADS + threadIdx.x; c < nchunk; c += stride) {
        const int64_t flat = c * E;
        const int64_t row = flat / cols;
        const int64_t col0[1] = {flat - row * cols};
        const bool ok[1] = {true};
        float v[1][E];
        if constexpr (E == 1) v[0][0] = load_any(P.input, P.input_dtype, flat);
        else load_vec<E>(P.input, P.input_dtype, flat, v[0]);
        for (int i = 0; i < P.n_pre; ++i) apply_op<1, E>(P.pre[i], P, v, row, col0, ok);
#pragma unroll
        for (int e = 0; e < E; ++e) acc = red_fold(P.reduce, acc, v[0][e]);
    }
    acc = group_reduce_of<THREADS, THREADS>(P.reduce, acc, lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = acc;
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void full_reduce_stage2(const float *partials, int n, int reduce, float inv_count,
                                                              void *out, int out_dtype) {
    __shared__ float lds[THREADS / WAVE];
    float acc = red_start(reduce);
#pragma unroll 4
    for (int i = threadIdx.x; i < n; i += THREADS) acc = red_fold(reduce, acc, partials[i]);
    acc = group_reduce_of<THREADS, THREADS>(reduce, acc, lds);
    if (reduce == AXHIP_RED_MEAN) acc *= inv_count;
    if (threadIdx.x == 0) store_any(out, out_dtype, 0, acc);
}

// ------------------------------------------------------------------ host side

namespace {

bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

int validate_chain(const AxhipChainOp *ops, int n, const AxhipRowsProgram &P, const char *which) {
    AXHIP_REQUIRE(n >= 0 && n <= AXHIP_MAX_CHAIN, AXHIP_ERR_INVALID_ARG, "fused rows: %s chain length %d out of range", which, n);
    for (int i = 0; i < n; ++i) {
        const int op = ops[i].op;
        const bool bin = is_binary_op(op);
        const bool un = is_unary_op(op);
        AXHIP_REQUIRE(bin || un, AXHIP_ERR_INVALID_ARG, "fused rows: %s[%d] has unknown op code %d", which, i, op);
        if (bin && ops[i].imm_kind != AXHIP_BK_IMM)
            AXHIP_REQUIRE(ops[i].operand >= 0 && ops[i].operand < P.n_operands, AXHIP_ERR_INVALID_ARG,
                          "fused rows: %s[%d] operand index %d out of range", which, i, ops[i].operand);
    }
    return AXHIP_OK;
}

// Picks the vector width E (elements per access): the widest for which every
// row start and every vector operand stays naturally aligned.
int pick_vector_width(const AxhipRowsProgram &P) {
    auto fits = [&](int e) {
        if (P.cols % e != 0) return false;
        auto ok = [&](const void *p, int dt) { return aligned_to(p, std::min<size_t>(16, e * dtype_size(dt))); };
        if (!ok(P.input, P.input_dtype)) return false;
        if (P.reduce == AXHIP_RED_NONE && !ok(P.output, P.output_dtype)) return false;
        for (int i = 0; i < P.n_operands; ++i)
            if ((P.operands[i].kind == AXHIP_BK_FULL || P.operands[i].kind == AXHIP_BK_ROWVEC) &&
                !ok(P.operands[i].ptr, P.operands[i].dtype))
                return false;
        return true;
    };
    // 8 elements per access only when every full-size stream is 16-bit: with an fp32 stream among them that stream's
    // 32 bytes per lane would go out as two accesses that each fill half of every 32-byte run (bf16 -> fp32 casts
    // ran at 42 % of the HBM peak that way)
    bool wide = P.input_dtype == AXHIP_DTYPE_F32 || (P.reduce == AXHIP_RED_NONE && P.output_dtype == AXHIP_DTYPE_F32);
    for (int i = 0; i < P.n_operands; ++i)
        if (P.operands[i].kind == AXHIP_BK_FULL && P.operands[i].dtype == AXHIP_DTYPE_F32) wide = true;
    if (!wide && fits(8)) return 8;
    if (fits(4)) return 4;
    return 1;
}

// Vector width for walking an elementwise program's arrays as one flat run (0: not possible): every full-size stream
// 16-byte aligned, rows of at least one chunk.
int flat_vector_width(const AxhipRowsProgram &P) {
    bool wide = P.input_dtype == AXHIP_DTYPE_F32 || P.output_dtype == AXHIP_DTYPE_F32;
    if (!aligned_to(P.input, 16) || !aligned_to(P.output, 16)) return 0;
    for (int i = 0; i < P.n_operands; ++i) {
        if (P.operands[i].kind != AXHIP_BK_FULL) continue;
        if (!aligned_to(P.operands[i].ptr, 16)) return 0;
        if (P.operands[i].dtype == AXHIP_DTYPE_F32) wide = true;
    }
    const int e = wide ? 4 : 8;
    return P.cols >= e ? e : 0;
}

int validate_program(const AxhipRowsProgram &P, const char *who) {
    AXHIP_REQUIRE(P.rows >= 0 && P.cols >= 0, AXHIP_ERR_INVALID_ARG, "%s: negative extent", who);
    AXHIP_REQUIRE(valid_dtype_or_u8(P.input_dtype) && valid_dtype_or_u8(P.output_dtype), AXHIP_ERR_INVALID_ARG, "%s: bad dtype", who);
    AXHIP_REQUIRE(P.n_operands >= 0 && P.n_operands <= AXHIP_MAX_OPERANDS, AXHIP_ERR_INVALID_ARG, "%s: bad operand count %d", who, P.n_operands);
    for (int i = 0; i < P.n_operands; ++i) {
        AXHIP_REQUIRE(P.operands[i].ptr != nullptr, AXHIP_ERR_INVALID_ARG, "%s: operand %d is NULL", who, i);
        AXHIP_REQUIRE(valid_dtype_or_u8(P.operands[i].dtype), AXHIP_ERR_INVALID_ARG, "%s: operand %d has bad dtype", who, i);
        AXHIP_REQUIRE(P.operands[i].kind >= AXHIP_BK_FULL && P.operands[i].kind <= AXHIP_BK_SCALAR, AXHIP_ERR_INVALID_ARG, "%s: operand %d has bad kind", who, i);
    }
    int rc = validate_chain(P.pre, P.n_pre, P, "pre");
    if (rc) return rc;
    rc = validate_chain(P.post, P.n_post, P, "post");
    if (rc) return rc;
    AXHIP_REQUIRE(P.row_op >= AXHIP_ROWOP_NONE && P.row_op <= AXHIP_ROWOP_RMSNORM, AXHIP_ERR_INVALID_ARG, "%s: bad row_op %d", who, P.row_op);
    AXHIP_REQUIRE(P.reduce >= AXHIP_RED_NONE && P.reduce <= AXHIP_RED_PROD, AXHIP_ERR_INVALID_ARG, "%s: bad reduce %d", who, P.reduce);
    for (int idx : {P.norm_weight, P.norm_bias})
        if (idx >= 0) {
            AXHIP_REQUIRE(idx < P.n_operands && P.operands[idx].kind == AXHIP_BK_ROWVEC, AXHIP_ERR_INVALID_ARG, "%s: norm weight/bias must be a ROWVEC operand", who);
        }
    if (P.rows > 0 && P.cols > 0) AXHIP_REQUIRE(P.input && P.output, AXHIP_ERR_INVALID_ARG, "%s: NULL input/output", who);
    return AXHIP_OK;
}


RowsPlan plan_rows(const AxhipRowsProgram &P) {
    RowsPlan pl{};
    if (P.rows == 0 || P.cols == 0) {
        pl.kind = RowsPlan::EMPTY;
        snprintf(pl.name, sizeof(pl.name), "empty");
        return pl;
    }
    pl.e = pick_vector_width(P);
    if (P.row_op == AXHIP_ROWOP_NONE && P.reduce == AXHIP_RED_NONE) {
        pl.kind = RowsPlan::ELEMENTWISE;
        pl.threads = 256;
        // a row length no vector divides, aligned arrays: one flat run of chunks instead of element by element
        const int flat_e = flat_vector_width(P);
        if (pl.e == 1 && flat_e > 1) {
            pl.kind = RowsPlan::ELEMENTWISE_FLAT;
            pl.e = flat_e;
            snprintf(pl.name, sizeof(pl.name), "elementwise_flat_e%d", pl.e);
            return pl;
        }
        snprintf(pl.name, sizeof(pl.name), "elementwise_e%d", pl.e);
        return pl;
    }
    // rows of odd length or alignment: keep the full vector width (the hardware takes 16-byte accesses at element
    // alignment) and treat the row's last, partial chunk element by element, as long as the row fits a resident plan
    const int natural = P.input_dtype != AXHIP_DTYPE_F32 ? 8 : 4;
    if (pl.e == 1 && P.cols >= natural && (P.cols + natural - 1) / natural <= 1024 * 4) { // (a narrower aligned vector, when one fits, measured faster)
        pl.e = natural;
        pl.ragged = true;
    }
    const int64_t chunks = (P.cols + pl.e - 1) / pl.e;
    pl.threads = 256;
    if (chunks <= 64 * 4) { // a row fits one wave with <= 4 chunks per lane
        pl.group = 64;
        pl.it = chunks <= 64 ? 1 : chunks <= 128 ? 2 : 4;
        pl.kind = RowsPlan::RESIDENT;
    } else if (chunks <= 256 * 8) {
        pl.group = 256;
        pl.it = chunks <= 256 ? 1 : chunks <= 512 ? 2 : chunks <= 1024 ? 4 : 8;
        pl.kind = RowsPlan::RESIDENT;
    } else if (chunks <= 1024 * 4) { // up to 64 KiB of 16-bit or 64 KiB of fp32 columns: still one read, in the registers of 1024 threads
        pl.group = 1024;
        pl.threads = 1024;
        pl.it = 4;
        pl.kind = RowsPlan::RESIDENT;
    } else {
        pl.kind = RowsPlan::STREAMED;
        pl.threads = 1024;
        pl.group = 1024;
        pl.it = 0;
    }
    if (pl.kind == RowsPlan::RESIDENT) snprintf(pl.name, sizeof(pl.name), "rows_resident_g%d_it%d_e%d%s", pl.group, pl.it, pl.e, pl.ragged ? "_ragged" : "");
    else snprintf(pl.name, sizeof(pl.name), "rows_streamed_e%d", pl.e);
    return pl;
}



int check_full_reduce_program(const AxhipRowsProgram *program, const char *who) {
    AXHIP_REQUIRE(program != nullptr, AXHIP_ERR_INVALID_ARG, "%s: program is NULL", who);
    const AxhipRowsProgram &P = *program;
    int rc = validate_program(P, who);
    if (rc) return rc;
    AXHIP_REQUIRE(P.row_op == AXHIP_ROWOP_NONE && P.n_post == 0, AXHIP_ERR_INVALID_ARG, "%s: row_op/post must be empty", who);
    AXHIP_REQUIRE(P.reduce != AXHIP_RED_NONE, AXHIP_ERR_INVALID_ARG, "%s: reduce is NONE", who);
    AXHIP_REQUIRE(P.rows > 0 && P.cols > 0, AXHIP_ERR_INVALID_ARG, "%s: empty input", who);
    return AXHIP_OK;
}

// Large aligned arrays under chains without per-column or per-row operands are one flat array: seen as rows of 512 or
// 2048 16-byte chunks it goes through the built-in row-reduction kernel of that plan, one partial per row (81-87 % of
// the HBM peak where the generic stage 1 -- one chunk in flight per thread, a division per chunk -- reaches 30-60 %).
// What is left behind the last whole row (less than a row) takes the generic stage 1, one partial per block.
// Only kernels that are built into the library: nothing is compiled here, so the no-allocation entry point can share
// the route.  Returns the number of partials written, 0 when the route does not apply.
int full_reduce_on_row_kernels(const AxhipRowsProgram &P, float *partials, hipStream_t s, int *rc) {
    *rc = AXHIP_OK;
    const int64_t count = P.rows * P.cols;
    if (!aligned_to(P.input, 16)) return 0;
    bool wide = P.input_dtype == AXHIP_DTYPE_F32;
    for (int i = 0; i < P.n_pre; ++i) {
        if (!is_binary_op(P.pre[i].op) || P.pre[i].imm_kind == AXHIP_BK_IMM) continue;
        const AxhipOperand &o = P.operands[P.pre[i].operand];
        if (o.kind == AXHIP_BK_ROWVEC || o.kind == AXHIP_BK_COLVEC) return 0;
        if (o.kind == AXHIP_BK_FULL) {
            if (!aligned_to(o.ptr, 16)) return 0;
            if (o.dtype == AXHIP_DTYPE_F32) wide = true;
        }
    }
    const int e = wide ? 4 : 8;
    const int64_t nchunk = count / e;
    if (nchunk < 512 * 256) return 0; // (2 MiB: below that the generic kernel's launch is what counts)
    const int64_t row_chunks = nchunk >= int64_t(2048) * 512 ? 2048 : 512;
    const int64_t rows = nchunk / row_chunks;
    if (rows > FULL_RED_ROWS) return 0;
    AxhipRowsProgram Q = P;
    Q.rows = rows;
    Q.cols = row_chunks * e;
    Q.reduce = P.reduce == AXHIP_RED_MEAN ? AXHIP_RED_SUM : P.reduce;
    Q.output = partials;
    Q.output_dtype = AXHIP_DTYPE_F32;
    if (!rows_prog_dispatch(Q, s, true, nullptr, 0, rc, /*builtin_only=*/true)) return 0;
    if (*rc) return 0;
    int written = static_cast<int>(rows);
    const int64_t done = rows * Q.cols, rest = count - done;
    if (rest > 0) {
        AxhipRowsProgram R = P;
        R.rows = 1;
        R.cols = rest;
        R.input = static_cast<const char *>(P.input) + done * dtype_size(P.input_dtype);
        for (int i = 0; i < R.n_operands; ++i)
            if (R.operands[i].kind == AXHIP_BK_FULL) R.operands[i].ptr = static_cast<const char *>(P.operands[i].ptr) + done * dtype_size(P.operands[i].dtype);
        const int blocks = static_cast<int>((rest + 255) / 256); // rest < 2048 * 8 elements: at most 64 blocks
        hipLaunchKernelGGL((full_reduce_stage1<256, 1>), dim3(blocks), dim3(256), 0, s, R, partials + written);
        written += blocks;
    }
    return written;
}

// stage 1 leaves its partials in `partials` (FULL_RED_PARTIALS floats), stage 2 reads exactly those
int launch_full_reduce(const AxhipRowsProgram &P, float *partials, hipStream_t s) {
    int rc = AXHIP_OK;
    const int on_rows = full_reduce_on_row_kernels(P, partials, s, &rc);
    if (rc) return rc;
    if (on_rows > 0) {
        AXHIP_CHECK_HIP(hipGetLastError());
        hipLaunchKernelGGL((full_reduce_stage2<1024>), dim3(1), dim3(1024), 0, s, partials, on_rows, P.reduce,
                           1.0f / static_cast<float>(P.rows * P.cols), P.output, P.output_dtype);
        AXHIP_CHECK_HIP(hipGetLastError());
        return AXHIP_OK;
    }
    AxhipRowsProgram Q = P;
    Q.reduce = AXHIP_RED_SUM; // only used by pick_vector_width to skip the output alignment test
    const int e = pick_vector_width(Q);
    const int64_t n = P.rows * P.cols;
    const int64_t nchunk = n / e;
    const int blocks = static_cast<int>(std::min<int64_t>((nchunk + 255) / 256, FULL_RED_BLOCKS));
    if (e == 8) hipLaunchKernelGGL((full_reduce_stage1<256, 8>), dim3(blocks), dim3(256), 0, s, P, partials);
    else if (e == 4) hipLaunchKernelGGL((full_reduce_stage1<256, 4>), dim3(blocks), dim3(256), 0, s, P, partials);
    else hipLaunchKernelGGL((full_reduce_stage1<256, 1>), dim3(blocks), dim3(256), 0, s, P, partials);
    AXHIP_CHECK_HIP(hipGetLastError());
    hipLaunchKernelGGL((full_reduce_stage2<256>), dim3(1), dim3(256), 0, s, partials, blocks, P.reduce,
                       1.0f / static_cast<float>(n), P.output, P.output_dtype);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

// Largest input axhip_fused_full_reduce_noalloc accepts (2^40 elements): the partials fit the fixed array whatever
// the size, the bound keeps rows * cols and the blocks' strided loops far inside 64-bit range.
constexpr int64_t FULL_REDUCE_NOALLOC_MAX_ELEMENTS = int64_t(1) << 40;

// Device address of `scratch` on the calling thread's current device, resolved once per device.
constexpr int MAX_SCRATCH_DEVICES = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[MAX_SCRATCH_DEVICES] = {};

int scratch_of_current_device(float **out) {
    int dev = -1;
    AXHIP_CHECK_HIP(hipGetDevice(&dev));
    AXHIP_REQUIRE(dev >= 0 && dev < MAX_SCRATCH_DEVICES, AXHIP_ERR_UNSUPPORTED, "device ordinal %d beyond the %d this library keeps scratch for", dev,
                  MAX_SCRATCH_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        AXHIP_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        AXHIP_REQUIRE(p != nullptr, AXHIP_ERR_WORKSPACE, "hipGetSymbolAddress returned no address for the reduction scratch");
        g_scratch_ptr[dev] = static_cast<float *>(p);
    }
    *out = g_scratch_ptr[dev];
    return AXHIP_OK;
}

} // namespace

// Called by axhip_init with the device current, so that the first no-allocation call on it finds the address resolved.
int rows_setup_device() {
    float *unused = nullptr;
    return scratch_of_current_device(&unused);
}

// A large elementwise chain (no row operation, no reduction) whose operands are full-size arrays, one-element arrays
// or immediates does not care where its rows end: seen as rows of 512 chunks (a wavefront per row, eight chunks per
// lane) any such array takes the same compiled kernel, whatever its own shape -- a vector of 2^26 elements included.
// False when the chain reads an operand by column or by row, when the size is no multiple of such a row, or when an
// array does not start on a 16-byte boundary: the program then runs with the shape it came with.
bool flat_chain_as_rows(const AxhipRowsProgram &P, AxhipRowsProgram *out) {
    if (P.row_op != AXHIP_ROWOP_NONE || P.reduce != AXHIP_RED_NONE) return false;
    auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (!al16(P.input) || !al16(P.output)) return false;
    for (int stage = 0; stage < 2; ++stage) {
        const AxhipChainOp *ops = stage ? P.post : P.pre;
        const int n = stage ? P.n_post : P.n_pre;
        for (int i = 0; i < n; ++i) {
            if (!is_binary_op(ops[i].op) || ops[i].imm_kind == AXHIP_BK_IMM) continue;
            if (ops[i].operand < 0 || ops[i].operand >= P.n_operands) return false;
            const AxhipOperand &o = P.operands[ops[i].operand];
            if (o.kind == AXHIP_BK_ROWVEC || o.kind == AXHIP_BK_COLVEC) return false;
            if (o.kind == AXHIP_BK_FULL && !al16(o.ptr)) return false;
        }
    }
    const int64_t row = 512 * rows_prog_chunk_elems(P), total = P.rows * P.cols;
    if (total % row != 0 || P.cols == row) return false;
    *out = P;
    out->rows = total / row;
    out->cols = row;
    return true;
}

} // namespace axhip

using namespace axhip;

extern "C" {

const char *axhip_fused_rows_kernel_name(const AxhipRowsProgram *P) {
    static thread_local char name[192];
    if (!P) return "invalid";
    AxhipRowsProgram flat;
    if (validate_program(*P, "axhip_fused_rows_kernel_name") == AXHIP_OK &&
        rows_prog_dispatch(flat_chain_as_rows(*P, &flat) ? flat : *P, nullptr, false, name, sizeof(name), nullptr))
        return name;
    RowsPlan pl = plan_rows(*P);
    snprintf(name, sizeof(name), "%s", pl.name);
    return name;
}

int axhip_fused_rows(const AxhipRowsProgram *program, void *stream) {
    AXHIP_REQUIRE(program != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_fused_rows: program is NULL");
    const AxhipRowsProgram &P = *program;
    int rc = validate_program(P, "axhip_fused_rows");
    if (rc) return rc;
    AXHIP_REQUIRE(P.rows < (int64_t(1) << 31), AXHIP_ERR_UNSUPPORTED, "axhip_fused_rows: more than 2^31 rows");
    rc = ensure_init();
    if (rc) return rc;
    RowsPlan pl = plan_rows(P);
    if (pl.kind == RowsPlan::EMPTY) return AXHIP_OK;
    hipStream_t s = resolve_stream(stream);
    // a kernel compiled for this program's shape (built in, or compiled now if this is its first launch) ...
    int launch_rc = AXHIP_OK;
    AxhipRowsProgram flat;
    if (rows_prog_dispatch(flat_chain_as_rows(P, &flat) ? flat : P, s, true, nullptr, 0, &launch_rc)) {
        if (launch_rc) return launch_rc;
        AXHIP_CHECK_HIP(hipGetLastError());
        return AXHIP_OK;
    }
    // ... or the interpreter
    rc = pl.e == 8 ? launch_plan_e<8>(P, pl, s) : pl.e == 4 ? launch_plan_e<4>(P, pl, s) : launch_plan_e<1>(P, pl, s);
    if (rc) return rc;
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_fused_rows_prepare(const AxhipRowsProgram *program) {
    AXHIP_REQUIRE(program != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_fused_rows_prepare: program is NULL");
    int rc = validate_program(*program, "axhip_fused_rows_prepare");
    if (rc) return rc;
    char name[192];
    AxhipRowsProgram flat;
    const AxhipRowsProgram &as_run = flat_chain_as_rows(*program, &flat) ? flat : *program;
    if (!rows_prog_dispatch(as_run, nullptr, false, name, sizeof(name), nullptr)) return AXHIP_OK; // the interpreter's: nothing to prepare
    if (strncmp(name, "rows_static_", 12) == 0) return AXHIP_OK;                                // built into the library
    std::string label, error;
    if (!rows_prog_compile_only(as_run, &label, &error)) {
        set_last_error("axhip_fused_rows_prepare: %s: %.400s", label.c_str(), error.c_str());
        return AXHIP_ERR_UNSUPPORTED;
    }
    return AXHIP_OK;
}

void axhip_fused_rows_jit_counters(int *from_disk, int *compiled) { rows_prog_jit_counters(from_disk, compiled); }

size_t axhip_full_reduce_workspace_bytes(void) { return FULL_RED_PARTIALS * sizeof(float); }

int axhip_fused_full_reduce(const AxhipRowsProgram *program, void *workspace, size_t workspace_bytes, void *stream) {
    int rc = check_full_reduce_program(program, "axhip_fused_full_reduce");
    if (rc) return rc;
    AXHIP_REQUIRE(workspace && workspace_bytes >= axhip_full_reduce_workspace_bytes() && aligned_to(workspace, 4), AXHIP_ERR_WORKSPACE,
                  "axhip_fused_full_reduce: workspace too small (%zu < %zu)", workspace_bytes, axhip_full_reduce_workspace_bytes());
    rc = ensure_init();
    if (rc) return rc;
    return launch_full_reduce(*program, static_cast<float *>(workspace), resolve_stream(stream));
}

int64_t axhip_full_reduce_noalloc_max_elements(void) { return FULL_REDUCE_NOALLOC_MAX_ELEMENTS; }

int axhip_fused_full_reduce_noalloc(const AxhipRowsProgram *program, void *stream) {
    int rc = check_full_reduce_program(program, "axhip_fused_full_reduce_noalloc");
    if (rc) return rc;
    // rows and cols are positive here; the division keeps the product from overflowing
    AXHIP_REQUIRE(program->rows <= FULL_REDUCE_NOALLOC_MAX_ELEMENTS / program->cols, AXHIP_ERR_UNSUPPORTED,
                  "axhip_fused_full_reduce_noalloc: %lld x %lld elements exceed the maximum of %lld", static_cast<long long>(program->rows),
                  static_cast<long long>(program->cols), static_cast<long long>(FULL_REDUCE_NOALLOC_MAX_ELEMENTS));
    rc = ensure_init();
    if (rc) return rc;
    float *partials = nullptr;
    rc = scratch_of_current_device(&partials);
    if (rc) return rc;
    // Nothing in the array has to start at zero: stage 1 writes every partial stage 2 reads.
    return launch_full_reduce(*program, partials, resolve_stream(stream));
}

} // extern "C"
