// Fused row programs: elementwise chain -> row op (softmax / layer norm / RMS
// norm) -> elementwise chain -> optional row reduction, one launch, every input
// element read from HBM once, nothing intermediate written.
//
// Layout: a [rows, cols] row-major view.  A row is held in registers as fp32:
// each thread owns IT chunks of E consecutive elements (E*elem = 16 or 32 bytes,
// so every global access is a full-width vector), chunk c = it*GROUP + lane_in_group,
// which makes consecutive lanes touch consecutive 16/32-byte segments.
// Reductions are wave64 shuffles plus one LDS hop when a row spans several waves.
#include "common.hpp"
#include "rows_ops.hpp"
#include "rows_prog.hpp"

#include <algorithm>
#include <cstring>
#include <mutex>
#include <string>

// Partial sums of axhip_fused_full_reduce_noalloc: one float per stage-1 block or row (16640 at most, 65 KiB).  Every
// device the library runs on holds its own copy until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress; kernels and copies take the per-device address kept in g_scratch_ptr.
static __device__ __align__(256) float scratch[16640];

namespace axhip {


// Loads the [IT][E] tile of a FULL or ROWVEC operand.  RAGGED (rows whose length is not a multiple of E, or whose
// start is not vector-aligned): nv[it] counts the chunk's valid elements; whole chunks use unaligned vector loads,
// the row's last, partial chunk is read element by element.
template <int IT, int E, bool RAGGED = false>
__device__ __forceinline__ void load_operand_tile(const AxhipOperand &o, const AxhipRowsProgram &P, int64_t row,
                                                  const int64_t (&col0)[IT], const bool (&ok)[IT], float (&w)[IT][E], const int *nv = nullptr) {
    const int64_t base = o.kind == AXHIP_BK_FULL ? row * P.cols : 0;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        if constexpr (RAGGED) {
            if (nv[it] == E) {
                load_vec<E, true>(o.ptr, o.dtype, base + col0[it], w[it]);
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) w[it][e] = e < nv[it] ? load_any(o.ptr, o.dtype, base + col0[it] + e) : 1.0f;
            }
        } else if (ok[it]) {
            if constexpr (E == 1) w[it][0] = load_any(o.ptr, o.dtype, base + col0[it]);
            else load_vec<E>(o.ptr, o.dtype, base + col0[it], w[it]);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) w[it][e] = 1.0f;
        }
    }
}

template <int IT, int E, bool RAGGED = false, bool GROUPS = true>
__device__ __forceinline__ void apply_op(const AxhipChainOp &c, const AxhipRowsProgram &P, float (&v)[IT][E],
                                         int64_t row, const int64_t (&col0)[IT], const bool (&ok)[IT], const int *nv = nullptr) {
    if (!is_binary_op(c.op)) {
        // results that are rounded to a 16-bit type do not need erff / expf / IEEE division: the polynomial
        // GELU (|error| <= 5e-5) and fast-exponential forms are far below the output resolution and keep
        // these chains on the memory roofline
        if (P.output_dtype != AXHIP_DTYPE_F32) {
            switch (c.op) {
            case AXHIP_OP_GELU: for_each_value<IT, E>(v, [](float a, int, int) { return gelu_fast(a); }); return;
            case AXHIP_OP_SILU: for_each_value<IT, E>(v, [](float a, int, int) { return a * __builtin_amdgcn_rcpf(1.0f + __expf(-a)); }); return;
            case AXHIP_OP_SIGMOID: for_each_value<IT, E>(v, [](float a, int, int) { return __builtin_amdgcn_rcpf(1.0f + __expf(-a)); }); return;
            case AXHIP_OP_TANH: for_each_value<IT, E>(v, [](float a, int, int) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * a)); }); return;
            default: break;
            }
        }
        apply_unary_tile<IT, E, GROUPS>(c.op, v);
        return;
    }
    if (c.imm_kind == AXHIP_BK_IMM) {
        const float s = c.imm;
        apply_binary_tile<IT, E, GROUPS>(c.op, v, [&](int, int) { return s; });
        return;
    }
    const AxhipOperand &o = P.operands[c.operand];
    if (o.kind == AXHIP_BK_SCALAR || o.kind == AXHIP_BK_COLVEC) {
        const float s = load_any(o.ptr, o.dtype, o.kind == AXHIP_BK_SCALAR ? 0 : row);
        apply_binary_tile<IT, E, GROUPS>(c.op, v, [&](int, int) { return s; });
        return;
    }
    float w[IT][E];
    load_operand_tile<IT, E, RAGGED>(o, P, row, col0, ok, w, nv);
    apply_binary_tile<IT, E, GROUPS>(c.op, v, [&](int it, int e) { return w[it][e]; });
}

// norm weight / bias: v = v * w  or  v = v + b with a ROWVEC operand
template <int IT, int E, bool MUL, bool RAGGED = false>
__device__ __forceinline__ void apply_affine(int operand, const AxhipRowsProgram &P, float (&v)[IT][E], int64_t row,
                                             const int64_t (&col0)[IT], const bool (&ok)[IT], const int *nv = nullptr) {
    float w[IT][E];
    load_operand_tile<IT, E, RAGGED>(P.operands[operand], P, row, col0, ok, w, nv);
#pragma unroll
    for (int it = 0; it < IT; ++it)
#pragma unroll
        for (int e = 0; e < E; ++e) v[it][e] = MUL ? v[it][e] * w[it][e] : v[it][e] + w[it][e];
}

// Reduce across the GROUP threads that share a row.  GROUP == 64: shuffles
// only.  GROUP == blockDim: shuffles, then one LDS exchange between waves.
template <int GROUP, int THREADS, int KIND /*0 sum, 1 max, 2 min, 3 product*/>
__device__ __forceinline__ float group_reduce(float x, float *lds) {
    x = KIND == 0 ? wave_sum(x) : KIND == 1 ? wave_max(x) : KIND == 2 ? wave_min(x) : wave_prod(x);
    if constexpr (GROUP > WAVE) {
        constexpr int NW = THREADS / WAVE;
        const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
        __syncthreads(); // lds may still be read by a previous reduction
        if (lane == 0) lds[wave] = x;
        __syncthreads();
        float y = lds[lane % NW];
#pragma unroll
        for (int o = NW / 2; o > 0; o >>= 1) {
            float z = __shfl_xor(y, o, WAVE);
            y = KIND == 0 ? y + z : KIND == 1 ? fmaxf(y, z) : KIND == 2 ? fminf(y, z) : y * z;
        }
        x = y;
    }
    return x;
}

// the reduction kinds as run-time values (AXHIP_RED_*; MEAN folds like SUM and is scaled by the caller)
__device__ __forceinline__ float red_start(int reduce) {
    return reduce == AXHIP_RED_MAX ? NEG_INF : reduce == AXHIP_RED_MIN ? POS_INF : reduce == AXHIP_RED_PROD ? 1.0f : 0.0f;
}
__device__ __forceinline__ float red_fold(int reduce, float acc, float x) {
    return reduce == AXHIP_RED_MAX ? fmaxf(acc, x) : reduce == AXHIP_RED_MIN ? fminf(acc, x) : reduce == AXHIP_RED_PROD ? acc * x : acc + x;
}
template <int GROUP, int THREADS>
__device__ __forceinline__ float group_reduce_of(int reduce, float acc, float *lds) {
    if (reduce == AXHIP_RED_MAX) return group_reduce<GROUP, THREADS, 1>(acc, lds);
    if (reduce == AXHIP_RED_MIN) return group_reduce<GROUP, THREADS, 2>(acc, lds);
    if (reduce == AXHIP_RED_PROD) return group_reduce<GROUP, THREADS, 3>(acc, lds);
    return group_reduce<GROUP, THREADS, 0>(acc, lds);
}

// One row per GROUP threads, the whole row resident in registers.
template <int THREADS, int GROUP, int IT, int E, bool RAGGED>
__global__ __launch_bounds__(THREADS) void rows_resident_kernel(const AxhipRowsProgram P) {
    __shared__ float lds[THREADS / WAVE];
    constexpr int ROWS_PER_BLOCK = THREADS / GROUP;
    const int lane_in_group = threadIdx.x % GROUP;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / GROUP;
    const bool row_ok = row < P.rows;
    const int64_t cols = P.cols;
    const int64_t r = row_ok ? row : 0; // idle groups mirror row 0 so barriers stay uniform; they never store

    float v[IT][E];
    int64_t col0[IT];
    bool ok[IT];
    int nv[IT]; // valid elements of the chunk: E, 0 past the end of the row, in between only for a RAGGED row's last chunk
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        col0[it] = (static_cast<int64_t>(it) * GROUP + lane_in_group) * E;
        ok[it] = col0[it] < cols;
        const int64_t left = cols - col0[it];
        nv[it] = left >= E ? E : left > 0 ? static_cast<int>(left) : 0;
        // idle lanes re-read the row's first chunk, so that no load sits behind a branch and all of them are in
        // flight together; what they read is replaced by zeros below
        const int64_t at = r * cols + (ok[it] ? col0[it] : 0);
        if constexpr (E == 1) {
            v[it][0] = load_any(P.input, P.input_dtype, at);
        } else if constexpr (RAGGED) {
            if (nv[it] == E || nv[it] == 0) {
                load_vec<E, true>(P.input, P.input_dtype, at, v[it]); // cols >= E: the first chunk is whole
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) v[it][e] = e < nv[it] ? load_any(P.input, P.input_dtype, at + e) : 0.0f;
            }
        } else {
            load_vec<E>(P.input, P.input_dtype, at, v[it]);
        }
    }
#pragma unroll
    for (int it = 0; it < IT; ++it)
        if (!ok[it]) {
#pragma unroll
            for (int e = 0; e < E; ++e) v[it][e] = 0.0f;
        }
    // is element e of chunk it part of the row
    auto valid = [&](int it, int e) { return RAGGED ? e < nv[it] : ok[it]; };

    const float inv_n = 1.0f / static_cast<float>(cols);
    // stage 0: pre chain then the row op; stage 1: post chain.  One loop so the
    // chain interpreter is instantiated once per kernel.
#pragma nounroll
    for (int stage = 0; stage < 2; ++stage) {
    const int n_ops = stage == 0 ? P.n_pre : P.n_post;
    for (int i = 0; i < n_ops; ++i) apply_op<IT, E, RAGGED, (THREADS < 1024)>(stage == 0 ? P.pre[i] : P.post[i], P, v, r, col0, ok, nv);
    if (stage == 1) break;
    if (P.row_op == AXHIP_ROWOP_SOFTMAX || P.row_op == AXHIP_ROWOP_LOGSOFTMAX) {
        float m = NEG_INF;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) m = fmaxf(m, v[it][e]);
        m = group_reduce<GROUP, THREADS, 1>(m, lds);
        const float mm = m == NEG_INF ? 0.0f : m;
        float s = 0.0f;
        if (P.row_op == AXHIP_ROWOP_SOFTMAX) {
#pragma unroll
            for (int it = 0; it < IT; ++it)
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    v[it][e] = valid(it, e) ? __expf(v[it][e] - mm) : 0.0f;
                    s += v[it][e];
                }
            s = group_reduce<GROUP, THREADS, 0>(s, lds);
            const float inv = 1.0f / s;
#pragma unroll
            for (int it = 0; it < IT; ++it)
#pragma unroll
                for (int e = 0; e < E; ++e) v[it][e] *= inv;
        } else {
#pragma unroll
            for (int it = 0; it < IT; ++it)
#pragma unroll
                for (int e = 0; e < E; ++e) s += valid(it, e) ? __expf(v[it][e] - mm) : 0.0f;
            s = group_reduce<GROUP, THREADS, 0>(s, lds);
            const float ls = __logf(s) + mm;
#pragma unroll
            for (int it = 0; it < IT; ++it)
#pragma unroll
                for (int e = 0; e < E; ++e) v[it][e] -= ls;
        }
    } else if (P.row_op == AXHIP_ROWOP_LAYERNORM || P.row_op == AXHIP_ROWOP_RMSNORM) {
        float mean = 0.0f;
        if (P.row_op == AXHIP_ROWOP_LAYERNORM) {
            float s = 0.0f;
#pragma unroll
            for (int it = 0; it < IT; ++it)
#pragma unroll
                for (int e = 0; e < E; ++e)
                    if (valid(it, e)) s += v[it][e];
            mean = group_reduce<GROUP, THREADS, 0>(s, lds) * inv_n;
        }
        float q = 0.0f;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) {
                    v[it][e] -= mean;
                    q += v[it][e] * v[it][e];
                }
        const float var = group_reduce<GROUP, THREADS, 0>(q, lds) * inv_n;
        const float rstd = 1.0f / sqrtf(var + P.eps);
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e) v[it][e] *= rstd;
        if (P.norm_weight >= 0) apply_affine<IT, E, true, RAGGED>(P.norm_weight, P, v, r, col0, ok, nv);
        if (P.norm_bias >= 0) apply_affine<IT, E, false, RAGGED>(P.norm_bias, P, v, r, col0, ok, nv);
    }

    } // stage loop

    if (P.reduce == AXHIP_RED_NONE) {
        if (row_ok) {
#pragma unroll
            for (int it = 0; it < IT; ++it)
                if (ok[it]) {
                    if constexpr (E == 1) {
                        store_any(P.output, P.output_dtype, r * cols + col0[it], v[it][0]);
                    } else if constexpr (RAGGED) {
                        if (nv[it] == E) {
                            store_vec<E, true>(P.output, P.output_dtype, r * cols + col0[it], v[it]);
                        } else {
#pragma unroll
                            for (int e = 0; e < E; ++e)
                                if (e < nv[it]) store_any(P.output, P.output_dtype, r * cols + col0[it] + e, v[it][e]);
                        }
                    } else {
                        store_vec<E>(P.output, P.output_dtype, r * cols + col0[it], v[it]);
                    }
                }
        }
        return;
    }
    float acc;
    if (P.reduce == AXHIP_RED_SUM || P.reduce == AXHIP_RED_MEAN) {
        acc = 0.0f;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) acc += v[it][e];
        acc = group_reduce<GROUP, THREADS, 0>(acc, lds);
        if (P.reduce == AXHIP_RED_MEAN) acc *= inv_n;
    } else if (P.reduce == AXHIP_RED_MAX) {
        acc = NEG_INF;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) acc = fmaxf(acc, v[it][e]);
        acc = group_reduce<GROUP, THREADS, 1>(acc, lds);
    } else if (P.reduce == AXHIP_RED_PROD) {
        acc = 1.0f;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) acc *= v[it][e];
        acc = group_reduce<GROUP, THREADS, 3>(acc, lds);
    } else {
        acc = POS_INF;
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (valid(it, e)) acc = fminf(acc, v[it][e]);
        acc = group_reduce<GROUP, THREADS, 2>(acc, lds);
    }
    if (row_ok && lane_in_group == 0) store_any(P.output, P.output_dtype, r, acc);
}

// Rows too long for registers: one row per block, streamed in up to three
// passes (two for statistics, one to produce the output).  The pre-chain is
// recomputed in every pass instead of spilling the row.
template <int THREADS, int E>
__global__ __launch_bounds__(THREADS) void rows_streamed_kernel(const AxhipRowsProgram P) {
    __shared__ float lds[THREADS / WAVE];
    const int64_t row = blockIdx.x;
    const int64_t cols = P.cols;
    const int64_t nchunk = cols / E;
    const float inv_n = 1.0f / static_cast<float>(cols);
    const bool is_sm = P.row_op == AXHIP_ROWOP_SOFTMAX || P.row_op == AXHIP_ROWOP_LOGSOFTMAX;
    const bool is_norm = P.row_op == AXHIP_ROWOP_LAYERNORM || P.row_op == AXHIP_ROWOP_RMSNORM;
    // pass 0: softmax max / layer-norm mean; pass 1: softmax sum / variance; pass 2: output
    const int first_pass = is_sm || P.row_op == AXHIP_ROWOP_LAYERNORM ? 0 : is_norm ? 1 : 2;

    float stat_a = 0.0f, stat_b = 1.0f; // softmax: (max, 1/sum or log-sum); norms: (mean, rstd)
    float out_acc = red_start(P.reduce);
#pragma nounroll
    for (int pass = first_pass; pass < 3; ++pass) {
        float acc = (pass == 0 && is_sm) ? NEG_INF : 0.0f;
        for (int64_t c = threadIdx.x; c < nchunk; c += THREADS) {
            float v[1][E];
            const int64_t col0[1] = {c * E};
            const bool ok[1] = {true};
            if constexpr (E == 1) v[0][0] = load_any(P.input, P.input_dtype, row * cols + col0[0]);
            else load_vec<E>(P.input, P.input_dtype, row * cols + col0[0], v[0]);
            for (int i = 0; i < P.n_pre; ++i) apply_op<1, E>(P.pre[i], P, v, row, col0, ok);
            if (pass == 0) {
#pragma unroll
                for (int e = 0; e < E; ++e) acc = is_sm ? fmaxf(acc, v[0][e]) : acc + v[0][e];
            } else if (pass == 1) {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const float d = v[0][e] - stat_a;
                    acc += is_sm ? __expf(d) : d * d;
                }
            } else {
                if (P.row_op == AXHIP_ROWOP_SOFTMAX) {
#pragma unroll
                    for (int e = 0; e < E; ++e) v[0][e] = __expf(v[0][e] - stat_a) * stat_b;
                } else if (P.row_op == AXHIP_ROWOP_LOGSOFTMAX) {
#pragma unroll
                    for (int e = 0; e < E; ++e) v[0][e] = v[0][e] - stat_a - stat_b;
                } else if (is_norm) {
#pragma unroll
                    for (int e = 0; e < E; ++e) v[0][e] = (v[0][e] - stat_a) * stat_b;
                    if (P.norm_weight >= 0) apply_affine<1, E, true>(P.norm_weight, P, v, row, col0, ok);
                    if (P.norm_bias >= 0) apply_affine<1, E, false>(P.norm_bias, P, v, row, col0, ok);
                }
                for (int i = 0; i < P.n_post; ++i) apply_op<1, E>(P.post[i], P, v, row, col0, ok);
                if (P.reduce == AXHIP_RED_NONE) {
                    if constexpr (E == 1) store_any(P.output, P.output_dtype, row * cols + col0[0], v[0][0]);
                    else store_vec<E>(P.output, P.output_dtype, row * cols + col0[0], v[0]);
                } else {
#pragma unroll
                    for (int e = 0; e < E; ++e) out_acc = red_fold(P.reduce, out_acc, v[0][e]);
                }
            }
        }
        if (pass == 0) {
            if (is_sm) {
                const float m = group_reduce<THREADS, THREADS, 1>(acc, lds);
                stat_a = m == NEG_INF ? 0.0f : m;
            } else {
                stat_a = group_reduce<THREADS, THREADS, 0>(acc, lds) * inv_n;
            }
        } else if (pass == 1) {
            const float t = group_reduce<THREADS, THREADS, 0>(acc, lds);
            if (is_sm) stat_b = P.row_op == AXHIP_ROWOP_SOFTMAX ? 1.0f / t : __logf(t);
            else stat_b = 1.0f / sqrtf(t * inv_n + P.eps);
        }
    }
    if (P.reduce != AXHIP_RED_NONE) {
        out_acc = group_reduce_of<THREADS, THREADS>(P.reduce, out_acc, lds);
        if (P.reduce == AXHIP_RED_MEAN) out_acc *= inv_n;
        if (threadIdx.x == 0) store_any(P.output, P.output_dtype, row, out_acc);
    }
}

// Flat elementwise chain (no row op, no reduction): grid-stride over chunks of
// E elements of the flattened [rows*cols] range.  Requires cols % E == 0 so a
// chunk never straddles two rows.
template <int THREADS, int E>
__global__ __launch_bounds__(THREADS) void elementwise_kernel(const AxhipRowsProgram P, const bool streaming) {
    const int64_t cols = P.cols;
    const int64_t nchunk = P.rows * cols / E;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * THREADS;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * THREADS + threadIdx.x; c < nchunk; c += stride) {
        const int64_t flat = c * E;
        const int64_t row = flat / cols;
        const int64_t col0[1] = {flat - row * cols};
        const bool ok[1] = {true};
        float v[1][E];
        if constexpr (E == 1) v[0][0] = load_any(P.input, P.input_dtype, flat);
        else load_vec<E>(P.input, P.input_dtype, flat, v[0]);
        for (int i = 0; i < P.n_pre + P.n_post; ++i) apply_op<1, E>(i < P.n_pre ? P.pre[i] : P.post[i - P.n_pre], P, v, row, col0, ok);
        if constexpr (E == 1) store_any(P.output, P.output_dtype, flat, v[0][0]);
        else store_vec<E>(P.output, P.output_dtype, flat, v[0], streaming);
    }
}

// The same for arrays whose row length no vector divides (cols >= E, every full-size stream 16-byte aligned): the
// array is walked as one flat run of E-element chunks, which may straddle two rows -- a full-size operand does not
// care, a per-column or per-row operand is picked element by element where the chunk crosses a row end (and with one
// unaligned vector load where it does not).  The n % E elements behind the last whole chunk go one by one.
template <int THREADS, int E>
__global__ __launch_bounds__(THREADS) void elementwise_flat_kernel(const AxhipRowsProgram P, const bool streaming) {
    const int64_t cols = P.cols;
    const int64_t n = P.rows * cols;
    const int64_t nchunk = n / E;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * THREADS;
    const int n_ops = P.n_pre + P.n_post;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * THREADS + threadIdx.x; c < nchunk; c += stride) {
        const int64_t flat = c * E;
        const int64_t row = flat / cols, col = flat - row * cols;
        const int64_t at[1] = {flat};
        const bool ok[1] = {true};
        float v[1][E];
        load_vec<E>(P.input, P.input_dtype, flat, v[0]);
        for (int i = 0; i < n_ops; ++i) {
            const AxhipChainOp &op = i < P.n_pre ? P.pre[i] : P.post[i - P.n_pre];
            const bool by_position = is_binary_op(op.op) && op.imm_kind != AXHIP_BK_IMM &&
                                     (P.operands[op.operand].kind == AXHIP_BK_ROWVEC || P.operands[op.operand].kind == AXHIP_BK_COLVEC);
            if (!by_position) {
                apply_op<1, E>(op, P, v, 0, at, ok); // row 0, "column" = flat index: what a full-size operand's address is computed from
                continue;
            }
            const AxhipOperand &o = P.operands[op.operand];
            float w[E];
            if (o.kind == AXHIP_BK_ROWVEC && col + E <= cols) {
                load_vec<E, true>(o.ptr, o.dtype, col, w);
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const bool next = col + e >= cols; // (cols >= E: a chunk crosses at most one row end)
                    w[e] = load_any(o.ptr, o.dtype, o.kind == AXHIP_BK_ROWVEC ? col + e - (next ? cols : 0) : row + (next ? 1 : 0));
                }
            }
            apply_binary_tile<1, E, true>(op.op, v, [&](int, int e) { return w[e]; });
        }
        store_vec<E>(P.output, P.output_dtype, flat, v[0], streaming);
    }
    const int64_t flat = nchunk * E + threadIdx.x;
    if (blockIdx.x == 0 && flat < n) {
        const int64_t row = flat / cols;
        const int64_t col0[1] = {flat - row * cols};
        const bool ok[1] = {true};
        float v[1][1];
        v[0][0] = load_any(P.input, P.input_dtype, flat);
        for (int i = 0; i < n_ops; ++i) apply_op<1, 1>(i < P.n_pre ? P.pre[i] : P.post[i - P.n_pre], P, v, row, col0, ok);
        store_any(P.output, P.output_dtype, flat, v[0][0]);
    }
}

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

struct RowsPlan {
    enum Kind { EMPTY, ELEMENTWISE, ELEMENTWISE_FLAT, RESIDENT, STREAMED } kind;
    int e, it, group, threads;
    bool ragged; // resident plan on rows that are not whole, aligned vectors: unaligned accesses, element-wise last chunk
    char name[64];
};

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

template <int GROUP, int IT, int E>
void launch_resident(const AxhipRowsProgram &P, bool ragged, hipStream_t s) {
    constexpr int THREADS = GROUP > 256 ? GROUP : 256;
    const int64_t rows_per_block = THREADS / GROUP;
    const unsigned grid = static_cast<unsigned>((P.rows + rows_per_block - 1) / rows_per_block);
    if constexpr (E > 1) {
        if (ragged) {
            hipLaunchKernelGGL((rows_resident_kernel<THREADS, GROUP, IT, E, true>), dim3(grid), dim3(THREADS), 0, s, P);
            return;
        }
    }
    hipLaunchKernelGGL((rows_resident_kernel<THREADS, GROUP, IT, E, false>), dim3(grid), dim3(THREADS), 0, s, P);
}

template <int GROUP, int E>
int launch_resident_it(const AxhipRowsProgram &P, int it, bool ragged, hipStream_t s) {
    switch (it) {
    case 1: launch_resident<GROUP, 1, E>(P, ragged, s); return AXHIP_OK;
    case 2: launch_resident<GROUP, 2, E>(P, ragged, s); return AXHIP_OK;
    case 4: launch_resident<GROUP, 4, E>(P, ragged, s); return AXHIP_OK;
    case 8:
        if constexpr (GROUP == 256) {
            launch_resident<GROUP, 8, E>(P, ragged, s);
            return AXHIP_OK;
        }
        [[fallthrough]];
    default:
        set_last_error("fused rows: no resident variant for it=%d", it);
        return AXHIP_ERR_UNSUPPORTED;
    }
}

template <int E>
int launch_plan_e(const AxhipRowsProgram &P, const RowsPlan &pl, hipStream_t s) {
    switch (pl.kind) {
    case RowsPlan::ELEMENTWISE: {
        const int64_t nchunk = P.rows * P.cols / E;
        const int64_t blocks = std::min<int64_t>((nchunk + 255) / 256, 256 * 32);
        const bool streaming = P.rows * P.cols * static_cast<int64_t>(dtype_size(P.output_dtype)) >= STREAMING_OUTPUT_BYTES;
        hipLaunchKernelGGL((elementwise_kernel<256, E>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, P, streaming);
        return AXHIP_OK;
    }
    case RowsPlan::ELEMENTWISE_FLAT: {
        if constexpr (E > 1) {
            const int64_t nchunk = P.rows * P.cols / E;
            const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>((nchunk + 255) / 256, 256 * 32));
            const bool streaming = P.rows * P.cols * static_cast<int64_t>(dtype_size(P.output_dtype)) >= STREAMING_OUTPUT_BYTES;
            hipLaunchKernelGGL((elementwise_flat_kernel<256, E>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, P, streaming);
        }
        return AXHIP_OK;
    }
    case RowsPlan::RESIDENT:
        if (pl.group == 1024) {
            launch_resident<1024, 4, E>(P, pl.ragged, s);
            return AXHIP_OK;
        }
        return pl.group == 64 ? launch_resident_it<64, E>(P, pl.it, pl.ragged, s) : launch_resident_it<256, E>(P, pl.it, pl.ragged, s);
    case RowsPlan::STREAMED:
        hipLaunchKernelGGL((rows_streamed_kernel<1024, E>), dim3(static_cast<unsigned>(P.rows)), dim3(1024), 0, s, P);
        return AXHIP_OK;
    default:
        return AXHIP_OK;
    }
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

} // namespace axhip

using namespace axhip;

extern "C" {

const char *axhip_fused_rows_kernel_name(const AxhipRowsProgram *P) {
    static thread_local char name[192];
    if (!P) return "invalid";
    if (validate_program(*P, "axhip_fused_rows_kernel_name") == AXHIP_OK && rows_prog_dispatch(*P, nullptr, false, name, sizeof(name), nullptr))
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
    if (rows_prog_dispatch(P, s, true, nullptr, 0, &launch_rc)) {
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
    if (!rows_prog_dispatch(*program, nullptr, false, name, sizeof(name), nullptr)) return AXHIP_OK; // the interpreter's: nothing to prepare
    if (strncmp(name, "rows_static_", 12) == 0) return AXHIP_OK;                                    // built into the library
    std::string label, error;
    if (!rows_prog_compile_only(*program, &label, &error)) {
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
