// The interpreter's row kernels and their launchers.  Shared by rows.hip (host side, and the scalar-width
// kernels) and rows_e4.hip / rows_e8.hip / rows_e8_ragged.hip, which instantiate the launchers of the 4- and 8-element
// vector widths: four translation units compile side by side instead of one after the other.
//
// Layout: a [rows, cols] row-major view.  A row is held in registers as fp32:
// each thread owns IT chunks of E consecutive elements (E*elem = 16 or 32 bytes,
// so every global access is a full-width vector), chunk c = it*GROUP + lane_in_group,
// which makes consecutive lanes touch consecutive 16/32-byte segments.
// Reductions are wave64 shuffles plus one LDS hop when a row spans several waves.
#pragma once
#include "common.hpp"
#include "rows_ops.hpp"
#include "rows_prog.hpp"

#include <algorithm>

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

// ------------------------------------------------------------------ launchers

struct RowsPlan {
    enum Kind { EMPTY, ELEMENTWISE, ELEMENTWISE_FLAT, RESIDENT, STREAMED } kind;
    int e, it, group, threads;
    bool ragged; // resident plan on rows that are not whole, aligned vectors: unaligned accesses, element-wise last chunk
    char name[64];
};

template <int GROUP, int IT, int E, bool RAGGED>
void launch_resident(const AxhipRowsProgram &P, hipStream_t s) {
    constexpr int THREADS = GROUP > 256 ? GROUP : 256;
    const int64_t rows_per_block = THREADS / GROUP;
    const unsigned grid = static_cast<unsigned>((P.rows + rows_per_block - 1) / rows_per_block);
    hipLaunchKernelGGL((rows_resident_kernel<THREADS, GROUP, IT, E, RAGGED>), dim3(grid), dim3(THREADS), 0, s, P);
}

// The resident kernels of one vector width and one raggedness: (group, chunks per lane) = (64 | 256, 1 | 2 | 4),
// (256, 8), (1024, 4).
template <int E, bool RAGGED>
int launch_resident_plan(const AxhipRowsProgram &P, int group, int it, hipStream_t s) {
    if (group == 1024) {
        launch_resident<1024, 4, E, RAGGED>(P, s);
        return AXHIP_OK;
    }
    const bool wave_rows = group == 64;
    switch (it) {
    case 1: wave_rows ? launch_resident<64, 1, E, RAGGED>(P, s) : launch_resident<256, 1, E, RAGGED>(P, s); return AXHIP_OK;
    case 2: wave_rows ? launch_resident<64, 2, E, RAGGED>(P, s) : launch_resident<256, 2, E, RAGGED>(P, s); return AXHIP_OK;
    case 4: wave_rows ? launch_resident<64, 4, E, RAGGED>(P, s) : launch_resident<256, 4, E, RAGGED>(P, s); return AXHIP_OK;
    case 8:
        if (!wave_rows) {
            launch_resident<256, 8, E, RAGGED>(P, s);
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
        if constexpr (E > 1) {
            if (pl.ragged) return launch_resident_plan<E, true>(P, pl.group, pl.it, s);
        }
        return launch_resident_plan<E, false>(P, pl.group, pl.it, s);
    case RowsPlan::STREAMED:
        hipLaunchKernelGGL((rows_streamed_kernel<1024, E>), dim3(static_cast<unsigned>(P.rows)), dim3(1024), 0, s, P);
        return AXHIP_OK;
    default:
        return AXHIP_OK;
    }
}

// instantiated in rows_e4.hip, rows_e8.hip and rows_e8_ragged.hip
extern template int launch_plan_e<4>(const AxhipRowsProgram &, const RowsPlan &, hipStream_t);
extern template int launch_plan_e<8>(const AxhipRowsProgram &, const RowsPlan &, hipStream_t);
extern template int launch_resident_plan<8, true>(const AxhipRowsProgram &, int, int, hipStream_t);

} // namespace axhip
