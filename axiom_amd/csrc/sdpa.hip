// Scaled-dot-product attention, forward, for gfx950.
//
// The kernels:
//   sdpa_mfma_pingpong_kernel   bf16 / f16, head_dim 128, no explicit mask,
//                       problems that fill the chip: the pipelined kernel's
//                       tiling with the two waves of a SIMD half a step apart
//                       (one in its matrix phase, one in its softmax phase) and
//                       persistent work-groups.
//   sdpa_mfma_pipelined_kernel  bf16 / f16, head_dim 64 / 128.  FlashAttention-2
//                       schedule on v_mfma_f32_32x32x16_{bf16,f16}: one
//                       workgroup = 4 or 8 wave64, each wave owns 32 query
//                       rows whose fragments stay in registers; K and V tiles
//                       of 64 keys go from HBM straight into swizzled LDS
//                       (buffer_load ... lds) two tiles ahead of their use;
//                       the softmax of tile j is interleaved with the two
//                       matrix products of tiles j+1 and j-1; fp32 online
//                       softmax in the exp2 domain; fp32 accumulators.
//   sdpa_mfma_kernel    bf16 / f16, head_dim 32: same arithmetic, K and V tiles
//                       staged through registers into LDS.
//   sdpa_generic_kernel any dtype, head_dim <= 256, fp32 FMA arithmetic; used
//                       for fp32 inputs and for head sizes the MFMA kernels do
//                       not cover.
//
// The MFMA kernels compute the TRANSPOSED score tile S^T = K * Q^T, so that in
// the 32x32 accumulator layout every lane owns ONE query column (lane % 32) and
// 16 key rows.  Row statistics of the softmax are then in-lane reductions plus a
// single exchange with lane ^ 32, and the exponentiated tile is already laid out
// as the B operand of the second product O^T += V^T * P^T: no trip through LDS
// for P.
#include "common.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <type_traits>

namespace axhip {

struct SdpaArgs {
    const void *q, *k, *v;
    void *o;
    const uint8_t *mask;
    int B, H, Sq, Skv, D;
    float scale;       // softmax scale
    float scale_log2e; // scale * log2(e)
    int causal;
    int nqb; // query blocks per (batch, head)
    int dtype;
    int64_t qs[3], ks[3], vs[3], os[3], ms[2];
    // key split of sdpa_mfma_kernel (decoding: few query rows, few heads, a long key sequence): `ksplit` work-groups
    // per (batch, head) take `kchunk` keys each and leave normalised fp32 partial outputs and the base-2 logarithm of
    // their softmax denominators (reference maximum included) for sdpa_splitk_merge_kernel
    int ksplit, kchunk;
    float *opart, *lse;
};

constexpr float NEG_INF_F = -__builtin_huge_valf();

// ---------------------------------------------------------------- MFMA kernel

constexpr int BM = 128; // query rows per workgroup (4 waves x 32)
constexpr int BN = 64;  // keys per LDS tile
// Growth of the running row maximum (log2 domain) that is tolerated before the
// accumulators are rescaled: exponentials stay below 2^8, far inside fp32/bf16/f16 range.
constexpr float RESCALE_THRESHOLD = 8.0f;

template <bool BF16>
__device__ __forceinline__ float16_t mfma_32x32x16(uint4_t a, uint4_t b, float16_t c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}

template <bool BF16> __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    if constexpr (BF16) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        typedef float float2_t __attribute__((ext_vector_type(2)));
        float2_t f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t)); // v_cvt_pk_bf16_f32, RNE
    } else {
        return pack_f16x2(lo, hi); // v_cvt_pk_f16_f32, RNE
    }
}

// acc + lo + hi of a packed pair, one v_dot2c instruction
template <bool BF16> __device__ __forceinline__ float add_pair(uint32_t packed, float acc) {
    if constexpr (BF16) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, packed), __builtin_bit_cast(bf16x2_t, 0x3F803F80u), acc, false);
    } else {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, packed), __builtin_bit_cast(half2_t, 0x3C003C00u), acc, false);
    }
}

// LDS transpose read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i
// receives element (i & 3) of the 8-byte rows addressed by lanes (i >> 2) + 4*j,
// j = 0..3.  Addressed as below, lane i of a group ends up with 4 consecutive keys
// of ONE head dimension although V sits in LDS in its natural [key][dim] layout.
__device__ __forceinline__ uint2_t lds_read_tr16(const uint16_t *p) {
    typedef short short4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_t lds_short4_t;
    short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t *)(p));
    return __builtin_bit_cast(uint2_t, v);
}

// D = 256: the two K and two V tile buffers (138 KiB) are dynamic LDS, one work-group per CU, one wave per SIMD
// with the registers that go with it (the output accumulators alone are 128).
// A head size below D (a.D, a multiple of 8) runs with zeros in the missing dims: Q fragments and K/V chunks beyond
// a.D are not fetched, the output keeps a.D columns.
template <int D> constexpr size_t sdpa_mfma_lds_bytes() { return 2 * BN * ((D + 8) + (D + 32)) * 2; }
extern __shared__ __attribute__((aligned(16))) unsigned char sdpa_dyn_lds[];

template <bool BF16, int D, bool HAS_MASK, bool SPLITK = false>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void sdpa_mfma_kernel(const SdpaArgs a_in) {
    static_assert(!SPLITK || !HAS_MASK, "the key split is for unmasked decoding steps");
    SdpaArgs a = a_in;
    int L = blockIdx.x, split = 0;
    if constexpr (SPLITK) { // this work-group's share of the keys: a shorter sequence from a later start
        split = L % a.ksplit;
        L /= a.ksplit;
        const int begin = split * a.kchunk;
        a.k = static_cast<const uint16_t *>(a.k) + begin * a.ks[2];
        a.v = static_cast<const uint16_t *>(a.v) + begin * a.vs[2];
        a.Skv = min(a.kchunk, a.Skv - begin);
    }
    constexpr int KS_STRIDE = D + 8;   // K row stride (elements): +16 B shifts consecutive rows by 4 banks
    constexpr int VS_STRIDE = D + 32;  // V row stride: +64 B shifts rows by 16 banks, what the 4-row transpose reads need
    constexpr int KT = D / 16;         // k-steps of the first product
    constexpr int DT = D / 32;         // 32-row tiles of O^T
    constexpr int KCH = D / 8;         // 16-byte chunks per K/V row
    constexpr int NLD = BN * KCH / 256 > 0 ? BN * KCH / 256 : 1; // 16-byte chunks per thread per tile
    constexpr int ROWS_PER_PASS = 256 / KCH; // rows covered by one chunk pass of the whole workgroup
    constexpr int KBUF = BN * KS_STRIDE, VBUF = BN * VS_STRIDE; // elements per tile buffer
    constexpr bool DYN = D >= 128; // (more than the 64 KiB of static LDS)
    __shared__ __attribute__((aligned(16))) uint16_t Ks_static[DYN ? 8 : 2 * KBUF];
    __shared__ __attribute__((aligned(16))) uint16_t Vs_static[DYN ? 8 : 2 * VBUF];
    uint16_t *const Ks = DYN ? reinterpret_cast<uint16_t *>(sdpa_dyn_lds) : Ks_static;
    uint16_t *const Vs = DYN ? reinterpret_cast<uint16_t *>(sdpa_dyn_lds) + 2 * KBUF : Vs_static;

    const int tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int ql = lane % 32, g = lane / 32;

    // Work-group -> (batch*head, query block).  Work-groups are dealt to the 8
    // XCDs round-robin by id; keeping one (batch, head) on one XCD lets its K/V
    // live in that XCD's L2.  Causal blocks are issued heaviest first.
    const int BH = a.B * a.H;
    int bh, qb;
    if (BH % 8 == 0) {
        const int xcd = L % 8, j = L / 8;
        bh = (j / a.nqb) * 8 + xcd;
        qb = j % a.nqb;
    } else {
        bh = L / a.nqb;
        qb = L % a.nqb;
    }
    if (a.causal) qb = a.nqb - 1 - qb;
    const int b = bh / a.H, h = bh % a.H;

    const uint16_t *Q = static_cast<const uint16_t *>(a.q) + b * a.qs[0] + h * a.qs[1];
    const uint16_t *K = static_cast<const uint16_t *>(a.k) + b * a.ks[0] + h * a.ks[1];
    const uint16_t *V = static_cast<const uint16_t *>(a.v) + b * a.vs[0] + h * a.vs[1];
    uint16_t *O = static_cast<uint16_t *>(a.o) + b * a.os[0] + h * a.os[1];
    const uint8_t *M = HAS_MASK ? a.mask + b * a.ms[0] + h * a.ms[1] : nullptr;

    const int q0 = qb * BM;
    const int qw0 = q0 + wave * 32; // first query row of this wave
    const int q = qw0 + ql;
    const bool q_ok = q < a.Sq;

    // K / V are fetched through buffer descriptors: rows past the end of the
    // sequence read as zero instead of touching memory.
    const int krow_bytes = static_cast<int>(a.ks[2]) * 2, vrow_bytes = static_cast<int>(a.vs[2]) * 2;
    const int dv = a.D; // the head size in memory (<= D, a multiple of 8)
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(K), 0, a.Skv > 0 ? (a.Skv - 1) * krow_bytes + dv * 2 : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(V), 0, a.Skv > 0 ? (a.Skv - 1) * vrow_bytes + dv * 2 : 0, 0x00020000);
    const int ld_row = tid / KCH, ld_cc = tid % KCH; // this thread's chunk in pass 0
    const bool ld_active = KCH * BN >= 256 || tid < KCH * BN;
    const bool ld_fetch = ld_active && ld_cc * 8 < dv; // (a chunk beyond the head size is staged as zeros)
    const int k_voff = ld_row * krow_bytes + ld_cc * 16, v_voff = ld_row * vrow_bytes + ld_cc * 16;

    // Q^T fragments (B operand): lane holds Q[q][16t + 8g .. +8]
    uint4_t qf[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        qf[t] = uint4_t{0, 0, 0, 0};
        if (q_ok && 16 * t + 8 * g < dv) qf[t] = *reinterpret_cast<const uint4_t *>(Q + static_cast<int64_t>(q) * a.qs[2] + 16 * t + 8 * g);
    }

    float16_t oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.0f;
    float m_run = NEG_INF_F; // reference maximum of the exponentials (scaled log2 domain); may lag the true maximum
    float l_run = 0.0f;      // this lane's share of the running denominator

    int kv_end = a.Skv;
    if (a.causal) kv_end = min(a.Skv, q0 + BM);
    const int ntiles = (kv_end + BN - 1) / BN;

    uint4_t kreg[NLD], vreg[NLD];
    auto load_tile = [&](int tile) {
#pragma unroll
        for (int n = 0; n < NLD; ++n) {
            // the whole offset rides in the vector operand: only that one is bounds-checked
            const int row0 = tile * BN + n * ROWS_PER_PASS;
            kreg[n] = uint4_t{0, 0, 0, 0};
            vreg[n] = uint4_t{0, 0, 0, 0};
            if (ld_fetch) {
                kreg[n] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, k_voff + row0 * krow_bytes, 0, 0);
                vreg[n] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, v_voff + row0 * vrow_bytes, 0, 0);
            }
        }
    };
    auto stage_tile = [&](int buf) {
        if (ld_active) {
#pragma unroll
            for (int n = 0; n < NLD; ++n) {
                const int row = ld_row + n * ROWS_PER_PASS;
                *reinterpret_cast<uint4_t *>(&Ks[buf * KBUF + row * KS_STRIDE + 8 * ld_cc]) = kreg[n];
                *reinterpret_cast<uint4_t *>(&Vs[buf * VBUF + row * VS_STRIDE + 8 * ld_cc]) = vreg[n];
            }
        }
    };

    // per-lane element offsets of the LDS fragment reads
    const int k_frag = ql * KS_STRIDE + 8 * g;                                         // + kt*32*KS_STRIDE + 16*t
    const int v_frag = (g * 4 + ((lane & 15) >> 2)) * VS_STRIDE + ((lane >> 4) & 1) * 16 + 4 * (lane & 3); // + ks*16*VS_STRIDE + dt*32

    // ntiles >= 1: the host never launches this kernel with an empty key sequence.
    // The prologue is deliberately unconditional and ends in an explicit vmcnt(0)
    // (Q and tile 0 have landed by then anyway): with that the compiler's in-loop
    // waits cover only the tile they need, not the prefetch issued just before.
    load_tile(0);
    stage_tile(0);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    if (ntiles > 1) load_tile(1);
    __syncthreads();

    for (int tile = 0; tile < ntiles; ++tile) {
        const int kv0 = tile * BN;
        const int buf = tile & 1;
        // registers hold tile+1: park it in the other buffer (every wave left that
        // buffer at the barrier that closed the previous iteration), then start on tile+2
        if (tile + 1 < ntiles) stage_tile(buf ^ 1);
        if (tile + 2 < ntiles) load_tile(tile + 2);

        // a wave whose last query row precedes this tile has nothing to add
        if (!(a.causal && kv0 > qw0 + 31)) {
            const uint16_t *Kb = Ks + buf * KBUF, *Vb = Vs + buf * VBUF;

            // explicit mask: the eight 4-byte words that cover this lane's keys of the tile (8 runs of 4 consecutive
            // keys), requested ahead of the score MFMAs; needs whole tiles and 4-byte aligned mask rows
            uint32_t mw[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            bool mask_words_tile = false;
            if constexpr (HAS_MASK) {
                mask_words_tile = a.Skv % 4 == 0 && (reinterpret_cast<uintptr_t>(M) & 3u) == 0 && kv0 + BN <= a.Skv;
                if (mask_words_tile && q_ok) {
                    const uint32_t *row = reinterpret_cast<const uint32_t *>(M + static_cast<int64_t>(q) * a.Skv + kv0 + 4 * g);
#pragma unroll
                    for (int w8 = 0; w8 < 8; ++w8) mw[w8] = row[(w8 / 4) * 8 + (w8 % 4) * 2];
                }
            }

            // ---- S^T = K Q^T : two 32-key sub-tiles
            float16_t s[2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[kt][i] = 0.0f;
#pragma unroll
                for (int t = 0; t < KT; ++t) {
                    const uint4_t kf = *reinterpret_cast<const uint4_t *>(&Kb[k_frag + kt * 32 * KS_STRIDE + 16 * t]);
                    s[kt] = mfma_32x32x16<BF16>(kf, qf[t], s[kt]);
                }
            }

            // ---- masking: only tiles that touch the diagonal, the key tail or an explicit mask
            const bool need_mask = (a.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > a.Skv) || HAS_MASK;
            if (need_mask) {
                const int kv_limit = a.causal ? min(a.Skv - 1, q) : a.Skv - 1; // last visible key of this row
                if (!HAS_MASK || mask_words_tile) {
                    // selects on values already in registers (for an explicit mask: the words fetched above)
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int kv = kv0 + kt * 32 + (i / 4) * 8 + g * 4 + (i % 4);
                            bool dead = kv > kv_limit;
                            if constexpr (HAS_MASK) dead = dead || ((mw[kt * 4 + i / 4] >> (8 * (i % 4))) & 0xFFu) != 0;
                            s[kt][i] = dead ? NEG_INF_F : s[kt][i];
                        }
                } else {
                    // ragged last tile, unaligned mask rows: byte by byte
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int kv = kv0 + kt * 32 + (i / 4) * 8 + g * 4 + (i % 4);
                            bool dead = kv > kv_limit;
                            if constexpr (HAS_MASK) {
                                if (q_ok && kv < a.Skv) dead = dead || M[static_cast<int64_t>(q) * a.Skv + kv] != 0;
                            }
                            s[kt][i] = dead ? NEG_INF_F : s[kt][i];
                        }
                }
            }

            // ---- online softmax (per lane: one query column, 32 of the 64 keys)
            float mloc = NEG_INF_F;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[kt][i]);
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
            const float m_new = fmaxf(m_run, mloc * a.scale_log2e);
            // rescale only when some row's maximum outgrew its reference by the threshold
            // (-inf - -inf = NaN compares false: a row with no visible key yet keeps -inf)
            if (__builtin_amdgcn_ballot_w64(m_new - m_run > RESCALE_THRESHOLD) != 0) {
                const float alpha = m_new == NEG_INF_F ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                l_run *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
            }
            const float m_use = m_run == NEG_INF_F ? 0.0f : m_run;
            uint4_t pf[4]; // P^T fragments (B operand), one per 16-key k-step
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                uint32_t w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][2 * i], a.scale_log2e, -m_use));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][2 * i + 1], a.scale_log2e, -m_use));
                    w[i] = pack2<BF16>(p0, p1);
                    l_run = add_pair<BF16>(w[i], l_run); // the denominator sums exactly what the MFMA multiplies
                }
                pf[2 * kt] = uint4_t{w[0], w[1], w[2], w[3]};
                pf[2 * kt + 1] = uint4_t{w[4], w[5], w[6], w[7]};
            }

            // ---- O^T += V^T P^T, V^T fragments through the LDS transpose read
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const uint16_t *p = &Vb[v_frag + ks * 16 * VS_STRIDE + dt * 32];
                    const uint2_t lo = lds_read_tr16(p);
                    const uint2_t hi = lds_read_tr16(p + 8 * VS_STRIDE);
                    const uint4_t vf = {lo.x, lo.y, hi.x, hi.y};
                    oacc[dt] = mfma_32x32x16<BF16>(vf, pf[ks], oacc[dt]);
                }
        }
        __syncthreads();
    }

    // ---- epilogue: O = O^T / l, written as 4 consecutive dims (8 bytes) per store
    const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if constexpr (SPLITK) {
        if (q_ok) {
            const int64_t slot = (static_cast<int64_t>(bh) * a.ksplit + split) * a.Sq + q;
            float *orow = a.opart + slot * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const float4_t w = {oacc[dt][4 * i4] * inv, oacc[dt][4 * i4 + 1] * inv, oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv};
                    *reinterpret_cast<float4_t *>(orow + dt * 32 + i4 * 8 + g * 4) = w;
                }
            if (g == 0) a.lse[slot] = l_tot > 0.0f ? m_run + __builtin_amdgcn_logf(l_tot) : NEG_INF_F; // (v_log_f32: base 2, as the exponentials)
        }
        return;
    }
    if (q_ok) {
        uint16_t *orow = O + static_cast<int64_t>(q) * a.os[2];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int d = dt * 32 + i4 * 8 + g * 4;
                uint2_t w = {pack2<BF16>(oacc[dt][4 * i4] * inv, oacc[dt][4 * i4 + 1] * inv),
                             pack2<BF16>(oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv)};
                if (d < dv) *reinterpret_cast<uint2_t *>(orow + d) = w;
            }
    }
}

// out = sum_s 2^(lse_s - max lse) O_s / sum_s 2^(lse_s - max lse) over the `ksplit` partial results of a (batch, head,
// query row); a thread per (row, four dims)
template <bool BF16>
__global__ __launch_bounds__(256) void sdpa_splitk_merge_kernel(const SdpaArgs a, int D) {
    const int64_t quads = D / 4, total = static_cast<int64_t>(a.B) * a.H * a.Sq * quads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t row = i / quads; // (batch, head, query row)
        const int d = static_cast<int>(i - row * quads) * 4;
        const int64_t bh = row / a.Sq;
        const int q = static_cast<int>(row - bh * a.Sq);
        float top = NEG_INF_F;
        for (int s = 0; s < a.ksplit; ++s) top = fmaxf(top, a.lse[(bh * a.ksplit + s) * a.Sq + q]);
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f}, den = 0.0f;
        if (top != NEG_INF_F)
            for (int s = 0; s < a.ksplit; ++s) {
                const int64_t slot = (bh * a.ksplit + s) * a.Sq + q;
                const float w = __builtin_amdgcn_exp2f(a.lse[slot] - top);
                const float4_t o = *reinterpret_cast<const float4_t *>(a.opart + slot * D + d);
                acc[0] += w * o[0]; acc[1] += w * o[1]; acc[2] += w * o[2]; acc[3] += w * o[3];
                den += w;
            }
        const float inv = den > 0.0f ? 1.0f / den : 0.0f;
        if (d < a.D) {
            uint16_t *orow = static_cast<uint16_t *>(a.o) + (bh / a.H) * a.os[0] + (bh % a.H) * a.os[1] + static_cast<int64_t>(q) * a.os[2];
            const uint2_t w = {pack2<BF16>(acc[0] * inv, acc[1] * inv), pack2<BF16>(acc[2] * inv, acc[3] * inv)};
            *reinterpret_cast<uint2_t *>(orow + d) = w;
        }
    }
}

// --------------------------------- pipelined MFMA kernel, head_dim 128 and 64
// Same tiling as sdpa_mfma_kernel, restructured for throughput:
//  * K and V tiles go HBM -> LDS directly (buffer_load ... lds), no staging
//    registers and no ds_write; rows sit unpadded (2 D bytes) in LDS with the 16-byte
//    chunk index XOR-swizzled by the row, which keeps both the K fragment reads
//    (16 consecutive rows, one chunk) and the V transpose reads (4 rows x 64 B)
//    free of bank conflicts.
//  * software pipeline: while the softmax of tile j runs on the VALU, the score
//    MFMAs of tile j+1 are already in flight, so one wave keeps both pipes busy.
//    K therefore runs one tile ahead of V in LDS.

typedef int int4_t __attribute__((ext_vector_type(4)));

// XOR applied to the 16-byte chunk index of an LDS row, per buffer and head size.  256-byte rows (D = 128) span all
// banks, so one function of row & 15 with 16 distinct values serves the K fragment reads (16 consecutive rows, one
// chunk) and the V transpose reads (4 rows x 64 bytes).  128-byte rows (D = 64) put two rows in one bank sweep: K rows
// are spread by (row >> 1) & 7, V rows of a 4-row transpose read alternate between the two halves of the row.
template <int D> __device__ __forceinline__ int swizzle_k(int row) { return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((row >> 1) & 7); }
template <int D> __device__ __forceinline__ int swizzle_v(int row) { return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : (((row >> 1) & 1) << 2); }

// One 16-byte element per lane from a buffer straight into LDS: lane i's data lands at
// lds_base + 16*i.  Out-of-range lanes (voffset beyond the descriptor) write zeros.
__device__ __forceinline__ void load_to_lds_16(const int4_t &rsrc, uint32_t lds_base_uniform, int voffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(lds_base_uniform), "v"(voffset), "s"(rsrc) : "memory");
}

__device__ __forceinline__ int4_t make_rsrc(const void *base, int bytes) {
    const uint64_t pa = reinterpret_cast<uint64_t>(base);
    return int4_t{static_cast<int>(static_cast<uint32_t>(pa)), static_cast<int>(static_cast<uint32_t>(pa >> 32) & 0xFFFFu), bytes, 0x00020000};
}

// NW waves per work-group (4: two work-groups share a CU; 8: one work-group per CU, each
// K/V tile fetched once for 256 query rows instead of 128).
// Head sizes between the compiled ones (a.D = 40 .. 56 on D = 64, 72 .. 120 on D = 128, multiples of 8) run as the next
// compiled size with zeros in the missing dims: the Q fragments beyond a.D stay zero, the lanes that would fetch a K/V
// chunk beyond a.D are sent outside the tile's descriptor (the load writes zeros to LDS), the output keeps a.D columns.
// SPLIT = 2 (problems too small to give every SIMD two waves otherwise): the work-group's waves form two halves that
// take the same 32 * NW / 2 query rows and one half of the keys each, through K/V tile buffers of their own; the second
// half hands its accumulators, reference maximum and row sums to the first through LDS at the end.  No causal mask, no
// explicit mask, at least two key tiles.
// (Four K and four V tile buffers with counted waits, so that a tile is requested three steps before its use, made the
// 4-wave head_dim-64 kernel 5 % slower on small problems: its step is not waiting for tiles.)
// (PAD: such a head size; the exact sizes keep a kernel without its tests.)
template <bool BF16, bool HAS_MASK, int NW, int D, int SPLIT = 1, bool PAD = false>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void sdpa_mfma_pipelined_kernel(const SdpaArgs a) {
    static_assert(D == 128 || D == 64, "head sizes with a direct-to-LDS pipeline");
    static_assert(SPLIT == 1 || (SPLIT == 2 && !HAS_MASK && NW == 4 && D == 64), "key split: the 64 KiB of static LDS hold two sets of head_dim-64 tiles");
    constexpr int NWH = NW / SPLIT;       // waves that share a key range
    constexpr int KT = D / 16;            // k-steps of the score product
    constexpr int DT = D / 32;            // 32-row tiles of O^T
    constexpr int BMW = 32 * NWH;         // query rows per work-group
    constexpr int ROWB = 2 * D;           // bytes per LDS row
    constexpr int CHUNKS = ROWB / 16;     // 16-byte chunks per row
    constexpr int RPL = 64 / CHUNKS;      // rows moved by one wave-wide load
    constexpr int NLOAD = BN / (RPL * NWH); // wave-wide loads per wave per tile
    constexpr int TILEB = BN * ROWB;      // 16 / 8 KiB per K or V tile
    __shared__ __attribute__((aligned(1024))) unsigned char lds_all[SPLIT * 4 * TILEB]; // per half: K0 K1 V0 V1

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int part = SPLIT == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid / WAVE / NWH); // which half of the keys
    const int wave = SPLIT == 1 ? tid / WAVE : __builtin_amdgcn_readfirstlane(tid / WAVE % NWH); // position among the waves of its half
    unsigned char *const lds = lds_all + part * 4 * TILEB;
    const int ql = lane % 32, g = lane / 32;

    // Work-group -> (batch*head, query block(s)).  Under a causal mask query block i needs
    // i+1 key blocks, so a work-group takes the pair (i, nqb-1-i): every work-group then
    // carries the same load and the launch has no ragged tail.  Work-groups are dealt to
    // the 8 XCDs round-robin by id; one (batch, head) stays on one XCD so that its K/V
    // live in that XCD's L2.
    const int L = blockIdx.x;
    const int BH = a.B * a.H;
    const int nqb = (a.Sq + BMW - 1) / BMW;
    const int per_bh = a.causal ? (nqb + 1) / 2 : nqb; // work-groups per (batch, head)
    int bh, slot;
    if (BH % 8 == 0) {
        const int xcd = L % 8, j = L / 8;
        bh = (j / per_bh) * 8 + xcd;
        slot = j % per_bh;
    } else {
        bh = L / per_bh;
        slot = L % per_bh;
    }
    const int b = bh / a.H, h = bh % a.H;
    const int npass = (a.causal && slot != nqb - 1 - slot) ? 2 : 1;

    const uint16_t *Q = static_cast<const uint16_t *>(a.q) + b * a.qs[0] + h * a.qs[1];
    const uint16_t *K = static_cast<const uint16_t *>(a.k) + b * a.ks[0] + h * a.ks[1];
    const uint16_t *V = static_cast<const uint16_t *>(a.v) + b * a.vs[0] + h * a.vs[1];
    uint16_t *O = static_cast<uint16_t *>(a.o) + b * a.os[0] + h * a.os[1];
    const uint8_t *M = HAS_MASK ? a.mask + b * a.ms[0] + h * a.ms[1] : nullptr;
    // Explicit masks are read as the eight 4-byte words that cover this lane's keys of a tile (the lane's 32 keys are
    // 8 runs of 4 consecutive ones), a step before the tile's score MFMAs are issued, and applied by starting the
    // masked elements' accumulators at -inf: the mask costs two VALU operations per score and no pass of its own.
    // Needs 4-byte aligned rows (else, and for the ragged last tile, single bytes are read after the MFMAs).
    const bool mask_words = HAS_MASK && a.Skv % 4 == 0 && (reinterpret_cast<uintptr_t>(M) & 3u) == 0;
    uint32_t mk[8] = {0, 0, 0, 0, 0, 0, 0, 0};

    const int dv = PAD ? a.D : D; // the head size in memory (<= D, a multiple of 8)
    const int krow_bytes = static_cast<int>(a.ks[2]) * 2, vrow_bytes = static_cast<int>(a.vs[2]) * 2;
    const int4_t krsrc = make_rsrc(K, (a.Skv - 1) * krow_bytes + dv * 2);
    const int4_t vrsrc = make_rsrc(V, (a.Skv - 1) * vrow_bytes + dv * 2);

    // ---- HBM -> LDS mapping.  A wave-wide load moves RPL rows; load n of wave w covers
    // tile rows RPL*NW*n + RPL*w + lane / CHUNKS; the lane fetches the chunk that belongs at
    // position lane % CHUNKS of the swizzled row (the swizzles only see row & 15).
    const int ld_r = RPL * wave + lane / CHUNKS;
    // (a chunk beyond the head size in memory: an offset that stays outside the descriptor whatever tile offset is
    // added to it -- a (batch, head) slice spans less than 2^31 bytes)
    const int k_chunk = (lane % CHUNKS) ^ swizzle_k<D>(ld_r), v_chunk = (lane % CHUNKS) ^ swizzle_v<D>(ld_r);
    const int k_voff = k_chunk * 8 < dv ? ld_r * krow_bytes + k_chunk * 16 : static_cast<int>(0x80000000u);
    const int v_voff = v_chunk * 8 < dv ? ld_r * vrow_bytes + v_chunk * 16 : static_cast<int>(0x80000000u);
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)); // LDS addresses fit 32 bits
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + RPL * wave * ROWB);
    // load n (0 .. NLOAD-1) of this wave's share of a K / V tile
    // (tile: counted from the first tile of this half's key range, tile0 -- set per pass below)
    int tile0 = 0;
    auto load_k1 = [&](int tile, int buf, int n) {
        load_to_lds_16(krsrc, lds_wave + buf * TILEB + n * RPL * NWH * ROWB, k_voff + ((tile0 + tile) * BN + RPL * NWH * n) * krow_bytes);
    };
    auto load_v1 = [&](int tile, int buf, int n) {
        load_to_lds_16(vrsrc, lds_wave + (2 + buf) * TILEB + n * RPL * NWH * ROWB, v_voff + ((tile0 + tile) * BN + RPL * NWH * n) * vrow_bytes);
    };
    auto load_k = [&](int tile, int buf) {
#pragma unroll
        for (int n = 0; n < NLOAD; ++n) load_k1(tile, buf, n);
    };
    auto load_v = [&](int tile, int buf) {
#pragma unroll
        for (int n = 0; n < NLOAD; ++n) load_v1(tile, buf, n);
    };

    // ---- LDS fragment offsets (bytes)
    int k_off[KT]; // K fragment of k-step t: row ql (+32 per sub-tile), chunk 2t+g
#pragma unroll
    for (int t = 0; t < KT; ++t) k_off[t] = ql * ROWB + (((2 * t + g) ^ swizzle_k<D>(ql)) * 16);
    int v_off[2][DT]; // V transpose read: rows g*4 + s2 (+8), dims dt*32 + (lane & 31)
    {
        const int s2 = (lane & 15) >> 2, cl = ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1), half = lane & 1;
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int row = g * 4 + s2 + 8 * hi;
                v_off[hi][dt] = row * ROWB + (((dt * 4 + cl) ^ swizzle_v<D>(row)) * 16) + half * 8;
            }
    }

    for (int pass = 0; pass < npass; ++pass) {
        // heavier block of the pair first
        const int qb = a.causal ? (pass == 0 ? nqb - 1 - slot : slot) : slot;
        const int q0 = qb * BMW;
        const int qw0 = q0 + wave * 32; // first query row of this wave
        const int q = qw0 + ql;
        const bool q_ok = q < a.Sq;

        // Q fragments, pre-multiplied by scale * log2(e) (rounded back to the 16-bit type): the
        // score MFMAs then deliver base-2 logits directly
        uint4_t qf[KT];
    #pragma unroll
        for (int t = 0; t < KT; ++t) {
            qf[t] = uint4_t{0, 0, 0, 0};
            if (q_ok && 16 * t + 8 * g < dv) qf[t] = *reinterpret_cast<const uint4_t *>(Q + static_cast<int64_t>(q) * a.qs[2] + 16 * t + 8 * g);
    #pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t w = qf[t][c];
                const float lo = BF16 ? bf16_bits_to_f32(w & 0xFFFFu) : f16_bits_to_f32(w & 0xFFFFu);
                const float hi = BF16 ? bf16_bits_to_f32(w >> 16) : f16_bits_to_f32(w >> 16);
                qf[t][c] = pack2<BF16>(lo * a.scale_log2e, hi * a.scale_log2e);
            }
        }

        float16_t oacc[DT];
    #pragma unroll
        for (int dt = 0; dt < DT; ++dt)
    #pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.0f;
        float m_run = NEG_INF_F, l_run = 0.0f;

        int kv_end = a.Skv;
        if (a.causal) kv_end = min(a.Skv, q0 + BMW);
        const int ntiles_all = (kv_end + BN - 1) / BN; // >= 1
        // key split: the first half takes the larger share; `nsteps` is what the work-group's barriers are counted by
        const int nsteps = SPLIT == 1 ? ntiles_all : (ntiles_all + 1) / 2;
        const int ntiles = SPLIT == 1 ? ntiles_all : part == 0 ? nsteps : ntiles_all - nsteps; // >= 1 (the launcher sees to two tiles)
        tile0 = SPLIT == 1 ? 0 : part * nsteps;

        // v_maximum3_f32: NaN-propagating maximum, which (unlike maxnum) needs no input canonicalisation
        auto max3 = [](float x, float y, float z) { return __builtin_elementwise_maximum(__builtin_elementwise_maximum(x, y), z); };
        // exchange between the two half-waves that share a query column
        auto max_across_halves = [&](float x) {
            const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
            return __builtin_elementwise_maximum(__uint_as_float(r[0]), __uint_as_float(r[1]));
        };
        // row maximum of a score tile, as four short chains instead of one long one
        auto row_max = [&](const float16_t (&s)[2]) {
            float m0 = max3(s[0][0], s[0][1], s[0][2]), m1 = max3(s[0][8], s[0][9], s[0][10]);
            float m2 = max3(s[1][0], s[1][1], s[1][2]), m3 = max3(s[1][8], s[1][9], s[1][10]);
            m0 = max3(m0, s[0][3], s[0][4]); m1 = max3(m1, s[0][11], s[0][12]);
            m2 = max3(m2, s[1][3], s[1][4]); m3 = max3(m3, s[1][11], s[1][12]);
            m0 = max3(m0, s[0][5], s[0][6]); m1 = max3(m1, s[0][13], s[0][14]);
            m2 = max3(m2, s[1][5], s[1][6]); m3 = max3(m3, s[1][13], s[1][14]);
            m0 = max3(m0, s[0][7], m1); m2 = max3(m2, s[1][7], m3);
            return max_across_halves(max3(m0, s[0][15], __builtin_elementwise_maximum(m2, s[1][15])));
        };

        // initial value of the score accumulators of tile `tile`: `base`, or -inf where the mask words (already in
        // mk) say so
        auto init_scores = [&](int tile, float base, float16_t (&s)[2]) {
            const bool use_words = HAS_MASK && mask_words && (tile0 + tile) * BN + BN <= a.Skv;
    #pragma unroll
            for (int kt = 0; kt < 2; ++kt)
    #pragma unroll
                for (int i = 0; i < 16; ++i) {
                    bool dead = false;
                    if constexpr (HAS_MASK) dead = use_words && ((mk[kt * 4 + i / 4] >> (8 * (i % 4))) & 0xFFu) != 0;
                    s[kt][i] = dead ? NEG_INF_F : base;
                }
        };

        // S^T = K Q^T for one tile (two 32-key sub-tiles); prologue only
        auto scores = [&](const unsigned char *Kb, float16_t (&s)[2]) {
            init_scores(0, 0.0f, s);
    #pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
    #pragma unroll
                for (int t = 0; t < KT; ++t) {
                    const uint4_t kf = *reinterpret_cast<const uint4_t *>(Kb + kt * 32 * ROWB + k_off[t]);
                    s[kt] = mfma_32x32x16<BF16>(kf, qf[t], s[kt]);
                }
            }
        };

        // the mask words of this lane's keys of one tile: bytes 32 kt + 8 i4 + 4 g .. + 3 of the tile's 64, kt < 2, i4 < 4
        auto load_mask_words = [&](int tile) {
            if constexpr (HAS_MASK) {
                const int kvb = (tile0 + tile) * BN;
                if (mask_words && q_ok && kvb + BN <= a.Skv) {
                    const uint32_t *row = reinterpret_cast<const uint32_t *>(M + static_cast<int64_t>(q) * a.Skv + kvb + 4 * g);
    #pragma unroll
                    for (int w8 = 0; w8 < 8; ++w8) mk[w8] = row[(w8 / 4) * 8 + (w8 % 4) * 2];
                }
            }
        };

        // Key masking of tile j (diagonal, key tail, explicit mask), then the row maximum.
        auto mask_and_max = [&](int kv0, float16_t (&s)[2]) {
            const int kv_limit = a.causal ? min(a.Skv - 1, q) : a.Skv - 1;
    #pragma unroll
            for (int kt = 0; kt < 2; ++kt)
    #pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int kv = kv0 + kt * 32 + (i / 4) * 8 + g * 4 + (i % 4);
                    bool dead = kv > kv_limit;
                    if constexpr (HAS_MASK) {
                        if (!(mask_words && kv0 + BN <= a.Skv) && q_ok && kv < a.Skv) dead = dead || M[static_cast<int64_t>(q) * a.Skv + kv] != 0;
                    }
                    if (dead) s[kt][i] = NEG_INF_F;
                }
            return row_max(s);
        };

        // Running maximum and the (rare) rescale of the accumulators.  The score accumulators of a
        // tile start at MINUS the reference maximum that was current when its MFMAs were issued, so
        // `cur` already holds logit - reference and the exponentials need no subtraction; mloc is
        // the tile's row maximum in that relative form.  When the reference moves, the accumulators
        // are rescaled and the tile re-referenced.
        auto update_max = [&](float mloc, float16_t (&cur)[2]) {
            const float ref = m_run == NEG_INF_F ? 0.0f : m_run;
            const float m_new = __builtin_elementwise_maximum(m_run, mloc + ref);
            if (__builtin_amdgcn_ballot_w64(m_new - m_run > RESCALE_THRESHOLD) != 0) {
                const float alpha = m_new == NEG_INF_F ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
                const float delta = (m_new == NEG_INF_F ? 0.0f : m_new) - ref;
                m_run = m_new;
                l_run *= alpha;
    #pragma unroll
                for (int dt = 0; dt < DT; ++dt)
    #pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
    #pragma unroll
                for (int kt = 0; kt < 2; ++kt)
    #pragma unroll
                    for (int i = 0; i < 16; ++i) cur[kt][i] -= delta;
            }
        };

        // The fused step body, hand-scheduled in NS + NP slots, one MFMA each (D = 128: 16 + 16, D = 64: 8 + 8):
        //   slots  0..NS-1      score MFMAs of the NEXT tile (K fragments from Kn)
        //   slots NS..NS+NP-1   O^T += V^T P^T of the CURRENT tile (V fragments from Vb)
        // LDS fragment reads run PF slots ahead of their MFMA.  The VALU work of the current
        // tile's softmax (exp2, pack, row sum: 16 pairs) is dealt out over the score slots (D = 128: one pair in
        // 12 of them and in the first four PV slots; D = 64: two pairs in each), always ahead of the P fragment
        // that the PV MFMAs need; the row maximum of the next tile is spread over PV slots.  A scheduling
        // barrier closes every slot so the compiler keeps this order.
        auto fused = [&](int j, const unsigned char *Kn, const unsigned char *Vb, const float16_t (&cur)[2], float16_t (&nxt)[2], float &mx_next) {
            const bool want_k = j + 2 < ntiles, want_v = j + 1 < ntiles;
            constexpr int PF = 3, RING = 4;
            const float m_use = m_run == NEG_INF_F ? 0.0f : m_run;
            uint4_t fr[RING];
            uint32_t w[16];
            float pm[4];
            constexpr int NS = 2 * KT, NP = 4 * DT;
            auto read_frag = [&](int m) {
                if (m < NS) {
                    fr[m % RING] = *reinterpret_cast<const uint4_t *>(Kn + (m / KT) * 32 * ROWB + k_off[m % KT]);
                } else {
                    const int ks = (m - NS) / DT, dt = (m - NS) % DT;
                    const uint2_t lo = lds_read_tr16(reinterpret_cast<const uint16_t *>(Vb + ks * 16 * ROWB + v_off[0][dt]));
                    const uint2_t hi = lds_read_tr16(reinterpret_cast<const uint16_t *>(Vb + ks * 16 * ROWB + v_off[1][dt]));
                    fr[m % RING] = uint4_t{lo.x, lo.y, hi.x, hi.y};
                }
            };
            auto exp_pair = [&](int pr) { // elements 2*pr, 2*pr+1 of the current tile
                const int kt = pr / 8, i = (pr % 8) * 2;
                const float p0 = __builtin_amdgcn_exp2f(cur[kt][i]);
                const float p1 = __builtin_amdgcn_exp2f(cur[kt][i + 1]);
                w[pr] = pack2<BF16>(p0, p1);
                l_run = add_pair<BF16>(w[pr], l_run);
            };
    #pragma unroll
            for (int m = 0; m < PF; ++m) read_frag(m);
    #pragma unroll
            for (int m = 0; m < NS + NP; ++m) {
                if (m + PF < NS + NP) read_frag(m + PF);
                if (m < NS) {
                    if constexpr (HAS_MASK) {
                        if (m == 0) { // both sub-tiles at once: the mask words are then free for the tile after
                            init_scores(j + 1, -m_use, nxt);
                            if (j + 2 < ntiles) load_mask_words(j + 2);
                        }
                    } else if (m % KT == 0) {
    #pragma unroll
                        for (int i = 0; i < 16; ++i) nxt[m / KT][i] = -m_use; // logits come out relative to the reference
                    }
                    nxt[m / KT] = mfma_32x32x16<BF16>(fr[m % RING], qf[m % KT], nxt[m / KT]);
                    if constexpr (D == 128) {
                        if (m % 4 != 3) exp_pair((m / 4) * 3 + m % 4);
                    } else {
                        exp_pair(2 * m);
                        exp_pair(2 * m + 1);
                    }
                } else {
                    const int idx = m - NS, ks = idx / DT, dt = idx % DT;
                    const uint4_t pf = {w[4 * ks], w[4 * ks + 1], w[4 * ks + 2], w[4 * ks + 3]};
                    oacc[dt] = mfma_32x32x16<BF16>(fr[m % RING], pf, oacc[dt]);
                    constexpr int MAX0 = D == 128 ? 4 : 0; // first PV slot that works on the next tile's maximum
                    if (D == 128 && idx < 4) exp_pair(12 + idx);
                    if (idx >= MAX0 && idx < MAX0 + 8) { // two partial maxima per slot over the next tile's 32 scores
                        const int c = idx - MAX0, kt = c / 4, i0 = (c % 4) * 4;
                        if (c % 4 < 2) {
                            pm[kt * 2 + c % 4] = max3(max3(nxt[kt][i0], nxt[kt][i0 + 1], nxt[kt][i0 + 2]), nxt[kt][i0 + 3], NEG_INF_F);
                        } else {
                            pm[kt * 2 + c % 4 - 2] = max3(max3(pm[kt * 2 + c % 4 - 2], nxt[kt][i0], nxt[kt][i0 + 1]), nxt[kt][i0 + 2], nxt[kt][i0 + 3]);
                        }
                    }
                    if (idx == (D == 128 ? MAX0 + 8 : MAX0 + 7)) mx_next = max_across_halves(max3(max3(pm[0], pm[1], pm[2]), pm[3], NEG_INF_F));
                }
                // the tile prefetch is spread over the slots instead of bursting at the step start:
                // K(j+2) in slots 1, 3, .., V(j+1) in slots 2, 4, ..
                if (m % 2 == 1 && m / 2 < NLOAD) {
                    if (want_k) load_k1(j + 2, j & 1, m / 2);
                } else if (m % 2 == 0 && m >= 2 && m / 2 - 1 < NLOAD) {
                    if (want_v) load_v1(j + 1, (j + 1) & 1, m / 2 - 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        // ---- prologue: K(0), V(0), K(1) in flight; first score tile
        load_mask_words(0);
        load_k(0, 0);
        load_v(0, 0);
        if (ntiles > 1) load_k(1, 1);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): Q fragments and this wave's share of the tiles
        __syncthreads();
        float16_t sA[2], sB[2];
        scores(lds, sA);
        if (ntiles > 1) load_mask_words(1); // for the scores of tile 1, issued in step 0
        float mxA = row_max(sA), mxB = NEG_INF_F; // unmasked row maxima, valid when the tile needs no masking
        __syncthreads(); // every wave is done with K buffer 0 before K(2) lands in it

        // One pipeline step: tile j is in `cur` (scores already computed), tile j+1's scores go to `nxt`.
        auto step = [&](int j, float16_t (&cur)[2], float mx_cur, float16_t (&nxt)[2], float &mx_nxt) {
            const int kv0 = (tile0 + j) * BN;
            const bool active = !(a.causal && kv0 > qw0 + 31) && (SPLIT == 1 || j < ntiles);
            const unsigned char *Vb = lds + (2 + (j & 1)) * TILEB;
            const unsigned char *Kn = lds + ((j + 1) & 1) * TILEB;
            if (active) {
                const bool need_mask = (a.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > a.Skv) || (HAS_MASK && !mask_words);
                float mloc = mx_cur;
                if (need_mask) mloc = mask_and_max(kv0, cur);
                update_max(mloc, cur);
                // The next tile's scores are issued unconditionally so that they share a basic
                // block with this tile's softmax; after the last tile (or the last one this wave
                // needs) they come from a stale K buffer and are never used: ~1.5 % extra MFMAs.
                fused(j, Kn, Vb, cur, nxt, mx_nxt);
            } else { // a wave with nothing to compute still fetches its share of the tiles
                if (j + 2 < ntiles) load_k(j + 2, j & 1);
                if (j + 1 < ntiles) load_v(j + 1, (j + 1) & 1);
            }
            __builtin_amdgcn_s_waitcnt(0x0F70); // this wave's async loads have landed
            __syncthreads();
        };
        for (int j = 0; j < nsteps; j += 2) {
            step(j, sA, mxA, sB, mxB);
            if (j + 1 < nsteps) step(j + 1, sB, mxB, sA, mxA);
        }

        if constexpr (SPLIT == 2) {
            // The second half's state goes to the first through LDS (the tile buffers are free: every step ends in a
            // barrier), value-major so that the 64 lanes of a wave touch consecutive words.  Both halves hold sums of
            // 2^(logit - reference) with a reference of their own: brought to the larger one and added.
            float *xch = reinterpret_cast<float *>(lds_all) + wave * (DT * 16 + 2) * WAVE + lane;
            if (part == 1) {
    #pragma unroll
                for (int dt = 0; dt < DT; ++dt)
    #pragma unroll
                    for (int i = 0; i < 16; ++i) xch[(dt * 16 + i) * WAVE] = oacc[dt][i];
                xch[DT * 16 * WAVE] = m_run;
                xch[(DT * 16 + 1) * WAVE] = l_run;
            }
            __syncthreads();
            if (part == 1) return; // (one pass: no causal mask)
            const float m_other = xch[DT * 16 * WAVE], l_other = xch[(DT * 16 + 1) * WAVE];
            const float m_new = __builtin_elementwise_maximum(m_run, m_other);
            const float a_mine = m_run == NEG_INF_F ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            const float a_other = m_other == NEG_INF_F ? 0.0f : __builtin_amdgcn_exp2f(m_other - m_new);
            l_run = l_run * a_mine + l_other * a_other;
    #pragma unroll
            for (int dt = 0; dt < DT; ++dt)
    #pragma unroll
                for (int i = 0; i < 16; ++i) oacc[dt][i] = oacc[dt][i] * a_mine + xch[(dt * 16 + i) * WAVE] * a_other;
        }

        const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        if (q_ok) {
            uint16_t *orow = O + static_cast<int64_t>(q) * a.os[2];
    #pragma unroll
            for (int dt = 0; dt < DT; ++dt)
    #pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const int d = dt * 32 + i4 * 8 + g * 4;
                    uint2_t w = {pack2<BF16>(oacc[dt][4 * i4] * inv, oacc[dt][4 * i4 + 1] * inv),
                                 pack2<BF16>(oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv)};
                    if (d < dv) *reinterpret_cast<uint2_t *>(orow + d) = w;
                }
        }
    }
}

// ------------------------------------------ ping-pong MFMA kernel, head_dim 128
// The pipelined kernel above lets both waves of a SIMD run the same mix of matrix and vector instructions at the same
// time: the older wave wins every arbitration, finishes its step early and the younger one trails behind it.  Here
// the eight waves of a work-group form two groups (waves 0-3 and 4-7: one wave of each group per SIMD) that run HALF A
// STEP APART.  Between two work-group barriers (one per 64-key tile)
//     group 0 issues the 2 * (KT + 2 DT) MFMAs of a step back to back -- O^T += V^T P^T of tile j and S^T = K Q^T of
//             tile j+1, alternating, fragments from LDS -- and then runs the softmax of tile j+1 on the VALU,
//     group 1 runs the softmax of tile j first and the same MFMAs after it,
// so a SIMD always has one wave in its matrix phase and one in its vector phase.  Measured against the pipelined
// kernel, back to back on one box (bf16 B4 H32 S4096 D128): causal 981 -> 1060 TFLOP/s, non-causal 1111 -> 1188.
// What else differs:
//  * row sums are fp32 adds of the exponentials.  v_dot2c_f32_bf16 (the pipelined kernel's choice) waits for the
//    matrix pipe: next to MFMAs every one of them costs about 18 cycles.
//  * the score accumulators of a tile exist once (the softmax of tile j ends before the MFMAs of tile j+1 start in
//    the same wave), which leaves registers for everything else without spills.
//  * a work-group is persistent: it walks the units blockIdx.x, blockIdx.x + gridDim.x, ... and requests the first K
//    and V tiles of the next segment (the second query block of a causal pair, or the next unit) during the last two
//    steps of the one at hand, so a segment does not start with an empty pipeline.
//  * the output is written as 16 bytes per lane after one exchange between the half-waves.
// No explicit mask and exact head sizes only (the pipelined kernel keeps those cases).
template <bool BF16, int D>
__global__ __launch_bounds__(512, 1) void sdpa_mfma_pingpong_kernel(const SdpaArgs a) {
    static_assert(D == 128, "tuned and tested for head_dim 128 (the index arithmetic also holds for 64)");
    constexpr int NW = 8, PF = 3; // PF: LDS fragment reads run this many MFMAs ahead
    constexpr int KT = D / 16, DT = D / 32, BMW = 32 * NW, ROWB = 2 * D, CHUNKS = ROWB / 16, RPL = 64 / CHUNKS;
    constexpr int NLOAD = BN / (RPL * NW), TILEB = BN * ROWB;
    constexpr int NM = D / 4; // MFMAs of a step: D / 8 for the scores of the next tile, D / 8 for the output of this one
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * TILEB]; // K0 K1 V0 V1

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int grp = wave >> 2;
    const int ql = lane % 32, g = lane / 32;

    const int BH = a.B * a.H;
    const int nqb = (a.Sq + BMW - 1) / BMW;
    const int per_bh = a.causal ? (nqb + 1) / 2 : nqb;
    const int n_wg = per_bh * BH; // units of work: a (batch, head) and a query block (a pair of them under a causal mask)
    const int krow_bytes = static_cast<int>(a.ks[2]) * 2, vrow_bytes = static_cast<int>(a.vs[2]) * 2;
    // A work-group walks the units blockIdx.x, blockIdx.x + gridDim.x, ... (units are dealt to the 8 XCDs round-robin by
    // id, and gridDim.x is a multiple of 8: one (batch, head) stays on one XCD); a unit is one or two segments (passes).
    struct Segment { int bh, qb, ntiles; };
    auto segment_of = [&](int L, int pass) {
        int bh, slot;
        if (BH % 8 == 0) {
            const int xcd = L % 8, j = L / 8;
            bh = (j / per_bh) * 8 + xcd;
            slot = j % per_bh;
        } else {
            bh = L / per_bh;
            slot = L % per_bh;
        }
        const int qb = a.causal ? (pass == 0 ? nqb - 1 - slot : slot) : slot;
        int kv_end = a.Skv;
        if (a.causal) kv_end = min(a.Skv, qb * BMW + BMW);
        return Segment{bh, qb, (kv_end + BN - 1) / BN};
    };
    auto passes_of = [&](int L) {
        const int slot = BH % 8 == 0 ? (L / 8) % per_bh : L % per_bh;
        return (a.causal && slot != nqb - 1 - slot) ? 2 : 1;
    };
    auto k_rsrc_of = [&](int bh) { return make_rsrc(static_cast<const uint16_t *>(a.k) + (bh / a.H) * a.ks[0] + (bh % a.H) * a.ks[1], (a.Skv - 1) * krow_bytes + D * 2); };
    auto v_rsrc_of = [&](int bh) { return make_rsrc(static_cast<const uint16_t *>(a.v) + (bh / a.H) * a.vs[0] + (bh % a.H) * a.vs[1], (a.Skv - 1) * vrow_bytes + D * 2); };

    const int ld_r = RPL * wave + lane / CHUNKS;
    const int k_chunk = (lane % CHUNKS) ^ swizzle_k<D>(ld_r), v_chunk = (lane % CHUNKS) ^ swizzle_v<D>(ld_r);
    const int k_voff = ld_r * krow_bytes + k_chunk * 16;
    const int v_voff = ld_r * vrow_bytes + v_chunk * 16;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + RPL * wave * ROWB);
    auto load_k = [&](const int4_t &krsrc, int tile, int buf) {
#pragma unroll
        for (int n = 0; n < NLOAD; ++n)
            load_to_lds_16(krsrc, lds_wave + buf * TILEB + n * RPL * NW * ROWB, k_voff + (tile * BN + RPL * NW * n) * krow_bytes);
    };
    auto load_v = [&](const int4_t &vrsrc, int tile, int buf) {
#pragma unroll
        for (int n = 0; n < NLOAD; ++n)
            load_to_lds_16(vrsrc, lds_wave + (2 + buf) * TILEB + n * RPL * NW * ROWB, v_voff + (tile * BN + RPL * NW * n) * vrow_bytes);
    };

    int k_off[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) k_off[t] = ql * ROWB + (((2 * t + g) ^ swizzle_k<D>(ql)) * 16);
    int v_off[2][DT];
    {
        const int s2 = (lane & 15) >> 2, cl = ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1), half = lane & 1;
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int row = g * 4 + s2 + 8 * hi;
                v_off[hi][dt] = row * ROWB + (((dt * 4 + cl) ^ swizzle_v<D>(row)) * 16) + half * 8;
            }
    }
    uint32_t touch = 0; // destination of the load that pulls the next segment's query rows into L2
    // work-group barrier without a memory fence of its own: tile loads are waited for explicitly, LDS fragment reads
    // have been consumed by the MFMAs in front of it
    auto bar = [] { asm volatile("s_barrier" ::: "memory"); };
    auto wait_tiles = [&] { __builtin_amdgcn_s_waitcnt(0x0F70); asm volatile("" :: "v"(touch)); }; // vmcnt(0) (and the touch register stays reserved until here)

    bool prefetched = false; // the first tiles of the segment at hand were requested during the previous one
    for (int L = blockIdx.x; L < n_wg; L += gridDim.x) {
    const int npass = passes_of(L);
    for (int pass = 0; pass < npass; ++pass) {
        const Segment seg = segment_of(L, pass);
        const int b = seg.bh / a.H, h = seg.bh % a.H;
        const uint16_t *Q = static_cast<const uint16_t *>(a.q) + b * a.qs[0] + h * a.qs[1];
        uint16_t *O = static_cast<uint16_t *>(a.o) + b * a.os[0] + h * a.os[1];
        const int4_t krsrc = k_rsrc_of(seg.bh), vrsrc = v_rsrc_of(seg.bh);
        // the segment after this one: its first K and V tiles are requested in this segment's last two steps
        const bool has_next = pass + 1 < npass || L + static_cast<int>(gridDim.x) < n_wg;
        const Segment nxt = has_next ? (pass + 1 < npass ? segment_of(L, pass + 1) : segment_of(L + gridDim.x, 0)) : seg;
        const int4_t krsrc_n = k_rsrc_of(nxt.bh), vrsrc_n = v_rsrc_of(nxt.bh);
        const int qb = seg.qb;
        const int q0 = qb * BMW;
        const int qw0 = q0 + wave * 32;
        const int q = qw0 + ql;
        const bool q_ok = q < a.Sq;
        const int ntiles = seg.ntiles; // >= 1
        const bool pf_next = has_next && ntiles % 2 == 0; // (an even count keeps tile t of the next segment in buffer t & 1)

        uint4_t qf[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            qf[t] = uint4_t{0, 0, 0, 0};
            if (q_ok) qf[t] = *reinterpret_cast<const uint4_t *>(Q + static_cast<int64_t>(q) * a.qs[2] + 16 * t + 8 * g);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t w = qf[t][c];
                const float lo = BF16 ? bf16_bits_to_f32(w & 0xFFFFu) : f16_bits_to_f32(w & 0xFFFFu);
                const float hi = BF16 ? bf16_bits_to_f32(w >> 16) : f16_bits_to_f32(w >> 16);
                qf[t][c] = pack2<BF16>(lo * a.scale_log2e, hi * a.scale_log2e);
            }
        }

        float16_t oacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.0f;
        float m_run = NEG_INF_F, l_run = 0.0f, l_run1 = 0.0f;

        auto max3 = [](float x, float y, float z) { return __builtin_elementwise_maximum(__builtin_elementwise_maximum(x, y), z); };
        auto max_across_halves = [&](float x) {
            const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
            return __builtin_elementwise_maximum(__uint_as_float(r[0]), __uint_as_float(r[1]));
        };
        auto row_max = [&](const float16_t (&s)[2]) {
            float m0 = max3(s[0][0], s[0][1], s[0][2]), m1 = max3(s[0][8], s[0][9], s[0][10]);
            float m2 = max3(s[1][0], s[1][1], s[1][2]), m3 = max3(s[1][8], s[1][9], s[1][10]);
            m0 = max3(m0, s[0][3], s[0][4]); m1 = max3(m1, s[0][11], s[0][12]);
            m2 = max3(m2, s[1][3], s[1][4]); m3 = max3(m3, s[1][11], s[1][12]);
            m0 = max3(m0, s[0][5], s[0][6]); m1 = max3(m1, s[0][13], s[0][14]);
            m2 = max3(m2, s[1][5], s[1][6]); m3 = max3(m3, s[1][13], s[1][14]);
            m0 = max3(m0, s[0][7], m1); m2 = max3(m2, s[1][7], m3);
            return max_across_halves(max3(m0, s[0][15], __builtin_elementwise_maximum(m2, s[1][15])));
        };
        auto mask_and_max = [&](int kv0, float16_t (&s)[2]) {
            const int kv_limit = a.causal ? min(a.Skv - 1, q) : a.Skv - 1;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int kv = kv0 + kt * 32 + (i / 4) * 8 + g * 4 + (i % 4);
                    if (kv > kv_limit) s[kt][i] = NEG_INF_F;
                }
            return row_max(s);
        };
        auto update_max = [&](float mloc, float16_t (&cur)[2]) {
            const float ref = m_run == NEG_INF_F ? 0.0f : m_run;
            const float m_new = __builtin_elementwise_maximum(m_run, mloc + ref);
            if (__builtin_amdgcn_ballot_w64(m_new - m_run > RESCALE_THRESHOLD) != 0) {
                const float alpha = m_new == NEG_INF_F ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
                const float ref_new = m_new == NEG_INF_F ? 0.0f : m_new;
                const float delta = ref_new - ref;
                m_run = m_new;
                l_run *= alpha;
                l_run1 *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) cur[kt][i] -= delta;
            }
        };

        float16_t s[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.0f;
        uint32_t w[16];

        // softmax of the tile in s (scores relative to the reference): masks, row maximum, rescale, P = 2^s packed to w
        auto softmax_phase = [&](int j) {
            const int kv0 = j * BN;
            const bool need_mask = (a.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > a.Skv);
            const float mloc = need_mask ? mask_and_max(kv0, s) : row_max(s);
            update_max(mloc, s);
#pragma unroll
            for (int pr = 0; pr < 16; ++pr) {
                const int kt = pr / 8, i = (pr % 8) * 2;
                const float p0 = __builtin_amdgcn_exp2f(s[kt][i]);
                const float p1 = __builtin_amdgcn_exp2f(s[kt][i + 1]);
                w[pr] = pack2<BF16>(p0, p1);
                l_run += p0; // (v_dot2c waits for the matrix pipe: 18 cycles each next to MFMAs)
                l_run1 += p1;
            }
            // the next tile's scores start from minus the reference: its logits come out relative to it
            const float m_use = m_run == NEG_INF_F ? 0.0f : m_run;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[kt][i] = -m_use;
        };
        // the NM MFMAs of a step: O^T += V^T P^T of tile j (P in w, V fragments from Vb) and S^T = K Q^T of tile j+1
        // (K fragments from Kn) alternate, so consecutive MFMAs never share an accumulator
        auto mfma_phase = [&](const unsigned char *Kn, const unsigned char *Vb) {
            constexpr int RING = PF + 1;
            uint4_t fr[RING];
            // slot m: even -> score MFMA (m / 2): sub-tile kt = (m/2) & 1, k-step t = (m/2) >> 1; odd -> PV MFMA (m / 2): ks = idx / DT, dt = idx % DT
            auto read_frag = [&](int m) {
                const int idx = m / 2;
                if (m % 2 == 0) {
                    fr[m % RING] = *reinterpret_cast<const uint4_t *>(Kn + (idx & 1) * 32 * ROWB + k_off[idx >> 1]);
                } else {
                    const int ks = idx / DT, dt = idx % DT;
                    const uint2_t lo = lds_read_tr16(reinterpret_cast<const uint16_t *>(Vb + ks * 16 * ROWB + v_off[0][dt]));
                    const uint2_t hi = lds_read_tr16(reinterpret_cast<const uint16_t *>(Vb + ks * 16 * ROWB + v_off[1][dt]));
                    fr[m % RING] = uint4_t{lo.x, lo.y, hi.x, hi.y};
                }
            };
#pragma unroll
            for (int m = 0; m < PF; ++m) read_frag(m);
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                if (m + PF < NM) read_frag(m + PF);
                const int idx = m / 2;
                if (m % 2 == 0) {
                    const int kt = idx & 1, t = idx >> 1;
                    s[kt] = mfma_32x32x16<BF16>(fr[m % RING], qf[t], s[kt]);
                } else {
                    const int ks = idx / DT, dt = idx % DT;
                    const uint4_t pf = {w[4 * ks], w[4 * ks + 1], w[4 * ks + 2], w[4 * ks + 3]};
                    oacc[dt] = mfma_32x32x16<BF16>(fr[m % RING], pf, oacc[dt]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        // ---- prologue: K(0), V(0), K(1); every wave computes the scores of tile 0
        if (!prefetched) {
            load_k(krsrc, 0, 0);
            load_v(vrsrc, 0, 0);
            if (ntiles > 1) load_k(krsrc, 1, 1);
        }
        wait_tiles();
        bar();
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (int t = 0; t < KT; ++t) {
                const uint4_t kf = *reinterpret_cast<const uint4_t *>(lds + kt * 32 * ROWB + k_off[t]);
                s[kt] = mfma_32x32x16<BF16>(kf, qf[t], s[kt]);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): K buffer 0 is read

        auto request = [&](int j, auto par) { // K(j+2) into the buffer of K(j), V(j+1) into the buffer of V(j-1)
            constexpr int PAR = decltype(par)::value;
            if (j + 2 < ntiles) load_k(krsrc, j + 2, PAR);
            else if (pf_next && j + 2 - ntiles < nxt.ntiles) load_k(krsrc_n, j + 2 - ntiles, PAR);
            if (j + 1 < ntiles) load_v(vrsrc, j + 1, 1 - PAR);
            else if (pf_next) load_v(vrsrc_n, 0, 1 - PAR);
        };
        auto active_at = [&](int j) { return !(a.causal && j * BN > qw0 + 31); };
        // One interval per tile, one barrier each: group 0 runs MFMAs(j+1) then softmax(j+1), group 1 softmax(j) then
        // MFMAs(j+1) -- the two waves of a SIMD are always in opposite phases.  PAR = j & 1 picks the tile buffers.
        auto interval0 = [&](int j, auto par) {
            constexpr int PAR = decltype(par)::value;
            wait_tiles();
            bar();
            request(j, par);
            if (active_at(j)) mfma_phase(lds + (1 - PAR) * TILEB, lds + (2 + PAR) * TILEB);
            if (j + 1 < ntiles && active_at(j + 1)) softmax_phase(j + 1);
        };
        auto interval1 = [&](int j, auto par) {
            constexpr int PAR = decltype(par)::value;
            wait_tiles();
            bar();
            request(j, par);
            if (active_at(j)) {
                softmax_phase(j);
                mfma_phase(lds + (1 - PAR) * TILEB, lds + (2 + PAR) * TILEB);
            }
        };
        if (grp == 0) {
            softmax_phase(0);
            for (int j = 0; j < ntiles; j += 2) {
                interval0(j, std::integral_constant<int, 0>{});
                if (j + 1 < ntiles) interval0(j + 1, std::integral_constant<int, 1>{});
            }
        } else {
            for (int j = 0; j < ntiles; j += 2) {
                interval1(j, std::integral_constant<int, 0>{});
                if (j + 1 < ntiles) interval1(j + 1, std::integral_constant<int, 1>{});
            }
        }
        if (!pf_next) bar(); // every wave is done with the tile buffers (nothing is written to them before the next segment's first barrier otherwise)
        prefetched = pf_next;

        l_run += l_run1;
        const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        // A lane holds 4 consecutive dims per (dt, i4); the half-waves trade every second group so that each lane
        // stores 8 consecutive dims (16 bytes): lanes 0-31 the even groups, lanes 32-63 the odd ones
        {
            uint16_t *orow = O + static_cast<int64_t>(q) * a.os[2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int ip = 0; ip < 2; ++ip) {
                    const int ia = 8 * ip, ib = 8 * ip + 4; // accumulator elements of groups i4 = 2 ip and 2 ip + 1
                    const uint32_t x0 = pack2<BF16>(oacc[dt][ia] * inv, oacc[dt][ia + 1] * inv), x1 = pack2<BF16>(oacc[dt][ia + 2] * inv, oacc[dt][ia + 3] * inv);
                    const uint32_t y0 = pack2<BF16>(oacc[dt][ib] * inv, oacc[dt][ib + 1] * inv), y1 = pack2<BF16>(oacc[dt][ib + 2] * inv, oacc[dt][ib + 3] * inv);
                    // after the exchange lanes 0-31 hold (own group 2 ip, partner's group 2 ip), lanes 32-63 (partner's group 2 ip + 1, own group 2 ip + 1)
                    const auto r0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
                    const auto r1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
                    const uint4_t wv = {r0[0], r1[0], r0[1], r1[1]};
                    const int d = dt * 32 + (2 * ip + g) * 8;
                    if (q_ok) *reinterpret_cast<uint4_t *>(orow + d) = wv;
                }
        }
    }
    }
}

// ------------------------------------------------------------- fp32 MFMA kernel
// fp32 inputs, head_dim 32 / 64 / 128, on v_mfma_f32_32x32x2_f32: fp32 products and fp32 accumulation, so nothing
// is given up against the FMA kernel below, at about ten times its rate.  Same transposed formulation as the 16-bit
// kernels: S^T = K Q^T leaves every lane with one query column and 16 of a sub-tile's 32 keys, and the
// exponentiated scores are, as they sit in the accumulator registers, the B operand (P^T, two keys per MFMA) of
// O^T += V^T P^T -- no conversion and no trip through LDS.  One work-group = 4 waves = 128 query rows; K and V tiles
// of 64 keys are staged through registers into padded LDS rows (K: +4 floats, conflict-free 16-byte fragment reads;
// V: +8 floats, so the two half-waves of a 4-byte read hit disjoint banks), double-buffered.  At 64 cycles per MFMA
// the kernel is bound by the matrix pipe; the softmax in between is a few percent.
template <int D> constexpr int sdpa_f32_lds_bytes() { return 2 * BN * ((D + 4) + (D + 8)) * 4; }

// SPLIT = 1, 2 or 4 waves share one 32-row query block and divide its keys among themselves (32-key sub-tiles in
// turn); their (reference maximum, denominator, O^T) states are merged through LDS at the end.  A wave's MFMAs form
// one dependent chain over its keys, so short problems (few work-groups, e.g. one batch of 8 heads x 512 rows) are
// bound by that chain's length rather than by the chip: splitting the keys shortens it SPLIT-fold.
template <bool HAS_MASK, int D, int SPLIT>
__global__ __launch_bounds__(256) void sdpa_mfma_f32_kernel(const SdpaArgs a) {
    static_assert(SPLIT == 1 || SPLIT == 2 || SPLIT == 4, "waves per query block");
    constexpr int KSTR = D + 4, VSTR = D + 8; // LDS row strides in floats
    constexpr int DT = D / 32;                // 32-row tiles of O^T
    constexpr int QJ = D / 8;                 // 16-byte Q / K fragments per lane
    constexpr int KCH = D / 4;                // 16-byte chunks per K / V row
    constexpr int NLD = BN * KCH / 256;       // chunks per thread per 64-key tile (2, 4, 8)
    constexpr int ROWS_PER_PASS = 256 / KCH;
    constexpr int BMW = 32 * (4 / SPLIT);     // query rows per work-group
    constexpr int TPI = SPLIT == 4 ? 2 : 1;   // 64-key tiles per iteration (one 32-key sub-tile per wave when split)
    constexpr int NSUB = SPLIT == 1 ? 2 : 1;  // sub-tiles a wave multiplies per iteration
    extern __shared__ __attribute__((aligned(16))) float f32_lds[];
    auto Ks = [&](int buf) { return f32_lds + buf * BN * KSTR; };                 // K tile `buf`
    auto Vs = [&](int buf) { return f32_lds + 2 * BN * KSTR + buf * BN * VSTR; }; // V tile `buf`

    const int tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int ql = lane % 32, g = lane / 32;
    const int rb = wave / SPLIT, part = wave % SPLIT; // query block within the work-group, share of its keys

    const int L = blockIdx.x;
    const int BH = a.B * a.H;
    int bh, qb;
    if (BH % 8 == 0) { // one (batch, head) stays on one XCD, whose L2 then holds its K / V
        const int xcd = L % 8, j = L / 8;
        bh = (j / a.nqb) * 8 + xcd;
        qb = j % a.nqb;
    } else {
        bh = L / a.nqb;
        qb = L % a.nqb;
    }
    if (a.causal) qb = a.nqb - 1 - qb; // heaviest blocks first
    const int b = bh / a.H, h = bh % a.H;

    const float *Q = static_cast<const float *>(a.q) + b * a.qs[0] + h * a.qs[1];
    const float *K = static_cast<const float *>(a.k) + b * a.ks[0] + h * a.ks[1];
    const float *V = static_cast<const float *>(a.v) + b * a.vs[0] + h * a.vs[1];
    float *O = static_cast<float *>(a.o) + b * a.os[0] + h * a.os[1];
    const uint8_t *M = HAS_MASK ? a.mask + b * a.ms[0] + h * a.ms[1] : nullptr;

    const int q0 = qb * BMW;
    const int qw0 = q0 + rb * 32;
    const int q = qw0 + ql;
    const bool q_ok = q < a.Sq;

    // K / V through buffer descriptors: rows past the end of the sequence read as zero
    const int krow_bytes = static_cast<int>(a.ks[2]) * 4, vrow_bytes = static_cast<int>(a.vs[2]) * 4;
    // A head size below D (a.D, a multiple of 4) runs with zeros in the missing dims: the lanes that would fetch a
    // chunk beyond it aim past the descriptors' ends (they stage zeros), Q fragments there stay zero, the output keeps
    // a.D columns.
    const int dv = a.D;
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(K), 0, (a.Skv - 1) * krow_bytes + dv * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(V), 0, (a.Skv - 1) * vrow_bytes + dv * 4, 0x00020000);
    const int ld_row = tid / KCH, ld_cc = tid % KCH;
    const bool ld_inside = ld_cc * 4 < dv;
    const int k_voff = ld_inside ? ld_row * krow_bytes + ld_cc * 16 : static_cast<int>(0x80000000u);
    const int v_voff = ld_inside ? ld_row * vrow_bytes + ld_cc * 16 : static_cast<int>(0x80000000u);

    // Q^T fragments (B operand): lane holds Q[q][8 j + 4 g .. + 3]; component c of fragment j meets K's component c
    float4_t qf[QJ];
#pragma unroll
    for (int j = 0; j < QJ; ++j) {
        qf[j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        if (q_ok && 8 * j + 4 * g < dv) qf[j] = *reinterpret_cast<const float4_t *>(Q + static_cast<int64_t>(q) * a.qs[2] + 8 * j + 4 * g);
    }

    float16_t oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.0f;
    float m_run = NEG_INF_F, l_run = 0.0f;

    int kv_end = a.Skv;
    if (a.causal) kv_end = min(a.Skv, q0 + BMW);
    const int nit = (kv_end + TPI * BN - 1) / (TPI * BN); // >= 1

    uint4_t kreg[TPI * NLD], vreg[TPI * NLD];
    auto load_it = [&](int it) {
#pragma unroll
        for (int tt = 0; tt < TPI; ++tt)
#pragma unroll
            for (int n = 0; n < NLD; ++n) {
                const int row0 = (it * TPI + tt) * BN + n * ROWS_PER_PASS;
                kreg[tt * NLD + n] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, k_voff + row0 * krow_bytes, 0, 0);
                vreg[tt * NLD + n] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, v_voff + row0 * vrow_bytes, 0, 0);
            }
    };
    auto stage_tile = [&](int tt, int buf) { // tile tt of the iteration held in registers -> LDS buffer buf
#pragma unroll
        for (int n = 0; n < NLD; ++n) {
            const int row = ld_row + n * ROWS_PER_PASS;
            *reinterpret_cast<uint4_t *>(Ks(buf) + row * KSTR + 4 * ld_cc) = kreg[tt * NLD + n];
            *reinterpret_cast<uint4_t *>(Vs(buf) + row * VSTR + 4 * ld_cc) = vreg[tt * NLD + n];
        }
    };

    const int k_frag = ql * KSTR + 4 * g; // + kt * 32 * KSTR + 8 j
    const int v_frag = 4 * g * VSTR + ql; // + (kt * 32 + 8 (e / 4) + e % 4) * VSTR + 32 dt

    // One iteration's share of this wave: NSUB sub-tiles of 32 keys.  Sub-tile u sits in LDS buffer sub_buf(u, buf)
    // at key offset 32 * sub_kt(u) and starts at key sub_kv(u, it) of the sequence.
    auto sub_kt = [&](int u) { return SPLIT == 1 ? u : part % 2; };
    auto sub_buf = [&](int buf) { return SPLIT == 4 ? part / 2 : buf; };
    auto sub_kv = [&](int u, int it) { return it * TPI * BN + (SPLIT == 4 ? (part / 2) * BN : 0) + 32 * sub_kt(u); };

    // explicit mask: the four 4-byte words per sub-tile that cover this lane's keys (4 runs of 4 consecutive ones).
    // They are requested before the iteration's K / V prefetch is issued and consumed after the score MFMAs.  Loads
    // return in order, so the wait for the words must not cover the prefetch behind them: every vector load of the
    // loop is issued unconditionally (lanes or iterations with nothing to fetch aim past the descriptor's end and
    // read zeros), which lets the wait be an exact count.  Rows must be 4-byte aligned and the sub-tile complete,
    // otherwise single bytes are read after the MFMAs.
    uint32_t mw[NSUB * 4];
    bool words_ok[NSUB];
    const __amdgpu_buffer_rsrc_t mrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(HAS_MASK ? M : nullptr), 0, HAS_MASK ? a.Sq * a.Skv : 0, 0x00020000);
    auto load_mask_words = [&](int it) {
        if constexpr (HAS_MASK) {
#pragma unroll
            for (int u = 0; u < NSUB; ++u) {
                const int kvs = sub_kv(u, it);
                words_ok[u] = a.Skv % 4 == 0 && (reinterpret_cast<uintptr_t>(M) & 3u) == 0 && kvs + 32 <= a.Skv;
                const int row_off = (words_ok[u] && q_ok) ? q * a.Skv + kvs + 4 * g : 0x7FFFFF00;
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) mw[u * 4 + w4] = __builtin_amdgcn_raw_buffer_load_b32(mrsrc, row_off + 8 * w4, 0, 0);
            }
        }
    };

    auto compute = [&](int it, int buf) {
        const int kv_first = sub_kv(0, it);
        if (a.causal && kv_first > qw0 + 31) return; // every key of this wave's share lies past its last query row
        const float *Kb = Ks(sub_buf(buf)), *Vb = Vs(sub_buf(buf));

        // ---- S^T = K Q^T: D / 2 MFMAs of two dims per 32-key sub-tile
        float16_t s[NSUB];
#pragma unroll
        for (int u = 0; u < NSUB; ++u) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[u][i] = 0.0f;
#pragma unroll
            for (int j = 0; j < QJ; ++j) {
                const float4_t kf = *reinterpret_cast<const float4_t *>(&Kb[k_frag + sub_kt(u) * 32 * KSTR + 8 * j]);
#pragma unroll
                for (int c = 0; c < 4; ++c) s[u] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[c], qf[j][c], s[u], 0, 0, 0);
            }
        }

        const int kv_last = sub_kv(NSUB - 1, it) + 31;
        const bool need_mask = (a.causal && kv_last > qw0) || (kv_last >= a.Skv) || HAS_MASK;
        if (need_mask) {
            const int kv_limit = a.causal ? min(a.Skv - 1, q) : a.Skv - 1;
            bool all_words = HAS_MASK;
            if constexpr (HAS_MASK) {
#pragma unroll
                for (int u = 0; u < NSUB; ++u) all_words = all_words && words_ok[u];
            }
            if (!HAS_MASK || all_words) {
                // the usual case, free of branches and loads: selects on values that are already in registers
#pragma unroll
                for (int u = 0; u < NSUB; ++u)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int kv = sub_kv(u, it) + (i / 4) * 8 + g * 4 + (i % 4);
                        bool dead = kv > kv_limit;
                        if constexpr (HAS_MASK) dead = dead || ((mw[u * 4 + i / 4] >> (8 * (i % 4))) & 0xFFu) != 0;
                        s[u][i] = dead ? NEG_INF_F : s[u][i];
                    }
            } else {
                // ragged last sub-tile or unaligned mask rows: byte by byte
#pragma unroll
                for (int u = 0; u < NSUB; ++u)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int kv = sub_kv(u, it) + (i / 4) * 8 + g * 4 + (i % 4);
                        bool dead = kv > kv_limit;
                        if constexpr (HAS_MASK) {
                            if (q_ok && kv < a.Skv) dead = dead || M[static_cast<int64_t>(q) * a.Skv + kv] != 0;
                        }
                        s[u][i] = dead ? NEG_INF_F : s[u][i];
                    }
            }
        }

        // ---- online softmax (per lane: one query column, half of each sub-tile's keys), base-2 domain
        float mloc = NEG_INF_F;
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[u][i]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
        const float m_new = fmaxf(m_run, mloc * a.scale_log2e);
        if (__builtin_amdgcn_ballot_w64(m_new - m_run > RESCALE_THRESHOLD) != 0) {
            const float alpha = m_new == NEG_INF_F ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
        }
        const float m_use = m_run == NEG_INF_F ? 0.0f : m_run;
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float pexp = __builtin_amdgcn_exp2f(__builtin_fmaf(s[u][i], a.scale_log2e, -m_use));
                s[u][i] = pexp;
                l_run += pexp;
            }

        // ---- O^T += V^T P^T: MFMA e of a sub-tile multiplies keys 8 (e / 4) + e % 4 (lower half-wave) and + 4 (upper)
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int e = 0; e < 16; ++e)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const float vf = Vb[v_frag + (sub_kt(u) * 32 + 8 * (e / 4) + e % 4) * VSTR + 32 * dt];
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf, s[u][e], oacc[dt], 0, 0, 0);
                }
    };

    if constexpr (SPLIT < 4) {
        // one tile per iteration, double-buffered: tile it + 1 is parked in the other buffer while tile it is multiplied
        load_it(0);
        stage_tile(0, 0);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        if (nit > 1) load_it(1);
        __syncthreads();
        for (int it = 0; it < nit; ++it) {
            const int buf = it & 1;
            if (it + 1 < nit) stage_tile(0, buf ^ 1);
            load_mask_words(it);
            load_it(it + 2); // past the last tile: zeros, nothing is fetched
            compute(it, buf);
            __syncthreads();
        }
    } else {
        // two tiles per iteration fill both buffers; the next pair waits in registers meanwhile
        load_it(0);
        for (int it = 0; it < nit; ++it) {
            stage_tile(0, 0);
            stage_tile(1, 1);
            load_mask_words(it);
            load_it(it + 1); // past the last tile: zeros, nothing is fetched
            __syncthreads();
            compute(it, 0);
            __syncthreads();
        }
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32, WAVE);
    if constexpr (SPLIT == 1) {
        // ---- epilogue: O = O^T / l, four consecutive dims per store
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        if (q_ok) {
            float *orow = O + static_cast<int64_t>(q) * a.os[2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    const float4_t w = {oacc[dt][4 * i4] * inv, oacc[dt][4 * i4 + 1] * inv, oacc[dt][4 * i4 + 2] * inv, oacc[dt][4 * i4 + 3] * inv};
                    if (dt * 32 + i4 * 8 + g * 4 < dv) *reinterpret_cast<float4_t *>(orow + dt * 32 + i4 * 8 + g * 4) = w;
                }
        }
    } else {
        // ---- merge the SPLIT partial states of each query block through LDS (the K / V buffers are free: every wave
        // has passed the barrier that closed the last iteration).  Wave `part` then finishes 4 / SPLIT of the 4
        // four-dim groups of every O^T tile.
        float4_t *part_o = reinterpret_cast<float4_t *>(f32_lds);   // [wave][dt][i4][lane]
        float *part_m = f32_lds + 4 * DT * 4 * 64 * 4;              // [wave][32]
        float *part_l = part_m + 4 * 32;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4)
                part_o[((wave * DT + dt) * 4 + i4) * 64 + lane] = float4_t{oacc[dt][4 * i4], oacc[dt][4 * i4 + 1], oacc[dt][4 * i4 + 2], oacc[dt][4 * i4 + 3]};
        if (g == 0) {
            part_m[wave * 32 + ql] = m_run;
            part_l[wave * 32 + ql] = l_tot;
        }
        __syncthreads();
        float m_star = NEG_INF_F;
#pragma unroll
        for (int p = 0; p < SPLIT; ++p) m_star = fmaxf(m_star, part_m[(rb * SPLIT + p) * 32 + ql]);
        float sc[SPLIT], l_star = 0.0f;
#pragma unroll
        for (int p = 0; p < SPLIT; ++p) {
            const float m_p = part_m[(rb * SPLIT + p) * 32 + ql];
            sc[p] = m_p == NEG_INF_F ? 0.0f : __builtin_amdgcn_exp2f(m_p - m_star);
            l_star += sc[p] * part_l[(rb * SPLIT + p) * 32 + ql];
        }
        const float inv = l_star > 0.0f ? 1.0f / l_star : 0.0f;
        if (q_ok) {
            float *orow = O + static_cast<int64_t>(q) * a.os[2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int k4 = 0; k4 < 4 / SPLIT; ++k4) {
                    const int i4 = part * (4 / SPLIT) + k4;
                    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int p = 0; p < SPLIT; ++p) {
                        const float4_t t = part_o[(((rb * SPLIT + p) * DT + dt) * 4 + i4) * 64 + lane];
                        acc[0] += sc[p] * t[0]; acc[1] += sc[p] * t[1]; acc[2] += sc[p] * t[2]; acc[3] += sc[p] * t[3];
                    }
                    const float4_t w = {acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
                    if (dt * 32 + i4 * 8 + g * 4 < dv) *reinterpret_cast<float4_t *>(orow + dt * 32 + i4 * 8 + g * 4) = w;
                }
        }
    }
}

// ------------------------------------------------------------- generic kernel
// 256 threads = 16 query rows x 16 lanes.  K/V tiles of 32 keys are widened to
// fp32 in LDS.  Lane c of a row computes scores for keys c, c+16 and output dims
// c, c+16, ...

constexpr int GM = 16, GN = 32, GMAXD = 256;

__global__ __launch_bounds__(256) void sdpa_generic_kernel(const SdpaArgs a) {
    extern __shared__ float smem[];
    const int D = a.D;
    const int ksd = D + 1;
    float *Qs = smem;                 // [GM][D]
    float *Ksm = Qs + GM * D;         // [GN][D+1]
    float *Vs = Ksm + GN * ksd;       // [GN][D]
    float *Ps = Vs + GN * D;          // [GM][GN]

    const int tid = threadIdx.x;
    const int r = tid / 16, c = tid % 16;
    const int bh = blockIdx.y;
    const int b = bh / a.H, h = bh % a.H;
    const int q0 = blockIdx.x * GM;
    const int q = q0 + r;
    const bool q_ok = q < a.Sq;
    const int64_t qoff = b * a.qs[0] + h * a.qs[1], koff = b * a.ks[0] + h * a.ks[1];
    const int64_t voff = b * a.vs[0] + h * a.vs[1], ooff = b * a.os[0] + h * a.os[1];
    const uint8_t *M = a.mask ? a.mask + b * a.ms[0] + h * a.ms[1] : nullptr;

    for (int i = tid; i < GM * D; i += 256) {
        const int rr = i / D, d = i % D;
        Qs[i] = (q0 + rr < a.Sq) ? load_any(a.q, a.dtype, qoff + static_cast<int64_t>(q0 + rr) * a.qs[2] + d) : 0.0f;
    }

    float acc[GMAXD / 16];
#pragma unroll
    for (int i = 0; i < GMAXD / 16; ++i) acc[i] = 0.0f;
    float m_run = NEG_INF_F, l_run = 0.0f;

    int kv_end = a.Skv;
    if (a.causal) kv_end = min(a.Skv, q0 + GM);
    for (int kv0 = 0; kv0 < kv_end; kv0 += GN) {
        __syncthreads();
        for (int i = tid; i < GN * D; i += 256) {
            const int rr = i / D, d = i % D;
            const bool ok = kv0 + rr < a.Skv;
            Ksm[rr * ksd + d] = ok ? load_any(a.k, a.dtype, koff + static_cast<int64_t>(kv0 + rr) * a.ks[2] + d) : 0.0f;
            Vs[rr * D + d] = ok ? load_any(a.v, a.dtype, voff + static_cast<int64_t>(kv0 + rr) * a.vs[2] + d) : 0.0f;
        }
        __syncthreads();
        float s[GN / 16];
#pragma unroll
        for (int jj = 0; jj < GN / 16; ++jj) {
            const int j = c + 16 * jj;
            float dot = 0.0f;
            for (int d = 0; d < D; ++d) dot = __builtin_fmaf(Qs[r * D + d], Ksm[j * ksd + d], dot);
            dot *= a.scale;
            const int kv = kv0 + j;
            bool dead = kv >= a.Skv || (a.causal && kv > q);
            if (M != nullptr && q_ok && kv < a.Skv) dead = dead || M[static_cast<int64_t>(q) * a.Skv + kv] != 0;
            s[jj] = dead ? NEG_INF_F : dot;
        }
        float mloc = NEG_INF_F;
#pragma unroll
        for (int jj = 0; jj < GN / 16; ++jj) mloc = fmaxf(mloc, s[jj]);
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, o, WAVE));
        const float m_new = fmaxf(m_run, mloc);
        const float m_use = m_new == NEG_INF_F ? 0.0f : m_new;
        const float alpha = __expf(m_run - m_use);
        m_run = m_new;
        float lsum = 0.0f;
#pragma unroll
        for (int jj = 0; jj < GN / 16; ++jj) {
            const float p = __expf(s[jj] - m_use);
            Ps[r * GN + c + 16 * jj] = p;
            lsum += p;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) lsum += __shfl_xor(lsum, o, WAVE);
        l_run = l_run * alpha + lsum;
        __syncthreads();
#pragma unroll
        for (int dd = 0; dd < GMAXD / 16; ++dd) {
            const int d = c + 16 * dd;
            if (d < D) {
                float t = acc[dd] * alpha;
                for (int j = 0; j < GN; ++j) t = __builtin_fmaf(Ps[r * GN + j], Vs[j * D + d], t);
                acc[dd] = t;
            }
        }
    }
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    if (q_ok) {
#pragma unroll
        for (int dd = 0; dd < GMAXD / 16; ++dd) {
            const int d = c + 16 * dd;
            if (d < D) store_any(a.o, a.dtype, ooff + static_cast<int64_t>(q) * a.os[2] + d, acc[dd] * inv);
        }
    }
}

// every element of an output given through its (batch, head, row) strides: no key at all means every row is "fully masked"
__global__ __launch_bounds__(256) void sdpa_zero_output_kernel(void *o, int dtype, int B, int H, int Sq, int D, int64_t sb, int64_t sh, int64_t ss) {
    const int64_t total = static_cast<int64_t>(B) * H * Sq * D;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int d = static_cast<int>(i % D);
        const int64_t r = i / D;
        const int sq = static_cast<int>(r % Sq), h = static_cast<int>((r / Sq) % H), b = static_cast<int>(r / Sq / H);
        store_any(o, dtype, b * sb + h * sh + sq * ss + d, 0.0f);
    }
}

// ------------------------------------------------------------------ host side
namespace {

enum class SdpaKind { EMPTY, MFMA, MFMA_F32, GENERIC, INVALID };

// which schedule the calling thread's last axhip_sdpa_fwd launched (diagnostic, for tests and A/B timing)
thread_local const char *last_schedule = "none";

// 0 = automatic; 4 / 8 forces the work-group width of the head_dim-128 kernel (AXHIP_SDPA_D128_WAVES)
int sdpa_d128_waves = [] {
    const char *e = getenv("AXHIP_SDPA_D128_WAVES");
    return e ? atoi(e) : 0;
}();

// AXHIP_SDPA_DECODE_SPLIT=0: decoding steps on the ordinary kernels (for A/B timing)
bool sdpa_decode_split = [] {
    const char *e = getenv("AXHIP_SDPA_DECODE_SPLIT");
    return !(e && e[0] == '0');
}();

// AXHIP_SDPA_KEY_SPLIT=0 keeps small head_dim-64 problems on the unsplit kernel (for A/B timing)
bool sdpa_key_split = [] {
    const char *e = getenv("AXHIP_SDPA_KEY_SPLIT");
    return !(e && e[0] == '0');
}();

// AXHIP_SDPA_F32_MFMA=0 sends fp32 attention to the FMA kernel (for A/B timing)
bool sdpa_f32_mfma = [] {
    const char *e = getenv("AXHIP_SDPA_F32_MFMA");
    return !(e && e[0] == '0');
}();

// AXHIP_SDPA_F32_SPLIT=1|2|4 forces the number of waves that share a query block in the fp32 kernel
int sdpa_f32_split = [] {
    const char *e = getenv("AXHIP_SDPA_F32_SPLIT");
    return e ? atoi(e) : 0;
}();

// AXHIP_SDPA_PINGPONG=0: unmasked head_dim-128 problems that fill the chip on the in-phase pipelined kernel (for A/B timing)
bool sdpa_pingpong = [] {
    const char *e = getenv("AXHIP_SDPA_PINGPONG");
    return !(e && e[0] == '0');
}();

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

SdpaKind pick_kernel(const AxhipSdpaParams &p, const void *q, const void *k, const void *v, const void *o) {
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0 || p.head_dim == 0) return SdpaKind::EMPTY;
    const bool half = p.dtype == AXHIP_DTYPE_BF16 || p.dtype == AXHIP_DTYPE_F16;
    // the 16-bit pipelined kernels also take the multiples of 8 between their compiled sizes (zeros in the missing dims);
    // so do the register-staged head_dim-32 and head_dim-256 kernels (8 .. 24, 136 .. 256)
    if (half && p.head_dim <= 256 && p.head_dim % 8 == 0) {
        bool ok = true;
        // 16-byte vector access to every row of q/k/v, 8-byte to o
        for (int i = 0; i < 3; ++i)
            ok = ok && p.q_strides[i] % 8 == 0 && p.k_strides[i] % 8 == 0 && p.v_strides[i] % 8 == 0 && p.o_strides[i] % 4 == 0;
        // K/V rows are addressed with 32-bit byte offsets inside one (batch, head) slice
        const int64_t span = (static_cast<int64_t>(p.seq_kv) + 64) * std::max(p.k_strides[2], p.v_strides[2]) * 2;
        ok = ok && span < (int64_t(1) << 31);
        ok = ok && (!q || aligned16(q)) && (!k || aligned16(k)) && (!v || aligned16(v)) && (!o || aligned16(o));
        if (ok) return SdpaKind::MFMA;
    }
    // fp32: every multiple of 4 up to 128, as the next of 32 / 64 / 128
    if (p.dtype == AXHIP_DTYPE_F32 && p.head_dim <= 128 && p.head_dim % 4 == 0 && sdpa_f32_mfma) {
        bool ok = true;
        for (int i = 0; i < 3; ++i) // 16-byte vector access to every row
            ok = ok && p.q_strides[i] % 4 == 0 && p.k_strides[i] % 4 == 0 && p.v_strides[i] % 4 == 0 && p.o_strides[i] % 4 == 0;
        const int64_t span = (static_cast<int64_t>(p.seq_kv) + 64) * std::max(p.k_strides[2], p.v_strides[2]) * 4;
        ok = ok && span < (int64_t(1) << 31);
        ok = ok && static_cast<int64_t>(p.seq_q) * p.seq_kv < (int64_t(1) << 31) - (1 << 20); // mask offsets are 32-bit
        ok = ok && (!q || aligned16(q)) && (!k || aligned16(k)) && (!v || aligned16(v)) && (!o || aligned16(o));
        if (ok) return SdpaKind::MFMA_F32;
    }
    if (p.head_dim <= GMAXD) return SdpaKind::GENERIC;
    return SdpaKind::INVALID;
}

int validate(const AxhipSdpaParams &p) {
    AXHIP_REQUIRE(valid_dtype(p.dtype), AXHIP_ERR_INVALID_ARG, "axhip_sdpa_fwd: bad dtype %d", p.dtype);
    AXHIP_REQUIRE(p.batch >= 0 && p.heads >= 0 && p.seq_q >= 0 && p.seq_kv >= 0 && p.head_dim >= 0, AXHIP_ERR_INVALID_ARG,
                  "axhip_sdpa_fwd: negative extent");
    for (int i = 0; i < 3; ++i)
        AXHIP_REQUIRE(p.q_strides[i] >= 0 && p.k_strides[i] >= 0 && p.v_strides[i] >= 0 && p.o_strides[i] >= 0, AXHIP_ERR_INVALID_ARG,
                      "axhip_sdpa_fwd: negative stride");
    AXHIP_REQUIRE(p.mask_strides[0] >= 0 && p.mask_strides[1] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_sdpa_fwd: negative mask stride");
    return AXHIP_OK;
}

// A decoding step -- one block of query rows, few (batch, head) slices, a long unmasked key sequence -- splits its keys
// between work-groups; the partial results need temporary memory.  Returns the number of key chunks (0: no split).
// (from 8 M key elements on: below that the second kernel and the temporary memory cost more than they gain --
// 20 heads of 1500 keys of 64: 12.5 us unsplit, 21.6 split; 32 heads of 4096 keys of 128: 78.7 -> 27.2 us)
struct DecodeSplit { int ksplit, kchunk, DD; size_t bytes; };
DecodeSplit decode_split_plan(const AxhipSdpaParams &p, bool has_mask) {
    DecodeSplit d{0, 0, 0, 0};
    const bool half = p.dtype == AXHIP_DTYPE_BF16 || p.dtype == AXHIP_DTYPE_F16;
    const int64_t slices = static_cast<int64_t>(p.batch) * p.heads;
    if (!half || has_mask || p.is_causal || p.seq_q <= 0 || p.seq_q > BM || slices <= 0 || slices > 384 || p.seq_kv < 1024 || p.head_dim <= 32 ||
        p.head_dim > 128 || p.head_dim % 8 != 0 || slices * p.seq_kv * p.head_dim < (int64_t(8) << 20) || !sdpa_decode_split)
        return d;
    d.DD = p.head_dim <= 64 ? 64 : 128;
    // (enough work-groups for four per CU: 128 (batch, head) slices of 16384 keys ran at 32 % of the HBM peak unsplit -- half
    // the CUs idle --, 256 slices of 8192 keys at 52 %)
    const int parts = static_cast<int>(std::min<int64_t>(std::min<int64_t>(64, ((slices <= 96 ? 512 : 1024) + slices - 1) / slices), p.seq_kv / 256));
    d.kchunk = ((p.seq_kv + parts - 1) / parts + BN - 1) / BN * BN;
    d.ksplit = (p.seq_kv + d.kchunk - 1) / d.kchunk;
    d.bytes = static_cast<size_t>(slices) * d.ksplit * p.seq_q * (d.DD + 1) * sizeof(float);
    return d;
}

template <bool BF16, int D> int launch_mfma(const SdpaArgs &a, hipStream_t s) {
    const unsigned grid = static_cast<unsigned>(a.nqb) * static_cast<unsigned>(a.B * a.H);
    constexpr size_t lds = D > 128 ? sdpa_mfma_lds_bytes<D>() : 0;
    if constexpr (D > 128) {
        static const bool configured = [] {
            return hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_mfma_kernel<BF16, D, true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess &&
                   hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_mfma_kernel<BF16, D, false>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess;
        }();
        AXHIP_REQUIRE(configured, AXHIP_ERR_UNSUPPORTED, "axhip_sdpa_fwd: cannot reserve %zu bytes of LDS", lds);
    }
    if (a.mask) hipLaunchKernelGGL((sdpa_mfma_kernel<BF16, D, true>), dim3(grid), dim3(256), lds, s, a);
    else hipLaunchKernelGGL((sdpa_mfma_kernel<BF16, D, false>), dim3(grid), dim3(256), lds, s, a);
    return AXHIP_OK;
}

template <int D, int SPLIT> int launch_mfma_f32(const SdpaArgs &a, hipStream_t s) {
    constexpr int lds = sdpa_f32_lds_bytes<D>();
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_mfma_f32_kernel<false, D, SPLIT>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (attr == hipSuccess)
            attr = hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_mfma_f32_kernel<true, D, SPLIT>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    });
    AXHIP_CHECK_HIP(attr);
    const unsigned grid = static_cast<unsigned>(a.nqb) * static_cast<unsigned>(a.B * a.H);
    if (a.mask) hipLaunchKernelGGL((sdpa_mfma_f32_kernel<true, D, SPLIT>), dim3(grid), dim3(256), lds, s, a);
    else hipLaunchKernelGGL((sdpa_mfma_f32_kernel<false, D, SPLIT>), dim3(grid), dim3(256), lds, s, a);
    return AXHIP_OK;
}

template <int D> int launch_mfma_f32_d(const SdpaArgs &a, int split, hipStream_t s) {
    return split == 1 ? launch_mfma_f32<D, 1>(a, s) : split == 2 ? launch_mfma_f32<D, 2>(a, s) : launch_mfma_f32<D, 4>(a, s);
}

} // namespace
} // namespace axhip

using namespace axhip;

extern "C" {

// diagnostic: resident work-groups per CU of the head_dim-128 bf16 kernel (waves = 4 or 8)
int axhip_sdpa_d128_occupancy(int waves) {
    int n = -1;
    hipError_t e = waves == 8
        ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, sdpa_mfma_pipelined_kernel<true, false, 8, 128>, 512, 0)
        : hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, sdpa_mfma_pipelined_kernel<true, false, 4, 128>, 256, 0);
    return e == hipSuccess ? n : -static_cast<int>(e);
}

const char *axhip_sdpa_last_schedule(void) { return last_schedule; }

const char *axhip_sdpa_kernel_name(const AxhipSdpaParams *p) {
    static thread_local char name[48];
    if (!p) return "invalid";
    switch (pick_kernel(*p, nullptr, nullptr, nullptr, nullptr)) {
    case SdpaKind::EMPTY: return "empty";
    case SdpaKind::MFMA:
        snprintf(name, sizeof(name), "mfma_%s_d%d", p->dtype == AXHIP_DTYPE_BF16 ? "bf16" : "f16", p->head_dim);
        return name;
    case SdpaKind::MFMA_F32:
        snprintf(name, sizeof(name), "mfma_f32_d%d", p->head_dim);
        return name;
    case SdpaKind::GENERIC: return "generic";
    default: return "invalid";
    }
}

size_t axhip_sdpa_workspace_bytes(const AxhipSdpaParams *params, int has_mask) {
    if (!params || validate(*params) != AXHIP_OK) return 0;
    if (pick_kernel(*params, nullptr, nullptr, nullptr, nullptr) != SdpaKind::MFMA) return 0;
    return CallScratch::rounded(decode_split_plan(*params, has_mask != 0).bytes);
}

int axhip_sdpa_fwd(const void *q, const void *k, const void *v, void *o, const uint8_t *mask,
                   const AxhipSdpaParams *params, void *stream) {
    return axhip_sdpa_fwd_ws(q, k, v, o, mask, params, nullptr, 0, stream);
}

int axhip_sdpa_fwd_ws(const void *q, const void *k, const void *v, void *o, const uint8_t *mask,
                      const AxhipSdpaParams *params, void *workspace, size_t workspace_bytes, void *stream) {
    AXHIP_REQUIRE(params != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_sdpa_fwd: params is NULL");
    const AxhipSdpaParams &p = *params;
    int rc = validate(p);
    if (rc) return rc;
    const SdpaKind kind = pick_kernel(p, q, k, v, o);
    last_schedule = "empty";
    if (kind == SdpaKind::EMPTY) return AXHIP_OK;
    if (p.seq_kv == 0) { // no key at all: every row is "fully masked" -> zeros
        AXHIP_REQUIRE(o != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_sdpa_fwd: NULL tensor");
        // one launch: the output viewed as (batch, head, row, dim) through its strides
        rc = ensure_init();
        if (rc) return rc;
        const int64_t total = static_cast<int64_t>(p.batch) * p.heads * p.seq_q * p.head_dim;
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((total + 255) / 256, 256 * 32));
        hipLaunchKernelGGL(sdpa_zero_output_kernel, dim3(blocks), dim3(256), 0, resolve_stream(stream), o, p.dtype, p.batch, p.heads, p.seq_q, p.head_dim,
                           p.o_strides[0], p.o_strides[1], p.o_strides[2]);
        AXHIP_CHECK_HIP(hipGetLastError());
        return AXHIP_OK;
    }
    AXHIP_REQUIRE(kind != SdpaKind::INVALID, AXHIP_ERR_UNSUPPORTED, "axhip_sdpa_fwd: head_dim %d > %d is not supported", p.head_dim, GMAXD);
    AXHIP_REQUIRE(q && k && v && o, AXHIP_ERR_INVALID_ARG, "axhip_sdpa_fwd: NULL tensor");
    AXHIP_REQUIRE(static_cast<int64_t>(p.batch) * p.heads < 65536 || kind != SdpaKind::GENERIC, AXHIP_ERR_UNSUPPORTED,
                  "axhip_sdpa_fwd: batch*heads too large for the generic kernel");
    rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);

    SdpaArgs a{};
    a.q = q; a.k = k; a.v = v; a.o = o; a.mask = mask;
    a.B = p.batch; a.H = p.heads; a.Sq = p.seq_q; a.Skv = p.seq_kv; a.D = p.head_dim;
    a.scale = p.scale > 0.0f ? p.scale : 1.0f / std::sqrt(static_cast<float>(p.head_dim));
    a.scale_log2e = a.scale * 1.44269504088896340736f;
    a.causal = p.is_causal ? 1 : 0;
    a.dtype = p.dtype;
    for (int i = 0; i < 3; ++i) { a.qs[i] = p.q_strides[i]; a.ks[i] = p.k_strides[i]; a.vs[i] = p.v_strides[i]; a.os[i] = p.o_strides[i]; }
    a.ms[0] = p.mask_strides[0]; a.ms[1] = p.mask_strides[1];

    if (kind == SdpaKind::MFMA) {
        a.nqb = (p.seq_q + BM - 1) / BM;
        AXHIP_REQUIRE(static_cast<int64_t>(a.nqb) * p.batch * p.heads < (int64_t(1) << 31), AXHIP_ERR_UNSUPPORTED, "axhip_sdpa_fwd: grid too large");
        const bool bf = p.dtype == AXHIP_DTYPE_BF16;
        // A decoding step -- one block of query rows, few (batch, head) slices, a long key sequence -- would give the
        // chip a work-group per slice: the keys are split between work-groups instead (flash decoding), partial
        // results in stream-ordered temporary memory, merged by a second kernel.
        const int64_t slices = static_cast<int64_t>(p.batch) * p.heads;
        const DecodeSplit ds = decode_split_plan(p, mask != nullptr);
        if (ds.ksplit > 0) {
            last_schedule = "decode_split";
            const int DD = ds.DD;
            a.kchunk = ds.kchunk;
            a.ksplit = ds.ksplit;
            const size_t rows = static_cast<size_t>(slices) * a.ksplit * p.seq_q;
            CallScratch scratch(workspace, workspace_bytes, s);
            void *tmp = nullptr;
            rc = scratch.take(&tmp, ds.bytes, "axhip_sdpa");
            if (rc) return rc;
            a.opart = static_cast<float *>(tmp);
            a.lse = a.opart + rows * DD;
            a.nqb = 1;
            const unsigned grid = static_cast<unsigned>(slices * a.ksplit);
            if (DD == 64) {
                if (bf) hipLaunchKernelGGL((sdpa_mfma_kernel<true, 64, false, true>), dim3(grid), dim3(256), 0, s, a);
                else hipLaunchKernelGGL((sdpa_mfma_kernel<false, 64, false, true>), dim3(grid), dim3(256), 0, s, a);
            } else {
                constexpr size_t lds = sdpa_mfma_lds_bytes<128>();
                static const bool configured = [] {
                    return hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_mfma_kernel<true, 128, false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess &&
                           hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_mfma_kernel<false, 128, false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess;
                }();
                AXHIP_REQUIRE(configured, AXHIP_ERR_UNSUPPORTED, "axhip_sdpa_fwd: cannot reserve %zu bytes of LDS", lds); // (scratch returns its memory on the way out)
                if (bf) hipLaunchKernelGGL((sdpa_mfma_kernel<true, 128, false, true>), dim3(grid), dim3(256), lds, s, a);
                else hipLaunchKernelGGL((sdpa_mfma_kernel<false, 128, false, true>), dim3(grid), dim3(256), lds, s, a);
            }
            const int64_t items = slices * p.seq_q * (DD / 4);
            const unsigned mgrid = static_cast<unsigned>(std::min<int64_t>((items + 255) / 256, 4096));
            if (bf) hipLaunchKernelGGL(sdpa_splitk_merge_kernel<true>, dim3(mgrid), dim3(256), 0, s, a, DD);
            else hipLaunchKernelGGL(sdpa_splitk_merge_kernel<false>, dim3(mgrid), dim3(256), 0, s, a, DD);
            rc = scratch.release();
            if (rc) return rc;
            AXHIP_CHECK_HIP(hipGetLastError());
            return AXHIP_OK;
        }
        last_schedule = "register_staged";
        switch (p.head_dim <= 32 ? 32 : p.head_dim > 128 ? 256 : 64) {
        case 32: rc = bf ? launch_mfma<true, 32>(a, s) : launch_mfma<false, 32>(a, s); break;
        case 256: rc = bf ? launch_mfma<true, 256>(a, s) : launch_mfma<false, 256>(a, s); break;
        default: {
            // 8-wave work-groups (256 query rows, each K/V tile fetched once for all of them) when that still gives
            // every CU a work-group; 4-wave work-groups (128 rows, two per CU) for shorter or narrower problems
            const int nqb8 = (p.seq_q + 255) / 256;
            const int64_t g8 = static_cast<int64_t>(a.causal ? (nqb8 + 1) / 2 : nqb8) * a.B * a.H;
            const bool wide = p.seq_q > 128 && sdpa_d128_waves != 4 && (g8 >= 256 || sdpa_d128_waves == 8);
            // Problems with 4-wave work-groups for at most half of the CUs split the keys between the two halves of a
            // work-group of 64 query rows instead: twice the work-groups, half the steps each (12 heads of 1024 rows:
            // 14.8 -> 10.6 us).  With a work-group for nearly every CU (Whisper's 20 heads of 1500 frames: 240) the
            // split changes nothing -- a SIMD issues the same instructions as one wave or as two.
            const int64_t g4 = static_cast<int64_t>((p.seq_q + 127) / 128) * a.B * a.H;
            if (p.head_dim > 32 && p.head_dim <= 64 && !mask && !a.causal && p.seq_kv > BN && g4 <= 128 && sdpa_key_split) {
                last_schedule = "key_split";
                const unsigned gs = static_cast<unsigned>((p.seq_q + 63) / 64) * static_cast<unsigned>(a.B * a.H);
                if (p.head_dim == 64) {
                    if (bf) hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<true, false, 4, 64, 2>), dim3(gs), dim3(256), 0, s, a);
                    else hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<false, false, 4, 64, 2>), dim3(gs), dim3(256), 0, s, a);
                } else {
                    if (bf) hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<true, false, 4, 64, 2, true>), dim3(gs), dim3(256), 0, s, a);
                    else hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<false, false, 4, 64, 2, true>), dim3(gs), dim3(256), 0, s, a);
                }
                break;
            }
            const int bmw = wide ? 256 : 128;
            const int nqbw = (p.seq_q + bmw - 1) / bmw;
            const unsigned g = static_cast<unsigned>(a.causal ? (nqbw + 1) / 2 : nqbw) * static_cast<unsigned>(a.B * a.H);
#define AXHIP_LAUNCH_DX(BF, MK, DD)                                                                                       \
    do {                                                                                                                  \
        if (p.head_dim == DD) {                                                                                           \
            if (wide) hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<BF, MK, 8, DD>), dim3(g), dim3(512), 0, s, a);            \
            else hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<BF, MK, 4, DD>), dim3(g), dim3(256), 0, s, a);                 \
        } else {                                                                                                          \
            if (wide) hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<BF, MK, 8, DD, 1, true>), dim3(g), dim3(512), 0, s, a);   \
            else hipLaunchKernelGGL((sdpa_mfma_pipelined_kernel<BF, MK, 4, DD, 1, true>), dim3(g), dim3(256), 0, s, a);        \
        }                                                                                                                 \
    } while (0)
#define AXHIP_LAUNCH_D(DD)                                                                                                \
    do {                                                                                                                  \
        if (bf && mask) AXHIP_LAUNCH_DX(true, true, DD);                                                                  \
        else if (bf) AXHIP_LAUNCH_DX(true, false, DD);                                                                    \
        else if (mask) AXHIP_LAUNCH_DX(false, true, DD);                                                                  \
        else AXHIP_LAUNCH_DX(false, false, DD);                                                                           \
    } while (0)
            last_schedule = wide ? "pipelined8" : "pipelined4";
            if (p.head_dim == 128 && !mask && wide && sdpa_pingpong) {
                last_schedule = "pingpong";
                // persistent work-groups, one per CU (a multiple of 8: a (batch, head) keeps its XCD)
                // (head_dim 64 stays on the pipelined kernel: with twice the softmax work per MFMA the two phases are
                // too uneven -- measured 846 against 867 TFLOP/s on bf16 B4 H32 S4096 causal)
                const unsigned gp = std::min<unsigned>(g, 256);
                if (bf) hipLaunchKernelGGL((sdpa_mfma_pingpong_kernel<true, 128>), dim3(gp), dim3(512), 0, s, a);
                else hipLaunchKernelGGL((sdpa_mfma_pingpong_kernel<false, 128>), dim3(gp), dim3(512), 0, s, a);
            } else if (p.head_dim <= 64) AXHIP_LAUNCH_D(64);
            else AXHIP_LAUNCH_D(128);
#undef AXHIP_LAUNCH_D
#undef AXHIP_LAUNCH_DX
        }
            break;
        }
    } else if (kind == SdpaKind::MFMA_F32) {
        last_schedule = "mfma_f32";
        // waves per 32-row query block, by how many such blocks there are for the 1024 SIMDs (thresholds from timings
        // of 128 .. 1024 blocks: below 0.75 blocks per SIMD the four-way split wins by up to 2.7x, above 1.5 none is needed)
        const int64_t blocks32 = static_cast<int64_t>((p.seq_q + 31) / 32) * p.batch * p.heads;
        int split = blocks32 >= 1536 ? 1 : blocks32 >= 768 ? 2 : 4;
        if (sdpa_f32_split == 1 || sdpa_f32_split == 2 || sdpa_f32_split == 4) split = sdpa_f32_split;
        const int bmw = 128 / split;
        a.nqb = (p.seq_q + bmw - 1) / bmw;
        AXHIP_REQUIRE(static_cast<int64_t>(a.nqb) * p.batch * p.heads < (int64_t(1) << 31), AXHIP_ERR_UNSUPPORTED, "axhip_sdpa_fwd: grid too large");
        rc = p.head_dim <= 32 ? launch_mfma_f32_d<32>(a, split, s) : p.head_dim <= 64 ? launch_mfma_f32_d<64>(a, split, s) : launch_mfma_f32_d<128>(a, split, s);
        if (rc) return rc;
    } else {
        last_schedule = "generic";
        a.nqb = (p.seq_q + GM - 1) / GM;
        const size_t lds = sizeof(float) * (static_cast<size_t>(GM) * a.D + static_cast<size_t>(GN) * (a.D + 1) + static_cast<size_t>(GN) * a.D + GM * GN);
        static std::once_flag attr_once;
        static hipError_t attr = hipSuccess;
        std::call_once(attr_once, [] { attr = hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_generic_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); });
        AXHIP_CHECK_HIP(attr);
        hipLaunchKernelGGL(sdpa_generic_kernel, dim3(a.nqb, a.B * a.H), dim3(256), lds, s, a);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

} // extern "C"
