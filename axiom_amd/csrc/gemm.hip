// C = op(A) op(B) (+ bias) (+ residual), activation epilogue.
//
//   gemm_mfma_nt_kernel   bf16 / f16, A [M,K] and B [N,K] both K-contiguous (the
//                         nn::Linear case x W^T): v_mfma_f32_32x32x16, workgroup
//                         tile 128x128x64 or 64x128x64, 4 waves, A/B tiles staged
//                         through LDS with up to three k-tiles in flight, fp32
//                         accumulation.
//   gemm_generic_kernel   any dtype / any transpose combination, 16x16 LDS tiles,
//                         fp32 FMA.
#include "common.hpp"
#include "gemm_skinny.hpp"

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <set>
#include <type_traits>

namespace axhip {

struct GemmArgs {
    const void *a, *b;
    void *c;
    const void *bias, *residual;
    int dtype, epilogue;
    int64_t M, N, K;
    int64_t a_rs, a_cs, b_rs, b_cs, ldc; // element strides of op(A)[m][k], op(B)[k][n]
    int64_t sa, sb, sc;                   // batch strides
};

// ------------------------------------------------------------------- generic
__global__ __launch_bounds__(256) void gemm_generic_kernel(const GemmArgs g) {
    __shared__ float As[16][17], Bs[16][17];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int64_t bz = blockIdx.z;
    const int64_t m = static_cast<int64_t>(blockIdx.y) * 16 + ty, n = static_cast<int64_t>(blockIdx.x) * 16 + tx;
    const int64_t aoff = bz * g.sa, boff = bz * g.sb, coff = bz * g.sc;
    float acc = 0.0f;
    for (int64_t k0 = 0; k0 < g.K; k0 += 16) {
        const int64_t ka = k0 + tx, kb = k0 + ty;
        As[ty][tx] = (m < g.M && ka < g.K) ? load_any(g.a, g.dtype, aoff + m * g.a_rs + ka * g.a_cs) : 0.0f;
        Bs[ty][tx] = (kb < g.K && n < g.N) ? load_any(g.b, g.dtype, boff + kb * g.b_rs + n * g.b_cs) : 0.0f;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; ++k) acc = __builtin_fmaf(As[ty][k], Bs[k][tx], acc);
        __syncthreads();
    }
    if (m < g.M && n < g.N) {
        if (g.bias) acc += load_any(g.bias, g.dtype, n);
        if (g.residual) acc += load_any(g.residual, g.dtype, coff + m * g.ldc + n);
        store_any(g.c, g.dtype, coff + m * g.ldc + n, gemm_epilogue(g.epilogue, acc));
    }
}

// Epilogue of the MFMA kernels: accumulator element e of 32x32 tile (i, j) is
// C[m_base + 32 i + 8 (e/4) + 4 g2 + e%4][n_base + 32 j + l32].  bias, residual and
// the activation are applied in fp32 before the one rounding to the output type.
// The activation is resolved outside the element loops.
template <bool BF16>
__device__ __forceinline__ float load16(const void *p, int64_t i) {
    const uint16_t b = static_cast<const uint16_t *>(p)[i];
    return BF16 ? bf16_bits_to_f32(b) : f16_bits_to_f32(b);
}
template <bool BF16>
__device__ __forceinline__ void store16(void *p, int64_t i, float x) {
    static_cast<uint16_t *>(p)[i] = BF16 ? f32_to_bf16_bits(x) : f32_to_f16_bits(x);
}

// C and the residual are addressed through buffer descriptors that cover exactly the valid
// rows of the block, so a row past the end of C is dropped by the hardware bounds check;
// columns past the end are masked per lane.  When all MI*32 rows are valid (FULL_ROWS)
// the row offset travels in the scalar offset of the instruction, otherwise it is added
// to the lane's offset, which is what the bounds check looks at.
// (Column tiles outside, rows inside: on the ring kernels' products the other nesting measured 3 - 5 % slower.)
// Requires MI*32 * ldc * 2 < 2^31.
template <bool BF16, int RESIDUAL_T, bool FULL_ROWS, int OP, int MI, int NJ> // RESIDUAL_T: 0 no, 1 yes, 2 decided at run time
__device__ __forceinline__ void gemm_store_tiles_as(const GemmArgs &g, const float16_t (&acc)[MI][NJ], int64_t m_base, int64_t n_base, int64_t coff, int l32, int g2) {
    const bool RESIDUAL = RESIDUAL_T == 1 || (RESIDUAL_T == 2 && g.residual != nullptr);
    const int ldc2 = static_cast<int>(g.ldc) * 2;
    const int cols_valid = static_cast<int>(min<int64_t>(32 * NJ, g.N - n_base));
    const int rows_valid = static_cast<int>(min<int64_t>(32 * MI, g.M - m_base));
    const int extent = (rows_valid - 1) * ldc2 + cols_valid * 2;
    const int64_t origin = coff + m_base * g.ldc + n_base;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(static_cast<uint16_t *>(g.c) + origin, 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(static_cast<const uint16_t *>(RESIDUAL ? g.residual : g.c)) + origin, 0, extent, 0x00020000);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int col = 32 * j + l32;
        if (col >= cols_valid) continue;
        const float bias = g.bias ? load16<BF16>(g.bias, n_base + col) : 0.0f;
        const int voff = 4 * g2 * ldc2 + col * 2;
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            float x[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                x[e] = acc[i][j][e] + bias;
                if (RESIDUAL) {
                    const int roff = (32 * i + 8 * (e / 4) + e % 4) * ldc2;
                    const uint16_t r = __builtin_amdgcn_raw_buffer_load_b16(rrsrc, FULL_ROWS ? voff : voff + roff, FULL_ROWS ? roff : 0, 0);
                    x[e] += BF16 ? bf16_bits_to_f32(r) : f16_bits_to_f32(r);
                }
            }
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const float y0 = gemm_epilogue16(OP, x[e]), y1 = gemm_epilogue16(OP, x[e + 1]);
                const uint32_t w = BF16 ? pack_bf16x2(y0, y1) : pack_f16x2(y0, y1);
                const int roff = (32 * i + 8 * (e / 4) + e % 4) * ldc2;
                __builtin_amdgcn_raw_buffer_store_b16(static_cast<uint16_t>(w & 0xFFFFu), crsrc, FULL_ROWS ? voff : voff + roff, FULL_ROWS ? roff : 0, 0);
                __builtin_amdgcn_raw_buffer_store_b16(static_cast<uint16_t>(w >> 16), crsrc, FULL_ROWS ? voff : voff + roff + ldc2, FULL_ROWS ? roff + ldc2 : 0, 0);
            }
        }
    }
}

template <bool BF16, int MI, int NJ>
__device__ __forceinline__ void gemm_store_tiles(const GemmArgs &g, const float16_t (&acc)[MI][NJ], int64_t m_base, int64_t n_base, int64_t coff, int l32, int g2) {
    if (m_base >= g.M || n_base >= g.N) return;
    const bool full_rows = m_base + MI * 32 <= g.M;
    // the cheap epilogues get a specialisation per (residual, full rows); the transcendental
    // ones are large when unrolled 128 times, and one general instance each is enough
#define AXHIP_GEMM_EPI_FAST(OP)                                                                                         \
    if (full_rows) {                                                                                                    \
        if (g.residual) gemm_store_tiles_as<BF16, 1, true, OP, MI, NJ>(g, acc, m_base, n_base, coff, l32, g2);          \
        else gemm_store_tiles_as<BF16, 0, true, OP, MI, NJ>(g, acc, m_base, n_base, coff, l32, g2);                     \
    } else {                                                                                                            \
        if (g.residual) gemm_store_tiles_as<BF16, 1, false, OP, MI, NJ>(g, acc, m_base, n_base, coff, l32, g2);         \
        else gemm_store_tiles_as<BF16, 0, false, OP, MI, NJ>(g, acc, m_base, n_base, coff, l32, g2);                    \
    }
#define AXHIP_GEMM_EPI_GENERAL(OP) gemm_store_tiles_as<BF16, 2, false, OP, MI, NJ>(g, acc, m_base, n_base, coff, l32, g2);
    switch (g.epilogue) {
    case AXHIP_OP_RELU: AXHIP_GEMM_EPI_FAST(AXHIP_OP_RELU) break;
    case AXHIP_OP_GELU: AXHIP_GEMM_EPI_GENERAL(AXHIP_OP_GELU) break;
    case AXHIP_OP_SILU: AXHIP_GEMM_EPI_GENERAL(AXHIP_OP_SILU) break;
    case AXHIP_OP_SIGMOID: AXHIP_GEMM_EPI_GENERAL(AXHIP_OP_SIGMOID) break;
    case AXHIP_OP_TANH: AXHIP_GEMM_EPI_GENERAL(AXHIP_OP_TANH) break;
    default: AXHIP_GEMM_EPI_FAST(0) break;
    }
#undef AXHIP_GEMM_EPI_FAST
#undef AXHIP_GEMM_EPI_GENERAL
}


// ------------------------------------------------------------------- MFMA NT
// Work-group tile BM x 128 x 64 (BM = 128 or 64), 4 waves in a 2 x 2 layout, each
// owning a (BM/2) x 64 block of C as 32x32 MFMA tiles.  A and B k-tiles travel
// HBM/L2 -> registers -> LDS; NPRE k-tiles are in flight in registers at any
// time, which is what hides the load latency when a small problem leaves one
// work-group per CU (the nn::Linear shapes of a single sequence).  The k loop is
// unrolled NPRE times so that each in-flight tile has its own registers.
constexpr int TN = 128, TK = 64;
constexpr int LDS_STRIDE = TK + 8; // 144 B rows: consecutive rows shift by 4 banks (+32)

template <bool BF16, int BM, int NPRE>
__global__ __launch_bounds__(256, BM == 128 ? 2 : 1) void gemm_mfma_nt_kernel(const GemmArgs g) {
    constexpr int MI = BM / 64;  // 32-row MFMA tiles per wave in M
    constexpr int NA = BM / 32;  // 16-byte chunks of A per thread per k-tile (BM rows x 8 chunks / 256 threads)
    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[TN * LDS_STRIDE];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int l32 = lane % 32, g2 = lane / 32;
    const int wm = (wave / 2) * (BM / 2), wn = (wave % 2) * 64;
    const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM, n0 = static_cast<int64_t>(blockIdx.x) * TN;
    const int64_t bz = blockIdx.z;
    const uint16_t *A = static_cast<const uint16_t *>(g.a) + bz * g.sa;
    const uint16_t *B = static_cast<const uint16_t *>(g.b) + bz * g.sb;

    float16_t acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    uint4_t ra[NPRE][NA], rb[NPRE][4];
    auto load_tiles = [&](int s, int64_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i;
            const int row = id / 8, cc = id % 8;
            const int64_t k = k0 + 8 * cc;
            if (i < NA) {
                ra[s][i < NA ? i : 0] = uint4_t{0, 0, 0, 0};
                if (m0 + row < g.M && k < g.K) ra[s][i < NA ? i : 0] = *reinterpret_cast<const uint4_t *>(A + (m0 + row) * g.a_rs + k);
            }
            rb[s][i] = uint4_t{0, 0, 0, 0};
            if (n0 + row < g.N && k < g.K) rb[s][i] = *reinterpret_cast<const uint4_t *>(B + (n0 + row) * g.b_cs + k);
        }
    };
    auto stage_tiles = [&](int s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i;
            const int row = id / 8, cc = id % 8;
            if (i < NA) *reinterpret_cast<uint4_t *>(&As[row * LDS_STRIDE + 8 * cc]) = ra[s][i < NA ? i : 0];
            *reinterpret_cast<uint4_t *>(&Bs[row * LDS_STRIDE + 8 * cc]) = rb[s][i];
        }
    };
    auto multiply_tile = [&]() {
#pragma unroll
        for (int ks = 0; ks < TK / 16; ++ks) {
            uint4_t af[MI], bf[2];
#pragma unroll
            for (int i = 0; i < MI; ++i) af[i] = *reinterpret_cast<const uint4_t *>(&As[(wm + 32 * i + l32) * LDS_STRIDE + 16 * ks + 8 * g2]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = *reinterpret_cast<const uint4_t *>(&Bs[(wn + 32 * j + l32) * LDS_STRIDE + 16 * ks + 8 * g2]);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if constexpr (BF16)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i]), __builtin_bit_cast(bf16x8_t, bf[j]), acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[i]), __builtin_bit_cast(half8_t, bf[j]), acc[i][j], 0, 0, 0);
                }
        }
    };

#pragma unroll
    for (int s = 0; s < NPRE; ++s)
        if (static_cast<int64_t>(s) * TK < g.K) load_tiles(s, static_cast<int64_t>(s) * TK);
    for (int64_t k0 = 0; k0 < g.K; k0 += NPRE * TK) {
#pragma unroll
        for (int s = 0; s < NPRE; ++s) {
            const int64_t k = k0 + static_cast<int64_t>(s) * TK;
            if (k < g.K) {
                __syncthreads(); // every wave is done reading the previous tile
                stage_tiles(s);
                __syncthreads();
                if (k + NPRE * TK < g.K) load_tiles(s, k + NPRE * TK);
                multiply_tile();
            }
        }
    }

    gemm_store_tiles<BF16, MI, 2>(g, acc, m0 + wm, n0 + wn, bz * g.sc, l32, g2);
}

// ----------------------------------------------------------- MFMA NT, 256x256
// Large products: work-group tile 256 x 256 x 64, 8 waves in a 2 x 4 layout, each owning 128 x 64 of C as 8 x 4
// tiles of v_mfma_f32_16x16x32 (128 accumulator registers).  The kernel runs on the chip's power limit, where time
// follows the energy a launch spends rather than its cycle count, and on operands that change every k-step the
// 16x16x32 form does the same flops for about 15 % less than 32x32x16 (a bare loop of either: 1.9 - 2.0 against
// 1.67 - 1.75 PFLOP/s).  A and B k-tiles go L2 -> LDS directly (buffer_load ... lds: no staging registers, no
// ds_write; staging through registers spends as many cycles and more power) into two 64 KiB buffers, one barrier per
// k-tile.  LDS rows are the 128 bytes of one k-tile row with the 16-byte chunk index XOR-ed by (row >> 1) & 7, which
// spreads the 16 rows of a fragment read over all banks.
// A k-tile is two k-steps of 32 MFMAs.  The A fragments are single-buffered: the registers of fragment row i are
// refilled for the next k-step right behind the row's fourth MFMA, 28 MFMAs before they are needed; the B fragments
// are double-buffered.  Every LDS read and every global load sits between two MFMAs (scheduling fences pin the
// order): a wave that meets a batch of reads, or several loads in a row -- a direct-to-LDS load holds the wave's
// issue for about 60 cycles --, starves the matrix pipe of its SIMD.  The barrier comes after the first fragment row
// of the second k-step: by then every wave has read the whole tile, so the buffer takes the tile after next (the
// loads are dealt out one per three MFMAs from there) and the reads turn to the next tile.
// Work-groups are dealt to the 8 XCDs so that each XCD owns a compact block of C tiles and its L2 sees every A / B
// panel few times.
typedef int int4_t __attribute__((ext_vector_type(4)));
constexpr int BIG = 256;              // tile rows (M) and columns (N)
constexpr int BIG_ROWB = TK * 2;      // bytes per LDS row
constexpr int BIG_TILEB = BIG * BIG_ROWB; // 32 KiB per A or B k-tile

// 16 bytes per lane from a buffer straight into LDS: lane i's data lands at lds_base + 16 i.
// Lanes whose voffset lies beyond the descriptor's extent write zeros.
__device__ __forceinline__ void gemm_load_to_lds(const int4_t &rsrc, uint32_t lds_base_uniform, int voffset, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_base_uniform), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}

__device__ __forceinline__ int4_t gemm_rsrc(const void *base, int bytes) {
    const uint64_t pa = reinterpret_cast<uint64_t>(base);
    return int4_t{static_cast<int>(static_cast<uint32_t>(pa)), static_cast<int>(static_cast<uint32_t>(pa >> 32) & 0xFFFFu), bytes, 0x00020000};
}

// The epilogue for 16x16 accumulator tiles computed as B-fragment x A-fragment^T: lane (l16, g4) holds, of tile
// (i, j), row 16 i + l16 and the four consecutive columns 16 j + 4 g4 .. + 3 -- one 8-byte store where C allows it
// (even ldc, 4-byte aligned origin), 2-byte stores otherwise.  C and the residual go through buffer descriptors that
// cover exactly the block's valid rows (a row past the end is dropped by the bounds check); columns are masked.
// Requires 128 * ldc * 2 < 2^31.
typedef float float4_t __attribute__((ext_vector_type(4)));
template <bool BF16, int RESIDUAL_T, int OP> // RESIDUAL_T: 0 no, 1 yes, 2 decided at run time
__device__ __forceinline__ void gemm_store_tiles16_as(const GemmArgs &g, const float4_t (&acc)[8][4], int64_t m_base, int64_t n_base, int64_t coff, int l16, int g4, unsigned char *stage) {
    const bool RESIDUAL = RESIDUAL_T == 1 || (RESIDUAL_T == 2 && g.residual != nullptr);
    const int ldc2 = static_cast<int>(g.ldc) * 2;
    const int cols_valid = static_cast<int>(min<int64_t>(64, g.N - n_base));
    const int rows_valid = static_cast<int>(min<int64_t>(128, g.M - m_base));
    const int extent = (rows_valid - 1) * ldc2 + cols_valid * 2;
    const int64_t origin = coff + m_base * g.ldc + n_base;
    uint16_t *cbase = static_cast<uint16_t *>(g.c) + origin;
    const uint16_t *rbase = static_cast<const uint16_t *>(RESIDUAL ? g.residual : g.c) + origin;
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(cbase, 0, extent, 0x00020000);
    const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(rbase), 0, extent, 0x00020000);
    const bool wide = (g.ldc & 1) == 0 && (reinterpret_cast<uintptr_t>(cbase) & 3u) == 0 && (reinterpret_cast<uintptr_t>(rbase) & 3u) == 0;
    float bias[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int col = 16 * j + 4 * g4 + e;
            bias[j][e] = g.bias && col < cols_valid ? load16<BF16>(g.bias, n_base + col) : 0.0f;
        }
    // A block with all 64 columns inside and 16-byte aligned rows goes through the wave's 16 KiB of LDS (free once the
    // k loop has ended): the finished 16-bit values are written in accumulator layout and read back row by row, so that
    // every global store carries 16 bytes per lane and a store instruction fills eight whole 128-byte lines.  While C is
    // written no MFMA runs anywhere on the chip (all work-groups end their k loops together), so the write phase is
    // pure HBM time: 8-byte stores, 32 bytes of a row per instruction, take 9.3 us for the 32 MiB of 4096^2 values.
    const bool staged = stage != nullptr && cols_valid == 64 && (g.ldc & 7) == 0 && (reinterpret_cast<uintptr_t>(cbase) & 15u) == 0;
    // rows outside, columns inside: the four stores that complete a row's 128-byte line follow one another (with the
    // column tiles outside, 16 rows apart in between, the same kernel takes 7 % longer on 4096^3)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = 16 * j + 4 * g4;
            if (col >= cols_valid) continue;
            const bool whole = wide && col + 4 <= cols_valid;
            const int voff = (16 * i + l16) * ldc2 + col * 2;
            float x[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = acc[i][j][e] + bias[j][e];
            if (RESIDUAL) {
                if (whole) {
                    const uint2_t r = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rrsrc, voff, 0, 0));
                    const uint32_t rw[2] = {r.x, r.y};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint16_t h = static_cast<uint16_t>(rw[e / 2] >> (16 * (e % 2)));
                        x[e] += BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < cols_valid) {
                            const uint16_t h = __builtin_amdgcn_raw_buffer_load_b16(rrsrc, voff + 2 * e, 0, 0);
                            x[e] += BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
                        }
                }
            }
            uint32_t w[2];
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
                const float y0 = gemm_epilogue16(OP, x[e]), y1 = gemm_epilogue16(OP, x[e + 1]);
                w[e / 2] = BF16 ? pack_bf16x2(y0, y1) : pack_f16x2(y0, y1);
            }
            if (staged) {
                const int r = 16 * i + l16; // 128-byte rows; the 16-byte chunk index is XOR-ed with the row so that neither pass meets bank conflicts
                *reinterpret_cast<uint2_t *>(stage + r * 128 + (((2 * j + (g4 >> 1)) ^ (r & 7)) * 16) + (g4 & 1) * 8) = uint2_t{w[0], w[1]};
            } else if (whole) {
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(decltype(__builtin_amdgcn_raw_buffer_load_b64(rrsrc, 0, 0, 0)), uint2_t{w[0], w[1]}), crsrc, voff, 0, 0);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < cols_valid)
                        __builtin_amdgcn_raw_buffer_store_b16(static_cast<uint16_t>(w[e / 2] >> (16 * (e % 2))), crsrc, voff + 2 * e, 0, 0);
            }
        }
    }
    if (staged) {
        const int lane = 16 * g4 + l16;
#pragma unroll
        for (int n = 0; n < 16; ++n) {
            const int r = 8 * n + (lane >> 3), q = lane & 7;
            const uint4_t v = *reinterpret_cast<const uint4_t *>(stage + r * 128 + ((q ^ (r & 7)) * 16));
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(decltype(__builtin_amdgcn_raw_buffer_load_b128(rrsrc, 0, 0, 0)), v), crsrc, r * ldc2 + q * 16, 0, 0);
        }
    }
}

template <bool BF16>
__device__ __forceinline__ void gemm_store_tiles16(const GemmArgs &g, const float4_t (&acc)[8][4], int64_t m_base, int64_t n_base, int64_t coff, int l16, int g4, unsigned char *stage) {
    if (m_base >= g.M || n_base >= g.N) return;
    // the cheap epilogues get a specialisation with and without residual; the transcendental ones are large when
    // unrolled 128 times, and one general instance each is enough
    switch (g.epilogue) {
    case AXHIP_OP_RELU:
        if (g.residual) gemm_store_tiles16_as<BF16, 1, AXHIP_OP_RELU>(g, acc, m_base, n_base, coff, l16, g4, stage);
        else gemm_store_tiles16_as<BF16, 0, AXHIP_OP_RELU>(g, acc, m_base, n_base, coff, l16, g4, stage);
        break;
    case AXHIP_OP_GELU: gemm_store_tiles16_as<BF16, 2, AXHIP_OP_GELU>(g, acc, m_base, n_base, coff, l16, g4, stage); break;
    case AXHIP_OP_SILU: gemm_store_tiles16_as<BF16, 2, AXHIP_OP_SILU>(g, acc, m_base, n_base, coff, l16, g4, stage); break;
    case AXHIP_OP_SIGMOID: gemm_store_tiles16_as<BF16, 2, AXHIP_OP_SIGMOID>(g, acc, m_base, n_base, coff, l16, g4, stage); break;
    case AXHIP_OP_TANH: gemm_store_tiles16_as<BF16, 2, AXHIP_OP_TANH>(g, acc, m_base, n_base, coff, l16, g4, stage); break;
    default:
        if (g.residual) gemm_store_tiles16_as<BF16, 1, 0>(g, acc, m_base, n_base, coff, l16, g4, stage);
        else gemm_store_tiles16_as<BF16, 0, 0>(g, acc, m_base, n_base, coff, l16, g4, stage);
        break;
    }
}

// Requires K % 64 == 0 and 256 * max(lda, ldb) * 2 < 2^31 (checked by the launcher).
template <bool BF16>
__global__ __launch_bounds__(512, 1) void gemm_mfma_nt_256_kernel(const GemmArgs g, const int tiles_m, const int tiles_n) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char big_lds[]; // A0 B0 A1 B1
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int l16 = lane % 16, g4 = lane / 16;

    // work-group -> C tile: XCD x (work-groups x, x+8, ...) owns a contiguous range of the
    // tile order; within it tiles run down groups of 4 tile rows
    const int per_xcd = gridDim.x / 8;
    const int t = (static_cast<int>(blockIdx.x) % 8) * per_xcd + static_cast<int>(blockIdx.x) / 8;
    if (t >= tiles_m * tiles_n) return;
    constexpr int GR = 4;
    const int group = t / (GR * tiles_n), first_m = group * GR;
    const int gsz = min(GR, tiles_m - first_m);
    const int rem = t - group * GR * tiles_n;
    const int tm = first_m + rem % gsz, tn = rem / gsz;
    const int64_t m0 = static_cast<int64_t>(tm) * BIG, n0 = static_cast<int64_t>(tn) * BIG;
    const int64_t bz = blockIdx.y;
    const uint16_t *A = static_cast<const uint16_t *>(g.a) + bz * g.sa + m0 * g.a_rs;
    const uint16_t *B = static_cast<const uint16_t *>(g.b) + bz * g.sb + n0 * g.b_cs;
    const int arow_bytes = static_cast<int>(g.a_rs) * 2, brow_bytes = static_cast<int>(g.b_cs) * 2;
    const int rows_a = static_cast<int>(min<int64_t>(BIG, g.M - m0)), rows_b = static_cast<int>(min<int64_t>(BIG, g.N - n0));
    const int4_t arsrc = gemm_rsrc(A, (rows_a - 1) * arow_bytes + static_cast<int>(g.K) * 2);
    const int4_t brsrc = gemm_rsrc(B, (rows_b - 1) * brow_bytes + static_cast<int>(g.K) * 2);

    // ---- L2 -> LDS mapping: one wave-wide load moves 8 rows of 128 bytes; load n of wave w
    // covers tile rows 64 n + 8 w + (lane >> 3); the lane fetches the chunk that belongs at
    // position lane & 7 of the swizzled row
    const int ld_r = 8 * wave + (lane >> 3);
    const int ld_c = (lane & 7) ^ ((ld_r >> 1) & 7);
    int a_voff[4], b_voff[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        a_voff[n] = (64 * n + ld_r) * arow_bytes + ld_c * 16;
        b_voff[n] = (64 * n + ld_r) * brow_bytes + ld_c * 16;
    }
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(big_lds));
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + 8 * wave * BIG_ROWB);
    auto load_one = [&](const int4_t &ar, const int4_t &br, int kt, int buf, int n) { // n: 0..3 of A, 4..7 of B
        const int soff = kt * BIG_ROWB;
        if (n < 4) gemm_load_to_lds(ar, lds_wave + buf * 2 * BIG_TILEB + n * 64 * BIG_ROWB, a_voff[n % 4], soff);
        else gemm_load_to_lds(br, lds_wave + buf * 2 * BIG_TILEB + BIG_TILEB + (n - 4) * 64 * BIG_ROWB, b_voff[n % 4], soff);
    };

    // ---- fragment reads: row l16 of a 16-row block, 16-byte chunk 4 s + g4 of the row's eight (s: k-step of the tile)
    const int wm = (wave / 4) * 128, wn = (wave % 4) * 64;
    int f_off[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) f_off[s] = l16 * BIG_ROWB + (((4 * s + g4) ^ ((l16 >> 1) & 7)) * 16);

    float4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    uint4_t fa[8], fb[2][4];
    auto read_a = [&](int buf, int s, int i) {
        fa[i] = *reinterpret_cast<const uint4_t *>(big_lds + buf * 2 * BIG_TILEB + (wm + 16 * i) * BIG_ROWB + f_off[s]);
    };
    auto read_b = [&](int slot, int buf, int s, int j) {
        fb[slot][j] = *reinterpret_cast<const uint4_t *>(big_lds + buf * 2 * BIG_TILEB + BIG_TILEB + (wn + 16 * j) * BIG_ROWB + f_off[s]);
    };
    // D = (B fragment) x (A fragment)^T: the lane holds four consecutive columns of one row of C
    auto mfma = [&](int slot, int i, int j) {
        if constexpr (BF16)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, fb[slot][j]), __builtin_bit_cast(bf16x8_t, fa[i]), acc[i][j], 0, 0, 0);
        else
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, fb[slot][j]), __builtin_bit_cast(half8_t, fa[i]), acc[i][j], 0, 0, 0);
    };
#define AXHIP_FENCE() __builtin_amdgcn_sched_barrier(0)

    const int nk = static_cast<int>(g.K / TK);
#pragma unroll
    for (int n = 0; n < 8; ++n) load_one(arsrc, brsrc, 0, 0, n);
    if (nk > 1) {
#pragma unroll
        for (int n = 0; n < 8; ++n) load_one(arsrc, brsrc, 1, 1, n);
        __builtin_amdgcn_s_waitcnt(0x0F78); // vmcnt(8): tile 0 has landed
    } else {
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) read_b(0, 0, 0, j);
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        // past the last tile the loads run on empty descriptors (every lane out of range: zeros into a buffer nobody
        // reads, no memory traffic) rather than behind eight branches
        const bool more = kt + 2 < nk;
        const int4_t ar = int4_t{arsrc.x, arsrc.y, more ? arsrc.z : 0, arsrc.w}, br = int4_t{brsrc.x, brsrc.y, more ? brsrc.z : 0, brsrc.w};
        AXHIP_FENCE();
        // k-step 0: B slot 0; the refills fetch k-step 1 of this tile
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mfma(0, i, j);
                AXHIP_FENCE();
                if (j == 2 && i < 4) {
                    read_b(1, buf, 1, i);
                    AXHIP_FENCE();
                }
                if (j == 3) {
                    read_a(buf, 1, i);
                    AXHIP_FENCE();
                }
            }
        // k-step 1: B slot 1; behind the barrier the refills fetch k-step 0 of the next tile (after the last tile: a
        // harmless read of stale LDS) and this tile's buffer takes the tile after next
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (i == 1) {
                __builtin_amdgcn_s_waitcnt(0x0F70); // this wave's share of tile kt+1 has landed
                __syncthreads();                    // ... everyone's has, and tile kt is no longer read
                AXHIP_FENCE();
                read_a(buf ^ 1, 0, 0);
                AXHIP_FENCE();
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mfma(1, i, j);
                AXHIP_FENCE();
                if (i >= 1) {
                    const int q = (i - 1) * 4 + j; // MFMAs since the barrier
                    if (q % 3 == 1 && q / 3 < 8) {
                        load_one(ar, br, kt + 2, buf, q / 3);
                        AXHIP_FENCE();
                    }
                    if (q % 2 == 0 && q >= 2 && q <= 8) {
                        read_b(0, buf ^ 1, 0, q / 2 - 1);
                        AXHIP_FENCE();
                    }
                    if (j == 3) {
                        read_a(buf ^ 1, 0, i);
                        AXHIP_FENCE();
                    }
                }
            }
        }
    }
#undef AXHIP_FENCE

    // the tile buffers become the staging area of the epilogue: no load of this work-group is still on its way into them
    // (past the last tile they write zeros), and every wave has its last fragments
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    gemm_store_tiles16<BF16>(g, acc, m0 + wm, n0 + wn, bz * g.sc, l16, g4, big_lds + wave * 16384);
}

// --------------------------------------------------- MFMA NT, multi-stage ring
// Mid-size products (too few 256 x 256 tiles to fill the chip): work-group tile TM x TN x 64,
// 4 waves in a 2 x 2 layout, and an S-stage ring of k-tiles in LDS filled by buffer_load ... lds.
// One work-group per CU cannot hide the L2 latency (about 1 us under load) behind a k-tile's
// 0.15 - 0.3 us of MFMA work by occupancy, so S - 1 k-tiles are kept in flight instead and the
// wait before a k-tile is a counted vmcnt that only covers the oldest one.  The k loop is unrolled
// by S so that every stage address is an immediate.  Same LDS row layout and XOR swizzle, same
// tile order over the XCDs and same epilogue as the 256 x 256 kernel.
// Requires K % 64 == 0 and max(TM, TN) * max(lda, ldb) * 2 < 2^31 (checked by the launcher).
template <bool BF16, int TM, int TNR, int S>
__global__ __launch_bounds__(256, 1) void gemm_mfma_nt_ring_kernel(const GemmArgs g, const int tiles_m, const int tiles_n) {
    constexpr int MI = TM / 64, NJ = TNR / 64;       // 32x32 MFMA tiles per wave
    constexpr int NLA = TM / 32, NLB = TNR / 32;      // wave-wide loads (8 rows each) per wave per k-tile
    constexpr int STAGEB = (TM + TNR) * BIG_ROWB;     // bytes per ring stage: A rows, then B rows
    extern __shared__ __attribute__((aligned(1024))) unsigned char big_lds[];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int l32 = lane % 32, g2 = lane / 32;

    const int per_xcd = gridDim.x / 8;
    const int t = (static_cast<int>(blockIdx.x) % 8) * per_xcd + static_cast<int>(blockIdx.x) / 8;
    if (t >= tiles_m * tiles_n) return;
    constexpr int GR = 4;
    const int group = t / (GR * tiles_n), first_m = group * GR;
    const int gsz = min(GR, tiles_m - first_m);
    const int rem = t - group * GR * tiles_n;
    const int tm = first_m + rem % gsz, tn = rem / gsz;
    const int64_t m0 = static_cast<int64_t>(tm) * TM, n0 = static_cast<int64_t>(tn) * TNR;
    const int64_t bz = blockIdx.y;
    const uint16_t *A = static_cast<const uint16_t *>(g.a) + bz * g.sa + m0 * g.a_rs;
    const uint16_t *B = static_cast<const uint16_t *>(g.b) + bz * g.sb + n0 * g.b_cs;
    const int arow_bytes = static_cast<int>(g.a_rs) * 2, brow_bytes = static_cast<int>(g.b_cs) * 2;
    const int rows_a = static_cast<int>(min<int64_t>(TM, g.M - m0)), rows_b = static_cast<int>(min<int64_t>(TNR, g.N - n0));
    const int4_t arsrc = gemm_rsrc(A, (rows_a - 1) * arow_bytes + static_cast<int>(g.K) * 2);
    const int4_t brsrc = gemm_rsrc(B, (rows_b - 1) * brow_bytes + static_cast<int>(g.K) * 2);

    // load n of wave w covers tile rows 32 n + 8 w + (lane >> 3)
    const int ld_r = 8 * wave + (lane >> 3);
    const int ld_c = (lane & 7) ^ ((ld_r >> 1) & 7);
    int a_voff[NLA], b_voff[NLB];
#pragma unroll
    for (int n = 0; n < NLA; ++n) a_voff[n] = (32 * n + ld_r) * arow_bytes + ld_c * 16;
#pragma unroll
    for (int n = 0; n < NLB; ++n) b_voff[n] = (32 * n + ld_r) * brow_bytes + ld_c * 16;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(big_lds));
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + 8 * wave * BIG_ROWB);
    auto load_tile = [&](int kt, int stage) {
        const int soff = kt * BIG_ROWB;
#pragma unroll
        for (int n = 0; n < NLA; ++n) gemm_load_to_lds(arsrc, lds_wave + stage * STAGEB + n * 32 * BIG_ROWB, a_voff[n], soff);
#pragma unroll
        for (int n = 0; n < NLB; ++n) gemm_load_to_lds(brsrc, lds_wave + stage * STAGEB + TM * BIG_ROWB + n * 32 * BIG_ROWB, b_voff[n], soff);
    };

    const int wm = (wave / 2) * (TM / 2), wn = (wave % 2) * (TNR / 2);
    int f_off[TK / 16];
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) f_off[ks] = l32 * BIG_ROWB + (((2 * ks + g2) ^ ((l32 >> 1) & 7)) * 16);

    float16_t acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    uint4_t fa[2][MI], fb[2][NJ];
    auto read_frags = [&](int slot, int stage, int ks) {
        const unsigned char *As = big_lds + stage * STAGEB + wm * BIG_ROWB;
        const unsigned char *Bs = big_lds + stage * STAGEB + (TM + wn) * BIG_ROWB;
#pragma unroll
        for (int j = 0; j < NJ; ++j) fb[slot][j] = *reinterpret_cast<const uint4_t *>(Bs + 32 * j * BIG_ROWB + f_off[ks]);
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[slot][i] = *reinterpret_cast<const uint4_t *>(As + 32 * i * BIG_ROWB + f_off[ks]);
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                if constexpr (BF16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fa[slot][i]), __builtin_bit_cast(bf16x8_t, fb[slot][j]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fa[slot][i]), __builtin_bit_cast(half8_t, fb[slot][j]), acc[i][j], 0, 0, 0);
            }
    };

    const int nk = static_cast<int>(g.K / TK);
    // s_waitcnt vmcnt(N) with the other counters left alone: N = loads of the S - 2 k-tiles that may still be in flight
    constexpr int INFLIGHT = (NLA + NLB) * (S - 2);
    static_assert(INFLIGHT < 64, "vmcnt is a 6-bit counter");
    constexpr int WAIT_OLDEST = (INFLIGHT & 0xF) | 0x0F70 | ((INFLIGHT >> 4) << 14);
#pragma unroll
    for (int st = 0; st < S - 1; ++st)
        if (st < nk) load_tile(st, st);

    // k-tile kt lives in ring stage ST (= kt % S, a compile-time value in the unrolled loop)
    auto step = [&](auto stage_tag, int kt) {
        constexpr int ST = decltype(stage_tag)::value;
        if (kt + S - 2 < nk) __builtin_amdgcn_s_waitcnt(WAIT_OLDEST); // everything older than the S - 2 newest k-tiles has landed
        else __builtin_amdgcn_s_waitcnt(0x0F70);                      // tail: fewer loads behind this one, wait for all
        __syncthreads(); // k-tile kt is complete for every wave, and k-tile kt - 1 (whose stage is refilled next) is no longer read
        if (kt + S - 1 < nk) load_tile(kt + S - 1, (ST + S - 1) % S);
        read_frags(0, ST, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < TK / 16; ++ks) {
            if (ks + 1 < TK / 16) read_frags((ks + 1) & 1, ST, ks + 1);
            __builtin_amdgcn_sched_barrier(0);
            multiply(ks & 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto steps = [&](auto self, auto stage_tag, int kt0) -> void { // step<0>(kt0), step<1>(kt0 + 1), ... step<S-1>
        constexpr int ST = decltype(stage_tag)::value;
        if constexpr (ST < S) {
            if (kt0 + ST < nk) {
                step(stage_tag, kt0 + ST);
                self(self, std::integral_constant<int, ST + 1>{}, kt0);
            }
        }
    };
    for (int kt0 = 0; kt0 < nk; kt0 += S) steps(steps, std::integral_constant<int, 0>{}, kt0);

    gemm_store_tiles<BF16, MI, NJ>(g, acc, m0 + wm, n0 + wn, bz * g.sc, l32, g2);
}

// ------------------------------------------------------------------ fp32, MFMA
// C = A B^T in fp32 on v_mfma_f32_32x32x2_f32 (fp32 products, fp32 accumulation: no precision is given up against
// the FMA kernel), A [M,K] and B [N,K] both K-contiguous.  Same skeleton as the 16-bit ring kernel: a k-tile is 32
// floats, i.e. the same 128-byte LDS rows, XOR swizzle and direct-to-LDS loads; a lane's 16-byte fragment read holds
// four k values that feed four successive MFMAs (which k a lane contributes to which MFMA is free as long as A and B
// agree).  K only has to be a multiple of 4: the chunks of the last k-tile that lie past K are sent out of the
// descriptor's range and arrive as zeros.  At 1/16 of the 16-bit MFMA rate the kernel is bound by the matrix pipe,
// not by the ring.
template <int TM, int TNR, int S>
__global__ __launch_bounds__(256, 1) void gemm_mfma_f32_ring_kernel(const GemmArgs g, const int tiles_m, const int tiles_n) {
    constexpr int MI = TM / 64, NJ = TNR / 64;
    constexpr int NLA = TM / 32, NLB = TNR / 32;
    constexpr int KF = 32;                            // floats per k-tile
    constexpr int STAGEB = (TM + TNR) * BIG_ROWB;
    extern __shared__ __attribute__((aligned(1024))) unsigned char big_lds[];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int l32 = lane % 32, g2 = lane / 32;

    const int per_xcd = gridDim.x / 8;
    const int t = (static_cast<int>(blockIdx.x) % 8) * per_xcd + static_cast<int>(blockIdx.x) / 8;
    if (t >= tiles_m * tiles_n) return;
    constexpr int GR = 4;
    const int group = t / (GR * tiles_n), first_m = group * GR;
    const int gsz = min(GR, tiles_m - first_m);
    const int rem = t - group * GR * tiles_n;
    const int tm = first_m + rem % gsz, tn = rem / gsz;
    const int64_t m0 = static_cast<int64_t>(tm) * TM, n0 = static_cast<int64_t>(tn) * TNR;
    const int64_t bz = blockIdx.y;
    const float *A = static_cast<const float *>(g.a) + bz * g.sa + m0 * g.a_rs;
    const float *B = static_cast<const float *>(g.b) + bz * g.sb + n0 * g.b_cs;
    const int arow_bytes = static_cast<int>(g.a_rs) * 4, brow_bytes = static_cast<int>(g.b_cs) * 4;
    const int rows_a = static_cast<int>(min<int64_t>(TM, g.M - m0)), rows_b = static_cast<int>(min<int64_t>(TNR, g.N - n0));
    const int K = static_cast<int>(g.K);
    const int4_t arsrc = gemm_rsrc(A, (rows_a - 1) * arow_bytes + K * 4);
    const int4_t brsrc = gemm_rsrc(B, (rows_b - 1) * brow_bytes + K * 4);

    const int ld_r = 8 * wave + (lane >> 3);
    const int ld_c = (lane & 7) ^ ((ld_r >> 1) & 7); // source chunk of this lane: floats 4 ld_c .. 4 ld_c + 3 of the k-tile
    int a_voff[NLA], b_voff[NLB];
#pragma unroll
    for (int n = 0; n < NLA; ++n) a_voff[n] = (32 * n + ld_r) * arow_bytes + ld_c * 16;
#pragma unroll
    for (int n = 0; n < NLB; ++n) b_voff[n] = (32 * n + ld_r) * brow_bytes + ld_c * 16;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(big_lds));
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + 8 * wave * BIG_ROWB);
    constexpr int OUT_OF_RANGE = 0x7FFFFFF0;
    auto load_tile = [&](int kt, int stage) {
        const int soff = kt * BIG_ROWB;
        const bool k_ok = kt * KF + ld_c * 4 < K; // false only for the trailing chunks of a ragged last k-tile
#pragma unroll
        for (int n = 0; n < NLA; ++n) gemm_load_to_lds(arsrc, lds_wave + stage * STAGEB + n * 32 * BIG_ROWB, k_ok ? a_voff[n] : OUT_OF_RANGE, soff);
#pragma unroll
        for (int n = 0; n < NLB; ++n) gemm_load_to_lds(brsrc, lds_wave + stage * STAGEB + TM * BIG_ROWB + n * 32 * BIG_ROWB, k_ok ? b_voff[n] : OUT_OF_RANGE, soff);
    };

    const int wm = (wave / 2) * (TM / 2), wn = (wave % 2) * (TNR / 2);
    int f_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) f_off[ks] = l32 * BIG_ROWB + (((2 * ks + g2) ^ ((l32 >> 1) & 7)) * 16);

    float16_t acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    float4_t fa[2][MI], fb[2][NJ];
    auto read_frags = [&](int slot, int stage, int ks) {
        const unsigned char *As = big_lds + stage * STAGEB + wm * BIG_ROWB;
        const unsigned char *Bs = big_lds + stage * STAGEB + (TM + wn) * BIG_ROWB;
#pragma unroll
        for (int j = 0; j < NJ; ++j) fb[slot][j] = *reinterpret_cast<const float4_t *>(Bs + 32 * j * BIG_ROWB + f_off[ks]);
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[slot][i] = *reinterpret_cast<const float4_t *>(As + 32 * i * BIG_ROWB + f_off[ks]);
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[slot][i][c], fb[slot][j][c], acc[i][j], 0, 0, 0);
    };

    const int nk = (K + KF - 1) / KF;
    constexpr int INFLIGHT = (NLA + NLB) * (S - 2);
    static_assert(INFLIGHT < 64, "vmcnt is a 6-bit counter");
    constexpr int WAIT_OLDEST = (INFLIGHT & 0xF) | 0x0F70 | ((INFLIGHT >> 4) << 14);
#pragma unroll
    for (int st = 0; st < S - 1; ++st)
        if (st < nk) load_tile(st, st);

    auto step = [&](auto stage_tag, int kt) {
        constexpr int ST = decltype(stage_tag)::value;
        if (kt + S - 2 < nk) __builtin_amdgcn_s_waitcnt(WAIT_OLDEST);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (kt + S - 1 < nk) load_tile(kt + S - 1, (ST + S - 1) % S);
        read_frags(0, ST, 0);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks + 1 < 4) read_frags((ks + 1) & 1, ST, ks + 1);
            multiply(ks & 1);
        }
    };
    auto steps = [&](auto self, auto stage_tag, int kt0) -> void {
        constexpr int ST = decltype(stage_tag)::value;
        if constexpr (ST < S) {
            if (kt0 + ST < nk) {
                step(stage_tag, kt0 + ST);
                self(self, std::integral_constant<int, ST + 1>{}, kt0);
            }
        }
    };
    for (int kt0 = 0; kt0 < nk; kt0 += S) steps(steps, std::integral_constant<int, 0>{}, kt0);

    // epilogue: accumulator element e of tile (i, j) is C[m + 32 i + 8 (e / 4) + 4 g2 + e % 4][n + 32 j + l32]
    float *Cb = static_cast<float *>(g.c) + bz * g.sc;
    const float *Rb = g.residual ? static_cast<const float *>(g.residual) + bz * g.sc : nullptr;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int64_t col = n0 + wn + 32 * j + l32;
        if (col >= g.N) continue;
        const float bias = g.bias ? static_cast<const float *>(g.bias)[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t row = m0 + wm + 32 * i + 8 * (e / 4) + 4 * g2 + e % 4;
                if (row >= g.M) continue;
                float x = acc[i][j][e] + bias;
                if (Rb) x += Rb[row * g.ldc + col];
                Cb[row * g.ldc + col] = gemm_epilogue(g.epilogue, x);
            }
    }
}

} // namespace axhip

using namespace axhip;

// AXHIP_GEMM_RING=0 routes mid-size products to the register-staged kernels (for A/B timing)
static bool ring_enabled() {
    static const bool on = [] { const char *e = std::getenv("AXHIP_GEMM_RING"); return !(e && e[0] == '0'); }();
    return on;
}

// AXHIP_GEMM_F32_MFMA=0 routes fp32 products to the FMA kernel (for A/B timing)
static bool f32_mfma_enabled() {
    static const bool on = [] { const char *e = std::getenv("AXHIP_GEMM_F32_MFMA"); return !(e && e[0] == '0'); }();
    return on;
}

// AXHIP_GEMM_SKINNY=0: products with at most 8 rows on the tiled kernels (for A/B timing)
static bool skinny_enabled() {
    static const bool on = [] { const char *e = std::getenv("AXHIP_GEMM_SKINNY"); return !(e && e[0] == '0'); }();
    return on;
}

// AXHIP_GEMM_RING_TILE=0..2 forces one ring tile shape (128x128, 64x128, 128x192) for A/B timing
static int ring_tile_override() {
    static const int v = [] { const char *e = std::getenv("AXHIP_GEMM_RING_TILE"); return (e && e[0] >= '0' && e[0] <= '2') ? e[0] - '0' : -1; }();
    return v;
}

namespace {
// whether (and into how many padded columns) a product is repacked before it runs on the k-contiguous kernels
struct Repack { bool on, a, b; int64_t kp; };
Repack repack_plan(const AxhipGemmParams &p) {
    const int64_t kvec = p.dtype == AXHIP_DTYPE_F32 ? 4 : 8;
    const bool pad_k = p.k % kvec != 0;
    Repack r{false, false, false, p.k};
    if ((p.trans_a || !p.trans_b || pad_k) && p.k >= 32 &&
        2.0 * static_cast<double>(p.m) * static_cast<double>(p.n) * static_cast<double>(p.k) * static_cast<double>(p.batch) >= double(1 << 30)) { // (about 70 us on the FMA kernel)
        r.on = true;
        r.kp = pad_k ? (p.k + 63) / 64 * 64 : p.k;
        r.a = p.trans_a || pad_k;
        r.b = !p.trans_b || pad_k;
    }
    return r;
}
size_t repack_bytes(const AxhipGemmParams &p) {
    const Repack r = repack_plan(p);
    if (!r.on) return 0;
    const size_t es = p.dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    size_t n = 0;
    if (r.a) n += CallScratch::rounded(static_cast<size_t>(p.stride_a == 0 ? 1 : p.batch) * p.m * r.kp * es);
    if (r.b) n += CallScratch::rounded(static_cast<size_t>(p.stride_b == 0 ? 1 : p.batch) * p.n * r.kp * es);
    return n;
}
int gemm_impl(const void *a, const void *b, void *c, const AxhipGemmParams *params, CallScratch *scratch_in, void *workspace, size_t workspace_bytes, void *stream);
} // namespace

extern "C" size_t axhip_gemm_workspace_bytes(const AxhipGemmParams *params) {
    if (!params || !valid_dtype(params->dtype) || params->m <= 0 || params->n <= 0 || params->k < 0 || params->batch <= 0) return 0;
    AxhipGemmParams part = *params;
    part.batch = std::min<int64_t>(part.batch, 65535); // larger batches run as consecutive launches that share the workspace
    return repack_bytes(part);
}

extern "C" int axhip_gemm(const void *a, const void *b, void *c, const AxhipGemmParams *params, void *stream) {
    return gemm_impl(a, b, c, params, nullptr, nullptr, 0, stream);
}

extern "C" int axhip_gemm_ws(const void *a, const void *b, void *c, const AxhipGemmParams *params, void *workspace, size_t workspace_bytes, void *stream) {
    return gemm_impl(a, b, c, params, nullptr, workspace, workspace_bytes, stream);
}

namespace {
int gemm_impl(const void *a, const void *b, void *c, const AxhipGemmParams *params, CallScratch *scratch_in, void *workspace, size_t workspace_bytes, void *stream) {
    AXHIP_REQUIRE(params != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_gemm: params is NULL");
    const AxhipGemmParams &p = *params;
    AXHIP_REQUIRE(valid_dtype(p.dtype), AXHIP_ERR_INVALID_ARG, "axhip_gemm: bad dtype %d", p.dtype);
    AXHIP_REQUIRE(p.m >= 0 && p.n >= 0 && p.k >= 0 && p.batch >= 0, AXHIP_ERR_INVALID_ARG, "axhip_gemm: negative extent");
    AXHIP_REQUIRE(p.lda >= 0 && p.ldb >= 0 && p.ldc >= p.n, AXHIP_ERR_INVALID_ARG, "axhip_gemm: bad leading dimension");
    AXHIP_REQUIRE(p.epilogue_op == 0 || p.epilogue_op == AXHIP_OP_RELU || p.epilogue_op == AXHIP_OP_GELU || p.epilogue_op == AXHIP_OP_SILU ||
                      p.epilogue_op == AXHIP_OP_SIGMOID || p.epilogue_op == AXHIP_OP_TANH,
                  AXHIP_ERR_INVALID_ARG, "axhip_gemm: unsupported epilogue op %d", p.epilogue_op);
    if (p.m == 0 || p.n == 0 || p.batch == 0) return AXHIP_OK;
    AXHIP_REQUIRE(a && b && c, AXHIP_ERR_INVALID_ARG, "axhip_gemm: NULL matrix");
    if (p.batch >= 65536) {
        // the batch index is a grid dimension (at most 65 535): a larger batch runs as consecutive launches
        const int64_t es = p.dtype == AXHIP_DTYPE_F32 ? 4 : 2;
        for (int64_t b0 = 0; b0 < p.batch; b0 += 65535) {
            AxhipGemmParams part = p;
            part.batch = std::min<int64_t>(65535, p.batch - b0);
            if (p.residual) part.residual = static_cast<const char *>(p.residual) + b0 * p.stride_c * es;
            const int rc_part = gemm_impl(static_cast<const char *>(a) + b0 * p.stride_a * es, static_cast<const char *>(b) + b0 * p.stride_b * es,
                                          static_cast<char *>(c) + b0 * p.stride_c * es, &part, nullptr, workspace, workspace_bytes, stream);
            if (rc_part) return rc_part;
        }
        return AXHIP_OK;
    }
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);

    // The matrix-core kernels read both operands along k, in 16-byte vectors.  An operand stored the other way (A as
    // [k, m], B as [k, n]: matmul(a, b) with a plain [k, n] right-hand side), or a reduction length that is not a whole
    // number of vectors, leaves only the FMA kernel below, a hundred times slower on a large product.  Such a product
    // is repacked first, into stream-ordered temporary memory (freed in stream order behind the product): the operand
    // that lies the other way is transposed; an unaligned k is zero-padded to the next multiple of 64 in both operands.
    const Repack rp = repack_plan(p);
    if (rp.on && !scratch_in) {
        const bool pad_k = rp.kp != p.k;
        const int64_t es = p.dtype == AXHIP_DTYPE_F32 ? 4 : 2, kp = rp.kp;
        AxhipGemmParams q = p;
        q.k = kp;
        CallScratch scratch(workspace, workspace_bytes, s);
        void *ta = nullptr, *tb = nullptr;
        // a contiguous [copies, rows, kp] image of an operand whose element (row, kk) lies at row * rs + kk * cs
        auto repacked = [&](const void *src, int64_t rows, int64_t rs, int64_t cs, int64_t batch_stride, void **out) -> int {
            const int64_t copies = batch_stride == 0 ? 1 : p.batch;
            const int rc_take = scratch.take(out, static_cast<size_t>(copies * rows * kp * es), "axhip_gemm");
            if (rc_take) return rc_take;
            const int64_t shape[3] = {copies, rows, p.k}, strides[3] = {batch_stride, rs, cs}, before[3] = {0, 0, 0}, after[3] = {0, 0, kp - p.k};
            if (pad_k) return axhip_pad(src, *out, p.dtype, 3, shape, strides, before, after, 0.0, stream);
            return axhip_strided_copy(src, p.dtype, *out, p.dtype, 3, shape, strides, stream);
        };
        if (rp.a) {
            rc = repacked(a, p.m, p.trans_a ? 1 : p.lda, p.trans_a ? p.lda : 1, p.stride_a, &ta);
            q.trans_a = 0; q.lda = kp; q.stride_a = p.stride_a == 0 ? 0 : p.m * kp;
        }
        if (!rc && rp.b) {
            rc = repacked(b, p.n, p.trans_b ? p.ldb : 1, p.trans_b ? 1 : p.ldb, p.stride_b, &tb);
            q.trans_b = 1; q.ldb = kp; q.stride_b = p.stride_b == 0 ? 0 : p.n * kp;
        }
        if (!rc) rc = gemm_impl(ta ? ta : a, tb ? tb : b, c, &q, &scratch, nullptr, 0, stream); // (q is not repacked again)
        const int freed = scratch.release();
        return rc ? rc : freed;
    }

    GemmArgs g{};
    g.a = a; g.b = b; g.c = c; g.bias = p.bias; g.residual = p.residual;
    g.dtype = p.dtype; g.epilogue = p.epilogue_op;
    g.M = p.m; g.N = p.n; g.K = p.k;
    g.a_rs = p.trans_a ? 1 : p.lda; g.a_cs = p.trans_a ? p.lda : 1;
    g.b_rs = p.trans_b ? 1 : p.ldb; g.b_cs = p.trans_b ? p.ldb : 1;
    g.ldc = p.ldc; g.sa = p.stride_a; g.sb = p.stride_b; g.sc = p.stride_c;

    const bool half = p.dtype != AXHIP_DTYPE_F32;
    auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool nt = !p.trans_a && p.trans_b && p.k % 8 == 0 && p.lda % 8 == 0 && p.ldb % 8 == 0 && p.stride_a % 8 == 0 &&
                    p.stride_b % 8 == 0 && al16(a) && al16(b) && p.ldc < (1 << 21);
    // (measured against the tiled kernels, whose k loop costs about 5.5 us per 1024 elements of k whatever N is: one or
    // two rows always win -- 1 x 4096 x 4096 23.2 -> 4.4 us --, up to four while W stays below 48 M elements, up to
    // eight on long-k products of up to 24 M elements; beyond that the per-lane sums make the kernel VALU-bound)
    // (fp32: the tiled fp32 kernels are an order of magnitude off on such shapes -- 1 x 4096 x 4096 138 -> 12 us --, so
    // every product of up to eight rows goes here)
    const int64_t w_elems = p.n * p.k;
    const bool skinny_pays = p.m <= 2 || (p.m <= 8 && p.dtype == AXHIP_DTYPE_F32) || (p.m <= 4 && w_elems <= (int64_t(48) << 20)) ||
                             (p.m <= 8 && p.k >= 2048 && w_elems <= (int64_t(24) << 20));
    const bool f32_nt = p.dtype == AXHIP_DTYPE_F32 && !p.trans_a && p.trans_b && p.k % 4 == 0 && p.lda % 4 == 0 && p.ldb % 4 == 0 && al16(a) && al16(b);
    // (the kernel carries leading dimensions as 32-bit element counts)
    const bool ld32 = p.lda < (int64_t(1) << 31) && p.ldb < (int64_t(1) << 31) && p.ldc < (int64_t(1) << 31);
    if (((half && nt) || f32_nt) && p.batch == 1 && skinny_pays && p.k >= 256 && p.n < (1 << 30) && p.k < (1 << 30) && ld32 && skinny_enabled()) {
        // a decoding step: bound by one read of W
        SkinnyArgs k{};
        k.x = a; k.w = b; k.c = c; k.bias = p.bias; k.residual = p.residual;
        k.dtype = p.dtype; k.epilogue = p.epilogue_op;
        k.N = static_cast<int>(p.n); k.K = static_cast<int>(p.k);
        k.ldx = static_cast<int>(p.lda); k.ldw = static_cast<int>(p.ldb); k.ldc = static_cast<int>(p.ldc);
        // A wavefront per row of W, each lane with four 16-byte pieces of it requested at a time: the fewest rows are
        // streamed at once, each in the longest runs (1 x 16384 x 16384: 88.8 us = 76 % of the HBM peak against
        // 95.2 / 101.2 us with two / four rows per wavefront; 1 x 50304 x 4096: 64.2 against 68.4 / 71.8 us; 1 x 4096 x
        // 4096 from the caches: 4.3 against 6.6 / 7.1 us).  Two rows per wavefront share the reads of x where two or
        // more rows of x meet a large W (2 x 16384 x 16384: 97.4 against 102.7 us).
        // AXHIP_GEMM_SKINNY_ROWS=1|2|4 (read once) forces the count.
        static const int forced_rows = [] { const char *e = std::getenv("AXHIP_GEMM_SKINNY_ROWS"); return e ? std::atoi(e) : 0; }();
        const int rows_per_wave = forced_rows == 1 || forced_rows == 2 || forced_rows == 4 ? forced_rows : (p.m >= 2 && w_elems >= (int64_t(64) << 20)) ? 2 : 1;
        const unsigned blocks = static_cast<unsigned>((p.n + 4 * rows_per_wave - 1) / (4 * rows_per_wave));
        launch_skinny(k, static_cast<int>(p.m), rows_per_wave, blocks, s);
    } else if (half && nt && p.k > 0 && p.k % TK == 0 && p.m >= BIG && p.n >= BIG && p.lda < (1 << 21) && p.ldb < (1 << 21) && p.batch < 65536 &&
        ((p.m + BIG - 1) / BIG) * ((p.n + BIG - 1) / BIG) * p.batch >= 128) {
        // 256 x 256 tiles once they give at least half the CUs a work-group
        const int tiles_m = static_cast<int>((p.m + BIG - 1) / BIG), tiles_n = static_cast<int>((p.n + BIG - 1) / BIG);
        const int per_xcd = (tiles_m * tiles_n + 7) / 8;
        const dim3 grid(static_cast<unsigned>(8 * per_xcd), static_cast<unsigned>(p.batch));
        constexpr size_t lds_bytes = 4 * BIG_TILEB;
        static const bool configured = [] {
            bool ok = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_nt_256_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) == hipSuccess;
            ok = ok && hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_nt_256_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) == hipSuccess;
            return ok;
        }();
        AXHIP_REQUIRE(configured, AXHIP_ERR_UNSUPPORTED, "axhip_gemm: cannot reserve %zu bytes of LDS", lds_bytes);
        if (p.dtype == AXHIP_DTYPE_BF16) hipLaunchKernelGGL((gemm_mfma_nt_256_kernel<true>), grid, dim3(512), lds_bytes, s, g, tiles_m, tiles_n);
        else hipLaunchKernelGGL((gemm_mfma_nt_256_kernel<false>), grid, dim3(512), lds_bytes, s, g, tiles_m, tiles_n);
    } else if (half && nt && p.k > 0 && p.k % TK == 0 && p.k >= 4 * TK && p.lda < (1 << 22) && p.ldb < (1 << 22) && p.batch < 65536 &&
               ring_enabled()) {
        // mid-size: the ring kernels
        const bool bf = p.dtype == AXHIP_DTYPE_BF16;
        auto launch = [&](auto kernel, int tm_rows, int tn_cols, size_t lds_bytes) -> int {
            static std::mutex mu;
            static std::set<const void *> configured;
            {
                std::lock_guard<std::mutex> lk(mu);
                if (!configured.count(reinterpret_cast<const void *>(kernel))) {
                    AXHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
                    configured.insert(reinterpret_cast<const void *>(kernel));
                }
            }
            const int tiles_m = static_cast<int>((p.m + tm_rows - 1) / tm_rows), tiles_n = static_cast<int>((p.n + tn_cols - 1) / tn_cols);
            const int per_xcd = (tiles_m * tiles_n + 7) / 8;
            hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(8 * per_xcd), static_cast<unsigned>(p.batch)), dim3(256), lds_bytes, s, g, tiles_m, tiles_n);
            return AXHIP_OK;
        };
        // Tile shape by modelled time: rounds of work-groups over the 256 CUs x (ring fill and epilogue + the tile's
        // k loop).  The k-loop cost per tile element is calibrated on the Whisper projections (64 x 128 tiles pay 1.4x
        // per element for their lower reuse of the LDS fragments, 128 x 192 tiles 1.13x for their shorter ring).  The
        // wide tile exists because a product such as 1500 x 3840 x 1280 makes 360 tiles of 128 x 128 (two rounds, the
        // second 40 % full) but 240 of 128 x 192.
        struct RingTile { int tm, tn; double per_elem; };
        static const RingTile candidates[] = {{128, 128, 1.0}, {64, 128, 1.42}, {128, 192, 1.13}};
        int best = 0;
        double best_cost = 0.0;
        for (int c = 0; c < 3; ++c) {
            const RingTile &rt = candidates[c];
            if (ring_tile_override() >= 0 && c != ring_tile_override()) continue;
            const int64_t tiles = ((p.m + rt.tm - 1) / rt.tm) * ((p.n + rt.tn - 1) / rt.tn) * p.batch;
            const double rounds = static_cast<double>((tiles + 255) / 256);
            // fixed part: 3 us, in units where a 128 x 128 x 1280 k loop costs 12.25 us
            const double cost = rounds * (3.0 + 12.25 * rt.per_elem * (rt.tm * rt.tn / 16384.0) * (static_cast<double>(p.k) / 1280.0));
            if (best_cost == 0.0 || cost < best_cost) { best_cost = cost; best = c; }
        }
        int rc2;
        switch (best) {
        case 0: rc2 = bf ? launch(gemm_mfma_nt_ring_kernel<true, 128, 128, 4>, 128, 128, 4 * 256 * BIG_ROWB) : launch(gemm_mfma_nt_ring_kernel<false, 128, 128, 4>, 128, 128, 4 * 256 * BIG_ROWB); break;
        case 1: rc2 = bf ? launch(gemm_mfma_nt_ring_kernel<true, 64, 128, 6>, 64, 128, 6 * 192 * BIG_ROWB) : launch(gemm_mfma_nt_ring_kernel<false, 64, 128, 6>, 64, 128, 6 * 192 * BIG_ROWB); break;
        default: rc2 = bf ? launch(gemm_mfma_nt_ring_kernel<true, 128, 192, 4>, 128, 192, 4 * 320 * BIG_ROWB) : launch(gemm_mfma_nt_ring_kernel<false, 128, 192, 4>, 128, 192, 4 * 320 * BIG_ROWB); break; // all 160 KiB of LDS
        }
        if (rc2) return rc2;
    } else if (half && nt && p.k > 0) {
        // Tall tiles (two work-groups per CU, one k-tile in flight) once they fill the chip;
        // otherwise 64-row tiles, one work-group per CU with three k-tiles in flight.
        const int64_t tiles128 = ((p.n + TN - 1) / TN) * ((p.m + 127) / 128) * p.batch;
        const bool bf = p.dtype == AXHIP_DTYPE_BF16;
        if (tiles128 >= 512) {
            dim3 grid(static_cast<unsigned>((p.n + TN - 1) / TN), static_cast<unsigned>((p.m + 127) / 128), static_cast<unsigned>(p.batch));
            if (bf) hipLaunchKernelGGL((gemm_mfma_nt_kernel<true, 128, 1>), grid, dim3(256), 0, s, g);
            else hipLaunchKernelGGL((gemm_mfma_nt_kernel<false, 128, 1>), grid, dim3(256), 0, s, g);
        } else {
            dim3 grid(static_cast<unsigned>((p.n + TN - 1) / TN), static_cast<unsigned>((p.m + 63) / 64), static_cast<unsigned>(p.batch));
            if (bf) hipLaunchKernelGGL((gemm_mfma_nt_kernel<true, 64, 3>), grid, dim3(256), 0, s, g);
            else hipLaunchKernelGGL((gemm_mfma_nt_kernel<false, 64, 3>), grid, dim3(256), 0, s, g);
        }
    } else if (p.dtype == AXHIP_DTYPE_F32 && !p.trans_a && p.trans_b && p.k >= 32 && p.k % 4 == 0 && p.lda % 4 == 0 && p.ldb % 4 == 0 &&
               p.stride_a % 4 == 0 && p.stride_b % 4 == 0 && al16(a) && al16(b) && p.lda < (1 << 21) && p.ldb < (1 << 21) && p.k < (1 << 24) &&
               p.batch < 65536 && p.m * p.n * p.batch >= 64 * 64 * 16 && f32_mfma_enabled()) {
        // fp32 x W^T on the fp32 MFMA; tile shape by rounds of work-groups x tile area (the kernel is bound by the matrix pipe)
        auto launch = [&](auto kernel, int tm_rows, int tn_cols, size_t lds_bytes) -> int {
            static std::mutex mu;
            static std::set<const void *> configured;
            {
                std::lock_guard<std::mutex> lk(mu);
                if (!configured.count(reinterpret_cast<const void *>(kernel))) {
                    AXHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
                    configured.insert(reinterpret_cast<const void *>(kernel));
                }
            }
            const int tiles_m = static_cast<int>((p.m + tm_rows - 1) / tm_rows), tiles_n = static_cast<int>((p.n + tn_cols - 1) / tn_cols);
            const int per_xcd = (tiles_m * tiles_n + 7) / 8;
            hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(8 * per_xcd), static_cast<unsigned>(p.batch)), dim3(256), lds_bytes, s, g, tiles_m, tiles_n);
            return AXHIP_OK;
        };
        static const int shapes[4][2] = {{128, 128}, {64, 128}, {128, 192}, {64, 64}};
        int best = 0;
        double best_cost = 0.0;
        for (int c = 0; c < 4; ++c) {
            const int64_t tiles = ((p.m + shapes[c][0] - 1) / shapes[c][0]) * ((p.n + shapes[c][1] - 1) / shapes[c][1]) * p.batch;
            const double cost = static_cast<double>((tiles + 255) / 256) * (0.05 + shapes[c][0] * shapes[c][1] / 16384.0);
            if (best_cost == 0.0 || cost < best_cost) { best_cost = cost; best = c; }
        }
        int rc2;
        switch (best) {
        case 0: rc2 = launch(gemm_mfma_f32_ring_kernel<128, 128, 3>, 128, 128, 3 * 256 * BIG_ROWB); break;
        case 1: rc2 = launch(gemm_mfma_f32_ring_kernel<64, 128, 3>, 64, 128, 3 * 192 * BIG_ROWB); break;
        case 3: rc2 = launch(gemm_mfma_f32_ring_kernel<64, 64, 3>, 64, 64, 3 * 128 * BIG_ROWB); break;
        default: rc2 = launch(gemm_mfma_f32_ring_kernel<128, 192, 3>, 128, 192, 3 * 320 * BIG_ROWB); break;
        }
        if (rc2) return rc2;
    } else {
        dim3 grid(static_cast<unsigned>((p.n + 15) / 16), static_cast<unsigned>((p.m + 15) / 16), static_cast<unsigned>(p.batch));
        AXHIP_REQUIRE(grid.y < 65536, AXHIP_ERR_UNSUPPORTED, "axhip_gemm: m too large for the generic kernel");
        hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, s, g);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}
} // namespace
