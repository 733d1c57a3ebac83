// C = op(A) op(B) (+ bias) (+ residual), activation epilogue.
//
//   gemm_mfma_nt_kernel   bf16 / f16, A [M,K] and B [N,K] both K-contiguous (the
//                         nn::Linear case x W^T): v_mfma_f32_32x32x16, workgroup
//                         tile 128x128x64, 4 waves each owning a 64x64 quadrant,
//                         A/B tiles staged through LDS, fp32 accumulation.
//   gemm_generic_kernel   any dtype / any transpose combination, 16x16 LDS tiles,
//                         fp32 FMA.
#include "common.hpp"

#include <algorithm>

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

__device__ __forceinline__ float gemm_epilogue(int op, float x) {
    switch (op) {
    case AXHIP_OP_RELU: return x > 0.0f ? x : 0.0f;
    case AXHIP_OP_GELU: return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
    case AXHIP_OP_SILU: return x / (1.0f + __expf(-x));
    case AXHIP_OP_SIGMOID: return 1.0f / (1.0f + __expf(-x));
    case AXHIP_OP_TANH: return tanhf(x);
    default: return x;
    }
}

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

// ------------------------------------------------------------------- MFMA NT
constexpr int TM = 128, TN = 128, TK = 64;
constexpr int LDS_STRIDE = TK + 8; // 144 B rows: consecutive rows shift by 4 banks (+32)

template <bool BF16>
__global__ __launch_bounds__(256, 2) void gemm_mfma_nt_kernel(const GemmArgs g) {
    __shared__ __attribute__((aligned(16))) uint16_t As[TM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[TN * LDS_STRIDE];
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int l32 = lane % 32, g2 = lane / 32;
    const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;
    const int64_t m0 = static_cast<int64_t>(blockIdx.y) * TM, n0 = static_cast<int64_t>(blockIdx.x) * TN;
    const int64_t bz = blockIdx.z;
    const uint16_t *A = static_cast<const uint16_t *>(g.a) + bz * g.sa;
    const uint16_t *B = static_cast<const uint16_t *>(g.b) + bz * g.sb;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // each thread moves 4 16-byte chunks of A and of B per k-tile: 128 rows x 8 chunks
    uint4_t ra[4], rb[4];
    auto load_tiles = [&](int64_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i;
            const int row = id / 8, cc = id % 8;
            const int64_t k = k0 + 8 * cc;
            ra[i] = uint4_t{0, 0, 0, 0};
            rb[i] = uint4_t{0, 0, 0, 0};
            if (m0 + row < g.M && k < g.K) ra[i] = *reinterpret_cast<const uint4_t *>(A + (m0 + row) * g.a_rs + k);
            if (n0 + row < g.N && k < g.K) rb[i] = *reinterpret_cast<const uint4_t *>(B + (n0 + row) * g.b_cs + k);
        }
    };
    auto stage_tiles = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i;
            const int row = id / 8, cc = id % 8;
            *reinterpret_cast<uint4_t *>(&As[row * LDS_STRIDE + 8 * cc]) = ra[i];
            *reinterpret_cast<uint4_t *>(&Bs[row * LDS_STRIDE + 8 * cc]) = rb[i];
        }
    };

    load_tiles(0);
    for (int64_t k0 = 0; k0 < g.K; k0 += TK) {
        __syncthreads();
        stage_tiles();
        __syncthreads();
        if (k0 + TK < g.K) load_tiles(k0 + TK);
#pragma unroll
        for (int ks = 0; ks < TK / 16; ++ks) {
            uint4_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const uint4_t *>(&As[(wm + 32 * i + l32) * LDS_STRIDE + 16 * ks + 8 * g2]);
                bf[i] = *reinterpret_cast<const uint4_t *>(&Bs[(wn + 32 * i + l32) * LDS_STRIDE + 16 * ks + 8 * g2]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if constexpr (BF16)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, af[i]), __builtin_bit_cast(bf16x8_t, bf[j]), acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, af[i]), __builtin_bit_cast(half8_t, bf[j]), acc[i][j], 0, 0, 0);
                }
        }
    }

    // accumulator element e of tile (i, j): row = 8*(e/4) + 4*g2 + e%4, col = l32
    const int64_t coff = bz * g.sc;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t n = n0 + wn + 32 * j + l32;
            if (n >= g.N) continue;
            const float bias = g.bias ? load_any(g.bias, g.dtype, n) : 0.0f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t m = m0 + wm + 32 * i + 8 * (e / 4) + 4 * g2 + (e % 4);
                if (m >= g.M) continue;
                float x = acc[i][j][e] + bias;
                if (g.residual) x += load_any(g.residual, g.dtype, coff + m * g.ldc + n);
                store_any(g.c, g.dtype, coff + m * g.ldc + n, gemm_epilogue(g.epilogue, x));
            }
        }
}

} // namespace axhip

using namespace axhip;

extern "C" int axhip_gemm(const void *a, const void *b, void *c, const AxhipGemmParams *params, void *stream) {
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
    AXHIP_REQUIRE(p.batch < 65536, AXHIP_ERR_UNSUPPORTED, "axhip_gemm: batch too large");
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);

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
                    p.stride_b % 8 == 0 && al16(a) && al16(b);
    if (half && nt && p.k > 0) {
        dim3 grid(static_cast<unsigned>((p.n + TN - 1) / TN), static_cast<unsigned>((p.m + TM - 1) / TM), static_cast<unsigned>(p.batch));
        if (p.dtype == AXHIP_DTYPE_BF16) hipLaunchKernelGGL(gemm_mfma_nt_kernel<true>, grid, dim3(256), 0, s, g);
        else hipLaunchKernelGGL(gemm_mfma_nt_kernel<false>, grid, dim3(256), 0, s, g);
    } else {
        dim3 grid(static_cast<unsigned>((p.n + 15) / 16), static_cast<unsigned>((p.m + 15) / 16), static_cast<unsigned>(p.batch));
        AXHIP_REQUIRE(grid.y < 65536, AXHIP_ERR_UNSUPPORTED, "axhip_gemm: m too large for the generic kernel");
        hipLaunchKernelGGL(gemm_generic_kernel, grid, dim3(256), 0, s, g);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}
