// ------------------------------------------------------------ skinny products
// x W^T with at most 8 rows of x (a decoding step: one token, or a handful, against a weight matrix), both operands
// along k.  The product is bound by reading W once, and a tiling by output tiles would give the chip N / 128
// work-groups.  Here a wavefront owns R rows of W (R = 1, 2 or 4: enough wavefronts for every SIMD) and walks k with
// its 64 lanes side by side -- every load covers 1 KiB of one row -- keeping M x R fp32 sums per lane
// (16-bit: v_dot2_f32 on the packed pairs, products exact, fp32 accumulation; fp32: FMAs), which the lanes add up at
// the end; lane 0
// applies bias, residual and activation.
#include "gemm_skinny.hpp"

namespace axhip {

// acc + the dot product of two 16-byte vectors of DT elements (fp32: four FMAs)
template <int DT> __device__ __forceinline__ float dot16b(const uint4_t &a, const uint4_t &b, float acc) {
    const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (DT == AXHIP_DTYPE_F32) {
            acc = __builtin_fmaf(__uint_as_float(aw[i]), __uint_as_float(bw[i]), acc);
        } else if constexpr (DT == AXHIP_DTYPE_BF16) {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, aw[i]), __builtin_bit_cast(bf16x2_t, bw[i]), acc, false);
        } else {
            typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, aw[i]), __builtin_bit_cast(half2_t, bw[i]), acc, false);
        }
    }
    return acc;
}

template <int DT, int M, int R>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const SkinnyArgs a) {
    constexpr int E = DT == AXHIP_DTYPE_F32 ? 4 : 8, ES = 16 / E; // elements per 16-byte vector, bytes per element
    const int lane = threadIdx.x % 64;
    const int n0 = (blockIdx.x * 4 + threadIdx.x / 64) * R;
    if (n0 >= a.N) return; // (whole wavefronts)
    float acc[M][R];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    const char *wrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) wrow[r] = static_cast<const char *>(a.w) + static_cast<int64_t>(min(n0 + r, a.N - 1)) * a.ldw * ES; // (rows past N: the last row again, not stored)
    constexpr int U = R == 1 ? 4 : R == 2 ? 2 : 1; // k steps requested together: U * R loads of W in flight per lane
    for (int k0 = lane * E; k0 < a.K; k0 += 64 * E * U) {
        uint4_t wf[U][R], xf[U][M];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + 64 * E * u;
            const bool inside = k < a.K; // (K is a multiple of E)
#pragma unroll
            for (int r = 0; r < R; ++r) wf[u][r] = inside ? *reinterpret_cast<const uint4_t *>(wrow[r] + static_cast<int64_t>(k) * ES) : uint4_t{0, 0, 0, 0};
#pragma unroll
            for (int m = 0; m < M; ++m)
                xf[u][m] = inside ? *reinterpret_cast<const uint4_t *>(static_cast<const char *>(a.x) + (static_cast<int64_t>(m) * a.ldx + k) * ES) : uint4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) acc[m][r] = dot16b<DT>(wf[u][r], xf[u][m], acc[m][r]);
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float v = acc[m][r];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, WAVE);
            const int n = n0 + r;
            if (lane == 0 && n < a.N) {
                if (a.bias) v += load_any(a.bias, a.dtype, n);
                if (a.residual) v += load_any(a.residual, a.dtype, static_cast<int64_t>(m) * a.ldc + n);
                store_any(a.c, a.dtype, static_cast<int64_t>(m) * a.ldc + n, gemm_epilogue(a.epilogue, v));
            }
        }
}

void launch_skinny(const SkinnyArgs &k, int m, int rows_per_wave, unsigned blocks, hipStream_t s) {
#define AXHIP_SKINNY_R(M, R)                                                                                              \
    do {                                                                                                                  \
        if (k.dtype == AXHIP_DTYPE_BF16) hipLaunchKernelGGL((gemm_skinny_kernel<AXHIP_DTYPE_BF16, M, R>), dim3(blocks), dim3(256), 0, s, k); \
        else if (k.dtype == AXHIP_DTYPE_F16) hipLaunchKernelGGL((gemm_skinny_kernel<AXHIP_DTYPE_F16, M, R>), dim3(blocks), dim3(256), 0, s, k); \
        else hipLaunchKernelGGL((gemm_skinny_kernel<AXHIP_DTYPE_F32, M, R>), dim3(blocks), dim3(256), 0, s, k);           \
    } while (0)
#define AXHIP_SKINNY(M)                                                                                                   \
    do {                                                                                                                  \
        if (rows_per_wave == 4) AXHIP_SKINNY_R(M, 4);                                                                     \
        else if (rows_per_wave == 2) AXHIP_SKINNY_R(M, 2);                                                                \
        else AXHIP_SKINNY_R(M, 1);                                                                                        \
    } while (0)
    switch (m) { // (x's row count is a template constant: the sums live in registers)
    case 1: AXHIP_SKINNY(1); break;
    case 2: AXHIP_SKINNY(2); break;
    case 3: AXHIP_SKINNY(3); break;
    case 4: AXHIP_SKINNY(4); break;
    case 5: AXHIP_SKINNY(5); break;
    case 6: AXHIP_SKINNY(6); break;
    case 7: AXHIP_SKINNY(7); break;
    default: AXHIP_SKINNY(8); break;
    }
#undef AXHIP_SKINNY
#undef AXHIP_SKINNY_R
}

} // namespace axhip
