// Shared by gemm.hip and gemm_skinny.hip: the activation epilogues and the skinny-product launcher.
#pragma once
#include "common.hpp"

namespace axhip {

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

// The same for results that are rounded to a 16-bit type: GELU through the polynomial
// form (|error| <= 5e-5) and tanh through one exponential, both far below the output
// resolution and a fraction of the code of erff / tanhf.
__device__ __forceinline__ float gemm_epilogue16(int op, float x) {
    switch (op) {
    case AXHIP_OP_GELU: return gelu_fast(x);
    case AXHIP_OP_TANH: return 1.0f - 2.0f / (1.0f + __expf(2.0f * x));
    default: return gemm_epilogue(op, x);
    }
}

// x W^T with at most 8 rows of x (a decoding step: one token, or a handful, against a weight matrix), both operands
// along k.  The product is bound by reading W once, and a tiling by output tiles would give the chip N / 128
// work-groups.  Here a wavefront owns R rows of W (R = 1, 2 or 4: enough wavefronts for every SIMD) and walks k with
// its 64 lanes side by side -- every load covers 1 KiB of one row -- keeping M x R fp32 sums per lane
// (16-bit: v_dot2_f32 on the packed pairs, products exact, fp32 accumulation; fp32: FMAs), which the lanes add up at
// the end; lane 0
// applies bias, residual and activation.
struct SkinnyArgs {
    const void *x, *w;
    void *c;
    const void *bias, *residual;
    int dtype, epilogue;
    int N, K, ldx, ldw, ldc;
};

// Launches gemm_skinny_kernel<dtype, m, rows_per_wave> (m = 1..8 rows of x, rows_per_wave = 1, 2 or 4) on `blocks`
// work-groups of four wavefronts.  Defined in gemm_skinny.hip, a translation unit of its own: its 72 kernels take
// longer to compile than every other product kernel together.
void launch_skinny(const SkinnyArgs &k, int m, int rows_per_wave, unsigned blocks, hipStream_t s);

} // namespace axhip
