// Strided gather into a contiguous buffer (with dtype conversion) and constant
// fill.  One thread per output element; the output side is fully coalesced.
#include "common.hpp"

#include <algorithm>

namespace axhip {

struct CopyArgs {
    const void *src;
    void *dst;
    int src_dtype, dst_dtype, ndim;
    int64_t total;
    int64_t shape[AXHIP_MAX_DIMS];
    int64_t strides[AXHIP_MAX_DIMS];
};

__global__ __launch_bounds__(256) void strided_copy_kernel(const CopyArgs a) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < a.total; i += stride) {
        int64_t rem = i, off = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const int64_t c = rem % a.shape[d];
            rem /= a.shape[d];
            off += c * a.strides[d];
        }
        store_any(a.dst, a.dst_dtype, i, load_any(a.src, a.src_dtype, off));
    }
}

__global__ __launch_bounds__(256) void fill_kernel(void *dst, int dtype, float value, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) store_any(dst, dtype, i, value);
}

} // namespace axhip

using namespace axhip;

extern "C" {

int axhip_strided_copy(const void *src, int32_t src_dtype, void *dst, int32_t dst_dtype, int32_t ndim,
                       const int64_t *shape, const int64_t *strides, void *stream) {
    AXHIP_REQUIRE(valid_dtype(src_dtype) && valid_dtype(dst_dtype), AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: bad dtype");
    AXHIP_REQUIRE(ndim >= 0 && ndim <= AXHIP_MAX_DIMS, AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: ndim %d out of range", ndim);
    AXHIP_REQUIRE(ndim == 0 || (shape && strides), AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: NULL shape/strides");
    CopyArgs a{};
    a.src = src; a.dst = dst; a.src_dtype = src_dtype; a.dst_dtype = dst_dtype; a.ndim = ndim;
    a.total = 1;
    for (int d = 0; d < ndim; ++d) {
        AXHIP_REQUIRE(shape[d] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: negative extent");
        AXHIP_REQUIRE(strides[d] >= 0, AXHIP_ERR_UNSUPPORTED, "axhip_strided_copy: negative strides (flipped views) are not supported");
        a.shape[d] = shape[d];
        a.strides[d] = strides[d];
        a.total *= shape[d];
    }
    if (a.total == 0) return AXHIP_OK;
    AXHIP_REQUIRE(src && dst, AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
    hipLaunchKernelGGL(strided_copy_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), a);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_fill(void *dst, int32_t dtype, double value, int64_t count, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_fill: bad dtype");
    AXHIP_REQUIRE(count >= 0, AXHIP_ERR_INVALID_ARG, "axhip_fill: negative count");
    if (count == 0) return AXHIP_OK;
    AXHIP_REQUIRE(dst != nullptr, AXHIP_ERR_INVALID_ARG, "axhip_fill: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    const int64_t blocks = std::min<int64_t>((count + 255) / 256, 256 * 64);
    hipLaunchKernelGGL(fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), dst, dtype,
                       static_cast<float>(value), count);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

} // extern "C"
