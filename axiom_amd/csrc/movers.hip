// Strided gather into a contiguous buffer (with dtype conversion), constant fill,
// constant padding, masked fill and embedding-row gather.  One thread per output
// element (16 bytes per thread for the row gather); the output side is fully coalesced.
#include "common.hpp"

#include <algorithm>
#include <climits>
#include <cstdint>

namespace axhip {

struct CopyArgs {
    const void *src;
    void *dst;
    int src_dtype, dst_dtype, ndim;
    int64_t total;
    int64_t shape[AXHIP_MAX_DIMS];
    int64_t strides[AXHIP_MAX_DIMS];
};

// IDX: int32_t when every index and offset fits (32-bit divisions cost a fraction of the 64-bit ones)
template <typename IDX>
__global__ __launch_bounds__(256) void strided_copy_kernel(const CopyArgs a) {
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, total = static_cast<IDX>(a.total);
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        IDX rem = i, off = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const IDX n = static_cast<IDX>(a.shape[d]);
            const IDX q = rem / n;
            off += (rem - q * n) * static_cast<IDX>(a.strides[d]);
            rem = q;
        }
        store_any(a.dst, a.dst_dtype, i, load_any(a.src, a.src_dtype, off));
    }
}

// Views whose innermost dimension is contiguous (head splits, slices, broadcasts of rows, plain casts): one thread
// moves V consecutive elements with 16-byte accesses; a.shape[ndim-1] counts such groups and a.strides[ndim-1] is V.
// RAW: same dtype on both sides, the bytes are moved as they are.
template <typename IDX, int V, bool RAW>
__global__ __launch_bounds__(256) void strided_copy_vec_kernel(const CopyArgs a) {
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, total = static_cast<IDX>(a.total);
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        IDX rem = i, off = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const IDX n = static_cast<IDX>(a.shape[d]);
            const IDX q = rem / n;
            off += (rem - q * n) * static_cast<IDX>(a.strides[d]);
            rem = q;
        }
        if constexpr (RAW) { // V elements = 16 bytes
            const int es = a.src_dtype == AXHIP_DTYPE_F32 ? 4 : 2;
            const uint4_t t = *reinterpret_cast<const uint4_t *>(static_cast<const char *>(a.src) + static_cast<int64_t>(off) * es);
            reinterpret_cast<uint4_t *>(a.dst)[i] = t;
        } else {
            float v[V];
            load_vec<V>(a.src, a.src_dtype, off, v);
            store_vec<V>(a.dst, a.dst_dtype, static_cast<int64_t>(i) * V, v);
        }
    }
}

// Views whose innermost (destination) dimension is strided in the source while another dimension J is contiguous
// there: transposes.  A work-group moves a 64 x 64 tile of (J, innermost) through LDS, so the reads run along J and
// the writes along the innermost dimension, both in full lines; the remaining dimensions select the tile's origin.
struct TransposeArgs {
    const void *src;
    void *dst;
    int src_dtype, dst_dtype, n_other;
    int64_t nJ, nL, src_stride_l, dst_stride_j; // the source stride of J and the destination stride of L are 1
    int64_t tiles_j, tiles_l;
    int64_t oshape[AXHIP_MAX_DIMS], osrc[AXHIP_MAX_DIMS], odst[AXHIP_MAX_DIMS];
};

__global__ __launch_bounds__(256) void transpose_copy_kernel(const TransposeArgs a) {
    __shared__ float tile[64][65];
    int64_t b = blockIdx.x;
    const int64_t tl = b % a.tiles_l;
    b /= a.tiles_l;
    const int64_t tj = b % a.tiles_j;
    int64_t o = b / a.tiles_j;
    int64_t src_base = 0, dst_base = 0;
    for (int d = a.n_other - 1; d >= 0; --d) {
        const int64_t c = o % a.oshape[d];
        o /= a.oshape[d];
        src_base += c * a.osrc[d];
        dst_base += c * a.odst[d];
    }
    const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
    const int64_t j0 = tj * 64, l0 = tl * 64;
#pragma unroll 4
    for (int r = ty; r < 64; r += 4) {
        const int64_t l = l0 + r, j = j0 + tx;
        if (l < a.nL && j < a.nJ) tile[r][tx] = load_any(a.src, a.src_dtype, src_base + l * a.src_stride_l + j);
    }
    __syncthreads();
#pragma unroll 4
    for (int r = ty; r < 64; r += 4) {
        const int64_t j = j0 + r, l = l0 + tx;
        if (l < a.nL && j < a.nJ) store_any(a.dst, a.dst_dtype, dst_base + j * a.dst_stride_j + l, tile[tx][r]);
    }
}

__global__ __launch_bounds__(256) void fill_kernel(void *dst, int dtype, float value, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) store_any(dst, dtype, i, value);
}

struct PadArgs {
    const void *src;
    void *dst;
    int dtype, ndim;
    int64_t total;
    float value;
    int64_t out_shape[AXHIP_MAX_DIMS], src_shape[AXHIP_MAX_DIMS], src_strides[AXHIP_MAX_DIMS], before[AXHIP_MAX_DIMS];
};

__global__ __launch_bounds__(256) void pad_kernel(const PadArgs a) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < a.total; i += stride) {
        int64_t rem = i, off = 0;
        bool inside = true;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const int64_t c = rem % a.out_shape[d] - a.before[d];
            rem /= a.out_shape[d];
            inside = inside && c >= 0 && c < a.src_shape[d];
            off += c * a.src_strides[d];
        }
        store_any(a.dst, a.dtype, i, inside ? load_any(a.src, a.dtype, off) : a.value);
    }
}

struct MaskedFillArgs {
    const void *src;
    const uint8_t *mask;
    void *dst;
    int dtype, ndim;
    int64_t total;
    float value;
    int64_t shape[AXHIP_MAX_DIMS], src_strides[AXHIP_MAX_DIMS], mask_strides[AXHIP_MAX_DIMS];
};

__global__ __launch_bounds__(256) void masked_fill_kernel(const MaskedFillArgs a) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < a.total; i += stride) {
        int64_t rem = i, soff = 0, moff = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const int64_t c = rem % a.shape[d];
            rem /= a.shape[d];
            soff += c * a.src_strides[d];
            moff += c * a.mask_strides[d];
        }
        store_any(a.dst, a.dtype, i, a.mask[moff] ? a.value : load_any(a.src, a.dtype, soff));
    }
}

// One thread moves `chunk` bytes (16, or the element size when rows are not 16-byte
// multiples) of one output row.
template <typename V>
__global__ __launch_bounds__(256) void gather_rows_kernel(const V *table, int64_t table_rows, int64_t row_chunks, const void *indices,
                                                           int index_bytes, int64_t n_indices, V *dst) {
    const int64_t total = n_indices * row_chunks, stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / row_chunks, c = i - r * row_chunks;
        const int64_t idx = index_bytes == 8 ? static_cast<const int64_t *>(indices)[r] : static_cast<const int32_t *>(indices)[r];
        V v{};
        if (idx >= 0 && idx < table_rows) v = table[idx * row_chunks + c];
        dst[i] = v;
    }
}

// ------------------------------------------------------------- argmax / argmin
// Index of the extreme along the middle extent of an (outer, axis, inner) view, with the scan's rule of the CPU path:
// start at index 0 with the type's lowest() (argmin: max()) as the value to beat, move on a strict comparison -- the
// first occurrence of the extreme wins, a NaN never does, a slice with nothing beyond the start value answers 0.
// A candidate is (value, index); "no candidate yet" carries index INT32_MAX, so that among equal values the lower
// index wins and the start value loses to a real element of the same value only by the strict comparison.
struct ArgBest {
    float v;
    int32_t i;
};
template <bool MIN> __device__ __forceinline__ void arg_take(ArgBest &b, float v, int32_t i) { // i increases along a thread's scan
    if (MIN ? v < b.v : v > b.v) {
        b.v = v;
        b.i = i;
    }
}
template <bool MIN> __device__ __forceinline__ void arg_merge(ArgBest &b, float v, int32_t i) { // candidates in any order
    if ((MIN ? v < b.v : v > b.v) || (v == b.v && i < b.i)) {
        b.v = v;
        b.i = i;
    }
}
template <bool MIN> __device__ __forceinline__ void arg_merge_wave(ArgBest &b) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float v = __shfl_xor(b.v, d, WAVE);
        const int32_t i = __shfl_xor(b.i, d, WAVE);
        arg_merge<MIN>(b, v, i);
    }
}

// inner == 1: a row per wavefront (THREADS = 64, four rows per work-group) or per work-group of 1024 threads.  A row
// starts wherever rows * cols puts it: elements up to the next 16-byte boundary and behind the last whole vector are
// read one by one, the body as 16-byte vectors.
template <bool MIN, int THREADS>
__global__ __launch_bounds__(THREADS == 64 ? 256 : THREADS) void argreduce_rows_kernel(const void *src, int dt, int64_t rows, int64_t cols, float start, int64_t *dst) {
    constexpr int RPB = THREADS == 64 ? 4 : 1;
    __shared__ float sv[THREADS == 64 ? 1 : THREADS / 64];
    __shared__ int32_t si[THREADS == 64 ? 1 : THREADS / 64];
    const int t = THREADS == 64 ? threadIdx.x % 64 : threadIdx.x;
    const int es = dt == AXHIP_DTYPE_F32 ? 4 : 2, E = 16 / es;
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * RPB + (THREADS == 64 ? threadIdx.x / 64 : 0); row < rows; row += static_cast<int64_t>(gridDim.x) * RPB) {
        const int64_t base = row * cols;
        const uintptr_t addr = reinterpret_cast<uintptr_t>(src) + static_cast<uintptr_t>(base) * es;
        const int64_t head = min(cols, static_cast<int64_t>(((16 - (addr & 15u)) & 15u) / es));
        const int64_t nvec = (cols - head) / E, tail0 = head + nvec * E;
        ArgBest b{start, INT32_MAX};
        if (t < head) arg_take<MIN>(b, load_any(src, dt, base + t), t);
        for (int64_t c = t; c < nvec; c += THREADS) {
            const int64_t at = head + c * E;
            if (es == 4) {
                float v[4];
                load_vec<4>(src, dt, base + at, v);
#pragma unroll
                for (int e = 0; e < 4; ++e) arg_take<MIN>(b, v[e], static_cast<int32_t>(at + e));
            } else {
                float v[8];
                load_vec<8>(src, dt, base + at, v);
#pragma unroll
                for (int e = 0; e < 8; ++e) arg_take<MIN>(b, v[e], static_cast<int32_t>(at + e));
            }
        }
        if (tail0 + t < cols) arg_take<MIN>(b, load_any(src, dt, base + tail0 + t), static_cast<int32_t>(tail0 + t));
        arg_merge_wave<MIN>(b);
        if constexpr (THREADS > 64) {
            const int w = threadIdx.x / 64;
            __syncthreads(); // the previous row's partials have been read
            if (threadIdx.x % 64 == 0) {
                sv[w] = b.v;
                si[w] = b.i;
            }
            __syncthreads();
            if (threadIdx.x == 0)
                for (int k = 1; k < THREADS / 64; ++k) arg_merge<MIN>(b, sv[k], si[k]);
        }
        if (t == 0) dst[row] = b.i == INT32_MAX ? 0 : b.i;
    }
}

// inner > 1: a thread per (outer, inner) position walks the axis; neighbouring threads read neighbouring addresses.
template <bool MIN>
__global__ __launch_bounds__(256) void argreduce_strided_kernel(const void *src, int dt, int64_t outer, int64_t axis, int64_t inner, float start, int64_t *dst) {
    const int64_t total = outer * inner;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; p < total; p += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t o = p / inner, i = p - o * inner;
        const int64_t first = o * axis * inner + i;
        ArgBest b{start, INT32_MAX};
        int64_t k = 0;
        for (; k + 4 <= axis; k += 4) { // four loads in flight per thread
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = load_any(src, dt, first + (k + u) * inner);
#pragma unroll
            for (int u = 0; u < 4; ++u) arg_take<MIN>(b, v[u], static_cast<int32_t>(k + u));
        }
        for (; k < axis; ++k) arg_take<MIN>(b, load_any(src, dt, first + k * inner), static_cast<int32_t>(k));
        dst[p] = b.i == INT32_MAX ? 0 : b.i;
    }
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
    hipStream_t s = resolve_stream(stream);

    // drop unit dimensions and merge neighbours that are contiguous in the source: fewer divisions per element
    int nd = 0;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] == 1) continue;
        if (nd > 0 && a.strides[nd - 1] == strides[d] * shape[d]) {
            a.shape[nd - 1] *= shape[d];
            a.strides[nd - 1] = strides[d];
        } else {
            a.shape[nd] = shape[d];
            a.strides[nd] = strides[d];
            ++nd;
        }
    }
    a.ndim = nd;
    int64_t max_off = 0;
    for (int d = 0; d < nd; ++d) max_off += (a.shape[d] - 1) * a.strides[d];
    const bool idx32 = a.total < (int64_t(1) << 31) - (1 << 23) && max_off < (int64_t(1) << 31) - (1 << 23); // room for the grid stride

    // vector path: innermost dimension contiguous and every row start aligned to the vector
    const bool raw = src_dtype == dst_dtype;
    const int v = raw ? (src_dtype == AXHIP_DTYPE_F32 ? 4 : 8) : (dst_dtype == AXHIP_DTYPE_F32 ? 4 : 8);
    const int src_es = src_dtype == AXHIP_DTYPE_F32 ? 4 : 2, dst_es = dst_dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    const int src_align = src_es == 4 ? 16 : v * 2; // bytes a vector load needs
    bool vec = nd >= 1 && a.strides[nd - 1] == 1 && a.shape[nd - 1] % v == 0 && reinterpret_cast<uintptr_t>(src) % src_align == 0 &&
               reinterpret_cast<uintptr_t>(dst) % (v * dst_es >= 16 ? 16 : 8) == 0;
    for (int d = 0; vec && d + 1 < nd; ++d) vec = (a.strides[d] * src_es) % src_align == 0;
    // transposes: the innermost dimension is strided, some other dimension is contiguous in the source
    int transpose_j = -1;
    if (!vec && nd >= 2 && a.strides[nd - 1] > 1 && a.shape[nd - 1] >= 16) {
        for (int d = 0; d + 1 < nd; ++d)
            if (a.strides[d] == 1 && a.shape[d] >= 16) transpose_j = d;
    }
    if (vec) {
        a.shape[nd - 1] /= v;
        a.strides[nd - 1] = v;
        a.total /= v;
        const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
        const dim3 grid(static_cast<unsigned>(blocks));
        auto launch = [&](auto idx_tag) {
            using IDX = decltype(idx_tag);
            if (raw && v == 4) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 4, true>), grid, dim3(256), 0, s, a);
            else if (raw) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 8, true>), grid, dim3(256), 0, s, a);
            else if (v == 4) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 4, false>), grid, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 8, false>), grid, dim3(256), 0, s, a);
        };
        if (idx32) launch(int32_t{});
        else launch(int64_t{});
    } else if (transpose_j >= 0) {
        TransposeArgs t{};
        t.src = src; t.dst = dst; t.src_dtype = src_dtype; t.dst_dtype = dst_dtype;
        const int L = nd - 1, J = transpose_j;
        t.nJ = a.shape[J]; t.nL = a.shape[L];
        t.src_stride_l = a.strides[L];
        t.tiles_j = (t.nJ + 63) / 64; t.tiles_l = (t.nL + 63) / 64;
        int64_t dst_stride = 1, blocks = t.tiles_j * t.tiles_l;
        int no = 0;
        int64_t dst_strides[AXHIP_MAX_DIMS]; // of the contiguous output
        for (int d = nd - 1; d >= 0; --d) {
            dst_strides[d] = dst_stride;
            dst_stride *= a.shape[d];
        }
        t.dst_stride_j = dst_strides[J];
        for (int d = 0; d < nd; ++d) {
            if (d == J || d == L) continue;
            t.oshape[no] = a.shape[d];
            t.osrc[no] = a.strides[d];
            t.odst[no] = dst_strides[d];
            blocks *= a.shape[d];
            ++no;
        }
        t.n_other = no;
        AXHIP_REQUIRE(blocks < (int64_t(1) << 31), AXHIP_ERR_UNSUPPORTED, "axhip_strided_copy: view too large");
        hipLaunchKernelGGL(transpose_copy_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, t);
    } else {
        const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
        const dim3 grid(static_cast<unsigned>(blocks));
        if (idx32) hipLaunchKernelGGL((strided_copy_kernel<int32_t>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((strided_copy_kernel<int64_t>), grid, dim3(256), 0, s, a);
    }
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

int axhip_pad(const void *src, void *dst, int32_t dtype, int32_t ndim, const int64_t *src_shape, const int64_t *src_strides,
              const int64_t *pad_before, const int64_t *pad_after, double value, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_pad: bad dtype");
    AXHIP_REQUIRE(ndim >= 1 && ndim <= AXHIP_MAX_DIMS, AXHIP_ERR_INVALID_ARG, "axhip_pad: ndim %d out of range", ndim);
    AXHIP_REQUIRE(src_shape && src_strides && pad_before && pad_after, AXHIP_ERR_INVALID_ARG, "axhip_pad: NULL shape/strides/pads");
    PadArgs a{};
    a.src = src; a.dst = dst; a.dtype = dtype; a.ndim = ndim; a.value = static_cast<float>(value);
    a.total = 1;
    int64_t src_total = 1;
    for (int d = 0; d < ndim; ++d) {
        AXHIP_REQUIRE(src_shape[d] >= 0 && pad_before[d] >= 0 && pad_after[d] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_pad: negative extent or pad");
        AXHIP_REQUIRE(src_strides[d] >= 0, AXHIP_ERR_UNSUPPORTED, "axhip_pad: negative strides (flipped views) are not supported");
        a.src_shape[d] = src_shape[d];
        a.src_strides[d] = src_strides[d];
        a.before[d] = pad_before[d];
        a.out_shape[d] = src_shape[d] + pad_before[d] + pad_after[d];
        a.total *= a.out_shape[d];
        src_total *= src_shape[d];
    }
    if (a.total == 0) return AXHIP_OK;
    AXHIP_REQUIRE(dst && (src || src_total == 0), AXHIP_ERR_INVALID_ARG, "axhip_pad: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
    hipLaunchKernelGGL(pad_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), a);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_masked_fill(const void *src, int32_t dtype, const uint8_t *mask, void *dst, int32_t ndim, const int64_t *shape,
                      const int64_t *src_strides, const int64_t *mask_strides, double value, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_masked_fill: bad dtype");
    AXHIP_REQUIRE(ndim >= 0 && ndim <= AXHIP_MAX_DIMS, AXHIP_ERR_INVALID_ARG, "axhip_masked_fill: ndim %d out of range", ndim);
    AXHIP_REQUIRE(ndim == 0 || (shape && src_strides && mask_strides), AXHIP_ERR_INVALID_ARG, "axhip_masked_fill: NULL shape/strides");
    MaskedFillArgs a{};
    a.src = src; a.mask = mask; a.dst = dst; a.dtype = dtype; a.ndim = ndim; a.value = static_cast<float>(value);
    a.total = 1;
    for (int d = 0; d < ndim; ++d) {
        AXHIP_REQUIRE(shape[d] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_masked_fill: negative extent");
        AXHIP_REQUIRE(src_strides[d] >= 0 && mask_strides[d] >= 0, AXHIP_ERR_UNSUPPORTED, "axhip_masked_fill: negative strides are not supported");
        a.shape[d] = shape[d];
        a.src_strides[d] = src_strides[d];
        a.mask_strides[d] = mask_strides[d];
        a.total *= shape[d];
    }
    if (a.total == 0) return AXHIP_OK;
    AXHIP_REQUIRE(src && mask && dst, AXHIP_ERR_INVALID_ARG, "axhip_masked_fill: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
    hipLaunchKernelGGL(masked_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), a);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_gather_rows(const void *table, int32_t dtype, int64_t table_rows, int64_t row_elems, const void *indices, int32_t index_bytes,
                      int64_t n_indices, void *dst, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_gather_rows: bad dtype");
    AXHIP_REQUIRE(index_bytes == 4 || index_bytes == 8, AXHIP_ERR_INVALID_ARG, "axhip_gather_rows: index_bytes must be 4 or 8");
    AXHIP_REQUIRE(table_rows >= 0 && row_elems >= 0 && n_indices >= 0, AXHIP_ERR_INVALID_ARG, "axhip_gather_rows: negative extent");
    if (n_indices == 0 || row_elems == 0) return AXHIP_OK;
    AXHIP_REQUIRE(indices && dst && (table || table_rows == 0), AXHIP_ERR_INVALID_ARG, "axhip_gather_rows: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    const int64_t esz = dtype == AXHIP_DTYPE_F32 ? 4 : 2, row_bytes = row_elems * esz;
    const bool wide = row_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(table) & 15u) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0;
    const int64_t chunks = wide ? row_bytes / 16 : row_elems;
    const int64_t blocks = std::min<int64_t>((n_indices * chunks + 255) / 256, 256 * 64);
    hipStream_t s = resolve_stream(stream);
    if (wide)
        hipLaunchKernelGGL(gather_rows_kernel<uint4_t>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, static_cast<const uint4_t *>(table),
                           table_rows, chunks, indices, index_bytes, n_indices, static_cast<uint4_t *>(dst));
    else if (esz == 4)
        hipLaunchKernelGGL(gather_rows_kernel<uint32_t>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, static_cast<const uint32_t *>(table),
                           table_rows, chunks, indices, index_bytes, n_indices, static_cast<uint32_t *>(dst));
    else
        hipLaunchKernelGGL(gather_rows_kernel<uint16_t>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, static_cast<const uint16_t *>(table),
                           table_rows, chunks, indices, index_bytes, n_indices, static_cast<uint16_t *>(dst));
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_argreduce(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t want_min, int64_t *dst, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_argreduce: bad dtype");
    AXHIP_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, AXHIP_ERR_INVALID_ARG, "axhip_argreduce: negative extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    AXHIP_REQUIRE(axis > 0, AXHIP_ERR_INVALID_ARG, "axhip_argreduce: an empty axis has no extreme");
    AXHIP_REQUIRE(axis < (int64_t(1) << 31) - 1, AXHIP_ERR_UNSUPPORTED, "axhip_argreduce: axis of %lld elements (indices are held in 32 bits)", static_cast<long long>(axis));
    AXHIP_REQUIRE(src && dst, AXHIP_ERR_INVALID_ARG, "axhip_argreduce: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);
    // lowest() of the element type (argmin: max()): the value the first element has to beat
    const float lowest = dtype == AXHIP_DTYPE_F32 ? -3.402823466e+38f : dtype == AXHIP_DTYPE_F16 ? -65504.0f : -3.3895313892515355e+38f;
    const float start = want_min ? -lowest : lowest;
    if (inner == 1) {
        const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
        if (axis * es <= 16384) {
            const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer + 3) / 4, 256 * 32));
            if (want_min) hipLaunchKernelGGL((argreduce_rows_kernel<true, 64>), dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, start, dst);
            else hipLaunchKernelGGL((argreduce_rows_kernel<false, 64>), dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, start, dst);
        } else {
            const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(outer, 256 * 8));
            if (want_min) hipLaunchKernelGGL((argreduce_rows_kernel<true, 1024>), dim3(blocks), dim3(1024), 0, s, src, dtype, outer, axis, start, dst);
            else hipLaunchKernelGGL((argreduce_rows_kernel<false, 1024>), dim3(blocks), dim3(1024), 0, s, src, dtype, outer, axis, start, dst);
        }
    } else {
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer * inner + 255) / 256, 256 * 32));
        if (want_min) hipLaunchKernelGGL(argreduce_strided_kernel<true>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, start, dst);
        else hipLaunchKernelGGL(argreduce_strided_kernel<false>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, start, dst);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

} // extern "C"
