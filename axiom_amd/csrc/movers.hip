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
// RAW: same dtype on both sides, the bytes are moved as they are.  UNALIGNED: the groups start anywhere in the source
// (a column slice from an odd column, the windows of a convolution): unaligned 16-byte loads, aligned stores.
template <typename IDX, int V, bool RAW, bool UNALIGNED = false>
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
            const uint4_t t = vec_load<UNALIGNED>(reinterpret_cast<const uint4_t *>(static_cast<const char *>(a.src) + static_cast<int64_t>(off) * es));
            reinterpret_cast<uint4_t *>(a.dst)[i] = t;
        } else {
            float v[V];
            load_vec<V, UNALIGNED>(a.src, a.src_dtype, off, v);
            store_vec<V>(a.dst, a.dst_dtype, static_cast<int64_t>(i) * V, v);
        }
    }
}

// Every other element of the source's innermost dimension (x[:, ::2], the windows of a stride-2 convolution), same type
// on both sides: a group of V results comes out of two unaligned 16-byte loads -- the second one starts an element
// early, so that it ends with the group's last picked element and nothing behind the view is touched -- with the
// wanted elements picked in registers, and leaves as one aligned 16-byte store.  a.shape[ndim-1] counts groups,
// a.strides[ndim-1] is 2 V.  HALF: groups of half a vector (rows of 1500 16-bit results: 8-byte loads and stores).
template <typename IDX, int ES, bool HALF>
__global__ __launch_bounds__(256) void strided_copy_every_other_kernel(const CopyArgs a) {
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, total = static_cast<IDX>(a.total);
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        IDX rem = i, off = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const IDX n = static_cast<IDX>(a.shape[d]);
            const IDX q = rem / n;
            off += (rem - q * n) * static_cast<IDX>(a.strides[d]);
            rem = q;
        }
        const char *p = static_cast<const char *>(a.src) + static_cast<int64_t>(off) * ES;
        if constexpr (HALF) {
            const uint2_t lo = vec_load<true>(reinterpret_cast<const uint2_t *>(p)), hi = vec_load<true>(reinterpret_cast<const uint2_t *>(p + 8 - ES));
            uint2_t t;
            if constexpr (ES == 4) t = uint2_t{lo.x, hi.y};
            else t = uint2_t{__builtin_amdgcn_perm(lo.y, lo.x, 0x05040100u), __builtin_amdgcn_perm(hi.y, hi.x, 0x07060302u)};
            reinterpret_cast<uint2_t *>(a.dst)[i] = t;
            continue;
        }
        const uint4_t lo = vec_load<true>(reinterpret_cast<const uint4_t *>(p));            // elements 0 .. V - 1
        const uint4_t hi = vec_load<true>(reinterpret_cast<const uint4_t *>(p + 16 - ES)); // elements V - 1 .. 2 V - 2
        uint4_t t;
        if constexpr (ES == 4) {
            t = uint4_t{lo.x, lo.z, hi.y, hi.w};
        } else { // lo: the low halves of consecutive words; hi (an element late): the high halves
            t = uint4_t{__builtin_amdgcn_perm(lo.y, lo.x, 0x05040100u), __builtin_amdgcn_perm(lo.w, lo.z, 0x05040100u),
                        __builtin_amdgcn_perm(hi.y, hi.x, 0x07060302u), __builtin_amdgcn_perm(hi.w, hi.z, 0x07060302u)};
        }
        reinterpret_cast<uint4_t *>(a.dst)[i] = t;
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

// The same for views that move whole 16-byte vectors on both sides (equal 2- or 4-byte element types; extents, strides
// and bases multiples of a vector -- or of half a vector on a side, LG / SG = 8: that side moves 8-byte pieces, e.g. the
// 3000-byte rows of a [.., 1500] 16-bit array): tiles of 16 x 16 vectors -- 128 x 128 16-bit or 64 x 64 32-bit
// elements, 256-byte runs on the read and on the write side.  A thread reads vectors along J, scatters their elements as 32-bit words into
// a tile that is stored transposed (16-bit: two neighbouring rows of L packed into one word first), and the tile
// leaves as 16-byte LDS reads along L.  Tile rows are 256 bytes = 16 chunks; chunk c of row j sits at c ^ (j / V mod 16),
// which spreads the words of one scatter over all 64 banks and keeps the 16 reads of a row apart.
template <int ES, int LG, int SG>
__global__ __launch_bounds__(256) void transpose_vec_kernel(const TransposeArgs a) {
    constexpr int V = 16 / ES, T = 16 * V; // elements per vector, tile edge
    // 16 bytes at `at`, of which the elements below `n` exist (whole pieces of LG bytes)
    auto load16 = [](const char *at, int64_t n) {
        if constexpr (LG == 16) {
            return n > 0 ? *reinterpret_cast<const uint4_t *>(at) : uint4_t{0, 0, 0, 0};
        } else {
            const uint2_t lo = n > 0 ? *reinterpret_cast<const uint2_t *>(at) : uint2_t{0, 0};
            const uint2_t hi = n > V / 2 ? *reinterpret_cast<const uint2_t *>(at + 8) : uint2_t{0, 0};
            return uint4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    __shared__ __attribute__((aligned(16))) uint32_t tile[T * 64];
    int64_t b = blockIdx.x;
    const int64_t tl = b % a.tiles_l;
    b /= a.tiles_l;
    // (work-groups that run side by side take tiles along a diagonal: with a power of two as row length, tiles of one
    // tile row or column start a multiple of 2 MiB apart on one of the two sides and would queue on the same channels)
    const int64_t tj = (b % a.tiles_j + tl) % a.tiles_j;
    int64_t o = b / a.tiles_j;
    int64_t src_base = 0, dst_base = 0;
    for (int d = a.n_other - 1; d >= 0; --d) {
        const int64_t c = o % a.oshape[d];
        o /= a.oshape[d];
        src_base += c * a.osrc[d];
        dst_base += c * a.odst[d];
    }
    const int tid = threadIdx.x, jv = tid % 16, hi = tid / 16;
    const int64_t j0 = tj * T, l0 = tl * T;
    const char *src = static_cast<const char *>(a.src);
    char *dst = static_cast<char *>(a.dst);
    const int64_t j_left = a.nJ - (j0 + jv * V); // elements of this thread's vectors that exist (whole pieces)
    if constexpr (ES == 2) {
        // pairs of rows: pair p = rows 2p, 2p + 1 of the tile; four per thread
        uint4_t r0[4], r1[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int64_t l = l0 + 2 * (hi + 16 * it);
            const int64_t at = (src_base + l * a.src_stride_l + j0 + jv * V) * ES;
            r0[it] = load16(src + at, l < a.nL ? j_left : 0);
            r1[it] = load16(src + at + a.src_stride_l * ES, l + 1 < a.nL ? j_left : 0);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int p = hi + 16 * it; // the pair's word: chunk p / 4, word p % 4 of row j
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const uint32_t w0 = r0[it][e / 2], w1 = r1[it][e / 2];
                const uint32_t word = e % 2 ? __builtin_amdgcn_perm(w1, w0, 0x07060302u) : __builtin_amdgcn_perm(w1, w0, 0x05040100u);
                tile[(jv * V + e) * 64 + (((p / 4) ^ jv) * 4) + p % 4] = word;
            }
        }
    } else {
        uint4_t r[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int64_t l = l0 + hi + 16 * it;
            r[it] = load16(src + (src_base + l * a.src_stride_l + j0 + jv * V) * ES, l < a.nL ? j_left : 0);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int l = hi + 16 * it;
#pragma unroll
            for (int e = 0; e < V; ++e) tile[(jv * V + e) * 64 + (((l / 4) ^ jv) * 4) + l % 4] = r[it][e];
        }
    }
    __syncthreads();
    // rows j of the transposed tile, 16 vectors along L each
    const int lv = tid % 16;
    const int64_t l_left = a.nL - (l0 + lv * V);
#pragma unroll
    for (int it = 0; it < T / 16; ++it) {
        const int j = hi + 16 * it;
        const uint4_t t = *reinterpret_cast<const uint4_t *>(&tile[j * 64 + ((lv ^ ((j / V) & 15)) * 4)]);
        char *to = dst + (dst_base + (j0 + j) * a.dst_stride_j + l0 + lv * V) * ES;
        if (j0 + j >= a.nJ) continue;
        if constexpr (SG == 16) {
            if (l_left > 0) *reinterpret_cast<uint4_t *>(to) = t;
        } else {
            if (l_left > 0) *reinterpret_cast<uint2_t *>(to) = uint2_t{t.x, t.y};
            if (l_left > V / 2) *reinterpret_cast<uint2_t *>(to + 8) = uint2_t{t.z, t.w};
        }
    }
}

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
    int mode; // AXHIP_PAD_*
    int64_t out_shape[AXHIP_MAX_DIMS], src_shape[AXHIP_MAX_DIMS], src_strides[AXHIP_MAX_DIMS], before[AXHIP_MAX_DIMS];
};

// Source coordinate of output coordinate c (already shifted by the leading pad) along an extent of n elements, -1
// where the constant goes.  Reflection leaves the border element out (… 2 1 | 0 1 2 … n-1 | n-2 n-3 …); the host
// has checked that a reflected pad is shorter than the extent, so one fold is enough.
template <typename IDX>
__device__ __forceinline__ IDX pad_source(IDX c, IDX n, int mode) {
    if (c >= 0 && c < n) return c;
    switch (mode) {
    case AXHIP_PAD_REFLECT: return c < 0 ? -c : 2 * n - c - 2;
    case AXHIP_PAD_REPLICATE: return c < 0 ? 0 : n - 1;
    case AXHIP_PAD_CIRCULAR: {
        const IDX m = c % n;
        return m < 0 ? m + n : m;
    }
    default: return -1;
    }
}

__global__ __launch_bounds__(256) void pad_kernel(const PadArgs a) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < a.total; i += stride) {
        int64_t rem = i, off = 0;
        bool inside = true;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const int64_t c = pad_source<int64_t>(rem % a.out_shape[d] - a.before[d], a.src_shape[d], a.mode);
            rem /= a.out_shape[d];
            inside = inside && c >= 0;
            off += c * a.src_strides[d];
        }
        store_any(a.dst, a.dtype, i, inside ? load_any(a.src, a.dtype, off) : a.value);
    }
}

// V elements of a constant pad's output row from source coordinate c0 on, for rows of V contiguous elements or more:
// the elements inside [0, n) come out of one unaligned 16-byte load placed inside the row and shifted into place in
// registers (the result is 16 of the 48 bytes constant | load | constant); the rest are the constant f.
template <typename IDX, int V>
__device__ __forceinline__ uint4_t pad_const_group(const char *row, IDX c0, IDX n, uint32_t f) {
    constexpr int ES = 16 / V;
    if (c0 + V <= 0 || c0 >= n) return uint4_t{f, f, f, f};
    const IDX at = c0 < 0 ? 0 : c0 > n - V ? n - V : c0;
    const uint4_t w = reinterpret_cast<const uint4_unaligned_t *>(row + static_cast<int64_t>(at) * ES)->v;
    if (at == c0) return w;
    const int b = 16 - static_cast<int>(at - c0) * ES, k = b >> 2, r = b & 3; // 0 < b < 32
    auto word = [&](int i) { return i == 4 ? w.x : i == 5 ? w.y : i == 6 ? w.z : i == 7 ? w.w : f; };
    uint32_t d[5];
#pragma unroll
    for (int j = 0; j < 5; ++j) d[j] = word(k + j);
    return uint4_t{__builtin_amdgcn_alignbyte(d[1], d[0], r), __builtin_amdgcn_alignbyte(d[2], d[1], r),
                   __builtin_amdgcn_alignbyte(d[3], d[2], r), __builtin_amdgcn_alignbyte(d[4], d[3], r)};
}

// The same with V consecutive elements of the innermost output dimension per thread (V elements are 16 bytes): one
// decomposition of the index per V elements.  A group whose sources are a run of the innermost source dimension --
// the interior, a wrapped-around run of a circular pad, or, backwards, the mirror image of a reflected pad -- is one
// 16-byte load and one 16-byte store (2- or 4-byte aligned: rows start wherever the extents put them); the groups on
// a border, a row's last, shorter group and strided sources go element by element.
// FLAT (output rows that are not whole groups, in an aligned output): the groups are the aligned 16-byte pieces of the
// whole output instead of pieces counted from each row's start, so that every store is aligned; a group that runs
// over a row's end goes element by element, the rest of it in the next row.
// IDX: int32_t when every index and offset fits.
template <typename IDX, int V, bool FLAT = false>
__global__ __launch_bounds__(256) void pad_vec_kernel(const PadArgs a) {
    const int L = a.ndim - 1;
    const IDX out_last = static_cast<IDX>(a.out_shape[L]), inner = (out_last + V - 1) / V;
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, n_rows = static_cast<IDX>(a.total / out_last);
    const IDX groups = FLAT ? static_cast<IDX>((a.total + V - 1) / V) : n_rows * inner;
    const IDX before = static_cast<IDX>(a.before[L]), n_src = static_cast<IDX>(a.src_shape[L]), st = static_cast<IDX>(a.src_strides[L]);
    constexpr int ES = 16 / V;
    uint4_t fill; // V copies of the constant in the element type
    if constexpr (V == 4) {
        fill = uint4_t{__float_as_uint(a.value), __float_as_uint(a.value), __float_as_uint(a.value), __float_as_uint(a.value)};
    } else {
        const uint32_t h = a.dtype == AXHIP_DTYPE_BF16 ? pack_bf16x2(a.value, a.value) : pack_f16x2(a.value, a.value);
        fill = uint4_t{h, h, h, h};
    }
    const bool rows_aligned = FLAT || (out_last % V == 0 && (reinterpret_cast<uintptr_t>(a.dst) & 15u) == 0); // every group's 16 bytes of output are aligned
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < groups; i += stride) {
        IDX row, col; // where the group starts
        if constexpr (FLAT) {
            row = i * V / out_last;
            col = i * V - row * out_last;
        } else {
            row = i / inner;
            col = (i - row * inner) * V;
        }
        IDX off = 0;
        const IDX c0 = col - before;
        const int nvalid = static_cast<int>(out_last - col < V ? out_last - col : V); // elements of the group in this row
        bool inside = true;
        auto outer = [&](IDX rem) { // the source offset of an output row, or that all of it is padding
            off = 0;
            inside = true;
            for (int d = L - 1; d >= 0; --d) {
                const IDX n = static_cast<IDX>(a.out_shape[d]);
                const IDX q = rem / n;
                const IDX c = pad_source<IDX>(rem - q * n - static_cast<IDX>(a.before[d]), static_cast<IDX>(a.src_shape[d]), a.mode);
                rem = q;
                inside = inside && c >= 0;
                off += c * static_cast<IDX>(a.src_strides[d]);
            }
        };
        outer(row);
        const int64_t out_index = static_cast<int64_t>(row) * out_last + static_cast<int64_t>(col);
        if (a.mode == AXHIP_PAD_CONSTANT && st == 1 && n_src >= V && (nvalid == V || (FLAT && row + 1 < n_rows))) {
            // constant pads of contiguous rows: every group, borders included, is one load (two where the group runs
            // over a row's end in a flat output) and one store
            const char *src = static_cast<const char *>(a.src);
            uint4_t w = inside ? pad_const_group<IDX, V>(src + static_cast<int64_t>(off) * ES, c0, n_src, fill.x) : fill;
            if (nvalid < V) {
                outer(row + 1);
                const uint4_t u = inside ? pad_const_group<IDX, V>(src + static_cast<int64_t>(off) * ES, -static_cast<IDX>(nvalid) - before, n_src, fill.x) : fill;
                const uint32_t wa[4] = {w.x, w.y, w.z, w.w}, ua[4] = {u.x, u.y, u.z, u.w};
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (V == 4) o[j] = j < nvalid ? wa[j] : ua[j];
                    else o[j] = ((2 * j < nvalid ? wa[j] : ua[j]) & 0xffffu) | ((2 * j + 1 < nvalid ? wa[j] : ua[j]) & 0xffff0000u);
                }
                w = uint4_t{o[0], o[1], o[2], o[3]};
            }
            char *out = static_cast<char *>(a.dst) + out_index * ES;
            if (rows_aligned) *reinterpret_cast<uint4_t *>(out) = w;
            else reinterpret_cast<uint4_unaligned_t *>(out)->v = w;
            continue;
        }
        if (nvalid == V && a.mode == AXHIP_PAD_CONSTANT && (!inside || c0 + V <= 0 || c0 >= n_src)) { // nothing but the constant
            char *out = static_cast<char *>(a.dst) + out_index * ES;
            if (rows_aligned) *reinterpret_cast<uint4_t *>(out) = fill;
            else reinterpret_cast<uint4_unaligned_t *>(out)->v = fill;
            continue;
        }
        if (inside && st == 1 && nvalid == V) {
            const IDX first = pad_source<IDX>(c0, n_src, a.mode), last = pad_source<IDX>(c0 + V - 1, n_src, a.mode);
            const bool forward = first >= 0 && last - first == V - 1, backward = last >= 0 && first - last == V - 1;
            if (forward || backward) {
                uint4_t w = reinterpret_cast<const uint4_unaligned_t *>(static_cast<const char *>(a.src) + (static_cast<int64_t>(off) + (forward ? first : last)) * ES)->v;
                if (backward) {
                    if constexpr (V == 4) w = uint4_t{w.w, w.z, w.y, w.x};
                    else w = uint4_t{(w.w >> 16) | (w.w << 16), (w.z >> 16) | (w.z << 16), (w.y >> 16) | (w.y << 16), (w.x >> 16) | (w.x << 16)};
                }
                char *out = static_cast<char *>(a.dst) + out_index * ES;
                if (rows_aligned) *reinterpret_cast<uint4_t *>(out) = w;
                else reinterpret_cast<uint4_unaligned_t *>(out)->v = w;
                continue;
            }
        }
        if (rows_aligned && nvalid == V) {
            float v[V];
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const IDX c = pad_source<IDX>(c0 + e, n_src, a.mode);
                v[e] = inside && c >= 0 ? load_any(a.src, a.dtype, off + c * st) : a.value;
            }
            store_vec<V>(a.dst, a.dtype, out_index, v);
            continue;
        }
        if constexpr (FLAT) { // the rest of the group is the start of the next row (rows hold V elements or more)
            if (row + 1 < n_rows) {
                float v[V]; // all loads first, one store
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const IDX c = pad_source<IDX>(c0 + e, n_src, a.mode);
                    if (e < nvalid) v[e] = inside && c >= 0 ? load_any(a.src, a.dtype, off + c * st) : a.value;
                }
                outer(row + 1);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const IDX c = pad_source<IDX>(e - nvalid - before, n_src, a.mode);
                    if (e >= nvalid) v[e] = inside && c >= 0 ? load_any(a.src, a.dtype, off + c * st) : a.value;
                }
                store_vec<V>(a.dst, a.dtype, out_index, v);
                continue;
            }
        }
        for (int e = 0; e < nvalid; ++e) {
            const IDX c = pad_source<IDX>(c0 + e, n_src, a.mode);
            store_any(a.dst, a.dtype, out_index + e, inside && c >= 0 ? load_any(a.src, a.dtype, off + c * st) : a.value);
        }
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

// The same over views whose innermost dimension is contiguous in the source and contiguous or broadcast in the mask
// (an attention mask over [batch, heads, queries, keys], a key-padding mask that repeats over the queries): one
// thread takes 16 bytes of the source and the 16 / ES mask bytes that go with them (one byte when the mask repeats
// along the row), picks per element in registers and stores 16 bytes.  a.shape[ndim-1] counts such groups;
// a.src_strides[ndim-1] is 16 / ES and a.mask_strides[ndim-1] is 16 / ES or 0.
template <typename IDX, int ES>
__global__ __launch_bounds__(256) void masked_fill_vec_kernel(const MaskedFillArgs a) {
    constexpr int V = 16 / ES;
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, total = static_cast<IDX>(a.total);
    uint32_t fill;
    if constexpr (ES == 4) fill = __float_as_uint(a.value);
    else fill = a.dtype == AXHIP_DTYPE_F16 ? f32_to_f16_bits(a.value) & 0xffffu : f32_to_bf16_bits(a.value) & 0xffffu;
    const bool mask_row = a.mask_strides[a.ndim - 1] != 0;
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        IDX rem = i, soff = 0, moff = 0;
        for (int d = a.ndim - 1; d >= 0; --d) {
            const IDX n = static_cast<IDX>(a.shape[d]);
            const IDX q = rem / n, c = rem - q * n;
            soff += c * static_cast<IDX>(a.src_strides[d]);
            moff += c * static_cast<IDX>(a.mask_strides[d]);
            rem = q;
        }
        uint4_t t = *reinterpret_cast<const uint4_t *>(static_cast<const char *>(a.src) + static_cast<int64_t>(soff) * ES);
        uint32_t m[2]; // the group's mask bytes, one per element
        if (mask_row) {
            if constexpr (V == 8) {
                const uint2_t mm = *reinterpret_cast<const uint2_t *>(a.mask + moff);
                m[0] = mm.x; m[1] = mm.y;
            } else {
                m[0] = *reinterpret_cast<const uint32_t *>(a.mask + moff); m[1] = 0;
            }
        } else {
            m[0] = m[1] = a.mask[moff] ? 0x01010101u : 0u;
        }
        uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if constexpr (ES == 4) {
                if ((m[0] >> (8 * k)) & 0xffu) w[k] = fill;
            } else {
                const uint32_t mk = m[k >> 1] >> (16 * (k & 1));
                if (mk & 0xffu) w[k] = (w[k] & 0xffff0000u) | fill;
                if (mk & 0xff00u) w[k] = (w[k] & 0x0000ffffu) | (fill << 16);
            }
        }
        t.x = w[0]; t.y = w[1]; t.z = w[2]; t.w = w[3];
        reinterpret_cast<uint4_t *>(a.dst)[i] = t;
    }
}

// where(cond, a, b): dst[i] = cond[i] ? a[i] : b[i] over an iteration space of up to 8 dimensions; the three inputs
// are strided views (stride 0 on broadcast dimensions), each of a type of its own; dst is contiguous.
struct WhereArgs {
    const void *cond, *a, *b;
    void *dst;
    int cond_dtype, a_dtype, b_dtype, dst_dtype, ndim;
    int64_t total;
    int64_t shape[AXHIP_MAX_DIMS], cond_strides[AXHIP_MAX_DIMS], a_strides[AXHIP_MAX_DIMS], b_strides[AXHIP_MAX_DIMS];
};

__global__ __launch_bounds__(256) void where_kernel(const WhereArgs w) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < w.total; i += stride) {
        int64_t rem = i, coff = 0, aoff = 0, boff = 0;
        for (int d = w.ndim - 1; d >= 0; --d) {
            const int64_t c = rem % w.shape[d];
            rem /= w.shape[d];
            coff += c * w.cond_strides[d];
            aoff += c * w.a_strides[d];
            boff += c * w.b_strides[d];
        }
        const bool pick = load_any(w.cond, w.cond_dtype, coff) != 0.0f;
        store_any(w.dst, w.dst_dtype, i, pick ? load_any(w.a, w.a_dtype, aoff) : load_any(w.b, w.b_dtype, boff));
    }
}

// the three inputs contiguous and of the output's extent (a and b may each be one broadcast element): V elements
// per thread, every access a whole vector
template <int V>
__global__ __launch_bounds__(256) void where_vec_kernel(const WhereArgs w, const bool a_scalar, const bool b_scalar) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256, chunks = w.total / V;
    const float a0 = a_scalar ? load_any(w.a, w.a_dtype, 0) : 0.0f, b0 = b_scalar ? load_any(w.b, w.b_dtype, 0) : 0.0f;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; c < chunks; c += stride) {
        float m[V], x[V], y[V];
        load_vec<V>(w.cond, w.cond_dtype, c * V, m);
        if (!a_scalar) load_vec<V>(w.a, w.a_dtype, c * V, x);
        if (!b_scalar) load_vec<V>(w.b, w.b_dtype, c * V, y);
#pragma unroll
        for (int e = 0; e < V; ++e) x[e] = m[e] != 0.0f ? (a_scalar ? a0 : x[e]) : (b_scalar ? b0 : y[e]);
        store_vec<V>(w.dst, w.dst_dtype, c * V, x);
    }
}

// Views whose innermost dimension each input either runs along or repeats over (a mask over [queries, keys] against
// [batch, heads, queries, keys] scores, a row vector, a column of per-row values): one thread takes V consecutive
// elements of a row -- a vector load from the inputs that run along it, one element from those that repeat -- and
// stores them as whole vectors.  w.shape[ndim-1] counts such groups; the inputs' strides there are V or 0.
template <typename IDX, int V>
__global__ __launch_bounds__(256) void where_rows_kernel(const WhereArgs w) {
    const int L = w.ndim - 1;
    const bool c_row = w.cond_strides[L] != 0, a_row = w.a_strides[L] != 0, b_row = w.b_strides[L] != 0;
    const IDX stride = static_cast<IDX>(gridDim.x) * 256, total = static_cast<IDX>(w.total);
    for (IDX i = static_cast<IDX>(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
        IDX rem = i, coff = 0, aoff = 0, boff = 0;
        for (int d = L; d >= 0; --d) {
            const IDX n = static_cast<IDX>(w.shape[d]);
            const IDX q = rem / n, c = rem - q * n;
            rem = q;
            coff += c * static_cast<IDX>(w.cond_strides[d]);
            aoff += c * static_cast<IDX>(w.a_strides[d]);
            boff += c * static_cast<IDX>(w.b_strides[d]);
        }
        float m[V], x[V], y[V];
        if (c_row) load_vec<V>(w.cond, w.cond_dtype, coff, m);
        else m[0] = load_any(w.cond, w.cond_dtype, coff);
        if (a_row) load_vec<V>(w.a, w.a_dtype, aoff, x);
        else x[0] = load_any(w.a, w.a_dtype, aoff);
        if (b_row) load_vec<V>(w.b, w.b_dtype, boff, y);
        else y[0] = load_any(w.b, w.b_dtype, boff);
        const float m0 = m[0], x0 = x[0], y0 = y[0];
#pragma unroll
        for (int e = 0; e < V; ++e) x[e] = (c_row ? m[e] : m0) != 0.0f ? (a_row ? x[e] : x0) : (b_row ? y[e] : y0);
        store_vec<V>(w.dst, w.dst_dtype, static_cast<int64_t>(i) * V, x);
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
// the E = 16 / sizeof(element) values of one 16-byte vector, as fp32
template <int DT> __device__ __forceinline__ void arg_unpack(const uint4_t raw, float (&v)[DT == AXHIP_DTYPE_F32 ? 4 : 8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if constexpr (DT == AXHIP_DTYPE_F32) {
            v[k] = __uint_as_float(w[k]);
        } else if constexpr (DT == AXHIP_DTYPE_BF16) {
            v[2 * k] = __uint_as_float(w[k] << 16);
            v[2 * k + 1] = __uint_as_float(w[k] & 0xFFFF0000u);
        } else {
            v[2 * k] = f16_bits_to_f32(w[k] & 0xFFFFu);
            v[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
        }
    }
}

// inner == 1.  THREADS = 64: `lanes` (a power of two up to 64) lanes of a wavefront per row, 64 / lanes rows per
// wavefront and four wavefronts per work-group; THREADS = 256 / 1024: a work-group per row.  A row starts wherever
// rows * cols puts it: elements up to the next 16-byte boundary and behind the last whole vector are read one by
// one, the body as 16-byte vectors, four of them requested before the first is looked at (a vector past the row's
// last one is fetched again from the last and not looked at: no branch between the loads).
template <bool MIN, int THREADS, int DT>
__global__ __launch_bounds__(THREADS == 64 ? 256 : THREADS) void argreduce_rows_kernel(const void *src, int64_t rows, int64_t cols, int lanes, float start, int64_t *dst) {
    constexpr int U = 4, E = DT == AXHIP_DTYPE_F32 ? 4 : 8, ES = 16 / E;
    __shared__ float sv[THREADS == 64 ? 1 : THREADS / 64];
    __shared__ int32_t si[THREADS == 64 ? 1 : THREADS / 64];
    const int span = THREADS == 64 ? lanes : THREADS;                 // threads per row
    const int t = THREADS == 64 ? threadIdx.x % lanes : threadIdx.x;  // position among them
    const int rpb = THREADS == 64 ? 256 / lanes : 1;                  // rows per work-group and sweep
    for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * rpb; row0 < rows; row0 += static_cast<int64_t>(gridDim.x) * rpb) {
        const int64_t row = row0 + (THREADS == 64 ? threadIdx.x / lanes : 0);
        const bool there = row < rows; // (a wavefront's lanes stay together for the exchanges below)
        const int64_t base = there ? row * cols : 0;
        const uintptr_t addr = reinterpret_cast<uintptr_t>(src) + static_cast<uintptr_t>(base) * ES;
        const int head = static_cast<int>(min(cols, static_cast<int64_t>(((16 - (addr & 15u)) & 15u) / ES)));
        const int nvec = there ? static_cast<int>((cols - head) / E) : 0, tail0 = head + nvec * E;
        const uint4_t *vec = reinterpret_cast<const uint4_t *>(addr + static_cast<uintptr_t>(head) * ES);
        ArgBest b{start, INT32_MAX};
        if (there)
            for (int h = t; h < head; h += span) arg_take<MIN>(b, load_any(src, DT, base + h), h); // (up to E - 1 of them)
        for (int c = t; c < nvec; c += span * U) {
            uint4_t raw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) raw[u] = vec[min(c + u * span, nvec - 1)];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int cc = c + u * span;
                if (cc < nvec) {
                    float v[E];
                    arg_unpack<DT>(raw[u], v);
#pragma unroll
                    for (int e = 0; e < E; ++e) arg_take<MIN>(b, v[e], head + cc * E + e);
                }
            }
        }
        if (there)
            for (int64_t h = tail0 + t; h < cols; h += span) arg_take<MIN>(b, load_any(src, DT, base + h), static_cast<int32_t>(h));
        // lanes of one row are neighbours: exchanges at distances below the row's span stay inside it
        for (int d = min(span, 64) >> 1; d >= 1; d >>= 1) {
            const float v = __shfl_xor(b.v, d, WAVE);
            const int32_t i = __shfl_xor(b.i, d, WAVE);
            arg_merge<MIN>(b, v, i);
        }
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
        if (there && t == 0) dst[row] = b.i == INT32_MAX ? 0 : b.i;
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

// inner > 1 with inner a multiple of the 16-byte vector and an aligned base: a thread owns the E neighbouring inner
// positions of one vector, TX such threads side by side read TX * 16 consecutive bytes, and the TY = 256 / TX thread
// rows of a work-group share the axis (k = ty, ty + TY, ..), merging through LDS at the end.  TX = 32 when that
// still gives the chip a thousand work-groups, else 8 (whole 128-byte lines still).
// part_v / part_i (both or neither): instead of the answer, the candidate of every position -- its value and its index
// within this axis segment, INT32_MAX for none -- for argreduce_merge_kernel.
template <bool MIN, int DT, int TX>
__global__ __launch_bounds__(256) void argreduce_strided_vec_kernel(const void *src, int64_t outer, int64_t axis, int64_t inner, float start, int64_t *dst,
                                                                    float *part_v, int32_t *part_i) {
    constexpr int TY = 256 / TX, U = 4, V = DT == AXHIP_DTYPE_F32 ? 4 : 8;
    __shared__ float sv[TY][TX][V + 1];
    __shared__ int32_t si[TY][TX][V + 1];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t ivecs = inner / V, groups = (ivecs + TX - 1) / TX, total = outer * groups;
    const int n = static_cast<int>(axis);
    for (int64_t g = blockIdx.x; g < total; g += gridDim.x) {
        const int64_t o = g / groups, iv = (g - o * groups) * TX + tx;
        const bool there = iv < ivecs;
        const uint4_t *first = reinterpret_cast<const uint4_t *>(src) + o * axis * ivecs + iv;
        ArgBest b[V];
#pragma unroll
        for (int e = 0; e < V; ++e) b[e] = ArgBest{start, INT32_MAX};
        if (there)
            for (int k = ty; k < n; k += TY * U) {
                uint4_t raw[U];
#pragma unroll
                for (int u = 0; u < U; ++u) raw[u] = first[static_cast<int64_t>(min(k + u * TY, n - 1)) * ivecs];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (k + u * TY < n) {
                        float v[V];
                        arg_unpack<DT>(raw[u], v);
#pragma unroll
                        for (int e = 0; e < V; ++e) arg_take<MIN>(b[e], v[e], k + u * TY);
                    }
            }
        __syncthreads(); // the previous group's partials have been read
#pragma unroll
        for (int e = 0; e < V; ++e) {
            sv[ty][tx][e] = b[e].v;
            si[ty][tx][e] = b[e].i;
        }
        __syncthreads();
        // thread (ty, tx) finishes elements ty, ty + TY, .. of column group tx
        if (there)
            for (int e = ty; e < V; e += TY) {
                ArgBest r{sv[0][tx][e], si[0][tx][e]};
                for (int y = 1; y < TY; ++y) arg_merge<MIN>(r, sv[y][tx][e], si[y][tx][e]);
                if (part_v) {
                    part_v[o * inner + iv * V + e] = r.v;
                    part_i[o * inner + iv * V + e] = r.i;
                } else {
                    dst[o * inner + iv * V + e] = r.i == INT32_MAX ? 0 : r.i;
                }
            }
    }
}

// Second pass of an argmax / argmin whose axis was cut into `parts` segments of `seg` elements: position p of result o
// has one candidate per segment, at [(o * parts + part) * inner + p].
template <bool MIN>
__global__ __launch_bounds__(256) void argreduce_merge_kernel(const float *part_v, const int32_t *part_i, int64_t outer, int64_t parts, int64_t seg, int64_t inner, float start,
                                                              int64_t *dst) {
    const int64_t total = outer * inner;
    for (int64_t q = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; q < total; q += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t o = q / inner, p = q - o * inner;
        ArgBest b{start, INT32_MAX};
        for (int64_t part = 0; part < parts; ++part) {
            const int64_t at = (o * parts + part) * inner + p;
            const int32_t i = part_i[at];
            if (i != INT32_MAX) arg_merge<MIN>(b, part_v[at], static_cast<int32_t>(part * seg) + i);
        }
        dst[q] = b.i == INT32_MAX ? 0 : b.i;
    }
}

// ------------------------------------------------ reductions along an inner axis
// Sum / max / min along the middle extent of a contiguous (outer, axis, inner) view, inner > 1: the layout of
// argreduce_strided_vec_kernel (a thread owns the V inner positions of one 16-byte vector, TX threads side by side,
// the TY = 256 / TX thread rows of a work-group share the axis and merge through LDS); fp32 accumulation, the result
// scaled (mean) and rounded to the output type.
template <int RED> __device__ __forceinline__ float red_identity() { return RED == AXHIP_RED_MAX ? -INFINITY : RED == AXHIP_RED_MIN ? INFINITY : RED == AXHIP_RED_PROD ? 1.0f : 0.0f; }
template <int RED> __device__ __forceinline__ float red_combine(float a, float b) { return RED == AXHIP_RED_MAX ? fmaxf(a, b) : RED == AXHIP_RED_MIN ? fminf(a, b) : RED == AXHIP_RED_PROD ? a * b : a + b; }

template <int RED, int DT, int TX>
__global__ __launch_bounds__(256) void reduce_strided_vec_kernel(const void *src, int64_t outer, int64_t axis, int64_t inner, float scale, void *dst, int dst_dt) {
    constexpr int TY = 256 / TX, U = 4, V = DT == AXHIP_DTYPE_F32 ? 4 : 8;
    __shared__ float sv[TY == 1 ? 1 : TY][TY == 1 ? 1 : TX][V + 1];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t ivecs = inner / V, groups = (ivecs + TX - 1) / TX, total = outer * groups;
    const int n = static_cast<int>(axis);
    for (int64_t g = blockIdx.x; g < total; g += gridDim.x) {
        const int64_t o = g / groups, iv = (g - o * groups) * TX + tx;
        const bool there = iv < ivecs;
        const uint4_t *first = reinterpret_cast<const uint4_t *>(src) + o * axis * ivecs + iv;
        float acc[V];
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = red_identity<RED>();
        if (there)
            for (int k = ty; k < n; k += TY * U) {
                uint4_t raw[U];
#pragma unroll
                for (int u = 0; u < U; ++u) raw[u] = first[static_cast<int64_t>(min(k + u * TY, n - 1)) * ivecs];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (k + u * TY < n) {
                        float v[V];
                        arg_unpack<DT>(raw[u], v);
#pragma unroll
                        for (int e = 0; e < V; ++e) acc[e] = red_combine<RED>(acc[e], v[e]);
                    }
            }
        if constexpr (TY == 1) { // a thread walked the whole (short) axis: nothing to merge, one vector store
            if (there) {
#pragma unroll
                for (int e = 0; e < V; ++e) acc[e] *= scale;
                store_vec<V>(dst, dst_dt, o * inner + iv * V, acc);
            }
        } else {
            __syncthreads(); // the previous group's partials have been read
#pragma unroll
            for (int e = 0; e < V; ++e) sv[ty][tx][e] = acc[e];
            __syncthreads();
            if (there)
                for (int e = ty; e < V; e += TY) {
                    float r = sv[0][tx][e];
                    for (int y = 1; y < TY; ++y) r = red_combine<RED>(r, sv[y][tx][e]);
                    store_any(dst, dst_dt, o * inner + iv * V + e, r * scale);
                }
        }
    }
}

// any inner extent and alignment: a thread per (outer, inner) position walks the axis
template <int RED>
__global__ __launch_bounds__(256) void reduce_strided_kernel(const void *src, int dt, int64_t outer, int64_t axis, int64_t inner, float scale, void *dst, int dst_dt) {
    const int64_t total = outer * inner;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; p < total; p += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t o = p / inner, i = p - o * inner;
        const int64_t first = o * axis * inner + i;
        float acc = red_identity<RED>();
        int64_t k = 0;
        for (; k + 4 <= axis; k += 4) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = load_any(src, dt, first + (k + u) * inner);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc = red_combine<RED>(acc, v[u]);
        }
        for (; k < axis; ++k) acc = red_combine<RED>(acc, load_any(src, dt, first + k * inner));
        store_any(dst, dst_dt, p, acc * scale);
    }
}

} // namespace axhip

namespace axhip {
// ----------------------------------------------- softmax along an inner axis
// softmax / log-softmax along the middle extent of a contiguous (outer, axis, inner) view, inner > 1, in the layout of
// reduce_strided_vec_kernel.  One sweep gathers a running maximum and the sum of 2^(x log2(e) - maximum) per inner
// position (rescaled once per four elements), the thread rows merge their pairs through LDS, a second sweep over the
// same elements writes the result: two reads of the input (the second mostly from the caches) and one write.
// HOLD > 0 (with TX = 256, a thread per vector walking the axis alone): the axis has at most HOLD elements and the thread
// keeps them in registers between the two sweeps -- one read of the input.
template <bool LOG, int DT, int TX, int HOLD = 0>
__global__ __launch_bounds__(256) void softmax_strided_vec_kernel(const void *src, int64_t outer, int64_t axis, int64_t inner, void *dst) {
    constexpr int TY = 256 / TX, U = 4, V = DT == AXHIP_DTYPE_F32 ? 4 : 8;
    static_assert(HOLD == 0 || (TX == 256 && HOLD % U == 0), "rows held in registers: one thread per vector");
    constexpr float LOG2E = 1.44269504088896340736f, LN2 = 0.69314718055994530942f;
    __shared__ float sm[TY][TX][V + 1], sl[TY][TX][V + 1];
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t ivecs = inner / V, groups = (ivecs + TX - 1) / TX, total = outer * groups;
    const int n = static_cast<int>(axis);
    for (int64_t g = blockIdx.x; g < total; g += gridDim.x) {
        const int64_t o = g / groups, iv = (g - o * groups) * TX + tx;
        const bool there = iv < ivecs;
        const uint4_t *first = reinterpret_cast<const uint4_t *>(src) + o * axis * ivecs + iv;
        float m[V], l[V];
#pragma unroll
        for (int e = 0; e < V; ++e) {
            m[e] = -INFINITY;
            l[e] = 0.0f;
        }
        uint4_t keep[HOLD > 0 ? HOLD : 1];
        if constexpr (HOLD > 0) {
            if (there) {
#pragma unroll
                for (int k = 0; k < HOLD; ++k) keep[k] = first[static_cast<int64_t>(min(k, n - 1)) * ivecs];
            }
        }
        auto gather = [&](int k, const uint4_t (&raw)[U]) { // running maximum and rescaled sum over U axis elements
                float t[U][V];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    arg_unpack<DT>(raw[u], t[u]);
#pragma unroll
                    for (int e = 0; e < V; ++e) t[u][e] = k + u * TY < n ? t[u][e] * LOG2E : -INFINITY;
                }
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float mx = fmaxf(fmaxf(fmaxf(t[0][e], t[1][e]), fmaxf(t[2][e], t[3][e])), m[e]);
                    const float ref = mx == -INFINITY ? 0.0f : mx; // (nothing finite yet: every term below is 2^-inf = 0)
                    float add = 0.0f;
#pragma unroll
                    for (int u = 0; u < U; ++u) add += __builtin_amdgcn_exp2f(t[u][e] - ref);
                    l[e] = l[e] * __builtin_amdgcn_exp2f(m[e] - ref) + add;
                    m[e] = mx;
                }
        };
        if (there) {
            if constexpr (HOLD > 0) {
#pragma unroll
                for (int k = 0; k < HOLD; k += U)
                    if (k < n) {
                        const uint4_t raw[U] = {keep[k], keep[k + 1], keep[k + 2], keep[k + 3]};
                        gather(k, raw);
                    }
            } else {
                for (int k = ty; k < n; k += TY * U) {
                    uint4_t raw[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) raw[u] = first[static_cast<int64_t>(min(k + u * TY, n - 1)) * ivecs];
                    gather(k, raw);
                }
            }
        }
        __syncthreads(); // the previous group's pairs have been read
#pragma unroll
        for (int e = 0; e < V; ++e) {
            sm[ty][tx][e] = m[e];
            sl[ty][tx][e] = l[e];
        }
        __syncthreads();
        float shift[V], inv[V]; // result = 2^(t - shift) * inv, or (t - shift) * ln 2 with the logarithm of the sum inside shift
#pragma unroll
        for (int e = 0; e < V; ++e) {
            float M = sm[0][tx][e];
            for (int y = 1; y < TY; ++y) M = fmaxf(M, sm[y][tx][e]);
            const float ref = M == -INFINITY ? 0.0f : M;
            float L = 0.0f;
            for (int y = 0; y < TY; ++y) L += sl[y][tx][e] * __builtin_amdgcn_exp2f(sm[y][tx][e] - ref);
            shift[e] = LOG ? M + __builtin_amdgcn_logf(L) : M; // (v_log_f32 is the base-2 logarithm)
            inv[e] = 1.0f / L;
        }
        auto emit = [&](int k, const uint4_t (&raw)[U]) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (k + u * TY < n) {
                        float v[V];
                        arg_unpack<DT>(raw[u], v);
#pragma unroll
                        for (int e = 0; e < V; ++e) v[e] = LOG ? (v[e] * LOG2E - shift[e]) * LN2 : __builtin_amdgcn_exp2f(v[e] * LOG2E - shift[e]) * inv[e];
                        store_vec<V>(dst, DT, (o * axis + k + u * TY) * inner + iv * V, v);
                    }
        };
        if (there) {
            if constexpr (HOLD > 0) {
#pragma unroll
                for (int k = 0; k < HOLD; k += U)
                    if (k < n) {
                        const uint4_t raw[U] = {keep[k], keep[k + 1], keep[k + 2], keep[k + 3]};
                        emit(k, raw);
                    }
            } else {
                for (int k = ty; k < n; k += TY * U) {
                    uint4_t raw[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) raw[u] = first[static_cast<int64_t>(min(k + u * TY, n - 1)) * ivecs];
                    emit(k, raw);
                }
            }
        }
    }
}

// A long axis read ONCE: a 1024-thread block holds an [axis, TX vectors] tile of the input in registers, as the raw
// 16-byte vectors it was loaded as -- thread (ty, tx) the rows ty, ty + TY, ... (RPT of them, TY = 1024 / TX) of
// vector column tx, so TX neighbouring lanes read TX * 16 consecutive bytes of a row --, works out the columns'
// maxima and sums across its threads (shuffles between the lanes of a wave that share a column, LDS between the
// waves) and writes the results from the same registers.  TX = 16, 8 or 4 for axes of up to 1024, 2048 or 4096
// elements (16 rows per thread at most: 64 registers of raw words).  With TX = 4 a row's 64 bytes are half a cache
// line: the two blocks that share the lines run on the same XCD (block b lands on XCD b % 8), so the second one finds
// them in that L2.
template <bool LOG, int DT, int RPT>
__global__ __launch_bounds__(1024) void softmax_axis_tile_kernel(const void *src, int64_t outer, int64_t axis, int64_t inner, int tx_log2, void *dst) {
    constexpr int V = DT == AXHIP_DTYPE_F32 ? 4 : 8;
    constexpr float LOG2E = 1.44269504088896340736f, LN2 = 0.69314718055994530942f;
    __shared__ float red[16][16][V + 1];
    const int TX = 1 << tx_log2, TY = 1024 >> tx_log2;
    const int tid = threadIdx.x, tx = tid & (TX - 1), ty = tid >> tx_log2, wave = tid / WAVE;
    const int64_t ivecs = inner / V, ctiles = (ivecs + TX - 1) / TX, tiles = outer * ctiles;
    const int share = TX >= 8 ? 1 : 8 / TX; // blocks per cache line of a row
    const int n = static_cast<int>(axis);
    const int64_t slot = blockIdx.x / 8, xcd = blockIdx.x % 8;
    const int64_t tile = ((slot / share) * 8 + xcd) * share + slot % share;
    if (tile >= tiles) return; // (whole block)
    const int64_t o = tile / ctiles, iv = (tile - o * ctiles) * TX + tx;
    const bool there = iv < ivecs;
    const uint4_t *first = reinterpret_cast<const uint4_t *>(src) + o * axis * ivecs + (there ? iv : 0);
    uint4_t raw[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) raw[r] = first[static_cast<int64_t>(min(ty + r * TY, n - 1)) * ivecs];
    // column statistic over the block: lanes of a wave that share tx, then the 16 waves
    auto across = [&](float (&x)[V], bool is_max) {
        for (int d = TX; d < WAVE; d <<= 1) {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float y = __shfl_xor(x[e], d, WAVE);
                x[e] = is_max ? fmaxf(x[e], y) : x[e] + y;
            }
        }
        __syncthreads(); // the previous statistic has been read
        if ((tid % WAVE) < TX) {
#pragma unroll
            for (int e = 0; e < V; ++e) red[wave][tx][e] = x[e];
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < V; ++e) {
            float a = red[0][tx][e];
            for (int w = 1; w < 16; ++w) a = is_max ? fmaxf(a, red[w][tx][e]) : a + red[w][tx][e];
            x[e] = a;
        }
    };
    float m[V], l[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
        m[e] = -INFINITY;
        l[e] = 0.0f;
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r)
        if (ty + r * TY < n) {
            float t[V];
            arg_unpack<DT>(raw[r], t);
#pragma unroll
            for (int e = 0; e < V; ++e) m[e] = fmaxf(m[e], t[e] * LOG2E);
        }
    across(m, true);
    float ref[V];
#pragma unroll
    for (int e = 0; e < V; ++e) ref[e] = m[e] == -INFINITY ? 0.0f : m[e]; // (nothing finite: every term is 2^-inf = 0)
#pragma unroll
    for (int r = 0; r < RPT; ++r)
        if (ty + r * TY < n) {
            float t[V];
            arg_unpack<DT>(raw[r], t);
#pragma unroll
            for (int e = 0; e < V; ++e) l[e] += __builtin_amdgcn_exp2f(t[e] * LOG2E - ref[e]);
        }
    across(l, false);
    float shift[V], inv[V]; // result = 2^(t - shift) * inv, or (t - shift) * ln 2 with the logarithm of the sum inside shift
#pragma unroll
    for (int e = 0; e < V; ++e) {
        shift[e] = LOG ? m[e] + __builtin_amdgcn_logf(l[e]) : ref[e]; // (v_log_f32 is the base-2 logarithm)
        inv[e] = 1.0f / l[e];
    }
    if (!there) return;
#pragma unroll
    for (int r = 0; r < RPT; ++r)
        if (ty + r * TY < n) {
            float v[V];
            arg_unpack<DT>(raw[r], v);
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = LOG ? (v[e] * LOG2E - shift[e]) * LN2 : __builtin_amdgcn_exp2f(v[e] * LOG2E - shift[e]) * inv[e];
            store_vec<V>(dst, DT, (o * axis + ty + r * TY) * inner + iv * V, v);
        }
}

// any inner extent and alignment: a thread per (outer, inner) position, three sweeps
template <bool LOG>
__global__ __launch_bounds__(256) void softmax_strided_kernel(const void *src, int dt, int64_t outer, int64_t axis, int64_t inner, void *dst) {
    const int64_t total = outer * inner;
    for (int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; p < total; p += static_cast<int64_t>(gridDim.x) * 256) {
        const int64_t o = p / inner, i = p - o * inner;
        const int64_t first = o * axis * inner + i;
        float m = -INFINITY;
        for (int64_t k = 0; k < axis; ++k) m = fmaxf(m, load_any(src, dt, first + k * inner));
        float l = 0.0f;
        for (int64_t k = 0; k < axis; ++k) l += __expf(load_any(src, dt, first + k * inner) - m);
        const float logl = __logf(l), inv = 1.0f / l;
        for (int64_t k = 0; k < axis; ++k) {
            const float x = load_any(src, dt, first + k * inner);
            store_any(dst, dt, first + k * inner, LOG ? x - m - logl : __expf(x - m) * inv);
        }
    }
}

// one launch: RED is sum, max or min; the result is multiplied by `scale`
int launch_reduce_axis(const void *src, int dtype, int64_t outer, int64_t axis, int64_t inner, int red, float scale, void *dst, int dst_dtype, hipStream_t s) {
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    const bool bytes = dtype == AXHIP_DTYPE_U8 || dst_dtype == AXHIP_DTYPE_U8;
    if (red != AXHIP_RED_PROD && !bytes && inner % (16 / es) == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) { // (products, truth values: the element-wise kernel)
        const int64_t ivecs = inner / (16 / es);
        // a short axis with plenty of results: a thread per vector walks it alone (no merge through LDS)
        const bool flat = axis <= 32 && outer * ((ivecs + 255) / 256) >= 1024 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0;
        // (32-vector column groups from 512 of them on: sum over axis 1 of bf16 [256, 1024, 512] 44.5 -> 38.2 us, 75 -> 88 %
        // of the HBM peak; AXHIP_REDUCE_AXIS_WIDE_FROM=<n>, read once, moves the threshold)
        static const int wide_from = [] { const char *e = getenv("AXHIP_REDUCE_AXIS_WIDE_FROM"); return e ? atoi(e) : 512; }();
        const bool wide = outer * ((ivecs + 31) / 32) >= wide_from;
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(outer * (flat ? (ivecs + 255) / 256 : wide ? (ivecs + 31) / 32 : (ivecs + 7) / 8), 256 * 64));
#define AXHIP_RED_VEC_TX(RED, DT, TX) hipLaunchKernelGGL((reduce_strided_vec_kernel<RED, DT, TX>), dim3(blocks), dim3(256), 0, s, src, outer, axis, inner, scale, dst, dst_dtype)
#define AXHIP_RED_VEC_DT(RED, DT)                                                                                                          \
    do {                                                                                                                                   \
        if (flat) AXHIP_RED_VEC_TX(RED, DT, 256);                                                                                          \
        else if (wide) AXHIP_RED_VEC_TX(RED, DT, 32);                                                                                      \
        else AXHIP_RED_VEC_TX(RED, DT, 8);                                                                                                 \
    } while (0)
#define AXHIP_RED_VEC(RED)                                                                                                                 \
    do {                                                                                                                                   \
        if (dtype == AXHIP_DTYPE_F32) AXHIP_RED_VEC_DT(RED, AXHIP_DTYPE_F32);                                                              \
        else if (dtype == AXHIP_DTYPE_F16) AXHIP_RED_VEC_DT(RED, AXHIP_DTYPE_F16);                                                         \
        else AXHIP_RED_VEC_DT(RED, AXHIP_DTYPE_BF16);                                                                                      \
    } while (0)
        if (red == AXHIP_RED_SUM) AXHIP_RED_VEC(AXHIP_RED_SUM);
        else if (red == AXHIP_RED_MAX) AXHIP_RED_VEC(AXHIP_RED_MAX);
        else AXHIP_RED_VEC(AXHIP_RED_MIN);
#undef AXHIP_RED_VEC
#undef AXHIP_RED_VEC_DT
#undef AXHIP_RED_VEC_TX
    } else {
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer * inner + 255) / 256, 256 * 32));
        if (red == AXHIP_RED_SUM) hipLaunchKernelGGL(reduce_strided_kernel<AXHIP_RED_SUM>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, scale, dst, dst_dtype);
        else if (red == AXHIP_RED_MAX) hipLaunchKernelGGL(reduce_strided_kernel<AXHIP_RED_MAX>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, scale, dst, dst_dtype);
        else if (red == AXHIP_RED_PROD) hipLaunchKernelGGL(reduce_strided_kernel<AXHIP_RED_PROD>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, scale, dst, dst_dtype);
        else hipLaunchKernelGGL(reduce_strided_kernel<AXHIP_RED_MIN>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, scale, dst, dst_dtype);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}
} // namespace axhip

using namespace axhip;

namespace {
// AXHIP_SOFTMAX_AXIS_TILE=0 (read at every call): long axes on the two-sweep kernel instead of the one-read tile kernel
bool softmax_axis_tile_enabled() {
    const char *e = getenv("AXHIP_SOFTMAX_AXIS_TILE");
    return !(e && e[0] == '0');
}
} // namespace

extern "C" {

int axhip_strided_copy(const void *src, int32_t src_dtype, void *dst, int32_t dst_dtype, int32_t ndim,
                       const int64_t *shape, const int64_t *strides, void *stream) {
    AXHIP_REQUIRE(valid_dtype_or_u8(src_dtype) && valid_dtype_or_u8(dst_dtype), AXHIP_ERR_INVALID_ARG, "axhip_strided_copy: bad dtype");
    const bool bytes = src_dtype == AXHIP_DTYPE_U8 || dst_dtype == AXHIP_DTYPE_U8; // truth values: the element-wise kernel
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
    // A cast of a contiguous array (nothing to gather) of 8 MiB or more is an elementwise chain with no operation: the
    // compiled row kernel of that chain moves it (bf16 -> fp32 [16384,4096]: 72.6 -> 57.4 us, 69 -> 88 % of the HBM peak).
    if (!bytes && src_dtype != dst_dtype && nd == 1 && a.strides[0] == 1 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0 &&
        a.total * (src_dtype == AXHIP_DTYPE_F32 ? 4 : 2) >= (int64_t(8) << 20) && a.total % 4096 == 0) {
        AxhipRowsProgram P{};
        P.rows = a.total / 4096; P.cols = 4096;
        P.input = src; P.input_dtype = src_dtype; P.output = dst; P.output_dtype = dst_dtype;
        P.norm_weight = P.norm_bias = -1;
        return axhip_fused_rows(&P, stream);
    }
    int64_t max_off = 0;
    for (int d = 0; d < nd; ++d) max_off += (a.shape[d] - 1) * a.strides[d];
    const bool idx32 = a.total < (int64_t(1) << 31) - (1 << 23) && max_off < (int64_t(1) << 31) - (1 << 23); // room for the grid stride

    // vector path: innermost dimension contiguous and every row start aligned to the vector
    const bool raw = src_dtype == dst_dtype;
    const int v = raw ? (src_dtype == AXHIP_DTYPE_F32 ? 4 : 8) : (dst_dtype == AXHIP_DTYPE_F32 ? 4 : 8);
    const int src_es = src_dtype == AXHIP_DTYPE_F32 ? 4 : 2, dst_es = dst_dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    const int src_align = src_es == 4 ? 16 : v * 2; // bytes a vector load needs
    bool vec = !bytes && nd >= 1 && a.strides[nd - 1] == 1 && a.shape[nd - 1] % v == 0 && reinterpret_cast<uintptr_t>(src) % src_align == 0 &&
               reinterpret_cast<uintptr_t>(dst) % (v * dst_es >= 16 ? 16 : 8) == 0;
    for (int d = 0; vec && d + 1 < nd; ++d) vec = (a.strides[d] * src_es) % src_align == 0;
    // the same with groups that start anywhere in the source (x[:, 1:], convolution windows): unaligned loads
    static const bool unaligned_on = [] { const char *e = getenv("AXHIP_COPY_UNALIGNED"); return !(e && e[0] == '0'); }();
    const bool vec_unaligned = !vec && unaligned_on && !bytes && nd >= 1 && a.strides[nd - 1] == 1 && a.shape[nd - 1] % v == 0 &&
                               reinterpret_cast<uintptr_t>(dst) % (v * dst_es >= 16 ? 16 : 8) == 0;
    vec = vec || vec_unaligned;
    // every other element, same type, whole groups of a vector or of half a vector
    const int gv = nd >= 1 && a.shape[nd - 1] % v == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 ? v : v / 2;
    const bool every_other = !vec && unaligned_on && !bytes && raw && nd >= 1 && a.strides[nd - 1] == 2 && a.shape[nd - 1] % gv == 0 &&
                             reinterpret_cast<uintptr_t>(dst) % (gv == v ? 16 : 8) == 0;
    // transposes: the innermost dimension is strided, some other dimension is contiguous in the source
    int transpose_j = -1;
    if (!vec && !bytes && nd >= 2 && a.strides[nd - 1] > 1 && a.shape[nd - 1] >= 16) {
        for (int d = 0; d + 1 < nd; ++d)
            if (a.strides[d] == 1 && a.shape[d] >= 16) transpose_j = d;
    }
    if (every_other) {
        a.shape[nd - 1] /= gv;
        a.strides[nd - 1] = 2 * gv;
        a.total /= gv;
        const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
        const dim3 grid(static_cast<unsigned>(blocks));
        auto launch = [&](auto idx_tag) {
            using IDX = decltype(idx_tag);
            if (src_es == 4 && gv == v) hipLaunchKernelGGL((strided_copy_every_other_kernel<IDX, 4, false>), grid, dim3(256), 0, s, a);
            else if (src_es == 4) hipLaunchKernelGGL((strided_copy_every_other_kernel<IDX, 4, true>), grid, dim3(256), 0, s, a);
            else if (gv == v) hipLaunchKernelGGL((strided_copy_every_other_kernel<IDX, 2, false>), grid, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((strided_copy_every_other_kernel<IDX, 2, true>), grid, dim3(256), 0, s, a);
        };
        if (idx32) launch(int32_t{});
        else launch(int64_t{});
    } else if (vec) {
        a.shape[nd - 1] /= v;
        a.strides[nd - 1] = v;
        a.total /= v;
        const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
        const dim3 grid(static_cast<unsigned>(blocks));
        auto launch = [&](auto idx_tag) {
            using IDX = decltype(idx_tag);
            if (vec_unaligned) {
                if (raw && v == 4) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 4, true, true>), grid, dim3(256), 0, s, a);
                else if (raw) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 8, true, true>), grid, dim3(256), 0, s, a);
                else if (v == 4) hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 4, false, true>), grid, dim3(256), 0, s, a);
                else hipLaunchKernelGGL((strided_copy_vec_kernel<IDX, 8, false, true>), grid, dim3(256), 0, s, a);
                return;
            }
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
        // whole 16-byte vectors (or 8-byte pieces) on both sides: the vector tiles
        const int es = src_dtype == AXHIP_DTYPE_F32 ? 4 : 2;
        auto side = [&](int64_t extent, int64_t stride, const int64_t *others, const void *base) { // bytes per access: 16, 8 or 0
            for (int g = 16; g >= 8; g /= 2) {
                const int64_t n = g / es;
                bool ok = extent % n == 0 && stride % n == 0 && (reinterpret_cast<uintptr_t>(base) & static_cast<uintptr_t>(g - 1)) == 0;
                for (int d = 0; d < no; ++d) ok = ok && others[d] % n == 0;
                if (ok) return g;
            }
            return 0;
        };
        const int lg = side(t.nJ, t.src_stride_l, t.osrc, src), sg = side(t.nL, t.dst_stride_j, t.odst, dst);
        const bool whole = src_dtype == dst_dtype && src_dtype != AXHIP_DTYPE_U8 && lg > 0 && sg > 0;
        static const bool vec_tiles = [] { const char *e = getenv("AXHIP_TRANSPOSE_VEC"); return !(e && e[0] == '0'); }();
        if (whole && vec_tiles) {
            const int64_t edge = 16 * (16 / es);
            t.tiles_j = (t.nJ + edge - 1) / edge; t.tiles_l = (t.nL + edge - 1) / edge;
            blocks = blocks / (((t.nJ + 63) / 64) * ((t.nL + 63) / 64)) * t.tiles_j * t.tiles_l;
            AXHIP_REQUIRE(blocks < (int64_t(1) << 31), AXHIP_ERR_UNSUPPORTED, "axhip_strided_copy: view too large");
            const dim3 grid(static_cast<unsigned>(blocks));
#define AXHIP_TRANSPOSE(ES)                                                                                              \
    do {                                                                                                                 \
        if (lg == 16 && sg == 16) hipLaunchKernelGGL((transpose_vec_kernel<ES, 16, 16>), grid, dim3(256), 0, s, t);      \
        else if (lg == 16) hipLaunchKernelGGL((transpose_vec_kernel<ES, 16, 8>), grid, dim3(256), 0, s, t);              \
        else if (sg == 16) hipLaunchKernelGGL((transpose_vec_kernel<ES, 8, 16>), grid, dim3(256), 0, s, t);              \
        else hipLaunchKernelGGL((transpose_vec_kernel<ES, 8, 8>), grid, dim3(256), 0, s, t);                             \
    } while (0)
            if (es == 2) AXHIP_TRANSPOSE(2);
            else AXHIP_TRANSPOSE(4);
#undef AXHIP_TRANSPOSE
            AXHIP_CHECK_HIP(hipGetLastError());
            return AXHIP_OK;
        }
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
    return axhip_pad_mode(src, dst, dtype, ndim, src_shape, src_strides, pad_before, pad_after, AXHIP_PAD_CONSTANT, value, stream);
}

int axhip_pad_mode(const void *src, void *dst, int32_t dtype, int32_t ndim, const int64_t *src_shape, const int64_t *src_strides,
                   const int64_t *pad_before, const int64_t *pad_after, int32_t mode, double value, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_pad: bad dtype");
    AXHIP_REQUIRE(mode >= AXHIP_PAD_CONSTANT && mode <= AXHIP_PAD_CIRCULAR, AXHIP_ERR_INVALID_ARG, "axhip_pad: bad mode %d", mode);
    AXHIP_REQUIRE(ndim >= 1 && ndim <= AXHIP_MAX_DIMS, AXHIP_ERR_INVALID_ARG, "axhip_pad: ndim %d out of range", ndim);
    AXHIP_REQUIRE(src_shape && src_strides && pad_before && pad_after, AXHIP_ERR_INVALID_ARG, "axhip_pad: NULL shape/strides/pads");
    PadArgs a{};
    a.src = src; a.dst = dst; a.dtype = dtype; a.ndim = ndim; a.value = static_cast<float>(value); a.mode = mode;
    a.total = 1;
    int64_t src_total = 1;
    for (int d = 0; d < ndim; ++d) {
        AXHIP_REQUIRE(src_shape[d] >= 0 && pad_before[d] >= 0 && pad_after[d] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_pad: negative extent or pad");
        if (mode == AXHIP_PAD_REFLECT && (pad_before[d] > 0 || pad_after[d] > 0))
            AXHIP_REQUIRE(pad_before[d] < src_shape[d] && pad_after[d] < src_shape[d], AXHIP_ERR_INVALID_ARG,
                          "axhip_pad: a reflected pad (%lld, %lld) must be shorter than the extent %lld", static_cast<long long>(pad_before[d]),
                          static_cast<long long>(pad_after[d]), static_cast<long long>(src_shape[d]));
        if (mode != AXHIP_PAD_CONSTANT && (pad_before[d] > 0 || pad_after[d] > 0))
            AXHIP_REQUIRE(src_shape[d] > 0, AXHIP_ERR_INVALID_ARG, "axhip_pad: nothing to repeat along an empty extent");
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
    const int V = dtype == AXHIP_DTYPE_F32 ? 4 : 8;
    if (ndim >= 1 && a.out_shape[ndim - 1] >= V && a.total > 0 && (reinterpret_cast<uintptr_t>(dst) & (dtype == AXHIP_DTYPE_F32 ? 3u : 1u)) == 0 &&
        (reinterpret_cast<uintptr_t>(src) & (dtype == AXHIP_DTYPE_F32 ? 3u : 1u)) == 0) {
        int64_t reach = a.total; // the largest index or source offset the kernel forms
        for (int d = 0; d < ndim; ++d) reach = std::max(reach, (a.src_shape[d] + a.out_shape[d]) * std::max<int64_t>(a.src_strides[d], 1));
        const bool small = reach < (int64_t(1) << 31) - (1 << 20);
        // Rows that are not whole 16-byte groups in an aligned output: the groups are cut from the whole output.
        static const bool flat_on = [] { const char *e = getenv("AXHIP_PAD_FLAT"); return !(e && e[0] == '0'); }();
        const bool flat = flat_on && a.out_shape[ndim - 1] % V != 0 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0;
        const int64_t n_groups = flat ? (a.total + V - 1) / V : a.total / a.out_shape[ndim - 1] * ((a.out_shape[ndim - 1] + V - 1) / V);
        const int64_t blocks = std::min<int64_t>((n_groups + 255) / 256, 256 * 64);
        hipStream_t s = resolve_stream(stream);
        if (flat) {
            if (V == 4) {
                if (small) hipLaunchKernelGGL((pad_vec_kernel<int32_t, 4, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
                else hipLaunchKernelGGL((pad_vec_kernel<int64_t, 4, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
            } else {
                if (small) hipLaunchKernelGGL((pad_vec_kernel<int32_t, 8, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
                else hipLaunchKernelGGL((pad_vec_kernel<int64_t, 8, true>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
            }
        } else if (V == 4) {
            if (small) hipLaunchKernelGGL((pad_vec_kernel<int32_t, 4>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
            else hipLaunchKernelGGL((pad_vec_kernel<int64_t, 4>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
        } else {
            if (small) hipLaunchKernelGGL((pad_vec_kernel<int32_t, 8>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
            else hipLaunchKernelGGL((pad_vec_kernel<int64_t, 8>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, a);
        }
        AXHIP_CHECK_HIP(hipGetLastError());
        return AXHIP_OK;
    }
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
    // Rows that are contiguous in the source and contiguous or repeated in the mask go 16 bytes a thread.
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2, v = 16 / es, last = ndim - 1;
    static const bool vec_on = [] { const char *e = getenv("AXHIP_MASKED_FILL_VEC"); return !(e && e[0] == '0'); }();
    bool vec = vec_on && ndim >= 1 && src_strides[last] == 1 && (mask_strides[last] == 0 || mask_strides[last] == 1) && shape[last] % v == 0 &&
               (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 == 0;
    const bool mask_row = vec && mask_strides[last] == 1;
    if (mask_row && reinterpret_cast<uintptr_t>(mask) % v != 0) vec = false;
    int64_t src_span = 0, mask_span = 0; // the largest element offsets
    for (int d = 0; d < ndim && vec; ++d) {
        src_span += (shape[d] - 1) * src_strides[d];
        mask_span += (shape[d] - 1) * mask_strides[d];
        if (d == last) continue;
        if (src_strides[d] % v != 0 || (mask_row && mask_strides[d] % v != 0)) vec = false;
    }
    if (vec) {
        a.shape[last] = shape[last] / v;
        a.src_strides[last] = v;
        a.mask_strides[last] = mask_row ? v : 0;
        a.total /= v;
        const bool idx32 = a.total < (1ll << 31) && src_span < (1ll << 31) && mask_span < (1ll << 31);
        const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 32);
        auto kernel = idx32 ? (es == 4 ? masked_fill_vec_kernel<uint32_t, 4> : masked_fill_vec_kernel<uint32_t, 2>)
                            : (es == 4 ? masked_fill_vec_kernel<int64_t, 4> : masked_fill_vec_kernel<int64_t, 2>);
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), a);
        AXHIP_CHECK_HIP(hipGetLastError());
        return AXHIP_OK;
    }
    const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 64);
    hipLaunchKernelGGL(masked_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, resolve_stream(stream), a);
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

int axhip_where(const void *cond, int32_t cond_dtype, const void *a, int32_t a_dtype, const void *b, int32_t b_dtype, void *dst, int32_t dst_dtype,
                int32_t ndim, const int64_t *shape, const int64_t *cond_strides, const int64_t *a_strides, const int64_t *b_strides, void *stream) {
    AXHIP_REQUIRE(valid_dtype_or_u8(cond_dtype) && valid_dtype_or_u8(a_dtype) && valid_dtype_or_u8(b_dtype) && valid_dtype_or_u8(dst_dtype),
                  AXHIP_ERR_INVALID_ARG, "axhip_where: bad dtype");
    AXHIP_REQUIRE(ndim >= 0 && ndim <= AXHIP_MAX_DIMS, AXHIP_ERR_INVALID_ARG, "axhip_where: ndim %d out of range", ndim);
    AXHIP_REQUIRE(ndim == 0 || (shape && cond_strides && a_strides && b_strides), AXHIP_ERR_INVALID_ARG, "axhip_where: NULL shape/strides");
    WhereArgs w{};
    w.cond = cond; w.a = a; w.b = b; w.dst = dst;
    w.cond_dtype = cond_dtype; w.a_dtype = a_dtype; w.b_dtype = b_dtype; w.dst_dtype = dst_dtype; w.ndim = ndim;
    w.total = 1;
    bool cond_flat = true, a_flat = true, b_flat = true, a_one = true, b_one = true; // contiguous over the whole extent / one element
    int64_t run = 1;
    for (int d = ndim - 1; d >= 0; --d) {
        AXHIP_REQUIRE(shape[d] >= 0, AXHIP_ERR_INVALID_ARG, "axhip_where: negative extent");
        AXHIP_REQUIRE(cond_strides[d] >= 0 && a_strides[d] >= 0 && b_strides[d] >= 0, AXHIP_ERR_UNSUPPORTED, "axhip_where: negative strides are not supported");
        w.shape[d] = shape[d];
        w.cond_strides[d] = cond_strides[d];
        w.a_strides[d] = a_strides[d];
        w.b_strides[d] = b_strides[d];
        if (shape[d] != 1) {
            cond_flat = cond_flat && cond_strides[d] == run;
            a_flat = a_flat && a_strides[d] == run;
            b_flat = b_flat && b_strides[d] == run;
            a_one = a_one && a_strides[d] == 0;
            b_one = b_one && b_strides[d] == 0;
        }
        run *= shape[d];
        w.total *= shape[d];
    }
    if (w.total == 0) return AXHIP_OK;
    AXHIP_REQUIRE(cond && a && b && dst, AXHIP_ERR_INVALID_ARG, "axhip_where: NULL buffer");
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);
    auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    const bool wide = (!a_one && a_dtype == AXHIP_DTYPE_F32) || (!b_one && b_dtype == AXHIP_DTYPE_F32) || dst_dtype == AXHIP_DTYPE_F32;
    const int v = wide ? 4 : 8;
    if (cond_flat && (a_flat || a_one) && (b_flat || b_one) && w.total % v == 0 && aligned(cond) && aligned(dst) && (a_one || aligned(a)) && (b_one || aligned(b))) {
        const int64_t blocks = std::min<int64_t>((w.total / v + 255) / 256, 256 * 64);
        if (v == 4) hipLaunchKernelGGL(where_vec_kernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, w, a_one, b_one);
        else hipLaunchKernelGGL(where_vec_kernel<8>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, w, a_one, b_one);
    } else {
        // Inputs that run along the innermost dimension or repeat over it, in whole aligned vectors: V elements a thread.
        static const bool rows_on = [] { const char *e = getenv("AXHIP_WHERE_ROWS"); return !(e && e[0] == '0'); }();
        const int L = ndim - 1;
        bool rows = rows_on && ndim >= 1 && shape[L] % v == 0 && aligned(dst);
        int64_t reach = w.total;
        auto fits = [&](const void *p, int dt, const int64_t *st) {
            const int es = dt == AXHIP_DTYPE_F32 ? 4 : dt == AXHIP_DTYPE_U8 ? 1 : 2;
            int64_t span = 0;
            for (int d = 0; d < ndim; ++d) span += (shape[d] - 1) * st[d];
            reach = std::max(reach, span + v);
            if (st[L] == 0) return true;
            if (st[L] != 1 || reinterpret_cast<uintptr_t>(p) % (static_cast<uintptr_t>(v) * es) != 0) return false;
            for (int d = 0; d < L; ++d)
                if (st[d] % v != 0) return false;
            return true;
        };
        rows = rows && fits(cond, cond_dtype, cond_strides) && fits(a, a_dtype, a_strides) && fits(b, b_dtype, b_strides);
        if (rows) {
            w.shape[L] /= v;
            w.total /= v;
            w.cond_strides[L] *= v; w.a_strides[L] *= v; w.b_strides[L] *= v;
            const bool small = reach < (int64_t(1) << 31) - (1 << 20);
            const int64_t blocks = std::min<int64_t>((w.total + 255) / 256, 256 * 32);
            auto kernel = v == 4 ? (small ? where_rows_kernel<uint32_t, 4> : where_rows_kernel<int64_t, 4>)
                                 : (small ? where_rows_kernel<uint32_t, 8> : where_rows_kernel<int64_t, 8>);
            hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, w);
        } else {
            const int64_t blocks = std::min<int64_t>((w.total + 255) / 256, 256 * 64);
            hipLaunchKernelGGL(where_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, w);
        }
    }
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

// segments the axis is cut into when few results stand over a long axis (1: no cut, no temporary memory)
static int64_t argreduce_parts(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner) {
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    if (inner <= 1 || inner % (16 / es) != 0 || (reinterpret_cast<uintptr_t>(src) & 15u) != 0) return 1;
    const int64_t ivecs = inner / (16 / es);
    int64_t parts = 1;
    if (outer * ((ivecs + 7) / 8) < 512 && axis >= 2048)
        for (int64_t p = 2; p <= 64 && outer * ((ivecs + 7) / 8) * parts < 1024; ++p)
            if (axis % p == 0 && axis / p >= 256) parts = p;
    return parts;
}

size_t axhip_argreduce_workspace_bytes(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner) {
    if (!valid_dtype(dtype) || outer <= 0 || axis <= 0 || inner <= 0) return 0;
    const int64_t parts = argreduce_parts(src, dtype, outer, axis, inner);
    return parts > 1 ? CallScratch::rounded(static_cast<size_t>(outer * parts * inner) * 8) : 0;
}

int axhip_argreduce(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t want_min, int64_t *dst, void *stream) {
    return axhip_argreduce_ws(src, dtype, outer, axis, inner, want_min, dst, nullptr, 0, stream);
}

int axhip_argreduce_ws(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t want_min, int64_t *dst, void *workspace,
                       size_t workspace_bytes, void *stream) {
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
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    if (inner == 1) {
        const int64_t row_bytes = axis * es;
#define AXHIP_ARG_ROWS_DT(T, DT, BLOCKS, LANES)                                                                                            \
    do {                                                                                                                                   \
        if (want_min) hipLaunchKernelGGL((argreduce_rows_kernel<true, T, DT>), dim3(BLOCKS), dim3(T == 64 ? 256 : T), 0, s, src, outer, axis, LANES, start, dst); \
        else hipLaunchKernelGGL((argreduce_rows_kernel<false, T, DT>), dim3(BLOCKS), dim3(T == 64 ? 256 : T), 0, s, src, outer, axis, LANES, start, dst);         \
    } while (0)
#define AXHIP_ARG_ROWS(T, BLOCKS, LANES)                                                                                                   \
    do {                                                                                                                                   \
        if (dtype == AXHIP_DTYPE_F32) AXHIP_ARG_ROWS_DT(T, AXHIP_DTYPE_F32, BLOCKS, LANES);                                                \
        else if (dtype == AXHIP_DTYPE_F16) AXHIP_ARG_ROWS_DT(T, AXHIP_DTYPE_F16, BLOCKS, LANES);                                           \
        else AXHIP_ARG_ROWS_DT(T, AXHIP_DTYPE_BF16, BLOCKS, LANES);                                                                        \
    } while (0)
        if (row_bytes <= 16384) {
            // lanes per row: one 16-byte vector each up to a whole wavefront, four vectors each beyond
            int lanes = 1;
            while (lanes < 64 && static_cast<int64_t>(lanes) * 16 < row_bytes) lanes *= 2;
            const int rpb = 256 / lanes;
            const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer + rpb - 1) / rpb, 256 * 32));
            AXHIP_ARG_ROWS(64, blocks, lanes);
        } else if (row_bytes <= 65536) {
            AXHIP_ARG_ROWS(256, static_cast<unsigned>(std::min<int64_t>(outer, 256 * 32)), 64);
        } else {
            AXHIP_ARG_ROWS(1024, static_cast<unsigned>(std::min<int64_t>(outer, 256 * 8)), 64);
        }
#undef AXHIP_ARG_ROWS
#undef AXHIP_ARG_ROWS_DT
    } else if (inner % (16 / es) == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
        const int64_t ivecs = inner / (16 / es);
        // Few results over a long axis: too few work-groups for the chip.  The axis is cut into `parts` equal segments
        // whose candidates (value, index) go to stream-ordered temporary memory and are merged by a second kernel.
        const int64_t parts = argreduce_parts(src, dtype, outer, axis, inner);
        const int64_t v_outer = outer * parts, v_axis = axis / parts;
        float *part_v = nullptr;
        int32_t *part_i = nullptr;
        CallScratch scratch(workspace, workspace_bytes, s);
        if (parts > 1) {
            void *tmp = nullptr;
            rc = scratch.take(&tmp, static_cast<size_t>(v_outer * inner) * 8, "axhip_argreduce");
            if (rc) return rc;
            part_v = static_cast<float *>(tmp);
            part_i = reinterpret_cast<int32_t *>(part_v + v_outer * inner);
        }
        const bool wide = v_outer * ((ivecs + 31) / 32) >= 1024;
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(v_outer * (wide ? (ivecs + 31) / 32 : (ivecs + 7) / 8), 256 * 64));
#define AXHIP_ARG_VEC_TX(DT, TX)                                                                                                           \
    do {                                                                                                                                   \
        if (want_min) hipLaunchKernelGGL((argreduce_strided_vec_kernel<true, DT, TX>), dim3(blocks), dim3(256), 0, s, src, v_outer, v_axis, inner, start, dst, part_v, part_i); \
        else hipLaunchKernelGGL((argreduce_strided_vec_kernel<false, DT, TX>), dim3(blocks), dim3(256), 0, s, src, v_outer, v_axis, inner, start, dst, part_v, part_i);         \
    } while (0)
#define AXHIP_ARG_VEC(DT)                                                                                                                  \
    do {                                                                                                                                   \
        if (wide) AXHIP_ARG_VEC_TX(DT, 32);                                                                                                \
        else AXHIP_ARG_VEC_TX(DT, 8);                                                                                                      \
    } while (0)
        if (dtype == AXHIP_DTYPE_F32) AXHIP_ARG_VEC(AXHIP_DTYPE_F32);
        else if (dtype == AXHIP_DTYPE_F16) AXHIP_ARG_VEC(AXHIP_DTYPE_F16);
        else AXHIP_ARG_VEC(AXHIP_DTYPE_BF16);
#undef AXHIP_ARG_VEC
#undef AXHIP_ARG_VEC_TX
        if (parts > 1) {
            const unsigned mblocks = static_cast<unsigned>(std::min<int64_t>((outer * inner + 255) / 256, 256 * 32));
            if (want_min) hipLaunchKernelGGL(argreduce_merge_kernel<true>, dim3(mblocks), dim3(256), 0, s, part_v, part_i, outer, parts, v_axis, inner, start, dst);
            else hipLaunchKernelGGL(argreduce_merge_kernel<false>, dim3(mblocks), dim3(256), 0, s, part_v, part_i, outer, parts, v_axis, inner, start, dst);
            rc = scratch.release();
            if (rc) return rc;
        }
    } else {
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer * inner + 255) / 256, 256 * 32));
        if (want_min) hipLaunchKernelGGL(argreduce_strided_kernel<true>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, start, dst);
        else hipLaunchKernelGGL(argreduce_strided_kernel<false>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, start, dst);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

// segments the axis is cut into when few results stand over a long axis (1: one pass, no temporary memory)
static int64_t reduce_axis_parts(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner) {
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    if (inner <= 1 || inner % (16 / es) != 0 || (reinterpret_cast<uintptr_t>(src) & 15u) != 0) return 1;
    // Large arrays of short inner rows (up to 8 KiB) do better in 32-vector column groups -- 512-byte runs per row
    // instead of 128 -- once the axis is cut so that there are about 1024 of them: sum over axis 1 of bf16
    // [64, 4096, 1024] 99.5 -> 91.8 us (67 -> 73 % of the HBM peak), [8, 8192, 4096] 97.2 -> 92.8 us.  Smaller arrays lose
    // to the second launch ([16, 2048, 2048]: 22.5 -> 25.9 us), long inner rows to the split itself (fp32
    // [1, 4096, 16384]: 40.0 -> 43.3 us): they keep the rule below.  AXHIP_REDUCE_AXIS_SPLIT32=0 (read once): never.
    static const bool split32 = [] { const char *e = getenv("AXHIP_REDUCE_AXIS_SPLIT32"); return !(e && e[0] == '0'); }();
    const int64_t groups8 = outer * ((inner / (16 / es) + 7) / 8), groups32 = outer * ((inner / (16 / es) + 31) / 32);
    int64_t parts = 1;
    if (split32 && outer * axis * inner * es >= (int64_t(256) << 20) && inner * es <= 8192) {
        if (groups32 < 512 && axis >= 1024)
            for (int64_t p = 2; p <= 64 && groups32 * parts < 1024; ++p)
                if (axis % p == 0 && axis / p >= 256) parts = p;
        return parts;
    }
    if (groups8 < 512 && axis >= 2048)
        for (int64_t p = 2; p <= 64 && groups8 * parts < 1024; ++p)
            if (axis % p == 0 && axis / p >= 256) parts = p;
    return parts;
}

size_t axhip_reduce_axis_workspace_bytes(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner) {
    if (!valid_dtype(dtype) || outer <= 0 || axis <= 0 || inner <= 0) return 0;
    const int64_t parts = reduce_axis_parts(src, dtype, outer, axis, inner);
    return parts > 1 ? CallScratch::rounded(static_cast<size_t>(outer * parts * inner) * 4) : 0;
}

int axhip_reduce_axis(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t reduce, void *dst, int32_t dst_dtype,
                      void *stream) {
    return axhip_reduce_axis_ws(src, dtype, outer, axis, inner, reduce, dst, dst_dtype, nullptr, 0, stream);
}

int axhip_reduce_axis_ws(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t reduce, void *dst, int32_t dst_dtype,
                         void *workspace, size_t workspace_bytes, void *stream) {
    AXHIP_REQUIRE(valid_dtype_or_u8(dtype) && valid_dtype_or_u8(dst_dtype), AXHIP_ERR_INVALID_ARG, "axhip_reduce_axis: bad dtype");
    AXHIP_REQUIRE(reduce >= AXHIP_RED_SUM && reduce <= AXHIP_RED_PROD, AXHIP_ERR_INVALID_ARG, "axhip_reduce_axis: bad reduction %d", reduce);
    AXHIP_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, AXHIP_ERR_INVALID_ARG, "axhip_reduce_axis: negative extent");
    if (outer == 0 || inner == 0) return AXHIP_OK;
    AXHIP_REQUIRE(axis > 0, AXHIP_ERR_INVALID_ARG, "axhip_reduce_axis: empty axis");
    AXHIP_REQUIRE(axis < (int64_t(1) << 31) - 64, AXHIP_ERR_UNSUPPORTED, "axhip_reduce_axis: axis of %lld elements", static_cast<long long>(axis));
    AXHIP_REQUIRE(src && dst, AXHIP_ERR_INVALID_ARG, "axhip_reduce_axis: NULL buffer");
    if (inner == 1) { // rows: the fused row kernels
        AxhipRowsProgram P{};
        P.rows = outer; P.cols = axis; P.input = src; P.input_dtype = dtype; P.output = dst; P.output_dtype = dst_dtype;
        P.norm_weight = P.norm_bias = -1; P.reduce = reduce;
        return axhip_fused_rows(&P, stream);
    }
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);
    const float scale = reduce == AXHIP_RED_MEAN ? 1.0f / static_cast<float>(axis) : 1.0f;
    const int red = reduce == AXHIP_RED_MEAN ? AXHIP_RED_SUM : reduce;
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    const bool vec = dtype != AXHIP_DTYPE_U8 && dst_dtype != AXHIP_DTYPE_U8 && inner % (16 / es) == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0;
    // Few results over a long axis (column sums of a tall matrix): too few work-groups for the chip.  The axis is cut
    // into `parts` equal segments, reduced to fp32 partials in stream-ordered temporary memory, and those reduced again.
    const int64_t parts = vec && red != AXHIP_RED_PROD ? reduce_axis_parts(src, dtype, outer, axis, inner) : 1;
    if (parts > 1) {
        CallScratch scratch(workspace, workspace_bytes, s);
        void *tmp = nullptr;
        rc = scratch.take(&tmp, static_cast<size_t>(outer * parts * inner) * 4, "axhip_reduce_axis");
        if (rc) return rc;
        rc = launch_reduce_axis(src, dtype, outer * parts, axis / parts, inner, red, 1.0f, tmp, AXHIP_DTYPE_F32, s);
        if (!rc) rc = launch_reduce_axis(tmp, AXHIP_DTYPE_F32, outer, parts, inner, red, scale, dst, dst_dtype, s);
        const int freed = scratch.release();
        return rc ? rc : freed;
    }
    return launch_reduce_axis(src, dtype, outer, axis, inner, red, scale, dst, dst_dtype, s);
}

int axhip_softmax_axis(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner, int32_t is_log, void *dst, void *stream) {
    AXHIP_REQUIRE(valid_dtype(dtype), AXHIP_ERR_INVALID_ARG, "axhip_softmax_axis: bad dtype");
    AXHIP_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, AXHIP_ERR_INVALID_ARG, "axhip_softmax_axis: negative extent");
    if (outer == 0 || inner == 0 || axis == 0) return AXHIP_OK;
    AXHIP_REQUIRE(axis < (int64_t(1) << 31) - 64, AXHIP_ERR_UNSUPPORTED, "axhip_softmax_axis: axis of %lld elements", static_cast<long long>(axis));
    AXHIP_REQUIRE(src && dst, AXHIP_ERR_INVALID_ARG, "axhip_softmax_axis: NULL buffer");
    if (inner == 1) { // rows: the fused row kernels
        AxhipRowsProgram P{};
        P.rows = outer; P.cols = axis; P.input = src; P.input_dtype = dtype; P.output = dst; P.output_dtype = dtype;
        P.norm_weight = P.norm_bias = -1; P.row_op = is_log ? AXHIP_ROWOP_LOGSOFTMAX : AXHIP_ROWOP_SOFTMAX;
        return axhip_fused_rows(&P, stream);
    }
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = resolve_stream(stream);
    const int es = dtype == AXHIP_DTYPE_F32 ? 4 : 2;
    if (inner % (16 / es) == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0) {
        const int64_t ivecs = inner / (16 / es);
        // a long axis that a block can hold: one read.  Where it pays against the two-sweep kernel (one 1024-thread block per
        // CU, whose load, arithmetic and store phases do not overlap): fp32 axes of 512 to 2048 elements (126 against 179 us
        // on [16, 2048, 2048]), 16-bit axes of 1024 to 4096 (274 against 348 us on [64, 2048, 2048]); shorter axes and
        // fp32 axes of 4096 (64-byte row pieces) stay on the two-sweep kernel
        const bool tile_pays = dtype == AXHIP_DTYPE_F32 ? axis >= 512 && axis <= 2048 : axis >= 1024 && axis <= 4096;
        if (tile_pays && softmax_axis_tile_enabled()) {
            const int tx_log2 = axis <= 1024 ? 4 : axis <= 2048 ? 3 : 2;
            const int TXv = 1 << tx_log2, TYv = 1024 >> tx_log2;
            const int64_t tiles = outer * ((ivecs + TXv - 1) / TXv);
            const int share = TXv >= 8 ? 1 : 8 / TXv;
            const int64_t nblocks = (tiles + 8 * share - 1) / (8 * share) * (8 * share);
            if (nblocks < (int64_t(1) << 31)) {
                const bool few = (axis + TYv - 1) / TYv <= 4; // rows per thread
#define AXHIP_SMT_R(LOG, DT, R) hipLaunchKernelGGL((softmax_axis_tile_kernel<LOG, DT, R>), dim3(static_cast<unsigned>(nblocks)), dim3(1024), 0, s, src, outer, axis, inner, tx_log2, dst)
#define AXHIP_SMT_DT(LOG, DT)                                                                                                              \
    do {                                                                                                                                   \
        if (few) AXHIP_SMT_R(LOG, DT, 4);                                                                                                  \
        else AXHIP_SMT_R(LOG, DT, 16);                                                                                                     \
    } while (0)
#define AXHIP_SMT(LOG)                                                                                                                     \
    do {                                                                                                                                   \
        if (dtype == AXHIP_DTYPE_F32) AXHIP_SMT_DT(LOG, AXHIP_DTYPE_F32);                                                                  \
        else if (dtype == AXHIP_DTYPE_F16) AXHIP_SMT_DT(LOG, AXHIP_DTYPE_F16);                                                             \
        else AXHIP_SMT_DT(LOG, AXHIP_DTYPE_BF16);                                                                                          \
    } while (0)
                if (is_log) AXHIP_SMT(true);
                else AXHIP_SMT(false);
#undef AXHIP_SMT
#undef AXHIP_SMT_DT
#undef AXHIP_SMT_R
                AXHIP_CHECK_HIP(hipGetLastError());
                return AXHIP_OK;
            }
        }
        // a short axis with plenty of results: a thread per vector walks it alone
        const bool flat = axis <= 32 && outer * ((ivecs + 255) / 256) >= 1024;
        const bool wide = outer * ((ivecs + 31) / 32) >= 1024;
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(outer * (flat ? (ivecs + 255) / 256 : wide ? (ivecs + 31) / 32 : (ivecs + 7) / 8), 256 * 64));
#define AXHIP_SM_TX(LOG, DT, TX) hipLaunchKernelGGL((softmax_strided_vec_kernel<LOG, DT, TX>), dim3(blocks), dim3(256), 0, s, src, outer, axis, inner, dst)
#define AXHIP_SM_DT(LOG, DT)                                                                                                               \
    do {                                                                                                                                   \
        if (flat && axis <= 16) hipLaunchKernelGGL((softmax_strided_vec_kernel<LOG, DT, 256, 16>), dim3(blocks), dim3(256), 0, s, src, outer, axis, inner, dst); \
        else if (flat) AXHIP_SM_TX(LOG, DT, 256);                                                                                          \
        else if (wide) AXHIP_SM_TX(LOG, DT, 32);                                                                                           \
        else AXHIP_SM_TX(LOG, DT, 8);                                                                                                      \
    } while (0)
#define AXHIP_SM(LOG)                                                                                                                      \
    do {                                                                                                                                   \
        if (dtype == AXHIP_DTYPE_F32) AXHIP_SM_DT(LOG, AXHIP_DTYPE_F32);                                                                   \
        else if (dtype == AXHIP_DTYPE_F16) AXHIP_SM_DT(LOG, AXHIP_DTYPE_F16);                                                              \
        else AXHIP_SM_DT(LOG, AXHIP_DTYPE_BF16);                                                                                           \
    } while (0)
        if (is_log) AXHIP_SM(true);
        else AXHIP_SM(false);
#undef AXHIP_SM
#undef AXHIP_SM_DT
#undef AXHIP_SM_TX
    } else {
        const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((outer * inner + 255) / 256, 256 * 32));
        if (is_log) hipLaunchKernelGGL(softmax_strided_kernel<true>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, dst);
        else hipLaunchKernelGGL(softmax_strided_kernel<false>, dim3(blocks), dim3(256), 0, s, src, dtype, outer, axis, inner, dst);
    }
    AXHIP_CHECK_HIP(hipGetLastError());
    return AXHIP_OK;
}

} // extern "C"
