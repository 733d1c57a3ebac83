// Shared host/device helpers for the gfx950 backend.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "axhip.h"

namespace axhip {

// ---------------------------------------------------------------- host side
void set_last_error(const char *fmt, ...);
hipStream_t resolve_stream(void *stream);
int ensure_init();
int rows_setup_device(); // per-device set-up of the fused-row kernels (rows.hip), run by axhip_init

#define AXHIP_CHECK_HIP(expr)                                                          \
    do {                                                                               \
        hipError_t _e = (expr);                                                        \
        if (_e != hipSuccess) {                                                        \
            ::axhip::set_last_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                    __FILE__, __LINE__);                               \
            return static_cast<int>(_e);                                               \
        }                                                                              \
    } while (0)

#define AXHIP_REQUIRE(cond, code, ...)                \
    do {                                              \
        if (!(cond)) {                                \
            ::axhip::set_last_error(__VA_ARGS__);     \
            return (code);                            \
        }                                             \
    } while (0)

// Temporary device memory of ONE call.  With a caller's workspace (the *_ws entry points) it hands out 256-byte
// aligned slices of that and allocates nothing; without one (workspace == NULL) every request is a stream-ordered
// allocation that is returned in stream order when the call ends.
class CallScratch {
public:
    CallScratch(void *workspace, size_t workspace_bytes, hipStream_t stream)
        : base_(static_cast<char *>(workspace)), bytes_(workspace_bytes), stream_(stream) {}
    CallScratch(const CallScratch &) = delete;
    CallScratch &operator=(const CallScratch &) = delete;
    ~CallScratch() { (void)release(); }
    static size_t rounded(size_t n) { return (n + 255) & ~static_cast<size_t>(255); }
    int take(void **out, size_t n, const char *who) {
        *out = nullptr;
        if (base_) {
            const size_t at = rounded(used_);
            if (at + n > bytes_) {
                set_last_error("%s: the workspace holds %zu bytes, the call needs %zu (ask %s_workspace_bytes)", who, bytes_, at + n, who);
                return AXHIP_ERR_WORKSPACE;
            }
            *out = base_ + at;
            used_ = at + n;
            return AXHIP_OK;
        }
        if (n_own_ >= MAX_OWN) {
            set_last_error("%s: too many temporary allocations in one call", who);
            return AXHIP_ERR_UNSUPPORTED;
        }
        const hipError_t e = hipMallocAsync(out, n, stream_);
        if (e != hipSuccess) {
            set_last_error("%s: hipMallocAsync of %zu bytes failed: %s", who, n, hipGetErrorString(e));
            return static_cast<int>(e);
        }
        own_[n_own_++] = *out;
        return AXHIP_OK;
    }
    // everything handed out so far may be handed out again (work on one stream runs in order)
    void rewind() { if (base_) used_ = 0; }
    int release() {
        hipError_t first = hipSuccess;
        for (int i = 0; i < n_own_; ++i) {
            const hipError_t e = hipFreeAsync(own_[i], stream_);
            if (first == hipSuccess) first = e;
        }
        n_own_ = 0;
        if (first != hipSuccess) set_last_error("hipFreeAsync failed: %s", hipGetErrorString(first));
        return static_cast<int>(first);
    }

private:
    static constexpr int MAX_OWN = 8;
    char *base_;
    size_t bytes_, used_ = 0;
    hipStream_t stream_;
    void *own_[MAX_OWN] = {};
    int n_own_ = 0;
};

inline bool valid_dtype(int dt) { return dt >= AXHIP_DTYPE_F32 && dt <= AXHIP_DTYPE_BF16; }
inline bool valid_dtype_or_u8(int dt) { return valid_dtype(dt) || dt == AXHIP_DTYPE_U8; }
inline size_t dtype_size(int dt) { return dt == AXHIP_DTYPE_F32 ? 4 : dt == AXHIP_DTYPE_U8 ? 1 : 2; }
// Outputs of at least this size are written with non-temporal stores: they cannot stay in the
// 256 MiB last-level cache next to the launch's inputs anyway, and a consumer that follows
// immediately could not find them there either.
constexpr int64_t STREAMING_OUTPUT_BYTES = 64ll << 20;

// -------------------------------------------------------------- device side
constexpr int WAVE = 64;

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

// bf16 <-> f32 with the same rounding as Axiom's bfloat16_t: round to nearest
// even, NaN canonicalised to 0x7FC0.
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? 0x7FC0u : r;
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f)); // v_cvt_f16_f32: RNE
}

// two fp32 values to one packed f16 pair (v_cvt_pk_f16_f32: round to nearest even)
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    float2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, half2_t));
}

// two fp32 values to one packed bf16 pair with the hardware conversion (v_cvt_pk_bf16_f32:
// round to nearest even; a NaN stays a quiet NaN)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const float2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

template <int DT> struct Elem;
template <> struct Elem<AXHIP_DTYPE_F32> {
    using type = float;
    __device__ static float load(const void *p, int64_t i) { return static_cast<const float *>(p)[i]; }
    __device__ static void store(void *p, int64_t i, float v) { static_cast<float *>(p)[i] = v; }
};
template <> struct Elem<AXHIP_DTYPE_F16> {
    using type = uint16_t;
    __device__ static float load(const void *p, int64_t i) { return f16_bits_to_f32(static_cast<const uint16_t *>(p)[i]); }
    __device__ static void store(void *p, int64_t i, float v) { static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(f32_to_f16_bits(v)); }
};
template <> struct Elem<AXHIP_DTYPE_BF16> {
    using type = uint16_t;
    __device__ static float load(const void *p, int64_t i) { return bf16_bits_to_f32(static_cast<const uint16_t *>(p)[i]); }
    __device__ static void store(void *p, int64_t i, float v) { static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v)); }
};

__device__ __forceinline__ float load_any(const void *p, int dt, int64_t i) {
    if (dt == AXHIP_DTYPE_F32) return static_cast<const float *>(p)[i];
    if (dt == AXHIP_DTYPE_U8) return static_cast<const uint8_t *>(p)[i] ? 1.0f : 0.0f;
    uint32_t h = static_cast<const uint16_t *>(p)[i];
    return dt == AXHIP_DTYPE_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}
__device__ __forceinline__ void store_any(void *p, int dt, int64_t i, float v) {
    if (dt == AXHIP_DTYPE_F32) {
        static_cast<float *>(p)[i] = v;
    } else if (dt == AXHIP_DTYPE_U8) {
        static_cast<uint8_t *>(p)[i] = v != 0.0f ? 1 : 0;
    } else {
        static_cast<uint16_t *>(p)[i] =
            static_cast<uint16_t>(dt == AXHIP_DTYPE_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v));
    }
}

// x * Phi(x) for 16-bit outputs: Phi(x) = 0.5 + u*P(u^2) with u = clamp(x, -C, C),
// P a degree-8 minimax fit; the result is clamped to [0, 1] so both tails are
// exact.  |error| <= 5e-5 absolute over the whole line, under half a bf16 ulp
// for |gelu| > 0.02, at 12 VALU operations and no transcendental (erff costs ~3x).
__device__ __forceinline__ float gelu_fast(float x) {
    constexpr float C = 4.45f;
    const float u = __builtin_amdgcn_fmed3f(x, -C, C);
    const float t = u * u;
    float p = 3.455728e-11f;
    p = __builtin_fmaf(p, t, -3.6776806e-09f);
    p = __builtin_fmaf(p, t, 1.7219786e-07f);
    p = __builtin_fmaf(p, t, -4.7068065e-06f);
    p = __builtin_fmaf(p, t, 8.4325635e-05f);
    p = __builtin_fmaf(p, t, -0.0010570257f);
    p = __builtin_fmaf(p, t, 0.009658655f);
    p = __builtin_fmaf(p, t, -0.06612378f);
    p = __builtin_fmaf(p, t, 0.39880943f);
    const float phi = __builtin_amdgcn_fmed3f(__builtin_fmaf(u, p, 0.5f), 0.0f, 1.0f);
    return x * phi;
}

// Vector accesses at element alignment only (rows of odd length): the same 16-byte instructions, which the
// hardware executes at any alignment; the packed types tell the compiler not to assume more.
struct __attribute__((packed, aligned(4))) float4_unaligned_t { float4_t v; };
struct __attribute__((packed, aligned(2))) uint4_unaligned_t { uint4_t v; };
struct __attribute__((packed, aligned(2))) uint2_unaligned_t { uint2_t v; };
template <bool UNALIGNED> __device__ __forceinline__ float4_t vec_load(const float4_t *p) {
    if constexpr (UNALIGNED) return reinterpret_cast<const float4_unaligned_t *>(p)->v;
    else return *p;
}
template <bool UNALIGNED> __device__ __forceinline__ uint4_t vec_load(const uint4_t *p) {
    if constexpr (UNALIGNED) return reinterpret_cast<const uint4_unaligned_t *>(p)->v;
    else return *p;
}
template <bool UNALIGNED> __device__ __forceinline__ uint2_t vec_load(const uint2_t *p) {
    if constexpr (UNALIGNED) return reinterpret_cast<const uint2_unaligned_t *>(p)->v;
    else return *p;
}
template <bool UNALIGNED> __device__ __forceinline__ void vec_store(float4_t *p, float4_t t) {
    if constexpr (UNALIGNED) reinterpret_cast<float4_unaligned_t *>(p)->v = t;
    else *p = t;
}
template <bool UNALIGNED> __device__ __forceinline__ void vec_store(uint4_t *p, uint4_t t) {
    if constexpr (UNALIGNED) reinterpret_cast<uint4_unaligned_t *>(p)->v = t;
    else *p = t;
}
template <bool UNALIGNED> __device__ __forceinline__ void vec_store(uint2_t *p, uint2_t t) {
    if constexpr (UNALIGNED) reinterpret_cast<uint2_unaligned_t *>(p)->v = t;
    else *p = t;
}

// Load / store N consecutive elements (N*sizeof(elem) is 16 or 32 bytes and, unless UNALIGNED, the
// address is aligned to min(16, that)) as fp32 values.
struct __attribute__((packed, aligned(1))) uint32_unaligned_t { uint32_t v; };

template <int N, bool UNALIGNED = false>
__device__ __forceinline__ void load_vec(const void *p, int dt, int64_t i, float (&v)[N]) {
    if (dt == AXHIP_DTYPE_U8) { // N bytes, in 32-bit words (the address is N-aligned unless UNALIGNED)
        static_assert(N % 4 == 0, "vector width");
        const uint8_t *q = static_cast<const uint8_t *>(p) + i;
#pragma unroll
        for (int j = 0; j < N / 4; ++j) {
            uint32_t w;
            if constexpr (UNALIGNED) w = reinterpret_cast<const uint32_unaligned_t *>(q + 4 * j)->v;
            else w = *reinterpret_cast<const uint32_t *>(q + 4 * j);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[4 * j + k] = ((w >> (8 * k)) & 0xFFu) ? 1.0f : 0.0f;
        }
    } else if (dt == AXHIP_DTYPE_F32) {
        const float4_t *q = reinterpret_cast<const float4_t *>(static_cast<const float *>(p) + i);
#pragma unroll
        for (int j = 0; j < N / 4; ++j) {
            float4_t t = vec_load<UNALIGNED>(q + j);
            v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
        }
    } else {
        static_assert(N % 4 == 0, "vector width");
        if constexpr (N % 8 == 0) {
            const uint4_t *q = reinterpret_cast<const uint4_t *>(static_cast<const uint16_t *>(p) + i);
#pragma unroll
            for (int j = 0; j < N / 8; ++j) {
                uint4_t t = vec_load<UNALIGNED>(q + j);
                uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (dt == AXHIP_DTYPE_BF16) {
                        v[8 * j + 2 * k] = __uint_as_float(w[k] << 16);
                        v[8 * j + 2 * k + 1] = __uint_as_float(w[k] & 0xFFFF0000u);
                    } else {
                        v[8 * j + 2 * k] = f16_bits_to_f32(w[k] & 0xFFFFu);
                        v[8 * j + 2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
                    }
                }
            }
        } else {
            const uint2_t *q = reinterpret_cast<const uint2_t *>(static_cast<const uint16_t *>(p) + i);
            uint2_t t = vec_load<UNALIGNED>(q);
            uint32_t w[2] = {t.x, t.y};
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (dt == AXHIP_DTYPE_BF16) {
                    v[2 * k] = __uint_as_float(w[k] << 16);
                    v[2 * k + 1] = __uint_as_float(w[k] & 0xFFFF0000u);
                } else {
                    v[2 * k] = f16_bits_to_f32(w[k] & 0xFFFFu);
                    v[2 * k + 1] = f16_bits_to_f32(w[k] >> 16);
                }
            }
        }
    }
}

// 16-byte non-temporal store.  Written as an instruction because a builtin non-temporal store in
// one arm of a run-time branch is merged with the ordinary store of the other arm, losing the hint.
__device__ __forceinline__ void store16_streaming(void *p, uint4_t v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(p), "v"(v) : "memory");
}

// `streaming`: non-temporal stores, for outputs far larger than the caches (they then do not
// push the inputs of the same launch out of the last-level cache)
template <int N, bool UNALIGNED = false>
__device__ __forceinline__ void store_vec(void *p, int dt, int64_t i, const float (&v)[N], bool streaming = false) {
    if (dt == AXHIP_DTYPE_U8) {
        static_assert(N % 4 == 0, "vector width");
        uint8_t *q = static_cast<uint8_t *>(p) + i;
#pragma unroll
        for (int j = 0; j < N / 4; ++j) {
            uint32_t w = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) w |= (v[4 * j + k] != 0.0f ? 1u : 0u) << (8 * k);
            if constexpr (UNALIGNED) reinterpret_cast<uint32_unaligned_t *>(q + 4 * j)->v = w;
            else *reinterpret_cast<uint32_t *>(q + 4 * j) = w;
        }
    } else if (dt == AXHIP_DTYPE_F32) {
        float4_t *q = reinterpret_cast<float4_t *>(static_cast<float *>(p) + i);
#pragma unroll
        for (int j = 0; j < N / 4; ++j) {
            float4_t t = {v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]};
            if (streaming) store16_streaming(&q[j], __builtin_bit_cast(uint4_t, t));
            else vec_store<UNALIGNED>(q + j, t);
        }
    } else {
        uint32_t w[N / 2];
#pragma unroll
        for (int k = 0; k < N / 2; ++k) {
            if (dt == AXHIP_DTYPE_BF16) {
                w[k] = pack_bf16x2(v[2 * k], v[2 * k + 1]);
            } else {
                w[k] = pack_f16x2(v[2 * k], v[2 * k + 1]);
            }
        }
        if constexpr (N % 8 == 0) {
            uint4_t *q = reinterpret_cast<uint4_t *>(static_cast<uint16_t *>(p) + i);
#pragma unroll
            for (int j = 0; j < N / 8; ++j) {
                uint4_t t = {w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]};
                if (streaming) store16_streaming(&q[j], t);
                else vec_store<UNALIGNED>(q + j, t);
            }
        } else {
            uint2_t *q = reinterpret_cast<uint2_t *>(static_cast<uint16_t *>(p) + i);
            uint2_t t = {w[0], w[1]};
            vec_store<UNALIGNED>(q, t);
        }
    }
}

// wavefront (64 lanes) all-reduce through cross-lane shuffles
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_prod(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v *= __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, WAVE));
    return v;
}

} // namespace axhip
