/*
 * axiom_oracle.c -- TEST INFRASTRUCTURE ONLY (see axiom_oracle.h).
 *
 * CPU restatement of Axiom's CPU algorithms for the SDPA and fused-chain hot
 * paths.  Written from the behaviour of the cited reference files, not copied
 * from them.  The shipped library never links this file.
 */
#include "axiom_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int axo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* Half-precision conversions                                               */
/* ------------------------------------------------------------------------ */

/* include/axiom/bfloat16.hpp:16-27: NaN -> 0x7FC0, otherwise add the
 * round-to-nearest-even bias 0x7FFF + lsb and truncate. */
uint16_t axo_f32_to_bf16(float f) {
    uint32_t u;
    if (f != f) return 0x7FC0u;
    memcpy(&u, &f, 4);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* include/axiom/bfloat16.hpp:41-46 */
float axo_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* include/axiom/float16.hpp:15,27 delegate to the FP16 library's
 * fp16_ieee_{from,to}_fp32_value, i.e. IEEE-754 binary16 with
 * round-to-nearest-even; restated from the standard. */
uint16_t axo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);        /* NaN */
    if (mag >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);       /* overflow -> inf (incl. ties at max+half ulp) */
    if (mag < 0x33000001u) return (uint16_t)sign;                    /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(mag >> 23) - 127;
    uint32_t m = (mag & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, half_bits;
    if (e < -14) {
        shift = (uint32_t)(13 + (-14 - e));   /* subnormal result */
        half_bits = 0;
    } else {
        shift = 13;
        half_bits = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    return (uint16_t)(sign | (half_bits + q));  /* carry propagates into the exponent */
}

float axo_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    uint32_t u;
    if (e == 0) {
        if (m == 0) {
            u = sign;
        } else {
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3FFu;
            u = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
        }
    } else if (e == 31) {
        u = sign | 0x7F800000u | (m << 13);
    } else {
        u = sign | ((e - 15 + 127) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline float ld(int dtype, const void *p, size_t i) {
    switch (dtype) {
    case AXO_F32: return ((const float *)p)[i];
    case AXO_F16: return axo_f16_to_f32(((const uint16_t *)p)[i]);
    default: return axo_bf16_to_f32(((const uint16_t *)p)[i]);
    }
}

static inline void st(int dtype, void *p, size_t i, float v) {
    switch (dtype) {
    case AXO_F32: ((float *)p)[i] = v; break;
    case AXO_F16: ((uint16_t *)p)[i] = axo_f32_to_f16(v); break;
    default: ((uint16_t *)p)[i] = axo_f32_to_bf16(v); break;
    }
}

/* value rounded to dtype and widened again */
static inline float rnd(int dtype, float v) {
    switch (dtype) {
    case AXO_F32: return v;
    case AXO_F16: return axo_f16_to_f32(axo_f32_to_f16(v));
    default: return axo_bf16_to_f32(axo_f32_to_bf16(v));
    }
}

void axo_convert(int sd, const void *src, int dd, void *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) st(dd, dst, i, ld(sd, src, i));
}

/* ------------------------------------------------------------------------ */
/* PCG-XSH-RR 64 -> 2x32 generator: include/axiom/random.hpp:12-68          */
/* ------------------------------------------------------------------------ */

static inline uint32_t pcg_step32(axo_pcg64 *g) {
    uint64_t old = g->state;
    g->state = old * 6364136223846793005ULL + g->inc;
    uint32_t xs = (uint32_t)(((old >> 18) ^ old) >> 27);
    uint32_t rot = (uint32_t)(old >> 59);
    return (xs >> rot) | (xs << ((32u - rot) & 31u));
}

uint64_t axo_pcg64_next(axo_pcg64 *g) {
    uint64_t hi = pcg_step32(g);
    uint64_t lo = pcg_step32(g);
    return (hi << 32) | lo;
}

/* random.hpp:24-30: state=0, inc=(stream<<1)|1, draw, state+=seed, draw */
void axo_pcg64_seed(axo_pcg64 *g, uint64_t seed, uint64_t stream) {
    g->state = 0;
    g->inc = (stream << 1) | 1u;
    (void)axo_pcg64_next(g);
    g->state += seed;
    (void)axo_pcg64_next(g);
}

/* random.hpp:85-87: 53-bit double in [0,1) */
static inline double pcg_double(axo_pcg64 *g) {
    return (double)(axo_pcg64_next(g) >> 11) * (1.0 / 9007199254740992.0);
}

void axo_fill_normal(axo_pcg64 *g, float *out, size_t n, float mean, float stddev) {
    const double two_pi = 6.283185307179586476925286766559;
    for (size_t i = 0; i < n; i += 2) {
        double u1 = 1.0 - pcg_double(g); /* (0,1] */
        double u2 = pcg_double(g);
        double r = sqrt(-2.0 * log(u1));
        out[i] = mean + stddev * (float)(r * cos(two_pi * u2));
        if (i + 1 < n) out[i + 1] = mean + stddev * (float)(r * sin(two_pi * u2));
    }
}

void axo_fill_uniform(axo_pcg64 *g, float *out, size_t n, float lo, float hi) {
    for (size_t i = 0; i < n; ++i) out[i] = lo + (hi - lo) * (float)pcg_double(g);
}

/* ------------------------------------------------------------------------ */
/* Native-tier sgemm: src/backends/cpu/blas/blas_native.cpp:28-185          */
/*   64x64 tiles of C held locally, K walked in chunks of 256, a*alpha      */
/*   formed first, then c += (a*alpha)*b sequentially over k.               */
/* ------------------------------------------------------------------------ */

#define GT_M 64
#define GT_N 64
#define GT_K 256

void axo_sgemm(int tA, int tB, size_t M, size_t N, size_t K, float alpha,
               const float *A, size_t lda, const float *B, size_t ldb, float beta,
               float *C, size_t ldc) {
    if (alpha == 0.0f) { /* blas_native.cpp:34-49 */
        for (size_t i = 0; i < M; ++i)
            for (size_t j = 0; j < N; ++j) {
                if (beta == 0.0f) C[i * ldc + j] = 0.0f;
                else if (beta != 1.0f) C[i * ldc + j] *= beta;
            }
        return;
    }
    for (size_t i0 = 0; i0 < M; i0 += GT_M) {
        for (size_t j0 = 0; j0 < N; j0 += GT_N) {
            float ct[GT_M][GT_N];
            size_t tm = (M - i0 < GT_M) ? M - i0 : GT_M;
            size_t tn = (N - j0 < GT_N) ? N - j0 : GT_N;
            for (size_t i = 0; i < tm; ++i)
                for (size_t j = 0; j < tn; ++j) {
                    if (beta == 0.0f) ct[i][j] = 0.0f;
                    else if (beta == 1.0f) ct[i][j] = C[(i0 + i) * ldc + j0 + j];
                    else ct[i][j] = C[(i0 + i) * ldc + j0 + j] * beta;
                }
            for (size_t k0 = 0; k0 < K; k0 += GT_K) {
                size_t tk = (K - k0 < GT_K) ? K - k0 : GT_K;
                for (size_t i = 0; i < tm; ++i)
                    for (size_t k = 0; k < tk; ++k) {
                        float a = (tA ? A[(k0 + k) * lda + i0 + i] : A[(i0 + i) * lda + k0 + k]) * alpha;
                        if (tB) {
                            for (size_t j = 0; j < tn; ++j) ct[i][j] += a * B[(j0 + j) * ldb + k0 + k];
                        } else {
                            const float *brow = B + (k0 + k) * ldb + j0;
                            for (size_t j = 0; j < tn; ++j) ct[i][j] += a * brow[j];
                        }
                    }
            }
            for (size_t i = 0; i < tm; ++i)
                for (size_t j = 0; j < tn; ++j) C[(i0 + i) * ldc + j0 + j] = ct[i][j];
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Tiled flash attention: src/backends/cpu/flash_attention_cpu.cpp:27-173   */
/* (one 64-row Q block against every 64-row K/V block; no causal skipping)  */
/* and its driver :177-281 (one slice per batch*head, OpenMP dynamic).      */
/* ------------------------------------------------------------------------ */

#define FA_BQ 64
#define FA_BKV 64

static void fa_tile(int dtype, const void *q, const void *k, const void *v, void *o,
                    size_t base_q, size_t base_kv, int Sq, int Skv, int D, float scale,
                    int causal, const uint8_t *mask, int q0) {
    int bq = Sq - q0 < FA_BQ ? Sq - q0 : FA_BQ;
    float *s = (float *)malloc(sizeof(float) * FA_BQ * FA_BKV);
    float *p = (float *)malloc(sizeof(float) * FA_BQ * FA_BKV);
    float *acc = (float *)calloc((size_t)bq * D, sizeof(float));
    float *qb = (float *)malloc(sizeof(float) * (size_t)bq * D);
    float *kb = (float *)malloc(sizeof(float) * (size_t)FA_BKV * D);
    float *vb = (float *)malloc(sizeof(float) * (size_t)FA_BKV * D);
    float m[FA_BQ], l[FA_BQ];
    for (int i = 0; i < bq; ++i) { m[i] = -INFINITY; l[i] = 0.0f; }
    for (int i = 0; i < bq; ++i)
        for (int d = 0; d < D; ++d) qb[(size_t)i * D + d] = ld(dtype, q, base_q + (size_t)(q0 + i) * D + d);

    for (int kv0 = 0; kv0 < Skv; kv0 += FA_BKV) {
        int bkv = Skv - kv0 < FA_BKV ? Skv - kv0 : FA_BKV;
        for (int i = 0; i < bkv; ++i)
            for (int d = 0; d < D; ++d) kb[(size_t)i * D + d] = ld(dtype, k, base_kv + (size_t)(kv0 + i) * D + d);
        /* :73-74  S = scale * Q K^T through the BLAS tier */
        axo_sgemm(0, 1, (size_t)bq, (size_t)bkv, (size_t)D, scale, qb, (size_t)D, kb, (size_t)D, 0.0f, s, (size_t)bkv);
        if (causal) /* :78-89  masked iff kv_pos > q_pos (top-left aligned) */
            for (int i = 0; i < bq; ++i)
                for (int j = 0; j < bkv; ++j)
                    if (kv0 + j > q0 + i) s[i * bkv + j] = -INFINITY;
        if (mask) /* :92-104  nonzero = masked out */
            for (int i = 0; i < bq; ++i)
                for (int j = 0; j < bkv; ++j)
                    if (mask[(size_t)(q0 + i) * Skv + kv0 + j]) s[i * bkv + j] = -INFINITY;
        for (int i = 0; i < bq; ++i) { /* :115-144 online softmax */
            float rmax = -INFINITY;
            for (int j = 0; j < bkv; ++j) rmax = fmaxf(rmax, s[i * bkv + j]);
            float mn = fmaxf(m[i], rmax);
            float alpha = expf(m[i] - mn);
            float rs = 0.0f;
            for (int j = 0; j < bkv; ++j) {
                float e = expf(s[i * bkv + j] - mn);
                p[i * bkv + j] = e;
                rs += e;
            }
            for (int d = 0; d < D; ++d) acc[(size_t)i * D + d] *= alpha;
            l[i] = alpha * l[i] + rs;
            m[i] = mn;
        }
        for (int i = 0; i < bkv; ++i)
            for (int d = 0; d < D; ++d) vb[(size_t)i * D + d] = ld(dtype, v, base_kv + (size_t)(kv0 + i) * D + d);
        /* :160-161  O += P V */
        axo_sgemm(0, 0, (size_t)bq, (size_t)D, (size_t)bkv, 1.0f, p, (size_t)bkv, vb, (size_t)D, 1.0f, acc, (size_t)D);
    }
    for (int i = 0; i < bq; ++i) { /* :165-172  O/l with the l>0 guard, cast to T */
        float inv = l[i] > 0.0f ? 1.0f / l[i] : 0.0f;
        for (int d = 0; d < D; ++d) st(dtype, o, base_q + (size_t)(q0 + i) * D + d, acc[(size_t)i * D + d] * inv);
    }
    free(s); free(p); free(acc); free(qb); free(kb); free(vb);
}

int axo_sdpa(int dtype, const void *q, const void *k, const void *v, void *o,
             int B, int H, int Sq, int Skv, int D, float scale, int is_causal,
             const uint8_t *mask, int mask_ndim, int mask_b, int mask_h,
             int slice_begin, int slice_end) {
    if (dtype < 0 || dtype > 2) return -1;
    if (mask && mask_ndim != 2 && mask_ndim != 4) return -2;
    if (scale <= 0.0f) scale = 1.0f / sqrtf((float)D); /* src/tensor/operations.cpp:4013-4015 */
    if (slice_end > B * H) slice_end = B * H;
#pragma omp parallel for schedule(dynamic)
    for (int sl = slice_begin; sl < slice_end; ++sl) {
        int b = sl / H, h = sl % H;
        size_t base_q = ((size_t)b * H + h) * (size_t)Sq * D;
        size_t base_kv = ((size_t)b * H + h) * (size_t)Skv * D;
        const uint8_t *ms = NULL;
        if (mask) {
            /* flash_attention_cpu.cpp:236-246 indexes a 4-D mask with the
             * mask's own extents; size-1 extents are broadcast here (the
             * reference only ever runs that case with B=H=1). */
            ms = mask;
            if (mask_ndim == 4) {
                size_t mb = mask_b == 1 ? 0 : (size_t)b, mh = mask_h == 1 ? 0 : (size_t)h;
                ms = mask + (mb * (size_t)mask_h + mh) * (size_t)Sq * Skv;
            }
        }
        for (int q0 = 0; q0 < Sq; q0 += FA_BQ)
            fa_tile(dtype, q, k, v, o, base_q, base_kv, Sq, Skv, D, scale, is_causal, ms, q0);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Softmax: src/backends/cpu/cpu_operations.cpp:3118-3162 (three passes per */
/* (outer, inner) lane: max, exp+sum, divide) and :3214-3233 (half types go */
/* through a float32 round trip).                                           */
/* ------------------------------------------------------------------------ */

static void softmax_f32(const float *in, float *out, size_t outer, size_t axis,
                        size_t inner, int is_log) {
    ptrdiff_t total = (ptrdiff_t)(outer * inner);
#pragma omp parallel for schedule(static) if (outer * inner * axis >= 65536)
    for (ptrdiff_t f = 0; f < total; ++f) {
        size_t o_ = (size_t)f / inner, i_ = (size_t)f % inner;
        float mx = -3.402823466e+38f; /* numeric_limits<float>::lowest() */
        for (size_t k = 0; k < axis; ++k) {
            float x = in[(o_ * axis + k) * inner + i_];
            mx = x > mx ? x : mx;
        }
        float sum = 0.0f;
        for (size_t k = 0; k < axis; ++k) {
            size_t idx = (o_ * axis + k) * inner + i_;
            float e = expf(in[idx] - mx);
            out[idx] = e;
            sum += e;
        }
        if (is_log) {
            float ls = logf(sum);
            for (size_t k = 0; k < axis; ++k) {
                size_t idx = (o_ * axis + k) * inner + i_;
                out[idx] = in[idx] - mx - ls;
            }
        } else {
            for (size_t k = 0; k < axis; ++k) out[(o_ * axis + k) * inner + i_] /= sum;
        }
    }
}

int axo_softmax(int dtype, const void *in, void *out, size_t outer, size_t axis,
                size_t inner, int is_log) {
    size_t n = outer * axis * inner;
    if (dtype == AXO_F32) {
        softmax_f32((const float *)in, (float *)out, outer, axis, inner, is_log);
        return 0;
    }
    if (dtype != AXO_F16 && dtype != AXO_BF16) return -1;
    float *a = (float *)malloc(n * sizeof(float)), *b = (float *)malloc(n * sizeof(float));
    axo_convert(dtype, in, AXO_F32, a, n);
    softmax_f32(a, b, outer, axis, inner, is_log);
    axo_convert(AXO_F32, b, dtype, out, n);
    free(a); free(b);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Elementwise functors: src/backends/cpu/cpu_operations.hpp:186-202        */
/* (add/sub/mul/div), :635-653 (gelu erf form, relu), and the scalar forms  */
/* beside them; :214-235 power (std::pow) and modulo (std::fmod), :237-291   */
/* comparisons and logical operations (any nonzero value is true), :360-381  */
/* atan2 / hypot, :395-400 logical not, :497-505 erf, :655-660 leaky ReLU,   */
/* :724-787 sign (0 for NaN) / floor / ceil / trunc / round (std::round),    */
/* :808-860 cbrt / isnan / isinf / isfinite.  Half types evaluate in float and round once per op         */
/* (include/axiom/bfloat16.hpp:55-73); gelu on a half type goes through     */
/* double (cpu_operations.hpp:643-646).                                     */
/* ------------------------------------------------------------------------ */

static inline float unary_f32(int op, float a) {
    switch (op) {
    case AXO_OP_RELU: return a > 0.0f ? a : 0.0f;
    case AXO_OP_GELU: return 0.5f * a * (1.0f + erff(a / 1.4142135623730951f));
    case AXO_OP_SQRT: return sqrtf(a);
    case AXO_OP_EXP: return expf(a);
    case AXO_OP_NEG: return -a;
    case AXO_OP_ABS: return fabsf(a);
    case AXO_OP_SIGMOID: {
        float e = expf(-fabsf(a)), d = 1.0f + e;
        return a >= 0.0f ? 1.0f / d : e / d;
    }
    case AXO_OP_TANH: return tanhf(a);
    case AXO_OP_SILU: return a / (1.0f + expf(-a));
    case AXO_OP_LOG: return logf(a);
    case AXO_OP_SQUARE: return a * a;
    case AXO_OP_RSQRT: return 1.0f / sqrtf(a);
    case AXO_OP_RECIP: return 1.0f / a;
    case AXO_OP_ERF: return erff(a);
    case AXO_OP_SIN: return sinf(a);
    case AXO_OP_COS: return cosf(a);
    case AXO_OP_TAN: return tanf(a);
    case AXO_OP_SIGN: return a > 0.0f ? 1.0f : a < 0.0f ? -1.0f : 0.0f;
    case AXO_OP_FLOOR: return floorf(a);
    case AXO_OP_CEIL: return ceilf(a);
    case AXO_OP_ROUND: return roundf(a);
    case AXO_OP_TRUNC: return truncf(a);
    case AXO_OP_CBRT: return cbrtf(a);
    case AXO_OP_ISNAN: return isnan(a) ? 1.0f : 0.0f;
    case AXO_OP_ISINF: return isinf(a) ? 1.0f : 0.0f;
    case AXO_OP_ISFINITE: return isfinite(a) ? 1.0f : 0.0f;
    case AXO_OP_NOT: return a != 0.0f ? 0.0f : 1.0f;
    default: return NAN;
    }
}

static inline float binary_f32(int op, float a, float b) {
    switch (op) {
    case AXO_OP_ADD: return a + b;
    case AXO_OP_SUB: return a - b;
    case AXO_OP_MUL: return a * b;
    case AXO_OP_DIV: return a / b;
    case AXO_OP_MAX: return a > b ? a : b;
    case AXO_OP_MIN: return a < b ? a : b;
    case AXO_OP_POW: return powf(a, b);
    case AXO_OP_RPOW: return powf(b, a);
    case AXO_OP_MOD: return fmodf(a, b);
    case AXO_OP_RMOD: return fmodf(b, a);
    case AXO_OP_ATAN2: return atan2f(a, b);
    case AXO_OP_RATAN2: return atan2f(b, a);
    case AXO_OP_HYPOT: return hypotf(a, b);
    case AXO_OP_EQ: return a == b ? 1.0f : 0.0f;
    case AXO_OP_NE: return a != b ? 1.0f : 0.0f;
    case AXO_OP_LT: return a < b ? 1.0f : 0.0f;
    case AXO_OP_LE: return a <= b ? 1.0f : 0.0f;
    case AXO_OP_GT: return a > b ? 1.0f : 0.0f;
    case AXO_OP_GE: return a >= b ? 1.0f : 0.0f;
    case AXO_OP_AND: return (a != 0.0f) && (b != 0.0f) ? 1.0f : 0.0f;
    case AXO_OP_OR: return (a != 0.0f) || (b != 0.0f) ? 1.0f : 0.0f;
    case AXO_OP_XOR: return (a != 0.0f) != (b != 0.0f) ? 1.0f : 0.0f;
    case AXO_OP_LEAKY_RELU: return a > 0.0f ? a : b * a; /* b: the slope */
    default: return NAN;
    }
}

int axo_unary(int op, int dtype, const void *in, void *out, size_t n) {
    if (dtype < 0 || dtype > 2) return -1;
#pragma omp parallel for schedule(static) if (n >= 65536)
    for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
        float a = ld(dtype, in, (size_t)i), r;
        if (dtype != AXO_F32 && op == AXO_OP_GELU)
            r = (float)(0.5 * (double)a * (1.0 + erf((double)a / 1.4142135623730951)));
        else
            r = unary_f32(op, a);
        st(dtype, out, (size_t)i, r);
    }
    return 0;
}

int axo_binary(int op, int dtype, const void *a, const void *b, void *out,
               size_t rows, size_t cols, int bk) {
    if (dtype < 0 || dtype > 2) return -1;
#pragma omp parallel for schedule(static) if (rows * cols >= 65536)
    for (ptrdiff_t r = 0; r < (ptrdiff_t)rows; ++r)
        for (size_t c = 0; c < cols; ++c) {
            size_t i = (size_t)r * cols + c;
            size_t j = bk == AXO_BK_FULL ? i : bk == AXO_BK_ROWVEC ? c : bk == AXO_BK_COLVEC ? (size_t)r : 0;
            st(dtype, out, i, binary_f32(op, ld(dtype, a, i), ld(dtype, b, j)));
        }
    return 0;
}

int axo_where(int dtype, const uint8_t *cond, const void *a, const void *b, void *out, size_t n) {
    if (dtype < 0 || dtype > 2) return -1;
    for (size_t i = 0; i < n; ++i) st(dtype, out, i, cond[i] ? ld(dtype, a, i) : ld(dtype, b, i));
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Last-axis reduction: src/backends/cpu/cpu_operations.cpp:1555-1617.      */
/* Float accumulation (also for half inputs, :1421-1424), mean divides the  */
/* row sum by the row length, half results are rounded back to the input    */
/* dtype (:1613-1614).  The reference reduces a row with a Highway SIMD     */
/* kernel whose lane count is machine-dependent; 8 interleaved partial sums */
/* stand in for it (the summation order is not part of the contract).       */
/* ------------------------------------------------------------------------ */

static float row_reduce(int red, int dtype, const void *in, size_t base, size_t n) {
    if (red == AXO_RED_SUM || red == AXO_RED_MEAN) {
        float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        size_t j = 0;
        for (; j + 8 <= n; j += 8)
            for (int t = 0; t < 8; ++t) lane[t] += ld(dtype, in, base + j + t);
        float s = ((lane[0] + lane[4]) + (lane[2] + lane[6])) + ((lane[1] + lane[5]) + (lane[3] + lane[7]));
        for (; j < n; ++j) s += ld(dtype, in, base + j);
        return s;
    }
    if (red == AXO_RED_PROD) { /* a running float product, in index order */
        float p = 1.0f;
        for (size_t j = 0; j < n; ++j) p *= ld(dtype, in, base + j);
        return p;
    }
    float r = ld(dtype, in, base);
    for (size_t j = 1; j < n; ++j) {
        float x = ld(dtype, in, base + j);
        r = red == AXO_RED_MAX ? (x > r ? x : r) : (x < r ? x : r);
    }
    return r;
}

int axo_reduce_last(int red, int dtype, const void *in, void *out, size_t rows, size_t cols) {
    if (dtype < 0 || dtype > 2 || red < 1 || red > 5 || cols == 0) return -1;
#pragma omp parallel for schedule(static) if (rows >= 64)
    for (ptrdiff_t r = 0; r < (ptrdiff_t)rows; ++r) {
        float s = row_reduce(red, dtype, in, (size_t)r * cols, cols);
        if (red == AXO_RED_MEAN) s /= (float)cols;
        st(dtype, out, (size_t)r, s);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* argmax / argmin over an axis: src/backends/cpu/cpu_operations.cpp:2157-2229 */
/* (argmin: the same loop with `<` and max(), :2258-2330).  The scan starts */
/* at index 0 with the type's lowest() (argmin: max()) as the value to beat */
/* and moves on a STRICT comparison in the input's own type: the first      */
/* occurrence of the extreme wins, a NaN never does, and a slice with       */
/* nothing above lowest() (all -inf, all NaN) answers 0.  Indices are int64 */
/* (:2186).  Half values compare as their exact float images.               */
/* ------------------------------------------------------------------------ */

int axo_argreduce(int want_min, int dtype, const void *in, int64_t *out, size_t outer, size_t axis, size_t inner) {
    if (dtype < 0 || dtype > 2) return -1;
    /* lowest() of the type: -FLT_MAX, -65504 (float16.hpp:82-), 0xFF7F as bfloat16 (bfloat16.hpp:116-118) */
    const float lowest = dtype == AXO_F32 ? -3.402823466e+38f : dtype == AXO_F16 ? -65504.0f : axo_bf16_to_f32(0xFF7F);
#pragma omp parallel for schedule(static) if (outer * inner >= 64)
    for (ptrdiff_t oi = 0; oi < (ptrdiff_t)(outer * inner); ++oi) {
        const size_t o = (size_t)oi / inner, i = (size_t)oi % inner;
        size_t best_idx = 0;
        float best = want_min ? -lowest : lowest;
        for (size_t k = 0; k < axis; ++k) {
            const float v = ld(dtype, in, (o * axis + k) * inner + i);
            if (want_min ? v < best : v > best) {
                best = v;
                best_idx = k;
            }
        }
        out[oi] = (int64_t)best_idx;
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* layer_norm on CPU: src/tensor/operations.cpp:1803-1817, a chain of       */
/*   mean -> subtract -> multiply -> mean -> add(eps) -> sqrt -> divide ->  */
/*   multiply(w) -> add(b).                                                 */
/* dtype flow for a half input: the Mean node is typed Float32              */
/* (src/graph/graph_registry.cpp:278-287) but the CPU reduction returns the */
/* input dtype (cpu_operations.cpp:1613-1614) and is only then widened      */
/* (src/graph/graph_executor.cpp:396-403): the first mean is rounded to the */
/* half type; every later op runs in float32 by promotion                   */
/* (src/tensor/operations.cpp:346-364), so the result is float32.           */
/* ------------------------------------------------------------------------ */

int axo_layer_norm(int dtype, const void *x, const void *w, const void *b,
                   float *out, size_t rows, size_t cols, float eps) {
    if (dtype < 0 || dtype > 2 || cols == 0) return -1;
#pragma omp parallel for schedule(static) if (rows >= 64)
    for (ptrdiff_t r = 0; r < (ptrdiff_t)rows; ++r) {
        size_t base = (size_t)r * cols;
        float mean = rnd(dtype, row_reduce(AXO_RED_SUM, dtype, x, base, cols) / (float)cols);
        float *y = out + base;
        for (size_t c = 0; c < cols; ++c) {
            float xc = ld(dtype, x, base + c) - mean;
            y[c] = xc * xc;
        }
        float var = row_reduce(AXO_RED_SUM, AXO_F32, y, 0, cols) / (float)cols;
        float sd = sqrtf(var + eps);
        for (size_t c = 0; c < cols; ++c) {
            float v = (ld(dtype, x, base + c) - mean) / sd;
            if (w) v = v * ld(dtype, w, c);
            if (b) v = v + ld(dtype, b, c);
            y[c] = v;
        }
    }
    return 0;
}

/* rms_norm on CPU: src/tensor/operations.cpp:1849-1857:                    */
/*   multiply(x,x) -> mean -> add(eps) -> sqrt -> divide(x, rms) -> mul(w). */
/* For a half input x*x is a half-typed op (rounded per element), its mean  */
/* is rounded to the half type as above, and the rest is float32.           */
int axo_rms_norm(int dtype, const void *x, const void *w, float *out,
                 size_t rows, size_t cols, float eps) {
    if (dtype < 0 || dtype > 2 || cols == 0) return -1;
#pragma omp parallel for schedule(static) if (rows >= 64)
    for (ptrdiff_t r = 0; r < (ptrdiff_t)rows; ++r) {
        size_t base = (size_t)r * cols;
        float *y = out + base;
        for (size_t c = 0; c < cols; ++c) {
            float v = ld(dtype, x, base + c);
            y[c] = rnd(dtype, v * v);
        }
        float ms = rnd(dtype, row_reduce(AXO_RED_SUM, AXO_F32, y, 0, cols) / (float)cols);
        float rms = sqrtf(ms + eps);
        for (size_t c = 0; c < cols; ++c) {
            float v = ld(dtype, x, base + c) / rms;
            if (w) v = v * ld(dtype, w, c);
            y[c] = v;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* matmul on CPU: src/backends/cpu/cpu_operations.cpp:1772-1883.  float32   */
/* goes to the BLAS tier; half types use the 64x64x256 tiled loop whose     */
/* accumulator is the half type itself, so every product and every += is    */
/* rounded (:1860).                                                         */
/* ------------------------------------------------------------------------ */

int axo_matmul(int dtype, const void *A, const void *B, void *C, size_t M,
               size_t N, size_t K, int tA, int tB) {
    if (dtype == AXO_F32) {
        axo_sgemm(tA, tB, M, N, K, 1.0f, (const float *)A, tA ? M : K, (const float *)B, tB ? K : N, 0.0f, (float *)C, N);
        return 0;
    }
    if (dtype != AXO_F16 && dtype != AXO_BF16) return -1;
    size_t ars = tA ? 1 : K, acs = tA ? M : 1, brs = tB ? 1 : N, bcs = tB ? K : 1;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (ptrdiff_t i0 = 0; i0 < (ptrdiff_t)M; i0 += GT_M)
        for (ptrdiff_t j0 = 0; j0 < (ptrdiff_t)N; j0 += GT_N) {
            float ct[GT_M][GT_N];
            size_t tm = (M - (size_t)i0 < GT_M) ? M - (size_t)i0 : GT_M;
            size_t tn = (N - (size_t)j0 < GT_N) ? N - (size_t)j0 : GT_N;
            for (size_t i = 0; i < tm; ++i)
                for (size_t j = 0; j < tn; ++j) ct[i][j] = 0.0f;
            for (size_t k0 = 0; k0 < K; k0 += GT_K) {
                size_t tk = (K - k0 < GT_K) ? K - k0 : GT_K;
                for (size_t i = 0; i < tm; ++i)
                    for (size_t k = 0; k < tk; ++k) {
                        float a = ld(dtype, A, ((size_t)i0 + i) * ars + (k0 + k) * acs);
                        for (size_t j = 0; j < tn; ++j) {
                            float bv = ld(dtype, B, (k0 + k) * brs + ((size_t)j0 + j) * bcs);
                            ct[i][j] = rnd(dtype, ct[i][j] + rnd(dtype, a * bv));
                        }
                    }
            }
            for (size_t i = 0; i < tm; ++i)
                for (size_t j = 0; j < tn; ++j) st(dtype, C, ((size_t)i0 + i) * N + (size_t)j0 + j, ct[i][j]);
        }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* The relu -> +1 -> *b -> softmax -> sum(1) chain as the CPU path runs it: */
/* three op-by-op elementwise passes (the {1}-shaped scalar operand keeps   */
/* the tiled fused loop from engaging, src/graph/graph_executor.cpp:205-218 */
/* and :641-690), an eager three-pass softmax (src/tensor/operations.cpp:   */
/* 1427-1434) and a last-axis row reduction.                                */
/* ------------------------------------------------------------------------ */

int axo_chain_relu_add_mul_softmax_sum(const float *a, const float *b, float *out,
                                       float *softmax_out, size_t rows, size_t cols) {
    size_t n = rows * cols;
    float one = 1.0f;
    float *t0 = (float *)malloc(n * sizeof(float));
    float *t1 = softmax_out ? softmax_out : (float *)malloc(n * sizeof(float));
    if (!t0 || !t1) return -1;
    axo_unary(AXO_OP_RELU, AXO_F32, a, t0, n);
    axo_binary(AXO_OP_ADD, AXO_F32, t0, &one, t0, rows, cols, AXO_BK_SCALAR);
    axo_binary(AXO_OP_MUL, AXO_F32, t0, b, t0, rows, cols, AXO_BK_FULL);
    axo_softmax(AXO_F32, t0, t1, rows, cols, 1, 0);
    axo_reduce_last(AXO_RED_SUM, AXO_F32, t1, out, rows, cols);
    free(t0);
    if (!softmax_out) free(t1);
    return 0;
}
