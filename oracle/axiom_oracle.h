/*
 * axiom_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU restatement of the arithmetic that Axiom's own CPU backend
 * performs on the two GPU hot paths (scaled-dot-product attention and the
 * fused elementwise / softmax / norm chains).  It exists so that the HIP
 * kernels can be checked against the reference's CPU algorithm on identical
 * inputs, and so that a CPU baseline can be timed beside the GPU numbers.
 *
 * Nothing in the shipped library links, loads or calls this file.  Only the
 * test suite, the smoke check and the benchmark's cpu_baseline leg may.
 *
 * Each function cites the reference file:line it follows (paths are relative
 * to the Axiom source tree).
 *
 * How each function is pinned (nothing here is "parity unpinned"):
 *   axo_f32_to_bf16 / axo_bf16_to_f32  bit patterns asserted by the
 *       reference's tests/test_bfloat16.cpp:14-57 and an exhaustive check
 *       against the round-to-nearest-even definition.
 *   axo_f32_to_f16 / axo_f16_to_f32    IEEE binary16, exhaustive over all
 *       65536 half patterns against numpy's float16.
 *   axo_pcg64_*    first outputs compared with the reference's own
 *       include/axiom/random.hpp compiled into oracle/_ref.
 *   axo_sgemm      compared with the reference's native BLAS tier compiled
 *       into oracle/_ref (bitwise) and with numpy float64 matmul.
 *   axo_sdpa       textbook softmax(scale*Q*K^T + mask)*V in float64 on the
 *       shape cases of tests/test_flash_attention.cpp:76-213,334-355; S=1
 *       gives O=V; a fully masked row gives 0; causal == explicit triangular
 *       mask.
 *   axo_softmax    rows sum to 1, equal inputs give equal outputs
 *       (tests/test_tensor_activations.cpp:11-52); float64 closed form.
 *   axo_unary/axo_binary   exact IEEE single-rounding identities; gelu(0)=0,
 *       erf(1)=0.8427 (tests/test_tensor_activations.cpp:310-375); the 12
 *       fused-pattern known answers of tests/test_fusion_extended.cpp:114-220.
 *       The wider operator table (op codes 40-77): the comparison vectors of
 *       tests/test_tensor_comparisons.cpp:24-113, the logical truth tables and
 *       atan2 / hypot values of tests/test_tensor_logical_bitwise.cpp:11-70,
 *       245-277, sign / floor / ceil / trunc / cbrt / isnan / isinf / isfinite /
 *       clip of tests/test_tensor_numpy_ops.cpp:13-88, erf of
 *       tests/test_tensor_activations.cpp:356-375, 3^4 = 81 of
 *       tests/test_tensor_operations.cpp:107-121; where the reference's tests
 *       hold no value, what the functor's definition fixes: fmod keeps the
 *       dividend's sign, round moves halves away from zero, sign(NaN) = 0,
 *       leaky ReLU's slope, the reversed forms against the forward ones, sin /
 *       cos / tan against libm in float64.
 *   axo_where      the vectors of tests/test_tensor_where.cpp:26-36, 176-205.
 *   axo_reduce_last  sum(a+b)=80 and 1 Mi ones*2 = 2097152
 *       (tests/test_fusion_extended.cpp:346-352,436-443); float64 reference;
 *       prod: 24 and {3, 8} of tests/test_tensor_numpy_ops.cpp:91-104,
 *       prod(sqrt([4,9,16])) = 24 of tests/test_fusion_extended.cpp:376-385;
 *       any / all as the extreme truth value, tests/test_tensor_activations.cpp:446-478.
 *   axo_layer_norm   mean~0 / var~1 (tests/test_tensor_normalization.cpp:9-74);
 *       float64 closed form.
 *   axo_rms_norm     [3,4] -> [3,4]/sqrt(12.5)
 *       (tests/test_tensor_normalization.cpp:80-141); [1,2,3,4][0]=1/sqrt(7.5)
 *       (tests/test_nn_layers.cpp:191-207).
 *   axo_matmul       float64 reference; Linear known answers 3/4/2/8
 *       (tests/test_nn_layers.cpp:12-73).
 *   axo_argreduce    the known answers of tests/test_tensor_argmax_argmin.cpp:4-112
 *       (1-D, both axes of [[1,5],[3,2]], arange(24) as (2,3,4)); numpy's
 *       argmax / argmin on data without NaN (same first-occurrence rule); the
 *       NaN / -inf cases by the scan's own definition on 3-element rows.
 */
#ifndef AXIOM_ORACLE_H
#define AXIOM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes, identical to the C-ABI's AXHIP_DTYPE_* */
enum { AXO_F32 = 0, AXO_F16 = 1, AXO_BF16 = 2 };

/* unary / binary / reduce op codes, identical to the C-ABI's AXHIP_OP_* */
enum {
    AXO_OP_ADD = 1, AXO_OP_SUB = 2, AXO_OP_MUL = 3, AXO_OP_DIV = 4,
    AXO_OP_MAX = 5, AXO_OP_MIN = 6,
    AXO_OP_RELU = 16, AXO_OP_GELU = 17, AXO_OP_SQRT = 18, AXO_OP_EXP = 19,
    AXO_OP_NEG = 20, AXO_OP_ABS = 21, AXO_OP_SIGMOID = 22, AXO_OP_TANH = 23,
    AXO_OP_SILU = 24, AXO_OP_LOG = 25, AXO_OP_SQUARE = 26, AXO_OP_RSQRT = 27,
    AXO_OP_RECIP = 28,
    /* binary: the running value is the first argument; R* forms take it as the second */
    AXO_OP_POW = 40, AXO_OP_RPOW = 41, AXO_OP_MOD = 42, AXO_OP_RMOD = 43, AXO_OP_ATAN2 = 44,
    AXO_OP_RATAN2 = 45, AXO_OP_HYPOT = 46, AXO_OP_EQ = 47, AXO_OP_NE = 48, AXO_OP_LT = 49,
    AXO_OP_LE = 50, AXO_OP_GT = 51, AXO_OP_GE = 52, AXO_OP_AND = 53, AXO_OP_OR = 54,
    AXO_OP_XOR = 55, AXO_OP_LEAKY_RELU = 56,
    /* unary */
    AXO_OP_ERF = 64, AXO_OP_SIN = 65, AXO_OP_COS = 66, AXO_OP_TAN = 67, AXO_OP_SIGN = 68,
    AXO_OP_FLOOR = 69, AXO_OP_CEIL = 70, AXO_OP_ROUND = 71, AXO_OP_TRUNC = 72, AXO_OP_CBRT = 73,
    AXO_OP_ISNAN = 74, AXO_OP_ISINF = 75, AXO_OP_ISFINITE = 76, AXO_OP_NOT = 77
};
enum { AXO_RED_SUM = 1, AXO_RED_MEAN = 2, AXO_RED_MAX = 3, AXO_RED_MIN = 4, AXO_RED_PROD = 5 };

/* broadcast kind of the second operand of a binary op over a [rows, cols] view */
enum { AXO_BK_FULL = 0, AXO_BK_ROWVEC = 1, AXO_BK_COLVEC = 2, AXO_BK_SCALAR = 3 };

uint16_t axo_f32_to_bf16(float f);
float axo_bf16_to_f32(uint16_t h);
uint16_t axo_f32_to_f16(float f);
float axo_f16_to_f32(uint16_t h);
void axo_convert(int src_dtype, const void *src, int dst_dtype, void *dst, size_t n);

typedef struct { uint64_t state, inc; } axo_pcg64;
void axo_pcg64_seed(axo_pcg64 *g, uint64_t seed, uint64_t stream);
uint64_t axo_pcg64_next(axo_pcg64 *g);
/* N(0,1) floats by Box-Muller over the generator's 53-bit doubles; the
 * reference draws through libstdc++'s std::normal_distribution, whose
 * algorithm is implementation-defined, so inputs are generated once on the
 * host and handed to both paths rather than regenerated. */
void axo_fill_normal(axo_pcg64 *g, float *out, size_t n, float mean, float stddev);
void axo_fill_uniform(axo_pcg64 *g, float *out, size_t n, float lo, float hi);

void axo_sgemm(int transA, int transB, size_t M, size_t N, size_t K, float alpha,
               const float *A, size_t lda, const float *B, size_t ldb, float beta,
               float *C, size_t ldc);

/* mask: NULL or uint8 (nonzero = masked out).  mask_ndim is 2 for (Sq,Skv) or
 * 4 for (mask_b, mask_h, Sq, Skv) with mask_b in {1,B}, mask_h in {1,H}.
 * slice_begin/slice_end select a range of (batch*head) slices to compute
 * (use 0, B*H for all); other slices of o are left untouched. */
int axo_sdpa(int dtype, const void *q, const void *k, const void *v, void *o,
             int B, int H, int Sq, int Skv, int D, float scale, int is_causal,
             const uint8_t *mask, int mask_ndim, int mask_b, int mask_h,
             int slice_begin, int slice_end);

int axo_softmax(int dtype, const void *in, void *out, size_t outer, size_t axis,
                size_t inner, int is_log);

/* Comparisons, logical operations and the is* tests write 1 or 0 in `dtype`
 * (the reference's Bool result: nonzero = true). */
int axo_unary(int op, int dtype, const void *in, void *out, size_t n);
/* out[i] = cond[i] ? a[i] : b[i]; cond is one byte per element, nonzero = true */
int axo_where(int dtype, const uint8_t *cond, const void *a, const void *b, void *out, size_t n);
int axo_binary(int op, int dtype, const void *a, const void *b, void *out,
               size_t rows, size_t cols, int b_kind);
/* last-axis reduction; out has `rows` elements of `dtype` (float accumulate,
 * result rounded to dtype for half types). */
int axo_reduce_last(int red, int dtype, const void *in, void *out, size_t rows,
                    size_t cols);

/* argmax (want_min = 0) / argmin over the middle extent of an (outer, axis,
 * inner) view; out has outer * inner int64 indices. */
int axo_argreduce(int want_min, int dtype, const void *in, int64_t *out, size_t outer,
                  size_t axis, size_t inner);

/* CPU layer_norm / rms_norm decompositions.  Output is ALWAYS float32, as on
 * the reference's CPU path (half inputs are promoted by the first op that
 * meets the float32 mean). w / b may be NULL (treated as absent). */
int axo_layer_norm(int dtype, const void *x, const void *w, const void *b,
                   float *out, size_t rows, size_t cols, float eps);
int axo_rms_norm(int dtype, const void *x, const void *w, float *out,
                 size_t rows, size_t cols, float eps);

/* C[M,N] = op(A) * op(B); float32 through axo_sgemm, half types through the
 * tiled loop that accumulates in the half type itself. */
int axo_matmul(int dtype, const void *A, const void *B, void *C, size_t M,
               size_t N, size_t K, int transA, int transB);

/* softmax((relu(a)+1)*b, -1).sum(1) for float32 a,b [rows, cols]; out [rows].
 * If softmax_out is non-NULL the intermediate softmax is stored there. */
int axo_chain_relu_add_mul_softmax_sum(const float *a, const float *b, float *out,
                                       float *softmax_out, size_t rows, size_t cols);

int axo_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
