/*
 * axhip.h -- C ABI of the gfx950 (MI355X) GPU backend for Axiom's two GPU hot
 * paths: scaled-dot-product attention and the fused elementwise / softmax /
 * norm chains that the lazy graph emits.
 *
 * Conventions
 *   - every function returns int: 0 on success, a positive value is a
 *     hipError_t, a negative value is one of AXHIP_ERR_*.  A human-readable
 *     message for the calling thread's last failure is at axhip_last_error().
 *   - the caller owns every buffer; kernels never allocate.  Pointers are
 *     device pointers unless a parameter says "host".  Four entry points need
 *     temporary device memory for some argument values (axhip_sdpa_fwd,
 *     axhip_gemm, axhip_argreduce, axhip_reduce_axis: each says when).  Their
 *     *_ws forms take it from the caller -- `workspace` of at least
 *     *_workspace_bytes(...) bytes, 256-byte aligned -- and allocate nothing;
 *     the plain forms (and a *_ws call with workspace == NULL) take it from the
 *     stream-ordered allocator (hipMallocAsync / hipFreeAsync on `stream`), a
 *     convenience that graph capture and no-allocation harnesses must avoid.
 *     A workspace that is too small fails with AXHIP_ERR_WORKSPACE before
 *     anything is launched.
 *   - `stream` is a hipStream_t passed as void* (NULL = the backend's own
 *     stream, created by axhip_init and shared process-wide).
 *   - no exception crosses this boundary.
 *
 * Each entry point names the Axiom interface it stands behind (paths relative
 * to the Axiom source tree).
 */
#ifndef AXHIP_H
#define AXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXHIP_OK 0
#define AXHIP_ERR_INVALID_ARG (-1)
#define AXHIP_ERR_UNSUPPORTED (-2)
#define AXHIP_ERR_NO_DEVICE (-3)
#define AXHIP_ERR_WORKSPACE (-4)

/* element types (DType subset of include/axiom/dtype.hpp:171-191) */
#define AXHIP_DTYPE_F32 0
#define AXHIP_DTYPE_F16 1
#define AXHIP_DTYPE_BF16 2
/* Bool / UInt8 (one byte; any nonzero byte reads as 1.0, a nonzero result is stored as 1): the result type of
 * comparisons, logical operations and any / all, and an input type of the fused chains and of axhip_strided_copy
 * and axhip_where.  Attention, GEMM and the other entry points take the three floating-point types only. */
#define AXHIP_DTYPE_U8 3

/* ------------------------------------------------------------------ runtime
 * Stands behind system::is_metal_available (src/tensor/system.cpp:11-29),
 * make_storage(bytes, Device::GPU) (src/tensor/storage.cpp:26-48),
 * MetalStorage::copy_to/copy_from (src/backends/metal/metal_storage.mm:66-142)
 * and MetalExecutionStream::synchronize (src/backends/metal/metal_common.mm:
 * 285-335).  The Apple unified-memory retag (src/tensor/tensor.cpp:1600-1623)
 * has no counterpart: transfers are explicit hipMemcpyAsync. */
int axhip_device_count(int *count);
int axhip_init(int device);
const char *axhip_last_error(void);
const char *axhip_version(void);
void *axhip_default_stream(void);
int axhip_malloc(void **ptr, size_t bytes);
int axhip_free(void *ptr);
int axhip_memcpy_h2d_async(void *dst_device, const void *src_host, size_t bytes, void *stream);
int axhip_memcpy_d2h_async(void *dst_host, const void *src_device, size_t bytes, void *stream);
int axhip_memcpy_d2d_async(void *dst_device, const void *src_device, size_t bytes, void *stream);
int axhip_stream_sync(void *stream);

/* --------------------------------------------------------------------- SDPA
 * Stands behind backends::metal::gpu_scaled_dot_product_attention
 * (src/backends/metal/metal_operations.hpp:47-50, dispatch in
 * src/backends/metal/flash_attention_dispatch.mm:168-304, kernel
 * src/backends/metal/flash_attention.metal:50-224), called from
 * ops::scaled_dot_product_attention (src/tensor/operations.cpp:3979-4044).
 *
 * q (B,H,Sq,D), k/v (B,H,Skv,D), o (B,H,Sq,D).  The last dimension is
 * contiguous; the other three carry explicit element strides so the
 * (B,S,H,D)->(B,H,S,D) head-split view of nn::MultiHeadAttention
 * (src/nn/attention.cpp:44-52) needs no copy.  mask is NULL or uint8,
 * nonzero = masked out (include/axiom/operations.hpp:650), laid out
 * (Sq,Skv) row-major per (batch, head) with element strides mask_strides
 * (0 = broadcast).  is_causal masks kv_pos > q_pos (top-left aligned,
 * src/backends/cpu/flash_attention_cpu.cpp:78-89).  scale <= 0 means
 * 1/sqrt(D) (src/tensor/operations.cpp:4013-4015).  A row whose keys are all
 * masked yields zeros.  fp32 accumulation; output in `dtype`.
 * bf16/f16 with D a multiple of 8 up to 256, and fp32 with D a multiple of
 * 4 up to 128, run on MFMA (16-byte aligned base
 * pointers, strides that are multiples of 8 elements; fp32: 4); everything
 * else up to D = 256 runs on the generic fp32-FMA kernel, which takes the
 * place of the reference's decomposed_attention fallback
 * (flash_attention_dispatch.mm:125-162).  axhip_sdpa_kernel_name tells which.
 * A decoding step (up to 128 query rows, at most 96 (batch, head) slices, a
 * long unmasked key sequence) splits its keys between work-groups and merges
 * the partial results through stream-ordered temporary memory
 * (hipMallocAsync on `stream`). */
typedef struct {
    int32_t dtype;
    int32_t batch, heads, seq_q, seq_kv, head_dim;
    float scale;
    int32_t is_causal;
    int64_t q_strides[3]; /* batch, head, seq (elements) */
    int64_t k_strides[3];
    int64_t v_strides[3];
    int64_t o_strides[3];
    int64_t mask_strides[2]; /* batch, head (elements; 0 = shared) */
} AxhipSdpaParams;

int axhip_sdpa_fwd(const void *q, const void *k, const void *v, void *o,
                   const uint8_t *mask, const AxhipSdpaParams *params_host, void *stream);
/* The same with the temporary memory of a decoding step handed in by the
 * caller (the role of the reference's caller-owned command buffers,
 * src/backends/metal/metal_common.hpp:53-123: the backend allocates nothing
 * behind the caller's back).  axhip_sdpa_workspace_bytes answers 0 for every
 * problem that needs none; has_mask: whether a mask will be passed. */
size_t axhip_sdpa_workspace_bytes(const AxhipSdpaParams *params_host, int has_mask);
int axhip_sdpa_fwd_ws(const void *q, const void *k, const void *v, void *o,
                      const uint8_t *mask, const AxhipSdpaParams *params_host,
                      void *workspace, size_t workspace_bytes, void *stream);
/* name of the kernel axhip_sdpa_fwd would launch for these parameters
 * ("mfma_bf16_d128", "generic", ...); the pointer stays valid for the life of
 * the process. */
const char *axhip_sdpa_kernel_name(const AxhipSdpaParams *params_host);
/* diagnostic: the schedule the calling thread's last axhip_sdpa_fwd launched ("pingpong", "pipelined8",
 * "pipelined4", "key_split", "decode_split", "register_staged", "mfma_f32", "generic", "empty"); several
 * schedules share one kernel name.  AXHIP_SDPA_PINGPONG=0 in the environment (read when the library loads)
 * sends "pingpong" problems to "pipelined8". */
const char *axhip_sdpa_last_schedule(void);

/* ------------------------------------------------------------ fused chains
 * Stands behind graph::materialize_gpu_graph (called from
 * src/graph/graph_registry.cpp:834-850, Metal implementation
 * src/backends/metal/mpsgraph_graph_compiler.mm:706-944), the CPU-planned
 * hooks execute_gpu_fused_chain / execute_gpu_fused_reduction
 * (include/axiom/graph/gpu_fusion.hpp:14-22), the norm fast paths
 * gpu_layer_norm / gpu_rms_norm (src/backends/metal/metal_operations.hpp:
 * 20-24; kernels src/backends/metal/kernels.metal:167-381,
 * src/backends/metal/mpsgraph_operations.mm:2139-2210) and the per-op GPU
 * registry entries (src/backends/metal/mpsgraph_operations.mm:2925-3150).
 *
 * A program describes ONE pass over a [rows, cols] row-major view:
 *     v = input
 *     v = pre[0..n_pre)(v)            elementwise chain
 *     v = row_op(v)                   softmax / log-softmax / layer norm / RMS norm over cols
 *     v = post[0..n_post)(v)          elementwise chain
 *     out = reduce(v) over cols       -> [rows], or out = v -> [rows, cols]
 * Every value is computed in fp32 and rounded once on store.  One kernel
 * launch, each input element read once, no intermediate ever written.
 *
 * Chain op codes follow ops::OpType (include/axiom/operations.hpp:55-208) for
 * the hot-path subset. */
#define AXHIP_OP_ADD 1
#define AXHIP_OP_SUB 2
#define AXHIP_OP_MUL 3
#define AXHIP_OP_DIV 4
#define AXHIP_OP_MAX 5
#define AXHIP_OP_MIN 6
#define AXHIP_OP_RSUB 7 /* operand - v  (chain value is the right-hand side) */
#define AXHIP_OP_RDIV 8 /* operand / v */
#define AXHIP_OP_RELU 16
#define AXHIP_OP_GELU 17
#define AXHIP_OP_SQRT 18
#define AXHIP_OP_EXP 19
#define AXHIP_OP_NEG 20
#define AXHIP_OP_ABS 21
#define AXHIP_OP_SIGMOID 22
#define AXHIP_OP_TANH 23
#define AXHIP_OP_SILU 24
#define AXHIP_OP_LOG 25
#define AXHIP_OP_SQUARE 26
#define AXHIP_OP_RSQRT 27
#define AXHIP_OP_RECIP 28
/* The wider operator table of the lazy graph (binary: 40-63, unary: 64-95), with the CPU functors' rules
 * (src/backends/cpu/cpu_operations.hpp:214-235 power / fmod, :237-291 comparisons and logical operations, :360-381
 * atan2 / hypot, :395-400 logical not, :497-505 erf, :655-660 leaky ReLU, :724-787 sign / floor / ceil / trunc /
 * round, :808-860 cbrt / isnan / isinf / isfinite).  Comparisons, logical operations and the is* tests yield 1.0 or
 * 0.0 inside a chain; stored to an AXHIP_DTYPE_U8 output that is the reference's Bool result.  A logical operation
 * reads any nonzero value (NaN included) as true. */
#define AXHIP_OP_POW 40    /* powf(v, operand) */
#define AXHIP_OP_RPOW 41   /* powf(operand, v) */
#define AXHIP_OP_MOD 42    /* fmodf(v, operand): the sign of the dividend, like the CPU functor */
#define AXHIP_OP_RMOD 43   /* fmodf(operand, v) */
#define AXHIP_OP_ATAN2 44  /* atan2f(v, operand) */
#define AXHIP_OP_RATAN2 45 /* atan2f(operand, v) */
#define AXHIP_OP_HYPOT 46
#define AXHIP_OP_EQ 47
#define AXHIP_OP_NE 48
#define AXHIP_OP_LT 49 /* v < operand; with the chain value on the right-hand side the planner emits GT */
#define AXHIP_OP_LE 50
#define AXHIP_OP_GT 51
#define AXHIP_OP_GE 52
#define AXHIP_OP_AND 53
#define AXHIP_OP_OR 54
#define AXHIP_OP_XOR 55
#define AXHIP_OP_LEAKY_RELU 56 /* v > 0 ? v : operand * v -- the slope is the operand (an immediate) */
#define AXHIP_OP_ERF 64
#define AXHIP_OP_SIN 65
#define AXHIP_OP_COS 66
#define AXHIP_OP_TAN 67
#define AXHIP_OP_SIGN 68 /* 1, -1, or 0 (also for NaN) */
#define AXHIP_OP_FLOOR 69
#define AXHIP_OP_CEIL 70
#define AXHIP_OP_ROUND 71 /* halves away from zero (std::round) */
#define AXHIP_OP_TRUNC 72
#define AXHIP_OP_CBRT 73
#define AXHIP_OP_ISNAN 74
#define AXHIP_OP_ISINF 75
#define AXHIP_OP_ISFINITE 76
#define AXHIP_OP_NOT 77 /* v == 0 */

#define AXHIP_ROWOP_NONE 0
#define AXHIP_ROWOP_SOFTMAX 1
#define AXHIP_ROWOP_LOGSOFTMAX 2
#define AXHIP_ROWOP_LAYERNORM 3 /* (x-mean)/sqrt(var+eps) [*w] [+b], population variance */
#define AXHIP_ROWOP_RMSNORM 4   /* x/sqrt(mean(x^2)+eps) [*w] */

#define AXHIP_RED_NONE 0
#define AXHIP_RED_SUM 1
#define AXHIP_RED_MEAN 2
#define AXHIP_RED_MAX 3
#define AXHIP_RED_MIN 4
#define AXHIP_RED_PROD 5 /* (any / all are NE 0 under MAX / MIN with an AXHIP_DTYPE_U8 result) */

/* how a binary op's second operand maps onto the [rows, cols] view */
#define AXHIP_BK_FULL 0   /* [rows, cols] */
#define AXHIP_BK_ROWVEC 1 /* [cols]  broadcast down the rows (weights, biases) */
#define AXHIP_BK_COLVEC 2 /* [rows]  one value per row (keep_dims reductions) */
#define AXHIP_BK_SCALAR 3 /* [1]     Axiom's make_scalar operand, device resident */
#define AXHIP_BK_IMM 4    /* immediate in AxhipChainOp.imm, no memory operand */

#define AXHIP_MAX_CHAIN 16
#define AXHIP_MAX_OPERANDS 8

typedef struct {
    const void *ptr;
    int32_t dtype;
    int32_t kind; /* AXHIP_BK_* */
} AxhipOperand;

typedef struct {
    int32_t op;      /* AXHIP_OP_* */
    int32_t operand; /* index into operands[] for binary ops, -1 otherwise */
    float imm;       /* value for AXHIP_BK_IMM */
    int32_t imm_kind; /* AXHIP_BK_IMM when imm is the operand, else 0 */
} AxhipChainOp;

typedef struct {
    int64_t rows, cols;
    const void *input;
    int32_t input_dtype;
    int32_t n_operands;
    AxhipOperand operands[AXHIP_MAX_OPERANDS];
    int32_t n_pre;
    AxhipChainOp pre[AXHIP_MAX_CHAIN];
    int32_t row_op; /* AXHIP_ROWOP_* */
    float eps;
    int32_t norm_weight; /* operand index (ROWVEC) or -1 */
    int32_t norm_bias;   /* operand index (ROWVEC) or -1 */
    int32_t n_post;
    AxhipChainOp post[AXHIP_MAX_CHAIN];
    int32_t reduce; /* AXHIP_RED_* over cols */
    void *output;   /* [rows] if reduce != NONE else [rows, cols] */
    int32_t output_dtype;
} AxhipRowsProgram;

int axhip_fused_rows(const AxhipRowsProgram *program_host, void *stream);
/* name of the kernel variant axhip_fused_rows would launch: "rows_static_..." a kernel of
 * this program shape built into the library, "rows_jit_..." one the library compiles (hipRTC)
 * when the shape is first launched -- the counterpart of the reference compiling a graph on
 * first use (mpsgraph_graph_compiler.mm:706-944) -- anything else the generic interpreter.
 * AXHIP_JIT=0 in the environment turns run-time compilation off. */
const char *axhip_fused_rows_kernel_name(const AxhipRowsProgram *program_host);
/* Compiles the kernel of a "rows_jit_" program now (for gfx950; needs no device) and reports
 * a compile error instead of leaving it to the first launch, which would fall back to the
 * interpreter.  Pointers in the program are only looked at for their alignment. */
int axhip_fused_rows_prepare(const AxhipRowsProgram *program_host);
/* diagnostic: how many "rows_jit_" kernels this process has so far loaded from the on-disk cache of
 * compiled code objects (AXHIP_CACHE_DIR, default $XDG_CACHE_HOME/axhip or $HOME/.cache/axhip; AXHIP_DISK_CACHE=0
 * turns it off) and how many it compiled with hipRTC.  Either pointer may be NULL. */
void axhip_fused_rows_jit_counters(int *from_disk, int *compiled);

/* Elementwise chain followed by a reduction over ALL elements -> one value
 * (the FusedReductionStep of include/axiom/graph/compiled_graph.hpp:41-70,
 * GPU hook execute_gpu_fused_reduction).  Uses program->pre only; row_op and
 * post must be empty; program->reduce selects the reduction; output is one
 * element.  workspace: device scratch of at least
 * axhip_full_reduce_workspace_bytes() bytes. */
size_t axhip_full_reduce_workspace_bytes(void);
int axhip_fused_full_reduce(const AxhipRowsProgram *program_host, void *workspace,
                            size_t workspace_bytes, void *stream);

/* axhip_fused_full_reduce for callers that cannot allocate device memory or
 * bring a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * Same program, same kernels and the same result, bit for bit; the partial
 * sums live in a 65 KiB array inside the library's device image (one copy on
 * every device the library runs on, held until the process ends), whose
 * address is resolved when axhip_init runs on the device.  The call itself
 * performs no hipMalloc / hipFree, calls no allocating routine and compiles
 * nothing (only kernels that are built into the library serve it).
 * Limits: rows * cols <= axhip_full_reduce_noalloc_max_elements() (2^40),
 * larger inputs return AXHIP_ERR_UNSUPPORTED.  All calls on one device share
 * that one array: two calls that overlap in time on the same device (different
 * streams, or different threads on different streams) race; calls on one
 * stream are ordered and safe.  Nothing in the array has to be cleared
 * between calls. */
int64_t axhip_full_reduce_noalloc_max_elements(void);
int axhip_fused_full_reduce_noalloc(const AxhipRowsProgram *program_host, void *stream);

/* ------------------------------------------------------------- data movers
 * Stands behind gpu_make_contiguous (src/backends/metal/metal_operations.hpp:
 * 60-63, kernel gather_strided src/backends/metal/kernels.metal:33-149) and
 * the GPU Cast op (src/tensor/tensor.cpp:1665-1670).  Copies a strided view
 * (<= 8 dims, non-negative element strides) into a contiguous row-major
 * buffer, converting dtype on the way (AXHIP_DTYPE_U8 on either side: the
 * Bool casts, nonzero <-> 1). */
#define AXHIP_MAX_DIMS 8
int axhip_strided_copy(const void *src, int32_t src_dtype, void *dst, int32_t dst_dtype,
                       int32_t ndim, const int64_t *shape_host, const int64_t *src_strides_host,
                       void *stream);
int axhip_fill(void *dst, int32_t dtype, double value, int64_t count, void *stream);

/* Constant padding (ops::pad, mode "constant": src/tensor/operations.cpp pad();
 * lazy Pad node, src/backends/metal/mpsgraph_graph_compiler.mm:335-573).  dst is
 * contiguous row-major with extents src_shape[d] + pad_before[d] + pad_after[d];
 * src may be a strided view (non-negative element strides).  One pass: each
 * output element is either copied or set to `value`. */
int axhip_pad(const void *src, void *dst, int32_t dtype, int32_t ndim, const int64_t *src_shape_host,
              const int64_t *src_strides_host, const int64_t *pad_before_host,
              const int64_t *pad_after_host, double value, void *stream);
/* The other modes of ops::pad (src/tensor/operations.cpp:2216-2246): reflect
 * (the border element is not repeated; each pad must be shorter than the
 * extent it reflects), replicate (the border element repeated) and circular
 * (wrap around); `value` only matters for AXHIP_PAD_CONSTANT. */
#define AXHIP_PAD_CONSTANT 0
#define AXHIP_PAD_REFLECT 1
#define AXHIP_PAD_REPLICATE 2
#define AXHIP_PAD_CIRCULAR 3
int axhip_pad_mode(const void *src, void *dst, int32_t dtype, int32_t ndim, const int64_t *src_shape_host,
                   const int64_t *src_strides_host, const int64_t *pad_before_host,
                   const int64_t *pad_after_host, int32_t mode, double value, void *stream);

/* masked_fill (include/axiom/operations.hpp:437-440): dst[i] = mask[i] ? value :
 * src[i] over an iteration space of <= 8 dims; src and the byte mask (Bool:
 * nonzero = fill) are strided views with element strides, 0 on broadcast dims;
 * dst is contiguous and has src's dtype. */
int axhip_masked_fill(const void *src, int32_t dtype, const uint8_t *mask, void *dst, int32_t ndim,
                      const int64_t *shape_host, const int64_t *src_strides_host,
                      const int64_t *mask_strides_host, double value, void *stream);

/* where (ops::where, include/axiom/operations.hpp:425-429 and
 * src/tensor/operations.cpp:1543-1566; GPU MPSGraphTernaryOperation::execute_where,
 * src/backends/metal/mpsgraph_operations.mm:637): dst[i] = cond[i] != 0 ?
 * a[i] : b[i] over an iteration space of <= 8 dims.  cond (normally
 * AXHIP_DTYPE_U8), a and b are strided views with element strides, 0 on
 * broadcast dims, each of its own element type; dst is contiguous. */
int axhip_where(const void *cond, int32_t cond_dtype, const void *a, int32_t a_dtype, const void *b,
                int32_t b_dtype, void *dst, int32_t dst_dtype, int32_t ndim, const int64_t *shape_host,
                const int64_t *cond_strides_host, const int64_t *a_strides_host,
                const int64_t *b_strides_host, void *stream);

/* Embedding lookup (ops::embedding, include/axiom/operations.hpp:483-486):
 * dst[i, :] = table[indices[i], :] for n_indices rows of row_elems elements.
 * index_bytes is 4 (int32) or 8 (int64).  An index outside [0, table_rows)
 * yields a row of zeros (the device cannot throw IndexError). */
int axhip_gather_rows(const void *table, int32_t dtype, int64_t table_rows, int64_t row_elems,
                      const void *indices, int32_t index_bytes, int64_t n_indices, void *dst,
                      void *stream);

/* argmax (want_min = 0) / argmin along the middle extent of a contiguous
 * (outer, axis, inner) view -> outer * inner int64 indices: the Reduction node
 * kinds ArgMax / ArgMin of the GPU graph compiler
 * (src/backends/metal/mpsgraph_graph_compiler.mm:628-658), with the CPU scan's
 * rule (src/backends/cpu/cpu_operations.cpp:2157-2229): the first occurrence of
 * the extreme wins, a NaN never does, and a slice with nothing above the type's
 * lowest() (argmin: below max()) -- all -inf, all NaN -- answers 0.  inner == 1
 * is the row form (greedy decoding over [batch, vocabulary] logits).  Few
 * results over a long inner-axis run go through stream-ordered temporary
 * memory (hipMallocAsync on `stream`). */
int axhip_argreduce(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner,
                    int32_t want_min, int64_t *dst, void *stream);
/* The same with that temporary memory handed in by the caller (0 bytes for
 * every shape that needs none; `src` only matters for its 16-byte alignment). */
size_t axhip_argreduce_workspace_bytes(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner);
int axhip_argreduce_ws(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner,
                       int32_t want_min, int64_t *dst, void *workspace, size_t workspace_bytes, void *stream);

/* Sum / mean / max / min (AXHIP_RED_*) along the middle extent of a contiguous
 * (outer, axis, inner) view -> outer * inner values of dst_dtype: Reduction
 * nodes over axes other than the last one
 * (src/backends/metal/mpsgraph_graph_compiler.mm:576-604 reduces over any axes),
 * without a transposing copy.  fp32 accumulation; the mean divides by the axis
 * length.  inner == 1 is a row reduction and goes to the fused row kernels.
 * Few results over a long axis are reduced in two passes through fp32
 * partials in stream-ordered temporary memory (hipMallocAsync on `stream`). */
int axhip_reduce_axis(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner,
                      int32_t reduce, void *dst, int32_t dst_dtype, void *stream);
/* The same with the fp32 partials in memory handed in by the caller (0 bytes
 * for every shape that needs none; `src` only matters for its alignment). */
size_t axhip_reduce_axis_workspace_bytes(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner);
int axhip_reduce_axis_ws(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner,
                         int32_t reduce, void *dst, int32_t dst_dtype, void *workspace, size_t workspace_bytes, void *stream);

/* softmax (is_log = 0) / log-softmax along the middle extent of a contiguous
 * (outer, axis, inner) view, dst of the same shape and dtype: Softmax /
 * LogSoftmax nodes over an axis other than the last one
 * (src/backends/metal/mpsgraph_graph_compiler.mm:287-300 takes any axis),
 * without the two transposing copies.  inner == 1 goes to the fused row
 * kernels. */
int axhip_softmax_axis(const void *src, int32_t dtype, int64_t outer, int64_t axis, int64_t inner,
                       int32_t is_log, void *dst, void *stream);

/* -------------------------------------------------------------------- GEMM
 * Stands behind the GPU MatMul registry entry and gpu_linear
 * (src/backends/metal/mpsgraph_operations.mm:2409-2532; lazy builder
 * src/backends/metal/mpsgraph_graph_compiler.mm:271-284), used by nn::Linear
 * as matmul(x, W, false, true) + bias (src/nn/linear.cpp:15-27).
 * C[b] = op(A[b]) * op(B[b]) (+ bias[N]) (+ residual[b]) for b < batch;
 * row-major, lda/ldb/ldc and batch strides in elements (stride 0 shares an
 * operand across the batch).  fp32 accumulation; bf16/f16 on MFMA.
 * The matrix-core kernels read both operands along k (trans_a = 0,
 * trans_b = 1: x W^T) in 16-byte vectors.  On a large product an operand
 * stored the other way is transposed first, and a k that is not a multiple of
 * 8 (fp32: 4) zero-padded, into temporary memory that the library takes and
 * returns in stream order (hipMallocAsync / hipFreeAsync on `stream`). */
typedef struct {
    int32_t dtype;
    int32_t trans_a, trans_b;
    int64_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t batch;
    int64_t stride_a, stride_b, stride_c;
    const void *bias;     /* [n] or NULL */
    const void *residual; /* same layout as C or NULL */
    int32_t epilogue_op;  /* 0 or AXHIP_OP_RELU / GELU / SILU / SIGMOID / TANH (MatMul+activation fusion) */
} AxhipGemmParams;

int axhip_gemm(const void *a, const void *b, void *c, const AxhipGemmParams *params_host, void *stream);
/* The same with the repacked operands in memory handed in by the caller (0
 * bytes for every product that is not repacked). */
size_t axhip_gemm_workspace_bytes(const AxhipGemmParams *params_host);
int axhip_gemm_ws(const void *a, const void *b, void *c, const AxhipGemmParams *params_host,
                  void *workspace, size_t workspace_bytes, void *stream);

/* sizeof() of the parameter structs as this library was compiled, so that a
 * foreign-language binding can verify its own struct layout at load time:
 * which = 0 AxhipSdpaParams, 1 AxhipRowsProgram, 2 AxhipGemmParams,
 * 3 AxhipOperand, 4 AxhipChainOp; anything else returns 0. */
size_t axhip_sizeof(int which);

#ifdef __cplusplus
}
#endif
#endif
