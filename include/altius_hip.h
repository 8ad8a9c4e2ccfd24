/*
 * altius_hip -- C ABI of the MI355X (gfx950) backend for the altius
 * interpreter's tensor kernels.
 *
 * This is the drop-in boundary: plain pointers and sizes, no C++ or framework
 * types.  A Rust crate binds it with an `extern "C"` block; the C++ session in
 * this repository and the Python test harness (ctypes) call the same symbols.
 *
 * Conventions
 *   - Every function returns AHIP_OK (0) or an AHIP_ERR_* code; nothing throws
 *     or aborts across the boundary.  ahip_last_error() gives the text of the
 *     most recent failure on a context (or on the calling thread when no
 *     context exists yet).
 *   - The caller owns every pointer it allocates.  Device pointers come from
 *     ahip_malloc (or any hipMalloc-compatible allocator on the same device).
 *   - All calls on one context are ordered on that context's stream.  A context
 *     must not be used from two threads at once; contexts are independent.
 *   - Tensors are dense, row-major, fp32 unless stated.  Strides are in
 *     elements.
 *
 * Citations name the reference interface each entry point stands in for
 * (paths relative to the altius checkout).
 */
#ifndef ALTIUS_HIP_H
#define ALTIUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AHIP_OK 0
#define AHIP_ERR_HIP 1         /* a HIP runtime call failed */
#define AHIP_ERR_ARG 2         /* invalid argument */
#define AHIP_ERR_SHAPE 3       /* SessionError::Shape (crates/session/src/lib.rs:16-18) */
#define AHIP_ERR_UNSUPPORTED 4 /* SessionError::Message: no kernel for this op / shape / dtype
                                  (crates/session/src/lib.rs:32-34) */
#define AHIP_ERR_OOM 5         /* device allocation failed */
#define AHIP_ERR_IO 6          /* ModelLoadError::Io: a model file could not be read */

#define AHIP_MAX_RANK 8

typedef struct ahip_ctx ahip_ctx;

/* ------------------------------------------------------------------------
 * Device shim: thin wrappers over hipSetDevice / hipStreamCreate / hipMalloc /
 * hipMemcpyAsync / hipEvent*.  The reference has no device layer; these stand
 * where its host allocator sits (Tensor::uninit_of_type,
 * crates/core/src/tensor.rs:116-132, called from
 * crates/session_interpreter/src/session.rs:159-162).
 * ---------------------------------------------------------------------- */

/* Creates a context on `device` with a stream of its own. */
int ahip_init(int device, ahip_ctx **ctx);
/* Same, but issues work on an existing hipStream_t (not destroyed with the context). */
int ahip_init_on_stream(int device, void *hip_stream, ahip_ctx **ctx);
int ahip_destroy(ahip_ctx *ctx);
/* ctx may be NULL: returns the calling thread's last context-less error. */
const char *ahip_last_error(ahip_ctx *ctx);
/* Number of visible devices, or a negative AHIP_ERR_* code. */
int ahip_device_count(void);

int ahip_malloc(ahip_ctx *ctx, size_t bytes, void **dptr);
int ahip_free(ahip_ctx *ctx, void *dptr);
int ahip_h2d_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes);
int ahip_d2h_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes);
int ahip_d2d_async(ahip_ctx *ctx, void *dst, const void *src, size_t bytes);
int ahip_memset_async(ahip_ctx *ctx, void *dst, int byte_value, size_t bytes);
int ahip_sync(ahip_ctx *ctx);

/* Pinned host memory for transfers that should overlap with kernels. */
int ahip_host_alloc(ahip_ctx *ctx, size_t bytes, void **hptr);
int ahip_host_free(ahip_ctx *ctx, void *hptr);

/* Events on the context's stream, for timing kernels where they run. */
int ahip_event_create(ahip_ctx *ctx, void **event);
int ahip_event_record(ahip_ctx *ctx, void *event);
int ahip_event_synchronize(ahip_ctx *ctx, void *event);
int ahip_event_elapsed_ms(ahip_ctx *ctx, void *start, void *stop, float *ms);
int ahip_event_destroy(ahip_ctx *ctx, void *event);

/* Code objects built elsewhere (hipcc --genco --offload-arch=gfx950) and loaded
 * at run time, then launched by kernel name on the context's stream.  Same role
 * as the reference's ClangSession, which dlopen()s a compiled model and calls
 * its exported entry (crates/session_clang/src/builder.rs:44-76,
 * crates/session_clang/src/session.rs:46-56).  image points to `bytes` bytes
 * of a gfx950 code object (raw or clang offload bundle); it may be freed after
 * the call.  grid counts BLOCKS per dimension; args[i] points to the i-th
 * kernel argument.  Unknown kernel names and launch shapes the device cannot
 * run (block of more than 1024 threads, zero extent, shared memory beyond
 * 160 KiB) are refused with AHIP_ERR_ARG before anything is launched. */
typedef struct ahip_module ahip_module;
int ahip_module_load(ahip_ctx *ctx, const void *image, size_t bytes, ahip_module **module);
int ahip_module_unload(ahip_ctx *ctx, ahip_module *module);
int ahip_launch(ahip_ctx *ctx, ahip_module *module, const char *kernel, const uint32_t grid[3],
                const uint32_t block[3], uint32_t shared_bytes, void **args);

/* ------------------------------------------------------------------------
 * Host-side index math (no device needed).
 * ---------------------------------------------------------------------- */

/* fixed_dim::broadcast of two shapes (crates/core/src/fixed_dim.rs:112-136).
 * out_dims holds max(a_rank, b_rank) entries.  AHIP_ERR_SHAPE if incompatible. */
int ahip_broadcast_shape(int a_rank, const int64_t *a_dims, int b_rank, const int64_t *b_dims,
                         int *out_rank, int64_t *out_dims);

/* Tensor::strides_for_broadcasting (crates/core/src/tensor.rs:369-406):
 * strides, in elements, with which a dense tensor of shape from_dims is read
 * when broadcast to to_dims; 0 on broadcast axes.  out_strides holds to_rank
 * entries.  AHIP_ERR_SHAPE if incompatible. */
int ahip_strides_for_broadcasting(int from_rank, const int64_t *from_dims, int to_rank,
                                  const int64_t *to_dims, int64_t *out_strides);

/* ------------------------------------------------------------------------
 * Operator kernels on device-resident fp32 tensors.  Outputs are pre-sized by
 * the caller and every element is written (the contract of the reference's
 * compute_* functions, crates/session_interpreter/src/session.rs:159-162).
 * ---------------------------------------------------------------------- */

enum ahip_binary_op { AHIP_ADD = 0, AHIP_SUB = 1, AHIP_MUL = 2, AHIP_DIV = 3, AHIP_POW = 4 };

/* compute_add / compute_sub / compute_mul / compute_div
 * (crates/session_interpreter/src/session.rs:384-526, 537-540) and compute_pow
 * (566-606).  `out` has shape out_dims[rank]; a_strides / b_strides come from
 * ahip_strides_for_broadcasting.  Pow multiplies a*a when b is a single
 * broadcast value equal to 2 and calls powf otherwise, as the reference does;
 * unlike the reference it also accepts a general broadcast exponent. */
int ahip_binary(ahip_ctx *ctx, int op, float *out, const float *a, const float *b, int rank,
                const int64_t *out_dims, const int64_t *a_strides, const int64_t *b_strides);

enum ahip_unary_op {
    AHIP_SQRT = 0,        /* compute_sqrt, session.rs:608-619 */
    AHIP_ERF = 1,         /* compute_erf, session.rs:924-931 (fastapprox::faster::erf) */
    AHIP_GELU = 2,        /* compute_gelu, session.rs:823-838 + fast_math.rs:281-355 */
    AHIP_SIGMOID = 3,     /* compute_sigmoid, session.rs:905-922 + fast_math.rs:189-279 */
    AHIP_HARDSIGMOID = 4, /* compute_hard_sigmoid, session.rs:805-812 (alpha, beta) */
    AHIP_RELU = 5,        /* compute_relu, session.rs:796-803 */
    AHIP_TANH = 6,        /* compute_tanh, session.rs:840-903, 933-938 (rational tanh) */
    AHIP_LEAKYRELU = 7,   /* compute_leaky_relu, session.rs:814-821 (alpha) */
    AHIP_EXP = 8,         /* no reference kernel (session.rs:224): expf */
    AHIP_ROUND = 9,       /* no reference kernel (session.rs:219-223): round half to even (ONNX Round) */
    AHIP_CLIP = 10,       /* no reference kernel (session.rs:201): clamp to [alpha, beta] (ONNX Clip) */
    AHIP_DIV_BY = 11      /* x / alpha: the division by H*W of compute_gavg_pool (session.rs:291) */
};

/* Flat element-wise op over n elements.  alpha/beta are read by HardSigmoid (alpha, beta),
 * LeakyRelu (alpha) and Clip (alpha = min, beta = max). */
int ahip_unary(ahip_ctx *ctx, int op, float *out, const float *in, size_t n, float alpha,
               float beta);

/* A chain of element-wise operators in one pass: Op::FusedElemwise (crates/core/src/op.rs:213-217),
 * which the reference emits in crates/core/src/optimize/elemwise_fusion.rs and runs only on its
 * code-generating backend (crates/session_clang/src/translator.rs:975-1143; the interpreter has no
 * kernel, session.rs:246).  Step t computes acc = op(lhs, rhs) (binary) or acc = op(lhs) (unary) for
 * every output element; an operand is inputs[k] broadcast to the output with input_strides[k] (from
 * ahip_strides_for_broadcasting) or AHIP_FUSED_ACC, the previous step's result; the last acc is the
 * output.  Each step applies exactly the per-element function of ahip_binary / ahip_unary, so the
 * result has the bits of the unfused chain.  pow_scalar_exponent selects the reference's
 * scalar-exponent Pow path (a*a when the exponent equals 2; session.rs:585-598), which the unfused
 * kernel takes when the exponent tensor has one element and the base has more.
 * AHIP_ERR_UNSUPPORTED (nothing launched) when the operands need more than three merged axes, or
 * there are more than AHIP_FUSED_MAX_INPUTS operands or AHIP_FUSED_MAX_STEPS steps: run the chain
 * operator by operator then. */
#define AHIP_FUSED_MAX_INPUTS 6
#define AHIP_FUSED_MAX_STEPS 16
#define AHIP_FUSED_ACC (-1)
typedef struct ahip_fused_step {
    int is_unary;            /* 0: op is an ahip_binary_op, 1: op is an ahip_unary_op */
    int op;
    int lhs, rhs;            /* index into inputs[] or AHIP_FUSED_ACC; rhs is ignored by unary steps */
    float alpha, beta;       /* parameters of unary steps (HardSigmoid, LeakyRelu, Clip) */
    int pow_scalar_exponent; /* AHIP_POW only */
} ahip_fused_step;
int ahip_fused_elemwise(ahip_ctx *ctx, float *out, int rank, const int64_t *out_dims, int n_inputs,
                        const float *const *inputs, const int64_t *const *input_strides, int n_steps,
                        const ahip_fused_step *steps);
/* ahip_fused_elemwise runs a chain through a kernel compiled for exactly that chain when the library
 * has one (the exporter's erf-GELU, the LayerNorm tail, scale-and-shift, bias + Relu or Gelu or residual, x * Sigmoid(x),
 * x * HardSigmoid(x)) and through a kernel that interprets the steps otherwise; both give the same bits.
 * enable = 0 sends every chain of this context to the interpreting kernel (default 1). */
int ahip_fused_use_compiled_chains(ahip_ctx *ctx, int enable);

/* compute_softmax over the last axis (session.rs:990-1026 + fast_math.rs:102-187):
 * `rows` rows of `len` contiguous elements. */
int ahip_softmax_lastaxis(ahip_ctx *ctx, float *out, const float *in, size_t rows, size_t len);
/* Not in the reference: Softmax that applies, while it loads the scores, the two operators exporters put in
 * front of it in attention -- Mul or Div by one value (scale_op 1 or 2, 0 for none), then Add of a mask
 * that holds one row of `len` values per `rows_per_mask` consecutive rows (mask may be NULL; [N,1,1,C] onto
 * [N,H,R,C] has rows_per_mask = H*R, one row for all has rows_per_mask = rows).  Each is the one IEEE
 * operation ahip_binary performs, so the result has the bits of Mul/Div -> Add -> Softmax run one after the
 * other, without their two passes over the scores.  AHIP_ERR_UNSUPPORTED (nothing launched) for tensors that
 * are not 16-byte aligned or rows longer than 1024: run the operators one after the other then. */
int ahip_softmax_lastaxis_prologue(ahip_ctx *ctx, float *out, const float *in, size_t rows, size_t len,
                                   int scale_op, float scale, const float *mask, size_t rows_per_mask);

/* compute_layer_normalization over the last axis (session.rs:1433-1486).
 * gamma and beta hold `len` values each. */
int ahip_layernorm_lastaxis(ahip_ctx *ctx, float *out, const float *in, const float *gamma,
                            const float *beta, size_t rows, size_t len, float eps);

enum ahip_reduce_kind {
    AHIP_REDUCE_MEAN = 0, /* sum * (1 / len) */
    AHIP_REDUCE_MAX = 1,
    AHIP_REDUCE_SUM = 2   /* plain sum: GlobalAveragePool divides it by H*W afterwards (session.rs:265-297) */
};

/* compute_reduce_mean / compute_reduce_max (session.rs:1292-1340), generalised
 * to any contiguous run of reduced axes: the input is viewed as
 * [outer, reduce, inner] and `out` as [outer, inner].  The reference's kernels
 * are the cases inner == 1 (ReduceMean over the last axis) and outer == 1,
 * inner == 1 (ReduceMax over everything).  ReduceMax ignores NaN (the reference
 * panics on NaN). */
int ahip_reduce(ahip_ctx *ctx, int kind, float *out, const float *in, size_t outer, size_t reduce,
                size_t inner);

/* ahip_reduce for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same kernels, same launch
 * shapes and therefore the same bits as ahip_reduce, but the partial results of a two-stage reduction go to
 * a fixed 1 MiB array inside the library's code object (resolved once per device by ahip_init) instead of
 * the context's scratch buffer, and the call itself performs no hipMalloc / hipFree.  A shape whose partial
 * results exceed ahip_reduce_static_capacity() floats fails with AHIP_ERR_UNSUPPORTED and launches nothing
 * (ahip_reduce would take its larger buffer or a one-stage kernel).  Every call on a GPU shares that GPU's
 * array, whatever its context.  Calls on one stream are ordered.  A two-stage call on another stream takes the
 * array over only if everything queued on the stream that used it last has finished (hipStreamQuery, no wait);
 * otherwise it fails with AHIP_ERR_UNSUPPORTED and launches nothing -- synchronize the other stream first.  Two
 * threads that call on different streams without such a handover would race: the library's record of the
 * last stream is what turns that into the error above.  Nothing in the array has to start at zero. */
int ahip_reduce_static(ahip_ctx *ctx, int kind, float *out, const float *in, size_t outer, size_t reduce,
                       size_t inner);
size_t ahip_reduce_static_capacity(void);

/* Data movement.  Element sizes are in bytes (1 = Bool, 4 = F32 / I32, 8 = I64); strides in
 * elements.  All of these move each byte once and accept any rank up to 8.
 *
 * ahip_copy_strided: element idx of the index space dims[rank] is read at sum(idx*in_strides)
 * and written at sum(idx*out_strides).  With a dense output it is Slice (offset base pointer,
 * strides scaled by the steps), Expand and Tile (stride 0) or a Transpose; with a dense input
 * and a windowed output it is one operand of Concat; Split is the reverse
 * (compute_concat / compute_split / compute_slice, session.rs:1134-1177, 1488-1558).
 * ahip_transpose: compute_transpose (session.rs:1179-1278); perm as in Op::Transpose.
 * ahip_gather: out[o, j, :] = data[o, indices[j], :] for outer x n_indices rows of `inner`
 * elements (compute_gather, session.rs:1560-1598, any index count); indices are i32 or i64
 * (index_size 4 or 8), negative ones count from the end.  An index out of range reads row 0
 * and makes the next ahip_sync on this context fail with AHIP_ERR_ARG.
 * ahip_where: out = cond ? x : y with broadcast strides (compute_where, session.rs:940-988).
 * ahip_greater: out (bool) = a > b (compute_greater, session.rs:541-562; any broadcast).
 * ahip_cast: Rust `as` between Bool / F32 / I32 / I64 (compute_cast, session.rs:1350-1378).
 * ahip_batchnorm: ((x - mean[c]) / sqrt(var[c] + eps)) * scale[c] + bias[c] on [n, c, hw]
 * (compute_batch_normalization, session.rs:1380-1431). */
int ahip_copy_strided(ahip_ctx *ctx, void *out, const void *in, int elem_size, int rank, const int64_t *dims,
                      const int64_t *out_strides, const int64_t *in_strides);
int ahip_transpose(ahip_ctx *ctx, void *out, const void *in, int elem_size, int rank, const int64_t *in_dims,
                   const int64_t *perm);
int ahip_gather(ahip_ctx *ctx, void *out, const void *data, const void *indices, int index_size, int elem_size,
                size_t outer, size_t axis_len, size_t n_indices, size_t inner);
int ahip_where(ahip_ctx *ctx, void *out, const void *cond, const void *x, const void *y, int elem_size, int rank,
               const int64_t *dims, const int64_t *cond_strides, const int64_t *x_strides, const int64_t *y_strides);
int ahip_greater(ahip_ctx *ctx, void *out, const float *a, const float *b, int rank, const int64_t *dims,
                 const int64_t *a_strides, const int64_t *b_strides);
int ahip_cast(ahip_ctx *ctx, void *out, const void *in, int from_elem_type, int to_elem_type, size_t n);
int ahip_batchnorm(ahip_ctx *ctx, float *out, const float *x, const float *scale, const float *bias, const float *mean,
                   const float *var, size_t n, size_t c, size_t hw, float epsilon);

/* C[b] = alpha * op(A[b]) * op(B[b]) + beta * C0, b in [0, batch): sgemm as compute_mat_mul and
 * compute_gemm call it (crates/session_interpreter/src/session.rs:621-794, gemm.rs:3-52), on the
 * matrix cores in fp32.  op(X) = X or its transpose (trans_a / trans_b); A is stored m x k (k x m
 * when transposed) with row pitch lda, B k x n (n x k) with row pitch ldb, C m x n with row pitch
 * ldc.  Batch strides are in elements; 0 shares one matrix between all batches (MatMul of
 * [b, m, k] by [k, n]).  c0 may be NULL; it is read at c0[i * c0_row_stride + j * c0_col_stride],
 * so (0, 1) broadcasts a bias row and (n, 1) reads a full matrix (Gemm's third input). */
int ahip_gemm(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t batch, size_t m,
              size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t a_batch_stride,
              size_t b_batch_stride, size_t c_batch_stride, size_t c0_row_stride, size_t c0_col_stride, float alpha,
              float beta);

/* ahip_gemm with the batch index split in two: batch z = (z / batch_inner, z % batch_inner), and operand X of
 * that batch starts at x + (z / batch_inner) * x_batch_strides[0] + (z % batch_inner) * x_batch_strides[1]
 * (elements; 0 shares).  Lets a product read or write the heads of a [b, t, h, d] tensor in place (b x h
 * matrices of t x d with row pitch h * d) instead of through a Transpose; the session uses it that way.  The
 * reference's sgemm call sites always copy (session.rs:1179-1278 Transpose, 621-684 MatMul). */
int ahip_gemm_batch2(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t batch_outer,
                     size_t batch_inner, size_t m, size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb,
                     size_t ldc, const size_t a_batch_strides[2], const size_t b_batch_strides[2],
                     const size_t c_batch_strides[2], size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta);

/* C = alpha * f(op(A)) * op(B) + beta * C0 for one batch, f = AHIP_GELU or AHIP_RELU applied to A's values
 * while the bf16 route (AHIP_GEMM_BF16X3) splits them: the activation between two products (Gelu between the
 * two MatMuls of a transformer MLP) costs no pass of its own and f(A) is never stored.  The values multiplied
 * are exactly those ahip_unary would have written.  AHIP_ERR_UNSUPPORTED, nothing launched, when this
 * product would not take the bf16 route under the context's algorithm setting (run ahip_unary, then
 * ahip_gemm).  No counterpart in the reference. */
int ahip_gemm_activated(ahip_ctx *ctx, int a_op, float *c, const float *a, const float *b, const float *c0, size_t m,
                        size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc,
                        size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta);

/* C = act(alpha * op(A) * op(B) + beta * C0) + residual for one batch, always on the fp32 kernel: the operators that
 * follow a product in a transformer block (Gelu after the MLP's first MatMul; the residual Add after its second one
 * and after attention's projection: compute_gelu session.rs:823-838, compute_add session.rs:537) done while C is
 * written, so that neither costs a pass or a launch of its own.  act: 0 (none), AHIP_GELU or AHIP_RELU; residual: NULL
 * or a matrix laid out like C (same pitch ldc).  Every step rounds as its own kernel would: the result has the bits
 * of ahip_gemm (with AHIP_GEMM_FP32) -> ahip_unary -> ahip_binary(AHIP_ADD).  No counterpart in the reference. */
int ahip_gemm_post(ahip_ctx *ctx, float *c, const float *a, const float *b, const float *c0, size_t m, size_t n, size_t k,
                   int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t c0_row_stride, size_t c0_col_stride,
                   float alpha, float beta, int act, const float *residual);

/* O = Softmax(scale(Q K^T) + mask) V for batch_outer * batch_inner independent (batch, head) pairs in one kernel: the
 * MatMul -> (Mul | Div by a scalar) -> (Add of a per-key mask) -> Softmax(last axis) -> MatMul chain of an attention block
 * (session.rs:621-684, 990-1026) without the [tq, tk] score tensor ever reaching memory.  Q is [tq, d] with row
 * pitch ldq, K and V [tk, d], O [tq, d]; operand X of batch z starts at x + (z / batch_inner) * x_batch_strides[0]
 * + (z % batch_inner) * x_batch_strides[1] (elements), so heads are read out of a [b, t, h * d] tensor and O is
 * written into one in place.  scale_op: 0 none, 1 scores * scale, 2 scores / scale.  mask (may be NULL): one value per
 * key, added after the scale, read at mask[(z / batch_inner) * mask_outer_stride + key] (stride 0: one row for all
 * batches; tk: one row per outer batch, the [b, 1, 1, tk] padding mask of BERT-style graphs).  Same exp and
 * reciprocal-multiply normalisation as ahip_softmax_lastaxis; the two products on the fp32 matrix cores, or, on a
 * context set to AHIP_GEMM_AUTO / AHIP_GEMM_BF16X3 and with at least one full block per CU, on the bf16 matrix cores
 * with every value as three bf16 planes (as accurate; an infinite value in Q, K or V then gives NaN).
 * AHIP_ERR_UNSUPPORTED (nothing launched) unless d == 64 and all pointers, pitches and batch strides are
 * multiples of 16 bytes: run the three operators then.  Any number of keys (they are streamed 64 at a time).  No counterpart in the reference. */
int ahip_attention(ahip_ctx *ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer,
                   size_t batch_inner, size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo,
                   const size_t q_batch_strides[2], const size_t k_batch_strides[2], const size_t v_batch_strides[2],
                   const size_t o_batch_strides[2], int scale_op, float scale, const float *mask, size_t mask_outer_stride);

/* Which kernel ahip_gemm (and the MatMul / Gemm / Conv2d operators of a session on this context) uses
 * for a single-batch product.  AHIP_GEMM_FP32: v_mfma_f32_32x32x2_f32 on the operands as they are.
 * AHIP_GEMM_BF16X3: every operand value is split exactly into three bf16 numbers and six bf16 MFMAs per
 * product accumulate in fp32 (the terms dropped are below 2^-23 of each product); measured against
 * float64 it is as close as a chain of fp32 multiply-adds, and about 1.6 times faster on large shapes.
 * AHIP_GEMM_AUTO: BF16X3 for large products whose C fills whole 256 x 256 tiles, FP32 otherwise.
 * The default is AHIP_GEMM_FP32, the only one with the reference's result for every operand value: on
 * the BF16X3 route an infinite operand value gives NaN in most of its row (inf in the leading plane meets
 * the lower planes of the other operand: inf * 0, or inf - inf) where fp32 arithmetic gives +-inf.  The reference has one sgemm
 * (gemm.rs:3-52) and no such switch. */
#define AHIP_GEMM_AUTO 0
#define AHIP_GEMM_FP32 1
#define AHIP_GEMM_BF16X3 2
int ahip_gemm_set_algorithm(ahip_ctx *ctx, int algorithm);
/* Tensors of at least `bytes` bytes are read and written with non-temporal 16-byte accesses; smaller ones are
 * left to the caches.  Default 64 MiB for a context of its own, whose caller hands over tensors from elsewhere
 * and reads results nobody knows when (Gelu over 77 MB in, 77 MB out: 70 % of the HBM peak become 73.5 %); a
 * session keeps 128 MiB for its context, because the node behind finds a smaller result in the 256 MB Infinity
 * Cache (a chain of five element-wise nodes over 77 MB tensors: 127 us against 140 us).  (size_t)-1 switches the
 * hint off, 0 applies it to everything.  No counterpart in the reference. */
int ahip_set_streaming_threshold(ahip_ctx *ctx, size_t bytes);
/* The element-wise operators (ahip_unary, ahip_binary) read a dense operand of at least `bytes` bytes with
 * non-temporal loads while storing the result the ordinary way, so that the next kernel finds it in the caches:
 * 5-10 % faster when the operand comes from HBM, 1-4 % slower when the kernel in front has just left it in the
 * caches.  Default 16 MiB, for callers that hand over tensors from elsewhere; a session sets it to the streaming
 * threshold above for its own context (its inputs were written by the node in front); (size_t)-1 does the same
 * here.  No counterpart in the reference. */
int ahip_set_load_streaming_threshold(ahip_ctx *ctx, size_t bytes);

/* The BF16X3 kernel cuts the tiles of a partly filled last round of blocks along k and lets the slice that
 * finishes last add the others' partial sums up out of one XCD's L2.  That needs all slices of a tile on one
 * XCD, which the kernel arranges by block id (the slices of a tile have equal ids mod 8, and consecutive ids go
 * to the eight XCDs in turn, starting wherever the queue's previous launch stopped).  ahip_init measures that
 * once per context with a probe launch (every block records its XCC id); the cut is used only if the probe
 * showed blocks 0..7 on eight different XCDs, every block i where block i % 8 ran, and a CU count that is a
 * multiple of eight -- otherwise tiles are not cut and the results are the same.  Every launch that cuts tiles
 * checks the XCC ids of each tile's slices again; a mismatch makes the next ahip_sync / ahip_session_run return
 * AHIP_ERR_HIP and switches the cut off for the context.  ahip_gemm_in_kernel_k_cut reports what the probe
 * showed and whether the cut is switched on; ahip_gemm_set_in_kernel_k_cut(ctx, 0) switches it off (it cannot
 * switch on what the probe did not show).  ahip_xcd_round_robin_holds is the decision itself on a recorded
 * placement (no GPU needed): 1 iff cu_count is a multiple of 8 (and >= 8), n_blocks >= 16,
 * xcc_of_block[0..7] are eight different values below 8 and xcc_of_block[i] == xcc_of_block[i % 8] for all i.
 * No counterpart in the reference. */
int ahip_gemm_in_kernel_k_cut(ahip_ctx *ctx, int *placement_shown, int *enabled);
int ahip_gemm_set_in_kernel_k_cut(ahip_ctx *ctx, int enable);
int ahip_xcd_round_robin_holds(int cu_count, const uint32_t *xcc_of_block, size_t n_blocks);
/* Declares the device buffer [ptr, ptr + bytes) immutable (model weights) until it is unregistered:
 * AHIP_GEMM_BF16X3 then splits an operand that lies inside it once and keeps the planes (1.5 times the
 * operand's size) instead of splitting it on every call.  Unregister before freeing or rewriting the
 * buffer.  No counterpart in the reference, whose sgemm reads fp32 operands directly. */
int ahip_gemm_register_constant(ahip_ctx *ctx, const void *ptr, size_t bytes);
int ahip_gemm_unregister_constant(ahip_ctx *ctx, const void *ptr);

/* Conv2d on NCHW (crates/session_interpreter/src/conv2d.rs:26-211): im2col into `col`
 * (scratch of batch*c*kh*kw*oh*ow floats, the reference's layout [b][c][kh][kw][oh][ow]) and one
 * batched GEMM per group.  w is [oc, c/group, kh, kw]; bias ([oc]) may be NULL.  oh / ow are the
 * output extents the caller inferred (shape.rs:38-88).
 * MaxPool (compute_max_pool, session.rs:324-382) over [planes, ih, iw] -> [planes, oh, ow]. */
int ahip_conv2d(ahip_ctx *ctx, float *out, const float *x, const float *w, const float *bias, float *col, size_t batch,
                size_t c, size_t ih, size_t iw, size_t oc, size_t oh, size_t ow, size_t kh, size_t kw, size_t stride_h,
                size_t stride_w, size_t dilation_h, size_t dilation_w, size_t pad_top, size_t pad_left, size_t group);
int ahip_maxpool(ahip_ctx *ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                 size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_top, size_t pad_left);
/* compute_resize (session.rs:1056-1132) over [planes, ih, iw] -> [planes, oh, ow]: nearest != 0 takes
 * x[(h / scale) as usize][(w / scale) as usize], otherwise the reference's bilinear blend (its only
 * other mode).  scale = output extent / input extent, per axis. */
int ahip_resize(ahip_ctx *ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                int nearest);

/* ------------------------------------------------------------------------
 * Graph IR: the same Model / Graph / Node / Value / Op structure as
 * altius_core (crates/core/src/model.rs:13-17, graph.rs:9-16, node.rs:7-14,
 * value.rs:9-13, op.rs:7-57), built through handles.  Value and node ids are
 * indices into the model's arenas.  None of these functions needs a device;
 * their error text is read with ahip_last_error(NULL).
 * ---------------------------------------------------------------------- */

typedef struct ahip_model ahip_model;
typedef struct ahip_tensor ahip_tensor;
typedef struct ahip_session_builder ahip_session_builder;
typedef struct ahip_session ahip_session;

/* TensorElemType (crates/core/src/tensor.rs:47-53) */
enum ahip_elem_type { AHIP_BOOL = 0, AHIP_F32 = 1, AHIP_I32 = 2, AHIP_I64 = 3 };

/* Op (crates/core/src/op.rs:7-57), same variants in the same order.  The
 * session executes the kinds marked (*); the others are representable so that
 * any altius graph can be described, and fail at build or run time with
 * AHIP_ERR_UNSUPPORTED, as the reference's unimplemented kernels do
 * (session.rs:200-245). */
enum ahip_op_kind {
    AHIP_OP_IDENTITY = 0 /* (*) */, AHIP_OP_CONV2D, AHIP_OP_ADD /* (*) */, AHIP_OP_SUB /* (*) */,
    AHIP_OP_MUL /* (*) */, AHIP_OP_DIV /* (*) */, AHIP_OP_POW /* (*) */, AHIP_OP_GREATER,
    AHIP_OP_SQRT /* (*) */, AHIP_OP_RELU /* (*) */, AHIP_OP_GELU /* (*) */, AHIP_OP_LEAKYRELU,
    AHIP_OP_SIGMOID /* (*) */, AHIP_OP_ERF /* (*) */, AHIP_OP_TANH /* (*) */, AHIP_OP_CLIP, AHIP_OP_WHERE,
    AHIP_OP_SOFTMAX /* (*) */, AHIP_OP_CAST, AHIP_OP_MAXPOOL, AHIP_OP_GLOBALAVERAGEPOOL, AHIP_OP_RESHAPE,
    AHIP_OP_FLATTEN, AHIP_OP_RESIZE, AHIP_OP_CONCAT, AHIP_OP_TRANSPOSE, AHIP_OP_SQUEEZE, AHIP_OP_UNSQUEEZE,
    AHIP_OP_REDUCEMIN, AHIP_OP_REDUCEMAX /* (*) */, AHIP_OP_REDUCEMEAN /* (*) */, AHIP_OP_ROUND, AHIP_OP_EXP,
    AHIP_OP_EXPAND, AHIP_OP_RANGE, AHIP_OP_LOOP, AHIP_OP_TILE, AHIP_OP_SPLIT, AHIP_OP_SLICE, AHIP_OP_GATHER,
    AHIP_OP_SHAPE, AHIP_OP_NONMAXSUPPRESSION, AHIP_OP_MATMUL, AHIP_OP_GEMM, AHIP_OP_BATCHNORMALIZATION,
    AHIP_OP_LAYERNORMALIZATION /* (*) */, AHIP_OP_HARDSIGMOID /* (*) */, AHIP_OP_CONSTANT,
    AHIP_OP_FUSEDELEMWISE, AHIP_OP_COUNT
};

/* Attributes of the executable operators (op.rs:84-99, 143-162, 195-200). */
typedef struct ahip_op_attrs {
    int64_t axis;                /* Softmax, LayerNormalization */
    int64_t axes[AHIP_MAX_RANK]; /* ReduceMax, ReduceMean */
    int32_t n_axes;
    int32_t keep_dims;           /* ReduceMax, ReduceMean */
    float alpha;                 /* HardSigmoid */
    float beta;                  /* HardSigmoid */
    float epsilon;               /* LayerNormalization */
    int64_t stash_type;          /* LayerNormalization */
} ahip_op_attrs;

/* Fills the ONNX defaults the reference's loader applies
 * (crates/core/src/onnx/load.rs:185-187, 277-288, 321-324, 340-344):
 * axis -1, no axes, keep_dims 1, alpha 0.2, beta 0.5, epsilon 1e-5, stash_type 1. */
void ahip_op_attrs_default(ahip_op_attrs *attrs);
const char *ahip_op_name(int op_kind); /* Op::name (op.rs:324-376) */

int ahip_model_new(int64_t opset_version, ahip_model **model);
int ahip_model_clone(const ahip_model *model, ahip_model **copy);
void ahip_model_free(ahip_model *model);
/* ValueArena::new_val / new_val_named (value.rs:19-31); name may be NULL. */
int ahip_model_new_value(ahip_model *model, const char *name, int64_t *value_id);
/* ValueArena::new_val_named_and_shaped (value.rs:33-42); a negative dim is a dynamic one. */
int ahip_model_new_value_shaped(ahip_model *model, const char *name, int elem_type, int rank,
                                const int64_t *dims, int64_t *value_id);
/* graph.inits.insert (graph.rs:13); data is copied, nbytes must match the shape. */
int ahip_model_add_initializer(ahip_model *model, int64_t value_id, int elem_type, int rank,
                               const int64_t *dims, const void *data, size_t nbytes);
/* Graph::add_node (graph.rs:18-22); name may be NULL.  With attrs == NULL the operator starts
 * from the defaults the ONNX loader applies to its kind (load.rs:171-361) and is then refined with
 * ahip_node_set_attr_*; a non-NULL block sets the seven fields of ahip_op_attrs as given. */
int ahip_model_add_node(ahip_model *model, int op_kind, const ahip_op_attrs *attrs, const char *name,
                        int n_inputs, const int64_t *inputs, int n_outputs, const int64_t *outputs,
                        int64_t *node_id);
int ahip_model_add_input(ahip_model *model, int64_t value_id);   /* graph.inputs.push */
int ahip_model_add_output(ahip_model *model, int64_t value_id);  /* graph.outputs.push */
/* Model::lookup_named_value (model.rs:19-28); AHIP_ERR_ARG when no value has that name. */
int ahip_model_lookup_named_value(const ahip_model *model, const char *name, int64_t *value_id);
/* which = 0: graph.inputs, 1: graph.outputs.  *n gets the full count even beyond capacity. */
int ahip_model_graph_io(const ahip_model *model, int which, int64_t *value_ids, int capacity, int *n);
/* Model::topo_sort_nodes (model.rs:62-101). */
int ahip_model_topo_sort(const ahip_model *model, int64_t *node_ids, int capacity, int *n);
/* Reads one node back.  inputs/outputs hold io_capacity entries each. */
int ahip_model_node_info(const ahip_model *model, int64_t node_id, int *op_kind, ahip_op_attrs *attrs,
                         int *n_inputs, int64_t *inputs, int *n_outputs, int64_t *outputs, int io_capacity);
/* infer_shapes (crates/core/src/analysis/shape.rs:659-692) and the shape it finds for one
 * value.  AHIP_ERR_SHAPE if inference fails, AHIP_ERR_ARG if that value's shape stays unknown. */
int ahip_model_infer_value_shape(const ahip_model *model, int64_t value_id, int *elem_type, int *rank,
                                 int64_t *dims);
/* create_execution_plan (crates/session/src/plan.rs:14-58): node ids in execution order,
 * and for node i the values freed after it: free_vals[free_offsets[i] .. free_offsets[i+1]).
 * free_offsets holds node_capacity + 1 entries. */
int ahip_model_execution_plan(const ahip_model *model, int64_t *node_ids, int *free_offsets,
                              int node_capacity, int64_t *free_vals, int free_capacity, int *n_nodes,
                              int *n_free);

/* ONNX files (crates/core/src/onnx/load.rs:55-63: load_onnx, load_onnx_from_buffer).  The
 * decoder reads the protobuf wire format itself; values are created in the reference's order
 * (initializers, graph inputs, graph outputs, then node inputs/outputs as met).  Errors mirror
 * ModelLoadError (load.rs:25-53): AHIP_ERR_IO for the file, AHIP_ERR_ARG for a malformed or
 * graph-less model, a missing required attribute or value type/shape, AHIP_ERR_UNSUPPORTED for
 * operators, element types and opset domains the reference does not load. */
int ahip_model_load_onnx(const char *path, ahip_model **model);
int ahip_model_load_onnx_buffer(const void *data, size_t bytes, ahip_model **model);
int64_t ahip_model_opset_version(const ahip_model *model);
int64_t ahip_model_num_values(const ahip_model *model);
int64_t ahip_model_num_nodes(const ahip_model *model);
/* One value: its name (NULL if unnamed; valid until the model changes), and its declared shape:
 * *rank is -1 when none is declared, dynamic dimensions read -1.  Any output pointer may be NULL. */
int ahip_model_value_info(const ahip_model *model, int64_t value_id, const char **name, int *elem_type,
                          int *rank, int64_t *dims, int dims_capacity);
/* A copy of the initializer bound to a value (graph.inits); AHIP_ERR_ARG if it has none. */
int ahip_model_initializer(const ahip_model *model, int64_t value_id, ahip_tensor **tensor);
/* Node name (NULL if unnamed). */
const char *ahip_model_node_name(const ahip_model *model, int64_t node_id);

/* Operator attributes by their ONNX names ("axis", "axes", "keepdims", "perm", "split", "to",
 * "kernel_shape", "strides", "pads", "dilations", "group", "auto_pad", "alpha", "beta",
 * "transA", "transB", "epsilon", "momentum", "training_mode", "stash_type", "start", "end",
 * "mode", "nearest_mode", "coordinate_transformation_mode", "cubic_coeff_a", "exclude_outside",
 * "extrapolation_value", "value"): every field of the attribute structs in op.rs:59-218.
 * AHIP_ERR_ARG when the node's operator does not carry an attribute of that name and kind. */
int ahip_node_set_attr_int(ahip_model *model, int64_t node_id, const char *name, int64_t value);
int ahip_node_set_attr_float(ahip_model *model, int64_t node_id, const char *name, float value);
int ahip_node_set_attr_ints(ahip_model *model, int64_t node_id, const char *name, const int64_t *values, int n);
int ahip_node_set_attr_string(ahip_model *model, int64_t node_id, const char *name, const char *value);
int ahip_node_set_attr_tensor(ahip_model *model, int64_t node_id, const char *name, const ahip_tensor *value);
int ahip_node_get_attr_int(const ahip_model *model, int64_t node_id, const char *name, int64_t *value);
int ahip_node_get_attr_float(const ahip_model *model, int64_t node_id, const char *name, float *value);
/* *n gets the full count even beyond capacity. */
int ahip_node_get_attr_ints(const ahip_model *model, int64_t node_id, const char *name, int64_t *values,
                            int capacity, int *n);
/* Copies at most capacity-1 characters and a terminator; *n gets the full length. */
int ahip_node_get_attr_string(const ahip_model *model, int64_t node_id, const char *name, char *value,
                              int capacity, int *n);
int ahip_node_get_attr_tensor(const ahip_model *model, int64_t node_id, const char *name, ahip_tensor **value);

/* Fusion passes (crates/core/src/optimize/{layer_norm_fusion,gelu_fusion,fast_gelu_fusion,
 * identity_elim}.rs).  *count (may be NULL) gets the number of rewrites. */
int ahip_fuse_layer_norm(ahip_model *model, int *count);
int ahip_fuse_gelu(ahip_model *model, int *count);
int ahip_fuse_fast_gelu(ahip_model *model, int *count);
int ahip_eliminate_identity(ahip_model *model, int *count);
/* fuse_elemwise_ops (crates/core/src/optimize/elemwise_fusion.rs:12-138): chains of element-wise
 * operators become one FusedElemwise node each, which the session runs as one kernel
 * (ahip_fused_elemwise) with the bits of the unfused chain.  AHIP_FUSE_REFERENCE_RULE restates the
 * reference's conditions (operators of Op::is_elemwise; the previous result must be the first operand of
 * the next node, the previous node binary, second operands of equal shape).  AHIP_FUSE_EXTENDED_RULE is
 * this backend's own: the previous result may be either operand, other operands may have any
 * broadcastable shape and come from anywhere outside the chain, and Erf / Gelu / Sigmoid / Tanh / Exp /
 * Round count as element-wise; f32 tensors of known shape only, at most 16 steps and 6 operands per chain.
 * Under both rules a value that is also a graph output ends its chain.  AHIP_ERR_SHAPE when shape
 * inference fails (the reference returns ShapeError).  The node's operators can be read back with
 * ahip_node_get_attr_string(model, node, "chain", ...) as a comma-separated list of names. */
/* Not in the reference: [Mul | Div by a one-element f32 initializer] -> [Add of a mask that is constant along
 * every axis but the first and the last] -> Softmax(last axis) becomes one Softmax node with inputs
 * (x, scale?, mask?), run as one kernel (ahip_softmax_lastaxis_prologue) with the bits of the separate nodes.
 * Readable afterwards as the integer attributes "prologue_scale" (0 none, 1 multiply, 2 divide) and
 * "prologue_mask" of the Softmax node. */
int ahip_fuse_softmax_prologue(ahip_model *model, int *count);
/* Not in the reference: MatMul(x, W) -> Add(., b), b holding one value per output column and the product having
 * no other reader, becomes a MatMul node with b as third input; the session adds it in the product's epilogue
 * (the same single addition per element, without the extra pass over the output). */
int ahip_fuse_matmul_bias(ahip_model *model, int *count);
/* fuse_transpose_matmul (crates/core/src/optimize/transpose_fusion.rs:10-104; switched off in the reference,
 * mod.rs:7, because its interpreter cannot run the node it emits): a Transpose of the last two axes in front of a
 * MatMul operand is folded into the product.  The MatMul node then reads the untransposed tensor and reports
 * "transA" / "transB" through ahip_node_get_attr_int; a Transpose with other readers stays for them. */
int ahip_fuse_transpose_matmul(ahip_model *model, int *count);
enum ahip_fuse_rule { AHIP_FUSE_REFERENCE_RULE = 0, AHIP_FUSE_EXTENDED_RULE = 1 };
int ahip_fuse_elemwise_ops(ahip_model *model, int rule, int *count);

/* Host tensors (crates/core/src/tensor.rs:61-76).  data is copied; NULL data gives zeros.
 * Storage of 64 KiB and more is pinned (page-locked) host memory from a process-wide pool when
 * a device is present, so that ahip_session_run moves it over PCIe by DMA; a freed tensor's
 * block is kept for the next tensor of its size class. */
int ahip_tensor_new(int elem_type, int rank, const int64_t *dims, const void *data, size_t nbytes,
                    ahip_tensor **tensor);
void ahip_tensor_free(ahip_tensor *tensor);
int ahip_tensor_elem_type(const ahip_tensor *tensor);
int ahip_tensor_rank(const ahip_tensor *tensor);
int ahip_tensor_dims(const ahip_tensor *tensor, int64_t *dims, int capacity);
size_t ahip_tensor_nbytes(const ahip_tensor *tensor);
const void *ahip_tensor_data(const ahip_tensor *tensor);
/* Writable view of the same bytes, to fill a tensor made with NULL data in place
 * (Tensor::data_mut, crates/core/src/tensor.rs:318). */
void *ahip_tensor_data_mut(ahip_tensor *tensor);

/* The pinned pool behind host tensors: bytes handed out, bytes cached for reuse, page-locking
 * allocations made so far and requests served from the cache (any pointer may be NULL).
 * ahip_host_pool_trim frees the cached blocks and returns the number of bytes freed. */
int ahip_host_pool_stats(size_t *live_bytes, size_t *cached_bytes, size_t *pinned_allocations, size_t *reuses);
size_t ahip_host_pool_trim(void);

/* ------------------------------------------------------------------------
 * Session: InterpreterSessionBuilder / InterpreterSession
 * (crates/session_interpreter/src/builder.rs:18-66, session.rs:61-134).
 * ---------------------------------------------------------------------- */

/* InterpreterSessionBuilder::new(model); the model is copied. */
int ahip_session_builder_new(const ahip_model *model, ahip_session_builder **builder);
void ahip_session_builder_free(ahip_session_builder *builder);
/* with_intra_op_num_threads: accepted for parity, device kernels use no host threads. */
int ahip_session_builder_with_intra_op_num_threads(ahip_session_builder *builder, size_t n);
int ahip_session_builder_with_profiling_enabled(ahip_session_builder *builder, int enable);
/* Not in the reference: the GPU to run on (default 0). */
int ahip_session_builder_with_device(ahip_session_builder *builder, int device);
/* Not in the reference: with enable != 0 the session records the kernels of a run as a HIP graph
 * the second time it sees a set of input shapes and replays that graph afterwards (one launch per
 * run instead of one per node).  Results are those of the node-by-node run.  Graphs whose shapes
 * or operands need the host during the run, and profiled sessions, keep running node by node. */
int ahip_session_builder_with_graph_replay(ahip_session_builder *builder, int enable);
/* Not in the reference (its run() times itself with Instant::now() only when profiling is on,
 * crates/session_interpreter/src/session.rs:74,117-125): with enable == 0 a run is no longer bracketed by
 * two events on the session's stream, and ahip_session_last_device_ms reports 0.  Default on.  Two event
 * records per run cost a few microseconds on the host and in the queue, which a caller of small graphs
 * that does not read the device time can do without. */
int ahip_session_builder_with_device_timing(ahip_session_builder *builder, int enable);
/* Not in the reference: the kernel the session's large single-batch MatMul / Gemm products take
 * (AHIP_GEMM_FP32, the default, AHIP_GEMM_AUTO or AHIP_GEMM_BF16X3; see ahip_gemm_set_algorithm).  The
 * default keeps the reference's semantics for every operand value (compute_mat_mul, session.rs:621-684: an
 * infinite operand gives +-inf); AUTO and BF16X3 are the faster route a caller opts into, where an infinite
 * operand gives NaN.  The session declares its float initializers constant to the GEMM, so the bf16 planes
 * of a weight are made on its first use and kept until the session is freed. */
int ahip_session_builder_with_gemm_algorithm(ahip_session_builder *builder, int algorithm);
/* Not in the reference, whose Split and Transpose always copy (session.rs:1179-1278, 1488-1548): with enable
 * != 0 (the default) a Split or Transpose whose result only MatMuls read, possibly through reshapes and further
 * transposes, hands out a strided view of its input, which the MatMul reads in place (ahip_gemm_batch2), and
 * a MatMul read only by a Transpose that keeps the last axis writes that Transpose's layout directly.  The
 * products are the same kernels on the same values: results do not change by a bit.  A view that some other
 * reader needs, or that the GEMM's addressing cannot express, is copied as before. */
int ahip_session_builder_with_strided_views(ahip_session_builder *builder, int enable);
/* Not in the reference, which runs MatMul, Softmax and MatMul as three kernels (session.rs:621-684, 990-1026):
 * with enable != 0 (default 0; needs strided views) a MatMul -> Softmax(last axis, with the scale and per-key
 * mask that ahip_fuse_softmax_prologue absorbed) -> MatMul chain with 64-wide heads runs as one ahip_attention
 * kernel that never writes the scores.  Its sums run in another order than the three operators': results
 * differ from theirs by up to 2e-4 relative, which is why a caller has to ask for it.  On the bf16 route, an
 * attention whose output only the product behind its Transpose and Reshape reads leaves the kernel as that
 * product's operand planes (the split of the same values). */
int ahip_session_builder_with_fused_attention(ahip_session_builder *builder, int enable);
/* Nodes of the last node-by-node run that were served without their copy (views taken, transposed layouts
 * written in place). */
int ahip_session_copies_avoided(const ahip_session *session, size_t *count);
/* Lanes the session holds so far (1 until two ahip_session_run calls have overlapped). */
int ahip_session_lanes(ahip_session *session, size_t *count);
/* build(): shape inference (AHIP_ERR_SHAPE on failure), execution plan, device context,
 * upload of the initializers.  The builder stays valid and must still be freed. */
int ahip_session_builder_build(ahip_session_builder *builder, ahip_session **session);

void ahip_session_free(ahip_session *session);
/* run(inputs): inputs are bound to graph.inputs in order; outputs come back in
 * graph.outputs order as new tensors the caller frees.  *n_outputs gets their
 * number; AHIP_ERR_ARG if output_capacity is too small.  Like
 * InterpreterSession::run(&self), which keeps its values in a map per calling
 * thread (crates/session_interpreter/src/session.rs:56,75-78), it may be called
 * from several threads at once: a session holds up to 16 lanes (a stream, a
 * buffer pool and a copy of the initializers each), builds a further one the first
 * time a call finds all of them busy, and queues calls beyond 16.  The profile
 * read back afterwards is that of the call that finished last. */
int ahip_session_run(ahip_session *session, int n_inputs, const ahip_tensor *const *inputs,
                     int output_capacity, ahip_tensor **outputs, int *n_outputs);
/* Not in the reference (its tensors are host memory): the same run on tensors that already live on
 * the session's GPU, so that nothing crosses PCIe.  Input i is `device_ptrs[i]`, caller-owned device
 * memory holding a dense row-major tensor of `elem_types[i]` (ahip_elem_type) and `dims[i][0..ranks[i])`.
 * The call enqueues the whole plan on the session's stream and returns without waiting: inputs are
 * read in stream order (they must hold their data before the call and stay valid until
 * ahip_session_synchronize), and the outputs hold their results once ahip_session_synchronize has
 * returned.  Outputs are device tensors in graph-output order; their memory belongs to the session's
 * pool, except that an output which is a reshaped view of an input is the caller's own pointer.
 * Free each with ahip_device_tensor_free (before or after the session; the pool lives until both
 * are gone).  A recorded HIP graph is not used on this path. */
typedef struct ahip_device_tensor ahip_device_tensor;
int ahip_session_run_device(ahip_session *session, int n_inputs, const void *const *device_ptrs,
                            const int *elem_types, const int *ranks, const int64_t *const *dims,
                            int output_capacity, ahip_device_tensor **outputs, int *n_outputs);
/* Waits for everything the session has enqueued; reports errors kernels leave in device flags
 * (an out-of-range Gather index) as AHIP_ERR_ARG. */
int ahip_session_synchronize(ahip_session *session);
void ahip_device_tensor_free(ahip_device_tensor *tensor);
void *ahip_device_tensor_ptr(const ahip_device_tensor *tensor);
int ahip_device_tensor_elem_type(const ahip_device_tensor *tensor);
int ahip_device_tensor_rank(const ahip_device_tensor *tensor);
int ahip_device_tensor_dims(const ahip_device_tensor *tensor, int64_t *dims, int capacity);
size_t ahip_device_tensor_nbytes(const ahip_device_tensor *tensor);
/* model(): a borrowed handle, valid while the session lives. */
const ahip_model *ahip_session_model(const ahip_session *session);
/* Per-operator device time of the last run when profiling is enabled
 * (session.rs:117-125, 251-255): entry `index` of `*count` entries. */
int ahip_session_profile(const ahip_session *session, int index, const char **op_name, double *ms,
                         int *count);
int ahip_session_last_run_ms(const ahip_session *session, double *ms);
/* Not in the reference: device time of the last run's kernels alone (between the uploads and the
 * downloads), measured by two events on the session's stream. */
int ahip_session_last_device_ms(const ahip_session *session, double *ms);
/* Number of hipMalloc calls the session's buffer pool has made so far. */
int ahip_session_device_allocations(const ahip_session *session, size_t *count);
/* Runs served by replaying a recorded HIP graph so far. */
int ahip_session_graph_replays(const ahip_session *session, size_t *count);

#ifdef __cplusplus
}
#endif

#endif
