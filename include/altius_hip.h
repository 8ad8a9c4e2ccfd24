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
    AHIP_RELU = 5         /* compute_relu, session.rs:796-803 */
};

/* Flat element-wise op over n elements.  alpha/beta are read by HardSigmoid only. */
int ahip_unary(ahip_ctx *ctx, int op, float *out, const float *in, size_t n, float alpha,
               float beta);

/* compute_softmax over the last axis (session.rs:990-1026 + fast_math.rs:102-187):
 * `rows` rows of `len` contiguous elements. */
int ahip_softmax_lastaxis(ahip_ctx *ctx, float *out, const float *in, size_t rows, size_t len);

/* compute_layer_normalization over the last axis (session.rs:1433-1486).
 * gamma and beta hold `len` values each. */
int ahip_layernorm_lastaxis(ahip_ctx *ctx, float *out, const float *in, const float *gamma,
                            const float *beta, size_t rows, size_t len, float eps);

enum ahip_reduce_kind { AHIP_REDUCE_MEAN = 0, AHIP_REDUCE_MAX = 1 };

/* compute_reduce_mean / compute_reduce_max (session.rs:1292-1340), generalised
 * to any contiguous run of reduced axes: the input is viewed as
 * [outer, reduce, inner] and `out` as [outer, inner].  The reference's kernels
 * are the cases inner == 1 (ReduceMean over the last axis) and outer == 1,
 * inner == 1 (ReduceMax over everything).  ReduceMax ignores NaN (the reference
 * panics on NaN). */
int ahip_reduce(ahip_ctx *ctx, int kind, float *out, const float *in, size_t outer, size_t reduce,
                size_t inner);

#ifdef __cplusplus
}
#endif

#endif
