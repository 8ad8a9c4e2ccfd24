// Device context and the launcher entry points shared by the C ABI and the
// session.  Everything here is host code; kernels live in the .hip files.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../../include/altius_hip.h"

namespace altius {

// A device buffer whose contents the caller has declared immutable (weights), and the bf16 planes the
// split GEMM has derived from an operand inside such a buffer.
struct ConstantBuffer {
    const void *ptr;
    size_t bytes;
};
struct PackedOperand {
    const void *owner;  // the ConstantBuffer the operand lies in
    const void *src;
    size_t rows, k, ld;
    bool k_contig;
    void *planes;
    size_t bytes;
};

// The streaming threshold of a session's context (see DeviceCtx::nt_threshold_bytes).
constexpr size_t SESSION_NT_THRESHOLD_BYTES = (size_t)128 << 20;

// One context = one device + one stream.  All work issued through a context is
// ordered on that stream.  A context is not thread-safe; use one per thread.
struct DeviceCtx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    // Partial results of two-stage reductions (device memory, owned).
    float *scratch = nullptr;
    size_t scratch_floats = 0;
    // Error flags kernels raise (device memory; int 0: Gather's index check, int 1: the slices of a GEMM tile
    // cut along k did not share an XCD); read back by check_device_flags after a synchronisation, only when a
    // kernel that can raise one has run.
    int *flags = nullptr;
    bool flags_armed = false;
    // Tensors of at least this many bytes are streamed with non-temporal accesses (a session raises it to
    // SESSION_NT_THRESHOLD_BYTES: its results are read by the node behind, out of the Infinity Cache if they fit).
    size_t nt_threshold_bytes = (size_t)64 << 20;
    size_t nt_load_threshold_bytes = (size_t)16 << 20;
    // Chains of element-wise steps that were instantiated at compile time run as straight-line code;
    // switched off, every chain takes the interpreting kernel (tests compare the two).
    bool fused_static_chains = true;
    // Which kernel large single-batch fp32 products take (AHIP_GEMM_*).  The default is the one whose
    // results equal fp32 arithmetic for every operand value, infinities included.
    int gemm_algorithm = AHIP_GEMM_FP32;
    // bf16 planes of the run-time operands of the split GEMM (device memory, owned, grows on demand;
    // the generation counts reallocations so that holders of recorded launches can tell).
    void *gemm_ws = nullptr;
    size_t gemm_ws_bytes = 0;
    uint64_t gemm_ws_generation = 0;
    // Partial sums and arrival counters of tiles the bf16 GEMM cuts along k (device memory, owned).
    void *gemm_partials = nullptr;
    size_t gemm_partials_bytes = 0;
    int *gemm_counters = nullptr;
    bool gemm_split_k = true;
    int cus_per_xcd = 0;  // compute units / 8, read when the context is created
    // Measured when the context is created (placement.hip): blocks whose ids agree mod 8 run on one XCD, and
    // eight consecutive blocks on eight different ones.  The bf16 GEMM lets the slices of a tile meet in one
    // XCD's L2 only when this holds and gemm_in_kernel_k_cut is on; otherwise it does not cut tiles inside the
    // kernel at all.
    bool xcd_round_robin = false;
    bool gemm_in_kernel_k_cut = true;
    std::vector<ConstantBuffer> gemm_constants;
    std::vector<PackedOperand> gemm_packed;
    std::string last_error;

    bool streaming(size_t bytes) const { return bytes >= nt_threshold_bytes; }
    // Element-wise kernels read an input of at least nt_load_threshold_bytes with non-temporal loads while storing
    // the result the ordinary way: an input that comes from HBM streams 5-10 % faster that way, one that the previous
    // kernel has just left in the caches 1-4 % slower.  A context assumes the first for 16 MiB and more; a session,
    // whose every input was written by the node in front, raises the threshold to nt_threshold_bytes.
    bool streaming_loads(size_t bytes) const { return bytes >= nt_threshold_bytes || bytes >= nt_load_threshold_bytes; }

    int fail(int code, const std::string &msg);
    int check(hipError_t e, const char *what);
};

// Sets the calling thread's "no context" error text (ahip_last_error(NULL)).
void set_global_error(const std::string &msg);
const char *global_error();

// Creates / tears down a context (stream + scratch buffer) on `device`.
int create_device_ctx(int device, hipStream_t stream, bool own_stream, DeviceCtx *ctx, std::string *error);
void destroy_device_ctx(DeviceCtx *ctx);
// The decision behind DeviceCtx::xcd_round_robin, on its own so that it can be tested without a GPU: true iff
// the CU count is a multiple of eight, blocks 0..7 of the probe launch ran on eight different XCDs and every
// block i ran where block i % 8 did.
bool xcd_round_robin_holds(int cu_count, const uint32_t *xcc_of_block, size_t n_blocks);
// Runs the probe launch on the context's stream (uses the scratch buffer) and sets ctx.xcd_round_robin.
int probe_xcd_placement(DeviceCtx &ctx, int cu_count);
// After the stream has been synchronised: reports and clears an error flag raised by a kernel.
int check_device_flags(DeviceCtx &ctx);

constexpr int MAX_RANK = 8;
constexpr size_t SCRATCH_FLOATS = 1u << 20;  // 4 MiB

int launch_binary(DeviceCtx &ctx, int op, float *out, const float *a, const float *b, int rank,
                  const int64_t *out_dims, const int64_t *a_strides, const int64_t *b_strides);
int launch_unary(DeviceCtx &ctx, int op, float *out, const float *in, size_t n, float alpha,
                 float beta);
// A chain of element-wise steps in one kernel (fused.hip); AHIP_ERR_UNSUPPORTED when the geometry
// needs the operator-by-operator route.
int launch_fused_elemwise(DeviceCtx &ctx, float *out, int rank, const int64_t *out_dims, int n_inputs, const float *const *inputs,
                          const int64_t *const *input_strides, int n_steps, const ahip_fused_step *steps);
int launch_softmax(DeviceCtx &ctx, float *out, const float *in, size_t rows, size_t len);
// Softmax of (in [*|/] scale) + mask over the last axis; scale_op 0 none / 1 multiply / 2 divide, mask (may be
// null) holds rows / rows_per_mask rows of len values.  AHIP_ERR_UNSUPPORTED when the geometry needs separate kernels.
int launch_softmax_prologue(DeviceCtx &ctx, float *out, const float *in, size_t rows, size_t len, int scale_op, float scale,
                            const float *mask, size_t rows_per_mask);
int launch_layernorm(DeviceCtx &ctx, float *out, const float *in, const float *gamma,
                     const float *beta, size_t rows, size_t len, float eps);
int launch_reduce(DeviceCtx &ctx, int kind, float *out, const float *in, size_t outer, size_t red,
                  size_t inner);
// The same reduction for callers that may not allocate: partial results go to a fixed array in the code
// object instead of the context's scratch buffer, and a shape whose partial results do not fit fails with
// AHIP_ERR_UNSUPPORTED.  reduce_static_setup resolves the array's address for `device`, which must be the
// calling thread's current device; create_device_ctx calls it.
int launch_reduce_static(DeviceCtx &ctx, int kind, float *out, const float *in, size_t outer, size_t red, size_t inner);
int reduce_static_setup(int device);
// A stream that is about to be destroyed (its work has been waited for) no longer owns the fixed array.
void reduce_static_forget_stream(int device, hipStream_t stream);
size_t reduce_static_capacity_floats();


// Data movement (movement.hip).  Strides are in elements; elem_size in bytes (1, 4 or 8).
int launch_copy_strided(DeviceCtx &ctx, void *out, const void *in, int elem_size, int rank, const int64_t *dims,
                        const int64_t *out_strides, const int64_t *in_strides);
int launch_transpose(DeviceCtx &ctx, void *out, const void *in, int elem_size, int rank, const int64_t *in_dims,
                     const int64_t *perm);
// *bad_flag (device memory, zeroed by the caller) becomes 1 if an index is out of range.
int launch_gather(DeviceCtx &ctx, void *out, const void *data, const void *indices, int index_size, int elem_size,
                  size_t outer, size_t axis_len, size_t n_idx, size_t inner, int *bad_flag);
int launch_where(DeviceCtx &ctx, void *out, const void *cond, const void *x, const void *y, int elem_size, int rank,
                 const int64_t *dims, const int64_t *c_strides, const int64_t *x_strides, const int64_t *y_strides);
int launch_greater(DeviceCtx &ctx, uint8_t *out, const float *a, const float *b, int rank, const int64_t *dims,
                   const int64_t *a_strides, const int64_t *b_strides);
int launch_cast(DeviceCtx &ctx, void *out, const void *in, int from_type, int to_type, size_t n);
int launch_batchnorm(DeviceCtx &ctx, float *out, const float *x, const float *scale, const float *bias, const float *mean,
                     const float *var, size_t n, size_t c, size_t hw, float eps);

// C[b] = alpha * op(A[b]) * op(B[b]) + beta * C0 for b in [0, batch) (matmul.hip).  op(X) is X or its
// transpose; lda / ldb / ldc are row pitches of the stored matrices; batch strides in elements
// (0 = one matrix shared by all batches); C0 may be null, and is read at
// c0[i * c0_row_stride + j * c0_col_stride] (strides of 0 broadcast a row vector or a scalar).
int launch_gemm(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t batch, size_t m, size_t n,
                size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t a_batch_stride,
                size_t b_batch_stride, size_t c_batch_stride, size_t c0_row_stride, size_t c0_col_stride, float alpha,
                float beta);

// The same with the batch index split in two, z = (z / batch_inner, z % batch_inner), each part with its own
// stride per operand: operands that are strided views of a larger tensor (the heads of a [b, t, h, d] tensor
// read in place as b x h matrices of t x d with row pitch h * d) need no copy.
// post (may be null): what the operators behind the product would do to its result, done while it is written, single
// batch only and always on the fp32 kernel: C = act(alpha * op(A) op(B) + beta * C0) + residual, act 0 or AHIP_GELU /
// AHIP_RELU, residual null or a matrix laid out like C (same pitch).  Each step rounds as its own kernel would.
struct GemmPost {
    int act = 0;
    const float *residual = nullptr;
};
int launch_gemm_batch2(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t batch_outer,
                       size_t batch_inner, size_t m, size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc,
                       const size_t a_batch_strides[2], const size_t b_batch_strides[2], const size_t c_batch_strides[2],
                       size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta, const GemmPost *post = nullptr);

// Many small products at once (matmul_small.hip): one block per matrix.  C = A B, A with unit stride along k.
bool gemm_small_batched_fits(size_t batch, size_t m, size_t n, size_t k);
int launch_gemm_small_batched(DeviceCtx &ctx, float *c, const float *a, const float *b, size_t batch_outer, size_t batch_inner, size_t m, size_t n,
                              size_t k, int trans_b, size_t lda, size_t ldb, size_t ldc, const size_t a_bs[2], const size_t b_bs[2],
                              const size_t c_bs[2]);

// O = Softmax(scale(Q K^T) + mask) V per batch, scores kept in registers (attention.hip).  Q [tq, d], K [tk, d], V [tk, d],
// O [tq, d] with row pitches ld*; batches as in launch_gemm_batch2; scale_op 0 none / 1 multiply / 2 divide; mask (may be
// null) one value per key, read at mask[outer batch * mask_outer_stride + key].
// AHIP_ERR_UNSUPPORTED (nothing launched) unless d == 64 and everything is 16-byte aligned.
int launch_attention(DeviceCtx &ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer, size_t batch_inner,
                     size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo, const size_t q_bs[2],
                     const size_t k_bs[2], const size_t v_bs[2], const size_t o_bs[2], int scale_op, float scale, const float *mask = nullptr,
                     size_t mask_outer_stride = 0, void *o_planes = nullptr);
// o_planes: O, taken as the matrix [batch_outer * tq, batch_inner * 64] (o is not written), leaves as the operand planes
// of the product on the bf16 route that reads it (gemm_planes_bytes(batch_outer * tq, batch_inner * 64) bytes).  Only
// where attention_writes_planes says so.
bool attention_writes_planes(const DeviceCtx &ctx, size_t batch_outer, size_t batch_inner, size_t tq);

// The same product for one batch through three bf16 planes per operand and six bf16 MFMAs per fp32
// product (gemm_split.hip): as accurate as an fp32 multiply-add chain, about 1.6 times the fp32 matrix
// cores' rate on large shapes.  launch_gemm takes this route by itself according to ctx.gemm_algorithm.
// a_op: 0, or AHIP_GELU / AHIP_RELU applied to A's values while they are split (C = alpha f(A) B + beta C0).
// a_planes (may be null): the first operand already as planes, as launch_layernorm_planes writes them (then a, lda
// and a_op are not used): rows = m, k = k, gemm_planes_bytes(m, k) bytes.
int launch_gemm_split(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t m, size_t n, size_t k,
                      int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t c0_row_stride, size_t c0_col_stride,
                      float alpha, float beta, int a_op = 0, const void *a_planes = nullptr);
size_t gemm_planes_bytes(size_t rows, size_t k);
// LayerNormalization over rows of `len` elements written as the planes of the first operand of a product on the
// bf16 route (rows = rows, k = len; gemm_planes_bytes(rows, len) bytes) instead of fp32 values: the planes that
// launch_layernorm followed by the operand split would give, bit for bit.  in2 (may be null): the rows are in + in2
// (a residual connection), and the sum is stored to sum_out as well.  Only for shapes layernorm_planes_fits accepts.
int launch_layernorm_planes(DeviceCtx &ctx, void *planes, float *sum_out, const float *in, const float *in2, const float *gamma,
                            const float *beta, size_t rows, size_t len, float eps);
bool layernorm_planes_fits(size_t rows, size_t len);
// The context's grow-only GEMM workspace, at least `bytes` large (stream-ordered use only).
int gemm_workspace(DeviceCtx &ctx, size_t bytes, void **p);
// Row sums (optionally times `scale`) or maxima of a [rows, len] matrix through LDS-staged groups of rows (rows.hip): for
// rows that are short or not whole float4s.  Returns -1 without launching when the shape is not one it is meant for.
int launch_reduce_rows_lds(DeviceCtx &ctx, bool is_max, float *out, const float *in, size_t rows, size_t len, float scale, bool scaled);
// Whether launch_gemm would send this single-batch product through launch_gemm_split.
bool gemm_takes_split(const DeviceCtx &ctx, size_t m, size_t n, size_t k);
// Large and tile-filling enough for the split kernel to win (the AHIP_GEMM_AUTO rule).
bool gemm_split_worthwhile(size_t m, size_t n, size_t k);
// Declares [ptr, ptr + bytes) immutable until unregistered: operands inside it are split once and the
// planes kept.  Unregistering frees them (after synchronising the stream).
int gemm_register_constant(DeviceCtx &ctx, const void *ptr, size_t bytes);
int gemm_unregister_constant(DeviceCtx &ctx, const void *ptr);
void gemm_release_all(DeviceCtx &ctx);

// col[b][c][fy][fx][oh][ow] for a convolution (movement.hip); maxpool over [planes, ih, iw].
int launch_im2col(DeviceCtx &ctx, float *col, const float *x, size_t batch, size_t c, size_t ih, size_t iw, size_t oh,
                  size_t ow, size_t kh, size_t kw, size_t sh, size_t sw, size_t dh, size_t dw, size_t pad_t, size_t pad_l);
int launch_maxpool(DeviceCtx &ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                   size_t kh, size_t kw, size_t sh, size_t sw, size_t pad_t, size_t pad_l);
// Conv2d = im2col + one batched GEMM per group (conv2d.cpp).  `col` is caller-provided scratch of
// batch * c * kh * kw * oh * ow floats; bias may be null.
int launch_conv2d(DeviceCtx &ctx, float *out, const float *x, const float *w, const float *bias, float *col, size_t batch,
                  size_t c, size_t ih, size_t iw, size_t oc, size_t oh, size_t ow, size_t kh, size_t kw, size_t sh, size_t sw,
                  size_t dh, size_t dw, size_t pad_t, size_t pad_l, size_t group);

// Resize on [planes, ih, iw] -> [planes, oh, ow]: nearest, or the reference's bilinear blend (movement.hip).
int launch_resize(DeviceCtx &ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                  int nearest);

}  // namespace altius
