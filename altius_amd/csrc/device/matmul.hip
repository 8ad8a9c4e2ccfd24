// fp32 matrix multiplication on the matrix cores: C = alpha * op(A) * op(B) + beta * C0, batched
// with broadcast batch strides.  Counterparts in the reference: compute_mat_mul
// (crates/session_interpreter/src/session.rs:621-684) and compute_gemm (686-794), both of which
// call sgemm (crates/session_interpreter/src/gemm.rs: the `matrixmultiply` crate or CBLAS).
//
// This is the one MFMA-bound kernel of the library.  A 256-thread block (4 wavefronts in a 2 x 2
// grid) owns a 128 x 128 tile of C; each wavefront accumulates a 64 x 64 sub-tile in four
// 32 x 32 accumulators with v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate: 256 flop per cycle
// per CU, 157 Tflop/s on the part).  K advances 16 at a time through double-buffered LDS tiles
// stored k-major ([k][m] and [k][n], pitch 132 floats) so that a fragment read is 32 consecutive
// floats per half-wave and the transposing store of a k-contiguous operand spreads over all banks.
// The global loads of tile t+1 are issued before the MFMA loop of tile t and land in LDS after it:
// one barrier per K tile.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.h"
#include "ctx.h"
#include "math.h"

namespace altius {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int PITCH = BM + 4;  // floats; (4k + m) mod 64 is a bijection over a transposing store's lanes
constexpr int THREADS = 256;

struct GemmArgs {
    const float *a, *b, *c0;
    float *c;
    uint32_t m, n, k;
    // Element (i, kk) of op(A) is a[i * a_rs + kk * a_cs]; (kk, j) of op(B) is b[kk * b_rs + j * b_cs].
    // One of the two strides of each operand is 1.
    uint32_t a_rs, a_cs, b_rs, b_cs;
    uint32_t ldc;
    // C0 (Gemm's third input) is read as c0[i * c0_rs + j * c0_cs]; either stride may be 0.
    uint32_t c0_rs, c0_cs;
    // Batch z = blockIdx.z is (z / batch_inner, z % batch_inner); operand X starts at
    // x + (z / batch_inner) * x_bs + (z % batch_inner) * x_bs2 (strides in elements, 0 = shared).
    uint64_t a_bs, b_bs, c_bs, a_bs2, b_bs2, c_bs2;
    uint32_t batch_inner;
    // Single-batch launches are one-dimensional: consecutive block ids go to the eight XCDs in turn, and
    // each XCD (one L2) is given a contiguous run of tiles, so the blocks it runs together share panels.
    // Within that order tiles go by groups of group_n tile columns, each group walked row of tiles by row of tiles,
    // so that the blocks an XCD runs together cover few columns of B (they stay in its L2) and many rows of A.
    uint32_t tiles_n, tiles_m, tiles, chunk, group_n;  // chunk = 0: the grid is (n tiles, m tiles, batches)
    float alpha, beta;
    int a_vec, b_vec;  // 16-byte loads are legal for this operand (alignment of base, strides, batch stride)
};

__device__ __forceinline__ float post_ops(float v, int act, const float *__restrict__ residual, size_t at) {
    if (act == AHIP_GELU) v = dev::gelu_elem(v);
    else if (act == AHIP_RELU) v = dev::relu_elem(v);
    if (residual) v = v + residual[at];
    return v;
}

// Loads this thread's share of a BK x 128 operand tile into registers.
// K_CONTIG: the operand's k axis is the contiguous one (A without transA, B with transB).
// `mn` is the tile's first row (A) or column (B), `lim` the extent of that axis.
// INSIDE: 16-byte loads are legal, the K tile is whole, and an operand whose mn axis is the contiguous one
// has an extent that is a multiple of 4 (decided per block and K tile, a scalar branch): no per-lane bounds
// checks, edge tiles clamp their addresses instead.
template <bool K_CONTIG, int WIDTH, bool INSIDE>
__device__ __forceinline__ void load_tile(float4 (&r)[WIDTH / 64], const float *__restrict__ p, uint32_t mn0, uint32_t lim,
                                          uint32_t k0, uint32_t kdim, uint32_t s_mn, uint32_t s_k, int vec, int tid) {
#pragma unroll
    for (int u = 0; u < WIDTH / 64; u++) {
        const int f = tid + THREADS * u;
        uint32_t mn, kk;
        if (K_CONTIG) {  // WIDTH rows of 16 floats: 4 float4 per row
            mn = mn0 + (f >> 2);
            kk = k0 + ((f & 3) << 2);
        } else {  // 16 rows of WIDTH floats: WIDTH / 4 float4 per row
            kk = k0 + f / (WIDTH / 4);
            mn = mn0 + ((f % (WIDTH / 4)) << 2);
        }
        if (INSIDE) {
            // Rows (or float4 columns) past the operand's edge re-read its last one: in bounds, and what they
            // contribute only reaches elements of C that are never stored.
            const uint32_t last = K_CONTIG ? lim - 1 : (lim - 4) & ~3u;
            if (mn > last) mn = last;
            r[u] = *reinterpret_cast<const float4 *>(K_CONTIG ? p + (size_t)mn * s_mn + kk : p + (size_t)kk * s_k + mn);
            continue;
        }
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (K_CONTIG) {
            if (mn < lim) {
                const float *q = p + (size_t)mn * s_mn + kk;
                if (vec && kk + 3 < kdim) {
                    v = *reinterpret_cast<const float4 *>(q);
                } else {
                    if (kk < kdim) v.x = q[0];
                    if (kk + 1 < kdim) v.y = q[1];
                    if (kk + 2 < kdim) v.z = q[2];
                    if (kk + 3 < kdim) v.w = q[3];
                }
            }
        } else {
            if (kk < kdim) {
                const float *q = p + (size_t)kk * s_k + mn;
                if (vec && mn + 3 < lim) {
                    v = *reinterpret_cast<const float4 *>(q);
                } else {
                    if (mn < lim) v.x = q[0];
                    if (mn + 1 < lim) v.y = q[1];
                    if (mn + 2 < lim) v.z = q[2];
                    if (mn + 3 < lim) v.w = q[3];
                }
            }
        }
        r[u] = v;
    }
}

// Stores the registers into the k-major LDS tile [BK][PITCH].
template <bool K_CONTIG, int WIDTH>
__device__ __forceinline__ void store_tile(float *__restrict__ t, const float4 (&r)[WIDTH / 64], int tid) {
#pragma unroll
    for (int u = 0; u < WIDTH / 64; u++) {
        const int f = tid + THREADS * u;
        if (K_CONTIG) {
            const int mn = f >> 2, kk = (f & 3) << 2;
            t[(kk + 0) * PITCH + mn] = r[u].x;
            t[(kk + 1) * PITCH + mn] = r[u].y;
            t[(kk + 2) * PITCH + mn] = r[u].z;
            t[(kk + 3) * PITCH + mn] = r[u].w;
        } else {
            const int kk = f / (WIDTH / 4), mn = (f % (WIDTH / 4)) << 2;
            *reinterpret_cast<float4 *>(t + kk * PITCH + mn) = r[u];
        }
    }
}

// TN = 128: wavefronts in a 2 x 2 grid, 64 x 64 each.  TN = 64 (narrow outputs such as attention's
// P x V with 64 columns): wavefronts stacked 4 x 1, 32 x 64 each.
template <bool A_KC, bool B_KC, int TN>
__global__ __launch_bounds__(THREADS) void gemm_f32_mfma(GemmArgs g) {
    constexpr int WI = TN == 128 ? 2 : 1;  // 32-row MFMA tiles per wavefront
    __shared__ __align__(16) float As[2][BK * PITCH];
    __shared__ __align__(16) float Bs[2][BK * PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = TN == 128 ? wave >> 1 : wave, wn = TN == 128 ? wave & 1 : 0;
    uint32_t tile_m = blockIdx.y, tile_n = blockIdx.x;
    if (g.chunk) {
        const uint32_t tile = (blockIdx.x & 7) * g.chunk + (blockIdx.x >> 3);
        if (tile >= g.tiles) return;
        const uint32_t per_group = g.tiles_m * g.group_n, grp = tile / per_group, r = tile - grp * per_group;
        const uint32_t width = min(g.group_n, g.tiles_n - grp * g.group_n);  // the last group may be narrower
        tile_m = r / width, tile_n = grp * g.group_n + r % width;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * TN;
    const uint32_t zo = blockIdx.z / g.batch_inner, zi = blockIdx.z % g.batch_inner;
    const float *a = g.a + (size_t)zo * g.a_bs + (size_t)zi * g.a_bs2;
    const float *b = g.b + (size_t)zo * g.b_bs + (size_t)zi * g.b_bs2;
    // Strides of the tile's mn axis and k axis for each operand.
    const uint32_t a_smn = g.a_rs, a_sk = g.a_cs, b_smn = g.b_cs, b_sk = g.b_rs;

    floatx16 acc[WI][2];
#pragma unroll
    for (int i = 0; i < WI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Operands that allow 16-byte loads everywhere run a loop without any bounds check on all K tiles but a
    // ragged last one (edge tiles clamp their addresses); the choice is a scalar branch around the whole
    // loop, so the loop is straight-line code between its barriers.
    const bool inside = g.a_vec && g.b_vec && (A_KC || (g.m & 3) == 0) && (B_KC || (g.n & 3) == 0);
    const int lr = lane & 31, lk = lane >> 5;
    auto main_loop = [&](auto inside_tag) {
        constexpr bool INSIDE = decltype(inside_tag)::value;
        float4 ra[BM / 64], rb[TN / 64];
        auto load = [&](uint32_t k0) {
            if (INSIDE && k0 + BK <= g.k) {
                load_tile<A_KC, BM, true>(ra, a, m0, g.m, k0, g.k, a_smn, a_sk, 1, tid);
                load_tile<B_KC, TN, true>(rb, b, n0, g.n, k0, g.k, b_smn, b_sk, 1, tid);
            } else {
                load_tile<A_KC, BM, false>(ra, a, m0, g.m, k0, g.k, a_smn, a_sk, g.a_vec, tid);
                load_tile<B_KC, TN, false>(rb, b, n0, g.n, k0, g.k, b_smn, b_sk, g.b_vec, tid);
            }
        };
        load(0);
        store_tile<A_KC, BM>(As[0], ra, tid);
        store_tile<B_KC, TN>(Bs[0], rb, tid);
        __syncthreads();

        const uint32_t nk = (g.k + BK - 1) / BK;
        for (uint32_t kt = 0; kt < nk; kt++) {
            const int cur = kt & 1;
            const bool more = kt + 1 < nk;
            if (more) load((kt + 1) * BK);
            const float *at = As[cur] + wm * (32 * WI) + lr;
            const float *bt = Bs[cur] + wn * 64 + lr;
#pragma unroll
            for (int kk = 0; kk < BK; kk += 2) {
                float av[WI];
#pragma unroll
                for (int i = 0; i < WI; i++) av[i] = at[(kk + lk) * PITCH + 32 * i];
                const float b0 = bt[(kk + lk) * PITCH], b1 = bt[(kk + lk) * PITCH + 32];
#pragma unroll
                for (int i = 0; i < WI; i++) {
                    acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], b0, acc[i][0], 0, 0, 0);
                    acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], b1, acc[i][1], 0, 0, 0);
                }
            }
            if (more) {
                store_tile<A_KC, BM>(As[cur ^ 1], ra, tid);
                store_tile<B_KC, TN>(Bs[cur ^ 1], rb, tid);
            }
            __syncthreads();
        }
    };
    if (inside) main_loop(std::true_type{});
    else main_loop(std::false_type{});

    // Accumulator r of lane l is C[8 * (r / 4) + 4 * (l / 32) + r % 4][l % 32] of its 32 x 32 tile.
    float *c = g.c + (size_t)zo * g.c_bs + (size_t)zi * g.c_bs2;
#pragma unroll
    for (int i = 0; i < WI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t col = n0 + wn * 64 + j * 32 + lr;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t row = m0 + wm * (32 * WI) + i * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                if (row < g.m && col < g.n) {
                    float v = g.alpha * acc[i][j][r];
                    if (g.c0) v += g.beta * g.c0[(size_t)row * g.c0_rs + (size_t)col * g.c0_cs];
                    c[(size_t)row * g.ldc + col] = v;
                }
            }
        }
}

// C = alpha * (sum over k slices, in slice order) + beta * C0: the second half of a product cut along k.
__global__ __launch_bounds__(256) void splitk_finish(float *__restrict__ c, const float *__restrict__ partials, uint32_t slices,
                                                     uint32_t m, uint32_t n, uint32_t ldc, const float *__restrict__ c0, uint32_t c0_rs,
                                                     uint32_t c0_cs, float alpha, float beta, int act,
                                                     const float *__restrict__ residual) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, total = (size_t)m * n;
    if (i >= total) return;
    float sum = partials[i];
    for (uint32_t s = 1; s < slices; s++) sum += partials[(size_t)s * total + i];
    const uint32_t row = (uint32_t)(i / n), col = (uint32_t)(i % n);
    float v = alpha * sum;
    if (c0) v += beta * c0[(size_t)row * c0_rs + (size_t)col * c0_cs];
    c[(size_t)row * ldc + col] = post_ops(v, act, residual, (size_t)row * ldc + col);
}

// c = act(c) + residual in place, for products that were not cut along k (their kernel's epilogue stays free of it:
// sixty-four inlined activations per thread slowed every launch down).
__global__ __launch_bounds__(256) void post_in_place(float *__restrict__ c, uint32_t m, uint32_t n, uint32_t ldc, int act,
                                                     const float *__restrict__ residual) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)m * n) return;
    const size_t at = (i / n) * ldc + i % n;
    c[at] = post_ops(c[at], act, residual, at);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

thread_local int split_k_inner = 0;  // the batched launch of the slices must not cut again (1), and keeps the tile width chosen for the whole product (2: the narrow one)

}  // namespace

bool gemm_takes_split(const DeviceCtx &ctx, size_t m, size_t n, size_t k) {
    return k > 0 && (ctx.gemm_algorithm == AHIP_GEMM_BF16X3 || (ctx.gemm_algorithm == AHIP_GEMM_AUTO && gemm_split_worthwhile(m, n, k)));
}

int launch_gemm(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t batch, size_t m, size_t n,
                size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t a_batch_stride,
                size_t b_batch_stride, size_t c_batch_stride, size_t c0_row_stride, size_t c0_col_stride, float alpha,
                float beta) {
    const size_t a_bs[2] = {a_batch_stride, 0}, b_bs[2] = {b_batch_stride, 0}, c_bs[2] = {c_batch_stride, 0};
    return launch_gemm_batch2(ctx, c, a, b, c0, batch, 1, m, n, k, trans_a, trans_b, lda, ldb, ldc, a_bs, b_bs, c_bs, c0_row_stride,
                              c0_col_stride, alpha, beta);
}

int launch_gemm_batch2(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t batch_outer,
                       size_t batch_inner, size_t m, size_t n, size_t k, int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc,
                       const size_t a_batch_strides[2], const size_t b_batch_strides[2], const size_t c_batch_strides[2],
                       size_t c0_row_stride, size_t c0_col_stride, float alpha, float beta, const GemmPost *post) {
    const size_t batch = batch_outer * batch_inner;
    if (batch == 0 || m == 0 || n == 0) return AHIP_OK;
    if (!c || (k && (!a || !b))) return ctx.fail(AHIP_ERR_ARG, "gemm: null pointer");
    const bool has_post = post && (post->act != 0 || post->residual);
    if (has_post && batch != 1) return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm: an activation or a residual needs a single batch");
    if (has_post && post->act != 0 && post->act != AHIP_GELU && post->act != AHIP_RELU)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm: only Gelu and Relu can follow the product in its kernel");
    if (!has_post && batch == 1 && gemm_takes_split(ctx, m, n, k))
        return launch_gemm_split(ctx, c, a, b, c0, m, n, k, trans_a, trans_b, lda, ldb, ldc, c0_row_stride, c0_col_stride, alpha, beta);
    const size_t lim = (size_t)1 << 31;
    if (m >= lim || n >= lim || k >= lim || lda >= lim || ldb >= lim || ldc >= lim || m * ldc >= ((size_t)1 << 40))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm: extent above 2^31");
    // Hundreds of small matrices (attention's two products per head): one block per matrix.
    // (its fetchers address a head's operand with 32-bit byte offsets: 2^29 floats per head at most)
    const size_t a_extent = (m - 1) * lda + k, b_extent = trans_b ? (n - 1) * ldb + k : (k ? k - 1 : 0) * ldb + n;
    if (!has_post && !trans_a && alpha == 1.0f && (!c0 || beta == 0.0f) && !split_k_inner && gemm_small_batched_fits(batch, m, n, k) &&
        a_extent < ((size_t)1 << 29) && b_extent < ((size_t)1 << 29))
        return launch_gemm_small_batched(ctx, c, a, b, batch_outer, batch_inner, m, n, k, trans_b, lda, ldb, ldc, a_batch_strides, b_batch_strides,
                                         c_batch_strides);
    // The 128 x 64 tile when it leaves fewer idle columns (n = 64: 64 instead of 128 computed), and for long
    // K loops: with half the accumulators per wavefront more blocks fit a CU and the last round of blocks
    // is fuller (measured at [50432,3072]x[3072,768]: 120.9 against 110.3 TFLOP/s; the wide tile stays ahead
    // only where K is short and the tile's fixed costs weigh more, as in attention's 64-deep products).
    // ... and when the wide tile would leave CUs without a block (the slices of a product cut along k).
    const size_t cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256;
    const bool narrow = split_k_inner ? split_k_inner == 2
                                      : n <= 64 || (n < 512 && n % 128 != 0 && n % 128 <= 64) || k >= 256 ||
                                            ((m + BM - 1) / BM) * ((n + BN - 1) / BN) * batch < cus;
    const size_t tn = narrow ? 64 : BN;
    const size_t gy = (m + BM - 1) / BM, gx = (n + tn - 1) / tn;
    if (gy > 65535 || batch > 65535) return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm: more than 65535 row tiles or batches");
    // A single product with few tiles and a long k (one image through a transformer layer) leaves most CUs idle
    // while each block walks all of k: cut k into slices that run as batches into a workspace, and add the
    // slices up in order afterwards (the bias and alpha / beta go there).
    if (batch == 1 && ctx.gemm_split_k && gx * gy <= cus && k >= 512 && !split_k_inner) {
        size_t slices = std::min<size_t>(std::min<size_t>((2 * cus + gx * gy - 1) / (gx * gy), k / 128), 16);
        while (slices > 1 && k % (slices * 16) != 0) slices--;  // equal slices of whole k tiles
        if (slices >= 2) {
            void *ws = nullptr;
            int rc = gemm_workspace(ctx, slices * m * n * sizeof(float), &ws);
            if (rc) return rc;
            const size_t ks = k / slices;
            // slice z of op(A) starts ks columns (or rows, transposed) further on; likewise op(B)
            const size_t a_bs[2] = {trans_a ? ks * lda : ks, 0}, b_bs[2] = {trans_b ? ks : ks * ldb, 0}, c_bs[2] = {m * n, 0};
            split_k_inner = narrow ? 2 : 1;
            rc = launch_gemm_batch2(ctx, static_cast<float *>(ws), a, b, nullptr, slices, 1, m, n, ks, trans_a, trans_b, lda, ldb, n, a_bs, b_bs,
                                    c_bs, 0, 0, 1.0f, 0.0f);
            split_k_inner = 0;
            if (rc) return rc;
            const size_t total = m * n;
            hipLaunchKernelGGL(splitk_finish, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx.stream, c, static_cast<const float *>(ws),
                               (uint32_t)slices, (uint32_t)m, (uint32_t)n, (uint32_t)ldc, (c0 && beta != 0.0f) ? c0 : nullptr,
                               (uint32_t)c0_row_stride, (uint32_t)c0_col_stride, alpha, beta, has_post ? post->act : 0,
                               has_post ? post->residual : nullptr);
            return ctx.check(hipGetLastError(), "gemm split-k finish launch");
        }
    }
    GemmArgs g;
    g.a = a;
    g.b = b;
    g.c0 = (c0 && beta != 0.0f) ? c0 : nullptr;
    g.c = c;
    g.m = (uint32_t)m;
    g.n = (uint32_t)n;
    g.k = (uint32_t)k;
    g.a_rs = trans_a ? 1u : (uint32_t)lda;
    g.a_cs = trans_a ? (uint32_t)lda : 1u;
    g.b_rs = trans_b ? 1u : (uint32_t)ldb;
    g.b_cs = trans_b ? (uint32_t)ldb : 1u;
    g.ldc = (uint32_t)ldc;
    g.c0_rs = (uint32_t)c0_row_stride;
    g.c0_cs = (uint32_t)c0_col_stride;
    g.a_bs = a_batch_strides[0];
    g.b_bs = b_batch_strides[0];
    g.c_bs = c_batch_strides[0];
    g.a_bs2 = a_batch_strides[1];
    g.b_bs2 = b_batch_strides[1];
    g.c_bs2 = c_batch_strides[1];
    g.batch_inner = (uint32_t)batch_inner;
    g.alpha = alpha;
    g.beta = beta;
    g.a_vec = aligned16(a) && lda % 4 == 0 && a_batch_strides[0] % 4 == 0 && a_batch_strides[1] % 4 == 0;
    g.b_vec = aligned16(b) && ldb % 4 == 0 && b_batch_strides[0] % 4 == 0 && b_batch_strides[1] % 4 == 0;
    g.tiles_n = (uint32_t)gx;
    g.tiles_m = (uint32_t)gy;
    g.tiles = (uint32_t)(gx * gy);
    {
        // Groups of about 768 columns (measured on [50432,768]x[768,2304..3072] and 4096^3 .. 8192^3: widths of
        // 6 to 16 tile columns are within 1 % of each other and up to 3 % ahead of whole rows of tiles; a single
        // column is 3-6 % behind), all groups equally wide.
        const size_t group = std::max<size_t>(1, 768 / tn), groups = (gx + group - 1) / group;
        g.group_n = (uint32_t)((gx + groups - 1) / groups);
    }
    g.chunk = batch == 1 && gx * gy >= 64 && gx * gy < lim / 8 ? (uint32_t)((gx * gy + 7) / 8) : 0;
    const dim3 grid = g.chunk ? dim3(g.chunk * 8) : dim3((unsigned)gx, (unsigned)gy, (unsigned)batch);
    const bool a_kc = !trans_a, b_kc = trans_b != 0;
#define GEMM(AK, BK_, TN_) hipLaunchKernelGGL((gemm_f32_mfma<AK, BK_, TN_>), grid, dim3(THREADS), 0, ctx.stream, g)
    if (narrow) {
        if (a_kc && b_kc) GEMM(true, true, 64);
        else if (a_kc) GEMM(true, false, 64);
        else if (b_kc) GEMM(false, true, 64);
        else GEMM(false, false, 64);
    } else {
        if (a_kc && b_kc) GEMM(true, true, 128);
        else if (a_kc) GEMM(true, false, 128);
        else if (b_kc) GEMM(false, true, 128);
        else GEMM(false, false, 128);
    }
#undef GEMM
    if (has_post)
        hipLaunchKernelGGL(post_in_place, dim3((unsigned)((m * n + 255) / 256)), dim3(256), 0, ctx.stream, c, (uint32_t)m, (uint32_t)n,
                           (uint32_t)ldc, post->act, post->residual);
    return ctx.check(hipGetLastError(), "gemm launch");
}

}  // namespace altius
