// Attention for one (batch, head) per block, without the score tensor ever reaching memory:
//   O = Softmax(scale(Q K^T) + mask) V,   Q [tq, 64], K [tk, 64], V [tk, 64], mask one value per key,
// the three operators compute_mat_mul -> compute_softmax -> compute_mat_mul of the reference
// (crates/session_interpreter/src/session.rs:621-684, 990-1026) on the fp32 matrix cores, with the
// reference's own exp (fast_math.rs:130-150, dev::softmax_exp).
//
// Both products are computed transposed, which keeps everything between them in registers.
// S^T = K Q^T: a wavefront owns 32 queries; for a tile of 32 keys it accumulates a 32 x 32 block whose
// accumulator register r of lane l is S[query l % 32][key 8 (r / 4) + 4 (l / 32) + r % 4].  A lane therefore
// holds one query's scores for half of the keys, and a row maximum or sum is an in-lane reduction plus one
// exchange with lane l ^ 32.  O^T = V^T P^T then takes the probabilities as the B operand exactly where they
// already are: the k slot of MFMA step kk in half-wave h is simply declared to be key 8 (kk / 4) + 4 h + kk % 4,
// and V is read from LDS in that order.
//
// Keys are streamed through LDS 64 at a time (double-buffered; the next chunk's loads are in flight during
// the products) with a running maximum and sum per query: when a later tile raises the maximum, what has
// been accumulated is rescaled by exp(old - new).  Any number of keys; 66 KiB of LDS and 128 registers, so
// two blocks share a CU and one block's staging and stores overlap the other's products.  O is normalised at
// the end (acc * 1/sum) rather than P before the second product.  A first version that kept all scores of a
// query in registers (at most 256 keys, K and V whole in 118 KB of LDS, one block per CU) took 533 us where
// this one takes 450 us (3072 heads of 197 x 64): its staging, products and stores could only add up.
#include <hip/hip_runtime.h>

#include "common.h"
#include "ctx.h"
#include "math.h"

namespace altius {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = 64;          // head width
constexpr int K_PITCH = 68;    // floats; 16-byte aligned rows whose b128 reads by 8 consecutive rows cover all banks
constexpr int MAX_WAVES = 8;   // query tiles per block

struct AttnArgs {
    const float *q, *k, *v;
    float *o;
    uint32_t tq, tk;
    uint32_t ldq, ldk, ldv, ldo;  // row pitches in elements
    // Batch z is (z / batch_inner, z % batch_inner): operand x of it starts at x + zo * x_bs[0] + zi * x_bs[1].
    uint64_t q_bs[2], k_bs[2], v_bs[2], o_bs[2];
    uint32_t batch_inner;
    int scale_op;  // 0 none, 1 scores * scale, 2 scores / scale
    float scale;
    // Added to the scaled scores, one value per key: mask[(z / batch_inner) * mask_outer_stride + key] (null: none).
    const float *mask;
    uint32_t mask_outer_stride;
};

constexpr int KC = 64;  // keys per chunk

// W: wavefronts (tiles of 32 queries) per block.  Fewer when there are few (batch, head) pairs, so that the queries of
// one pair spread over several CUs; every block stages the keys and values it needs itself.
template <int W>
__global__ __launch_bounds__(64 * W, W == 8 ? 4 : 1) void attention_stream_d64(AttnArgs g) {
    __shared__ __align__(16) float ks[2][KC * K_PITCH];
    __shared__ __align__(16) float vs[2][KC * D];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, lr = lane & 31;
    const uint32_t zo = blockIdx.x / g.batch_inner, zi = blockIdx.x % g.batch_inner;
    const float *q = g.q + zo * g.q_bs[0] + zi * g.q_bs[1];
    const float *k = g.k + zo * g.k_bs[0] + zi * g.k_bs[1];
    const float *v = g.v + zo * g.v_bs[0] + zi * g.v_bs[1];
    float *o = g.o + zo * g.o_bs[0] + zi * g.o_bs[1];
    const float *mask = g.mask ? g.mask + (size_t)zo * g.mask_outer_stride : nullptr;
    const uint32_t query = (blockIdx.y * W + wave) * 32 + lr;
    const bool active = (blockIdx.y * W + wave) * 32 < g.tq;  // wavefronts without queries still help staging
    const uint32_t nchunks = (g.tk + KC - 1) / KC;

    // Staging: the block's threads move 4 W rows of 16 float4 per pass, 16 / W passes per operand and chunk.
    constexpr int PASSES = 16 / W, ROWS = 4 * W;
    const uint32_t r0 = tid >> 4, c4 = tid & 15;
    f32x4 stage[PASSES];
    auto fetch = [&](const float *base, uint32_t ld, uint32_t chunk) {
#pragma unroll
        for (int it = 0; it < PASSES; it++) {
            const uint32_t row = chunk * KC + it * ROWS + r0;
            stage[it] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (row < g.tk) stage[it] = *reinterpret_cast<const f32x4 *>(base + (size_t)row * ld + c4 * 4);
        }
    };
    auto park = [&](float *dst, int pitch) {
#pragma unroll
        for (int it = 0; it < PASSES; it++) *reinterpret_cast<f32x4 *>(dst + (it * ROWS + r0) * pitch + c4 * 4) = stage[it];
    };
    fetch(k, g.ldk, 0);
    park(ks[0], K_PITCH);
    fetch(v, g.ldv, 0);
    park(vs[0], D);

    float qf[32];
    if (active && query < g.tq) {
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const f32x4 t = *reinterpret_cast<const f32x4 *>(q + (size_t)query * g.ldq + 32 * h + 4 * c);
            qf[4 * c] = t.x, qf[4 * c + 1] = t.y, qf[4 * c + 2] = t.z, qf[4 * c + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int c = 0; c < 32; c++) qf[c] = 0.0f;
    }
    __syncthreads();

    float mx = -INFINITY, sum = 0.0f;
    floatx16 acc[2];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[0][r] = 0.0f, acc[1][r] = 0.0f;

    for (uint32_t c = 0; c < nchunks; c++) {
        const int buf = c & 1;
        const bool more = c + 1 < nchunks;
        const uint32_t key0 = c * KC;
        const int tiles = g.tk - key0 > 32 ? 2 : 1;
        if (more) fetch(k, g.ldk, c + 1);  // in flight during the first tile
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (active && j < tiles) {
                // Scores of 32 keys: S^T tile = K tile x Q^T.
                floatx16 st;
#pragma unroll
                for (int r = 0; r < 16; r++) st[r] = 0.0f;
                const float *kr = &ks[buf][(32 * j + lr) * K_PITCH + 32 * h];
#pragma unroll
                for (int cc = 0; cc < 8; cc++) {
                    const f32x4 kf = *reinterpret_cast<const f32x4 *>(kr + 4 * cc);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.x, qf[4 * cc], st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.y, qf[4 * cc + 1], st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.z, qf[4 * cc + 2], st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.w, qf[4 * cc + 3], st, 0, 0, 0);
                }
                float cmax = -INFINITY;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const uint32_t key = key0 + 32 * j + 8 * (r >> 2) + 4 * h + (r & 3);
                    float x = st[r];
                    if (g.scale_op == 1) x = x * g.scale;
                    else if (g.scale_op == 2) x = x / g.scale;
                    if (mask && key < g.tk) x = x + mask[key];
                    st[r] = x;
                    if (key < g.tk) cmax = dev::nanmax(cmax, x);
                }
                cmax = dev::nanmax(cmax, __shfl_xor(cmax, 32));
                const float mnew = dev::nanmax(mx, cmax);
                if (mnew != mx) {  // what has been summed so far was taken relative to the old maximum
                    const float corr = mx == -INFINITY ? 0.0f : dev::softmax_exp(mx, mnew);
                    sum *= corr;
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[0][r] *= corr, acc[1][r] *= corr;
                    mx = mnew;
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const uint32_t key = key0 + 32 * j + 8 * (r >> 2) + 4 * h + (r & 3);
                    const float e = key < g.tk ? dev::softmax_exp(st[r], mx) : 0.0f;
                    st[r] = e;
                    sum += e;
                }
#pragma unroll
                for (int kk = 0; kk < 16; kk++) {
                    const int key = 32 * j + 8 * (kk >> 2) + 4 * h + (kk & 3);
                    const float v0 = vs[buf][key * D + lr], v1 = vs[buf][key * D + 32 + lr];
                    acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(v0, st[kk], acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(v1, st[kk], acc[1], 0, 0, 0);
                }
            }
            if (j == 0 && more) {
                park(ks[buf ^ 1], K_PITCH);
                fetch(v, g.ldv, c + 1);  // in flight during the second tile
            }
        }
        if (more) park(vs[buf ^ 1], D);
        __syncthreads();  // the next chunk is in place, and nobody reads this one any more
    }

    if (active && query < g.tq) {
        sum += __shfl_xor(sum, 32);
        const float recip = 1.0f / sum;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const f32x4 out = {acc[t][4 * g4] * recip, acc[t][4 * g4 + 1] * recip, acc[t][4 * g4 + 2] * recip, acc[t][4 * g4 + 3] * recip};
                *reinterpret_cast<f32x4 *>(o + (size_t)query * g.ldo + 32 * t + 8 * g4 + 4 * h) = out;
            }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

int launch_attention(DeviceCtx &ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer, size_t batch_inner,
                     size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo, const size_t q_bs[2],
                     const size_t k_bs[2], const size_t v_bs[2], const size_t o_bs[2], int scale_op, float scale, const float *mask,
                     size_t mask_outer_stride) {
    const size_t batch = batch_outer * batch_inner;
    if (batch == 0 || tq == 0) return AHIP_OK;
    if (!o || !q || !k || !v) return ctx.fail(AHIP_ERR_ARG, "attention: null pointer");
    if (scale_op < 0 || scale_op > 2) return ctx.fail(AHIP_ERR_ARG, "attention: scale_op must be 0, 1 or 2");
    if (d != (size_t)D || tk == 0) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: needs 64-wide heads and at least one key");
    const size_t lim = (size_t)1 << 31;
    if (mask_outer_stride >= lim) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: mask stride above 2^31");
    if (tq >= lim || tk >= lim || ldq >= lim || ldk >= lim || ldv >= lim || ldo >= lim || batch >= lim)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: extent above 2^31");
    auto vec_ok = [](const void *p, size_t ld, const size_t bs[2]) { return aligned16(p) && ld % 4 == 0 && bs[0] % 4 == 0 && bs[1] % 4 == 0; };
    if (!vec_ok(q, ldq, q_bs) || !vec_ok(k, ldk, k_bs) || !vec_ok(v, ldv, v_bs) || !vec_ok(o, ldo, o_bs))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: operands must be 16-byte aligned with pitches that are multiples of 4");
    if (ldq < (size_t)D || ldk < (size_t)D || ldv < (size_t)D || ldo < (size_t)D)
        return ctx.fail(AHIP_ERR_ARG, "attention: a row pitch is below the head width");
    AttnArgs g;
    g.q = q, g.k = k, g.v = v, g.o = o;
    g.tq = (uint32_t)tq, g.tk = (uint32_t)tk;
    g.ldq = (uint32_t)ldq, g.ldk = (uint32_t)ldk, g.ldv = (uint32_t)ldv, g.ldo = (uint32_t)ldo;
    for (int i = 0; i < 2; i++) g.q_bs[i] = q_bs[i], g.k_bs[i] = k_bs[i], g.v_bs[i] = v_bs[i], g.o_bs[i] = o_bs[i];
    g.batch_inner = (uint32_t)batch_inner;
    g.scale_op = scale_op;
    g.scale = scale;
    g.mask = mask;
    g.mask_outer_stride = (uint32_t)mask_outer_stride;
    // As many query tiles per block as still leave a block for most CUs.
    const size_t q_tiles = (tq + 31) / 32, cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256;
    size_t w = MAX_WAVES;
    while (w > 1 && batch * ((q_tiles + w - 1) / w) < cus) w /= 2;
    const size_t gy = (q_tiles + w - 1) / w;
    if (gy > 65535) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: too many queries");
    const dim3 grid((unsigned)batch, (unsigned)gy);
    if (w == 8) hipLaunchKernelGGL(attention_stream_d64<8>, grid, dim3(512), 0, ctx.stream, g);
    else if (w == 4) hipLaunchKernelGGL(attention_stream_d64<4>, grid, dim3(256), 0, ctx.stream, g);
    else if (w == 2) hipLaunchKernelGGL(attention_stream_d64<2>, grid, dim3(128), 0, ctx.stream, g);
    else hipLaunchKernelGGL(attention_stream_d64<1>, grid, dim3(64), 0, ctx.stream, g);
    return ctx.check(hipGetLastError(), "attention launch");
}

}  // namespace altius
