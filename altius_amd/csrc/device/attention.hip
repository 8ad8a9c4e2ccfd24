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
#include "split3.h"

namespace altius {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = 64;          // head width
constexpr int K_PITCH = 68;    // floats; 16-byte aligned rows whose b128 reads by 8 consecutive rows cover all banks
constexpr int MAX_WAVES = 8;   // query tiles per block

typedef uint32_t u32x4_attn __attribute__((ext_vector_type(4)));

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
    // attention_stream_d64_bf16<.., PLANES>: O, a [batch_outer * tq, batch_inner * 64] matrix, leaves as the three bf16
    // planes of the first operand of the product that reads it ([plane][k / 8][row][8], o_rp rows, o_kgs k groups).
    u32x4_attn *o_planes;
    uint32_t o_rp, o_kgs;
};

constexpr int KC = 64;  // keys per chunk

// One tile of 32 keys for a wavefront's 32 queries: scores S^T = K tile x Q^T, the running maximum and sum
// brought up to date (what was accumulated is rescaled when the maximum rises), then O^T += V tile^T x P^T.
// ktile / vtile: the tile's first row in LDS (pitches K_PITCH and D); key_base: its first key's index.
__device__ __forceinline__ void attend_tile(int scale_op, float scale, uint32_t tk, const float *__restrict__ mask, const float *ktile,
                                            const float *vtile, uint32_t key_base, const float (&qf)[32], int h, int lr, float &mx,
                                            float &sum, floatx16 (&acc)[2]) {
    floatx16 st;
#pragma unroll
    for (int r = 0; r < 16; r++) st[r] = 0.0f;
    const float *kr = ktile + lr * K_PITCH + 32 * h;
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
        const uint32_t key = key_base + 8 * (r >> 2) + 4 * h + (r & 3);
        float x = st[r];
        if (scale_op == 1) x = x * scale;
        else if (scale_op == 2) x = x / scale;
        if (mask && key < tk) x = x + mask[key];
        st[r] = x;
        if (key < tk) cmax = dev::nanmax(cmax, x);
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
        const uint32_t key = key_base + 8 * (r >> 2) + 4 * h + (r & 3);
        const float e = key < tk ? dev::softmax_exp(st[r], mx) : 0.0f;
        st[r] = e;
        sum += e;
    }
#pragma unroll
    for (int kk = 0; kk < 16; kk++) {
        const int key = 8 * (kk >> 2) + 4 * h + (kk & 3);
        const float v0 = vtile[key * D + lr], v1 = vtile[key * D + 32 + lr];
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(v0, st[kk], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(v1, st[kk], acc[1], 0, 0, 0);
    }
}

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
                attend_tile(g.scale_op, g.scale, g.tk, mask, &ks[buf][32 * j * K_PITCH], &vs[buf][32 * j * D], key0 + 32 * j, qf, h, lr, mx, sum, acc);
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

// ---------------------------------------------------------------- the same on the bf16 matrix cores
// Both products with every fp32 operand value as the exact sum of three bf16 numbers and six
// v_mfma_f32_32x32x16_bf16 per k step (the scheme of gemm_split.hip): 48 MFMAs of 8 passes per tile of 32 keys
// instead of 64 fp32 MFMAs of 16 passes.  K and V are split once per block on their way into LDS, Q once per
// wavefront into registers; the probabilities are split where they are, in the accumulator registers of S^T, whose
// layout is again the B operand's: half-wave h supplies the 8 k slots of a 16-key step from accumulator registers
// 8 u .. 8 u + 7, i.e. keys 16 u + 8 (i / 4) + 4 h + i % 4, and V^T is laid out in LDS in that key order.
// Keys go through LDS 32 at a time, double-buffered: 57 KiB, two blocks per CU.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int KCB = 32;       // keys per chunk (one tile)
constexpr int KB_PITCH = 72;  // 16-bit words per K row in LDS: 64 d and a pad that spreads 16-byte reads of 16 rows over all banks
constexpr int VB_PITCH = 40;  // 16-bit words per V^T row (one d): 32 key slots and a pad, likewise

#define ALTIUS_MFMA_BF16(A, B, C) \
    C = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A), __builtin_bit_cast(bf16x8, B), C, 0, 0, 0)

// Smallest terms first.
__device__ __forceinline__ void six_products(const u32x4 (&a)[3], const u32x4 &b0, const u32x4 &b1, const u32x4 &b2, floatx16 &c) {
    ALTIUS_MFMA_BF16(a[0], b2, c);
    ALTIUS_MFMA_BF16(a[2], b0, c);
    ALTIUS_MFMA_BF16(a[1], b1, c);
    ALTIUS_MFMA_BF16(a[0], b1, c);
    ALTIUS_MFMA_BF16(a[1], b0, c);
    ALTIUS_MFMA_BF16(a[0], b0, c);
}

// Two probabilities (in [0, 1]: no rounding up to infinity, no NaN payloads to keep) as three pairs of bf16.
__device__ __forceinline__ void split_pair(float e0, float e1, uint32_t &p0, uint32_t &p1, uint32_t &p2) {
    p0 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){e0, e1}, bf16x2));
    const float r0 = e0 - __uint_as_float(p0 << 16), r1 = e1 - __uint_as_float(p0 & 0xffff0000u);
    p1 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){r0, r1}, bf16x2));
    const float s0 = r0 - __uint_as_float(p1 << 16), s1 = r1 - __uint_as_float(p1 & 0xffff0000u);
    p2 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){s0, s1}, bf16x2));
}

// FULL: every key of the tile exists.  SCALE_OP and MASK are the launch's, so that the sixteen scores of a lane go
// through straight-line code.
template <bool FULL, int SCALE_OP, bool MASK>
__device__ __forceinline__ void attend_tile_bf16(float scale, uint32_t tk, const float *__restrict__ mask, const uint16_t *kp,
                                                 const uint16_t *vp, uint32_t key_base, const u32x4 (&qp)[3][4], int h, int lr, float &mx,
                                                 float &sum, floatx16 (&acc)[2]) {
    floatx16 st;
#pragma unroll
    for (int r = 0; r < 16; r++) st[r] = 0.0f;
#pragma unroll
    for (int s = 0; s < 4; s++) {
        u32x4 kf[3];
#pragma unroll
        for (int p = 0; p < 3; p++) kf[p] = *reinterpret_cast<const u32x4 *>(kp + p * (KCB * KB_PITCH) + lr * KB_PITCH + 16 * s + 8 * h);
        six_products(kf, qp[0][s], qp[1][s], qp[2][s], st);
    }
    float cmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const uint32_t key = key_base + 8 * (r >> 2) + 4 * h + (r & 3);
        float x = st[r];
        if (SCALE_OP == 1) x = x * scale;
        else if (SCALE_OP == 2) x = x / scale;
        if (MASK && (FULL || key < tk)) x = x + mask[key];
        st[r] = x;
        if (FULL || key < tk) cmax = dev::nanmax(cmax, x);
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
        const uint32_t key = key_base + 8 * (r >> 2) + 4 * h + (r & 3);
        const float e = (FULL || key < tk) ? dev::softmax_exp(st[r], mx) : 0.0f;
        st[r] = e;
        sum += e;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        u32x4 pf[3];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t p0, p1, p2;
            split_pair(st[8 * u + 2 * i], st[8 * u + 2 * i + 1], p0, p1, p2);
            pf[0][i] = p0, pf[1][i] = p1, pf[2][i] = p2;
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
            u32x4 vf[3];
#pragma unroll
            for (int p = 0; p < 3; p++)
                vf[p] = *reinterpret_cast<const u32x4 *>(vp + p * (D * VB_PITCH) + (32 * t + lr) * VB_PITCH + (2 * u + h) * 8);
            six_products(vf, pf[0], pf[1], pf[2], acc[t]);
        }
    }
}

template <int SCALE_OP, bool MASK, bool PLANES>
__global__ __launch_bounds__(512, 2) void attention_stream_d64_bf16(AttnArgs g) {
    constexpr int W = 8;
    __shared__ __align__(16) uint16_t kps[2][3 * KCB * KB_PITCH];
    __shared__ __align__(16) uint16_t vps[2][3 * D * VB_PITCH];
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
    const uint32_t nchunks = (g.tk + KCB - 1) / KCB;

    // Staging: thread (key r0, float4 c4) moves one float4 of K and one of V per chunk.
    const uint32_t r0 = tid >> 4, c4 = tid & 15;
    // Where key r0 sits in a V^T row: group (u, h) of 8 slots, slot i within it (see above).
    const uint32_t vslot = ((r0 >> 4) * 2 + ((r0 & 7) >> 2)) * 8 + 4 * ((r0 & 15) >> 3) + (r0 & 3);
    f32x4 kst, vst;
    auto fetch = [&](uint32_t chunk) {
        const uint32_t row = chunk * KCB + r0;
        kst = vst = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (row < g.tk) {
            kst = *reinterpret_cast<const f32x4 *>(k + (size_t)row * g.ldk + c4 * 4);
            vst = *reinterpret_cast<const f32x4 *>(v + (size_t)row * g.ldv + c4 * 4);
        }
    };
    auto park = [&](int buf) {
        uint32_t hk[3][2], hv[3][2];
#pragma unroll
        for (int e = 0; e < 2; e++) {
            dev::split3_pair(kst[2 * e], kst[2 * e + 1], hk[0][e], hk[1][e], hk[2][e]);
            dev::split3_pair(vst[2 * e], vst[2 * e + 1], hv[0][e], hv[1][e], hv[2][e]);
        }
#pragma unroll
        for (int p = 0; p < 3; p++) {
            *reinterpret_cast<u32x2 *>(&kps[buf][p * (KCB * KB_PITCH) + r0 * KB_PITCH + 4 * c4]) = u32x2{hk[p][0], hk[p][1]};
#pragma unroll
            for (int e = 0; e < 4; e++)
                vps[buf][p * (D * VB_PITCH) + (4 * c4 + e) * VB_PITCH + vslot] = (uint16_t)(e & 1 ? hv[p][e >> 1] >> 16 : hv[p][e >> 1]);
        }
    };
    fetch(0);
    park(0);

    u32x4 qp[3][4];
    if (active && query < g.tq) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const float *src = q + (size_t)query * g.ldq + 16 * s + 8 * h;
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(src), hi = *reinterpret_cast<const f32x4 *>(src + 4);
            uint32_t hq[3][4];
#pragma unroll
            for (int e = 0; e < 2; e++) {
                dev::split3_pair(lo[2 * e], lo[2 * e + 1], hq[0][e], hq[1][e], hq[2][e]);
                dev::split3_pair(hi[2 * e], hi[2 * e + 1], hq[0][2 + e], hq[1][2 + e], hq[2][2 + e]);
            }
#pragma unroll
            for (int p = 0; p < 3; p++) qp[p][s] = u32x4{hq[p][0], hq[p][1], hq[p][2], hq[p][3]};
        }
    } else {
#pragma unroll
        for (int p = 0; p < 3; p++)
#pragma unroll
            for (int s = 0; s < 4; s++) qp[p][s] = u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    float mx = -INFINITY, sum = 0.0f;
    floatx16 acc[2];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[0][r] = 0.0f, acc[1][r] = 0.0f;

    for (uint32_t c = 0; c < nchunks; c++) {
        const int buf = c & 1;
        const bool more = c + 1 < nchunks;
        if (more) fetch(c + 1);  // in flight during the tile
        if (active) {
            if ((c + 1) * KCB <= g.tk) attend_tile_bf16<true, SCALE_OP, MASK>(g.scale, g.tk, mask, kps[buf], vps[buf], c * KCB, qp, h, lr, mx, sum, acc);
            else attend_tile_bf16<false, SCALE_OP, MASK>(g.scale, g.tk, mask, kps[buf], vps[buf], c * KCB, qp, h, lr, mx, sum, acc);
        }
        if (more) park(buf ^ 1);
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
                if (PLANES) {
                    // The lane's four values are half h of the 16-byte chunk (row zo tq + query, k group 8 zi + 4 t + g4).
                    uint32_t lo[3], hi[3];
                    dev::split3_pair(out[0], out[1], lo[0], lo[1], lo[2]);
                    dev::split3_pair(out[2], out[3], hi[0], hi[1], hi[2]);
                    const size_t row = (size_t)zo * g.tq + query, kg = (size_t)zi * 8 + 4 * t + g4;
#pragma unroll
                    for (int p = 0; p < 3; p++)
                        reinterpret_cast<u32x2 *>(g.o_planes + ((size_t)p * g.o_kgs + kg) * g.o_rp + row)[h] = u32x2{lo[p], hi[p]};
                } else {
                    *reinterpret_cast<f32x4 *>(o + (size_t)query * g.ldo + 32 * t + 8 * g4 + 4 * h) = out;
                }
            }
    }
}

// The same for few (batch, head) pairs, where a wavefront walking all keys alone is the whole run time: a block
// of SW wavefronts owns ONE tile of 32 queries and deals the key tiles out among its wavefronts (tile t of a
// chunk of 32 SW keys goes to wavefront t).  Each keeps its own running maximum, sum and O^T; at the end the
// partial results meet in LDS and wavefront 0 combines them, every part scaled by exp(its maximum - the overall
// one), exactly the rescaling the streaming kernel applies when its maximum rises.
constexpr int SW = 4;
constexpr int SC = 32 * SW;  // keys per chunk

__global__ __launch_bounds__(64 * SW, 1) void attention_keysplit_d64(AttnArgs g) {
    __shared__ __align__(16) float ks[SC * K_PITCH];
    __shared__ __align__(16) float vs[SC * D];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, lr = lane & 31;
    const uint32_t zo = blockIdx.x / g.batch_inner, zi = blockIdx.x % g.batch_inner;
    const float *q = g.q + zo * g.q_bs[0] + zi * g.q_bs[1];
    const float *k = g.k + zo * g.k_bs[0] + zi * g.k_bs[1];
    const float *v = g.v + zo * g.v_bs[0] + zi * g.v_bs[1];
    float *o = g.o + zo * g.o_bs[0] + zi * g.o_bs[1];
    const float *mask = g.mask ? g.mask + (size_t)zo * g.mask_outer_stride : nullptr;
    const uint32_t query = blockIdx.y * 32 + lr;
    const uint32_t nchunks = (g.tk + SC - 1) / SC;

    // Staging: 256 threads move 16 rows of 16 float4 per pass, 8 passes per operand and chunk.
    constexpr int PASSES = SC / 16;
    const uint32_t r0 = tid >> 4, c4 = tid & 15;
    f32x4 kst[PASSES], vst[PASSES];
    auto fetch = [&](f32x4 (&st)[PASSES], const float *base, uint32_t ld, uint32_t chunk) {
#pragma unroll
        for (int it = 0; it < PASSES; it++) {
            const uint32_t row = chunk * SC + it * 16 + r0;
            st[it] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (row < g.tk) st[it] = *reinterpret_cast<const f32x4 *>(base + (size_t)row * ld + c4 * 4);
        }
    };
    auto park = [&](const f32x4 (&st)[PASSES], float *dst, int pitch) {
#pragma unroll
        for (int it = 0; it < PASSES; it++) *reinterpret_cast<f32x4 *>(dst + (it * 16 + r0) * pitch + c4 * 4) = st[it];
    };
    fetch(kst, k, g.ldk, 0);
    fetch(vst, v, g.ldv, 0);
    float qf[32];
    if (query < g.tq) {
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const f32x4 t = *reinterpret_cast<const f32x4 *>(q + (size_t)query * g.ldq + 32 * h + 4 * c);
            qf[4 * c] = t.x, qf[4 * c + 1] = t.y, qf[4 * c + 2] = t.z, qf[4 * c + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int c = 0; c < 32; c++) qf[c] = 0.0f;
    }
    park(kst, ks, K_PITCH);
    park(vst, vs, D);
    __syncthreads();

    float mx = -INFINITY, sum = 0.0f;
    floatx16 acc[2];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[0][r] = 0.0f, acc[1][r] = 0.0f;

    for (uint32_t c = 0; c < nchunks; c++) {
        const bool more = c + 1 < nchunks;
        if (more) {  // in flight during this chunk's products
            fetch(kst, k, g.ldk, c + 1);
            fetch(vst, v, g.ldv, c + 1);
        }
        const uint32_t key_base = c * SC + 32 * wave;
        if (key_base < g.tk) attend_tile(g.scale_op, g.scale, g.tk, mask, &ks[32 * wave * K_PITCH], &vs[32 * wave * D], key_base, qf, h, lr, mx, sum, acc);
        __syncthreads();  // nobody reads this chunk any more
        if (more) {
            park(kst, ks, K_PITCH);
            park(vst, vs, D);
            __syncthreads();
        }
    }

    // Partial results meet in LDS (the staging area is free now): per wavefront 64 lanes x 32 accumulators, laid
    // out [register][lane] so that every access is a row of consecutive floats, then maximum and sum per query.
    sum += __shfl_xor(sum, 32);
    float *part = ks;                      // [SW][32][64]
    float *stat = vs;                      // [SW][2][32]
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) part[(wave * 32 + 16 * t + r) * 64 + lane] = acc[t][r];
        if (h == 0) stat[(wave * 2) * 32 + lr] = mx, stat[(wave * 2 + 1) * 32 + lr] = sum;
    }
    __syncthreads();
    if (wave == 0 && query < g.tq) {
        float top = mx;
#pragma unroll
        for (int w = 1; w < SW; w++) top = dev::nanmax(top, stat[(w * 2) * 32 + lr]);
        const float own = mx == -INFINITY ? 0.0f : dev::softmax_exp(mx, top);
        float total = sum * own;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[0][r] *= own, acc[1][r] *= own;
#pragma unroll
        for (int w = 1; w < SW; w++) {
            const float m = stat[(w * 2) * 32 + lr];
            const float f = m == -INFINITY ? 0.0f : dev::softmax_exp(m, top);
            total += stat[(w * 2 + 1) * 32 + lr] * f;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[t][r] += part[(w * 32 + 16 * t + r) * 64 + lane] * f;
        }
        const float recip = 1.0f / total;
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

// Whether launch_attention would run the kernel that can write O as operand planes: enough (batch, head) pairs for full
// blocks on a context whose products may take the bf16 route.
bool attention_writes_planes(const DeviceCtx &ctx, size_t batch_outer, size_t batch_inner, size_t tq) {
    const size_t q_tiles = (tq + 31) / 32, cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256, batch = batch_outer * batch_inner;
    return ctx.gemm_algorithm != AHIP_GEMM_FP32 && tq > 0 && batch * ((q_tiles + 7) / 8) >= cus && batch * q_tiles >= 2 * cus &&
           batch_outer * tq < ((size_t)1 << 31) - 256;
}

int launch_attention(DeviceCtx &ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer, size_t batch_inner,
                     size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo, const size_t q_bs[2],
                     const size_t k_bs[2], const size_t v_bs[2], const size_t o_bs[2], int scale_op, float scale, const float *mask,
                     size_t mask_outer_stride, void *o_planes) {
    const size_t batch = batch_outer * batch_inner;
    if (batch == 0 || tq == 0) return AHIP_OK;
    if ((!o && !o_planes) || !q || !k || !v) return ctx.fail(AHIP_ERR_ARG, "attention: null pointer");
    if (o_planes && !attention_writes_planes(ctx, batch_outer, batch_inner, tq))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: operand planes are written by the bf16 kernel on full blocks only");
    if (scale_op < 0 || scale_op > 2) return ctx.fail(AHIP_ERR_ARG, "attention: scale_op must be 0, 1 or 2");
    if (d != (size_t)D || tk == 0) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: needs 64-wide heads and at least one key");
    const size_t lim = (size_t)1 << 31;
    if (mask_outer_stride >= lim) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: mask stride above 2^31");
    if (tq >= lim || tk >= lim || ldq >= lim || ldk >= lim || ldv >= lim || ldo >= lim || batch >= lim)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: extent above 2^31");
    auto vec_ok = [](const void *p, size_t ld, const size_t bs[2]) { return aligned16(p) && ld % 4 == 0 && bs[0] % 4 == 0 && bs[1] % 4 == 0; };
    if (!vec_ok(q, ldq, q_bs) || !vec_ok(k, ldk, k_bs) || !vec_ok(v, ldv, v_bs) || (!o_planes && !vec_ok(o, ldo, o_bs)))
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
    g.o_planes = static_cast<u32x4_attn *>(o_planes);
    g.o_rp = (uint32_t)((batch_outer * tq + 255) / 256 * 256);
    g.o_kgs = (uint32_t)(batch_inner * 8);
    const size_t q_tiles = (tq + 31) / 32, cus = ctx.cus_per_xcd ? (size_t)ctx.cus_per_xcd * 8 : 256;
    if (q_tiles > 65535) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: too many queries");
    if (batch * q_tiles < 2 * cus) {
        // One query tile per block would still leave the GPU thin: the keys are split over a block's wavefronts
        // as well (ViT-B/16 at batch 1: 84 tiles; measured faster up to about two tiles per CU).
        hipLaunchKernelGGL(attention_keysplit_d64, dim3((unsigned)batch, (unsigned)q_tiles), dim3(64 * SW), 0, ctx.stream, g);
        return ctx.check(hipGetLastError(), "attention launch");
    }
    // As many query tiles per block as still leave a block for most CUs.
    size_t w = MAX_WAVES;
    while (w > 2 && batch * ((q_tiles + w - 1) / w) < cus) w /= 2;
    const dim3 grid((unsigned)batch, (unsigned)((q_tiles + w - 1) / w));
    // Where products may take the bf16 matrix cores (an infinite operand then gives NaN, as in the GEMM on that
    // route), full blocks do.
    if (w == 8 && ctx.gemm_algorithm != AHIP_GEMM_FP32) {
#define ALTIUS_ATT(S, M)                                                                                             \
    do {                                                                                                             \
        if (o_planes) hipLaunchKernelGGL((attention_stream_d64_bf16<S, M, true>), grid, dim3(512), 0, ctx.stream, g);  \
        else hipLaunchKernelGGL((attention_stream_d64_bf16<S, M, false>), grid, dim3(512), 0, ctx.stream, g);         \
    } while (0)
        if (mask) {
            if (scale_op == 0) ALTIUS_ATT(0, true);
            else if (scale_op == 1) ALTIUS_ATT(1, true);
            else ALTIUS_ATT(2, true);
        } else {
            if (scale_op == 0) ALTIUS_ATT(0, false);
            else if (scale_op == 1) ALTIUS_ATT(1, false);
            else ALTIUS_ATT(2, false);
        }
#undef ALTIUS_ATT
    } else if (w == 8) hipLaunchKernelGGL(attention_stream_d64<8>, grid, dim3(512), 0, ctx.stream, g);
    else if (w == 4) hipLaunchKernelGGL(attention_stream_d64<4>, grid, dim3(256), 0, ctx.stream, g);
    else hipLaunchKernelGGL(attention_stream_d64<2>, grid, dim3(128), 0, ctx.stream, g);
    return ctx.check(hipGetLastError(), "attention launch");
}

}  // namespace altius
