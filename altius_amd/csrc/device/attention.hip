// Attention for one (batch, head) per block, without the score tensor ever reaching memory:
//   O = Softmax(scale(Q K^T) + mask) V,   Q [tq, 64], K [tk, 64], V [tk, 64], tk <= 256, mask one value per key,
// the three operators compute_mat_mul -> compute_softmax -> compute_mat_mul of the reference
// (crates/session_interpreter/src/session.rs:621-684, 990-1026) on the fp32 matrix cores, with the
// reference's own exp (fast_math.rs:130-150, dev::softmax_exp) and its reciprocal-multiply
// normalisation.
//
// Both products are computed transposed, which keeps everything between them in registers.
// S^T = K Q^T: a wavefront owns 32 queries; for each tile of 32 keys it accumulates a 32 x 32 block
// whose accumulator register r of lane l is S[query l % 32][key 8 (r / 4) + 4 (l / 32) + r % 4].
// A lane therefore holds one query's scores for half of the keys, and a row maximum or sum is an
// in-lane reduction plus one exchange with lane l ^ 32.  O^T = V^T P^T then takes the probabilities
// as the B operand exactly where they already are: the k slot of MFMA step kk in half-wave h is
// simply declared to be key 8 (kk / 4) + 4 h + kk % 4, and V is read from LDS in that order.
// K and V are both staged in LDS up front (one barrier): afterwards the wavefronts of a block run free of each
// other, so one wavefront's softmax arithmetic overlaps another's MFMAs on the same SIMD.
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

template <int NT>
__global__ __launch_bounds__(64 * MAX_WAVES) void attention_d64(AttnArgs g) {
    __shared__ __align__(16) float ks[NT * 32 * K_PITCH];
    __shared__ __align__(16) float vs[NT * 32 * D];
    __shared__ volatile int qk_done[MAX_WAVES / 2];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, lr = lane & 31;
    const uint32_t zo = blockIdx.x / g.batch_inner, zi = blockIdx.x % g.batch_inner;
    const float *q = g.q + zo * g.q_bs[0] + zi * g.q_bs[1];
    const float *k = g.k + zo * g.k_bs[0] + zi * g.k_bs[1];
    const float *v = g.v + zo * g.v_bs[0] + zi * g.v_bs[1];
    float *o = g.o + zo * g.o_bs[0] + zi * g.o_bs[1];
    const uint32_t query = (blockIdx.y * MAX_WAVES + wave) * 32 + lr;

    // K and V -> LDS, rows past tk zero.  The block always has 512 threads: 32 rows of 16 float4 per pass, all
    // 2 NT loads of a thread in flight before the first store.
    {
        f32x4 kreg[NT], vreg[NT];
        const uint32_t r0 = tid >> 4, c4 = tid & 15;
#pragma unroll
        for (int it = 0; it < NT; it++) {
            const uint32_t row = it * 32 + r0;
            kreg[it] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            vreg[it] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (row < g.tk) {
                kreg[it] = *reinterpret_cast<const f32x4 *>(k + (size_t)row * g.ldk + c4 * 4);
                vreg[it] = *reinterpret_cast<const f32x4 *>(v + (size_t)row * g.ldv + c4 * 4);
            }
        }
#pragma unroll
        for (int it = 0; it < NT; it++) {
            const uint32_t row = it * 32 + r0;
            *reinterpret_cast<f32x4 *>(&ks[row * K_PITCH + c4 * 4]) = kreg[it];
            *reinterpret_cast<f32x4 *>(&vs[row * D + c4 * 4]) = vreg[it];
        }
    }
    // This lane's half of its query's row: d = 32 h + kk.
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
    if (tid < MAX_WAVES / 2) qk_done[tid] = 0;
    __syncthreads();

    if ((blockIdx.y * MAX_WAVES + wave) * 32 >= g.tq) return;  // helped with the staging; no queries of its own

    // Wavefronts w and w + 4 share a SIMD.  The second one holds back until the first has issued its score
    // products, so that from then on one of them is in its softmax arithmetic (VALU) while the other is in a
    // product (MFMA).  Only a scheduling hint: the wait is bounded and nothing depends on it.
    if (wave >= MAX_WAVES / 2) {
        for (int spin = 0; spin < (1 << 16) && qk_done[wave - MAX_WAVES / 2] == 0; spin++) __builtin_amdgcn_s_sleep(16);
    }

    floatx16 s[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[j][r] = 0.0f;
        const float *kr = &ks[(32 * j + lr) * K_PITCH + 32 * h];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const f32x4 kf = *reinterpret_cast<const f32x4 *>(kr + 4 * c);
            s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.x, qf[4 * c], s[j], 0, 0, 0);
            s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.y, qf[4 * c + 1], s[j], 0, 0, 0);
            s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.z, qf[4 * c + 2], s[j], 0, 0, 0);
            s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf.w, qf[4 * c + 3], s[j], 0, 0, 0);
        }
    }

    if (wave < MAX_WAVES / 2 && lane == 0) qk_done[wave] = 1;

    // Softmax over the keys of this lane's query: scale, maximum (NaNs ignored, as the reference's fold does),
    // exp, sum, one reciprocal.  Keys past tk take no part.
    const float *mask = g.mask ? g.mask + (size_t)zo * g.mask_outer_stride : nullptr;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = 32 * j + 8 * (r >> 2) + 4 * h + (r & 3);
            float x = s[j][r];
            if (g.scale_op == 1) x = x * g.scale;
            else if (g.scale_op == 2) x = x / g.scale;
            if (mask && key < g.tk) x = x + mask[key];
            s[j][r] = x;
            if (key < g.tk) mx = dev::nanmax(mx, x);
        }
    mx = dev::nanmax(mx, __shfl_xor(mx, 32));
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = 32 * j + 8 * (r >> 2) + 4 * h + (r & 3);
            const float e = key < g.tk ? dev::softmax_exp(s[j][r], mx) : 0.0f;
            s[j][r] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 32);
    const float recip = 1.0f / sum;
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[j][r] *= recip;

    floatx16 acc[2];
#pragma unroll
    for (int r = 0; r < 16; r++) acc[0][r] = 0.0f, acc[1][r] = 0.0f;
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
            const int key = 32 * j + 8 * (kk >> 2) + 4 * h + (kk & 3);
            const float v0 = vs[key * D + lr], v1 = vs[key * D + 32 + lr];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(v0, s[j][kk], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(v1, s[j][kk], acc[1], 0, 0, 0);
        }

    // acc[t][r] is O[query][32 t + 8 (r / 4) + 4 h + r % 4]: four consecutive d per group of registers.
    if (query < g.tq) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const f32x4 out = {acc[t][4 * g4], acc[t][4 * g4 + 1], acc[t][4 * g4 + 2], acc[t][4 * g4 + 3]};
                *reinterpret_cast<f32x4 *>(o + (size_t)query * g.ldo + 32 * t + 8 * g4 + 4 * h) = out;
            }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int NT>
void launch_nt(DeviceCtx &ctx, const AttnArgs &g, dim3 grid, unsigned threads) {
    hipLaunchKernelGGL(attention_d64<NT>, grid, dim3(threads), 0, ctx.stream, g);
}

}  // namespace

int launch_attention(DeviceCtx &ctx, float *o, const float *q, const float *k, const float *v, size_t batch_outer, size_t batch_inner,
                     size_t tq, size_t tk, size_t d, size_t ldq, size_t ldk, size_t ldv, size_t ldo, const size_t q_bs[2],
                     const size_t k_bs[2], const size_t v_bs[2], const size_t o_bs[2], int scale_op, float scale, const float *mask,
                     size_t mask_outer_stride) {
    const size_t batch = batch_outer * batch_inner;
    if (batch == 0 || tq == 0) return AHIP_OK;
    if (!o || !q || !k || !v) return ctx.fail(AHIP_ERR_ARG, "attention: null pointer");
    if (scale_op < 0 || scale_op > 2) return ctx.fail(AHIP_ERR_ARG, "attention: scale_op must be 0, 1 or 2");
    if (d != (size_t)D || tk == 0 || tk > 256) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: needs 64-wide heads and 1..256 keys");
    const size_t lim = (size_t)1 << 31;
    if (mask_outer_stride >= lim) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: mask stride above 2^31");
    if (tq >= lim || ldq >= lim || ldk >= lim || ldv >= lim || ldo >= lim || batch >= lim)
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
    const size_t q_tiles = (tq + 31) / 32;
    const size_t gy = (q_tiles + MAX_WAVES - 1) / MAX_WAVES;
    if (gy > 65535) return ctx.fail(AHIP_ERR_UNSUPPORTED, "attention: too many queries");
    const unsigned threads = 64 * MAX_WAVES;
    const dim3 grid((unsigned)batch, (unsigned)gy);
    switch ((tk + 31) / 32) {
    case 1: launch_nt<1>(ctx, g, grid, threads); break;
    case 2: launch_nt<2>(ctx, g, grid, threads); break;
    case 3: launch_nt<3>(ctx, g, grid, threads); break;
    case 4: launch_nt<4>(ctx, g, grid, threads); break;
    case 5: launch_nt<5>(ctx, g, grid, threads); break;
    case 6: launch_nt<6>(ctx, g, grid, threads); break;
    case 7: launch_nt<7>(ctx, g, grid, threads); break;
    default: launch_nt<8>(ctx, g, grid, threads); break;
    }
    return ctx.check(hipGetLastError(), "attention launch");
}

}  // namespace altius
