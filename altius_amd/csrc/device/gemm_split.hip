// fp32 matrix multiplication on the bf16 matrix cores: every fp32 operand value x is written as
// x = h0 + h1 + h2 with three bf16 numbers (8 + 8 + 8 significand bits: the sum is exact), and
//   a * b = a0 b0 + (a0 b1 + a1 b0) + (a0 b2 + a1 b1 + a2 b0) + [a1 b2 + a2 b1 + a2 b2]
// is accumulated in fp32 by six v_mfma_f32_32x32x16_bf16 per tile and k step; the bracket, below
// 2^-23 |a b| with random signs, is dropped.  Against a float64 product the result is as close as
// a chain of fp32 fused multiply-adds (the reference's sgemm, crates/session_interpreter/src/gemm.rs:3-52,
// called by compute_mat_mul and compute_gemm, session.rs:621-794), and six bf16 MFMAs cost 6 / 16 of
// one fp32 MFMA per product.
//
// Two kernels.  split_planes turns an operand into three planes stored [plane][k / 8][row][8]
// (16-byte chunks: 8 consecutive k of one row), rows and k padded with zeros to whole tiles, so
// that both the GEMM's global reads and its LDS layout are plain contiguous copies.  gemm_bf16x3
// computes a 256 x 256 tile of C per 512-thread block (8 wavefronts, 64 x 128 each) in k steps of
// 16 through three LDS buffers that are filled by direct global->LDS loads issued two steps ahead;
// one barrier per step, with the block's two groups of four wavefronts half a step apart (a SIMD's two
// wavefronts take turns at the matrix pipe).  The epilogue transposes the accumulators through LDS so that
// C is written in whole 512-byte row segments.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.h"
#include "ctx.h"
#include "math.h"
#include "split3.h"

namespace altius {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- operand -> three bf16 planes

using dev::split3_pair;

// An activation applied to the operand's values on their way into the planes (PRE: 0 none, else an AHIP_* unary
// code): the product reads f(A) without f(A) ever being stored as fp32.
template <int PRE>
__device__ __forceinline__ float pre(float x) {
    if (PRE == AHIP_GELU) return dev::gelu_elem(x);
    if (PRE == AHIP_RELU) return dev::relu_elem(x);
    return x;
}

__device__ __forceinline__ void store_planes(u32x4 *__restrict__ planes, const float (&v)[8], uint32_t row, uint32_t kg, uint32_t rp,
                                             uint32_t kgs) {
    uint32_t h[3][4];
#pragma unroll
    for (int j = 0; j < 4; j++) split3_pair(v[2 * j], v[2 * j + 1], h[0][j], h[1][j], h[2][j]);
#pragma unroll
    for (int p = 0; p < 3; p++) planes[((size_t)p * kgs + kg) * rp + row] = u32x4{h[p][0], h[p][1], h[p][2], h[p][3]};
}

// Any strides: element (row, k) is src[row * s_r + k * s_k].  Consecutive lanes take consecutive rows,
// which is the contiguous direction of an operand stored k-major (A transposed, B as given).
template <int PRE>
__global__ __launch_bounds__(256) void split_planes(const float *__restrict__ src, u32x4 *__restrict__ planes, uint32_t rows, uint32_t k,
                                                    size_t s_r, size_t s_k, uint32_t rp, uint32_t kgs) {
    const uint32_t row = blockIdx.x * 64 + (threadIdx.x & 63);
    const uint32_t kg = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (kg >= kgs) return;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t kk = kg * 8 + j;
        v[j] = (row < rows && kk < k) ? pre<PRE>(src[(size_t)row * s_r + (size_t)kk * s_k]) : 0.0f;
    }
    store_planes(planes, v, row, kg, rp, kgs);
}

// Rows contiguous in k and 16-byte aligned: four adjacent lanes read 128 contiguous bytes of a row,
// sixteen rows per wavefront; each (plane, k group) store of a wavefront is 256 contiguous bytes.
template <int PRE>
__global__ __launch_bounds__(256) void split_planes_rows(const float *__restrict__ src, u32x4 *__restrict__ planes, uint32_t rows,
                                                         uint32_t k, size_t s_r, uint32_t rp, uint32_t kgs, int k_fastest) {
    const uint32_t row = (k_fastest ? blockIdx.y : blockIdx.x) * 64 + (threadIdx.x >> 2);
    const uint32_t kg = (k_fastest ? blockIdx.x : blockIdx.y) * 4 + (threadIdx.x & 3);
    if (kg >= kgs) return;
    float v[8];
    const uint32_t k0 = kg * 8;
    if (row < rows && k0 + 8 <= k) {
        const f32x4 lo = *reinterpret_cast<const f32x4 *>(src + (size_t)row * s_r + k0);
        const f32x4 hi = *reinterpret_cast<const f32x4 *>(src + (size_t)row * s_r + k0 + 4);
        v[0] = pre<PRE>(lo.x), v[1] = pre<PRE>(lo.y), v[2] = pre<PRE>(lo.z), v[3] = pre<PRE>(lo.w);
        v[4] = pre<PRE>(hi.x), v[5] = pre<PRE>(hi.y), v[6] = pre<PRE>(hi.z), v[7] = pre<PRE>(hi.w);
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (row < rows && k0 + j < k) ? pre<PRE>(src[(size_t)row * s_r + k0 + j]) : 0.0f;
    }
    store_planes(planes, v, row, kg, rp, kgs);
}

// ---------------------------------------------------------------- LayerNormalization straight into planes
// LayerNormalization over the last axis (crates/session_interpreter/src/session.rs:1433-1486) whose only reader is
// the first operand of a product on this route: the normalised rows are written as that operand's planes and never
// as fp32 (232 MB instead of 155 MB written, and the 155 MB + 232 MB of the operand split saved, on [50432, 768]).
// A block of sixteen wavefronts takes sixteen rows, a wavefront per row with the row in registers: lane l holds
// float4 l, l + 64, ... and the additions run in the order of the stand-alone wavefront-per-row kernel
// (layernorm_wave in rows.hip), so mean, variance and every output value have its bits.  A lane's four values are
// half of a 16-byte chunk of each plane; the halves go to LDS as [plane][k group][row], and from there the block
// stores 256 contiguous bytes (sixteen rows of one k group) at a time.  ADD: the rows are a + b (a residual
// connection); the sum is also stored as fp32 for its other readers.
constexpr int LNP_ROWS = 16, LNP_THREADS = 1024;
constexpr int LNP_KG_PITCH = LNP_ROWS * 4 + 4;  // 32-bit words per k group in LDS: sixteen 16-byte chunks and a pad

template <int NCH, bool ADD>
__global__ __launch_bounds__(LNP_THREADS) void layernorm_planes(u32x4 *__restrict__ planes, float *__restrict__ sum_out,
                                                                const float *__restrict__ in, const float *__restrict__ in2,
                                                                const float *__restrict__ gamma, const float *__restrict__ beta, uint32_t rows,
                                                                uint32_t len, float eps, uint32_t rp, uint32_t kgs) {
    extern __shared__ __align__(16) uint32_t lnp_lds[];  // [3][kgs][LNP_KG_PITCH]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t row0 = blockIdx.x * LNP_ROWS, grow = row0 + wave;
    const uint32_t v4 = len / 4;  // float4 per row
    float v[NCH * 4];
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const uint32_t c = lane + 64 * k;
        f32x4 t = {0.0f, 0.0f, 0.0f, 0.0f};
        if (grow < rows && c < v4) {
            const size_t off = (size_t)grow * len + 4 * c;
            t = *reinterpret_cast<const f32x4 *>(in + off);
            if (ADD) {
                const f32x4 u = *reinterpret_cast<const f32x4 *>(in2 + off);
                t = f32x4{t.x + u.x, t.y + u.y, t.z + u.z, t.w + u.w};
                *reinterpret_cast<f32x4 *>(sum_out + off) = t;
            }
        }
        v[4 * k] = t.x, v[4 * k + 1] = t.y, v[4 * k + 2] = t.z, v[4 * k + 3] = t.w;
    }
    const float inv_n = 1.0f / (float)len;
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < NCH * 4; s++) sum += v[s];
    const float mean = dev::wave_reduce<dev::SumOp>(sum) * inv_n;
    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < NCH * 4; s++) {
        const bool valid = (uint32_t)(lane + 64 * (s / 4)) < v4;
        v[s] = v[s] - mean;
        ss += valid ? v[s] * v[s] : 0.0f;
    }
    ss = dev::wave_reduce<dev::SumOp>(ss);
    const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));
    // this lane's half chunks of the three planes -> LDS
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const uint32_t c = lane + 64 * k;  // float4 number: k group c / 2, half c % 2
        if (c < 2 * kgs) {
            uint32_t h[3][2];
            float y[4];
            const bool live = grow < rows && c < v4;
            f32x4 gm = {0.0f, 0.0f, 0.0f, 0.0f}, bt = {0.0f, 0.0f, 0.0f, 0.0f};
            if (live) gm = *reinterpret_cast<const f32x4 *>(gamma + 4 * c), bt = *reinterpret_cast<const f32x4 *>(beta + 4 * c);
            const float g4[4] = {gm.x, gm.y, gm.z, gm.w}, b4[4] = {bt.x, bt.y, bt.z, bt.w};
#pragma unroll
            for (int j = 0; j < 4; j++) y[j] = live ? __builtin_fmaf(v[4 * k + j] * inv_std, g4[j], b4[j]) : 0.0f;
            split3_pair(y[0], y[1], h[0][0], h[1][0], h[2][0]);
            split3_pair(y[2], y[3], h[0][1], h[1][1], h[2][1]);
#pragma unroll
            for (int p = 0; p < 3; p++) {
                uint32_t *dst = lnp_lds + ((size_t)p * kgs + (c >> 1)) * LNP_KG_PITCH + wave * 4 + (c & 1) * 2;
                dst[0] = h[p][0];
                dst[1] = h[p][1];
            }
        }
    }
    __syncthreads();
    // LDS -> planes: consecutive threads take consecutive rows of one (plane, k group): 256 contiguous bytes
    const uint32_t chunks = 3 * kgs * LNP_ROWS;
    for (uint32_t i = tid; i < chunks; i += LNP_THREADS) {
        const uint32_t r = i & (LNP_ROWS - 1), pk = i / LNP_ROWS;  // pk = plane * kgs + k group
        const u32x4 o = *reinterpret_cast<const u32x4 *>(lnp_lds + (size_t)pk * LNP_KG_PITCH + r * 4);
        planes[(size_t)pk * rp + row0 + r] = o;
    }
}

// ---------------------------------------------------------------- the product

constexpr int TM = 256, TN = 256, THREADS = 512;
constexpr size_t GEMM_COUNTERS = 256;  // tiles cut along k per launch: at most 8 XCDs x 31

// One k step of 16 (two k groups of 8) of both operand tiles.
struct Stage {
    u32x4 a[3][2][TM];
    u32x4 b[3][2][TN];
};
constexpr uint32_t PLANE_BYTES = 2 * 256 * 16;  // distance between two planes of one operand inside a Stage
static_assert(sizeof(Stage) == 6 * PLANE_BYTES, "Stage layout");

struct SplitGemmArgs {
    const u32x4 *ap, *bp;  // planes of op(A) (rows = m) and of op(B) transposed (rows = n)
    float *c;
    const float *c0;
    uint32_t m, n, mp, np, kgs, ldc;
    uint32_t c0_rs, c0_cs;
    float alpha, beta;
    uint32_t tiles_n, tiles, chunk;
    // Each XCD's run of `chunk` tiles: the first `full` are whole tiles (one block each); each of the rest is
    // computed by `sf` blocks over `sf` slices of k, whose partial sums meet in `partials` (see the kernel).
    uint32_t full, sf;
    float *partials;
    int *counters;
    int *misplaced;  // raised when the slices of a tile did not all run on one XCD
    int c_vec;    // 16-byte stores into C are aligned
    int c_stream;  // C is large: write it with non-temporal stores
};

typedef __attribute__((address_space(3))) void *lds_ptr;
typedef const __attribute__((address_space(1))) void *global_ptr;

// Wavefront w fills rows [64 (w & 3), +64) of k group (w >> 2) of all three planes of both operands:
// six loads of 1 KiB, each lane's 16 bytes landing at consecutive LDS addresses.
__device__ __forceinline__ void issue(Stage &s, const u32x4 *ga, const u32x4 *gb, size_t a_plane, size_t b_plane, int sub) {
#pragma unroll
    for (int p = 0; p < 3; p++) {
        __builtin_amdgcn_global_load_lds((global_ptr)(ga + p * a_plane), (lds_ptr)(&s.a[p][0][0] + sub), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr)(gb + p * b_plane), (lds_ptr)(&s.b[p][0][0] + sub), 16, 0, 0);
    }
}

// The fragment reads are written as asm: the compiler's wait-count pass drains every outstanding
// global->LDS load before an LDS read that it cannot prove independent of them, which would undo
// the two-steps-ahead prefetch.  The "+v" operands of the waits tie each use to its wait.
#define DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off) : "memory")
#define MFMA(A, B, C) C = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A), __builtin_bit_cast(bf16x8, B), C, 0, 0, 0)

// A wavefront's operands for one stage: 64 x 16 of A and 16 x 128 of B in three planes each, 18 reads of 16 bytes per
// lane.  They are all requested at once and the 48 MFMAs follow when they have arrived.
struct Fragments {
    u32x4 a[2][3], b[4][3];
};

__device__ __forceinline__ void read_fragments(Fragments &f, uint32_t a_addr, uint32_t b_addr) {
#pragma unroll
    for (int p = 0; p < 3; p++) {
        DS_READ(f.a[0][p], a_addr, 0 + 0);
        DS_READ(f.a[1][p], a_addr, 512);
        DS_READ(f.b[0][p], b_addr, 0 + 0);
        DS_READ(f.b[1][p], b_addr, 512);
        DS_READ(f.b[2][p], b_addr, 1024);
        DS_READ(f.b[3][p], b_addr, 1536);
        a_addr += PLANE_BYTES;
        b_addr += PLANE_BYTES;
    }
}

// Smallest terms first for every accumulator; consecutive MFMAs go to different accumulators.
__device__ __forceinline__ void multiply_fragments(Fragments &f, floatx16 (&acc)[2][4]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.a[0][0]), "+v"(f.a[0][1]), "+v"(f.a[0][2]), "+v"(f.a[1][0]), "+v"(f.a[1][1]), "+v"(f.a[1][2]), "+v"(f.b[0][0]),
                   "+v"(f.b[0][1]), "+v"(f.b[0][2]), "+v"(f.b[1][0]), "+v"(f.b[1][1]), "+v"(f.b[1][2]), "+v"(f.b[2][0]), "+v"(f.b[2][1]),
                   "+v"(f.b[2][2]), "+v"(f.b[3][0]), "+v"(f.b[3][1]), "+v"(f.b[3][2]));
    constexpr int PA[6] = {0, 2, 1, 0, 1, 0}, PB[6] = {2, 0, 1, 1, 0, 0};
#pragma unroll
    for (int t = 0; t < 6; t++)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) MFMA(f.a[i][PA[t]], f.b[j][PB[t]], acc[i][j]);
}

__device__ __forceinline__ void slot_barrier(bool loads_left_in_flight) {
    // lgkmcnt(0): this wavefront's fragment reads have left LDS before anybody may overwrite the stage.
    if (loads_left_in_flight) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__global__ __launch_bounds__(THREADS, 1) void gemm_bf16x3(SplitGemmArgs g) {
    __shared__ Stage S[3];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, lr = lane & 31, lk = lane >> 5;
    // Consecutive block ids are dealt to the eight XCDs in turn; give each XCD (one L2) a contiguous
    // run of tiles so that the blocks it runs together share operand panels.
    // The last, partly filled round of an XCD is cut along k instead: its tiles are computed by sf blocks each,
    // so that round takes 1 / sf of a tile's time.
    const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    uint32_t local = slot, part = 0, nparts = 1;
    if (slot >= g.full) {
        local = g.full + (slot - g.full) / g.sf;
        part = (slot - g.full) % g.sf;
        nparts = g.sf;
    }
    const uint32_t tile = xcd * g.chunk + local;
    if (local >= g.chunk || tile >= g.tiles) return;
    const uint32_t m0 = (tile / g.tiles_n) * TM, n0 = (tile % g.tiles_n) * TN;
    const size_t a_plane = (size_t)g.kgs * g.mp, b_plane = (size_t)g.kgs * g.np;

    floatx16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const uint32_t all_stages = g.kgs / 2, first = part * all_stages / nparts, nst = (part + 1) * all_stages / nparts - first;
    const uint32_t a_addr = (uint32_t)(uintptr_t)(lds_ptr)&S[0].a[0][lk][wm * 64 + lr];
    const uint32_t b_addr = (uint32_t)(uintptr_t)(lds_ptr)&S[0].b[0][lk][wn * 128 + lr];
    const int sub = (wave >> 2) * 256 + (wave & 3) * 64;
    const size_t a_step = (size_t)2 * g.mp, b_step = (size_t)2 * g.np;
    const u32x4 *ga = g.ap + first * a_step + (size_t)(wave >> 2) * g.mp + m0 + (wave & 3) * 64 + lane;
    const u32x4 *gb = g.bp + first * b_step + (size_t)(wave >> 2) * g.np + n0 + (wave & 3) * 64 + lane;
    issue(S[0], ga, gb, a_plane, b_plane, sub);
    if (nst > 1) issue(S[1], ga + a_step, gb + b_step, a_plane, b_plane, sub);
    // One barrier per stage.  Between two barriers group 0 (wavefronts 0-3) reads stage t and multiplies it, group 1
    // multiplies stage t - 1 and reads stage t: wavefronts w and w + 4 share a SIMD, and while one waits for its
    // fragments the other keeps the matrix pipe busy.  Before barrier t every wavefront's own loads of stage t have
    // landed and its reads of stage t - 1 have left LDS (slot_barrier), so stage t + 2 may go where stage t - 1 was.
    Fragments f;
    if (wave < 4) {
        for (uint32_t t = 0; t < nst; t++) {
            slot_barrier(t + 1 < nst);
            read_fragments(f, a_addr + (t % 3) * (uint32_t)sizeof(Stage), b_addr + (t % 3) * (uint32_t)sizeof(Stage));
            if (t + 2 < nst) issue(S[(t + 2) % 3], ga + (t + 2) * a_step, gb + (t + 2) * b_step, a_plane, b_plane, sub);
            multiply_fragments(f, acc);
        }
    } else {
        slot_barrier(nst > 1);
        for (uint32_t t = 0; t < nst; t++) {
            if (t > 0) multiply_fragments(f, acc);
            read_fragments(f, a_addr + (t % 3) * (uint32_t)sizeof(Stage), b_addr + (t % 3) * (uint32_t)sizeof(Stage));
            if (t + 2 < nst) issue(S[(t + 2) % 3], ga + (t + 2) * a_step, gb + (t + 2) * b_step, a_plane, b_plane, sub);
            if (t + 1 < nst) slot_barrier(t + 2 < nst);
        }
        multiply_fragments(f, acc);
    }

    // A tile cut along k: every block leaves its partial sums in `partials` (coalesced 16-byte stores), and the block that arrives last adds them up in slice order, so the result does not
    // depend on who was last, and goes on to the epilogue.  All slices of a tile run on one XCD (one L2).
    if (nparts > 1) {
        __shared__ int arrived;
        const uint32_t idx = xcd * (g.chunk - g.full) + (local - g.full);
        // Four accumulator registers per 16-byte store: [register / 4][thread][4].
        f32x4 *mine = reinterpret_cast<f32x4 *>(g.partials + ((size_t)idx * nparts + part) * (TM * TN)) + tid;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++)
                    mine[(size_t)((i * 4 + j) * 4 + r4) * THREADS] =
                        f32x4{acc[i][j][4 * r4], acc[i][j][4 * r4 + 1], acc[i][j][4 * r4 + 2], acc[i][j][4 * r4 + 3]};
        // The partial sums only have to reach this XCD's L2, where the other slices' blocks read them: stores
        // write through the L1, and vmcnt(0) says the L2 has them.  (A device-wide release fence here would
        // write the whole L2 back, once per wavefront.)
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // The launcher cuts tiles only on a context that has measured that blocks whose ids agree mod 8 share an
        // XCD.  Every launch checks it again per tile: a slice counts itself in with 1 in the low byte and 1 in
        // the 3-bit field of the XCD it really ran on (at most 8 slices, so at most 7 ahead of the last one).
        uint32_t xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        xcc &= 7u;
        if (tid == 0) arrived = atomicAdd(&g.counters[idx], (int)(1u + (1u << (8 + 3 * xcc))));
        __syncthreads();
        if ((arrived & 0xff) != (int)nparts - 1) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // nothing stale in this CU's L1
        if (tid == 0) {
            atomicExch(&g.counters[idx], 0);  // ready for the next launch
            // A slice that ran on another XCD left its partial sums in another L2: say so instead of adding up
            // whatever this L2 holds at those addresses.
            if (((uint32_t)arrived >> 8) != ((nparts - 1) << (3 * xcc))) atomicExch(g.misplaced, 1);
        }
        // Sum in slice order, 64 registers' worth of 16-byte loads in flight at a time.
        const f32x4 *all = reinterpret_cast<const f32x4 *>(g.partials + (size_t)idx * nparts * (TM * TN)) + tid;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
        for (uint32_t q = 0; q < nparts; q++) {
            const f32x4 *src = all + (size_t)q * (TM * TN / 4);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                f32x4 tmp[16];
#pragma unroll
                for (int e = 0; e < 16; e++) tmp[e] = src[(size_t)(i * 16 + e) * THREADS];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int r4 = 0; r4 < 4; r4++) {
                        const f32x4 t = tmp[j * 4 + r4];
                        acc[i][j][4 * r4] += t.x, acc[i][j][4 * r4 + 1] += t.y, acc[i][j][4 * r4 + 2] += t.z, acc[i][j][4 * r4 + 3] += t.w;
                    }
            }
        }
    }

    // Epilogue: each wavefront transposes 32 x 128 of its sub-tile at a time through a private LDS
    // region (pitch 132 floats), then stores rows of 128 floats, 16 bytes per lane.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    constexpr int EP = 132;
    float *stage = reinterpret_cast<float *>(&S[0]) + wave * (32 * EP);
    // A bias row (c0_rs == 0) is the same for every row of the tile: read it once, ahead of the stores.
    const uint32_t gcol = n0 + wn * 128 + lr * 4;
    const bool row_bias = g.c0 && g.c0_rs == 0;
    float bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (row_bias) {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (gcol + e < g.n) bias[e] = g.c0[(size_t)(gcol + e) * g.c0_cs];
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) stage[(8 * (r >> 2) + 4 * lk + (r & 3)) * EP + j * 32 + lr] = acc[i][j][r];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll 4
        for (int q = 0; q < 16; q++) {
            const int row = 2 * q + lk;
            const f32x4 t = *reinterpret_cast<const f32x4 *>(stage + row * EP + lr * 4);
            const uint32_t grow = m0 + wm * 64 + i * 32 + row;
            if (grow >= g.m || gcol >= g.n) continue;
            float v[4] = {g.alpha * t.x, g.alpha * t.y, g.alpha * t.z, g.alpha * t.w};
            const bool whole = gcol + 3 < g.n;
            if (row_bias) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] += g.beta * bias[e];
            } else if (g.c0) {
                const float *c0 = g.c0 + (size_t)grow * g.c0_rs + (size_t)gcol * g.c0_cs;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (gcol + e < g.n) v[e] += g.beta * c0[(size_t)e * g.c0_cs];
            }
            float *dst = g.c + (size_t)grow * g.ldc + gcol;
            if (whole && g.c_vec) {
                const f32x4 o = {v[0], v[1], v[2], v[3]};
                if (g.c_stream) __builtin_nontemporal_store(o, reinterpret_cast<f32x4 *>(dst));
                else *reinterpret_cast<f32x4 *>(dst) = o;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (gcol + e < g.n) dst[e] = v[e];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

inline size_t round_up(size_t x, size_t q) { return (x + q - 1) / q * q; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Geometry of one operand's planes.
struct PlaneDims {
    size_t rp, kgs, bytes;
};
PlaneDims plane_dims(size_t rows, size_t k) {
    PlaneDims d;
    d.rp = round_up(rows, 256);
    d.kgs = round_up(k, 16) / 8;
    d.bytes = (size_t)3 * d.kgs * d.rp * 16;
    return d;
}

template <int PRE>
void launch_split(DeviceCtx &ctx, void *planes, const float *src, size_t rows, size_t k, size_t ld, bool k_contig, const PlaneDims &d) {
    const dim3 grid((unsigned)(d.rp / 64), (unsigned)((d.kgs + 3) / 4));
    if (k_contig && aligned16(src) && ld % 4 == 0) {
        // Blocks that run together read neighbouring pieces of the same rows (a 12 KB row of the MLP's inner activation
        // is otherwise fetched 128 bytes at a time at 96 different moments): 5 % on [50432, 3072].
        const int k_fastest = d.rp / 64 <= 65535;
        const dim3 g2 = k_fastest ? dim3(grid.y, grid.x) : grid;
        hipLaunchKernelGGL(split_planes_rows<PRE>, g2, dim3(256), 0, ctx.stream, src, static_cast<u32x4 *>(planes), (uint32_t)rows,
                           (uint32_t)k, ld, (uint32_t)d.rp, (uint32_t)d.kgs, k_fastest);
    } else
        hipLaunchKernelGGL(split_planes<PRE>, grid, dim3(256), 0, ctx.stream, src, static_cast<u32x4 *>(planes), (uint32_t)rows,
                           (uint32_t)k, k_contig ? ld : (size_t)1, k_contig ? (size_t)1 : ld, (uint32_t)d.rp, (uint32_t)d.kgs);
}

int run_split(DeviceCtx &ctx, void *planes, const float *src, size_t rows, size_t k, size_t ld, bool k_contig, int pre_op = 0) {
    const PlaneDims d = plane_dims(rows, k);
    if (pre_op == AHIP_GELU) launch_split<AHIP_GELU>(ctx, planes, src, rows, k, ld, k_contig, d);
    else if (pre_op == AHIP_RELU) launch_split<AHIP_RELU>(ctx, planes, src, rows, k, ld, k_contig, d);
    else launch_split<0>(ctx, planes, src, rows, k, ld, k_contig, d);
    return ctx.check(hipGetLastError(), "split_planes launch");
}

// Planes of an operand that lies in a registered constant buffer are made once and kept.
const void *cached_planes(DeviceCtx &ctx, const float *src, size_t rows, size_t k, size_t ld, bool k_contig, int *rc) {
    *rc = AHIP_OK;
    for (const PackedOperand &p : ctx.gemm_packed)
        if (p.src == src && p.rows == rows && p.k == k && p.ld == ld && p.k_contig == k_contig) return p.planes;
    const char *lo = reinterpret_cast<const char *>(src);
    // Last element read: row rows-1 at k-1.
    const size_t span = k_contig ? ((rows - 1) * ld + k) : ((k - 1) * ld + rows);
    const ConstantBuffer *owner = nullptr;
    for (const ConstantBuffer &cb : ctx.gemm_constants) {
        const char *base = static_cast<const char *>(cb.ptr);
        if (lo >= base && lo + span * sizeof(float) <= base + cb.bytes) owner = &cb;
    }
    if (!owner) return nullptr;
    const PlaneDims d = plane_dims(rows, k);
    void *planes = nullptr;
    if (hipMalloc(&planes, d.bytes) != hipSuccess) {
        (void)hipGetLastError();
        *rc = ctx.fail(AHIP_ERR_OOM, "gemm: no memory for the bf16 planes of a constant operand");
        return nullptr;
    }
    *rc = run_split(ctx, planes, src, rows, k, ld, k_contig);
    if (*rc) {
        (void)hipFree(planes);
        return nullptr;
    }
    PackedOperand p;
    p.owner = owner->ptr;
    p.src = src;
    p.rows = rows;
    p.k = k;
    p.ld = ld;
    p.k_contig = k_contig;
    p.planes = planes;
    p.bytes = d.bytes;
    ctx.gemm_packed.push_back(p);
    return planes;
}

int ensure_workspace(DeviceCtx &ctx, size_t bytes) {
    if (bytes <= ctx.gemm_ws_bytes) return AHIP_OK;
    // Work already queued may still read the old buffer.
    int rc = ctx.check(hipStreamSynchronize(ctx.stream), "hipStreamSynchronize");
    if (rc) return rc;
    if (ctx.gemm_ws) (void)hipFree(ctx.gemm_ws);
    ctx.gemm_ws = nullptr;
    ctx.gemm_ws_bytes = 0;
    ctx.gemm_ws_generation++;
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return ctx.fail(AHIP_ERR_OOM, "gemm: no memory for the bf16 planes of the operands");
    }
    ctx.gemm_ws = p;
    ctx.gemm_ws_bytes = bytes;
    return AHIP_OK;
}

int ensure_partials(DeviceCtx &ctx, size_t bytes) {
    if (!ctx.gemm_counters) {
        void *c = nullptr;
        // Zeroed once, in stream order ahead of the first kernel that counts in it; the kernels leave it zeroed.
        if (hipMalloc(&c, GEMM_COUNTERS * sizeof(int)) != hipSuccess ||
            hipMemsetAsync(c, 0, GEMM_COUNTERS * sizeof(int), ctx.stream) != hipSuccess) {
            (void)hipGetLastError();
            if (c) (void)hipFree(c);
            return ctx.fail(AHIP_ERR_OOM, "gemm: no memory for the slice counters");
        }
        ctx.gemm_counters = static_cast<int *>(c);
    }
    if (bytes <= ctx.gemm_partials_bytes) return AHIP_OK;
    int rc = ctx.check(hipStreamSynchronize(ctx.stream), "hipStreamSynchronize");
    if (rc) return rc;
    if (ctx.gemm_partials) (void)hipFree(ctx.gemm_partials);
    ctx.gemm_partials = nullptr;
    ctx.gemm_partials_bytes = 0;
    ctx.gemm_ws_generation++;
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return ctx.fail(AHIP_ERR_OOM, "gemm: no memory for the partial sums of tiles cut along k");
    }
    ctx.gemm_partials = p;
    ctx.gemm_partials_bytes = bytes;
    return AHIP_OK;
}

}  // namespace

int gemm_workspace(DeviceCtx &ctx, size_t bytes, void **p) {
    const int rc = ensure_workspace(ctx, bytes);
    *p = rc ? nullptr : ctx.gemm_ws;
    return rc;
}

bool gemm_split_worthwhile(size_t m, size_t n, size_t k) {
    // Large products whose C fills most of its 256 x 256 tiles.  Products with few rows (one image through a
    // transformer layer: [197, 768] x [768, 2304]) are faster on the fp32 kernel with k cut into batches: its
    // tiles are smaller and nothing has to be split into planes first (30 against 49 us for that shape).
    if (m < 1024 || n < 256 || k < 128) return false;
    const double useful = (double)m * (double)n / ((double)round_up(m, TM) * (double)round_up(n, TN));
    return useful >= 0.8 && (double)m * (double)n * (double)k >= 2147483648.0;
}

int launch_gemm_split(DeviceCtx &ctx, float *c, const float *a, const float *b, const float *c0, size_t m, size_t n, size_t k,
                      int trans_a, int trans_b, size_t lda, size_t ldb, size_t ldc, size_t c0_row_stride, size_t c0_col_stride,
                      float alpha, float beta, int a_op, const void *a_planes) {
    if (a_op != 0 && a_op != AHIP_GELU && a_op != AHIP_RELU)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm (bf16 x 3): only Gelu and Relu can be folded into the operand split");
    if (a_planes && (a_op || trans_a)) return ctx.fail(AHIP_ERR_ARG, "gemm (bf16 x 3): planes of the first operand come as they are");
    if (m == 0 || n == 0) return AHIP_OK;
    if (!c || (!a && !a_planes) || !b || k == 0) return ctx.fail(AHIP_ERR_ARG, "gemm (bf16 x 3): null pointer or k = 0");
    const size_t lim = (size_t)1 << 31;
    if (m >= lim - 256 || n >= lim - 256 || k >= lim - 16 || lda >= lim || ldb >= lim || ldc >= lim || c0_row_stride >= lim ||
        c0_col_stride >= lim)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm (bf16 x 3): extent above 2^31");
    const PlaneDims da = plane_dims(m, k), db = plane_dims(n, k);
    const size_t tiles_n = db.rp / TN, tiles = tiles_n * (da.rp / TM);
    if (tiles >= lim / 8 || (da.kgs + 3) / 4 > 65535) return ctx.fail(AHIP_ERR_UNSUPPORTED, "gemm (bf16 x 3): too many tiles");
    const bool a_kc = !trans_a, b_kc = trans_b != 0;
    int rc = AHIP_OK;
    const void *pa = a_planes ? a_planes : a_op ? nullptr : cached_planes(ctx, a, m, k, lda, a_kc, &rc);  // cached planes hold the plain values
    if (rc) return rc;
    const void *pb = cached_planes(ctx, b, n, k, ldb, b_kc, &rc);
    if (rc) return rc;
    const size_t a_off = 0, b_off = pa ? 0 : round_up(da.bytes, 256);
    const size_t need = (pa ? 0 : round_up(da.bytes, 256)) + (pb ? 0 : db.bytes);
    if (need) {
        rc = ensure_workspace(ctx, need);
        if (rc) return rc;
    }
    if (!pa) {
        void *p = static_cast<char *>(ctx.gemm_ws) + a_off;
        rc = run_split(ctx, p, a, m, k, lda, a_kc, a_op);
        if (rc) return rc;
        pa = p;
    }
    if (!pb) {
        void *p = static_cast<char *>(ctx.gemm_ws) + b_off;
        rc = run_split(ctx, p, b, n, k, ldb, b_kc);
        if (rc) return rc;
        pb = p;
    }
    SplitGemmArgs g;
    g.ap = static_cast<const u32x4 *>(pa);
    g.bp = static_cast<const u32x4 *>(pb);
    g.c = c;
    g.c0 = (c0 && beta != 0.0f) ? c0 : nullptr;
    g.m = (uint32_t)m;
    g.n = (uint32_t)n;
    g.mp = (uint32_t)da.rp;
    g.np = (uint32_t)db.rp;
    g.kgs = (uint32_t)da.kgs;
    g.ldc = (uint32_t)ldc;
    g.c0_rs = (uint32_t)c0_row_stride;
    g.c0_cs = (uint32_t)c0_col_stride;
    g.alpha = alpha;
    g.beta = beta;
    g.tiles_n = (uint32_t)tiles_n;
    g.tiles = (uint32_t)tiles;
    g.chunk = (uint32_t)((tiles + 7) / 8);
    // An XCD works through its run of tiles one round of `per` blocks at a time (one block per CU).  If the last
    // round is partly filled, cut each of its tiles along k into as many slices as fill it.
    const uint32_t per = ctx.cus_per_xcd ? (uint32_t)ctx.cus_per_xcd : 32u, stages = g.kgs / 2;
    g.full = g.chunk / per * per;
    g.sf = 1;
    const uint32_t rem = g.chunk - g.full;
    // Only where the slices of a tile have been shown to share an L2 (block id mod 8 = XCD, DeviceCtx::xcd_round_robin).
    if (rem && ctx.gemm_split_k && ctx.gemm_in_kernel_k_cut && ctx.xcd_round_robin) {
        uint32_t sf = per / rem;
        sf = std::min(sf, 8u);
        sf = std::min(sf, stages / 4);
        if (sf >= 2 && (size_t)8 * rem <= GEMM_COUNTERS) g.sf = sf;
    }
    if (g.sf == 1) g.full = g.chunk;
    g.partials = nullptr;
    g.counters = nullptr;
    g.misplaced = ctx.flags ? ctx.flags + 1 : nullptr;
    if (g.sf > 1) {
        if (!g.misplaced) return ctx.fail(AHIP_ERR_HIP, "gemm: the context has no error flags");
        ctx.flags_armed = true;
        rc = ensure_partials(ctx, (size_t)8 * (g.chunk - g.full) * g.sf * TM * TN * sizeof(float));
        if (rc) return rc;
        g.partials = static_cast<float *>(ctx.gemm_partials);
        g.counters = ctx.gemm_counters;  // allocated by ensure_partials on first use
        if (!g.partials || !g.counters) return ctx.fail(AHIP_ERR_HIP, "gemm: the buffers for tiles cut along k are missing");
    }
    const uint32_t slots = g.full + (g.chunk - g.full) * g.sf;
    g.c_vec = aligned16(c) && ldc % 4 == 0;
    g.c_stream = ctx.streaming(m * n * sizeof(float));
    hipLaunchKernelGGL(gemm_bf16x3, dim3(slots * 8), dim3(THREADS), 0, ctx.stream, g);
    return ctx.check(hipGetLastError(), "gemm (bf16 x 3) launch");
}

size_t gemm_planes_bytes(size_t rows, size_t k) { return plane_dims(rows, k).bytes; }

int launch_layernorm_planes(DeviceCtx &ctx, void *planes, float *sum_out, const float *in, const float *in2, const float *gamma,
                            const float *beta, size_t rows, size_t len, float eps) {
    if (!planes || !in || !gamma || !beta || (in2 && !sum_out)) return ctx.fail(AHIP_ERR_ARG, "layernorm (planes): null pointer");
    if (!layernorm_planes_fits(rows, len) || !aligned16(in) || !aligned16(gamma) || !aligned16(beta) ||
        (in2 && (!aligned16(in2) || !aligned16(sum_out))))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm (planes): rows must be whole 128-byte lines of 256 to 1024 elements, 16-byte aligned");
    const PlaneDims d = plane_dims(rows, len);
    const dim3 grid((unsigned)(d.rp / LNP_ROWS));
    const size_t shmem = (size_t)3 * d.kgs * LNP_KG_PITCH * sizeof(uint32_t);
    const int nch = (int)((len / 4 + 63) / 64);
#define ALTIUS_LNP(N)                                                                                                                   \
    do {                                                                                                                                \
        if (in2)                                                                                                                        \
            hipLaunchKernelGGL((layernorm_planes<N, true>), grid, dim3(LNP_THREADS), shmem, ctx.stream, static_cast<u32x4 *>(planes), sum_out, in, \
                               in2, gamma, beta, (uint32_t)rows, (uint32_t)len, eps, (uint32_t)d.rp, (uint32_t)d.kgs);                  \
        else                                                                                                                            \
            hipLaunchKernelGGL((layernorm_planes<N, false>), grid, dim3(LNP_THREADS), shmem, ctx.stream, static_cast<u32x4 *>(planes), sum_out, in, \
                               in2, gamma, beta, (uint32_t)rows, (uint32_t)len, eps, (uint32_t)d.rp, (uint32_t)d.kgs);                  \
    } while (0)
    switch (nch) {
    case 1: ALTIUS_LNP(1); break;
    case 2: ALTIUS_LNP(2); break;
    case 3: ALTIUS_LNP(3); break;
    default: ALTIUS_LNP(4); break;
    }
#undef ALTIUS_LNP
    return ctx.check(hipGetLastError(), "layernorm (planes) launch");
}

// The row lengths the stand-alone LayerNormalization gives to its wavefront-per-row kernel (whole 128-byte lines
// filling three quarters of the wavefront's 256-element chunks, at most 1024 elements): only there does the planes
// kernel reproduce its summation order.
bool layernorm_planes_fits(size_t rows, size_t len) {
    const size_t slots = (len + 255) / 256 * 256;
    return rows > 0 && rows < ((size_t)1 << 31) - 256 && len >= 32 && len <= 1024 && len % 32 == 0 && len * 4 >= slots * 3;
}

int gemm_register_constant(DeviceCtx &ctx, const void *ptr, size_t bytes) {
    if (!ptr || !bytes) return ctx.fail(AHIP_ERR_ARG, "gemm_register_constant: null buffer");
    for (ConstantBuffer &cb : ctx.gemm_constants)
        if (cb.ptr == ptr) {
            cb.bytes = bytes;
            return AHIP_OK;
        }
    ctx.gemm_constants.push_back(ConstantBuffer{ptr, bytes});
    return AHIP_OK;
}

int gemm_unregister_constant(DeviceCtx &ctx, const void *ptr) {
    auto it = std::find_if(ctx.gemm_constants.begin(), ctx.gemm_constants.end(), [&](const ConstantBuffer &cb) { return cb.ptr == ptr; });
    if (it == ctx.gemm_constants.end()) return AHIP_OK;
    ctx.gemm_constants.erase(it);
    bool any = false;
    for (const PackedOperand &p : ctx.gemm_packed) any = any || p.owner == ptr;
    if (!any) return AHIP_OK;
    // Kernels that read the planes may still be queued.
    int rc = ctx.check(hipStreamSynchronize(ctx.stream), "hipStreamSynchronize");
    for (size_t i = 0; i < ctx.gemm_packed.size();) {
        if (ctx.gemm_packed[i].owner == ptr) {
            (void)hipFree(ctx.gemm_packed[i].planes);
            ctx.gemm_packed.erase(ctx.gemm_packed.begin() + (long)i);
        } else {
            i++;
        }
    }
    return rc;
}

void gemm_release_all(DeviceCtx &ctx) {
    for (PackedOperand &p : ctx.gemm_packed) (void)hipFree(p.planes);
    ctx.gemm_packed.clear();
    ctx.gemm_constants.clear();
    if (ctx.gemm_ws) (void)hipFree(ctx.gemm_ws);
    ctx.gemm_ws = nullptr;
    ctx.gemm_ws_bytes = 0;
    if (ctx.gemm_partials) (void)hipFree(ctx.gemm_partials);
    ctx.gemm_partials = nullptr;
    ctx.gemm_partials_bytes = 0;
    if (ctx.gemm_counters) (void)hipFree(ctx.gemm_counters);
    ctx.gemm_counters = nullptr;
}

}  // namespace altius
