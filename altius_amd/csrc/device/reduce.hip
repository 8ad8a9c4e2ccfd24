// ReduceMean / ReduceMax for gfx950 over an [outer, reduce, inner] view.
//
//   inner == 1 (reduced axes are the trailing ones):
//     rows under 4096     -> one wavefront per row, lanes stride through the
//                            row (16-byte loads when rows stay aligned), lane
//                            butterfly at the end (short rows: a few lanes per
//                            row, or groups of rows through LDS);
//     longer rows         -> 256-thread blocks, each reducing a row or a
//                            contiguous chunk of one through LDS; with more
//                            than one chunk per row the partials go to the
//                            context's scratch buffer and a second, tiny launch
//                            folds them.
//   inner > 1 (e.g. axis 1 of [256,768,197], the tokens of [N,197,768]):
//     rows of whole float4s -> lanes own float4 columns, the four wavefronts
//                            of a block deal the rows between them and combine
//                            through LDS (reduce_cols_vec4); a thread per
//                            column for up to four rows (reduce_cols_few_rows);
//     other widths to 1024 -> spans of rows that make whole 128-byte lines,
//                            16-byte loads (reduce_cols_span);
//     slabs of a few KB   -> groups of slabs through LDS, a thread per output
//                            (reduce_small_slabs);
//     anything else       -> lanes own single columns (reduce_cols).
//     The reduced axis can additionally be split over blocks, again through
//     the scratch buffer.
//
// Reference: crates/session_interpreter/src/session.rs:1292-1340.  ReduceMean
// multiplies the sum by the f32 reciprocal of the reduced length, as the
// reference does (session.rs:1331,1338).  Max is order-independent and exact;
// sums are accumulated in a different order than the reference's 8 strided
// accumulators.

#include <algorithm>
#include <numeric>
#include <mutex>

#include "common.h"
#include "ctx.h"

namespace altius {
namespace {

using namespace dev;

// Partial results for callers that may not allocate (launch_reduce_static): a fixed array in the code
// object, one copy per GPU for the life of the process.  Host code never uses this name as an address;
// it asks the runtime for the array's device address once per device (reduce_static_setup) and passes
// that pointer to the kernels like any other buffer.
constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)1 << 18;  // 1 MiB
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
std::mutex g_static_mutex;
float *g_static_scratch[MAX_DEVICES] = {};
// The stream whose launch last used each device's fixed array (guarded by g_static_mutex).  Calls on one stream are
// ordered; a call on another stream may take the array over only once everything queued on that stream has finished.
hipStream_t g_static_owner[MAX_DEVICES] = {};
bool g_static_owned[MAX_DEVICES] = {};

constexpr int ROW_BLOCK = 256;
constexpr int ROW_WAVES = ROW_BLOCK / WAVE;

template <class OP> __device__ __forceinline__ float fold4(float acc, const float4 &v) {
    acc = OP::apply(acc, v.x);
    acc = OP::apply(acc, v.y);
    acc = OP::apply(acc, v.z);
    acc = OP::apply(acc, v.w);
    return acc;
}

// Accumulates x[begin..end) strided over `nthreads` lanes starting at `tid`.
// VEC == 4 requires x + begin 16-byte aligned; the range length may be ragged.
template <class OP, int VEC, bool NT = false>
__device__ __forceinline__ float strided_fold(const float *__restrict__ x, size_t begin, size_t end, int tid,
                                              int nthreads) {
    float acc0 = OP::identity(), acc1 = OP::identity(), acc2 = OP::identity(), acc3 = OP::identity();
    if (VEC == 4) {
        const float4 *x4 = reinterpret_cast<const float4 *>(x + begin);
        const size_t n4 = (end - begin) >> 2;
        size_t i = tid;
        for (; i + 3 * (size_t)nthreads < n4; i += 4 * (size_t)nthreads) {
            const float4 a = load4<NT>(reinterpret_cast<const float *>(x4 + i));
            const float4 b = load4<NT>(reinterpret_cast<const float *>(x4 + i + nthreads));
            const float4 c = load4<NT>(reinterpret_cast<const float *>(x4 + i + 2 * (size_t)nthreads));
            const float4 d = load4<NT>(reinterpret_cast<const float *>(x4 + i + 3 * (size_t)nthreads));
            acc0 = fold4<OP>(acc0, a);
            acc1 = fold4<OP>(acc1, b);
            acc2 = fold4<OP>(acc2, c);
            acc3 = fold4<OP>(acc3, d);
        }
        {
            // Up to three more per lane: all issued before the first is folded.
            const size_t i1 = i + nthreads, i2 = i + 2 * (size_t)nthreads;
            const float id = OP::identity();
            float4 a = make_float4(id, id, id, id), b = a, c = a;
            if (i < n4) a = load4<NT>(reinterpret_cast<const float *>(x4 + i));
            if (i1 < n4) b = load4<NT>(reinterpret_cast<const float *>(x4 + i1));
            if (i2 < n4) c = load4<NT>(reinterpret_cast<const float *>(x4 + i2));
            acc0 = fold4<OP>(acc0, a);
            acc1 = fold4<OP>(acc1, b);
            acc2 = fold4<OP>(acc2, c);
        }
        for (size_t j = begin + (n4 << 2) + tid; j < end; j += nthreads) acc1 = OP::apply(acc1, x[j]);
    } else {
        size_t i = begin + tid;
        for (; i + 3 * (size_t)nthreads < end; i += 4 * (size_t)nthreads) {
            const float a = x[i];
            const float b = x[i + nthreads];
            const float c = x[i + 2 * (size_t)nthreads];
            const float d = x[i + 3 * (size_t)nthreads];
            acc0 = OP::apply(acc0, a);
            acc1 = OP::apply(acc1, b);
            acc2 = OP::apply(acc2, c);
            acc3 = OP::apply(acc3, d);
        }
        for (; i < end; i += nthreads) acc0 = OP::apply(acc0, x[i]);
    }
    return OP::apply(OP::apply(acc0, acc1), OP::apply(acc2, acc3));
}

// The same for a range that starts anywhere: single elements up to the first 16-byte boundary, then float4s.
template <class OP, bool NT>
__device__ __forceinline__ float peeled_fold(const float *__restrict__ x, size_t begin, size_t end, int tid, int nthreads) {
    const size_t lead = (4 - ((reinterpret_cast<uintptr_t>(x + begin) >> 2) & 3)) & 3;
    const size_t head = lead < end - begin ? lead : end - begin;
    float acc = OP::identity();
    if ((size_t)tid < head) acc = x[begin + tid];
    return OP::apply(acc, strided_fold<OP, 4, NT>(x, begin + head, end, tid, nthreads));
}

// VEC: 4 = rows of whole float4s on 16-byte boundaries, 0 = rows that start anywhere (peeled_fold), 1 = single elements.
template <class OP, int VEC, bool SCALE, bool NT>
__global__ __launch_bounds__(ROW_BLOCK) void reduce_rows_wave(float *__restrict__ out,
                                                              const float *__restrict__ in, size_t outer,
                                                              size_t red, float scale) {
    const int lane = threadIdx.x & (WAVE - 1);
    const size_t row = (size_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (row >= outer) return;
    float acc = VEC == 0 ? peeled_fold<OP, NT>(in + row * red, 0, red, lane, WAVE) : strided_fold<OP, VEC == 0 ? 1 : VEC, NT>(in + row * red, 0, red, lane, WAVE);
    acc = wave_reduce<OP>(acc);
    if (lane == 0) out[row] = SCALE ? acc * scale : acc;
}

// Rows of 4 to 256 elements that are whole float4s: SUB = 1 to 64 lanes per row, one 16-byte load per lane, so a
// wavefront's load is one contiguous piece of the tensor holding 64 / SUB whole rows (lanes past the row's last
// float4 idle when the float4 count is not a power of two).  Each wavefront takes U such pieces, all loads requested
// before the first is folded.
template <class OP, int SUB, int U, bool SCALE, bool NT>
__global__ __launch_bounds__(ROW_BLOCK) void reduce_rows_sub4(float *__restrict__ out, const float *__restrict__ in, size_t outer,
                                                              uint32_t red, float scale) {
    constexpr int RPP = WAVE / SUB;  // rows per wavefront pass
    const int lane = threadIdx.x & (WAVE - 1);
    const int s = lane & (SUB - 1), rr = lane / SUB;
    const size_t wave = (size_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    const size_t row0 = wave * (size_t)(RPP * U) + rr;
    const bool has = (uint32_t)(4 * s) < red;
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t row = row0 + (size_t)u * RPP;
        const float id = OP::identity();
        v[u] = has && row < outer ? load4<NT>(in + row * red + 4 * s) : make_float4(id, id, id, id);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t row = row0 + (size_t)u * RPP;
        float acc = OP::apply(OP::apply(v[u].x, v[u].y), OP::apply(v[u].z, v[u].w));
        if (SUB > 1) acc = subwave_allreduce<OP, SUB < 4 ? 4 : SUB>(acc);
        if (s == 0 && row < outer) out[row] = SCALE ? acc * scale : acc;
    }
}

// grid = (splits, outer).  Block (s, o) folds chunk s of row o into
// dst[o * splits + s].
template <class OP, int VEC, bool SCALE, bool NT = false>
__global__ __launch_bounds__(ROW_BLOCK) void reduce_rows_block(float *__restrict__ dst,
                                                               const float *__restrict__ in, size_t red,
                                                               size_t chunk, float scale) {
    __shared__ float lds[ROW_WAVES];
    const size_t o = blockIdx.y, s = blockIdx.x;
    const size_t begin = s * chunk;
    size_t end = begin + chunk;
    if (end > red) end = red;
    float acc = OP::identity();
    if (begin < end)
        acc = VEC == 0 ? peeled_fold<OP, NT>(in + o * red, begin, end, threadIdx.x, ROW_BLOCK)
                       : strided_fold<OP, VEC == 0 ? 1 : VEC, NT>(in + o * red, begin, end, threadIdx.x, ROW_BLOCK);
    acc = block_reduce<OP, ROW_WAVES>(acc, lds);
    if (threadIdx.x == 0) dst[o * gridDim.x + s] = SCALE ? acc * scale : acc;
}

// ---------------------------------------------------------------------------
// inner > 1
// ---------------------------------------------------------------------------
constexpr int COL_BLOCK = 512;
constexpr int COL_WAVES = COL_BLOCK / WAVE;
constexpr int ROW_UNROLL = 4;

// grid = (outer * splits, column tiles).  Block (o*splits + s, t) folds rows
// [s*chunk, (s+1)*chunk) of slab o for columns [t*64*CPL, (t+1)*64*CPL) into
// dst[(o*splits + s) * inner + column].
template <class OP, int CPL, bool SCALE>
__global__ __launch_bounds__(COL_BLOCK) void reduce_cols(float *__restrict__ dst, const float *__restrict__ in,
                                                         uint32_t red, uint32_t inner, uint32_t splits,
                                                         uint32_t chunk, float scale) {
    __shared__ float lds[COL_WAVES][CPL * WAVE];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const uint32_t o = blockIdx.x / splits, s = blockIdx.x % splits;
    const uint32_t c0 = blockIdx.y * (CPL * WAVE) + lane;
    const uint32_t r_begin = s * chunk;
    uint32_t r_end = r_begin + chunk;
    if (r_end > red) r_end = red;
    const float *slab = in + (size_t)o * red * inner;

    float acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) acc[j] = OP::identity();

    uint32_t r = r_begin + wave;
    for (; r + (ROW_UNROLL - 1) * COL_WAVES < r_end; r += ROW_UNROLL * COL_WAVES) {
        float v[ROW_UNROLL][CPL];
#pragma unroll
        for (int u = 0; u < ROW_UNROLL; u++) {
            const float *row = slab + (size_t)(r + u * COL_WAVES) * inner;
#pragma unroll
            for (int j = 0; j < CPL; j++) {
                const uint32_t c = c0 + j * WAVE;
                v[u][j] = c < inner ? row[c] : OP::identity();
            }
        }
#pragma unroll
        for (int u = 0; u < ROW_UNROLL; u++)
#pragma unroll
            for (int j = 0; j < CPL; j++) acc[j] = OP::apply(acc[j], v[u][j]);
    }
    for (; r < r_end; r += COL_WAVES) {
        const float *row = slab + (size_t)r * inner;
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            const uint32_t c = c0 + j * WAVE;
            if (c < inner) acc[j] = OP::apply(acc[j], row[c]);
        }
    }

#pragma unroll
    for (int j = 0; j < CPL; j++) lds[wave][j * WAVE + lane] = acc[j];
    __syncthreads();
    for (int t = threadIdx.x; t < CPL * WAVE; t += COL_BLOCK) {
        float a = OP::identity();
#pragma unroll
        for (int w = 0; w < COL_WAVES; w++) a = OP::apply(a, lds[w][t]);
        const uint32_t c = blockIdx.y * (CPL * WAVE) + t;
        if (c < inner) dst[(size_t)blockIdx.x * inner + c] = SCALE ? a * scale : a;
    }
}

// inner a multiple of 4 (rows of whole float4s, 16-byte aligned): lanes own float4 columns.  A block takes a tile of
// tile4 = min(inner / 4, 64) float4 columns; where a row of the tile is narrower than a wavefront, the wavefront's
// lanes cover rpp = 64 / tile4 consecutive rows of it at once (inner = 8: 32 rows, one contiguous KiB per load), so
// the four wavefronts step through the reduced axis 4 * rpp rows at a time, CV_U loads in flight each.  The lanes'
// float4 accumulators meet in LDS, where the first tile4 threads fold the 4 * rpp partial results of their column.
// grid = (outer * splits * tiles of 64 float4 columns).
constexpr int CV_BLOCK = 256, CV_WAVES = CV_BLOCK / WAVE, CV_U = 4;

template <class OP> __device__ __forceinline__ float4 apply4(const float4 &a, const float4 &b) {
    return make_float4(OP::apply(a.x, b.x), OP::apply(a.y, b.y), OP::apply(a.z, b.z), OP::apply(a.w, b.w));
}

template <class OP, bool SCALE, bool NT>
__global__ __launch_bounds__(CV_BLOCK) void reduce_cols_vec4(float *__restrict__ dst, const float *__restrict__ in, uint32_t red,
                                                             uint32_t inner, uint32_t splits, uint32_t chunk, uint32_t tile4,
                                                             uint32_t rpp, uint32_t tiles, float scale) {
    __shared__ float4 lds[CV_WAVES][WAVE];
    const uint32_t lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    // Consecutive blocks take the column tiles of one (slab, split): together they read whole rows.
    const uint32_t part = blockIdx.x / tiles, tile = blockIdx.x - part * tiles;
    const uint32_t o = part / splits, s = part % splits;
    const uint32_t lr = lane / tile4, lc = lane - lr * tile4;
    const uint32_t v4 = inner >> 2, c4 = tile * WAVE + lc;
    const uint32_t r_begin = s * chunk;
    uint32_t r_end = r_begin + chunk;
    if (r_end > red) r_end = red;
    const uint32_t step = CV_WAVES * rpp;  // rows per pass of the block
    const float id = OP::identity();
    float4 acc = make_float4(id, id, id, id);
    if (lr < rpp && c4 < v4) {
        const float *col = in + (size_t)o * red * inner + 4 * (size_t)c4;
        uint32_t r = r_begin + wave * rpp + lr;
        for (; r + (CV_U - 1) * step < r_end; r += CV_U * step) {
            float4 v[CV_U];
#pragma unroll
            for (int u = 0; u < CV_U; u++) v[u] = load4<NT>(col + (size_t)(r + u * step) * inner);
#pragma unroll
            for (int u = 0; u < CV_U; u++) acc = apply4<OP>(acc, v[u]);
        }
        {
            // Up to CV_U - 1 more rows: all requested before the first is folded.
            float4 v[CV_U - 1];
#pragma unroll
            for (int u = 0; u < CV_U - 1; u++)
                v[u] = r + u * step < r_end ? load4<NT>(col + (size_t)(r + u * step) * inner) : make_float4(id, id, id, id);
#pragma unroll
            for (int u = 0; u < CV_U - 1; u++) acc = apply4<OP>(acc, v[u]);
        }
    }
    lds[wave][lane] = acc;
    __syncthreads();
    const uint32_t t = threadIdx.x, out4 = tile * WAVE + t;
    if (t < tile4 && out4 < v4) {
        float4 a = make_float4(id, id, id, id);
        for (uint32_t w = 0; w < CV_WAVES; w++)
            for (uint32_t q = 0; q < rpp; q++) a = apply4<OP>(a, lds[w][q * tile4 + t]);
        if (SCALE) a = make_float4(a.x * scale, a.y * scale, a.z * scale, a.w * scale);
        *reinterpret_cast<float4 *>(dst + (size_t)part * inner + 4 * (size_t)out4) = a;
    }
}

// Very few rows of many float4 columns ([768, 2, 65536]): a thread owns one float4 column of one slab and
// walks all of its rows, CV_U loads in flight; nothing to combine.  Threads number the (slab, column) pairs, so a slab
// narrower than a block leaves no thread idle.  grid = (outer * columns / 256 float4).
template <class OP, bool SCALE, bool NT>
__global__ __launch_bounds__(CV_BLOCK) void reduce_cols_few_rows(float *__restrict__ dst, const float *__restrict__ in, size_t outer,
                                                                 uint32_t red, uint32_t inner, float scale) {
    const uint32_t v4 = inner >> 2;
    const size_t g = (size_t)blockIdx.x * CV_BLOCK + threadIdx.x;
    const size_t o = g / v4;
    if (o >= outer) return;
    const uint32_t c4 = (uint32_t)(g - o * v4);
    const float *col = in + o * red * inner + 4 * (size_t)c4;
    const float id = OP::identity();
    float4 acc = make_float4(id, id, id, id);
    uint32_t r = 0;
    for (; r + CV_U <= red; r += CV_U) {
        float4 v[CV_U];
#pragma unroll
        for (int u = 0; u < CV_U; u++) v[u] = load4<NT>(col + (size_t)(r + u) * inner);
#pragma unroll
        for (int u = 0; u < CV_U; u++) acc = apply4<OP>(acc, v[u]);
    }
    for (; r < red; r++) acc = apply4<OP>(acc, load4<NT>(col + (size_t)r * inner));
    if (SCALE) acc = make_float4(acc.x * scale, acc.y * scale, acc.z * scale, acc.w * scale);
    *reinterpret_cast<float4 *>(dst + o * inner + 4 * (size_t)c4) = acc;
}

// Slabs of a few KB at most ([N, 7, 7] over axis 1, [N, 196, 3]): a block takes `group` consecutive slabs -- one
// contiguous, 16-byte aligned piece of the tensor (group is a multiple of 4) -- into LDS with 16-byte loads, and then a
// thread per output value walks its column there.  A block or a wavefront per slab would leave most lanes idle on 49
// values, and lanes reading single columns from memory would fetch every 128-byte line many times.
// grid = (outer / group); dynamic LDS = group * red * inner floats.
constexpr int SS_BLOCK = 256;
constexpr size_t SS_MAX_SLAB = 2048, SS_GROUP_FLOATS = 8192;

template <class OP, bool SCALE, bool NT>
__global__ __launch_bounds__(SS_BLOCK) void reduce_small_slabs(float *__restrict__ dst, const float *__restrict__ in, size_t outer,
                                                               uint32_t red, uint32_t inner, uint32_t group, uint32_t parts, float scale) {
    extern __shared__ __align__(16) float ss_lds[];
    const uint32_t slab = red * inner;
    const size_t o0 = (size_t)blockIdx.x * group;
    const uint32_t n_slabs = outer - o0 < group ? (uint32_t)(outer - o0) : group;
    const uint32_t floats = n_slabs * slab, n4 = floats >> 2;
    const float *src = in + o0 * slab;
    for (uint32_t i0 = threadIdx.x; i0 < n4; i0 += 4 * SS_BLOCK) {  // four loads requested before the first goes to LDS
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i0 + u * SS_BLOCK < n4) v[u] = load4<NT>(src + 4 * (size_t)(i0 + u * SS_BLOCK));
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (i0 + u * SS_BLOCK < n4) reinterpret_cast<float4 *>(ss_lds)[i0 + u * SS_BLOCK] = v[u];
    }
    for (uint32_t i = (n4 << 2) + threadIdx.x; i < floats; i += SS_BLOCK) ss_lds[i] = src[i];  // the tensor's ragged end
    __syncthreads();
    const uint32_t outs = n_slabs * inner;
    if (parts > 1) {
        // Few outputs per block (a group of [196, 3] slabs has 36): `parts` threads share an output's column, thread p of
        // them taking rows p, p + parts, ..., so that most of the block walks LDS instead of a seventh of it 196 rows each.
        // The partial results go through LDS (the slabs are done with by then) and are combined in a fixed order.
        const uint32_t j = threadIdx.x / parts, p = threadIdx.x - j * parts;  // outs * parts <= SS_BLOCK
        float acc = OP::identity();
        if (j < outs) {
            const uint32_t ol = j / inner, c = j - ol * inner;
            const float *q = ss_lds + ol * slab + c;
            float a0 = OP::identity(), a1 = a0;
            uint32_t r = p;
            for (; r + parts < red; r += 2 * parts) {
                a0 = OP::apply(a0, q[r * inner]);
                a1 = OP::apply(a1, q[(r + parts) * inner]);
            }
            if (r < red) a0 = OP::apply(a0, q[r * inner]);
            acc = OP::apply(a0, a1);
        }
        __syncthreads();
        if (j < outs) ss_lds[threadIdx.x] = acc;  // parts <= red: the partial results fit where the group's slabs were
        __syncthreads();
        if (threadIdx.x < outs) {
            float a = ss_lds[threadIdx.x * parts];
            for (uint32_t k = 1; k < parts; k++) a = OP::apply(a, ss_lds[threadIdx.x * parts + k]);
            dst[o0 * inner + threadIdx.x] = SCALE ? a * scale : a;
        }
        return;
    }
    for (uint32_t j = threadIdx.x; j < outs; j += SS_BLOCK) {
        const uint32_t ol = j / inner, c = j - ol * inner;
        const float *p = ss_lds + ol * slab + c;
        float a0 = OP::identity(), a1 = a0, a2 = a0, a3 = a0;
        uint32_t r = 0;
        for (; r + 4 <= red; r += 4) {
            a0 = OP::apply(a0, p[r * inner]);
            a1 = OP::apply(a1, p[(r + 1) * inner]);
            a2 = OP::apply(a2, p[(r + 2) * inner]);
            a3 = OP::apply(a3, p[(r + 3) * inner]);
        }
        for (; r < red; r++) a0 = OP::apply(a0, p[r * inner]);
        const float acc = OP::apply(OP::apply(a0, a1), OP::apply(a2, a3));
        dst[o0 * inner + j] = SCALE ? acc * scale : acc;
    }
}

// The same reduction with 16-byte loads even when rows are only 4-byte aligned
// (inner = 197, say).  A "span" is P consecutive rows, P chosen so that a span is
// a whole number of 128-byte lines (32 rows when inner is odd).  Because every
// span is exactly P rows long, float4 number j of every span holds the same four
// (row-in-span, column) positions, so thread t accumulates float4 t, t + 1024, ...
// of span after span element by element, and only at the end do the P*inner
// accumulators go through LDS, where column c collects positions c, c + inner,
// c + 2*inner, ...  The loads of the next span are issued before the current one
// is folded in, so each wave has U to 2*U 16-byte loads in flight on whole,
// line-aligned 1-KiB pieces.  Rows left over when the reduced extent is
// not a multiple of P are folded in at the end by the last split.
// grid = (outer * splits); dynamic LDS = P * inner floats.
constexpr int SPAN_BLOCK = 1024;

template <class OP, int U, bool SCALE, bool NT>
__global__ __launch_bounds__(SPAN_BLOCK) void reduce_cols_span(float *__restrict__ dst, const float *__restrict__ in,
                                                               uint32_t red, uint32_t inner, uint32_t span_rows,
                                                               uint32_t splits, uint32_t spans_per_split, float scale) {
    extern __shared__ __align__(16) float span_lds[];
    const uint32_t tid = threadIdx.x;
    const uint32_t o = blockIdx.x / splits, s = blockIdx.x % splits;
    const uint32_t span_floats = span_rows * inner;
    const uint32_t nf4 = span_floats >> 2;
    const uint32_t nspans = red / span_rows;
    const uint32_t sp_begin = s * spans_per_split;
    uint32_t sp_end = sp_begin + spans_per_split;
    if (sp_end > nspans) sp_end = nspans;
    const float *slab = in + (size_t)o * red * inner;

    float4 acc[U];
#pragma unroll
    for (int u = 0; u < U; u++) acc[u] = make_float4(OP::identity(), OP::identity(), OP::identity(), OP::identity());

    // Software pipeline: the loads of span i+1 are in flight while span i is folded in.  Lanes
    // whose float4 index lies past the span re-read its last float4 instead of being masked off:
    // straight-line code lets the loads of the next span overtake the wait for the current one.
    uint32_t off[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t j = tid + SPAN_BLOCK * u;
        off[u] = 4 * (j < nf4 ? j : nf4 - 1);
    }
    auto load_span = [&](uint32_t sp, float4 (&v)[U]) {
        const float *p = slab + (size_t)sp * span_floats;
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = load4<NT>(p + off[u]);
    };
    auto fold_span = [&](const float4 (&v)[U]) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            acc[u].x = OP::apply(acc[u].x, v[u].x);
            acc[u].y = OP::apply(acc[u].y, v[u].y);
            acc[u].z = OP::apply(acc[u].z, v[u].z);
            acc[u].w = OP::apply(acc[u].w, v[u].w);
        }
    };
    // The loop body has no conditional loads, so the wait before each fold can allow exactly
    // the U younger loads to stay in flight.  (A third span in flight was measured: slower.)
    if (sp_begin < sp_end) {
        float4 va[U], vb[U];
        uint32_t sp = sp_begin;
        load_span(sp, va);
        for (; sp + 2 < sp_end; sp += 2) {  // va holds span sp
            load_span(sp + 1, vb);
            fold_span(va);
            load_span(sp + 2, va);
            fold_span(vb);
        }
        if (sp + 1 < sp_end) {
            load_span(sp + 1, vb);
            fold_span(va);
            fold_span(vb);
        } else {
            fold_span(va);
        }
    }

#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t j = tid + SPAN_BLOCK * u;
        if (j < nf4) *reinterpret_cast<float4 *>(span_lds + 4 * j) = acc[u];
    }
    __syncthreads();
    for (uint32_t c = tid; c < inner; c += SPAN_BLOCK) {
        float a = OP::identity();
        for (uint32_t p = 0; p < span_rows; p++) a = OP::apply(a, span_lds[p * inner + c]);
        if (s == splits - 1)
            for (uint32_t r = nspans * span_rows; r < red; r++) a = OP::apply(a, slab[(size_t)r * inner + c]);
        dst[(size_t)blockIdx.x * inner + c] = SCALE ? a * scale : a;
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr size_t MAX_GRID_X = 0x7FFFFFFFu;
constexpr size_t MAX_GRID_Y = 65535;

template <class OP, bool SCALE>
void rows_wave_launch(hipStream_t s, float *out, const float *in, size_t outer, size_t red, float scale,
                      bool nt = false) {
    const bool vec4 = (red % 4 == 0) && aligned16(in);
    const size_t blocks = (outer + ROW_WAVES - 1) / ROW_WAVES;
    if (vec4 && nt)
        hipLaunchKernelGGL((reduce_rows_wave<OP, 4, SCALE, true>), dim3((unsigned)blocks), dim3(ROW_BLOCK), 0, s, out,
                           in, outer, red, scale);
    else if (vec4)
        hipLaunchKernelGGL((reduce_rows_wave<OP, 4, SCALE, false>), dim3((unsigned)blocks), dim3(ROW_BLOCK), 0, s, out,
                           in, outer, red, scale);
    else if (red >= 64 && nt)  // long enough for a body of float4s behind the row's first elements
        hipLaunchKernelGGL((reduce_rows_wave<OP, 0, SCALE, true>), dim3((unsigned)blocks), dim3(ROW_BLOCK), 0, s, out,
                           in, outer, red, scale);
    else if (red >= 64)
        hipLaunchKernelGGL((reduce_rows_wave<OP, 0, SCALE, false>), dim3((unsigned)blocks), dim3(ROW_BLOCK), 0, s, out,
                           in, outer, red, scale);
    else
        hipLaunchKernelGGL((reduce_rows_wave<OP, 1, SCALE, false>), dim3((unsigned)blocks), dim3(ROW_BLOCK), 0, s, out,
                           in, outer, red, scale);
}

template <class OP, bool SCALE>
void rows_block_launch(hipStream_t s, float *dst, const float *in, size_t outer, size_t red, size_t splits,
                       size_t chunk, float scale, bool nt = false) {
    // Chunks start 16-byte aligned when the row pitch and the chunk length are multiples of 4.
    const bool vec4 = aligned16(in) && (red % 4 == 0 || outer == 1) && (chunk % 4 == 0);
    const dim3 grid((unsigned)splits, (unsigned)outer);
    if (vec4 && nt)
        hipLaunchKernelGGL((reduce_rows_block<OP, 4, SCALE, true>), grid, dim3(ROW_BLOCK), 0, s, dst, in, red, chunk,
                           scale);
    else if (vec4)
        hipLaunchKernelGGL((reduce_rows_block<OP, 4, SCALE>), grid, dim3(ROW_BLOCK), 0, s, dst, in, red, chunk,
                           scale);
    else if (nt)
        hipLaunchKernelGGL((reduce_rows_block<OP, 0, SCALE, true>), grid, dim3(ROW_BLOCK), 0, s, dst, in, red, chunk,
                           scale);
    else
        hipLaunchKernelGGL((reduce_rows_block<OP, 0, SCALE, false>), grid, dim3(ROW_BLOCK), 0, s, dst, in, red, chunk,
                           scale);
}

// Whether reduce_cols_vec4 takes this geometry, and its grid's second extent.
inline bool cols_vec4_fits(const float *dst, const float *in, size_t inner) {
    return inner % 4 == 0 && aligned16(in) && aligned16(dst);
}
inline size_t cols_vec4_tiles(size_t inner) { return (inner / 4 + WAVE - 1) / WAVE; }

template <class OP, bool SCALE>
void cols_launch(hipStream_t s, float *dst, const float *in, size_t outer, size_t red, size_t inner,
                 size_t splits, size_t chunk, float scale, bool nt = false) {
    if (cols_vec4_fits(dst, in, inner)) {
        const size_t v4 = inner / 4, tile4 = v4 < (size_t)WAVE ? v4 : (size_t)WAVE, rpp = WAVE / tile4;
        const size_t tiles = cols_vec4_tiles(inner);
        const dim3 grid((unsigned)(outer * splits * tiles));
        if (nt)
            hipLaunchKernelGGL((reduce_cols_vec4<OP, SCALE, true>), grid, dim3(CV_BLOCK), 0, s, dst, in, (uint32_t)red, (uint32_t)inner,
                               (uint32_t)splits, (uint32_t)chunk, (uint32_t)tile4, (uint32_t)rpp, (uint32_t)tiles, scale);
        else
            hipLaunchKernelGGL((reduce_cols_vec4<OP, SCALE, false>), grid, dim3(CV_BLOCK), 0, s, dst, in, (uint32_t)red, (uint32_t)inner,
                               (uint32_t)splits, (uint32_t)chunk, (uint32_t)tile4, (uint32_t)rpp, (uint32_t)tiles, scale);
        return;
    }
    const size_t cpl = inner <= 64 ? 1 : inner <= 128 ? 2 : 4;
    const size_t tiles = (inner + cpl * WAVE - 1) / (cpl * WAVE);
    const dim3 grid((unsigned)(outer * splits), (unsigned)tiles);
    const dim3 block(COL_BLOCK);
    if (cpl == 1)
        hipLaunchKernelGGL((reduce_cols<OP, 1, SCALE>), grid, block, 0, s, dst, in, (uint32_t)red,
                           (uint32_t)inner, (uint32_t)splits, (uint32_t)chunk, scale);
    else if (cpl == 2)
        hipLaunchKernelGGL((reduce_cols<OP, 2, SCALE>), grid, block, 0, s, dst, in, (uint32_t)red,
                           (uint32_t)inner, (uint32_t)splits, (uint32_t)chunk, scale);
    else
        hipLaunchKernelGGL((reduce_cols<OP, 4, SCALE>), grid, block, 0, s, dst, in, (uint32_t)red,
                           (uint32_t)inner, (uint32_t)splits, (uint32_t)chunk, scale);
}

template <class OP, bool SCALE>
void cols_span_launch(hipStream_t s, float *dst, const float *in, size_t outer, size_t red, size_t inner,
                      size_t span_rows, size_t splits, size_t spans_per_split, float scale, bool nt) {
    const dim3 grid((unsigned)(outer * splits));
    const dim3 block(SPAN_BLOCK);
    const size_t shmem = span_rows * inner * sizeof(float);
    const int u = (int)((span_rows * inner / 4 + SPAN_BLOCK - 1) / SPAN_BLOCK);
#define ALTIUS_LAUNCH(N, T)                                                                                   \
    hipLaunchKernelGGL((reduce_cols_span<OP, N, SCALE, T>), grid, block, shmem, s, dst, in, (uint32_t)red,    \
                       (uint32_t)inner, (uint32_t)span_rows, (uint32_t)splits, (uint32_t)spans_per_split, scale)
    if (nt) {
        if (u <= 1) ALTIUS_LAUNCH(1, true);
        else if (u == 2) ALTIUS_LAUNCH(2, true);
        else ALTIUS_LAUNCH(4, true);
    } else {
        if (u <= 1) ALTIUS_LAUNCH(1, false);
        else if (u == 2) ALTIUS_LAUNCH(2, false);
        else ALTIUS_LAUNCH(4, false);
    }
#undef ALTIUS_LAUNCH
}

size_t gcd_size(size_t a, size_t b) {
    while (b) {
        const size_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Where the partial results of a two-stage reduction go.  fixed: the buffer cannot be replaced by a
// one-stage launch or anything else when it is too small; the call fails instead, naming the sizes.
struct Partials {
    float *ptr;
    size_t floats;
    bool fixed;
};

int partials_too_small(DeviceCtx &ctx, size_t needed, const Partials &pt) {
    return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: this shape needs " + std::to_string(needed) + " floats of partial results, the " +
                                              (pt.fixed ? "fixed buffer of the no-allocation entry point" : "context's scratch buffer") + " holds " +
                                              std::to_string(pt.floats));
}

// Before a launch writes partial results: the context's own buffer is its own business; the fixed array of the
// no-allocation entry point is shared by every context and stream of the GPU, and a second stream gets it only when
// the first has drained (hipStreamQuery: no allocation, no wait).  Otherwise the call fails instead of racing.
int claim_partials(DeviceCtx &ctx, const Partials &pt) {
    if (!pt.fixed || ctx.device < 0 || ctx.device >= MAX_DEVICES) return AHIP_OK;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_static_owned[ctx.device] && g_static_owner[ctx.device] != ctx.stream) {
        const hipError_t e = hipStreamQuery(g_static_owner[ctx.device]);
        if (e == hipErrorNotReady)
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce (no-allocation entry point): the fixed buffer is still in use by work queued on "
                                                  "another stream of this GPU; synchronize that stream first, or use ahip_reduce");
        (void)hipGetLastError();  // finished, or a stream that no longer exists: the array is free either way
    }
    g_static_owner[ctx.device] = ctx.stream;
    g_static_owned[ctx.device] = true;
    return AHIP_OK;
}

template <class OP, bool SCALE>
int reduce_impl(DeviceCtx &ctx, const Partials &pt, float *out, const float *in, size_t outer, size_t red, size_t inner,
                float scale) {
    hipStream_t s = ctx.stream;
    if (inner == 1) {
        // Rows of up to 256 elements that are whole float4s: a few lanes per row, straight from memory.
        if (red % 4 == 0 && red >= 16 && red <= 256 && aligned16(in)) {
            constexpr int U = 4;
            const size_t v4 = red / 4;
            const int sub = v4 <= 4 ? 4 : v4 <= 8 ? 8 : v4 <= 16 ? 16 : v4 <= 32 ? 32 : 64;
            const size_t rows_per_wave = (size_t)(WAVE / sub) * U;
            const size_t blocks = (outer + rows_per_wave * ROW_WAVES - 1) / (rows_per_wave * ROW_WAVES);
            if (blocks <= MAX_GRID_X) {
                const bool nt = ctx.streaming(outer * red * sizeof(float));
                const dim3 grid((unsigned)blocks), block(ROW_BLOCK);
#define ALTIUS_SUB4(SUBV)                                                                                                          \
    do {                                                                                                                           \
        if (nt) hipLaunchKernelGGL((reduce_rows_sub4<OP, SUBV, U, SCALE, true>), grid, block, 0, s, out, in, outer, (uint32_t)red, scale);  \
        else hipLaunchKernelGGL((reduce_rows_sub4<OP, SUBV, U, SCALE, false>), grid, block, 0, s, out, in, outer, (uint32_t)red, scale);    \
    } while (0)
                switch (sub) {
                case 4: ALTIUS_SUB4(4); break;
                case 8: ALTIUS_SUB4(8); break;
                case 16: ALTIUS_SUB4(16); break;
                case 32: ALTIUS_SUB4(32); break;
                default: ALTIUS_SUB4(64); break;
                }
#undef ALTIUS_SUB4
                return ctx.check(hipGetLastError(), "reduce rows (lane groups) launch");
            }
        }
        // Short rows and rows that are not whole 128-byte lines (a wavefront per row would fetch the lines two rows
        // share twice: 10 % more traffic on rows of 1000): groups of rows staged through LDS, a few lanes per row.
        if (red <= 1024 && (red % 32 != 0 || red < 256)) {
            const int rc = launch_reduce_rows_lds(ctx, std::is_same<OP, MaxOp>::value, out, in, outer, red, scale, SCALE);
            if (rc >= 0) return rc;
        }
        // A wavefront per row below 4096 elements, a block of four above (measured over 96 M elements, non-temporal loads
        // in both: 4096: 84 against 88 % of the HBM peak, 8192: 82 / 88, 16384: 77 / 87; 3072: 86.5 / 85.5).
        if (red < 4096 || outer >= 65536) {
            if ((outer + ROW_WAVES - 1) / ROW_WAVES > MAX_GRID_X)
                return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: too many rows for one launch");
            rows_wave_launch<OP, SCALE>(s, out, in, outer, red, scale, ctx.streaming(outer * red * sizeof(float)));
            return ctx.check(hipGetLastError(), "reduce rows (wave) launch");
        }
        if (outer > MAX_GRID_Y) return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: too many rows for one launch");
        // Aim for a few thousand blocks; every block gets at least 4096 elements.
        size_t splits = 1;
        if (outer < 1024) {
            splits = (4096 + outer - 1) / outer;
            const size_t max_splits = (red + 4095) / 4096;
            if (splits > max_splits) splits = max_splits;
            if (splits < 1) splits = 1;
        }
        size_t chunk = (red + splits - 1) / splits;
        chunk = (chunk + 1023) / 1024 * 1024;
        splits = (red + chunk - 1) / chunk;
        const bool nt = ctx.streaming(outer * red * sizeof(float));
        if (splits == 1) {
            rows_block_launch<OP, SCALE>(s, out, in, outer, red, 1, chunk, scale, nt);
            return ctx.check(hipGetLastError(), "reduce rows (block) launch");
        }
        if (outer * splits > pt.floats) return partials_too_small(ctx, outer * splits, pt);
        if (int rc = claim_partials(ctx, pt)) return rc;
        rows_block_launch<OP, false>(s, pt.ptr, in, outer, red, splits, chunk, 1.0f, nt);
        rows_wave_launch<OP, SCALE>(s, out, pt.ptr, outer, splits, scale);
        return ctx.check(hipGetLastError(), "reduce rows (two-stage) launch");
    }

    // inner > 1
    if (red >= ((size_t)1 << 32) || inner >= ((size_t)1 << 31))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: axis extent exceeds 32-bit index range");
    // Small slabs whose rows are not whole float4s, or too few and too narrow to keep half of reduce_cols_vec4's lanes busy.
    if (red * inner <= SS_MAX_SLAB && aligned16(in) && (inner % 4 != 0 || red * std::min<size_t>(inner / 4, WAVE) < CV_BLOCK / 2)) {
        const size_t slab = red * inner;
        // Slabs per group: a multiple of 4 (16-byte loads), and of as many slabs as have whole 128-byte lines of results where
        // a group holds that many (32 slabs of 7 x 7: 68 -> 72 % of the HBM peak), so that no line of the output is written
        // in part by two blocks.  (Lines of the input shared by two groups cost nothing measurable: [196, 3] slabs run
        // a point better in groups of 12 than in groups of 8, which end on line boundaries.)
        const size_t limit = SS_GROUP_FLOATS / slab;  // SS_MAX_SLAB * 4 <= SS_GROUP_FLOATS: at least 4
        const size_t whole_lines = 32 / std::gcd<size_t>(inner, 32);
        const size_t step = whole_lines >= 4 && whole_lines <= limit ? whole_lines : 4;
        size_t group = limit / step * step;
        while (group > step && (outer + group - 1) / group < 2048) group -= step;  // rather more blocks than fuller ones
        const size_t blocks = (outer + group - 1) / group;
        if (blocks <= MAX_GRID_X) {
            const bool nt = ctx.streaming(outer * slab * sizeof(float));
            const dim3 grid((unsigned)blocks), block(SS_BLOCK);
            const size_t shmem = group * slab * sizeof(float);
            // threads per output where a group has few of them: as many as the block has, at most 8, rows for each
            const size_t per_output = std::min<size_t>({(size_t)SS_BLOCK / (group * inner), (size_t)8, red / 4});
            const uint32_t parts = per_output >= 2 ? (uint32_t)per_output : 1u;
            if (nt) hipLaunchKernelGGL((reduce_small_slabs<OP, SCALE, true>), grid, block, shmem, s, out, in, outer, (uint32_t)red, (uint32_t)inner, (uint32_t)group, parts, scale);
            else hipLaunchKernelGGL((reduce_small_slabs<OP, SCALE, false>), grid, block, shmem, s, out, in, outer, (uint32_t)red, (uint32_t)inner, (uint32_t)group, parts, scale);
            return ctx.check(hipGetLastError(), "reduce (small slabs) launch");
        }
    }
    // Rows that are not multiples of 16 bytes, moderate width: the span variant with 16-byte loads.
    if (inner % 4 != 0 && inner <= 1024 && aligned16(in) && (outer == 1 || (red * inner) % 4 == 0)) {
        const size_t span_rows = 32 / gcd_size(inner, 32);  // smallest P with P * inner * 4 bytes a multiple of 128
        const size_t nspans = red / span_rows;
        if (span_rows * inner <= (size_t)4 * 4 * SPAN_BLOCK && nspans >= 4) {
            // One 16-wave block per slab fills the chip once there are about as many slabs as CUs;
            // with fewer slabs the reduced axis is split over blocks and a second launch folds the parts.
            size_t fsplits = 1;
            if (outer < 192) {
                fsplits = (512 + outer - 1) / outer;
                const size_t max_splits = nspans / 4 > 0 ? nspans / 4 : 1;
                if (fsplits > max_splits) fsplits = max_splits;
            }
            size_t sps = (nspans + fsplits - 1) / fsplits;
            fsplits = (nspans + sps - 1) / sps;
            const bool nt = ctx.streaming(outer * red * inner * sizeof(float));
            if (outer * fsplits <= MAX_GRID_X) {
                if (fsplits == 1) {
                    cols_span_launch<OP, SCALE>(s, out, in, outer, red, inner, span_rows, 1, sps, scale, nt);
                    return ctx.check(hipGetLastError(), "reduce cols (span) launch");
                }
                if (outer * fsplits * inner <= pt.floats) {
                    if (int rc = claim_partials(ctx, pt)) return rc;
                    cols_span_launch<OP, false>(s, pt.ptr, in, outer, red, inner, span_rows, fsplits, sps, 1.0f, nt);
                    cols_launch<OP, SCALE>(s, out, pt.ptr, outer, fsplits, inner, 1, fsplits, scale);
                    return ctx.check(hipGetLastError(), "reduce cols (span, two-stage) launch");
                }
                if (pt.fixed) return partials_too_small(ctx, outer * fsplits * inner, pt);
            }
        }
    }

    const bool nt = ctx.streaming(outer * red * inner * sizeof(float));
    const bool vec4 = cols_vec4_fits(out, in, inner);
    // Up to four rows (fewer than reduce_cols_vec4's wavefronts could share) of at least a wavefront's worth of float4
    // columns: a thread per column, no partial results ([768,2,65536]: 84 % of the HBM peak against 53 %; from eight
    // rows on the other kernel is ahead, [12288,8,1024]: 78 against 83 %).
    if (vec4 && red <= 4 && inner >= 4 * (size_t)WAVE && (outer * (inner / 4) + CV_BLOCK - 1) / CV_BLOCK <= MAX_GRID_X) {
        const dim3 grid((unsigned)((outer * (inner / 4) + CV_BLOCK - 1) / CV_BLOCK));
        if (nt) hipLaunchKernelGGL((reduce_cols_few_rows<OP, SCALE, true>), grid, dim3(CV_BLOCK), 0, s, out, in, outer, (uint32_t)red, (uint32_t)inner, scale);
        else hipLaunchKernelGGL((reduce_cols_few_rows<OP, SCALE, false>), grid, dim3(CV_BLOCK), 0, s, out, in, outer, (uint32_t)red, (uint32_t)inner, scale);
        return ctx.check(hipGetLastError(), "reduce cols (few rows) launch");
    }
    const size_t cpl = inner <= 64 ? 1 : inner <= 128 ? 2 : 4;
    const size_t tiles = vec4 ? cols_vec4_tiles(inner) : (inner + cpl * WAVE - 1) / (cpl * WAVE);
    if (!vec4 && tiles > MAX_GRID_Y) return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: inner extent too large");
    size_t splits = 1;
    const size_t blocks = outer * tiles;
    // Rows one pass of a block covers (its wavefronts take different rows; a wavefront of reduce_cols_vec4 covers
    // several where a row is narrower than its 64 lanes): a block keeps at least eight passes.
    const size_t rows_per_pass = vec4 ? (size_t)CV_WAVES * (WAVE / std::min<size_t>(inner / 4, WAVE)) : 4;
    if (blocks < 1024 && red >= 16 * rows_per_pass) {
        splits = (1024 + blocks - 1) / blocks;
        const size_t max_splits = red / (8 * rows_per_pass);
        if (splits > max_splits) splits = max_splits;
        if (splits < 1) splits = 1;
    }
    size_t chunk = (red + splits - 1) / splits;
    splits = (red + chunk - 1) / chunk;
    if (outer * splits * (vec4 ? tiles : 1) > MAX_GRID_X)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "reduce: outer extent too large for one launch");
    if (splits == 1) {
        cols_launch<OP, SCALE>(s, out, in, outer, red, inner, 1, chunk, scale, nt);
        return ctx.check(hipGetLastError(), "reduce cols launch");
    }
    if (outer * splits * inner > pt.floats) {
        if (pt.fixed) return partials_too_small(ctx, outer * splits * inner, pt);
        // Not enough scratch for the partials: do it in one stage.
        cols_launch<OP, SCALE>(s, out, in, outer, red, inner, 1, red, scale, nt);
        return ctx.check(hipGetLastError(), "reduce cols launch");
    }
    if (int rc = claim_partials(ctx, pt)) return rc;
    cols_launch<OP, false>(s, pt.ptr, in, outer, red, inner, splits, chunk, 1.0f, nt);
    cols_launch<OP, SCALE>(s, out, pt.ptr, outer, splits, inner, 1, splits, scale);
    return ctx.check(hipGetLastError(), "reduce cols (two-stage) launch");
}

int reduce_with(DeviceCtx &ctx, const Partials &pt, int kind, float *out, const float *in, size_t outer, size_t red, size_t inner) {
    if (kind != AHIP_REDUCE_MEAN && kind != AHIP_REDUCE_MAX && kind != AHIP_REDUCE_SUM)
        return ctx.fail(AHIP_ERR_ARG, "reduce: unknown kind");
    if (outer == 0 || inner == 0) return AHIP_OK;
    if (red == 0) return ctx.fail(AHIP_ERR_ARG, "reduce: empty reduced axis");
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "reduce: null tensor pointer");
    if (kind == AHIP_REDUCE_MEAN) {
        const float r_axis_len = 1.0f / (float)red;
        return reduce_impl<SumOp, true>(ctx, pt, out, in, outer, red, inner, r_axis_len);
    }
    if (kind == AHIP_REDUCE_SUM) return reduce_impl<SumOp, false>(ctx, pt, out, in, outer, red, inner, 1.0f);
    return reduce_impl<MaxOp, false>(ctx, pt, out, in, outer, red, inner, 1.0f);
}

}  // namespace

int launch_reduce(DeviceCtx &ctx, int kind, float *out, const float *in, size_t outer, size_t red,
                  size_t inner) {
    return reduce_with(ctx, Partials{ctx.scratch, ctx.scratch_floats, false}, kind, out, in, outer, red, inner);
}

int reduce_static_setup(int device) {
    if (device < 0 || device >= MAX_DEVICES) return AHIP_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_static_scratch[device]) return AHIP_OK;
    float *ptr = nullptr;
    // The calling thread's current device is `device`: each GPU holds its own copy of the array at its own address.
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return AHIP_ERR_HIP;
    }
    g_static_scratch[device] = ptr;
    return AHIP_OK;
}

size_t reduce_static_capacity_floats() { return STATIC_SCRATCH_FLOATS; }

void reduce_static_forget_stream(int device, hipStream_t stream) {
    if (device < 0 || device >= MAX_DEVICES) return;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_static_owned[device] && g_static_owner[device] == stream) g_static_owned[device] = false;
}

int launch_reduce_static(DeviceCtx &ctx, int kind, float *out, const float *in, size_t outer, size_t red, size_t inner) {
    float *ptr = nullptr;
    if (ctx.device >= 0 && ctx.device < MAX_DEVICES) {
        std::lock_guard<std::mutex> lock(g_static_mutex);
        ptr = g_static_scratch[ctx.device];
    }
    if (!ptr) return ctx.fail(AHIP_ERR_HIP, "reduce (no-allocation entry point): the fixed buffer's address was not resolved on this device");
    return reduce_with(ctx, Partials{ptr, STATIC_SCRATCH_FLOATS, true}, kind, out, in, outer, red, inner);
}

}  // namespace altius
