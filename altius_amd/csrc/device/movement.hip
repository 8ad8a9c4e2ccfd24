// Data-movement kernels: strided copies (Transpose, Slice, Concat, Split, Expand, Tile), a tiled
// transpose for permutations that move the innermost axis, Gather, Where, Cast, Greater and
// BatchNormalization.  Counterparts in the reference interpreter:
// crates/session_interpreter/src/session.rs:1134-1278 (concat, transpose), 1488-1598 (split, slice,
// gather), 940-988 (where), 1350-1378 (cast), 1380-1431 (batch normalisation), 541-562 (greater).
// All of them move each byte once: the roofline is HBM bandwidth, the care goes into keeping both
// the read and the write side coalesced.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>

#include "common.h"
#include "ctx.h"

namespace altius {

namespace {

using dev::FastDiv;
using dev::make_fastdiv;

constexpr int BLOCK = 256;

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned128(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 127u) == 0; }

// ---- generic strided copy --------------------------------------------------------------------
// Logical index space dims[0..rank) (axis 0 innermost here); element `idx` is read at
// sum(idx[d] * in_str[d]) and written at sum(idx[d] * out_str[d]).  Either side may be dense,
// windowed (Concat / Split / Slice), permuted (Transpose) or repeated (stride 0: Expand, Tile).
struct CopyGeom {
    FastDiv dims[MAX_RANK];
    uint32_t in_str[MAX_RANK];
    uint32_t out_str[MAX_RANK];
    int rank;
};

// T is the storage unit: 1, 4, 8 or 16 bytes (16 = four 4-byte elements moved together when the
// innermost axis is contiguous on both sides and everything is 16-byte aligned).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// NT (16-byte units only): non-temporal accesses, for tensors too large to be found in a cache afterwards.
template <class T, bool NT = false>
__global__ __launch_bounds__(BLOCK) void copy_strided(T *__restrict__ out, const T *__restrict__ in, CopyGeom g,
                                                      uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t rest = i, src = 0, dst = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.rank) {
            const uint32_t q = g.dims[d].div(rest);
            const uint32_t r = rest - q * g.dims[d].d;
            src += r * g.in_str[d];
            dst += r * g.out_str[d];
            rest = q;
        }
    }
    if (NT) {
        static_assert(!NT || sizeof(T) == 16, "non-temporal copies move 16-byte units");
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in + src));
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + dst));
    } else {
        out[dst] = in[src];
    }
}

// The element-wise copy with four elements per thread, BLOCK apart (each access of a wavefront stays as coalesced as
// it was): the four loads are requested before the first store, and a block's index arithmetic overlaps them.
template <class T>
__global__ __launch_bounds__(BLOCK) void copy_strided_x4(T *__restrict__ out, const T *__restrict__ in, CopyGeom g, uint32_t total) {
    const uint32_t first = blockIdx.x * (4 * BLOCK) + threadIdx.x;
    uint32_t src[4], dst[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        uint32_t rest = first + k * BLOCK;
        src[k] = dst[k] = 0;
#pragma unroll
        for (int d = 0; d < MAX_RANK; d++) {
            if (d < g.rank) {
                const uint32_t q = g.dims[d].div(rest);
                const uint32_t r = rest - q * g.dims[d].d;
                src[k] += r * g.in_str[d];
                dst[k] += r * g.out_str[d];
                rest = q;
            }
        }
    }
    T v[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (first + k * BLOCK < total) v[k] = in[src[k]];
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (first + k * BLOCK < total) out[dst[k]] = v[k];
}

// ---- tiled transpose -------------------------------------------------------------------------
// For permutations whose output-innermost axis is not the input-innermost axis.  View the tensor
// as [batch..., R, ..., C, ...] where C is the input's contiguous axis and R the axis that becomes
// contiguous in the output.  A block moves a TILE x TILE patch of (R, C) through LDS: rows of the
// patch are read along C (coalesced), columns are written along R (coalesced).  The remaining axes
// are enumerated by blockIdx.z through the same index decomposition as copy_strided.
constexpr int TILE = 64;

struct TransGeom {
    uint32_t r_len, c_len;          // extents of R and C
    uint32_t r_in_str, c_out_str;   // stride of R in the input, of C in the output (both sides' other stride is 1)
    FastDiv bdims[MAX_RANK];        // the remaining axes (any order; innermost first)
    uint32_t b_in_str[MAX_RANK];
    uint32_t b_out_str[MAX_RANK];
    int brank;
};

// Which patch a block takes where pieces of a patch start and end inside cache lines (single elements at odd
// addresses; 16-byte accesses along rows whose pitch is not a whole number of 128-byte lines).  The patch next door
// completes such a line, so each XCD takes a run of neighbouring patches (dev::piece_of_block): [50257, 768] ->
// [768, 50257] wrote 11 % more bytes than the result holds and ran at 65 % of the HBM peak with patches dealt out row by
// row, 74 % this way; the other way round 69 -> 85 %.  A run goes along one axis in a band of `band` patches across:
// neighbours along the run's axis are `band` blocks apart, neighbours across it follow each other.
// along_r: runs go along R (whose pieces are written), else along C (whose pieces are read).
__device__ __forceinline__ void patch_of_block(bool along_r, uint32_t band, uint32_t &bx, uint32_t &by) {
    const uint32_t nx = gridDim.x, ny = gridDim.y;
    const uint32_t turn = dev::piece_of_block(blockIdx.y * nx + blockIdx.x, nx * ny);
    const uint32_t n_run = along_r ? ny : nx, n_across = along_r ? nx : ny;
    const uint32_t whole = n_across / band * band, in_whole = whole * n_run;  // patches in bands of full width
    uint32_t run, across;
    if (turn < in_whole) {
        const uint32_t b = turn / (band * n_run), rest = turn - b * band * n_run;
        run = rest / band, across = b * band + rest - run * band;
    } else {
        const uint32_t w = n_across - whole, rest = turn - in_whole;  // the last, narrower band
        run = rest / w, across = whole + rest - run * w;
    }
    bx = along_r ? across : run, by = along_r ? run : across;
}

template <class T>
__global__ __launch_bounds__(BLOCK) void transpose_tiled(T *__restrict__ out, const T *__restrict__ in, TransGeom g) {
    __shared__ T tile[TILE][TILE + 1];
    uint32_t rest = blockIdx.z, src0 = 0, dst0 = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.brank) {
            const uint32_t q = g.bdims[d].div(rest);
            const uint32_t r = rest - q * g.bdims[d].d;
            src0 += r * g.b_in_str[d];
            dst0 += r * g.b_out_str[d];
            rest = q;
        }
    }
    uint32_t bx, by;
    patch_of_block(true, 8, bx, by);  // both sides move single elements
    const uint32_t c0 = bx * TILE, r0 = by * TILE;
    const uint32_t tx = threadIdx.x & (TILE - 1), ty = threadIdx.x / TILE;  // 64 x 4
    // read: lane tx walks C, ty (+4k) walks R; all sixteen loads are requested before the first goes to LDS
    T v[TILE / (BLOCK / TILE)];
#pragma unroll
    for (int k = 0; k < TILE; k += BLOCK / TILE) {
        const uint32_t r = r0 + ty + k, c = c0 + tx;
        if (r < g.r_len && c < g.c_len) v[k / (BLOCK / TILE)] = in[src0 + r * g.r_in_str + c];
    }
#pragma unroll
    for (int k = 0; k < TILE; k += BLOCK / TILE) tile[ty + k][tx] = v[k / (BLOCK / TILE)];
    __syncthreads();
    // write: lane tx walks R, ty (+4k) walks C
#pragma unroll 4
    for (int k = 0; k < TILE; k += BLOCK / TILE) {
        const uint32_t c = c0 + ty + k, r = r0 + tx;
        if (r < g.r_len && c < g.c_len) out[dst0 + c * g.c_out_str + r] = tile[tx][ty + k];
    }
}

// The same patch with 16-byte accesses on both sides, for 4-byte elements when both extents, both strides and every
// batch offset are multiples of 4, the tensors are 16-byte aligned and the rows written start on 128-byte boundaries:
// a thread reads four float4 along C and writes four float4 along R (each gathered from four LDS rows).  The pitch
// of 65 words keeps both the row-wise stores and the column-wise gathers of a wavefront on 64 different banks.
// LINES: the rows read start on 128-byte boundaries too.
template <bool NT, bool LINES>
__global__ __launch_bounds__(BLOCK) void transpose_tiled_vec4(uint32_t *__restrict__ out, const uint32_t *__restrict__ in, TransGeom g) {
    __shared__ uint32_t tile[TILE][TILE + 1];
    uint32_t rest = blockIdx.z, src0 = 0, dst0 = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.brank) {
            const uint32_t q = g.bdims[d].div(rest);
            const uint32_t r = rest - q * g.bdims[d].d;
            src0 += r * g.b_in_str[d];
            dst0 += r * g.b_out_str[d];
            rest = q;
        }
    }
    uint32_t bx, by;
    if (LINES) {
        // Pitches of whole lines: tiles are dealt diagonally.  Blocks that run together (consecutive blockIdx.x) then differ
        // in R as well as in C, so with a pitch that is a large power of two their rows do not all fall on the same memory
        // channels.
        bx = blockIdx.x, by = blockIdx.y + blockIdx.x;
        by = by >= gridDim.y ? by % gridDim.y : by;
    } else {
        patch_of_block(true, 8, bx, by);
    }
    const uint32_t c0 = bx * TILE, r0 = by * TILE;
    const uint32_t q4 = threadIdx.x & 15, line = threadIdx.x >> 4;  // 16 float4 per 64-wide line, 16 lines per pass
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t r = r0 + line + 16 * k, c = c0 + 4 * q4;
        v[k] = u32x4{0, 0, 0, 0};
        if (r < g.r_len && c < g.c_len) {
            const u32x4 *p = reinterpret_cast<const u32x4 *>(in + src0 + (size_t)r * g.r_in_str + c);
            v[k] = NT ? __builtin_nontemporal_load(p) : *p;
        }
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        uint32_t *row = &tile[line + 16 * k][4 * q4];
        row[0] = v[k].x, row[1] = v[k].y, row[2] = v[k].z, row[3] = v[k].w;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t c = c0 + line + 16 * k, r = r0 + 4 * q4;
        if (r < g.r_len && c < g.c_len) {
            const uint32_t col = line + 16 * k;
            const u32x4 w = {tile[4 * q4][col], tile[4 * q4 + 1][col], tile[4 * q4 + 2][col], tile[4 * q4 + 3][col]};
            u32x4 *p = reinterpret_cast<u32x4 *>(out + dst0 + (size_t)c * g.c_out_str + r);
            if (NT) __builtin_nontemporal_store(w, p);
            else *p = w;
        }
    }
}

// The 64 x 64 patch of 4-byte elements when only one side lines up for 16-byte accesses (an odd R extent:
// [50257, 768] -> [768, 50257], or rows written that do not start on 128-byte boundaries; or an odd C extent the
// other way round): that side moves float4s as in transpose_tiled_vec4, the other single elements as in
// transpose_tiled.  (16-byte stores are no way out on the written side: a wavefront's store is four separate 256-byte
// pieces, and where those straddle cache lines they run at half the speed of the single elements.)
template <bool LOAD4, bool NT>
__global__ __launch_bounds__(BLOCK) void transpose_tiled_mixed(uint32_t *__restrict__ out, const uint32_t *__restrict__ in, TransGeom g) {
    __shared__ uint32_t tile[TILE][TILE + 1];
    uint32_t rest = blockIdx.z, src0 = 0, dst0 = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.brank) {
            const uint32_t q = g.bdims[d].div(rest);
            const uint32_t r = rest - q * g.bdims[d].d;
            src0 += r * g.b_in_str[d];
            dst0 += r * g.b_out_str[d];
            rest = q;
        }
    }
    uint32_t bx, by;
    patch_of_block(LOAD4, 8, bx, by);  // runs along the axis that moves single elements
    const uint32_t c0 = bx * TILE, r0 = by * TILE;
    const uint32_t q4 = threadIdx.x & 15, line = threadIdx.x >> 4;           // the float4 side: 16 float4 per line, 16 lines per pass
    const uint32_t tx = threadIdx.x & (TILE - 1), ty = threadIdx.x / TILE;  // the element side: 64 x 4
    if (LOAD4) {
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t r = r0 + line + 16 * k, c = c0 + 4 * q4;
            v[k] = u32x4{0, 0, 0, 0};
            if (r < g.r_len && c < g.c_len) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(in + src0 + (size_t)r * g.r_in_str + c);
                v[k] = NT ? __builtin_nontemporal_load(p) : *p;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t *row = &tile[line + 16 * k][4 * q4];
            row[0] = v[k].x, row[1] = v[k].y, row[2] = v[k].z, row[3] = v[k].w;
        }
    } else {
        uint32_t v[TILE / (BLOCK / TILE)];
#pragma unroll
        for (int k = 0; k < TILE; k += BLOCK / TILE) {
            const uint32_t r = r0 + ty + k, c = c0 + tx;
            if (r < g.r_len && c < g.c_len) v[k / (BLOCK / TILE)] = in[src0 + (size_t)r * g.r_in_str + c];
        }
#pragma unroll
        for (int k = 0; k < TILE; k += BLOCK / TILE) tile[ty + k][tx] = v[k / (BLOCK / TILE)];
    }
    __syncthreads();
    if (LOAD4) {
#pragma unroll 4
        for (int k = 0; k < TILE; k += BLOCK / TILE) {
            const uint32_t c = c0 + ty + k, r = r0 + tx;
            if (r < g.r_len && c < g.c_len) out[dst0 + (size_t)c * g.c_out_str + r] = tile[tx][ty + k];
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t c = c0 + line + 16 * k, r = r0 + 4 * q4;
            if (r < g.r_len && c < g.c_len) {
                const uint32_t col = line + 16 * k;
                const u32x4 w = {tile[4 * q4][col], tile[4 * q4 + 1][col], tile[4 * q4 + 2][col], tile[4 * q4 + 3][col]};
                u32x4 *p = reinterpret_cast<u32x4 *>(out + dst0 + (size_t)c * g.c_out_str + r);
                if (NT) __builtin_nontemporal_store(w, p);
                else *p = w;
            }
        }
    }
}

// Matrices whose transposed image is dense ([.., R, C] -> [.., C, R] with R of up to a thousand elements: 197 tokens x
// 768 channels) but too large for one block: a block takes a panel of TC columns, all R rows of them.  It reads R
// segments of TC elements (whole 128-byte lines with TC = 32) and writes one dense span of TC x R elements, which
// starts and ends on a 128-byte boundary whatever R is: 16-byte accesses on both sides and no line written by two
// blocks, where 64 x 64 patches leave 5 of the last patch's 64 rows in use and cut every output row at odd addresses.
// LDS holds the panel transposed, [TC][pitch] with an odd pitch.
constexpr int PANEL = 32;
constexpr int PANEL_BLOCK = 512;  // 197 rows of 8 float4: one round of four loads per thread
template <int TC, bool NT>
__global__ __launch_bounds__(PANEL_BLOCK) void transpose_panel(uint32_t *__restrict__ out, const uint32_t *__restrict__ in, TransGeom g, uint32_t pitch,
                                                         FastDiv rdiv) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    uint32_t *lds = reinterpret_cast<uint32_t *>(smem_raw);  // element (c, r) of the panel at c * pitch + r
    uint32_t rest = blockIdx.y, src0 = 0, dst0 = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.brank) {
            const uint32_t q = g.bdims[d].div(rest);
            const uint32_t r = rest - q * g.bdims[d].d;
            src0 += r * g.b_in_str[d];
            dst0 += r * g.b_out_str[d];
            rest = q;
        }
    }
    const uint32_t c0 = blockIdx.x * TC;
    constexpr uint32_t Q = TC / 4;                 // float4 per row segment
    const uint32_t n4 = g.r_len * Q;               // float4 of the panel, on either side
    const uint32_t *src = in + src0 + c0;
    uint32_t *dst = out + dst0 + (size_t)c0 * g.r_len;
    constexpr int U = 4;  // loads requested before the first is scattered into LDS
    for (uint32_t i0 = threadIdx.x; i0 < n4; i0 += U * PANEL_BLOCK) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * PANEL_BLOCK;
            if (i < n4) {
                const u32x4 *p = reinterpret_cast<const u32x4 *>(src + (size_t)(i / Q) * g.r_in_str + 4 * (i % Q));
                v[u] = NT ? __builtin_nontemporal_load(p) : *p;
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * PANEL_BLOCK;
            if (i < n4) {
                const uint32_t r = i / Q, c = 4 * (i % Q);
                lds[c * pitch + r] = v[u].x, lds[(c + 1) * pitch + r] = v[u].y, lds[(c + 2) * pitch + r] = v[u].z, lds[(c + 3) * pitch + r] = v[u].w;
            }
        }
    }
    __syncthreads();
    const bool image = pitch == g.r_len;  // an odd R: LDS holds the span as it goes out, 16 bytes at a time
    for (uint32_t i = threadIdx.x; i < n4; i += PANEL_BLOCK) {
        u32x4 t;
        if (image) {
            t = *reinterpret_cast<const u32x4 *>(lds + 4 * i);
        } else {
            uint32_t c = rdiv.div(4 * i), r = 4 * i - c * g.r_len;  // the span is [c][r]
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                w[k] = lds[c * pitch + r];
                if (++r == g.r_len) {
                    r = 0;
                    c++;
                }
            }
            t = u32x4{w[0], w[1], w[2], w[3]};
        }
        if (NT) __builtin_nontemporal_store(t, reinterpret_cast<u32x4 *>(dst + 4 * (size_t)i));
        else *reinterpret_cast<u32x4 *>(dst + 4 * (size_t)i) = t;
    }
}

// Batched transpose of small matrices that are contiguous on both sides (attention's K^T:
// [.., 197, 64] -> [.., 64, 197]).  One block moves one whole r_len x c_len matrix: it reads the
// matrix as one contiguous span, scatters it into LDS transposed, and writes the result as one
// contiguous span, so both global sides run at full 16-byte width whatever the extents are.
// The LDS row pitch is odd, which keeps the transposed stores conflict-free.
template <class T, int VEC, int TB = BLOCK, bool NT = false>
__global__ __launch_bounds__(TB) void transpose_small(T *__restrict__ out, const T *__restrict__ in, uint32_t r_len,
                                                      uint32_t c_len, uint32_t pitch, FastDiv cdiv, FastDiv rdiv) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *lds = reinterpret_cast<T *>(smem_raw);  // [c_len][pitch], element (c, r) at c * pitch + r
    const uint32_t n = r_len * c_len;
    const T *src = in + (size_t)blockIdx.x * n;
    T *dst = out + (size_t)blockIdx.x * n;
    // Four loads per thread are requested before the first is scattered into LDS (the trip count is not known at
    // compile time, so the loop would otherwise wait for every load in turn).
    constexpr int U = 4;
    for (uint32_t i0 = threadIdx.x * VEC; i0 < n; i0 += U * TB * VEC) {
        T v[U][VEC];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * TB * VEC;
            if (i < n) {
                if (VEC == 4) {
                    const u32x4 t = NT ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + i)) : *reinterpret_cast<const u32x4 *>(src + i);
                    v[u][0] = (T)t.x; v[u][1 % VEC] = (T)t.y; v[u][2 % VEC] = (T)t.z; v[u][3 % VEC] = (T)t.w;
                } else {
                    v[u][0] = src[i];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t i = i0 + u * TB * VEC;
            if (i < n) {
                uint32_t r = cdiv.div(i), c = i - r * c_len;  // input is [r][c]
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    lds[c * pitch + r] = v[u][k];
                    if (++c == c_len) {
                        c = 0;
                        r++;
                    }
                }
            }
        }
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x * VEC; i < n; i += TB * VEC) {
        uint32_t c = rdiv.div(i), r = i - c * r_len;  // output is [c][r]
        T v[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            v[k] = lds[c * pitch + r];
            if (++r == r_len) {
                r = 0;
                c++;
            }
        }
        if (VEC == 4) {
            u32x4 t;
            t.x = (uint32_t)v[0]; t.y = (uint32_t)v[1 % VEC]; t.z = (uint32_t)v[2 % VEC]; t.w = (uint32_t)v[3 % VEC];
            if (NT) __builtin_nontemporal_store(t, reinterpret_cast<u32x4 *>(dst + i));
            else *reinterpret_cast<u32x4 *>(dst + i) = t;
        } else {
            dst[i] = v[0];
        }
    }
}

// ---- gather ----------------------------------------------------------------------------------
// out[o, j, :] = data[o, idx[j], :] with `inner` contiguous elements per row; negative indices
// count from the end (ONNX).  Out-of-range indices read row 0 and raise the flag in *bad.
template <class T, class I>
__global__ __launch_bounds__(BLOCK) void gather_rows(T *__restrict__ out, const T *__restrict__ data,
                                                     const I *__restrict__ idx, uint32_t axis_len, uint32_t n_idx,
                                                     FastDiv inner, FastDiv idx_div, uint32_t total,
                                                     int *__restrict__ bad) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    const uint32_t row = inner.div(i);        // o * n_idx + j
    const uint32_t col = i - row * inner.d;
    const uint32_t o = idx_div.div(row);
    const uint32_t j = row - o * idx_div.d;
    long long k = (long long)idx[j];
    if (k < 0) k += axis_len;
    if (k < 0 || k >= (long long)axis_len) {
        *bad = 1;
        k = 0;
    }
    out[i] = data[((size_t)o * axis_len + (size_t)k) * inner.d + col];
}

// ---- where -----------------------------------------------------------------------------------
struct WhereGeom {
    FastDiv dims[MAX_RANK];
    uint32_t c_str[MAX_RANK], x_str[MAX_RANK], y_str[MAX_RANK];
    int rank;
};

template <class T>
__global__ __launch_bounds__(BLOCK) void where_strided(T *__restrict__ out, const uint8_t *__restrict__ cond,
                                                       const T *__restrict__ x, const T *__restrict__ y, WhereGeom g,
                                                       uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t rest = i, ci = 0, xi = 0, yi = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.rank) {
            const uint32_t q = g.dims[d].div(rest);
            const uint32_t r = rest - q * g.dims[d].d;
            ci += r * g.c_str[d];
            xi += r * g.x_str[d];
            yi += r * g.y_str[d];
            rest = q;
        }
    }
    out[i] = cond[ci] ? x[xi] : y[yi];
}

// ---- greater ---------------------------------------------------------------------------------
struct CmpGeom {
    FastDiv dims[MAX_RANK];
    uint32_t a_str[MAX_RANK], b_str[MAX_RANK];
    int rank;
};

__global__ __launch_bounds__(BLOCK) void greater_strided(uint8_t *__restrict__ out, const float *__restrict__ a,
                                                         const float *__restrict__ b, CmpGeom g, uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t rest = i, ai = 0, bi = 0;
#pragma unroll
    for (int d = 0; d < MAX_RANK; d++) {
        if (d < g.rank) {
            const uint32_t q = g.dims[d].div(rest);
            const uint32_t r = rest - q * g.dims[d].d;
            ai += r * g.a_str[d];
            bi += r * g.b_str[d];
            rest = q;
        }
    }
    out[i] = a[ai] > b[bi] ? 1 : 0;
}

// ---- cast ------------------------------------------------------------------------------------
// Rust `as` semantics (session.rs:1350-1378): int -> float rounds to nearest, float -> int
// truncates and saturates with NaN -> 0, wider -> narrower int wraps, anything -> bool is != 0.
template <class To, class From> __device__ __forceinline__ To cast_one(From v) { return (To)v; }
template <> __device__ __forceinline__ int32_t cast_one<int32_t, float>(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
template <> __device__ __forceinline__ long long cast_one<long long, float>(float v) {
    if (v != v) return 0;
    if (v >= 9223372036854775808.0f) return INT64_MAX;
    if (v <= -9223372036854775808.0f) return INT64_MIN;
    return (long long)v;
}
struct BoolTag {
    uint8_t v;
};
template <class From> __device__ __forceinline__ uint8_t to_bool(From v) { return v != (From)0 ? 1 : 0; }

template <class To, class From, bool TO_BOOL>
__global__ __launch_bounds__(BLOCK) void cast_flat(To *__restrict__ out, const From *__restrict__ in, size_t n) {
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n) return;
    if (TO_BOOL)
        out[i] = (To)to_bool<From>(in[i]);
    else
        out[i] = cast_one<To, From>(in[i]);
}

// ---- batch normalisation ---------------------------------------------------------------------
// y = ((x - mean[c]) / sqrt(var[c] + eps)) * scale[c] + bias[c] on NCHW, in the reference's
// operation order (session.rs:1424-1427): true division, no fused multiply-add.
template <int VEC>
__global__ __launch_bounds__(BLOCK) void batchnorm_nchw(float *__restrict__ out, const float *__restrict__ x,
                                                        const float *__restrict__ scale, const float *__restrict__ bias,
                                                        const float *__restrict__ mean, const float *__restrict__ var,
                                                        FastDiv hw, FastDiv ch, uint32_t total, float eps) {
    const uint32_t i = (blockIdx.x * BLOCK + threadIdx.x) * VEC;
    if (i >= total) return;
    const uint32_t plane = hw.div(i);  // n * C + c ; VEC divides H*W, so the VEC elements share a plane
    const uint32_t c = plane - ch.div(plane) * ch.d;
    const float m = mean[c], d = sqrtf(var[c] + eps), s = scale[c], b = bias[c];
    if (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(x + i);
        float4 r;
        r.x = ((v.x - m) / d) * s + b;
        r.y = ((v.y - m) / d) * s + b;
        r.z = ((v.z - m) / d) * s + b;
        r.w = ((v.w - m) / d) * s + b;
        *reinterpret_cast<float4 *>(out + i) = r;
    } else {
        out[i] = ((x[i] - m) / d) * s + b;
    }
}

// ---- im2col and max pooling -------------------------------------------------------------------
// col[b][c][fy][fx][oh][ow] = x[b][c][oh*sh - pad_t + fy*dh][ow*sw - pad_l + fx*dw], zero outside the
// image: the layout the reference builds (conv2d.rs:82-150, 213-333), K-major so that the
// convolution is W[oc, K] x col[K, oh*ow] per image and group.
struct ConvGeom {
    FastDiv ow, oh, kw, kh, c;
    uint32_t ih, iw, sh, sw, dh, dw, pad_t, pad_l;
};

__global__ __launch_bounds__(BLOCK) void im2col_kernel(float *__restrict__ col, const float *__restrict__ x, ConvGeom g,
                                                       uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t r = i;
    uint32_t q = g.ow.div(r);
    const uint32_t ow = r - q * g.ow.d;
    r = q;
    q = g.oh.div(r);
    const uint32_t oh = r - q * g.oh.d;
    r = q;
    q = g.kw.div(r);
    const uint32_t fx = r - q * g.kw.d;
    r = q;
    q = g.kh.div(r);
    const uint32_t fy = r - q * g.kh.d;
    const uint32_t plane = q;  // b * C + c
    const int y = (int)(oh * g.sh + fy * g.dh) - (int)g.pad_t;
    const int xx = (int)(ow * g.sw + fx * g.dw) - (int)g.pad_l;
    float v = 0.0f;
    if (y >= 0 && y < (int)g.ih && xx >= 0 && xx < (int)g.iw) v = x[((size_t)plane * g.ih + (uint32_t)y) * g.iw + (uint32_t)xx];
    col[i] = v;
}

// compute_max_pool (session.rs:324-382): the window is clipped to the image, NaN never wins
// (f32::max), and a window that holds nothing (or only f32::MIN) yields 0.0.
__global__ __launch_bounds__(BLOCK) void maxpool_kernel(float *__restrict__ out, const float *__restrict__ x, FastDiv ow,
                                                        FastDiv oh, uint32_t ih, uint32_t iw, uint32_t kh, uint32_t kw,
                                                        uint32_t sh, uint32_t sw, uint32_t pad_t, uint32_t pad_l,
                                                        uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t q = ow.div(i);
    const uint32_t ox = i - q * ow.d;
    const uint32_t plane = oh.div(q);
    const uint32_t oy = q - plane * oh.d;
    const int y0 = (int)(oy * sh) - (int)pad_t, x0 = (int)(ox * sw) - (int)pad_l;
    const float lowest = -3.40282347e+38f;  // f32::MIN
    float m = lowest;
    const float *p = x + (size_t)plane * ih * iw;
    for (uint32_t fy = 0; fy < kh; fy++) {
        const int y = y0 + (int)fy;
        if (y < 0 || y >= (int)ih) continue;
        for (uint32_t fx = 0; fx < kw; fx++) {
            const int xx = x0 + (int)fx;
            if (xx < 0 || xx >= (int)iw) continue;
            m = fmaxf(p[(uint32_t)y * iw + (uint32_t)xx], m);
        }
    }
    out[i] = m == lowest ? 0.0f : m;
}

// ---- resize ----------------------------------------------------------------------------------
// compute_resize (session.rs:1056-1132) on NCHW: "nearest" takes x[(h / scale) as usize][(w / scale) as usize];
// every other mode is the reference's bilinear blend with half-pixel centres clamped at 0.  The
// reference derives one scale from the heights and uses it for both axes; here each axis has its own
// (identical whenever the two agree, which is the only case in which the reference stays in bounds).
template <bool NEAREST>
__global__ __launch_bounds__(BLOCK) void resize_kernel(float *__restrict__ out, const float *__restrict__ x, FastDiv ow,
                                                       FastDiv oh, uint32_t ih, uint32_t iw, float scale_h, float scale_w,
                                                       uint32_t total) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= total) return;
    uint32_t q = ow.div(i);
    const uint32_t w = i - q * ow.d;
    const uint32_t plane = oh.div(q);
    const uint32_t h = q - plane * oh.d;
    const float *p = x + (size_t)plane * ih * iw;
    if (NEAREST) {
        uint32_t y = (uint32_t)((float)h / scale_h), xx = (uint32_t)((float)w / scale_w);
        y = y < ih ? y : ih - 1;
        xx = xx < iw ? xx : iw - 1;
        out[i] = p[y * iw + xx];
    } else {
        const float ihf = fmaxf((float)h / scale_h - 0.5f, 0.0f), iwf = fmaxf((float)w / scale_w - 0.5f, 0.0f);
        const uint32_t y = (uint32_t)ihf, xx = (uint32_t)iwf;
        const uint32_t y0 = y < ih - 1 ? y : ih - 1, y1 = y + 1 < ih - 1 ? y + 1 : ih - 1;
        const uint32_t x0 = xx < iw - 1 ? xx : iw - 1, x1 = xx + 1 < iw - 1 ? xx + 1 : iw - 1;
        const float v00 = p[y0 * iw + x0], v01 = p[y0 * iw + x1], v10 = p[y1 * iw + x0], v11 = p[y1 * iw + x1];
        const float fy = ihf - (float)y, fx = iwf - (float)xx;
        const float hd = v00 + (v10 - v00) * fy;
        const float hw = v01 + (v11 - v01) * fy;
        out[i] = hd + (hw - hd) * fx;
    }
}

struct Vec16 {
    uint32_t a, b, c, d;
};

int fits32(DeviceCtx &ctx, size_t total, const char *what) {
    if (total >= ((size_t)1 << 31)) return ctx.fail(AHIP_ERR_UNSUPPORTED, std::string(what) + ": more than 2^31 elements");
    return AHIP_OK;
}

template <class T>
void launch_copy(hipStream_t s, void *out, const void *in, const CopyGeom &g, uint32_t total) {
    if (sizeof(T) < 16 && total >= 16 * BLOCK) {  // elements past `total` are decomposed too (and dropped): no address is formed from them
        hipLaunchKernelGGL((copy_strided_x4<T>), dim3((total + 4 * BLOCK - 1) / (4 * BLOCK)), dim3(BLOCK), 0, s, static_cast<T *>(out),
                           static_cast<const T *>(in), g, total);
        return;
    }
    hipLaunchKernelGGL((copy_strided<T>), dim3((total + BLOCK - 1) / BLOCK), dim3(BLOCK), 0, s, static_cast<T *>(out),
                       static_cast<const T *>(in), g, total);
}

}  // namespace

int launch_copy_strided(DeviceCtx &ctx, void *out, const void *in, int elem_size, int rank, const int64_t *dims,
                        const int64_t *out_strides, const int64_t *in_strides) {
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "copy: rank must be 0..8");
    if (elem_size != 1 && elem_size != 4 && elem_size != 8) return ctx.fail(AHIP_ERR_ARG, "copy: element size must be 1, 4 or 8");
    // Drop size-1 axes, then merge neighbours that are contiguous on both sides.
    std::vector<int64_t> d, so, si;
    size_t total = 1;
    for (int i = 0; i < rank; i++) {
        if (dims[i] < 0 || out_strides[i] < 0 || in_strides[i] < 0) return ctx.fail(AHIP_ERR_ARG, "copy: negative extent or stride");
        total *= (size_t)dims[i];
        if (dims[i] == 1) continue;
        d.push_back(dims[i]);
        so.push_back(out_strides[i]);
        si.push_back(in_strides[i]);
    }
    if (total == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "copy: null pointer");
    for (size_t i = d.size(); i-- > 1;) {
        // axis i-1 (outer) and i (inner) merge when outer stride == inner stride * inner extent on both sides
        if (so[i - 1] == so[i] * d[i] && si[i - 1] == si[i] * d[i]) {
            d[i - 1] *= d[i];
            so[i - 1] = so[i];
            si[i - 1] = si[i];
            d.erase(d.begin() + i);
            so.erase(so.begin() + i);
            si.erase(si.begin() + i);
        }
    }
    if (int rc = fits32(ctx, total, "copy")) return rc;
    size_t max_in = 0, max_out = 0;
    for (size_t i = 0; i < d.size(); i++) {
        max_in += (size_t)(d[i] - 1) * (size_t)si[i];
        max_out += (size_t)(d[i] - 1) * (size_t)so[i];
    }
    if (max_in >= ((size_t)1 << 31) || max_out >= ((size_t)1 << 31))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "copy: an operand spans more than 2^31 elements");
    if (d.empty()) {
        d.push_back(1);
        so.push_back(1);
        si.push_back(1);
    }
    // 16-byte units when the innermost axis is contiguous on both sides and everything lines up.
    int unit = elem_size;
    if (elem_size == 4 && so.back() == 1 && si.back() == 1 && d.back() % 4 == 0 && aligned16(out) && aligned16(in)) {
        bool ok = true;
        for (size_t i = 0; i + 1 < d.size(); i++) ok = ok && so[i] % 4 == 0 && si[i] % 4 == 0;
        if (ok) {
            unit = 16;
            d.back() /= 4;
            for (size_t i = 0; i + 1 < d.size(); i++) {
                so[i] /= 4;
                si[i] /= 4;
            }
            total /= 4;
        }
    }
    CopyGeom g;
    g.rank = (int)d.size();
    for (int i = 0; i < MAX_RANK; i++) {
        g.dims[i] = make_fastdiv(1);
        g.in_str[i] = g.out_str[i] = 0;
    }
    for (int i = 0; i < g.rank; i++) {  // innermost first
        const size_t j = d.size() - 1 - (size_t)i;
        g.dims[i] = make_fastdiv((uint32_t)d[j]);
        g.in_str[i] = (uint32_t)si[j];
        g.out_str[i] = (uint32_t)so[j];
    }
    switch (unit) {
    case 1: launch_copy<uint8_t>(ctx.stream, out, in, g, (uint32_t)total); break;
    case 4: launch_copy<uint32_t>(ctx.stream, out, in, g, (uint32_t)total); break;
    case 8: launch_copy<uint64_t>(ctx.stream, out, in, g, (uint32_t)total); break;
    default:
        if (ctx.streaming(total * 16))
            hipLaunchKernelGGL((copy_strided<uint4, true>), dim3((unsigned)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream,
                               static_cast<uint4 *>(out), static_cast<const uint4 *>(in), g, (uint32_t)total);
        else
            launch_copy<uint4>(ctx.stream, out, in, g, (uint32_t)total);
        break;
    }
    return ctx.check(hipGetLastError(), "copy_strided launch");
}

int launch_transpose(DeviceCtx &ctx, void *out, const void *in, int elem_size, int rank, const int64_t *in_dims,
                     const int64_t *perm) {
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "transpose: rank must be 0..8");
    if (elem_size != 1 && elem_size != 4 && elem_size != 8) return ctx.fail(AHIP_ERR_ARG, "transpose: element size must be 1, 4 or 8");
    bool seen[MAX_RANK] = {};
    for (int i = 0; i < rank; i++) {
        if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]]) return ctx.fail(AHIP_ERR_ARG, "transpose: perm must name every axis once");
        seen[perm[i]] = true;
        if (in_dims[i] < 0) return ctx.fail(AHIP_ERR_ARG, "transpose: negative extent");
    }
    // Strides of the input, then the logical (output-ordered) view: out axis i reads input axis perm[i].
    int64_t in_str[MAX_RANK], od[MAX_RANK], os[MAX_RANK], is[MAX_RANK];
    int64_t acc = 1;
    for (int i = rank - 1; i >= 0; i--) {
        in_str[i] = acc;
        acc *= in_dims[i];
    }
    const size_t total = (size_t)acc;
    if (total == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "transpose: null pointer");
    acc = 1;
    for (int i = rank - 1; i >= 0; i--) {
        od[i] = in_dims[perm[i]];
        is[i] = in_str[perm[i]];
        os[i] = acc;
        acc *= od[i];
    }
    // Collapse: drop size-1 axes and merge output-adjacent axes that are also adjacent in the input.
    std::vector<int64_t> d, so, si;
    for (int i = 0; i < rank; i++) {
        if (od[i] == 1) continue;
        d.push_back(od[i]);
        so.push_back(os[i]);
        si.push_back(is[i]);
    }
    for (size_t i = d.size(); i-- > 1;) {
        if (si[i - 1] == si[i] * d[i]) {  // output strides are dense by construction
            d[i - 1] *= d[i];
            so[i - 1] = so[i];
            si[i - 1] = si[i];
            d.erase(d.begin() + i);
            so.erase(so.begin() + i);
            si.erase(si.begin() + i);
        }
    }
    if (int rc = fits32(ctx, total, "transpose")) return rc;
    // The innermost output axis is contiguous in the input too (or nothing is left to permute):
    // rows of `d.back()` elements move whole -> strided copy, 16 bytes at a time when it lines up.
    if (d.size() <= 1 || si.back() == 1) {
        const int r = (int)d.size();
        return launch_copy_strided(ctx, out, in, elem_size, r, d.data(), so.data(), si.data());
    }
    // Tiled path: C = the axis with input stride 1, R = the innermost output axis.
    size_t c_axis = d.size();
    for (size_t i = 0; i < d.size(); i++)
        if (si[i] == 1) c_axis = i;
    if (c_axis == d.size()) return ctx.fail(AHIP_ERR_ARG, "transpose: no contiguous input axis");  // cannot happen for a dense input
    TransGeom g;
    g.r_len = (uint32_t)d.back();
    g.r_in_str = (uint32_t)si.back();
    g.c_len = (uint32_t)d[c_axis];
    g.c_out_str = (uint32_t)so[c_axis];
    g.brank = 0;
    size_t batches = 1;
    for (int i = 0; i < MAX_RANK; i++) {
        g.bdims[i] = make_fastdiv(1);
        g.b_in_str[i] = g.b_out_str[i] = 0;
    }
    for (size_t i = d.size() - 1; i-- > 0;) {  // innermost of the rest first
        if (i == c_axis) continue;
        g.bdims[g.brank] = make_fastdiv((uint32_t)d[i]);
        g.b_in_str[g.brank] = (uint32_t)si[i];
        g.b_out_str[g.brank] = (uint32_t)so[i];
        g.brank++;
        batches *= (size_t)d[i];
    }
    // A short R or C axis wastes most of a 64 x 64 tile; one element per thread in output order
    // keeps the writes dense and the reads in runs of r_len-strided segments.
    if (g.r_len < 16 || g.c_len < 16)
        return launch_copy_strided(ctx, out, in, elem_size, (int)d.size(), d.data(), so.data(), si.data());
    // Whole small matrices, contiguous on both sides: one block each through LDS.
    {
        const size_t n = (size_t)g.r_len * g.c_len;
        const uint32_t pitch = g.r_len | 1u;
        const size_t lds_bytes = (size_t)g.c_len * pitch * (size_t)elem_size;
        if (g.r_in_str == g.c_len && g.c_out_str == g.r_len && lds_bytes <= 64 * 1024 && n >= 1024 && batches <= 0x7fffffffull) {
            // every other axis must step over whole matrices: true by construction after collapsing
            // when C and R are the two innermost axes of both sides
            bool whole = c_axis + 2 == d.size();
            size_t expect = n;
            for (size_t i = c_axis; whole && i-- > 0;) {
                whole = si[i] == (int64_t)expect && so[i] == (int64_t)expect;
                expect *= (size_t)d[i];
            }
            if (whole) {
                const FastDiv cdiv = make_fastdiv(g.c_len), rdiv = make_fastdiv(g.r_len);
                const dim3 grid((unsigned)batches);
                const bool vec = elem_size == 4 && n % 4 == 0 && aligned16(out) && aligned16(in);
                // Matrices of 8192 elements and more get a block of 1024 threads (one matrix's LDS image allows two or
                // three blocks per CU: with 256 threads each the CU would be nearly empty).
                if (elem_size == 4 && vec && n >= 8192 && ctx.streaming(total * 4))
                    hipLaunchKernelGGL((transpose_small<uint32_t, 4, 1024, true>), grid, dim3(1024), lds_bytes, ctx.stream,
                                       static_cast<uint32_t *>(out), static_cast<const uint32_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                else if (elem_size == 4 && vec && n >= 8192)
                    hipLaunchKernelGGL((transpose_small<uint32_t, 4, 1024, false>), grid, dim3(1024), lds_bytes, ctx.stream,
                                       static_cast<uint32_t *>(out), static_cast<const uint32_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                else if (elem_size == 4 && vec)
                    hipLaunchKernelGGL((transpose_small<uint32_t, 4>), grid, dim3(BLOCK), lds_bytes, ctx.stream,
                                       static_cast<uint32_t *>(out), static_cast<const uint32_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                else if (elem_size == 4)
                    hipLaunchKernelGGL((transpose_small<uint32_t, 1>), grid, dim3(BLOCK), lds_bytes, ctx.stream,
                                       static_cast<uint32_t *>(out), static_cast<const uint32_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                else if (elem_size == 8)
                    hipLaunchKernelGGL((transpose_small<uint64_t, 1>), grid, dim3(BLOCK), lds_bytes, ctx.stream,
                                       static_cast<uint64_t *>(out), static_cast<const uint64_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                else
                    hipLaunchKernelGGL((transpose_small<uint8_t, 1>), grid, dim3(BLOCK), lds_bytes, ctx.stream,
                                       static_cast<uint8_t *>(out), static_cast<const uint8_t *>(in), g.r_len, g.c_len, pitch, cdiv, rdiv);
                return ctx.check(hipGetLastError(), "transpose_small launch");
            }
        }
    }
    // Dense transposed matrices with a short R axis, too large for one block: panels of 32 or 64 columns (with 16, which a
    // longer R axis would need to fit LDS, the segments read are half lines and the 64 x 64 patches are ahead).
    if (elem_size == 4 && g.c_out_str == g.r_len && g.c_len % PANEL == 0 && g.r_in_str % 4 == 0 && aligned16(out) && aligned16(in) && batches <= 65535 &&
        (size_t)PANEL * (g.r_len | 1u) * 4 <= 64 * 1024) {
        bool lines_up = true;
        for (int i = 0; i < g.brank; i++) lines_up = lines_up && g.b_in_str[i] % 4 == 0 && g.b_out_str[i] % 4 == 0;
        if (lines_up) {
            const uint32_t pitch = g.r_len | 1u;
            // twice as wide where that still fits LDS: the segments read are two whole lines
            const bool wide = g.c_len % (2 * PANEL) == 0 && (size_t)2 * PANEL * pitch * 4 <= 64 * 1024;
            const uint32_t tc = wide ? 2 * PANEL : PANEL;
            const dim3 grid((unsigned)(g.c_len / tc), (unsigned)batches);
            const size_t lds_bytes = (size_t)tc * pitch * 4;
            const FastDiv rdiv = make_fastdiv(g.r_len);
            uint32_t *o = static_cast<uint32_t *>(out);
            const uint32_t *x = static_cast<const uint32_t *>(in);
            const bool nt = ctx.streaming(total * 4);
            if (wide && nt) hipLaunchKernelGGL((transpose_panel<2 * PANEL, true>), grid, dim3(PANEL_BLOCK), lds_bytes, ctx.stream, o, x, g, pitch, rdiv);
            else if (wide) hipLaunchKernelGGL((transpose_panel<2 * PANEL, false>), grid, dim3(PANEL_BLOCK), lds_bytes, ctx.stream, o, x, g, pitch, rdiv);
            else if (nt) hipLaunchKernelGGL((transpose_panel<PANEL, true>), grid, dim3(PANEL_BLOCK), lds_bytes, ctx.stream, o, x, g, pitch, rdiv);
            else hipLaunchKernelGGL((transpose_panel<PANEL, false>), grid, dim3(PANEL_BLOCK), lds_bytes, ctx.stream, o, x, g, pitch, rdiv);
            return ctx.check(hipGetLastError(), "transpose_panel launch");
        }
    }
    const size_t gx = (g.c_len + TILE - 1) / TILE, gy = (g.r_len + TILE - 1) / TILE;
    if (gy > 65535 || batches > 65535) {
        // Grid limits: fall back to the one-element-per-thread copy (still correct, reads uncoalesced).
        return launch_copy_strided(ctx, out, in, elem_size, (int)d.size(), d.data(), so.data(), si.data());
    }
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batches);
    switch (elem_size) {
    case 1:
        hipLaunchKernelGGL((transpose_tiled<uint8_t>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<uint8_t *>(out),
                           static_cast<const uint8_t *>(in), g);
        break;
    case 4: {
        // 16-byte loads along C where every row of a patch starts on a 16-byte boundary.  16-byte stores along R only where
        // every row of a patch starts on a 128-byte boundary as well: a wavefront's store is four 256-byte pieces, and pieces
        // that straddle lines run at half the rate of single elements ([8196, 8196]: 38 % of the HBM peak against 74 %);
        // loads do not mind.
        const bool in_lines = g.r_in_str % 32 == 0 && aligned128(in), out_lines = g.c_out_str % 32 == 0 && aligned128(out);
        bool in4 = g.c_len % 4 == 0 && g.r_in_str % 4 == 0 && aligned16(in), out4 = g.r_len % 4 == 0 && out_lines, lines = in_lines && out_lines;
        for (int i = 0; i < g.brank; i++) {
            in4 = in4 && g.b_in_str[i] % 4 == 0, out4 = out4 && g.b_out_str[i] % 32 == 0;
            lines = lines && g.b_in_str[i] % 32 == 0 && g.b_out_str[i] % 32 == 0;
        }
        uint32_t *o = static_cast<uint32_t *>(out);
        const uint32_t *x = static_cast<const uint32_t *>(in);
        const bool nt = ctx.streaming(total * 4);
        if (in4 && out4 && nt && lines) hipLaunchKernelGGL((transpose_tiled_vec4<true, true>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (in4 && out4 && nt) hipLaunchKernelGGL((transpose_tiled_vec4<true, false>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (in4 && out4 && lines) hipLaunchKernelGGL((transpose_tiled_vec4<false, true>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (in4 && out4) hipLaunchKernelGGL((transpose_tiled_vec4<false, false>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (in4 && nt) hipLaunchKernelGGL((transpose_tiled_mixed<true, true>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (in4) hipLaunchKernelGGL((transpose_tiled_mixed<true, false>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (out4 && nt) hipLaunchKernelGGL((transpose_tiled_mixed<false, true>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else if (out4) hipLaunchKernelGGL((transpose_tiled_mixed<false, false>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        else hipLaunchKernelGGL((transpose_tiled<uint32_t>), grid, dim3(BLOCK), 0, ctx.stream, o, x, g);
        break;
    }
    default:
        hipLaunchKernelGGL((transpose_tiled<uint64_t>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<uint64_t *>(out),
                           static_cast<const uint64_t *>(in), g);
        break;
    }
    return ctx.check(hipGetLastError(), "transpose_tiled launch");
}

int launch_gather(DeviceCtx &ctx, void *out, const void *data, const void *indices, int index_size, int elem_size,
                  size_t outer, size_t axis_len, size_t n_idx, size_t inner, int *bad_flag) {
    if (elem_size != 1 && elem_size != 4 && elem_size != 8) return ctx.fail(AHIP_ERR_ARG, "gather: element size must be 1, 4 or 8");
    if (index_size != 4 && index_size != 8) return ctx.fail(AHIP_ERR_ARG, "gather: indices must be i32 or i64");
    const size_t total = outer * n_idx * inner;
    if (total == 0) return AHIP_OK;
    if (axis_len == 0) return ctx.fail(AHIP_ERR_SHAPE, "gather: the gathered axis is empty");
    if (!out || !data || !indices || !bad_flag) return ctx.fail(AHIP_ERR_ARG, "gather: null pointer");
    if (int rc = fits32(ctx, std::max(total, outer * axis_len * inner), "gather")) return rc;
    // Rows of whole 16-byte units move as such (embedding rows, class tokens).
    if (elem_size == 4 && inner % 4 == 0 && aligned16(out) && aligned16(data)) {
        const FastDiv in4 = make_fastdiv((uint32_t)(inner / 4)), nd4 = make_fastdiv((uint32_t)n_idx);
        const uint32_t total4 = (uint32_t)(total / 4);
        const dim3 grid4((total4 + BLOCK - 1) / BLOCK);
        if (index_size == 8)
            hipLaunchKernelGGL((gather_rows<uint4, long long>), grid4, dim3(BLOCK), 0, ctx.stream, static_cast<uint4 *>(out),
                               static_cast<const uint4 *>(data), static_cast<const long long *>(indices), (uint32_t)axis_len,
                               (uint32_t)n_idx, in4, nd4, total4, bad_flag);
        else
            hipLaunchKernelGGL((gather_rows<uint4, int>), grid4, dim3(BLOCK), 0, ctx.stream, static_cast<uint4 *>(out),
                               static_cast<const uint4 *>(data), static_cast<const int *>(indices), (uint32_t)axis_len,
                               (uint32_t)n_idx, in4, nd4, total4, bad_flag);
        return ctx.check(hipGetLastError(), "gather launch");
    }
    const FastDiv in = make_fastdiv((uint32_t)inner), nd = make_fastdiv((uint32_t)n_idx);
    const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
#define GATHER(T, I)                                                                                                   \
    hipLaunchKernelGGL((gather_rows<T, I>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<T *>(out),                  \
                       static_cast<const T *>(data), static_cast<const I *>(indices), (uint32_t)axis_len,             \
                       (uint32_t)n_idx, in, nd, (uint32_t)total, bad_flag)
    if (index_size == 8) {
        if (elem_size == 1) GATHER(uint8_t, long long);
        else if (elem_size == 4) GATHER(uint32_t, long long);
        else GATHER(uint64_t, long long);
    } else {
        if (elem_size == 1) GATHER(uint8_t, int);
        else if (elem_size == 4) GATHER(uint32_t, int);
        else GATHER(uint64_t, int);
    }
#undef GATHER
    return ctx.check(hipGetLastError(), "gather launch");
}

int launch_where(DeviceCtx &ctx, void *out, const void *cond, const void *x, const void *y, int elem_size, int rank,
                 const int64_t *dims, const int64_t *c_strides, const int64_t *x_strides, const int64_t *y_strides) {
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "where: rank must be 0..8");
    if (elem_size != 1 && elem_size != 4 && elem_size != 8) return ctx.fail(AHIP_ERR_ARG, "where: element size must be 1, 4 or 8");
    size_t total = 1;
    for (int i = 0; i < rank; i++) {
        if (dims[i] < 0) return ctx.fail(AHIP_ERR_ARG, "where: negative extent");
        total *= (size_t)dims[i];
    }
    if (total == 0) return AHIP_OK;
    if (!out || !cond || !x || !y) return ctx.fail(AHIP_ERR_ARG, "where: null pointer");
    if (int rc = fits32(ctx, total, "where")) return rc;
    WhereGeom g;
    g.rank = rank;
    for (int i = 0; i < MAX_RANK; i++) {
        g.dims[i] = make_fastdiv(1);
        g.c_str[i] = g.x_str[i] = g.y_str[i] = 0;
    }
    for (int i = 0; i < rank; i++) {
        const int j = rank - 1 - i;
        g.dims[i] = make_fastdiv((uint32_t)dims[j]);
        g.c_str[i] = (uint32_t)c_strides[j];
        g.x_str[i] = (uint32_t)x_strides[j];
        g.y_str[i] = (uint32_t)y_strides[j];
    }
    const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
    const uint8_t *c = static_cast<const uint8_t *>(cond);
    switch (elem_size) {
    case 1:
        hipLaunchKernelGGL((where_strided<uint8_t>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<uint8_t *>(out), c,
                           static_cast<const uint8_t *>(x), static_cast<const uint8_t *>(y), g, (uint32_t)total);
        break;
    case 4:
        hipLaunchKernelGGL((where_strided<uint32_t>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<uint32_t *>(out), c,
                           static_cast<const uint32_t *>(x), static_cast<const uint32_t *>(y), g, (uint32_t)total);
        break;
    default:
        hipLaunchKernelGGL((where_strided<uint64_t>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<uint64_t *>(out), c,
                           static_cast<const uint64_t *>(x), static_cast<const uint64_t *>(y), g, (uint32_t)total);
        break;
    }
    return ctx.check(hipGetLastError(), "where launch");
}

int launch_greater(DeviceCtx &ctx, uint8_t *out, const float *a, const float *b, int rank, const int64_t *dims,
                   const int64_t *a_strides, const int64_t *b_strides) {
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "greater: rank must be 0..8");
    size_t total = 1;
    for (int i = 0; i < rank; i++) {
        if (dims[i] < 0) return ctx.fail(AHIP_ERR_ARG, "greater: negative extent");
        total *= (size_t)dims[i];
    }
    if (total == 0) return AHIP_OK;
    if (!out || !a || !b) return ctx.fail(AHIP_ERR_ARG, "greater: null pointer");
    if (int rc = fits32(ctx, total, "greater")) return rc;
    CmpGeom g;
    g.rank = rank;
    for (int i = 0; i < MAX_RANK; i++) {
        g.dims[i] = make_fastdiv(1);
        g.a_str[i] = g.b_str[i] = 0;
    }
    for (int i = 0; i < rank; i++) {
        const int j = rank - 1 - i;
        g.dims[i] = make_fastdiv((uint32_t)dims[j]);
        g.a_str[i] = (uint32_t)a_strides[j];
        g.b_str[i] = (uint32_t)b_strides[j];
    }
    hipLaunchKernelGGL(greater_strided, dim3((unsigned)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream, out, a, b,
                       g, (uint32_t)total);
    return ctx.check(hipGetLastError(), "greater launch");
}

int launch_cast(DeviceCtx &ctx, void *out, const void *in, int from_type, int to_type, size_t n) {
    if (n == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "cast: null pointer");
    const dim3 grid((unsigned)((n + BLOCK - 1) / BLOCK));
    if (grid.x == 0 || (n + BLOCK - 1) / BLOCK > 0x7fffffffull) return ctx.fail(AHIP_ERR_UNSUPPORTED, "cast: too many elements");
#define CAST(TO, FROM, B)                                                                                              \
    hipLaunchKernelGGL((cast_flat<TO, FROM, B>), grid, dim3(BLOCK), 0, ctx.stream, static_cast<TO *>(out),            \
                       static_cast<const FROM *>(in), n)
    const int F = AHIP_F32, I4 = AHIP_I32, I8 = AHIP_I64, BO = AHIP_BOOL;
    if (from_type == to_type) {
        const size_t bytes = n * (from_type == BO ? 1 : from_type == I8 ? 8 : 4);
        return ctx.check(hipMemcpyAsync(out, in, bytes, hipMemcpyDeviceToDevice, ctx.stream), "hipMemcpyAsync(cast)");
    }
    if (from_type == F && to_type == I4) CAST(int32_t, float, false);
    else if (from_type == F && to_type == I8) CAST(long long, float, false);
    else if (from_type == F && to_type == BO) CAST(uint8_t, float, true);
    else if (from_type == I4 && to_type == F) CAST(float, int32_t, false);
    else if (from_type == I4 && to_type == I8) CAST(long long, int32_t, false);
    else if (from_type == I4 && to_type == BO) CAST(uint8_t, int32_t, true);
    else if (from_type == I8 && to_type == F) CAST(float, long long, false);
    else if (from_type == I8 && to_type == I4) CAST(int32_t, long long, false);
    else if (from_type == I8 && to_type == BO) CAST(uint8_t, long long, true);
    else if (from_type == BO && to_type == F) CAST(float, uint8_t, false);
    else if (from_type == BO && to_type == I4) CAST(int32_t, uint8_t, false);
    else if (from_type == BO && to_type == I8) CAST(long long, uint8_t, false);
    else return ctx.fail(AHIP_ERR_ARG, "cast: unknown element type");
#undef CAST
    return ctx.check(hipGetLastError(), "cast launch");
}

int launch_batchnorm(DeviceCtx &ctx, float *out, const float *x, const float *scale, const float *bias, const float *mean,
                     const float *var, size_t n, size_t c, size_t hw, float eps) {
    const size_t total = n * c * hw;
    if (total == 0) return AHIP_OK;
    if (!out || !x || !scale || !bias || !mean || !var) return ctx.fail(AHIP_ERR_ARG, "batchnorm: null pointer");
    if (int rc = fits32(ctx, total, "batchnorm")) return rc;
    const FastDiv fhw = make_fastdiv((uint32_t)hw), fc = make_fastdiv((uint32_t)c);
    if (hw % 4 == 0 && aligned16(out) && aligned16(x)) {
        hipLaunchKernelGGL((batchnorm_nchw<4>), dim3((unsigned)((total / 4 + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream,
                           out, x, scale, bias, mean, var, fhw, fc, (uint32_t)total, eps);
    } else {
        hipLaunchKernelGGL((batchnorm_nchw<1>), dim3((unsigned)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream, out,
                           x, scale, bias, mean, var, fhw, fc, (uint32_t)total, eps);
    }
    return ctx.check(hipGetLastError(), "batchnorm launch");
}

int launch_im2col(DeviceCtx &ctx, float *col, const float *x, size_t batch, size_t c, size_t ih, size_t iw, size_t oh,
                  size_t ow, size_t kh, size_t kw, size_t sh, size_t sw, size_t dh, size_t dw, size_t pad_t, size_t pad_l) {
    const size_t total = batch * c * kh * kw * oh * ow;
    if (total == 0) return AHIP_OK;
    if (!col || !x) return ctx.fail(AHIP_ERR_ARG, "im2col: null pointer");
    if (int rc = fits32(ctx, std::max(total, batch * c * ih * iw), "im2col")) return rc;
    ConvGeom g;
    g.ow = make_fastdiv((uint32_t)ow);
    g.oh = make_fastdiv((uint32_t)oh);
    g.kw = make_fastdiv((uint32_t)kw);
    g.kh = make_fastdiv((uint32_t)kh);
    g.c = make_fastdiv((uint32_t)c);
    g.ih = (uint32_t)ih;
    g.iw = (uint32_t)iw;
    g.sh = (uint32_t)sh;
    g.sw = (uint32_t)sw;
    g.dh = (uint32_t)dh;
    g.dw = (uint32_t)dw;
    g.pad_t = (uint32_t)pad_t;
    g.pad_l = (uint32_t)pad_l;
    hipLaunchKernelGGL(im2col_kernel, dim3((unsigned)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream, col, x, g,
                       (uint32_t)total);
    return ctx.check(hipGetLastError(), "im2col launch");
}

int launch_maxpool(DeviceCtx &ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                   size_t kh, size_t kw, size_t sh, size_t sw, size_t pad_t, size_t pad_l) {
    const size_t total = planes * oh * ow;
    if (total == 0) return AHIP_OK;
    if (!out || !x) return ctx.fail(AHIP_ERR_ARG, "maxpool: null pointer");
    if (int rc = fits32(ctx, std::max(total, planes * ih * iw), "maxpool")) return rc;
    hipLaunchKernelGGL(maxpool_kernel, dim3((unsigned)((total + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, ctx.stream, out, x,
                       make_fastdiv((uint32_t)ow), make_fastdiv((uint32_t)oh), (uint32_t)ih, (uint32_t)iw, (uint32_t)kh,
                       (uint32_t)kw, (uint32_t)sh, (uint32_t)sw, (uint32_t)pad_t, (uint32_t)pad_l, (uint32_t)total);
    return ctx.check(hipGetLastError(), "maxpool launch");
}

int launch_resize(DeviceCtx &ctx, float *out, const float *x, size_t planes, size_t ih, size_t iw, size_t oh, size_t ow,
                  int nearest) {
    const size_t total = planes * oh * ow;
    if (total == 0) return AHIP_OK;
    if (ih == 0 || iw == 0) return ctx.fail(AHIP_ERR_SHAPE, "resize: empty input plane");
    if (!out || !x) return ctx.fail(AHIP_ERR_ARG, "resize: null pointer");
    if (int rc = fits32(ctx, std::max(total, planes * ih * iw), "resize")) return rc;
    const float sh = (float)oh / (float)ih, sw = (float)ow / (float)iw;
    const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
    if (nearest)
        hipLaunchKernelGGL((resize_kernel<true>), grid, dim3(BLOCK), 0, ctx.stream, out, x, make_fastdiv((uint32_t)ow),
                           make_fastdiv((uint32_t)oh), (uint32_t)ih, (uint32_t)iw, sh, sw, (uint32_t)total);
    else
        hipLaunchKernelGGL((resize_kernel<false>), grid, dim3(BLOCK), 0, ctx.stream, out, x, make_fastdiv((uint32_t)ow),
                           make_fastdiv((uint32_t)oh), (uint32_t)ih, (uint32_t)iw, sh, sw, (uint32_t)total);
    return ctx.check(hipGetLastError(), "resize launch");
}

}  // namespace altius
