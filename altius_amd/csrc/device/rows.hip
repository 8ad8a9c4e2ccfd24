// Softmax and LayerNormalization over the last axis for gfx950.
//
// Rows of up to 1024 elements: one 64-lane wavefront per row, the row held in
// registers (read once, written once), max / sum reductions as lane butterflies.
// Lane l owns elements (l + 64*k)*VEC .. +VEC-1, so every load instruction of
// the wave covers one contiguous 256-byte (VEC=1) or 1-KiB (VEC=4) span.
// Rows that are not whole 128-byte lines, and short rows: groups of rows staged
// through LDS, a few lanes per row.
// Rows of up to 65536 elements: one block of 192 to 1024 threads per row, the row
// in the block's registers (2 to 20 float4 per thread), the two reductions
// through LDS; rows that start anywhere are addressed as buffers from their
// first 128-byte boundary on.
// Longer rows: one block per row walking it three times (from the caches after
// the first pass), single elements up to the first 16-byte boundary and float4s
// from there.
//
// Reference arithmetic:
//   Softmax  crates/session_interpreter/src/session.rs:990-1026,
//            crates/session_interpreter/src/fast_math.rs:102-187
//   LayerNorm crates/session_interpreter/src/session.rs:1433-1486
// The per-element values follow the reference bit for bit; the row sums are
// accumulated in a different order (lane butterfly instead of 8 strided
// accumulators), which moves results by a few ulp.

#include "common.h"
#include "ctx.h"
#include "math.h"

#include <math.h>

#include <type_traits>

namespace altius {
namespace {

using namespace dev;

constexpr int BLOCK = 256;
constexpr int WAVES_PER_BLOCK = BLOCK / WAVE;

// Register image of one row spread over a wavefront.
template <int VEC, int NCH> struct RowRegs {
    float v[NCH * VEC];

    // Loads the row; slots past `len` are set to `fill`.  NT: non-temporal 16-byte accesses, for tensors
    // too large to be found in a cache by the next kernel.
    template <bool NT = false, bool FULL = false>
    __device__ __forceinline__ void load(const float *__restrict__ row, int len, int lane, float fill) {
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const int e = (lane + WAVE * k) * VEC;
            if (VEC == 4) {
                if (FULL || e < len) {
                    const float4 t = load4<NT>(row + e);
                    v[k * VEC + 0] = t.x;
                    v[k * VEC + 1 % VEC] = t.y;
                    v[k * VEC + 2 % VEC] = t.z;
                    v[k * VEC + 3 % VEC] = t.w;
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; j++) v[k * VEC + j] = fill;
                }
            } else {
                v[k] = e < len ? row[e] : fill;
            }
        }
    }
    template <bool NT = false, bool FULL = false>
    __device__ __forceinline__ void store(float *__restrict__ row, int len, int lane) const {
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const int e = (lane + WAVE * k) * VEC;
            if (FULL || e < len) {
                if (VEC == 4) {
                    float4 t;
                    t.x = v[k * VEC + 0];
                    t.y = v[k * VEC + 1 % VEC];
                    t.z = v[k * VEC + 2 % VEC];
                    t.w = v[k * VEC + 3 % VEC];
                    store4<NT>(row + e, t);
                } else {
                    row[e] = v[k];
                }
            }
        }
    }
    // Element index of slot s, for per-column operands.
    static __device__ __forceinline__ int index(int lane, int s) {
        return (lane + WAVE * (s / VEC)) * VEC + (s % VEC);
    }
};

// ---------------------------------------------------------------------------
// Softmax
// ---------------------------------------------------------------------------
// What may happen to the scores on their way into Softmax, in this order: a multiplication or
// division by one value (the 1/sqrt(d) of attention), then the addition of a mask that holds one
// row per `rows_per_mask` consecutive score rows ([N,1,1,C] onto [N,H,R,C]: H*R rows).  Each is the
// single IEEE operation the stand-alone Mul / Div / Add kernel performs, so Softmax sees the same
// bits; what disappears is one pass over the scores per operation.
struct SoftmaxPrologue {
    int scale_code;  // 0: none, 1: x * scale, 2: x / scale
    float scale;
    const float *mask;  // null: none
    uint32_t rows_per_mask;
    uint32_t mask_rows;
};

// FULL: the row fills every slot (len == NCH * 64 * VEC: 256, 512, 768, 1024), known when the kernel is built, so
// that no load, store or summand is guarded: 36 of the 311 vector instructions of a 768-element row are such guards.
template <int VEC, int NCH, bool PRO, bool NT, bool FULL = false>
__global__ __launch_bounds__(BLOCK) void softmax_wave(float *__restrict__ out, const float *__restrict__ in,
                                                      size_t rows, int len_arg, const SoftmaxPrologue pro) {
    const int len = FULL ? NCH * WAVE * VEC : len_arg;
    const int lane = threadIdx.x & (WAVE - 1);
    const size_t row = (size_t)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *x = in + row * (size_t)len;
    float *o = out + row * (size_t)len;

    RowRegs<VEC, NCH> r;
    const float nan = __builtin_nanf("");
    r.template load<NT, FULL>(x, len, lane, nan);
    if (PRO) {
        // The mask row is shared by rows_per_mask score rows: it comes from the caches, and its load
        // is issued before the scores are looked at.
        RowRegs<VEC, NCH> m;
        if (pro.mask) m.template load<false, FULL>(pro.mask + (size_t)((uint32_t)row / pro.rows_per_mask) * len, len, lane, 0.0f);
        if (pro.scale_code == 1) {
#pragma unroll
            for (int s = 0; s < NCH * VEC; s++) r.v[s] = r.v[s] * pro.scale;
        } else if (pro.scale_code == 2) {
#pragma unroll
            for (int s = 0; s < NCH * VEC; s++) r.v[s] = r.v[s] / pro.scale;
        }
        if (pro.mask) {
#pragma unroll
            for (int s = 0; s < NCH * VEC; s++) r.v[s] = r.v[s] + m.v[s];  // slots past the row stay NaN
        }
    }

    float mx = nan;  // fold(NAN, max): NaN elements are ignored
#pragma unroll
    for (int s = 0; s < NCH * VEC; s++) mx = nanmax(r.v[s], mx);
    mx = wave_reduce<MaxOp>(mx);

    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < NCH * VEC; s++) {
        const bool valid = FULL || RowRegs<VEC, NCH>::index(lane, s) < len;
        const float e = softmax_exp(r.v[s], mx);
        r.v[s] = e;
        sum += valid ? e : 0.0f;
    }
    sum = wave_reduce<SumOp>(sum);
    const float recip = 1.0f / sum;
#pragma unroll
    for (int s = 0; s < NCH * VEC; s++) r.v[s] *= recip;
    r.template store<NT, FULL>(o, len, lane);
}

// Rows whose length is not a multiple of 4 (197 tokens, say) start at addresses
// that are only 4-byte aligned, and a wave per row would leave a quarter of its
// lanes idle in the last chunk.  This kernel decouples the memory layout from
// the compute layout through LDS.  A block of 16 wavefronts takes a group of
// consecutive rows whose span starts and ends on a 128-byte boundary (32 rows
// when the length is odd), so no cache line is shared between blocks or between
// the load/store instructions of different waves:
//   1. the span is copied to LDS with 16-byte loads, thread t taking float4
//      t and t + 1024; both loads are issued before the first LDS write.
//      Measured on this part: copy bandwidth falls with the number of loads a
//      wave issues back to back (6.6 TB/s at 1-2, 6.1 at 4, 5.5 at 13) and with
//      spans that share cache lines between waves, hence wide blocks, shallow
//      bursts and line-aligned groups;
//   2. rows are processed from LDS with SUB = 16, 32 or 64 lanes per row
//      (64/SUB rows per wave pass, passes dealt round-robin to the waves), NCH
//      chunks per lane, max and sum all-reduced inside each lane group with DPP
//      rotations; results overwrite the row in LDS;
//   3. the span is written back with 16-byte stores.
// With SUB*NCH just above the row length nearly every lane slot of the
// arithmetic does useful work (197 -> 16 x 13 = 208 slots).
constexpr int LDS_BLOCK = 1024;                                      // threads of the wide block; the narrow one has half
constexpr int STAGE_LDS = 2;                                         // float4 per lane staged through registers
constexpr size_t LDS_GROUP_FLOATS = (size_t)STAGE_LDS * LDS_BLOCK * 4;  // 8192 floats = 32 KiB of LDS at most

template <int BT, int SUB, int NCH, bool NT, bool PRO>
__global__ __launch_bounds__(BT) void softmax_lds(float *__restrict__ out, const float *__restrict__ in,
                                                         size_t rows, int len, int group_rows, const SoftmaxPrologue pro) {
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const size_t row0 = (size_t)blockIdx.x * group_rows;
    const int nrows = rows - row0 < (size_t)group_rows ? (int)(rows - row0) : group_rows;
    const int n = nrows * len;
    const int n4 = n >> 2;
    const float *src = in + row0 * (size_t)len;
    float *dst = out + row0 * (size_t)len;

    // Whether float4 number tid + 1024u exists is decided per block (scalar branch) except for the
    // one partially filled step.
    float4 stage[STAGE_LDS];
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        const float *p = src + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            stage[u] = load4<NT>(p);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) stage[u] = load4<NT>(p);
        }
    }
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        float *q = lds + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            *reinterpret_cast<float4 *>(q) = stage[u];
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) *reinterpret_cast<float4 *>(q) = stage[u];
        }
    }
    for (int i = (n4 << 2) + tid; i < n; i += BT) lds[i] = src[i];  // ragged end of the last group
    // The group's rows use at most two consecutive mask rows (the host checks rows_per_mask >=
    // group_rows); they go to LDS behind the scores, once per block.
    float *mask_lds = lds + (size_t)group_rows * len;
    uint32_t second_mask_from = 0xFFFFFFFFu;  // first row of the group (block-relative) that uses the second mask row
    if (PRO && pro.mask) {
        const uint32_t m0 = (uint32_t)(row0 / pro.rows_per_mask);
        const size_t boundary = (size_t)(m0 + 1) * pro.rows_per_mask;  // first score row of mask row m0 + 1
        const bool two = boundary < row0 + (size_t)nrows;
        if (two) second_mask_from = (uint32_t)(boundary - row0);
        const int count = two ? 2 * len : len;
        const float *m = pro.mask + (size_t)m0 * len;
        for (int i = tid; i < count; i += BT) mask_lds[i] = m[i];
    }
    __syncthreads();

    constexpr int RPP = WAVE / SUB;  // rows per wave pass
    constexpr int LAST = NCH - 1;    // NCH == ceil(len / SUB): only the last chunk can be partial
    const int s = lane & (SUB - 1);
    const int rr = lane / SUB;
    const bool last_valid = s + SUB * LAST < len;
    const float nan = __builtin_nanf("");
    for (int r0 = wave * RPP; r0 < nrows; r0 += (BT / WAVE) * RPP) {
        // Lane groups past the end of a ragged last group redo its last row: they compute and
        // store the same values as the group that owns it.
        const int r = r0 + rr < nrows ? r0 + rr : nrows - 1;
        float *row = lds + r * len + s;

        float x[NCH];
#pragma unroll
        for (int k = 0; k < LAST; k++) x[k] = row[SUB * k];
        x[LAST] = last_valid ? row[SUB * LAST] : nan;
        if (PRO) {
            if (pro.scale_code == 1) {
#pragma unroll
                for (int k = 0; k < NCH; k++) x[k] = x[k] * pro.scale;
            } else if (pro.scale_code == 2) {
#pragma unroll
                for (int k = 0; k < NCH; k++) x[k] = x[k] / pro.scale;
            }
            if (pro.mask) {
                const float *mrow = mask_lds + ((uint32_t)r >= second_mask_from ? len : 0) + s;
#pragma unroll
                for (int k = 0; k < LAST; k++) x[k] = x[k] + mrow[SUB * k];
                if (last_valid) x[LAST] = x[LAST] + mrow[SUB * LAST];
            }
        }
        float mx = nan;  // fold(NAN, max): NaN elements are ignored
#pragma unroll
        for (int k = 0; k < NCH; k++) mx = nanmax(x[k], mx);
        mx = subwave_allreduce<MaxOp, SUB>(mx);

        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            x[k] = softmax_exp(x[k], mx);
            sum += (k < LAST || last_valid) ? x[k] : 0.0f;
        }
        sum = subwave_allreduce<SumOp, SUB>(sum);
        const float recip = 1.0f / sum;
#pragma unroll
        for (int k = 0; k < LAST; k++) row[SUB * k] = x[k] * recip;
        if (last_valid) row[SUB * LAST] = x[LAST] * recip;
    }
    __syncthreads();

#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        const float *q = lds + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            stage[u] = *reinterpret_cast<const float4 *>(q);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) stage[u] = *reinterpret_cast<const float4 *>(q);
        }
    }
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        float *p = dst + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            store4<NT>(p, stage[u]);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) store4<NT>(p, stage[u]);
        }
    }
    for (int i = (n4 << 2) + tid; i < n; i += BT) dst[i] = lds[i];
}

// LayerNormalization of rows that a wavefront per row with 16-byte accesses does not fit (not whole float4s, or
// short): the same staging as softmax_lds (a line-aligned group of rows through LDS, 16-byte global accesses), SUB
// lanes per row with the row in NCH registers per lane, read from LDS once and written back once.  A lane works on
// the same columns of every row it meets, so its scale and bias values are read once per block (from LDS, where they
// are staged with coalesced loads).
// Two blocks of sixteen wavefronts share a CU (one loads or stores while the other computes), which leaves each lane
// 64 registers: the second launch bound says so to the register allocator.
template <int BT, int SUB, int NCH, bool NT>
__global__ __launch_bounds__(BT, 8) void layernorm_lds(float *__restrict__ out, const float *__restrict__ in,
                                                           const float *__restrict__ gamma, const float *__restrict__ beta, size_t rows,
                                                           int len, int group_rows, float eps) {
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const size_t row0 = (size_t)blockIdx.x * group_rows;
    const int nrows = rows - row0 < (size_t)group_rows ? (int)(rows - row0) : group_rows;
    const int n = nrows * len;
    const int n4 = n >> 2;
    const float *src = in + row0 * (size_t)len;
    float *dst = out + row0 * (size_t)len;
    float4 stage[STAGE_LDS];
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        const float *p = src + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            stage[u] = load4<NT>(p);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) stage[u] = load4<NT>(p);
        }
    }
    constexpr int RPP = WAVE / SUB;  // rows per wave pass
    constexpr int LAST = NCH - 1;    // NCH == ceil(len / SUB): only the last chunk can be partial
    const int s = lane & (SUB - 1);
    const int rr = lane / SUB;
    const bool last_valid = s + SUB * LAST < len;
    // Scale and bias go to LDS behind the rows with coalesced loads, once per block, and from there into each
    // lane's registers.
    float *g_lds = lds + (size_t)group_rows * len, *b_lds = g_lds + len;
    for (int i = tid; i < len; i += BT) g_lds[i] = gamma[i], b_lds[i] = beta[i];
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        float *q = lds + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            *reinterpret_cast<float4 *>(q) = stage[u];
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) *reinterpret_cast<float4 *>(q) = stage[u];
        }
    }
    for (int i = (n4 << 2) + tid; i < n; i += BT) lds[i] = src[i];  // ragged end of the last group
    __syncthreads();

    // Up to 10 chunks the lane's scale and bias values stay in registers for all of its rows; beyond that they would
    // not fit beside the row (64 registers per lane) and are read from LDS where they are used.
    constexpr bool GB_REGS = NCH <= 10;
    constexpr int NGB = GB_REGS ? NCH : 1;
    float g[NGB], b[NGB];
    if (GB_REGS) {
#pragma unroll
        for (int k = 0; k < NGB; k++) {
            const bool valid = k < LAST || last_valid;
            g[k] = valid ? g_lds[s + SUB * k] : 0.0f;
            b[k] = valid ? b_lds[s + SUB * k] : 0.0f;
        }
    }
    const float inv_n = 1.0f / (float)len;
    for (int r0 = wave * RPP; r0 < nrows; r0 += (BT / WAVE) * RPP) {
        // Lane groups past the end of a ragged last group redo its last row: they compute and store the same
        // values as the group that owns it.
        const int r = r0 + rr < nrows ? r0 + rr : nrows - 1;
        float *row = lds + r * len + s;
        float x[NCH];
#pragma unroll
        for (int k = 0; k < LAST; k++) x[k] = row[SUB * k];
        x[LAST] = last_valid ? row[SUB * LAST] : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < NCH; k++) sum += x[k];
        const float mean = subwave_allreduce<SumOp, SUB>(sum) * inv_n;
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            x[k] = x[k] - mean;
            const float d2 = x[k] * x[k];
            ss += (k < LAST || last_valid) ? d2 : 0.0f;
        }
        ss = subwave_allreduce<SumOp, SUB>(ss);
        const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            if (k < LAST || last_valid) {
                const float gk = GB_REGS ? g[GB_REGS ? k : 0] : g_lds[s + SUB * k];
                const float bk = GB_REGS ? b[GB_REGS ? k : 0] : b_lds[s + SUB * k];
                row[SUB * k] = __builtin_fmaf(x[k] * inv_std, gk, bk);
            }
        }
    }
    __syncthreads();

#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        const float *q = lds + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            stage[u] = *reinterpret_cast<const float4 *>(q);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) stage[u] = *reinterpret_cast<const float4 *>(q);
        }
    }
#pragma unroll
    for (int u = 0; u < STAGE_LDS; u++) {
        float *p = dst + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            store4<NT>(p, stage[u]);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) store4<NT>(p, stage[u]);
        }
    }
    for (int i = (n4 << 2) + tid; i < n; i += BT) dst[i] = lds[i];
}

// Sum or maximum of every row, for rows that are short or not whole float4s (7 x 7 feature maps, 197 tokens): a
// wavefront per row would leave most lanes idle and read 4 bytes per lane.  Same staging as softmax_lds: a
// line-aligned group of rows goes to LDS with 16-byte loads, then SUB lanes fold each row and lane 0 of the group
// writes out[row] (times `scale` for a mean).
template <int BT, int ST, class OP, int SUB, bool SCALE, bool NT>
__global__ __launch_bounds__(BT) void reduce_rows_lds(float *__restrict__ out, const float *__restrict__ in, size_t rows,
                                                             int len, int group_rows, float scale) {
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const size_t row0 = (size_t)blockIdx.x * group_rows;
    const int nrows = rows - row0 < (size_t)group_rows ? (int)(rows - row0) : group_rows;
    const int n = nrows * len;
    const int n4 = n >> 2;
    const float *src = in + row0 * (size_t)len;
    float4 stage[ST];
#pragma unroll
    for (int u = 0; u < ST; u++) {
        const float *p = src + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            stage[u] = load4<NT>(p);
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) stage[u] = load4<NT>(p);
        }
    }
#pragma unroll
    for (int u = 0; u < ST; u++) {
        float *q = lds + 4 * (tid + BT * u);
        if (BT * (u + 1) <= n4) {
            *reinterpret_cast<float4 *>(q) = stage[u];
        } else if (BT * u < n4) {
            if (tid + BT * u < n4) *reinterpret_cast<float4 *>(q) = stage[u];
        }
    }
    for (int i = (n4 << 2) + tid; i < n; i += BT) lds[i] = src[i];  // ragged end of the last group
    __syncthreads();

    constexpr int RPP = WAVE / SUB;  // rows per wave pass
    const int s = lane & (SUB - 1);
    const int rr = lane / SUB;
    for (int r0 = wave * RPP; r0 < nrows; r0 += (BT / WAVE) * RPP) {
        const int r = r0 + rr < nrows ? r0 + rr : nrows - 1;  // lane groups past the end redo the last row and write nothing
        const float *row = lds + r * len;
        float acc = OP::identity();
        for (int k = s; k < len; k += SUB) acc = OP::apply(acc, row[k]);
        acc = subwave_allreduce<OP, SUB>(acc);
        if (s == 0 && r0 + rr < nrows) out[row0 + r] = SCALE ? acc * scale : acc;
    }
}

// One block per row, any length and any 4-byte alignment: max pass, sum pass, write pass.  Every pass walks the row as
// `head` single elements up to the first 16-byte boundary, a body of whole float4s with four loads in flight per thread,
// and up to three single elements at the end; the second and third pass find the row in the caches (a row that does
// not fit them would have to be read three times by any kernel that cannot hold it).  SAME: the output row starts at
// the same offset from a 16-byte boundary as the input row, so the body is stored as float4s too.
// The shape of a row as the streaming kernels walk it.
struct RowWalk {
    uint32_t head, tail;
    size_t body4;
    __device__ __forceinline__ RowWalk(const float *x, size_t len) {
        const size_t lead = (4 - ((reinterpret_cast<uintptr_t>(x) >> 2) & 3)) & 3;
        head = (uint32_t)(lead < len ? lead : len);
        body4 = (len - head) >> 2;
        tail = (uint32_t)(len - head - (body4 << 2));
    }
};

// Folds f(element) over the row into `acc` with `join`; f4 handles a float4 of the body.
template <int THREADS, class F1, class F4>
__device__ __forceinline__ void walk_row(const float *__restrict__ x, const RowWalk &w, F1 one, F4 four) {
    const uint32_t tid = threadIdx.x;
    if (tid < w.head) one(x[tid], (size_t)tid);
    const float *body = x + w.head;
    size_t i = tid;
    for (; i + 3 * (size_t)THREADS < w.body4; i += 4 * (size_t)THREADS) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const float4 *>(body + 4 * (i + u * (size_t)THREADS));
#pragma unroll
        for (int u = 0; u < 4; u++) four(v[u], w.head + 4 * (i + u * (size_t)THREADS));
    }
    for (; i < w.body4; i += THREADS) four(*reinterpret_cast<const float4 *>(body + 4 * i), w.head + 4 * i);
    if (tid < w.tail) {
        const size_t at = w.head + (w.body4 << 2) + tid;
        one(x[at], at);
    }
}

template <int THREADS, bool NT>
__global__ __launch_bounds__(THREADS) void softmax_block_stream(float *__restrict__ out, const float *__restrict__ in, size_t len) {
    __shared__ float lds[THREADS / WAVE];
    const float *x = in + (size_t)blockIdx.x * len;
    float *o = out + (size_t)blockIdx.x * len;
    const RowWalk w(x, len);
    const bool same = ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(o)) & 15u) == 0;

    float mx = __builtin_nanf("");
    walk_row<THREADS>(x, w, [&](float v, size_t) { mx = nanmax(v, mx); },
                      [&](const float4 &v, size_t) { mx = nanmax(nanmax(v.x, v.y), nanmax(nanmax(v.z, v.w), mx)); });
    mx = block_reduce<MaxOp, THREADS / WAVE>(mx, lds);

    float sum = 0.0f;
    walk_row<THREADS>(x, w, [&](float v, size_t) { sum += softmax_exp(v, mx); },
                      [&](const float4 &v, size_t) {
                          sum += (softmax_exp(v.x, mx) + softmax_exp(v.y, mx)) + (softmax_exp(v.z, mx) + softmax_exp(v.w, mx));
                      });
    sum = block_reduce<SumOp, THREADS / WAVE>(sum, lds);
    const float recip = 1.0f / sum;

    walk_row<THREADS>(x, w, [&](float v, size_t at) { o[at] = softmax_exp(v, mx) * recip; },
                      [&](const float4 &v, size_t at) {
                          const float4 e = make_float4(softmax_exp(v.x, mx) * recip, softmax_exp(v.y, mx) * recip,
                                                       softmax_exp(v.z, mx) * recip, softmax_exp(v.w, mx) * recip);
                          if (same) {
                              store4<NT>(o + at, e);
                          } else {
                              o[at] = e.x, o[at + 1] = e.y, o[at + 2] = e.z, o[at + 3] = e.w;
                          }
                      });
}

// ---------------------------------------------------------------------------
// LayerNormalization
// ---------------------------------------------------------------------------
template <int VEC, int NCH, bool NT, bool FULL = false>
__global__ __launch_bounds__(BLOCK) void layernorm_wave(float *__restrict__ out, const float *__restrict__ in,
                                                        const float *__restrict__ gamma,
                                                        const float *__restrict__ beta, size_t rows, int len_arg,
                                                        float eps) {
    const int len = FULL ? NCH * WAVE * VEC : len_arg;  // see softmax_wave
    const int lane = threadIdx.x & (WAVE - 1);
    size_t row = (size_t)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
    constexpr bool EARLY = NCH <= 4;
    // Rows of two chunks and more (whole float4s): the block's four wavefronts fetch scale and bias once between them
    // and pass them on through LDS (a wavefront of its own reads 2 x the row's bytes of them from the caches per
    // row): 512 / 768 / 1024 elements gain about one point of the HBM peak, 384 two; with one chunk (256) the barrier
    // costs 3.  Up to four chunks they are read back into registers at once (SHARE); with five they wait in the
    // requesting thread's registers during the reductions and go through LDS just before they are used (LATE).
    constexpr bool SHARE = EARLY && VEC == 4 && NCH >= 2;
    constexpr bool LATE = !EARLY && VEC == 4;
    constexpr int GB = 2 * NCH * WAVE;  // float4s of scale and bias
    __shared__ float4 gb_lds[SHARE || LATE ? GB : 1];
    auto fetch_gb = [&](int i) {
        const int e = 4 * (i < NCH * WAVE ? i : i - NCH * WAVE);
        return FULL || e < len ? *reinterpret_cast<const float4 *>((i < NCH * WAVE ? gamma : beta) + e) : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    const bool active = row < rows;
    if (!SHARE && !LATE && !active) return;
    if (!active) row = rows - 1;  // keeps the block's barrier company; stores nothing
    const float *x = in + row * (size_t)len;
    float *o = out + row * (size_t)len;

    RowRegs<VEC, NCH> r;
    r.template load<NT, FULL>(x, len, lane, 0.0f);
    // Scale and bias are requested right behind the row, so that they arrive during the two reductions.
    RowRegs<VEC, EARLY ? NCH : 1> g, b;
    constexpr int STAGED = LATE ? (GB + BLOCK - 1) / BLOCK : 1;
    float4 staged[STAGED];
    if (SHARE) {
        for (int i = threadIdx.x; i < GB; i += BLOCK) gb_lds[i] = fetch_gb(i);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const float4 gv = gb_lds[lane + WAVE * k], bv = gb_lds[NCH * WAVE + lane + WAVE * k];
            g.v[(k * 4 + 0) % (EARLY ? NCH * VEC : 1)] = gv.x, g.v[(k * 4 + 1) % (EARLY ? NCH * VEC : 1)] = gv.y;
            g.v[(k * 4 + 2) % (EARLY ? NCH * VEC : 1)] = gv.z, g.v[(k * 4 + 3) % (EARLY ? NCH * VEC : 1)] = gv.w;
            b.v[(k * 4 + 0) % (EARLY ? NCH * VEC : 1)] = bv.x, b.v[(k * 4 + 1) % (EARLY ? NCH * VEC : 1)] = bv.y;
            b.v[(k * 4 + 2) % (EARLY ? NCH * VEC : 1)] = bv.z, b.v[(k * 4 + 3) % (EARLY ? NCH * VEC : 1)] = bv.w;
        }
        if (!active) return;
    } else if (LATE) {
#pragma unroll
        for (int u = 0; u < STAGED; u++) {
            const int i = threadIdx.x + u * BLOCK;
            if (i < GB) staged[u] = fetch_gb(i);
        }
    } else if (EARLY) {
        g.template load<false, FULL>(gamma, len, lane, 0.0f);
        b.template load<false, FULL>(beta, len, lane, 0.0f);
    }

    const float inv_n = 1.0f / (float)len;
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < NCH * VEC; s++) sum += r.v[s];
    const float mean = wave_reduce<SumOp>(sum) * inv_n;

    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < NCH * VEC; s++) {
        const bool valid = FULL || RowRegs<VEC, NCH>::index(lane, s) < len;
        const float d = r.v[s] - mean;
        r.v[s] = d;
        ss += valid ? d * d : 0.0f;
    }
    ss = wave_reduce<SumOp>(ss);
    const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));

    if (EARLY) {
#pragma unroll
        for (int s = 0; s < NCH * VEC; s++) r.v[s] = __builtin_fmaf(r.v[s] * inv_std, g.v[EARLY ? s : 0], b.v[EARLY ? s : 0]);
    } else if (LATE) {
#pragma unroll
        for (int u = 0; u < STAGED; u++) {
            const int i = threadIdx.x + u * BLOCK;
            if (i < GB) gb_lds[i] = staged[u];
        }
        __syncthreads();
        if (!active) return;
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const float4 gv = gb_lds[lane + WAVE * k], bv = gb_lds[NCH * WAVE + lane + WAVE * k];
            r.v[(k * 4 + 0) % (NCH * VEC)] = __builtin_fmaf(r.v[(k * 4 + 0) % (NCH * VEC)] * inv_std, gv.x, bv.x);
            r.v[(k * 4 + 1) % (NCH * VEC)] = __builtin_fmaf(r.v[(k * 4 + 1) % (NCH * VEC)] * inv_std, gv.y, bv.y);
            r.v[(k * 4 + 2) % (NCH * VEC)] = __builtin_fmaf(r.v[(k * 4 + 2) % (NCH * VEC)] * inv_std, gv.z, bv.z);
            r.v[(k * 4 + 3) % (NCH * VEC)] = __builtin_fmaf(r.v[(k * 4 + 3) % (NCH * VEC)] * inv_std, gv.w, bv.w);
        }
    } else {
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const int e = (lane + WAVE * k) * VEC;
            if (FULL || e < len) {
#pragma unroll
                for (int j = 0; j < VEC; j++) r.v[k * VEC + j] = __builtin_fmaf(r.v[k * VEC + j] * inv_std, gamma[e + j], beta[e + j]);
            }
        }
    }
    r.template store<NT, FULL>(o, len, lane);
}

// One block per row, any length and alignment: sum pass, squared-deviation pass, write pass (see softmax_block_stream).
// Scale and bias are read as float4s where the row's body lines up with theirs.
template <int THREADS, bool NT>
__global__ __launch_bounds__(THREADS) void layernorm_block_stream(float *__restrict__ out, const float *__restrict__ in,
                                                                  const float *__restrict__ gamma, const float *__restrict__ beta,
                                                                  size_t len, float eps) {
    __shared__ float lds[THREADS / WAVE];
    const float *x = in + (size_t)blockIdx.x * len;
    float *o = out + (size_t)blockIdx.x * len;
    const RowWalk w(x, len);
    const bool same = ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(o)) & 15u) == 0;
    // gamma + head and beta + head are 16-byte aligned
    const bool gb4 = ((reinterpret_cast<uintptr_t>(gamma + w.head) | reinterpret_cast<uintptr_t>(beta + w.head)) & 15u) == 0;
    const float inv_n = 1.0f / (float)len;

    float sum = 0.0f;
    walk_row<THREADS>(x, w, [&](float v, size_t) { sum += v; }, [&](const float4 &v, size_t) { sum += (v.x + v.y) + (v.z + v.w); });
    const float mean = block_reduce<SumOp, THREADS / WAVE>(sum, lds) * inv_n;

    float ss = 0.0f;
    walk_row<THREADS>(x, w,
                      [&](float v, size_t) {
                          const float d = v - mean;
                          ss += d * d;
                      },
                      [&](const float4 &v, size_t) {
                          const float a = v.x - mean, b = v.y - mean, c = v.z - mean, d = v.w - mean;
                          ss += (a * a + b * b) + (c * c + d * d);
                      });
    ss = block_reduce<SumOp, THREADS / WAVE>(ss, lds);
    const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));

    walk_row<THREADS>(x, w, [&](float v, size_t at) { o[at] = __builtin_fmaf((v - mean) * inv_std, gamma[at], beta[at]); },
                      [&](const float4 &v, size_t at) {
                          float4 g, b;
                          if (gb4) {
                              g = *reinterpret_cast<const float4 *>(gamma + at), b = *reinterpret_cast<const float4 *>(beta + at);
                          } else {
                              g = make_float4(gamma[at], gamma[at + 1], gamma[at + 2], gamma[at + 3]);
                              b = make_float4(beta[at], beta[at + 1], beta[at + 2], beta[at + 3]);
                          }
                          const float4 e = make_float4(__builtin_fmaf((v.x - mean) * inv_std, g.x, b.x), __builtin_fmaf((v.y - mean) * inv_std, g.y, b.y),
                                                       __builtin_fmaf((v.z - mean) * inv_std, g.z, b.z), __builtin_fmaf((v.w - mean) * inv_std, g.w, b.w));
                          if (same) {
                              store4<NT>(o + at, e);
                          } else {
                              o[at] = e.x, o[at + 1] = e.y, o[at + 2] = e.z, o[at + 3] = e.w;
                          }
                      });
}

// Long rows that are whole float4s: a block of THREADS threads per row with the row in registers (NCH float4 per
// thread, read once); the two reductions go through LDS.  Few loads per thread and many threads per row: on this
// part a wavefront that issues many 16-byte loads back to back streams more slowly than many wavefronts issuing a
// few each.
template <int THREADS, int NCH, bool NT>
__global__ __launch_bounds__(THREADS) void softmax_block_regs(float *__restrict__ out, const float *__restrict__ in, size_t len) {
    __shared__ float lds[THREADS / WAVE];
    const float *x = in + (size_t)blockIdx.x * len;
    float *o = out + (size_t)blockIdx.x * len;
    const float nan = __builtin_nanf("");
    // Element indices inside a row (at most 65536 elements): 32-bit from four float4 per thread on; below that the
    // 64-bit ones, which the compiler folds into the addresses, are 5 points of the HBM peak ahead.
    using idx_t = std::conditional_t<(NCH >= 4), int, ptrdiff_t>;
    const idx_t n = (idx_t)len;
    float4 r[NCH];
    float mx = nan;  // NaN elements (and the slots past the row) are ignored by the maximum
    // At most two 16-byte loads per thread are requested at a time; with four chunks the second pair goes out
    // once the first has been folded into the maximum.
    constexpr int BURST = NCH >= 4 && NCH % 2 == 0 ? NCH / 2 : NCH;
#pragma unroll
    for (int k0 = 0; k0 < NCH; k0 += BURST) {
#pragma unroll
        for (int k = k0; k < k0 + BURST; k++) {
            const idx_t e = ((idx_t)threadIdx.x + (idx_t)THREADS * k) * 4;
            r[k] = e < n ? load4<NT>(x + e) : make_float4(nan, nan, nan, nan);
        }
#pragma unroll
        for (int k = k0; k < k0 + BURST; k++) mx = nanmax(nanmax(r[k].x, r[k].y), nanmax(nanmax(r[k].z, r[k].w), mx));
        if (BURST != NCH) asm volatile("" ::: "memory");
    }
    mx = block_reduce<MaxOp, THREADS / WAVE>(mx, lds);
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const idx_t e = ((idx_t)threadIdx.x + (idx_t)THREADS * k) * 4;
        r[k].x = softmax_exp(r[k].x, mx), r[k].y = softmax_exp(r[k].y, mx), r[k].z = softmax_exp(r[k].z, mx), r[k].w = softmax_exp(r[k].w, mx);
        if (e < n) sum += (r[k].x + r[k].y) + (r[k].z + r[k].w);
    }
    sum = block_reduce<SumOp, THREADS / WAVE>(sum, lds);
    const float recip = 1.0f / sum;
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const idx_t e = ((idx_t)threadIdx.x + (idx_t)THREADS * k) * 4;
        if (e < n) store4<NT>(o + e, make_float4(r[k].x * recip, r[k].y * recip, r[k].z * recip, r[k].w * recip));
    }
}

template <int THREADS, int NCH, bool NT>
__global__ __launch_bounds__(THREADS) void layernorm_block_regs(float *__restrict__ out, const float *__restrict__ in,
                                                                const float *__restrict__ gamma, const float *__restrict__ beta, size_t len,
                                                                float eps) {
    __shared__ float lds[THREADS / WAVE];
    const float *x = in + (size_t)blockIdx.x * len;
    float *o = out + (size_t)blockIdx.x * len;
    const float inv_n = 1.0f / (float)len;
    float4 r[NCH];
    float sum = 0.0f;
    constexpr int BURST = NCH >= 4 && NCH % 2 == 0 ? NCH / 2 : NCH;  // see softmax_block_regs
#pragma unroll
    for (int k0 = 0; k0 < NCH; k0 += BURST) {
#pragma unroll
        for (int k = k0; k < k0 + BURST; k++) {
            const size_t e = ((size_t)threadIdx.x + (size_t)THREADS * k) * 4;
            r[k] = e < len ? load4<NT>(x + e) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int k = k0; k < k0 + BURST; k++) sum += (r[k].x + r[k].y) + (r[k].z + r[k].w);
        if (BURST != NCH) asm volatile("" ::: "memory");
    }
    // Scale and bias are requested right behind the row where the registers allow it, so that they arrive during the
    // two reductions instead of after them.
    constexpr bool EARLY = NCH <= 2;  // measured: 3 to 4.5 points of the HBM peak for two float4 per thread (2048 ... 8192), 1 to 3 lost with three
    float4 g[EARLY ? NCH : 1], b[EARLY ? NCH : 1];
    if (EARLY) {
#pragma unroll
        for (int k = 0; k < NCH; k++) {
            const size_t e = ((size_t)threadIdx.x + (size_t)THREADS * k) * 4;
            g[k] = b[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < len) g[k] = *reinterpret_cast<const float4 *>(gamma + e), b[k] = *reinterpret_cast<const float4 *>(beta + e);
        }
    }
    const float mean = block_reduce<SumOp, THREADS / WAVE>(sum, lds) * inv_n;
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const bool valid = ((size_t)threadIdx.x + (size_t)THREADS * k) * 4 < len;
        r[k].x -= mean, r[k].y -= mean, r[k].z -= mean, r[k].w -= mean;
        if (valid) ss += (r[k].x * r[k].x + r[k].y * r[k].y) + (r[k].z * r[k].z + r[k].w * r[k].w);
    }
    ss = block_reduce<SumOp, THREADS / WAVE>(ss, lds);
    const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const size_t e = ((size_t)threadIdx.x + (size_t)THREADS * k) * 4;
        if (e < len) {
            if (!EARLY) g[0] = *reinterpret_cast<const float4 *>(gamma + e), b[0] = *reinterpret_cast<const float4 *>(beta + e);
            const float4 gk = g[EARLY ? k : 0], bk = b[EARLY ? k : 0];
            store4<NT>(o + e, make_float4(__builtin_fmaf(r[k].x * inv_std, gk.x, bk.x), __builtin_fmaf(r[k].y * inv_std, gk.y, bk.y),
                                          __builtin_fmaf(r[k].z * inv_std, gk.z, bk.z), __builtin_fmaf(r[k].w * inv_std, gk.w, bk.w)));
        }
    }
}

// ---------------------------------------------------------------------------
// Rows addressed as buffers
// ---------------------------------------------------------------------------
// A raw buffer's 16-byte accesses need 4-byte alignment only and are checked against the buffer's size in hardware:
// what lies past the end reads as zero and is not stored, without a branch, and one 32-bit offset per thread
// addresses the input row, the output row, scale and bias alike (the descriptors sit in scalar registers).  That is
// what rows that start anywhere need (a length that is not a multiple of 4, or a base pointer that is only 4-byte
// aligned), and what lets a thread hold two rows, or 26 float4 of one, in its registers.
//
// A row of `len` elements as its block holds it (EDGES): a head of up to 31 elements that ends at the row's first
// 128-byte boundary, one each in the block's first threads; the body, whole float4s from that boundary on, float4
// number tid + stride * k in chunk k of thread tid, so that every load and store instruction of a wavefront covers
// eight whole 128-byte lines (rows of 36 K and 50 K elements: 3 to 5 points of the HBM peak over float4s taken where
// the row starts); and a tail of up to three elements behind the body, again in the first threads.  The body's
// descriptor ends with the body, so a float4 is in range or out of range as a whole.  Without EDGES the row is all
// body: whole float4s, and 128-byte lines when its tensor is a stack of them.
typedef uint32_t u32x4_row __attribute__((ext_vector_type(4)));
typedef float f32x4_row __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ float4 load_at(__amdgpu_buffer_rsrc_t row, uint32_t byte_offset) {
    const f32x4_row f = __builtin_bit_cast(f32x4_row, __builtin_amdgcn_raw_buffer_load_b128(row, byte_offset, 0, NT ? 2 : 0));
    return make_float4(f[0], f[1], f[2], f[3]);
}
template <bool NT>
__device__ __forceinline__ void store_at(__amdgpu_buffer_rsrc_t row, uint32_t byte_offset, float4 v) {
    const f32x4_row f = {v.x, v.y, v.z, v.w};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_row, f), row, byte_offset, 0, NT ? 2 : 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_buffer(const float *row, uint32_t len) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(row), 0, (int)(len * 4u), 0x00020000);  // raw buffer of 32-bit words
}

struct RowBuf {
    const float *p;
    uint32_t len;
    uint32_t head;  // elements ahead of the body
    __device__ __forceinline__ uint32_t body() const { return (len - head) & ~3u; }
    __device__ __forceinline__ uint32_t tail() const { return (len - head) & 3u; }
    __device__ __forceinline__ __amdgpu_buffer_rsrc_t body_rsrc() const { return row_buffer(p + head, body()); }
    __device__ __forceinline__ __amdgpu_buffer_rsrc_t head_rsrc() const { return row_buffer(p, head); }
    __device__ __forceinline__ __amdgpu_buffer_rsrc_t tail_rsrc() const { return row_buffer(p + head + body(), tail()); }
};

// Elements of the row that starts at `row` ahead of its first 128-byte boundary (0 to 31).
__device__ __forceinline__ uint32_t elements_to_line(const float *row) {
    return ((128u - ((uint32_t)reinterpret_cast<uintptr_t>(row) & 127u)) & 127u) >> 2;
}

// One element of a row's head or tail per thread: element tid of the piece, zero (and nothing stored) past its end.
__device__ __forceinline__ float load_edge(__amdgpu_buffer_rsrc_t piece, uint32_t tid) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(piece, tid * 4u, 0, 0));
}
__device__ __forceinline__ void store_edge(__amdgpu_buffer_rsrc_t piece, uint32_t tid, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), piece, tid * 4u, 0, 0);
}

// Byte offset of a thread's float4 in chunk k; `stride` threads share the row.  The thread's own offset is hidden from
// the compiler's value numbering at every use: left to itself it keeps one register per chunk alive from the row's
// load to its store (18 to 26 registers of a long row) instead of an addition per access.
__device__ __forceinline__ uint32_t chunk_offset(uint32_t tid, uint32_t stride, int k) {
    uint32_t own = tid * 16u;
    asm volatile("" : "+v"(own));
    return own + (uint32_t)k * stride * 16u;
}

// `stride` threads share the row (a block's, or a wavefront's 64); tid is the thread's number among them.
template <int NCH, bool NT, bool EDGES>
__device__ __forceinline__ void request_row(float4 (&r)[NCH], float &h, float &t, const RowBuf &row, uint32_t tid, uint32_t stride) {
    const __amdgpu_buffer_rsrc_t body = row.body_rsrc();
#pragma unroll
    for (int k = 0; k < NCH; k++) r[k] = load_at<NT>(body, chunk_offset(tid, stride, k));
    h = EDGES ? load_edge(row.head_rsrc(), tid) : 0.0f;
    t = EDGES ? load_edge(row.tail_rsrc(), tid) : 0.0f;
}

template <int NCH, bool NT, bool EDGES>
__device__ __forceinline__ void store_row(const float4 (&r)[NCH], float h, float t, const RowBuf &row, uint32_t tid, uint32_t stride) {
    const __amdgpu_buffer_rsrc_t body = row.body_rsrc();
#pragma unroll
    for (int k = 0; k < NCH; k++) store_at<NT>(body, chunk_offset(tid, stride, k), r[k]);
    if (EDGES) store_edge(row.head_rsrc(), tid, h), store_edge(row.tail_rsrc(), tid, t);
}

// Reduction over a block of any whole number of wavefronts (at most 16); `lds` holds 16 floats.
template <class OP> __device__ __forceinline__ float block_reduce_any(float v, float *lds) {
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    v = wave_reduce<OP>(v);
    __syncthreads();  // protects lds against a previous use
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = OP::identity();
    for (int w = 0; w < nwaves; w++) r = OP::apply(r, lds[w]);
    return r;
}

// The two reductions of a row: over the wavefront, or over the block through LDS.
template <class OP, bool WAVE_ROW> __device__ __forceinline__ float row_reduce(float v, float *lds) {
    if constexpr (WAVE_ROW) return wave_reduce<OP>(v);
    else return block_reduce_any<OP>(v, lds);
}

// Softmax of the row in r (and h, t), written to o.
template <int NCH, bool NT, bool EDGES, bool WAVE_ROW>
__device__ __forceinline__ void softmax_row_in_regs(float4 (&r)[NCH], float h, float t, const RowBuf &o, uint32_t tid, uint32_t stride, float *lds) {
    const float nan = __builtin_nanf("");
    const uint32_t body = o.body();
    float mx = nan;  // NaN elements (and the slots past the row) are ignored by the maximum
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        if ((tid + stride * k) * 4u >= body) r[k] = make_float4(nan, nan, nan, nan);
        mx = nanmax(nanmax(r[k].x, r[k].y), nanmax(nanmax(r[k].z, r[k].w), mx));
    }
    if (EDGES) {
        h = tid < o.head ? h : nan, t = tid < o.tail() ? t : nan;
        mx = nanmax(nanmax(h, t), mx);
    }
    mx = row_reduce<MaxOp, WAVE_ROW>(mx, lds);
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        r[k].x = softmax_exp(r[k].x, mx), r[k].y = softmax_exp(r[k].y, mx), r[k].z = softmax_exp(r[k].z, mx), r[k].w = softmax_exp(r[k].w, mx);
        if ((tid + stride * k) * 4u < body) sum += (r[k].x + r[k].y) + (r[k].z + r[k].w);
        __builtin_amdgcn_sched_barrier(0);  // one chunk's temporaries at a time
    }
    if (EDGES) {
        h = softmax_exp(h, mx), t = softmax_exp(t, mx);
        sum += (tid < o.head ? h : 0.0f) + (tid < o.tail() ? t : 0.0f);
    }
    sum = row_reduce<SumOp, WAVE_ROW>(sum, lds);
    const float recip = 1.0f / sum;
#pragma unroll
    for (int k = 0; k < NCH; k++) r[k] = make_float4(r[k].x * recip, r[k].y * recip, r[k].z * recip, r[k].w * recip);
    store_row<NCH, NT, EDGES>(r, h * recip, t * recip, o, tid, stride);
}

// LayerNormalization of the row in r (and h, t), written to o; scale and bias are cut into head, body and tail as the
// row is.  GB: when scale and bias are requested: 0 chunk by chunk behind the reductions, 1 between the two reductions
// (they then wait in registers during the second).
template <int NCH, bool NT, bool EDGES, bool WAVE_ROW, int GB>
__device__ __forceinline__ void layernorm_row_in_regs(float4 (&r)[NCH], float h, float t, const RowBuf &o, const RowBuf &gamma, const RowBuf &beta,
                                                      float eps, uint32_t tid, uint32_t stride, float *lds) {
    const uint32_t body = o.body();
    const float inv_n = 1.0f / (float)o.len;
    const __amdgpu_buffer_rsrc_t ob = o.body_rsrc(), gb = gamma.body_rsrc(), bb = beta.body_rsrc();
    float4 g[GB ? NCH : 1], b[GB ? NCH : 1];
    float gh = 0.0f, bh = 0.0f, gt = 0.0f, bt = 0.0f;
    auto request_gb = [&]() {
#pragma unroll
        for (int k = 0; k < (GB ? NCH : 0); k++)
            g[GB ? k : 0] = load_at<false>(gb, chunk_offset(tid, stride, k)), b[GB ? k : 0] = load_at<false>(bb, chunk_offset(tid, stride, k));
        if (EDGES) {
            gh = load_edge(gamma.head_rsrc(), tid), bh = load_edge(beta.head_rsrc(), tid);
            gt = load_edge(gamma.tail_rsrc(), tid), bt = load_edge(beta.tail_rsrc(), tid);
        }
    };
    float sum = 0.0f;  // slots past the row hold zeros
#pragma unroll
    for (int k = 0; k < NCH; k++) sum += (r[k].x + r[k].y) + (r[k].z + r[k].w);
    if (EDGES) sum += h + t;
    const float mean = row_reduce<SumOp, WAVE_ROW>(sum, lds) * inv_n;
    if (GB == 1) request_gb();
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        r[k].x -= mean, r[k].y -= mean, r[k].z -= mean, r[k].w -= mean;
        if ((tid + stride * k) * 4u < body) ss += (r[k].x * r[k].x + r[k].y * r[k].y) + (r[k].z * r[k].z + r[k].w * r[k].w);
    }
    if (EDGES) {
        h -= mean, t -= mean;
        ss += (tid < o.head ? h * h : 0.0f) + (tid < o.tail() ? t * t : 0.0f);
    }
    ss = row_reduce<SumOp, WAVE_ROW>(ss, lds);
    const float inv_std = 1.0f / sqrtf(__builtin_fmaf(ss, inv_n, eps));
    if (GB == 0) request_gb();  // the edges' scale and bias only
#pragma unroll
    for (int k = 0; k < NCH; k++) {
        const float4 gk = GB ? g[GB ? k : 0] : load_at<false>(gb, chunk_offset(tid, stride, k));
        const float4 bk = GB ? b[GB ? k : 0] : load_at<false>(bb, chunk_offset(tid, stride, k));
        store_at<NT>(ob, chunk_offset(tid, stride, k),
                     make_float4(__builtin_fmaf(r[k].x * inv_std, gk.x, bk.x), __builtin_fmaf(r[k].y * inv_std, gk.y, bk.y),
                                 __builtin_fmaf(r[k].z * inv_std, gk.z, bk.z), __builtin_fmaf(r[k].w * inv_std, gk.w, bk.w)));
        if (!GB && k % 2 == 1) __builtin_amdgcn_sched_barrier(0);  // scale and bias of two chunks at a time
    }
    if (EDGES) {
        store_edge(o.head_rsrc(), tid, __builtin_fmaf(h * inv_std, gh, bh));
        store_edge(o.tail_rsrc(), tid, __builtin_fmaf(t * inv_std, gt, bt));
    }
}

// One block per row, the row wherever it starts; the block is any whole number of wavefronts (its threads share the
// row's float4s NCH each, so a row of 1025 float4 takes 576 threads and not the next power of two).
// MINW: wavefronts per SIMD to leave room for: 8 (64 registers a thread: blocks of 1024 threads fit a CU two at a time,
// and one loads or stores while the other reduces) up to eight float4 per thread; 4 (128 registers) beyond, where a row
// takes blocks of 512 threads with 18 or 20 float4 each, two to a CU, or of 1024 threads, one to a CU.
template <int NCH, bool NT, bool EDGES, int MINW>
__global__ __launch_bounds__(1024, MINW) void softmax_block_anywhere(float *__restrict__ out, const float *__restrict__ in, uint32_t len) {
    __shared__ float lds[16];
    const float *x = in + (size_t)blockIdx.x * len;
    const uint32_t head = EDGES ? elements_to_line(x) : 0;
    float4 r[NCH];
    float h, t;
    request_row<NCH, NT, EDGES>(r, h, t, RowBuf{x, len, head}, threadIdx.x, blockDim.x);
    softmax_row_in_regs<NCH, NT, EDGES, false>(r, h, t, RowBuf{out + (size_t)blockIdx.x * len, len, head}, threadIdx.x, blockDim.x, lds);
}

template <int NCH, bool NT, bool EDGES, int MINW, int GB>
__global__ __launch_bounds__(1024, MINW) void layernorm_block_anywhere(float *__restrict__ out, const float *__restrict__ in,
                                                                       const float *__restrict__ gamma, const float *__restrict__ beta, uint32_t len,
                                                                       float eps) {
    __shared__ float lds[16];
    const float *x = in + (size_t)blockIdx.x * len;
    const uint32_t head = EDGES ? elements_to_line(x) : 0;
    float4 r[NCH];
    float h, t;
    request_row<NCH, NT, EDGES>(r, h, t, RowBuf{x, len, head}, threadIdx.x, blockDim.x);
    layernorm_row_in_regs<NCH, NT, EDGES, false, GB>(r, h, t, RowBuf{out + (size_t)blockIdx.x * len, len, head}, RowBuf{gamma, len, head},
                                                     RowBuf{beta, len, head}, eps, threadIdx.x, blockDim.x, lds);
}

// The block-per-row kernels for rows that take 1024 threads and four float4 each: two such blocks are all a CU holds,
// and a block that loads its row, reduces, reduces again and stores leaves the memory pipeline idle while it reduces.
// Here a block walks rows blockIdx.x, blockIdx.x + gridDim.x, ... and requests the next row before it works on the one
// it holds; both rows fit 64 registers per thread together with everything else.  Which thread holds which elements
// and the order of every sum are those of softmax_block_regs / layernorm_block_regs: same bits.
template <int THREADS, int NCH, bool NT>
__global__ __launch_bounds__(THREADS, 2048 / THREADS * (THREADS / WAVE) / 4) void softmax_block_pipe(float *__restrict__ out, const float *__restrict__ in,
                                                                                                      uint32_t len, size_t rows) {
    __shared__ float lds[16];
    size_t row = blockIdx.x;
    const size_t step = gridDim.x;
    float4 next[NCH];
    float h, t;  // unused: these rows are whole float4s
    request_row<NCH, NT, false>(next, h, t, RowBuf{in + row * len, len, 0}, threadIdx.x, THREADS);
    while (row + step < rows) {
        float4 r[NCH];
#pragma unroll
        for (int k = 0; k < NCH; k++) r[k] = next[k];
        request_row<NCH, NT, false>(next, h, t, RowBuf{in + (row + step) * len, len, 0}, threadIdx.x, THREADS);
        softmax_row_in_regs<NCH, NT, false, false>(r, 0.0f, 0.0f, RowBuf{out + row * len, len, 0}, threadIdx.x, THREADS, lds);
        row += step;
    }
    softmax_row_in_regs<NCH, NT, false, false>(next, 0.0f, 0.0f, RowBuf{out + row * len, len, 0}, threadIdx.x, THREADS, lds);
}

template <int THREADS, int NCH, bool NT>
__global__ __launch_bounds__(THREADS, 2048 / THREADS * (THREADS / WAVE) / 4) void layernorm_block_pipe(float *__restrict__ out, const float *__restrict__ in,
                                                                                                        const float *__restrict__ gamma,
                                                                                                        const float *__restrict__ beta, uint32_t len,
                                                                                                        size_t rows, float eps) {
    __shared__ float lds[16];
    size_t row = blockIdx.x;
    const size_t step = gridDim.x;
    const RowBuf g{gamma, len, 0}, b{beta, len, 0};
    float4 next[NCH];
    float h, t;
    request_row<NCH, NT, false>(next, h, t, RowBuf{in + row * len, len, 0}, threadIdx.x, THREADS);
    while (row + step < rows) {
        float4 r[NCH];
#pragma unroll
        for (int k = 0; k < NCH; k++) r[k] = next[k];
        request_row<NCH, NT, false>(next, h, t, RowBuf{in + (row + step) * len, len, 0}, threadIdx.x, THREADS);
        layernorm_row_in_regs<NCH, NT, false, false, 0>(r, 0.0f, 0.0f, RowBuf{out + row * len, len, 0}, g, b, eps, threadIdx.x, THREADS, lds);
        row += step;
    }
    layernorm_row_in_regs<NCH, NT, false, false, 0>(next, 0.0f, 0.0f, RowBuf{out + row * len, len, 0}, g, b, eps, threadIdx.x, THREADS, lds);
}

// Threads per row and float4 per thread for a row of `len` elements in the block-per-row kernels.
struct BlockLayout {
    int threads, nch;
};
// Measured over rows of 1536 to 16384 elements: two float4 per thread is the best shape (256 x 2 to 2048 elements,
// 384 x 2 to 3072, 512 x 2 to 4096, 768 x 2 to 6144, 1024 x 2 to 8192: 79-81 % of peak for Softmax, 75-78 % for
// LayerNormalization, which then requests scale and bias behind the row; with three float4 on fewer threads
// LayerNormalization loses 2-4 points at 2560, 4608 and 5120), 1024 x 3 for 12288, and a 16 K row has to take four
// (the kernels that request a row ahead).  Fewer threads with more float4 each (512 x 4..8, 256 x 5..16) are 3-8
// points behind at every length from 5120 up.
inline BlockLayout block_layout(size_t len) {
    const size_t v = len / 4;  // float4 per row
    const int threads = v <= 512 ? 256 : v <= 768 ? 384 : v <= 1024 ? 512 : v <= 1536 ? 768 : 1024;
    int nch = (int)((v + threads - 1) / threads);
    if (nch > 4 && nch <= 16) nch = nch <= 6 ? 6 : nch <= 8 ? 8 : nch <= 12 ? 12 : 16;  // rows beyond 16 K: the layouts that exist
    return BlockLayout{threads, nch};
}

// Blocks of 1024 threads and four float4 per thread (rows of more than 12288 elements) with more than two rows each to
// walk take the kernel that requests a row ahead (`resident` = the blocks the device holds at a time): 70-72 % of the
// HBM peak become 75 % for Softmax over rows of 16384, 72-73 % become 74 % for LayerNormalization.  With two or three
// float4 per thread the plain kernels are 2-5 points ahead of it.
template <int THREADS, int NCH>
void softmax_block_go(bool nt, hipStream_t s, size_t rows, size_t resident, float *out, const float *in, size_t len) {
    if constexpr (THREADS == 1024 && NCH == 4) if (rows > 2 * resident) {
        const dim3 grid((unsigned)resident);
        if (nt) hipLaunchKernelGGL((softmax_block_pipe<THREADS, NCH, true>), grid, dim3(THREADS), 0, s, out, in, (uint32_t)len, rows);
        else hipLaunchKernelGGL((softmax_block_pipe<THREADS, NCH, false>), grid, dim3(THREADS), 0, s, out, in, (uint32_t)len, rows);
        return;
    }
    const dim3 grid((unsigned)rows);
    if (nt) hipLaunchKernelGGL((softmax_block_regs<THREADS, NCH, true>), grid, dim3(THREADS), 0, s, out, in, len);
    else hipLaunchKernelGGL((softmax_block_regs<THREADS, NCH, false>), grid, dim3(THREADS), 0, s, out, in, len);
}
// Threads of a block and float4 per thread for a row of len / 4 whole float4s that starts anywhere (the elements ahead
// of them and behind them ride along in the first threads).  The threads are the whole wavefronts that hold the row at
// the chosen float4 per thread.  Blocks of 640 to 768 threads run 2 to 4 points of the HBM peak ahead of blocks of 896
// to 1024 with fewer float4 each (three of them fit a CU where two of the larger do): Softmax takes two float4 per thread
// up to 768 threads, then the fewest that 1024 threads cover the row with; LayerNormalization, which also waits for its
// scale and bias, keeps to 768 threads (832 with four float4) up to eight float4 per thread and takes sixteen on at most
// 512 threads from there to 8 K float4.  Beyond 8 K float4 both take blocks of 512 threads with 18 or 20 each, then
// blocks of 1024 threads, one to a CU.
struct AnyLayout {
    int threads, nch;
};
inline AnyLayout any_layout(size_t len, bool layer_norm) {
    const size_t v = len / 4;
    int nch;
    if (layer_norm) nch = v <= 1536 ? 2 : v <= 2304 ? 3 : v <= 3328 ? 4 : v <= 4608 ? 6 : v <= 6144 ? 8 : v <= 8192 ? 16 : 0;
    else nch = v <= 1536 ? 2 : v <= 3072 ? 3 : v <= 4096 ? 4 : v <= 6144 ? 6 : v <= 8192 ? 8 : 0;
    if (nch) return AnyLayout{(int)(((v + nch - 1) / nch + WAVE - 1) / WAVE * WAVE), nch};
    if (v <= 512 * 18) return AnyLayout{512, 18};
    if (v <= 512 * 20) return AnyLayout{512, 20};
    return AnyLayout{1024, v <= 12288 ? 12 : v <= 13312 ? 13 : 16};
}
#define ALTIUS_ANY_LAYOUTS(L)                                                                                       \
    switch ((L).nch) {                                                                                              \
        ALTIUS_GO(2, 8) ALTIUS_GO(3, 8) ALTIUS_GO(4, 8) ALTIUS_GO(6, 8) ALTIUS_GO(8, 8)                             \
        ALTIUS_GO(12, 4) ALTIUS_GO(13, 4) ALTIUS_GO(16, 4) ALTIUS_GO(18, 4) ALTIUS_GO(20, 4)                        \
    }

// A launch with the template's flags NT and EDGES taken from run-time values; AFTER: the template arguments behind them.
#define ALTIUS_NT_EDGES(KERNEL, NCH, AFTER, ...)                                                            \
    do {                                                                                                    \
        if (nt && edges) hipLaunchKernelGGL((KERNEL<NCH, true, true, AFTER>), __VA_ARGS__);                 \
        else if (nt) hipLaunchKernelGGL((KERNEL<NCH, true, false, AFTER>), __VA_ARGS__);                    \
        else if (edges) hipLaunchKernelGGL((KERNEL<NCH, false, true, AFTER>), __VA_ARGS__);                 \
        else hipLaunchKernelGGL((KERNEL<NCH, false, false, AFTER>), __VA_ARGS__);                           \
    } while (0)
#define ALTIUS_COMMA ,

inline bool aligned128(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 127u) == 0; }

// Softmax / LayerNormalization over rows of more than 1024 and at most 65536 elements that start anywhere.
bool softmax_anywhere_launch(bool nt, hipStream_t s, size_t rows, float *out, const float *in, size_t len) {
    const bool edges = !(len % 32 == 0 && aligned128(in) && aligned128(out));  // not a stack of whole 128-byte lines
    const AnyLayout lay = any_layout(len, false);
    const dim3 grid((unsigned)rows), block((unsigned)lay.threads);
#define ALTIUS_GO(N, W)                                                                              \
    case N:                                                                                          \
        ALTIUS_NT_EDGES(softmax_block_anywhere, N, W, grid, block, 0, s, out, in, (uint32_t)len);    \
        return true;
    ALTIUS_ANY_LAYOUTS(lay)
#undef ALTIUS_GO
    return false;
}
bool layernorm_anywhere_launch(bool nt, hipStream_t s, size_t rows, float *out, const float *in, const float *gamma, const float *beta, size_t len,
                               float eps) {
    const bool edges = !(len % 32 == 0 && aligned128(in) && aligned128(out));
    const AnyLayout lay = any_layout(len, true);
    const dim3 grid((unsigned)rows), block((unsigned)lay.threads);
    // Scale and bias between the two reductions: 2 to 3.5 points of the HBM peak for blocks of up to 512 threads with
    // two float4 each (rows of up to 4 K elements), 5 lost with 640 and 768 threads; behind the reductions otherwise.
    if (lay.nch == 2 && lay.threads <= 512) {
        ALTIUS_NT_EDGES(layernorm_block_anywhere, 2, 8 ALTIUS_COMMA 1, grid, block, 0, s, out, in, gamma, beta, (uint32_t)len, eps);
        return true;
    }
#define ALTIUS_GO(N, W)                                                                                                                 \
    case N:                                                                                                                             \
        ALTIUS_NT_EDGES(layernorm_block_anywhere, N, W ALTIUS_COMMA 0, grid, block, 0, s, out, in, gamma, beta, (uint32_t)len, eps);     \
        return true;
    ALTIUS_ANY_LAYOUTS(lay)
#undef ALTIUS_GO
    return false;
}
template <int THREADS, int NCH>
void layernorm_block_go(bool nt, hipStream_t s, size_t rows, size_t resident, float *out, const float *in, const float *gamma, const float *beta,
                        size_t len, float eps) {
    if constexpr (THREADS == 1024 && NCH == 4) if (rows > 2 * resident) {
        const dim3 grid((unsigned)resident);
        if (nt) hipLaunchKernelGGL((layernorm_block_pipe<THREADS, NCH, true>), grid, dim3(THREADS), 0, s, out, in, gamma, beta, (uint32_t)len, rows, eps);
        else hipLaunchKernelGGL((layernorm_block_pipe<THREADS, NCH, false>), grid, dim3(THREADS), 0, s, out, in, gamma, beta, (uint32_t)len, rows, eps);
        return;
    }
    const dim3 grid((unsigned)rows);
    if (nt) hipLaunchKernelGGL((layernorm_block_regs<THREADS, NCH, true>), grid, dim3(THREADS), 0, s, out, in, gamma, beta, len, eps);
    else hipLaunchKernelGGL((layernorm_block_regs<THREADS, NCH, false>), grid, dim3(THREADS), 0, s, out, in, gamma, beta, len, eps);
}
// GO(THREADS, NCH) for the layout of a row; false if there is none.
#define ALTIUS_BLOCK_LAYOUTS(L)                                                          \
    switch ((L).threads * 100 + (L).nch) {                                               \
        ALTIUS_GO(256, 2) ALTIUS_GO(384, 2) ALTIUS_GO(512, 2) ALTIUS_GO(768, 2) ALTIUS_GO(1024, 2) ALTIUS_GO(1024, 3) ALTIUS_GO(1024, 4) \
        ALTIUS_GO(1024, 6) ALTIUS_GO(1024, 8) ALTIUS_GO(1024, 12) ALTIUS_GO(1024, 16)                                                                       \
    }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Picks the register layout for a wave-per-row kernel: VEC=4 when rows stay
// 16-byte aligned, and the smallest chunk count that covers the row.
template <template <int, int> class Launcher, class... Args>
bool dispatch_wave(bool vec4, size_t len, Args... args) {
    if (vec4) {
        const size_t chunks = (len / 4 + WAVE - 1) / WAVE;
        switch (chunks) {
        case 1: Launcher<4, 1>::go(args...); return true;
        case 2: Launcher<4, 2>::go(args...); return true;
        case 3: Launcher<4, 3>::go(args...); return true;
        case 4: Launcher<4, 4>::go(args...); return true;
        }
        return false;
    }
    const size_t chunks = (len + WAVE - 1) / WAVE;
    if (chunks <= 1) { Launcher<1, 1>::go(args...); return true; }
    if (chunks <= 2) { Launcher<1, 2>::go(args...); return true; }
    if (chunks <= 4) { Launcher<1, 4>::go(args...); return true; }
    if (chunks <= 8) { Launcher<1, 8>::go(args...); return true; }
    if (chunks <= 12) { Launcher<1, 12>::go(args...); return true; }
    if (chunks <= 16) { Launcher<1, 16>::go(args...); return true; }
    return false;
}

// Rows of 1025 to 1280 elements that are whole float4s: still a wavefront per row with the row in registers
// (5 float4 per lane), read once.
template <template <int, int> class Launcher, class... Args>
bool dispatch_wave_long(size_t len, Args... args) {
    const size_t chunks = (len / 4 + WAVE - 1) / WAVE;
    if (chunks <= 5) { Launcher<4, 5>::go(args...); return true; }
    return false;
}

template <int VEC, int NCH> struct SoftmaxLauncher {
    static void go(hipStream_t s, float *out, const float *in, size_t rows, int len, const SoftmaxPrologue *pro, bool nt) {
        const dim3 grid((unsigned)((rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK));
        const SoftmaxPrologue none{0, 0.0f, nullptr, 1, 0};
        if constexpr (VEC == 4 && NCH <= 4) {  // with five chunks the five unguarded loads in a row cost 3 points
            if (len == NCH * WAVE * VEC) {  // every slot of the wavefront's chunks is an element
                if (pro && nt) hipLaunchKernelGGL((softmax_wave<VEC, NCH, true, true, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, *pro);
                else if (pro) hipLaunchKernelGGL((softmax_wave<VEC, NCH, true, false, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, *pro);
                else if (nt) hipLaunchKernelGGL((softmax_wave<VEC, NCH, false, true, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, none);
                else hipLaunchKernelGGL((softmax_wave<VEC, NCH, false, false, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, none);
                return;
            }
        }
        if (pro && nt && VEC == 4)
            hipLaunchKernelGGL((softmax_wave<VEC, NCH, true, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, *pro);
        else if (pro)
            hipLaunchKernelGGL((softmax_wave<VEC, NCH, true, false>), grid, dim3(BLOCK), 0, s, out, in, rows, len, *pro);
        else if (nt && VEC == 4)
            hipLaunchKernelGGL((softmax_wave<VEC, NCH, false, true>), grid, dim3(BLOCK), 0, s, out, in, rows, len, none);
        else
            hipLaunchKernelGGL((softmax_wave<VEC, NCH, false, false>), grid, dim3(BLOCK), 0, s, out, in, rows, len, none);
    }
};

template <int VEC, int NCH> struct LayerNormLauncher {
    static void go(hipStream_t s, float *out, const float *in, const float *gamma, const float *beta,
                   size_t rows, int len, float eps, bool nt) {
        const size_t blocks = (rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
        if constexpr (VEC == 4 && NCH <= 5) {
            if (len == NCH * WAVE * VEC) {
                if (nt) hipLaunchKernelGGL((layernorm_wave<VEC, NCH, true, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, gamma, beta, rows, len, eps);
                else hipLaunchKernelGGL((layernorm_wave<VEC, NCH, false, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, gamma, beta, rows, len, eps);
                return;
            }
        }
        if (nt && VEC == 4)
            hipLaunchKernelGGL((layernorm_wave<VEC, NCH, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in,
                               gamma, beta, rows, len, eps);
        else
            hipLaunchKernelGGL((layernorm_wave<VEC, NCH, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in,
                               gamma, beta, rows, len, eps);
    }
};

// Launches softmax_lds with the lane-group width and chunk count that waste the
// fewest lane slots for this row length (len <= 1024): 16 lanes per row up to
// 256 elements, 32 up to 512, 64 above.
template <int BT, int SUB, int NCH>
void softmax_lds_go_bt(bool nt, dim3 grid, size_t shmem, hipStream_t s, float *out, const float *in, size_t rows,
                       int len, int g, const SoftmaxPrologue *pro) {
    const SoftmaxPrologue none{0, 0.0f, nullptr, 1, 0};
    if (pro) {
        if (nt)
            hipLaunchKernelGGL((softmax_lds<BT, SUB, NCH, true, true>), grid, dim3(BT), shmem, s, out, in, rows, len, g, *pro);
        else
            hipLaunchKernelGGL((softmax_lds<BT, SUB, NCH, false, true>), grid, dim3(BT), shmem, s, out, in, rows, len, g, *pro);
    } else if (nt) {
        hipLaunchKernelGGL((softmax_lds<BT, SUB, NCH, true, false>), grid, dim3(BT), shmem, s, out, in, rows, len, g, none);
    } else {
        hipLaunchKernelGGL((softmax_lds<BT, SUB, NCH, false, false>), grid, dim3(BT), shmem, s, out, in, rows, len, g, none);
    }
}
template <int SUB, int NCH>
void softmax_lds_go(int threads, bool nt, dim3 grid, size_t shmem, hipStream_t s, float *out, const float *in, size_t rows,
                    int len, int g, const SoftmaxPrologue *pro) {
    if (threads == LDS_BLOCK) softmax_lds_go_bt<LDS_BLOCK, SUB, NCH>(nt, grid, shmem, s, out, in, rows, len, g, pro);
    else softmax_lds_go_bt<LDS_BLOCK / 2, SUB, NCH>(nt, grid, shmem, s, out, in, rows, len, g, pro);
}

size_t gcd_size(size_t a, size_t b) {
    while (b) {
        const size_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Rows per block: the smallest count whose span is a whole number of 128-byte lines (or of
// 64/32/16 bytes when that would not fit), repeated up to the LDS budget.
size_t softmax_lds_group_rows(size_t len, size_t budget_floats = LDS_GROUP_FLOATS) {
    for (size_t align_floats = 32; align_floats >= 4; align_floats /= 2) {
        const size_t base = align_floats / gcd_size(len, align_floats);
        if (base * len <= budget_floats) {
            size_t m = budget_floats / (base * len);
            const size_t max_rows = 1024;
            if (base * m > max_rows) m = max_rows / base > 0 ? max_rows / base : 1;
            return base * m;
        }
    }
    return 4;  // unreachable for len <= 1024: 4 rows are at most 4096 floats
}

// Threads of a block of the LDS-staged kernels.  Half-wide blocks (512 threads, 16 KiB groups) put four blocks on a CU
// instead of two, and every block loads, computes and stores in turn: Softmax and LayerNormalization gain 2-3 points
// of the HBM peak at 49, 64, 100, 128 and 1000 elements.  Where the smallest line-aligned group of rows does not fit
// 16 KiB (197: 32 rows are 25 KiB) the narrow block would have to cut groups inside a 128-byte line and loses 2-5
// points (one point of that comes back when the two blocks that share a line are dealt to one XCD): those keep the
// wide block.
// A tensor of up to 64 MiB is a launch of a few rounds of blocks at most and mostly cache-resident: there the narrow
// block wins with groups cut at 64-byte boundaries too (18 912 rows of 197: 8.4 -> 7.0 us; 75 648 rows: 24.1 -> 23.4 us;
// from 128 MiB on it loses).
inline int lds_block_threads(size_t len, size_t rows = ~(size_t)0) {
    if (32 / gcd_size(len, 32) * len <= LDS_GROUP_FLOATS / 2) return LDS_BLOCK / 2;
    const bool small = rows <= ((size_t)64 << 20) / sizeof(float) / len;
    if (small && 16 / gcd_size(len, 16) * len <= LDS_GROUP_FLOATS / 2) return LDS_BLOCK / 2;
    return LDS_BLOCK;
}

// Lanes per row and chunks per lane for a row of L <= 1024 elements in the LDS-staged kernels: the narrowest lane
// group that covers the row in at most 16 chunks.  Narrow groups mean more rows per wavefront pass, and the work a
// pass does once per row group (the two all-reduces, the division, the loop) is shared by more rows: 4 lanes up to
// 64 elements (unless the length is a multiple of 8: the sixteen rows of a pass would then meet in the same LDS
// banks), 8 up to 128, 16 up to 256, 32 up to 512, 64 above.
#define ALTIUS_LDS_LAYOUTS(L)                                                                                       \
    if ((L) <= 64 && (L) % 8 != 0) {                                                                                \
        switch (((L) + 3) / 4) {                                                                                    \
            ALTIUS_GO(4, 1) ALTIUS_GO(4, 2) ALTIUS_GO(4, 3) ALTIUS_GO(4, 4) ALTIUS_GO(4, 5) ALTIUS_GO(4, 6)         \
            ALTIUS_GO(4, 7) ALTIUS_GO(4, 8) ALTIUS_GO(4, 9) ALTIUS_GO(4, 10) ALTIUS_GO(4, 11) ALTIUS_GO(4, 12)      \
            ALTIUS_GO(4, 13) ALTIUS_GO(4, 14) ALTIUS_GO(4, 15) ALTIUS_GO(4, 16)                                     \
        }                                                                                                           \
    } else if ((L) <= 128) {                                                                                               \
        switch (((L) + 7) / 8) {                                                                                    \
            ALTIUS_GO(8, 1) ALTIUS_GO(8, 2) ALTIUS_GO(8, 3) ALTIUS_GO(8, 4) ALTIUS_GO(8, 5) ALTIUS_GO(8, 6)         \
            ALTIUS_GO(8, 7) ALTIUS_GO(8, 8) ALTIUS_GO(8, 9) ALTIUS_GO(8, 10) ALTIUS_GO(8, 11) ALTIUS_GO(8, 12)      \
            ALTIUS_GO(8, 13) ALTIUS_GO(8, 14) ALTIUS_GO(8, 15) ALTIUS_GO(8, 16)                                     \
        }                                                                                                           \
    } else if ((L) <= 256) {                                                                                        \
        switch (((L) + 15) / 16) {                                                                                  \
            ALTIUS_GO(16, 9) ALTIUS_GO(16, 10) ALTIUS_GO(16, 11) ALTIUS_GO(16, 12) ALTIUS_GO(16, 13)                \
            ALTIUS_GO(16, 14) ALTIUS_GO(16, 15) ALTIUS_GO(16, 16)                                                   \
        }                                                                                                           \
    } else if ((L) <= 512) {                                                                                        \
        switch (((L) + 31) / 32) {                                                                                  \
            ALTIUS_GO(32, 9) ALTIUS_GO(32, 10) ALTIUS_GO(32, 11) ALTIUS_GO(32, 12) ALTIUS_GO(32, 13)                \
            ALTIUS_GO(32, 14) ALTIUS_GO(32, 15) ALTIUS_GO(32, 16)                                                   \
        }                                                                                                           \
    } else {                                                                                                        \
        switch (((L) + 63) / 64) {                                                                                  \
            ALTIUS_GO(64, 9) ALTIUS_GO(64, 10) ALTIUS_GO(64, 11) ALTIUS_GO(64, 12) ALTIUS_GO(64, 13)                \
            ALTIUS_GO(64, 14) ALTIUS_GO(64, 15) ALTIUS_GO(64, 16)                                                   \
        }                                                                                                           \
    }

bool softmax_lds_launch(hipStream_t s, float *out, const float *in, size_t rows, size_t len, bool nt,
                        const SoftmaxPrologue *pro = nullptr) {
    static_assert(4 * 1024 <= LDS_GROUP_FLOATS, "four rows of the longest supported length must fit");
    const int threads = lds_block_threads(len, rows);
    size_t g = softmax_lds_group_rows(len, (size_t)STAGE_LDS * threads * 4);
    // A group may straddle one boundary between mask rows, not more: with a mask, groups are cut
    // down to a line-aligned row count that does not exceed the rows of one mask row.
    if (pro && pro->mask && pro->rows_per_mask < g) {
        size_t base = 32 / gcd_size(len, 32);
        while (base > 1 && base > pro->rows_per_mask) base /= 2;  // fall back to 64-, 32-, 16-byte aligned groups
        g = pro->rows_per_mask / base * base;
        if (g == 0) return false;
    }
    const size_t groups = (rows + g - 1) / g;
    if (groups > 0x7FFFFFFFu) return false;
    const dim3 grid((unsigned)groups);
    const size_t shmem = (g * len + (pro && pro->mask ? 2 * len : 0)) * sizeof(float);
    const int L = (int)len, G = (int)g;
#define ALTIUS_GO(SUB, N)                                                    \
    case N:                                                                  \
        softmax_lds_go<SUB, N>(threads, nt, grid, shmem, s, out, in, rows, L, G, pro); \
        return true;
    ALTIUS_LDS_LAYOUTS(L)
#undef ALTIUS_GO
    return false;
}

template <int BT, int SUB, int NCH>
void layernorm_lds_go_bt(bool nt, dim3 grid, size_t shmem, hipStream_t s, float *out, const float *in, const float *gamma, const float *beta,
                         size_t rows, int len, int g, float eps) {
    if (nt) hipLaunchKernelGGL((layernorm_lds<BT, SUB, NCH, true>), grid, dim3(BT), shmem, s, out, in, gamma, beta, rows, len, g, eps);
    else hipLaunchKernelGGL((layernorm_lds<BT, SUB, NCH, false>), grid, dim3(BT), shmem, s, out, in, gamma, beta, rows, len, g, eps);
}
template <int SUB, int NCH>
void layernorm_lds_go(int threads, bool nt, dim3 grid, size_t shmem, hipStream_t s, float *out, const float *in, const float *gamma,
                      const float *beta, size_t rows, int len, int g, float eps) {
    if (threads == LDS_BLOCK) layernorm_lds_go_bt<LDS_BLOCK, SUB, NCH>(nt, grid, shmem, s, out, in, gamma, beta, rows, len, g, eps);
    else layernorm_lds_go_bt<LDS_BLOCK / 2, SUB, NCH>(nt, grid, shmem, s, out, in, gamma, beta, rows, len, g, eps);
}

bool layernorm_lds_launch(hipStream_t s, float *out, const float *in, const float *gamma, const float *beta, size_t rows, size_t len, float eps,
                          bool nt) {
    const int threads = lds_block_threads(len, rows);
    const size_t g = softmax_lds_group_rows(len, (size_t)STAGE_LDS * threads * 4);
    const size_t groups = (rows + g - 1) / g;
    if ((g * len) % 4 != 0 || groups > 0x7FFFFFFFu) return false;
    const dim3 grid((unsigned)groups);
    const size_t shmem = (g * len + 2 * len) * sizeof(float);
    const int L = (int)len, G = (int)g;
#define ALTIUS_GO(SUB, N)                                                                     \
    case N:                                                                                   \
        layernorm_lds_go<SUB, N>(threads, nt, grid, shmem, s, out, in, gamma, beta, rows, L, G, eps); \
        return true;
    ALTIUS_LDS_LAYOUTS(L)
#undef ALTIUS_GO
    return false;
}

// A wavefront per row with 16-byte accesses suits rows that are whole 128-byte lines (no line shared between the
// loads of two wavefronts) and fill at least three quarters of the wavefront's 256-element chunks; every other
// row of up to 1024 elements goes through LDS in line-aligned groups.
inline bool wave_row_fits(size_t len) {
    const size_t slots = (len + 255) / 256 * 256;
    return len % 32 == 0 && len * 4 >= slots * 3;
}

constexpr size_t MAX_WAVE_ROW = 1024;
constexpr size_t MAX_LONG_ROW = 1280;  // rows kept in a wavefront's registers when they are whole float4s (at 1536 a block per row is 2 points ahead)
constexpr size_t MAX_BLOCK_REG_ROW = 65536;  // ... and in a block's registers
constexpr size_t MAX_GRID = 0x7FFFFFFFu;
}  // namespace

// Threads of the streaming kernels' block: two float4 per thread and pass up to 8192 elements, then the widest block.
inline int stream_block_threads(size_t len) { return len <= 2048 ? 256 : len <= 4096 ? 512 : 1024; }

int launch_softmax(DeviceCtx &ctx, float *out, const float *in, size_t rows, size_t len) {
    if (rows == 0 || len == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "softmax: null tensor pointer");
    if (len <= MAX_WAVE_ROW) {
        if ((rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK > MAX_GRID)
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: too many rows for one launch");
        const bool aligned = aligned16(out) && aligned16(in);
        const bool vec4 = (len % 4 == 0) && aligned;
        // A wave per row with 16-byte accesses is ideal when the row fills (most of) the wave's
        // 256-element chunks; otherwise go through LDS, which needs aligned buffers only.
        const bool wave_fits = vec4 && wave_row_fits(len);
        if (aligned && !wave_fits) {
            if (!softmax_lds_launch(ctx.stream, out, in, rows, len, ctx.streaming(rows * len * sizeof(float))))
                return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: too many rows for one launch");
        } else if (!dispatch_wave<SoftmaxLauncher>(vec4, len, ctx.stream, out, in, rows, (int)len, (const SoftmaxPrologue *)nullptr,
                                                    ctx.streaming(rows * len * sizeof(float)))) {
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: no wave layout for this row length");
        }
    } else if (len <= MAX_LONG_ROW && len % 4 == 0 && aligned16(out) && aligned16(in) &&
               (rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK <= MAX_GRID) {
        dispatch_wave_long<SoftmaxLauncher>(len, ctx.stream, out, in, rows, (int)len, (const SoftmaxPrologue *)nullptr,
                                            ctx.streaming(rows * len * sizeof(float)));
    } else if (len <= MAX_BLOCK_REG_ROW && len % 4 == 0 && aligned16(out) && aligned16(in) && rows <= MAX_GRID) {
        const bool nt = ctx.streaming(rows * len * sizeof(float));
        const BlockLayout lay = block_layout(len);
        const size_t resident = (size_t)2 * (ctx.cus_per_xcd ? ctx.cus_per_xcd * 8 : 256);
        bool launched = false;
#define ALTIUS_GO(T, N)                                                         \
    case T * 100 + N:                                                           \
        softmax_block_go<T, N>(nt, ctx.stream, rows, resident, out, in, len);   \
        launched = true;                                                        \
        break;
        ALTIUS_BLOCK_LAYOUTS(lay)
#undef ALTIUS_GO
        if (!launched) return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: no block layout for this row length");
    } else if (len > MAX_WAVE_ROW && len <= MAX_BLOCK_REG_ROW && rows <= MAX_GRID) {
        // Rows that start anywhere, input and output each where it lies.
        if (!softmax_anywhere_launch(ctx.streaming(rows * len * sizeof(float)), ctx.stream, rows, out, in, len))
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: no block layout for this row length");
    } else {
        if (rows > MAX_GRID) return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax: too many rows for one launch");
        const bool nt = ctx.streaming(rows * len * sizeof(float));
        const int threads = stream_block_threads(len);
#define ALTIUS_GO(T)                                                                                                          \
    do {                                                                                                                      \
        if (nt) hipLaunchKernelGGL((softmax_block_stream<T, true>), dim3((unsigned)rows), dim3(T), 0, ctx.stream, out, in, len);  \
        else hipLaunchKernelGGL((softmax_block_stream<T, false>), dim3((unsigned)rows), dim3(T), 0, ctx.stream, out, in, len);    \
    } while (0)
        if (threads == 256) ALTIUS_GO(256);
        else if (threads == 512) ALTIUS_GO(512);
        else ALTIUS_GO(1024);
#undef ALTIUS_GO
    }
    return ctx.check(hipGetLastError(), "softmax launch");
}

int launch_softmax_prologue(DeviceCtx &ctx, float *out, const float *in, size_t rows, size_t len, int scale_op, float scale,
                            const float *mask, size_t rows_per_mask) {
    if (scale_op < 0 || scale_op > 2) return ctx.fail(AHIP_ERR_ARG, "softmax: scale_op must be 0 (none), 1 (multiply) or 2 (divide)");
    if (rows == 0 || len == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "softmax: null tensor pointer");
    if (mask && (rows_per_mask == 0 || rows % rows_per_mask != 0))
        return ctx.fail(AHIP_ERR_ARG, "softmax: the row count must be a multiple of rows_per_mask");
    if (scale_op == 0 && !mask) return launch_softmax(ctx, out, in, rows, len);
    // The same kernel choice as launch_softmax, so that the row sums are accumulated in the same order and
    // the result has the bits of the separate operators.  Unaligned tensors and rows beyond 1024 elements
    // are left to the caller's operator-by-operator route.
    if (len > MAX_WAVE_ROW || !aligned16(out) || !aligned16(in) || rows >= ((size_t)1 << 32) || rows_per_mask >= ((size_t)1 << 32))
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax prologue: needs 16-byte aligned tensors and rows of at most 1024 elements");
    SoftmaxPrologue pro{scale_op, scale, mask, (uint32_t)(mask ? rows_per_mask : 1), (uint32_t)(mask ? rows / rows_per_mask : 0)};
    const bool wave_fits = wave_row_fits(len);
    if (wave_fits) {
        if (mask && !aligned16(mask)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax prologue: the mask must be 16-byte aligned");
        if ((rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK > MAX_GRID || !dispatch_wave<SoftmaxLauncher>(true, len, ctx.stream, out, in, rows, (int)len, (const SoftmaxPrologue *)&pro,
                                                                                         ctx.streaming(rows * len * sizeof(float))))
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax prologue: too many rows for one launch");
    } else if (!softmax_lds_launch(ctx.stream, out, in, rows, len, ctx.streaming(rows * len * sizeof(float)), &pro)) {
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "softmax prologue: too many rows for one launch");
    }
    return ctx.check(hipGetLastError(), "softmax (prologue) launch");
}

int launch_layernorm(DeviceCtx &ctx, float *out, const float *in, const float *gamma, const float *beta,
                     size_t rows, size_t len, float eps) {
    if (rows == 0 || len == 0) return AHIP_OK;
    if (!out || !in || !gamma || !beta) return ctx.fail(AHIP_ERR_ARG, "layernorm: null tensor pointer");
    if (len <= MAX_WAVE_ROW && rows >= 64 && aligned16(out) && aligned16(in)) {
        // Rows that fill (most of) a wavefront's 256-element chunks with whole float4s take the wavefront-per-row
        // kernel; every other row of up to 1024 elements goes through LDS in line-aligned groups (the rule Softmax uses).
        const bool wave_fits = wave_row_fits(len) && aligned16(gamma) && aligned16(beta);
        if (!wave_fits && layernorm_lds_launch(ctx.stream, out, in, gamma, beta, rows, len, eps, ctx.streaming(rows * len * sizeof(float))))
            return ctx.check(hipGetLastError(), "layernorm (LDS groups) launch");
    }
    if (len <= MAX_WAVE_ROW) {
        if ((rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK > MAX_GRID)
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm: too many rows for one launch");
        const bool vec4 =
            (len % 4 == 0) && aligned16(out) && aligned16(in) && aligned16(gamma) && aligned16(beta);
        if (!dispatch_wave<LayerNormLauncher>(vec4, len, ctx.stream, out, in, gamma, beta, rows, (int)len,
                                              eps, ctx.streaming(rows * len * sizeof(float))))
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm: no wave layout for this row length");
    } else if (len <= MAX_LONG_ROW && len % 4 == 0 && aligned16(out) && aligned16(in) &&
               (rows + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK <= MAX_GRID) {
        dispatch_wave_long<LayerNormLauncher>(len, ctx.stream, out, in, gamma, beta, rows, (int)len, eps,
                                              ctx.streaming(rows * len * sizeof(float)));
    } else if (len <= MAX_BLOCK_REG_ROW && len % 4 == 0 && aligned16(out) && aligned16(in) && aligned16(gamma) && aligned16(beta) &&
               rows <= MAX_GRID) {
        const bool nt = ctx.streaming(rows * len * sizeof(float));
        const BlockLayout lay = block_layout(len);
        const size_t resident = (size_t)2 * (ctx.cus_per_xcd ? ctx.cus_per_xcd * 8 : 256);
        bool launched = false;
#define ALTIUS_GO(T, N)                                                                      \
    case T * 100 + N:                                                                        \
        layernorm_block_go<T, N>(nt, ctx.stream, rows, resident, out, in, gamma, beta, len, eps); \
        launched = true;                                                                     \
        break;
        ALTIUS_BLOCK_LAYOUTS(lay)
#undef ALTIUS_GO
        if (!launched) return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm: no block layout for this row length");
    } else if (len > MAX_WAVE_ROW && len <= MAX_BLOCK_REG_ROW && rows <= MAX_GRID) {
        // Rows that start anywhere (see launch_softmax).
        if (!layernorm_anywhere_launch(ctx.streaming(rows * len * sizeof(float)), ctx.stream, rows, out, in, gamma, beta, len, eps))
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm: no block layout for this row length");
    } else {
        if (rows > MAX_GRID) return ctx.fail(AHIP_ERR_UNSUPPORTED, "layernorm: too many rows for one launch");
        const bool nt = ctx.streaming(rows * len * sizeof(float));
        const int threads = stream_block_threads(len);
#define ALTIUS_GO(T)                                                                                                                          \
    do {                                                                                                                                      \
        if (nt) hipLaunchKernelGGL((layernorm_block_stream<T, true>), dim3((unsigned)rows), dim3(T), 0, ctx.stream, out, in, gamma, beta, len, eps);  \
        else hipLaunchKernelGGL((layernorm_block_stream<T, false>), dim3((unsigned)rows), dim3(T), 0, ctx.stream, out, in, gamma, beta, len, eps);    \
    } while (0)
        if (threads == 256) ALTIUS_GO(256);
        else if (threads == 512) ALTIUS_GO(512);
        else ALTIUS_GO(1024);
#undef ALTIUS_GO
    }
    return ctx.check(hipGetLastError(), "layernorm launch");
}

// Row sums / maxima through reduce_rows_lds; -1 (nothing launched) when the shape is not one it is meant for.
int launch_reduce_rows_lds(DeviceCtx &ctx, bool is_max, float *out, const float *in, size_t rows, size_t len, float scale, bool scaled) {
    if (len == 0 || len > 1024 || rows < 64 || !aligned16(in)) return -1;
    // Read-only: blocks of 512 threads, four to a CU (72-75 % of the HBM peak with 1024 become 83-90 %); two float4 per
    // thread where a line-aligned group of rows fits 16 KiB, four where it takes 32 KiB (197).
    constexpr int RT = LDS_BLOCK / 2;
    const bool deep = lds_block_threads(len) == LDS_BLOCK;
    const size_t g = softmax_lds_group_rows(len, (size_t)(deep ? 4 : 2) * RT * 4);
    if ((g * len) % 4 != 0) return -1;  // groups must start 16-byte aligned
    const size_t groups = (rows + g - 1) / g;
    if (groups > 0x7FFFFFFFu) return -1;
    const bool nt = ctx.streaming(rows * len * sizeof(float));
    const dim3 grid((unsigned)groups);
    const size_t shmem = g * len * sizeof(float);
    const int L = (int)len, G = (int)g;
#define ALTIUS_RED(OP, SUB, SC)                                                                                                   \
    do {                                                                                                                          \
        if (deep && nt) hipLaunchKernelGGL((reduce_rows_lds<RT, 4, OP, SUB, SC, true>), grid, dim3(RT), shmem, ctx.stream, out, in, rows, L, G, scale);  \
        else if (deep) hipLaunchKernelGGL((reduce_rows_lds<RT, 4, OP, SUB, SC, false>), grid, dim3(RT), shmem, ctx.stream, out, in, rows, L, G, scale);  \
        else if (nt) hipLaunchKernelGGL((reduce_rows_lds<RT, 2, OP, SUB, SC, true>), grid, dim3(RT), shmem, ctx.stream, out, in, rows, L, G, scale);     \
        else hipLaunchKernelGGL((reduce_rows_lds<RT, 2, OP, SUB, SC, false>), grid, dim3(RT), shmem, ctx.stream, out, in, rows, L, G, scale);           \
    } while (0)
#define ALTIUS_RED_SUB(SUB)                                   \
    do {                                                      \
        if (is_max) ALTIUS_RED(MaxOp, SUB, false);            \
        else if (scaled) ALTIUS_RED(SumOp, SUB, true);        \
        else ALTIUS_RED(SumOp, SUB, false);                   \
    } while (0)
    if (len <= 64 && len % 8 != 0) ALTIUS_RED_SUB(4);
    else if (len <= 128) ALTIUS_RED_SUB(8);
    else if (len <= 256) ALTIUS_RED_SUB(16);
    else if (len <= 512) ALTIUS_RED_SUB(32);
    else ALTIUS_RED_SUB(64);
#undef ALTIUS_RED_SUB
#undef ALTIUS_RED
    return ctx.check(hipGetLastError(), "reduce rows (LDS groups) launch");
}

}  // namespace altius
