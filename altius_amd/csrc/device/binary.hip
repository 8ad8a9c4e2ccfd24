// Broadcast binary ops (Add/Sub/Mul/Div/Pow) for gfx950.
//
// The output is always dense, so every kernel walks the flat output index and
// stores 16 bytes per lane.  An operand is one of
//   FULL    -- same layout as the output: 16-byte load at the flat index,
//   SCALAR  -- one value for the whole tensor,
//   STRIDED -- anything else: its offset is rebuilt from the output coordinate
//              with the per-axis strides the host precomputed (0 on broadcast
//              axes); the coordinate is decomposed once per lane and advanced
//              with carries, so no division is spent per element.
// The host first drops size-1 axes and merges adjacent axes that both operands
// walk contiguously, which turns e.g. [256,12,197,197] + [256,1,1,197] into a
// rank-3 problem and every same-shape or scalar case into a rank-1 one.
//
// Reference semantics: crates/session_interpreter/src/session.rs:384-526
// (Add/Sub/Mul/Div: one IEEE operation per element) and 566-606 (Pow).

#include "common.h"
#include "ctx.h"

#include <math.h>

namespace altius {
namespace {

using namespace dev;

enum Mode : int { FULL = 0, SCALAR = 1, STRIDED = 2 };

struct OpAdd { static __device__ __forceinline__ float f(float a, float b) { return a + b; } };
struct OpSub { static __device__ __forceinline__ float f(float a, float b) { return a - b; } };
struct OpMul { static __device__ __forceinline__ float f(float a, float b) { return a * b; } };
struct OpDiv { static __device__ __forceinline__ float f(float a, float b) { return a / b; } };
struct OpPow { static __device__ __forceinline__ float f(float a, float b) { return powf(a, b); } };
// Pow with one exponent for the whole tensor (session.rs:585-598): a*a when it
// equals 2, powf otherwise.  The exponent is uniform, so the branch is too.
struct OpPowScalarExp {
    static __device__ __forceinline__ float f(float a, float b) { return b == 2.0f ? a * a : powf(a, b); }
};

constexpr int BLOCK = 256;

// ---------------------------------------------------------------------------
// Flat kernel: both operands are FULL or SCALAR.  One float4 per lane.
// ---------------------------------------------------------------------------
template <class OP, int MA, int MB, bool NT, bool NTL = NT>
__global__ __launch_bounds__(BLOCK) void binary_flat_vec4(float *__restrict__ out,
                                                          const float *__restrict__ a,
                                                          const float *__restrict__ b, size_t n) {
    const size_t n4 = n >> 2;
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    float sa = 0.f, sb = 0.f;
    if (MA == SCALAR) sa = a[0];
    if (MB == SCALAR) sb = b[0];
    if (i < n4) {
        const float4 x = MA == FULL ? load4<NTL>(a + 4 * i) : make_float4(sa, sa, sa, sa);
        const float4 y = MB == FULL ? load4<NTL>(b + 4 * i) : make_float4(sb, sb, sb, sb);
        float4 r;
        r.x = OP::f(x.x, y.x);
        r.y = OP::f(x.y, y.y);
        r.z = OP::f(x.z, y.z);
        r.w = OP::f(x.w, y.w);
        store4<NT>(out + 4 * i, r);
    }
    // The last (n % 4) elements.
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t j = (n4 << 2) + threadIdx.x;
        out[j] = OP::f(MA == FULL ? a[j] : sa, MB == FULL ? b[j] : sb);
    }
}

// The same on tensors that lie on 4-byte boundaries only: this part's 16-byte global accesses need no more.
template <class OP, int MA, int MB, bool NT>
__global__ __launch_bounds__(BLOCK) void binary_flat_vec4_any(float *__restrict__ out, const float *__restrict__ a,
                                                              const float *__restrict__ b, size_t n) {
    const size_t n4 = n >> 2;
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    float sa = 0.f, sb = 0.f;
    if (MA == SCALAR) sa = a[0];
    if (MB == SCALAR) sb = b[0];
    if (i < n4) {
        const float4 x = MA == FULL ? load4_dword_aligned<NT>(a + 4 * i) : make_float4(sa, sa, sa, sa);
        const float4 y = MB == FULL ? load4_dword_aligned<NT>(b + 4 * i) : make_float4(sb, sb, sb, sb);
        store4_dword_aligned<NT>(out + 4 * i, make_float4(OP::f(x.x, y.x), OP::f(x.y, y.y), OP::f(x.z, y.z), OP::f(x.w, y.w)));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t j = (n4 << 2) + threadIdx.x;
        out[j] = OP::f(MA == FULL ? a[j] : sa, MB == FULL ? b[j] : sb);
    }
}

// Same, one element per lane, for the smallest tensors that are not 16-byte aligned.
template <class OP, int MA, int MB>
__global__ __launch_bounds__(BLOCK) void binary_flat_scalar(float *__restrict__ out,
                                                            const float *__restrict__ a,
                                                            const float *__restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n) return;
    out[i] = OP::f(MA == FULL ? a[i] : a[0], MB == FULL ? b[i] : b[0]);
}

// ---------------------------------------------------------------------------
// Strided kernel.
// ---------------------------------------------------------------------------
using dev::FastDiv;
using dev::make_fastdiv;

struct Geom {
    // Axis 0 is the innermost (fastest) output axis.
    FastDiv dims[MAX_RANK];
    uint32_t a_str[MAX_RANK];
    uint32_t b_str[MAX_RANK];
    int mode_a, mode_b;  // Mode
    // The operand can be read 16 bytes at a time: innermost stride 1, innermost
    // extent and every other stride multiples of 4, base 16-byte aligned.
    int a_vec, b_vec;
};

// Offsets of one operand for VEC consecutive output elements that start at
// column c0 of a row: elements past the end of the row continue in the next
// row (VEC <= innermost extent, so at most one row change).
template <int VEC> struct Span {
    uint32_t row, next;  // operand offset of column 0 of this row / of the next row
    __device__ __forceinline__ uint32_t at(int j, uint32_t c0, uint32_t d0, uint32_t s0) const {
        const uint32_t c = c0 + j;
        return c >= d0 ? next + (c - d0) * s0 : row + c * s0;
    }
};

// 16 bytes from an address that is only 4-byte aligned (global memory allows it).
struct __attribute__((packed, aligned(4))) Float4U {
    float x, y, z, w;
};

// Reads VEC consecutive output elements' worth of one operand.
template <int VEC, bool NT>
__device__ __forceinline__ void fetch(float (&v)[VEC], const float *__restrict__ p, int mode, int vec_ok,
                                      const Span<VEC> &sp, uint32_t c0, uint32_t d0, uint32_t s0, uint32_t i0,
                                      uint32_t n, bool whole, bool same_row) {
    if (mode == FULL) {
        if (VEC == 4 && whole) {
            const float4 t = load4<NT>(p + i0);
            v[0] = t.x; v[1 % VEC] = t.y; v[2 % VEC] = t.z; v[3 % VEC] = t.w;
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) v[j] = i0 + j < n ? p[i0 + j] : 0.f;
        }
    } else if (mode == SCALAR) {
        const float s = p[0];
#pragma unroll
        for (int j = 0; j < VEC; j++) v[j] = s;
    } else if (VEC == 4 && vec_ok) {  // aligned, and no row change inside the four elements
        const float4 t = *reinterpret_cast<const float4 *>(p + sp.row + c0);
        v[0] = t.x; v[1 % VEC] = t.y; v[2 % VEC] = t.z; v[3 % VEC] = t.w;
    } else if (VEC == 4 && whole && same_row && s0 == 1) {
        const Float4U t = *reinterpret_cast<const Float4U *>(p + sp.row + c0);
        v[0] = t.x; v[1 % VEC] = t.y; v[2 % VEC] = t.z; v[3 % VEC] = t.w;
    } else if (VEC == 4 && whole && same_row && s0 == 0) {
        const float s = p[sp.row];
#pragma unroll
        for (int j = 0; j < VEC; j++) v[j] = s;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) v[j] = i0 + j < n ? p[sp.at(j, c0, d0, s0)] : 0.f;
    }
}

template <class OP, int RANK, int VEC, bool NT>
__global__ __launch_bounds__(BLOCK) void binary_strided(float *__restrict__ out,
                                                        const float *__restrict__ a,
                                                        const float *__restrict__ b, uint32_t n,
                                                        const Geom g) {
    const uint32_t nvec = (n + VEC - 1) / VEC;
    const uint32_t t = blockIdx.x * BLOCK + threadIdx.x;
    if (t >= nvec) return;
    const uint32_t i0 = t * VEC;
    const bool whole = i0 + VEC <= n;

    // Coordinates of element i0; row offsets of both operands; the same for the next row.
    const uint32_t d0 = g.dims[0].d;
    uint32_t q = g.dims[0].div(i0);
    const uint32_t c0 = i0 - q * d0;
    Span<VEC> sa, sb;
    sa.row = sb.row = 0;
    sa.next = sb.next = 0;
    bool carry = true;  // the next row increments axis 1, and further axes while they wrap
#pragma unroll
    for (int d = 1; d < RANK; d++) {
        uint32_t c;
        if (d < RANK - 1) {
            const uint32_t q2 = g.dims[d].div(q);
            c = q - q2 * g.dims[d].d;
            q = q2;
        } else {
            c = q;
        }
        sa.row += c * g.a_str[d];
        sb.row += c * g.b_str[d];
        uint32_t cn = c;
        if (carry) {
            cn = c + 1;
            carry = cn == g.dims[d].d && d < RANK - 1;
            if (carry) cn = 0;
        }
        sa.next += cn * g.a_str[d];
        sb.next += cn * g.b_str[d];
    }
    const bool same_row = c0 + VEC <= d0;

    float x[VEC], y[VEC];
    fetch<VEC, NT>(x, a, g.mode_a, g.a_vec, sa, c0, d0, g.a_str[0], i0, n, whole, same_row);
    fetch<VEC, NT>(y, b, g.mode_b, g.b_vec, sb, c0, d0, g.b_str[0], i0, n, whole, same_row);

    if (VEC == 4 && whole) {
        float4 r;
        r.x = OP::f(x[0], y[0]);
        r.y = OP::f(x[1 % VEC], y[1 % VEC]);
        r.z = OP::f(x[2 % VEC], y[2 % VEC]);
        r.w = OP::f(x[3 % VEC], y[3 % VEC]);
        store4<NT>(out + i0, r);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++)
            if (i0 + j < n) out[i0 + j] = OP::f(x[j], y[j]);
    }
}

// ---------------------------------------------------------------------------
// Row-broadcast kernel: out[n][r][c] = full[n][r][c] op small[n][c] (an attention
// mask [N,1,1,C] on scores [N,H,S,C], a bias [C] on [.., C]).  The block's one or
// two rows of the small operand are staged in LDS, so the only global traffic per
// lane is one 16-byte load and one 16-byte store, as in a plain copy; gathering
// the small operand from global memory instead costs as many L1 accesses as the
// main stream.
// ---------------------------------------------------------------------------
struct RowBcast {
    FastDiv rc;     // R * C: elements per outer index
    FastDiv c;      // C: row length
    uint32_t n;     // number of outer indices (rows of the small operand)
    uint32_t total; // N * R * C
};

template <class OP, bool SMALL_IS_A, bool NT, bool NTL = NT>
__global__ __launch_bounds__(BLOCK) void binary_rowbcast(float *__restrict__ out, const float *__restrict__ full,
                                                         const float *__restrict__ small, const RowBcast g) {
    extern __shared__ float rows_lds[];  // two rows of C floats
    const uint32_t C = g.c.d;
    const uint32_t block_start = blockIdx.x * (BLOCK * 4);
    const uint32_t n_first = g.rc.div(block_start);  // uniform
    // The 16-byte load of the dense operand goes out first, so its latency covers the staging of
    // the small operand and the index arithmetic.
    const uint32_t i0 = block_start + threadIdx.x * 4;
    const bool whole = i0 + 4 <= g.total;
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (whole) x = load4<NTL>(full + i0);
    {
        // Row n_first, and the next one only if this block really reaches into it.
        uint32_t block_last = block_start + BLOCK * 4 - 1;
        if (block_last >= g.total) block_last = g.total - 1;
        const uint32_t want = g.rc.div(block_last) != n_first ? 2 * C : C;
        const float *src = small + (size_t)n_first * C;
        for (uint32_t i = threadIdx.x; i < want; i += BLOCK) rows_lds[i] = src[i];
    }
    __syncthreads();

    if (i0 >= g.total) return;
    const uint32_t n = g.rc.div(i0);
    const uint32_t rem = i0 - n * g.rc.d;            // offset inside outer index n
    const uint32_t row = g.c.div(rem);
    const uint32_t c0 = rem - row * C;               // column of element 0
    const uint32_t base = (n - n_first) * C;         // LDS offset of row n

    float y[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t c = c0 + j, b = base;
        if (c >= C) {                                // next row of the output ...
            c -= C;
            if (rem + j >= g.rc.d) b += C;           // ... which may belong to the next outer index
        }
        y[j] = rows_lds[b + c];
    }
    if (whole) {
        float4 r;
        r.x = SMALL_IS_A ? OP::f(y[0], x.x) : OP::f(x.x, y[0]);
        r.y = SMALL_IS_A ? OP::f(y[1], x.y) : OP::f(x.y, y[1]);
        r.z = SMALL_IS_A ? OP::f(y[2], x.z) : OP::f(x.z, y[2]);
        r.w = SMALL_IS_A ? OP::f(y[3], x.w) : OP::f(x.w, y[3]);
        store4<NT>(out + i0, r);
    } else {
        for (int j = 0; j < 4 && i0 + j < g.total; j++) {
            const float xs = full[i0 + j];
            out[i0 + j] = SMALL_IS_A ? OP::f(y[j], xs) : OP::f(xs, y[j]);
        }
    }
}

// A vector of two or three values on the innermost axis ([N,H,W,3] op [3]): shorter than a lane's four elements, which
// therefore cycle through it more than once; the vector lives in three registers.
template <class OP, bool SMALL_IS_A, bool NT>
__global__ __launch_bounds__(BLOCK) void binary_short_vector(float *__restrict__ out, const float *__restrict__ full,
                                                             const float *__restrict__ small, const FastDiv c, uint32_t total) {
    const uint32_t i0 = (blockIdx.x * BLOCK + threadIdx.x) * 4;
    if (i0 >= total) return;
    const bool whole = i0 + 4 <= total;
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (whole) x = load4<NT>(full + i0);
    const uint32_t C = c.d;
    const float v0 = small[0], v1 = small[1], v2 = small[C > 2 ? 2 : 0];
    uint32_t idx = i0 - c.div(i0) * C;
    float y[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        y[j] = idx == 0 ? v0 : idx == 1 ? v1 : v2;
        idx = idx + 1 == C ? 0 : idx + 1;
    }
    if (whole) {
        float4 r;
        r.x = SMALL_IS_A ? OP::f(y[0], x.x) : OP::f(x.x, y[0]);
        r.y = SMALL_IS_A ? OP::f(y[1], x.y) : OP::f(x.y, y[1]);
        r.z = SMALL_IS_A ? OP::f(y[2], x.z) : OP::f(x.z, y[2]);
        r.w = SMALL_IS_A ? OP::f(y[3], x.w) : OP::f(x.w, y[3]);
        store4<NT>(out + i0, r);
    } else {
        for (int j = 0; j < 4 && i0 + j < total; j++) {
            const float xs = full[i0 + j];
            out[i0 + j] = SMALL_IS_A ? OP::f(y[j], xs) : OP::f(xs, y[j]);
        }
    }
}

// ---------------------------------------------------------------------------
// Kernel for rows that are whole float4s with a small operand that is constant along or across the row:
//   out[r][c] = full[r][c] op small[c]            a bias or scale vector on rows longer than the row-broadcast kernel stages
//   out[n][r][c] = full[n][r][c] op small[n][c]   the same with one vector per outer index (an attention mask on long rows)
//   out[r][c] = full[r][c] op small[r]            a per-row mean or deviation, a squeeze-excite gate [N,C,1,1] on [N,C,H,W]
//   out[n][k][c] = full[n][k][c] op small[k]      a per-channel scale or bias [C,1,1] on [N,C,H,W]
// A lane's four elements lie in one row, so the dense 16-byte load goes out before any index arithmetic and the small
// operand costs one more load: 16 bytes that hit in L1, or one dword that most lanes of the wavefront share.
// ---------------------------------------------------------------------------
enum { SMALL_VECTOR = 0, SMALL_VECTOR_OUTER = 1, SMALL_COLUMN = 2, SMALL_COLUMN_MOD = 3 };

// c: the row length.  o: elements per outer index (SMALL_VECTOR_OUTER) or the number of values the rows cycle
// through (SMALL_COLUMN_MOD); unused otherwise.
template <class OP, int KIND, bool SMALL_IS_A, bool NT, bool NTL = NT>
__global__ __launch_bounds__(BLOCK) void binary_rows4(float *__restrict__ out, const float *__restrict__ full,
                                                      const float *__restrict__ small, uint32_t total,
                                                      const FastDiv c, const FastDiv o) {
    const uint32_t i0 = (blockIdx.x * BLOCK + threadIdx.x) * 4;
    if (i0 >= total) return;  // total is a multiple of 4
    const float4 x = load4<NTL>(full + i0);
    const uint32_t row = c.div(i0);
    float4 y;
    if (KIND == SMALL_VECTOR) {
        y = *reinterpret_cast<const float4 *>(small + (i0 - row * c.d));
    } else if (KIND == SMALL_VECTOR_OUTER) {
        y = *reinterpret_cast<const float4 *>(small + (o.div(i0) * c.d + (i0 - row * c.d)));
    } else {
        const float v = small[KIND == SMALL_COLUMN ? row : row - o.div(row) * o.d];
        y = make_float4(v, v, v, v);
    }
    float4 r;
    r.x = SMALL_IS_A ? OP::f(y.x, x.x) : OP::f(x.x, y.x);
    r.y = SMALL_IS_A ? OP::f(y.y, x.y) : OP::f(x.y, y.y);
    r.z = SMALL_IS_A ? OP::f(y.z, x.z) : OP::f(x.z, y.z);
    r.w = SMALL_IS_A ? OP::f(y.w, x.w) : OP::f(x.w, y.w);
    store4<NT>(out + i0, r);
}

// One value per row (or per channel) on rows of any length from 4 up (7 x 7 feature maps): a lane's four elements
// lie in at most two rows, so it reads this row's value and, only if its elements reach into it, the next row's.
// MOD: the rows cycle through o.d values.
template <class OP, bool MOD, bool SMALL_IS_A, bool NT>
__global__ __launch_bounds__(BLOCK) void binary_rows_any(float *__restrict__ out, const float *__restrict__ full,
                                                         const float *__restrict__ small, uint32_t total,
                                                         const FastDiv c, const FastDiv o) {
    const uint32_t i0 = (blockIdx.x * BLOCK + threadIdx.x) * 4;
    if (i0 >= total) return;
    const bool whole = i0 + 4 <= total;
    float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
    if (whole) x = load4<NT>(full + i0);
    const uint32_t row = c.div(i0), c0 = i0 - row * c.d;
    const uint32_t in_row = c.d - c0;  // elements of this lane that still belong to `row` (if < 4)
    const float v0 = small[MOD ? row - o.div(row) * o.d : row];
    float v1 = v0;
    if (in_row < 4 && i0 + in_row < total) {
        const uint32_t next = row + 1;
        v1 = small[MOD ? next - o.div(next) * o.d : next];
    }
    const float y[4] = {v0, in_row > 1 ? v0 : v1, in_row > 2 ? v0 : v1, in_row > 3 ? v0 : v1};
    if (whole) {
        float4 r;
        r.x = SMALL_IS_A ? OP::f(y[0], x.x) : OP::f(x.x, y[0]);
        r.y = SMALL_IS_A ? OP::f(y[1], x.y) : OP::f(x.y, y[1]);
        r.z = SMALL_IS_A ? OP::f(y[2], x.z) : OP::f(x.z, y[2]);
        r.w = SMALL_IS_A ? OP::f(y[3], x.w) : OP::f(x.w, y[3]);
        store4<NT>(out + i0, r);
    } else {
        for (int j = 0; j < 4 && i0 + j < total; j++) {
            const float xs = full[i0 + j];
            out[i0 + j] = SMALL_IS_A ? OP::f(y[j], xs) : OP::f(xs, y[j]);
        }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class OP, int MA, int MB>
void flat_dispatch(hipStream_t s, float *out, const float *a, const float *b, size_t n, bool vec, bool nt, bool ntl) {
    if (vec) {
        size_t blocks = ((n >> 2) + BLOCK - 1) / BLOCK;
        if (blocks == 0) blocks = 1;
        if (nt)
            hipLaunchKernelGGL((binary_flat_vec4<OP, MA, MB, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s,
                               out, a, b, n);
        else if (ntl)
            hipLaunchKernelGGL((binary_flat_vec4<OP, MA, MB, false, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s,
                               out, a, b, n);
        else
            hipLaunchKernelGGL((binary_flat_vec4<OP, MA, MB, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, s,
                               out, a, b, n);
    } else if (n >= 4 * BLOCK && ((reinterpret_cast<uintptr_t>(out) | (MA == FULL ? reinterpret_cast<uintptr_t>(a) : 0) |
                                   (MB == FULL ? reinterpret_cast<uintptr_t>(b) : 0)) & 3u) == 0) {
        // 16-byte accesses on 4-byte boundaries: the output and every full operand must at least be float-aligned
        // (a pointer at a byte offset takes the single-element kernel below)
        const size_t blocks = ((n >> 2) + BLOCK - 1) / BLOCK;
        if (nt) hipLaunchKernelGGL((binary_flat_vec4_any<OP, MA, MB, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, a, b, n);
        else hipLaunchKernelGGL((binary_flat_vec4_any<OP, MA, MB, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, a, b, n);
    } else {
        const size_t blocks = (n + BLOCK - 1) / BLOCK;
        hipLaunchKernelGGL((binary_flat_scalar<OP, MA, MB>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, a,
                           b, n);
    }
}

template <class OP>
void flat_launch(hipStream_t s, int ma, int mb, float *out, const float *a, const float *b, size_t n, bool vec,
                 bool nt, bool ntl) {
    if (ma == FULL && mb == FULL) flat_dispatch<OP, FULL, FULL>(s, out, a, b, n, vec, nt, ntl);
    else if (ma == FULL && mb == SCALAR) flat_dispatch<OP, FULL, SCALAR>(s, out, a, b, n, vec, nt, ntl);
    else if (ma == SCALAR && mb == FULL) flat_dispatch<OP, SCALAR, FULL>(s, out, a, b, n, vec, nt, ntl);
    else flat_dispatch<OP, SCALAR, SCALAR>(s, out, a, b, n, vec, nt, false);
}

template <class OP, int RANK>
void strided_dispatch(hipStream_t s, float *out, const float *a, const float *b, uint32_t n, const Geom &g,
                      bool vec, bool nt) {
    if (vec) {
        const uint32_t nvec = (n + 3) / 4;
        const dim3 grid((nvec + BLOCK - 1) / BLOCK);
        if (nt)
            hipLaunchKernelGGL((binary_strided<OP, RANK, 4, true>), grid, dim3(BLOCK), 0, s, out, a, b, n, g);
        else
            hipLaunchKernelGGL((binary_strided<OP, RANK, 4, false>), grid, dim3(BLOCK), 0, s, out, a, b, n, g);
    } else {
        hipLaunchKernelGGL((binary_strided<OP, RANK, 1, false>), dim3((n + BLOCK - 1) / BLOCK), dim3(BLOCK), 0,
                           s, out, a, b, n, g);
    }
}

template <class OP>
void strided_launch(hipStream_t s, int rank, float *out, const float *a, const float *b, uint32_t n,
                    const Geom &g, bool vec, bool nt) {
    if (rank <= 2) strided_dispatch<OP, 2>(s, out, a, b, n, g, vec, nt);
    else if (rank == 3) strided_dispatch<OP, 3>(s, out, a, b, n, g, vec, nt);
    else if (rank == 4) strided_dispatch<OP, 4>(s, out, a, b, n, g, vec, nt);
    else strided_dispatch<OP, MAX_RANK>(s, out, a, b, n, g, vec, nt);
}

template <class OP>
void rowbcast_launch(hipStream_t s, bool small_is_a, bool nt, bool ntl, float *out, const float *full, const float *small,
                     const RowBcast &g) {
    const dim3 grid((g.total + BLOCK * 4 - 1) / (BLOCK * 4));
    const size_t shmem = (size_t)2 * g.c.d * sizeof(float);
    if (small_is_a) {
        if (nt) hipLaunchKernelGGL((binary_rowbcast<OP, true, true>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
        else if (ntl) hipLaunchKernelGGL((binary_rowbcast<OP, true, false, true>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
        else hipLaunchKernelGGL((binary_rowbcast<OP, true, false>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
    } else {
        if (nt) hipLaunchKernelGGL((binary_rowbcast<OP, false, true>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
        else if (ntl) hipLaunchKernelGGL((binary_rowbcast<OP, false, false, true>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
        else hipLaunchKernelGGL((binary_rowbcast<OP, false, false>), grid, dim3(BLOCK), shmem, s, out, full, small, g);
    }
}

template <class OP>
void short_vector_launch(hipStream_t s, bool small_is_a, bool nt, float *out, const float *full, const float *small, uint32_t c, uint32_t total) {
    const dim3 grid((total + BLOCK * 4 - 1) / (BLOCK * 4));
    const FastDiv fd = make_fastdiv(c);
    if (small_is_a) {
        if (nt) hipLaunchKernelGGL((binary_short_vector<OP, true, true>), grid, dim3(BLOCK), 0, s, out, full, small, fd, total);
        else hipLaunchKernelGGL((binary_short_vector<OP, true, false>), grid, dim3(BLOCK), 0, s, out, full, small, fd, total);
    } else {
        if (nt) hipLaunchKernelGGL((binary_short_vector<OP, false, true>), grid, dim3(BLOCK), 0, s, out, full, small, fd, total);
        else hipLaunchKernelGGL((binary_short_vector<OP, false, false>), grid, dim3(BLOCK), 0, s, out, full, small, fd, total);
    }
}

template <class OP, int KIND>
void rows4_launch_kind(hipStream_t s, bool small_is_a, bool nt, bool ntl, float *out, const float *full, const float *small, uint32_t total,
                       const FastDiv &c, const FastDiv &o) {
    const dim3 grid((total / 4 + BLOCK - 1) / BLOCK);
#define ALTIUS_ROWS4(A, N, L) hipLaunchKernelGGL((binary_rows4<OP, KIND, A, N, L>), grid, dim3(BLOCK), 0, s, out, full, small, total, c, o)
    if (small_is_a) {
        if (nt) ALTIUS_ROWS4(true, true, true);
        else if (ntl) ALTIUS_ROWS4(true, false, true);
        else ALTIUS_ROWS4(true, false, false);
    } else {
        if (nt) ALTIUS_ROWS4(false, true, true);
        else if (ntl) ALTIUS_ROWS4(false, false, true);
        else ALTIUS_ROWS4(false, false, false);
    }
#undef ALTIUS_ROWS4
}

template <class OP>
void rows_any_launch(hipStream_t s, bool mod, bool small_is_a, bool nt, float *out, const float *full, const float *small,
                     uint32_t total, const FastDiv &c, const FastDiv &o) {
    const dim3 grid(((total + 3) / 4 + BLOCK - 1) / BLOCK);
#define ALTIUS_ROWS_ANY(M, A, N) hipLaunchKernelGGL((binary_rows_any<OP, M, A, N>), grid, dim3(BLOCK), 0, s, out, full, small, total, c, o)
#define ALTIUS_ROWS_ANY_M(M)                                  \
    if (small_is_a) {                                         \
        if (nt) ALTIUS_ROWS_ANY(M, true, true);               \
        else ALTIUS_ROWS_ANY(M, true, false);                 \
    } else {                                                  \
        if (nt) ALTIUS_ROWS_ANY(M, false, true);              \
        else ALTIUS_ROWS_ANY(M, false, false);                \
    }
    if (mod) { ALTIUS_ROWS_ANY_M(true) } else { ALTIUS_ROWS_ANY_M(false) }
#undef ALTIUS_ROWS_ANY_M
#undef ALTIUS_ROWS_ANY
}

template <class OP>
void rows4_launch(hipStream_t s, int kind, bool small_is_a, bool nt, bool ntl, float *out, const float *full, const float *small,
                  uint32_t total, const FastDiv &c, const FastDiv &o) {
    switch (kind) {
    case SMALL_VECTOR: rows4_launch_kind<OP, SMALL_VECTOR>(s, small_is_a, nt, ntl, out, full, small, total, c, o); break;
    case SMALL_VECTOR_OUTER: rows4_launch_kind<OP, SMALL_VECTOR_OUTER>(s, small_is_a, nt, ntl, out, full, small, total, c, o); break;
    case SMALL_COLUMN: rows4_launch_kind<OP, SMALL_COLUMN>(s, small_is_a, nt, ntl, out, full, small, total, c, o); break;
    default: rows4_launch_kind<OP, SMALL_COLUMN_MOD>(s, small_is_a, nt, ntl, out, full, small, total, c, o); break;
    }
}

}  // namespace

int launch_binary(DeviceCtx &ctx, int op, float *out, const float *a, const float *b, int rank,
                  const int64_t *out_dims, const int64_t *a_strides, const int64_t *b_strides) {
    if (op < AHIP_ADD || op > AHIP_POW) return ctx.fail(AHIP_ERR_ARG, "binary: unknown op");
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "binary: rank out of range");
    if (rank > 0 && (!out_dims || !a_strides || !b_strides))
        return ctx.fail(AHIP_ERR_ARG, "binary: null dims/strides");

    // Drop size-1 axes, then merge neighbours that both operands walk contiguously.
    int64_t dims[MAX_RANK], as[MAX_RANK], bs[MAX_RANK];
    int r = 0;
    size_t total = 1;
    for (int i = 0; i < rank; i++) {
        if (out_dims[i] < 0 || a_strides[i] < 0 || b_strides[i] < 0)
            return ctx.fail(AHIP_ERR_ARG, "binary: negative dim or stride");
        total *= (size_t)out_dims[i];
    }
    if (total == 0) return AHIP_OK;
    if (!out || !a || !b) return ctx.fail(AHIP_ERR_ARG, "binary: null tensor pointer");
    for (int i = 0; i < rank; i++) {
        if (out_dims[i] == 1) continue;
        if (r > 0 && as[r - 1] == a_strides[i] * out_dims[i] && bs[r - 1] == b_strides[i] * out_dims[i]) {
            dims[r - 1] *= out_dims[i];
            as[r - 1] = a_strides[i];
            bs[r - 1] = b_strides[i];
        } else {
            dims[r] = out_dims[i];
            as[r] = a_strides[i];
            bs[r] = b_strides[i];
            r++;
        }
    }
    if (r == 0) {  // a single element
        dims[0] = 1;
        as[0] = bs[0] = 0;
        r = 1;
    }

    // Classify the operands.
    auto classify = [&](const int64_t *st) {
        bool all_zero = true, contiguous = true;
        int64_t expect = 1;
        for (int i = r - 1; i >= 0; i--) {
            if (st[i] != 0) all_zero = false;
            if (st[i] != expect) contiguous = false;
            expect *= dims[i];
        }
        if (total == 1) return (int)SCALAR;
        return all_zero ? (int)SCALAR : contiguous ? (int)FULL : (int)STRIDED;
    };
    const int ma = classify(as), mb = classify(bs);

    // Pow takes the a*a shortcut only where the reference takes its
    // scalar-exponent path, i.e. not for equal shapes.
    const bool square = op == AHIP_POW && mb == SCALAR && ma != SCALAR;

    hipStream_t s = ctx.stream;
    if (total > ((size_t)1 << 38)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "binary: more than 2^38 elements");
    const bool nt = ctx.streaming(total * sizeof(float)), ntl = ctx.streaming_loads(total * sizeof(float));
    if (ma != STRIDED && mb != STRIDED) {
        const bool vec = aligned16(out) && (ma != FULL || aligned16(a)) && (mb != FULL || aligned16(b));
        switch (op) {
        case AHIP_ADD: flat_launch<OpAdd>(s, ma, mb, out, a, b, total, vec, nt, ntl); break;
        case AHIP_SUB: flat_launch<OpSub>(s, ma, mb, out, a, b, total, vec, nt, ntl); break;
        case AHIP_MUL: flat_launch<OpMul>(s, ma, mb, out, a, b, total, vec, nt, ntl); break;
        case AHIP_DIV: flat_launch<OpDiv>(s, ma, mb, out, a, b, total, vec, nt, ntl); break;
        case AHIP_POW:
            if (square) flat_launch<OpPowScalarExp>(s, ma, mb, out, a, b, total, vec, nt, ntl);
            else flat_launch<OpPow>(s, ma, mb, out, a, b, total, vec, nt, ntl);
            break;
        }
        return ctx.check(hipGetLastError(), "binary flat launch");
    }

    // Strided path: 32-bit index math, so split the outermost axis if needed.
    const size_t LIMIT = (size_t)1 << 31;
    size_t inner_elems = 1;
    for (int i = 1; i < r; i++) inner_elems *= (size_t)dims[i];
    if (inner_elems >= LIMIT)
        return ctx.fail(AHIP_ERR_UNSUPPORTED, "binary: broadcast inner extent exceeds 2^31 elements");
    for (int i = 0; i < r; i++)
        if ((uint64_t)as[i] >= LIMIT || (uint64_t)bs[i] >= LIMIT)
            return ctx.fail(AHIP_ERR_UNSUPPORTED, "binary: operand stride exceeds 2^31 elements");

    // One operand dense, the other a row per outer index: [N,R,C] op [N,1,C] (strides [C,0,1]) or
    // [R,C] op [C] (strides [0,1]).
    {
        const int64_t *ss = ma == STRIDED ? as : bs;  // strides of the small operand
        const int other = ma == STRIDED ? mb : ma;
        const bool pattern3 = r == 3 && ss[0] == dims[2] && ss[1] == 0 && ss[2] == 1;
        const bool pattern2 = r == 2 && ss[0] == 0 && ss[1] == 1;
        const int64_t C = dims[r - 1];
        // A block covers BLOCK*4 consecutive elements and stages two rows of the small operand, so
        // an outer index must span at least that many elements.
        if (other == FULL && pattern2 && (C == 2 || C == 3) && total < LIMIT && aligned16(out) && aligned16(ma == STRIDED ? b : a)) {
            const bool small_is_a = ma == STRIDED;
            const float *full = small_is_a ? b : a;
            const float *small = small_is_a ? a : b;
            switch (op) {
            case AHIP_ADD: short_vector_launch<OpAdd>(s, small_is_a, nt, out, full, small, (uint32_t)C, (uint32_t)total); break;
            case AHIP_SUB: short_vector_launch<OpSub>(s, small_is_a, nt, out, full, small, (uint32_t)C, (uint32_t)total); break;
            case AHIP_MUL: short_vector_launch<OpMul>(s, small_is_a, nt, out, full, small, (uint32_t)C, (uint32_t)total); break;
            case AHIP_DIV: short_vector_launch<OpDiv>(s, small_is_a, nt, out, full, small, (uint32_t)C, (uint32_t)total); break;
            case AHIP_POW: short_vector_launch<OpPow>(s, small_is_a, nt, out, full, small, (uint32_t)C, (uint32_t)total); break;
            }
            return ctx.check(hipGetLastError(), "binary short-vector launch");
        }
        const bool two_rows_suffice = pattern2 || (r == 3 && dims[1] * dims[2] >= BLOCK * 4);
        if (other == FULL && (pattern3 || pattern2) && two_rows_suffice && C >= 4 && C <= 512 && total < LIMIT &&
            aligned16(out) &&
            aligned16(ma == STRIDED ? b : a)) {
            RowBcast rb;
            rb.c = make_fastdiv((uint32_t)C);
            rb.rc = make_fastdiv((uint32_t)(pattern3 ? dims[1] * dims[2] : dims[0] * dims[1]));
            rb.n = pattern3 ? (uint32_t)dims[0] : 1u;
            rb.total = (uint32_t)total;
            const bool small_is_a = ma == STRIDED;
            const float *full = small_is_a ? b : a;
            const float *small = small_is_a ? a : b;
            switch (op) {
            case AHIP_ADD: rowbcast_launch<OpAdd>(s, small_is_a, nt, ntl, out, full, small, rb); break;
            case AHIP_SUB: rowbcast_launch<OpSub>(s, small_is_a, nt, ntl, out, full, small, rb); break;
            case AHIP_MUL: rowbcast_launch<OpMul>(s, small_is_a, nt, ntl, out, full, small, rb); break;
            case AHIP_DIV: rowbcast_launch<OpDiv>(s, small_is_a, nt, ntl, out, full, small, rb); break;
            case AHIP_POW: rowbcast_launch<OpPow>(s, small_is_a, nt, ntl, out, full, small, rb); break;
            }
            return ctx.check(hipGetLastError(), "binary row-broadcast launch");
        }
    }

    // Rows of whole float4s, one operand dense and the other constant along or across the row (see binary_rows4).
    {
        const int64_t *ss = ma == STRIDED ? as : bs;
        const int other = ma == STRIDED ? mb : ma;
        const bool small_is_a = ma == STRIDED;
        const float *full = small_is_a ? b : a;
        const float *small = small_is_a ? a : b;
        int kind = -1;
        uint32_t second = 1;
        if (r == 2 && ss[0] == 0 && ss[1] == 1) kind = SMALL_VECTOR;
        else if (r == 2 && ss[0] == 1 && ss[1] == 0) kind = SMALL_COLUMN;
        else if (r == 3 && ss[0] == dims[2] && ss[1] == 0 && ss[2] == 1) kind = SMALL_VECTOR_OUTER, second = (uint32_t)(dims[1] * dims[2]);
        else if (r == 3 && ss[0] == 0 && ss[1] == 1 && ss[2] == 0) kind = SMALL_COLUMN_MOD, second = (uint32_t)dims[1];
        const bool vector = kind == SMALL_VECTOR || kind == SMALL_VECTOR_OUTER;
        if (other == FULL && kind >= 0 && dims[r - 1] % 4 == 0 && total < LIMIT && aligned16(out) && aligned16(full) &&
            (!vector || aligned16(small))) {
            const FastDiv c = make_fastdiv((uint32_t)dims[r - 1]), o = make_fastdiv(second);
            switch (op) {
            case AHIP_ADD: rows4_launch<OpAdd>(s, kind, small_is_a, nt, ntl, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_SUB: rows4_launch<OpSub>(s, kind, small_is_a, nt, ntl, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_MUL: rows4_launch<OpMul>(s, kind, small_is_a, nt, ntl, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_DIV: rows4_launch<OpDiv>(s, kind, small_is_a, nt, ntl, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_POW: rows4_launch<OpPow>(s, kind, small_is_a, nt, ntl, out, full, small, (uint32_t)total, c, o); break;
            }
            return ctx.check(hipGetLastError(), "binary row-aligned broadcast launch");
        }
        // One value per row or per channel on rows of any other length from 4 up.
        if (other == FULL && (kind == SMALL_COLUMN || kind == SMALL_COLUMN_MOD) && dims[r - 1] >= 4 && total < LIMIT && aligned16(out) &&
            aligned16(full)) {
            const FastDiv c = make_fastdiv((uint32_t)dims[r - 1]), o = make_fastdiv(second);
            const bool mod = kind == SMALL_COLUMN_MOD;
            switch (op) {
            case AHIP_ADD: rows_any_launch<OpAdd>(s, mod, small_is_a, nt, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_SUB: rows_any_launch<OpSub>(s, mod, small_is_a, nt, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_MUL: rows_any_launch<OpMul>(s, mod, small_is_a, nt, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_DIV: rows_any_launch<OpDiv>(s, mod, small_is_a, nt, out, full, small, (uint32_t)total, c, o); break;
            case AHIP_POW: rows_any_launch<OpPow>(s, mod, small_is_a, nt, out, full, small, (uint32_t)total, c, o); break;
            }
            return ctx.check(hipGetLastError(), "binary per-row broadcast launch");
        }
    }

    Geom g;
    for (int d = 0; d < MAX_RANK; d++) {
        g.dims[d] = make_fastdiv(1);
        g.a_str[d] = g.b_str[d] = 0;
    }
    for (int d = 0; d < r; d++) {  // reverse: innermost first
        g.dims[d] = make_fastdiv((uint32_t)dims[r - 1 - d]);
        g.a_str[d] = (uint32_t)as[r - 1 - d];
        g.b_str[d] = (uint32_t)bs[r - 1 - d];
    }
    g.mode_a = ma;
    g.mode_b = mb;
    auto vec_ok = [&](const float *p, const uint32_t *st) {
        if (!aligned16(p) || st[0] != 1 || (g.dims[0].d & 3)) return 0;
        for (int d = 1; d < r; d++)
            if (st[d] & 3) return 0;
        return 1;
    };
    g.a_vec = vec_ok(a, g.a_str);
    g.b_vec = vec_ok(b, g.b_str);

    const size_t outer = (size_t)dims[0];
    size_t rows_per_launch = (LIMIT - 1) / inner_elems;
    if (rows_per_launch == 0) rows_per_launch = 1;
    for (size_t o0 = 0; o0 < outer; o0 += rows_per_launch) {
        const size_t o1 = o0 + rows_per_launch < outer ? o0 + rows_per_launch : outer;
        const uint32_t n = (uint32_t)((o1 - o0) * inner_elems);
        Geom gl = g;
        gl.dims[r - 1] = make_fastdiv((uint32_t)(o1 - o0));
        float *po = out + o0 * inner_elems;
        const float *pa = a + o0 * (size_t)as[0];
        const float *pb = b + o0 * (size_t)bs[0];
        // Four elements per lane need an innermost extent of at least 4 (one row change at most).
        const bool vec = aligned16(po) && (ma != FULL || aligned16(pa)) && (mb != FULL || aligned16(pb)) &&
                         gl.dims[0].d >= 4;
        if (!vec) gl.a_vec = gl.b_vec = 0;
        else {
            gl.a_vec = g.a_vec && aligned16(pa);
            gl.b_vec = g.b_vec && aligned16(pb);
        }
        switch (op) {
        case AHIP_ADD: strided_launch<OpAdd>(s, r, po, pa, pb, n, gl, vec, nt); break;
        case AHIP_SUB: strided_launch<OpSub>(s, r, po, pa, pb, n, gl, vec, nt); break;
        case AHIP_MUL: strided_launch<OpMul>(s, r, po, pa, pb, n, gl, vec, nt); break;
        case AHIP_DIV: strided_launch<OpDiv>(s, r, po, pa, pb, n, gl, vec, nt); break;
        case AHIP_POW:
            if (square) strided_launch<OpPowScalarExp>(s, r, po, pa, pb, n, gl, vec, nt);
            else strided_launch<OpPow>(s, r, po, pa, pb, n, gl, vec, nt);
            break;
        }
    }
    return ctx.check(hipGetLastError(), "binary strided launch");
}

}  // namespace altius
