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
// Flat kernel: both operands are FULL or SCALAR.  UNROLL float4 per lane,
// block-contiguous so that a block's accesses stay coalesced.
// ---------------------------------------------------------------------------
template <class OP, int MA, int MB, int UNROLL>
__global__ __launch_bounds__(BLOCK) void binary_flat_vec4(float *__restrict__ out,
                                                          const float *__restrict__ a,
                                                          const float *__restrict__ b, size_t n) {
    const size_t n4 = n >> 2;
    const size_t base = (size_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    float sa = 0.f, sb = 0.f;
    if (MA == SCALAR) sa = a[0];
    if (MB == SCALAR) sb = b[0];
    float4 va[UNROLL], vb[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * BLOCK;
        if (i < n4) {
            if (MA == FULL) va[u] = reinterpret_cast<const float4 *>(a)[i];
            if (MB == FULL) vb[u] = reinterpret_cast<const float4 *>(b)[i];
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * BLOCK;
        if (i < n4) {
            float4 x = MA == FULL ? va[u] : make_float4(sa, sa, sa, sa);
            float4 y = MB == FULL ? vb[u] : make_float4(sb, sb, sb, sb);
            float4 r;
            r.x = OP::f(x.x, y.x);
            r.y = OP::f(x.y, y.y);
            r.z = OP::f(x.z, y.z);
            r.w = OP::f(x.w, y.w);
            reinterpret_cast<float4 *>(out)[i] = r;
        }
    }
    // The last (n % 4) elements.
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t i = (n4 << 2) + threadIdx.x;
        out[i] = OP::f(MA == FULL ? a[i] : sa, MB == FULL ? b[i] : sb);
    }
}

// Same, one element per lane, for buffers that are not 16-byte aligned.
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
struct Geom {
    // Axis 0 is the innermost (fastest) output axis.
    uint32_t dims[MAX_RANK];
    uint32_t a_str[MAX_RANK];
    uint32_t b_str[MAX_RANK];
    int mode_a, mode_b;  // Mode
    // The operand can be read 16 bytes at a time: innermost stride 1, innermost
    // extent and every other stride multiples of 4, base 16-byte aligned.
    int a_vec, b_vec;
};

template <int RANK> struct Cursor {
    uint32_t c[RANK];
    uint32_t a_off, b_off;

    __device__ __forceinline__ void init(const Geom &g, uint32_t flat) {
        a_off = 0;
        b_off = 0;
#pragma unroll
        for (int d = 0; d < RANK; d++) {
            const uint32_t q = flat / g.dims[d];
            c[d] = flat - q * g.dims[d];
            flat = q;
            a_off += c[d] * g.a_str[d];
            b_off += c[d] * g.b_str[d];
        }
    }
    // Advances by one output element.
    __device__ __forceinline__ void next(const Geom &g) {
        c[0]++;
        a_off += g.a_str[0];
        b_off += g.b_str[0];
        if (c[0] == g.dims[0]) {
#pragma unroll
            for (int d = 0; d < RANK - 1; d++) {
                if (c[d] != g.dims[d]) break;
                c[d] = 0;
                a_off -= g.dims[d] * g.a_str[d];
                b_off -= g.dims[d] * g.b_str[d];
                c[d + 1]++;
                a_off += g.a_str[d + 1];
                b_off += g.b_str[d + 1];
            }
        }
    }
};

template <class OP, int RANK, int VEC>
__global__ __launch_bounds__(BLOCK) void binary_strided(float *__restrict__ out,
                                                        const float *__restrict__ a,
                                                        const float *__restrict__ b, uint32_t n,
                                                        const Geom g) {
    const uint32_t nvec = (n + VEC - 1) / VEC;
    const uint32_t t = blockIdx.x * BLOCK + threadIdx.x;
    if (t >= nvec) return;
    const uint32_t i0 = t * VEC;
    const bool whole = i0 + VEC <= n;

    Cursor<RANK> cur;
    cur.init(g, i0);

    float x[VEC], y[VEC];
    const bool same_row = cur.c[0] + VEC <= g.dims[0];

    // Operand a.
    if (g.mode_a == FULL) {
        if (VEC == 4 && whole) {
            const float4 v = *reinterpret_cast<const float4 *>(a + i0);
            x[0] = v.x; x[1 % VEC] = v.y; x[2 % VEC] = v.z; x[3 % VEC] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) x[j] = i0 + j < n ? a[i0 + j] : 0.f;
        }
    } else if (g.mode_a == SCALAR) {
        const float s = a[0];
#pragma unroll
        for (int j = 0; j < VEC; j++) x[j] = s;
    }
    // Operand b.
    if (g.mode_b == FULL) {
        if (VEC == 4 && whole) {
            const float4 v = *reinterpret_cast<const float4 *>(b + i0);
            y[0] = v.x; y[1 % VEC] = v.y; y[2 % VEC] = v.z; y[3 % VEC] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) y[j] = i0 + j < n ? b[i0 + j] : 0.f;
        }
    } else if (g.mode_b == SCALAR) {
        const float s = b[0];
#pragma unroll
        for (int j = 0; j < VEC; j++) y[j] = s;
    }
    // Strided operands.
    if (g.mode_a == STRIDED || g.mode_b == STRIDED) {
        if (VEC == 4 && whole && same_row) {
            if (g.mode_a == STRIDED) {
                if (g.a_vec) {
                    const float4 v = *reinterpret_cast<const float4 *>(a + cur.a_off);
                    x[0] = v.x; x[1 % VEC] = v.y; x[2 % VEC] = v.z; x[3 % VEC] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; j++) x[j] = a[cur.a_off + j * g.a_str[0]];
                }
            }
            if (g.mode_b == STRIDED) {
                if (g.b_vec) {
                    const float4 v = *reinterpret_cast<const float4 *>(b + cur.b_off);
                    y[0] = v.x; y[1 % VEC] = v.y; y[2 % VEC] = v.z; y[3 % VEC] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; j++) y[j] = b[cur.b_off + j * g.b_str[0]];
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                if (i0 + j < n) {
                    if (g.mode_a == STRIDED) x[j] = a[cur.a_off];
                    if (g.mode_b == STRIDED) y[j] = b[cur.b_off];
                    if (j + 1 < VEC) cur.next(g);
                }
            }
        }
    }

    if (VEC == 4 && whole) {
        float4 r;
        r.x = OP::f(x[0], y[0]);
        r.y = OP::f(x[1 % VEC], y[1 % VEC]);
        r.z = OP::f(x[2 % VEC], y[2 % VEC]);
        r.w = OP::f(x[3 % VEC], y[3 % VEC]);
        *reinterpret_cast<float4 *>(out + i0) = r;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++)
            if (i0 + j < n) out[i0 + j] = OP::f(x[j], y[j]);
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class OP, int MA, int MB>
void flat_dispatch(hipStream_t s, float *out, const float *a, const float *b, size_t n, bool vec) {
    if (vec) {
        constexpr int UNROLL = 4;
        const size_t n4 = n >> 2;
        size_t blocks = (n4 + (size_t)BLOCK * UNROLL - 1) / ((size_t)BLOCK * UNROLL);
        if (blocks == 0) blocks = 1;
        hipLaunchKernelGGL((binary_flat_vec4<OP, MA, MB, UNROLL>), dim3((unsigned)blocks), dim3(BLOCK),
                           0, s, out, a, b, n);
    } else {
        const size_t blocks = (n + BLOCK - 1) / BLOCK;
        hipLaunchKernelGGL((binary_flat_scalar<OP, MA, MB>), dim3((unsigned)blocks), dim3(BLOCK), 0, s,
                           out, a, b, n);
    }
}

template <class OP>
void flat_launch(hipStream_t s, int ma, int mb, float *out, const float *a, const float *b, size_t n,
                 bool vec) {
    if (ma == FULL && mb == FULL) flat_dispatch<OP, FULL, FULL>(s, out, a, b, n, vec);
    else if (ma == FULL && mb == SCALAR) flat_dispatch<OP, FULL, SCALAR>(s, out, a, b, n, vec);
    else if (ma == SCALAR && mb == FULL) flat_dispatch<OP, SCALAR, FULL>(s, out, a, b, n, vec);
    else flat_dispatch<OP, SCALAR, SCALAR>(s, out, a, b, n, vec);
}

template <class OP, int RANK>
void strided_dispatch(hipStream_t s, float *out, const float *a, const float *b, uint32_t n,
                      const Geom &g, bool vec) {
    if (vec) {
        const uint32_t nvec = (n + 3) / 4;
        hipLaunchKernelGGL((binary_strided<OP, RANK, 4>), dim3((nvec + BLOCK - 1) / BLOCK), dim3(BLOCK),
                           0, s, out, a, b, n, g);
    } else {
        hipLaunchKernelGGL((binary_strided<OP, RANK, 1>), dim3((n + BLOCK - 1) / BLOCK), dim3(BLOCK), 0,
                           s, out, a, b, n, g);
    }
}

template <class OP>
void strided_launch(hipStream_t s, int rank, float *out, const float *a, const float *b, uint32_t n,
                    const Geom &g, bool vec) {
    if (rank <= 2) strided_dispatch<OP, 2>(s, out, a, b, n, g, vec);
    else if (rank == 3) strided_dispatch<OP, 3>(s, out, a, b, n, g, vec);
    else if (rank == 4) strided_dispatch<OP, 4>(s, out, a, b, n, g, vec);
    else strided_dispatch<OP, MAX_RANK>(s, out, a, b, n, g, vec);
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
    if (ma != STRIDED && mb != STRIDED) {
        const bool vec = aligned16(out) && (ma != FULL || aligned16(a)) && (mb != FULL || aligned16(b));
        switch (op) {
        case AHIP_ADD: flat_launch<OpAdd>(s, ma, mb, out, a, b, total, vec); break;
        case AHIP_SUB: flat_launch<OpSub>(s, ma, mb, out, a, b, total, vec); break;
        case AHIP_MUL: flat_launch<OpMul>(s, ma, mb, out, a, b, total, vec); break;
        case AHIP_DIV: flat_launch<OpDiv>(s, ma, mb, out, a, b, total, vec); break;
        case AHIP_POW:
            if (square) flat_launch<OpPowScalarExp>(s, ma, mb, out, a, b, total, vec);
            else flat_launch<OpPow>(s, ma, mb, out, a, b, total, vec);
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

    Geom g;
    for (int d = 0; d < MAX_RANK; d++) {
        g.dims[d] = 1;
        g.a_str[d] = g.b_str[d] = 0;
    }
    for (int d = 0; d < r; d++) {  // reverse: innermost first
        g.dims[d] = (uint32_t)dims[r - 1 - d];
        g.a_str[d] = (uint32_t)as[r - 1 - d];
        g.b_str[d] = (uint32_t)bs[r - 1 - d];
    }
    g.mode_a = ma;
    g.mode_b = mb;
    auto vec_ok = [&](const float *p, const uint32_t *st) {
        if (!aligned16(p) || st[0] != 1 || (g.dims[0] & 3)) return 0;
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
        gl.dims[r - 1] = (uint32_t)(o1 - o0);
        float *po = out + o0 * inner_elems;
        const float *pa = a + o0 * (size_t)as[0];
        const float *pb = b + o0 * (size_t)bs[0];
        const bool vec = aligned16(po) && (ma != FULL || aligned16(pa)) && (mb != FULL || aligned16(pb));
        if (!vec) gl.a_vec = gl.b_vec = 0;
        else {
            gl.a_vec = g.a_vec && aligned16(pa);
            gl.b_vec = g.b_vec && aligned16(pb);
        }
        switch (op) {
        case AHIP_ADD: strided_launch<OpAdd>(s, r, po, pa, pb, n, gl, vec); break;
        case AHIP_SUB: strided_launch<OpSub>(s, r, po, pa, pb, n, gl, vec); break;
        case AHIP_MUL: strided_launch<OpMul>(s, r, po, pa, pb, n, gl, vec); break;
        case AHIP_DIV: strided_launch<OpDiv>(s, r, po, pa, pb, n, gl, vec); break;
        case AHIP_POW:
            if (square) strided_launch<OpPowScalarExp>(s, r, po, pa, pb, n, gl, vec);
            else strided_launch<OpPow>(s, r, po, pa, pb, n, gl, vec);
            break;
        }
    }
    return ctx.check(hipGetLastError(), "binary strided launch");
}

}  // namespace altius
