// Shared device-side helpers for the gfx950 kernels: 64-lane wavefront
// reductions, block reductions through LDS, and bit casts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace altius {
namespace dev {

constexpr int WAVE = 64;

// Neighbouring pieces of work under one L2.  Blocks i, i + 8, i + 16, ... of a launch run on one of the part's eight
// XCDs, each with an L2 of its own, so blocks that take pieces i and i + 1 of a tensor never share one: a cache line
// that two neighbouring pieces both touch (rows, slabs or patches that do not end on a 128-byte boundary) is fetched
// twice and goes out to memory as two partial lines.  This maps block `id` of `n` to a piece such that each XCD takes
// a run of consecutive pieces, in the order of its blocks: the parts of such a line then meet in one L2 while it is
// still there.  A bijection of 0 .. n - 1; where blocks really land is a matter of speed only.
__device__ __forceinline__ uint32_t piece_of_block(uint32_t id, uint32_t n) {
    const uint32_t xcd = id & 7u, each = n >> 3, more = n & 7u;
    return xcd * each + (xcd < more ? xcd : more) + (id >> 3);
}

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// 16-byte global accesses, optionally with the non-temporal hint.  Streaming
// kernels over tensors far larger than the 256 MB Infinity Cache run ~8 % faster
// with it; smaller tensors are left cacheable so the next kernel can hit.
typedef float v4f __attribute__((ext_vector_type(4)));

template <bool NT> __device__ __forceinline__ float4 load4(const float *p) {
    if (NT) {
        const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
        return make_float4(t.x, t.y, t.z, t.w);
    }
    return *reinterpret_cast<const float4 *>(p);
}
// The same for addresses that are only 4-byte aligned: the part's 16-byte global accesses need no more than that, and
// the compiler emits them for a vector type declared with that alignment.
typedef float v4f_dword __attribute__((ext_vector_type(4), aligned(4)));
template <bool NT> __device__ __forceinline__ float4 load4_dword_aligned(const float *p) {
    const v4f_dword t = NT ? __builtin_nontemporal_load(reinterpret_cast<const v4f_dword *>(p)) : *reinterpret_cast<const v4f_dword *>(p);
    return make_float4(t.x, t.y, t.z, t.w);
}
template <bool NT> __device__ __forceinline__ void store4_dword_aligned(float *p, const float4 &v) {
    const v4f_dword t = {v.x, v.y, v.z, v.w};
    if (NT) __builtin_nontemporal_store(t, reinterpret_cast<v4f_dword *>(p));
    else *reinterpret_cast<v4f_dword *>(p) = t;
}
template <bool NT> __device__ __forceinline__ void store4(float *p, const float4 &v) {
    if (NT) {
        v4f t;
        t.x = v.x;
        t.y = v.y;
        t.z = v.z;
        t.w = v.w;
        __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
    } else {
        *reinterpret_cast<float4 *>(p) = v;
    }
}

// Division of an index below 2^31 by a fixed divisor as multiply-high, add, shift (the
// divisor's magic numbers are computed once on the host).
struct FastDiv {
    uint32_t d, mul, shift;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return (__umulhi(n, mul) + n) >> shift; }
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    uint32_t shift = 0;
    while (shift < 32 && ((uint64_t)1 << shift) < d) shift++;
    const uint64_t one = 1;
    f.mul = (uint32_t)(((one << 32) * ((one << shift) - d)) / d + 1);
    f.shift = shift;
    return f;
}

// The non-NaN operand wins (f32::max in the reference).
__device__ __forceinline__ float nanmax(float a, float b) { return fmaxf(a, b); }

struct SumOp {
    static __device__ __forceinline__ float identity() { return 0.0f; }
    static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
struct MaxOp {
    // NaN is the identity of a NaN-ignoring max.
    static __device__ __forceinline__ float identity() { return __builtin_nanf(""); }
    static __device__ __forceinline__ float apply(float a, float b) { return nanmax(a, b); }
};

// Cross-lane moves that cost no LDS access: DPP row rotations inside each row
// of 16 lanes, ds_swizzle for the 16-lane exchange inside each half wave.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
constexpr int DPP_ROW_ROR = 0x120;  // + n: rotate right by n lanes within a row of 16

constexpr int DPP_QUAD_XOR1 = 0xB1;     // quad_perm [1,0,3,2]: lane ^ 1
constexpr int DPP_QUAD_XOR2 = 0x4E;     // quad_perm [2,3,0,1]: lane ^ 2
constexpr int DPP_ROW_HALF_MIRROR = 0x141;  // lane i of each group of 8 reads lane 7 - i

// All-reduce over aligned groups of SUB lanes (SUB = 4, 8, 16, 32 or 64); every lane
// ends with the result of its group.  Rotation and exchange steps combine the
// same two partial results in every lane of a pair and OP is commutative, so all
// lanes of a group hold bit-identical values.
template <class OP, int SUB> __device__ __forceinline__ float subwave_allreduce(float v) {
    static_assert(SUB == 4 || SUB == 8 || SUB == 16 || SUB == 32 || SUB == 64, "group size");
    if (SUB <= 8) {
        v = OP::apply(v, dpp_move<DPP_QUAD_XOR1>(v));
        v = OP::apply(v, dpp_move<DPP_QUAD_XOR2>(v));
        // every lane of a quad now holds the quad's result, so the mirror image is the other quad's
        if (SUB == 8) v = OP::apply(v, dpp_move<DPP_ROW_HALF_MIRROR>(v));
        return v;
    }
    v = OP::apply(v, dpp_move<DPP_ROW_ROR + 8>(v));
    v = OP::apply(v, dpp_move<DPP_ROW_ROR + 4>(v));
    v = OP::apply(v, dpp_move<DPP_ROW_ROR + 2>(v));
    v = OP::apply(v, dpp_move<DPP_ROW_ROR + 1>(v));
    if (SUB >= 32) {
        // lane ^ 16: swizzle bit mode, and_mask 0x1F, or_mask 0, xor_mask 0x10
        v = OP::apply(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)));
    }
    if (SUB == 64) v = OP::apply(v, __shfl_xor(v, 32, WAVE));
    return v;
}

// All-reduce over the 64 lanes of a wavefront.
template <class OP> __device__ __forceinline__ float wave_reduce(float v) {
    return subwave_allreduce<OP, WAVE>(v);
}

// Reduction over a whole block of NWAVES wavefronts.  `lds` holds NWAVES floats.
// Every thread ends with the result.  Contains two barriers.
template <class OP, int NWAVES>
__device__ __forceinline__ float block_reduce(float v, float *lds) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    v = wave_reduce<OP>(v);
    __syncthreads();  // protects lds against a previous use
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = OP::identity();
#pragma unroll
    for (int w = 0; w < NWAVES; w++) r = OP::apply(r, lds[w]);
    return r;
}

}  // namespace dev
}  // namespace altius
