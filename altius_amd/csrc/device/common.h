// Shared device-side helpers for the gfx950 kernels: 64-lane wavefront
// reductions, block reductions through LDS, and bit casts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace altius {
namespace dev {

constexpr int WAVE = 64;

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

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

// Butterfly over the 64 lanes of a wavefront; every lane ends with the result.
template <class OP> __device__ __forceinline__ float wave_reduce(float v) {
#pragma unroll
    for (int m = WAVE / 2; m >= 1; m >>= 1) v = OP::apply(v, __shfl_xor(v, m, WAVE));
    return v;
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
