// An fp32 value as the exact sum of three bf16 numbers (8 + 8 + 8 significand bits), the form in which the
// products on the bf16 matrix cores take their operands (gemm_split.hip, attention.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace altius {
namespace dev {

__device__ __forceinline__ uint32_t round_bf16(uint32_t u) { return (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u; }

// The upper halves of three floats whose sum is x.  Round-to-nearest at each step keeps the
// residuals small and sign-symmetric; each residual is exact (it has at most 16, then 8 significant
// bits).  A value that would round up to infinity is truncated instead; infinities and NaNs stay in
// the first plane alone.
__device__ __forceinline__ void split3(float x, uint32_t &h0, uint32_t &h1, uint32_t &h2) {
    const uint32_t u = __float_as_uint(x);
    const bool finite = (u & 0x7f800000u) != 0x7f800000u;
    uint32_t r0 = round_bf16(u);
    if ((r0 & 0x7f800000u) == 0x7f800000u) {
        r0 = u & 0xffff0000u;
        if (!finite && (u & 0x007fffffu)) r0 |= 0x00400000u;  // a NaN whose payload sat in the low half
    }
    const float e1 = finite ? x - __uint_as_float(r0) : 0.0f;
    const uint32_t r1 = round_bf16(__float_as_uint(e1));
    const float e2 = e1 - __uint_as_float(r1);
    const uint32_t r2 = round_bf16(__float_as_uint(e2));
    h0 = r0 >> 16;
    h1 = r1 >> 16;
    h2 = r2 >> 16;
}

// The same for two values at once with the hardware's float -> bf16 conversion (round to nearest even, like
// round_bf16): the low half of p_i is x0's plane i, the high half x1's.  A value that the conversion rounds up to
// infinity, an infinity or a NaN (exponent bits all ones in a first plane) takes split3's route.
__device__ __forceinline__ void split3_pair(float x0, float x1, uint32_t &p0, uint32_t &p1, uint32_t &p2) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    p0 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){x0, x1}, bf16x2));
    const float r0 = x0 - __uint_as_float(p0 << 16), r1 = x1 - __uint_as_float(p0 & 0xffff0000u);
    p1 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){r0, r1}, bf16x2));
    const float s0 = r0 - __uint_as_float(p1 << 16), s1 = r1 - __uint_as_float(p1 & 0xffff0000u);
    p2 = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){s0, s1}, bf16x2));
    if (__builtin_expect(((p0 & 0x7f80u) == 0x7f80u) | ((p0 & 0x7f800000u) == 0x7f800000u), 0)) {
        uint32_t a[3], b[3];
        split3(x0, a[0], a[1], a[2]);
        split3(x1, b[0], b[1], b[2]);
        p0 = a[0] | (b[0] << 16), p1 = a[1] | (b[1] << 16), p2 = a[2] | (b[2] << 16);
    }
}

}  // namespace dev
}  // namespace altius
