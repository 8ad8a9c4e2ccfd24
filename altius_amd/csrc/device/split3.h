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

}  // namespace dev
}  // namespace altius
