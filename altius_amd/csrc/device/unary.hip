// Flat unary ops (Sqrt/Erf/Gelu/Sigmoid/HardSigmoid/Relu) for gfx950.
// One 16-byte load and one 16-byte store per lane and step, UNROLL steps per
// lane, block-contiguous.  Per-element formulas are in math.h.
//
// Reference: crates/session_interpreter/src/session.rs:608-619, 796-838,
// 905-931 and crates/session_interpreter/src/fast_math.rs.

#include "common.h"
#include "ctx.h"
#include "math.h"

#include <math.h>

namespace altius {
namespace {

using namespace dev;

struct FSqrt { __device__ __forceinline__ float operator()(float x) const { return sqrtf(x); } };
struct FErf { __device__ __forceinline__ float operator()(float x) const { return erf_elem(x); } };
struct FGelu { __device__ __forceinline__ float operator()(float x) const { return gelu_elem(x); } };
struct FSigmoid { __device__ __forceinline__ float operator()(float x) const { return sigmoid_elem(x); } };
struct FRelu { __device__ __forceinline__ float operator()(float x) const { return relu_elem(x); } };
struct FHardSigmoid {
    float alpha, beta;
    __device__ __forceinline__ float operator()(float x) const { return hard_sigmoid_elem(x, alpha, beta); }
};

constexpr int BLOCK = 256;

template <class F, int UNROLL>
__global__ __launch_bounds__(BLOCK) void unary_vec4(float *__restrict__ out, const float *__restrict__ in,
                                                    size_t n, F f) {
    const size_t n4 = n >> 2;
    const size_t base = (size_t)blockIdx.x * (BLOCK * UNROLL) + threadIdx.x;
    float4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * BLOCK;
        if (i < n4) v[u] = reinterpret_cast<const float4 *>(in)[i];
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const size_t i = base + (size_t)u * BLOCK;
        if (i < n4) {
            float4 r;
            r.x = f(v[u].x);
            r.y = f(v[u].y);
            r.z = f(v[u].z);
            r.w = f(v[u].w);
            reinterpret_cast<float4 *>(out)[i] = r;
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t i = (n4 << 2) + threadIdx.x;
        out[i] = f(in[i]);
    }
}

template <class F>
__global__ __launch_bounds__(BLOCK) void unary_scalar(float *__restrict__ out, const float *__restrict__ in,
                                                      size_t n, F f) {
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < n) out[i] = f(in[i]);
}

template <class F> void launch(hipStream_t s, float *out, const float *in, size_t n, F f) {
    const bool vec = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(in)) & 15u) == 0;
    if (vec) {
        constexpr int UNROLL = 4;
        size_t blocks = ((n >> 2) + (size_t)BLOCK * UNROLL - 1) / ((size_t)BLOCK * UNROLL);
        if (blocks == 0) blocks = 1;
        hipLaunchKernelGGL((unary_vec4<F, UNROLL>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
    } else {
        hipLaunchKernelGGL((unary_scalar<F>), dim3((unsigned)((n + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, s,
                           out, in, n, f);
    }
}

}  // namespace

int launch_unary(DeviceCtx &ctx, int op, float *out, const float *in, size_t n, float alpha, float beta) {
    if (op < AHIP_SQRT || op > AHIP_RELU) return ctx.fail(AHIP_ERR_ARG, "unary: unknown op");
    if (n == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "unary: null tensor pointer");
    if (n > ((size_t)1 << 40)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "unary: more than 2^40 elements");
    switch (op) {
    case AHIP_SQRT: launch(ctx.stream, out, in, n, FSqrt{}); break;
    case AHIP_ERF: launch(ctx.stream, out, in, n, FErf{}); break;
    case AHIP_GELU: launch(ctx.stream, out, in, n, FGelu{}); break;
    case AHIP_SIGMOID: launch(ctx.stream, out, in, n, FSigmoid{}); break;
    case AHIP_HARDSIGMOID: launch(ctx.stream, out, in, n, FHardSigmoid{alpha, beta}); break;
    case AHIP_RELU: launch(ctx.stream, out, in, n, FRelu{}); break;
    }
    return ctx.check(hipGetLastError(), "unary launch");
}

}  // namespace altius
