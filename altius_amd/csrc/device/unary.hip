// Flat unary ops (Sqrt/Erf/Gelu/Sigmoid/HardSigmoid/Relu) for gfx950.
// One 16-byte load and one 16-byte store per lane.  Per-element formulas are in
// math.h.
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
struct FTanh { __device__ __forceinline__ float operator()(float x) const { return tanh_elem(x); } };
struct FRelu { __device__ __forceinline__ float operator()(float x) const { return relu_elem(x); } };
struct FHardSigmoid {
    float alpha, beta;
    __device__ __forceinline__ float operator()(float x) const { return hard_sigmoid_elem(x, alpha, beta); }
};

struct FLeakyRelu {
    float alpha;
    __device__ __forceinline__ float operator()(float x) const { return leaky_relu_elem(x, alpha); }
};
struct FClip {
    float lo, hi;
    __device__ __forceinline__ float operator()(float x) const { return clip_elem(x, lo, hi); }
};
// Exp and Round have no kernel in the reference interpreter (session.rs:219-224): correctly
// rounded-to-1-ulp expf, and round-half-to-even as ONNX defines Round.
// x / alpha with a true division: the second half of GlobalAveragePool (sum / area, session.rs:291).
struct FDivBy {
    float d;
    __device__ __forceinline__ float operator()(float x) const { return x / d; }
};
struct FExp { __device__ __forceinline__ float operator()(float x) const { return expf(x); } };
struct FRound { __device__ __forceinline__ float operator()(float x) const { return rintf(x); } };

constexpr int BLOCK = 256;

// One float4 per lane: on this part a streaming kernel is fastest with the
// smallest per-lane footprint and the occupancy that comes with it.
// NT: non-temporal stores (and loads) for tensors too large to be found in a cache by the next kernel.  NTL alone:
// non-temporal loads of a mid-sized input that nobody reads again, while the result is stored the ordinary way so
// that the next kernel finds it in the Infinity Cache.
template <class F, bool NT, bool NTL = NT>
__global__ __launch_bounds__(BLOCK) void unary_vec4(float *__restrict__ out, const float *__restrict__ in,
                                                    size_t n, F f) {
    const size_t n4 = n >> 2;
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < n4) {
        const float4 v = load4<NTL>(in + 4 * i);
        float4 r;
        r.x = f(v.x);
        r.y = f(v.y);
        r.z = f(v.z);
        r.w = f(v.w);
        store4<NT>(out + 4 * i, r);
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t j = (n4 << 2) + threadIdx.x;
        out[j] = f(in[j]);
    }
}

// Tensors on 4-byte boundaries only: the same four elements per lane through 16-byte accesses that are not aligned.
template <class F, bool NT>
__global__ __launch_bounds__(BLOCK) void unary_vec4_any(float *__restrict__ out, const float *__restrict__ in, size_t n, F f) {
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    const size_t n4 = n >> 2;
    if (i < n4) {
        const float4 v = load4_dword_aligned<NT>(in + 4 * i);
        store4_dword_aligned<NT>(out + 4 * i, make_float4(f(v.x), f(v.y), f(v.z), f(v.w)));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const size_t j = (n4 << 2) + threadIdx.x;
        out[j] = f(in[j]);
    }
}

template <class F>
__global__ __launch_bounds__(BLOCK) void unary_scalar(float *__restrict__ out, const float *__restrict__ in,
                                                      size_t n, F f) {
    const size_t i = (size_t)blockIdx.x * BLOCK + threadIdx.x;
    if (i < n) out[i] = f(in[i]);
}

template <class F> void launch(hipStream_t s, float *out, const float *in, size_t n, F f, bool nt, bool ntl) {
    const uintptr_t off_in = reinterpret_cast<uintptr_t>(in) & 15u, off_out = reinterpret_cast<uintptr_t>(out) & 15u;
    const bool vec = (off_in | off_out) == 0;
    if (vec) {
        size_t blocks = ((n >> 2) + BLOCK - 1) / BLOCK;
        if (blocks == 0) blocks = 1;
        if (nt)
            hipLaunchKernelGGL((unary_vec4<F, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
        else if (ntl)
            hipLaunchKernelGGL((unary_vec4<F, false, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
        else
            hipLaunchKernelGGL((unary_vec4<F, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
    } else if (n >= 4 * BLOCK && ((off_in | off_out) & 3u) == 0) {
        const size_t blocks = ((n >> 2) + BLOCK - 1) / BLOCK;
        if (nt) hipLaunchKernelGGL((unary_vec4_any<F, true>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
        else hipLaunchKernelGGL((unary_vec4_any<F, false>), dim3((unsigned)blocks), dim3(BLOCK), 0, s, out, in, n, f);
    } else {
        hipLaunchKernelGGL((unary_scalar<F>), dim3((unsigned)((n + BLOCK - 1) / BLOCK)), dim3(BLOCK), 0, s,
                           out, in, n, f);
    }
}

}  // namespace

int launch_unary(DeviceCtx &ctx, int op, float *out, const float *in, size_t n, float alpha, float beta) {
    if (op < AHIP_SQRT || op > AHIP_DIV_BY) return ctx.fail(AHIP_ERR_ARG, "unary: unknown op");
    if (n == 0) return AHIP_OK;
    if (!out || !in) return ctx.fail(AHIP_ERR_ARG, "unary: null tensor pointer");
    if (n > ((size_t)1 << 38)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "unary: more than 2^38 elements");
    const bool nt = ctx.streaming(n * sizeof(float)), ntl = ctx.streaming_loads(n * sizeof(float));
    switch (op) {
    case AHIP_SQRT: launch(ctx.stream, out, in, n, FSqrt{}, nt, ntl); break;
    case AHIP_ERF: launch(ctx.stream, out, in, n, FErf{}, nt, ntl); break;
    case AHIP_GELU: launch(ctx.stream, out, in, n, FGelu{}, nt, ntl); break;
    case AHIP_SIGMOID: launch(ctx.stream, out, in, n, FSigmoid{}, nt, ntl); break;
    case AHIP_HARDSIGMOID: launch(ctx.stream, out, in, n, FHardSigmoid{alpha, beta}, nt, ntl); break;
    case AHIP_RELU: launch(ctx.stream, out, in, n, FRelu{}, nt, ntl); break;
    case AHIP_TANH: launch(ctx.stream, out, in, n, FTanh{}, nt, ntl); break;
    case AHIP_LEAKYRELU: launch(ctx.stream, out, in, n, FLeakyRelu{alpha}, nt, ntl); break;
    case AHIP_EXP: launch(ctx.stream, out, in, n, FExp{}, nt, ntl); break;
    case AHIP_ROUND: launch(ctx.stream, out, in, n, FRound{}, nt, ntl); break;
    case AHIP_CLIP: launch(ctx.stream, out, in, n, FClip{alpha, beta}, nt, ntl); break;
    case AHIP_DIV_BY: launch(ctx.stream, out, in, n, FDivBy{alpha}, nt, ntl); break;
    }
    return ctx.check(hipGetLastError(), "unary launch");
}

}  // namespace altius
