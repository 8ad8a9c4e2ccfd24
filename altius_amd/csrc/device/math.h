// Per-element arithmetic of the interpreter's approximated functions, written
// for the device.  The formulas follow the reference bit for bit: explicit
// fmaf exactly where the reference uses mul_add, separate multiply/add
// elsewhere (the translation unit is compiled with -ffp-contract=off), IEEE
// correctly rounded division and square root.
#pragma once

#include "common.h"

namespace altius {
namespace dev {

// Constants of crates/session_interpreter/src/fast_math.rs:105-117,190-203.
constexpr float ROUNDING_BIAS = 12582912.0f;
constexpr float LOG2RECIPROCAL = 1.44269504088896341f;
constexpr float LOG2HIGH = -6.93145752e-1f;
constexpr float LOG2LOW = -1.42860677e-6f;
constexpr float POLY_0 = 0.0013780593872f;
constexpr float POLY_1 = 0.0083731245250f;
constexpr float POLY_2 = 0.0416695363820f;
constexpr float POLY_3 = 0.1666647195816f;
constexpr float POLY_4 = 0.4999998509884f;
constexpr float POLY_56 = 1.0000000000000f;
constexpr int32_t MINIMUM_EXPONENT = -1056964608;
constexpr int32_t MAXIMUM_EXPONENT = 0x3F800000;

// f32::clamp: comparisons only, NaN passes through.
__device__ __forceinline__ float rclamp(float x, float lo, float hi) {
    x = x < lo ? lo : x;
    x = x > hi ? hi : x;
    return x;
}

// exp(x - max) as Softmax computes it (fast_math.rs:130-150): clamp below at
// -88.37626, round-to-nearest range reduction with the 1.5*2^23 bias, two-step
// Cody-Waite remainder, degree-6 Horner polynomial, exponent bits stuffed in.
__device__ __forceinline__ float softmax_exp(float x, float mx) {
    float v = nanmax(x - mx, -88.37626f);
    float biased = __builtin_fmaf(v, LOG2RECIPROCAL, ROUNDING_BIAS);
    float m = biased - ROUNDING_BIAS;
    v = __builtin_fmaf(m, LOG2HIGH, v);
    v = __builtin_fmaf(m, LOG2LOW, v);
    uint32_t normal = (f2u(biased) << 23) + (uint32_t)MAXIMUM_EXPONENT;
    float p = POLY_0;
    p = __builtin_fmaf(p, v, POLY_1);
    p = __builtin_fmaf(p, v, POLY_2);
    p = __builtin_fmaf(p, v, POLY_3);
    p = __builtin_fmaf(p, v, POLY_4);
    p = __builtin_fmaf(p, v, POLY_56);
    p = __builtin_fmaf(p, v, POLY_56);
    return p * u2f(normal);
}

// Op::Sigmoid (fast_math.rs:214-244): exp(-x) with the exponent split into an
// "overflow" and a "normal" part, then a true division.
__device__ __forceinline__ float sigmoid_elem(float x) {
    float v = rclamp(-x, -103.9720840454f, 88.7762626647950f);
    float biased = __builtin_fmaf(v, LOG2RECIPROCAL, ROUNDING_BIAS);
    float m = biased - ROUNDING_BIAS;
    v = __builtin_fmaf(m, LOG2HIGH, v);
    v = __builtin_fmaf(m, LOG2LOW, v);
    int32_t overflow = (int32_t)(f2u(biased) << 23);
    int32_t normal = overflow < MAXIMUM_EXPONENT ? overflow : MAXIMUM_EXPONENT;
    normal = normal > MINIMUM_EXPONENT ? normal : MINIMUM_EXPONENT;
    uint32_t of = (uint32_t)overflow - (uint32_t)normal + (uint32_t)MAXIMUM_EXPONENT;
    uint32_t nf = (uint32_t)normal + (uint32_t)MAXIMUM_EXPONENT;
    float p = POLY_0;
    p = __builtin_fmaf(p, v, POLY_1);
    p = __builtin_fmaf(p, v, POLY_2);
    p = __builtin_fmaf(p, v, POLY_3);
    p = __builtin_fmaf(p, v, POLY_4);
    p = __builtin_fmaf(p, v, POLY_56);
    v = v * u2f(of);
    p = __builtin_fmaf(p, v, u2f(of));
    p = p * u2f(nf);
    return 1.0f / (1.0f + p);
}

// The 13/6-degree rational tanh shared by Op::Tanh (session.rs:860-877) and
// Op::Gelu (fast_math.rs:306-322), applied to an already clamped argument.
__device__ __forceinline__ float rational_tanh(float v) {
    constexpr float ALPHA_13 = -2.76076847742355e-16f;
    constexpr float ALPHA_11 = 2.00018790482477e-13f;
    constexpr float ALPHA_9 = -8.60467152213735e-11f;
    constexpr float ALPHA_7 = 5.12229709037114e-08f;
    constexpr float ALPHA_5 = 1.48572235717979e-05f;
    constexpr float ALPHA_3 = 6.37261928875436e-04f;
    constexpr float ALPHA_1 = 4.89352455891786e-03f;
    constexpr float BETA_6 = 1.19825839466702e-06f;
    constexpr float BETA_4 = 1.18534705686654e-04f;
    constexpr float BETA_2 = 2.26843463243900e-03f;
    constexpr float BETA_0 = 4.89352518554385e-03f;
    float v2 = v * v;
    float p = __builtin_fmaf(v2, ALPHA_13, ALPHA_11);
    p = __builtin_fmaf(p, v2, ALPHA_9);
    p = __builtin_fmaf(p, v2, ALPHA_7);
    p = __builtin_fmaf(p, v2, ALPHA_5);
    p = __builtin_fmaf(p, v2, ALPHA_3);
    p = __builtin_fmaf(p, v2, ALPHA_1);
    p = p * v;
    float q = __builtin_fmaf(v2, BETA_6, BETA_4);
    q = __builtin_fmaf(q, v2, BETA_2);
    q = __builtin_fmaf(q, v2, BETA_0);
    return p / q;
}

// Op::Tanh (session.rs:840-903).
__device__ __forceinline__ float tanh_elem(float x) { return rational_tanh(rclamp(x, -9.0f, 9.0f)); }

// Op::Gelu (fast_math.rs:304-323): 0.5x(1 + tanh(x(B + Cx^2))); the inner
// product is plain multiplies and an add, no fma.
__device__ __forceinline__ float gelu_elem(float i) {
    constexpr float B = 0.7978845608028654f;
    constexpr float C = 0.035677408136300125f;
    const float v = rclamp(i * (C * i * i + B), -9.0f, 9.0f);
    return (rational_tanh(v) + 1.0f) * (i * 0.5f);
}

// Op::Erf: fastapprox::faster::erf (crate fastapprox 0.3.1; call site
// crates/session_interpreter/src/session.rs:929).  pow2 writes
// 2^23 * (p + 126.94269504) into the float's bits with a saturating
// float-to-u32 conversion (NaN -> 0), as Rust's `as u32` does.
__device__ __forceinline__ uint32_t f32_as_u32_saturating(float f) {
    if (!(f > 0.0f)) return 0u;
    if (f >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)f;
}
__device__ __forceinline__ float erf_elem(float x) {
    constexpr float K = 3.3509633149424609f;
    float p = K * x;
    float clipp = p < -126.0f ? -126.0f : p;
    float pow2 = u2f(f32_as_u32_saturating(8388608.0f * (clipp + 126.94269504f)));
    float erfc = 2.0f / (1.0f + pow2);
    return 1.0f - erfc;
}

// Op::HardSigmoid (session.rs:810): fma then clamp.
__device__ __forceinline__ float hard_sigmoid_elem(float x, float alpha, float beta) {
    return rclamp(__builtin_fmaf(alpha, x, beta), 0.0f, 1.0f);
}

// Op::ReLU (session.rs:801): x.max(0.0); NaN -> 0.0.
__device__ __forceinline__ float relu_elem(float x) { return x > 0.0f ? x : 0.0f; }


// Op::LeakyReLU (session.rs:819): alpha * x below zero, x otherwise (NaN and -0.0 pass through).
__device__ __forceinline__ float leaky_relu_elem(float x, float alpha) { return x < 0.0f ? alpha * x : x; }

// Op::Clip: min(max(x, lo), hi) as ONNX defines it; the reference interpreter has no kernel
// (session.rs:201).  NaN stays NaN.
__device__ __forceinline__ float clip_elem(float x, float lo, float hi) { return x != x ? x : rclamp(x, lo, hi); }

}  // namespace dev
}  // namespace altius
