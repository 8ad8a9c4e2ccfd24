// A stand-alone code object: not linked into libaltius_hip.so but built with `hipcc --genco` and
// loaded at run time through ahip_module_load / ahip_launch.  It is the smallest example of the
// "compiled model" route the reference's ClangSession takes (crates/session_clang/src/builder.rs:44-76):
// kernels generated outside the library, bound by name.
#include <hip/hip_runtime.h>

#include <cstdint>

// out[i] = fma(alpha, in[i], beta) clamped to [0, 1]: HardSigmoid as the reference computes it
// (crates/session_interpreter/src/session.rs:805-812), one element per thread.
extern "C" __global__ void __launch_bounds__(256)
ahip_module_hard_sigmoid(float *__restrict__ out, const float *__restrict__ in, float alpha, float beta, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = __builtin_fmaf(alpha, in[i], beta);
    // NaN stays NaN: both comparisons are false for it.
    out[i] = v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v);
}

// out[r] = sum of the `len` floats of row r accumulated through dynamic shared memory: exercises
// the shared_bytes argument of ahip_launch.  One block per row; blockDim.x floats of shared memory.
extern "C" __global__ void ahip_module_row_sum(float *__restrict__ out, const float *__restrict__ in, uint32_t len) {
    extern __shared__ float partial[];
    const float *row = in + (uint64_t)blockIdx.x * len;
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < len; i += blockDim.x) acc += row[i];
    partial[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.0f;
        for (uint32_t t = 0; t < blockDim.x; t++) s += partial[t];
        out[blockIdx.x] = s;
    }
}
