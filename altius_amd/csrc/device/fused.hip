// A chain of element-wise operators in one pass over memory (Op::FusedElemwise,
// crates/core/src/op.rs:213-217; the reference emits it in
// crates/core/src/optimize/elemwise_fusion.rs and compiles it to one C loop in
// crates/session_clang/src/translator.rs:975-1143).
//
// The chain is data, not code: the host passes a short program (one step per
// operator) in the kernel arguments and every lane runs it on four consecutive
// output elements held in registers.  Step codes and operand selectors are the
// same for all lanes, so the dispatch is scalar branching and the vector unit
// only sees the arithmetic.  Every step applies the same per-element function
// as the stand-alone kernel of its operator (math.h, IEEE + - * /, sqrtf, powf),
// so the result equals the unfused chain bit for bit; what disappears is the
// round trip through memory between the steps.
//
// Two executors share the program format.  Chains that models actually contain (the exporter's
// erf-GELU, the tail of its LayerNorm, scale-and-shift, bias + activation or residual, x * sigmoid(x)) are also
// instantiated at compile time: the host compares the program with each instantiated signature and,
// on a match, launches straight-line code that runs at the speed of a copy.  Everything else goes to
// the interpreting kernel, whose per-step dispatch costs scalar-unit time.
//
// Operands are dense tensors broadcast to the output.  After the host has
// dropped size-1 axes and merged axes that every operand walks contiguously the
// output is at most [N, R, C] and each operand has one stride per axis (0 on
// broadcast axes): same shape (R*C, C, 1), one value (0, 0, 0), a row vector
// such as a bias (0, 0, 1), one value per row such as a mean (1, 0) and an
// attention mask [N, 1, C] (C, 0, 1) are all instances.

#include "common.h"
#include "ctx.h"
#include "math.h"

#include <math.h>

#include <utility>

namespace altius {
namespace {

using namespace dev;

constexpr int BLOCK = 256;
constexpr int MAX_IN = AHIP_FUSED_MAX_INPUTS;
constexpr int MAX_STEPS = AHIP_FUSED_MAX_STEPS;
constexpr uint32_t ACC = 0xFF;  // operand selector: the previous step's result

// Step codes: binary operators, then unary ones.
enum Code : uint32_t {
    C_ADD, C_SUB, C_MUL, C_DIV, C_POW, C_POW_SCALAR_EXP,
    C_SQRT, C_ERF, C_GELU, C_SIGMOID, C_HARDSIGMOID, C_RELU, C_TANH, C_LEAKYRELU, C_EXP, C_ROUND, C_CLIP, C_DIV_BY,
};

struct Step {
    uint32_t code, lhs, rhs;
    float alpha, beta;
};

struct Operand {
    const float *p;
    uint32_t s0, s1, s2;  // strides of the innermost, middle and outermost merged axis
    uint32_t vec;         // innermost stride 1 and everything 16-byte aligned: one float4 load (2: a dense operand, streamed)
};

struct Program {
    Operand in[MAX_IN];
    Step steps[MAX_STEPS];
    uint32_t n_in, n_steps;
    uint32_t n_vec;  // operands [0, n_vec) are read four elements at a time (vec4 kernel; 0 in the one-element kernel)
    uint32_t rank;   // merged rank: 1 (flat), 2 or 3
    FastDiv c, r;    // innermost and middle extents
    uint32_t total;  // output elements (< 2^32)
};

__device__ __forceinline__ float apply(uint32_t code, float a, float b, float alpha, float beta) {
    switch (code) {
    case C_ADD: return a + b;
    case C_SUB: return a - b;
    case C_MUL: return a * b;
    case C_DIV: return a / b;
    case C_POW: return powf(a, b);
    case C_POW_SCALAR_EXP: return b == 2.0f ? a * a : powf(a, b);
    case C_SQRT: return sqrtf(a);
    case C_ERF: return erf_elem(a);
    case C_GELU: return gelu_elem(a);
    case C_SIGMOID: return sigmoid_elem(a);
    case C_HARDSIGMOID: return hard_sigmoid_elem(a, alpha, beta);
    case C_RELU: return relu_elem(a);
    case C_TANH: return tanh_elem(a);
    case C_LEAKYRELU: return leaky_relu_elem(a, alpha);
    case C_EXP: return expf(a);
    case C_ROUND: return rintf(a);
    case C_CLIP: return clip_elem(a, alpha, beta);
    default: return a / alpha;  // C_DIV_BY
    }
}

// The lane's operands.  The host orders them: slots [0, n_vec) are read VEC elements at a time,
// slots [n_vec, n_in) hold one value for all VEC elements (a broadcast along the innermost axis).
template <int VEC> struct Regs {
    float vec[MAX_IN][VEC];
    float one[MAX_IN];
};

// The interpreter.  All operands and the running result live in one register file that is indexed
// with the step's (uniform) selectors: the compiler turns that into indexed register reads, two
// scalar instructions per value, where a branch per possible slot would cost a dozen.  The scalar
// unit issues at the rate of the vector unit on this part, so a step's cost is its scalar
// instructions as much as its arithmetic.
template <int VEC> __device__ __forceinline__ void run_steps(const Program &prog, const Regs<VEC> &in, float (&acc)[VEC]) {
    constexpr uint32_t ACC_SLOT = MAX_IN;
    float file[(MAX_IN + 1) * VEC];
#pragma unroll
    for (int k = 0; k < MAX_IN; k++) {
#pragma unroll
        for (int j = 0; j < VEC; j++)
            file[k * VEC + j] = k >= (int)prog.n_in ? 0.0f : k < (int)prog.n_vec ? in.vec[k][j] : in.one[k];
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) file[ACC_SLOT * VEC + j] = 0.0f;

    // The descriptor of step t+1 is fetched while step t computes (unused slots hold a harmless step).
    Step next = prog.steps[0];
    for (uint32_t t = 0; t < prog.n_steps; t++) {
        const Step st = next;
        next = prog.steps[t + 1 < MAX_STEPS ? t + 1 : t];
        const uint32_t la = (st.lhs < ACC_SLOT ? st.lhs : ACC_SLOT) * VEC, lb = (st.rhs < ACC_SLOT ? st.rhs : ACC_SLOT) * VEC;
        float a[VEC], b[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            a[j] = file[la + j];
            b[j] = file[lb + j];
        }
        // One dispatch per step, not per element: the switch is around the lane's elements.
        switch (st.code) {
#define ALTIUS_STEP(CODE)                                                                                                   \
    case CODE:                                                                                                              \
        _Pragma("unroll") for (int j = 0; j < VEC; j++) file[ACC_SLOT * VEC + j] = apply(CODE, a[j], b[j], st.alpha, st.beta); \
        break;
            ALTIUS_STEP(C_ADD)
            ALTIUS_STEP(C_SUB)
            ALTIUS_STEP(C_MUL)
            ALTIUS_STEP(C_DIV)
            ALTIUS_STEP(C_POW)
            ALTIUS_STEP(C_POW_SCALAR_EXP)
            ALTIUS_STEP(C_SQRT)
            ALTIUS_STEP(C_ERF)
            ALTIUS_STEP(C_GELU)
            ALTIUS_STEP(C_SIGMOID)
            ALTIUS_STEP(C_HARDSIGMOID)
            ALTIUS_STEP(C_RELU)
            ALTIUS_STEP(C_TANH)
            ALTIUS_STEP(C_LEAKYRELU)
            ALTIUS_STEP(C_EXP)
            ALTIUS_STEP(C_ROUND)
            ALTIUS_STEP(C_CLIP)
        default:
#pragma unroll
            for (int j = 0; j < VEC; j++) file[ACC_SLOT * VEC + j] = apply(C_DIV_BY, a[j], b[j], st.alpha, st.beta);
#undef ALTIUS_STEP
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[j] = file[ACC_SLOT * VEC + j];
}

// ---- chains fixed at compile time ----------------------------------------------------------------
// S<code, lhs, rhs>: one step; operands are slot numbers (after the host's reordering) or ACC.
template <uint32_t CODE, uint32_t LHS, uint32_t RHS = ACC> struct S {
    static constexpr uint32_t code = CODE, lhs = LHS, rhs = RHS;
};

template <uint32_t SEL, uint32_t NVEC, int VEC>
__device__ __forceinline__ float operand(const Regs<VEC> &in, const float (&acc)[VEC], int j) {
    if (SEL == ACC) return acc[j];
    return SEL < NVEC ? in.vec[SEL < MAX_IN ? SEL : 0][j] : in.one[SEL < MAX_IN ? SEL : 0];
}

// NVEC 16-byte operands in slots [0, NVEC), broadcast operands in [NVEC, NIN), then the steps.
template <uint32_t NVEC, uint32_t NIN, class... STEPS> struct Chain {
    static constexpr uint32_t n_vec = NVEC, n_in = NIN, n_steps = sizeof...(STEPS);

    static bool matches(const Program &p) {
        if (p.n_vec != NVEC || p.n_in != NIN || p.n_steps != n_steps) return false;
        const uint32_t code[] = {STEPS::code...}, lhs[] = {STEPS::lhs...}, rhs[] = {STEPS::rhs...};
        for (uint32_t t = 0; t < n_steps; t++)
            if (p.steps[t].code != code[t] || p.steps[t].lhs != lhs[t] || p.steps[t].rhs != rhs[t]) return false;
        return true;
    }

    template <class ST, int VEC>
    static __device__ __forceinline__ void step(const Step &st, const Regs<VEC> &in, float (&acc)[VEC]) {
        float r[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++)
            r[j] = apply(ST::code, operand<ST::lhs, NVEC, VEC>(in, acc, j), operand<ST::rhs, NVEC, VEC>(in, acc, j), st.alpha, st.beta);
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[j] = r[j];
    }

    template <int VEC> static __device__ __forceinline__ void run(const Program &prog, const Regs<VEC> &in, float (&acc)[VEC]) {
        uint32_t t = 0;
        (step<STEPS, VEC>(prog.steps[t++], in, acc), ...);
    }
};

// The interpreter, with the same interface.
struct AnyChain {
    template <int VEC> static __device__ __forceinline__ void run(const Program &prog, const Regs<VEC> &in, float (&acc)[VEC]) {
        run_steps<VEC>(prog, in, acc);
    }
};

// Commutative steps are stored with the previous result as left operand (the host normalises them).
// Div -> Erf -> Add 1 -> Mul x -> Mul 0.5 on (x | sqrt 2, 1, 0.5)
using ErfGeluChain = Chain<1, 4, S<C_DIV, 0, 1>, S<C_ERF, ACC>, S<C_ADD, ACC, 2>, S<C_MUL, ACC, 0>, S<C_MUL, ACC, 3>>;
// (var + eps) -> Sqrt -> d / . -> Mul gamma -> Add beta on (d, gamma, beta | var, eps)
using LayerNormTailChain = Chain<3, 5, S<C_ADD, 3, 4>, S<C_SQRT, ACC>, S<C_DIV, 0, ACC>, S<C_MUL, ACC, 1>, S<C_ADD, ACC, 2>>;
// d / std -> Mul gamma -> Add beta on (d, gamma, beta | std)
using NormaliseScaleShiftChain = Chain<3, 4, S<C_DIV, 0, 3>, S<C_MUL, ACC, 1>, S<C_ADD, ACC, 2>>;
// x * a + b with 16-byte operands: scale and shift, or a residual
using MulAddChain = Chain<3, 3, S<C_MUL, 0, 1>, S<C_ADD, ACC, 2>>;
// x + b -> Relu (bias or residual, then the activation)
using AddReluChain = Chain<2, 2, S<C_ADD, 0, 1>, S<C_RELU, ACC>>;
// x + b -> Gelu (a linear layer's bias, then the fused activation)
using AddGeluChain = Chain<2, 2, S<C_ADD, 0, 1>, S<C_GELU, ACC>>;
// x + b + r (bias, then the residual)
using AddAddChain = Chain<3, 3, S<C_ADD, 0, 1>, S<C_ADD, ACC, 2>>;
// x * Sigmoid(x)
using SiluChain = Chain<1, 1, S<C_SIGMOID, 0>, S<C_MUL, ACC, 0>>;
// x * HardSigmoid(x)  (hard swish)
using HardSwishChain = Chain<1, 1, S<C_HARDSIGMOID, 0>, S<C_MUL, ACC, 0>>;

// Four consecutive output elements per lane.  The host guarantees that the innermost extent is a
// multiple of 4 (the four elements share a row), that the operands in slots [0, n_vec) have innermost
// stride 1 and 16-byte aligned rows, and that the others have innermost stride 0.
template <class CHAIN, bool NT>
__global__ __launch_bounds__(BLOCK) void fused_elemwise_vec4(float *__restrict__ out, const Program prog) {
    const uint32_t i0 = (blockIdx.x * BLOCK + threadIdx.x) * 4u;
    if (i0 >= prog.total) return;
    uint32_t col = i0, row = 0, slab = 0;
    if (prog.rank > 1) {
        const uint32_t t = prog.c.div(i0);
        col = i0 - t * prog.c.d;
        row = t;
        if (prog.rank > 2) {
            slab = prog.r.div(t);
            row = t - slab * prog.r.d;
        }
    }
    // Every load is issued before any loaded value is looked at, so they are all in flight together.
    Regs<4> in;
#pragma unroll
    for (int k = 0; k < MAX_IN; k++) {
        if (k < (int)prog.n_vec) {
            const Operand &o = prog.in[k];
            const float *p = o.p + (size_t)slab * o.s2 + (size_t)row * o.s1 + col;
            // Only dense operands take the streaming hint; a broadcast row is re-read by every block.
            const float4 v = o.vec == 2 ? load4<NT>(p) : load4<false>(p);
            in.vec[k][0] = v.x;
            in.vec[k][1] = v.y;
            in.vec[k][2] = v.z;
            in.vec[k][3] = v.w;
        }
    }
#pragma unroll
    for (int k = 0; k < MAX_IN; k++) {
        if (k >= (int)prog.n_vec && k < (int)prog.n_in) {
            const Operand &o = prog.in[k];
            in.one[k] = o.p[(size_t)slab * o.s2 + (size_t)row * o.s1];
        }
    }
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    CHAIN::template run<4>(prog, in, acc);
    store4<NT>(out + i0, make_float4(acc[0], acc[1], acc[2], acc[3]));
}

// One element per lane: any innermost extent, any strides, any alignment.
__global__ __launch_bounds__(BLOCK) void fused_elemwise_scalar(float *__restrict__ out, const Program prog) {
    const uint32_t i = blockIdx.x * BLOCK + threadIdx.x;
    if (i >= prog.total) return;
    uint32_t col = i, row = 0, slab = 0;
    if (prog.rank > 1) {
        const uint32_t t = prog.c.div(i);
        col = i - t * prog.c.d;
        row = t;
        if (prog.rank > 2) {
            slab = prog.r.div(t);
            row = t - slab * prog.r.d;
        }
    }
    Regs<1> in;
#pragma unroll
    for (int k = 0; k < MAX_IN; k++) {
        if (k < (int)prog.n_in) {
            const Operand &o = prog.in[k];
            in.one[k] = o.p[(size_t)slab * o.s2 + (size_t)row * o.s1 + (size_t)col * o.s0];
        }
    }
    float acc[1] = {0.0f};
    run_steps<1>(prog, in, acc);
    out[i] = acc[0];
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class CHAIN> void launch_vec4(hipStream_t s, dim3 grid, bool nt, float *out, const Program &prog) {
    if (nt) hipLaunchKernelGGL((fused_elemwise_vec4<CHAIN, true>), grid, dim3(BLOCK), 0, s, out, prog);
    else hipLaunchKernelGGL((fused_elemwise_vec4<CHAIN, false>), grid, dim3(BLOCK), 0, s, out, prog);
}

template <class CHAIN> bool try_static(hipStream_t s, dim3 grid, bool nt, float *out, const Program &prog) {
    if (!CHAIN::matches(prog)) return false;
    launch_vec4<CHAIN>(s, grid, nt, out, prog);
    return true;
}

}  // namespace

int launch_fused_elemwise(DeviceCtx &ctx, float *out, int rank, const int64_t *out_dims, int n_inputs, const float *const *inputs,
                          const int64_t *const *input_strides, int n_steps, const ahip_fused_step *steps) {
    if (rank < 0 || rank > MAX_RANK) return ctx.fail(AHIP_ERR_ARG, "fused: rank out of range");
    if (n_inputs < 1 || n_inputs > MAX_IN) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: between 1 and 6 operands are supported");
    if (n_steps < 1 || n_steps > MAX_STEPS) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: between 1 and 16 steps are supported");
    if ((rank > 0 && !out_dims) || !inputs || !input_strides || !steps) return ctx.fail(AHIP_ERR_ARG, "fused: null argument");
    size_t total = 1;
    for (int i = 0; i < rank; i++) {
        if (out_dims[i] < 0) return ctx.fail(AHIP_ERR_ARG, "fused: negative dimension");
        total *= (size_t)out_dims[i];
    }
    for (int k = 0; k < n_inputs; k++) {
        if (rank > 0 && !input_strides[k]) return ctx.fail(AHIP_ERR_ARG, "fused: null strides");
        for (int i = 0; i < rank; i++)
            if (input_strides[k][i] < 0) return ctx.fail(AHIP_ERR_ARG, "fused: negative stride");
    }

    Program prog;
    for (int t = 0; t < n_steps; t++) {
        const ahip_fused_step &s = steps[t];
        Step &d = prog.steps[t];
        auto sel = [&](int v, uint32_t *o) {
            if (v == AHIP_FUSED_ACC) {
                if (t == 0) return false;  // nothing has been computed yet
                *o = ACC;
                return true;
            }
            if (v < 0 || v >= n_inputs) return false;
            *o = (uint32_t)v;
            return true;
        };
        d.alpha = s.alpha;
        d.beta = s.beta;
        d.rhs = ACC;
        if (!sel(s.lhs, &d.lhs)) return ctx.fail(AHIP_ERR_ARG, "fused: bad operand selector");
        if (s.is_unary) {
            static const Code unary[] = {C_SQRT, C_ERF, C_GELU, C_SIGMOID, C_HARDSIGMOID, C_RELU, C_TANH,
                                         C_LEAKYRELU, C_EXP, C_ROUND, C_CLIP, C_DIV_BY};
            if (s.op < AHIP_SQRT || s.op > AHIP_DIV_BY) return ctx.fail(AHIP_ERR_ARG, "fused: unknown unary op");
            d.code = unary[s.op];
        } else {
            if (s.op < AHIP_ADD || s.op > AHIP_POW) return ctx.fail(AHIP_ERR_ARG, "fused: unknown binary op");
            if (!sel(s.rhs, &d.rhs)) return ctx.fail(AHIP_ERR_ARG, "fused: bad operand selector");
            d.code = s.op == AHIP_POW && s.pow_scalar_exponent ? (uint32_t)C_POW_SCALAR_EXP : (uint32_t)(C_ADD + s.op);
        }
    }
    for (int t = n_steps; t < MAX_STEPS; t++) prog.steps[t] = Step{C_ADD, ACC, ACC, 0.0f, 0.0f};
    // a + b and a * b have the bits of b + a and b * a: keep the previous result on the left.
    for (int t = 0; t < n_steps; t++) {
        Step &d = prog.steps[t];
        if ((d.code == C_ADD || d.code == C_MUL) && d.rhs == ACC && d.lhs != ACC) std::swap(d.lhs, d.rhs);
    }
    if (total == 0) return AHIP_OK;
    if (!out) return ctx.fail(AHIP_ERR_ARG, "fused: null output pointer");
    for (int k = 0; k < n_inputs; k++)
        if (!inputs[k]) return ctx.fail(AHIP_ERR_ARG, "fused: null operand pointer");
    if (total >= ((size_t)1 << 32) - 4 * BLOCK) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: 2^32 or more elements");

    // Drop size-1 axes; merge neighbours that every operand walks as one contiguous (or one broadcast) axis.
    int64_t dims[MAX_RANK], st[MAX_IN][MAX_RANK];
    int r = 0;
    for (int i = 0; i < rank; i++) {
        if (out_dims[i] == 1) continue;
        bool merge = r > 0;
        for (int k = 0; k < n_inputs && merge; k++) merge = st[k][r - 1] == input_strides[k][i] * out_dims[i];
        if (merge) {
            dims[r - 1] *= out_dims[i];
            for (int k = 0; k < n_inputs; k++) st[k][r - 1] = input_strides[k][i];
        } else {
            dims[r] = out_dims[i];
            for (int k = 0; k < n_inputs; k++) st[k][r] = input_strides[k][i];
            r++;
        }
    }
    if (r == 0) {
        dims[0] = 1;
        for (int k = 0; k < n_inputs; k++) st[k][0] = 0;
        r = 1;
    }
    if (r > 3) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: operands need more than three merged axes");
    for (int k = 0; k < n_inputs; k++)
        for (int i = 0; i < r; i++)
            if ((uint64_t)st[k][i] >= ((uint64_t)1 << 32)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: operand stride exceeds 2^32 elements");

    prog.n_in = (uint32_t)n_inputs;
    prog.n_steps = (uint32_t)n_steps;
    prog.rank = (uint32_t)r;
    prog.total = (uint32_t)total;
    prog.c = make_fastdiv((uint32_t)dims[r - 1]);
    prog.r = make_fastdiv(r >= 2 ? (uint32_t)dims[r - 2] : 1u);
    // FastDiv is exact for indices below 2^31.
    if (r > 1 && total >= ((size_t)1 << 31)) return ctx.fail(AHIP_ERR_UNSUPPORTED, "fused: broadcast operands with 2^31 or more elements");
    // Four elements per lane need rows that are multiples of four long (a flat problem: a length that is;
    // otherwise the one-element kernel reads the operands once all the same, and such tensors are small
    // in practice), and operands that are either 16-byte loadable or constant along the innermost axis.
    bool vec = aligned16(out) && (r == 1 ? total % 4 == 0 : dims[r - 1] % 4 == 0);
    Operand ops[MAX_IN];
    for (int k = 0; k < n_inputs; k++) {
        Operand &o = ops[k];
        o.p = inputs[k];
        o.s0 = (uint32_t)st[k][r - 1];
        o.s1 = r >= 2 ? (uint32_t)st[k][r - 2] : 0u;
        o.s2 = r >= 3 ? (uint32_t)st[k][r - 3] : 0u;
        o.vec = o.s0 == 1 && aligned16(o.p) && o.s1 % 4 == 0 && o.s2 % 4 == 0;
        const bool dense = o.s0 == 1 && (r < 2 || (int64_t)o.s1 == dims[r - 1]) && (r < 3 || (int64_t)o.s2 == dims[r - 1] * dims[r - 2]);
        if (o.vec && dense) o.vec = 2;
        if (o.s0 != 0 && !o.vec) vec = false;
    }
    // Slot order of the vec4 kernel: 16-byte operands first, then the broadcast ones.
    int slot_of[MAX_IN];
    int n_vec = 0;
    if (vec) {
        int next = 0;
        for (int k = 0; k < n_inputs; k++)
            if (ops[k].vec) slot_of[k] = next++;
        n_vec = next;
        for (int k = 0; k < n_inputs; k++)
            if (!ops[k].vec) slot_of[k] = next++;
    } else {
        for (int k = 0; k < n_inputs; k++) slot_of[k] = k;
    }
    for (int k = 0; k < MAX_IN; k++) prog.in[k] = Operand{nullptr, 0, 0, 0, 0};
    for (int k = 0; k < n_inputs; k++) prog.in[slot_of[k]] = ops[k];
    for (int t = 0; t < n_steps; t++) {
        if (prog.steps[t].lhs != ACC) prog.steps[t].lhs = (uint32_t)slot_of[prog.steps[t].lhs];
        if (prog.steps[t].rhs != ACC) prog.steps[t].rhs = (uint32_t)slot_of[prog.steps[t].rhs];
    }
    prog.n_vec = (uint32_t)n_vec;

    const bool nt = ctx.streaming(total * sizeof(float));
    if (vec) {
        const dim3 grid((unsigned)((total / 4 + BLOCK - 1) / BLOCK));
        hipStream_t s = ctx.stream;
        const bool fixed = ctx.fused_static_chains &&
                           (try_static<ErfGeluChain>(s, grid, nt, out, prog) || try_static<LayerNormTailChain>(s, grid, nt, out, prog) ||
                            try_static<NormaliseScaleShiftChain>(s, grid, nt, out, prog) || try_static<MulAddChain>(s, grid, nt, out, prog) ||
                            try_static<AddReluChain>(s, grid, nt, out, prog) || try_static<AddGeluChain>(s, grid, nt, out, prog) ||
                            try_static<AddAddChain>(s, grid, nt, out, prog) || try_static<SiluChain>(s, grid, nt, out, prog) ||
                            try_static<HardSwishChain>(s, grid, nt, out, prog));
        if (!fixed) launch_vec4<AnyChain>(s, grid, nt, out, prog);
    } else {
        const dim3 grid((unsigned)((total + BLOCK - 1) / BLOCK));
        hipLaunchKernelGGL(fused_elemwise_scalar, grid, dim3(BLOCK), 0, ctx.stream, out, prog);
    }
    return ctx.check(hipGetLastError(), "fused launch");
}

}  // namespace altius
