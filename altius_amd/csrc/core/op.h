// Operator kinds and attributes of the graph IR.
// Mirrors altius_core::op::Op (crates/core/src/op.rs:7-57): the same 49 kinds in the
// same order, so a graph built for the interpreter names the same operators here.
// Attributes are kept for the operators this backend executes.
#pragma once

#include <stdint.h>

#include <vector>

#include "tensor.h"

namespace altius {

enum class OpKind : int {
    Identity = 0, Conv2d, Add, Sub, Mul, Div, Pow, Greater, Sqrt, ReLU, Gelu, LeakyReLU, Sigmoid, Erf, Tanh,
    Clip, Where, Softmax, Cast, MaxPool, GlobalAveragePool, Reshape, Flatten, Resize, Concat, Transpose,
    Squeeze, Unsqueeze, ReduceMin, ReduceMax, ReduceMean, Round, Exp, Expand, Range, Loop, Tile, Split,
    Slice, Gather, Shape, NonMaxSuppression, MatMul, Gemm, BatchNormalization, LayerNormalization,
    HardSigmoid, Constant, FusedElemwise,
    Count
};

const char *op_kind_name(OpKind k);

struct Op {
    OpKind kind = OpKind::Identity;

    // Softmax.axis, LayerNormalization.axis (op.rs:96-99, 195-200)
    int64_t axis = -1;
    // ReduceMax / ReduceMean / ReduceMin (op.rs:143-162)
    std::vector<int64_t> axes;
    bool keep_dims = true;
    // HardSigmoid.alpha/beta (op.rs:84-88), LeakyReLU.alpha
    float alpha = 0.2f;
    float beta = 0.5f;
    // LayerNormalization (op.rs:195-200)
    float epsilon = 1e-5f;
    int64_t stash_type = 1;
    // Cast.to
    TensorElemType to = TensorElemType::F32;

    Op() = default;
    explicit Op(OpKind k) : kind(k) {}

    static Op softmax(int64_t axis) {
        Op o(OpKind::Softmax);
        o.axis = axis;
        return o;
    }
    static Op hard_sigmoid(float alpha, float beta) {
        Op o(OpKind::HardSigmoid);
        o.alpha = alpha;
        o.beta = beta;
        return o;
    }
    static Op reduce_mean(std::vector<int64_t> axes, bool keep_dims) {
        Op o(OpKind::ReduceMean);
        o.axes = std::move(axes);
        o.keep_dims = keep_dims;
        return o;
    }
    static Op reduce_max(std::vector<int64_t> axes, bool keep_dims) {
        Op o(OpKind::ReduceMax);
        o.axes = std::move(axes);
        o.keep_dims = keep_dims;
        return o;
    }
    static Op layer_normalization(int64_t axis, float epsilon, int64_t stash_type) {
        Op o(OpKind::LayerNormalization);
        o.axis = axis;
        o.epsilon = epsilon;
        o.stash_type = stash_type;
        return o;
    }

    const char *name() const { return op_kind_name(kind); }
};

}  // namespace altius
