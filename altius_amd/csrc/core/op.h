// Operator kinds and attributes of the graph IR.
// Mirrors altius_core::op::Op (crates/core/src/op.rs:7-57): the same 49 kinds in the
// same order, so a graph built for the interpreter names the same operators here.
// Every attribute the reference's loader reads is kept (op.rs:59-218), under one struct.
#pragma once

#include <stdint.h>

#include <memory>
#include <optional>
#include <string>
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

struct FusedElemwise;

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
    // Conv2d / MaxPool (op.rs:59-83)
    std::string auto_pad;
    std::vector<int64_t> dilations, kernel_shape, strides, padding;
    int64_t group = 1;
    // Transpose.perm, Split.split (op.rs:127-130, 165-168)
    std::vector<int64_t> perm, split;
    // Gemm (op.rs:183-188); alpha / beta above
    bool trans_a = false, trans_b = false;
    // BatchNormalization (op.rs:190-195); epsilon above
    float momentum = 1e-5f;
    bool training_mode = false;
    // Shape (op.rs:177-181)
    int64_t start = 0;
    std::optional<int64_t> end;
    // Resize (op.rs:113-121)
    std::string coordinate_transformation_mode, mode, nearest_mode;
    float cubic_coeff_a = -0.75f, extrapolation_value = 0.0f;
    int64_t exclude_outside = 0;
    // Constant.value (op.rs:206-210)
    std::shared_ptr<Tensor> value;
    // FusedElemwise (op.rs:213-217)
    std::shared_ptr<const FusedElemwise> fused;
    // Not in the reference: a Softmax that absorbed the Mul / Div by one value and the mask Add in front
    // of it (fuse_softmax_prologue).  Its inputs are then x, the scale value if prologue_scale != 0
    // (1: x * scale, 2: x / scale), and the mask if prologue_mask.
    int prologue_scale = 0;
    bool prologue_mask = false;

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
    // Op::is_elemwise (op.rs:387-412): the operators fuse_elemwise_ops chains together.
    bool is_elemwise() const {
        switch (kind) {
        case OpKind::Add: case OpKind::Sub: case OpKind::Mul: case OpKind::Div: case OpKind::Pow: case OpKind::Greater:
        case OpKind::Sqrt: case OpKind::ReLU: case OpKind::LeakyReLU: case OpKind::HardSigmoid:
            return true;
        default:
            return false;
        }
    }

    // Attribute access by ONNX attribute name ("axis", "perm", "kernel_shape", "transB", ...): the
    // one vocabulary shared by the ONNX loader and the C ABI.  Setters return false for a name
    // this operator kind does not carry.
    bool set_int(const std::string &name, int64_t v);
    bool set_float(const std::string &name, float v);
    bool set_ints(const std::string &name, const std::vector<int64_t> &v);
    bool set_string(const std::string &name, const std::string &v);
    bool get_int(const std::string &name, int64_t *v) const;
    bool get_float(const std::string &name, float *v) const;
    bool get_ints(const std::string &name, std::vector<int64_t> *v) const;
    bool get_string(const std::string &name, std::string *v) const;
};

// The payload of Op::FusedElemwise (op.rs:213-217): the value ids the fused node reads, in the order
// of its inputs, and the operators it stands for with the value ids they were wired with.  Every
// step but the first reads the output of the step before it.
struct FusedElemwise {
    struct Step {
        Op op;
        std::vector<size_t> inputs, outputs;  // ValueIds
    };
    std::vector<size_t> input_map;
    std::vector<Step> chain;
};

// The operator a freshly loaded ONNX node of this type starts from: kind plus the defaults the
// reference's loader applies for absent attributes (crates/core/src/onnx/load.rs:171-361).
// Returns false for an op_type the reference does not know.
bool op_from_onnx_type(const std::string &op_type, int64_t opset_version, Op *op);
// Attributes the reference's loader insists on (`get_attribute(..)?`): missing ones are an error.
std::vector<std::string> required_onnx_attributes(const Op &op, int64_t opset_version);
// ONNX op_type string of a kind ("Relu" for ReLU, "Conv" for Conv2d, ...); nullptr for kinds
// that have no ONNX spelling (Gelu, FusedElemwise).
const char *onnx_type_of(OpKind k);

}  // namespace altius
