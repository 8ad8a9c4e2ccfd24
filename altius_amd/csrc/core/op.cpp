// Operator attributes by ONNX name, and the ONNX op_type <-> OpKind table with the defaults
// the reference's loader applies (crates/core/src/onnx/load.rs:171-361).
#include "op.h"

namespace altius {

namespace {

bool is(OpKind k, std::initializer_list<OpKind> ks) {
    for (OpKind x : ks)
        if (x == k) return true;
    return false;
}

}  // namespace

bool Op::set_int(const std::string &n, int64_t v) {
    if (n == "axis" && is(kind, {OpKind::Softmax, OpKind::LayerNormalization, OpKind::Concat, OpKind::Flatten,
                                 OpKind::Gather, OpKind::Split})) {
        axis = v;
    } else if (n == "keepdims" && is(kind, {OpKind::ReduceMin, OpKind::ReduceMax, OpKind::ReduceMean})) {
        keep_dims = v != 0;
    } else if (n == "stash_type" && kind == OpKind::LayerNormalization) {
        stash_type = v;
    } else if (n == "to" && kind == OpKind::Cast) {
        // ONNX TensorProto.DataType numbering: FLOAT 1, INT32 6, INT64 7, BOOL 9 (load.rs:426-440).
        switch (v) {
        case 1: to = TensorElemType::F32; break;
        case 6: to = TensorElemType::I32; break;
        case 7: to = TensorElemType::I64; break;
        case 9: to = TensorElemType::Bool; break;
        default: return false;
        }
    } else if (n == "group" && kind == OpKind::Conv2d) {
        group = v;
    } else if (n == "transA" && kind == OpKind::Gemm) {
        trans_a = v == 1;
    } else if (n == "transB" && kind == OpKind::Gemm) {
        trans_b = v == 1;
    } else if (n == "training_mode" && kind == OpKind::BatchNormalization) {
        training_mode = v != 0;
    } else if (n == "start" && kind == OpKind::Shape) {
        start = v;
    } else if (n == "end" && kind == OpKind::Shape) {
        end = v;
    } else if (n == "exclude_outside" && kind == OpKind::Resize) {
        exclude_outside = v;
    } else {
        return false;
    }
    return true;
}

bool Op::get_int(const std::string &n, int64_t *v) const {
    if (kind == OpKind::Softmax && n == "prologue_scale") {
        *v = prologue_scale;
        return true;
    }
    if (kind == OpKind::Softmax && n == "prologue_mask") {
        *v = prologue_mask ? 1 : 0;
        return true;
    }
    if (kind == OpKind::MatMul && (n == "transA" || n == "transB")) {  // set by fuse_transpose_matmul
        *v = (n == "transA" ? trans_a : trans_b) ? 1 : 0;
        return true;
    }
    if (n == "axis" && is(kind, {OpKind::Softmax, OpKind::LayerNormalization, OpKind::Concat, OpKind::Flatten,
                                 OpKind::Gather, OpKind::Split})) {
        *v = axis;
    } else if (n == "keepdims" && is(kind, {OpKind::ReduceMin, OpKind::ReduceMax, OpKind::ReduceMean})) {
        *v = keep_dims ? 1 : 0;
    } else if (n == "stash_type" && kind == OpKind::LayerNormalization) {
        *v = stash_type;
    } else if (n == "to" && kind == OpKind::Cast) {
        switch (to) {
        case TensorElemType::F32: *v = 1; break;
        case TensorElemType::I32: *v = 6; break;
        case TensorElemType::I64: *v = 7; break;
        case TensorElemType::Bool: *v = 9; break;
        }
    } else if (n == "group" && kind == OpKind::Conv2d) {
        *v = group;
    } else if (n == "transA" && kind == OpKind::Gemm) {
        *v = trans_a ? 1 : 0;
    } else if (n == "transB" && kind == OpKind::Gemm) {
        *v = trans_b ? 1 : 0;
    } else if (n == "training_mode" && kind == OpKind::BatchNormalization) {
        *v = training_mode ? 1 : 0;
    } else if (n == "start" && kind == OpKind::Shape) {
        *v = start;
    } else if (n == "end" && kind == OpKind::Shape && end) {
        *v = *end;
    } else if (n == "exclude_outside" && kind == OpKind::Resize) {
        *v = exclude_outside;
    } else {
        return false;
    }
    return true;
}

bool Op::set_float(const std::string &n, float v) {
    if (n == "alpha" && is(kind, {OpKind::HardSigmoid, OpKind::LeakyReLU, OpKind::Gemm})) {
        alpha = v;
    } else if (n == "beta" && is(kind, {OpKind::HardSigmoid, OpKind::Gemm})) {
        beta = v;
    } else if (n == "epsilon" && is(kind, {OpKind::LayerNormalization, OpKind::BatchNormalization})) {
        epsilon = v;
    } else if (n == "momentum" && kind == OpKind::BatchNormalization) {
        momentum = v;
    } else if (n == "cubic_coeff_a" && kind == OpKind::Resize) {
        cubic_coeff_a = v;
    } else if (n == "extrapolation_value" && kind == OpKind::Resize) {
        extrapolation_value = v;
    } else {
        return false;
    }
    return true;
}

bool Op::get_float(const std::string &n, float *v) const {
    if (n == "alpha" && is(kind, {OpKind::HardSigmoid, OpKind::LeakyReLU, OpKind::Gemm})) {
        *v = alpha;
    } else if (n == "beta" && is(kind, {OpKind::HardSigmoid, OpKind::Gemm})) {
        *v = beta;
    } else if (n == "epsilon" && is(kind, {OpKind::LayerNormalization, OpKind::BatchNormalization})) {
        *v = epsilon;
    } else if (n == "momentum" && kind == OpKind::BatchNormalization) {
        *v = momentum;
    } else if (n == "cubic_coeff_a" && kind == OpKind::Resize) {
        *v = cubic_coeff_a;
    } else if (n == "extrapolation_value" && kind == OpKind::Resize) {
        *v = extrapolation_value;
    } else {
        return false;
    }
    return true;
}

bool Op::set_ints(const std::string &n, const std::vector<int64_t> &v) {
    if (n == "axes" && is(kind, {OpKind::ReduceMin, OpKind::ReduceMax, OpKind::ReduceMean, OpKind::Squeeze,
                                 OpKind::Unsqueeze})) {
        axes = v;
    } else if (n == "perm" && kind == OpKind::Transpose) {
        perm = v;
    } else if (n == "split" && kind == OpKind::Split) {
        split = v;
    } else if (n == "kernel_shape" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        kernel_shape = v;
    } else if (n == "strides" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        strides = v;
    } else if (n == "pads" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        padding = v;
    } else if (n == "dilations" && kind == OpKind::Conv2d) {
        dilations = v;
    } else {
        return false;
    }
    return true;
}

bool Op::get_ints(const std::string &n, std::vector<int64_t> *v) const {
    if (n == "axes" && is(kind, {OpKind::ReduceMin, OpKind::ReduceMax, OpKind::ReduceMean, OpKind::Squeeze,
                                 OpKind::Unsqueeze})) {
        *v = axes;
    } else if (n == "perm" && kind == OpKind::Transpose) {
        *v = perm;
    } else if (n == "split" && kind == OpKind::Split) {
        *v = split;
    } else if (n == "kernel_shape" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        *v = kernel_shape;
    } else if (n == "strides" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        *v = strides;
    } else if (n == "pads" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        *v = padding;
    } else if (n == "dilations" && kind == OpKind::Conv2d) {
        *v = dilations;
    } else {
        return false;
    }
    return true;
}

bool Op::set_string(const std::string &n, const std::string &v) {
    if (n == "auto_pad" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        auto_pad = v;
    } else if (n == "coordinate_transformation_mode" && kind == OpKind::Resize) {
        coordinate_transformation_mode = v;
    } else if (n == "mode" && kind == OpKind::Resize) {
        mode = v;
    } else if (n == "nearest_mode" && kind == OpKind::Resize) {
        nearest_mode = v;
    } else {
        return false;
    }
    return true;
}

bool Op::get_string(const std::string &n, std::string *v) const {
    if (n == "auto_pad" && is(kind, {OpKind::Conv2d, OpKind::MaxPool})) {
        *v = auto_pad;
    } else if (n == "coordinate_transformation_mode" && kind == OpKind::Resize) {
        *v = coordinate_transformation_mode;
    } else if (n == "mode" && kind == OpKind::Resize) {
        *v = mode;
    } else if (n == "nearest_mode" && kind == OpKind::Resize) {
        *v = nearest_mode;
    } else if (n == "chain" && kind == OpKind::FusedElemwise && fused) {
        // Not an ONNX attribute: the fused operators' names in order, comma-separated, for inspection.
        v->clear();
        for (const auto &step : fused->chain) *v += (v->empty() ? "" : ",") + std::string(step.op.name());
    } else {
        return false;
    }
    return true;
}

namespace {

struct OnnxName {
    const char *type;
    OpKind kind;
};

// load.rs:171-361, in the order of its match arms.
const OnnxName kOnnxNames[] = {
    {"Identity", OpKind::Identity}, {"Add", OpKind::Add}, {"Sub", OpKind::Sub}, {"Mul", OpKind::Mul},
    {"Div", OpKind::Div}, {"Greater", OpKind::Greater}, {"Pow", OpKind::Pow}, {"Sqrt", OpKind::Sqrt},
    {"Relu", OpKind::ReLU}, {"Sigmoid", OpKind::Sigmoid}, {"Erf", OpKind::Erf}, {"Tanh", OpKind::Tanh},
    {"Where", OpKind::Where}, {"Softmax", OpKind::Softmax}, {"Round", OpKind::Round}, {"Exp", OpKind::Exp},
    {"Expand", OpKind::Expand}, {"Range", OpKind::Range}, {"Tile", OpKind::Tile}, {"Split", OpKind::Split},
    {"Slice", OpKind::Slice}, {"Gather", OpKind::Gather}, {"NonMaxSuppression", OpKind::NonMaxSuppression},
    {"Reshape", OpKind::Reshape}, {"MatMul", OpKind::MatMul}, {"GlobalAveragePool", OpKind::GlobalAveragePool},
    {"Conv", OpKind::Conv2d}, {"LeakyRelu", OpKind::LeakyReLU}, {"Resize", OpKind::Resize},
    {"Concat", OpKind::Concat}, {"Transpose", OpKind::Transpose}, {"Squeeze", OpKind::Squeeze},
    {"Unsqueeze", OpKind::Unsqueeze}, {"ReduceMin", OpKind::ReduceMin}, {"ReduceMax", OpKind::ReduceMax},
    {"ReduceMean", OpKind::ReduceMean}, {"Loop", OpKind::Loop}, {"Cast", OpKind::Cast}, {"MaxPool", OpKind::MaxPool},
    {"HardSigmoid", OpKind::HardSigmoid}, {"Flatten", OpKind::Flatten}, {"Gemm", OpKind::Gemm},
    {"BatchNormalization", OpKind::BatchNormalization}, {"LayerNormalization", OpKind::LayerNormalization},
    {"Clip", OpKind::Clip}, {"Shape", OpKind::Shape}, {"Constant", OpKind::Constant},
};

}  // namespace

const char *onnx_type_of(OpKind k) {
    for (const auto &e : kOnnxNames)
        if (e.kind == k) return e.type;
    return nullptr;
}

bool op_from_onnx_type(const std::string &op_type, int64_t opset_version, Op *op) {
    (void)opset_version;
    for (const auto &e : kOnnxNames) {
        if (op_type != e.type) continue;
        Op o(e.kind);
        switch (e.kind) {
        case OpKind::Softmax: o.axis = -1; break;                          // load.rs:185-187
        case OpKind::Split: o.axis = 0; break;                             // load.rs:193-197
        case OpKind::Gather: o.axis = 0; break;                            // load.rs:199-201
        case OpKind::Flatten: o.axis = 1; break;                           // load.rs:325-327
        case OpKind::LayerNormalization:                                   // load.rs:340-344
            o.axis = -1;
            o.stash_type = 1;
            o.epsilon = 1e-5f;
            break;
        case OpKind::Conv2d:                                               // load.rs:206-230
            o.auto_pad = "NOTSET";
            o.strides = {1, 1};
            o.padding = {0, 0};
            o.dilations = {1, 1};
            o.group = 1;
            break;
        case OpKind::MaxPool:                                              // load.rs:302-320
            o.auto_pad = "NOTSET";
            o.padding = {0, 0};
            break;
        case OpKind::LeakyReLU: o.alpha = 0.01f; break;                    // load.rs:231-233
        case OpKind::HardSigmoid:                                          // load.rs:321-324
            o.alpha = 0.2f;
            o.beta = 0.5f;
            break;
        case OpKind::Gemm:                                                 // load.rs:328-333
            o.alpha = 1.0f;
            o.beta = 1.0f;
            break;
        case OpKind::BatchNormalization:                                   // load.rs:334-339
            o.epsilon = 1e-5f;
            o.momentum = 1e-5f;
            break;
        case OpKind::Resize:                                               // load.rs:234-262
            o.coordinate_transformation_mode = "half_pixel";
            o.cubic_coeff_a = -0.75f;
            o.mode = "nearest";
            o.nearest_mode = "round_prefer_floor";
            break;
        case OpKind::ReduceMin:
        case OpKind::ReduceMax:
        case OpKind::ReduceMean: o.keep_dims = true; break;                // load.rs:277-288
        default: break;
        }
        *op = std::move(o);
        return true;
    }
    return false;
}

std::vector<std::string> required_onnx_attributes(const Op &op, int64_t opset_version) {
    switch (op.kind) {
    case OpKind::Conv2d: return {"kernel_shape"};                          // load.rs:211-213
    case OpKind::Concat: return {"axis"};                                  // load.rs:263-265
    case OpKind::Transpose: return {"perm"};                               // load.rs:266-268
    case OpKind::Squeeze:                                                  // load.rs:269-272
        if (opset_version < 12) return {"axes"};
        return {};
    case OpKind::ReduceMin: return {"axes"};                               // load.rs:277-280
    case OpKind::ReduceMean: return {"axes"};                              // load.rs:285-288
    case OpKind::Cast: return {"to"};                                      // load.rs:295-301
    case OpKind::MaxPool: return {"kernel_shape", "strides"};              // load.rs:309-313
    case OpKind::Loop: return {"body"};                                    // load.rs:289-294
    default: return {};
    }
}

}  // namespace altius
