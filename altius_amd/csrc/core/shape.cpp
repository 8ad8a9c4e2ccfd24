#include "shape.h"

#include <algorithm>

namespace altius {

namespace {

bool fail(ShapeError *err, std::string msg) {
    if (err) err->message = std::move(msg);
    return false;
}

// Normalises negative axes; rejects axes outside the rank.
bool normalise_axes(const Op &op, size_t rank, std::vector<size_t> *out, ShapeError *err) {
    for (int64_t a : op.axes) {
        const int64_t n = a < 0 ? a + (int64_t)rank : a;
        if (n < 0 || n >= (int64_t)rank)
            return fail(err, std::string(op.name()) + ": axis " + std::to_string(a) + " out of range for rank " +
                                 std::to_string(rank));
        out->push_back((size_t)n);
    }
    return true;
}

FixedDimensions reduced_dims(const FixedDimensions &in, const std::vector<size_t> &axes, bool keep_dims) {
    std::vector<FixedDimension> d;
    for (size_t i = 0; i < in.len(); i++) {
        const bool reduced = std::find(axes.begin(), axes.end(), i) != axes.end();
        if (!reduced)
            d.push_back(in[i]);
        else if (keep_dims)
            d.push_back(1);
    }
    if (d.empty()) d.push_back(1);  // a full reduction without keepdims yields [1]
    return FixedDimensions(std::move(d));
}

}  // namespace

bool compute_output_shapes(const Model &model, Op &op, const std::vector<const Tensor *> &inputs,
                           size_t num_outputs, std::vector<TypedFixedShape> *out, ShapeError *err) {
    out->clear();
    auto need_inputs = [&](size_t n) {
        if (inputs.size() >= n) return true;
        return fail(err, std::string(op.name()) + ": expected " + std::to_string(n) + " inputs");
    };
    switch (op.kind) {
    case OpKind::Add:
    case OpKind::Sub:
    case OpKind::Mul:
    case OpKind::Div:
    case OpKind::Pow: {
        if (!need_inputs(2)) return false;
        auto shape = inputs[0]->dims().broadcast(inputs[1]->dims());
        if (!shape)
            return fail(err, std::string(op.name()) + ": cannot broadcast " + inputs[0]->dims().to_string() +
                                 " with " + inputs[1]->dims().to_string());
        out->push_back({*shape, inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::ReduceMax: {
        if (!need_inputs(1)) return false;
        if (model.opset_version > 13)
            return fail(err, "ReduceMax: opset " + std::to_string(model.opset_version) +
                                 " passes axes as an input; only opset <= 13 is supported");
        const FixedDimensions &in = inputs[0]->dims();
        std::vector<size_t> axes;
        if (op.axes.empty()) {
            for (size_t i = 0; i < in.len(); i++) axes.push_back(i);
        } else if (!normalise_axes(op, in.len(), &axes, err)) {
            return false;
        }
        out->push_back({reduced_dims(in, axes, op.keep_dims), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::ReduceMean: {
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        std::vector<size_t> axes;  // no axes attribute: nothing is reduced
        if (!normalise_axes(op, in.len(), &axes, err)) return false;
        out->push_back({reduced_dims(in, axes, op.keep_dims), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Identity:
    case OpKind::Sqrt:
    case OpKind::ReLU:
    case OpKind::Gelu:
    case OpKind::Sigmoid:
    case OpKind::Erf:
    case OpKind::Tanh:
    case OpKind::HardSigmoid:
    case OpKind::Softmax: {
        if (!need_inputs(1)) return false;
        out->push_back({inputs[0]->dims(), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::LayerNormalization: {
        if (!need_inputs(3)) return false;
        if (num_outputs != 1) return fail(err, "LayerNormalization: exactly one output is supported");
        if (op.stash_type != 1) return fail(err, "LayerNormalization: stash_type must be 1");
        out->push_back({inputs[0]->dims(), inputs[0]->elem_ty()});
        return true;
    }
    default:
        return fail(err, std::string(op.name()) + ": Unsupported op");
    }
}

bool infer_shapes(const Model &model, InferredShapes *shapes, std::map<ValueId, TypedFixedShape> *value_shapes,
                  ShapeError *err) {
    std::map<ValueId, Tensor> values;
    for (const auto &kv : model.graph.inits)
        values[kv.first] = Tensor::empty_of_type(kv.second.elem_ty(), kv.second.dims());
    for (ValueId id : model.graph.inputs) {
        const auto &shape = model.graph.values[id].shape;
        if (!shape) continue;
        auto fixed = shape->dims.as_fixed_dims();
        if (!fixed) return fail(err, "Must be fixed dimension");
        values[id] = Tensor::empty_of_type(shape->elem_ty, *fixed);
    }
    for (NodeId nid : model.topo_sort_nodes()) {
        const Node &node = model.graph.nodes[nid];
        std::vector<const Tensor *> inputs;
        bool known = true;
        for (ValueId in : node.inputs) {
            auto it = values.find(in);
            if (it == values.end()) {
                known = false;
                break;
            }
            inputs.push_back(&it->second);
        }
        if (!known) continue;
        Op op = node.op;
        std::vector<TypedFixedShape> out;
        if (!compute_output_shapes(model, op, inputs, node.outputs.size(), &out, err)) return false;
        for (size_t i = 0; i < node.outputs.size() && i < out.size(); i++)
            values[node.outputs[i]] = Tensor::empty_of_type(out[i].elem_ty, out[i].dims);
        if (shapes) (*shapes)[nid] = {op, out};
    }
    if (value_shapes)
        for (const auto &kv : values) (*value_shapes)[kv.first] = {kv.second.dims(), kv.second.elem_ty()};
    return true;
}

}  // namespace altius
