#include "shape.h"

#include <algorithm>
#include <cmath>

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

bool needs_data(ShapeError *err, const std::string &what) {
    if (err) {
        err->message = what + " is not known before the graph runs";
        err->needs_data = true;
    }
    return false;
}

// Integer contents of a shape-like operand (i64, or i32 widened).
bool read_ints(const Tensor &t, std::vector<int64_t> *out, const char *what, ShapeError *err) {
    const size_t n = t.dims().total_elems();
    if (t.elem_ty() != TensorElemType::I64 && t.elem_ty() != TensorElemType::I32)
        return fail(err, std::string(what) + " must be an integer tensor");
    if (n == 0) return true;
    if (!t.has_data()) return needs_data(err, what);
    if (t.elem_ty() == TensorElemType::I64) {
        const int64_t *p = reinterpret_cast<const int64_t *>(t.data_as_bytes());
        out->assign(p, p + n);
    } else {
        const int32_t *p = reinterpret_cast<const int32_t *>(t.data_as_bytes());
        out->assign(p, p + n);
    }
    return true;
}

// Total padding along H and W for Conv2d / MaxPool, normalising op.padding to
// [top, left, bottom, right] (shape.rs:47-72, 113-124).
bool pool_padding(Op &op, const FixedDimensions &in, size_t *pad_h, size_t *pad_w, ShapeError *err) {
    if (!op.auto_pad.empty() && op.auto_pad != "NOTSET") {
        if (op.auto_pad != "SAME_UPPER") return fail(err, std::string(op.name()) + ": auto_pad " + op.auto_pad + " is not supported");
        const size_t s0 = (size_t)op.strides[0], s1 = (size_t)op.strides[1];
        const size_t out0 = (size_t)std::ceil((float)in[2] / (float)s0), out1 = (size_t)std::ceil((float)in[3] / (float)s1);
        const size_t need0 = (out0 - 1) * s0 + (size_t)op.kernel_shape[0], need1 = (out1 - 1) * s1 + (size_t)op.kernel_shape[1];
        const size_t p0 = need0 > in[2] ? need0 - in[2] : 0, p1 = need1 > in[3] ? need1 - in[3] : 0;
        op.padding = {(int64_t)(p0 / 2), (int64_t)(p1 / 2), (int64_t)(p0 - p0 / 2), (int64_t)(p1 - p1 / 2)};
        *pad_h = p0;
        *pad_w = p1;
        return true;
    }
    for (int64_t p : op.padding)
        if (p < 0) return fail(err, std::string(op.name()) + ": negative padding");
    if (op.padding.size() == 2) {
        op.padding = {op.padding[0], op.padding[1], op.padding[0], op.padding[1]};
    } else if (op.padding.size() != 4) {
        return fail(err, std::string(op.name()) + ": Unknown padding pattern");
    }
    *pad_h = (size_t)(op.padding[0] + op.padding[2]);
    *pad_w = (size_t)(op.padding[1] + op.padding[3]);
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
    case OpKind::LeakyReLU:
    case OpKind::Gelu:
    case OpKind::Sigmoid:
    case OpKind::Erf:
    case OpKind::Tanh:
    case OpKind::Clip:
    case OpKind::HardSigmoid:
    case OpKind::Round:
    case OpKind::Exp:
    case OpKind::Softmax:
    case OpKind::BatchNormalization: {
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
    case OpKind::FusedElemwise: {  // shape.rs:616-650: the chain's steps one after the other
        if (!op.fused || op.fused->chain.empty()) return fail(err, "FusedElemwise: empty chain");
        const FusedElemwise &f = *op.fused;
        if (!need_inputs(f.input_map.size())) return false;
        std::map<size_t, const Tensor *> outer;
        for (size_t i = 0; i < f.input_map.size(); i++) outer[f.input_map[i]] = inputs[i];
        Tensor prev;
        bool have_prev = false;
        size_t prev_id = 0;
        std::vector<TypedFixedShape> step_out;
        for (const auto &step : f.chain) {
            if (step.outputs.size() != 1) return fail(err, "FusedElemwise: a step must have one output");
            std::vector<const Tensor *> ins;
            for (size_t v : step.inputs) {
                auto it = outer.find(v);
                if (it != outer.end()) ins.push_back(it->second);
                else if (have_prev && v == prev_id) ins.push_back(&prev);
                else return fail(err, "FusedElemwise: a step reads a value that is neither an input nor the previous result");
            }
            Op step_op = step.op;
            step_out.clear();
            if (!compute_output_shapes(model, step_op, ins, 1, &step_out, err)) return false;
            if (step_out.empty()) return fail(err, "FusedElemwise: a step produced no shape");
            prev = Tensor::empty_of_type(step_out[0].elem_ty, step_out[0].dims);
            have_prev = true;
            prev_id = step.outputs[0];
        }
        out->push_back(step_out[0]);
        return true;
    }
    case OpKind::Cast: {  // shape.rs:612-615
        if (!need_inputs(1)) return false;
        out->push_back({inputs[0]->dims(), op.to});
        return true;
    }
    case OpKind::Greater: {  // shape.rs:95-100
        if (!need_inputs(2)) return false;
        auto shape = inputs[0]->dims().broadcast(inputs[1]->dims());
        if (!shape) return fail(err, "Greater: cannot broadcast " + inputs[0]->dims().to_string() + " with " + inputs[1]->dims().to_string());
        out->push_back({*shape, TensorElemType::Bool});
        return true;
    }
    case OpKind::Where: {  // shape.rs:101-106 broadcasts x and y; the condition is broadcast in as well here
        if (!need_inputs(3)) return false;
        auto shape = broadcast({&inputs[0]->dims(), &inputs[1]->dims(), &inputs[2]->dims()});
        if (!shape) return fail(err, "Where: operands do not broadcast");
        out->push_back({*shape, inputs[1]->elem_ty()});
        return true;
    }
    case OpKind::Conv2d: {  // shape.rs:38-88
        if (!need_inputs(2)) return false;
        const FixedDimensions &in = inputs[0]->dims(), &w = inputs[1]->dims();
        if (in.len() != 4 || w.len() != 4) return fail(err, "Conv2d: input and weight must have four dimensions");
        if (op.kernel_shape.size() != 2 || op.strides.size() != 2 || op.dilations.size() != 2)
            return fail(err, "Conv2d: kernel_shape, strides and dilations must have two entries");
        for (int i = 0; i < 2; i++)
            if (op.kernel_shape[i] <= 0 || op.strides[i] <= 0 || op.dilations[i] <= 0) return fail(err, "Conv2d: non-positive kernel, stride or dilation");
        size_t pad_h, pad_w;
        if (!pool_padding(op, in, &pad_h, &pad_w, err)) return false;
        const size_t eff_h = (size_t)op.dilations[0] * ((size_t)op.kernel_shape[0] - 1) + 1;
        const size_t eff_w = (size_t)op.dilations[1] * ((size_t)op.kernel_shape[1] - 1) + 1;
        if (in[2] + pad_h < eff_h || in[3] + pad_w < eff_w) return fail(err, "Conv2d: kernel larger than the padded input");
        out->push_back({FixedDimensions({in[0], w[0], (in[2] + pad_h - eff_h) / (size_t)op.strides[0] + 1,
                                         (in[3] + pad_w - eff_w) / (size_t)op.strides[1] + 1}),
                        inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::MaxPool: {  // shape.rs:107-139
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        if (in.len() != 4) return fail(err, "MaxPool: input must have four dimensions");
        if (op.kernel_shape.size() != 2 || op.strides.size() != 2) return fail(err, "MaxPool: kernel_shape and strides must have two entries");
        for (int i = 0; i < 2; i++)
            if (op.kernel_shape[i] <= 0 || op.strides[i] <= 0) return fail(err, "MaxPool: non-positive kernel or stride");
        size_t pad_h, pad_w;
        if (!pool_padding(op, in, &pad_h, &pad_w, err)) return false;
        if (in[2] + pad_h < (size_t)op.kernel_shape[0] || in[3] + pad_w < (size_t)op.kernel_shape[1])
            return fail(err, "MaxPool: kernel larger than the padded input");
        out->push_back({FixedDimensions({in[0], in[1], (in[2] + pad_h - (size_t)op.kernel_shape[0]) / (size_t)op.strides[0] + 1,
                                         (in[3] + pad_w - (size_t)op.kernel_shape[1]) / (size_t)op.strides[1] + 1}),
                        inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::GlobalAveragePool: {  // shape.rs:140-147
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        if (in.len() != 4) return fail(err, "GlobalAveragePool: input must have four dimensions");
        out->push_back({FixedDimensions({in[0], in[1], 1, 1}), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Expand: {  // shape.rs:148-161 takes the shape operand as is; ONNX broadcasts it with the input
        if (!need_inputs(2)) return false;
        std::vector<int64_t> shape;
        if (!read_ints(*inputs[1], &shape, "Expand: shape", err)) return false;
        std::vector<FixedDimension> d;
        for (int64_t x : shape) {
            if (x < 0) return fail(err, "Expand: negative dimension");
            d.push_back((size_t)x);
        }
        const FixedDimensions want(std::move(d));
        auto b = inputs[0]->dims().broadcast(want);
        if (!b) return fail(err, "Expand: " + inputs[0]->dims().to_string() + " does not broadcast to " + want.to_string());
        out->push_back({*b, inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Range: {  // shape.rs:162-177
        if (!need_inputs(3)) return false;
        if (inputs[0]->elem_ty() != TensorElemType::I64) return fail(err, "Range only supports i64 for now");
        std::vector<int64_t> s, l, d;
        if (!read_ints(*inputs[0], &s, "Range: start", err) || !read_ints(*inputs[1], &l, "Range: limit", err) ||
            !read_ints(*inputs[2], &d, "Range: delta", err))
            return false;
        if (s.empty() || l.empty() || d.empty() || d[0] == 0) return fail(err, "Range: start, limit and a non-zero delta are needed");
        const int64_t n = std::max<int64_t>(0, (int64_t)std::ceil((float)(l[0] - s[0]) / (float)d[0]));
        out->push_back({FixedDimensions({(size_t)n}), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Reshape: {  // shape.rs:178-199, plus ONNX's "0 copies the input dimension"
        if (!need_inputs(2)) return false;
        std::vector<int64_t> shape;
        if (!read_ints(*inputs[1], &shape, "Reshape: shape", err)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        size_t known = 1;
        int wild = -1;
        std::vector<FixedDimension> d(shape.size());
        for (size_t i = 0; i < shape.size(); i++) {
            if (shape[i] == -1) {
                if (wild >= 0) return fail(err, "Reshape: more than one -1");
                wild = (int)i;
            } else if (shape[i] == 0) {
                if (i >= in.len()) return fail(err, "Reshape: 0 refers to a dimension the input does not have");
                d[i] = in[i];
                known *= d[i];
            } else if (shape[i] < 0) {
                return fail(err, "Reshape: negative dimension");
            } else {
                d[i] = (size_t)shape[i];
                known *= d[i];
            }
        }
        const size_t total = in.total_elems();
        if (wild >= 0) {
            if (known == 0 || total % known) return fail(err, "Reshape: cannot infer the -1 dimension");
            d[(size_t)wild] = total / known;
        } else if (known != total) {
            return fail(err, "Reshape: " + in.to_string() + " does not hold as many elements as the new shape");
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Flatten: {  // shape.rs:200-209
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        int64_t axis = op.axis < 0 ? op.axis + (int64_t)in.len() : op.axis;
        if (axis < 0 || axis > (int64_t)in.len()) return fail(err, "Flatten: axis out of range");
        size_t x = 1, y = 1;
        for (size_t i = 0; i < in.len(); i++) (i < (size_t)axis ? x : y) *= in[i];
        out->push_back({FixedDimensions({x, y}), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Resize: {  // shape.rs:210-260
        if (inputs.size() == 4) {
            std::vector<int64_t> sizes;
            if (!read_ints(*inputs[3], &sizes, "Resize: sizes", err)) return false;
            if (sizes.size() != 4) return fail(err, "Resize: sizes must have four entries");
            std::vector<FixedDimension> d;
            for (int64_t x : sizes) {
                if (x < 0) return fail(err, "Resize: negative size");
                d.push_back((size_t)x);
            }
            out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
            return true;
        }
        if (inputs.size() == 3) {
            const FixedDimensions &in = inputs[0]->dims();
            if (in.len() != 4) return fail(err, "Resize: input must have four dimensions");
            const Tensor &sc = *inputs[2];
            if (sc.elem_ty() != TensorElemType::F32) return fail(err, "Resize: scales must be f32");
            if (!sc.has_data() || sc.dims().total_elems() == 0) return needs_data(err, "Resize: scales");
            if (sc.dims().total_elems() != 4) return fail(err, "Resize: scales must have four entries");
            const float *f = sc.data_f32();
            std::vector<FixedDimension> d;
            for (int i = 0; i < 4; i++) d.push_back((size_t)std::floor((float)in[(size_t)i] * f[i]));
            out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
            return true;
        }
        return fail(err, "Resize: Unsupported pattern");
    }
    case OpKind::Concat: {  // shape.rs:261-269
        if (!need_inputs(1)) return false;
        const FixedDimensions &first = inputs[0]->dims();
        const int64_t axis = op.axis < 0 ? op.axis + (int64_t)first.len() : op.axis;
        if (axis < 0 || axis >= (int64_t)first.len()) return fail(err, "Concat: axis out of range");
        std::vector<FixedDimension> d = first.as_vec();
        size_t sum = 0;
        for (const Tensor *t : inputs) {
            if (t->dims().len() != first.len()) return fail(err, "Concat: inputs differ in rank");
            for (size_t i = 0; i < first.len(); i++)
                if (i != (size_t)axis && t->dims()[i] != first[i]) return fail(err, "Concat: inputs differ outside the axis");
            sum += t->dims()[(size_t)axis];
        }
        d[(size_t)axis] = sum;
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Transpose: {  // shape.rs:270-281
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        if (op.perm.size() != in.len()) return fail(err, "Transpose: perm must name every axis once");
        std::vector<bool> seen(in.len(), false);
        std::vector<FixedDimension> d(in.len());
        for (size_t i = 0; i < in.len(); i++) {
            const int64_t p = op.perm[i];
            if (p < 0 || p >= (int64_t)in.len() || seen[(size_t)p]) return fail(err, "Transpose: perm must name every axis once");
            seen[(size_t)p] = true;
            d[i] = in[(size_t)p];
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Squeeze: {  // shape.rs:282-314
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        std::vector<int64_t> axes = op.axes;
        if (model.opset_version >= 12 && inputs.size() >= 2) {
            axes.clear();
            if (!read_ints(*inputs[1], &axes, "Squeeze: axes", err)) return false;
        }
        std::vector<FixedDimension> d;
        for (size_t i = 0; i < in.len(); i++) {
            bool drop = false;
            for (int64_t a : axes) drop = drop || (a < 0 ? a + (int64_t)in.len() : a) == (int64_t)i;
            if (axes.empty()) drop = in[i] == 1;  // no axes: every size-1 dimension goes (ONNX)
            if (drop && in[i] != 1) return fail(err, "Squeeze: dimension " + std::to_string(i) + " is not 1");
            if (!drop) d.push_back(in[i]);
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Unsqueeze: {  // shape.rs:315-337
        if (!need_inputs(1)) return false;
        std::vector<int64_t> axes = op.axes;
        if (model.opset_version >= 13) {
            if (!need_inputs(2)) return false;
            axes.clear();
            if (!read_ints(*inputs[1], &axes, "Unsqueeze: axes", err)) return false;
        }
        std::vector<FixedDimension> d = inputs[0]->dims().as_vec();
        const int64_t out_rank = (int64_t)(d.size() + axes.size());
        std::vector<int64_t> sorted;
        for (int64_t a : axes) sorted.push_back(a < 0 ? a + out_rank : a);
        std::sort(sorted.begin(), sorted.end());
        for (int64_t a : sorted) {
            if (a < 0 || a > (int64_t)d.size()) return fail(err, "Unsqueeze: axis out of range");
            d.insert(d.begin() + a, 1);
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::ReduceMin: {  // shape.rs:338-353
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        std::vector<size_t> axes;
        if (!normalise_axes(op, in.len(), &axes, err)) return false;
        out->push_back({reduced_dims(in, axes, op.keep_dims), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Loop: return fail(err, "Loop: Unsupported op");  // shape.rs:412-422
    case OpKind::Tile: {  // shape.rs:423-434
        if (!need_inputs(2)) return false;
        std::vector<int64_t> reps;
        if (!read_ints(*inputs[1], &reps, "Tile: repeats", err)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        if (reps.size() != in.len()) return fail(err, "Tile: repeats must have one entry per dimension");
        std::vector<FixedDimension> d;
        for (size_t i = 0; i < in.len(); i++) {
            if (reps[i] < 0) return fail(err, "Tile: negative repeat");
            d.push_back(in[i] * (size_t)reps[i]);
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Split: {  // shape.rs:435-462
        if (!need_inputs(1)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        const int64_t axis = op.axis < 0 ? op.axis + (int64_t)in.len() : op.axis;
        if (axis < 0 || axis >= (int64_t)in.len()) return fail(err, "Split: axis out of range");
        std::vector<int64_t> split = op.split;
        if (model.opset_version >= 13 && inputs.size() >= 2) {
            split.clear();
            if (!read_ints(*inputs[1], &split, "Split: split", err)) return false;
        }
        if (split.empty()) {  // equal parts, one per output (ONNX)
            if (num_outputs == 0 || in[(size_t)axis] % num_outputs) return fail(err, "Split: the axis does not divide evenly over the outputs");
            split.assign(num_outputs, (int64_t)(in[(size_t)axis] / num_outputs));
        }
        size_t sum = 0;
        for (int64_t x : split) {
            if (x < 0) return fail(err, "Split: negative part");
            sum += (size_t)x;
        }
        if (sum != in[(size_t)axis]) return fail(err, "Split: parts do not add up to the axis");
        for (int64_t x : split) {
            std::vector<FixedDimension> d = in.as_vec();
            d[(size_t)axis] = (size_t)x;
            out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        }
        return true;
    }
    case OpKind::Slice: {  // shape.rs:463-503; negative and oversized bounds are clamped as ONNX defines
        if (!need_inputs(3)) return false;
        const FixedDimensions &in = inputs[0]->dims();
        std::vector<int64_t> starts, ends, axes, steps;
        if (!read_ints(*inputs[1], &starts, "Slice: starts", err) || !read_ints(*inputs[2], &ends, "Slice: ends", err)) return false;
        if (inputs.size() > 3 && inputs[3]->dims().total_elems() > 0) {
            if (!read_ints(*inputs[3], &axes, "Slice: axes", err)) return false;
        } else {
            for (size_t i = 0; i < starts.size(); i++) axes.push_back((int64_t)i);
        }
        if (inputs.size() > 4 && inputs[4]->dims().total_elems() > 0) {
            if (!read_ints(*inputs[4], &steps, "Slice: steps", err)) return false;
        } else {
            steps.assign(starts.size(), 1);
        }
        if (ends.size() != starts.size() || axes.size() != starts.size() || steps.size() != starts.size())
            return fail(err, "Slice: starts, ends, axes and steps differ in length");
        std::vector<FixedDimension> d = in.as_vec();
        for (size_t i = 0; i < starts.size(); i++) {
            const int64_t ax = axes[i] < 0 ? axes[i] + (int64_t)in.len() : axes[i];
            if (ax < 0 || ax >= (int64_t)in.len()) return fail(err, "Slice: axis out of range");
            if (steps[i] <= 0) return fail(err, "Slice: only positive steps are supported");
            const int64_t n = (int64_t)in[(size_t)ax];
            int64_t s = starts[i] < 0 ? starts[i] + n : starts[i];
            int64_t e = ends[i] < 0 ? ends[i] + n : ends[i];
            s = std::min(std::max<int64_t>(s, 0), n);
            e = std::min(std::max<int64_t>(e, 0), n);
            d[(size_t)ax] = e > s ? (size_t)((e - s + steps[i] - 1) / steps[i]) : 0;
        }
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Gather: {  // shape.rs:504-524; any index shape (ONNX), of which the reference takes two
        if (!need_inputs(2)) return false;
        const FixedDimensions &data = inputs[0]->dims(), &idx = inputs[1]->dims();
        const int64_t axis = op.axis < 0 ? op.axis + (int64_t)data.len() : op.axis;
        if (axis < 0 || axis >= (int64_t)data.len()) return fail(err, "Gather: axis out of range");
        std::vector<FixedDimension> d;
        for (size_t i = 0; i < (size_t)axis; i++) d.push_back(data[i]);
        if (!(idx.len() == 0)) for (size_t i = 0; i < idx.len(); i++) d.push_back(idx[i]);
        for (size_t i = (size_t)axis + 1; i < data.len(); i++) d.push_back(data[i]);
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Shape: {  // shape.rs:525-533 (start 0, no end); start/end as ONNX defines them otherwise
        if (!need_inputs(1)) return false;
        const int64_t rank = (int64_t)inputs[0]->dims().len();
        int64_t s = op.start < 0 ? op.start + rank : op.start;
        int64_t e = op.end ? (*op.end < 0 ? *op.end + rank : *op.end) : rank;
        s = std::min(std::max<int64_t>(s, 0), rank);
        e = std::min(std::max<int64_t>(e, 0), rank);
        out->push_back({FixedDimensions({(size_t)std::max<int64_t>(0, e - s)}), TensorElemType::I64});
        return true;
    }
    case OpKind::NonMaxSuppression: return fail(err, "NonMaxSuppression: Unsupported op");  // shape.rs:534-538
    case OpKind::MatMul: {  // shape.rs:539-569, generalised to NumPy matmul broadcasting of the batch axes
        if (!need_inputs(2)) return false;
        const FixedDimensions &a = inputs[0]->dims(), &b = inputs[1]->dims();
        if (a.len() < 2 || b.len() < 2) return fail(err, "MatMul: operands must have at least two dimensions");
        // trans_a / trans_b are set by fuse_transpose_matmul only: the stored operand is the transposed one.
        const size_t m = op.trans_a ? a[a.len() - 1] : a[a.len() - 2], k = op.trans_a ? a[a.len() - 2] : a[a.len() - 1];
        const size_t k2 = op.trans_b ? b[b.len() - 1] : b[b.len() - 2], n = op.trans_b ? b[b.len() - 2] : b[b.len() - 1];
        if (k != k2) return fail(err, "MatMul: A shape: " + a.to_string() + ", B shape: " + b.to_string());
        std::vector<FixedDimension> ab(a.as_vec().begin(), a.as_vec().end() - 2), bb(b.as_vec().begin(), b.as_vec().end() - 2);
        auto batch = FixedDimensions(ab).broadcast(FixedDimensions(bb));
        if (!batch) return fail(err, "MatMul: A shape: " + a.to_string() + ", B shape: " + b.to_string());
        std::vector<FixedDimension> d = batch->as_vec();
        d.push_back(m);
        d.push_back(n);
        out->push_back({FixedDimensions(std::move(d)), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Gemm: {  // shape.rs:570-589
        if (!need_inputs(2)) return false;
        const FixedDimensions &a = inputs[0]->dims(), &b = inputs[1]->dims();
        if (a.len() != 2 || b.len() != 2) return fail(err, "Gemm: A and B must have two dimensions");
        const size_t a0 = op.trans_a ? a[1] : a[0], a1 = op.trans_a ? a[0] : a[1];
        const size_t b0 = op.trans_b ? b[1] : b[0], b1 = op.trans_b ? b[0] : b[1];
        if (a1 != b0) return fail(err, "Gemm: inner dimensions differ: " + a.to_string() + " and " + b.to_string());
        out->push_back({FixedDimensions({a0, b1}), inputs[0]->elem_ty()});
        return true;
    }
    case OpKind::Constant: {  // shape.rs:590 refuses it; the value's own shape is the answer
        if (!op.value) return fail(err, "Constant: no value");
        out->push_back({op.value->dims(), op.value->elem_ty()});
        return true;
    }
    default:
        return fail(err, std::string(op.name()) + ": Unsupported op");
    }
}

bool infer_shapes(const Model &model, InferredShapes *shapes, std::map<ValueId, TypedFixedShape> *value_shapes,
                  ShapeError *err) {
    std::map<ValueId, Tensor> values;
    for (const auto &kv : model.graph.inits) values[kv.first] = kv.second;  // contents too: shapes may depend on them
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
        ShapeError local;
        if (!compute_output_shapes(model, op, inputs, node.outputs.size(), &out, &local)) {
            if (local.needs_data) continue;  // decided at run time
            if (err) *err = local;
            return false;
        }
        for (size_t i = 0; i < node.outputs.size() && i < out.size(); i++)
            values[node.outputs[i]] = Tensor::empty_of_type(out[i].elem_ty, out[i].dims);
        if (shapes) (*shapes)[nid] = {op, out};
    }
    if (value_shapes)
        for (const auto &kv : values) (*value_shapes)[kv.first] = {kv.second.dims(), kv.second.elem_ty()};
    return true;
}

}  // namespace altius
