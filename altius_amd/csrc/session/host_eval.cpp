#include "host_eval.h"

#include <algorithm>
#include <cstring>

namespace altius {

namespace {

bool is_int_like(TensorElemType t) { return t != TensorElemType::F32; }

// Integer / bool contents widened to int64.
bool read_i64(const Tensor &t, std::vector<int64_t> *out) {
    const size_t n = t.dims().total_elems();
    if (!t.has_data()) return false;
    out->resize(n);
    const uint8_t *p = t.data_as_bytes();
    switch (t.elem_ty()) {
    case TensorElemType::I64: std::memcpy(out->data(), p, n * 8); return true;
    case TensorElemType::I32:
        for (size_t i = 0; i < n; i++) (*out)[i] = reinterpret_cast<const int32_t *>(p)[i];
        return true;
    case TensorElemType::Bool:
        for (size_t i = 0; i < n; i++) (*out)[i] = p[i] ? 1 : 0;
        return true;
    case TensorElemType::F32: return false;
    }
    return false;
}

Tensor make_tensor(const TypedFixedShape &s, const std::vector<int64_t> &v) {
    const size_t n = s.dims.total_elems();
    switch (s.elem_ty) {
    case TensorElemType::I64: return Tensor::from_raw(s.dims, s.elem_ty, v.data(), n * 8);
    case TensorElemType::I32: {
        std::vector<int32_t> w(n);
        for (size_t i = 0; i < n; i++) w[i] = (int32_t)v[i];
        return Tensor::from_raw(s.dims, s.elem_ty, w.data(), n * 4);
    }
    case TensorElemType::Bool: {
        std::vector<uint8_t> w(n);
        for (size_t i = 0; i < n; i++) w[i] = v[i] != 0;
        return Tensor::from_raw(s.dims, s.elem_ty, w.data(), n);
    }
    case TensorElemType::F32: {
        std::vector<float> w(n);
        for (size_t i = 0; i < n; i++) w[i] = (float)v[i];  // Rust `as f32`: round to nearest
        return Tensor::from_raw(s.dims, s.elem_ty, w.data(), n * 4);
    }
    }
    return Tensor();
}

bool fail(std::string *error, const std::string &msg) {
    if (error) *error = msg;
    return false;
}

// Offsets of every element of `dims` read through `strides` (row-major walk).
void walk(const FixedDimensions &dims, const std::vector<int64_t> &strides, std::vector<size_t> *offsets) {
    const size_t n = dims.total_elems(), r = dims.len();
    offsets->resize(n);
    std::vector<size_t> idx(r, 0);
    for (size_t i = 0; i < n; i++) {
        int64_t off = 0;
        for (size_t d = 0; d < r; d++) off += (int64_t)idx[d] * strides[d];
        (*offsets)[i] = (size_t)off;
        for (size_t d = r; d-- > 0;) {
            if (++idx[d] < dims[d]) break;
            idx[d] = 0;
        }
    }
}

std::vector<int64_t> i64_strides(const FixedDimensions &f) {
    std::vector<int64_t> s;
    for (auto x : f.as_vec()) s.push_back((int64_t)x);
    return s;
}

}  // namespace

bool host_evaluable(const Op &op) {
    switch (op.kind) {
    case OpKind::Shape:
    case OpKind::Constant:
    case OpKind::Identity:
    case OpKind::Reshape:
    case OpKind::Flatten:
    case OpKind::Squeeze:
    case OpKind::Unsqueeze:
    case OpKind::Gather:
    case OpKind::Concat:
    case OpKind::Slice:
    case OpKind::Cast:
    case OpKind::Add:
    case OpKind::Sub:
    case OpKind::Mul:
    case OpKind::Div:
    case OpKind::Range:
    case OpKind::Expand:
    case OpKind::Where:
    case OpKind::Greater: return true;
    default: return false;
    }
}

bool evaluate_on_host(const Model &model, const Op &op, const std::vector<const Tensor *> &in,
                      const std::vector<TypedFixedShape> &shapes, std::vector<Tensor> *outputs, std::string *error) {
    (void)model;
    outputs->clear();
    if (shapes.empty()) return fail(error, std::string(op.name()) + ": no output shape");
    const TypedFixedShape &os = shapes[0];
    // What runs here is the integer arithmetic on shapes and indices that exporters leave in a graph: small tensors.
    // A result of 2^26 elements and more (a Range whose limit is a mistake) is refused instead of filling host memory.
    if (os.dims.total_elems() >= ((size_t)1 << 26))
        return fail(error, std::string(op.name()) + ": a result of " + std::to_string(os.dims.total_elems()) + " elements is too large to evaluate on the host");
    auto input = [&](size_t i) -> const Tensor * { return i < in.size() ? in[i] : nullptr; };
    auto ints = [&](size_t i, std::vector<int64_t> *v) {
        const Tensor *t = input(i);
        return t && read_i64(*t, v);
    };
    switch (op.kind) {
    case OpKind::Shape: {  // compute_shape (session.rs:1600-1608), with start / end
        if (!input(0)) return fail(error, "Shape: missing input");
        const auto &d = input(0)->dims();
        const int64_t rank = (int64_t)d.len();
        int64_t s = op.start < 0 ? op.start + rank : op.start;
        s = std::min(std::max<int64_t>(s, 0), rank);
        std::vector<int64_t> v;
        for (size_t i = 0; i < os.dims.total_elems(); i++) v.push_back((int64_t)d[(size_t)s + i]);
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Constant:
        if (!op.value) return fail(error, "Constant: no value");
        outputs->push_back(*op.value);
        return true;
    case OpKind::Identity:
    case OpKind::Reshape:
    case OpKind::Flatten:
    case OpKind::Squeeze:
    case OpKind::Unsqueeze: {
        if (!input(0) || !input(0)->has_data()) return fail(error, std::string(op.name()) + ": input contents unknown");
        Tensor t = input(0)->reshaped(os.dims);
        if (!t.has_data() && os.dims.total_elems()) return fail(error, std::string(op.name()) + ": element count changes");
        outputs->push_back(std::move(t));
        return true;
    }
    default: break;
    }
    // Everything below computes on integer values.
    if (op.kind != OpKind::Cast && op.kind != OpKind::Where && op.kind != OpKind::Greater && !is_int_like(os.elem_ty))
        return fail(error, std::string(op.name()) + ": float tensors are computed on the device");
    switch (op.kind) {
    case OpKind::Cast: {
        std::vector<int64_t> v;
        if (!ints(0, &v)) return fail(error, "Cast: only integer and bool sources are evaluated on the host");
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Gather: {
        std::vector<int64_t> data, idx;
        if (!ints(0, &data) || !ints(1, &idx)) return fail(error, "Gather: operands unknown on the host");
        const auto &d = input(0)->dims();
        const int64_t axis = op.axis < 0 ? op.axis + (int64_t)d.len() : op.axis;
        size_t outer = 1, inner = 1;
        for (size_t i = 0; i < (size_t)axis; i++) outer *= d[i];
        for (size_t i = (size_t)axis + 1; i < d.len(); i++) inner *= d[i];
        const size_t len = d[(size_t)axis];
        std::vector<int64_t> v;
        for (size_t o = 0; o < outer; o++)
            for (int64_t k : idx) {
                if (k < 0) k += (int64_t)len;
                if (k < 0 || k >= (int64_t)len) return fail(error, "Gather: an index is outside the gathered axis");
                for (size_t i = 0; i < inner; i++) v.push_back(data[(o * len + (size_t)k) * inner + i]);
            }
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Concat: {
        if (in.empty() || !input(0)) return fail(error, "Concat: no inputs");
        const size_t rank = os.dims.len();
        const int64_t axis = op.axis < 0 ? op.axis + (int64_t)rank : op.axis;
        size_t outer = 1, inner = 1;
        for (size_t i = 0; i < (size_t)axis; i++) outer *= os.dims[i];
        for (size_t i = (size_t)axis + 1; i < rank; i++) inner *= os.dims[i];
        std::vector<std::vector<int64_t>> parts(in.size());
        for (size_t k = 0; k < in.size(); k++)
            if (!ints(k, &parts[k])) return fail(error, "Concat: operands unknown on the host");
        std::vector<int64_t> v;
        for (size_t o = 0; o < outer; o++)
            for (size_t k = 0; k < in.size(); k++) {
                const size_t chunk = in[k]->dims()[(size_t)axis] * inner;
                v.insert(v.end(), parts[k].begin() + (long)(o * chunk), parts[k].begin() + (long)((o + 1) * chunk));
            }
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Slice: {
        std::vector<int64_t> data, starts, ends, axes, steps;
        if (!ints(0, &data) || !ints(1, &starts) || !ints(2, &ends)) return fail(error, "Slice: operands unknown on the host");
        if (input(3) && input(3)->dims().total_elems()) {
            if (!ints(3, &axes)) return fail(error, "Slice: axes unknown on the host");
        } else {
            for (size_t i = 0; i < starts.size(); i++) axes.push_back((int64_t)i);
        }
        if (input(4) && input(4)->dims().total_elems()) {
            if (!ints(4, &steps)) return fail(error, "Slice: steps unknown on the host");
        } else {
            steps.assign(starts.size(), 1);
        }
        const auto &d = input(0)->dims();
        std::vector<int64_t> str = i64_strides(d.strides()), base_str = str;
        int64_t base = 0;
        for (size_t i = 0; i < starts.size(); i++) {
            const int64_t ax = axes[i] < 0 ? axes[i] + (int64_t)d.len() : axes[i];
            const int64_t n = (int64_t)d[(size_t)ax];
            int64_t s = starts[i] < 0 ? starts[i] + n : starts[i];
            s = std::min(std::max<int64_t>(s, 0), n);
            base += s * base_str[(size_t)ax];
            str[(size_t)ax] = base_str[(size_t)ax] * steps[i];
        }
        std::vector<size_t> offs;
        walk(os.dims, str, &offs);
        std::vector<int64_t> v;
        for (size_t o : offs) v.push_back(data[(size_t)base + o]);
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Add:
    case OpKind::Sub:
    case OpKind::Mul:
    case OpKind::Div: {
        std::vector<int64_t> a, b;
        if (!ints(0, &a) || !ints(1, &b)) return fail(error, std::string(op.name()) + ": operands unknown on the host");
        auto sa = input(0)->dims().strides_for_broadcasting_to(os.dims), sb = input(1)->dims().strides_for_broadcasting_to(os.dims);
        if (!sa || !sb) return fail(error, std::string(op.name()) + ": operands do not broadcast");
        std::vector<size_t> oa, ob;
        walk(os.dims, i64_strides(*sa), &oa);
        walk(os.dims, i64_strides(*sb), &ob);
        std::vector<int64_t> v(oa.size());
        for (size_t i = 0; i < oa.size(); i++) {
            const int64_t x = a[oa[i]], y = b[ob[i]];
            switch (op.kind) {
            case OpKind::Add: v[i] = (int64_t)((uint64_t)x + (uint64_t)y); break;
            case OpKind::Sub: v[i] = (int64_t)((uint64_t)x - (uint64_t)y); break;
            case OpKind::Mul: v[i] = (int64_t)((uint64_t)x * (uint64_t)y); break;
            default:
                if (y == 0) return fail(error, "Div: integer division by zero");
                v[i] = (x == INT64_MIN && y == -1) ? INT64_MIN : x / y;
                break;
            }
        }
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Range: {
        std::vector<int64_t> s, l, d;
        if (!ints(0, &s) || !ints(1, &l) || !ints(2, &d) || s.empty() || d.empty()) return fail(error, "Range: operands unknown on the host");
        std::vector<int64_t> v;
        for (size_t i = 0; i < os.dims.total_elems(); i++) v.push_back(s[0] + (int64_t)i * d[0]);
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Expand: {
        std::vector<int64_t> a;
        if (!ints(0, &a)) return fail(error, "Expand: operand unknown on the host");
        auto sa = input(0)->dims().strides_for_broadcasting_to(os.dims);
        if (!sa) return fail(error, "Expand: operand does not broadcast");
        std::vector<size_t> oa;
        walk(os.dims, i64_strides(*sa), &oa);
        std::vector<int64_t> v;
        for (size_t o : oa) v.push_back(a[o]);
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Where: {
        std::vector<int64_t> c, x, y;
        if (!ints(0, &c) || !ints(1, &x) || !ints(2, &y)) return fail(error, "Where: operands unknown on the host");
        auto sc = input(0)->dims().strides_for_broadcasting_to(os.dims), sx = input(1)->dims().strides_for_broadcasting_to(os.dims),
             sy = input(2)->dims().strides_for_broadcasting_to(os.dims);
        if (!sc || !sx || !sy) return fail(error, "Where: operands do not broadcast");
        std::vector<size_t> oc, ox, oy;
        walk(os.dims, i64_strides(*sc), &oc);
        walk(os.dims, i64_strides(*sx), &ox);
        walk(os.dims, i64_strides(*sy), &oy);
        std::vector<int64_t> v(oc.size());
        for (size_t i = 0; i < oc.size(); i++) v[i] = c[oc[i]] ? x[ox[i]] : y[oy[i]];
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    case OpKind::Greater: {
        std::vector<int64_t> a, b;
        if (!ints(0, &a) || !ints(1, &b)) return fail(error, "Greater: only integer operands are evaluated on the host");
        auto sa = input(0)->dims().strides_for_broadcasting_to(os.dims), sb = input(1)->dims().strides_for_broadcasting_to(os.dims);
        if (!sa || !sb) return fail(error, "Greater: operands do not broadcast");
        std::vector<size_t> oa, ob;
        walk(os.dims, i64_strides(*sa), &oa);
        walk(os.dims, i64_strides(*sb), &ob);
        std::vector<int64_t> v(oa.size());
        for (size_t i = 0; i < oa.size(); i++) v[i] = a[oa[i]] > b[ob[i]];
        outputs->push_back(make_tensor(os, v));
        return true;
    }
    default: return fail(error, std::string(op.name()) + ": not evaluated on the host");
    }
}

}  // namespace altius
