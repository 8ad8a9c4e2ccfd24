#include "load.h"

#include <cerrno>
#include <cstdio>
#include <cstring>
#include <map>
#include <unordered_map>

namespace altius {

std::string ModelLoadError::to_string() const {
    switch (kind) {
    case Io: return message;
    case NoGraph: return "Model does not contain any graph";
    case InvalidModel: return "Model is invalid: " + message;
    case DuplicateOpset: return "Model contains duplicated opsets";
    case NoValueType: return "Value type is not specified";
    case NoValueShape: return "Value shape is not specified";
    case NoAttribute: return "Attribute '" + message + "' is not specified";
    case Todo: return "Something went wrong: " + message;
    }
    return message;
}

namespace {

// ---- protobuf wire format -----------------------------------------------------------------
// A message is a sequence of (tag = field << 3 | wire type, payload).  Wire types: 0 varint,
// 1 fixed64, 2 length-delimited, 5 fixed32 (groups, 3 and 4, do not occur in onnx.proto).

struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
    std::string str() const { return std::string(reinterpret_cast<const char *>(p), n); }
};

struct Field {
    uint32_t number = 0;
    uint32_t wire = 0;
    uint64_t varint = 0;  // wire 0; also the raw bits of wire 1 / 5
    Span bytes;           // wire 2
};

class Reader {
public:
    explicit Reader(Span s) : p_(s.p), end_(s.p + s.n) {}
    bool done() const { return p_ >= end_; }
    bool failed() const { return failed_; }

    bool varint(uint64_t *v) {
        uint64_t r = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p_ >= end_) return fail();
            const uint8_t b = *p_++;
            r |= uint64_t(b & 0x7f) << shift;
            if (!(b & 0x80)) {
                *v = r;
                return true;
            }
        }
        return fail();  // more than 10 bytes
    }

    bool next(Field *f) {
        uint64_t tag;
        if (!varint(&tag)) return false;
        f->number = uint32_t(tag >> 3);
        f->wire = uint32_t(tag & 7);
        if (f->number == 0) return fail();
        switch (f->wire) {
        case 0: return varint(&f->varint);
        case 1:
            if (size_t(end_ - p_) < 8) return fail();
            std::memcpy(&f->varint, p_, 8);
            p_ += 8;
            return true;
        case 2: {
            uint64_t len;
            if (!varint(&len)) return false;
            if (len > size_t(end_ - p_)) return fail();
            f->bytes = Span{p_, size_t(len)};
            p_ += len;
            return true;
        }
        case 5: {
            if (size_t(end_ - p_) < 4) return fail();
            uint32_t v;
            std::memcpy(&v, p_, 4);
            f->varint = v;
            p_ += 4;
            return true;
        }
        default: return fail();
        }
    }

private:
    bool fail() {
        failed_ = true;
        p_ = end_;
        return false;
    }
    const uint8_t *p_, *end_;
    bool failed_ = false;
};

// Repeated scalar fields arrive packed (wire 2) or one element per tag; accept both.
bool read_packed_varints(const Field &f, std::vector<int64_t> *out) {
    if (f.wire == 0) {
        out->push_back(int64_t(f.varint));
        return true;
    }
    if (f.wire != 2) return false;
    Reader r(f.bytes);
    while (!r.done()) {
        uint64_t v;
        if (!r.varint(&v)) return false;
        out->push_back(int64_t(v));
    }
    return true;
}

bool read_packed_floats(const Field &f, std::vector<float> *out) {
    if (f.wire == 5) {
        const uint32_t bits = uint32_t(f.varint);
        float v;
        std::memcpy(&v, &bits, 4);
        out->push_back(v);
        return true;
    }
    if (f.wire != 2 || f.bytes.n % 4) return false;
    const size_t n = f.bytes.n / 4, at = out->size();
    out->resize(at + n);
    if (n) std::memcpy(out->data() + at, f.bytes.p, f.bytes.n);
    return true;
}

float float_of(const Field &f) {
    const uint32_t bits = uint32_t(f.varint);
    float v;
    std::memcpy(&v, &bits, 4);
    return v;
}

// ---- the messages the loader looks at -------------------------------------------------------

struct TensorP {  // TensorProto
    std::vector<int64_t> dims;
    int32_t data_type = 0;
    std::vector<float> float_data;
    std::vector<int64_t> int32_data, int64_data;
    std::string name;
    Span raw_data;
    bool has_raw = false;
};

struct AttributeP {  // AttributeProto
    std::string name;
    int32_t type = 0;  // AttributeType; 0 when the writer left it out (IR version < 2)
    float f = 0;
    int64_t i = 0;
    bool has_i = false, has_f = false;
    std::string s;
    TensorP t;
    bool has_t = false, has_g = false;
    std::vector<float> floats;
    std::vector<int64_t> ints;
};

struct NodeP {  // NodeProto
    std::vector<std::string> input, output;
    std::string name, op_type;
    std::vector<AttributeP> attribute;
};

struct DimP {  // TensorShapeProto.Dimension
    bool has_value = false, has_param = false;
    int64_t value = 0;
    std::string param;
};

struct ValueInfoP {  // ValueInfoProto with TypeProto.Tensor flattened in
    std::string name;
    bool has_type = false, has_tensor_type = false, other_type = false, has_shape = false;
    int32_t elem_type = 0;
    std::vector<DimP> dims;
};

struct GraphP {
    std::vector<NodeP> node;
    std::vector<TensorP> initializer;
    std::vector<ValueInfoP> input, output;
};

struct OpsetP {
    std::string domain;
    int64_t version = 0;
};

bool parse_tensor(Span s, TensorP *t) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        switch (f.number) {
        case 1:
            if (!read_packed_varints(f, &t->dims)) return false;
            break;
        case 2: t->data_type = int32_t(f.varint); break;
        case 4:
            if (!read_packed_floats(f, &t->float_data)) return false;
            break;
        case 5:
            if (!read_packed_varints(f, &t->int32_data)) return false;
            break;
        case 7:
            if (!read_packed_varints(f, &t->int64_data)) return false;
            break;
        case 8: t->name = f.bytes.str(); break;
        case 9:
            t->raw_data = f.bytes;
            t->has_raw = true;
            break;
        default: break;  // segment, strings, doubles, external data: not read by the reference either
        }
    }
    return !r.failed();
}

bool parse_attribute(Span s, AttributeP *a) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        switch (f.number) {
        case 1: a->name = f.bytes.str(); break;
        case 2:
            a->f = float_of(f);
            a->has_f = true;
            break;
        case 3:
            a->i = int64_t(f.varint);
            a->has_i = true;
            break;
        case 20: a->type = int32_t(f.varint); break;
        case 4: a->s = f.bytes.str(); break;
        case 5:
            if (!parse_tensor(f.bytes, &a->t)) return false;
            a->has_t = true;
            break;
        case 6: a->has_g = true; break;
        case 7:
            if (!read_packed_floats(f, &a->floats)) return false;
            break;
        case 8:
            if (!read_packed_varints(f, &a->ints)) return false;
            break;
        default: break;
        }
    }
    return !r.failed();
}

bool parse_node(Span s, NodeP *n) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        switch (f.number) {
        case 1: n->input.push_back(f.bytes.str()); break;
        case 2: n->output.push_back(f.bytes.str()); break;
        case 3: n->name = f.bytes.str(); break;
        case 4: n->op_type = f.bytes.str(); break;
        case 5: {
            AttributeP a;
            if (!parse_attribute(f.bytes, &a)) return false;
            n->attribute.push_back(std::move(a));
            break;
        }
        default: break;
        }
    }
    return !r.failed();
}

bool parse_shape(Span s, std::vector<DimP> *dims) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        if (f.number != 1) continue;
        DimP d;
        Reader rd(f.bytes);
        Field g;
        while (!rd.done()) {
            if (!rd.next(&g)) return false;
            if (g.number == 1) {
                d.has_value = true;
                d.value = int64_t(g.varint);
            } else if (g.number == 2) {
                d.has_param = true;
                d.param = g.bytes.str();
            }
        }
        dims->push_back(std::move(d));
    }
    return !r.failed();
}

bool parse_value_info(Span s, ValueInfoP *v) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        if (f.number == 1) {
            v->name = f.bytes.str();
        } else if (f.number == 2) {  // TypeProto
            v->has_type = true;
            Reader rt(f.bytes);
            Field g;
            while (!rt.done()) {
                if (!rt.next(&g)) return false;
                if (g.number == 1) {  // TypeProto.Tensor
                    v->has_tensor_type = true;
                    Reader rr(g.bytes);
                    Field h;
                    while (!rr.done()) {
                        if (!rr.next(&h)) return false;
                        if (h.number == 1) {
                            v->elem_type = int32_t(h.varint);
                        } else if (h.number == 2) {
                            v->has_shape = true;
                            if (!parse_shape(h.bytes, &v->dims)) return false;
                        }
                    }
                } else if (g.number == 4 || g.number == 5 || g.number == 8 || g.number == 9) {
                    v->other_type = true;  // sequence, map, sparse tensor, optional
                }
            }
        }
    }
    return !r.failed();
}

bool parse_graph(Span s, GraphP *g) {
    Reader r(s);
    Field f;
    while (!r.done()) {
        if (!r.next(&f)) return false;
        switch (f.number) {
        case 1: {
            NodeP n;
            if (!parse_node(f.bytes, &n)) return false;
            g->node.push_back(std::move(n));
            break;
        }
        case 5: {
            TensorP t;
            if (!parse_tensor(f.bytes, &t)) return false;
            g->initializer.push_back(std::move(t));
            break;
        }
        case 11:
        case 12: {
            ValueInfoP v;
            if (!parse_value_info(f.bytes, &v)) return false;
            (f.number == 11 ? g->input : g->output).push_back(std::move(v));
            break;
        }
        default: break;
        }
    }
    return !r.failed();
}

// ---- proto -> Model ---------------------------------------------------------------------------

bool fail(ModelLoadError *err, ModelLoadError::Kind kind, std::string msg = {}) {
    if (err) {
        err->kind = kind;
        err->message = std::move(msg);
    }
    return false;
}

// TensorProto.DataType -> TensorElemType (load.rs:426-440).
bool elem_type_of(int32_t data_type, TensorElemType *ty) {
    switch (data_type) {
    case 1: *ty = TensorElemType::F32; return true;
    case 6: *ty = TensorElemType::I32; return true;
    case 7: *ty = TensorElemType::I64; return true;
    case 9: *ty = TensorElemType::Bool; return true;
    default: return false;
    }
}

const char *data_type_name(int32_t t) {
    static const char *names[] = {"Undefined", "Float", "Uint8", "Int8", "Uint16", "Int16", "Int32", "Int64", "String",
                                  "Bool", "Float16", "Double", "Uint32", "Uint64", "Complex64", "Complex128", "Bfloat16"};
    return t >= 0 && t <= 16 ? names[t] : "Unknown";
}

// get_tensor (load.rs:384-424): typed data when raw_data is empty, raw little-endian bytes otherwise.
bool tensor_of(const TensorP &t, Tensor *out, ModelLoadError *err) {
    for (int64_t d : t.dims)
        if (d < 0) return fail(err, ModelLoadError::InvalidModel, "negative tensor dimension");
    FixedDimensions dims = FixedDimensions::from_i64(t.dims.data(), t.dims.size());
    const size_t n = dims.total_elems();
    TensorElemType ty;
    if (!elem_type_of(t.data_type, &ty))
        return fail(err, ModelLoadError::Todo, std::string("Unsupported data type for tensor: ") + data_type_name(t.data_type));
    const size_t want = n * elem_size(ty);
    const bool raw = t.has_raw && t.raw_data.n > 0;
    if (raw) {
        if (t.raw_data.n != want)
            return fail(err, ModelLoadError::InvalidModel, "tensor '" + t.name + "': raw_data size does not match its shape");
        *out = Tensor::from_raw(std::move(dims), ty, t.raw_data.p, want);
        return true;
    }
    switch (ty) {
    case TensorElemType::F32:
        if (t.float_data.size() != n)
            return fail(err, ModelLoadError::InvalidModel, "tensor '" + t.name + "': float_data size does not match its shape");
        *out = Tensor::from_raw(std::move(dims), ty, t.float_data.data(), want);
        return true;
    case TensorElemType::I64:
        if (t.int64_data.size() != n)
            return fail(err, ModelLoadError::InvalidModel, "tensor '" + t.name + "': int64_data size does not match its shape");
        *out = Tensor::from_raw(std::move(dims), ty, t.int64_data.data(), want);
        return true;
    case TensorElemType::I32: {
        if (t.int32_data.size() != n)
            return fail(err, ModelLoadError::InvalidModel, "tensor '" + t.name + "': int32_data size does not match its shape");
        std::vector<int32_t> v(n);
        for (size_t i = 0; i < n; i++) v[i] = int32_t(t.int32_data[i]);
        *out = Tensor::from_raw(std::move(dims), ty, v.data(), want);
        return true;
    }
    case TensorElemType::Bool:
        // The reference reads Bool from raw_data only (load.rs:413-417); an empty tensor is the one legal case left.
        if (n != 0) return fail(err, ModelLoadError::InvalidModel, "tensor '" + t.name + "': Bool data must be raw_data");
        *out = Tensor::from_raw(std::move(dims), ty, nullptr, 0);
        return true;
    }
    return false;
}

const AttributeP *find_attribute(const NodeP &n, const char *name) {
    for (const auto &a : n.attribute)
        if (a.name == name) return &a;
    return nullptr;
}

bool build_op(const NodeP &n, int64_t opset, Op *op, ModelLoadError *err) {
    if (!op_from_onnx_type(n.op_type, opset, op)) return fail(err, ModelLoadError::Todo, "Unsupported op: " + n.op_type);
    for (const std::string &req : required_onnx_attributes(*op, opset))
        if (!find_attribute(n, req.c_str())) return fail(err, ModelLoadError::NoAttribute, req);
    for (const auto &a : n.attribute) {
        // From opset 12 the reference no longer reads Squeeze.axes (load.rs:269-272).
        if (op->kind == OpKind::Squeeze && opset >= 12) continue;
        if (op->kind == OpKind::Constant && a.name == "value") {
            if (!a.has_t) return fail(err, ModelLoadError::Todo, "Constant.value must be specified for now");
            Tensor t;
            if (!tensor_of(a.t, &t, err)) return false;
            op->value = std::make_shared<Tensor>(std::move(t));
            continue;
        }
        if (op->kind == OpKind::Cast && a.name == "to") {
            if (!op->set_int("to", a.i))
                return fail(err, ModelLoadError::Todo,
                            std::string("Unsupported tensor element type: ") + data_type_name(int32_t(a.i)));
            continue;
        }
        // An attribute lands in the field of its kind; names this operator does not carry are
        // ignored, as the reference ignores attributes it never asks for.  The type tag decides
        // when present (a writer may leave out a zero-valued payload); otherwise the payload does.
        switch (a.type) {
        case 1: op->set_float(a.name, a.f); continue;    // FLOAT
        case 2: op->set_int(a.name, a.i); continue;      // INT
        case 3: op->set_string(a.name, a.s); continue;   // STRING
        case 7: op->set_ints(a.name, a.ints); continue;  // INTS
        default: break;
        }
        if (!a.ints.empty() && op->set_ints(a.name, a.ints)) continue;
        if (!a.s.empty() && op->set_string(a.name, a.s)) continue;
        if (a.has_i && op->set_int(a.name, a.i)) continue;
        if (a.has_f) op->set_float(a.name, a.f);
    }
    if (op->kind == OpKind::Constant && !op->value)
        return fail(err, ModelLoadError::Todo, "Constant.value must be specified for now");
    return true;
}

bool model_from_proto(const GraphP &g, const std::vector<OpsetP> &opsets, Model *model, ModelLoadError *err) {
    *model = Model();
    // load.rs:70-84
    bool have = false;
    for (const auto &o : opsets) {
        if (o.domain.empty() || o.domain == "ai.onnx") {
            if (have) return fail(err, ModelLoadError::DuplicateOpset);
            model->opset_version = o.version;
            have = true;
        } else {
            return fail(err, ModelLoadError::Todo, "Custom domain ('" + o.domain + "') not supported yet");
        }
    }
    if (!have) return fail(err, ModelLoadError::DuplicateOpset);  // the reference reports the same kind here

    std::unordered_map<std::string, ValueId> name_to_val;
    Graph &graph = model->graph;

    // Initializers (load.rs:86-96).
    for (const auto &init : g.initializer) {
        Tensor t;
        if (!tensor_of(init, &t, err)) return false;
        auto it = name_to_val.find(init.name);
        ValueId id;
        if (it == name_to_val.end()) {
            TypedShape ts{Dimensions::from_fixed(t.dims()), t.elem_ty()};
            id = graph.values.new_val_named_and_shaped(init.name, std::move(ts));
            name_to_val.emplace(init.name, id);
        } else {
            id = it->second;
        }
        graph.inits[id] = std::move(t);
    }

    // Inputs and outputs (load.rs:98-142).
    for (int which = 0; which < 2; which++) {
        const auto &infos = which == 0 ? g.input : g.output;
        auto &ids = which == 0 ? graph.inputs : graph.outputs;
        for (const auto &x : infos) {
            if (!x.has_type || (!x.has_tensor_type && !x.other_type)) return fail(err, ModelLoadError::NoValueType);
            if (!x.has_tensor_type) return fail(err, ModelLoadError::Todo, "Graph input must be tensor type");
            if (!x.has_shape) return fail(err, ModelLoadError::NoValueShape);
            std::vector<Dimension> dims;
            for (const auto &d : x.dims) {
                if (d.has_value) {
                    if (d.value < 0) return fail(err, ModelLoadError::InvalidModel, "negative dimension in '" + x.name + "'");
                    dims.push_back(Dimension::Fixed(size_t(d.value)));
                } else if (d.has_param) {
                    dims.push_back(Dimension::Dynamic(d.param));
                } else {
                    return fail(err, ModelLoadError::InvalidModel, "dimension of '" + x.name + "' has neither value nor name");
                }
            }
            auto it = name_to_val.find(x.name);
            ValueId id;
            if (it != name_to_val.end()) {
                id = it->second;
            } else {
                TensorElemType ty;
                if (!elem_type_of(x.elem_type, &ty))
                    return fail(err, ModelLoadError::Todo,
                                std::string("Unsupported tensor element type: ") + data_type_name(x.elem_type));
                id = graph.values.new_val_named_and_shaped(x.name, TypedShape{Dimensions(std::move(dims)), ty});
                name_to_val.emplace(x.name, id);
            }
            ids.push_back(id);
        }
    }

    // Initializers listed as inputs are not inputs (load.rs:144-148).
    std::vector<ValueId> kept;
    for (ValueId v : graph.inputs)
        if (!graph.inits.count(v)) kept.push_back(v);
    graph.inputs = std::move(kept);

    // Nodes (load.rs:150-369).
    auto value_of = [&](const std::string &name) {
        auto it = name_to_val.find(name);
        if (it != name_to_val.end()) return it->second;
        const ValueId id = graph.values.new_val_named(name);
        name_to_val.emplace(name, id);
        return id;
    };
    for (const auto &n : g.node) {
        Op op;
        if (!build_op(n, model->opset_version, &op, err)) return false;
        Node node(std::move(op));
        node.with_name(n.name);
        for (const auto &i : n.input) node.with_in(value_of(i));
        for (const auto &o : n.output) node.with_out(value_of(o));
        graph.add_node(std::move(node));
    }
    return true;
}

}  // namespace

bool load_onnx_from_buffer(const void *data, size_t bytes, Model *model, ModelLoadError *err) {
    if (!model || (!data && bytes)) return fail(err, ModelLoadError::InvalidModel, "null buffer");
    Reader r(Span{static_cast<const uint8_t *>(data), bytes});
    Field f;
    GraphP graph;
    bool has_graph = false;
    std::vector<OpsetP> opsets;
    while (!r.done()) {
        if (!r.next(&f)) return fail(err, ModelLoadError::InvalidModel, "truncated or malformed protobuf");
        if (f.number == 7 && f.wire == 2) {  // ModelProto.graph
            // A field that occurs twice is merged by protobuf; ONNX writers emit it once.
            if (!parse_graph(f.bytes, &graph)) return fail(err, ModelLoadError::InvalidModel, "malformed GraphProto");
            has_graph = true;
        } else if (f.number == 8 && f.wire == 2) {  // ModelProto.opset_import
            OpsetP o;
            Reader ro(f.bytes);
            Field g;
            while (!ro.done()) {
                if (!ro.next(&g)) return fail(err, ModelLoadError::InvalidModel, "malformed OperatorSetIdProto");
                if (g.number == 1) o.domain = g.bytes.str();
                else if (g.number == 2) o.version = int64_t(g.varint);
            }
            opsets.push_back(std::move(o));
        }
    }
    if (!has_graph) return fail(err, ModelLoadError::NoGraph);
    return model_from_proto(graph, opsets, model, err);
}

bool load_onnx(const std::string &path, Model *model, ModelLoadError *err) {
    FILE *fp = std::fopen(path.c_str(), "rb");
    if (!fp) return fail(err, ModelLoadError::Io, path + ": " + std::strerror(errno));
    std::vector<uint8_t> buf;
    uint8_t chunk[1 << 16];
    size_t got;
    while ((got = std::fread(chunk, 1, sizeof(chunk), fp)) > 0) buf.insert(buf.end(), chunk, chunk + got);
    const bool bad = std::ferror(fp);
    std::fclose(fp);
    if (bad) return fail(err, ModelLoadError::Io, path + ": read error");
    return load_onnx_from_buffer(buf.data(), buf.size(), model, err);
}

}  // namespace altius
