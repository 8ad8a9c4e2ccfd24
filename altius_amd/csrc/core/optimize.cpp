#include "optimize.h"

#include "shape.h"

#include <algorithm>

namespace altius {

namespace {

using Users = std::map<ValueId, std::set<NodeId>>;

// The user of `value` whose operator is `kind`, if any.
std::optional<NodeId> user_of_kind(const Model &m, const Users &users, ValueId value, OpKind kind) {
    auto it = users.find(value);
    if (it == users.end()) return std::nullopt;
    for (NodeId id : it->second)
        if (m.graph.nodes[id].op.kind == kind) return id;
    return std::nullopt;
}

const Tensor *init_of(const Model &m, ValueId v) {
    auto it = m.graph.inits.find(v);
    return it == m.graph.inits.end() ? nullptr : &it->second;
}

// The initializer is f32, has at least one element and its first element equals `want`.
bool init_first_is(const Model &m, ValueId v, float want) {
    const Tensor *t = init_of(m, v);
    return t && t->elem_ty() == TensorElemType::F32 && t->nbytes() >= sizeof(float) && t->data_f32()[0] == want;
}

bool init_allclose(const Model &m, ValueId v, float want) {
    const Tensor *t = init_of(m, v);
    return t && t->allclose_f32({want});
}

// Points every reader of `from` (nodes and graph outputs) at `to`.
void replace_value(Model &m, const Users &users, ValueId from, ValueId to) {
    auto it = users.find(from);
    if (it != users.end())
        for (NodeId u : it->second)
            for (ValueId &in : m.graph.nodes[u].inputs)
                if (in == from) in = to;
    for (ValueId &out : m.graph.outputs)
        if (out == from) out = to;
}

// Matches are collected on the graph as it was, and rewritten one after the other in topological order: where one
// pattern starts at the value another one ends in (two chains back to back), the later one has to read what the
// earlier rewrite put in that value's place.
struct Renamed {
    std::map<ValueId, ValueId> to;
    ValueId operator()(ValueId v) const {
        auto it = to.find(v);
        return it == to.end() ? v : it->second;
    }
};

}  // namespace

size_t fuse_layer_norm(Model &model) {
    const auto users = model.get_value_users();
    struct Match {
        ValueId data, end, scale, bias;
        float epsilon;
    };
    std::vector<Match> matches;
    std::vector<NodeId> doomed;

    for (NodeId mean_id : model.topo_sort_nodes()) {
        const Node &mean = model.graph.nodes[mean_id];
        if (mean.op.kind != OpKind::ReduceMean || mean.outputs.empty() || mean.inputs.empty()) continue;
        static const OpKind chain[] = {OpKind::Sub,  OpKind::Pow, OpKind::ReduceMean, OpKind::Add,
                                       OpKind::Sqrt, OpKind::Div, OpKind::Mul,        OpKind::Add};
        std::vector<NodeId> ids{mean_id};
        ValueId cur = mean.outputs[0];
        bool ok = true;
        for (OpKind k : chain) {
            auto next = user_of_kind(model, users, cur, k);
            if (!next || model.graph.nodes[*next].outputs.empty()) {
                ok = false;
                break;
            }
            ids.push_back(*next);
            cur = model.graph.nodes[*next].outputs[0];
        }
        if (!ok) continue;
        const Node &add = model.graph.nodes[ids[4]];
        const Node &mul = model.graph.nodes[ids[7]];
        const Node &add2 = model.graph.nodes[ids[8]];
        if (add.inputs.size() < 2 || mul.inputs.size() < 2 || add2.inputs.size() < 2) continue;
        const Tensor *eps = init_of(model, add.inputs[1]);
        if (!eps || eps->elem_ty() != TensorElemType::F32 || eps->nbytes() < sizeof(float)) continue;
        matches.push_back({mean.inputs[0], add2.outputs[0], mul.inputs[1], add2.inputs[1], eps->data_f32()[0]});
        doomed.insert(doomed.end(), ids.begin(), ids.end());
    }

    Renamed now;
    for (const Match &m : matches) {
        const ValueId ln_out = model.graph.values.new_val();
        Node ln(Op::layer_normalization(-1, m.epsilon, 1));
        ln.with_in(now(m.data)).with_in(now(m.scale)).with_in(now(m.bias)).with_out(ln_out);
        model.graph.add_node(std::move(ln));
        replace_value(model, users, m.end, ln_out);
        now.to[m.end] = ln_out;
    }
    for (NodeId id : doomed) model.graph.nodes[id].deleted = true;
    model.remove_unnecessary_nodes();
    return matches.size();
}

size_t fuse_gelu(Model &model) {
    const auto users = model.get_value_users();
    struct Match {
        ValueId start, end;
    };
    std::vector<Match> matches;
    std::vector<NodeId> doomed;

    for (NodeId div_id : model.topo_sort_nodes()) {
        const Node &div = model.graph.nodes[div_id];
        if (div.op.kind != OpKind::Div || div.inputs.size() < 2 || div.outputs.empty()) continue;
        if (!init_allclose(model, div.inputs[1], 1.4142099618911743f)) continue;
        const ValueId x = div.inputs[0];

        auto erf_id = user_of_kind(model, users, div.outputs[0], OpKind::Erf);
        if (!erf_id) continue;
        const Node &erf = model.graph.nodes[*erf_id];

        auto add_id = user_of_kind(model, users, erf.outputs[0], OpKind::Add);
        if (!add_id) continue;
        const Node &add = model.graph.nodes[*add_id];
        if (add.inputs.size() < 2) continue;
        const ValueId add_other = add.inputs[0] == erf.outputs[0] ? add.inputs[1] : add.inputs[0];
        if (!init_first_is(model, add_other, 1.0f)) continue;

        auto mul1_id = user_of_kind(model, users, add.outputs[0], OpKind::Mul);
        if (!mul1_id) continue;
        const Node &mul1 = model.graph.nodes[*mul1_id];
        if (mul1.inputs.size() < 2) continue;
        const ValueId mul1_other = mul1.inputs[0] == add.outputs[0] ? mul1.inputs[1] : mul1.inputs[0];
        if (mul1_other != x) continue;

        auto mul2_id = user_of_kind(model, users, mul1.outputs[0], OpKind::Mul);
        if (!mul2_id) continue;
        const Node &mul2 = model.graph.nodes[*mul2_id];
        if (mul2.inputs.size() < 2) continue;
        const ValueId mul2_other = mul2.inputs[0] == mul1.outputs[0] ? mul2.inputs[1] : mul2.inputs[0];
        if (!init_first_is(model, mul2_other, 0.5f)) continue;

        matches.push_back({x, mul2.outputs[0]});
        for (NodeId id : {div_id, *erf_id, *add_id, *mul1_id, *mul2_id}) doomed.push_back(id);
    }

    Renamed now;
    for (const Match &m : matches) {
        const ValueId gelu_out = model.graph.values.new_val();
        Node gelu{Op(OpKind::Gelu)};
        gelu.with_in(now(m.start)).with_out(gelu_out);
        model.graph.add_node(std::move(gelu));
        replace_value(model, users, m.end, gelu_out);
        now.to[m.end] = gelu_out;
    }
    for (NodeId id : doomed) model.graph.nodes[id].deleted = true;
    model.remove_unnecessary_nodes();
    return matches.size();
}

size_t fuse_fast_gelu(Model &model) {
    const auto users = model.get_value_users();
    const auto parents = model.get_value_parents();
    struct Match {
        ValueId start, end;
    };
    std::vector<Match> matches;
    std::vector<NodeId> doomed;

    // The single user of `v`, required to have operator `kind`.
    auto sole_user = [&](ValueId v, OpKind kind) -> std::optional<NodeId> {
        auto it = users.find(v);
        if (it == users.end() || it->second.size() != 1) return std::nullopt;
        const NodeId id = *it->second.begin();
        if (model.graph.nodes[id].op.kind != kind) return std::nullopt;
        return id;
    };

    for (NodeId src_id : model.topo_sort_nodes()) {
        const Node &src = model.graph.nodes[src_id];
        if (src.outputs.size() != 1) continue;
        const ValueId x = src.outputs[0];

        auto pow_id = user_of_kind(model, users, x, OpKind::Pow);
        if (!pow_id) continue;
        const Node &pow = model.graph.nodes[*pow_id];
        if (pow.inputs.size() < 2 || !init_first_is(model, pow.inputs[1], 3.0f)) continue;

        auto mul1_id = sole_user(pow.outputs[0], OpKind::Mul);
        if (!mul1_id) continue;
        const Node &mul1 = model.graph.nodes[*mul1_id];
        if (mul1.inputs.size() < 2 || !init_allclose(model, mul1.inputs[1], 0.044714998453855515f)) continue;

        auto add1_id = sole_user(mul1.outputs[0], OpKind::Add);
        if (!add1_id) continue;
        const Node &add1 = model.graph.nodes[*add1_id];
        if (add1.inputs.empty() || add1.inputs[0] != x) continue;

        auto mul2_id = sole_user(add1.outputs[0], OpKind::Mul);
        if (!mul2_id) continue;
        const Node &mul2 = model.graph.nodes[*mul2_id];
        if (mul2.inputs.size() < 2 || !init_allclose(model, mul2.inputs[1], 0.7978845834732056f)) continue;

        auto tanh_id = sole_user(mul2.outputs[0], OpKind::Tanh);
        if (!tanh_id) continue;
        const Node &tanh = model.graph.nodes[*tanh_id];

        auto add2_id = sole_user(tanh.outputs[0], OpKind::Add);
        if (!add2_id) continue;
        const Node &add2 = model.graph.nodes[*add2_id];
        if (add2.inputs.size() < 2 || !init_first_is(model, add2.inputs[1], 1.0f)) continue;

        auto mul3_id = sole_user(add2.outputs[0], OpKind::Mul);
        if (!mul3_id) continue;
        const Node &mul3 = model.graph.nodes[*mul3_id];
        if (mul3.inputs.size() < 2 || mul3.inputs[1] != add2.outputs[0]) continue;

        auto mul4_parent = parents.find(mul3.inputs[0]);
        if (mul4_parent == parents.end()) continue;
        const NodeId mul4_id = mul4_parent->second;
        const Node &mul4 = model.graph.nodes[mul4_id];
        if (mul4.op.kind != OpKind::Mul || mul4.inputs.size() < 2 || mul4.inputs[0] != x) continue;
        if (!init_first_is(model, mul4.inputs[1], 0.5f)) continue;
        auto mul4_users = users.find(mul4.outputs[0]);
        if (mul4_users == users.end() || mul4_users->second.size() != 1) continue;

        matches.push_back({x, mul3.outputs[0]});
        for (NodeId id : {*pow_id, *mul1_id, *add1_id, *mul2_id, *tanh_id, *add2_id, *mul3_id, mul4_id})
            doomed.push_back(id);
    }

    Renamed now;
    for (const Match &m : matches) {
        const ValueId gelu_out = model.graph.values.new_val();
        Node gelu{Op(OpKind::Gelu)};
        gelu.with_in(now(m.start)).with_out(gelu_out);
        model.graph.add_node(std::move(gelu));
        replace_value(model, users, m.end, gelu_out);
        now.to[m.end] = gelu_out;
    }
    for (NodeId id : doomed) model.graph.nodes[id].deleted = true;
    model.remove_unnecessary_nodes();
    return matches.size();
}

size_t eliminate_identity(Model &model) {
    const auto users = model.get_value_users();
    size_t count = 0;
    for (NodeId id : model.topo_sort_nodes()) {
        Node &node = model.graph.nodes[id];
        if (node.op.kind != OpKind::Identity || node.inputs.size() != 1 || node.outputs.size() != 1) continue;
        const ValueId in = node.inputs[0], out = node.outputs[0];
        auto it = users.find(out);
        if (it == users.end()) continue;  // feeds a graph output (or nothing): kept
        for (NodeId u : it->second)
            for (ValueId &v : model.graph.nodes[u].inputs)
                if (v == out) v = in;
        node.deleted = true;
        count++;
    }
    model.remove_unnecessary_nodes();
    return count;
}

namespace {

bool extended_elemwise(const Op &op) {
    switch (op.kind) {
    case OpKind::Add: case OpKind::Sub: case OpKind::Mul: case OpKind::Div: case OpKind::Pow:
    case OpKind::Sqrt: case OpKind::ReLU: case OpKind::LeakyReLU: case OpKind::HardSigmoid:
    case OpKind::Erf: case OpKind::Gelu: case OpKind::Sigmoid: case OpKind::Tanh: case OpKind::Exp: case OpKind::Round:
        return true;
    default:
        return false;
    }
}

}  // namespace

bool fuse_elemwise_ops(Model &model, ElemwiseFusionRule rule, size_t *count, std::string *err) {
    if (count) *count = 0;
    const std::vector<NodeId> order = model.topo_sort_nodes();
    const auto users = model.get_value_users();
    const auto parents = model.get_value_parents();
    std::map<ValueId, TypedFixedShape> shapes;
    ShapeError serr;
    if (!infer_shapes(model, nullptr, &shapes, &serr)) {
        if (err) *err = serr.message;
        return false;
    }
    const auto &outs = model.graph.outputs;
    auto is_graph_output = [&](ValueId v) { return std::find(outs.begin(), outs.end(), v) != outs.end(); };
    auto shape_of = [&](ValueId v) -> const TypedFixedShape * {
        auto it = shapes.find(v);
        return it == shapes.end() ? nullptr : &it->second;
    };
    auto f32_known = [&](ValueId v) {
        const TypedFixedShape *s = shape_of(v);
        return s && s->elem_ty == TensorElemType::F32;
    };
    const bool extended = rule == ElemwiseFusionRule::ExtendedRule;
    constexpr size_t MAX_STEPS = 16, MAX_OPERANDS = 6;

    std::vector<std::vector<NodeId>> chains;
    std::set<NodeId> visited;
    for (NodeId start : order) {
        if (visited.count(start)) continue;
        std::vector<NodeId> chain;
        std::set<ValueId> operands;  // distinct values the chain reads from outside (extended rule's limit)
        std::optional<NodeId> last;
        NodeId cur = start;
        for (;;) {
            const Node &node = model.graph.nodes[cur];
            bool fusible = node.outputs.size() == 1 && !node.inputs.empty() && !visited.count(cur);
            std::set<ValueId> more = operands;
            if (fusible && !extended) {
                fusible = node.op.is_elemwise();
                for (ValueId in : node.inputs) {
                    if (!fusible) break;
                    auto p = parents.find(in);
                    fusible = p == parents.end() || !last || p->second == *last;
                }
                if (fusible && last) {
                    const Node &prev = model.graph.nodes[*last];
                    fusible = prev.inputs.size() == 2 && prev.outputs[0] == node.inputs[0];
                    if (fusible && node.inputs.size() == 2) {
                        const TypedFixedShape *a = shape_of(node.inputs[1]), *b = shape_of(prev.inputs[1]);
                        fusible = a && b && a->dims == b->dims && a->elem_ty == b->elem_ty;
                    } else if (fusible) {
                        fusible = node.inputs.size() == 1;
                    }
                }
            } else if (fusible) {
                fusible = extended_elemwise(node.op) && node.inputs.size() <= 2 && f32_known(node.outputs[0]) &&
                          chain.size() < MAX_STEPS;
                bool reads_prev = !last;
                for (ValueId in : node.inputs) {
                    if (!fusible) break;
                    if (last && in == model.graph.nodes[*last].outputs[0]) {
                        reads_prev = true;
                        continue;
                    }
                    fusible = f32_known(in);
                    more.insert(in);
                }
                fusible = fusible && reads_prev && more.size() <= MAX_OPERANDS;
            }
            if (!fusible) break;
            chain.push_back(cur);
            operands = std::move(more);
            last = cur;
            auto u = users.find(node.outputs[0]);
            if (u == users.end() || u->second.size() != 1 || is_graph_output(node.outputs[0])) break;
            cur = *u->second.begin();
        }
        if (chain.size() > 1) {
            visited.insert(chain.begin(), chain.end());
            chains.push_back(std::move(chain));
        }
    }

    for (const auto &chain : chains) {
        auto fused = std::make_shared<FusedElemwise>();
        std::optional<NodeId> prev;
        for (NodeId id : chain) {
            const Node &node = model.graph.nodes[id];
            for (ValueId in : node.inputs) {
                if (prev && model.graph.nodes[*prev].outputs[0] == in) continue;
                if (std::find(fused->input_map.begin(), fused->input_map.end(), in) == fused->input_map.end())
                    fused->input_map.push_back(in);
            }
            fused->chain.push_back({node.op, node.inputs, node.outputs});
            prev = id;
        }
        Op op(OpKind::FusedElemwise);
        const std::vector<ValueId> ins = fused->input_map;
        op.fused = std::move(fused);
        Node node(std::move(op));
        node.with_ins(ins).with_out(model.graph.nodes[chain.back()].outputs[0]);
        model.graph.add_node(std::move(node));
        for (NodeId id : chain) model.graph.nodes[id].deleted = true;
    }
    model.remove_unnecessary_nodes();
    if (count) *count = chains.size();
    return true;
}

size_t fuse_softmax_prologue(Model &model) {
    const auto users = model.get_value_users();
    const auto parents = model.get_value_parents();
    std::map<ValueId, TypedFixedShape> shapes;
    ShapeError serr;
    if (!infer_shapes(model, nullptr, &shapes, &serr)) return 0;
    const auto &outs = model.graph.outputs;
    auto single_use = [&](ValueId v) {
        auto u = users.find(v);
        return u != users.end() && u->second.size() == 1 && std::find(outs.begin(), outs.end(), v) == outs.end();
    };
    auto dims_of = [&](ValueId v) -> const FixedDimensions * {
        auto it = shapes.find(v);
        return it == shapes.end() || it->second.elem_ty != TensorElemType::F32 ? nullptr : &it->second.dims;
    };
    auto one_value_init = [&](ValueId v) {
        const Tensor *t = init_of(model, v);
        return t && t->elem_ty() == TensorElemType::F32 && t->dims().total_elems() == 1 && t->nbytes() == sizeof(float);
    };
    // Constant along every axis but the first and the last, and not growing x.
    auto mask_fits = [&](const FixedDimensions &m, const FixedDimensions &x) {
        if (x.len() < 1 || m.len() > x.len() || m.len() == 0) return false;
        const size_t off = x.len() - m.len();
        for (size_t i = 0; i < m.len(); i++) {
            const size_t xi = i + off;
            if (xi == x.len() - 1) {
                if (m[i] != x[xi]) return false;
            } else if (xi == 0) {
                if (m[i] != x[xi] && m[i] != 1) return false;
            } else if (m[i] != 1) {
                return false;
            }
        }
        return true;
    };

    size_t count = 0;
    std::vector<NodeId> doomed;
    for (NodeId sid : model.topo_sort_nodes()) {
        Node &sm = model.graph.nodes[sid];
        if (sm.op.kind != OpKind::Softmax || sm.inputs.size() != 1 || sm.op.prologue_scale || sm.op.prologue_mask) continue;
        const FixedDimensions *xd = dims_of(sm.inputs[0]);
        if (!xd || xd->len() == 0 || !(sm.op.axis == -1 || sm.op.axis == (int64_t)xd->len() - 1)) continue;

        ValueId x = sm.inputs[0];
        std::optional<ValueId> mask, scale;
        int scale_code = 0;
        std::vector<NodeId> absorbed;
        // the mask Add, directly in front of the Softmax
        auto p = parents.find(x);
        if (p != parents.end() && single_use(x)) {
            const Node &add = model.graph.nodes[p->second];
            if (add.op.kind == OpKind::Add && add.inputs.size() == 2 && add.outputs.size() == 1) {
                for (int side = 0; side < 2 && !mask; side++) {
                    const ValueId data = add.inputs[side], m = add.inputs[1 - side];
                    const FixedDimensions *dd = dims_of(data), *md = dims_of(m);
                    if (dd && md && *dd == *xd && mask_fits(*md, *xd)) {
                        mask = m;
                        x = data;
                        absorbed.push_back(p->second);
                    }
                }
            }
        }
        // the scale, in front of that
        p = parents.find(x);
        if (p != parents.end() && single_use(x)) {
            const Node &sc = model.graph.nodes[p->second];
            if ((sc.op.kind == OpKind::Mul || sc.op.kind == OpKind::Div) && sc.inputs.size() == 2 && sc.outputs.size() == 1) {
                const bool mul = sc.op.kind == OpKind::Mul;
                for (int side = 0; side < (mul ? 2 : 1) && !scale; side++) {  // x / c only; c * x or x * c
                    const ValueId data = sc.inputs[side], c = sc.inputs[1 - side];
                    const FixedDimensions *dd = dims_of(data);
                    if (dd && *dd == *xd && one_value_init(c)) {
                        scale = c;
                        scale_code = mul ? 1 : 2;
                        x = data;
                        absorbed.push_back(p->second);
                    }
                }
            }
        }
        if (!mask && !scale) continue;
        sm.inputs.assign(1, x);
        if (scale) sm.inputs.push_back(*scale);
        if (mask) sm.inputs.push_back(*mask);
        sm.op.prologue_scale = scale_code;
        sm.op.prologue_mask = mask.has_value();
        doomed.insert(doomed.end(), absorbed.begin(), absorbed.end());
        count++;
    }
    for (NodeId id : doomed) model.graph.nodes[id].deleted = true;
    if (count) model.remove_unnecessary_nodes();
    return count;
}

size_t fuse_matmul_bias(Model &model) {
    const auto users = model.get_value_users();
    std::map<ValueId, TypedFixedShape> shapes;
    ShapeError serr;
    if (!infer_shapes(model, nullptr, &shapes, &serr)) return 0;
    const auto &outs = model.graph.outputs;
    size_t count = 0;
    std::vector<NodeId> doomed;
    for (NodeId mid : model.topo_sort_nodes()) {
        Node &mm = model.graph.nodes[mid];
        if (mm.op.kind != OpKind::MatMul || mm.inputs.size() != 2 || mm.outputs.size() != 1) continue;
        const ValueId prod = mm.outputs[0];
        auto u = users.find(prod);
        if (u == users.end() || u->second.size() != 1 || std::find(outs.begin(), outs.end(), prod) != outs.end()) continue;
        const NodeId aid = *u->second.begin();
        const Node &add = model.graph.nodes[aid];
        if (add.op.kind != OpKind::Add || add.inputs.size() != 2 || add.outputs.size() != 1 || add.inputs[0] == add.inputs[1]) continue;
        const ValueId bias = add.inputs[0] == prod ? add.inputs[1] : add.inputs[0];
        auto ps = shapes.find(prod), bs = shapes.find(bias), os = shapes.find(add.outputs[0]);
        if (ps == shapes.end() || bs == shapes.end() || os == shapes.end()) continue;
        if (ps->second.elem_ty != TensorElemType::F32 || bs->second.elem_ty != TensorElemType::F32) continue;
        const FixedDimensions &pd = ps->second.dims, &bd = bs->second.dims;
        if (pd.len() < 2 || os->second.dims != pd || bd.len() == 0 || bd.len() > pd.len()) continue;
        // one value per column: the last extent equals N, every other extent is 1
        bool row_vector = bd[bd.len() - 1] == pd[pd.len() - 1];
        for (size_t i = 0; i + 1 < bd.len(); i++) row_vector = row_vector && bd[i] == 1;
        if (!row_vector) continue;
        mm.inputs.push_back(bias);
        mm.outputs[0] = add.outputs[0];
        doomed.push_back(aid);
        count++;
    }
    for (NodeId id : doomed) model.graph.nodes[id].deleted = true;
    if (count) model.remove_unnecessary_nodes();
    return count;
}

size_t fuse_transpose_matmul(Model &model) {
    const auto users = model.get_value_users();
    const auto parents = model.get_value_parents();
    const auto &outs = model.graph.outputs;
    auto swaps_last_two = [](const std::vector<int64_t> &perm) {
        const size_t r = perm.size();
        if (r < 2 || r > 4) return false;
        for (size_t i = 0; i + 2 < r; i++)
            if (perm[i] != (int64_t)i) return false;
        return perm[r - 2] == (int64_t)r - 1 && perm[r - 1] == (int64_t)r - 2;
    };
    size_t count = 0;
    std::set<NodeId> maybe_dead;
    for (NodeId mid : model.topo_sort_nodes()) {
        Node &mm = model.graph.nodes[mid];
        if (mm.op.kind != OpKind::MatMul || mm.inputs.size() < 2) continue;
        bool changed = false;
        for (int side = 0; side < 2; side++) {
            auto p = parents.find(mm.inputs[side]);
            if (p == parents.end()) continue;
            const Node &tr = model.graph.nodes[p->second];
            if (tr.op.kind != OpKind::Transpose || tr.inputs.size() != 1 || !swaps_last_two(tr.op.perm)) continue;
            bool &flag = side == 0 ? mm.op.trans_a : mm.op.trans_b;
            mm.inputs[side] = tr.inputs[0];
            flag = !flag;
            maybe_dead.insert(p->second);
            changed = true;
        }
        if (changed) count++;
    }
    // A folded Transpose goes away when nothing else reads it.
    if (count) {
        const auto now = model.get_value_users();
        for (NodeId id : maybe_dead) {
            const ValueId out = model.graph.nodes[id].outputs[0];
            auto u = now.find(out);
            const bool read = u != now.end() && !u->second.empty();
            if (!read && std::find(outs.begin(), outs.end(), out) == outs.end()) model.graph.nodes[id].deleted = true;
        }
        model.remove_unnecessary_nodes();
    }
    (void)users;
    return count;
}

}  // namespace altius
