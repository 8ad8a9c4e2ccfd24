#include "model.h"

#include <algorithm>
#include <cmath>

namespace altius {

const char *op_kind_name(OpKind k) {
    static const char *names[] = {
        "Identity", "Conv2d", "Add", "Sub", "Mul", "Div", "Pow", "Greater", "Sqrt", "ReLU", "Gelu", "LeakyReLU",
        "Sigmoid", "Erf", "Tanh", "Clip", "Where", "Softmax", "Cast", "MaxPool", "GlobalAveragePool", "Reshape",
        "Flatten", "Resize", "Concat", "Transpose", "Squeeze", "Unsqueeze", "ReduceMin", "ReduceMax",
        "ReduceMean", "Round", "Exp", "Expand", "Range", "Loop", "Tile", "Split", "Slice", "Gather", "Shape",
        "NonMaxSuppression", "MatMul", "Gemm", "BatchNormalization", "LayerNormalization", "HardSigmoid",
        "Constant", "FusedElemwise"};
    const int i = static_cast<int>(k);
    if (i < 0 || i >= static_cast<int>(OpKind::Count)) return "?";
    return names[i];
}

bool Tensor::allclose_f32(const std::vector<float> &other) const {
    if (elem_ty_ != TensorElemType::F32) return false;
    const size_t n = data_->size / sizeof(float);
    if (n != other.size()) return false;
    const float *x = data_f32();
    for (size_t i = 0; i < n; i++) {
        const float a = x[i], b = other[i];
        const float atol = 1e-5f, rtol = 1e-8f;
        const bool close = std::abs(a - b) <= atol + rtol * std::abs(b);
        const bool same_inf = std::isinf(a) && std::isinf(b) && (std::signbit(a) == std::signbit(b));
        if (!close && !same_inf) return false;
    }
    return true;
}

std::optional<ValueId> Model::lookup_named_value(const std::string &name) const {
    for (ValueId id = 0; id < graph.values.size(); id++) {
        const auto &v = graph.values[id];
        if (v.name && *v.name == name) return id;
    }
    return std::nullopt;
}

std::map<ValueId, std::set<NodeId>> Model::get_value_users() const {
    std::map<ValueId, std::set<NodeId>> users;
    for (NodeId id = 0; id < graph.nodes.size(); id++) {
        const Node &n = graph.nodes[id];
        if (n.deleted) continue;
        for (ValueId in : n.inputs) users[in].insert(id);
    }
    return users;
}

std::map<ValueId, NodeId> Model::get_value_parents() const {
    std::map<ValueId, NodeId> parents;
    for (NodeId id = 0; id < graph.nodes.size(); id++) {
        const Node &n = graph.nodes[id];
        if (n.deleted) continue;
        for (ValueId out : n.outputs) parents[out] = id;
    }
    return parents;
}

std::vector<NodeId> Model::topo_sort_nodes() const {
    const auto users = get_value_users();
    const auto parents = get_value_parents();
    std::set<ValueId> available(graph.inputs.begin(), graph.inputs.end());
    for (const auto &kv : graph.inits) available.insert(kv.first);

    std::map<NodeId, size_t> pending;  // number of distinct inputs still to be produced
    std::vector<NodeId> ready;
    for (NodeId id = 0; id < graph.nodes.size(); id++) {
        const Node &n = graph.nodes[id];
        if (n.deleted) continue;
        std::set<ValueId> need;
        for (ValueId in : n.inputs)
            if (!available.count(in) && parents.count(in)) need.insert(in);
        pending[id] = need.size();
        if (need.empty()) ready.push_back(id);
    }
    // Deterministic order: lowest node id first among the ready ones.
    std::sort(ready.begin(), ready.end(), std::greater<NodeId>());

    std::vector<NodeId> order;
    while (!ready.empty()) {
        const NodeId id = ready.back();
        ready.pop_back();
        order.push_back(id);
        std::vector<NodeId> released;
        for (ValueId out : graph.nodes[id].outputs) {
            auto it = users.find(out);
            if (it == users.end()) continue;
            for (NodeId u : it->second) {
                auto p = pending.find(u);
                if (p == pending.end() || p->second == 0) continue;
                if (--p->second == 0) released.push_back(u);
            }
        }
        std::sort(released.begin(), released.end(), std::greater<NodeId>());
        ready.insert(ready.end(), released.begin(), released.end());
    }
    return order;
}

void Model::remove_unnecessary_nodes() {
    const std::vector<NodeId> order = topo_sort_nodes();
    std::vector<Node> kept;
    kept.reserve(order.size());
    for (NodeId id : order) kept.push_back(std::move(graph.nodes[id]));
    graph.nodes = std::move(kept);
}

}  // namespace altius
