// Graph IR: values, nodes, graph and model.
// Mirrors altius_core::{value, node, graph, model} (crates/core/src/value.rs,
// node.rs, graph.rs, model.rs:13-132).  Ids are indices into the arenas.
#pragma once

#include <map>
#include <optional>
#include <set>
#include <string>
#include <vector>

#include "op.h"
#include "tensor.h"

namespace altius {

using ValueId = size_t;
using NodeId = size_t;

struct Value {
    std::optional<std::string> name;
    std::optional<TypedShape> shape;
};

class ValueArena {
public:
    ValueId new_val() {
        v_.push_back(Value{});
        return v_.size() - 1;
    }
    ValueId new_val_named(std::string name) {
        v_.push_back(Value{std::move(name), std::nullopt});
        return v_.size() - 1;
    }
    ValueId new_val_named_and_shaped(std::string name, TypedShape shape) {
        v_.push_back(Value{std::move(name), std::move(shape)});
        return v_.size() - 1;
    }
    const Value &operator[](ValueId id) const { return v_.at(id); }
    Value &operator[](ValueId id) { return v_.at(id); }
    size_t size() const { return v_.size(); }

private:
    std::vector<Value> v_;
};

struct Node {
    Op op;
    std::optional<std::string> name;
    std::vector<ValueId> inputs;
    std::vector<ValueId> outputs;
    bool deleted = false;

    explicit Node(Op o) : op(std::move(o)) {}
    Node &with_name(std::string n) {
        name = std::move(n);
        return *this;
    }
    Node &with_in(ValueId id) {
        inputs.push_back(id);
        return *this;
    }
    Node &with_ins(const std::vector<ValueId> &ids) {
        inputs.insert(inputs.end(), ids.begin(), ids.end());
        return *this;
    }
    Node &with_out(ValueId id) {
        outputs.push_back(id);
        return *this;
    }
    Node &with_outs(const std::vector<ValueId> &ids) {
        outputs.insert(outputs.end(), ids.begin(), ids.end());
        return *this;
    }
};

struct Graph {
    std::vector<Node> nodes;  // arena; NodeId indexes it
    ValueArena values;
    std::map<ValueId, Tensor> inits;
    std::vector<ValueId> inputs;
    std::vector<ValueId> outputs;

    NodeId add_node(Node node) {
        nodes.push_back(std::move(node));
        return nodes.size() - 1;
    }
};

struct Model {
    Graph graph;
    int64_t opset_version = 0;

    std::optional<ValueId> lookup_named_value(const std::string &name) const;
    // value -> nodes reading it (model.rs:30-44); deleted nodes are skipped.
    std::map<ValueId, std::set<NodeId>> get_value_users() const;
    // value -> node producing it (model.rs:46-60).
    std::map<ValueId, NodeId> get_value_parents() const;
    // Kahn's algorithm over live nodes; graph inputs and initializers count as
    // available, as do inputs nobody produces (optional inputs) (model.rs:62-101).
    std::vector<NodeId> topo_sort_nodes() const;
    // Drops deleted nodes and renumbers the rest in topological order (model.rs:104-121).
    void remove_unnecessary_nodes();
};

}  // namespace altius
