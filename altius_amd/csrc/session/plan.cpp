#include "plan.h"

namespace altius {

std::vector<NodeExecutionPlan> create_execution_plan(const Model &model) {
    const std::vector<NodeId> order = model.topo_sort_nodes();
    std::map<NodeId, size_t> position;
    for (size_t i = 0; i < order.size(); i++) position[order[i]] = i;
    const auto users = model.get_value_users();

    // For every node output that somebody reads, the reader that runs last frees it.
    std::map<NodeId, std::vector<ValueId>> frees;
    for (NodeId id : order) {
        for (ValueId out : model.graph.nodes[id].outputs) {
            auto it = users.find(out);
            if (it == users.end()) continue;
            NodeId last = id;
            size_t last_pos = 0;
            bool found = false;
            for (NodeId u : it->second) {
                auto p = position.find(u);
                if (p == position.end()) continue;
                if (!found || p->second > last_pos) {
                    last = u;
                    last_pos = p->second;
                    found = true;
                }
            }
            if (found) frees[last].push_back(out);
        }
    }

    std::vector<NodeExecutionPlan> plan;
    plan.reserve(order.size());
    for (NodeId id : order) {
        NodeExecutionPlan p{id, {}};
        auto it = frees.find(id);
        if (it != frees.end()) p.free_vals = it->second;
        plan.push_back(std::move(p));
    }
    return plan;
}

}  // namespace altius
