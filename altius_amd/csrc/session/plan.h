// Execution plan: nodes in topological order, each with the values whose last
// reader it is.  Mirrors altius_session::plan (crates/session/src/plan.rs:6-58).
#pragma once

#include <vector>

#include "../core/model.h"

namespace altius {

struct NodeExecutionPlan {
    NodeId node_id;
    // Values produced by nodes that can be released once this node has run.
    // Graph outputs have no readers and are never listed.
    std::vector<ValueId> free_vals;
};

std::vector<NodeExecutionPlan> create_execution_plan(const Model &model);

}  // namespace altius
