// Shape inference for the operators this backend executes.
// Mirrors altius_core::analysis::shape (crates/core/src/analysis/shape.rs): the
// binary arm (89-94), ReduceMax (354-386), ReduceMean (387-411), the element-wise
// arm (590-605), LayerNormalization (606-611) and Identity (34-37); infer_shapes
// (659-692) and infer_shape (694-719).  Where the reference panics (unwrap on an
// impossible broadcast, asserts) these functions return a ShapeError.
#pragma once

#include <map>
#include <string>
#include <utility>
#include <vector>

#include "model.h"

namespace altius {

struct ShapeError {
    std::string message;
};

using InferredShapes = std::map<NodeId, std::pair<Op, std::vector<TypedFixedShape>>>;

// Output shapes of `op` for the given inputs (only dims and element types of the
// inputs are read).  Returns false and fills *err on failure.
bool compute_output_shapes(const Model &model, Op &op, const std::vector<const Tensor *> &inputs,
                           size_t num_outputs, std::vector<TypedFixedShape> *out, ShapeError *err);

// Infers output shapes node by node in topological order, starting from the
// initializers and the graph inputs that carry a fixed shape.  Nodes whose
// inputs are not all known are skipped (they are inferred at run time).
bool infer_shapes(const Model &model, InferredShapes *shapes, std::map<ValueId, TypedFixedShape> *value_shapes,
                  ShapeError *err);

}  // namespace altius
