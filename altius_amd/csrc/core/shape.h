// Shape inference.
// Mirrors altius_core::analysis::shape (crates/core/src/analysis/shape.rs:21-657): every
// arm of compute_output_shapes, plus infer_shapes (659-692) and infer_shape (694-719).
// Where the reference panics (unwrap on an impossible broadcast, asserts) these functions
// return a ShapeError.
#pragma once

#include <map>
#include <string>
#include <utility>
#include <vector>

#include "model.h"

namespace altius {

struct ShapeError {
    std::string message;
    // The shape depends on the CONTENTS of an input (Reshape's shape, Slice's bounds, ...) that
    // is not available: static inference skips such a node, the session infers it at run time.
    bool needs_data = false;
};

using InferredShapes = std::map<NodeId, std::pair<Op, std::vector<TypedFixedShape>>>;

// Output shapes of `op` for the given inputs.  Dims and element types are always read; the
// contents only of the integer / scale operands that decide a shape.  `op` may be rewritten
// (Conv2d / MaxPool paddings are normalised to four entries, shape.rs:38-72).  Returns false
// and fills *err on failure.
bool compute_output_shapes(const Model &model, Op &op, const std::vector<const Tensor *> &inputs,
                           size_t num_outputs, std::vector<TypedFixedShape> *out, ShapeError *err);

// Infers output shapes node by node in topological order, starting from the
// initializers and the graph inputs that carry a fixed shape.  Nodes whose
// inputs are not all known are skipped (they are inferred at run time).
bool infer_shapes(const Model &model, InferredShapes *shapes, std::map<ValueId, TypedFixedShape> *value_shapes,
                  ShapeError *err);

}  // namespace altius
