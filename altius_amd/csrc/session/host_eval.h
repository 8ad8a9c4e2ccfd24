// Shape arithmetic on the host.
//
// Exported transformer graphs compute reshape targets with small integer subgraphs
// (Shape -> Gather -> Unsqueeze -> Concat -> Reshape, Slice bounds, Range ...).  Those tensors hold
// a handful of int64 values that the host needs anyway to size the next device buffer, so the
// session evaluates them here instead of launching kernels and reading the result back.  Only
// integer and bool tensors (and casts out of them) go this way; every float tensor of the model
// is computed on the device.
#pragma once

#include <string>
#include <vector>

#include "../core/model.h"

namespace altius {

// True if `op` is one of the operators evaluate_on_host implements.
bool host_evaluable(const Op &op);

// Computes the outputs of `op` from host tensors.  `inputs[i]` may be nullptr for an omitted
// optional input.  `shapes` are the inferred output shapes.  Returns false with a message for
// anything outside the supported integer cases.
bool evaluate_on_host(const Model &model, const Op &op, const std::vector<const Tensor *> &inputs,
                      const std::vector<TypedFixedShape> &shapes, std::vector<Tensor> *outputs, std::string *error);

}  // namespace altius
