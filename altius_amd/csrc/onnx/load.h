// ONNX model files -> Model (crates/core/src/onnx/load.rs:55-372), read with a small
// protobuf wire-format decoder written against the field numbers of onnx.proto.
#pragma once

#include <string>

#include "../core/model.h"

namespace altius {

// Mirrors ModelLoadError (load.rs:25-53).
struct ModelLoadError {
    enum Kind { Io, NoGraph, InvalidModel, DuplicateOpset, NoValueType, NoValueShape, NoAttribute, Todo };
    Kind kind = Todo;
    std::string message;
    std::string to_string() const;
};

bool load_onnx(const std::string &path, Model *model, ModelLoadError *err);
bool load_onnx_from_buffer(const void *data, size_t bytes, Model *model, ModelLoadError *err);

}  // namespace altius
