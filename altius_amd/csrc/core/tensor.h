// Host tensor: dense, row-major, typed bytes behind a shared pointer.
// Mirrors altius_core::tensor (crates/core/src/tensor.rs:15-21, 47-76).
#pragma once

#include <cstdlib>
#include <cstring>
#include <memory>
#include <optional>
#include <vector>

#include "fixed_dim.h"

namespace altius {

enum class TensorElemType : int { Bool = 0, F32 = 1, I32 = 2, I64 = 3 };

inline size_t elem_size(TensorElemType t) {
    switch (t) {
    case TensorElemType::Bool: return 1;
    case TensorElemType::F32: return 4;
    case TensorElemType::I32: return 4;
    case TensorElemType::I64: return 8;
    }
    return 0;
}

inline const char *elem_name(TensorElemType t) {
    switch (t) {
    case TensorElemType::Bool: return "Bool";
    case TensorElemType::F32: return "F32";
    case TensorElemType::I32: return "I32";
    case TensorElemType::I64: return "I64";
    }
    return "?";
}

// Type and fixed shape of a tensor (tensor.rs:23-28).
struct TypedFixedShape {
    FixedDimensions dims;
    TensorElemType elem_ty = TensorElemType::F32;
};

// Type and possibly symbolic shape of a graph value (tensor.rs:30-35).
struct TypedShape {
    Dimensions dims;
    TensorElemType elem_ty = TensorElemType::F32;
};

// Host storage of a tensor: a byte block that knows how to give itself back.  Blocks come from
// malloc unless the creator of the tensor names another allocator: the session and the C ABI
// place the tensors that cross PCIe in pinned (page-locked) memory so that uploads and downloads
// are plain DMA transfers.
struct HostBlock {
    uint8_t *ptr = nullptr;
    size_t size = 0;
    void (*release)(uint8_t *ptr, size_t size, void *user) = nullptr;
    void *user = nullptr;

    HostBlock() = default;
    HostBlock(const HostBlock &) = delete;
    HostBlock &operator=(const HostBlock &) = delete;
    ~HostBlock() {
        if (ptr && release) release(ptr, size, user);
    }
};

// Returns an uninitialised block of `bytes` bytes, or nullptr when memory is exhausted.
using HostAllocator = std::shared_ptr<HostBlock> (*)(size_t bytes);

std::shared_ptr<HostBlock> malloc_host_block(size_t bytes);  // plain malloc; the default allocator
// `preferred` if it is given and succeeds, else malloc.
std::shared_ptr<HostBlock> allocate_host_block(size_t bytes, HostAllocator preferred);

class Tensor {
public:
    Tensor() : data_(std::make_shared<HostBlock>()) {}

    // Copies `bytes` (elem_size * total_elems) from `data`.
    static Tensor from_raw(FixedDimensions dims, TensorElemType ty, const void *data, size_t bytes,
                           HostAllocator alloc = nullptr) {
        Tensor t;
        t.stride_ = dims.strides();
        t.dims_ = std::move(dims);
        t.elem_ty_ = ty;
        t.data_ = allocate_host_block(bytes, alloc);
        if (!t.data_) {  // out of memory: a tensor without data (has_data() is false)
            t.data_ = std::make_shared<HostBlock>();
            return t;
        }
        if (bytes && data) std::memcpy(t.data_->ptr, data, bytes);
        return t;
    }
    static Tensor from_f32(FixedDimensions dims, const std::vector<float> &v) {
        return from_raw(std::move(dims), TensorElemType::F32, v.data(), v.size() * sizeof(float));
    }
    static Tensor zeros_of_type(TensorElemType ty, FixedDimensions dims, HostAllocator alloc = nullptr) {
        Tensor t = uninit_of_type(ty, std::move(dims), alloc);
        if (t.data_->size) std::memset(t.data_->ptr, 0, t.data_->size);
        return t;
    }
    // Shape and type without storage: what shape inference passes around (tensor.rs:96-103).
    static Tensor empty_of_type(TensorElemType ty, FixedDimensions dims) {
        Tensor t;
        t.stride_ = dims.strides();
        t.dims_ = std::move(dims);
        t.elem_ty_ = ty;
        return t;
    }
    // Storage of the right size, contents unspecified (tensor.rs:116-132).
    static Tensor uninit_of_type(TensorElemType ty, FixedDimensions dims, HostAllocator alloc = nullptr) {
        const size_t bytes = dims.total_elems() * elem_size(ty);
        return from_raw(std::move(dims), ty, nullptr, bytes, alloc);
    }

    // The same bytes under another shape of as many elements (Tensor::copy_data_from shares the
    // buffer in the reference too, tensor.rs:340-342); an empty tensor if the counts differ.
    Tensor reshaped(FixedDimensions dims) const {
        Tensor t;
        if (dims.total_elems() != dims_.total_elems()) return t;
        t.stride_ = dims.strides();
        t.dims_ = std::move(dims);
        t.elem_ty_ = elem_ty_;
        t.data_ = data_;
        return t;
    }

    const FixedDimensions &dims() const { return dims_; }
    const FixedDimensions &strides() const { return stride_; }
    TensorElemType elem_ty() const { return elem_ty_; }
    size_t nbytes() const { return data_->size; }
    const uint8_t *data_as_bytes() const { return data_->ptr; }
    uint8_t *data_as_bytes_mut() { return data_->ptr; }
    bool has_data() const { return data_->size == dims_.total_elems() * elem_size(elem_ty_); }

    // Typed view; nullptr when the element type does not match.
    const float *data_f32() const {
        return elem_ty_ == TensorElemType::F32 ? reinterpret_cast<const float *>(data_->ptr) : nullptr;
    }

    // Tensor::allclose for f32 (tensor.rs:350-362, 517-522): |a-b| <= 1e-5 + 1e-8*|b|.
    bool allclose_f32(const std::vector<float> &other) const;

    // Strides for reading this tensor broadcast to `dims` (tensor.rs:369-406).
    std::optional<FixedDimensions> strides_for_broadcasting(const FixedDimensions &dims) const {
        return dims_.strides_for_broadcasting_to(dims);
    }

private:
    FixedDimensions dims_;
    FixedDimensions stride_;
    std::shared_ptr<HostBlock> data_;
    TensorElemType elem_ty_ = TensorElemType::F32;
};

}  // namespace altius
