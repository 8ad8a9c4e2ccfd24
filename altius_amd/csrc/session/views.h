// Helpers shared by the session's node loop (hip_session.cpp) and its copy-avoidance code (views.cpp):
// error helpers, which operators alias or read strided views, and stride arithmetic on shapes.
#pragma once

#include <cstdint>
#include <vector>

#include "hip_session.h"

#include <string>

namespace altius {
namespace detail {

inline bool fail(SessionError *err, SessionError::Kind kind, std::string msg) {
    if (err) {
        err->kind = kind;
        err->message = std::move(msg);
    }
    return false;
}

// Turns an AHIP_ERR_* code from the device layer into a SessionError.
inline bool fail_code(SessionError *err, int code, const std::string &msg) {
    SessionError::Kind k = SessionError::Hip;
    if (code == AHIP_ERR_OOM) k = SessionError::OutOfMemory;
    else if (code == AHIP_ERR_UNSUPPORTED) k = SessionError::Message;
    else if (code == AHIP_ERR_SHAPE) k = SessionError::Shape;
    else if (code == AHIP_ERR_ARG) k = SessionError::Argument;
    return fail(err, k, msg);
}

inline bool is_alias_op(OpKind k) {
    return k == OpKind::Reshape || k == OpKind::Flatten || k == OpKind::Squeeze || k == OpKind::Unsqueeze;
}

// Operators that read a strided view in place (or pass it on as another view).
inline bool reads_views(OpKind k) { return is_alias_op(k) || k == OpKind::MatMul || k == OpKind::Transpose || k == OpKind::Split; }

inline std::vector<int64_t> dense_strides(const FixedDimensions &dims) {
    std::vector<int64_t> s(dims.len());
    int64_t acc = 1;
    for (size_t i = dims.len(); i-- > 0;) {
        s[i] = acc;
        acc *= (int64_t)dims[i];
    }
    return s;
}

inline std::vector<int64_t> strides_of(const DeviceTensor &t) { return t.strides.empty() ? dense_strides(t.dims) : t.strides; }

// Axes of extent 1 may carry any stride.
inline bool is_dense(const FixedDimensions &dims, const std::vector<int64_t> &strides) {
    const std::vector<int64_t> d = dense_strides(dims);
    for (size_t i = 0; i < dims.len(); i++)
        if (dims[i] != 1 && strides[i] != d[i]) return false;
    return true;
}

// Strides of the same elements under new_dims, if they exist without a copy (each run of new axes
// must tile a run of old axes that is itself uniformly strided).
inline bool reshape_strides(const FixedDimensions &old_dims, const std::vector<int64_t> &old_strides, const FixedDimensions &new_dims,
                     std::vector<int64_t> *out) {
    std::vector<size_t> od;
    std::vector<int64_t> os;
    for (size_t i = 0; i < old_dims.len(); i++)
        if (old_dims[i] != 1) od.push_back(old_dims[i]), os.push_back(old_strides[i]);
    out->assign(new_dims.len(), 0);
    size_t oi = 0, ni = 0;
    while (ni < new_dims.len() && oi < od.size()) {
        if (new_dims[ni] == 1) {
            (*out)[ni++] = 1;
            continue;
        }
        size_t np = new_dims[ni], op = od[oi], nj = ni + 1, oj = oi + 1;
        while (np != op) {
            if (np < op) {
                if (nj >= new_dims.len()) return false;
                np *= new_dims[nj++];
            } else {
                if (oj >= od.size()) return false;
                op *= od[oj++];
            }
        }
        for (size_t q = oi; q + 1 < oj; q++)
            if (os[q] != (int64_t)od[q + 1] * os[q + 1]) return false;
        int64_t st = os[oj - 1];
        for (size_t q = nj; q-- > ni;) {
            (*out)[q] = st;
            st *= (int64_t)new_dims[q];
        }
        ni = nj;
        oi = oj;
    }
    for (; ni < new_dims.len(); ni++) {
        if (new_dims[ni] != 1) return false;
        (*out)[ni] = 1;
    }
    return oi == od.size();
}

// [outer, axis, inner] view of `dims` around `axis`.
inline void split_at(const FixedDimensions &dims, size_t axis, size_t *outer, size_t *len, size_t *inner) {
    *outer = *inner = 1;
    for (size_t i = 0; i < axis; i++) *outer *= dims[i];
    *len = dims[axis];
    for (size_t i = axis + 1; i < dims.len(); i++) *inner *= dims[i];
}


}  // namespace detail
}  // namespace altius
