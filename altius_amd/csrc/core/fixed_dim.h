// Fixed tensor dimensions and NumPy-style broadcasting index math.
// Mirrors altius_core::fixed_dim (crates/core/src/fixed_dim.rs) and
// altius_core::dim (crates/core/src/dim.rs).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <initializer_list>
#include <optional>
#include <string>
#include <vector>

namespace altius {

using FixedDimension = size_t;

class FixedDimensions {
public:
    FixedDimensions() = default;
    FixedDimensions(std::vector<FixedDimension> d) : d_(std::move(d)) {}
    FixedDimensions(std::initializer_list<FixedDimension> d) : d_(d) {}

    static FixedDimensions from_i64(const int64_t *dims, size_t n) {
        std::vector<FixedDimension> v(n);
        for (size_t i = 0; i < n; i++) v[i] = (FixedDimension)dims[i];
        return FixedDimensions(std::move(v));
    }

    size_t len() const { return d_.size(); }
    bool is_empty() const { return d_.empty(); }
    // Rank 0, or rank 1 with extent 0 or 1 (fixed_dim.rs:26-28).
    bool is_scalar() const { return d_.empty() || (d_.size() == 1 && (d_[0] == 0 || d_[0] == 1)); }
    // The product of the extents.  A product that does not fit comes back as SATURATED instead of wrapped: no tensor
    // is that large, so every allocation sized from it fails cleanly (times an element size it still does not wrap).
    static constexpr size_t SATURATED = ~size_t(0) / 16;
    size_t total_elems() const {
        size_t n = 1;
        for (auto x : d_)
            if (x == 0) return 0;
        for (auto x : d_) {
            if (n > SATURATED / x) return SATURATED;
            n *= x;
        }
        return n;
    }
    const std::vector<FixedDimension> &as_vec() const { return d_; }
    std::vector<FixedDimension> &as_vec_mut() { return d_; }
    FixedDimension operator[](size_t i) const { return d_[i]; }
    FixedDimension &operator[](size_t i) { return d_[i]; }
    bool operator==(const FixedDimensions &o) const { return d_ == o.d_; }
    bool operator!=(const FixedDimensions &o) const { return d_ != o.d_; }

    // Row-major strides in elements: stride[i] = product of dims[i+1..].
    FixedDimensions strides() const;

    // Strides with which a dense tensor of this shape is read when broadcast to
    // `to` (right-aligned): the tensor's own stride where the extents agree, 0
    // where this extent is 1 or the axis is missing; nullopt if incompatible
    // (fixed_dim.rs:64-101, tensor.rs:369-406).
    std::optional<FixedDimensions> strides_for_broadcasting_to(const FixedDimensions &to) const;

    std::optional<FixedDimensions> broadcast(const FixedDimensions &other) const;

    std::string to_string() const;

private:
    std::vector<FixedDimension> d_;
};

// Broadcast shape of any number of shapes (fixed_dim.rs:112-136).
std::optional<FixedDimensions> broadcast(const std::vector<const FixedDimensions *> &shapes);

// A dimension that may be symbolic (dim.rs:9-13).
struct Dimension {
    bool fixed = true;
    FixedDimension value = 0;
    std::string name;  // when !fixed

    static Dimension Fixed(FixedDimension v) { return Dimension{true, v, {}}; }
    static Dimension Dynamic(std::string n) { return Dimension{false, 0, std::move(n)}; }
    bool operator==(const Dimension &o) const {
        return fixed == o.fixed && (fixed ? value == o.value : name == o.name);
    }
};

class Dimensions {
public:
    Dimensions() = default;
    explicit Dimensions(std::vector<Dimension> d) : d_(std::move(d)) {}
    static Dimensions from_fixed(const FixedDimensions &f) {
        std::vector<Dimension> v;
        for (auto x : f.as_vec()) v.push_back(Dimension::Fixed(x));
        return Dimensions(std::move(v));
    }
    bool is_fixed() const {
        for (auto &x : d_)
            if (!x.fixed) return false;
        return true;
    }
    bool is_dynamic() const { return !is_fixed(); }
    std::optional<FixedDimensions> as_fixed_dims() const {
        if (is_dynamic()) return std::nullopt;
        std::vector<FixedDimension> v;
        for (auto &x : d_) v.push_back(x.value);
        return FixedDimensions(std::move(v));
    }
    const std::vector<Dimension> &as_vec() const { return d_; }

private:
    std::vector<Dimension> d_;
};

}  // namespace altius
