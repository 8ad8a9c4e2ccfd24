#include "fixed_dim.h"

#include <algorithm>

namespace altius {

FixedDimensions FixedDimensions::strides() const {
    std::vector<FixedDimension> s(d_.size());
    FixedDimension run = 1;
    for (size_t i = d_.size(); i-- > 0;) {
        s[i] = run;
        run *= d_[i];
    }
    return FixedDimensions(std::move(s));
}

std::optional<FixedDimensions> FixedDimensions::strides_for_broadcasting_to(const FixedDimensions &to) const {
    const size_t nf = d_.size(), nt = to.len();
    if (nt < nf) return std::nullopt;
    const FixedDimensions own = strides();
    std::vector<FixedDimension> out(nt, 0);  // axes this tensor lacks are broadcast
    for (size_t k = 0; k < nf; k++) {
        const size_t fi = nf - 1 - k, ti = nt - 1 - k;
        if (to[ti] == d_[fi])
            out[ti] = own[fi];  // also when both extents are 1: the real stride is kept
        else if (d_[fi] == 1)
            out[ti] = 0;
        else
            return std::nullopt;
    }
    return FixedDimensions(std::move(out));
}

std::optional<FixedDimensions> FixedDimensions::broadcast(const FixedDimensions &other) const {
    return altius::broadcast({this, &other});
}

std::string FixedDimensions::to_string() const {
    std::string s = "[";
    for (size_t i = 0; i < d_.size(); i++) {
        if (i) s += ", ";
        s += std::to_string(d_[i]);
    }
    return s + "]";
}

std::optional<FixedDimensions> broadcast(const std::vector<const FixedDimensions *> &shapes) {
    if (shapes.empty()) return std::nullopt;
    size_t rank = 0;
    for (auto *s : shapes) rank = std::max(rank, s->len());
    std::vector<FixedDimension> out(rank, 1);
    for (size_t k = 0; k < rank; k++) {  // k counts axes from the right
        FixedDimension extent = 1;
        for (auto *s : shapes) {
            if (k >= s->len()) continue;
            const FixedDimension d = (*s)[s->len() - 1 - k];
            if (d == 1) continue;
            if (extent != 1 && d != extent) return std::nullopt;
            extent = d;
        }
        out[rank - 1 - k] = extent;
    }
    return FixedDimensions(std::move(out));
}

}  // namespace altius
