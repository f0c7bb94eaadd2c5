#include "strided_shape.h"

namespace kn {

std::vector<int64_t> simple_strides(const std::vector<size_t> &shape) {
    std::vector<int64_t> r(shape.size());
    int64_t next = 1;
    for (size_t a = shape.size(); a-- > 0;) {
        r[a] = next;
        next *= (int64_t) shape[a];
    }
    return r;
}

static bool compute_dense(const std::vector<size_t> &shape, const std::vector<int64_t> &strides) {
    if (concrete_size(shape) == 0) return true;
    std::vector<std::pair<size_t, int64_t>> pairs;
    for (size_t a = 0; a < shape.size(); a++) pairs.push_back({shape[a], std::llabs(strides[a])});
    std::stable_sort(pairs.begin(), pairs.end(), [](auto &x, auto &y) { return x.second > y.second; });
    std::vector<size_t> ss;
    std::vector<int64_t> st;
    for (auto &p : pairs) {
        ss.push_back(p.first);
        st.push_back(p.second);
    }
    return simple_strides(ss) == st;
}

StridedShape::StridedShape(std::vector<size_t> shape, std::vector<int64_t> strides)
    : shape_(std::move(shape)), strides_(std::move(strides)) {
    if (shape_.size() != strides_.size()) fail("Shape and stride rank mismatch");
    simple_ = strides_ == simple_strides(shape_);
    dense_ = compute_dense(shape_, strides_);
    if (simple_) KN_ASSERT(dense_, "simple strides should imply dense strides");
}

StridedShape StridedShape::slice(size_t axis, SliceRange range) const {
    if (axis >= rank()) fail("Axis ", axis, " out of bounds for ", str());
    range.assert_in_bounds(shape_[axis]);
    auto ns = shape_;
    auto nst = strides_;
    ns[axis] = (range.end - range.start) / range.step;
    nst[axis] *= (int64_t) range.step;
    return StridedShape(ns, nst);
}

StridedShape StridedShape::flip(size_t axis) const {
    if (axis >= rank()) fail("Axis ", axis, " out of bounds for ", str());
    auto nst = strides_;
    nst[axis] *= -1;
    return StridedShape(shape_, nst);
}

StridedShape StridedShape::broadcast(const std::vector<size_t> &new_shape) const {
    if (rank() != new_shape.size()) fail("Can only broadcast to same rank, got ", str(), " and ", vec_str(new_shape));
    std::vector<int64_t> nst(rank());
    for (size_t i = 0; i < rank(); i++) {
        if (new_shape[i] == shape_[i]) nst[i] = strides_[i];
        else {
            if (shape_[i] != 1) fail("Broadcast mismatch between ", str(), " and ", vec_str(new_shape), " at axis ", i);
            nst[i] = 0;
        }
    }
    return StridedShape(new_shape, nst);
}

std::vector<std::pair<size_t, int64_t>> StridedShape::continuous_groups() const {
    std::vector<std::pair<size_t, int64_t>> groups;
    if (size() == 0 || rank() == 0) {
        groups.push_back({0, 1});
        return groups;
    }
    size_t group_size = 1;
    bool have_prev = false;
    int64_t prev_stride = 0;
    for (size_t a = 0; a < rank(); a++) {
        if (have_prev && prev_stride != (int64_t) shape_[a] * strides_[a]) {
            groups.push_back({group_size, prev_stride});
            group_size = 1;
        }
        group_size *= shape_[a];
        prev_stride = strides_[a];
        have_prev = true;
    }
    groups.push_back({group_size, prev_stride});
    return groups;
}

std::optional<StridedShape> StridedShape::view(const std::vector<size_t> &new_shape) const {
    if (size() != concrete_size(new_shape))
        fail("Size cannot change during view, cannot go from ", str(), " to ", vec_str(new_shape));
    if (size() == 0 || rank() == 0) return StridedShape::simple(new_shape);

    std::vector<int64_t> nst(new_shape.size(), 0);
    size_t next_d = 0;
    for (auto &[group_size, group_stride] : continuous_groups()) {
        size_t left = group_size;
        while (left > 1) {
            if (next_d < new_shape.size() && new_shape[next_d] != 0 && left % new_shape[next_d] == 0) {
                left /= new_shape[next_d];
                nst[next_d] = (int64_t) left * group_stride;
                next_d++;
            } else {
                return std::nullopt;
            }
        }
    }
    for (size_t d = next_d; d < new_shape.size(); d++) {
        KN_ASSERT(new_shape[d] == 1);
        nst[d] = 1;
    }
    return StridedShape(new_shape, nst);
}

StridedShape StridedShape::permute(const std::vector<size_t> &permutation) const {
    KN_ASSERT(permutation.size() == rank());
    std::vector<size_t> ns;
    std::vector<int64_t> nst;
    for (size_t i : permutation) {
        KN_ASSERT(i < rank());
        ns.push_back(shape_[i]);
        nst.push_back(strides_[i]);
    }
    return StridedShape(ns, nst);
}

StridedShape StridedShape::repeat_unary(size_t axis, size_t count) const {
    KN_ASSERT(axis < rank() && shape_[axis] == 1);
    auto ns = shape_;
    auto nst = strides_;
    ns[axis] = count;
    nst[axis] = 0;
    return StridedShape(ns, nst);
}

StridedShape StridedShape::remove(size_t axis) const {
    if (axis >= rank()) fail("Axis ", axis, " out of bounds for ", str());
    auto ns = shape_;
    auto nst = strides_;
    ns.erase(ns.begin() + axis);
    nst.erase(nst.begin() + axis);
    return StridedShape(ns, nst);
}

std::pair<int64_t, int64_t> StridedShape::offset_bounds() const {
    int64_t lo = 0, hi = 0;
    if (size() == 0) return {0, 0};
    for (size_t a = 0; a < rank(); a++) {
        int64_t span = (int64_t) (shape_[a] - 1) * strides_[a];
        if (span < 0) lo += span;
        else hi += span;
    }
    return {lo, hi};
}

std::string StridedShape::str() const {
    return "StridedShape { shape: " + vec_str(shape_) + ", strides: " + vec_str(strides_) + " }";
}

}  // namespace kn
