// Shape + element strides, and the zero-copy layout algebra on top of it.
// Mirrors kn-cuda-eval/src/shape.rs:25-285 (StridedShape) and kn-cuda-eval/src/offset_tensor.rs:52-114 (views of a
// pointer). Strides are in elements and may be zero (broadcast) or negative (flip).
#pragma once

#include <algorithm>

#include "graph.h"

namespace kn {

std::vector<int64_t> simple_strides(const std::vector<size_t> &shape);

class StridedShape {
public:
    StridedShape() : simple_(true), dense_(true) {}
    StridedShape(std::vector<size_t> shape, std::vector<int64_t> strides);
    static StridedShape simple(std::vector<size_t> shape) {
        auto st = simple_strides(shape);
        return StridedShape(std::move(shape), std::move(st));
    }

    const std::vector<size_t> &shape() const { return shape_; }
    const std::vector<int64_t> &strides() const { return strides_; }
    size_t rank() const { return shape_.size(); }
    size_t size() const { return concrete_size(shape_); }
    // row-major contiguous
    bool has_simple_strides() const { return simple_; }
    // covers every element of its span exactly once, in some axis order and direction
    bool has_dense_strides() const { return dense_; }
    bool operator==(const StridedShape &o) const { return shape_ == o.shape_ && strides_ == o.strides_; }
    bool operator!=(const StridedShape &o) const { return !(*this == o); }

    StridedShape slice(size_t axis, SliceRange range) const;
    StridedShape flip(size_t axis) const;
    StridedShape broadcast(const std::vector<size_t> &new_shape) const;
    // shape.rs:135-189: succeeds iff every contiguous group of axes splits evenly into the new dims
    std::optional<StridedShape> view(const std::vector<size_t> &new_shape) const;
    StridedShape permute(const std::vector<size_t> &permutation) const;
    StridedShape repeat_unary(size_t axis, size_t count) const;
    StridedShape remove(size_t axis) const;

    // (group_size, group_stride) of every maximal run of axes that is contiguous in memory (shape.rs:191-217)
    std::vector<std::pair<size_t, int64_t>> continuous_groups() const;
    // lowest and highest element offset touched, relative to the view's origin
    std::pair<int64_t, int64_t> offset_bounds() const;
    std::string str() const;

private:
    std::vector<size_t> shape_;
    std::vector<int64_t> strides_;
    bool simple_, dense_;
};

// Where a planned tensor lives. The arena has three regions, each resolved to a base address when the
// executor is realised on a device: constants (uploaded once), a block of zeros, and the shared region whose
// slots are reused between values with disjoint live ranges.
enum class BufferKind : uint8_t { Constant = 0, Shared = 1, Zero = 2 };

struct PlanPtr {
    BufferKind kind = BufferKind::Shared;
    size_t index = 0;          // Constant: constant slot, Shared: shared buffer index
    int64_t offset_bytes = 0;  // offset of the view's origin inside the buffer
    bool operator==(const PlanPtr &o) const {
        return kind == o.kind && index == o.index && offset_bytes == o.offset_bytes;
    }
};

struct PlanTensor {
    PlanPtr ptr;
    DType dtype = DType::F32;
    StridedShape shape;

    bool operator==(const PlanTensor &o) const { return ptr == o.ptr && dtype == o.dtype && shape == o.shape; }

    PlanTensor with(int64_t offset_elem, StridedShape new_shape) const {
        PlanTensor r = *this;
        r.ptr.offset_bytes += offset_elem * (int64_t) dtype_bytes(dtype);
        r.shape = std::move(new_shape);
        return r;
    }
    PlanTensor permute(const std::vector<size_t> &p) const { return with(0, shape.permute(p)); }
    std::optional<PlanTensor> view(const std::vector<size_t> &new_shape) const {
        auto s = shape.view(new_shape);
        if (!s) return std::nullopt;
        return with(0, *s);
    }
    PlanTensor broadcast(const std::vector<size_t> &new_shape) const { return with(0, shape.broadcast(new_shape)); }
    PlanTensor slice(size_t axis, SliceRange range) const {
        StridedShape rs = shape.slice(axis, range);
        int64_t offset = rs.size() != 0 ? shape.strides()[axis] * (int64_t) range.start : 0;
        return with(offset, rs);
    }
    PlanTensor flip(size_t axis) const {
        size_t len = shape.shape()[axis];
        int64_t offset = (shape.size() != 0 && len != 0) ? (int64_t) (len - 1) * shape.strides()[axis] : 0;
        return with(offset, shape.flip(axis));
    }
};

}  // namespace kn
