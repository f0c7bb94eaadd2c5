// Symbolic shapes: every dimension is `fixed_factor * batch^batch_exp`.
// Mirrors kn-graph/src/shape.rs (Size :31-38, :234-317, :421-507; Shape :26-29, :48-219;
// infer_batch_size :353-419).
#pragma once

#include <optional>

#include "common.h"

namespace kn {

struct Size {
    uint32_t batch_exp = 0;
    uint64_t fixed_factor = 0;

    Size() = default;
    // shape.rs:239-251: a zero factor always normalises to the plain constant 0
    Size(uint32_t exp, uint64_t factor) : batch_exp(factor == 0 ? 0 : exp), fixed_factor(factor) {}
    static Size fixed(uint64_t n) { return Size(0, n); }
    static Size zero() { return Size(0, 0); }
    static Size one() { return Size(0, 1); }
    static Size batch() { return Size(1, 1); }

    bool operator==(const Size &o) const { return batch_exp == o.batch_exp && fixed_factor == o.fixed_factor; }
    bool operator!=(const Size &o) const { return !(*this == o); }
    bool is_zero() const { return fixed_factor == 0; }
    bool is_fixed() const { return batch_exp == 0; }

    uint64_t eval(uint64_t batch_size) const {
        uint64_t r = fixed_factor;
        for (uint32_t k = 0; k < batch_exp; k++) r *= batch_size;
        return r;
    }
    std::optional<uint64_t> try_unwrap_fixed() const {
        if (batch_exp == 0) return fixed_factor;
        return std::nullopt;
    }
    uint64_t unwrap_fixed(const char *what) const {
        if (batch_exp != 0) fail(what, " must be fixed, but got size ", str());
        return fixed_factor;
    }

    Size operator*(const Size &o) const { return Size(batch_exp + o.batch_exp, fixed_factor * o.fixed_factor); }
    // shape.rs:421-455: addition and subtraction only exist between equal powers of the batch size
    std::optional<Size> add(const Size &o) const {
        if (is_zero()) return o;
        if (o.is_zero()) return *this;
        if (batch_exp != o.batch_exp) return std::nullopt;
        return Size(batch_exp, fixed_factor + o.fixed_factor);
    }
    std::optional<Size> sub(const Size &o) const {
        if (o.is_zero()) return *this;
        if (batch_exp != o.batch_exp || fixed_factor < o.fixed_factor) return std::nullopt;
        return Size(batch_exp, fixed_factor - o.fixed_factor);
    }
    // shape.rs:303-316 exact division
    std::optional<Size> div(const Size &o) const {
        KN_ASSERT(o.fixed_factor != 0, "division by a zero size");
        if (batch_exp < o.batch_exp) return std::nullopt;
        if (fixed_factor % o.fixed_factor != 0) return std::nullopt;
        return Size(batch_exp - o.batch_exp, fixed_factor / o.fixed_factor);
    }

    // shape.rs:536-546
    std::string str() const {
        std::ostringstream ss;
        if (batch_exp == 0) ss << fixed_factor;
        else if (fixed_factor == 1 && batch_exp == 1) ss << "B";
        else if (batch_exp == 1) ss << fixed_factor << "B";
        else if (fixed_factor == 1) ss << "B^" << batch_exp;
        else ss << fixed_factor << "B^" << batch_exp;
        return ss.str();
    }
};

using ConcreteShape = std::vector<size_t>;

inline size_t concrete_size(const ConcreteShape &s) {
    size_t n = 1;
    for (size_t d : s) n *= d;
    return n;
}

struct Shape {
    std::vector<Size> dims;

    Shape() = default;
    explicit Shape(std::vector<Size> d) : dims(std::move(d)) {}
    static Shape fixed(const std::vector<size_t> &d) {
        Shape s;
        for (size_t x : d) s.dims.push_back(Size::fixed(x));
        return s;
    }
    static Shape ones(size_t rank) { return Shape(std::vector<Size>(rank, Size::one())); }
    static Shape scalar() { return Shape(); }

    size_t rank() const { return dims.size(); }
    bool operator==(const Shape &o) const { return dims == o.dims; }
    bool operator!=(const Shape &o) const { return !(*this == o); }
    const Size &operator[](size_t axis) const {
        assert_has_axis(axis);
        return dims[axis];
    }
    void assert_has_axis(size_t axis) const {
        if (axis >= rank()) fail("Axis ", axis, " out of bounds for ", str());
    }

    Size size() const {
        Size r = Size::one();
        for (auto &d : dims) r = r * d;
        return r;
    }
    ConcreteShape eval(uint64_t batch_size) const {
        ConcreteShape r;
        for (auto &d : dims) r.push_back(d.eval(batch_size));
        return r;
    }
    std::optional<ConcreteShape> as_fixed() const {
        ConcreteShape r;
        for (auto &d : dims) {
            if (!d.is_fixed()) return std::nullopt;
            r.push_back(d.fixed_factor);
        }
        return r;
    }
    ConcreteShape unwrap_fixed(const char *what) const {
        ConcreteShape r;
        for (auto &d : dims) r.push_back(d.unwrap_fixed(what));
        return r;
    }

    Shape concat(const Shape &o) const {
        Shape r = *this;
        r.dims.insert(r.dims.end(), o.dims.begin(), o.dims.end());
        return r;
    }
    // shape.rs:143-162: every listed axis is replaced by the whole of `replacement`
    Shape replace_all(const std::vector<size_t> &axes, const Shape &replacement) const {
        for (size_t a = 0; a < axes.size(); a++) {
            assert_has_axis(axes[a]);
            for (size_t b = 0; b < a; b++)
                if (axes[a] == axes[b]) fail("Axes must be unique, got ", vec_str(axes));
        }
        Shape r;
        for (size_t i = 0; i < rank(); i++) {
            bool hit = false;
            for (size_t a : axes) hit |= (a == i);
            if (hit) r.dims.insert(r.dims.end(), replacement.dims.begin(), replacement.dims.end());
            else r.dims.push_back(dims[i]);
        }
        return r;
    }
    Shape replace(size_t axis, const Shape &replacement) const { return replace_all({axis}, replacement); }
    // shape.rs:164-175
    Shape keep(size_t axis, Size rest) const {
        assert_has_axis(axis);
        Shape r = *this;
        for (size_t i = 0; i < rank(); i++)
            if (i != axis) r.dims[i] = rest;
        return r;
    }
    Shape insert(size_t axis, Size size) const {
        if (axis > rank()) fail("Axis ", axis, " out of bounds for inserting into ", str());
        Shape r = *this;
        r.dims.insert(r.dims.begin() + axis, size);
        return r;
    }
    std::pair<Shape, Shape> split(size_t index) const {
        if (index > rank()) fail("Split index ", index, " out of bounds for ", str());
        return {Shape(std::vector<Size>(dims.begin(), dims.begin() + index)),
                Shape(std::vector<Size>(dims.begin() + index, dims.end()))};
    }

    std::string str() const {
        std::string r = "(";
        for (size_t i = 0; i < dims.size(); i++) {
            if (i) r += " x ";
            r += dims[i].str();
        }
        return r + ")";
    }
    uint64_t hash() const {
        uint64_t h = dims.size();
        for (auto &d : dims) h = hash_combine(hash_combine(h, d.batch_exp), d.fixed_factor);
        return h;
    }
};

enum class ShapeMismatch { None = 0, DifferentLength = 1, ConstantMismatch = 2, BatchConflict = 3, ImpossibleBatchValue = 4 };

// shape.rs:360-419. On success `*batch` holds the inferred batch size, or is empty when any size fits.
ShapeMismatch infer_batch_size(const std::vector<Shape> &expected, const std::vector<ConcreteShape> &actual,
                               std::optional<uint64_t> *batch);

}  // namespace kn
