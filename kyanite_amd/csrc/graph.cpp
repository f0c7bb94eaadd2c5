#include "graph.h"

#include <algorithm>
#include <functional>

namespace kn {

const char *op_kind_name(OpKind k) {
    static const char *names[] = {"Input", "Constant", "View", "Broadcast", "Permute", "Slice", "Flip", "Gather",
                                  "Concat", "Conv", "MatMul", "Unary", "Binary", "Softmax", "Layernorm", "Reduce"};
    return names[(int) k];
}
const char *unary_op_name(UnaryOp op) {
    static const char *names[] = {"Abs", "Neg", "Sin", "Cos", "Exp", "Log", "Sqrt", "Sigmoid", "Tanh", "Erf",
                                  "Mish", "Softplus", "ValueCast", "BitCast"};
    return names[(int) op];
}
const char *binary_op_name(BinaryOp op) {
    static const char *names[] = {"Add", "Sub", "Mul", "Div", "Min", "Max", "Pow"};
    return names[(int) op];
}
const char *reduce_op_name(ReduceOp op) {
    static const char *names[] = {"Sum", "Mean", "Prod", "Max", "Min"};
    return names[(int) op];
}

// ------------------------------------------------------------------------------------------------ SliceRange

SliceRange SliceRange::make(size_t start, size_t end, size_t step) {
    SliceRange r{start, end, step};
    r.assert_valid();
    return r;
}

void SliceRange::assert_valid() const {
    if (end < start) fail("Invalid range ", start, ":", end, ":", step, ": bounds cannot be decreasing");
    if (step == 0) fail("Invalid range ", start, ":", end, ":", step, ": step cannot be 0");
    if ((end - start) % step != 0)
        fail("Invalid range ", start, ":", end, ":", step, ": bounds must differ by a multiple of step");
}

void SliceRange::assert_in_bounds(size_t size) const {
    assert_valid();
    if (!(start == end || (start < size && end - (step - 1) <= size)))
        fail("SliceRange ", start, ":", end, ":", step, " out of bounds for axis of size ", size);
}

bool ConvDetails::operator==(const ConvDetails &o) const {
    return dtype == o.dtype && batch_size == o.batch_size && input_channels == o.input_channels &&
           output_channels == o.output_channels && input_h == o.input_h && input_w == o.input_w &&
           kernel_h == o.kernel_h && kernel_w == o.kernel_w && stride_y == o.stride_y && stride_x == o.stride_x &&
           padding_y == o.padding_y && padding_x == o.padding_x && output_h == o.output_h && output_w == o.output_w;
}

// ------------------------------------------------------------------------------------------------ Operation

bool Operation::equals(const Operation &o) const {
    if (kind != o.kind || inputs != o.inputs) return false;
    switch (kind) {
        case OpKind::Input: return index == o.index;
        case OpKind::Constant: return tensor.equals(o.tensor);
        case OpKind::View: case OpKind::Broadcast: case OpKind::MatMul: return true;
        case OpKind::Permute: case OpKind::Flip: case OpKind::Gather: case OpKind::Concat: case OpKind::Softmax:
            return axes == o.axes;
        case OpKind::Slice: return axes == o.axes && range == o.range;
        case OpKind::Conv: return conv == o.conv;
        case OpKind::Unary:
            if (unary != o.unary) return false;
            if (unary == UnaryOp::ValueCast || unary == UnaryOp::BitCast) return cast_to == o.cast_to;
            return true;
        case OpKind::Binary: return binary == o.binary;
        case OpKind::Layernorm: {
            // eps compares as a total float: NaN equals NaN
            bool same = (std::isnan(eps) && std::isnan(o.eps)) || eps == o.eps;
            return axes == o.axes && same;
        }
        case OpKind::Reduce: return axes == o.axes && reduce == o.reduce;
    }
    return false;
}

uint64_t Operation::hash() const {
    uint64_t h = (uint64_t) kind;
    for (Value v : inputs) h = hash_combine(h, v);
    for (size_t a : axes) h = hash_combine(h, a);
    switch (kind) {
        case OpKind::Input: h = hash_combine(h, index); break;
        case OpKind::Constant: h = hash_combine(h, tensor.hash()); break;
        case OpKind::Slice: h = hash_combine(hash_combine(hash_combine(h, range.start), range.end), range.step); break;
        case OpKind::Unary: h = hash_combine(h, (uint64_t) unary * 16 + (uint64_t) cast_to); break;
        case OpKind::Binary: h = hash_combine(h, (uint64_t) binary); break;
        case OpKind::Reduce: h = hash_combine(h, (uint64_t) reduce); break;
        default: break;
    }
    return h;
}

// ------------------------------------------------------------------------------------------------ scalar semantics

std::optional<DType> unary_output_dtype(UnaryOp op, DType x, DType cast_to) {
    switch (op) {
        case UnaryOp::Abs: case UnaryOp::Neg:
            return dtype_is_signed(x) ? std::optional<DType>(x) : std::nullopt;
        case UnaryOp::ValueCast: return cast_to;
        case UnaryOp::BitCast:
            return dtype_bytes(x) == dtype_bytes(cast_to) ? std::optional<DType>(cast_to) : std::nullopt;
        default: return dtype_is_float(x) ? std::optional<DType>(x) : std::nullopt;
    }
}

double erf_approx(double x) {
    // graph.rs:1791-1815: Abramowitz and Stegun, max error 3e-7
    static const double A[] = {1.0, 0.0705230784, 0.0422820123, 0.0092705272, 0.0001520143, 0.0002765672, 0.0000430638};
    double sign = std::isnan(x) ? x : (std::signbit(x) ? -1.0 : 1.0);
    double xa = std::fabs(x);
    double d = 0, p = 1;
    for (double a : A) {
        d += a * p;
        p *= xa;
    }
    double d2 = d * d, d4 = d2 * d2, d8 = d4 * d4, d16 = d8 * d8;
    return sign * (1.0 - 1.0 / d16);
}

template <typename F>
static F unary_float(UnaryOp op, F x) {
    switch (op) {
        case UnaryOp::Abs: return std::fabs(x);
        case UnaryOp::Neg: return -x;
        case UnaryOp::Sin: return std::sin(x);
        case UnaryOp::Cos: return std::cos(x);
        case UnaryOp::Exp: return std::exp(x);
        case UnaryOp::Log: return std::log(x);
        case UnaryOp::Sqrt: return std::sqrt(x);
        case UnaryOp::Sigmoid: return (F) 1 / ((F) 1 + std::exp(-x));
        case UnaryOp::Tanh: return std::tanh(x);
        case UnaryOp::Erf: return (F) erf_approx((double) x);
        case UnaryOp::Mish: return x * std::tanh(std::log1p(std::exp(x)));
        case UnaryOp::Softplus: return std::log1p(std::exp(-std::fabs(x))) + std::max(x, (F) 0);
        default: fail("not a float operation");
    }
}

static DScalar wrap_sint(DType t, int64_t v) {
    switch (t) {
        case DType::I8: return DScalar::sint(t, (int8_t) v);
        case DType::I16: return DScalar::sint(t, (int16_t) v);
        case DType::I32: return DScalar::sint(t, (int32_t) v);
        default: return DScalar::sint(t, v);
    }
}
static DScalar wrap_uint(DType t, uint64_t v) {
    switch (t) {
        case DType::U8: return DScalar::uint(t, (uint8_t) v);
        case DType::U16: return DScalar::uint(t, (uint16_t) v);
        case DType::U32: return DScalar::uint(t, (uint32_t) v);
        default: return DScalar::uint(t, v);
    }
}

DScalar unary_map(UnaryOp op, DType cast_to, const DScalar &x) {
    if (op == UnaryOp::ValueCast) return x.value_cast(cast_to);
    if (op == UnaryOp::BitCast) {
        DScalar y;
        if (!x.bit_cast(cast_to, &y)) fail("Cannot bitcast ", dtype_name(x.dtype), " to ", dtype_name(cast_to));
        return y;
    }
    if (x.is_float()) {
        if (x.dtype == DType::F64) return DScalar::f64(unary_float<double>(op, x.f));
        float y = unary_float<float>(op, (float) x.f);
        return x.dtype == DType::F16 ? DScalar::f16(y) : DScalar::f32(y);
    }
    if (x.is_signed_int() && (op == UnaryOp::Abs || op == UnaryOp::Neg)) {
        // two's complement wrapping, as a release build of the reference does
        uint64_t u = (uint64_t) x.i;
        uint64_t r = (op == UnaryOp::Neg || x.i < 0) ? (0 - u) : u;
        return wrap_sint(x.dtype, (int64_t) r);
    }
    fail("Operation ", unary_op_name(op), " not supported on dtype ", dtype_name(x.dtype));
}

template <typename F>
static F binary_float(BinaryOp op, F l, F r) {
    switch (op) {
        case BinaryOp::Add: return l + r;
        case BinaryOp::Sub: return l - r;
        case BinaryOp::Mul: return l * r;
        case BinaryOp::Div: return l / r;
        case BinaryOp::Min: return std::fmin(l, r);
        case BinaryOp::Max: return std::fmax(l, r);
        case BinaryOp::Pow: return std::pow(l, r);
    }
    return 0;
}

DScalar binary_map(BinaryOp op, const DScalar &l, const DScalar &r) {
    if (l.dtype != r.dtype) fail("Mismatched dtypes: left ", dtype_name(l.dtype), ", right ", dtype_name(r.dtype));
    DType t = l.dtype;
    if (op == BinaryOp::Pow && t != DType::F32 && t != DType::F16 && t != DType::F64)
        fail("Pow is only supported for floats, got ", dtype_name(t));
    if (t == DType::F64) return DScalar::f64(binary_float<double>(op, l.f, r.f));
    if (t == DType::F32) return DScalar::f32(binary_float<float>(op, (float) l.f, (float) r.f));
    if (t == DType::F16) return DScalar::f16(binary_float<float>(op, (float) l.f, (float) r.f));
    if (t == DType::Bool) {
        // dtype.rs:726-757: add = or, mul = and, sub = div = and-not; min/max follow false < true
        bool a = l.u != 0, b = r.u != 0;
        switch (op) {
            case BinaryOp::Add: case BinaryOp::Max: return DScalar::boolean(a || b);
            case BinaryOp::Mul: case BinaryOp::Min: return DScalar::boolean(a && b);
            case BinaryOp::Sub: case BinaryOp::Div: return DScalar::boolean(a && !b);
            default: fail("unsupported bool operation");
        }
    }
    if (dtype_is_signed(t)) {
        int64_t a = l.i, b = r.i;
        switch (op) {
            case BinaryOp::Add: return wrap_sint(t, (int64_t) ((uint64_t) a + (uint64_t) b));
            case BinaryOp::Sub: return wrap_sint(t, (int64_t) ((uint64_t) a - (uint64_t) b));
            case BinaryOp::Mul: return wrap_sint(t, (int64_t) ((uint64_t) a * (uint64_t) b));
            case BinaryOp::Div:
                if (b == 0) fail("attempt to divide by zero");
                if (b == -1) return wrap_sint(t, (int64_t) (0 - (uint64_t) a));
                return wrap_sint(t, a / b);
            case BinaryOp::Min: return wrap_sint(t, std::min(a, b));
            case BinaryOp::Max: return wrap_sint(t, std::max(a, b));
            default: fail("unsupported int operation");
        }
    }
    uint64_t a = l.u, b = r.u;
    switch (op) {
        case BinaryOp::Add: return wrap_uint(t, a + b);
        case BinaryOp::Sub: return wrap_uint(t, a - b);
        case BinaryOp::Mul: return wrap_uint(t, a * b);
        case BinaryOp::Div:
            if (b == 0) fail("attempt to divide by zero");
            return wrap_uint(t, a / b);
        case BinaryOp::Min: return wrap_uint(t, std::min(a, b));
        case BinaryOp::Max: return wrap_uint(t, std::max(a, b));
        default: fail("unsupported int operation");
    }
}

DScalar reduce_identity(ReduceOp op, DType dtype) {
    Specials s = dtype_specials(dtype);
    switch (op) {
        case ReduceOp::Sum: case ReduceOp::Mean: return s.zero;
        case ReduceOp::Prod: return s.one;
        case ReduceOp::Min: return s.max;
        case ReduceOp::Max: return s.min;
    }
    return s.zero;
}

// ------------------------------------------------------------------------------------------------ queries

bool Graph::is_hidden(Value v) const {
    check_contains(v);
    return std::find(inputs.begin(), inputs.end(), v) == inputs.end() &&
           std::find(outputs.begin(), outputs.end(), v) == outputs.end();
}

bool Graph::is_hidden_with_uses(Value v, size_t users) const {
    return is_hidden(v) && values[v].non_output_uses == users;
}

bool Graph::is_const(Value v) const {
    // iterative, values are topologically ordered
    check_contains(v);
    std::vector<Value> stack{v};
    std::vector<uint8_t> seen(values.size(), 0);
    while (!stack.empty()) {
        Value c = stack.back();
        stack.pop_back();
        if (seen[c]) continue;
        seen[c] = 1;
        const Operation &op = values[c].operation;
        if (op.kind == OpKind::Input) return false;
        for (Value in : op.inputs) stack.push_back(in);
    }
    return true;
}

std::optional<DScalar> Graph::as_single_const(Value v) const {
    const ValueInfo &info = (*this)[v];
    const Operation &op = info.operation;
    switch (op.kind) {
        case OpKind::Input: return std::nullopt;
        case OpKind::Constant: {
            size_t n = op.tensor.len();
            if (n == 0) return std::nullopt;
            DScalar e = op.tensor.at(0);
            // elements compare with the primitive `==` here (graph.rs:495-498): a NaN constant is never "single"
            auto prim_eq = [](const DScalar &a, const DScalar &b) {
                if (a.is_float()) return a.f == b.f;
                return a == b;
            };
            for (size_t k = 0; k < n; k++)
                if (!prim_eq(op.tensor.at(k), e)) return std::nullopt;
            return e;
        }
        case OpKind::View: case OpKind::Broadcast: case OpKind::Permute: case OpKind::Slice: case OpKind::Flip:
        case OpKind::Gather:
            return as_single_const(op.inputs[0]);
        case OpKind::Concat: {
            if (op.inputs.empty()) return std::nullopt;
            auto f = as_single_const(op.inputs[0]);
            if (!f) return std::nullopt;
            for (Value x : op.inputs)
                if (!is_const_filled_with(x, *f)) return std::nullopt;
            return f;
        }
        case OpKind::Unary: {
            auto x = as_single_const(op.inputs[0]);
            if (!x) return std::nullopt;
            return unary_map(op.unary, op.cast_to, *x);
        }
        case OpKind::Binary: {
            auto l = as_single_const(op.inputs[0]);
            if (!l) return std::nullopt;
            auto r = as_single_const(op.inputs[1]);
            if (!r) return std::nullopt;
            return binary_map(op.binary, *l, *r);
        }
        default: return std::nullopt;
    }
}

bool Graph::is_const_filled_with(Value v, const DScalar &expected) const {
    auto actual = as_single_const(v);
    return actual && *actual == expected;
}

// ------------------------------------------------------------------------------------------------ push

Value Graph::push(Shape shape, DType dtype, Operation operation) {
    uint64_t h = hash_combine(hash_combine(shape.hash(), (uint64_t) dtype), operation.hash());
    auto range = back_map_.equal_range(h);
    for (auto it = range.first; it != range.second; ++it) {
        const ValueInfo &cand = values[it->second];
        if (cand.dtype == dtype && cand.shape == shape && cand.operation.equals(operation)) return it->second;
    }
    for (Value in : operation.inputs) {
        check_contains(in);
        values[in].non_output_uses += 1;
    }
    Value v = (Value) values.size();
    ValueInfo info;
    info.shape = std::move(shape);
    info.dtype = dtype;
    info.operation = std::move(operation);
    values.push_back(std::move(info));
    back_map_.emplace(h, v);
    return v;
}

void Graph::set_debug_id(Value v, std::string id) {
    check_contains(v);
    values[v].debug_id = std::move(id);
}

// ------------------------------------------------------------------------------------------------ builder

Value Graph::input(Shape shape, DType dtype) {
    Operation op;
    op.kind = OpKind::Input;
    op.index = inputs.size();
    Value v = push(std::move(shape), dtype, std::move(op));
    inputs.push_back(v);
    return v;
}

Value Graph::constant_tensor(HostTensor tensor) {
    Shape shape = Shape::fixed(tensor.shape);
    DType dtype = tensor.dtype;
    Operation op;
    op.kind = OpKind::Constant;
    op.tensor = std::move(tensor);
    return push(std::move(shape), dtype, std::move(op));
}

Value Graph::constant(const Shape &shape, DType dtype, const void *data) {
    ConcreteShape dims = shape.unwrap_fixed("constant shape");
    return constant_tensor(HostTensor(dtype, dims, data));
}

Value Graph::scalar_dyn(const DScalar &value) { return constant_tensor(HostTensor::scalar(value)); }

Value Graph::view(Value input, const Shape &new_shape) {
    const ValueInfo &info = (*this)[input];
    if (new_shape == info.shape) return input;
    if (info.shape.size() != new_shape.size())
        fail("New shape ", new_shape.str(), " must have the same size as old shape ", info.shape.str());
    // only keep the last view operation
    Value inner = info.operation.kind == OpKind::View ? info.operation.inputs[0] : input;
    Operation op;
    op.kind = OpKind::View;
    op.inputs = {inner};
    return push(new_shape, info.dtype, std::move(op));
}

Value Graph::broadcast(Value input, const Shape &new_shape) {
    Shape input_shape = (*this)[input].shape;
    DType dtype = (*this)[input].dtype;
    if (input_shape.rank() > new_shape.rank())
        fail("Cannot broadcast to a lower rank shape (from ", input_shape.str(), " to ", new_shape.str(), ")");
    Shape view_shape = Shape::ones(new_shape.rank() - input_shape.rank()).concat(input_shape);
    Value curr = view(input, view_shape);
    for (size_t i = 0; i < new_shape.rank(); i++) {
        if (!(view_shape.dims[i] == new_shape.dims[i] || view_shape.dims[i] == Size::one()))
            fail("Cannot broadcast from ", input_shape.str(), " to ", new_shape.str(), " because of axis (",
                 view_shape.dims[i].str(), ", ", new_shape.dims[i].str(), ")");
    }
    if (view_shape == new_shape) return curr;
    Operation op;
    op.kind = OpKind::Broadcast;
    op.inputs = {curr};
    return push(new_shape, dtype, std::move(op));
}

Value Graph::repeat_unary(Value input, size_t axis, Size count) {
    const ValueInfo &info = (*this)[input];
    if (info.shape[axis] != Size::one())
        fail("Input shape ", info.shape.str(), " does not have dim 1 for axis ", axis);
    if (count == Size::one()) return input;
    Shape new_shape = info.shape.replace(axis, Shape({count}));
    Operation op;
    op.kind = OpKind::Broadcast;
    op.inputs = {input};
    return push(new_shape, info.dtype, std::move(op));
}

Value Graph::flatten(Value input, size_t start_axis) {
    const Shape &old = (*this)[input].shape;
    if (start_axis > old.rank()) fail("Flatten start axis ", start_axis, " out of bounds for ", old.str());
    Shape ns;
    Size flat = Size::one();
    for (size_t i = 0; i < old.rank(); i++) {
        if (i < start_axis) ns.dims.push_back(old.dims[i]);
        else flat = flat * old.dims[i];
    }
    ns.dims.push_back(flat);
    return view(input, ns);
}

Value Graph::permute(Value input, std::vector<size_t> permutation) {
    const ValueInfo &info = (*this)[input];
    if (permutation.size() != info.shape.rank())
        fail("Permutation rank must match input shape, got ", vec_str(permutation), " and ", info.shape.str());
    for (size_t a = 0; a < permutation.size(); a++) {
        if (permutation[a] >= info.shape.rank()) fail("Permutation axis out of bounds, got ", vec_str(permutation));
        for (size_t b = 0; b < a; b++)
            if (permutation[a] == permutation[b])
                fail("Permutation cannot contain repeated axis, got ", vec_str(permutation));
    }
    // fuse consecutive permute operations
    Value inner = input;
    std::vector<size_t> full = permutation;
    if (info.operation.kind == OpKind::Permute) {
        inner = info.operation.inputs[0];
        for (size_t k = 0; k < permutation.size(); k++) full[k] = info.operation.axes[permutation[k]];
    }
    const Shape &inner_shape = (*this)[inner].shape;
    Shape result;
    for (size_t i : full) result.dims.push_back(inner_shape[i]);
    Operation op;
    op.kind = OpKind::Permute;
    op.inputs = {inner};
    op.axes = full;
    return push(result, info.dtype, std::move(op));
}

Value Graph::slice(Value input, size_t axis, SliceRange range) {
    const ValueInfo &info = (*this)[input];
    info.shape.assert_has_axis(axis);
    size_t input_size = info.shape.dims[axis].unwrap_fixed("Slice axis length");
    range.assert_in_bounds(input_size);
    size_t new_size = (range.end - range.start) / range.step;
    if (range == SliceRange{0, input_size, 1}) return input;
    Shape new_shape = info.shape.replace(axis, Shape::fixed({new_size}));
    Operation op;
    op.kind = OpKind::Slice;
    op.inputs = {input};
    op.axes = {axis};
    op.range = range;
    return push(new_shape, info.dtype, std::move(op));
}

Value Graph::index(Value input, size_t axis, size_t index) {
    Shape new_shape = (*this)[input].shape.replace(axis, Shape());
    Value sliced = slice(input, axis, SliceRange::single(index));
    return view(sliced, new_shape);
}

Value Graph::flip(Value input, size_t axis) {
    const ValueInfo &info = (*this)[input];
    info.shape.assert_has_axis(axis);
    Operation op;
    op.kind = OpKind::Flip;
    op.inputs = {input};
    op.axes = {axis};
    return push(info.shape, info.dtype, std::move(op));
}

Value Graph::repeat(Value input, size_t axis, Size count) { return repeat_impl(input, axis, count, false); }
Value Graph::repeat_interleave(Value input, size_t axis, Size count) { return repeat_impl(input, axis, count, true); }

Value Graph::repeat_impl(Value input, size_t axis, Size count, bool inner) {
    Shape input_shape = (*this)[input].shape;
    input_shape.assert_has_axis(axis);
    if (input_shape[axis] == Size::one()) return repeat_unary(input, axis, count);
    Size new_size = input_shape[axis] * count;
    size_t dummy_axis = inner ? axis + 1 : axis;
    // insert dummy axis, repeat dummy axis, flatten into main axis
    Value extra = view(input, input_shape.insert(dummy_axis, Size::one()));
    Value broad = repeat_unary(extra, dummy_axis, count);
    return view(broad, input_shape.replace(axis, Shape({new_size})));
}

Value Graph::gather(Value input, size_t axis, Value indices) {
    Shape input_shape = (*this)[input].shape;
    DType dtype = (*this)[input].dtype;
    Shape indices_shape = (*this)[indices].shape;
    DType indices_dtype = (*this)[indices].dtype;
    input_shape.assert_has_axis(axis);
    if (!dtype_is_int(indices_dtype)) fail("Indices must be integers, got ", dtype_name(indices_dtype));

    Shape result_shape = input_shape.replace(axis, indices_shape);
    Shape result_shape_flat = input_shape.replace(axis, Shape({indices_shape.size()}));

    // arbitrary rank indices are supported here, the operation itself only takes rank 1
    Value flat_indices = flatten(indices, 0);
    Size flat_size = (*this)[flat_indices].shape.dims.at(0);

    Value result_flat;
    if (auto index = as_single_const(indices)) {
        // replace gather with simpler slice + repeat operators
        if (index->is_signed_int() && index->i < 0) fail("Gather index ", index->i, " is negative");
        size_t idx = index->is_signed_int() ? (size_t) index->i : (size_t) index->u;
        Value single = slice(input, axis, SliceRange::single(idx));
        result_flat = repeat(single, axis, flat_size);
        KN_ASSERT((*this)[result_flat].shape == result_shape_flat);
    } else {
        Operation op;
        op.kind = OpKind::Gather;
        op.inputs = {input, flat_indices};
        op.axes = {axis};
        result_flat = push(result_shape_flat, dtype, std::move(op));
    }
    return view(result_flat, result_shape);
}

Value Graph::concat(std::vector<Value> ins, size_t axis, const std::optional<Shape> &base_shape_opt,
                    std::optional<DType> dtype_opt) {
    Shape base_shape;
    if (base_shape_opt) base_shape = *base_shape_opt;
    else {
        if (ins.empty()) fail("Cannot infer concatenation shape without any inputs");
        base_shape = (*this)[ins[0]].shape.replace(axis, Shape::fixed({0}));
    }
    DType dtype;
    if (dtype_opt) dtype = *dtype_opt;
    else {
        if (ins.empty()) fail("Cannot infer concatenation dtype without any inputs");
        dtype = (*this)[ins[0]].dtype;
    }

    Size size_along_axis = Size::zero();
    for (Value v : ins) {
        const ValueInfo &info = (*this)[v];
        if (info.shape.replace(axis, Shape::fixed({0})) != base_shape)
            fail("All concatenated values must match base shape on non-concatenated axes");
        if (info.dtype != dtype) fail("All concatenated values must have the same dtype");
        auto sum = size_along_axis.add(info.shape.dims[axis]);
        if (!sum) fail("Could not add all concatenation sizes");
        size_along_axis = *sum;
    }
    Shape result_shape = base_shape.replace(axis, Shape({size_along_axis}));

    // drop empty inputs
    std::vector<Value> kept;
    for (Value v : ins)
        if (!(*this)[v].shape.size().is_zero()) kept.push_back(v);
    if (kept.size() == 1) return kept[0];

    Operation op;
    op.kind = OpKind::Concat;
    op.inputs = kept;
    op.axes = {axis};
    return push(result_shape, dtype, std::move(op));
}

Value Graph::pad(Value input, const std::vector<std::pair<size_t, size_t>> &pad_amount, Value pad_value) {
    const ValueInfo &info = (*this)[input];
    const ValueInfo &pinfo = (*this)[pad_value];
    if (info.shape.rank() != pad_amount.size()) fail("Padding length must match input rank");
    if (info.dtype != pinfo.dtype) fail("Padding value dtype must match input dtype");
    if (pinfo.shape.rank() != 0) fail("Padding value must be scalar");
    Value curr = input;
    for (size_t i = 0; i < pad_amount.size(); i++) {
        Shape curr_shape = (*this)[curr].shape;
        Value before = broadcast(pad_value, curr_shape.replace(i, Shape::fixed({pad_amount[i].first})));
        Value after = broadcast(pad_value, curr_shape.replace(i, Shape::fixed({pad_amount[i].second})));
        curr = concat({before, curr, after}, i, std::nullopt, std::nullopt);
    }
    return curr;
}

Value Graph::conv(Value input, Value filter, size_t stride_y, size_t stride_x, size_t padding_y, size_t padding_x) {
    const ValueInfo &iinfo = (*this)[input];
    const ValueInfo &finfo = (*this)[filter];
    if (iinfo.dtype != finfo.dtype) fail("Convolution input and filter must have the same dtype");
    if (iinfo.shape.rank() != 4) fail("Convolution input must have rank 4");
    if (finfo.shape.rank() != 4) fail("Convolution filter must have rank 4");
    if (stride_y == 0 || stride_x == 0) fail("Convolution stride cannot be 0");

    ConvDetails d;
    d.dtype = iinfo.dtype;
    d.batch_size = iinfo.shape.dims[0];
    d.input_channels = iinfo.shape.dims[1].unwrap_fixed("Conv input channels");
    d.input_h = iinfo.shape.dims[2].unwrap_fixed("Conv input height");
    d.input_w = iinfo.shape.dims[3].unwrap_fixed("Conv input width");
    d.output_channels = finfo.shape.dims[0].unwrap_fixed("Conv output channels");
    size_t in_c_check = finfo.shape.dims[1].unwrap_fixed("Filter input channels");
    d.kernel_h = finfo.shape.dims[2].unwrap_fixed("Conv kernel height");
    d.kernel_w = finfo.shape.dims[3].unwrap_fixed("Conv kernel width");
    if (d.kernel_h % 2 != 1) fail("Kernel height must be odd, got ", d.kernel_h);
    if (d.kernel_w % 2 != 1) fail("Kernel width must be odd, got ", d.kernel_w);
    if (d.input_channels != in_c_check) fail("Input channel mismatch");
    size_t padded_h = d.input_h + 2 * padding_y, padded_w = d.input_w + 2 * padding_x;
    if (!(padded_h >= d.kernel_h && padded_w >= d.kernel_w)) fail("Kernel must fit inside of padded input");
    d.stride_y = stride_y;
    d.stride_x = stride_x;
    d.padding_y = padding_y;
    d.padding_x = padding_x;
    d.output_h = (padded_h - (d.kernel_h - 1) - 1) / stride_y + 1;
    d.output_w = (padded_w - (d.kernel_w - 1) - 1) / stride_x + 1;
    Shape out({d.batch_size, Size::fixed(d.output_channels), Size::fixed(d.output_h), Size::fixed(d.output_w)});

    Operation op;
    op.kind = OpKind::Conv;
    op.inputs = {input, filter};
    op.conv = d;
    return push(out, iinfo.dtype, std::move(op));
}

Value Graph::linear(Value input, Value weight) {
    Value wt = permute(weight, {1, 0});
    return mat_mul(input, wt);
}

Value Graph::mat_mul(Value left, Value right) {
    Shape ls = (*this)[left].shape, rs = (*this)[right].shape;
    if (!(ls.rank() >= 2 && rs.rank() >= 2))
        fail("Matmul operands must have rank >= 2, got shapes ", ls.str(), " and ", rs.str());
    auto [lhead, ltail] = ls.split(ls.rank() - 2);
    auto [rhead, rtail] = rs.split(rs.rank() - 2);
    if (ltail.dims[1] != rtail.dims[0])
        fail("Inner matmul dimension must match, got shapes ", ls.str(), " and ", rs.str());
    Shape result_tail({ltail.dims[0], rtail.dims[1]});
    Shape result_head = broadcast_shape_symmetric(lhead, rhead);
    Size batch = result_head.size();
    Value lb = broadcast(left, result_head.concat(ltail));
    Value rb = broadcast(right, result_head.concat(rtail));
    Value lf = view(lb, ltail.insert(0, batch));
    Value rf = view(rb, rtail.insert(0, batch));
    Value rflat = batched_mat_mul(lf, rf);
    return view(rflat, result_head.concat(result_tail));
}

Value Graph::batched_mat_mul(Value left, Value right) {
    const ValueInfo &l = (*this)[left];
    const ValueInfo &r = (*this)[right];
    if (l.dtype != r.dtype) fail("Matmul operands must have same dtype");
    if (l.shape.rank() != 3) fail("Expected rank 3 shape, got ", l.shape.str());
    if (r.shape.rank() != 3) fail("Expected rank 3 shape, got ", r.shape.str());
    if (!(l.shape.dims[0] == r.shape.dims[0] && l.shape.dims[2] == r.shape.dims[1]))
        fail("Batched matmul dimension mismatch, got shapes ", l.shape.str(), " and ", r.shape.str());
    Shape result({l.shape.dims[0], l.shape.dims[1], r.shape.dims[2]});
    Operation op;
    op.kind = OpKind::MatMul;
    op.inputs = {left, right};
    return push(result, l.dtype, std::move(op));
}

Value Graph::softmax(Value input, size_t axis) {
    const ValueInfo &info = (*this)[input];
    if (info.dtype != DType::F32 && info.dtype != DType::F16) fail("Softmax input must be f32 or f16");
    info.shape.assert_has_axis(axis);
    Operation op;
    op.kind = OpKind::Softmax;
    op.inputs = {input};
    op.axes = {axis};
    return push(info.shape, info.dtype, std::move(op));
}

Value Graph::layernorm(Value input, size_t axis, float eps) {
    const ValueInfo &info = (*this)[input];
    if (info.dtype != DType::F32 && info.dtype != DType::F16) fail("Layernorm input must be f32 or f16");
    info.shape.assert_has_axis(axis);
    Operation op;
    op.kind = OpKind::Layernorm;
    op.inputs = {input};
    op.axes = {axis};
    op.eps = eps;
    return push(info.shape, info.dtype, std::move(op));
}

Value Graph::reduce(Value input, std::vector<size_t> axes, ReduceOp rop) {
    const ValueInfo &info = (*this)[input];
    for (size_t a : axes) info.shape.assert_has_axis(a);
    if (rop == ReduceOp::Mean && info.dtype != DType::F32 && info.dtype != DType::F16) fail("Mean input must be f32 or f16");
    if (axes.empty()) return input;
    Shape new_shape = info.shape.replace_all(axes, Shape());
    Operation op;
    op.kind = OpKind::Reduce;
    op.inputs = {input};
    op.axes = std::move(axes);
    op.reduce = rop;
    return push(new_shape, info.dtype, std::move(op));
}

Value Graph::sigmoid(Value input) { return unary(UnaryOp::Sigmoid, input); }

Value Graph::relu(Value input) {
    Specials s = dtype_specials((*this)[input].dtype);
    return clamp_dyn(input, s.zero, s.max);
}

Value Graph::clamp_dyn(Value input, const DScalar &min, const DScalar &max) {
    DType dtype = (*this)[input].dtype;
    if (!(dtype == min.dtype && dtype == max.dtype))
        fail("Clamp bounds must match value type, got min=", min.to_string(), " and max=", max.to_string(), " for ",
             dtype_name(dtype));
    // min/max are intentionally flipped to yield MAX(MIN(x, max), min)
    Value curr = input;
    Specials s = dtype_specials(dtype);
    if (max != s.max) curr = binary(BinaryOp::Min, curr, scalar_dyn(max));
    if (min != s.min) curr = binary(BinaryOp::Max, curr, scalar_dyn(min));
    return curr;
}

Value Graph::unary(UnaryOp uop, Value input, DType cast_to) {
    const ValueInfo &info = (*this)[input];
    auto out = unary_output_dtype(uop, info.dtype, cast_to);
    if (!out) fail("Operation ", unary_op_name(uop), " not supported on dtype ", dtype_name(info.dtype));
    bool is_cast = uop == UnaryOp::ValueCast || uop == UnaryOp::BitCast;
    if (is_cast && *out == info.dtype) return input;
    if (uop == UnaryOp::BitCast) {
        // skip to the innermost bitcast value
        while (values[input].operation.kind == OpKind::Unary && values[input].operation.unary == UnaryOp::BitCast)
            input = values[input].operation.inputs[0];
    }
    Operation op;
    op.kind = OpKind::Unary;
    op.inputs = {input};
    op.unary = uop;
    op.cast_to = is_cast ? cast_to : DType::F32;
    return push((*this)[input].shape, *out, std::move(op));
}

Value Graph::binary(BinaryOp bop, Value left, Value right) {
    Shape ls = (*this)[left].shape, rs = (*this)[right].shape;
    DType ld = (*this)[left].dtype, rd = (*this)[right].dtype;
    Shape result_shape = broadcast_shape_symmetric(ls, rs);
    if (ld != rd)
        fail("Binary operation ", binary_op_name(bop), " requires matching dtypes, got ", dtype_name(ld), " and ",
             dtype_name(rd));
    Specials s = dtype_specials(ld);
    bool skip = false;
    switch (bop) {
        case BinaryOp::Sub: case BinaryOp::Add: skip = is_const_zero(right); break;
        case BinaryOp::Mul: case BinaryOp::Div: case BinaryOp::Pow: skip = is_const_one(right); break;
        case BinaryOp::Min: skip = is_const_filled_with(right, s.max); break;
        case BinaryOp::Max: skip = is_const_filled_with(right, s.min); break;
    }
    if (skip) return left;
    Value l = broadcast(left, result_shape);
    Value r = broadcast(right, result_shape);
    Operation op;
    op.kind = OpKind::Binary;
    op.inputs = {l, r};
    op.binary = bop;
    return push(result_shape, ld, std::move(op));
}

std::vector<Value> Graph::call(const Graph &other, const std::vector<Value> &ins) {
    if (ins.size() != other.inputs.size()) fail("Wrong number of inputs");
    for (size_t k = 0; k < ins.size(); k++)
        if ((*this)[ins[k]].shape != other[other.inputs[k]].shape) fail("Wrong input shape");
    std::vector<Value> map(other.values.size());
    for (Value ov = 0; ov < other.values.size(); ov++) {
        const ValueInfo &info = other.values[ov];
        if (info.operation.kind == OpKind::Input) {
            map[ov] = ins[info.operation.index];
        } else {
            Operation op = info.operation;
            for (Value &in : op.inputs) in = map[in];
            map[ov] = push(info.shape, info.dtype, std::move(op));
        }
    }
    std::vector<Value> result;
    for (Value o : other.outputs) result.push_back(map[o]);
    return result;
}

void Graph::output(Value v) {
    check_contains(v);
    outputs.push_back(v);
}

std::vector<Shape> Graph::input_shapes() const {
    std::vector<Shape> r;
    for (Value v : inputs) r.push_back(values[v].shape);
    return r;
}
std::vector<Shape> Graph::output_shapes() const {
    std::vector<Shape> r;
    for (Value v : outputs) r.push_back(values[v].shape);
    return r;
}

Shape broadcast_shape_symmetric(const Shape &left, const Shape &right) {
    size_t rank = std::max(left.rank(), right.rank());
    Shape l = Shape::ones(rank - left.rank()).concat(left);
    Shape r = Shape::ones(rank - right.rank()).concat(right);
    Shape result;
    for (size_t i = 0; i < rank; i++) {
        if (l.dims[i] == Size::one()) result.dims.push_back(r.dims[i]);
        else if (r.dims[i] == Size::one()) result.dims.push_back(l.dims[i]);
        else if (l.dims[i] == r.dims[i]) result.dims.push_back(l.dims[i]);
        else fail("Cannot broadcast ", l.dims[i].str(), " and ", r.dims[i].str(), " in shapes ", l.str(), " and ", r.str());
    }
    return result;
}

std::string Graph::str() const {
    std::ostringstream ss;
    ss << "Graph {\n  inputs: " << vec_str(inputs) << ",\n  outputs: " << vec_str(outputs) << ",\n  values: [\n";
    for (Value v = 0; v < values.size(); v++) {
        const ValueInfo &info = values[v];
        const Operation &op = info.operation;
        ss << "    Value(" << v << ") = " << info.shape.str() << " " << dtype_name(info.dtype) << " " << op_kind_name(op.kind);
        ss << " { inputs: " << vec_str(op.inputs);
        switch (op.kind) {
            case OpKind::Input: ss << ", index: " << op.index; break;
            case OpKind::Constant: ss << ", len: " << op.tensor.len(); break;
            case OpKind::Permute: ss << ", permutation: " << vec_str(op.axes); break;
            case OpKind::Slice: ss << ", axis: " << op.axis() << ", range: " << op.range.start << ":" << op.range.end << ":" << op.range.step; break;
            case OpKind::Flip: case OpKind::Gather: case OpKind::Concat: case OpKind::Softmax: ss << ", axis: " << op.axis(); break;
            case OpKind::Layernorm: ss << ", axis: " << op.axis() << ", eps: " << op.eps; break;
            case OpKind::Unary:
                ss << ", op: " << unary_op_name(op.unary);
                if (op.unary == UnaryOp::ValueCast || op.unary == UnaryOp::BitCast) ss << "(" << dtype_name(op.cast_to) << ")";
                break;
            case OpKind::Binary: ss << ", op: " << binary_op_name(op.binary); break;
            case OpKind::Reduce: ss << ", axes: " << vec_str(op.axes) << ", op: " << reduce_op_name(op.reduce); break;
            case OpKind::Conv:
                ss << ", kernel: " << op.conv.kernel_h << "x" << op.conv.kernel_w << ", stride: " << op.conv.stride_y << "x"
                   << op.conv.stride_x << ", padding: " << op.conv.padding_y << "x" << op.conv.padding_x;
                break;
            default: break;
        }
        ss << " }, uses: " << info.non_output_uses;
        if (!info.debug_id.empty()) ss << ", id: \"" << info.debug_id << "\"";
        ss << "\n";
    }
    ss << "  ],\n}\n";
    return ss.str();
}

// ------------------------------------------------------------------------------------------------ shape inference

ShapeMismatch infer_batch_size(const std::vector<Shape> &expected, const std::vector<ConcreteShape> &actual,
                               std::optional<uint64_t> *batch) {
    std::vector<Size> e;
    std::vector<size_t> a;
    for (auto &s : expected) e.insert(e.end(), s.dims.begin(), s.dims.end());
    for (auto &s : actual) a.insert(a.end(), s.begin(), s.end());
    *batch = std::nullopt;
    size_t n = std::min(e.size(), a.size());
    for (size_t k = 0; k < n; k++) {
        uint64_t factor = e[k].fixed_factor;
        uint32_t exp = e[k].batch_exp;
        if (exp == 0) {
            if (a[k] != factor) return ShapeMismatch::ConstantMismatch;
        } else if (*batch) {
            if (a[k] != e[k].eval(**batch)) return ShapeMismatch::BatchConflict;
        } else {
            uint64_t approx = (uint64_t) std::pow((double) a[k] / (double) factor, 1.0 / (double) exp);
            bool found = false;
            for (int delta : {0, 1, -1, 2, -2}) {
                if (delta < 0 && approx < (uint64_t) -delta) continue;
                uint64_t cand = approx + delta;
                if (Size(exp, factor).eval(cand) == a[k]) {
                    *batch = cand;
                    found = true;
                    break;
                }
            }
            if (!found) return ShapeMismatch::ImpossibleBatchValue;
        }
    }
    if (e.size() != a.size()) return ShapeMismatch::DifferentLength;
    return ShapeMismatch::None;
}

}  // namespace kn
