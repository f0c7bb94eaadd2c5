// The graph IR and its canonicalising builder.
// Mirrors kn-graph/src/graph.rs: Operation :106-162, Graph :77-84 and the builder methods :535-1363.
#pragma once

#include <unordered_map>

#include "dtype.h"
#include "shape.h"

namespace kn {

using Value = uint32_t;  // index into Graph::values, values are append-only and topologically ordered

// Codes are part of the serialised format and the C ABI.
enum class OpKind : uint8_t {
    Input = 0, Constant = 1, View = 2, Broadcast = 3, Permute = 4, Slice = 5, Flip = 6, Gather = 7,
    Concat = 8, Conv = 9, MatMul = 10, Unary = 11, Binary = 12, Softmax = 13, Layernorm = 14, Reduce = 15,
};

enum class UnaryOp : uint8_t {
    Abs = 0, Neg = 1, Sin = 2, Cos = 3, Exp = 4, Log = 5, Sqrt = 6, Sigmoid = 7, Tanh = 8, Erf = 9, Mish = 10,
    Softplus = 11, ValueCast = 12, BitCast = 13,
};
constexpr int UNARY_OP_COUNT = 14;

enum class BinaryOp : uint8_t { Add = 0, Sub = 1, Mul = 2, Div = 3, Min = 4, Max = 5, Pow = 6 };
constexpr int BINARY_OP_COUNT = 7;

enum class ReduceOp : uint8_t { Sum = 0, Mean = 1, Prod = 2, Max = 3, Min = 4 };
constexpr int REDUCE_OP_COUNT = 5;

const char *op_kind_name(OpKind k);
const char *unary_op_name(UnaryOp op);
const char *binary_op_name(BinaryOp op);
const char *reduce_op_name(ReduceOp op);

struct SliceRange {
    size_t start = 0, end = 0, step = 1;
    bool operator==(const SliceRange &o) const { return start == o.start && end == o.end && step == o.step; }
    static SliceRange make(size_t start, size_t end, size_t step);  // validated, graph.rs:1550-1554
    static SliceRange single(size_t index) { return make(index, index + 1, 1); }
    void assert_valid() const;                   // graph.rs:1568-1583
    void assert_in_bounds(size_t size) const;    // graph.rs:1585-1594
};

struct ConvDetails {  // graph.rs:313-330
    DType dtype = DType::F32;
    Size batch_size;
    size_t input_channels = 0, output_channels = 0;
    size_t input_h = 0, input_w = 0, kernel_h = 0, kernel_w = 0;
    size_t stride_y = 1, stride_x = 1, padding_y = 0, padding_x = 0;
    size_t output_h = 0, output_w = 0;

    bool keeps_spatial_shape() const { return input_h == output_h && input_w == output_w; }
    bool has_stride() const { return stride_y != 1 || stride_x != 1; }
    bool operator==(const ConvDetails &o) const;
};

// One flat record instead of a Rust enum: `kind` says which fields are meaningful.
struct Operation {
    OpKind kind = OpKind::Input;
    std::vector<Value> inputs;  // operands in the order graph.rs:220-251 lists them
    size_t index = 0;           // Input
    HostTensor tensor;          // Constant
    std::vector<size_t> axes;   // Permute: permutation; Slice/Flip/Gather/Concat/Softmax/Layernorm: {axis}; Reduce: axes
    SliceRange range;           // Slice
    ConvDetails conv;           // Conv
    UnaryOp unary = UnaryOp::Abs;
    DType cast_to = DType::F32;  // Unary ValueCast / BitCast target
    BinaryOp binary = BinaryOp::Add;
    ReduceOp reduce = ReduceOp::Sum;
    float eps = 0;  // Layernorm

    size_t axis() const { return axes.at(0); }
    bool equals(const Operation &o) const;
    uint64_t hash() const;
};

struct ValueInfo {
    Shape shape;
    DType dtype;
    Operation operation;
    std::string debug_id;
    size_t non_output_uses = 0;
};

class Graph {
public:
    std::vector<ValueInfo> values;
    std::vector<Value> inputs;
    std::vector<Value> outputs;

    const ValueInfo &operator[](Value v) const {
        check_contains(v);
        return values[v];
    }
    void check_contains(Value v) const {
        if (v >= values.size()) fail("Value ", v, " does not belong to this graph");
    }
    size_t len() const { return values.size(); }

    bool is_hidden(Value v) const;                           // graph.rs:416-419
    bool is_hidden_with_uses(Value v, size_t users) const;   // graph.rs:421-423
    bool is_const(Value v) const;                            // graph.rs:425-432
    std::optional<DScalar> as_single_const(Value v) const;   // graph.rs:490-527
    bool is_const_filled_with(Value v, const DScalar &expected) const;
    bool is_const_zero(Value v) const { return is_const_filled_with(v, dtype_specials((*this)[v].dtype).zero); }
    bool is_const_one(Value v) const { return is_const_filled_with(v, dtype_specials((*this)[v].dtype).one); }
    // graph.rs:435-474 restricted to what the optimizer needs: layout operations, gather, concat,
    // unary, binary and reduce are folded; conv, matmul, softmax and layernorm are not.
    std::optional<HostTensor> as_const(Value v) const;

    Value push(Shape shape, DType dtype, Operation operation);  // graph.rs:535-574 (deduplicating)
    void set_debug_id(Value v, std::string id);

    Value input(Shape shape, DType dtype);
    Value constant_tensor(HostTensor tensor);
    Value constant(const Shape &shape, DType dtype, const void *data);
    Value scalar_dyn(const DScalar &value);
    Value view(Value input, const Shape &new_shape);
    Value broadcast(Value input, const Shape &new_shape);
    Value repeat_unary(Value input, size_t axis, Size count);
    Value flatten(Value input, size_t start_axis);
    Value permute(Value input, std::vector<size_t> permutation);
    Value slice(Value input, size_t axis, SliceRange range);
    Value index(Value input, size_t axis, size_t index);
    Value flip(Value input, size_t axis);
    Value repeat(Value input, size_t axis, Size count);
    Value repeat_interleave(Value input, size_t axis, Size count);
    Value gather(Value input, size_t axis, Value indices);
    Value concat(std::vector<Value> inputs, size_t axis, const std::optional<Shape> &base_shape,
                 std::optional<DType> dtype);
    Value pad(Value input, const std::vector<std::pair<size_t, size_t>> &pad_amount, Value pad_value);
    Value conv(Value input, Value filter, size_t stride_y, size_t stride_x, size_t padding_y, size_t padding_x);
    Value linear(Value input, Value weight);
    Value mat_mul(Value left, Value right);
    Value batched_mat_mul(Value left, Value right);
    Value softmax(Value input, size_t axis);
    Value layernorm(Value input, size_t axis, float eps);
    Value reduce(Value input, std::vector<size_t> axes, ReduceOp op);
    Value sigmoid(Value input);
    Value relu(Value input);
    Value clamp_dyn(Value input, const DScalar &min, const DScalar &max);
    Value unary(UnaryOp op, Value input, DType cast_to = DType::F32);
    Value binary(BinaryOp op, Value left, Value right);
    Value add(Value l, Value r) { return binary(BinaryOp::Add, l, r); }
    Value sub(Value l, Value r) { return binary(BinaryOp::Sub, l, r); }
    Value mul(Value l, Value r) { return binary(BinaryOp::Mul, l, r); }
    Value pow(Value l, Value r) { return binary(BinaryOp::Pow, l, r); }
    std::vector<Value> call(const Graph &other, const std::vector<Value> &inputs);  // graph.rs:1319-1351
    void output(Value v);

    std::vector<Shape> input_shapes() const;
    std::vector<Shape> output_shapes() const;
    std::string str() const;

    // Flat little-endian binary form that crosses the C ABI; values stay in topological order.
    std::vector<uint8_t> serialize() const;
    static Graph deserialize(const uint8_t *data, size_t len);

private:
    Value repeat_impl(Value input, size_t axis, Size count, bool inner);
    std::unordered_multimap<uint64_t, Value> back_map_;
};

Shape broadcast_shape_symmetric(const Shape &left, const Shape &right);  // graph.rs:1431-1448

// Scalar semantics of the elementwise and reduce operations (graph.rs:1597-1815).
std::optional<DType> unary_output_dtype(UnaryOp op, DType x, DType cast_to);
DScalar unary_map(UnaryOp op, DType cast_to, const DScalar &x);
DScalar binary_map(BinaryOp op, const DScalar &l, const DScalar &r);
DScalar reduce_identity(ReduceOp op, DType dtype);
double erf_approx(double x);

}  // namespace kn
