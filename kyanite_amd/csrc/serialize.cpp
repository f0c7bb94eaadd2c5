// Flat binary form of a Graph. This is what a host language hands across the C ABI: it can be produced by
// walking the public `Graph::values()` / `graph[value]` API of the reference (graph.rs:354-361, :391-394).
//
// Layout (little endian):
//   u32 magic 'KNHG', u32 version
//   u32 value_count, then per value:
//     u8 dtype, u32 rank, rank x (u64 fixed_factor, u32 batch_exp), u8 op kind, op payload, u32 debug_id_len, bytes
//   u32 input_count, input values; u32 output_count, output values
// Payloads:
//   Input: u32 index | Constant: u64 byte_count, raw dense row-major bytes | View, Broadcast: u32 input
//   Permute: u32 input, u32 n, n x u32 | Slice: u32 input, u32 axis, u64 start, u64 end, u64 step
//   Flip: u32 input, u32 axis | Gather: u32 input, u32 axis, u32 indices | Concat: u32 n, n x u32 input, u32 axis
//   Conv: u32 input, u32 filter, u64 x 8 (stride_y, stride_x, padding_y, padding_x, kernel_h, kernel_w, output_h, output_w)
//   MatMul: u32 left, u32 right | Unary: u32 input, u8 op, u8 cast dtype | Binary: u32 left, u32 right, u8 op
//   Softmax: u32 input, u32 axis | Layernorm: u32 input, u32 axis, f32 eps | Reduce: u32 input, u32 n, n x u32 axis, u8 op
#include "graph.h"

namespace kn {

static constexpr uint32_t MAGIC = 0x47484e4b;  // "KNHG"
static constexpr uint32_t VERSION = 1;

namespace {
struct Writer {
    std::vector<uint8_t> out;
    void raw(const void *p, size_t n) {
        const uint8_t *b = (const uint8_t *) p;
        out.insert(out.end(), b, b + n);
    }
    void u8(uint8_t v) { out.push_back(v); }
    void u32(uint64_t v) {
        KN_ASSERT(v <= 0xffffffffull);
        uint32_t x = (uint32_t) v;
        raw(&x, 4);
    }
    void u64(uint64_t v) { raw(&v, 8); }
    void f32(float v) { raw(&v, 4); }
};

struct Reader {
    const uint8_t *p;
    size_t len, pos = 0;
    void need(size_t n) {
        if (pos + n > len || pos + n < pos) fail("graph blob is truncated");
    }
    void raw(void *dst, size_t n) {
        need(n);
        std::memcpy(dst, p + pos, n);
        pos += n;
    }
    uint8_t u8() { uint8_t v; raw(&v, 1); return v; }
    uint32_t u32() { uint32_t v; raw(&v, 4); return v; }
    uint64_t u64() { uint64_t v; raw(&v, 8); return v; }
    float f32() { float v; raw(&v, 4); return v; }
};
}  // namespace

std::vector<uint8_t> Graph::serialize() const {
    Writer w;
    w.u32(MAGIC);
    w.u32(VERSION);
    w.u32(values.size());
    for (const ValueInfo &info : values) {
        const Operation &op = info.operation;
        w.u8((uint8_t) info.dtype);
        w.u32(info.shape.rank());
        for (const Size &d : info.shape.dims) {
            w.u64(d.fixed_factor);
            w.u32(d.batch_exp);
        }
        w.u8((uint8_t) op.kind);
        switch (op.kind) {
            case OpKind::Input: w.u32(op.index); break;
            case OpKind::Constant:
                w.u64(op.tensor.nbytes());
                w.raw(op.tensor.bytes(), op.tensor.nbytes());
                break;
            case OpKind::View: case OpKind::Broadcast: w.u32(op.inputs[0]); break;
            case OpKind::Permute:
                w.u32(op.inputs[0]);
                w.u32(op.axes.size());
                for (size_t a : op.axes) w.u32(a);
                break;
            case OpKind::Slice:
                w.u32(op.inputs[0]);
                w.u32(op.axis());
                w.u64(op.range.start);
                w.u64(op.range.end);
                w.u64(op.range.step);
                break;
            case OpKind::Flip: case OpKind::Softmax:
                w.u32(op.inputs[0]);
                w.u32(op.axis());
                break;
            case OpKind::Gather:
                w.u32(op.inputs[0]);
                w.u32(op.axis());
                w.u32(op.inputs[1]);
                break;
            case OpKind::Concat:
                w.u32(op.inputs.size());
                for (Value v : op.inputs) w.u32(v);
                w.u32(op.axis());
                break;
            case OpKind::Conv:
                w.u32(op.inputs[0]);
                w.u32(op.inputs[1]);
                for (size_t v : {op.conv.stride_y, op.conv.stride_x, op.conv.padding_y, op.conv.padding_x,
                                 op.conv.kernel_h, op.conv.kernel_w, op.conv.output_h, op.conv.output_w})
                    w.u64(v);
                break;
            case OpKind::MatMul:
                w.u32(op.inputs[0]);
                w.u32(op.inputs[1]);
                break;
            case OpKind::Unary:
                w.u32(op.inputs[0]);
                w.u8((uint8_t) op.unary);
                w.u8((uint8_t) op.cast_to);
                break;
            case OpKind::Binary:
                w.u32(op.inputs[0]);
                w.u32(op.inputs[1]);
                w.u8((uint8_t) op.binary);
                break;
            case OpKind::Layernorm:
                w.u32(op.inputs[0]);
                w.u32(op.axis());
                w.f32(op.eps);
                break;
            case OpKind::Reduce:
                w.u32(op.inputs[0]);
                w.u32(op.axes.size());
                for (size_t a : op.axes) w.u32(a);
                w.u8((uint8_t) op.reduce);
                break;
        }
        w.u32(info.debug_id.size());
        w.raw(info.debug_id.data(), info.debug_id.size());
    }
    w.u32(inputs.size());
    for (Value v : inputs) w.u32(v);
    w.u32(outputs.size());
    for (Value v : outputs) w.u32(v);
    return std::move(w.out);
}

// Rebuilds the values exactly as written (no builder canonicalisation is re-run), checking every
// operand index, shape and dtype relation the executor later relies on.
namespace {

// What the builder methods of Graph guarantee about a value, checked for a value that comes out of a blob instead:
// the operation's axes and operands are in range and the stored shape and dtype are the ones the operation yields.
// The planner and the kernels index with these without looking again.
void check_value(const Graph &g, uint32_t vi, const Shape &shape, DType dtype, const Operation &op) {
    auto bad = [&](const char *what) { fail("graph blob: value ", vi, ": ", what); };
    auto in = [&](size_t k) -> const ValueInfo & { return g.values[op.inputs[k]]; };
    auto is_float = [](DType d) { return d == DType::F32 || d == DType::F16; };
    switch (op.kind) {
        case OpKind::Input: case OpKind::Constant: break;
        case OpKind::View:
            if (in(0).dtype != dtype || in(0).shape.size() != shape.size()) bad("view changes the dtype or the size");
            break;
        case OpKind::Broadcast: {
            const Shape &is = in(0).shape;
            if (in(0).dtype != dtype || is.rank() != shape.rank()) bad("broadcast changes the dtype or the rank");
            for (size_t a = 0; a < shape.rank(); a++)
                if (!(is.dims[a] == shape.dims[a] || is.dims[a] == Size::one())) bad("broadcast of an axis that is not 1");
            break;
        }
        case OpKind::Permute: {
            const Shape &is = in(0).shape;
            if (in(0).dtype != dtype || op.axes.size() != is.rank() || shape.rank() != is.rank()) bad("permutation rank mismatch");
            std::vector<bool> seen(is.rank(), false);
            for (size_t a = 0; a < op.axes.size(); a++) {
                if (op.axes[a] >= is.rank() || seen[op.axes[a]]) bad("not a permutation of the axes");
                seen[op.axes[a]] = true;
                if (shape.dims[a] != is.dims[op.axes[a]]) bad("permuted shape mismatch");
            }
            break;
        }
        case OpKind::Slice: {
            const Shape &is = in(0).shape;
            size_t axis = op.axes[0];
            if (in(0).dtype != dtype || axis >= is.rank() || !is.dims[axis].is_fixed()) bad("slice axis out of range or not fixed");
            op.range.assert_in_bounds(is.dims[axis].fixed_factor);
            size_t n = (op.range.end - op.range.start) / op.range.step;
            if (shape != is.replace(axis, Shape::fixed({n}))) bad("sliced shape mismatch");
            break;
        }
        case OpKind::Flip: case OpKind::Softmax: case OpKind::Layernorm:
            if (in(0).dtype != dtype || in(0).shape != shape || op.axes[0] >= shape.rank()) bad("axis out of range, or shape or dtype changed");
            if (op.kind != OpKind::Flip && !is_float(dtype)) bad("softmax and layernorm need f32 or f16");
            break;
        case OpKind::Gather: {
            const Shape &is = in(0).shape;
            const ValueInfo &idx = in(1);
            size_t axis = op.axes[0];
            if (in(0).dtype != dtype || axis >= is.rank()) bad("gather axis out of range or dtype changed");
            if (idx.shape.rank() != 1 || !dtype_is_int(idx.dtype)) bad("gather indices must be a rank 1 integer value");
            if (shape != is.replace(axis, idx.shape)) bad("gathered shape mismatch");
            break;
        }
        case OpKind::Concat: {
            size_t axis = op.axes[0];
            if (axis >= shape.rank()) bad("concat axis out of range");
            Shape base = shape.replace(axis, Shape::fixed({0}));
            Size along = Size::zero();
            for (size_t k = 0; k < op.inputs.size(); k++) {
                if (in(k).dtype != dtype || in(k).shape.rank() != shape.rank() || in(k).shape.replace(axis, Shape::fixed({0})) != base)
                    bad("concat operand does not match the result off the axis");
                auto sum = along.add(in(k).shape.dims[axis]);
                if (!sum) bad("concat sizes do not add");
                along = *sum;
            }
            if (along != shape.dims[axis]) bad("concat size along the axis mismatch");
            break;
        }
        case OpKind::Conv: {
            const ConvDetails &d = op.conv;
            if (in(0).dtype != dtype || in(1).dtype != dtype) bad("conv operands must have the dtype of the result");
            if (d.kernel_h % 2 != 1 || d.kernel_w % 2 != 1) bad("conv kernel sizes must be odd");
            if (shape != Shape({d.batch_size, Size::fixed(d.output_channels), Size::fixed(d.output_h), Size::fixed(d.output_w)}))
                bad("conv output shape mismatch");
            break;
        }
        case OpKind::MatMul: {
            const Shape &l = in(0).shape, &r = in(1).shape;
            if (in(0).dtype != dtype || in(1).dtype != dtype) bad("matmul operands must have the dtype of the result");
            if (l.rank() != 3 || r.rank() != 3 || l.dims[0] != r.dims[0] || l.dims[2] != r.dims[1]) bad("matmul operand shapes mismatch");
            if (shape != Shape({l.dims[0], l.dims[1], r.dims[2]})) bad("matmul output shape mismatch");
            break;
        }
        case OpKind::Unary: {
            auto out = unary_output_dtype(op.unary, in(0).dtype, op.cast_to);
            if (!out || *out != dtype || in(0).shape != shape) bad("unary operation does not yield this dtype and shape");
            break;
        }
        case OpKind::Binary:
            if (in(0).dtype != dtype || in(1).dtype != dtype || in(0).shape != shape || in(1).shape != shape)
                bad("binary operands must have the shape and dtype of the result");
            break;
        case OpKind::Reduce:
            if (in(0).dtype != dtype || op.axes.empty()) bad("reduce changes the dtype or has no axes");
            if (op.reduce == ReduceOp::Mean && !is_float(dtype)) bad("mean needs f32 or f16");
            if (shape != in(0).shape.replace_all(op.axes, Shape())) bad("reduced shape mismatch");  // checks range and uniqueness
            break;
    }
}

}  // namespace

Graph Graph::deserialize(const uint8_t *data, size_t len) {
    Reader r{data, len};
    if (r.u32() != MAGIC) fail("graph blob has a wrong magic number");
    if (r.u32() != VERSION) fail("graph blob has an unsupported version");
    Graph g;
    uint32_t count = r.u32();
    for (uint32_t vi = 0; vi < count; vi++) {
        uint8_t dt = r.u8();
        if (!dtype_valid(dt)) fail("graph blob: invalid dtype ", (int) dt);
        DType dtype = (DType) dt;
        uint32_t rank = r.u32();
        if (rank > 64) fail("graph blob: unreasonable rank ", rank);
        Shape shape;
        for (uint32_t k = 0; k < rank; k++) {
            uint64_t factor = r.u64();
            uint32_t exp = r.u32();
            shape.dims.push_back(Size(exp, factor));
        }
        uint8_t kind_code = r.u8();
        if (kind_code > (uint8_t) OpKind::Reduce) fail("graph blob: invalid operation kind ", (int) kind_code);
        Operation op;
        op.kind = (OpKind) kind_code;
        auto operand = [&]() {
            uint32_t v = r.u32();
            if (v >= vi) fail("graph blob: operand ", v, " of value ", vi, " is not an earlier value");
            return (Value) v;
        };
        switch (op.kind) {
            case OpKind::Input:
                op.index = r.u32();
                if (op.index != g.inputs.size()) fail("graph blob: inputs must be numbered in order");
                break;
            case OpKind::Constant: {
                uint64_t nbytes = r.u64();
                ConcreteShape dims = shape.unwrap_fixed("constant shape");
                if (nbytes != concrete_size(dims) * dtype_bytes(dtype)) fail("graph blob: constant byte count mismatch");
                r.need(nbytes);
                op.tensor = HostTensor(dtype, dims, r.p + r.pos);
                r.pos += nbytes;
                break;
            }
            case OpKind::View: case OpKind::Broadcast: op.inputs = {operand()}; break;
            case OpKind::Permute: {
                op.inputs = {operand()};
                uint32_t n = r.u32();
                if (n != rank) fail("graph blob: permutation rank mismatch");
                for (uint32_t k = 0; k < n; k++) op.axes.push_back(r.u32());
                break;
            }
            case OpKind::Slice:
                op.inputs = {operand()};
                op.axes = {r.u32()};
                op.range.start = r.u64();
                op.range.end = r.u64();
                op.range.step = r.u64();
                op.range.assert_valid();
                break;
            case OpKind::Flip: case OpKind::Softmax:
                op.inputs = {operand()};
                op.axes = {r.u32()};
                break;
            case OpKind::Gather: {
                Value in = operand();
                op.axes = {r.u32()};
                Value idx = operand();
                op.inputs = {in, idx};
                break;
            }
            case OpKind::Concat: {
                uint32_t n = r.u32();
                for (uint32_t k = 0; k < n; k++) op.inputs.push_back(operand());
                op.axes = {r.u32()};
                break;
            }
            case OpKind::Conv: {
                Value in = operand(), f = operand();
                op.inputs = {in, f};
                ConvDetails &d = op.conv;
                d.stride_y = r.u64(); d.stride_x = r.u64(); d.padding_y = r.u64(); d.padding_x = r.u64();
                d.kernel_h = r.u64(); d.kernel_w = r.u64(); d.output_h = r.u64(); d.output_w = r.u64();
                const Shape &is = g.values[in].shape;
                const Shape &fs = g.values[f].shape;
                if (is.rank() != 4 || fs.rank() != 4 || rank != 4) fail("graph blob: conv operands must have rank 4");
                d.dtype = dtype;
                d.batch_size = is.dims[0];
                d.input_channels = is.dims[1].unwrap_fixed("Conv input channels");
                d.input_h = is.dims[2].unwrap_fixed("Conv input height");
                d.input_w = is.dims[3].unwrap_fixed("Conv input width");
                d.output_channels = fs.dims[0].unwrap_fixed("Conv output channels");
                if (d.stride_y == 0 || d.stride_x == 0) fail("graph blob: conv stride cannot be 0");
                if (fs.dims[1] != Size::fixed(d.input_channels) || fs.dims[2] != Size::fixed(d.kernel_h) ||
                    fs.dims[3] != Size::fixed(d.kernel_w))
                    fail("graph blob: conv filter shape mismatch");
                size_t ph = d.input_h + 2 * d.padding_y, pw = d.input_w + 2 * d.padding_x;
                if (ph < d.kernel_h || pw < d.kernel_w || d.output_h != (ph - d.kernel_h) / d.stride_y + 1 ||
                    d.output_w != (pw - d.kernel_w) / d.stride_x + 1)
                    fail("graph blob: conv output size mismatch");
                break;
            }
            case OpKind::MatMul: {
                Value a = operand(), b = operand();
                op.inputs = {a, b};
                break;
            }
            case OpKind::Unary: {
                op.inputs = {operand()};
                uint8_t u = r.u8(), c = r.u8();
                if (u >= UNARY_OP_COUNT || !dtype_valid(c)) fail("graph blob: invalid unary operation");
                op.unary = (UnaryOp) u;
                op.cast_to = (DType) c;
                break;
            }
            case OpKind::Binary: {
                Value a = operand(), b = operand();
                op.inputs = {a, b};
                uint8_t bo = r.u8();
                if (bo >= BINARY_OP_COUNT) fail("graph blob: invalid binary operation");
                op.binary = (BinaryOp) bo;
                break;
            }
            case OpKind::Layernorm:
                op.inputs = {operand()};
                op.axes = {r.u32()};
                op.eps = r.f32();
                break;
            case OpKind::Reduce: {
                op.inputs = {operand()};
                uint32_t n = r.u32();
                for (uint32_t k = 0; k < n; k++) op.axes.push_back(r.u32());
                uint8_t ro = r.u8();
                if (ro >= REDUCE_OP_COUNT) fail("graph blob: invalid reduce operation");
                op.reduce = (ReduceOp) ro;
                break;
            }
        }
        uint32_t id_len = r.u32();
        r.need(id_len);
        std::string debug_id((const char *) r.p + r.pos, id_len);
        r.pos += id_len;

        check_value(g, vi, shape, dtype, op);
        bool is_input = op.kind == OpKind::Input;
        size_t before = g.values.size();
        Value v = g.push(shape, dtype, std::move(op));
        if (g.values.size() == before) fail("graph blob: value ", vi, " duplicates value ", v);
        g.values[v].debug_id = debug_id;
        if (is_input) g.inputs.push_back(v);
    }
    uint32_t n_in = r.u32();
    if (n_in != g.inputs.size()) fail("graph blob: input list does not match the Input values");
    for (uint32_t k = 0; k < n_in; k++)
        if (r.u32() != g.inputs[k]) fail("graph blob: input list does not match the Input values");
    uint32_t n_out = r.u32();
    for (uint32_t k = 0; k < n_out; k++) {
        uint32_t v = r.u32();
        if (v >= g.values.size()) fail("graph blob: output ", v, " out of range");
        g.outputs.push_back(v);
    }
    if (r.pos != len) fail("graph blob has trailing bytes");
    return g;
}

}  // namespace kn
