// Host-side folding of constant sub-graphs, used while building and optimizing graphs
// (the role `Graph::as_const` plays at kn-graph/src/graph.rs:435-474). Only cheap operations are folded:
// layout operations, gather, concat, unary, binary and reduce. Conv, matmul, softmax and layernorm over
// constants are left alone (the result is "not a constant"), so no numerical kernel runs on the host.
#include <functional>

#include "graph.h"

namespace kn {

namespace {

// Materialise a strided view of `src` (element strides, element offset) as a dense tensor.
HostTensor strided_to_dense(const HostTensor &src, const std::vector<size_t> &shape,
                            const std::vector<int64_t> &strides, int64_t offset) {
    HostTensor out(src.dtype, shape);
    size_t es = dtype_bytes(src.dtype);
    size_t n = out.len();
    if (n == 0) return out;
    size_t rank = shape.size();
    std::vector<size_t> idx(rank, 0);
    const uint8_t *sp = src.bytes();
    uint8_t *dp = out.bytes_mut();
    int64_t cur = offset;
    for (size_t flat = 0; flat < n; flat++) {
        std::memcpy(dp + flat * es, sp + cur * (int64_t) es, es);
        for (size_t a = rank; a-- > 0;) {
            idx[a]++;
            cur += strides[a];
            if (idx[a] < shape[a]) break;
            cur -= strides[a] * (int64_t) shape[a];
            idx[a] = 0;
        }
    }
    return out;
}

std::vector<int64_t> dense_strides(const std::vector<size_t> &shape) {
    std::vector<int64_t> s(shape.size());
    int64_t next = 1;
    for (size_t a = shape.size(); a-- > 0;) {
        s[a] = next;
        next *= (int64_t) shape[a];
    }
    return s;
}

}  // namespace

std::optional<HostTensor> Graph::as_const(Value root) const {
    check_contains(root);
    if (!is_const(root)) return std::nullopt;

    std::unordered_map<Value, std::optional<HostTensor>> cache;
    std::vector<Value> stack{root};
    while (!stack.empty()) {
        Value v = stack.back();
        if (cache.count(v)) {
            stack.pop_back();
            continue;
        }
        const ValueInfo &info = values[v];
        const Operation &op = info.operation;
        bool missing = false;
        for (Value in : op.inputs) {
            if (!cache.count(in)) {
                stack.push_back(in);
                missing = true;
            }
        }
        if (missing) continue;
        stack.pop_back();

        bool operand_failed = false;
        for (Value in : op.inputs) operand_failed |= !cache[in].has_value();
        auto shape_opt = info.shape.as_fixed();
        if (operand_failed || !shape_opt) {
            cache[v] = std::nullopt;
            continue;
        }
        const ConcreteShape &out_shape = *shape_opt;
        auto arg = [&](size_t k) -> const HostTensor & { return *cache[op.inputs[k]]; };

        std::optional<HostTensor> result;
        switch (op.kind) {
            case OpKind::Input: break;
            case OpKind::Constant: result = op.tensor; break;
            case OpKind::View: result = arg(0).reshape(out_shape); break;
            case OpKind::Broadcast: {
                const HostTensor &x = arg(0);
                auto st = dense_strides(x.shape);
                for (size_t a = 0; a < st.size(); a++)
                    if (x.shape[a] != out_shape[a]) st[a] = 0;
                result = strided_to_dense(x, out_shape, st, 0);
                break;
            }
            case OpKind::Permute: {
                const HostTensor &x = arg(0);
                auto st = dense_strides(x.shape);
                std::vector<int64_t> ps;
                for (size_t a : op.axes) ps.push_back(st[a]);
                result = strided_to_dense(x, out_shape, ps, 0);
                break;
            }
            case OpKind::Slice: {
                const HostTensor &x = arg(0);
                auto st = dense_strides(x.shape);
                int64_t offset = concrete_size(out_shape) ? st[op.axis()] * (int64_t) op.range.start : 0;
                st[op.axis()] *= (int64_t) op.range.step;
                result = strided_to_dense(x, out_shape, st, offset);
                break;
            }
            case OpKind::Flip: {
                const HostTensor &x = arg(0);
                auto st = dense_strides(x.shape);
                size_t a = op.axis();
                int64_t offset = x.len() ? st[a] * (int64_t) (x.shape[a] - 1) : 0;
                st[a] = -st[a];
                result = strided_to_dense(x, out_shape, st, offset);
                break;
            }
            case OpKind::Gather: {
                const HostTensor &x = arg(0);
                const HostTensor &idx = arg(1);
                size_t a = op.axis();
                HostTensor out(x.dtype, out_shape);
                size_t es = dtype_bytes(x.dtype);
                size_t outer = 1, inner = 1;
                for (size_t k = 0; k < a; k++) outer *= x.shape[k];
                for (size_t k = a + 1; k < x.rank(); k++) inner *= x.shape[k];
                size_t n_idx = idx.len();
                bool ok = true;
                for (size_t o = 0; o < outer && ok; o++) {
                    for (size_t j = 0; j < n_idx; j++) {
                        DScalar s = idx.at(j);
                        int64_t i = s.is_signed_int() ? s.i : (int64_t) s.u;
                        if (i < 0 || (size_t) i >= x.shape[a]) {
                            ok = false;
                            break;
                        }
                        std::memcpy(out.bytes_mut() + ((o * n_idx + j) * inner) * es,
                                    x.bytes() + ((o * x.shape[a] + (size_t) i) * inner) * es, inner * es);
                    }
                }
                if (ok) result = out;
                break;
            }
            case OpKind::Concat: {
                size_t a = op.axis();
                HostTensor out(info.dtype, out_shape);
                size_t es = dtype_bytes(info.dtype);
                size_t outer = 1, inner = 1;
                for (size_t k = 0; k < a; k++) outer *= out_shape[k];
                for (size_t k = a + 1; k < out_shape.size(); k++) inner *= out_shape[k];
                size_t start = 0;
                for (size_t k = 0; k < op.inputs.size(); k++) {
                    const HostTensor &x = arg(k);
                    size_t len = x.shape[a];
                    for (size_t o = 0; o < outer; o++)
                        std::memcpy(out.bytes_mut() + ((o * out_shape[a] + start) * inner) * es,
                                    x.bytes() + (o * len * inner) * es, len * inner * es);
                    start += len;
                }
                result = out;
                break;
            }
            case OpKind::Unary: {
                const HostTensor &x = arg(0);
                HostTensor out(info.dtype, out_shape);
                size_t n = out.len();
                for (size_t k = 0; k < n; k++) out.set(k, unary_map(op.unary, op.cast_to, x.at(k)));
                result = out;
                break;
            }
            case OpKind::Binary: {
                const HostTensor &l = arg(0);
                const HostTensor &r = arg(1);
                HostTensor out(info.dtype, out_shape);
                size_t n = out.len();
                for (size_t k = 0; k < n; k++) out.set(k, binary_map(op.binary, l.at(k), r.at(k)));
                result = out;
                break;
            }
            case OpKind::Reduce: {
                // sequential left fold along each lane, one axis at a time (cpu.rs:259-272, graph.rs:1770-1786)
                HostTensor curr = arg(0);
                BinaryOp bop = op.reduce == ReduceOp::Prod  ? BinaryOp::Mul
                               : op.reduce == ReduceOp::Min ? BinaryOp::Min
                               : op.reduce == ReduceOp::Max ? BinaryOp::Max
                                                            : BinaryOp::Add;
                for (size_t a : op.axes) {
                    std::vector<size_t> ns = curr.shape;
                    size_t len = ns[a];
                    ns[a] = 1;
                    HostTensor next(curr.dtype, ns);
                    size_t outer = 1, inner = 1;
                    for (size_t k = 0; k < a; k++) outer *= curr.shape[k];
                    for (size_t k = a + 1; k < curr.rank(); k++) inner *= curr.shape[k];
                    for (size_t o = 0; o < outer; o++) {
                        for (size_t i = 0; i < inner; i++) {
                            DScalar acc = reduce_identity(op.reduce, curr.dtype);
                            for (size_t j = 0; j < len; j++) acc = binary_map(bop, acc, curr.at((o * len + j) * inner + i));
                            if (op.reduce == ReduceOp::Mean) acc = DScalar::f32((float) acc.f / (float) len);
                            next.set(o * inner + i, acc);
                        }
                    }
                    curr = next;
                }
                result = curr.reshape(out_shape);
                break;
            }
            case OpKind::Conv: case OpKind::MatMul: case OpKind::Softmax: case OpKind::Layernorm: break;
        }
        cache[v] = std::move(result);
    }
    return cache[root];
}

}  // namespace kn
