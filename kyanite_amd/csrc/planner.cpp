#include "planner.h"

#include <algorithm>
#include <cmath>
#include <map>

namespace kn {

const char *step_kind_name(StepKind k) {
    static const char *names[] = {"Conv", "MatMul", "ScalarOp", "ReduceOp", "SoftmaxOp", "LayernormOp", "GatherOp"};
    return names[(int) k];
}

namespace {
std::string conv_tail_note(const ConvParams &conv) {
    int parts = 1;
    const long long head = conv_tail_split(conv, &parts);
    if (parts <= 1) return std::string();
    return " [the tiles after " + std::to_string(head) + " in " + std::to_string(parts) + " slices of the input channels]";
}
}  // namespace

std::string Step::str() const {
    std::ostringstream ss;
    ss << step_kind_name(kind) << " value=" << debug_value;
    if (!debug_id.empty()) ss << " id=\"" << debug_id << "\"";
    if (kind == StepKind::MatMul && attention)
        ss << " attention " << (gemm_f16 ? "f16" : "f32") << (attention_has_mask ? (attention_has_classes ? " +mask (constant, classified by block)" : " +mask") : "") << " b=" << attn.batch << " lq=" << attn.lq << " lk=" << attn.lk << " dk=" << attn.dk << " dv=" << attn.dv
           << (gemm_f16 && attention_f16_shares_keys(attn) ? " [128 queries share each block of keys]" : "");
    else if (kind == StepKind::MatMul) {
        ss << (gemm_f16 ? " f16" : " f32") << " b=" << gemm.batch << " m=" << gemm.m << " n=" << gemm.n << " k=" << gemm.k
           << (gemm_has_addend ? " +add" : "") << (gemm_has_addend2 ? " +add" : "") << (gemm.relu ? " relu" : "");
        if (gemm.groups > 1) ss << " x" << gemm.groups << " grouped";
        if (gemm.pair_op) ss << " (x w_g) sigmoid(x w_g) (x w_u), n counts both";
        ss << " [" << describe_gemm_plan(plan_gemm_launch(gemm, gemm_f16), gemm_f16) << "]";
    }
    else if (kind == StepKind::Conv)
        ss << " n=" << conv.batch << " c=" << conv.in_c << "->" << conv.out_c << " hw=" << conv.in_h << "x" << conv.in_w << " k="
           << conv.kernel_h << "x" << conv.kernel_w << (conv_has_bias ? " +bias" : "") << (conv_has_res ? " +res" : "")
           << (conv.relu ? " relu" : "") << (conv_channel_split(conv) > 1 ? " [input channels in " + std::to_string(conv_channel_split(conv)) + " slices]" : std::string())
           << conv_tail_note(conv);
    else ss << " [" << kernel.strategy << "] grid=" << kernel.grid << "x" << kernel.block;
    ss << " operands:";
    for (auto &op : operands) ss << " " << dtype_name(op.tensor.dtype) << vec_str(op.tensor.shape.shape());
    return ss.str();
}

double Step::flops() const {
    if (kind == StepKind::MatMul && attention) return 2.0 * attn.batch * attn.lq * attn.lk * (attn.dk + attn.dv);
    if (kind == StepKind::MatMul) return 2.0 * gemm.batch * gemm.m * gemm.n * gemm.k * (gemm.groups > 1 ? gemm.groups : 1);
    if (kind == StepKind::Conv)
        return 2.0 * conv.batch * conv.out_c * conv.out_h * conv.out_w * conv.in_c * conv.kernel_h * conv.kernel_w;
    return 0.0;
}

double Step::bytes() const {
    double total = 0.0;
    for (size_t i = 0; i < operands.size(); i++) {
        // split-K scratch is not algorithmic traffic
        if (kind == StepKind::MatMul && !attention && i >= (gemm.pair_op ? 4u : gemm.groups > 1 ? 1u + 2u * (unsigned) gemm.groups : 3u + (gemm_has_addend ? 1u : 0u) + (gemm_has_addend2 ? 1u : 0u))) break;
        auto &op = operands[i];
        double elements = 1.0;
        const auto &shape = op.tensor.shape.shape();
        const auto &strides = op.tensor.shape.strides();
        for (size_t a = 0; a < shape.size(); a++)
            if (strides[a] != 0) elements *= (double) shape[a];
        total += elements * (double) dtype_bytes(op.tensor.dtype);
    }
    return total;
}

size_t Plan::resolve(const PlanPtr &ptr) const {
    size_t base;
    switch (ptr.kind) {
        case BufferKind::Constant: base = constant_offsets.at(ptr.index); break;
        case BufferKind::Zero: base = zero_offset; break;
        default:
            base = shared_offsets.at(ptr.index);
            if (base == SIZE_MAX) fail("Unused shared buffer ", ptr.index, " is actually used");
            break;
    }
    int64_t r = (int64_t) base + ptr.offset_bytes;
    KN_ASSERT(r >= 0);
    return (size_t) r;
}

namespace {

template <typename T>
struct Visit {
    bool ok;
    Value need;
    T value;
    static Visit done(T v) { return {true, 0, std::move(v)}; }
    static Visit missing(Value v) { return {false, v, T()}; }
};

#define KN_TRY(name, expr)                                          \
    auto name##_visit = (expr);                                     \
    if (!name##_visit.ok) return {false, name##_visit.need, {}};    \
    auto &name = name##_visit.value

// The expression under construction for one fused elementwise kernel (planner.rs:994-1060), with common
// sub-expressions computed once.
struct ScalarBlock {
    std::vector<PlanTensor> operands;  // operands[0] is reserved for the result
    ScalarExpr expr;
    std::map<Value, size_t> value_nodes;
    std::vector<std::optional<size_t>> loaded;  // per operand: the node that holds its loaded value
    // the layernorm / softmax whose result this block post-processes, or the reduction over the last axis whose
    // result it reads back broadcast along that axis (a mean of squares in an RMS norm)
    std::optional<Value> row_value;
    size_t row_node = 0;

    size_t load_operand(const PlanTensor &t) {
        for (size_t x = 1; x < operands.size(); x++) {
            if (operands[x] == t) return *loaded[x];
        }
        operands.push_back(t);
        ScalarNode n;
        n.kind = ScalarNode::Load;
        n.dtype = t.dtype;
        n.operand = operands.size() - 1;
        expr.nodes.push_back(n);
        loaded.push_back(expr.nodes.size() - 1);
        return expr.nodes.size() - 1;
    }
};

struct FusedRow {
    RowKernelDesc::Kind kind;
    ReduceOp reduce_op = ReduceOp::Sum;
    size_t axis;
    float eps;
    std::vector<PlanTensor> inputs;  // 1 or 2 tensors
    ScalarExpr pre;                  // Load operand indices are 1-based positions into `inputs`
};

class Planner {
public:
    Planner(const Graph &g, size_t batch, const PlannerOptions &o) : graph(g), batch_size(batch), options(o) {}

    const Graph &graph;
    size_t batch_size;
    PlannerOptions options;

    std::vector<size_t> shared_sizes;
    std::vector<HostTensor> constants;
    std::unordered_map<Value, PlanTensor> map;
    std::vector<Step> steps;

    using VT = Visit<PlanTensor>;

    PlanTensor visit_completely(Value value) {
        std::vector<Value> stack{value};
        while (true) {
            VT r = visit_single_cached(stack.back());
            if (r.ok) {
                stack.pop_back();
                if (stack.empty()) return r.value;
            } else {
                stack.push_back(r.need);
            }
        }
    }

    PlanTensor visit_completely_ensure_simple_strides(Value value) {
        visit_completely(value);
        VT r = visit_ensure_simple_strides(value);
        KN_ASSERT(r.ok);
        return r.value;
    }

    // (kernels are compiled when the whole plan stands: steps may still be joined until then)
    void compile_steps() {
        if (!options.compile) return;
        for (Step &step : steps)
            if (step.kind != StepKind::Conv && step.kind != StepKind::MatMul) step.code = compile_kernel(step.kernel.source);
    }

private:
    VT visit(Value value) {
        auto it = map.find(value);
        if (it != map.end()) return VT::done(it->second);
        return VT::missing(value);
    }

    void insert_mapping(Value value, const PlanTensor &t) {
        if (t.shape.shape() != graph[value].shape.eval(batch_size)) fail("Got wrong result shape for value ", value);
        bool inserted = map.emplace(value, t).second;
        KN_ASSERT(inserted);
    }

    VT visit_single_cached(Value value) {
        auto it = map.find(value);
        if (it != map.end()) return VT::done(it->second);
        KN_TRY(result, visit_single_new(value));
        const ValueInfo &info = graph[value];
        KN_ASSERT(result.dtype == info.dtype);
        // a fused conv or row kernel may already have registered this value
        if (!map.count(value)) insert_mapping(value, result);
        return VT::done(result);
    }

    bool can_fuse(Value v) const { return graph.is_hidden_with_uses(v, 1); }

    PlanPtr alloc_buffer_shared(size_t bytes) {
        shared_sizes.push_back(bytes);
        return PlanPtr{BufferKind::Shared, shared_sizes.size() - 1, 0};
    }

    PlanTensor alloc_tensor_shared(const ConcreteShape &shape, DType dtype) {
        PlanTensor t;
        t.ptr = alloc_buffer_shared(dtype_bytes(dtype) * concrete_size(shape));
        t.dtype = dtype;
        t.shape = StridedShape::simple(shape);
        return t;
    }

    // One launch, or two with partial results in between when the reduction has few results and much to read.
    void push_reduce(Value value, const PlanTensor &input, const PlanTensor &output, const std::vector<size_t> &axes,
                     ReduceOp rop, const ScalarExpr *pre) {
        ReduceSplit split;
        Step step;
        step.kind = StepKind::ReduceOp;
        step.kernel = make_reduce_kernel(kop(input), kop(output), axes, rop, pre, options.split_reduce ? &split : nullptr);
        if (split.parts <= 1) {
            step.operands = {{input, OperandKind::In}, {output, OperandKind::Out}};
            push(std::move(step), value);
            return;
        }
        PlanTensor partial = alloc_tensor_shared({split.parts * split.kept_size}, split.partial_dtype);
        step.operands = {{input, OperandKind::In}, {partial, OperandKind::Out}};
        push(std::move(step), value);
        Step fold;
        fold.kind = StepKind::ReduceOp;
        fold.kernel = std::move(split.final);
        fold.operands = {{partial, OperandKind::In}, {output, OperandKind::Out}};
        push(std::move(fold), value);
    }

    void push(Step step, Value debug_value) {
        step.debug_value = debug_value;
        step.debug_id = graph[debug_value].debug_id;
        if (step.kind != StepKind::Conv && step.kind != StepKind::MatMul) {
            if (step.kernel.grid == 0) return;  // nothing to compute (empty tensors)
            if (step.kind == StepKind::ScalarOp && !steps.empty() && try_join_elementwise(steps.back(), step)) return;
        }
        steps.push_back(std::move(step));
    }

    // Two elementwise steps in a row that walk the same shape and do not touch each other's tensors - the rotary
    // embeddings of q and of k - become one launch with the outputs of both: small kernels cost their launch and one
    // round trip to memory each, whatever they compute. Large ones, which run at the rate of the memory, stay apart.
    bool try_join_elementwise(Step &prev, const Step &next) {
        constexpr size_t max_elements = 1u << 22, max_outputs = 4, max_operands = 12;
        if (!options.join_elementwise || prev.kind != StepKind::ScalarOp || prev.scalar_exprs.empty() || next.scalar_exprs.empty()) return false;
        const auto &shape = prev.operands[0].tensor.shape.shape();
        if (next.operands[0].tensor.shape.shape() != shape || concrete_size(shape) > max_elements) return false;
        const size_t out_a = prev.scalar_exprs.size(), out_b = next.scalar_exprs.size();
        if (out_a + out_b > max_outputs) return false;
        auto same_buffer = [](const PlanTensor &x, const PlanTensor &y) { return x.ptr.kind == y.ptr.kind && x.ptr.index == y.ptr.index; };
        // neither reads or writes what the other writes
        for (size_t i = 0; i < prev.operands.size(); i++)
            for (size_t j = 0; j < next.operands.size(); j++)
                if ((i < out_a || j < out_b) && same_buffer(prev.operands[i].tensor, next.operands[j].tensor)) return false;
        std::vector<PlanTensor> operands;
        for (size_t i = 0; i < out_a; i++) operands.push_back(prev.operands[i].tensor);
        for (size_t j = 0; j < out_b; j++) operands.push_back(next.operands[j].tensor);
        const size_t n_out = out_a + out_b;
        std::vector<ScalarExpr> exprs;
        auto take = [&](const Step &from, size_t own_outputs) {
            for (ScalarExpr expr : from.scalar_exprs) {
                for (auto &node : expr.nodes) {
                    if (node.kind != ScalarNode::Load) continue;
                    KN_ASSERT(node.operand >= own_outputs && node.operand < from.operands.size());
                    const PlanTensor &t = from.operands[node.operand].tensor;
                    size_t at = n_out;
                    while (at < operands.size() && !(operands[at] == t)) at++;
                    if (at == operands.size()) operands.push_back(t);
                    node.operand = at;
                }
                exprs.push_back(std::move(expr));
            }
        };
        take(prev, out_a);
        take(next, out_b);
        if (operands.size() > max_operands) return false;
        std::vector<KernelOperand> kops;
        for (auto &t : operands) kops.push_back(kop(t));
        KernelSpec joined = make_scalar_kernel_multi(kops, exprs);
        if (joined.grid == 0) return false;
        prev.kernel = std::move(joined);
        prev.scalar_exprs = std::move(exprs);
        prev.operands.clear();
        for (size_t k = 0; k < operands.size(); k++) prev.operands.push_back({operands[k], k < n_out ? OperandKind::Out : OperandKind::In});
        return true;
    }

    static KernelOperand kop(const PlanTensor &t) { return KernelOperand{t.dtype, t.shape, t.ptr.offset_bytes}; }

    VT visit_single_new(Value value) {
        {
            auto fused = try_visit_fused_conv(value);
            if (!fused.ok) return VT::missing(fused.need);
            if (fused.value) return VT::done(*fused.value);
        }
        if (options.fuse_attention) {
            auto fused = try_visit_fused_attention(value);
            if (!fused.ok) return VT::missing(fused.need);
            if (fused.value) return VT::done(*fused.value);
        }
        if (options.fuse_matmul_epilogue) {
            auto fused = try_visit_fused_matmul(value);
            if (!fused.ok) return VT::missing(fused.need);
            if (fused.value) return VT::done(*fused.value);
        }
        if (options.fuse_gated_matmul) {
            auto fused = try_visit_gated_matmul(value);
            if (!fused.ok) return VT::missing(fused.need);
            if (fused.value) return VT::done(*fused.value);
        }
        const ValueInfo &info = graph[value];
        ConcreteShape result_shape = info.shape.eval(batch_size);
        DType result_dtype = info.dtype;
        const Operation &op = info.operation;

        switch (op.kind) {
            case OpKind::Input: return VT::done(alloc_tensor_shared(result_shape, result_dtype));
            case OpKind::Constant: {
                PlanTensor t;
                constants.push_back(op.tensor);
                t.ptr = PlanPtr{BufferKind::Constant, constants.size() - 1, 0};
                t.dtype = op.tensor.dtype;
                t.shape = StridedShape::simple(result_shape);
                return VT::done(t);
            }
            case OpKind::View: {
                KN_TRY(input, visit(op.inputs[0]));
                // try a pure stride edit, otherwise restride into a dense copy first
                if (auto v = input.view(result_shape)) return VT::done(*v);
                PlanTensor dense = alloc_tensor_shared(input.shape.shape(), input.dtype);
                plan_copy_tensor(input, dense, value);
                auto v = dense.view(result_shape);
                KN_ASSERT(v.has_value());
                return VT::done(*v);
            }
            case OpKind::Broadcast: {
                KN_TRY(input, visit(op.inputs[0]));
                return VT::done(input.broadcast(result_shape));
            }
            case OpKind::Permute: return visit_permute(op.inputs[0], op.axes);
            case OpKind::Slice: {
                KN_TRY(input, visit(op.inputs[0]));
                return VT::done(input.slice(op.axis(), op.range));
            }
            case OpKind::Flip: {
                KN_TRY(input, visit(op.inputs[0]));
                return VT::done(input.flip(op.axis()));
            }
            case OpKind::Gather: {
                KN_TRY(input, visit(op.inputs[0]));
                KN_TRY(indices, visit(op.inputs[1]));
                PlanTensor output = alloc_tensor_shared(result_shape, result_dtype);
                Step step;
                step.kind = StepKind::GatherOp;
                step.kernel = make_gather_kernel(kop(input), kop(indices), kop(output), op.axis());
                step.operands = {{input, OperandKind::In}, {indices, OperandKind::In}, {output, OperandKind::Out}};
                push(std::move(step), value);
                return VT::done(output);
            }
            case OpKind::Concat: {
                // planner.rs:394-412 copies every input into its slice of the result. An input that is an
                // elementwise chain nobody else uses is computed straight into its slice instead (one kernel
                // less per input and no intermediate buffer).
                struct Piece {
                    std::optional<PlanTensor> tensor;  // a materialised input, copied
                    std::optional<ScalarBlock> block;  // or a chain evaluated in place
                    Value value;
                };
                std::vector<Piece> pieces;
                for (Value x : op.inputs) {
                    Piece piece;
                    piece.value = x;
                    const OpKind kind = graph[x].operation.kind;
                    if (!map.count(x) && can_fuse(x) && (kind == OpKind::Unary || kind == OpKind::Binary)) {
                        ScalarBlock block;
                        block.operands.push_back(PlanTensor());  // placeholder for the result
                        block.loaded.push_back(std::nullopt);
                        auto root = visit_fused_scalar_recurse(x, block, true);
                        if (!root.ok) return VT::missing(root.need);
                        if (!block.row_value) piece.block = std::move(block);
                    }
                    if (!piece.block) {
                        KN_TRY(t, visit(x));
                        piece.tensor = t;
                    }
                    pieces.push_back(std::move(piece));
                }
                PlanTensor result = alloc_tensor_shared(result_shape, result_dtype);
                size_t axis = op.axis(), start = 0;
                // chains of the same shape (the two halves of a rotary embedding) share one launch and their loads
                struct Pending {
                    PlanTensor target;
                    ScalarBlock *block;
                    Value value;
                };
                std::vector<Pending> pending;
                auto flush = [&]() {
                    if (pending.empty()) return;
                    if (pending.size() == 1) {
                        pending[0].block->operands[0] = pending[0].target;
                        plan_scalar_op(pending[0].block->expr, pending[0].block->operands, pending[0].value);
                    } else {
                        const size_t n_out = pending.size();
                        std::vector<PlanTensor> operands;
                        for (auto &pd : pending) operands.push_back(pd.target);
                        std::vector<ScalarExpr> exprs;
                        for (auto &pd : pending) {
                            ScalarExpr expr = pd.block->expr;
                            for (auto &node : expr.nodes) {
                                if (node.kind != ScalarNode::Load) continue;
                                const PlanTensor &t = pd.block->operands[node.operand];
                                size_t at = n_out;
                                while (at < operands.size() && !(operands[at] == t)) at++;
                                if (at == operands.size()) operands.push_back(t);
                                node.operand = at;
                            }
                            exprs.push_back(std::move(expr));
                        }
                        std::vector<KernelOperand> kops;
                        for (auto &t : operands) kops.push_back(kop(t));
                        Step step;
                        step.kind = StepKind::ScalarOp;
                        step.kernel = make_scalar_kernel_multi(kops, exprs);
                        step.scalar_exprs = exprs;
                        for (size_t k = 0; k < operands.size(); k++)
                            step.operands.push_back({operands[k], k < n_out ? OperandKind::Out : OperandKind::In});
                        push(std::move(step), pending[0].value);
                    }
                    pending.clear();
                };
                for (auto &piece : pieces) {
                    size_t len = graph[piece.value].shape.eval(batch_size)[axis];
                    PlanTensor target = result.slice(axis, SliceRange{start, start + len, 1});
                    if (piece.block) {
                        if (!pending.empty() && (pending[0].target.shape.shape() != target.shape.shape() || pending.size() >= 4)) flush();
                        pending.push_back({target, &*piece.block, piece.value});
                    } else {
                        flush();
                        plan_copy_tensor(*piece.tensor, target, value);
                    }
                    start += len;
                }
                flush();
                return VT::done(result);
            }
            case OpKind::Conv: fail("Conv should have been handled by the conv fuser (only rank-4 f32 convolutions are supported)");
            case OpKind::MatMul: {
                if (options.group_matmuls) {
                    auto grouped = try_visit_matmul_group(value);
                    if (!grouped.ok) return VT::missing(grouped.need);
                    if (grouped.value) return VT::done(*grouped.value);
                }
                return visit_matmul(value, op.inputs[0], op.inputs[1], true);
            }
            case OpKind::Unary: case OpKind::Binary: return visit_fused_scalar(value);
            case OpKind::Softmax: case OpKind::Layernorm: {
                KN_ASSERT(result_dtype == DType::F32 || result_dtype == DType::F16);
                auto row = visit_row_inputs(value);
                if (!row.ok) return VT::missing(row.need);
                // no elementwise consumer was fused: the epilogue is the identity
                ScalarExpr post;
                ScalarNode n;
                n.kind = ScalarNode::Load;
                n.dtype = result_dtype;
                n.operand = SIZE_MAX;
                post.nodes.push_back(n);
                return VT::done(push_row_kernel(value, value, row.value, post, {}));
            }
            case OpKind::Reduce: {
                if (op.reduce == ReduceOp::Mean) KN_ASSERT(result_dtype == DType::F32 || result_dtype == DType::F16);
                // An elementwise chain of ONE tensor that only this reduction uses (the square in a mean of
                // squares) is evaluated on the loaded elements instead of being written out and read back.
                const Value in_v = op.inputs[0];
                const OpKind in_kind = graph[in_v].operation.kind;
                if (!map.count(in_v) && can_fuse(in_v) && (in_kind == OpKind::Unary || in_kind == OpKind::Binary)) {
                    ScalarBlock block;
                    block.operands.push_back(PlanTensor());  // placeholder for a result
                    block.loaded.push_back(std::nullopt);
                    auto root = visit_fused_scalar_recurse(in_v, block, true);
                    if (!root.ok) return VT::missing(root.need);
                    if (!block.row_value && block.operands.size() == 2) {
                        const PlanTensor &input = block.operands[1];
                        PlanTensor output = alloc_tensor_shared(result_shape, result_dtype);
                        push_reduce(value, input, output, op.axes, op.reduce, &block.expr);
                        return VT::done(output);
                    }
                }
                KN_TRY(input, visit(in_v));
                PlanTensor output = alloc_tensor_shared(result_shape, result_dtype);
                push_reduce(value, input, output, op.axes, op.reduce, nullptr);
                return VT::done(output);
            }
        }
        fail("unreachable");
    }

    // planner.rs:554-567
    VT visit_permute(Value input, const std::vector<size_t> &permutation) {
        if (can_fuse(input) && permutation == std::vector<size_t>{1, 0, 2} && !map.count(input)) {
            const Operation &iop = graph[input].operation;
            if (iop.kind == OpKind::MatMul) {
                if (options.fuse_attention) {
                    auto fused = try_visit_fused_attention(input, false);
                    if (!fused.ok) return VT::missing(fused.need);
                    if (fused.value) {
                        insert_mapping(input, *fused.value);
                        return VT::done(fused.value->permute(permutation));
                    }
                }
                // avoid a non-dense result for the typical attention matmul: write directly in [m, b, n] order
                KN_TRY(mm, visit_matmul(input, iop.inputs[0], iop.inputs[1], false));
                insert_mapping(input, mm);
                return VT::done(mm.permute(permutation));
            }
        }
        if (options.fuse_attention && can_fuse(input) && permutation == std::vector<size_t>{0, 2, 1, 3} && !map.count(input)) {
            // attention over [batch, heads] whose result goes back to [batch, tokens, heads, width] order: the
            // kernel stores in that order itself instead of a copy after it
            const Operation &vop = graph[input].operation;
            const Value mm = vop.kind == OpKind::View ? vop.inputs[0] : input;
            if (vop.kind == OpKind::View && graph[mm].operation.kind == OpKind::MatMul && can_fuse(mm) && !map.count(mm)) {
                const ConcreteShape split = graph[input].shape.eval(batch_size), flat = graph[mm].shape.eval(batch_size);
                if (split.size() == 4 && flat.size() == 3 && split[0] * split[1] == flat[0] && split[2] == flat[1] && split[3] == flat[2]) {
                    auto fused = try_visit_fused_attention(mm, true, split[1]);
                    if (!fused.ok) return VT::missing(fused.need);
                    if (fused.value) {
                        insert_mapping(input, *fused.value);
                        return VT::done(fused.value->permute(permutation));
                    }
                }
            }
        }
        KN_TRY(t, visit(input));
        return VT::done(t.permute(permutation));
    }

    // planner.rs:569-582
    VT visit_ensure_simple_strides(Value value) {
        KN_TRY(inner, visit(value));
        if (inner.shape.has_simple_strides()) return VT::done(inner);
        PlanTensor dense = alloc_tensor_shared(inner.shape.shape(), inner.dtype);
        plan_copy_tensor(inner, dense, value);
        return VT::done(dense);
    }

    // planner.rs:584-604: `alpha * x` with a single-valued constant alpha
    Visit<std::pair<std::optional<DScalar>, PlanTensor>> visit_scalable_value(Value value) {
        using R = Visit<std::pair<std::optional<DScalar>, PlanTensor>>;
        const Operation &op = graph[value].operation;
        if (op.kind == OpKind::Binary && op.binary == BinaryOp::Mul && !map.count(value)) {
            if (auto alpha = graph.as_single_const(op.inputs[0])) {
                auto t = visit(op.inputs[1]);
                if (!t.ok) return R::missing(t.need);
                return R::done({alpha, t.value});
            }
            if (auto alpha = graph.as_single_const(op.inputs[1])) {
                auto t = visit(op.inputs[0]);
                if (!t.ok) return R::missing(t.need);
                return R::done({alpha, t.value});
            }
        }
        auto t = visit(value);
        if (!t.ok) return R::missing(t.need);
        return R::done({std::nullopt, t.value});
    }

    // The operands and prologue of a softmax (planner.rs:418-441) or layernorm (:443-476, :522-552) value.
    Visit<FusedRow> visit_row_inputs(Value value) {
        using R = Visit<FusedRow>;
        const Operation &op = graph[value].operation;
        FusedRow row;
        row.axis = op.axis();
        row.eps = op.eps;
        const DType dt = graph[value].dtype;
        auto load = [&](size_t operand) {
            ScalarNode n;
            n.kind = ScalarNode::Load;
            n.dtype = dt;
            n.operand = operand;
            row.pre.nodes.push_back(n);
            return row.pre.nodes.size() - 1;
        };
        auto scaled = [&](const std::optional<DScalar> &alpha, size_t x) {
            if (!alpha) return x;
            ScalarNode c;
            c.kind = ScalarNode::Const;
            c.dtype = dt;
            c.constant = *alpha;
            row.pre.nodes.push_back(c);
            ScalarNode m;
            m.kind = ScalarNode::Binary;
            m.dtype = dt;
            m.binary = BinaryOp::Mul;
            m.a = x;
            m.b = row.pre.nodes.size() - 1;
            row.pre.nodes.push_back(m);
            return row.pre.nodes.size() - 1;
        };
        Value input = op.inputs[0];
        row.kind = op.kind == OpKind::Softmax ? RowKernelDesc::Softmax : RowKernelDesc::Layernorm;
        // `a0 * x0 + a1 * x1` in front of the row operation (planner.rs:522-604 for layernorm; here for softmax as
        // well, which covers `scale * scores + mask`); the operands may be laid out differently (a broadcast mask)
        // (a sum that something else uses as well is stored for that user anyway, bias or residual in the store of
        // the matmul that feeds it where that applies: the row kernel then reads the one tensor)
        const Operation &iop = graph[input].operation;
        if (iop.kind == OpKind::Binary && iop.binary == BinaryOp::Add && !map.count(input) && can_fuse(input)) {
            auto l = visit_scalable_value(iop.inputs[0]);
            if (!l.ok) return R::missing(l.need);
            auto r = visit_scalable_value(iop.inputs[1]);
            if (!r.ok) return R::missing(r.need);
            if (l.value.second.shape.shape() == r.value.second.shape.shape()) {
                row.inputs = {l.value.second, r.value.second};
                size_t a = scaled(l.value.first, load(1));
                size_t b = scaled(r.value.first, load(2));
                ScalarNode add;
                add.kind = ScalarNode::Binary;
                add.dtype = dt;
                add.binary = BinaryOp::Add;
                add.a = a;
                add.b = b;
                row.pre.nodes.push_back(add);
                return R::done(row);
            }
            auto total = visit(input);
            if (!total.ok) return R::missing(total.need);
            row.inputs = {total.value};
            load(1);
            return R::done(row);
        }
        auto sv = visit_scalable_value(input);
        if (!sv.ok) return R::missing(sv.need);
        row.inputs = {sv.value.second};
        scaled(sv.value.first, load(1));
        return R::done(row);
    }

    // A softmax or layernorm whose rows no workgroup can hold. The row kernel reads such a row again per pass, with
    // the one workgroup that owns it: a few rows of a million elements move at what a few compute units can pull
    // (8 rows of 4 Mi floats: 1.6 ms, 0.17 TB/s), and columns of a tall matrix in runs of 64 bytes per row of lanes
    // ([4096, 16384] along axis 0: 309 us). As two steps that each use the whole chip the tensor is read twice and
    // written once at the rate of the memory: the statistics of every row as a reduction that folds pairs (maximum
    // and sum of exponentials in one pass, or mean and variance; slices of the reduced index side by side when the
    // rows are few), then an elementwise kernel over (x, statistics) that also applies the epilogue.
    bool two_pass_rows_ok(const FusedRow &row, const KernelSpec &kernel, DType result_dtype, size_t rows,
                          const std::vector<PlanTensor> &extra) const {
        if (!options.split_reduce || (result_dtype != DType::F32 && result_dtype != DType::F16) || row.kind == RowKernelDesc::Reduce) return false;
        if (row.inputs.size() != 1 || row.pre.nodes.size() != 1 || row.inputs[0].dtype != result_dtype) return false;
        for (size_t k = 1; k < extra.size(); k++)
            if (extra[k].dtype != result_dtype) return false;
        if (kernel.row_access == KernelSpec::ColumnsStreamed) return true;
        // lanes along the rows: a workgroup per row is enough once there are four per compute unit
        return kernel.row_access == KernelSpec::RowsStreamed && rows < 1024;
    }

    void plan_two_pass_rows(Value value, const FusedRow &row, const PlanTensor &output, const ScalarExpr &post,
                            const std::vector<PlanTensor> &extra) {
        const PlanTensor &x = row.inputs[0];
        const std::vector<size_t> shape = x.shape.shape();
        const size_t axis = row.axis;
        std::vector<size_t> kept, unit = shape, planes{2};
        for (size_t a = 0; a < shape.size(); a++)
            if (a != axis) kept.push_back(shape[a]);
        unit[axis] = 1;
        planes.insert(planes.end(), kept.begin(), kept.end());
        const bool softmax = row.kind == RowKernelDesc::Softmax;

        // step 1: (maximum, 1 / sum of exponentials) or (mean, 1 / sqrt(variance + eps)) of every row, as two planes
        PlanTensor stats = alloc_tensor_shared(planes, DType::F32);
        auto plane = [&](size_t which) { return *stats.slice(0, SliceRange{which, which + 1, 1}).view(kept); };
        const PlanTensor first = plane(0), second = plane(1);
        ReduceStat stat;
        stat.kind = softmax ? ReduceStat::MaxSumExp : ReduceStat::MeanRstd;
        stat.eps = row.eps;
        stat.plane = concrete_size(kept);
        {
            ReduceSplit split;
            Step step;
            step.kind = StepKind::ReduceOp;
            step.kernel = make_reduce_kernel(kop(x), kop(first), {axis}, ReduceOp::Sum, nullptr, &split, &stat);
            step.kernel.strategy = std::string(softmax ? "maximum and sum of exponentials: " : "mean and variance: ") + step.kernel.strategy;
            if (split.parts <= 1) {
                step.operands = {{x, OperandKind::In}, {stats, OperandKind::Out}};
                push(std::move(step), value);
            } else {
                PlanTensor partial = alloc_tensor_shared({split.parts * split.kept_size * split.partial_words}, split.partial_dtype);
                step.operands = {{x, OperandKind::In}, {partial, OperandKind::Out}};
                push(std::move(step), value);
                Step fold;
                fold.kind = StepKind::ReduceOp;
                fold.kernel = std::move(split.final);
                fold.operands = {{partial, OperandKind::In}, {stats, OperandKind::Out}};
                push(std::move(fold), value);
            }
        }

        // step 2: post(exp(x - maximum) * (1 / sum)) or post((x - mean) * (1 / sqrt(variance + eps)))
        auto along = [&](const PlanTensor &s) { return s.view(unit)->broadcast(shape); };
        ScalarExpr expr;
        auto node = [&](ScalarNode::Kind kind) {
            ScalarNode n;
            n.kind = kind;
            n.dtype = DType::F32;
            return n;
        };
        auto push_node = [&](ScalarNode n) {
            expr.nodes.push_back(std::move(n));
            return expr.nodes.size() - 1;
        };
        auto load = [&](size_t operand) {
            ScalarNode n = node(ScalarNode::Load);
            n.operand = operand;
            return push_node(n);
        };
        auto binary = [&](BinaryOp op, size_t a, size_t b) {
            ScalarNode n = node(ScalarNode::Binary);
            n.binary = op;
            n.a = a;
            n.b = b;
            return push_node(n);
        };
        // (halves: computed in f32 from the loaded half and rounded once, like the row kernel's result)
        const DType dt = x.dtype;
        auto cast = [&](size_t a, DType to) {
            ScalarNode n = node(ScalarNode::Unary);
            n.unary = UnaryOp::ValueCast;
            n.cast_to = to;
            n.dtype = to;
            n.a = a;
            return push_node(n);
        };
        size_t lx = load(1);
        expr.nodes[lx].dtype = dt;
        if (dt != DType::F32) lx = cast(lx, DType::F32);
        const size_t la = load(2), lb = load(3);
        size_t centred = binary(BinaryOp::Sub, lx, la);
        if (softmax) {
            ScalarNode e = node(ScalarNode::Unary);
            e.unary = UnaryOp::Exp;
            e.a = centred;
            centred = push_node(e);
        }
        size_t normalised = binary(BinaryOp::Mul, centred, lb);
        if (dt != DType::F32) normalised = cast(normalised, dt);
        // the epilogue behind it: its loads of the normalised value become references to that node, its other loads
        // move behind (output, x, the two statistics)
        std::vector<PlanTensor> operands{output, x, along(first), along(second)};
        for (size_t k = 1; k < extra.size(); k++) operands.push_back(extra[k]);
        std::vector<size_t> at(post.nodes.size());
        for (size_t i = 0; i < post.nodes.size(); i++) {
            ScalarNode n = post.nodes[i];
            KN_ASSERT(n.kind != ScalarNode::Raw);
            if (n.kind == ScalarNode::Load && n.operand == SIZE_MAX) {
                at[i] = normalised;
                continue;
            }
            if (n.kind == ScalarNode::Load) n.operand = 4 + n.operand - 1;
            if (n.kind == ScalarNode::Unary || n.kind == ScalarNode::Binary) n.a = at[n.a];
            if (n.kind == ScalarNode::Binary) n.b = at[n.b];
            at[i] = push_node(n);
        }
        // (the result of an expression is its last node: the epilogue's, or the normalised value of an epilogue that
        // is nothing but that value)
        KN_ASSERT(at.back() == expr.nodes.size() - 1);
        plan_scalar_op(expr, operands, value);
    }

    // Emit the row kernel for `row_value`, storing `post(normalised, extra...)` as the result of `result_value`.
    // Load nodes of `post` index into `extra` (1-based, 0 is unused); SIZE_MAX is the normalised value.
    PlanTensor push_row_kernel(Value row_value, Value result_value, const FusedRow &row, const ScalarExpr &post_in,
                               const std::vector<PlanTensor> &extra) {
        const ValueInfo &info = graph[result_value];
        PlanTensor output = alloc_tensor_shared(info.shape.eval(batch_size), info.dtype);
        RowKernelDesc desc;
        desc.kind = row.kind;
        desc.reduce_op = row.reduce_op;
        desc.axis = row.axis;
        desc.eps = row.eps;
        // operand order: output, row inputs, epilogue operands
        std::vector<PlanTensor> all{output};
        for (auto &t : row.inputs) all.push_back(t);
        size_t extra_base = all.size();
        for (size_t k = 1; k < extra.size(); k++) all.push_back(extra[k]);
        for (auto &t : all) desc.operands.push_back(kop(t));
        desc.pre = row.pre;
        desc.post = post_in;
        for (auto &n : desc.post.nodes)
            if (n.kind == ScalarNode::Load && n.operand != SIZE_MAX) n.operand = extra_base + n.operand - 1;

        Step step;
        step.kind = row.kind == RowKernelDesc::Softmax ? StepKind::SoftmaxOp
                                                      : (row.kind == RowKernelDesc::Reduce ? StepKind::ReduceOp : StepKind::LayernormOp);
        step.kernel = make_row_kernel(desc);
        {
            const auto &full = output.shape.shape();
            const size_t rows = full[row.axis] == 0 ? 0 : concrete_size(full) / full[row.axis];
            if (two_pass_rows_ok(row, step.kernel, info.dtype, rows, extra)) {
                plan_two_pass_rows(row_value, row, output, post_in, extra);
                return output;
            }
        }
        step.operands.push_back({output, OperandKind::Out});
        for (size_t k = 1; k < all.size(); k++) step.operands.push_back({all[k], OperandKind::In});
        push(std::move(step), row_value);
        return output;
    }

    // planner.rs:606-648
    // Not in the reference (its matmuls are plain library calls): an elementwise tail of a matmul of the form
    //   max(., 0)?  <-  (. + d)?  <-  view*  <-  MatMul
    // whose intermediate values are hidden and used once is folded into the matmul's store, d being any tensor of
    // the result's shape (a broadcast bias, a residual). Returns nullopt when `value` is not such a tail.
    Visit<std::optional<PlanTensor>> try_visit_fused_matmul(Value value) {
        using R = Visit<std::optional<PlanTensor>>;
        const DType dt = graph[value].dtype;
        if (dt != DType::F32 && dt != DType::F16) return R::done(std::nullopt);
        Value curr = value;
        bool relu = false;
        {
            const Operation &op = graph[curr].operation;
            if (op.kind == OpKind::Binary && op.binary == BinaryOp::Max) {
                Value l = op.inputs[0], r = op.inputs[1];
                if (graph.is_const_zero(l)) curr = r;
                else if (graph.is_const_zero(r)) curr = l;
                else return R::done(std::nullopt);
                if (!can_fuse(curr)) return R::done(std::nullopt);
                relu = true;
            }
        }
        // through views down to the matmul, as long as every link is hidden and used once (`from` itself is the
        // operand of the operation above and has been checked by the caller)
        auto matmul_under = [&](Value from) -> std::optional<Value> {
            Value v = from;
            while (graph[v].operation.kind == OpKind::View) {
                Value inner = graph[v].operation.inputs[0];
                if (!can_fuse(inner)) return std::nullopt;
                v = inner;
            }
            if (graph[v].operation.kind != OpKind::MatMul) return std::nullopt;
            return v;
        };
        // `(matmul + d) + d2` (a bias, then the skip connection of a transformer block): the sum next to the matmul
        // and its shape, then optionally the sum above it, each hidden and used once except for `curr` itself
        std::optional<Value> addend, addend2;
        std::optional<Value> mm;
        {
            auto sum_over_matmul = [&](Value sum, std::optional<Value> &other) -> std::optional<Value> {
                const Operation &op = graph[sum].operation;
                if (op.kind != OpKind::Binary || op.binary != BinaryOp::Add) return std::nullopt;
                const Value l = op.inputs[0], r = op.inputs[1];
                std::optional<Value> found;
                if (can_fuse(l)) found = matmul_under(l);
                if (found) other = r;
                else if (can_fuse(r) && (found = matmul_under(r))) other = l;
                return found;
            };
            const Operation &op = graph[curr].operation;
            if (op.kind == OpKind::Binary && op.binary == BinaryOp::Add) {
                mm = sum_over_matmul(curr, addend);
                if (!mm) {
                    // one more sum in between, of the same shape (views between the two sums are not followed)
                    for (int side = 0; side < 2 && !mm; side++) {
                        const Value inner = op.inputs[side], outer = op.inputs[1 - side];
                        if (!can_fuse(inner) || map.count(inner) || graph[inner].shape != graph[curr].shape) continue;
                        mm = sum_over_matmul(inner, addend);
                        if (mm) addend2 = outer;
                    }
                }
            } else if (relu) {
                mm = matmul_under(curr);
            }
        }
        if (!mm || (!relu && !addend)) return R::done(std::nullopt);
        if (map.count(*mm)) return R::done(std::nullopt);

        const ConcreteShape final_shape = graph[value].shape.eval(batch_size);
        const ConcreteShape mm_shape = graph[*mm].shape.eval(batch_size);
        std::optional<PlanTensor> addend_t, addend2_t;
        for (int which = 0; which < 2; which++) {
            const std::optional<Value> &from = which == 0 ? addend : addend2;
            if (!from) continue;
            auto at = visit(*from);
            if (!at.ok) return R::missing(at.need);
            // the operand in the matmul's own [b, m, n] shape; an operand whose layout cannot follow the views
            // between the matmul and the sum is not fused
            KN_ASSERT(at.value.shape.shape() == final_shape);
            auto viewed = at.value.view(mm_shape);
            if (!viewed) return R::done(std::nullopt);
            (which == 0 ? addend_t : addend2_t) = viewed;
        }
        const Operation &mop = graph[*mm].operation;
        auto result = visit_matmul(value, mop.inputs[0], mop.inputs[1], true, addend_t, relu, addend2_t);
        if (!result.ok) return R::missing(result.need);
        auto viewed = result.value.view(final_shape);
        KN_ASSERT(viewed.has_value(), "a dense matmul result can always be viewed");
        return R::done(*viewed);
    }

    // An operand [b, rows, cols] of the fused attention as [b1, b2, rows, cols] with b1 * b2 = b. The batch of an
    // attention is usually (batch, heads) flattened, and the flattening of a permuted [batch, tokens, heads, width]
    // tensor is no stride edit: the kernel takes two batch strides instead of a dense copy of the operand.
    VT visit_split_batch(Value v) {
        const Operation &op = graph[v].operation;
        const ConcreteShape flat = graph[v].shape.eval(batch_size);
        if (op.kind == OpKind::View && !map.count(v)) {
            KN_TRY(inner, visit(op.inputs[0]));
            const auto &shape = inner.shape.shape();
            if (shape.size() == 4 && shape[0] * shape[1] == flat[0] && shape[2] == flat[1] && shape[3] == flat[2]) return VT::done(inner);
        }
        if (op.kind == OpKind::Permute && op.axes == std::vector<size_t>{0, 2, 1} && !map.count(v)) {
            // K^T: the transposition commutes with the split of the batch
            KN_TRY(inner, visit_split_batch(op.inputs[0]));
            return VT::done(inner.permute({0, 1, 3, 2}));
        }
        KN_TRY(t, visit(v));
        auto split = t.view({1, flat[0], flat[1], flat[2]});
        KN_ASSERT(split.has_value(), "a leading axis of size 1 is a stride edit");
        return VT::done(*split);
    }

    // matmul(softmax(matmul(q, kt) [* or / constant] [+ mask], last axis), v) in f32 (no mask) or f16, every
    // intermediate value hidden and used once: the scores stay on the compute unit instead of passing through memory
    // between three or more launches (planner.rs:606-648, :418-476 plan them separately).
    // `split_inner` > 0: the result is wanted as [b / split_inner, split_inner, lq, dv], laid out in memory as
    // [b / split_inner, lq, split_inner, dv] (what `permute [0, 2, 1, 3]` of it turns into a dense tensor)
    Visit<std::optional<PlanTensor>> try_visit_fused_attention(Value value, bool batch_first = true, size_t split_inner = 0) {
        using R = Visit<std::optional<PlanTensor>>;
        const ValueInfo &info = graph[value];
        const DType dt = info.dtype;
        if (info.operation.kind != OpKind::MatMul || (dt != DType::F32 && dt != DType::F16)) return R::done(std::nullopt);
        const bool f16 = dt == DType::F16;
        const Value probs = info.operation.inputs[0], v_v = info.operation.inputs[1];
        const Operation &sop = graph[probs].operation;
        if (sop.kind != OpKind::Softmax || sop.axis() != 2 || !can_fuse(probs) || map.count(probs)) return R::done(std::nullopt);
        Value scores = sop.inputs[0];
        if (!can_fuse(scores) || map.count(scores)) return R::done(std::nullopt);
        // f16 only: `... + mask`, either way round; the mask is any tensor of the scores' shape (usually a broadcast)
        std::optional<Value> mask_v;
        if (f16 && graph[scores].operation.kind == OpKind::Binary && graph[scores].operation.binary == BinaryOp::Add) {
            const Value l = graph[scores].operation.inputs[0], r = graph[scores].operation.inputs[1];
            auto leads_to_matmul = [&](Value v) {
                if (!can_fuse(v) || map.count(v)) return false;
                const Operation &op = graph[v].operation;
                if (op.kind == OpKind::MatMul) return true;
                return op.kind == OpKind::Binary && op.binary == BinaryOp::Mul;
            };
            if (leads_to_matmul(l)) { scores = l; mask_v = r; }
            else if (leads_to_matmul(r)) { scores = r; mask_v = l; }
            else return R::done(std::nullopt);
        }
        float scale = 1.0f;
        bool has_scale = false;
        {
            const Operation &op = graph[scores].operation;
            // f16 rounds the scaled scores, so a division is not the same as a multiplication there
            if (op.kind == OpKind::Binary && (op.binary == BinaryOp::Mul || (op.binary == BinaryOp::Div && !f16))) {
                Value l = op.inputs[0], r = op.inputs[1];
                auto rc = graph.as_single_const(r);
                auto lc = op.binary == BinaryOp::Mul ? graph.as_single_const(l) : std::nullopt;
                Value inner;
                std::optional<DScalar> factor;
                if (rc) { inner = l; factor = rc; }
                else if (lc) { inner = r; factor = lc; }
                else return R::done(std::nullopt);
                if (factor->dtype != dt || !can_fuse(inner) || map.count(inner)) return R::done(std::nullopt);
                scale = op.binary == BinaryOp::Mul ? (float) factor->f : 1.0f / (float) factor->f;
                // the f32 kernel folds the scale into Q and takes the maximum of the scaled scores
                if (!std::isfinite(scale) || (!f16 && !(scale > 0.0f))) return R::done(std::nullopt);
                has_scale = true;
                scores = inner;
            }
        }
        const Operation &mop = graph[scores].operation;
        if (mop.kind != OpKind::MatMul || graph[scores].dtype != dt) return R::done(std::nullopt);
        const Value q_v = mop.inputs[0], kt_v = mop.inputs[1];
        const ConcreteShape q_shape = graph[q_v].shape.eval(batch_size), kt_shape = graph[kt_v].shape.eval(batch_size);
        const ConcreteShape v_shape = graph[v_v].shape.eval(batch_size);
        const size_t b = q_shape[0], lq = q_shape[1], dk = q_shape[2], lk = kt_shape[2], dv = v_shape[2];
        if (b == 0 || lq == 0 || lk == 0 || b > 65535 || lq > INT32_MAX || lk > INT32_MAX) return R::done(std::nullopt);
        if (dk > 1024 || dv > 1024) return R::done(std::nullopt);
        if (!(f16 ? attention_f16_supported((int) dk, (int) dv) : attention_supported((int) dk, (int) dv))) return R::done(std::nullopt);

        auto q = visit_split_batch(q_v);
        if (!q.ok) return R::missing(q.need);
        auto kt = visit_split_batch(kt_v);
        if (!kt.ok) return R::missing(kt.need);
        auto v = visit_split_batch(v_v);
        if (!v.ok) return R::missing(v.need);
        // one split of the batch for the whole launch: the one the result asks for, else that of the operands
        size_t inner_batch = split_inner > 0 ? split_inner : 1;
        if (split_inner == 0)
            for (const PlanTensor *t : {&q.value, &kt.value, &v.value})
                if (t->shape.shape()[0] > 1) inner_batch = std::max(inner_batch, t->shape.shape()[1]);
        if (b % inner_batch != 0) return R::done(std::nullopt);
        {
            const Value from[3] = {q_v, kt_v, v_v};
            PlanTensor *operand[3] = {&q.value, &kt.value, &v.value};
            for (int i = 0; i < 3; i++) {
                const auto &shape = operand[i]->shape.shape();
                auto again = operand[i]->view({b / inner_batch, inner_batch, shape[2], shape[3]});
                if (!again) {
                    // split in another way: the flat operand (a dense copy), whose batch axis splits in any way
                    auto flat = visit(from[i]);
                    if (!flat.ok) return R::missing(flat.need);
                    again = flat.value.view({b / inner_batch, inner_batch, shape[2], shape[3]});
                    KN_ASSERT(again.has_value(), "splitting an axis is a stride edit");
                }
                *operand[i] = *again;
            }
        }
        std::optional<PlanTensor> mask;
        if (mask_v) {
            auto m = visit(*mask_v);
            if (!m.ok) return R::missing(m.need);
            mask = m.value;
        }
        // strides of [b1, b2, rows, cols]
        const auto &qs = q.value.shape.strides(), &ks = kt.value.shape.strides(), &vs = v.value.shape.strides();
        if (f16) {
            // rows of Q, K and V are read as 128 bit vectors
            auto rows_ok = [](const PlanTensor &t, long long row_stride, long long inner_stride) {
                const auto &st = t.shape.strides();
                return inner_stride == 1 && row_stride % 8 == 0 && st[0] % 8 == 0 && st[1] % 8 == 0 && t.ptr.offset_bytes % 16 == 0;
            };
            if (!rows_ok(q.value, qs[2], qs[3]) || !rows_ok(kt.value, ks[3], ks[2]) || !rows_ok(v.value, vs[2], vs[3]))
                return R::done(std::nullopt);
            // a block of 64 keys is addressed with 32 bit offsets from the block's base
            if (ks[3] < 0 || ks[3] > (1 << 20) || vs[2] < 0 || vs[2] > (1 << 20)) return R::done(std::nullopt);
            // the 32 queries of a workgroup are addressed with 32 bit byte offsets from the batch entry's base
            if (qs[2] < 0 || (long long) lq * qs[2] >= (1ll << 30)) return R::done(std::nullopt);
        } else {
            // the kernel addresses a block of 64 keys with 32 bit offsets from the block's base
            auto fits = [](const PlanTensor &t) {
                for (size_t a = 2; a < 4; a++) {
                    const long long s = t.shape.strides()[a];
                    if (s < 0 || s > (1ll << 20)) return false;
                }
                return true;
            };
            if (!fits(kt.value) || !fits(v.value)) return R::done(std::nullopt);
        }

        // the result as the caller sees it, and as [b1, b2, lq, dv] for the kernel
        PlanTensor result, result_split;
        if (split_inner > 0) {
            result = alloc_tensor_shared({b / inner_batch, lq, inner_batch, dv}, dt).permute({0, 2, 1, 3});
            result_split = result;
        } else {
            result = batch_first ? alloc_tensor_shared({b, lq, dv}, dt) : alloc_tensor_shared({lq, b, dv}, dt).permute({1, 0, 2});
            auto split = result.view({b / inner_batch, inner_batch, lq, dv});
            KN_ASSERT(split.has_value(), "splitting an axis is a stride edit");
            result_split = *split;
        }
        Step step;
        step.kind = StepKind::MatMul;
        step.attention = true;
        step.gemm_f16 = f16;
        AttentionParams &a = step.attn;
        a.batch = (int) b; a.lq = (int) lq; a.lk = (int) lk; a.dk = (int) dk; a.dv = (int) dv;
        a.scale = scale;
        a.has_scale = has_scale ? 1 : 0;
        a.batch_inner = (int) inner_batch;
        const auto &os = result_split.shape.strides();
        a.q_sb = qs[0]; a.q_sb2 = qs[1]; a.q_sm = qs[2]; a.q_sk = qs[3];
        a.k_sb = ks[0]; a.k_sb2 = ks[1]; a.k_sk = ks[2]; a.k_sn = ks[3];  // the operand is K^T: [b, dk, lk]
        a.v_sb = vs[0]; a.v_sb2 = vs[1]; a.v_sk = vs[2]; a.v_sn = vs[3];
        a.o_sb = os[0]; a.o_sb2 = os[1]; a.o_sm = os[2]; a.o_sn = os[3];
        step.operands = {{q.value, OperandKind::In}, {kt.value, OperandKind::In}, {v.value, OperandKind::In}};
        if (mask) {
            KN_ASSERT(mask->shape.shape() == ConcreteShape({b, lq, lk}));
            const auto &ms = mask->shape.strides();
            a.m_sb = ms[0]; a.m_sq = ms[1]; a.m_sk = ms[2];
            a.mask_vec = ms[2] == 1 && ms[1] % 4 == 0 && ms[0] % 4 == 0 && mask->ptr.offset_bytes % 8 == 0;
            step.attention_has_mask = true;
            step.operands.push_back({*mask, OperandKind::In});
            // a constant mask (the causal triangle of a decoder) is looked at once, here: the kernel then neither
            // fetches nor computes the blocks it removes and does not read it where it is zero
            if (f16 && mask->ptr.kind == BufferKind::Constant && mask->dtype == DType::F16 && lk <= 64 * 4 * ATTENTION_F16_BLOCK &&
                ms[0] >= 0 && ms[1] >= 0 && ms[2] >= 0) {
                const HostTensor &src = constants[mask->ptr.index];
                const size_t batches = ms[0] == 0 ? 1 : b;
                const int64_t last = mask->ptr.offset_bytes / 2 + (int64_t) (batches - 1) * ms[0] + (int64_t) (lq - 1) * ms[1] + (int64_t) (lk - 1) * ms[2];
                KN_ASSERT(mask->ptr.offset_bytes >= 0 && mask->ptr.offset_bytes % 2 == 0 && last < (int64_t) src.len());
                std::vector<unsigned char> classes = attention_f16_block_classes(src.bytes() + mask->ptr.offset_bytes, (int) batches,
                                                                                 (int) lq, (int) lk, ms[0], ms[1], ms[2]);
                bool useful = false;
                for (unsigned char cl : classes) useful |= cl != 0;
                if (useful) {
                    constants.push_back(HostTensor(DType::U8, {classes.size()}, classes.data()));
                    PlanTensor t;
                    t.ptr = PlanPtr{BufferKind::Constant, constants.size() - 1, 0};
                    t.dtype = DType::U8;
                    t.shape = StridedShape::simple({classes.size()});
                    step.operands.push_back({t, OperandKind::In});
                    step.attention_has_classes = true;
                }
            }
        }
        step.operands.push_back({result, OperandKind::Out});
        push(std::move(step), value);
        return R::done(result);
    }

    // Matmuls of the same left operand with constant right operands of one shape and layout (the q / k / v or gate /
    // up projections of a transformer layer) run as ONE grouped launch: more tiles to fill the chip with, the left
    // operand fetched once per tile row, and launches saved. The reference launches them one by one
    // (planner.rs:606-648).
    std::unordered_map<Value, std::vector<Value>> matmuls_by_left;
    std::vector<Value> some_user;  // one of the values that use a value (the only one for values used once)
    bool matmuls_by_left_built = false;

    // whether the matmul is likely to be folded into the `+ tensor` / relu that consumes it (try_visit_fused_matmul):
    // such a matmul stays out of groups
    bool feeds_fused_epilogue(Value mm) const {
        Value v = mm;
        while (can_fuse(v)) {
            const Value user = some_user[v];
            const Operation &op = graph[user].operation;
            if (op.kind == OpKind::View) { v = user; continue; }
            if (op.kind != OpKind::Binary) return false;
            if (op.binary == BinaryOp::Add) return true;
            return op.binary == BinaryOp::Max && (graph.is_const_zero(op.inputs[0]) || graph.is_const_zero(op.inputs[1]));
        }
        return false;
    }

    const std::vector<Value> &matmul_siblings(Value left) {
        if (!matmuls_by_left_built) {
            matmuls_by_left_built = true;
            // only values that some output depends on
            std::vector<char> seen(graph.len(), 0);
            some_user.assign(graph.len(), 0);
            std::vector<Value> stack(graph.outputs.begin(), graph.outputs.end());
            while (!stack.empty()) {
                Value v = stack.back();
                stack.pop_back();
                if (seen[v]) continue;
                seen[v] = 1;
                for (Value in : graph[v].operation.inputs) {
                    some_user[in] = v;
                    stack.push_back(in);
                }
            }
            for (Value v = 0; v < graph.len(); v++) {
                const Operation &op = graph[v].operation;
                if (seen[v] && op.kind == OpKind::MatMul && graph.is_const(op.inputs[1]) && !graph.is_const(op.inputs[0]) &&
                    !feeds_fused_epilogue(v))
                    matmuls_by_left[op.inputs[0]].push_back(v);
            }
        }
        static const std::vector<Value> none;
        auto it = matmuls_by_left.find(left);
        return it == matmuls_by_left.end() ? none : it->second;
    }

    // `(g * sigmoid(g)) * u` with g = x w_g and u = x w_u, two f16 matmuls of one left operand with constant right
    // operands of one shape, every intermediate value hidden and used only here (the gate twice): the feed-forward gate
    // of a LLaMA style block. Planned as ONE launch of the matmul kernel that loads global -> LDS directly: its tiles
    // interleave 16 columns of g with the same 16 columns of u, and the store computes the gated product, so neither
    // product is written to memory and the elementwise launch behind them is gone (the reference plans two cuBLAS calls
    // and a scalar kernel, planner.rs:606-648, :835-954). Roundings are those of the separate operations.
    Visit<std::optional<PlanTensor>> try_visit_gated_matmul(Value value) {
        using R = Visit<std::optional<PlanTensor>>;
        const ValueInfo &info = graph[value];
        const Operation &top = info.operation;
        if (info.dtype != DType::F16 || top.kind != OpKind::Binary || top.binary != BinaryOp::Mul) return R::done(std::nullopt);
        // through single-use hidden views down to a matmul; `from` itself has been checked by the caller
        auto matmul_under = [&](Value from) -> std::optional<Value> {
            Value v = from;
            while (graph[v].operation.kind == OpKind::View) {
                Value inner = graph[v].operation.inputs[0];
                if (!can_fuse(inner) || graph[inner].shape.rank() == 0) return std::nullopt;
                v = inner;
            }
            if (graph[v].operation.kind != OpKind::MatMul || map.count(v)) return std::nullopt;
            return v;
        };
        std::optional<Value> gate_mm, up_mm;
        for (int side = 0; side < 2 && !gate_mm; side++) {
            const Value inner = top.inputs[side], up_side = top.inputs[1 - side];
            const Operation &iop = graph[inner].operation;
            if (!can_fuse(inner) || !can_fuse(up_side) || iop.kind != OpKind::Binary || iop.binary != BinaryOp::Mul) continue;
            if (graph[inner].shape != info.shape || graph[up_side].shape != info.shape) continue;
            for (int s = 0; s < 2; s++) {
                const Value sig = iop.inputs[s], gate = iop.inputs[1 - s];
                const Operation &sop = graph[sig].operation;
                if (!can_fuse(sig) || sop.kind != OpKind::Unary || sop.unary != UnaryOp::Sigmoid || sop.inputs[0] != gate) continue;
                if (!graph.is_hidden_with_uses(gate, 2) || graph[gate].shape != info.shape || map.count(gate) || map.count(up_side)) continue;
                auto g = matmul_under(gate), u = matmul_under(up_side);
                if (!g || !u || *g == *u) continue;
                gate_mm = g;
                up_mm = u;
                break;
            }
        }
        if (!gate_mm) return R::done(std::nullopt);
        const Operation &gop = graph[*gate_mm].operation, &uop = graph[*up_mm].operation;
        if (gop.inputs[0] != uop.inputs[0] || !graph.is_const(gop.inputs[1]) || !graph.is_const(uop.inputs[1]) || graph.is_const(gop.inputs[0])) return R::done(std::nullopt);
        if (graph[*gate_mm].dtype != DType::F16 || graph[*gate_mm].shape != graph[*up_mm].shape ||
            graph[gop.inputs[1]].shape != graph[uop.inputs[1]].shape)
            return R::done(std::nullopt);

        auto left = visit(gop.inputs[0]);
        if (!left.ok) return R::missing(left.need);
        auto gate_w = visit(gop.inputs[1]);
        if (!gate_w.ok) return R::missing(gate_w.need);
        auto up_w = visit(uop.inputs[1]);
        if (!up_w.ok) return R::missing(up_w.need);
        if (gate_w.value.shape.strides() != up_w.value.shape.strides()) return R::done(std::nullopt);
        KN_ASSERT(left.value.shape.rank() == 3 && gate_w.value.shape.rank() == 3);
        const PlanTensor wg = pack_right_operand(left.value, gate_w.value, DType::F16), wu = pack_right_operand(left.value, up_w.value, DType::F16);
        if (wg.shape.strides() != wu.shape.strides()) return R::done(std::nullopt);

        const PlanTensor &l = left.value;
        const size_t b = l.shape.shape()[0], m = l.shape.shape()[1], k = l.shape.shape()[2], n = wg.shape.shape()[2];
        if (b != 1 || m * n == 0 || m > INT32_MAX || 2 * n > INT32_MAX || k > INT32_MAX) return R::done(std::nullopt);
        Step step;
        step.kind = StepKind::MatMul;
        step.gemm_f16 = true;
        GemmParams &g = step.gemm;
        g.tuning = options.gemm;
        g.batch = 1; g.m = (int) m; g.n = (int) (2 * n); g.k = (int) k;
        g.a_sb = l.shape.strides()[0]; g.a_sm = l.shape.strides()[1]; g.a_sk = l.shape.strides()[2];
        g.b_sb = wg.shape.strides()[0]; g.b_sk = wg.shape.strides()[1]; g.b_sn = wg.shape.strides()[2];
        g.c_sb = (long long) (m * n); g.c_sm = (long long) n; g.c_sn = 1;
        g.pair_op = GEMM_PAIR_SWIGLU;
        // only on the kernel that loads global -> LDS directly, whole K per workgroup (operands in the arena are aligned)
        const GemmLaunchPlan lp = plan_gemm_launch(g, true);
        if (!lp.direct || lp.swapped || lp.split_k > 1 || lp.dot) return R::done(std::nullopt);
        // both weights lie within the reach of the kernel's 32 bit offsets wherever the arena puts them
        if (dtype_bytes(DType::F16) * (n * (size_t) std::llabs(g.b_sn) + k) * 2 >= ((size_t) 1 << 31)) return R::done(std::nullopt);

        PlanTensor result = alloc_tensor_shared({1, m, n}, DType::F16);
        step.operands = {{l, OperandKind::In}, {wg, OperandKind::In}, {wu, OperandKind::In}, {result, OperandKind::Out}};
        push_gemm_scratch(step);  // (a sparse last round of tiles is shared between workgroups)
        push(std::move(step), value);
        auto viewed = result.view(info.shape.eval(batch_size));
        KN_ASSERT(viewed.has_value(), "a dense matmul result can always be viewed");
        return R::done(*viewed);
    }

    Visit<std::optional<PlanTensor>> try_visit_matmul_group(Value value) {
        using R = Visit<std::optional<PlanTensor>>;
        const ValueInfo &info = graph[value];
        const DType dt = info.dtype;
        if (dt != DType::F32 && dt != DType::F16) return R::done(std::nullopt);
        const Value left_v = info.operation.inputs[0];
        std::vector<Value> members{value};
        for (Value other : matmul_siblings(left_v)) {
            if (other == value || map.count(other) || members.size() >= (size_t) GEMM_MAX_GROUPS) continue;
            if (graph[other].dtype != dt || graph[other].shape != info.shape) continue;
            if (graph[graph[other].operation.inputs[1]].shape != graph[info.operation.inputs[1]].shape) continue;
            members.push_back(other);
        }
        // `value` itself has to be one of the candidates (constant right operand, reachable)
        {
            const auto &sib = matmul_siblings(left_v);
            if (members.size() < 2 || std::find(sib.begin(), sib.end(), value) == sib.end()) return R::done(std::nullopt);
        }
        auto left = visit(left_v);
        if (!left.ok) return R::missing(left.need);
        std::vector<PlanTensor> rights;
        for (Value m : members) {
            auto r = visit(graph[m].operation.inputs[1]);
            if (!r.ok) return R::missing(r.need);
            rights.push_back(r.value);
        }
        // keep the members whose right operand is laid out like the first one's
        std::vector<Value> kept{members[0]};
        std::vector<PlanTensor> kept_rights{rights[0]};
        for (size_t i = 1; i < members.size(); i++)
            if (rights[i].shape.strides() == rights[0].shape.strides()) {
                kept.push_back(members[i]);
                kept_rights.push_back(rights[i]);
            }
        if (kept.size() < 2) return R::done(std::nullopt);
        KN_ASSERT(left.value.shape.rank() == 3 && kept_rights[0].shape.rank() == 3);
        for (auto &r : kept_rights) r = pack_right_operand(left.value, r, dt);

        const PlanTensor &l = left.value, &r0 = kept_rights[0];
        const size_t b = l.shape.shape()[0], m = l.shape.shape()[1], k = l.shape.shape()[2], n = r0.shape.shape()[2];
        if (b * m * n == 0 || b > INT32_MAX || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return R::done(std::nullopt);
        Step step;
        step.kind = StepKind::MatMul;
        step.gemm_f16 = dt == DType::F16;
        GemmParams &g = step.gemm;
            g.tuning = options.gemm;
        g.batch = (int) b; g.m = (int) m; g.n = (int) n; g.k = (int) k;
        g.a_sb = l.shape.strides()[0]; g.a_sm = l.shape.strides()[1]; g.a_sk = l.shape.strides()[2];
        g.b_sb = r0.shape.strides()[0]; g.b_sk = r0.shape.strides()[1]; g.b_sn = r0.shape.strides()[2];
        g.c_sb = (long long) (m * n); g.c_sm = (long long) n; g.c_sn = 1;
        g.groups = (int) kept.size();
        if (!gemm_group_ok(g, step.gemm_f16)) return R::done(std::nullopt);

        step.operands.push_back({l, OperandKind::In});
        for (auto &r : kept_rights) step.operands.push_back({r, OperandKind::In});
        std::vector<PlanTensor> results;
        for (size_t i = 0; i < kept.size(); i++) {
            results.push_back(alloc_tensor_shared({b, m, n}, dt));
            step.operands.push_back({results.back(), OperandKind::Out});
        }
        push_gemm_scratch(step);
        push(std::move(step), value);
        for (size_t i = 1; i < kept.size(); i++) insert_mapping(kept[i], results[i]);
        return R::done(results[0]);
    }

    // A constant right operand of a matmul whose n axis is the contiguous one ([k, n] weights, as `x @ w` exports
    // them) is laid out again, once, on the host, as [n, k]: with K contiguous in both operands the matmul takes the
    // direct global -> LDS path (f16, 512 x 11008 x 4096 twice in one launch: 157 us -> 116 us; f32,
    // 1024 x 4672 x 2048: 281 -> 175 us). That holds for a left operand of any height: under a few rows the product
    // is a pass over the weights, which that path streams at twice the rate (f16, 8 x 32000 x 4096: 96 -> 40 us).
    // The original constant stays out of the arena when nothing else reads it.
    std::map<std::tuple<size_t, int64_t, std::vector<size_t>, std::vector<int64_t>>, PlanTensor> packed_rights;

    PlanTensor pack_right_operand(const PlanTensor &left, const PlanTensor &right, DType dt) {
        if (!options.pack_matmul_constants || right.ptr.kind != BufferKind::Constant) return right;
        if (dt != DType::F16 && dt != DType::F32) return right;
        const auto &shape = right.shape.shape();
        const auto &strides = right.shape.strides();
        const size_t b = shape[0], k = shape[1], n = shape[2];
        if (b == 0 || n < 2 || k < 64 || k % 64 != 0 || strides[2] != 1 || strides[1] == 1) return right;
        if (left.shape.strides()[2] != 1) return right;
        if (strides[0] < 0 || strides[1] < 0) return right;
        auto key = std::make_tuple(right.ptr.index, right.ptr.offset_bytes, shape, strides);
        auto it = packed_rights.find(key);
        if (it != packed_rights.end()) return it->second;

        const HostTensor &src = constants[right.ptr.index];
        const size_t elem = dtype_bytes(dt);
        const size_t copies = strides[0] == 0 ? 1 : b;
        // every element the view reads lies inside the constant
        {
            const int64_t last = right.ptr.offset_bytes / (int64_t) elem + (int64_t) (copies - 1) * strides[0] +
                                 (int64_t) (k - 1) * strides[1] + (int64_t) (n - 1);
            KN_ASSERT(right.ptr.offset_bytes >= 0 && right.ptr.offset_bytes % (int64_t) elem == 0 && last < (int64_t) src.len());
        }
        HostTensor packed(dt, {copies, n, k});
        constexpr size_t TILE = 64;  // both the reads and the writes of a tile stay in cache
        auto turn = [&](auto *to, const auto *from) {
            for (size_t c = 0; c < copies; c++)
                for (size_t k0 = 0; k0 < k; k0 += TILE)
                    for (size_t n0 = 0; n0 < n; n0 += TILE) {
                        const size_t k1 = std::min(k, k0 + TILE), n1 = std::min(n, n0 + TILE);
                        for (size_t ni = n0; ni < n1; ni++) {
                            auto *row = to + (c * n + ni) * k;
                            const auto *col = from + c * (size_t) strides[0] + ni;
                            for (size_t ki = k0; ki < k1; ki++) row[ki] = col[ki * (size_t) strides[1]];
                        }
                    }
        };
        if (elem == 2) turn((uint16_t *) packed.bytes_mut(), (const uint16_t *) (src.bytes() + right.ptr.offset_bytes));
        else turn((uint32_t *) packed.bytes_mut(), (const uint32_t *) (src.bytes() + right.ptr.offset_bytes));
        constants.push_back(std::move(packed));
        PlanTensor t;
        t.ptr = PlanPtr{BufferKind::Constant, constants.size() - 1, 0};
        t.dtype = dt;
        t.shape = StridedShape::simple({copies, n, k});
        t = t.permute({0, 2, 1});
        if (copies != b) t = t.broadcast({b, k, n});
        packed_rights.emplace(std::move(key), t);
        return t;
    }

    // A launch that splits the K axis needs scratch for its f32 partial products: a shared buffer that is live for
    // this step only. Where workgroups share tiles inside one launch they also need counters, which start at zero
    // and which every launch leaves at zero again: a zero-filled constant of the step's own.
    void push_gemm_scratch(Step &step) {
        const GemmLaunchPlan lp = plan_gemm_launch(step.gemm, step.gemm_f16);
        if (lp.workspace_bytes > 0)
            step.operands.push_back({alloc_tensor_shared({lp.workspace_bytes / 4}, DType::F32), OperandKind::Out});
        if (lp.counter_bytes > 0) {
            constants.push_back(HostTensor(DType::I32, {lp.counter_bytes / 4}));
            PlanTensor t;
            t.ptr = PlanPtr{BufferKind::Constant, constants.size() - 1, 0};
            t.dtype = DType::I32;
            t.shape = StridedShape::simple({lp.counter_bytes / 4});
            step.operands.push_back({t, OperandKind::Out});
        }
    }

    // A right operand of an f16 matmul that is not a constant and has n as its contiguous axis ([k, n] activations,
    // `x @ y`) is copied into [n, k] order first when the left operand has enough rows to pay for the copy: the
    // matmul then runs on the direct global -> LDS kernel instead of the one that transposes 16 bit elements through
    // LDS stores (4096^3: 546 us -> 149 us including the 18 us copy, which turns 64 x 64 tiles through LDS).
    PlanTensor transpose_right_operand(const PlanTensor &left, const PlanTensor &right, DType dt, Value debug_value) {
        if (!options.pack_matmul_constants || dt != DType::F16 || right.ptr.kind == BufferKind::Constant) return right;
        const auto &shape = right.shape.shape();
        const auto &strides = right.shape.strides();
        const size_t b = shape[0], k = shape[1], n = shape[2], m = left.shape.shape()[1];
        if (b == 0 || n < 16 || k < 64 || k % 64 != 0 || strides[2] != 1 || strides[1] == 1 || m < 256) return right;
        if (left.shape.strides()[2] != 1) return right;
        const size_t copies = strides[0] == 0 ? 1 : b;
        PlanTensor source = copies == b ? right : right.slice(0, SliceRange{0, 1, 1});
        PlanTensor dense = alloc_tensor_shared({copies, n, k}, dt);
        plan_copy_tensor(source.permute({0, 2, 1}), dense, debug_value);
        PlanTensor t = dense.permute({0, 2, 1});
        if (copies != b) t = t.broadcast({b, k, n});
        return t;
    }

    VT visit_matmul(Value value, Value left_v, Value right_v, bool batch_first,
                    const std::optional<PlanTensor> &addend = std::nullopt, bool relu = false,
                    const std::optional<PlanTensor> &addend2 = std::nullopt) {
        const DType dt = graph[value].dtype;
        if (dt != DType::F32 && dt != DType::F16) fail("GPU matmul only supports f32 and f16, got ", dtype_name(dt));
        KN_TRY(left, visit(left_v));
        KN_TRY(right_as_given, visit(right_v));
        KN_ASSERT(left.shape.rank() == 3 && right_as_given.shape.rank() == 3);
        const PlanTensor right = transpose_right_operand(left, pack_right_operand(left, right_as_given, dt), dt, value);
        size_t b = left.shape.shape()[0], m = left.shape.shape()[1], k = left.shape.shape()[2], n = right.shape.shape()[2];
        PlanTensor result = batch_first ? alloc_tensor_shared({b, m, n}, dt)
                                        : alloc_tensor_shared({m, b, n}, dt).permute({1, 0, 2});
        if (b * m * n != 0) {
            KN_ASSERT(b <= INT32_MAX && m <= INT32_MAX && n <= INT32_MAX && k <= INT32_MAX);
            Step step;
            step.kind = StepKind::MatMul;
            step.gemm_f16 = dt == DType::F16;
            GemmParams &g = step.gemm;
            g.tuning = options.gemm;
            g.batch = (int) b; g.m = (int) m; g.n = (int) n; g.k = (int) k;
            g.a_sb = left.shape.strides()[0]; g.a_sm = left.shape.strides()[1]; g.a_sk = left.shape.strides()[2];
            g.b_sb = right.shape.strides()[0]; g.b_sk = right.shape.strides()[1]; g.b_sn = right.shape.strides()[2];
            g.c_sb = result.shape.strides()[0]; g.c_sm = result.shape.strides()[1]; g.c_sn = result.shape.strides()[2];
            step.operands = {{left, OperandKind::In}, {right, OperandKind::In}, {result, OperandKind::Out}};
            if (addend) {
                KN_ASSERT(addend->dtype == dt && addend->shape.shape() == ConcreteShape({b, m, n}));
                g.d_sb = addend->shape.strides()[0]; g.d_sm = addend->shape.strides()[1]; g.d_sn = addend->shape.strides()[2];
                step.gemm_has_addend = true;
                step.operands.push_back({*addend, OperandKind::In});
            }
            if (addend2) {
                KN_ASSERT(addend.has_value() && addend2->dtype == dt && addend2->shape.shape() == ConcreteShape({b, m, n}));
                g.d2_sb = addend2->shape.strides()[0]; g.d2_sm = addend2->shape.strides()[1]; g.d2_sn = addend2->shape.strides()[2];
                step.gemm_has_addend2 = true;
                step.operands.push_back({*addend2, OperandKind::In});
            }
            g.relu = relu ? 1 : 0;
            push_gemm_scratch(step);
            push(std::move(step), value);
        }
        return VT::done(result);
    }

    // planner.rs:669-833: relu?( conv(x, w) [+ bias] [+ res] )
    Visit<std::optional<PlanTensor>> try_visit_fused_conv(Value value) {
        using R = Visit<std::optional<PlanTensor>>;
        if (graph[value].dtype != DType::F32 || graph[value].shape.rank() != 4) return R::done(std::nullopt);
        Value curr = value;
        bool relu = false;
        {
            const Operation &op = graph[curr].operation;
            if (op.kind == OpKind::Binary && op.binary == BinaryOp::Max) {
                Value l = op.inputs[0], r = op.inputs[1];
                // only the activation input has to be exclusive to this relu: the zero it is compared with is a
                // constant that the builder shares between all relus of the same shape
                if (graph.is_const_zero(l)) curr = r;
                else if (graph.is_const_zero(r)) curr = l;
                else return R::done(std::nullopt);
                if (!can_fuse(curr)) return R::done(std::nullopt);
                relu = true;
            }
        }
        std::optional<Value> bias, res;
        while (true) {
            const Operation &op = graph[curr].operation;
            if (!(op.kind == OpKind::Binary && op.binary == BinaryOp::Add)) break;
            Value l = op.inputs[0], r = op.inputs[1];
            if (!can_fuse(l)) return R::done(std::nullopt);
            bool is_res = graph[l].shape == graph[r].shape;
            std::optional<Value> bias_inner;
            const Operation &rop = graph[r].operation;
            if (rop.kind == OpKind::Broadcast) {
                Value ri = rop.inputs[0];
                if (graph[l].shape.keep(1, Size::one()) == graph[ri].shape) bias_inner = ri;
            }
            if (bias_inner) {
                if (bias) return R::done(std::nullopt);
                bias = bias_inner;
            } else if (is_res) {
                if (res) return R::done(std::nullopt);
                res = r;
            } else {
                return R::done(std::nullopt);
            }
            curr = l;
        }
        const Operation &cop = graph[curr].operation;
        if (cop.kind != OpKind::Conv) return R::done(std::nullopt);
        Value input_v = cop.inputs[0], filter_v = cop.inputs[1];
        const ConvDetails &d = cop.conv;
        KN_ASSERT(d.dtype == DType::F32);
        // the residual has to be shaped like the input; otherwise the conv is retried later without it
        if (res && graph[input_v].shape != graph[*res].shape) return R::done(std::nullopt);

        auto input = visit_ensure_simple_strides(input_v);
        if (!input.ok) return R::missing(input.need);
        auto filter = visit_ensure_simple_strides(filter_v);
        if (!filter.ok) return R::missing(filter.need);
        std::optional<PlanTensor> bias_t, res_t;
        if (bias) {
            auto bt = visit(*bias);
            if (!bt.ok) return R::missing(bt.need);
            bias_t = bt.value;
        }
        if (res) {
            auto rt = visit_ensure_simple_strides(*res);
            if (!rt.ok) return R::missing(rt.need);
            res_t = rt.value;
        }
        ConcreteShape out_shape = graph[curr].shape.eval(batch_size);
        PlanTensor output = alloc_tensor_shared(out_shape, DType::F32);
        if (res_t) KN_ASSERT(res_t->shape.shape() == out_shape, "conv residual must match the output shape");

        // A 1 x 1 convolution with stride 1 is a matrix product per image, out[n] = W [K, C] x in[n] [C, H W], with the
        // bias added along the rows and the residual laid out like the result: it runs on the matmul kernels, which read
        // the image with 128 bit loads along its contiguous axis (128 -> 32 channels on 1024 boards of 8 x 8: 36 us as
        // an implicit GEMM that gathers single elements).
        const bool pointwise = d.kernel_h == 1 && d.kernel_w == 1 && d.stride_y == 1 && d.stride_x == 1 && d.padding_y == 0 && d.padding_x == 0;
        if (pointwise && options.pointwise_conv_as_matmul && concrete_size(out_shape) != 0 && out_shape[0] <= 65535 &&
            d.input_h * d.input_w <= INT32_MAX) {
            const int64_t hw = (int64_t) (d.input_h * d.input_w), cin = (int64_t) d.input_channels, cout = (int64_t) d.output_channels;
            Step step;
            step.kind = StepKind::MatMul;
            GemmParams &g = step.gemm;
            g.tuning = options.gemm;
            g.batch = (int) out_shape[0]; g.m = (int) cout; g.n = (int) hw; g.k = (int) cin;
            g.a_sb = 0; g.a_sm = cin; g.a_sk = 1;
            g.b_sb = cin * hw; g.b_sk = hw; g.b_sn = 1;
            g.c_sb = cout * hw; g.c_sm = hw; g.c_sn = 1;
            step.operands = {{filter.value, OperandKind::In}, {input.value, OperandKind::In}, {output, OperandKind::Out}};
            if (bias_t) {
                g.d_sb = 0; g.d_sm = bias_t->shape.strides()[1]; g.d_sn = 0;
                step.gemm_has_addend = true;
                step.operands.push_back({*bias_t, OperandKind::In});
            }
            if (res_t) {
                if (bias_t) {
                    g.d2_sb = cout * hw; g.d2_sm = hw; g.d2_sn = 1;
                    step.gemm_has_addend2 = true;
                } else {
                    g.d_sb = cout * hw; g.d_sm = hw; g.d_sn = 1;
                    step.gemm_has_addend = true;
                }
                step.operands.push_back({*res_t, OperandKind::In});
            }
            g.relu = relu ? 1 : 0;
            push_gemm_scratch(step);
            push(std::move(step), value);
        } else if (concrete_size(out_shape) != 0) {
            Step step;
            step.kind = StepKind::Conv;
            ConvParams &p = step.conv;
            p.channel_split = options.split_conv_channels;
            p.plane_any_width = options.plane_conv_any_width;
            KN_ASSERT(out_shape[0] <= INT32_MAX);
            p.batch = (int) out_shape[0];
            p.in_c = (int) d.input_channels; p.in_h = (int) d.input_h; p.in_w = (int) d.input_w;
            p.out_c = (int) d.output_channels; p.out_h = (int) d.output_h; p.out_w = (int) d.output_w;
            p.kernel_h = (int) d.kernel_h; p.kernel_w = (int) d.kernel_w;
            p.stride_y = (int) d.stride_y; p.stride_x = (int) d.stride_x;
            p.pad_y = (int) d.padding_y; p.pad_x = (int) d.padding_x;
            p.relu = relu ? 1 : 0;
            p.bias_stride = bias_t ? bias_t->shape.strides()[1] : 0;
            step.conv_has_bias = bias_t.has_value();
            step.conv_has_res = res_t.has_value();
            step.operands = {{input.value, OperandKind::In}, {filter.value, OperandKind::In}};
            if (bias_t) step.operands.push_back({*bias_t, OperandKind::In});
            if (res_t) step.operands.push_back({*res_t, OperandKind::In});
            step.operands.push_back({output, OperandKind::Out});
            // partial results of a launch that splits the input channels
            if (const size_t bytes = conv_workspace_bytes(p))
                step.operands.push_back({alloc_tensor_shared({bytes / 4}, DType::F32), OperandKind::Out});
            // counters of the tiles whose parts are summed inside the launch: zero, and left at zero by every launch
            if (const size_t bytes = conv_counter_bytes(p)) {
                constants.push_back(HostTensor(DType::I32, {bytes / 4}));
                PlanTensor t;
                t.ptr = PlanPtr{BufferKind::Constant, constants.size() - 1, 0};
                t.dtype = DType::I32;
                t.shape = StridedShape::simple({bytes / 4});
                step.operands.push_back({t, OperandKind::Out});
            }
            push(std::move(step), value);
        }
        return R::done(output);
    }

    // planner.rs:835-871
    VT visit_fused_scalar(Value value) {
        const ValueInfo &info = graph[value];
        ScalarBlock block;
        block.operands.push_back(PlanTensor());  // placeholder for the result
        block.loaded.push_back(std::nullopt);
        auto root = visit_fused_scalar_recurse(value, block, true);
        if (!root.ok) return VT::missing(root.need);
        KN_ASSERT(root.value == block.expr.result());

        if (block.row_value) {
            // the chain hangs off a layernorm / softmax (or reads a statistic of its own rows): it becomes the
            // epilogue of that row kernel
            auto row = graph[*block.row_value].operation.kind == OpKind::Reduce ? visit_reduce_row_inputs(*block.row_value)
                                                                                 : visit_row_inputs(*block.row_value);
            if (!row.ok) return VT::missing(row.need);
            return VT::done(push_row_kernel(*block.row_value, value, row.value, block.expr, block.operands));
        }

        PlanTensor result = alloc_tensor_shared(info.shape.eval(batch_size), info.dtype);
        block.operands[0] = result;
        plan_scalar_op(block.expr, block.operands, value);
        return VT::done(result);
    }

    // planner.rs:873-923; returns the node index that holds `value`
    Visit<size_t> visit_fused_scalar_recurse(Value value, ScalarBlock &block, bool is_root) {
        using R = Visit<size_t>;
        auto known = block.value_nodes.find(value);
        if (known != block.value_nodes.end()) return R::done(known->second);

        size_t node;
        auto mapped = map.find(value);
        if (mapped != map.end()) {
            node = block.load_operand(mapped->second);
        } else {
            // give the conv fuser the first shot, so that this chain does not steal its relu, add or bias
            auto fused = try_visit_fused_conv(value);
            if (!fused.ok) return R::missing(fused.need);
            // `matmul + bias` or `matmul + residual` that more than this chain uses: stored by the matmul itself and
            // loaded here, instead of computed again in every chain that uses it
            if (!fused.value && !is_root && options.fuse_matmul_epilogue && !can_fuse(value)) {
                fused = try_visit_fused_matmul(value);
                if (!fused.ok) return R::missing(fused.need);
            }
            if (fused.value) {
                if (!map.count(value)) insert_mapping(value, *fused.value);
                node = block.load_operand(*fused.value);
            } else {
                const ValueInfo &info = graph[value];
                const Operation &op = info.operation;
                ScalarNode n;
                n.dtype = info.dtype;
                if (op.kind == OpKind::Unary) {
                    auto a = visit_fused_scalar_recurse(op.inputs[0], block, false);
                    if (!a.ok) return a;
                    n.kind = ScalarNode::Unary;
                    n.unary = op.unary;
                    n.cast_to = op.cast_to;
                    n.a = a.value;
                } else if (op.kind == OpKind::Binary) {
                    auto a = visit_fused_scalar_recurse(op.inputs[0], block, false);
                    if (!a.ok) return a;
                    auto b = visit_fused_scalar_recurse(op.inputs[1], block, false);
                    if (!b.ok) return b;
                    n.kind = ScalarNode::Binary;
                    n.binary = op.binary;
                    n.a = a.value;
                    n.b = b.value;
                } else {
                    KN_ASSERT(!is_root);
                    if (auto c = graph.as_single_const(value)) {
                        n.kind = ScalarNode::Const;
                        n.constant = *c;
                    } else if (options.fuse_row_epilogue && !block.row_value && can_fuse(value) &&
                               (op.kind == OpKind::Layernorm || op.kind == OpKind::Softmax)) {
                        block.row_value = value;
                        n.kind = ScalarNode::Load;
                        n.operand = SIZE_MAX;
                    } else if (op.kind == OpKind::Broadcast && is_small_elementwise(op.inputs[0])) {
                        // A broadcast elementwise chain that nobody else uses (`rsqrt(mean + eps)` of a norm) is
                        // evaluated per element here instead of in a launch of its own.
                        auto inner = inline_under_broadcast(op.inputs[0], info.shape.eval(batch_size), block);
                        if (!inner.ok) return inner;
                        block.value_nodes[value] = inner.value;
                        return R::done(inner.value);
                    } else {
                        auto t = visit(value);
                        if (!t.ok) return R::missing(t.need);
                        node = block.load_operand(t.value);
                        block.value_nodes[value] = node;
                        return R::done(node);
                    }
                }
                block.expr.nodes.push_back(n);
                node = block.expr.nodes.size() - 1;
            }
        }
        block.value_nodes[value] = node;
        return R::done(node);
    }

    bool is_small_elementwise(Value v) const {
        const OpKind kind = graph[v].operation.kind;
        return (kind == OpKind::Unary || kind == OpKind::Binary) && can_fuse(v) && !map.count(v);
    }

    // The nodes of the elementwise chain under a Broadcast, with its leaf tensors broadcast to `target`.
    Visit<size_t> inline_under_broadcast(Value value, const ConcreteShape &target, ScalarBlock &block) {
        using R = Visit<size_t>;
        auto known = block.value_nodes.find(value);
        if (known != block.value_nodes.end()) return R::done(known->second);
        const ValueInfo &info = graph[value];
        const Operation &op = info.operation;
        ScalarNode n;
        n.dtype = info.dtype;
        if (is_small_elementwise(value)) {
            auto a = inline_under_broadcast(op.inputs[0], target, block);
            if (!a.ok) return a;
            n.a = a.value;
            if (op.kind == OpKind::Unary) {
                n.kind = ScalarNode::Unary;
                n.unary = op.unary;
                n.cast_to = op.cast_to;
            } else {
                auto b = inline_under_broadcast(op.inputs[1], target, block);
                if (!b.ok) return b;
                n.kind = ScalarNode::Binary;
                n.binary = op.binary;
                n.b = b.value;
            }
        } else if (auto c = graph.as_single_const(value)) {
            n.kind = ScalarNode::Const;
            n.constant = *c;
        } else if (auto reduce = row_reduce_under(value, target, block)) {
            // A statistic of the very rows this kernel writes (the mean of squares of an RMS norm): the kernel
            // becomes a row kernel that computes it itself, instead of a reduce launch in front of it.
            block.row_value = *reduce;
            n.kind = ScalarNode::Load;
            n.operand = SIZE_MAX;
        } else {
            auto t = visit(value);
            if (!t.ok) return R::missing(t.need);
            const size_t node = block.load_operand(t.value.broadcast(target));
            block.value_nodes[value] = node;
            return R::done(node);
        }
        block.expr.nodes.push_back(n);
        block.value_nodes[value] = block.expr.nodes.size() - 1;
        return R::done(block.expr.nodes.size() - 1);
    }

    // `value`, seen through views that only it uses, is a Sum / Mean / Max / Min over the last axis of a tensor of
    // shape `target`, kept as a column ([..., 1]) that the caller broadcasts back along that axis
    std::optional<Value> row_reduce_under(Value value, const ConcreteShape &target, const ScalarBlock &block) const {
        if (!options.fuse_row_epilogue || block.row_value || target.empty() || target.back() < 2) return std::nullopt;
        ConcreteShape column = target;
        column.back() = 1;
        if (graph[value].shape.eval(batch_size) != column) return std::nullopt;
        Value v = value;
        while (graph[v].operation.kind == OpKind::View) {
            if (!can_fuse(v) || map.count(v)) return std::nullopt;
            v = graph[v].operation.inputs[0];
        }
        const Operation &op = graph[v].operation;
        if (op.kind != OpKind::Reduce || !can_fuse(v) || map.count(v)) return std::nullopt;
        if (op.reduce != ReduceOp::Sum && op.reduce != ReduceOp::Mean && op.reduce != ReduceOp::Max && op.reduce != ReduceOp::Min)
            return std::nullopt;
        if (op.axes != std::vector<size_t>{target.size() - 1}) return std::nullopt;
        if (graph[op.inputs[0]].shape.eval(batch_size) != target) return std::nullopt;
        const DType dt = graph[v].dtype;
        if ((dt != DType::F32 && dt != DType::F16) || graph[op.inputs[0]].dtype != dt) return std::nullopt;
        return v;
    }

    // The operands and prologue of a reduction that a row kernel computes for itself: an elementwise chain that
    // only the reduction uses is evaluated on the loaded elements (like in the reduce kernel).
    Visit<FusedRow> visit_reduce_row_inputs(Value reduce) {
        using R = Visit<FusedRow>;
        const Operation &op = graph[reduce].operation;
        FusedRow row;
        row.kind = RowKernelDesc::Reduce;
        row.reduce_op = op.reduce;
        row.axis = op.axes[0];
        row.eps = 0;
        const Value in_v = op.inputs[0];
        const OpKind in_kind = graph[in_v].operation.kind;
        if (!map.count(in_v) && can_fuse(in_v) && (in_kind == OpKind::Unary || in_kind == OpKind::Binary)) {
            ScalarBlock pre;
            pre.operands.push_back(PlanTensor());
            pre.loaded.push_back(std::nullopt);
            auto root = visit_fused_scalar_recurse(in_v, pre, true);
            if (!root.ok) return R::missing(root.need);
            if (!pre.row_value) {
                row.inputs.assign(pre.operands.begin() + 1, pre.operands.end());
                row.pre = pre.expr;
                return R::done(row);
            }
        }
        auto t = visit(in_v);
        if (!t.ok) return R::missing(t.need);
        row.inputs = {t.value};
        ScalarNode n;
        n.kind = ScalarNode::Load;
        n.dtype = t.value.dtype;
        n.operand = 1;
        row.pre.nodes.push_back(n);
        return R::done(row);
    }

    // planner.rs:926-931
    void plan_copy_tensor(const PlanTensor &old_t, const PlanTensor &new_t, Value debug_value) {
        KN_ASSERT(old_t.shape.shape() == new_t.shape.shape() && old_t.dtype == new_t.dtype);
        ScalarExpr expr;
        ScalarNode n;
        n.kind = ScalarNode::Load;
        n.dtype = old_t.dtype;
        n.operand = 1;
        expr.nodes.push_back(n);
        plan_scalar_op(expr, {new_t, old_t}, debug_value);
    }

    // planner.rs:933-954
    void plan_scalar_op(const ScalarExpr &expr, const std::vector<PlanTensor> &operands, Value debug_value) {
        std::vector<KernelOperand> kops;
        for (auto &t : operands) kops.push_back(kop(t));
        Step step;
        step.kind = StepKind::ScalarOp;
        step.kernel = make_scalar_kernel(kops, expr);
        step.scalar_exprs = {expr};
        step.operands.push_back({operands[0], OperandKind::Out});
        for (size_t k = 1; k < operands.size(); k++) step.operands.push_back({operands[k], OperandKind::In});
        push(std::move(step), debug_value);
    }
};

size_t align_up(size_t v) { return (v + ARENA_ALIGN - 1) / ARENA_ALIGN * ARENA_ALIGN; }

}  // namespace

Plan plan_graph(const Graph &graph, size_t batch_size, const PlannerOptions &options) {
    GeneratorScope generator_scope(options.generator);
    Planner planner(graph, batch_size, options);
    Plan plan;

    // allocate inputs (even if they are not actually used), then plan everything the outputs need
    for (Value in : graph.inputs) plan.inputs.push_back(planner.visit_completely(in));
    for (Value out : graph.outputs) plan.outputs.push_back(planner.visit_completely_ensure_simple_strides(out));

    planner.compile_steps();

    size_t buffer_count = planner.shared_sizes.size();
    size_t step_count = planner.steps.size();

    // live ranges of the shared buffers over step indices (planner.rs:134-164)
    std::vector<std::pair<size_t, size_t>> live(buffer_count, {step_count, 0});
    auto touch = [&](const PlanPtr &p, size_t si) {
        if (p.kind != BufferKind::Shared) return;
        live[p.index].first = std::min(live[p.index].first, si);
        live[p.index].second = std::max(live[p.index].second, si);
    };
    for (size_t si = 0; si < step_count; si++)
        for (auto &op : planner.steps[si].operands) touch(op.tensor.ptr, si);
    for (auto &t : plan.outputs)
        if (t.ptr.kind == BufferKind::Shared) live[t.ptr.index].second = step_count;
    for (auto &t : plan.inputs) {
        if (t.ptr.kind != BufferKind::Shared) continue;
        live[t.ptr.index].first = 0;
        if (options.preserve_inputs) live[t.ptr.index].second = step_count;
    }

    // ---- arena layout: constants first
    // (a constant that no step reads, because a matmul took a copy in another layout instead, gets no room)
    std::vector<char> constant_used(planner.constants.size(), 0);
    for (auto &step : planner.steps)
        for (auto &op : step.operands)
            if (op.tensor.ptr.kind == BufferKind::Constant) constant_used[op.tensor.ptr.index] = 1;
    for (auto &t : plan.outputs)
        if (t.ptr.kind == BufferKind::Constant) constant_used[t.ptr.index] = 1;
    size_t cursor = 0;
    for (size_t ci = 0; ci < planner.constants.size(); ci++) {
        const HostTensor &c = planner.constants[ci];
        plan.constant_offsets.push_back(cursor);
        if (!constant_used[ci]) continue;
        plan.uploads.push_back({cursor, c});
        plan.mem_usage.dedicated_bytes += c.nbytes();
        cursor = align_up(cursor + c.nbytes());
    }
    plan.zero_offset = cursor;
    size_t shared_base = cursor;
    if (options.stream_weights_bytes != 0 && plan.mem_usage.dedicated_bytes >= options.stream_weights_bytes) {
        for (auto &step : planner.steps) {
            if (step.kind != StepKind::MatMul || step.attention || step.operands.size() < 2) continue;
            // (the right operands follow the left one: one, one per product of a group, or the two of a gated pair)
            const size_t rights = step.gemm.pair_op ? 2 : (size_t) std::max(step.gemm.groups, 1);
            // (a weight that many row tiles of the left operand share is read more than once: not a stream)
            bool constant = step.operands.size() > rights && (long long) step.gemm.batch * step.gemm.m <= 1024;
            for (size_t k = 1; k <= rights && constant; k++) constant = step.operands[k].tensor.ptr.kind == BufferKind::Constant;
            step.gemm.tuning.stream_b = constant;
        }
    }

    // ---- shared region: first-fit placement of live intervals. A buffer whose last use is step s may share
    // memory with one whose first use is step s + 1, never with one that is touched by step s itself.
    plan.shared_offsets.assign(buffer_count, SIZE_MAX);
    plan.shared_sizes = planner.shared_sizes;
    std::vector<size_t> order;
    for (size_t b = 0; b < buffer_count; b++)
        if (live[b].first <= live[b].second) order.push_back(b);
    std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) {
        if (live[x].first != live[y].first) return live[x].first < live[y].first;
        return planner.shared_sizes[x] > planner.shared_sizes[y];
    });
    struct Active {
        size_t offset, size, end;
    };
    std::vector<Active> active;
    size_t shared_extent = 0;
    for (size_t b : order) {
        size_t start = live[b].first, end = live[b].second;
        size_t size = align_up(std::max<size_t>(planner.shared_sizes[b], 1));
        active.erase(std::remove_if(active.begin(), active.end(), [&](const Active &a) { return a.end < start; }), active.end());
        std::sort(active.begin(), active.end(), [](const Active &x, const Active &y) { return x.offset < y.offset; });
        size_t offset = 0;
        for (auto &a : active) {
            if (offset + size <= a.offset) break;
            offset = std::max(offset, a.offset + a.size);
        }
        active.push_back({offset, size, end});
        plan.shared_offsets[b] = shared_base + offset;
        shared_extent = std::max(shared_extent, offset + size);
        plan.mem_usage.hypo_shared_bytes_total += planner.shared_sizes[b];
    }
    plan.mem_usage.shared_bytes = shared_extent;
    plan.arena_bytes = std::max<size_t>(shared_base + shared_extent, ARENA_ALIGN);

    // the amount of memory that is live at the same time, as a lower bound for the shared region
    {
        std::vector<int64_t> delta(step_count + 2, 0);
        for (size_t b : order) {
            delta[live[b].first] += (int64_t) planner.shared_sizes[b];
            delta[live[b].second + 1] -= (int64_t) planner.shared_sizes[b];
        }
        int64_t curr = 0;
        for (int64_t d : delta) {
            curr += d;
            plan.mem_usage.hypo_shared_bytes_peak = std::max<size_t>(plan.mem_usage.hypo_shared_bytes_peak, (size_t) curr);
        }
    }

    // ---- every access of every step has to stay inside its buffer: checked here, on the host, so that a planning
    // mistake is reported as an error instead of faulting on the device
    auto buffer_bytes = [&](const PlanPtr &p) {
        return p.kind == BufferKind::Constant ? planner.constants[p.index].nbytes() : planner.shared_sizes[p.index];
    };
    for (auto &step : planner.steps) {
        for (auto &op : step.operands) {
            const PlanTensor &t = op.tensor;
            if (t.shape.size() == 0) continue;
            auto [lo, hi] = t.shape.offset_bounds();
            int64_t es = (int64_t) dtype_bytes(t.dtype);
            int64_t first = t.ptr.offset_bytes + lo * es, last = t.ptr.offset_bytes + (hi + 1) * es;
            if (first < 0 || last > (int64_t) buffer_bytes(t.ptr))
                fail("planned operand of ", step.str(), " reaches outside its buffer: bytes [", first, ", ", last, ") of ",
                     buffer_bytes(t.ptr));
        }
    }

    plan.steps = std::move(planner.steps);
    return plan;
}

}  // namespace kn
