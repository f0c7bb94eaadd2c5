// optimize_graph: rebuilds a graph through the public builder while applying four rewrites, in this order
// (kn-graph/src/optimizer/core.rs:87-113): layernorm pattern -> Layernorm, min/max chains -> one clamp,
// per-channel affine operations folded into a neighbouring convolution (optimizer/affine.rs), and division
// by a constant -> multiplication by its inverse. Only f32 values are rewritten (core.rs:90-93).
#include "optimizer.h"

#include <map>

namespace kn {

namespace {

// A visit either yields the mapped value, or names an old value that has to be visited first
// (core.rs:21, optimizer/recurse.rs:6-22): this keeps deep graphs off the call stack.
struct Visit {
    bool ok;
    Value value;
    static Visit done(Value v) { return {true, v}; }
    static Visit need(Value v) { return {false, v}; }
};

using Vec = std::vector<float>;

struct AffineOp {
    bool is_scale;  // else add
    Vec data;
};

struct ScaleBias {
    std::optional<Vec> scale, bias;
};

struct AffineGroup {
    size_t before_channels, after_channels;
    Value old_input;
    std::vector<AffineOp> before, after;
    bool has_conv = false;
    ConvDetails details;
    HostTensor filter;
};

class Optimizer {
public:
    Optimizer(const OptimizerSettings &s, const Graph &old) : settings(s), old_graph(old) {}

    OptimizerSettings settings;
    const Graph &old_graph;
    Graph new_graph;
    std::unordered_map<Value, Value> map;

    void insert_mapping(Value old, Value neu) {
        KN_ASSERT(old_graph[old].shape == new_graph[neu].shape);
        bool inserted = map.emplace(old, neu).second;
        KN_ASSERT(inserted);
    }

    Value visit_completely(Value old) {
        std::vector<Value> stack{old};
        while (true) {
            Value curr = stack.back();
            Visit r = visit_single_cached(curr);
            if (r.ok) {
                stack.pop_back();
                if (stack.empty()) return r.value;
            } else {
                stack.push_back(r.value);
            }
        }
    }

private:
    Visit visit(Value old) {
        auto it = map.find(old);
        return it != map.end() ? Visit::done(it->second) : Visit::need(old);
    }

    Visit visit_single_cached(Value old) {
        auto it = map.find(old);
        if (it != map.end()) return Visit::done(it->second);
        Visit r = visit_single_new(old);
        if (r.ok) insert_mapping(old, r.value);
        return r;
    }

    Visit visit_single_new(Value old_value) {
        std::optional<Value> fused;
        Visit f = try_fuse(old_value, &fused);
        if (!f.ok) return f;
        if (fused) {
            new_graph.set_debug_id(*fused, old_graph[old_value].debug_id);
            return Visit::done(*fused);
        }
        // fallback, copy the old operation with mapped operands
        const ValueInfo &info = old_graph[old_value];
        for (Value in : info.operation.inputs) {
            Visit r = visit(in);
            if (!r.ok) return r;
        }
        Operation op = info.operation;
        for (Value &in : op.inputs) in = map.at(in);
        Value nv = new_graph.push(info.shape, info.dtype, std::move(op));
        if (info.operation.kind == OpKind::Input) new_graph.inputs.push_back(nv);
        new_graph.set_debug_id(nv, info.debug_id);
        return Visit::done(nv);
    }

    // Each try_* returns need(v) to ask for an operand first; otherwise done() with `*out` set when it fused.
    Visit try_fuse(Value old_start, std::optional<Value> *out) {
        *out = std::nullopt;
        if (old_graph[old_start].dtype != DType::F32) return Visit::done(0);
        Visit r = Visit::done(0);
        if (settings.fuse_layernorm) {
            r = try_fuse_layernorm(old_start, out);
            if (!r.ok || *out) return r;
        }
        r = try_fuse_clamp(old_start, out);
        if (!r.ok || *out) return r;
        r = try_fuse_conv_affine(old_start, out);
        if (!r.ok || *out) return r;
        if (settings.div_to_mul) {
            r = try_convert_div_to_mul(old_start, out);
            if (!r.ok || *out) return r;
        }
        return Visit::done(0);
    }

    // core.rs:115-210: (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) with every intermediate used only here
    Visit try_fuse_layernorm(Value value, std::optional<Value> *out) {
        std::map<Value, size_t> fused_values;
        std::vector<Value> order;
        auto op = [&](Value v) -> const Operation & {
            if (!fused_values.count(v)) order.push_back(v);
            fused_values[v] += 1;
            return old_graph[v].operation;
        };
        const Operation &root = old_graph[value].operation;
        if (!(root.kind == OpKind::Binary && root.binary == BinaryOp::Div)) return Visit::done(0);
        Value zeroed0 = root.inputs[0], std_broadcast = root.inputs[1];

        const Operation &o_zeroed = op(zeroed0);
        if (!(o_zeroed.kind == OpKind::Binary && o_zeroed.binary == BinaryOp::Sub)) return Visit::done(0);
        Value input0 = o_zeroed.inputs[0], mean_broadcast = o_zeroed.inputs[1];
        const Operation &o_mb = op(mean_broadcast);
        if (o_mb.kind != OpKind::Broadcast) return Visit::done(0);
        const Operation &o_mv = op(o_mb.inputs[0]);
        if (o_mv.kind != OpKind::View) return Visit::done(0);
        const Operation &o_mean = op(o_mv.inputs[0]);
        if (!(o_mean.kind == OpKind::Reduce && o_mean.reduce == ReduceOp::Mean)) return Visit::done(0);
        Value input1 = o_mean.inputs[0];
        const std::vector<size_t> &axes0 = o_mean.axes;

        const Operation &o_sb = op(std_broadcast);
        if (o_sb.kind != OpKind::Broadcast) return Visit::done(0);
        const Operation &o_std = op(o_sb.inputs[0]);
        if (!(o_std.kind == OpKind::Unary && o_std.unary == UnaryOp::Sqrt)) return Visit::done(0);
        const Operation &o_stable = op(o_std.inputs[0]);
        if (!(o_stable.kind == OpKind::Binary && o_stable.binary == BinaryOp::Add)) return Visit::done(0);
        Value var_view = o_stable.inputs[0], const_eps = o_stable.inputs[1];
        const Operation &o_vv = op(var_view);
        if (o_vv.kind != OpKind::View) return Visit::done(0);
        const Operation &o_var = op(o_vv.inputs[0]);
        if (!(o_var.kind == OpKind::Reduce && o_var.reduce == ReduceOp::Mean)) return Visit::done(0);
        const std::vector<size_t> &axes1 = o_var.axes;
        const Operation &o_pow = op(o_var.inputs[0]);
        if (!(o_pow.kind == OpKind::Binary && o_pow.binary == BinaryOp::Pow)) return Visit::done(0);
        Value zeroed1 = o_pow.inputs[0], const_2 = o_pow.inputs[1];
        op(zeroed1);  // count the second use of the zeroed value

        if (input0 != input1 || zeroed0 != zeroed1 || axes0 != axes1) return Visit::done(0);
        for (auto &[fv, count] : fused_values)
            if (!old_graph.is_hidden_with_uses(fv, count)) return Visit::done(0);

        if (axes0.size() != 1) return Visit::done(0);
        auto eps = old_graph.as_single_const(const_eps);
        if (!eps || eps->dtype != DType::F32) return Visit::done(0);
        if (!old_graph.is_const_filled_with(const_2, DScalar::f32(2.0f))) return Visit::done(0);

        Visit in = visit(input0);
        if (!in.ok) return in;
        *out = new_graph.layernorm(in.value, axes0[0], (float) eps->f);
        return Visit::done(0);
    }

    // core.rs:299-326
    template <typename F>
    Visit follow_if(Value start, F next, std::optional<Value> *result) {
        Value curr = start;
        while (true) {
            if (!old_graph.is_hidden_with_uses(curr, 1)) break;
            std::optional<Value> n;
            Visit r = next(curr, old_graph[curr].operation, &n);
            if (!r.ok) return r;
            if (!n) break;
            curr = *n;
        }
        *result = curr == start ? std::nullopt : std::optional<Value>(curr);
        return Visit::done(0);
    }

    // core.rs:212-243: several sequential min/max with single constants become one clamp
    Visit try_fuse_clamp(Value old_start, std::optional<Value> *out) {
        float total_min = -INFINITY, total_max = INFINITY;
        std::optional<Value> old_input;
        Visit r = follow_if(
            old_start,
            [&](Value, const Operation &op, std::optional<Value> *n) {
                if (op.kind == OpKind::Binary && (op.binary == BinaryOp::Min || op.binary == BinaryOp::Max)) {
                    auto c = old_graph.as_single_const(op.inputs[1]);
                    if (c && c->dtype == DType::F32) {
                        float v = (float) c->f;
                        if (op.binary == BinaryOp::Min) total_max = std::fmin(total_max, v);
                        else total_min = std::fmax(total_min, v);
                        *n = op.inputs[0];
                    }
                }
                return Visit::done(0);
            },
            &old_input);
        if (!r.ok) return r;
        if (!old_input) return Visit::done(0);
        Visit in = visit(*old_input);
        if (!in.ok) return in;
        *out = new_graph.clamp_dyn(in.value, DScalar::f32(total_min), DScalar::f32(total_max));
        return Visit::done(0);
    }

    // core.rs:263-297
    Visit try_convert_div_to_mul(Value old_start, std::optional<Value> *out) {
        const Operation &op = old_graph[old_start].operation;
        if (!(op.kind == OpKind::Binary && op.binary == BinaryOp::Div)) return Visit::done(0);
        auto right = old_graph.as_const(op.inputs[1]);
        if (!right || right->dtype != DType::F32) return Visit::done(0);
        HostTensor inv(DType::F32, right->shape);
        const float *src = (const float *) right->bytes();
        float *dst = (float *) inv.bytes_mut();
        for (size_t k = 0; k < inv.len(); k++) dst[k] = 1.0f / src[k];
        Visit left = visit(op.inputs[0]);
        if (!left.ok) return left;
        Value new_right = new_graph.constant_tensor(inv);
        *out = new_graph.mul(left.value, new_right);
        return Visit::done(0);
    }

    // ------------------------------------------------------------------------------ affine.rs

    Visit try_fuse_conv_affine(Value old_start, std::optional<Value> *out) {
        const Shape &shape = old_graph[old_start].shape;
        if (shape.rank() != 4) return Visit::done(0);
        auto after_channels = shape.dims[1].try_unwrap_fixed();
        if (!after_channels) return Visit::done(0);

        AffineGroup group;
        group.before_channels = group.after_channels = *after_channels;
        std::vector<AffineOp> before_rev, after_rev;

        std::optional<Value> old_input;
        Visit r = follow_if(
            old_start,
            [&](Value, const Operation &op, std::optional<Value> *n) {
                grow_affine_group(group, before_rev, after_rev, op, n);
                return Visit::done(0);
            },
            &old_input);
        if (!r.ok) return r;
        if (!old_input) return Visit::done(0);

        group.old_input = *old_input;
        group.before.assign(before_rev.rbegin(), before_rev.rend());
        group.after.assign(after_rev.rbegin(), after_rev.rend());

        Visit in = visit(group.old_input);
        if (!in.ok) return in;
        *out = apply_fused(group, in.value);
        return Visit::done(0);
    }

    // affine.rs:47-114
    void grow_affine_group(AffineGroup &g, std::vector<AffineOp> &before_rev, std::vector<AffineOp> &after_rev,
                           const Operation &op, std::optional<Value> *next) {
        if (op.kind == OpKind::Conv) {
            auto filter = old_graph.as_const(op.inputs[1]);
            if (!filter || filter->dtype != DType::F32) return;
            if (!g.has_conv && op.conv.keeps_spatial_shape() && !op.conv.has_stride()) {
                g.has_conv = true;
                g.details = op.conv;
                g.filter = *filter;
                g.before_channels = op.conv.input_channels;
                *next = op.inputs[0];
            }
            return;
        }
        if (op.kind == OpKind::Binary && (op.binary == BinaryOp::Add || op.binary == BinaryOp::Sub ||
                                          op.binary == BinaryOp::Mul || op.binary == BinaryOp::Div)) {
            Value left = op.inputs[0], right = op.inputs[1];
            const Operation &rop = old_graph[right].operation;
            if (rop.kind != OpKind::Broadcast) return;
            Value right_inner = rop.inputs[0];
            const Shape &rs = old_graph[right_inner].shape;
            size_t channels = g.before_channels;
            if (!(rs.rank() == 4 && rs.dims[0] == Size::one() && rs.dims[2] == Size::one() && rs.dims[3] == Size::one() &&
                  rs.dims[1] == Size::fixed(channels)))
                return;
            auto data_t = old_graph.as_const(right_inner);
            if (!data_t || data_t->dtype != DType::F32) return;
            const float *p = (const float *) data_t->bytes();
            Vec data(p, p + channels);
            AffineOp a;
            switch (op.binary) {
                case BinaryOp::Add: a = {false, data}; break;
                case BinaryOp::Sub:
                    for (float &x : data) x = -x;
                    a = {false, data};
                    break;
                case BinaryOp::Mul: a = {true, data}; break;
                default:
                    for (float &x : data) x = 1.0f / x;
                    a = {true, data};
                    break;
            }
            (g.has_conv ? before_rev : after_rev).push_back(std::move(a));
            *next = left;
        }
    }

    // affine.rs:341-373
    static ScaleBias fuse_affine_list(size_t channels, const std::vector<AffineOp> &ops) {
        ScaleBias r;
        for (const AffineOp &op : ops) {
            KN_ASSERT(op.data.size() == channels);
            if (!op.is_scale) {
                if (!r.bias) r.bias = op.data;
                else
                    for (size_t c = 0; c < channels; c++) (*r.bias)[c] += op.data[c];
            } else {
                if (!r.scale) r.scale = op.data;
                else
                    for (size_t c = 0; c < channels; c++) (*r.scale)[c] *= op.data[c];
                if (r.bias)
                    for (size_t c = 0; c < channels; c++) (*r.bias)[c] *= op.data[c];
            }
        }
        return r;
    }

    // affine.rs:313-334
    Value apply_scale_bias(const ScaleBias &sb, Value input) {
        Value curr = input;
        if (sb.scale) {
            Value c = new_graph.constant_tensor(HostTensor(DType::F32, {1, sb.scale->size(), 1, 1}, sb.scale->data()));
            curr = new_graph.binary(BinaryOp::Mul, curr, c);
        }
        if (sb.bias) {
            Value c = new_graph.constant_tensor(HostTensor(DType::F32, {1, sb.bias->size(), 1, 1}, sb.bias->data()));
            curr = new_graph.binary(BinaryOp::Add, curr, c);
        }
        return curr;
    }

    Value apply_fused(const AffineGroup &g, Value input) {
        if (!g.has_conv) {
            KN_ASSERT(g.before.empty());
            return apply_scale_bias(fuse_affine_list(g.after_channels, g.after), input);
        }
        ScaleBias before = fuse_affine_list(g.before_channels, g.before);
        ScaleBias after = fuse_affine_list(g.after_channels, g.after);
        return apply_fused_conv(input, before, g, after);
    }

    // affine.rs:169-253
    Value apply_fused_conv(Value input, const ScaleBias &before, const AffineGroup &g, const ScaleBias &after) {
        const ConvDetails &d = g.details;
        KN_ASSERT(!d.has_stride());
        size_t K = d.output_channels, C = d.input_channels, kh = d.kernel_h, kw = d.kernel_w;
        std::vector<size_t> fshape{K, C, kh, kw};
        Vec filter((const float *) g.filter.bytes(), (const float *) g.filter.bytes() + K * C * kh * kw);
        size_t per_k = C * kh * kw, per_c = kh * kw;

        // fuse output scale into kernel
        if (after.scale)
            for (size_t k = 0; k < K; k++)
                for (size_t j = 0; j < per_k; j++) filter[k * per_k + j] *= (*after.scale)[k];

        // try to pull the input bias through the convolution (affine.rs:255-305)
        bool pulled = true;
        std::optional<HostTensor> bias_before_as_after;
        if (before.bias) {
            bool all_zero = true;
            for (float x : *before.bias) all_zero &= (x == 0.0f);
            if (all_zero) {
                // nothing to add
            } else if (d.padding_y == 0 && d.padding_x == 0) {
                HostTensor t(DType::F32, {1, K, 1, 1});
                float *tp = (float *) t.bytes_mut();
                for (size_t k = 0; k < K; k++) {
                    float total = 0;
                    for (size_t c = 0; c < C; c++) {
                        float s = 0;
                        for (size_t j = 0; j < per_c; j++) s += filter[k * per_k + c * per_c + j];
                        total += s * (*before.bias)[c];
                    }
                    tp[k] = total;
                }
                bias_before_as_after = t;
            } else if (settings.force_bias_through_conv) {
                // the bias differs at the edges, so it becomes a full [1, K, H, W] constant:
                // the convolution of the spatially broadcast bias with the (already scaled) filter
                HostTensor t(DType::F32, {1, K, d.output_h, d.output_w});
                float *tp = (float *) t.bytes_mut();
                for (size_t k = 0; k < K; k++)
                    for (size_t oy = 0; oy < d.output_h; oy++)
                        for (size_t ox = 0; ox < d.output_w; ox++) {
                            float acc = 0;
                            for (size_t c = 0; c < C; c++)
                                for (size_t fy = 0; fy < kh; fy++)
                                    for (size_t fx = 0; fx < kw; fx++) {
                                        int64_t iy = (int64_t) oy + (int64_t) fy - (int64_t) d.padding_y;
                                        int64_t ix = (int64_t) ox + (int64_t) fx - (int64_t) d.padding_x;
                                        if (iy < 0 || ix < 0 || iy >= (int64_t) d.input_h || ix >= (int64_t) d.input_w) continue;
                                        acc += (*before.bias)[c] * filter[k * per_k + c * per_c + fy * kw + fx];
                                    }
                            tp[(k * d.output_h + oy) * d.output_w + ox] = acc;
                        }
                bias_before_as_after = t;
            } else {
                pulled = false;
            }
        }

        std::optional<HostTensor> bias_after_shaped;
        if (after.bias) bias_after_shaped = HostTensor(DType::F32, {1, K, 1, 1}, after.bias->data());

        Value curr = input;
        if (pulled) {
            std::optional<HostTensor> total_bias;
            if (bias_before_as_after && bias_after_shaped) {
                // broadcast add of [1,K,h,w] and [1,K,1,1]
                HostTensor t = HostTensor(DType::F32, bias_before_as_after->shape, bias_before_as_after->bytes());
                float *tp = (float *) t.bytes_mut();
                size_t spatial = t.len() / K;
                const float *bp = (const float *) bias_after_shaped->bytes();
                for (size_t k = 0; k < K; k++)
                    for (size_t j = 0; j < spatial; j++) tp[k * spatial + j] += bp[k];
                total_bias = t;
            } else if (bias_before_as_after) {
                total_bias = bias_before_as_after;
            } else if (bias_after_shaped) {
                total_bias = bias_after_shaped;
            }
            // fuse input scale into kernel
            if (before.scale)
                for (size_t k = 0; k < K; k++)
                    for (size_t c = 0; c < C; c++)
                        for (size_t j = 0; j < per_c; j++) filter[k * per_k + c * per_c + j] *= (*before.scale)[c];

            Value vf = new_graph.constant_tensor(HostTensor(DType::F32, fshape, filter.data()));
            curr = new_graph.conv(curr, vf, 1, 1, d.padding_y, d.padding_x);
            if (total_bias) {
                Value vb = new_graph.constant_tensor(*total_bias);
                curr = new_graph.binary(BinaryOp::Add, curr, vb);
            }
        } else {
            ScaleBias b{before.scale, before.bias};
            curr = apply_scale_bias(b, curr);
            Value vf = new_graph.constant_tensor(HostTensor(DType::F32, fshape, filter.data()));
            curr = new_graph.conv(curr, vf, 1, 1, d.padding_y, d.padding_x);
            if (bias_after_shaped) {
                Value vb = new_graph.constant_tensor(*bias_after_shaped);
                curr = new_graph.binary(BinaryOp::Add, curr, vb);
            }
        }
        return curr;
    }
};

}  // namespace

Graph optimize_graph(const Graph &graph, const OptimizerSettings &settings) {
    if (!settings.optimize) return graph;
    Optimizer opt(settings, graph);
    // all inputs are copied over in the same order, then every output is rebuilt
    for (Value old_input : graph.inputs) {
        Value ni = opt.new_graph.input(graph[old_input].shape, graph[old_input].dtype);
        opt.insert_mapping(old_input, ni);
    }
    for (Value old_output : graph.outputs) {
        Value no = opt.visit_completely(old_output);
        opt.new_graph.output(no);
    }
    return std::move(opt.new_graph);
}

}  // namespace kn
