// The extern "C" surface declared in include/knhip.h. Every entry point catches all exceptions and converts
// them into a status code plus a thread-local message.
#include "../../include/knhip.h"

#include <cstring>
#include <new>

#include "executor.h"
#include "matmul_api.h"
#include "optimizer.h"

using namespace kn;

struct knhip_graph {
    Graph graph;
};
struct knhip_executor {
    HipExecutor ex;
    knhip_executor(int device, const Graph &g, size_t batch, const ExecutorOptions &options) : ex(device, g, batch, options) {}
};

namespace {

thread_local std::string g_last_error;

template <typename F>
int guarded(F f) {
    try {
        return f();
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return KNHIP_ERROR;
    } catch (...) {
        g_last_error = "unknown failure";
        return KNHIP_ERROR;
    }
}

#define KN_REQUIRE(cond)                                       \
    do {                                                       \
        if (!(cond)) fail("invalid argument: " #cond " does not hold"); \
    } while (0)

Shape to_shape(const knhip_size_t *dims, size_t rank) {
    KN_REQUIRE(dims != nullptr || rank == 0);
    Shape s;
    for (size_t i = 0; i < rank; i++) s.dims.push_back(Size(dims[i].batch_exp, dims[i].fixed_factor));
    return s;
}

DType to_dtype(int code) {
    if (!dtype_valid(code)) fail("invalid dtype code ", code);
    return (DType) code;
}

int copy_out(const std::string &s, char *buf, size_t cap, size_t *needed) {
    if (needed) *needed = s.size() + 1;
    if (buf == nullptr || cap < s.size() + 1) {
        if (buf == nullptr && cap == 0) return KNHIP_OK;  // size query
        g_last_error = "buffer too small";
        return KNHIP_BUFFER_TOO_SMALL;
    }
    std::memcpy(buf, s.c_str(), s.size() + 1);
    return KNHIP_OK;
}

template <typename T, typename U>
int copy_list(const std::vector<T> &v, U *buf, size_t cap, size_t *count) {
    if (count) *count = v.size();
    if (buf == nullptr && cap == 0) return KNHIP_OK;
    if (cap < v.size()) {
        g_last_error = "buffer too small";
        return KNHIP_BUFFER_TOO_SMALL;
    }
    for (size_t i = 0; i < v.size(); i++) buf[i] = (U) v[i];
    return KNHIP_OK;
}

// Every call names its device and selects it first (handle.rs:60-64): the caller's thread may have switched.
template <typename F>
int on_device(int device, F f) {
    return guarded([&] {
        HipDevice::check(device);
        hip_check(hipSetDevice(device), "hipSetDevice");
        f();
        return KNHIP_OK;
    });
}

}  // namespace

namespace kn {

void set_last_error(const std::string &message) { g_last_error = message; }

namespace {

// grid.y carries the batch index: at most this many batch entries per launch, longer batches run as several launches
constexpr int MATMUL_BATCH_SLAB = 65535;

GemmLaunchPlan matmul_plan_slab(const knhip_matmul_args &a, int first, int count, MatmulWorkspace *ws) {
    const size_t elem = a.dtype == KNHIP_F16 ? 2 : 4;
    GemmParams p{};
    p.a = a.a ? (const char *) a.a + (int64_t) first * a.a_batch_stride * (int64_t) elem : nullptr;
    p.b = a.b ? (const char *) a.b + (int64_t) first * a.b_batch_stride * (int64_t) elem : nullptr;
    p.c = a.c ? (char *) a.c + (int64_t) first * a.c_batch_stride * (int64_t) elem : nullptr;
    p.batch = count;
    p.m = a.m;
    p.n = a.n;
    p.k = a.k;
    p.a_sb = a.a_batch_stride; p.a_sm = a.a_row_stride; p.a_sk = a.a_col_stride;
    p.b_sb = a.b_batch_stride; p.b_sk = a.b_row_stride; p.b_sn = a.b_col_stride;
    p.c_sb = a.c_batch_stride; p.c_sm = a.c_row_stride; p.c_sn = a.c_col_stride;
    GemmLaunchPlan lp = plan_gemm_launch(p, a.dtype == KNHIP_F16);
    ws->counter_bytes = lp.counter_bytes;
    ws->partial_bytes = lp.workspace_bytes;
    return lp;
}

}  // namespace

MatmulPlan matmul_api_plan(const knhip_matmul_args &a) {
    if (a.dtype != KNHIP_F32 && a.dtype != KNHIP_F16) fail("batched_mat_mul: dtype must be f32 or f16, got code ", a.dtype);
    if (a.batch < 0 || a.m < 0 || a.n < 0 || a.k < 0) fail("batched_mat_mul: negative size");
    const bool empty = a.batch == 0 || a.m == 0 || a.n == 0;
    if (!empty && (a.c == nullptr || (a.k > 0 && (a.a == nullptr || a.b == nullptr)))) fail("batched_mat_mul: null operand");
    MatmulPlan plan;
    plan.f16 = a.dtype == KNHIP_F16;
    plan.empty = empty;
    // the slabs run one after the other on the stream and share the workspace, which has room for the largest
    for (int first = 0; first < a.batch || plan.slabs.empty(); first += MATMUL_BATCH_SLAB) {
        MatmulWorkspace ws;
        plan.slabs.push_back(matmul_plan_slab(a, first, std::min(MATMUL_BATCH_SLAB, a.batch - first), &ws));
        plan.slab_workspaces.push_back(ws);
        plan.workspace.counter_bytes = std::max(plan.workspace.counter_bytes, ws.counter_bytes);
        plan.workspace.partial_bytes = std::max(plan.workspace.partial_bytes, ws.partial_bytes);
        if (a.batch == 0) break;
    }
    return plan;
}

void matmul_api_launch(MatmulPlan &plan, void *workspace, size_t workspace_bytes, ihipStream_t *stream) {
    if (plan.empty) return;
    const size_t total = plan.workspace.total();
    if (total > 0) {
        if (workspace == nullptr || workspace_bytes < total)
            fail("batched_mat_mul: this product needs ", total, " bytes of workspace, got ", workspace_bytes);
        if ((uintptr_t) workspace % 256 != 0) fail("batched_mat_mul: the workspace must be 256 byte aligned");
    }
    for (size_t i = 0; i < plan.slabs.size(); i++) {
        GemmLaunchPlan &lp = plan.slabs[i];
        const MatmulWorkspace &ws = plan.slab_workspaces[i];
        if (ws.counter_bytes > 0) {
            // the tile counters start at zero (a fill kernel, not a memset: the call may be under stream capture)
            hip_check((hipError_t) launch_fill_zero(workspace, ws.counter_bytes, stream), "counter fill launch");
            lp.p.counters = workspace;
        }
        // (the partial products sit behind the room of the largest slab's counters)
        if (ws.partial_bytes > 0) lp.p.workspace = (char *) workspace + plan.workspace.partial_offset();
        hip_check((hipError_t) (plan.f16 ? launch_gemm_f16(lp, stream) : launch_gemm_f32(lp, stream)), "matmul launch");
    }
}

}  // namespace kn

extern "C" {

const char *knhip_last_error(void) { return g_last_error.c_str(); }

// ---------------------------------------------------------------------------------------------- device shim

int knhip_device_count(int *count) {
    return guarded([&] {
        KN_REQUIRE(count != nullptr);
        *count = HipDevice::count();
        return KNHIP_OK;
    });
}

int knhip_device_name(int device, char *buf, size_t cap, size_t *needed) {
    return guarded([&] { return copy_out(HipDevice::name(device), buf, cap, needed); });
}

int knhip_malloc(int device, size_t bytes, void **ptr) {
    return guarded([&] {
        KN_REQUIRE(ptr != nullptr);
        HipDevice::check(device);
        hip_check(hipSetDevice(device), "hipSetDevice");
        hip_check(hipMalloc(ptr, std::max<size_t>(bytes, 1)), "hipMalloc");
        return KNHIP_OK;
    });
}

int knhip_free(int device, void *ptr) {
    return guarded([&] {
        HipDevice::check(device);
        hip_check(hipSetDevice(device), "hipSetDevice");
        hip_check(hipFree(ptr), "hipFree");
        return KNHIP_OK;
    });
}

static int do_memcpy(int device, void *dst, const void *src, size_t bytes, hipMemcpyKind kind) {
    return guarded([&] {
        HipDevice::check(device);
        KN_REQUIRE(bytes == 0 || (dst != nullptr && src != nullptr));
        hip_check(hipSetDevice(device), "hipSetDevice");
        if (bytes) hip_check(hipMemcpy(dst, src, bytes, kind), "hipMemcpy");
        return KNHIP_OK;
    });
}
int knhip_memcpy_h2d(int device, void *dst, const void *src, size_t bytes) { return do_memcpy(device, dst, src, bytes, hipMemcpyHostToDevice); }
int knhip_memcpy_d2h(int device, void *dst, const void *src, size_t bytes) { return do_memcpy(device, dst, src, bytes, hipMemcpyDeviceToHost); }
int knhip_memcpy_d2d(int device, void *dst, const void *src, size_t bytes) { return do_memcpy(device, dst, src, bytes, hipMemcpyDeviceToDevice); }

static int do_memcpy_async(int device, void *dst, const void *src, size_t bytes, hipMemcpyKind kind, void *stream) {
    return guarded([&] {
        HipDevice::check(device);
        KN_REQUIRE(bytes == 0 || (dst != nullptr && src != nullptr));
        hip_check(hipSetDevice(device), "hipSetDevice");
        if (bytes) hip_check(hipMemcpyAsync(dst, src, bytes, kind, (hipStream_t) stream), "hipMemcpyAsync");
        return KNHIP_OK;
    });
}
int knhip_memcpy_h2d_async(int device, void *dst, const void *src, size_t bytes, void *stream) {
    return do_memcpy_async(device, dst, src, bytes, hipMemcpyHostToDevice, stream);
}
int knhip_memcpy_d2h_async(int device, void *dst, const void *src, size_t bytes, void *stream) {
    return do_memcpy_async(device, dst, src, bytes, hipMemcpyDeviceToHost, stream);
}
int knhip_memcpy_d2d_async(int device, void *dst, const void *src, size_t bytes, void *stream) {
    return do_memcpy_async(device, dst, src, bytes, hipMemcpyDeviceToDevice, stream);
}

int knhip_stream_create(int device, void **stream) {
    return on_device(device, [&] {
        KN_REQUIRE(stream != nullptr);
        hipStream_t s = nullptr;
        hip_check(hipStreamCreate(&s), "hipStreamCreate");  // default priority
        *stream = s;
    });
}
int knhip_stream_destroy(int device, void *stream) {
    return on_device(device, [&] {
        KN_REQUIRE(stream != nullptr);
        hip_check(hipStreamDestroy((hipStream_t) stream), "hipStreamDestroy");
    });
}
int knhip_stream_synchronize(int device, void *stream) {
    return on_device(device, [&] { hip_check(hipStreamSynchronize((hipStream_t) stream), "hipStreamSynchronize"); });
}
int knhip_stream_wait_event(int device, void *stream, void *event) {
    return on_device(device, [&] {
        KN_REQUIRE(event != nullptr);
        hip_check(hipStreamWaitEvent((hipStream_t) stream, (hipEvent_t) event, 0), "hipStreamWaitEvent");
    });
}
int knhip_event_create(int device, void **event) {
    return on_device(device, [&] {
        KN_REQUIRE(event != nullptr);
        hipEvent_t e = nullptr;
        hip_check(hipEventCreate(&e), "hipEventCreate");
        *event = e;
    });
}
int knhip_event_destroy(int device, void *event) {
    return on_device(device, [&] {
        KN_REQUIRE(event != nullptr);
        hip_check(hipEventDestroy((hipEvent_t) event), "hipEventDestroy");
    });
}
int knhip_event_record(int device, void *event, void *stream) {
    return on_device(device, [&] {
        KN_REQUIRE(event != nullptr);
        hip_check(hipEventRecord((hipEvent_t) event, (hipStream_t) stream), "hipEventRecord");
    });
}
int knhip_event_synchronize(int device, void *event) {
    return on_device(device, [&] {
        KN_REQUIRE(event != nullptr);
        hip_check(hipEventSynchronize((hipEvent_t) event), "hipEventSynchronize");
    });
}
int knhip_event_elapsed_seconds(int device, void *start, void *end, float *seconds) {
    return on_device(device, [&] {
        KN_REQUIRE(start != nullptr && end != nullptr && seconds != nullptr);
        float ms = 0;
        hip_check(hipEventElapsedTime(&ms, (hipEvent_t) start, (hipEvent_t) end), "hipEventElapsedTime");
        *seconds = ms / 1000.0f;
    });
}

int knhip_batched_mat_mul_workspace_bytes(const knhip_matmul_args *args, size_t *bytes) {
    return guarded([&] {
        KN_REQUIRE(args != nullptr && bytes != nullptr);
        *bytes = matmul_api_plan(*args).workspace.total();
        return KNHIP_OK;
    });
}

int knhip_batched_mat_mul(int device, void *stream, const knhip_matmul_args *args, void *workspace, size_t workspace_bytes) {
    return on_device(device, [&] {
        KN_REQUIRE(args != nullptr);
        MatmulPlan plan = matmul_api_plan(*args);
        matmul_api_launch(plan, workspace, workspace_bytes, (ihipStream_t *) stream);
    });
}

int knhip_host_alloc(size_t bytes, void **ptr) {
    return guarded([&] {
        KN_REQUIRE(ptr != nullptr);
        hip_check(hipHostMalloc(ptr, std::max<size_t>(bytes, 1), hipHostMallocDefault), "hipHostMalloc");
        return KNHIP_OK;
    });
}

int knhip_host_free(void *ptr) {
    return guarded([&] {
        hip_check(hipHostFree(ptr), "hipHostFree");
        return KNHIP_OK;
    });
}

int knhip_device_synchronize(int device) {
    return guarded([&] {
        HipDevice::check(device);
        hip_check(hipSetDevice(device), "hipSetDevice");
        hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");
        return KNHIP_OK;
    });
}

// ---------------------------------------------------------------------------------------------- graph

int knhip_graph_new(knhip_graph **out) {
    return guarded([&] {
        KN_REQUIRE(out != nullptr);
        *out = new knhip_graph();
        return KNHIP_OK;
    });
}

int knhip_graph_clone(const knhip_graph *graph, knhip_graph **out) {
    return guarded([&] {
        KN_REQUIRE(graph != nullptr && out != nullptr);
        *out = new knhip_graph{graph->graph};
        return KNHIP_OK;
    });
}

void knhip_graph_free(knhip_graph *graph) { delete graph; }

int knhip_graph_deserialize(const uint8_t *blob, size_t len, knhip_graph **out) {
    return guarded([&] {
        KN_REQUIRE(blob != nullptr && out != nullptr);
        *out = new knhip_graph{Graph::deserialize(blob, len)};
        return KNHIP_OK;
    });
}

int knhip_graph_serialize(const knhip_graph *graph, uint8_t *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(graph != nullptr);
        std::vector<uint8_t> blob = graph->graph.serialize();
        if (needed) *needed = blob.size();
        if (buf == nullptr && cap == 0) return KNHIP_OK;
        if (cap < blob.size()) {
            g_last_error = "buffer too small";
            return KNHIP_BUFFER_TOO_SMALL;
        }
        std::memcpy(buf, blob.data(), blob.size());
        return KNHIP_OK;
    });
}

int knhip_graph_str(const knhip_graph *graph, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(graph != nullptr);
        return copy_out(graph->graph.str(), buf, cap, needed);
    });
}

#define KN_BUILD(expr)                          \
    return guarded([&] {                        \
        KN_REQUIRE(g != nullptr && out != nullptr); \
        *out = (expr);                          \
        return KNHIP_OK;                        \
    })

int knhip_graph_input(knhip_graph *g, const knhip_size_t *dims, size_t rank, int dtype, knhip_value *out) {
    KN_BUILD(g->graph.input(to_shape(dims, rank), to_dtype(dtype)));
}

int knhip_graph_constant(knhip_graph *g, const knhip_size_t *dims, size_t rank, int dtype, const void *data,
                         size_t data_bytes, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr);
        Shape shape = to_shape(dims, rank);
        DType dt = to_dtype(dtype);
        ConcreteShape cs = shape.unwrap_fixed("constant shape");
        if (data_bytes != concrete_size(cs) * dtype_bytes(dt))
            fail("constant data has ", data_bytes, " bytes, shape ", shape.str(), " of ", dtype_name(dt), " needs ",
                 concrete_size(cs) * dtype_bytes(dt));
        KN_REQUIRE(data != nullptr || data_bytes == 0);
        *out = g->graph.constant(shape, dt, data);
        return KNHIP_OK;
    });
}

int knhip_graph_view(knhip_graph *g, knhip_value input, const knhip_size_t *dims, size_t rank, knhip_value *out) {
    KN_BUILD(g->graph.view(input, to_shape(dims, rank)));
}
int knhip_graph_broadcast(knhip_graph *g, knhip_value input, const knhip_size_t *dims, size_t rank, knhip_value *out) {
    KN_BUILD(g->graph.broadcast(input, to_shape(dims, rank)));
}
int knhip_graph_repeat_unary(knhip_graph *g, knhip_value input, size_t axis, knhip_size_t count, knhip_value *out) {
    KN_BUILD(g->graph.repeat_unary(input, axis, Size(count.batch_exp, count.fixed_factor)));
}
int knhip_graph_flatten(knhip_graph *g, knhip_value input, size_t start_axis, knhip_value *out) {
    KN_BUILD(g->graph.flatten(input, start_axis));
}
int knhip_graph_permute(knhip_graph *g, knhip_value input, const size_t *permutation, size_t rank, knhip_value *out) {
    KN_BUILD(g->graph.permute(input, std::vector<size_t>(permutation, permutation + rank)));
}
int knhip_graph_slice(knhip_graph *g, knhip_value input, size_t axis, size_t start, size_t end, size_t step, knhip_value *out) {
    KN_BUILD(g->graph.slice(input, axis, SliceRange::make(start, end, step)));
}
int knhip_graph_index(knhip_graph *g, knhip_value input, size_t axis, size_t index, knhip_value *out) {
    KN_BUILD(g->graph.index(input, axis, index));
}
int knhip_graph_flip(knhip_graph *g, knhip_value input, size_t axis, knhip_value *out) { KN_BUILD(g->graph.flip(input, axis)); }
int knhip_graph_repeat(knhip_graph *g, knhip_value input, size_t axis, knhip_size_t count, int interleave, knhip_value *out) {
    KN_BUILD(interleave ? g->graph.repeat_interleave(input, axis, Size(count.batch_exp, count.fixed_factor))
                        : g->graph.repeat(input, axis, Size(count.batch_exp, count.fixed_factor)));
}
int knhip_graph_gather(knhip_graph *g, knhip_value input, size_t axis, knhip_value indices, knhip_value *out) {
    KN_BUILD(g->graph.gather(input, axis, indices));
}
int knhip_graph_concat(knhip_graph *g, const knhip_value *inputs, size_t count, size_t axis, const knhip_size_t *base_dims,
                       size_t base_rank, int dtype, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr && (inputs != nullptr || count == 0));
        std::optional<Shape> base;
        if (base_dims != nullptr) base = to_shape(base_dims, base_rank);
        std::optional<DType> dt;
        if (dtype >= 0) dt = to_dtype(dtype);
        *out = g->graph.concat(std::vector<Value>(inputs, inputs + count), axis, base, dt);
        return KNHIP_OK;
    });
}
int knhip_graph_pad(knhip_graph *g, knhip_value input, const size_t *pad_amount, size_t rank, knhip_value pad_value, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr && (pad_amount != nullptr || rank == 0));
        std::vector<std::pair<size_t, size_t>> pads;
        for (size_t i = 0; i < rank; i++) pads.push_back({pad_amount[2 * i], pad_amount[2 * i + 1]});
        *out = g->graph.pad(input, pads, pad_value);
        return KNHIP_OK;
    });
}
int knhip_graph_conv(knhip_graph *g, knhip_value input, knhip_value filter, size_t stride_y, size_t stride_x, size_t padding_y,
                     size_t padding_x, knhip_value *out) {
    KN_BUILD(g->graph.conv(input, filter, stride_y, stride_x, padding_y, padding_x));
}
int knhip_graph_linear(knhip_graph *g, knhip_value input, knhip_value weight, knhip_value *out) { KN_BUILD(g->graph.linear(input, weight)); }
int knhip_graph_mat_mul(knhip_graph *g, knhip_value left, knhip_value right, knhip_value *out) { KN_BUILD(g->graph.mat_mul(left, right)); }
int knhip_graph_batched_mat_mul(knhip_graph *g, knhip_value left, knhip_value right, knhip_value *out) {
    KN_BUILD(g->graph.batched_mat_mul(left, right));
}
int knhip_graph_softmax(knhip_graph *g, knhip_value input, size_t axis, knhip_value *out) { KN_BUILD(g->graph.softmax(input, axis)); }
int knhip_graph_layernorm(knhip_graph *g, knhip_value input, size_t axis, float eps, knhip_value *out) {
    KN_BUILD(g->graph.layernorm(input, axis, eps));
}
int knhip_graph_reduce(knhip_graph *g, knhip_value input, const size_t *axes, size_t count, int op, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr && (axes != nullptr || count == 0));
        if (op < 0 || op >= REDUCE_OP_COUNT) fail("invalid reduce op ", op);
        *out = g->graph.reduce(input, std::vector<size_t>(axes, axes + count), (ReduceOp) op);
        return KNHIP_OK;
    });
}
int knhip_graph_clamp(knhip_graph *g, knhip_value input, const void *min, const void *max, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr && min != nullptr && max != nullptr);
        DType dt = g->graph[input].dtype;
        *out = g->graph.clamp_dyn(input, DScalar::load(dt, min), DScalar::load(dt, max));
        return KNHIP_OK;
    });
}
int knhip_graph_relu(knhip_graph *g, knhip_value input, knhip_value *out) { KN_BUILD(g->graph.relu(input)); }
int knhip_graph_unary(knhip_graph *g, int op, int cast_dtype, knhip_value input, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr);
        if (op < 0 || op >= UNARY_OP_COUNT) fail("invalid unary op ", op);
        bool is_cast = op == KNHIP_UNARY_VALUE_CAST || op == KNHIP_UNARY_BIT_CAST;
        DType to = is_cast ? to_dtype(cast_dtype) : DType::F32;
        *out = g->graph.unary((UnaryOp) op, input, to);
        return KNHIP_OK;
    });
}
int knhip_graph_binary(knhip_graph *g, int op, knhip_value left, knhip_value right, knhip_value *out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr);
        if (op < 0 || op >= BINARY_OP_COUNT) fail("invalid binary op ", op);
        *out = g->graph.binary((BinaryOp) op, left, right);
        return KNHIP_OK;
    });
}
int knhip_graph_call(knhip_graph *g, const knhip_graph *callee, const knhip_value *inputs, size_t input_count,
                     knhip_value *outputs, size_t output_cap, size_t *output_count) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && callee != nullptr && (inputs != nullptr || input_count == 0));
        if (callee->graph.outputs.size() > output_cap) {
            if (output_count) *output_count = callee->graph.outputs.size();
            g_last_error = "buffer too small";
            return KNHIP_BUFFER_TOO_SMALL;
        }
        std::vector<Value> r = g->graph.call(callee->graph, std::vector<Value>(inputs, inputs + input_count));
        return copy_list(r, outputs, output_cap, output_count);
    });
}
int knhip_graph_output(knhip_graph *g, knhip_value value) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        g->graph.output(value);
        return KNHIP_OK;
    });
}
int knhip_graph_set_debug_id(knhip_graph *g, knhip_value value, const char *id) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && id != nullptr);
        g->graph.set_debug_id(value, id);
        return KNHIP_OK;
    });
}

int knhip_graph_value_count(const knhip_graph *g, size_t *count) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && count != nullptr);
        *count = g->graph.len();
        return KNHIP_OK;
    });
}
int knhip_graph_inputs(const knhip_graph *g, knhip_value *buf, size_t cap, size_t *count) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        return copy_list(g->graph.inputs, buf, cap, count);
    });
}
int knhip_graph_outputs(const knhip_graph *g, knhip_value *buf, size_t cap, size_t *count) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        return copy_list(g->graph.outputs, buf, cap, count);
    });
}
int knhip_graph_value_info(const knhip_graph *g, knhip_value value, knhip_value_info *info) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && info != nullptr);
        const ValueInfo &vi = g->graph[value];
        const Operation &op = vi.operation;
        std::memset(info, 0, sizeof *info);
        info->dtype = (int) vi.dtype;
        info->op = (int) op.kind;
        info->sub_op = op.kind == OpKind::Unary ? (int) op.unary : op.kind == OpKind::Binary ? (int) op.binary
                       : op.kind == OpKind::Reduce ? (int) op.reduce : -1;
        bool is_cast = op.kind == OpKind::Unary && (op.unary == UnaryOp::ValueCast || op.unary == UnaryOp::BitCast);
        info->cast_dtype = is_cast ? (int) op.cast_to : -1;
        info->rank = vi.shape.rank();
        info->operand_count = op.inputs.size();
        info->axis_count = op.kind == OpKind::Conv ? 4 : op.axes.size();
        info->non_output_uses = vi.non_output_uses;
        info->slice_start = op.range.start;
        info->slice_end = op.range.end;
        info->slice_step = op.range.step;
        info->eps = op.eps;
        info->is_hidden = g->graph.is_hidden(value) ? 1 : 0;
        return KNHIP_OK;
    });
}
int knhip_graph_value_shape(const knhip_graph *g, knhip_value value, knhip_size_t *dims, size_t cap) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        const Shape &s = g->graph[value].shape;
        if (cap < s.rank()) {
            g_last_error = "buffer too small";
            return KNHIP_BUFFER_TOO_SMALL;
        }
        for (size_t i = 0; i < s.rank(); i++) dims[i] = knhip_size_t{s.dims[i].fixed_factor, s.dims[i].batch_exp};
        return KNHIP_OK;
    });
}
int knhip_graph_value_operands(const knhip_graph *g, knhip_value value, knhip_value *buf, size_t cap) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        return copy_list(g->graph[value].operation.inputs, buf, cap, (size_t *) nullptr);
    });
}
int knhip_graph_value_axes(const knhip_graph *g, knhip_value value, size_t *buf, size_t cap) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr);
        const Operation &op = g->graph[value].operation;
        if (op.kind == OpKind::Conv) {
            std::vector<size_t> geometry = {op.conv.stride_y, op.conv.stride_x, op.conv.padding_y, op.conv.padding_x};
            return copy_list(geometry, buf, cap, (size_t *) nullptr);
        }
        return copy_list(op.axes, buf, cap, (size_t *) nullptr);
    });
}
int knhip_graph_value_constant(const knhip_graph *g, knhip_value value, const void **data, size_t *bytes) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && data != nullptr && bytes != nullptr);
        const Operation &op = g->graph[value].operation;
        if (op.kind != OpKind::Constant) fail("value ", value, " is not a constant");
        *data = op.tensor.bytes();
        *bytes = op.tensor.nbytes();
        return KNHIP_OK;
    });
}
int knhip_graph_as_single_const(const knhip_graph *g, knhip_value value, int *is_single, void *element) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && is_single != nullptr && element != nullptr);
        auto c = g->graph.as_single_const(value);
        *is_single = c.has_value() ? 1 : 0;
        if (c) c->store(element);
        return KNHIP_OK;
    });
}

int knhip_graph_as_const(const knhip_graph *g, knhip_value value, int *is_const, void *data, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && is_const != nullptr && needed != nullptr);
        auto c = g->graph.as_const(value);
        *is_const = c.has_value() ? 1 : 0;
        *needed = c ? c->nbytes() : 0;
        if (c && data != nullptr && cap >= c->nbytes() && c->nbytes() > 0) std::memcpy(data, c->bytes(), c->nbytes());
        return KNHIP_OK;
    });
}

int knhip_graph_infer_batch_size(const knhip_graph *g, const size_t *actual, const size_t *ranks, size_t input_count,
                                 int *status, int *has_batch, uint64_t *batch) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && status != nullptr && has_batch != nullptr && batch != nullptr);
        KN_REQUIRE(input_count == 0 || (actual != nullptr && ranks != nullptr));
        std::vector<ConcreteShape> shapes;
        size_t pos = 0;
        for (size_t i = 0; i < input_count; i++) {
            shapes.push_back(ConcreteShape(actual + pos, actual + pos + ranks[i]));
            pos += ranks[i];
        }
        std::optional<uint64_t> b;
        *status = (int) infer_batch_size(g->graph.input_shapes(), shapes, &b);
        *has_batch = b.has_value() ? 1 : 0;
        *batch = b.value_or(0);
        return KNHIP_OK;
    });
}

int knhip_optimizer_settings_default(knhip_optimizer_settings *settings) {
    return guarded([&] {
        KN_REQUIRE(settings != nullptr);
        OptimizerSettings d;
        *settings = knhip_optimizer_settings{d.optimize, d.force_bias_through_conv, d.fuse_layernorm, d.div_to_mul};
        return KNHIP_OK;
    });
}

int knhip_graph_optimize(const knhip_graph *g, const knhip_optimizer_settings *settings, knhip_graph **out) {
    return guarded([&] {
        KN_REQUIRE(g != nullptr && out != nullptr);
        OptimizerSettings s;
        if (settings) {
            s.optimize = settings->optimize != 0;
            s.force_bias_through_conv = settings->force_bias_through_conv != 0;
            s.fuse_layernorm = settings->fuse_layernorm != 0;
            s.div_to_mul = settings->div_to_mul != 0;
        }
        *out = new knhip_graph{optimize_graph(g->graph, s)};
        return KNHIP_OK;
    });
}

// ---------------------------------------------------------------------------------------------- executor

int knhip_executor_options_default(knhip_executor_options *o) {
    return guarded([&] {
        KN_REQUIRE(o != nullptr);
        const ExecutorOptions d;
        std::memset(o, 0, sizeof *o);
        o->struct_bytes = sizeof *o;
        o->plan_only = d.plan_only;
        o->preserve_inputs = d.planner.preserve_inputs;
        o->step_by_step = !d.fuse_small;
        o->fuse_attention = d.planner.fuse_attention;
        o->fuse_gated_matmul = d.planner.fuse_gated_matmul;
        o->group_matmuls = d.planner.group_matmuls;
        o->pack_matmul_constants = d.planner.pack_matmul_constants;
        o->pointwise_conv_as_matmul = d.planner.pointwise_conv_as_matmul;
        o->join_elementwise = d.planner.join_elementwise;
        o->split_reduce = d.planner.split_reduce;
        o->tiled_transpose = d.planner.generator.tiled_transpose;
        o->split_conv_channels = d.planner.split_conv_channels;
        o->plane_conv_any_width = d.planner.plane_conv_any_width;
        o->direct_gemm = d.planner.gemm.direct;
        o->split_k = d.planner.gemm.split_k;
        o->tail_split = d.planner.gemm.tail_split;
        o->dot_products = d.planner.gemm.dot_products;
        o->streaming_bytes = d.planner.generator.streaming_bytes;
        o->mapped_io_bytes = d.mapped_io_bytes;
        o->stream_weights_bytes = d.planner.stream_weights_bytes;
        return KNHIP_OK;
    });
}

namespace {

ExecutorOptions executor_options_from(const knhip_executor_options *o) {
    ExecutorOptions e;
    if (o == nullptr) return e;
    if (o->struct_bytes != sizeof *o)
        fail("knhip_executor_options.struct_bytes is ", o->struct_bytes, ", this library expects ", sizeof *o,
             " (fill the struct with knhip_executor_options_default first)");
    e.plan_only = o->plan_only != 0;
    e.fuse_small = o->step_by_step == 0;
    e.mapped_io_bytes = (size_t) o->mapped_io_bytes;
    PlannerOptions &p = e.planner;
    p.preserve_inputs = o->preserve_inputs != 0;
    p.fuse_attention = o->fuse_attention != 0;
    p.fuse_gated_matmul = o->fuse_gated_matmul != 0;
    p.group_matmuls = o->group_matmuls != 0;
    p.pack_matmul_constants = o->pack_matmul_constants != 0;
    p.pointwise_conv_as_matmul = o->pointwise_conv_as_matmul != 0;
    p.join_elementwise = o->join_elementwise != 0;
    p.split_reduce = o->split_reduce != 0;
    p.generator.tiled_transpose = o->tiled_transpose != 0;
    p.generator.streaming_bytes = (size_t) o->streaming_bytes;
    p.split_conv_channels = o->split_conv_channels != 0;
    p.plane_conv_any_width = o->plane_conv_any_width != 0;
    p.gemm.direct = o->direct_gemm != 0;
    p.gemm.split_k = o->split_k != 0;
    p.gemm.tail_split = o->tail_split != 0;
    p.gemm.dot_products = o->dot_products != 0;
    p.stream_weights_bytes = (size_t) o->stream_weights_bytes;
    return e;
}

}  // namespace

int knhip_executor_new(int device, const knhip_graph *graph, size_t batch_size, const knhip_executor_options *options,
                       knhip_executor **out) {
    return guarded([&] {
        KN_REQUIRE(graph != nullptr && out != nullptr);
        *out = new knhip_executor(device, graph->graph, batch_size, executor_options_from(options));
        return KNHIP_OK;
    });
}

int knhip_executor_new_from_blob(int device, const uint8_t *blob, size_t len, size_t batch_size,
                                 const knhip_executor_options *options, knhip_executor **out) {
    return guarded([&] {
        KN_REQUIRE(blob != nullptr && out != nullptr);
        Graph g = Graph::deserialize(blob, len);
        *out = new knhip_executor(device, g, batch_size, executor_options_from(options));
        return KNHIP_OK;
    });
}

void knhip_executor_free(knhip_executor *ex) {
    try {
        delete ex;
    } catch (...) {
    }
}

int knhip_executor_io_count(const knhip_executor *ex, size_t *inputs, size_t *outputs) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && inputs != nullptr && outputs != nullptr);
        *inputs = ex->ex.plan().inputs.size();
        *outputs = ex->ex.plan().outputs.size();
        return KNHIP_OK;
    });
}

int knhip_executor_io_info(const knhip_executor *ex, int is_output, size_t index, int *dtype, size_t *rank, size_t *dims, size_t cap) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && dtype != nullptr && rank != nullptr);
        const auto &list = is_output ? ex->ex.plan().outputs : ex->ex.plan().inputs;
        if (index >= list.size()) fail("index ", index, " out of range");
        const PlanTensor &t = list[index];
        *dtype = (int) t.dtype;
        *rank = t.shape.rank();
        if (dims == nullptr && cap == 0) return KNHIP_OK;
        if (cap < t.shape.rank()) {
            g_last_error = "buffer too small";
            return KNHIP_BUFFER_TOO_SMALL;
        }
        for (size_t i = 0; i < t.shape.rank(); i++) dims[i] = t.shape.shape()[i];
        return KNHIP_OK;
    });
}

int knhip_executor_evaluate(knhip_executor *ex, const void *const *inputs, const size_t *input_bytes, size_t input_count,
                            void *const *outputs, const size_t *output_bytes, size_t output_count) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        const Plan &plan = ex->ex.plan();
        if (input_count != plan.inputs.size()) fail("Wrong input count: expected ", plan.inputs.size(), ", got ", input_count);
        if (output_count != plan.outputs.size()) fail("Wrong output count: expected ", plan.outputs.size(), ", got ", output_count);
        KN_REQUIRE(input_count == 0 || (inputs != nullptr && input_bytes != nullptr));
        KN_REQUIRE(output_count == 0 || (outputs != nullptr && output_bytes != nullptr));
        for (size_t i = 0; i < input_count; i++) {
            const PlanTensor &t = plan.inputs[i];
            size_t expected = t.shape.size() * dtype_bytes(t.dtype);
            if (input_bytes[i] != expected) fail("Wrong size for input ", i, ": expected ", expected, " bytes, got ", input_bytes[i]);
            KN_REQUIRE(inputs[i] != nullptr || expected == 0);
        }
        for (size_t i = 0; i < output_count; i++) {
            const PlanTensor &t = plan.outputs[i];
            size_t expected = t.shape.size() * dtype_bytes(t.dtype);
            if (output_bytes[i] != expected) fail("Wrong size for output ", i, ": expected ", expected, " bytes, got ", output_bytes[i]);
            KN_REQUIRE(outputs[i] != nullptr || expected == 0);
        }
        ex->ex.evaluate(inputs, outputs);
        return KNHIP_OK;
    });
}

int knhip_executor_run_async(knhip_executor *ex) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        ex->ex.run_async();
        return KNHIP_OK;
    });
}

int knhip_executor_synchronize(knhip_executor *ex) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        ex->ex.synchronize();
        return KNHIP_OK;
    });
}

int knhip_executor_time_runs(knhip_executor *ex, size_t iterations, float *elapsed_ms) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && elapsed_ms != nullptr);
        *elapsed_ms = ex->ex.time_runs(iterations);
        return KNHIP_OK;
    });
}

int knhip_executor_input_ptr(const knhip_executor *ex, size_t index, void **ptr) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && ptr != nullptr);
        *ptr = ex->ex.input_ptr(index);
        return KNHIP_OK;
    });
}

int knhip_executor_output_ptr(const knhip_executor *ex, size_t index, void **ptr) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && ptr != nullptr);
        *ptr = ex->ex.output_ptr(index);
        return KNHIP_OK;
    });
}

int knhip_executor_stream(const knhip_executor *ex, void **stream) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && stream != nullptr);
        *stream = (void *) ex->ex.stream();
        return KNHIP_OK;
    });
}

int knhip_executor_set_profile(knhip_executor *ex, int enabled) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        ex->ex.set_profile(enabled != 0);
        return KNHIP_OK;
    });
}

int knhip_executor_last_profile(const knhip_executor *ex, int *available, knhip_profile *profile) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && available != nullptr && profile != nullptr);
        const auto &p = ex->ex.last_profile();
        *available = p.has_value() ? 1 : 0;
        std::memset(profile, 0, sizeof *profile);
        if (p) {
            for (int k = 0; k < STEP_KIND_COUNT; k++) profile->per_kind[k] = p->per_kind[k];
            profile->total_cpu = p->total_cpu;
            profile->total_gpu = p->total_gpu;
            profile->timing_overhead = p->timing_overhead;
            profile->step_count = p->step_seconds.size();
        }
        return KNHIP_OK;
    });
}

int knhip_executor_profile_step_seconds(const knhip_executor *ex, float *buf, size_t cap) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        const auto &p = ex->ex.last_profile();
        if (!p) fail("no profile available");
        return copy_list(p->step_seconds, buf, cap, (size_t *) nullptr);
    });
}

int knhip_executor_profile_str(const knhip_executor *ex, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        const auto &p = ex->ex.last_profile();
        if (!p) fail("no profile available");
        return copy_out(p->str(), buf, cap, needed);
    });
}

int knhip_executor_mem_usage(const knhip_executor *ex, knhip_mem_usage *usage) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && usage != nullptr);
        const Plan &p = ex->ex.plan();
        *usage = knhip_mem_usage{p.mem_usage.dedicated_bytes, p.mem_usage.shared_bytes, p.mem_usage.zero_bytes,
                                 p.mem_usage.hypo_shared_bytes_peak, p.mem_usage.hypo_shared_bytes_total, p.arena_bytes};
        return KNHIP_OK;
    });
}

int knhip_executor_step_count(const knhip_executor *ex, size_t *count) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && count != nullptr);
        *count = ex->ex.plan().steps.size();
        return KNHIP_OK;
    });
}

int knhip_executor_step_kind(const knhip_executor *ex, size_t index, int *kind) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && kind != nullptr);
        *kind = (int) ex->ex.plan().steps.at(index).kind;
        return KNHIP_OK;
    });
}

int knhip_executor_step_str(const knhip_executor *ex, size_t index, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        return copy_out(ex->ex.plan().steps.at(index).str(), buf, cap, needed);
    });
}

int knhip_executor_set_graph_mode(knhip_executor *ex, int enabled) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        ex->ex.set_graph_mode(enabled != 0);
        return KNHIP_OK;
    });
}

int knhip_executor_step_work(const knhip_executor *ex, size_t index, double *flops, double *bytes) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr && flops != nullptr && bytes != nullptr);
        const kn::Step &step = ex->ex.plan().steps.at(index);
        *flops = step.flops();
        *bytes = step.bytes();
        return KNHIP_OK;
    });
}

int knhip_executor_step_source(const knhip_executor *ex, size_t index, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        return copy_out(ex->ex.plan().steps.at(index).kernel.source, buf, cap, needed);
    });
}

int knhip_executor_fused_source(const knhip_executor *ex, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        return copy_out(ex->ex.fused_source(), buf, cap, needed);
    });
}

int knhip_executor_str(const knhip_executor *ex, char *buf, size_t cap, size_t *needed) {
    return guarded([&] {
        KN_REQUIRE(ex != nullptr);
        return copy_out(ex->ex.str(), buf, cap, needed);
    });
}

int knhip_strided_flags(const size_t *shape, const int64_t *strides, size_t rank, int *simple, int *dense) {
    return guarded([&] {
        KN_REQUIRE(simple != nullptr && dense != nullptr && (rank == 0 || (shape != nullptr && strides != nullptr)));
        StridedShape s(std::vector<size_t>(shape, shape + rank), std::vector<int64_t>(strides, strides + rank));
        *simple = s.has_simple_strides() ? 1 : 0;
        *dense = s.has_dense_strides() ? 1 : 0;
        return KNHIP_OK;
    });
}

int knhip_strided_view(const size_t *shape, const int64_t *strides, size_t rank, const size_t *new_shape, size_t new_rank,
                       int *ok, int64_t *new_strides) {
    return guarded([&] {
        KN_REQUIRE(ok != nullptr && (rank == 0 || (shape != nullptr && strides != nullptr)));
        KN_REQUIRE(new_rank == 0 || (new_shape != nullptr && new_strides != nullptr));
        StridedShape s(std::vector<size_t>(shape, shape + rank), std::vector<int64_t>(strides, strides + rank));
        auto v = s.view(std::vector<size_t>(new_shape, new_shape + new_rank));
        *ok = v.has_value() ? 1 : 0;
        if (v)
            for (size_t i = 0; i < new_rank; i++) new_strides[i] = v->strides()[i];
        return KNHIP_OK;
    });
}

int knhip_strided_slice(const size_t *shape, const int64_t *strides, size_t rank, size_t axis, size_t start, size_t end,
                        size_t step, size_t *out_shape, int64_t *out_strides) {
    return guarded([&] {
        KN_REQUIRE(shape != nullptr && strides != nullptr && out_shape != nullptr && out_strides != nullptr);
        StridedShape s(std::vector<size_t>(shape, shape + rank), std::vector<int64_t>(strides, strides + rank));
        StridedShape r = s.slice(axis, SliceRange::make(start, end, step));
        for (size_t i = 0; i < rank; i++) {
            out_shape[i] = r.shape()[i];
            out_strides[i] = r.strides()[i];
        }
        return KNHIP_OK;
    });
}

int knhip_compile_stats(size_t *compiled, size_t *memory_hits, size_t *disk_hits) {
    return guarded([&] {
        KN_REQUIRE(compiled != nullptr && memory_hits != nullptr && disk_hits != nullptr);
        CompileStats s = compile_stats();
        *compiled = s.compiled;
        *memory_hits = s.memory_hits;
        *disk_hits = s.disk_hits;
        return KNHIP_OK;
    });
}

}  // extern "C"
