// Kernels on caller-owned device tensors, outside any executor: the strided copy behind DeviceTensor::copy_from
// (kn-cuda-eval/src/device_tensor.rs:73-126) and the five autokernel types the reference exports from
// kn-cuda-eval/src/autokernel/ (ScalarKernel scalar.rs:33-154, ReduceKernel reduce.rs:35-153, SoftmaxKernel
// softmax.rs:28-108, LayernormKernel layernorm.rs:33-136, GatherKernel gather.rs:30-129). They are the executor's own
// generators (kernels.h) behind constructors that take shapes, strides and element types the way the reference's do.
#include <hip/hip_runtime.h>

#include <map>
#include <mutex>

#include "../../include/knhip.h"
#include "executor.h"
#include "kernels.h"
#include "matmul_api.h"
#include "rtc.h"

namespace kn {

namespace {

// Loaded code objects, per device, for the life of the process (the reference's kernel cache is never cleared
// either, autokernel/common.rs:14-21): a queued launch keeps needing its module after the call that queued it returned.
std::mutex g_modules_mutex;
std::map<std::pair<int, uint64_t>, hipModule_t> g_modules;

hipFunction_t function_for(int device, const KernelSpec &spec) {
    std::shared_ptr<const CodeObject> code = compile_kernel(spec.source);
    std::lock_guard<std::mutex> lock(g_modules_mutex);
    auto key = std::make_pair(device, code->key);
    auto it = g_modules.find(key);
    if (it == g_modules.end()) {
        hipModule_t module = nullptr;
        hipError_t e = hipModuleLoadData(&module, code->binary.data());
        if (e != hipSuccess && code->from_disk) {
            // a code object from the disk cache that the runtime refuses is built again, once
            (void) hipGetLastError();
            code = recompile_kernel(spec.source);
            e = hipModuleLoadData(&module, code->binary.data());
        }
        hip_check(e, "hipModuleLoadData");
        it = g_modules.emplace(key, module).first;
    }
    hipFunction_t function = nullptr;
    hip_check(hipModuleGetFunction(&function, it->second, spec.name.c_str()), "hipModuleGetFunction");
    return function;
}

DType dtype_of(int code) {
    if (code < 0 || code > KNHIP_F16) fail("invalid element type code ", code);
    return (DType) code;
}

// Alignment the generators may assume: a tensor given without an address is taken to start on a 256 byte boundary
// (what the allocator hands out); one given with its address is taken as aligned as that address is.
KernelOperand operand_of(const knhip_tensor &t) {
    if (t.rank > 0 && (t.shape == nullptr || t.strides == nullptr)) fail("tensor descriptor without shape or strides");
    KernelOperand op;
    op.dtype = dtype_of(t.dtype);
    op.shape = StridedShape(std::vector<size_t>(t.shape, t.shape + t.rank), std::vector<int64_t>(t.strides, t.strides + t.rank));
    op.offset_bytes = (int64_t) ((uintptr_t) t.ptr % 256);
    return op;
}

ScalarNode load_node(size_t operand, DType dtype) {
    ScalarNode n;
    n.kind = ScalarNode::Load;
    n.operand = operand;
    n.dtype = dtype;
    return n;
}
ScalarNode const_node(float v) {
    ScalarNode n;
    n.kind = ScalarNode::Const;
    n.dtype = DType::F32;
    n.constant = DScalar::f32(v);
    return n;
}
ScalarNode binary_node(BinaryOp op, size_t a, size_t b) {
    ScalarNode n;
    n.kind = ScalarNode::Binary;
    n.dtype = DType::F32;
    n.binary = op;
    n.a = a;
    n.b = b;
    return n;
}

}  // namespace

}  // namespace kn

using namespace kn;

struct knhip_kernel {
    int device = -1;  // -1: compiled only, cannot run
    KernelSpec spec;
    hipFunction_t function = nullptr;
    // run() takes the addresses in the order of the constructor's tensors; slot i of the launch reads argument order[i]
    std::vector<size_t> order;
    std::vector<unsigned> assumed_align;  // per run() argument: the address modulo 16 the kernel was built for
    std::vector<bool> optional;           // per run() argument: may be NULL
    std::string what;
};

namespace {

template <typename F>
int guarded(F f) {
    try {
        f();
        return KNHIP_OK;
    } catch (const std::exception &e) {
        set_last_error(e.what());
        return KNHIP_ERROR;
    } catch (...) {
        set_last_error("unknown failure");
        return KNHIP_ERROR;
    }
}

// `device` < 0: the kernel is generated and compiled for gfx950 and can be inspected, but not run (no GPU needed)
void finish(knhip_kernel &k, int device, const std::vector<const knhip_tensor *> &args) {
    k.device = device;
    for (const knhip_tensor *t : args) {
        k.assumed_align.push_back(t ? (unsigned) ((uintptr_t) t->ptr % 16) : 0u);
        k.optional.push_back(t == nullptr);
    }
    if (k.spec.grid == 0) return;  // nothing to do: an empty tensor
    if (device < 0) {
        (void) compile_kernel(k.spec.source);
        return;
    }
    HipDevice::check(device);
    hip_check(hipSetDevice(device), "hipSetDevice");
    k.function = function_for(device, k.spec);
}

void launch(const knhip_kernel &k, void *stream, void *const *ptrs, size_t count) {
    if (count != k.assumed_align.size()) fail(k.what, ": run takes ", k.assumed_align.size(), " addresses, got ", count);
    if (k.spec.grid == 0) return;
    if (k.device < 0) fail(k.what, ": this kernel was built without a device and cannot run");
    for (size_t i = 0; i < count; i++) {
        if (ptrs[i] == nullptr) {
            if (!k.optional[i]) fail(k.what, ": address ", i, " is null");
            continue;
        }
        if ((uintptr_t) ptrs[i] % 16 != k.assumed_align[i])
            fail(k.what, ": address ", i, " is ", (uintptr_t) ptrs[i] % 16, " modulo 16, the kernel was built for ", k.assumed_align[i],
                 " (pass the tensor's address to the constructor, or keep tensors 16 byte aligned)");
    }
    std::vector<void *> args(k.spec.n_ptrs, nullptr);
    KN_ASSERT(k.order.size() == k.spec.n_ptrs);
    for (size_t slot = 0; slot < k.order.size(); slot++) args[slot] = ptrs[k.order[slot]];
    hip_check(hipSetDevice(k.device), "hipSetDevice");
    void *params[] = {args.data()};
    hip_check(hipModuleLaunchKernel(k.function, k.spec.grid, 1, 1, k.spec.block, 1, 1, 0, (hipStream_t) stream, params, nullptr),
              "hipModuleLaunchKernel");
}

void require_same_shape(const KernelOperand &a, const KernelOperand &b, const char *what) {
    if (a.shape.shape() != b.shape.shape()) fail(what, ": shapes differ, ", a.shape.str(), " against ", b.shape.str());
}

}  // namespace

extern "C" {

int knhip_strided_copy(int device, void *stream, const knhip_tensor *dst, const knhip_tensor *src) {
    return guarded([&] {
        if (dst == nullptr || src == nullptr) fail("strided_copy: null tensor");
        const KernelOperand d = operand_of(*dst), s = operand_of(*src);
        if (d.dtype != s.dtype) fail("strided_copy: tensors must have the same dtype");
        require_same_shape(d, s, "strided_copy");
        const size_t elements = d.shape.size();
        if (elements == 0) return;
        if (dst->ptr == nullptr || src->ptr == nullptr) fail("strided_copy: null address");
        for (size_t a = 0; a < d.shape.rank(); a++)
            if (d.shape.shape()[a] > 1 && d.shape.strides()[a] == 0) fail("strided_copy: the destination has a broadcast axis: ", d.shape.str());
        HipDevice::check(device);
        hip_check(hipSetDevice(device), "hipSetDevice");
        if (d.shape == s.shape && d.shape.has_dense_strides()) {
            // same dense layout on both sides: one linear copy of the span (device_tensor.rs:115-118); a view whose
            // origin is not its lowest address (negative strides) starts that far below it
            const int64_t low = d.shape.offset_bounds().first * (int64_t) dtype_bytes(d.dtype);
            hip_check(hipMemcpyAsync((char *) dst->ptr + low, (const char *) src->ptr + low, elements * dtype_bytes(d.dtype),
                                     hipMemcpyDeviceToDevice, (hipStream_t) stream),
                      "hipMemcpyAsync");
            return;
        }
        // the restride fallback of device_tensor.rs:119-124: the elementwise kernel with the operation `y = x`
        ScalarExpr copy;
        copy.nodes = {load_node(1, s.dtype)};
        knhip_kernel k;
        k.what = "strided_copy";
        k.spec = make_scalar_kernel({d, s}, copy);
        k.order = {0, 1};
        finish(k, device, {dst, src});
        void *ptrs[2] = {dst->ptr, const_cast<void *>((const void *) src->ptr)};
        launch(k, stream, ptrs, 2);
    });
}

int knhip_scalar_kernel_new(int device, const char *operation, const knhip_tensor *operands, size_t operand_count, knhip_kernel **out) {
    return guarded([&] {
        if (operation == nullptr || operands == nullptr || out == nullptr) fail("scalar_kernel: null argument");
        if (operand_count < 1) fail("scalar_kernel: at least the result operand is needed");
        std::string text = operation;
        while (!text.empty() && isspace((unsigned char) text.back())) text.pop_back();
        if (text.empty() || text.back() != ';') fail("Operation should end with ';', got \"", operation, "\"");  // scalar.rs:51-55
        std::vector<KernelOperand> ops;
        std::vector<const knhip_tensor *> args;
        for (size_t i = 0; i < operand_count; i++) {
            ops.push_back(operand_of(operands[i]));
            args.push_back(&operands[i]);
            require_same_shape(ops[0], ops[i], "scalar_kernel");
        }
        for (size_t a = 0; a < ops[0].shape.rank(); a++)
            if (ops[0].shape.shape()[a] > 1 && ops[0].shape.strides()[a] == 0) fail("scalar_kernel: the result has a broadcast axis: ", ops[0].shape.str());
        ScalarExpr expr;
        for (size_t i = 1; i < operand_count; i++) expr.nodes.push_back(load_node(i, ops[i].dtype));
        ScalarNode raw;
        raw.kind = ScalarNode::Raw;
        raw.dtype = ops[0].dtype;
        raw.raw = text;
        expr.nodes.push_back(raw);
        auto k = std::make_unique<knhip_kernel>();
        k->what = "scalar_kernel";
        k->spec = make_scalar_kernel(ops, expr);
        for (size_t i = 0; i < operand_count; i++) k->order.push_back(i);
        finish(*k, device, args);
        *out = k.release();
    });
}

int knhip_reduce_kernel_new(int device, int reduce_op, const knhip_tensor *input, const knhip_tensor *output, const size_t *axes,
                            size_t axis_count, knhip_kernel **out) {
    return guarded([&] {
        if (input == nullptr || output == nullptr || out == nullptr || (axis_count > 0 && axes == nullptr)) fail("reduce_kernel: null argument");
        if (reduce_op < KNHIP_REDUCE_SUM || reduce_op > KNHIP_REDUCE_MIN) fail("reduce_kernel: invalid operation code ", reduce_op);
        const KernelOperand in = operand_of(*input), res = operand_of(*output);
        if (in.dtype != res.dtype) fail("reduce_kernel: input and output must have the same dtype");
        if ((ReduceOp) reduce_op == ReduceOp::Mean && in.dtype != DType::F32) fail("reduce_kernel: mean is only supported for f32");  // planner.rs:487-489
        std::vector<size_t> reduced(axes, axes + axis_count);
        std::vector<bool> is_reduced(in.shape.rank(), false);
        for (size_t a : reduced) {
            if (a >= in.shape.rank()) fail("Reduced axis out of bounds for shape ", in.shape.str());       // reduce.rs:49-55
            if (is_reduced[a]) fail("Reduced axes must be unique");                                          // reduce.rs:43-47
            is_reduced[a] = true;
        }
        std::vector<size_t> kept;
        for (size_t a = 0; a < in.shape.rank(); a++)
            if (!is_reduced[a]) kept.push_back(in.shape.shape()[a]);
        if (kept != res.shape.shape()) fail("reduce_kernel: the output shape ", res.shape.str(), " is not the input's kept axes");
        auto k = std::make_unique<knhip_kernel>();
        k->what = "reduce_kernel";
        k->spec = make_reduce_kernel(in, res, reduced, (ReduceOp) reduce_op);
        k->order = {0, 1};
        finish(*k, device, {input, output});
        *out = k.release();
    });
}

int knhip_softmax_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *output, size_t axis, float input_scale,
                             knhip_kernel **out) {
    return guarded([&] {
        if (input == nullptr || output == nullptr || out == nullptr) fail("softmax_kernel: null argument");
        const KernelOperand in = operand_of(*input), res = operand_of(*output);
        if (in.dtype != DType::F32 || res.dtype != DType::F32) fail("softmax_kernel: f32 only");
        require_same_shape(in, res, "softmax_kernel");
        if (axis >= in.shape.rank()) fail("softmax_kernel: axis ", axis, " out of bounds for ", in.shape.str());
        RowKernelDesc desc;
        desc.kind = RowKernelDesc::Softmax;
        desc.axis = axis;
        desc.operands = {res, in};
        desc.pre.nodes = {load_node(1, DType::F32)};
        if (input_scale != 1.0f) {
            desc.pre.nodes.push_back(const_node(input_scale));
            desc.pre.nodes.push_back(binary_node(BinaryOp::Mul, 0, 1));
        }
        desc.post.nodes = {load_node(SIZE_MAX, DType::F32)};
        auto k = std::make_unique<knhip_kernel>();
        k->what = "softmax_kernel";
        k->spec = make_row_kernel(desc);
        k->order = {1, 0};  // the generator takes the result first, run() takes (input, output)
        finish(*k, device, {input, output});
        *out = k.release();
    });
}

int knhip_layernorm_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *output, size_t axis, float eps, float alpha0,
                               float alpha1, float beta, knhip_kernel **out) {
    return guarded([&] {
        if (input == nullptr || output == nullptr || out == nullptr) fail("layernorm_kernel: null argument");
        const KernelOperand in = operand_of(*input), res = operand_of(*output);
        if (in.dtype != DType::F32 || res.dtype != DType::F32) fail("layernorm_kernel: f32 only");
        require_same_shape(in, res, "layernorm_kernel");
        if (axis >= in.shape.rank()) fail("layernorm_kernel: axis ", axis, " out of bounds for ", in.shape.str());
        // x = alpha0 * input0 + alpha1 * input1, y = beta * (x - mean) / sqrt(var + eps)   (layernorm.cu:31-96)
        const bool second = alpha1 != 0.0f;
        RowKernelDesc desc;
        desc.kind = RowKernelDesc::Layernorm;
        desc.axis = axis;
        desc.eps = eps;
        desc.operands = {res, in};
        if (second) desc.operands.push_back(in);  // input1 has input0's shape and strides (layernorm.rs:107-110)
        auto &pre = desc.pre.nodes;
        pre = {load_node(1, DType::F32)};
        if (alpha0 != 1.0f || second) {
            pre.push_back(const_node(alpha0));
            pre.push_back(binary_node(BinaryOp::Mul, 0, 1));
        }
        if (second) {
            const size_t first = pre.size() - 1;
            pre.push_back(load_node(2, DType::F32));
            pre.push_back(const_node(alpha1));
            pre.push_back(binary_node(BinaryOp::Mul, first + 1, first + 2));
            pre.push_back(binary_node(BinaryOp::Add, first, first + 3));
        }
        auto &post = desc.post.nodes;
        post = {load_node(SIZE_MAX, DType::F32)};
        if (beta != 1.0f) {
            post.push_back(const_node(beta));
            post.push_back(binary_node(BinaryOp::Mul, 1, 0));
        }
        auto k = std::make_unique<knhip_kernel>();
        k->what = "layernorm_kernel";
        k->spec = make_row_kernel(desc);
        // run() takes (input0, input1 or NULL, output)
        k->order = second ? std::vector<size_t>{2, 0, 1} : std::vector<size_t>{2, 0};
        finish(*k, device, {input, second ? input : nullptr, output});
        if (!second) k->optional[1] = true;
        *out = k.release();
    });
}

int knhip_gather_kernel_new(int device, const knhip_tensor *input, const knhip_tensor *indices, const knhip_tensor *output, size_t axis,
                            knhip_kernel **out) {
    return guarded([&] {
        if (input == nullptr || indices == nullptr || output == nullptr || out == nullptr) fail("gather_kernel: null argument");
        const KernelOperand in = operand_of(*input), idx = operand_of(*indices), res = operand_of(*output);
        if (in.dtype != res.dtype) fail("gather_kernel: input and output must have the same dtype");
        if (!dtype_is_int(idx.dtype)) fail("gather_kernel: indices must be integers");
        if (idx.shape.rank() != 1) fail("gather_kernel: indices must have rank 1");                          // gather.rs:45
        if (in.shape.rank() != res.shape.rank() || axis >= in.shape.rank()) fail("gather_kernel: rank or axis mismatch");
        if (idx.shape.size() != res.shape.shape()[axis]) fail("gather_kernel: the output's axis must have one entry per index");
        if (in.shape.remove(axis).shape() != res.shape.remove(axis).shape()) fail("gather_kernel: kept axes differ");
        auto k = std::make_unique<knhip_kernel>();
        k->what = "gather_kernel";
        k->spec = make_gather_kernel(in, idx, res, axis);
        k->order = {0, 1, 2};
        finish(*k, device, {input, indices, output});
        *out = k.release();
    });
}

int knhip_kernel_run(const knhip_kernel *kernel, void *stream, void *const *ptrs, size_t count) {
    return guarded([&] {
        if (kernel == nullptr || (count > 0 && ptrs == nullptr)) fail("kernel_run: null argument");
        launch(*kernel, stream, ptrs, count);
    });
}

int knhip_kernel_info(const knhip_kernel *kernel, char *strategy, size_t cap, size_t *needed, unsigned *grid, unsigned *block) {
    int status = guarded([&] {
        if (kernel == nullptr) fail("kernel_info: null argument");
        if (grid) *grid = kernel->spec.grid;
        if (block) *block = kernel->spec.block;
        if (needed) *needed = kernel->spec.strategy.size() + 1;
    });
    if (status != KNHIP_OK || (strategy == nullptr && cap == 0)) return status;
    if (cap < kernel->spec.strategy.size() + 1) {
        set_last_error("buffer too small");
        return KNHIP_BUFFER_TOO_SMALL;
    }
    std::memcpy(strategy, kernel->spec.strategy.c_str(), kernel->spec.strategy.size() + 1);
    return KNHIP_OK;
}

void knhip_kernel_free(knhip_kernel *kernel) { delete kernel; }

}  // extern "C"
