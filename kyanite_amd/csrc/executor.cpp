#include "executor.h"

// declared here instead of including <hip/hip_ext.h>, whose templates need the HIP compiler
extern "C" hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX, uint32_t globalWorkSizeY,
                                               uint32_t globalWorkSizeZ, uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                               uint32_t localWorkSizeZ, size_t sharedMemBytes, hipStream_t hStream,
                                               void **kernelParams, void **extra, hipEvent_t startEvent, hipEvent_t stopEvent,
                                               uint32_t flags);

#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <thread>

namespace kn {

// The host side of big staging copies, spread over a few threads: one thread copies 10 to 20 GB/s out of memory, less
// than the copy engine moves across the bus, so a tensor of hundreds of MB would wait for the host otherwise.
class HostCopyPool {
public:
    explicit HostCopyPool(size_t workers) {
        for (size_t i = 0; i < workers; i++) threads_.emplace_back([this] { work(); });
    }
    ~HostCopyPool() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            stop_ = true;
        }
        wake_.notify_all();
        for (auto &t : threads_) t.join();
    }
    // returns when all of [dst, dst + bytes) is written
    void copy(void *dst, const void *src, size_t bytes) {
        const size_t parts = threads_.size() + 1;
        const size_t part = (bytes / parts + 4095) & ~(size_t) 4095;
        size_t own = std::min(part, bytes);
        {
            std::lock_guard<std::mutex> lock(mutex_);
            for (size_t off = own; off < bytes; off += part) {
                jobs_.push_back({(char *) dst + off, (const char *) src + off, std::min(part, bytes - off)});
                pending_++;
            }
        }
        wake_.notify_all();
        std::memcpy(dst, src, own);
        std::unique_lock<std::mutex> lock(mutex_);
        done_.wait(lock, [this] { return pending_ == 0; });
    }

private:
    struct Job {
        char *dst;
        const char *src;
        size_t bytes;
    };
    void work() {
        std::unique_lock<std::mutex> lock(mutex_);
        while (true) {
            wake_.wait(lock, [this] { return stop_ || !jobs_.empty(); });
            if (stop_) return;
            Job job = jobs_.front();
            jobs_.pop_front();
            lock.unlock();
            std::memcpy(job.dst, job.src, job.bytes);
            lock.lock();
            if (--pending_ == 0) done_.notify_all();
        }
    }
    std::vector<std::thread> threads_;
    std::mutex mutex_;
    std::condition_variable wake_, done_;
    std::deque<Job> jobs_;
    size_t pending_ = 0;
    bool stop_ = false;
};

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) fail("HIP failure in ", what, ": ", hipGetErrorName(e), " (", hipGetErrorString(e), ")");
}

int HipDevice::count() {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) return 0;
    return n;
}

void HipDevice::check(int device) {
    int n = count();
    if (device < 0 || device >= n) fail("HIP device ", device, " is not available (", n, " device(s) visible)");
}

std::string HipDevice::name(int device) {
    check(device);
    hipDeviceProp_t prop;
    hip_check(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    return std::string(prop.name) + " (" + prop.gcnArchName + ")";
}

std::string Profile::str() const {
    std::ostringstream ss;
    ss << "Profile {\n  steps: [\n";
    for (auto &s : steps) ss << "    " << s << "\n";
    ss << "  ]\n";
    for (int k = 0; k < STEP_KIND_COUNT; k++) ss << "  " << step_kind_name((StepKind) k) << ": " << per_kind[k] << " s\n";
    ss << "  total_cpu: " << total_cpu << " s\n  total_gpu: " << total_gpu << " s\n  timing_overhead: " << timing_overhead << " s\n}\n";
    return ss.str();
}

namespace {

// A code object from the disk cache that the runtime refuses to load is dropped and built again, once.
hipModule_t load_code_object(std::shared_ptr<const CodeObject> &code, const std::string &source) {
    hipModule_t module = nullptr;
    hipError_t e = hipModuleLoadData(&module, code->binary.data());
    if (e != hipSuccess && code->from_disk) {
        (void) hipGetLastError();
        code = recompile_kernel(source);
        e = hipModuleLoadData(&module, code->binary.data());
    }
    hip_check(e, "hipModuleLoadData");
    return module;
}

}  // namespace

HipExecutor::HipExecutor(int device, const Graph &graph, size_t batch_size, const ExecutorOptions &executor_options)
    : device_(device), batch_size_(batch_size), plan_only_(executor_options.plan_only) {
    const bool plan_only = executor_options.plan_only, fuse_small = executor_options.fuse_small;
    if (!plan_only) HipDevice::check(device);
    const PlannerOptions &options = executor_options.planner;
    plan_ = plan_graph(graph, batch_size, options);
    if (fuse_small && plan_.steps.size() > 1) {
        std::vector<FusedPart> parts;
        bool ok = true;
        for (auto &step : plan_.steps) {
            FusedPart part;
            part.n_ptrs = step.operands.size();
            if (step.kind == StepKind::MatMul && !step.attention) {
                part.gemm = step.gemm;
                part.f16 = step.gemm_f16;
                part.has_addend = step.gemm_has_addend;
                part.has_addend2 = step.gemm_has_addend2;
            } else if (step.kind != StepKind::MatMul && step.kind != StepKind::Conv) {
                part.kernel = &step.kernel;
            } else {
                ok = false;
            }
            parts.push_back(part);
        }
        if (ok) fused_spec_ = make_fused_graph_kernel(parts);
        if (fused_spec_) {
            fused_code_ = compile_kernel(fused_spec_->source);
            // What launch_fused passes: the pointer table by value (at least one slot), the address of the completion
            // word and the number of the launch. The compiled kernel must expect exactly that many bytes of arguments.
            const size_t host_bytes = 8 * std::max<size_t>(fused_spec_->n_ptrs, 1) + 8 + 4;
            const size_t kernel_bytes = kernarg_segment_bytes(*fused_code_);
            if (kernel_bytes != host_bytes)
                fail("the one-kernel plan expects ", kernel_bytes, " bytes of launch arguments, the launch passes ", host_bytes);
        }
    }
    if (plan_only) return;

    hip_check(hipSetDevice(device_), "hipSetDevice");
    hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
    hip_check(hipMalloc((void **) &arena_, plan_.arena_bytes), "hipMalloc(arena)");
    // constants are uploaded once; the shared region needs no initialisation
    for (auto &up : plan_.uploads) {
        if (up.tensor.nbytes() == 0) continue;
        hip_check(hipMemcpy(arena_ + up.arena_offset, up.tensor.bytes(), up.tensor.nbytes(), hipMemcpyHostToDevice),
                  "hipMemcpy(constant)");
    }
    // plan-time copies of the constants are not needed any more
    plan_.uploads.clear();
    plan_.uploads.shrink_to_fit();

    // Page-locked staging for `evaluate`. Up to a few hundred MB it is set up here, so that the first evaluation is
    // as fast as the rest; beyond that it waits for the first `evaluate`, and a caller that keeps its own device
    // buffers and only ever calls `run_async` never pays for it.
    size_t staging_bytes = 0;
    for (auto &t : plan_.inputs) staging_bytes += t.shape.size() * dtype_bytes(t.dtype);
    for (auto &t : plan_.outputs) staging_bytes += t.shape.size() * dtype_bytes(t.dtype);
    if (staging_bytes <= ((size_t) 256 << 20)) allocate_staging();

    // load every distinct code object once and resolve the launch arguments
    std::map<uint64_t, hipModule_t> loaded;
    launches_.resize(plan_.steps.size());
    for (size_t si = 0; si < plan_.steps.size(); si++) {
        Step &step = plan_.steps[si];
        Launch &l = launches_[si];
        realise_launch(si, l, false);
        if (step.kind != StepKind::MatMul && step.kind != StepKind::Conv) {
            KN_ASSERT(step.code != nullptr, "kernel was not compiled");
            KN_ASSERT(l.ptrs.size() == step.kernel.n_ptrs);
            auto it = loaded.find(step.code->key);
            if (it == loaded.end()) {
                hipModule_t module = load_code_object(step.code, step.kernel.source);
                modules_.push_back(module);
                it = loaded.emplace(step.code->key, module).first;
            }
            hip_check(hipModuleGetFunction(&l.function, it->second, step.kernel.name.c_str()), "hipModuleGetFunction");
        }
    }

    // Mapped inputs / outputs for small graphs: every input and output in a shared buffer of its own, a few KB in all
    const size_t mapped_limit = executor_options.mapped_io_bytes;
    size_t io_bytes = 0;
    bool separate = true;
    std::vector<size_t> seen;
    auto own_buffer = [&](const PlanTensor &t) {
        io_bytes += t.shape.size() * dtype_bytes(t.dtype);
        if (t.ptr.kind != BufferKind::Shared || t.ptr.offset_bytes != 0 || !t.shape.has_simple_strides()) separate = false;
        for (size_t b : seen) separate &= b != t.ptr.index;
        seen.push_back(t.ptr.index);
    };
    for (auto &t : plan_.inputs) own_buffer(t);
    for (auto &t : plan_.outputs) own_buffer(t);
    if (separate && mapped_limit > 0 && io_bytes <= mapped_limit && !plan_.steps.empty()) {
        allocate_staging();
        mapped_launches_.resize(plan_.steps.size());
        for (size_t si = 0; si < plan_.steps.size(); si++) {
            mapped_launches_[si].function = launches_[si].function;
            realise_launch(si, mapped_launches_[si], true);
        }
        mapped_io_ = true;
    }
    if (fused_spec_) {
        hip_check(hipHostMalloc((void **) &fused_done_, 64, hipHostMallocCoherent), "hipHostMalloc");
        *fused_done_ = 0;
        hipModule_t module = load_code_object(fused_code_, fused_spec_->source);
        modules_.push_back(module);
        hip_check(hipModuleGetFunction(&fused_function_, module, fused_spec_->name.c_str()), "hipModuleGetFunction");
        for (auto &l : launches_) fused_ptrs_.insert(fused_ptrs_.end(), l.ptrs.begin(), l.ptrs.end());
        for (auto &l : mapped_launches_) fused_mapped_ptrs_.insert(fused_mapped_ptrs_.end(), l.ptrs.begin(), l.ptrs.end());
        KN_ASSERT(fused_ptrs_.size() == fused_spec_->n_ptrs && (!mapped_io_ || fused_mapped_ptrs_.size() == fused_spec_->n_ptrs));
        // (the kernel's table has at least one slot: the launch must never read it through a null data pointer)
        if (fused_ptrs_.empty()) fused_ptrs_.push_back(nullptr);
        if (mapped_io_ && fused_mapped_ptrs_.empty()) fused_mapped_ptrs_.push_back(nullptr);
    }
}

void HipExecutor::allocate_staging() {
    if (staging_ready_) return;
    auto pinned = [](const PlanTensor &t) {
        void *p = nullptr;
        hip_check(hipHostMalloc(&p, std::max<size_t>(t.shape.size() * dtype_bytes(t.dtype), 1), hipHostMallocCoherent), "hipHostMalloc");
        return p;
    };
    for (auto &t : plan_.inputs) pinned_inputs_.push_back(pinned(t));
    for (auto &t : plan_.outputs) pinned_outputs_.push_back(pinned(t));
    staging_ready_ = true;
}

const std::string &HipExecutor::fused_source() const {
    static const std::string none;
    return fused_spec_ ? fused_spec_->source : none;
}

void HipExecutor::launch_fused(bool mapped) {
    fused_seq_++;
    void *args[] = {mapped ? fused_mapped_ptrs_.data() : fused_ptrs_.data(), &fused_done_, &fused_seq_};
    hip_check(hipModuleLaunchKernel(fused_function_, 1, 1, 1, fused_spec_->block, 1, 1, 0, stream_, args, nullptr), "hipModuleLaunchKernel");
}

// The address of every operand of step `index`, and the launch parameters of the matrix-core kernels built from them.
void HipExecutor::realise_launch(size_t index, Launch &l, bool mapped) {
    Step &step = plan_.steps[index];
    l.ptrs.clear();
    for (auto &op : step.operands) {
        uint8_t *address = arena_ + plan_.resolve(op.tensor.ptr);
        if (mapped && op.tensor.ptr.kind == BufferKind::Shared) {
            // an operand inside the buffer of an input or output: the same place inside its page-locked buffer
            for (size_t i = 0; i < plan_.inputs.size(); i++)
                if (plan_.inputs[i].ptr.index == op.tensor.ptr.index) address = (uint8_t *) pinned_inputs_[i] + op.tensor.ptr.offset_bytes;
            for (size_t i = 0; i < plan_.outputs.size(); i++)
                if (plan_.outputs[i].ptr.index == op.tensor.ptr.index) address = (uint8_t *) pinned_outputs_[i] + op.tensor.ptr.offset_bytes;
        }
        l.ptrs.push_back(address);
    }
    if (step.kind == StepKind::MatMul && step.attention) {
        l.attn = step.attn;
        l.attn.q = l.ptrs[0];
        l.attn.k = l.ptrs[1];
        l.attn.v = l.ptrs[2];
        l.attn.mask = step.attention_has_mask ? l.ptrs[3] : nullptr;
        l.attn.block_class = step.attention_has_classes ? l.ptrs[4] : nullptr;
        l.attn.o = l.ptrs.back();
    } else if (step.kind == StepKind::MatMul && step.gemm.groups > 1) {
        GemmParams gemm = step.gemm;
        const size_t groups = (size_t) gemm.groups;
        const GemmLaunchPlan lp = plan_gemm_launch(gemm, step.gemm_f16);
        size_t next = 1 + 2 * groups;
        KN_ASSERT(l.ptrs.size() == next + (lp.workspace_bytes > 0) + (lp.counter_bytes > 0));
        gemm.a = l.ptrs[0];
        for (size_t g = 0; g < groups; g++) {
            gemm.b_group[g] = l.ptrs[1 + g];
            gemm.c_group[g] = l.ptrs[1 + groups + g];
        }
        gemm.b = gemm.b_group[0];
        gemm.c = gemm.c_group[0];
        gemm.workspace = lp.workspace_bytes > 0 ? l.ptrs[next++] : nullptr;
        gemm.counters = lp.counter_bytes > 0 ? l.ptrs[next++] : nullptr;
        l.gemm_plan = plan_gemm_launch(gemm, step.gemm_f16);
    } else if (step.kind == StepKind::MatMul && step.gemm.pair_op) {
        // a gated pair: left operand, the two right operands, the result
        GemmParams gemm = step.gemm;
        KN_ASSERT(l.ptrs.size() >= 4);
        gemm.a = l.ptrs[0];
        gemm.b = l.ptrs[1];
        gemm.b_pair = l.ptrs[2];
        gemm.c = l.ptrs[3];
        {
            const GemmLaunchPlan lp = plan_gemm_launch(gemm, step.gemm_f16);
            size_t next = 4;
            KN_ASSERT(l.ptrs.size() == next + (lp.workspace_bytes > 0) + (lp.counter_bytes > 0));
            gemm.workspace = lp.workspace_bytes > 0 ? l.ptrs[next++] : nullptr;
            gemm.counters = lp.counter_bytes > 0 ? l.ptrs[next++] : nullptr;
        }
        // the kernel reaches both right operands with 32 bit byte offsets from the lower of the two
        const long long apart = std::llabs((const char *) gemm.b_pair - (const char *) gemm.b);
        if (apart + ((long long) (gemm.n / 2) * gemm.b_sn + gemm.k) * 2 >= 0xffffffffll)
            fail("the two weights of a gated matmul lie ", apart, " bytes apart in the arena, out of the kernel's reach; "
                 "build the executor with fuse_gated_matmul = 0");
        l.gemm_plan = plan_gemm_launch(gemm, step.gemm_f16);
    } else if (step.kind == StepKind::MatMul) {
        GemmParams gemm = step.gemm;
        gemm.a = l.ptrs[0];
        gemm.b = l.ptrs[1];
        gemm.c = l.ptrs[2];
        size_t next = 3;
        gemm.addend = step.gemm_has_addend ? l.ptrs[next++] : nullptr;
        gemm.addend2 = step.gemm_has_addend2 ? l.ptrs[next++] : nullptr;
        const GemmLaunchPlan lp = plan_gemm_launch(gemm, step.gemm_f16);
        KN_ASSERT(l.ptrs.size() == next + (lp.workspace_bytes > 0) + (lp.counter_bytes > 0));
        gemm.workspace = lp.workspace_bytes > 0 ? l.ptrs[next++] : nullptr;
        gemm.counters = lp.counter_bytes > 0 ? l.ptrs[next++] : nullptr;
        l.gemm_plan = plan_gemm_launch(gemm, step.gemm_f16);
    } else if (step.kind == StepKind::Conv) {
        size_t k = 0;
        l.conv = step.conv;
        l.conv.input = (const float *) l.ptrs[k++];
        l.conv.filter = (const float *) l.ptrs[k++];
        l.conv.bias = step.conv_has_bias ? (const float *) l.ptrs[k++] : nullptr;
        l.conv.res = step.conv_has_res ? (const float *) l.ptrs[k++] : nullptr;
        l.conv.output = (float *) l.ptrs[k++];
        l.conv.workspace = k < l.ptrs.size() ? (float *) l.ptrs[k++] : nullptr;
        l.conv.counters = k < l.ptrs.size() ? (int *) l.ptrs[k++] : nullptr;
    }
}

HipExecutor::~HipExecutor() {
    if (plan_only_) return;
    // failures while tearing down are ignored on purpose (the reference does the same in its drop handlers)
    (void) hipSetDevice(device_);
    if (stream_) (void) hipStreamSynchronize(stream_);
    if (graph_exec_) (void) hipGraphExecDestroy(graph_exec_);
    if (fused_done_) (void) hipHostFree(fused_done_);
    for (hipEvent_t e : chunk_events_) (void) hipEventDestroy(e);
    for (void *p : pinned_inputs_) (void) hipHostFree(p);
    for (void *p : pinned_outputs_) (void) hipHostFree(p);
    for (hipModule_t m : modules_) (void) hipModuleUnload(m);
    if (arena_) (void) hipFree(arena_);
    if (stream_) (void) hipStreamDestroy(stream_);
}

void *HipExecutor::input_ptr(size_t i) const {
    KN_ASSERT(!plan_only_ && i < plan_.inputs.size());
    return arena_ + plan_.resolve(plan_.inputs[i].ptr);
}

void *HipExecutor::output_ptr(size_t i) const {
    KN_ASSERT(!plan_only_ && i < plan_.outputs.size());
    return arena_ + plan_.resolve(plan_.outputs[i].ptr);
}

void HipExecutor::synchronize() {
    KN_ASSERT(!plan_only_);
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
}

float HipExecutor::time_runs(size_t iterations) {
    KN_ASSERT(!plan_only_);
    bool was_profiling = profile_;
    profile_ = false;
    hip_check(hipSetDevice(device_), "hipSetDevice");
    hipEvent_t start, stop;
    hip_check(hipEventCreate(&start), "hipEventCreate");
    hip_check(hipEventCreate(&stop), "hipEventCreate");
    hip_check(hipEventRecord(start, stream_), "hipEventRecord");
    for (size_t i = 0; i < iterations; i++) run_async();
    hip_check(hipEventRecord(stop, stream_), "hipEventRecord");
    hip_check(hipEventSynchronize(stop), "hipEventSynchronize");
    float ms = 0;
    hip_check(hipEventElapsedTime(&ms, start, stop), "hipEventElapsedTime");
    (void) hipEventDestroy(start);
    (void) hipEventDestroy(stop);
    profile_ = was_profiling;
    return ms;
}

void HipExecutor::launch_step(size_t index, hipEvent_t start, hipEvent_t stop, bool mapped) {
    Step &step = plan_.steps[index];
    Launch &l = mapped ? mapped_launches_[index] : launches_[index];
    bool jit = step.kind != StepKind::MatMul && step.kind != StepKind::Conv;
    if (start && jit && (uint64_t) step.kernel.grid * step.kernel.block <= 0xffffffffull) {
        // the events are attached to the dispatch itself, so they time the kernel without any launch gaps
        void *args[] = {l.ptrs.data()};
        hip_check(hipExtModuleLaunchKernel(l.function, step.kernel.grid * step.kernel.block, 1, 1, step.kernel.block, 1, 1, 0,
                                           stream_, args, nullptr, start, stop, 0),
                  "hipExtModuleLaunchKernel");
        return;
    }
    if (start) hip_check(hipEventRecord(start, stream_), "hipEventRecord");
    switch (step.kind) {
        case StepKind::MatMul:
            if (step.attention) {
                hip_check((hipError_t) (step.gemm_f16 ? launch_attention_f16(l.attn, stream_) : launch_attention_f32(l.attn, stream_)),
                          "attention launch");
                break;
            }
            hip_check((hipError_t) (step.gemm_f16 ? launch_gemm_f16(l.gemm_plan, stream_) : launch_gemm_f32(l.gemm_plan, stream_)),
                      "matmul launch");
            break;
        case StepKind::Conv: hip_check((hipError_t) launch_conv_f32(l.conv, stream_), "conv launch"); break;
        default: {
            void *args[] = {l.ptrs.data()};
            hip_check(hipModuleLaunchKernel(l.function, step.kernel.grid, 1, 1, step.kernel.block, 1, 1, 0, stream_, args, nullptr),
                      "hipModuleLaunchKernel");
            break;
        }
    }
    if (stop) hip_check(hipEventRecord(stop, stream_), "hipEventRecord");
}

void HipExecutor::run_async() {
    if (plan_only_) fail("this executor was created without a device and cannot run");
    int current = -1;
    hip_check(hipGetDevice(&current), "hipGetDevice");
    if (current != device_) hip_check(hipSetDevice(device_), "hipSetDevice");

    if (!profile_) {
        last_profile_ = std::nullopt;
        if (fused_function_ && !graph_mode_) {
            launch_fused(false);
            return;
        }
        if (graph_mode_ && !plan_.steps.empty()) {
            if (!graph_exec_) {
                // the launch list is fixed for the lifetime of the executor (same kernels, same arena addresses)
                hipGraph_t graph = nullptr;
                hip_check(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
                try {
                    for (size_t si = 0; si < plan_.steps.size(); si++) launch_step(si);
                } catch (...) {
                    (void) hipStreamEndCapture(stream_, &graph);
                    if (graph) (void) hipGraphDestroy(graph);
                    throw;
                }
                hip_check(hipStreamEndCapture(stream_, &graph), "hipStreamEndCapture");
                hipError_t e = hipGraphInstantiate(&graph_exec_, graph, nullptr, nullptr, 0);
                (void) hipGraphDestroy(graph);
                hip_check(e, "hipGraphInstantiate");
            }
            hip_check(hipGraphLaunch(graph_exec_, stream_), "hipGraphLaunch");
            return;
        }
        for (size_t si = 0; si < plan_.steps.size(); si++) launch_step(si);
        return;
    }

    // executor.rs:208-257: one event pair per step
    using clock = std::chrono::steady_clock;
    size_t n = plan_.steps.size();
    std::vector<hipEvent_t> events(2 * n + 2);
    for (auto &e : events) hip_check(hipEventCreate(&e), "hipEventCreate");
    hip_check(hipEventRecord(events[2 * n], stream_), "hipEventRecord");
    hip_check(hipEventSynchronize(events[2 * n]), "hipEventSynchronize");
    auto start_cpu = clock::now();
    for (size_t si = 0; si < n; si++) {
        launch_step(si, events[2 * si], events[2 * si + 1]);
    }
    hip_check(hipEventRecord(events[2 * n + 1], stream_), "hipEventRecord");
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    auto end_cpu = clock::now();

    Profile profile;
    for (size_t si = 0; si < n; si++) {
        float ms = 0;
        hip_check(hipEventElapsedTime(&ms, events[2 * si], events[2 * si + 1]), "hipEventElapsedTime");
        profile.per_kind[(int) plan_.steps[si].kind] += ms * 1e-3f;
        profile.step_seconds.push_back(ms * 1e-3f);
        char buf[64];
        snprintf(buf, sizeof buf, "%4zu time %10.4f ms, step ", si, ms);
        profile.steps.push_back(buf + plan_.steps[si].str());
    }
    float total_ms = 0;
    hip_check(hipEventElapsedTime(&total_ms, events[2 * n], events[2 * n + 1]), "hipEventElapsedTime");
    profile.total_gpu = total_ms * 1e-3f;
    profile.total_cpu = std::chrono::duration<float>(end_cpu - start_cpu).count();
    for (auto &e : events) (void) hipEventDestroy(e);
    profile.timing_overhead = std::chrono::duration<float>(clock::now() - end_cpu).count();
    last_profile_ = std::move(profile);
}

void HipExecutor::host_copy(void *dst, const void *src, size_t bytes) {
    // below a few MB a second thread would still be waking up when the first one is done
    if (bytes < ((size_t) 2 << 20)) {
        std::memcpy(dst, src, bytes);
        return;
    }
    if (!copy_pool_) copy_pool_ = std::make_unique<HostCopyPool>(3);
    copy_pool_->copy(dst, src, bytes);
}

// The chunk a tensor of `bytes` moves in between page-locked staging and the device: a quarter of it, between
// `kCopyChunkLeast` and `kCopyChunkBytes`, so that tensors of a few MB already overlap the host's copy with the copy
// engine's (a 512 token LLaMA evaluation with 4 MB in and out 0.885 -> 0.853 ms, the UNet block with 10.5 MB each
// way 1.90 -> 1.75 ms, the ResNet tower with 19 MB of policies 4.21 -> 4.13 ms against one chunk of 8 MB).
size_t HipExecutor::copy_chunk_bytes(size_t bytes) {
    const size_t grain = (size_t) 256 << 10;
    const size_t quarter = (bytes / 4 + grain - 1) & ~(grain - 1);
    return std::min(kCopyChunkBytes, std::max(quarter, kCopyChunkLeast));
}

void HipExecutor::evaluate(const void *const *inputs, void *const *outputs) {
    if (plan_only_) fail("this executor was created without a device and cannot run");
    hip_check(hipSetDevice(device_), "hipSetDevice");
    allocate_staging();
    // The staging buffers are free: every evaluate ends with a synchronisation, and run_async never touches them.
    // Device work a caller queued through run_async is ordered before the copies below by the stream itself.
    const bool mapped = mapped_io_ && !profile_ && !graph_mode_;
    for (size_t i = 0; i < plan_.inputs.size(); i++) {
        const size_t bytes = plan_.inputs[i].shape.size() * dtype_bytes(plan_.inputs[i].dtype);
        KN_ASSERT(plan_.inputs[i].shape.has_simple_strides());
        const size_t chunk = copy_chunk_bytes(bytes);
        for (size_t off = 0; off < bytes; off += chunk) {
            const size_t n = std::min(chunk, bytes - off);
            host_copy((char *) pinned_inputs_[i] + off, (const char *) inputs[i] + off, n);
            if (!mapped)
                hip_check(hipMemcpyAsync((char *) input_ptr(i) + off, (char *) pinned_inputs_[i] + off, n, hipMemcpyHostToDevice, stream_),
                          "hipMemcpyAsync(H2D)");
        }
    }
    struct Chunk {
        size_t output, offset, bytes;
    };
    std::vector<Chunk> chunks;
    for (size_t i = 0; i < plan_.outputs.size(); i++) {
        const size_t bytes = plan_.outputs[i].shape.size() * dtype_bytes(plan_.outputs[i].dtype);
        const size_t chunk = copy_chunk_bytes(bytes);
        for (size_t off = 0; off < bytes; off += chunk) chunks.push_back({i, off, std::min(chunk, bytes - off)});
    }
    // an event behind every chunk but the last, so that the host can copy a chunk out while the next ones still move
    // (outputs that do not make the smallest chunk between them wait for the stream once instead)
    size_t output_bytes = 0;
    for (auto &ch : chunks) output_bytes += ch.bytes;
    const size_t n_events = output_bytes > kCopyChunkLeast ? chunks.size() - 1 : 0;
    if (mapped) {
        last_profile_ = std::nullopt;
        if (fused_function_) launch_fused(true);
        else for (size_t si = 0; si < plan_.steps.size(); si++) launch_step(si, nullptr, nullptr, true);
    } else {
        run_async();
        while (chunk_events_.size() < n_events) {
            hipEvent_t e = nullptr;
            hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
            chunk_events_.push_back(e);
        }
        for (size_t c = 0; c < chunks.size(); c++) {
            const Chunk &ch = chunks[c];
            hip_check(hipMemcpyAsync((char *) pinned_outputs_[ch.output] + ch.offset, (char *) output_ptr(ch.output) + ch.offset, ch.bytes,
                                     hipMemcpyDeviceToHost, stream_),
                      "hipMemcpyAsync(D2H)");
            if (c < n_events) hip_check(hipEventRecord(chunk_events_[c], stream_), "hipEventRecord");
        }
    }
    // The fused kernel of a small graph reports its own completion: after its last store every thread fences at
    // system scope and one thread writes this evaluation's number into a page-locked word, which the host polls.
    // That is a bus write away from the end of the kernel, where the runtime's own completion path adds about 6 us.
    bool done = false;
    if (mapped && fused_function_) {
        // (an acquire load: the outputs are read from page-locked memory right behind it)
        for (int spin = 0; spin < 400000 && !done; spin++) done = __atomic_load_n(fused_done_, __ATOMIC_ACQUIRE) == fused_seq_;
    }
    bool synchronized = done;
    if (mapped && !done) {
        hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
        synchronized = true;
    }
    for (size_t c = 0; c < chunks.size(); c++) {
        const Chunk &ch = chunks[c];
        if (c < n_events && !mapped) {
            hip_check(hipEventSynchronize(chunk_events_[c]), "hipEventSynchronize");
        } else if (!synchronized) {
            hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
            synchronized = true;
        }
        host_copy((char *) outputs[ch.output] + ch.offset, (char *) pinned_outputs_[ch.output] + ch.offset, ch.bytes);
    }
    if (!synchronized) hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    for (size_t i = 0; i < plan_.outputs.size(); i++) {
        if (plan_.outputs[i].dtype != DType::Bool) continue;
        const uint8_t *bytes = (const uint8_t *) outputs[i];
        for (size_t k = 0, n = plan_.outputs[i].shape.size(); k < n; k++)
            if (bytes[k] > 1) fail("bool output ", i, " holds a value other than 0 or 1");
    }
}

std::string HipExecutor::str() const {
    std::ostringstream ss;
    ss << "HipExecutor {\n  device: " << device_ << ",\n  batch_size: " << batch_size_ << ",\n  arena_bytes: " << plan_.arena_bytes
       << ",\n  mem_usage: { dedicated: " << plan_.mem_usage.dedicated_bytes << ", shared: " << plan_.mem_usage.shared_bytes
       << ", zero: " << plan_.mem_usage.zero_bytes << ", hypo_peak: " << plan_.mem_usage.hypo_shared_bytes_peak
       << ", hypo_total: " << plan_.mem_usage.hypo_shared_bytes_total << " },\n  steps: [\n";
    for (auto &s : plan_.steps) ss << "    " << s.str() << "\n";
    ss << "  ]" << (fused_spec_ ? ",\n  launched as one kernel: " + fused_spec_->strategy : std::string()) << "\n}\n";
    return ss.str();
}

}  // namespace kn
