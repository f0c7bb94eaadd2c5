// HipExecutor: the MI355X counterpart of CudaExecutor (kn-cuda-eval/src/executor.rs:20-37, :60-258).
// new(device, graph, batch_size) plans the graph into one device arena; evaluate(inputs) copies the inputs in,
// launches the planned steps in order on one stream and copies the outputs back.
#pragma once

#include <hip/hip_runtime_api.h>

#include "fused_graph.h"
#include "planner.h"

namespace kn {

struct Profile {  // executor.rs:43-58
    std::vector<std::string> steps;
    std::vector<float> step_seconds;
    float per_kind[STEP_KIND_COUNT] = {0};
    float total_cpu = 0, total_gpu = 0, timing_overhead = 0;
    std::string str() const;
};

class HipDevice {  // kn-cuda-sys/src/wrapper/handle.rs:37-103
public:
    static int count();
    static void check(int device);  // fails when the device does not exist
    static std::string name(int device);
};

// What an executor is built with beyond (device, graph, batch size); the defaults are the reference's behaviour plus
// every planned path of this library switched on. One executor's options do not touch another's.
struct ExecutorOptions {
    bool plan_only = false;   // build and compile the plan without touching a device (no allocation, no launches)
    bool fuse_small = true;   // a plan of a few tiny steps is launched as one kernel (fused_graph.h)
    // `evaluate` of a graph whose inputs and outputs are at most this many bytes in all reads and writes them in
    // page-locked host memory instead of copying them to and from the arena (0: never)
    size_t mapped_io_bytes = 64 * 1024;
    // (`planner.preserve_inputs` keeps the input buffers from being reused for later values, for callers that write
    // the inputs on the device once and then call run_async many times)
    PlannerOptions planner;
};

class HostCopyPool;

class HipExecutor {
public:
    HipExecutor(int device, const Graph &graph, size_t batch_size, const ExecutorOptions &options = ExecutorOptions());
    ~HipExecutor();
    HipExecutor(const HipExecutor &) = delete;
    HipExecutor &operator=(const HipExecutor &) = delete;

    // Dense host buffers in, dense host buffers out (executor.rs:117-195; the C ABI has checked counts and sizes).
    // Every byte crosses host memory once on each side: caller -> page-locked staging -> device and back. Tensors of
    // more than `kCopyChunkLeast` move in chunks (a quarter of the tensor, `kCopyChunkBytes` at most), so that the
    // copy engine works on one chunk while the host copies the next one (inputs) or the one before (outputs), with
    // the host copies of chunks spread over a few threads.
    void evaluate(const void *const *inputs, void *const *outputs);
    static constexpr size_t kCopyChunkBytes = (size_t) 8 << 20, kCopyChunkLeast = (size_t) 2 << 20;
    static size_t copy_chunk_bytes(size_t bytes);
    // launch the steps on the executor's stream without any synchronisation (executor.rs:197-258)
    void run_async();
    void synchronize();
    // `iterations` back-to-back runs timed with events on the executor's stream; elapsed milliseconds in total
    float time_runs(size_t iterations);

    // Replay the launch list as one HIP graph (captured from the executor's stream on the first run after switching
    // it on) instead of launching every step: one submission per evaluation, for graphs of small kernels where the
    // launches dominate. Profiled runs always launch step by step.
    void set_graph_mode(bool on) { graph_mode_ = on; }
    bool graph_mode() const { return graph_mode_; }

    void set_profile(bool on) { profile_ = on; }
    const std::optional<Profile> &last_profile() const { return last_profile_; }

    int device() const { return device_; }
    size_t batch_size() const { return batch_size_; }
    const Plan &plan() const { return plan_; }
    hipStream_t stream() const { return stream_; }
    // device addresses of the (dense, row-major) input and output tensors
    void *input_ptr(size_t i) const;
    void *output_ptr(size_t i) const;
    std::string str() const;
    // whether the whole plan runs as one generated kernel, and that kernel's source
    bool fused() const { return fused_spec_.has_value(); }
    const std::string &fused_source() const;

private:
    // the launch arguments of one step with every operand at its final address
    struct Launch {
        hipFunction_t function = nullptr;
        std::vector<void *> ptrs;
        GemmLaunchPlan gemm_plan{};
        AttentionParams attn{};
        ConvParams conv{};
    };
    // `mapped`: the variant of the launch whose inputs and outputs are the page-locked host buffers themselves
    void launch_step(size_t index, hipEvent_t start = nullptr, hipEvent_t stop = nullptr, bool mapped = false);
    void realise_launch(size_t index, Launch &l, bool mapped);

    int device_;
    size_t batch_size_;
    bool plan_only_;
    Plan plan_;
    uint8_t *arena_ = nullptr;
    hipStream_t stream_ = nullptr;
    std::vector<hipModule_t> modules_;
    std::vector<Launch> launches_;
    // Small graphs (inputs and outputs of a few KB): `evaluate` runs the steps on launches whose input / output
    // operands point at the page-locked staging buffers, which the device reads and writes across the bus, so an
    // evaluation is the launches and one synchronisation, without copy commands in between.
    std::vector<Launch> mapped_launches_;
    bool mapped_io_ = false;
    // A plan of a few tiny steps as ONE generated kernel, one workgroup (fused_graph.h); runs that are not profiled
    // launch it instead of the steps.
    std::optional<KernelSpec> fused_spec_;
    std::shared_ptr<const CodeObject> fused_code_;
    hipFunction_t fused_function_ = nullptr;
    std::vector<void *> fused_ptrs_, fused_mapped_ptrs_;
    uint32_t *fused_done_ = nullptr;  // page-locked word that the fused kernel writes the number of its launch into
    uint32_t fused_seq_ = 0;
    void launch_fused(bool mapped);
    std::vector<void *> pinned_inputs_, pinned_outputs_;
    bool staging_ready_ = false;
    void allocate_staging();
    std::unique_ptr<HostCopyPool> copy_pool_;   // threads for the host side of big copies, started on first need
    std::vector<hipEvent_t> chunk_events_;      // one per output chunk of the largest evaluation so far
    void host_copy(void *dst, const void *src, size_t bytes);
    bool profile_ = false;
    std::optional<Profile> last_profile_;
    bool graph_mode_ = false;
    hipGraphExec_t graph_exec_ = nullptr;
};

void hip_check(hipError_t e, const char *what);

}  // namespace kn
