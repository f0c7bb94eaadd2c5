// Planner: turns a Graph plus a concrete batch size into a launch list over one device arena.
// Keeps the planning semantics of kn-cuda-eval/src/planner.rs (layout propagation :345-364, fused convolution
// matcher :669-833, scalar chain fusion :835-954, softmax / layernorm operand folding :418-476, :522-604, matmul
// :606-648, live ranges :134-164), but plans into byte offsets of a single arena instead of separate allocations,
// and fuses elementwise work that follows a layernorm or softmax into that kernel's single pass over the row.
#pragma once

#include <memory>

#include "kernels.h"
#include "mfma_kernels.h"
#include "rtc.h"

namespace kn {

enum class StepKind : uint8_t { Conv = 0, MatMul = 1, ScalarOp = 2, ReduceOp = 3, SoftmaxOp = 4, LayernormOp = 5, GatherOp = 6 };
constexpr int STEP_KIND_COUNT = 7;
const char *step_kind_name(StepKind k);

enum class OperandKind : uint8_t { In, Out, InOut, Scratch };  // step.rs:82-94

struct StepOperand {
    PlanTensor tensor;
    OperandKind kind;
};

struct Step {
    StepKind kind = StepKind::ScalarOp;
    Value debug_value = 0;
    std::string debug_id;
    // every tensor the step touches, in kernel argument order
    std::vector<StepOperand> operands;
    // run-time compiled kernels
    KernelSpec kernel;
    std::shared_ptr<const CodeObject> code;
    // ScalarOp steps: the expression of every output (operands: the outputs first, then what is loaded), kept so that
    // neighbouring elementwise steps of one shape can still be joined into one launch
    std::vector<ScalarExpr> scalar_exprs;
    // matrix-core kernels; the pointers are filled in when the plan is realised
    GemmParams gemm{};
    bool gemm_f16 = false;  // element type of a MatMul step: f16 (f32 accumulation) instead of f32
    bool gemm_has_addend = false;  // operand 3 is the tensor added in the epilogue
    bool gemm_has_addend2 = false;  // operand 4 is a second one, added after the first
    // a MatMul step that is a whole softmax(scale * Q K^T [+ mask]) V chain in one launch; operands Q, K, V, [mask,] O
    bool attention = false;
    bool attention_has_mask = false;  // operand 3 is the additive mask, the result comes last
    bool attention_has_classes = false;  // operand 4 is the per-block classification of a constant mask
    AttentionParams attn{};
    ConvParams conv{};
    bool conv_has_bias = false, conv_has_res = false;

    std::string str() const;
    // Algorithmic work of one launch: multiply-add flops of a MatMul / Conv step (0 otherwise) and the bytes of
    // every distinct operand element (a broadcast axis counts once), which is what a perfect kernel would move.
    double flops() const;
    double bytes() const;
};

struct MemoryUsage {  // planner.rs:67-81
    size_t dedicated_bytes = 0;  // constants
    size_t shared_bytes = 0;     // inputs, outputs, hidden values
    size_t zero_bytes = 0;
    size_t hypo_shared_bytes_peak = 0;   // lower bound: what is live at the same time
    size_t hypo_shared_bytes_total = 0;  // without any reuse
};

struct ConstantUpload {
    size_t arena_offset;
    HostTensor tensor;
};

struct Plan {
    std::vector<PlanTensor> inputs, outputs;
    std::vector<Step> steps;
    MemoryUsage mem_usage;
    // arena layout: [constants | zeros | shared], every buffer aligned to ARENA_ALIGN
    size_t arena_bytes = 0;
    std::vector<size_t> constant_offsets;  // per constant slot
    size_t zero_offset = 0;
    std::vector<size_t> shared_offsets;  // per shared buffer; SIZE_MAX for buffers that are never used
    std::vector<size_t> shared_sizes;
    std::vector<ConstantUpload> uploads;

    // resolve a planned pointer to a byte offset inside the arena
    size_t resolve(const PlanPtr &ptr) const;
};

constexpr size_t ARENA_ALIGN = 256;

struct PlannerOptions {
    bool compile = true;          // compile the generated kernels (can be switched off to inspect the plan only)
    bool fuse_row_epilogue = true;  // fold elementwise consumers of a layernorm / softmax into the row kernel
    bool fuse_matmul_epilogue = true;  // fold `+ d` and `max(., 0)` after a matmul into the matmul's store
    bool fuse_attention = true;  // matmul, softmax, matmul chains in f32 run as one launch
    bool pack_matmul_constants = true;  // constant [k, n] right operands of matmuls are laid out again as [n, k]
    // (x w_g) * sigmoid(x w_g) * (x w_u) in f16 with constant weights: one launch whose store computes the gated product
    bool fuse_gated_matmul = true;
    bool group_matmuls = true;   // matmuls that share their left operand and have constant right operands share a launch
    bool pointwise_conv_as_matmul = true;  // 1 x 1 convolutions with stride 1 run as one matrix product per image
    bool join_elementwise = true;  // small elementwise steps of one shape that do not depend on each other share a launch
    bool split_reduce = true;  // a reduction with few results and a long reduced index runs as two launches
    // keep input buffers out of the reuse pool, so that inputs written once stay valid over many run_async calls
    bool preserve_inputs = false;
    GemmTuning gemm;                   // launch paths of the matmul kernels
    // A plan with this many bytes of constants or more reads the constant right operands of its matmuls as streams
    // (GemmTuning::stream_b): they cannot stay in the last-level cache (256 MB) from one evaluation to the next.
    // 0: never.
    size_t stream_weights_bytes = (size_t) 256 << 20;
    bool split_conv_channels = true;   // convolutions with few tiles fold slices of their input channels side by side
    bool plane_conv_any_width = true;  // 3 x 3 convolutions on images without a power-of-two width on the plane kernel
    GeneratorOptions generator;        // what the generated kernels may use (streaming accesses, transposing tiles)
};

Plan plan_graph(const Graph &graph, size_t batch_size, const PlannerOptions &options);

}  // namespace kn
