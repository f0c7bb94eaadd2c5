// A whole small graph as one kernel launch (see fused_graph.cpp).
#pragma once

#include <optional>
#include <vector>

#include "kernels.h"
#include "mfma_kernels.h"

namespace kn {

constexpr size_t FUSED_MAX_STEPS = 16;
constexpr uint32_t FUSED_MAX_WORKGROUPS = 4;             // workgroups of a generated step that the one workgroup walks through
constexpr long long FUSED_MAX_MATMUL_OUTPUTS = 2048;     // output elements of a matmul step
constexpr long long FUSED_MAX_MATMUL_MACS = 256 * 1024;  // multiply-adds of a matmul step

// One step of the plan: a generated kernel, or a matmul given by its launch parameters (pointers unused).
struct FusedPart {
    const KernelSpec *kernel = nullptr;
    GemmParams gemm{};
    bool f16 = false, has_addend = false, has_addend2 = false;
    size_t n_ptrs = 0;  // operands of the step, in the order of its launch
};

// nullopt when a step is too large for one workgroup or of a kind that has no single-workgroup form
std::optional<KernelSpec> make_fused_graph_kernel(const std::vector<FusedPart> &parts);

}  // namespace kn
