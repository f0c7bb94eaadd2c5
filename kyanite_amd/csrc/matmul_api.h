// The stand-alone batched matrix product of the C ABI (knhip_batched_mat_mul and its variant on static scratch):
// argument checks, launch plan and launch, shared by both entry points.
#pragma once

#include <cstddef>
#include <string>
#include <vector>

#include "../../include/knhip.h"
#include "mfma_kernels.h"

namespace kn {

// counters first (rounded up to 256 bytes), then the partial products
struct MatmulWorkspace {
    size_t counter_bytes = 0, partial_bytes = 0;
    size_t partial_offset() const { return (counter_bytes + 255) / 256 * 256; }
    size_t total() const { return partial_bytes > 0 ? partial_offset() + partial_bytes : counter_bytes; }
};

// One call of the C ABI as launches: a batch of more than 65535 entries (the batch index rides on grid.y) runs as
// several launches, one after the other on the stream, that share one workspace with room for the largest.
struct MatmulPlan {
    bool f16 = false, empty = false;
    std::vector<GemmLaunchPlan> slabs;             // oriented launch plans, without workspace addresses
    std::vector<MatmulWorkspace> slab_workspaces;  // what each of them needs
    MatmulWorkspace workspace;                     // what the call needs
};

// checks the arguments (throws KnError) and plans the launches
MatmulPlan matmul_api_plan(const knhip_matmul_args &args);
// queues the planned product on `stream`; `workspace` holds at least plan.workspace.total() bytes when that is not
// zero. Allocates nothing.
void matmul_api_launch(MatmulPlan &plan, void *workspace, size_t workspace_bytes, ihipStream_t *stream);
// stores the message that knhip_last_error() returns on the calling thread
void set_last_error(const std::string &message);

}  // namespace kn
