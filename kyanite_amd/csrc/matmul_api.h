// The stand-alone batched matrix product of the C ABI (knhip_batched_mat_mul and its variant on static scratch):
// argument checks, launch plan and launch, shared by both entry points.
#pragma once

#include <cstddef>
#include <string>

#include "../../include/knhip.h"
#include "mfma_kernels.h"

namespace kn {

// counters first (rounded up to 256 bytes), then the partial products
struct MatmulWorkspace {
    size_t counter_bytes = 0, partial_bytes = 0;
    size_t partial_offset() const { return (counter_bytes + 255) / 256 * 256; }
    size_t total() const { return partial_bytes > 0 ? partial_offset() + partial_bytes : counter_bytes; }
};

// checks the arguments (throws KnError) and returns the oriented launch plan without workspace addresses
GemmLaunchPlan matmul_api_plan(const knhip_matmul_args &args, MatmulWorkspace *ws);
// queues the product on `stream`; `workspace` holds at least ws.total() bytes when that is not zero. Allocates nothing.
void matmul_api_launch(const knhip_matmul_args &args, void *workspace, size_t workspace_bytes, ihipStream_t *stream);
// stores the message that knhip_last_error() returns on the calling thread
void set_last_error(const std::string &message);

}  // namespace kn
