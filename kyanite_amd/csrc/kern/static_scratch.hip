// knhip_batched_mat_mul_static: the stand-alone batched matrix product for callers that cannot allocate (code under
// HIP graph capture, serving loops, harnesses that forbid hipMalloc). It is knhip_batched_mat_mul with the workspace
// argument replaced by a static device array: the f32 partial products of a split K axis and the tile counters live
// in `scratch` below, KNHIP_STATIC_SCRATCH_BYTES per GPU, held from the first use of the library on that GPU until
// the process ends. The call itself allocates nothing: no hipMalloc, no hipFree, no allocating library routine.
//
// Every call on one GPU shares that GPU's array, and the array keeps what the last call left in it: the counters
// are cleared by a kernel at the start of every call, the partial products are written before they are read.
// Two calls whose work overlaps on one GPU (different streams, or threads) race on the array; callers order them.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../executor.h"
#include "../matmul_api.h"

namespace {

static __device__ __align__(256) unsigned char scratch[KNHIP_STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
// In host code `scratch` is only a stand-in for the symbol, not a device address; every GPU holds its own copy of
// the array at its own address, looked up once per device with that device current.
void *g_scratch_ptr[MAX_DEVICES] = {};
std::once_flag g_scratch_once[MAX_DEVICES];

void *scratch_of_current_device(int device) {
    if (device < 0 || device >= MAX_DEVICES) kn::fail("batched_mat_mul_static: device index ", device, " out of range");
    std::call_once(g_scratch_once[device], [&] {
        void *ptr = nullptr;
        kn::hip_check(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
        if (ptr == nullptr || (uintptr_t) ptr % 256 != 0) kn::fail("batched_mat_mul_static: bad address for the static scratch");
        g_scratch_ptr[device] = ptr;
    });
    return g_scratch_ptr[device];
}

}  // namespace

// The address lookup is no stream operation and may be refused while a stream capture is open: a caller that will
// capture resolves it ahead of time with this call (any earlier knhip_batched_mat_mul_static on the device does too).
extern "C" int knhip_static_scratch_prepare(int device) {
    try {
        kn::HipDevice::check(device);
        kn::hip_check(hipSetDevice(device), "hipSetDevice");
        (void) scratch_of_current_device(device);
        return KNHIP_OK;
    } catch (const std::exception &e) {
        kn::set_last_error(e.what());
        return KNHIP_ERROR;
    } catch (...) {
        kn::set_last_error("unknown failure");
        return KNHIP_ERROR;
    }
}

extern "C" int knhip_batched_mat_mul_static(int device, void *stream, const knhip_matmul_args *args) {
    try {
        if (args == nullptr) kn::fail("invalid argument: args is null");
        kn::HipDevice::check(device);
        kn::hip_check(hipSetDevice(device), "hipSetDevice");
        kn::MatmulPlan plan = kn::matmul_api_plan(*args);
        const size_t total = plan.workspace.total();
        if (total > (size_t) KNHIP_STATIC_SCRATCH_BYTES)
            kn::fail("batched_mat_mul_static: this product needs ", total, " bytes of scratch, the static scratch holds ",
                     (size_t) KNHIP_STATIC_SCRATCH_BYTES, "; use knhip_batched_mat_mul with a workspace of the caller's");
        void *ptr = scratch_of_current_device(device);
        kn::matmul_api_launch(plan, total > 0 ? ptr : nullptr, total > 0 ? (size_t) KNHIP_STATIC_SCRATCH_BYTES : 0,
                              (ihipStream_t *) stream);
        return KNHIP_OK;
    } catch (const std::exception &e) {
        kn::set_last_error(e.what());
        return KNHIP_ERROR;
    } catch (...) {
        kn::set_last_error("unknown failure");
        return KNHIP_ERROR;
    }
}
