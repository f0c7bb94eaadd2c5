// What the matrix cores of the device deliver when nothing else limits them: a register-only loop of independent
// v_mfma_f32_32x32x16_f16 or v_mfma_f32_32x32x2_f32 (the inner loop of a 128 x 128 wave tile without any memory traffic), one wave per SIMD, and
// the shader clock it runs at, read as clock64() against the constant-rate wall_clock64(). With normally distributed
// operands the matrix cores draw more power than with small integers and the clock drops; the rate measured here
// on such data is the ceiling that matmul and convolution kernels should be read against.
#include <hip/hip_runtime.h>

#include <cmath>
#include <vector>

#include "../executor.h"
#include "../matmul_api.h"

namespace {

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_probe_kernel(const _Float16 *src, float *out, long long *clocks, int iters) {
    halfx8 a[4], b[4];
    for (int i = 0; i < 4; i++) {
        a[i] = *(const halfx8 *) (src + ((threadIdx.x + 256 * i) % 1024) * 8);
        b[i] = *(const halfx8 *) (src + 8192 + ((threadIdx.x + 256 * i) % 1024) * 8);
    }
    floatx16 acc[4][4];
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++)
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++)
            for (int v = 0; v < 16; v++) s += acc[i][j][v];
    if (s == 12345.678f) out[0] = s;  // (keeps the loop alive)
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = w1 - w0;
    }
}

__global__ __launch_bounds__(256) void mfma_probe_f32_kernel(const float *src, float *out, long long *clocks, int iters) {
    float a[4], b[4];
    for (int i = 0; i < 4; i++) {
        a[i] = src[(threadIdx.x + 256 * i) % 16384];
        b[i] = src[(threadIdx.x + 256 * i + 8192) % 16384];
    }
    floatx16 acc[4][4];
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++)
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0;
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++)
            for (int v = 0; v < 16; v++) s += acc[i][j][v];
    if (s == 12345.678f) out[0] = s;  // (keeps the loop alive)
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = c1 - c0;
        clocks[1] = w1 - w0;
    }
}

}  // namespace

extern "C" int knhip_device_mfma_probe(int device, int mode, int iterations, double *tflops, double *shader_mhz) {
    void *src = nullptr;
    float *out = nullptr;
    long long *clocks = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int status = KNHIP_OK;
    try {
        if (tflops == nullptr || shader_mhz == nullptr || iterations <= 0 || iterations > 1000000 || mode < 0 || mode > 7) kn::fail("invalid argument");
        const bool normal_data = mode & 1, f32 = mode & 2, rectified = mode & 4;
        kn::HipDevice::check(device);
        kn::hip_check(hipSetDevice(device), "hipSetDevice");
        int cus = 0, wall_khz = 0;
        kn::hip_check(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device), "hipDeviceGetAttribute");
        kn::hip_check(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, device), "hipDeviceGetAttribute");
        // 16384 values: small integers, or N(0, 1) from a fixed linear congruential stream; rectified: the second
        // half, which feeds the B operands, is max(x, 0) like the output of a relu
        std::vector<float> values(16384);
        unsigned long long state = 0x9e3779b97f4a7c15ull;
        auto uniform = [&]() {
            state = state * 6364136223846793005ull + 1442695040888963407ull;
            return ((double) (state >> 11) + 1.0) / 9007199254740994.0;
        };
        for (size_t i = 0; i < values.size(); i++) {
            float x;
            if (normal_data) x = (float) (std::sqrt(-2.0 * std::log(uniform())) * std::cos(6.283185307179586 * uniform()));
            else x = (float) ((int) (uniform() * 5.0) - 2);
            if (rectified && i >= values.size() / 2) x = x > 0.0f ? x : 0.0f;
            values[i] = x;
        }
        std::vector<_Float16> halves(values.begin(), values.end());
        const size_t bytes = f32 ? values.size() * 4 : halves.size() * 2;
        kn::hip_check(hipMalloc(&src, bytes), "hipMalloc");
        kn::hip_check(hipMalloc((void **) &out, 64), "hipMalloc");
        kn::hip_check(hipMalloc((void **) &clocks, 64), "hipMalloc");
        kn::hip_check(hipMemcpy(src, f32 ? (const void *) values.data() : (const void *) halves.data(), bytes, hipMemcpyHostToDevice), "hipMemcpy");
        kn::hip_check(hipEventCreate(&e0), "hipEventCreate");
        kn::hip_check(hipEventCreate(&e1), "hipEventCreate");
        auto launch = [&]() {
            if (f32) hipLaunchKernelGGL(mfma_probe_f32_kernel, dim3(cus), dim3(256), 0, 0, (const float *) src, out, clocks, iterations);
            else hipLaunchKernelGGL(mfma_probe_kernel, dim3(cus), dim3(256), 0, 0, (const _Float16 *) src, out, clocks, iterations);
        };
        // one untimed launch, then the timed one
        launch();
        kn::hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");
        kn::hip_check(hipEventRecord(e0, 0), "hipEventRecord");
        launch();
        kn::hip_check(hipEventRecord(e1, 0), "hipEventRecord");
        kn::hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
        float ms = 0;
        kn::hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        long long h[2] = {0, 0};
        kn::hip_check(hipMemcpy(h, clocks, 16, hipMemcpyDeviceToHost), "hipMemcpy");
        const double flops_per_mfma = f32 ? 2.0 * 32 * 32 * 2 : 2.0 * 32 * 32 * 16;
        *tflops = (double) cus * 4 * 16 * flops_per_mfma * iterations / (ms * 1e-3) / 1e12;
        *shader_mhz = h[1] > 0 ? (double) h[0] / (double) h[1] * wall_khz / 1e3 : 0.0;
    } catch (const std::exception &e) {
        kn::set_last_error(e.what());
        status = KNHIP_ERROR;
    }
    if (e0) (void) hipEventDestroy(e0);
    if (e1) (void) hipEventDestroy(e1);
    if (src) (void) hipFree(src);
    if (out) (void) hipFree(out);
    if (clocks) (void) hipFree(clocks);
    return status;
}
