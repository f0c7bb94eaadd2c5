// f32 matrix multiply and fused convolution on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One workgroup of 4 waves computes a 128 x 128 tile of D = A * B; every wave owns a 64 x 64 quadrant as 2 x 2
// MFMA tiles of 32 x 32 (64 accumulator registers per lane). The K dimension is walked in slices of 16 that are
// staged through LDS as As[k][m] and Bs[k][n]; the next slice is fetched into registers while the current one is
// multiplied. Operand elements are addressed through small functors, so the same main loop serves strided
// batched GEMM (any row/column/batch strides) and convolution as an implicit GEMM (the B operand gathers input
// patches on the fly, with zero padding) with bias + residual + relu applied to the accumulators before the store.
#include <hip/hip_runtime.h>

#include "../mfma_kernels.h"

namespace kn {

namespace {

constexpr int BM = 128, BN = 128, BK = 16, THREADS = 256;
constexpr int LDS_STRIDE = BM + 4;  // keeps rows 16 byte aligned and shifts successive k rows by 4 banks

typedef float floatx16 __attribute__((ext_vector_type(16)));

// ---- operand accessors for plain strided GEMM
struct GemmA {
    const float *p;
    long long sm, sk;
    int M, K;
    __device__ __forceinline__ float load(int m, int k) const { return (m < M && k < K) ? p[m * sm + k * sk] : 0.0f; }
    __device__ __forceinline__ bool lanes_along_k() const { return (sk < 0 ? -sk : sk) < (sm < 0 ? -sm : sm); }
};
struct GemmB {
    const float *p;
    long long sk, sn;
    int K, N;
    __device__ __forceinline__ float load(int k, int n) const { return (k < K && n < N) ? p[k * sk + n * sn] : 0.0f; }
    __device__ __forceinline__ bool lanes_along_k() const { return (sk < 0 ? -sk : sk) < (sn < 0 ? -sn : sn); }
};
struct GemmStore {
    float *p;
    long long sm, sn;
    int M, N;
    __device__ __forceinline__ void store(int m, int n, float v) const {
        if (m < M && n < N) p[m * sm + n * sn] = v;
    }
};

// ---- operand accessors for convolution: D[ko][pos] = sum_k filter[ko][k] * patch[k][pos]
struct ConvA {  // the filter, dense [out_c, in_c * kh * kw]
    const float *p;
    int M, K;
    __device__ __forceinline__ float load(int m, int k) const { return (m < M && k < K) ? p[(long long) m * K + k] : 0.0f; }
    __device__ __forceinline__ bool lanes_along_k() const { return true; }
};
struct ConvB {  // input patches, gathered from the dense NCHW input; n runs over (image, oy, ox)
    const float *p;
    int K, N;  // K = in_c * kh * kw, N = batch * out_h * out_w
    int in_c, in_h, in_w, out_h, out_w, kh, kw, sy, sx, py, px;
    __device__ __forceinline__ float load(int k, int n) const {
        if (k >= K || n >= N) return 0.0f;
        int khw = kh * kw, ohw = out_h * out_w;
        int c = k / khw, r = k - c * khw;
        int fy = r / kw, fx = r - fy * kw;
        int img = n / ohw, pos = n - img * ohw;
        int oy = pos / out_w, ox = pos - oy * out_w;
        int iy = oy * sy + fy - py, ix = ox * sx + fx - px;
        if (iy < 0 || iy >= in_h || ix < 0 || ix >= in_w) return 0.0f;
        return p[(((long long) img * in_c + c) * in_h + iy) * in_w + ix];
    }
    __device__ __forceinline__ bool lanes_along_k() const { return false; }
};
struct ConvStore {
    float *p;
    const float *bias;
    const float *res;
    long long bias_stride;
    int M, N, ohw;  // out_c, batch * out_h * out_w, out_h * out_w
    int relu;
    __device__ __forceinline__ void store(int m, int n, float v) const {
        if (m < M && n < N) {
            int img = n / ohw, pos = n - img * ohw;
            long long o = ((long long) img * M + m) * ohw + pos;
            if (res) v += res[o];
            if (bias) v += bias[m * bias_stride];
            if (relu) v = fmaxf(v, 0.0f);
            p[o] = v;
        }
    }
};

template <typename A, typename B, typename S>
__device__ __forceinline__ void mfma_tile_loop(const A &a, const B &b, const S &s, int K) {
    __shared__ float As[BK][LDS_STRIDE];
    __shared__ float Bs[BK][LDS_STRIDE];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    // each thread moves 8 elements of each operand per slice; lanes run along the axis that is contiguous in memory
    const bool a_k = a.lanes_along_k(), b_k = b.lanes_along_k();
    float ra[8], rb[8];

    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int e = t + THREADS * i;
            int am = a_k ? (e >> 4) : (e & (BM - 1));
            int ak = a_k ? (e & (BK - 1)) : (e >> 7);
            ra[i] = a.load(m0 + am, k0 + ak);
            int bn = b_k ? (e >> 4) : (e & (BN - 1));
            int bk = b_k ? (e & (BK - 1)) : (e >> 7);
            rb[i] = b.load(k0 + bk, n0 + bn);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            int e = t + THREADS * i;
            int am = a_k ? (e >> 4) : (e & (BM - 1));
            int ak = a_k ? (e & (BK - 1)) : (e >> 7);
            As[ak][am] = ra[i];
            int bn = b_k ? (e >> 4) : (e & (BN - 1));
            int bk = b_k ? (e & (BK - 1)) : (e >> 7);
            Bs[bk][bn] = rb[i];
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();  // the previous slice has been consumed
        stage();
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const int kr = kk + (lane >> 5), c = lane & 31;
            const float a0 = As[kr][wm * 64 + c], a1 = As[kr][wm * 64 + 32 + c];
            const float b0 = Bs[kr][wn * 64 + c], b1 = Bs[kr][wn * 64 + 32 + c];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
    }

    // accumulator layout of the 32x32 tile: register v of lane l holds row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                int col = n0 + wn * 64 + j * 32 + (lane & 31);
                s.store(row, col, acc[i][j][v]);
            }
}

__global__ __launch_bounds__(THREADS) void gemm_f32_kernel(GemmParams p) {
    const int bz = blockIdx.z;
    GemmA a{p.a + bz * p.a_sb, p.a_sm, p.a_sk, p.m, p.k};
    GemmB b{p.b + bz * p.b_sb, p.b_sk, p.b_sn, p.k, p.n};
    GemmStore s{p.c + bz * p.c_sb, p.c_sm, p.c_sn, p.m, p.n};
    mfma_tile_loop(a, b, s, p.k);
}

__global__ __launch_bounds__(THREADS) void conv_f32_kernel(ConvParams p) {
    const int K = p.in_c * p.kernel_h * p.kernel_w, ohw = p.out_h * p.out_w, N = p.batch * ohw;
    ConvA a{p.filter, p.out_c, K};
    ConvB b{p.input, K, N, p.in_c, p.in_h, p.in_w, p.out_h, p.out_w,
            p.kernel_h, p.kernel_w, p.stride_y, p.stride_x, p.pad_y, p.pad_x};
    ConvStore s{p.output, p.bias, p.res, p.bias_stride, p.out_c, N, ohw, p.relu};
    mfma_tile_loop(a, b, s, K);
}

}  // namespace

int launch_gemm_f32(const GemmParams &params, ihipStream_t *stream) {
    GemmParams p = params;
    if (p.batch <= 0 || p.m <= 0 || p.n <= 0) return 0;
    // put the axis of C that is contiguous in memory on the MFMA column (lane) axis: D^T = B^T * A^T
    auto mag = [](long long x) { return x < 0 ? -x : x; };
    if (mag(p.c_sm) < mag(p.c_sn)) {
        GemmParams q = p;
        q.a = p.b; q.b = p.a;
        q.m = p.n; q.n = p.m;
        q.a_sb = p.b_sb; q.a_sm = p.b_sn; q.a_sk = p.b_sk;
        q.b_sb = p.a_sb; q.b_sk = p.a_sk; q.b_sn = p.a_sm;
        q.c_sm = p.c_sn; q.c_sn = p.c_sm;
        p = q;
    }
    dim3 grid((p.n + BN - 1) / BN, (p.m + BM - 1) / BM, p.batch);
    if (grid.y > 65535 || grid.z > 65535) return (int) hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(THREADS), 0, stream, p);
    return (int) hipGetLastError();
}

int launch_conv_f32(const ConvParams &p, ihipStream_t *stream) {
    long long positions = (long long) p.batch * p.out_h * p.out_w;
    if (positions <= 0 || p.out_c <= 0) return 0;
    if (positions > 0x7fffffffll) return (int) hipErrorInvalidValue;
    dim3 grid((unsigned) ((positions + BN - 1) / BN), (p.out_c + BM - 1) / BM, 1);
    if (grid.y > 65535) return (int) hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(conv_f32_kernel, grid, dim3(THREADS), 0, stream, p);
    return (int) hipGetLastError();
}

}  // namespace kn
