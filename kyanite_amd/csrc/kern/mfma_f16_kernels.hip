// f16 matrix multiply with f32 accumulation on the CDNA4 matrix cores (v_mfma_f32_32x32x16_f16).
//
// Same decomposition as the f32 kernel: a workgroup of 4 waves (2 x 2) owns a T x T tile of D = A * B (T = 128 or
// 64), every wave (T / 2) x (T / 2) of it as 32 x 32 MFMA tiles. K is walked in slices of BK that sit in LDS as
// As[m][k] and Bs[n][k], K contiguous with rows padded by 8 halves: a lane's MFMA operand (8 consecutive k of one
// row) is one 128 bit LDS read, and operands whose K axis is contiguous in memory (activations, `linear` weights,
// K^T of attention) move global -> register -> LDS as 128 bit vectors without being transposed.
// The slices are double buffered in LDS: while slice s is multiplied, slice s + 1 waits in registers and slice
// s + 2 is in flight from memory; one barrier per slice. The result is rounded to f16 once, at the store.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "../mfma_kernels.h"

namespace kn {

namespace {

typedef _Float16 half_t;
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));


enum LoadMode { Scalar = 0, VecOuter = 1, VecK = 2 };

struct Operand {
    const half_t *p;
    long long so, sk;  // element strides of the outer (m or n) and the K axis
    int outer_size, K;
};

// Fetches a T x BK slice into registers and writes it to LDS as [outer][k]. Vector modes need every vector to lie
// completely inside or outside the matrix, which the host guarantees (sizes divisible by 8 along the vector axis).
// THREADS: size of the workgroup that shares the slice.
template <int MODE, int T, int BK, int THREADS>
struct Loader {
    static constexpr int NVEC = T * BK / 8 / THREADS;  // 128 bit vectors per thread and slice
    static constexpr int LDS_K = BK + 8;
    static_assert(NVEC >= 1, "slice too small for the workgroup");
    Operand op;
    int o0;
    halfx8 r[NVEC];

    __device__ __forceinline__ Loader(const Operand &operand, int outer0) : op(operand), o0(outer0) {}

    __device__ __forceinline__ void fetch(int k0) {
        const int t = threadIdx.x;
#pragma unroll
        for (int h = 0; h < NVEC; h++) {
            if (MODE == VecK) {
                // BK / 8 vectors cover the k of one row
                const int o = t / (BK / 8) + (THREADS * 8 / BK) * h, k = (t % (BK / 8)) * 8;
                const bool ok = (o0 + o) < op.outer_size && (k0 + k) < op.K;
                if (ok) r[h] = *(const halfx8 *) (op.p + (long long) (o0 + o) * op.so + (k0 + k));
                else r[h] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
            } else if (MODE == VecOuter) {
                // T / 8 vectors cover the T outer indices of one k
                const int k = t / (T / 8) + (THREADS * 8 / T) * h, o = (t % (T / 8)) * 8;
                const bool ok = (o0 + o) < op.outer_size && (k0 + k) < op.K;
                if (ok) r[h] = *(const halfx8 *) (op.p + (long long) (k0 + k) * op.sk + (o0 + o));
                else r[h] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
            } else {
                // lanes run along k within a row
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int e = (t + THREADS * h) * 8 + j;
                    const int o = e / BK, k = e % BK;
                    const bool ok = (o0 + o) < op.outer_size && (k0 + k) < op.K;
                    r[h][j] = ok ? op.p[(long long) (o0 + o) * op.so + (long long) (k0 + k) * op.sk] : (half_t) 0;
                }
            }
        }
    }

    __device__ __forceinline__ void stage(half_t (*lds)[LDS_K]) const {
        const int t = threadIdx.x;
#pragma unroll
        for (int h = 0; h < NVEC; h++) {
            if (MODE == VecK) {
                const int o = t / (BK / 8) + (THREADS * 8 / BK) * h, k = (t % (BK / 8)) * 8;
                *(halfx8 *) &lds[o][k] = r[h];
            } else if (MODE == VecOuter) {
                const int k = t / (T / 8) + (THREADS * 8 / T) * h, o = (t % (T / 8)) * 8;
#pragma unroll
                for (int j = 0; j < 8; j++) lds[o + j][k] = r[h][j];
            } else {
                const int e = (t + THREADS * h) * 8;
                *(halfx8 *) &lds[e / BK][e % BK] = r[h];
            }
        }
    }
};

// Tiles are numbered in bands of 8 tile rows, column by column within a band, so 8 k consecutive numbers are a patch
// of 8 x k tiles. Workgroups are handed to the 8 XCDs (each with its own L2) in turn, workgroup i to XCD i % 8;
// the renumbering below gives every XCD runs of `xcd_chunk` consecutive tile numbers (as many as it runs at a time),
// so that the workgroups sharing an L2 cover one compact patch and find each other's operand tiles there.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int xcd_chunk, int *tm, int *tn) {
    int id = blockIdx.x;
    if (xcd_chunk > 0) {
        const int per_round = 8 * xcd_chunk;
        const int full = (int) (gridDim.x / per_round) * per_round;  // the tail keeps its numbers
        if (id < full) {
            const int xcd = id & 7, local = id >> 3;
            id = ((local / xcd_chunk) * 8 + xcd) * xcd_chunk + local % xcd_chunk;
        }
    }
    const int group_rows = 8;
    const int per_group = group_rows * tiles_n;
    const int g = id / per_group, in_g = id - g * per_group;
    const int rows_here = min(group_rows, tiles_m - g * group_rows);
    *tm = g * group_rows + in_g % rows_here;
    *tn = in_g / rows_here;
}

// TI: MFMA tiles per wave and axis; WM: waves along M (2 along N), so the workgroup tile is (32 TI WM) x (64 TI):
// 128 x 128 (TI 2, WM 2), 64 x 64 (TI 1, WM 2) or 256 x 128 with 8 waves (TI 2, WM 4), which fetches a quarter less
// from L2 per flop. BK: depth of a K slice; NBUF: LDS buffers per operand (2 = double buffered, one barrier per
// slice; 1 = two barriers per slice)
template <int A_MODE, int B_MODE, int TI, int BK, int NBUF, int WM>
__global__ __launch_bounds__(128 * WM) void gemm_f16_kernel(GemmParams p, int k_chunk, int xcd_chunk) {
    constexpr int TM = 32 * TI * WM, TN = 64 * TI, LDS_K = BK + 8, THREADS = 128 * WM;
    __shared__ __attribute__((aligned(16))) half_t As[NBUF][TM][LDS_K];
    __shared__ __attribute__((aligned(16))) half_t Bs[NBUF][TN][LDS_K];

    // a grouped launch lines the tiles of its products up along n
    const int tiles_m = (p.m + TM - 1) / TM, tiles_n = (p.n + TN - 1) / TN;
    int tm, tn;
    tile_of_block(tiles_m, tiles_n * p.groups, xcd_chunk, &tm, &tn);
    const int group = tn / tiles_n;
    tn -= group * tiles_n;
    const void *b_base = p.groups > 1 ? p.b_group[group] : p.b;
    void *c_base = p.groups > 1 ? p.c_group[group] : p.c;
    const int bz = blockIdx.y;
    const int m0 = tm * TM, n0 = tn * TN;
    // split K: workgroup z of gridDim.z multiplies its own range of k and stores an f32 partial product
    const int k_begin = blockIdx.z * k_chunk, k_end = min(p.k, k_begin + k_chunk);
    Loader<A_MODE, TM, BK, THREADS> la(Operand{(const half_t *) p.a + bz * p.a_sb, p.a_sm, p.a_sk, p.m, k_end}, m0);
    Loader<B_MODE, TN, BK, THREADS> lb(Operand{(const half_t *) b_base + bz * p.b_sb, p.b_sn, p.b_sk, p.n, k_end}, n0);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1, c = lane & 31, half = lane >> 5;

    floatx16 acc[TI][TI];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int slices = (k_end - k_begin + BK - 1) / BK;
    la.fetch(k_begin);
    lb.fetch(k_begin);
    la.stage(As[0]);
    lb.stage(Bs[0]);
    __syncthreads();
    if (slices > 1) {
        la.fetch(k_begin + BK);
        lb.fetch(k_begin + BK);
    }
    for (int s = 0; s < slices; s++) {
        const int cur = NBUF == 2 ? (s & 1) : 0;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            // lane l supplies 8 consecutive k (starting at 8 * (l / 32)) of row / column l % 32
            halfx8 a[TI], b[TI];
#pragma unroll
            for (int i = 0; i < TI; i++) a[i] = *(const halfx8 *) &As[cur][wm * 32 * TI + 32 * i + c][kk + 8 * half];
#pragma unroll
            for (int j = 0; j < TI; j++) b[j] = *(const halfx8 *) &Bs[cur][wn * 32 * TI + 32 * j + c][kk + 8 * half];
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TI; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (NBUF == 1) __syncthreads();  // the slice has been consumed by every wave
        if (s + 1 < slices) {
            // double buffered: the other buffer was last read in iteration s - 1, which every wave has left through
            // the barrier below
            la.stage(As[NBUF == 2 ? cur ^ 1 : 0]);
            lb.stage(Bs[NBUF == 2 ? cur ^ 1 : 0]);
        }
        __syncthreads();
        if (s + 2 < slices) {
            la.fetch(k_begin + (s + 2) * BK);
            lb.fetch(k_begin + (s + 2) * BK);
        }
    }

    // accumulator layout of the 32x32 tile: register v of lane l holds row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32
    half_t *out = (half_t *) c_base + bz * p.c_sb;
    float *partial = (float *) p.workspace + ((long long) bz * gridDim.z + blockIdx.z) * p.m * p.n;
    const bool split = gridDim.z > 1;
    // the epilogue of a split launch is applied by the pass that sums the partial products
    const half_t *addend = p.addend ? (const half_t *) p.addend + bz * p.d_sb : nullptr;
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TI; j++) {
            const int col = n0 + wn * 32 * TI + 32 * j + c;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 32 * TI + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
                if (row < p.m && col < p.n) {
                    if (split) {
                        partial[(long long) row * p.n + col] = acc[i][j][v];
                    } else {
                        half_t r = (half_t) acc[i][j][v];
                        if (addend) r = (half_t) ((float) r + (float) addend[(long long) row * p.d_sm + (long long) col * p.d_sn]);
                        if (p.relu) r = r > (half_t) 0 ? r : (half_t) 0;
                        out[(long long) row * p.c_sm + (long long) col * p.c_sn] = r;
                    }
                }
            }
        }
}

// `so` / `sk`: element strides of the outer and the K axis; vectors of 8 halves must be aligned and must not
// straddle the edge of the matrix.
int pick_mode(const void *ptr, long long so, long long sk, int outer_size, int k, long long batch_stride, int batch) {
    const bool aligned = ((uintptr_t) ptr % 16 == 0) && (batch <= 1 || batch_stride % 8 == 0);
    if (!aligned) return Scalar;
    if (sk == 1 && so % 8 == 0 && k % 8 == 0) return VecK;
    if (so == 1 && sk % 8 == 0 && outer_size % 8 == 0) return VecOuter;
    return Scalar;
}

template <int A_MODE, int TI, int BK, int NBUF, int WM>
void launch_b(int b_mode, dim3 grid, hipStream_t stream, const GemmParams &p, int kc, int xc) {
    const dim3 block(128 * WM);
    switch (b_mode) {
        case VecOuter: hipLaunchKernelGGL((gemm_f16_kernel<A_MODE, VecOuter, TI, BK, NBUF, WM>), grid, block, 0, stream, p, kc, xc); break;
        case VecK: hipLaunchKernelGGL((gemm_f16_kernel<A_MODE, VecK, TI, BK, NBUF, WM>), grid, block, 0, stream, p, kc, xc); break;
        default: hipLaunchKernelGGL((gemm_f16_kernel<A_MODE, Scalar, TI, BK, NBUF, WM>), grid, block, 0, stream, p, kc, xc); break;
    }
}

template <int TI, int BK, int NBUF, int WM>
void launch_a(int a_mode, int b_mode, dim3 grid, hipStream_t stream, const GemmParams &p, int kc, int xc) {
    switch (a_mode) {
        case VecOuter: launch_b<VecOuter, TI, BK, NBUF, WM>(b_mode, grid, stream, p, kc, xc); break;
        case VecK: launch_b<VecK, TI, BK, NBUF, WM>(b_mode, grid, stream, p, kc, xc); break;
        default: launch_b<Scalar, TI, BK, NBUF, WM>(b_mode, grid, stream, p, kc, xc); break;
    }
}

}  // namespace

int launch_gemm_f16(const GemmParams &params, ihipStream_t *stream) {
    if (params.batch <= 0 || params.m <= 0 || params.n <= 0) return 0;
    const GemmLaunchPlan lp = plan_gemm_launch(params, true);
    const GemmParams &p = lp.p;
    const int t = lp.small_tile ? 64 : 128, t_m = lp.tall_tile ? 256 : t;
    const int groups = p.groups > 1 ? p.groups : 1;
    if (groups > GEMM_MAX_GROUPS || (groups > 1 && (lp.split_k > 1 || p.addend || p.a != params.a))) return (int) hipErrorInvalidValue;
    const long long tiles = (long long) ((p.m + t_m - 1) / t_m) * ((p.n + t - 1) / t) * groups;
    if (tiles > 0x7fffffffll || p.batch > 65535 || (long long) p.m * p.n > 0x7fffffffll * 256) return (int) hipErrorInvalidConfiguration;
    if (lp.split_k > 1 && p.workspace == nullptr) return (int) hipErrorInvalidValue;
    dim3 grid((unsigned) tiles, (unsigned) p.batch, (unsigned) lp.split_k);
    const int a_mode = pick_mode(p.a, p.a_sm, p.a_sk, p.m, p.k, p.a_sb, p.batch);
    int b_mode = pick_mode(groups > 1 ? p.b_group[0] : p.b, p.b_sn, p.b_sk, p.n, p.k, p.b_sb, p.batch);
    for (int g = 1; g < groups; g++) {  // the loader that every operand of the group allows
        const int mode = pick_mode(p.b_group[g], p.b_sn, p.b_sk, p.n, p.k, p.b_sb, p.batch);
        if (mode != b_mode) b_mode = Scalar;
    }
    // Measured on 128 x 128 tiles (TFLOP/s at 4096^3 / 8192^3): BK 64 single buffered 594 / 757, BK 64 double
    // buffered 643 / 718, BK 128 single buffered 672 / 744. All of them sit at the rate at which the L2 can feed
    // the compute units at this tile size (64 flop per byte fetched from L2, about 12 TB/s -> 770 TFLOP/s).
    // workgroups an XCD (32 compute units) runs at a time: 1 per compute unit for the tall tiles, else 2
    static const int xc_env = getenv("KNHIP_XCD_CHUNK") ? atoi(getenv("KNHIP_XCD_CHUNK")) : -1;
    const int xc = xc_env >= 0 ? xc_env : (lp.tall_tile ? 32 : 64);
    if (lp.small_tile) launch_a<1, 64, 2, 2>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    else if (lp.tall_tile) launch_a<2, 64, 1, 4>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    else launch_a<2, 128, 1, 2>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    int e = (int) hipGetLastError();
    if (e == 0 && lp.split_k > 1) e = launch_gemm_reduce_partials(p, lp.split_k, true, stream);
    return e;
}

}  // namespace kn
