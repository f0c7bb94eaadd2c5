// f16 matrix multiply with f32 accumulation on the CDNA4 matrix cores (v_mfma_f32_32x32x16_f16).
//
// Same decomposition as the f32 kernel: a workgroup of 4 waves (2 x 2) owns a T x T tile of D = A * B (T = 128 or
// 64), every wave (T / 2) x (T / 2) of it as 32 x 32 MFMA tiles. K is walked in slices of BK that sit in LDS as
// As[m][k] and Bs[n][k], K contiguous with rows padded by 8 halves: a lane's MFMA operand (8 consecutive k of one
// row) is one 128 bit LDS read, and operands whose K axis is contiguous in memory (activations, `linear` weights,
// K^T of attention) move global -> register -> LDS as 128 bit vectors without being transposed.
// The slices are double buffered in LDS: while slice s is multiplied, slice s + 1 waits in registers and slice
// s + 2 is in flight from memory; one barrier per slice. The result is rounded to f16 once, at the store.
//
// When both operands have K contiguous, 16 byte aligned rows and K is a multiple of 64, a second kernel moves the
// slices global -> LDS directly (global_load_lds_dwordx4: every lane names its own 16 source bytes, the wave's 64
// vectors land side by side in LDS), with no trip through registers and no LDS write instructions. Rows are then
// exactly 128 bytes with no padding, and bank conflicts are avoided by an XOR swizzle instead: the 16 byte chunk q
// of row r sits at position q ^ swz(r), swz(r) = (r / 2) % 8, which the loading lane arranges by choosing its source
// chunk and the reading lane by flipping address bits. A 128 bit read is served 16 lanes at a time from 64 banks
// (256 bytes, two rows): the 16 rows r .. r + 15 of such a group then hit 16 different (row parity, position)
// pairs. (With swz(r) = r % 8, which would do for 32 banks, the counters showed every second LDS cycle as a
// conflict.)
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "../mfma_kernels.h"

namespace kn {

namespace {

typedef _Float16 half_t;
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
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
// so that the workgroups sharing an L2 cover one compact patch and find each other's operand tiles there. With 4
// tile rows (m = 512) and 96 tile columns, a B tile whose 4 users sit on 4 XCDs is fetched from memory 4 times:
// 103 us against 61 us for 512 x 12288 x 4096.
__device__ __forceinline__ void tile_of_block(int id, int total, int tiles_m, int tiles_n, int xcd_chunk, int *tm, int *tn) {
    if (xcd_chunk > 0) {
        const int per_round = 8 * xcd_chunk;
        const int full = total / per_round * per_round;
        const int xcd = id & 7;
        if (id < full) {
            const int local = id >> 3;
            id = ((local / xcd_chunk) * 8 + xcd) * xcd_chunk + local % xcd_chunk;
        } else {
            // the last, partial round: one run per XCD again, as long as that XCD's share of the rest
            const int rest = total - full, share = rest >> 3, extra = rest & 7;
            id = full + xcd * share + min(xcd, extra) + ((id - full) >> 3);
        }
    }
    const int group_rows = 8;
    const int per_group = group_rows * tiles_n;
    const int g = id / per_group, in_g = id - g * per_group;
    const int rows_here = min(group_rows, tiles_m - g * group_rows);
    *tm = g * group_rows + in_g % rows_here;
    *tn = in_g / rows_here;
}

// Stores the MI x NI MFMA tiles of a wave whose first row / column are row0 / col0. Accumulator layout of a 32 x 32
// tile: register v of lane l holds row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32.
template <typename T, int MI, int NI>
__device__ __forceinline__ void store_tiles(const GemmParams &p, const floatx16 (&acc)[MI][NI], void *c_base, int bz, int row0, int col0) {
    const int lane = threadIdx.x & 63, c = lane & 31, half = lane >> 5;
    T *out = (T *) c_base + bz * p.c_sb;
    float *partial = (float *) p.workspace + ((long long) bz * gridDim.z + blockIdx.z) * p.m * p.n;
    const bool split = gridDim.z > 1;
    // the epilogue of a split launch is applied by the pass that sums the partial products
    const T *addend = p.addend ? (const T *) p.addend + bz * p.d_sb : nullptr;
    const T *addend2 = p.addend2 ? (const T *) p.addend2 + bz * p.d2_sb : nullptr;
    // Tiles that lie inside the matrix, with offsets that fit 32 bits, skip the bounds checks and the 64 bit
    // address arithmetic (which otherwise cost about a tenth of a 512 x 12288 x 4096 launch).
    const long long reach = (long long) (p.m - 1) * p.c_sm + p.n, d_reach = (long long) (p.m - 1) * p.d_sm + (long long) (p.n - 1) * p.d_sn;
    const long long d2_reach = (long long) (p.m - 1) * p.d2_sm + (long long) (p.n - 1) * p.d2_sn;
    const bool fast = !split && p.c_sn == 1 && p.c_sm > 0 && reach < 0x7fffffffll && row0 + 32 * MI <= p.m && col0 + 32 * NI <= p.n &&
                      (!addend || (p.d_sm >= 0 && p.d_sn >= 0 && d_reach < 0x7fffffffll)) &&
                      (!addend2 || (p.d2_sm >= 0 && p.d2_sn >= 0 && d2_reach < 0x7fffffffll));
    if (fast) {
        const int c_sm = (int) p.c_sm, d_sm = (int) p.d_sm, d_sn = (int) p.d_sn, d2_sm = (int) p.d2_sm, d2_sn = (int) p.d2_sn;
        T *tile = out + (row0 + 4 * half) * c_sm + col0 + c;
        const T *d_tile = addend ? addend + (row0 + 4 * half) * d_sm + (col0 + c) * d_sn : nullptr;
        const T *d2_tile = addend2 ? addend2 + (row0 + 4 * half) * d2_sm + (col0 + c) * d2_sn : nullptr;
        const bool relu = p.relu != 0;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++) {
                // every addend of the MFMA tile is requested before its first store: the compiler cannot move a
                // load over a store that might alias it, and one round trip per element is the tail of the workgroup
                T d[16], d2[16];
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = 32 * i + 8 * (v >> 2) + (v & 3);
                    d[v] = d_tile ? d_tile[r * d_sm + 32 * j * d_sn] : (T) 0;
                    d2[v] = d2_tile ? d2_tile[r * d2_sm + 32 * j * d2_sn] : (T) 0;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = 32 * i + 8 * (v >> 2) + (v & 3);
                    T x = (T) acc[i][j][v];
                    if (d_tile) x = (T) ((float) x + (float) d[v]);
                    if (d2_tile) x = (T) ((float) x + (float) d2[v]);
                    if (relu) x = x > (T) 0 ? x : (T) 0;
                    tile[r * c_sm + 32 * j] = x;
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const int col = col0 + 32 * j + c;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = row0 + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
                if (row < p.m && col < p.n) {
                    if (split) {
                        partial[(long long) row * p.n + col] = acc[i][j][v];
                    } else {
                        T r = (T) acc[i][j][v];
                        if (addend) r = (T) ((float) r + (float) addend[(long long) row * p.d_sm + (long long) col * p.d_sn]);
                        if (addend2) r = (T) ((float) r + (float) addend2[(long long) row * p.d2_sm + (long long) col * p.d2_sn]);
                        if (p.relu) r = r > (T) 0 ? r : (T) 0;
                        out[(long long) row * p.c_sm + (long long) col * p.c_sn] = r;
                    }
                }
            }
        }
}

// The store of a gated pair (GemmParams::pair_op): lanes c and c + 16 of an MFMA tile hold G and U of one element of
// C, column 16 * (virtual column / 32) + c % 16. Each of the two lanes computes and stores half of the tile's rows: the
// lower lane registers 0 .. 7, the upper one registers 8 .. 15, and one lane exchange per pair of registers hands each
// the factor it lacks (the lower lane sends its register v + 8 and gets the partner's register v, the upper lane the
// other way round). Roundings as the separate operations place them: the two products, the sigmoid (the hardware's 2^x
// and reciprocal, like the generated elementwise kernels use for halves) and both multiplications are each rounded to f16.
template <int MI, int NI>
__device__ __forceinline__ void store_tiles_gated(const GemmParams &p, const floatx16 (&acc)[MI][NI], int bz, int row0, int col0) {
    const int lane = threadIdx.x & 63, c = lane & 31, half = lane >> 5;
    const bool low = c < 16;
    const int n_out = p.n / 2;
    half_t *out = (half_t *) p.c + bz * p.c_sb;
    auto r16 = [](float x) { return (float) (half_t) x; };
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const int col = ((col0 + 32 * j) >> 5) * 16 + (c & 15);
#pragma unroll
            for (int v = 0; v < 8; v++) {
                const float lo = acc[i][j][v], hi = acc[i][j][v + 8];
                const float got = __shfl_xor(low ? hi : lo, 16);
                const float g = r16(low ? lo : got), u = r16(low ? got : hi);
                const float sig = r16(__frcp_rn(1.0f + __expf(-g)));
                const float act = r16(r16(g * sig) * u);
                const int w = low ? v : v + 8;
                const int row = row0 + 32 * i + 8 * (w >> 2) + 4 * half + (w & 3);
                if (row < p.m && col < n_out) out[(long long) row * p.c_sm + (long long) col * p.c_sn] = (half_t) act;
            }
        }
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
    tile_of_block((int) blockIdx.x, (int) gridDim.x, tiles_m, tiles_n * p.groups, xcd_chunk, &tm, &tn);
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

    store_tiles<half_t, TI, TI>(p, acc, c_base, bz, m0 + wm * 32 * TI, n0 + wn * 32 * TI);
}

constexpr int DIRECT_ROW = 128;  // bytes of a row of a slice: 64 halves or 32 floats

template <int N>
__device__ __forceinline__ void wait_for_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// One slice of both operands on its way, global -> LDS: load i of the wave fills the 1024 bytes at dst + 1024 i,
// lane l the 16 bytes at 16 l of them from its own source address, which then moves on by `advance` elements.
// (The host pass of the compiler does not know the load instruction, hence the guard.)
template <typename T, int A_LD, int B_LD>
__device__ __forceinline__ void issue_loads(const T *(&a_src)[A_LD], const T *(&b_src)[B_LD], char *dst_a, char *dst_b, int advance) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int i = 0; i < A_LD; i++) {
        __builtin_amdgcn_global_load_lds(a_src[i], dst_a + i * 1024, 16, 0, 0);
        a_src[i] += advance;
    }
#pragma unroll
    for (int i = 0; i < B_LD; i++) {
        __builtin_amdgcn_global_load_lds(b_src[i], dst_b + i * 1024, 16, 0, 0);
        b_src[i] += advance;
    }
#endif
}

// compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// One K step of a wave's MI x NI MFMA tiles from the operands in `ca` / `cb`, 16 bytes per lane and tile row: 8 halves
// for one v_mfma_f32_32x32x16_f16 per tile, or 4 floats for four v_mfma_f32_32x32x2_f32 (element u of the vector
// multiplies k = 8 t + u in the lower half of the wave and 8 t + 4 + u in the upper, in A and B alike). Other work is
// slotted in between the MFMAs so that the matrix cores never wait for it: `pre(m)` runs right in front of MFMA m,
// and the scheduling barriers keep the compiler from moving it. The operands of the following step are read during
// this one (read r goes in front of MFMA r, the operands the next step needs first are read first), so a wave
// needs no second wave on its SIMD to cover LDS latency.
template <typename T, int MI, int NI, int ROW, typename V, typename Pre>
__device__ __forceinline__ void mfma_step(floatx16 (&acc)[MI][NI], const V (&ca)[MI], const V (&cb)[NI], V (&na)[MI], V (&nb)[NI],
                                          const char *src_a, const char *src_b, Pre &&pre) {
    constexpr int U = sizeof(T) == 2 ? 1 : 4, R = MI + NI, M = MI * NI * U;
    auto read_next = [&](auto rc) {
        constexpr int r = decltype(rc)::value;
        // order of need in the next step (i-major MFMAs): a[0], b[0 .. NI - 1], a[1 ..]
        if constexpr (r == 0) na[0] = *(const V *) src_a;
        else if constexpr (r <= NI) nb[r - 1] = *(const V *) (src_b + (r - 1) * 32 * ROW);
        else na[r - NI] = *(const V *) (src_a + (r - NI) * 32 * ROW);
    };
    // with fewer MFMAs than reads, the surplus reads go first
    static_for<0, (R > M ? R - M : 0)>([&](auto rc) { read_next(rc); });
    static_for<0, M>([&](auto mc) {
        constexpr int m = decltype(mc)::value, r = m + (R > M ? R - M : 0);
        constexpr int u = m / (MI * NI), i = (m % (MI * NI)) / NI, j = m % NI;
        pre(mc);
        if constexpr (r < R) read_next(std::integral_constant<int, r>{});
        if constexpr (sizeof(T) == 2) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ca[i], cb[j], acc[i][j], 0, 0, 0);
        else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[i][u], cb[j][u], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    });
}

// The direct-to-LDS kernel: a workgroup of WM x WN waves owns a (32 MI WM) x (32 NI WN) tile, a wave MI x NI MFMA
// tiles of it. K is walked in slices of 64 through a ring of NSTAGE LDS stages; every stage holds the rows of A,
// then those of B, 128 bytes each. One load instruction of a wave fills 8 rows (64 chunks of 16 bytes): lane l fills chunk
// position l % 8 of row l / 8, so it fetches chunk (l % 8) ^ swz(row) of that row. Rows past the edge of a matrix
// repeat its last row; they only feed results that are not stored.
// Per slice: wait for the own loads of this slice (those of the NSTAGE - 2 slices after it may still be in
// flight), barrier (now everybody's have landed, and everybody is done reading the stage of the slice before),
// start the loads of slice s + NSTAGE - 1 into that stage, multiply.
//
// Tiles can share the launch in two ways. The first `head_tiles` tiles (in launch order) are computed by one
// workgroup each, over all of K. Every further tile is shared by `tail_split` workgroups, which take
// `tail_k_chunk` of K each, park their f32 partial tile in the workspace and count themselves in on the tile's
// counter; whoever comes last adds the partial tiles up (always in the order of K, so the result does not depend on
// who that is), applies the epilogue, stores, and puts the counter back to zero for the next launch. A launch
// with too few tiles for the chip splits all of them (head_tiles = 0); one whose tile count leaves the last round
// of workgroups mostly idle splits just that round, so that it is short instead of sparse.
struct DirectSchedule {
    int k_chunk;     // split over gridDim.z, partial products summed by a second launch (batched products)
    int xcd_chunk;
    int head_tiles, tail_split, tail_k_chunk;
};

// BSTREAM: the loads of the right operand carry the non-temporal hint (GemmTuning::stream_b)
template <typename T, int MI, int NI, int WM, int WN, int NSTAGE, bool BSTREAM>
__global__ __launch_bounds__(64 * WM * WN) void gemm_direct_kernel(GemmParams p, DirectSchedule sched) {
    constexpr int WAVES = WM * WN, TM = 32 * MI * WM, TN = 32 * NI * WN, ROW = DIRECT_ROW, BK = ROW / (int) sizeof(T), VEC = 16 / (int) sizeof(T);
    constexpr int A_BYTES = TM * ROW, STAGE = (TM + TN) * ROW;
    constexpr int ROWS_PER_LOAD = 1024 / ROW, CHUNKS = ROW / 16;  // one load instruction of a wave moves 1024 bytes
    constexpr int A_LD = TM / ROWS_PER_LOAD / WAVES, B_LD = TN / ROWS_PER_LOAD / WAVES;  // load instructions per wave and stage
    static_assert(A_LD >= 1 && B_LD >= 1 && NSTAGE >= 2, "tile too small for the workgroup");
    static_assert(TM % (ROWS_PER_LOAD * WAVES) == 0 && TN % (ROWS_PER_LOAD * WAVES) == 0, "rows of a stage do not divide over the waves");
    static_assert((NSTAGE - 2) * (A_LD + B_LD) < 64, "the counter of loads in flight has 6 bits");
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tiles_m = (p.m + TM - 1) / TM, tiles_n = (p.n + TN - 1) / TN;
    const int tiles = tiles_m * tiles_n * p.groups;
    // which tile, and which part of K
    int tile_id = (int) blockIdx.x, chunk = 0;
    const bool shared_tile = tile_id >= sched.head_tiles;
    if (shared_tile) {
        const int t = tile_id - sched.head_tiles;
        tile_id = sched.head_tiles + t / sched.tail_split;
        chunk = t % sched.tail_split;
    }
    int tm, tn;
    if (shared_tile) tile_of_block(tile_id, tiles, tiles_m, tiles_n * p.groups, 0, &tm, &tn);
    else tile_of_block(tile_id, sched.head_tiles, tiles_m, tiles_n * p.groups, sched.xcd_chunk, &tm, &tn);
    const int group = tn / tiles_n;
    tn -= group * tiles_n;
    const void *b_base = p.groups > 1 ? p.b_group[group] : p.b;
    void *c_base = p.groups > 1 ? p.c_group[group] : p.c;
    const int bz = blockIdx.y;
    const int m0 = tm * TM, n0 = tn * TN;
    int k_begin = blockIdx.z * sched.k_chunk, k_end = min(p.k, k_begin + sched.k_chunk);
    if (shared_tile) {
        k_begin = chunk * sched.tail_k_chunk;
        k_end = min(p.k, k_begin + sched.tail_k_chunk);
    }
    const int slices = (k_end - k_begin) / BK;

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WN, wn = wave % WN, c = lane & 31, half = lane >> 5;

    floatx16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // MFMA operand of lane (row c, half h) at step t: chunk 2 t + h of its row, found at (2 t + h) ^ swz(c), which is
    // the address of step 0 with bits 5 and 6 flipped by t
    auto swz = [](int row) { return (row >> 1) & 7; };
    const unsigned a_rd = (wm * 32 * MI + c) * ROW + ((half ^ swz(c)) * 16);
    const unsigned b_rd = A_BYTES + (wn * 32 * NI + c) * ROW + ((half ^ swz(c)) * 16);

    // Software pipelined main loop. Every lane keeps 32 bit byte offsets from the tile's uniform base
    // pointers, which move on by one slice per issue on the scalar unit. A slice is walked in 4 steps of 16 k; the
    // operands of step t + 1 are read from LDS between the MFMAs of step t. In the last step of a slice the wave
    // waits for its own loads of the next slice, meets the others at the barrier (everybody's loads have landed,
    // and everybody has read the last operands of this slice), sends the loads of the slice NSTAGE further on into
    // the stage just read, and reads the first operands of the next slice, all between the MFMAs of that step.
    constexpr int LD = A_LD + B_LD;
    const int lr = lane / CHUNKS, pos = lane % CHUNKS;
    const char *a_tile = (const char *) ((const T *) p.a + bz * p.a_sb + k_begin + (long long) m0 * p.a_sm);
    // (a gated pair reads rows of two matrices: offsets from the lower of the two bases, see below)
    const char *pair_lo = (const char *) p.b < (const char *) p.b_pair ? (const char *) p.b : (const char *) p.b_pair;
    const char *b_tile = p.pair_op ? pair_lo + ((long long) bz * p.b_sb + k_begin) * (long long) sizeof(T)
                                   : (const char *) ((const T *) b_base + bz * p.b_sb + k_begin + (long long) n0 * p.b_sn);
    unsigned a_off[A_LD], b_off[B_LD];
#pragma unroll
    for (int i = 0; i < A_LD; i++) {
        const int row = (wave * A_LD + i) * ROWS_PER_LOAD + lr;
        a_off[i] = (unsigned) (((long long) (min(m0 + row, p.m - 1) - m0) * p.a_sm + VEC * (pos ^ swz(row))) * (long long) sizeof(T));
    }
#pragma unroll
    for (int i = 0; i < B_LD; i++) {
        const int row = (wave * B_LD + i) * ROWS_PER_LOAD + lr;
        b_off[i] = (unsigned) (((long long) (min(n0 + row, p.n - 1) - n0) * p.b_sn + VEC * (pos ^ swz(row))) * (long long) sizeof(T));
        if (p.pair_op) {
            // virtual column -> (matrix, column): the first 16 columns of a block of 32 are G's, the others U's
            const int vcol = n0 + row, col = min((vcol >> 5) * 16 + (vcol & 15), p.n / 2 - 1);
            const char *base = (vcol & 16) ? (const char *) p.b_pair : (const char *) p.b;
            b_off[i] = (unsigned) ((long long) (base - pair_lo) + ((long long) col * p.b_sn + VEC * (pos ^ swz(row))) * (long long) sizeof(T));
        }
    }
    char *const dst_a = lds + wave * A_LD * 1024, *const dst_b = lds + A_BYTES + wave * B_LD * 1024;
    // load l of a slice: the first A_LD fill rows of A, the others rows of B
    auto issue_load = [&](auto lc, unsigned stage) {
        constexpr int l = decltype(lc)::value;
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (l < A_LD) __builtin_amdgcn_global_load_lds((const void *) (a_tile + a_off[l]), dst_a + stage + l * 1024, 16, 0, 0);
        else __builtin_amdgcn_global_load_lds((const void *) (b_tile + b_off[l - A_LD]), dst_b + stage + (l - A_LD) * 1024, 16, 0, BSTREAM ? 2 : 0);
#endif
    };
    int fetched = 0;  // slices whose loads have been issued
    auto advance = [&]() {
        // once no slice is left, the last one is fetched again, into a stage nobody reads any more
        fetched++;
        if (fetched < slices) {
            a_tile += ROW;
            b_tile += ROW;
        }
    };
#pragma unroll
    for (int j = 0; j < NSTAGE - 1; j++) {
        static_for<0, LD>([&](auto lc) { issue_load(lc, (unsigned) (j * STAGE)); });
        advance();
    }
    // operand addresses of the steps within a stage
    constexpr int STEPS = ROW / 32;
    unsigned a_rd_t[STEPS], b_rd_t[STEPS];
#pragma unroll
    for (int t = 0; t < STEPS; t++) {
        a_rd_t[t] = a_rd ^ (32 * t);
        b_rd_t[t] = b_rd ^ (32 * t);
    }
    typedef typename std::conditional<sizeof(T) == 2, halfx8, floatx4>::type V;
    V ra[2][MI], rb[2][NI];
    wait_for_loads<(NSTAGE - 2) * LD>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    static_for<0, LD>([&](auto lc) { issue_load(lc, (unsigned) ((NSTAGE - 1) * STAGE)); });
    advance();
#pragma unroll
    for (int i = 0; i < MI; i++) ra[0][i] = *(const V *) (lds + a_rd_t[0] + i * 32 * ROW);
#pragma unroll
    for (int j = 0; j < NI; j++) rb[0][j] = *(const V *) (lds + b_rd_t[0] + j * 32 * ROW);
    unsigned stage_off = 0;
    auto nothing = [](auto) {};
    for (int s = 0; s < slices; s++) {
        const char *st = lds + stage_off;
        const unsigned next_off = stage_off + STAGE == NSTAGE * STAGE ? 0 : stage_off + STAGE;
        // (STEPS is even: the operand registers alternate, step t multiplies set t % 2 and fills the other)
        static_for<0, STEPS - 1>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            mfma_step<T, MI, NI, ROW>(acc, ra[t & 1], rb[t & 1], ra[(t + 1) & 1], rb[(t + 1) & 1], st + a_rd_t[t + 1], st + b_rd_t[t + 1], nothing);
        });
        // the turn of the ring: the own loads of slice s + 1 have landed, the own reads of slice s are complete
        wait_for_loads<(NSTAGE - 2) * LD>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        const char *nx = lds + next_off;
        constexpr int M = MI * NI * (sizeof(T) == 2 ? 1 : 4), PER = (LD + M - 1) / M;
        mfma_step<T, MI, NI, ROW>(acc, ra[1], rb[1], ra[0], rb[0], nx + a_rd_t[0], nx + b_rd_t[0], [&](auto mc) {
            constexpr int m = decltype(mc)::value;
            static_for<0, PER>([&](auto uc) {
                constexpr int l = m * PER + decltype(uc)::value;
                if constexpr (l < LD) issue_load(std::integral_constant<int, l>{}, stage_off);
            });
        });
        advance();
        stage_off = next_off;
    }
    wait_for_loads<0>();

    if (shared_tile && sched.tail_split > 1) {
        // park the partial tile: [workgroup of the tile][wave][MFMA tile][register / 4][lane][register % 4], so that
        // a wave moves 1 KB per instruction
        const int shared_index = tile_id - sched.head_tiles;
        // The partial tiles travel between workgroups that may sit on different XCDs, each with an L2 of its own:
        // they are written and read with device scope accesses (sc1), which go past those caches, instead of
        // fences that would write back and invalidate a whole L2 (measured: 163 us instead of 69 us for
        // 512 x 4096 x 11008).
        constexpr int SC1 = 16;  // auxiliary bits of the buffer instructions: device scope
        float *tile_slots = (float *) p.workspace + (size_t) shared_index * sched.tail_split * (TM * TN);
        const __amdgpu_buffer_rsrc_t slots = __builtin_amdgcn_make_buffer_rsrc(tile_slots, 0, sched.tail_split * (TM * TN) * 4, 0x00020000);
        const int thread_off = (wave * (MI * NI * 16 * 64) + lane * 4) * 4;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NI; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const floatx4 x = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, x), slots,
                                                           chunk * (TM * TN * 4) + thread_off + ((i * NI + j) * 4 + q) * 1024, 0, SC1);
                }
        // the stores have been acknowledged before the workgroup counts itself in
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // (also: every wave is done with the LDS stages)
        int *counter = (int *) p.counters + shared_index, *arrived = (int *) lds;
        if (threadIdx.x == 0) *arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*(volatile int *) arrived != sched.tail_split - 1) return;
        // the last one in: sum over the parts of K in their order
        floatx16 sum[MI][NI];
        for (int part = 0; part < sched.tail_split; part++) {
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const floatx4 x = __builtin_bit_cast(
                            floatx4, __builtin_amdgcn_raw_buffer_load_b128(slots, part * (TM * TN * 4) + thread_off + ((i * NI + j) * 4 + q) * 1024, 0, SC1));
#pragma unroll
                        for (int u = 0; u < 4; u++) sum[i][j][4 * q + u] = part == 0 ? x[u] : sum[i][j][4 * q + u] + x[u];
                    }
        }
        if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if constexpr (sizeof(T) == 2) {
            if (p.pair_op) {
                store_tiles_gated<MI, NI>(p, sum, bz, m0 + wm * 32 * MI, n0 + wn * 32 * NI);
                return;
            }
        }
        store_tiles<T, MI, NI>(p, sum, c_base, bz, m0 + wm * 32 * MI, n0 + wn * 32 * NI);
        return;
    }
    if constexpr (sizeof(T) == 2) {
        if (p.pair_op) {
            store_tiles_gated<MI, NI>(p, acc, bz, m0 + wm * 32 * MI, n0 + wn * 32 * NI);
            return;
        }
    }
    store_tiles<T, MI, NI>(p, acc, c_base, bz, m0 + wm * 32 * MI, n0 + wn * 32 * NI);
}

template <typename T, int MI, int NI, int WM, int WN, int NSTAGE>
int launch_direct(dim3 grid, hipStream_t stream, const GemmParams &p, const DirectSchedule &sched) {
    constexpr int LDS_BYTES = NSTAGE * (32 * MI * WM + 32 * NI * WN) * DIRECT_ROW;
    auto kernel = p.tuning.stream_b ? gemm_direct_kernel<T, MI, NI, WM, WN, NSTAGE, true> : gemm_direct_kernel<T, MI, NI, WM, WN, NSTAGE, false>;
    // more than 64 KB of dynamic LDS has to be asked for, once per device
    static bool allowed[2][64] = {};
    int device = 0;
    if (LDS_BYTES > 64 * 1024) {
        int e = (int) hipGetDevice(&device);
        if (e == 0 && (device < 0 || device >= 64)) e = (int) hipErrorInvalidDevice;
        if (e == 0 && !allowed[p.tuning.stream_b][device]) {
            e = (int) hipFuncSetAttribute((const void *) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
            if (e == 0) allowed[p.tuning.stream_b][device] = true;
        }
        if (e != 0) return e;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * WM * WN), LDS_BYTES, stream, p, sched);
    return 0;
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

int launch_gemm_f32_direct(const GemmLaunchPlan &lp, ihipStream_t *stream, bool *launched) {
    *launched = false;
    const GemmParams &p = lp.p;
    if (!lp.direct || lp.k_chunk % 32 != 0) return 0;
    const int groups = p.groups > 1 ? p.groups : 1;
    bool aligned = (uintptr_t) p.a % 16 == 0;
    for (int g = 0; g < groups; g++) aligned = aligned && (uintptr_t) (groups > 1 ? p.b_group[g] : p.b) % 16 == 0;
    if (!aligned) return 0;
    const int t_m = lp.skinny_tile ? 32 : (lp.small_tile ? 64 : 128), t_n = lp.skinny_tile ? 128 : t_m;
    const long long tiles = (long long) ((p.m + t_m - 1) / t_m) * ((p.n + t_n - 1) / t_n) * groups;
    if (tiles > 0x7fffffffll) return (int) hipErrorInvalidConfiguration;
    dim3 grid((unsigned) tiles, (unsigned) p.batch, (unsigned) lp.split_k);
    DirectSchedule sched{lp.k_chunk, 64, (int) tiles, 1, p.k};
    if (lp.tail_split > 1) {
        if (p.workspace == nullptr || p.counters == nullptr) return (int) hipErrorInvalidValue;
        sched.head_tiles = lp.head_tiles;
        sched.tail_split = lp.tail_split;
        sched.tail_k_chunk = lp.tail_k_chunk;
        grid.x = (unsigned) (lp.head_tiles + (tiles - lp.head_tiles) * lp.tail_split);
    }
    // (64 x 64 tiles on three stages: 48 KB of LDS, so three workgroups share a compute unit; on four stages and two
    // workgroups the 8192 x 320 x 320 projections of a transformer block took 26.7 us instead of 24.9 us)
    const int e = lp.skinny_tile ? launch_direct<float, 1, 1, 1, 4, 3>(grid, stream, p, sched)
                  : lp.small_tile ? launch_direct<float, 1, 1, 2, 2, 3>(grid, stream, p, sched) : launch_direct<float, 2, 2, 2, 2, 2>(grid, stream, p, sched);
    if (e != 0) return e;
    *launched = true;
    return (int) hipGetLastError();
}

int launch_gemm_f16(const GemmLaunchPlan &lp, ihipStream_t *stream) {
    const GemmParams &p = lp.p;
    if (p.batch <= 0 || p.m <= 0 || p.n <= 0) return 0;
    if (lp.dot) return launch_gemm_dot(lp, true, stream);
    const int groups = p.groups > 1 ? p.groups : 1;
    if (groups > GEMM_MAX_GROUPS || (groups > 1 && (lp.split_k > 1 || p.addend || lp.swapped))) return (int) hipErrorInvalidValue;
    if (p.addend2 != nullptr && p.addend == nullptr) return (int) hipErrorInvalidValue;
    if (p.batch > 65535 || (long long) p.m * p.n > 0x7fffffffll * 256) return (int) hipErrorInvalidConfiguration;
    if (lp.split_k > 1 && p.workspace == nullptr) return (int) hipErrorInvalidValue;
    if (p.pair_op) {
        // a gated pair: only what the plan promised (direct kernel, one product per launch, whole K per workgroup), and
        // both matrices within reach of the 32 bit offsets from the lower of the two
        const long long apart = (const char *) p.b_pair - (const char *) p.b, span = ((long long) (p.n / 2) * p.b_sn + p.k) * 2;
        if (p.pair_op != GEMM_PAIR_SWIGLU || p.b_pair == nullptr || groups > 1 || p.addend || lp.split_k > 1 || lp.swapped ||
            !lp.direct || p.n % 2 != 0 || (apart < 0 ? -apart : apart) + span >= 0xffffffffll || (uintptr_t) p.b_pair % 16 != 0)
            return (int) hipErrorInvalidValue;
    }
    const int a_mode = pick_mode(p.a, p.a_sm, p.a_sk, p.m, p.k, p.a_sb, p.batch);
    int b_mode = pick_mode(groups > 1 ? p.b_group[0] : p.b, p.b_sn, p.b_sk, p.n, p.k, p.b_sb, p.batch);
    for (int g = 1; g < groups; g++) {  // the loader that every operand of the group allows
        const int mode = pick_mode(p.b_group[g], p.b_sn, p.b_sk, p.n, p.k, p.b_sb, p.batch);
        if (mode != b_mode) b_mode = Scalar;
    }
    // both operands K contiguous and K (and every split of it) whole slices: the direct-to-LDS kernel
    const bool direct = lp.direct && a_mode == VecK && b_mode == VecK && lp.k_chunk % 64 == 0;
    if (p.pair_op && !direct) return (int) hipErrorInvalidValue;
    // (128 x 64 tiles exist in the direct kernel only; without it they run as 64 x 64)
    // (so do 256 x 256 and 256 x 192 tiles, which otherwise run as 256 x 128)
    const bool narrow = lp.narrow_tile && direct, small = lp.small_tile || (lp.narrow_tile && !direct);
    const bool wide = lp.wide_tile && direct, mid = lp.mid_tile && direct;
    const int t_n = small || narrow ? 64 : (wide ? 256 : (mid ? 192 : 128)), t_m = lp.tall_tile ? 256 : (small ? 64 : 128);
    const long long tiles = (long long) ((p.m + t_m - 1) / t_m) * ((p.n + t_n - 1) / t_n) * groups;
    if (tiles > 0x7fffffffll) return (int) hipErrorInvalidConfiguration;
    dim3 grid((unsigned) tiles, (unsigned) p.batch, (unsigned) lp.split_k);
    // Measured on 128 x 128 tiles of the kernel that stages through registers (TFLOP/s at 4096^3 / 8192^3): BK 64
    // single buffered 594 / 757, BK 64 double buffered 643 / 718, BK 128 single buffered 672 / 744.
    // workgroups an XCD (32 compute units) runs at a time: 1 per compute unit for the tall tiles, else 2
    const int xc = lp.tall_tile || narrow ? 32 : 64;  // (also for the 256 x 256 tiles)
    if (direct) {
        DirectSchedule sched{lp.k_chunk, xc, (int) tiles, 1, p.k};
        if (lp.tail_split > 1) {
            if (p.workspace == nullptr || p.counters == nullptr) return (int) hipErrorInvalidValue;
            sched.head_tiles = lp.head_tiles;
            sched.tail_split = lp.tail_split;
            sched.tail_k_chunk = lp.tail_k_chunk;
            grid.x = (unsigned) (lp.head_tiles + (tiles - lp.head_tiles) * lp.tail_split);
        }
        int e;
        if (small) e = launch_direct<half_t, 1, 1, 2, 2, 4>(grid, stream, p, sched);
        else if (narrow) e = launch_direct<half_t, 2, 1, 2, 2, 4>(grid, stream, p, sched);
        else if (wide) e = launch_direct<half_t, 4, 2, 2, 4, 2>(grid, stream, p, sched);
        else if (mid) e = launch_direct<half_t, 2, 3, 4, 2, 2>(grid, stream, p, sched);
        else if (lp.tall_tile) e = launch_direct<half_t, 2, 2, 4, 2, 3>(grid, stream, p, sched);
        else e = launch_direct<half_t, 2, 2, 2, 2, 2>(grid, stream, p, sched);
        if (e != 0) return e;
    } else if (small) launch_a<1, 64, 2, 2>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    else if (lp.tall_tile) launch_a<2, 64, 1, 4>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    else launch_a<2, 128, 1, 2>(a_mode, b_mode, grid, stream, p, lp.k_chunk, xc);
    int e = (int) hipGetLastError();
    if (e == 0 && lp.split_k > 1) e = launch_gemm_reduce_partials(p, lp.split_k, true, stream);
    return e;
}

}  // namespace kn
