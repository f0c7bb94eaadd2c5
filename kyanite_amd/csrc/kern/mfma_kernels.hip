// f32 matrix multiply and fused convolution on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One workgroup of 4 waves computes a 128 x 128 tile of D = A * B; every wave owns a 64 x 64 quadrant as 2 x 2
// MFMA tiles of 32 x 32 (64 accumulator registers per lane). Problems with too few such tiles to fill the chip
// use 64 x 64 tiles instead (one MFMA tile per wave). The K dimension is walked in slices of 16 that are
// staged through LDS as As[k][m] and Bs[k][n]; the next slice is fetched into registers while the current one is
// multiplied. Operand slices are fetched by small loader objects, so the same main loop serves strided batched
// GEMM (any row / column / batch strides) and convolution as an implicit GEMM (the B operand gathers input
// patches on the fly, with zero padding), with bias + residual + relu applied to the accumulators before the store.
//
// Loaders come in three flavours, picked on the host per operand:
//   VecOuter  the non-K axis is contiguous (stride 1) and rows are 16 byte aligned: one 128 bit load moves 4
//             neighbouring m (or n) of one k, stored to LDS as one 128 bit write
//   VecK      the K axis is contiguous: one 128 bit load moves 4 neighbouring k of one m (or n)
//   Scalar    anything else (arbitrary strides), and every tile that sticks out of the matrix
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "../mfma_kernels.h"

namespace kn {

namespace {

// BM x BN is the large tile of the convolution kernels; the generic kernels take their tile (64 or 128 wide per
// axis) from the loaders, the plane kernel from its template arguments. LDS rows are padded by 4 floats: rows stay 16 byte aligned and successive k rows shift
// by 4 banks.
constexpr int BM = 128, BN = 128, THREADS = 256;

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

enum LoadMode { Scalar = 0, VecOuter = 1, VecK = 2 };

// A [outer, K] operand addressed as p[outer * so + k * sk]; `outer` is m for A and n for B.
struct StridedOperand {
    const float *p;
    long long so, sk;
    int outer_size, K;
};

// Fetches one BK x WIDTH slice (WIDTH = 64 or 128) of a strided operand into registers and writes it to LDS as
// [k][outer]. BK is 16, or 64 for the 64 wide tiles of problems with a long K axis: those are chosen when there is
// little work per compute unit, and deeper slices keep more bytes in flight per round trip to memory (measured:
// 8 x 4096 x 4096 171 -> 148 us, 512 x 4096 x 4096 224 -> 212 us; with K of a few hundred the shallow slices win).
template <int MODE, int WIDTH, int BK_>
struct StridedLoader {
    static constexpr int BK = BK_;
    static constexpr int EPT = BK * WIDTH / THREADS;  // elements per thread
    // Rows padded by 4 keep the 128 bit stores of the VecOuter mode aligned. The transposing stores of the VecK mode
    // write 4 * (BK / 4) different k rows per wave: with 64 deep slices an odd stride spreads them over all banks
    // (two lanes per bank, the minimum), a multiple of 4 would pile them onto two groups of four banks.
    static constexpr int LDS_STRIDE = (MODE == VecK && BK > 16) ? WIDTH + 1 : WIDTH + 4;
    StridedOperand op;
    int o0;        // first outer index of this workgroup's tile
    bool interior; // the tile lies completely inside the matrix along the outer axis
    float r[EPT];

    __device__ __forceinline__ StridedLoader(const StridedOperand &operand, int outer0)
        : op(operand), o0(outer0), interior(outer0 + WIDTH <= operand.outer_size) {}

    __device__ __forceinline__ void fetch(int k0) {
        const int t = threadIdx.x;
        if (MODE == VecOuter && interior && k0 + BK <= op.K) {
            // thread -> (k = t / (WIDTH / 4) (+ ..), outer = 4 * (t % (WIDTH / 4)) ..)
#pragma unroll
            for (int h = 0; h < EPT / 4; h++) {
                const int k = t / (WIDTH / 4) + (THREADS * 4 / WIDTH) * h, o = (t % (WIDTH / 4)) * 4;
                const floatx4 v = *(const floatx4 *) (op.p + (long long) (o0 + o) * op.so + (long long) (k0 + k) * op.sk);
#pragma unroll
                for (int j = 0; j < 4; j++) r[4 * h + j] = v[j];
            }
        } else if (MODE == VecK && interior && k0 + BK <= op.K) {
            // thread -> (outer = t / 4 (+64), k = 4 * (t % 4) ..)
#pragma unroll
            for (int h = 0; h < EPT / 4; h++) {
                const int o = t / (BK / 4) + (THREADS * 4 / BK) * h, k = (t % (BK / 4)) * 4;
                const floatx4 v = *(const floatx4 *) (op.p + (long long) (o0 + o) * op.so + (long long) (k0 + k) * op.sk);
#pragma unroll
                for (int j = 0; j < 4; j++) r[4 * h + j] = v[j];
            }
        } else {
            // lanes run along whichever axis has the smaller stride
            const bool along_k = (op.sk < 0 ? -op.sk : op.sk) < (op.so < 0 ? -op.so : op.so);
#pragma unroll
            for (int i = 0; i < EPT; i++) {
                const int e = t + THREADS * i;
                const int o = along_k ? (e / BK) : (e % WIDTH);
                const int k = along_k ? (e % BK) : (e / WIDTH);
                const bool ok = (o0 + o) < op.outer_size && (k0 + k) < op.K;
                r[i] = ok ? op.p[(long long) (o0 + o) * op.so + (long long) (k0 + k) * op.sk] : 0.0f;
            }
        }
    }

    // the layout decision has to match the one `fetch` took for the same slice
    __device__ __forceinline__ void stage(float (*lds)[LDS_STRIDE], int k0) const {
        const int t = threadIdx.x;
        if (MODE == VecOuter && interior && k0 + BK <= op.K) {
#pragma unroll
            for (int h = 0; h < EPT / 4; h++) {
                const int k = t / (WIDTH / 4) + (THREADS * 4 / WIDTH) * h, o = (t % (WIDTH / 4)) * 4;
                floatx4 v;
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = r[4 * h + j];
                *(floatx4 *) &lds[k][o] = v;
            }
        } else if (MODE == VecK && interior && k0 + BK <= op.K) {
#pragma unroll
            for (int h = 0; h < EPT / 4; h++) {
                const int o = t / (BK / 4) + (THREADS * 4 / BK) * h, k = (t % (BK / 4)) * 4;
#pragma unroll
                for (int j = 0; j < 4; j++) lds[k + j][o] = r[4 * h + j];
            }
        } else {
            const bool along_k = (op.sk < 0 ? -op.sk : op.sk) < (op.so < 0 ? -op.so : op.so);
#pragma unroll
            for (int i = 0; i < EPT; i++) {
                const int e = t + THREADS * i;
                const int o = along_k ? (e / BK) : (e % WIDTH);
                const int k = along_k ? (e % BK) : (e / WIDTH);
                lds[k][o] = r[i];
            }
        }
    }
};

// Input patches of a convolution as the B operand: k = (c, fy, fx), n = (image, oy, ox). Every thread keeps one
// fixed n for the whole K loop, so the position is decomposed once; KH / KW are compile-time constants (0 = read
// them from the parameters) so that splitting k costs multiplications instead of divisions.
template <int KH, int KW, int WIDTH, int BK_>
struct PatchLoader {
    static constexpr int BK = BK_;
    static constexpr int EPT = BK * WIDTH / THREADS;
    static constexpr int LDS_STRIDE = WIDTH + 4;
    const float *base;  // input of this thread's image, or null when n is out of range
    int K, in_h, in_w, kh, kw;
    int pos_off;               // iy0 * in_w + ix0: where tap (0, 0) of channel 0 lies for this thread's position
    unsigned long long taps;   // bit fy * kw + fx: the tap lies inside the image for this thread's position
    int iy0, ix0;              // (filters of more than 64 taps test the bounds per element instead)
    float r[EPT];

    __device__ __forceinline__ PatchLoader(const ConvParams &p, int n0) {
        kh = KH ? KH : p.kernel_h;
        kw = KW ? KW : p.kernel_w;
        K = p.in_c * kh * kw;
        in_h = p.in_h;
        in_w = p.in_w;
        const int n = n0 + (threadIdx.x % WIDTH);
        const int ohw = p.out_h * p.out_w;
        const long long total = (long long) p.batch * ohw;
        taps = 0;
        if (n < total) {
            const int img = n / ohw, pos = n - img * ohw;
            const int oy = pos / p.out_w, ox = pos - oy * p.out_w;
            iy0 = oy * p.stride_y - p.pad_y;
            ix0 = ox * p.stride_x - p.pad_x;
            base = p.input + (long long) img * p.in_c * in_h * in_w;
            if (kh * kw <= 64)
                for (int fy = 0; fy < kh; fy++)
                    for (int fx = 0; fx < kw; fx++)
                        if (iy0 + fy >= 0 && iy0 + fy < in_h && ix0 + fx >= 0 && ix0 + fx < in_w) taps |= 1ull << (fy * kw + fx);
        } else {
            base = nullptr;
            iy0 = ix0 = 0;
        }
        pos_off = iy0 * in_w + ix0;
    }

    // Every thread of a wave loads the same k (a wave covers 64 of the WIDTH positions of one k), so the split of k
    // into (channel, tap) and the tap's offset run on the scalar unit; a lane adds its position and tests one bit.
    __device__ __forceinline__ void fetch(int k0) {
        const int khw = kh * kw;
        const int k_row = __builtin_amdgcn_readfirstlane((int) threadIdx.x / WIDTH);
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int k = k0 + k_row + (THREADS / WIDTH) * i;
            const int c = k / khw, rem = k - c * khw;
            const int fy = rem / kw, fx = rem - fy * kw;
            if (khw <= 64) {
                const bool ok = k < K && ((taps >> rem) & 1ull) != 0;  // (no image: no taps)
                r[i] = ok ? base[(c * in_h + fy) * in_w + fx + pos_off] : 0.0f;  // inside one image: below 2^31, checked on the host
            } else {
                const int iy = iy0 + fy, ix = ix0 + fx;
                const bool ok = base != nullptr && k < K && iy >= 0 && iy < in_h && ix >= 0 && ix < in_w;
                r[i] = ok ? base[((long long) c * in_h + iy) * in_w + ix] : 0.0f;
            }
        }
    }

    __device__ __forceinline__ void stage(float (*lds)[LDS_STRIDE], int) const {
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int k = threadIdx.x / WIDTH + (THREADS / WIDTH) * i;
            lds[k][threadIdx.x % WIDTH] = r[i];
        }
    }
};

struct GemmStore {
    float *p;
    long long sm, sn;
    int M, N;
    const float *addend;  // optional epilogue operand (null = none), with its own strides
    long long dm, dn;
    const float *addend2;  // a second one, added after the first
    long long d2m, d2n;
    int relu;
    // what `prepare` derives for the two columns this lane owns
    const float *d_col[2];  // addend at (row 0, column), or null
    float d_bias[2];        // its value when the addend does not depend on the row (a bias): loaded once
    bool row_invariant;

    __device__ __forceinline__ void prepare(int col0, int col1) {
        const int cols[2] = {col0, col1};
        row_invariant = addend != nullptr && dm == 0;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            d_col[j] = addend != nullptr && cols[j] < N ? addend + (long long) cols[j] * dn : nullptr;
            d_bias[j] = row_invariant && d_col[j] ? *d_col[j] : 0.0f;
        }
    }
    __device__ __forceinline__ void store(int m, int n, int j, float v) const {
        if (m < M && n < N) {
            if (addend) v += row_invariant ? d_bias[j] : d_col[j][(long long) m * dm];
            if (addend2) v += addend2[(long long) m * d2m + (long long) n * d2n];
            if (relu) v = fmaxf(v, 0.0f);
            p[(long long) m * sm + (long long) n * sn] = v;
        }
    }
};

struct ConvStore {
    float *p;
    const float *bias;
    const float *res;
    long long bias_stride;
    int M, ohw;  // out_c, out_h * out_w
    long long N; // batch * out_h * out_w
    int relu;
    long long col_base[2];  // offset of (image, 0, position) for the two columns this lane owns
    bool col_ok[2];

    __device__ __forceinline__ void prepare(int col0, int col1) {
        const int cols[2] = {col0, col1};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            col_ok[j] = cols[j] < N;
            const int img = cols[j] / ohw, pos = cols[j] - img * ohw;
            col_base[j] = (long long) img * M * ohw + pos;
        }
    }
    __device__ __forceinline__ void store(int m, int, int j, float v) const {
        if (m < M && col_ok[j]) {
            const long long o = col_base[j] + (long long) m * ohw;
            if (res) v += res[o];
            if (bias) v += bias[m * bias_stride];
            if (relu) v = fmaxf(v, 0.0f);
            p[o] = v;
        }
    }
};

// MI x NI: MFMA tiles per wave; the workgroup tile is (64 * MI) x (64 * NI) with the 4 waves arranged 2 x 2.
template <int MI, int NI, typename LA, typename LB, typename S>
__device__ __forceinline__ void mfma_tile_loop(LA &la, LB &lb, S &s, int k_begin, int K, int m0, int n0) {
    constexpr int BK = LA::BK;
    static_assert(LA::BK == LB::BK, "both operands advance by the same slice");
    __shared__ __attribute__((aligned(16))) float As[BK][LA::LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[BK][LB::LDS_STRIDE];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    floatx16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    la.fetch(k_begin);
    lb.fetch(k_begin);
    for (int k0 = k_begin; k0 < K; k0 += BK) {
        __syncthreads();  // the previous slice has been consumed
        la.stage(As, k0);
        lb.stage(Bs, k0);
        __syncthreads();
        if (k0 + BK < K) {
            la.fetch(k0 + BK);
            lb.fetch(k0 + BK);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const int kr = kk + (lane >> 5), c = lane & 31;
            float a[MI], b[NI];
#pragma unroll
            for (int i = 0; i < MI; i++) a[i] = As[kr][wm * 32 * MI + 32 * i + c];
#pragma unroll
            for (int j = 0; j < NI; j++) b[j] = Bs[kr][wn * 32 * NI + 32 * j + c];
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }

    // accumulator layout of the 32x32 tile: register v of lane l holds row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32
    const int col0 = n0 + wn * 32 * NI + (lane & 31);
    s.prepare(col0, col0 + 32);
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 32 * MI + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                s.store(row, col0 + 32 * j, j, acc[i][j][v]);
            }
}

// Tiles are numbered so that the workgroups that run at the same time (consecutive ids) share rows of tiles:
// groups of 8 tile rows are walked column by column.
__device__ __forceinline__ void tile_of_id(int id, int tiles_m, int tiles_n, int *tm, int *tn) {
    const int group_rows = 8;
    const int per_group = group_rows * tiles_n;
    const int g = id / per_group, in_g = id - g * per_group;
    const int rows_here = min(group_rows, tiles_m - g * group_rows);
    *tm = g * group_rows + in_g % rows_here;
    *tn = in_g / rows_here;
}
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int *tm, int *tn) { tile_of_id(blockIdx.x, tiles_m, tiles_n, tm, tn); }

// TI: MFMA tiles per wave and axis (2 -> 128 x 128 workgroup tile, 1 -> 64 x 64); BK: depth of a K slice
template <int A_MODE, int B_MODE, int TI, int BK>
__global__ __launch_bounds__(THREADS) void gemm_f32_kernel(GemmParams p, int k_chunk) {
    constexpr int T = 64 * TI;
    // a grouped launch lines the tiles of its products up along n
    const int tiles_m = (p.m + T - 1) / T, tiles_n = (p.n + T - 1) / T;
    int tm, tn;
    tile_of_block(tiles_m, tiles_n * p.groups, &tm, &tn);
    const int group = tn / tiles_n;
    tn -= group * tiles_n;
    const void *b_base = p.groups > 1 ? p.b_group[group] : p.b;
    void *c_base = p.groups > 1 ? p.c_group[group] : p.c;
    const int bz = blockIdx.y;
    const int m0 = tm * T, n0 = tn * T;
    // split K: workgroup z of gridDim.z multiplies its own range of k and stores an f32 partial product
    const int k_begin = blockIdx.z * k_chunk, k_end = min(p.k, k_begin + k_chunk);
    StridedLoader<A_MODE, T, BK> la(StridedOperand{(const float *) p.a + bz * p.a_sb, p.a_sm, p.a_sk, p.m, k_end}, m0);
    StridedLoader<B_MODE, T, BK> lb(StridedOperand{(const float *) b_base + bz * p.b_sb, p.b_sn, p.b_sk, p.n, k_end}, n0);
    // the epilogue of a split launch is applied by the pass that sums the partial products
    GemmStore s = gridDim.z > 1
        ? GemmStore{(float *) p.workspace + ((long long) bz * gridDim.z + blockIdx.z) * p.m * p.n, p.n, 1, p.m, p.n,
                    nullptr, 0, 0, nullptr, 0, 0, 0, {nullptr, nullptr}, {0.0f, 0.0f}, false}
        : GemmStore{(float *) c_base + bz * p.c_sb, p.c_sm, p.c_sn, p.m, p.n,
                    p.addend ? (const float *) p.addend + bz * p.d_sb : nullptr, p.d_sm, p.d_sn,
                    p.addend2 ? (const float *) p.addend2 + bz * p.d2_sb : nullptr, p.d2_sm, p.d2_sn, p.relu,
                    {nullptr, nullptr}, {0.0f, 0.0f}, false};
    mfma_tile_loop<TI, TI>(la, lb, s, k_begin, k_end, m0, n0);
}

template <int A_MODE, int KH, int KW, int TI>
__global__ __launch_bounds__(THREADS) void conv_f32_kernel(ConvParams p) {
    constexpr int T = 64 * TI, BK = 16;
    const int kh = KH ? KH : p.kernel_h, kw = KW ? KW : p.kernel_w;
    const int K = p.in_c * kh * kw, ohw = p.out_h * p.out_w;
    const long long N = (long long) p.batch * ohw;
    const int tiles_m = (p.out_c + T - 1) / T, tiles_n = (int) ((N + T - 1) / T);
    int tm, tn;
    tile_of_block(tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * T, n0 = tn * T;
    // a launch that splits the input channels: slice blockIdx.y multiplies its own range of k and stores an f32 partial
    // result; bias, residual and activation are applied by the pass that sums the slices
    const int k_begin = p.splits > 1 ? blockIdx.y * p.split_channels * kh * kw : 0;
    const int k_end = p.splits > 1 ? min(K, k_begin + p.split_channels * kh * kw) : K;
    StridedLoader<A_MODE, T, BK> la(StridedOperand{p.filter, K, 1, p.out_c, k_end}, m0);
    PatchLoader<KH, KW, T, BK> lb(p, n0);
    lb.K = k_end;
    ConvStore s = p.splits > 1
        ? ConvStore{p.workspace + (long long) blockIdx.y * p.out_c * N, nullptr, nullptr, 0, p.out_c, ohw, N, 0, {0, 0}, {false, false}}
        : ConvStore{p.output, p.bias, p.res, p.bias_stride, p.out_c, ohw, N, p.relu, {0, 0}, {false, false}};
    mfma_tile_loop<TI, TI>(la, lb, s, k_begin, k_end, m0, n0);
}

// ---------------------------------------------------------------------------------------------------------------
// "Plane" convolution: 3 x 3 or 5 x 5 filter, stride 1, same-size output (image width a power of two in the variant described first). Instead of gathering the im2col
// matrix, every K slice (CB input channels x KH x KW taps) stages the raw input rows that the tile's TN = 128 or
// 64 output positions touch into LDS once, as [channel][group][row][W], and the MFMA B operand is read straight from those
// planes: position n of the tile sits at a fixed per-lane offset, tap (c, fy, fx) adds a wave-uniform offset. Every
// plane row has PLANE_PAD zero floats in front of it, so a tap left of the image reads the row's own padding and a
// tap right of it the next row's (rows above / below the image are stored as zero rows): no masking in the K loop.
// Global -> LDS traffic for B drops by KH * KW and no per-element index arithmetic is left in the K loop.
// A tile is either R = TN / W whole output rows of one image (H * W >= TN) or G = TN / (H * W) whole images.
constexpr int CB = 8;             // input channels per K slice of a 3 x 3 filter
// (a 5 x 5 filter takes 4: 100 filter rows per slice in LDS instead of 200)
constexpr int plane_slice_channels(int kh, int kw) { return kh * kw > 9 ? CB / 2 : CB; }
constexpr int PLANE_MAX_VEC = 3;  // 128 bit loads per thread and slice for the B planes
constexpr int PLANE_PAD = 4;      // zero floats in front of every plane row: what a tap left or right of the image reads
constexpr int PLANE_SLACK = 4;    // zero floats in front of / behind all planes
constexpr int PLANE_LDS = 2 * PLANE_MAX_VEC * THREADS * 4 + 2 * PLANE_SLACK;  // rows of 4 pixels double with the padding

struct PlaneGeom {
    int rows;            // R: output rows per group
    int groups;          // G: images per tile (1 when a tile is part of one image)
    int tiles_per_image; // H * W / 128, or 0 when a tile holds whole images
    int plane_rows;      // R + KH - 1
    int w4_shift, g_shift, rw_shift;  // log2 of W / 4, G, R * W
    int n_vec;           // CB * G * plane_rows * W / 4
    int row_stride;      // W + PLANE_PAD
    // Any image size (template flag ANYW): a tile is TN consecutive positions of the (image, y, x) order, wherever
    // they start. Every image counts H + 2 (5 x 5: H + 4) padded rows (empty rows above and below), so that the rows
    // above / below an output row are the padded rows before / after its own, across image boundaries too; the tile
    // stages the padded rows from the first one its first output row reads to the last one its last reads,
    // `plane_rows` at most, float by float (`n_scalar` = slice channels * plane_rows * W of them per slice).
    int n_scalar;
    int by4;  // the image width is a multiple of 4 and the input 16 byte aligned: staged four floats at a time
};
constexpr int PLANE_MAX_SCALAR = 8;  // 32 bit loads per thread and slice for the B planes of the ANYW variant
constexpr int PLANE_MAX_VEC4 = 4;    // 128 bit loads per thread and slice for the same when the width is a multiple of 4

// NJ: MFMA tiles per wave along the positions (2 -> 128 positions per workgroup tile, 1 -> 64); MI: the same along
// the output channels (2 -> 128 channels per tile, 1 -> 64); RAGGED: the channel count is not a multiple of CB (the
// 21 planes of a board game's input): the last slice takes zeros for the channels past the end, and the filter rows,
// whose length is no multiple of 4 floats then, are read float by float.
template <int KH, int KW, int NJ, int MI, bool RAGGED, int ANYW = 0>
__global__ __launch_bounds__(THREADS) void conv_plane_kernel(ConvParams p, PlaneGeom g) {
    // ANYW: 0 the power-of-two variant; 1 any image size, planes staged float by float; 2 the same with an image width
    // that is a multiple of 4, staged four floats at a time
    constexpr int EW = ANYW == 2 ? 4 : 1, ANY_SLOTS = ANYW == 2 ? PLANE_MAX_VEC4 : PLANE_MAX_SCALAR;
    constexpr int TN = 64 * NJ;  // positions per tile
    constexpr int BM = 64 * MI;  // output channels per tile
    constexpr int CBK = plane_slice_channels(KH, KW);
    constexpr int KS = CBK * KH * KW;     // K slice
    constexpr int A_VEC = KS / 4;         // 128 bit loads per filter row and slice
    constexpr int A_ITERS = (BM * A_VEC + THREADS - 1) / THREADS;
    // rows k and k + 1, which the two halves of a wave read together, lie 32 of the 64 LDS banks apart
    constexpr int A_STRIDE = BM + 32;
    static_assert(KS % 4 == 0 && KS % 2 == 0, "slice shape");
    __shared__ float As[KS][A_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[PLANE_LDS];

    const int W = p.in_w, H = p.in_h, C = p.in_c;
    const int K = C * KH * KW, ohw = H * W;
    const long long N = (long long) p.batch * ohw;
    const int tiles_m = (p.out_c + BM - 1) / BM, tiles_n = (int) ((N + TN - 1) / TN);
    // the tiles of a sparse last round are shared by `tail_parts` workgroups each, a slice of the input channels per part
    int tile_id = blockIdx.x, tail_part = -1;
    if (p.tail_parts > 1 && tile_id >= p.tail_head) {
        const int t_id = tile_id - p.tail_head;
        tile_id = p.tail_head + t_id / p.tail_parts;
        tail_part = t_id % p.tail_parts;
    }
    int tm, tn;
    tile_of_id(tile_id, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * TN;
    int img0 = 0, oy0 = 0;
    if (ANYW) {
    } else if (g.tiles_per_image) {
        img0 = tn / g.tiles_per_image;
        oy0 = (tn - img0 * g.tiles_per_image) * g.rows;
    } else {
        img0 = tn * g.groups;
    }

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1, half = lane >> 5, c32 = lane & 31;
    const int RS = g.row_stride;
    const int plane = g.plane_rows * RS, gplane = ANYW ? plane : plane << g.g_shift;  // LDS floats per (c, g) and per c
    // ANYW: the first padded row the tile's first output row reads (with PY = KH / 2 empty rows above and below every
    // image, output row rho of the (image, y) order is padded row rho + 2 * PY * (rho / H) + PY)
    constexpr int PY = KH / 2;
    const int rho0 = n0 / W, pi_base = rho0 + 2 * PY * (rho0 / H);

    // ---- B planes: what this thread moves per slice (the same places every slice, only the channel base moves)
    constexpr int B_SLOTS = ANYW ? ANY_SLOTS : PLANE_MAX_VEC;
    const float *b_src[PLANE_MAX_VEC];
    int b_dst[B_SLOTS];  // -1: nothing to move
    int b_channel[B_SLOTS];  // inside the slice
    int s_off[ANY_SLOTS];  // ANYW: offset of the float(s) inside the input, from channel 0 of the slice; -1: zeros
    if (ANYW) {
        const int wq = W / EW;  // loads per image row
#pragma unroll
        for (int i = 0; i < ANY_SLOTS; i++) {
            const int e = t + THREADS * i;
            const int x = (e % wq) * EW, t1 = e / wq;
            const int c = t1 / g.plane_rows, prow = t1 - c * g.plane_rows;
            const int pi = pi_base + prow, img = pi / (H + 2 * PY), iy = pi - img * (H + 2 * PY) - PY;
            const bool inside = e * EW < g.n_scalar && iy >= 0 && iy < H && img < p.batch;
            // (the empty rows above and below an image are never written: they keep the zeros of the first fill)
            b_dst[i] = inside ? PLANE_SLACK + t1 * RS + PLANE_PAD + x : -1;
            s_off[i] = inside ? ((img * C + c) * H + iy) * W + x : -1;  // below 2^31: checked on the host
            b_channel[i] = c;
        }
    }
#pragma unroll
    for (int i = 0; i < (ANYW ? 0 : PLANE_MAX_VEC); i++) {
        const int e = t + THREADS * i;
        const int w4 = e & ((1 << g.w4_shift) - 1), t1 = e >> g.w4_shift;
        const int t2 = t1 / g.plane_rows, prow = t1 - t2 * g.plane_rows;
        const int gg = t2 & (g.groups - 1), c = t2 >> g.g_shift;
        const int iy = oy0 + prow - p.pad_y, img = img0 + gg;
        const bool ok = e < g.n_vec && iy >= 0 && iy < H && img < p.batch;
        b_dst[i] = e < g.n_vec ? PLANE_SLACK + t1 * RS + PLANE_PAD + 4 * w4 : -1;
        b_src[i] = ok ? p.input + (((long long) img * C + c) * H + iy) * W + 4 * w4 : nullptr;
        b_channel[i] = c;
    }
    // ---- A (filter) rows: K contiguous
    const float *a_src[A_ITERS];
    int a_dst[A_ITERS], a_k[A_ITERS];  // a_k: the first of the 4 floats inside the slice
#pragma unroll
    for (int i = 0; i < A_ITERS; i++) {
        // (consecutive lanes take consecutive filter rows, so that their transposing stores hit different banks)
        const int e = t + THREADS * i, q = e / BM, row = e - q * BM;
        a_src[i] = q < A_VEC && (m0 + row) < p.out_c ? p.filter + (long long) (m0 + row) * K + 4 * q : nullptr;
        a_dst[i] = q < A_VEC ? 4 * q * A_STRIDE + row : -1;
        a_k[i] = 4 * q;
    }
    // ---- where this lane's output positions sit inside a plane, and which taps stay inside the image
    int lane_base[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int n = wn * 32 * NJ + 32 * j + c32;
        if (ANYW) {
            // (positions past the end take the place of the last one; their results are never stored)
            const int pos = (int) min((long long) n0 + n, N - 1), rho = pos / W, col = pos - rho * W;
            lane_base[j] = PLANE_SLACK + (rho + 2 * PY * (rho / H) - pi_base) * RS + PLANE_PAD + col - p.pad_x;
            continue;
        }
        const int gl = n >> g.rw_shift, rem = n & ((1 << g.rw_shift) - 1), col = rem & (W - 1), r = rem >> (g.w4_shift + 2);
        lane_base[j] = PLANE_SLACK + gl * plane + r * RS + PLANE_PAD + col - p.pad_x;
    }

    floatx4 ra[A_ITERS], rb[PLANE_MAX_VEC];
    float rs[ANYW == 1 ? ANY_SLOTS : 1];
    floatx4 rv[ANYW == 2 ? ANY_SLOTS : 1];
    auto fetch_planes_any = [&](int c0) {
        const float *from = p.input + (long long) c0 * ohw;
#pragma unroll
        for (int i = 0; i < ANY_SLOTS; i++) {
            const bool wanted = s_off[i] >= 0 && (!RAGGED || c0 + b_channel[i] < C);
            if constexpr (ANYW == 2) rv[i] = wanted ? *(const floatx4 *) (from + s_off[i]) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            else rs[i] = wanted ? from[s_off[i]] : 0.0f;
        }
    };
    auto fetch = [&](int c0) {
        const long long a_off = (long long) c0 * KH * KW, b_off = (long long) c0 * ohw;
        if (ANYW) {
            fetch_planes_any(c0);
            if (RAGGED) {
#pragma unroll
                for (int i = 0; i < A_ITERS; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        ra[i][j] = a_src[i] && a_off + a_k[i] + j < K ? (a_src[i] + a_off)[j] : 0.0f;
            } else {
#pragma unroll
                for (int i = 0; i < A_ITERS; i++)
                    ra[i] = a_src[i] ? *(const floatx4 *) (a_src[i] + a_off) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            }
            return;
        }
        if (RAGGED) {
#pragma unroll
            for (int i = 0; i < A_ITERS; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    ra[i][j] = a_src[i] && a_off + a_k[i] + j < K ? (a_src[i] + a_off)[j] : 0.0f;
#pragma unroll
            for (int i = 0; i < PLANE_MAX_VEC; i++)
                rb[i] = b_src[i] && c0 + b_channel[i] < C ? *(const floatx4 *) (b_src[i] + b_off) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            return;
        }
#pragma unroll
        for (int i = 0; i < A_ITERS; i++)
            ra[i] = a_src[i] ? *(const floatx4 *) (a_src[i] + a_off) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < PLANE_MAX_VEC; i++)
            rb[i] = b_src[i] ? *(const floatx4 *) (b_src[i] + b_off) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    };
    auto stage = [&]() {
        float *a_flat = &As[0][0];
#pragma unroll
        for (int i = 0; i < A_ITERS; i++)
            if ((BM * A_VEC) % THREADS == 0 || a_dst[i] >= 0) {
#pragma unroll
                for (int j = 0; j < 4; j++) a_flat[a_dst[i] + j * A_STRIDE] = ra[i][j];
            }
        if (ANYW) {
#pragma unroll
            for (int i = 0; i < ANY_SLOTS; i++)
                if (b_dst[i] >= 0) {
                    if constexpr (ANYW == 2) *(floatx4 *) &Bs[b_dst[i]] = rv[i];
                    else Bs[b_dst[i]] = rs[i];
                }
            return;
        }
#pragma unroll
        for (int i = 0; i < PLANE_MAX_VEC; i++)
            if (b_dst[i] >= 0) *(floatx4 *) &Bs[b_dst[i]] = rb[i];
    };

    floatx16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // a launch that splits the input channels: slice blockIdx.y takes its own range of them
    int c_begin = p.splits > 1 ? blockIdx.y * p.split_channels : 0;
    int c_end = p.splits > 1 ? min(C, c_begin + p.split_channels) : C;
    if (tail_part >= 0) {
        c_begin = tail_part * p.tail_channels;
        c_end = min(C, c_begin + p.tail_channels);
    }
    // the padding is never written again
    for (int i = t; i < PLANE_LDS; i += THREADS) Bs[i] = 0.0f;
    fetch(c_begin);
    for (int c0 = c_begin; c0 < c_end; c0 += CBK) {
        __syncthreads();
        stage();
        __syncthreads();
        if (c0 + CBK < c_end) fetch(c0 + CBK);
        // The operands of step kk + 2 are requested from LDS before the MFMAs of step kk are issued, and the wave
        // raises its priority while it issues MFMAs. Measured on this loop alone (no global loads, two waves per
        // SIMD): operands read right before their MFMAs and masked with selects 126 TFLOP/s, without the selects 140,
        // read one step ahead and with the priority 147, the bare MFMAs 155.
        float a_next[MI], b_next[NJ];
        auto read_operands = [&](int kk) {
            // taps of k = kk (lower half of the wave) and k = kk + 1 (upper half); all compile-time
            const int ca = kk / (KH * KW), fya = (kk / KW) % KH, fxa = kk % KW;
            const int cb = (kk + 1) / (KH * KW), fyb = ((kk + 1) / KW) % KH, fxb = (kk + 1) % KW;
            const int off_a = ca * gplane + fya * RS + fxa, off_b = cb * gplane + fyb * RS + fxb;
            const int koff = half ? off_b : off_a;
#pragma unroll
            for (int i = 0; i < MI; i++) a_next[i] = As[kk + half][wm * 32 * MI + 32 * i + c32];
#pragma unroll
            for (int j = 0; j < NJ; j++) b_next[j] = Bs[lane_base[j] + koff];
        };
        read_operands(0);
#pragma unroll
        for (int kk = 0; kk < KS; kk += 2) {
            float a[MI], b[NJ];
#pragma unroll
            for (int i = 0; i < MI; i++) a[i] = a_next[i];
#pragma unroll
            for (int j = 0; j < NJ; j++) b[j] = b_next[j];
            if (kk + 2 < KS) read_operands(kk + 2);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // Epilogue. Bias and residual are requested for a whole MFMA tile row at once (addresses clamped into the tensor
    // instead of branches around the loads), so their latencies overlap; only the stores are predicated.
    // (the partial results of a split launch get bias, residual and activation from the pass that sums them)
    const int part = tail_part >= 0 ? tail_part : (p.splits > 1 ? (int) blockIdx.y : -1);
    if (part >= 0 && p.counters) {
        // Summed inside the launch: every workgroup of a tile parks its partial tile, [part][wave][MFMA tile][register / 4]
        // [lane][register % 4], and counts itself in; the last one to arrive adds the parts up in their order and goes
        // on to the epilogue. The partial tiles travel between workgroups that may sit on different XCDs, each with an L2
        // of its own: they are written and read with device scope accesses, which go past those caches. What orders the
        // exchange: every wave waits for the acknowledgements of its own stores, the barrier collects the waves, and only
        // then one thread adds to the tile's counter; the workgroup that reads `parts - 1` there is behind all the others'
        // stores. It puts the counter back to zero for the next launch, which the stream orders behind this one.
        constexpr int SC1 = 16;  // auxiliary bits of the buffer instructions: device scope
        const int parts = tail_part >= 0 ? p.tail_parts : p.splits;
        const int shared_index = tail_part >= 0 ? tile_id - p.tail_head : tile_id;
        float *tile_slots = p.workspace + (size_t) shared_index * parts * (BM * TN);
        const __amdgpu_buffer_rsrc_t slots = __builtin_amdgcn_make_buffer_rsrc(tile_slots, 0, parts * (BM * TN) * 4, 0x00020000);
        const int thread_off = (wave * (MI * NJ * 16 * 64) + lane * 4) * 4;
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const floatx4 x = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, x), slots,
                                                           part * (BM * TN * 4) + thread_off + ((i * NJ + j) * 4 + q) * 1024, 0, SC1);
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // (also: every wave is done with the LDS operands)
        int *counter = p.counters + shared_index, *arrived = (int *) &As[0][0];
        if (threadIdx.x == 0) *arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*(volatile int *) arrived != parts - 1) return;
        // (the parts of a small tile are requested four at a time before the first is added: one round trip for four)
        constexpr int AHEAD = MI * NJ == 1 ? 4 : 1;
        for (int from0 = 0; from0 < parts; from0 += AHEAD) {
            floatx4 x[AHEAD][MI][NJ][4];
#pragma unroll
            for (int a = 0; a < AHEAD; a++)
#pragma unroll
                for (int i = 0; i < MI; i++)
#pragma unroll
                    for (int j = 0; j < NJ; j++)
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            // (parts past the last read the last one again; they are not added)
                            const int from = min(from0 + a, parts - 1);
                            x[a][i][j][q] = __builtin_bit_cast(
                                floatx4, __builtin_amdgcn_raw_buffer_load_b128(slots, from * (BM * TN * 4) + thread_off + ((i * NJ + j) * 4 + q) * 1024, 0, SC1));
                        }
#pragma unroll
            for (int a = 0; a < AHEAD; a++)
                if (from0 + a < parts) {
#pragma unroll
                    for (int i = 0; i < MI; i++)
#pragma unroll
                        for (int j = 0; j < NJ; j++)
#pragma unroll
                            for (int q = 0; q < 4; q++)
#pragma unroll
                                for (int u = 0; u < 4; u++)
                                    acc[i][j][4 * q + u] = from0 + a == 0 ? x[a][i][j][q][u] : acc[i][j][4 * q + u] + x[a][i][j][q][u];
                }
        }
        if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const bool to_scratch = part >= 0 && !p.counters;
    ConvStore s = to_scratch
        ? ConvStore{p.workspace + (long long) part * p.out_c * N, nullptr, nullptr, 0, p.out_c, ohw, N, 0, {0, 0}, {false, false}}
        : ConvStore{p.output, p.bias, p.res, p.bias_stride, p.out_c, ohw, N, p.relu, {0, 0}, {false, false}};
    const int col0 = n0 + wn * 32 * NJ + c32;
    s.prepare(col0, col0 + 32);
#pragma unroll
    for (int i = 0; i < MI; i++) {
        int row_off[16];  // inside one image: below 2^31 (checked on the host)
        float bias_v[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int row = m0 + wm * 32 * MI + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
            const int row_c = min(row, p.out_c - 1);
            row_off[v] = row_c * ohw;
            bias_v[v] = s.bias ? s.bias[row_c * s.bias_stride] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const long long base = s.col_ok[j] ? s.col_base[j] : 0ll;
            float res_v[16];
            if (s.res) {
#pragma unroll
                for (int v = 0; v < 16; v++) res_v[v] = s.res[base + row_off[v]];
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = m0 + wm * 32 * MI + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
                float x = acc[i][j][v];
                if (s.res) x += res_v[v];
                x += bias_v[v];
                if (s.relu) x = fmaxf(x, 0.0f);
                if (row < p.out_c && s.col_ok[j]) s.p[base + row_off[v]] = x;
            }
        }
    }
}

int log2_exact(int x) {
    int s = 0;
    while ((1 << s) < x) s++;
    return (1 << s) == x ? s : -1;
}

// Fills `g` and returns true when the plane kernel covers this convolution.
bool plane_geometry(const ConvParams &p, int tn, PlaneGeom *g) {
    const bool three = p.kernel_h == 3 && p.kernel_w == 3 && p.pad_y == 1 && p.pad_x == 1;
    const bool five = p.kernel_h == 5 && p.kernel_w == 5 && p.pad_y == 2 && p.pad_x == 2;
    if (!(three || five) || p.stride_y != 1 || p.stride_x != 1 || p.out_h != p.in_h || p.out_w != p.in_w) return false;
    const int cb = plane_slice_channels(p.kernel_h, p.kernel_w);
    // (5 x 5 with channels that do not fill their slices of four gathers faster: the 22 planes of a Go network's stem on
    // 19 x 19 -> 192 channels at batch 256 383 us here, 319 us on the patch kernel)
    if (five && p.in_c % cb != 0) return false;
    // (a channel count that is no multiple of the slice runs on the variant that reads the filter float by float)
    if (p.in_c <= 0 || (uintptr_t) p.input % 16 != 0 || (p.in_c % cb == 0 && (uintptr_t) p.filter % 16 != 0)) return false;
    const int W = p.in_w, H = p.in_h;
    if (W < 4 || W > tn || log2_exact(W) < 0) return false;
    const long long hw = (long long) H * W;
    if (hw >= tn) {
        if (hw % tn != 0) return false;
        g->rows = tn / W;
        g->groups = 1;
        g->tiles_per_image = (int) (hw / tn);
    } else {
        if (tn % hw != 0) return false;
        g->rows = H;
        g->groups = (int) (tn / hw);
        g->tiles_per_image = 0;
    }
    g->plane_rows = g->rows + p.kernel_h - 1;
    g->w4_shift = log2_exact(W / 4);
    g->g_shift = log2_exact(g->groups);
    g->rw_shift = log2_exact(g->rows * W);
    g->n_vec = cb * g->groups * g->plane_rows * W / 4;
    g->row_stride = W + PLANE_PAD;
    if (g->g_shift < 0 || g->rw_shift < 0 || g->n_vec > PLANE_MAX_VEC * THREADS) return false;
    if (cb * g->groups * g->plane_rows * g->row_stride + 2 * PLANE_SLACK > PLANE_LDS) return false;
    return true;
}

// The same for the variant that takes any image size (3 x 3 or 5 x 5, stride 1, same-size output): tiles of `tn`
// consecutive positions.
bool plane_geometry_any(const ConvParams &p, int tn, PlaneGeom *g) {
    const bool three = p.kernel_h == 3 && p.kernel_w == 3 && p.pad_y == 1 && p.pad_x == 1;
    const bool five = p.kernel_h == 5 && p.kernel_w == 5 && p.pad_y == 2 && p.pad_x == 2;
    if (!(three || five) || p.stride_y != 1 || p.stride_x != 1 || p.out_h != p.in_h || p.out_w != p.in_w) return false;
    const int cb = plane_slice_channels(p.kernel_h, p.kernel_w);
    if (five && p.in_c % cb != 0) return false;
    if (p.in_c <= 0 || (p.in_c % cb == 0 && (uintptr_t) p.filter % 16 != 0)) return false;
    const int W = p.in_w, H = p.in_h;
    if (W < 2 || H < 1 || (long long) p.batch * p.in_c * H * W >= (1ll << 31)) return false;
    // output rows that `tn` consecutive positions can touch, image boundaries between them, and the padded rows
    // from the one above the first to the one below the last
    const int touched = (tn - 2) / W + 2, crossings = (touched - 2) / H + 1;
    *g = PlaneGeom{};
    g->groups = 1;
    g->plane_rows = touched + 2 * p.pad_y * crossings + 2 * p.pad_y;
    g->row_stride = W + PLANE_PAD;
    g->n_scalar = cb * g->plane_rows * W;
    g->by4 = W % 4 == 0 && (uintptr_t) p.input % 16 == 0;
    if (g->n_scalar > (g->by4 ? 4 * PLANE_MAX_VEC4 : PLANE_MAX_SCALAR) * THREADS) return false;
    if (cb * g->plane_rows * g->row_stride + 2 * PLANE_SLACK > PLANE_LDS) return false;
    return true;
}

// Pick the widest loader an operand allows: `so` / `sk` are the strides of the outer and the K axis.
int pick_mode(const void *ptr, long long so, long long sk, long long batch_stride, int batch) {
    const bool aligned = ((uintptr_t) ptr % 16 == 0) && (batch <= 1 || batch_stride % 4 == 0);
    if (!aligned) return Scalar;
    if (so == 1 && sk % 4 == 0) return VecOuter;
    if (sk == 1 && so % 4 == 0) return VecK;
    return Scalar;
}

template <int A_MODE, int TI, int BK>
void launch_gemm_b(int b_mode, dim3 grid, hipStream_t stream, const GemmParams &p, int kc) {
    switch (b_mode) {
        case VecOuter: hipLaunchKernelGGL((gemm_f32_kernel<A_MODE, VecOuter, TI, BK>), grid, dim3(THREADS), 0, stream, p, kc); break;
        case VecK: hipLaunchKernelGGL((gemm_f32_kernel<A_MODE, VecK, TI, BK>), grid, dim3(THREADS), 0, stream, p, kc); break;
        default: hipLaunchKernelGGL((gemm_f32_kernel<A_MODE, Scalar, TI, BK>), grid, dim3(THREADS), 0, stream, p, kc); break;
    }
}

template <int TI, int BK>
void launch_gemm_a(int a_mode, int b_mode, dim3 grid, hipStream_t stream, const GemmParams &p, int kc) {
    switch (a_mode) {
        case VecOuter: launch_gemm_b<VecOuter, TI, BK>(b_mode, grid, stream, p, kc); break;
        case VecK: launch_gemm_b<VecK, TI, BK>(b_mode, grid, stream, p, kc); break;
        default: launch_gemm_b<Scalar, TI, BK>(b_mode, grid, stream, p, kc); break;
    }
}

// Sums the split-K partial products [batch][split][m][n] (f32, dense) into C and applies the epilogue. VEC = 4:
// every thread owns four neighbouring columns (n a multiple of 4, C and the addend contiguous or broadcast along n).
template <typename OutT, int VEC>
__global__ __launch_bounds__(256) void gemm_reduce_partials_kernel(GemmParams p, int split) {
    const long long mn = (long long) p.m * p.n;
    const long long e = ((long long) blockIdx.x * 256 + threadIdx.x) * VEC;
    if (e >= mn) return;
    const int bz = blockIdx.y;
    const float *part = (const float *) p.workspace + (long long) bz * split * mn + e;
    float total[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) total[j] = 0.0f;
    if (VEC == 4) {
        // four parts requested at a time (the order of the sum stays that of K)
        int s = 0;
        for (; s + 4 <= split; s += 4) {
            floatx4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = *(const floatx4 *) (part + (s + u) * mn);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int j = 0; j < VEC; j++) total[j] += v[u][j];
        }
        for (; s < split; s++) {
            const floatx4 v = *(const floatx4 *) (part + s * mn);
#pragma unroll
            for (int j = 0; j < VEC; j++) total[j] += v[j];
        }
    } else {
        for (int s = 0; s < split; s++) total[0] += part[s * mn];
    }
    const long long row = e / p.n, col = e - row * p.n;
    OutT *out = (OutT *) p.c + bz * p.c_sb + row * p.c_sm + col * p.c_sn;
    const OutT *addend = p.addend ? (const OutT *) p.addend + bz * p.d_sb + row * p.d_sm + col * p.d_sn : nullptr;
    const OutT *addend2 = p.addend2 ? (const OutT *) p.addend2 + bz * p.d2_sb + row * p.d2_sm + col * p.d2_sn : nullptr;
    // (the addends are requested before the first store: a load may not pass a store that might alias it)
    OutT d[VEC], d2[VEC];
    typedef OutT OutVec __attribute__((ext_vector_type(VEC)));
    // contiguous, aligned columns move as one vector
    auto as_vector = [](const OutT *ptr, long long stride) { return VEC > 1 && stride == 1 && (uintptr_t) ptr % (VEC * sizeof(OutT)) == 0; };
    if (addend && as_vector(addend, p.d_sn)) {
        const OutVec v = *(const OutVec *) addend;
#pragma unroll
        for (int j = 0; j < VEC; j++) d[j] = v[j];
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) d[j] = addend ? addend[j * p.d_sn] : (OutT) 0;
    }
    if (addend2 && as_vector(addend2, p.d2_sn)) {
        const OutVec v = *(const OutVec *) addend2;
#pragma unroll
        for (int j = 0; j < VEC; j++) d2[j] = v[j];
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) d2[j] = addend2 ? addend2[j * p.d2_sn] : (OutT) 0;
    }
    OutVec result;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        // rounding to the output type after the product and after the sum, like separate operations would
        float v = (float) (OutT) total[j];
        if (addend) v = (float) (OutT) (v + (float) d[j]);
        if (addend2) v = (float) (OutT) (v + (float) d2[j]);
        if (p.relu) v = fmaxf(v, 0.0f);
        result[j] = (OutT) v;
    }
    if (as_vector(out, p.c_sn)) {
        *(OutVec *) out = result;
    } else {
#pragma unroll
        for (int j = 0; j < VEC; j++) out[j * p.c_sn] = result[j];
    }
}

template <int KH, int KW, int TI>
void launch_conv_k(int a_mode, dim3 grid, hipStream_t stream, const ConvParams &p) {
    if (a_mode == VecK) hipLaunchKernelGGL((conv_f32_kernel<VecK, KH, KW, TI>), grid, dim3(THREADS), 0, stream, p);
    else hipLaunchKernelGGL((conv_f32_kernel<Scalar, KH, KW, TI>), grid, dim3(THREADS), 0, stream, p);
}

template <int TI>
void launch_conv_t(int a_mode, dim3 grid, hipStream_t stream, const ConvParams &p) {
    if (p.kernel_h == 3 && p.kernel_w == 3) launch_conv_k<3, 3, TI>(a_mode, grid, stream, p);
    else if (p.kernel_h == 1 && p.kernel_w == 1) launch_conv_k<1, 1, TI>(a_mode, grid, stream, p);
    else if (p.kernel_h == 5 && p.kernel_w == 5) launch_conv_k<5, 5, TI>(a_mode, grid, stream, p);
    else if (p.kernel_h == 7 && p.kernel_w == 7) launch_conv_k<7, 7, TI>(a_mode, grid, stream, p);
    else launch_conv_k<0, 0, TI>(a_mode, grid, stream, p);
}

// convolutions: 128 x 128 tiles unless there are too few of them to give every compute unit two workgroups
int small_tile_threshold() { return 512; }

}  // namespace

__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned *p, size_t words) {
    const size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
    if (i < words) p[i] = 0u;
}

int launch_fill_zero(void *ptr, size_t bytes, ihipStream_t *stream) {
    if (bytes == 0) return 0;
    if (bytes % 4 != 0 || (uintptr_t) ptr % 4 != 0 || bytes / 4 > 0x7fffffffull * 256) return (int) hipErrorInvalidValue;
    const size_t words = bytes / 4;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned) ((words + 255) / 256)), dim3(256), 0, stream, (unsigned *) ptr, words);
    return (int) hipGetLastError();
}

int launch_gemm_reduce_partials(const GemmParams &p, int split, bool f16, ihipStream_t *stream) {
    const long long mn = (long long) p.m * p.n;
    const bool vec = p.n % 4 == 0 && p.c_sn == 1 && (uintptr_t) p.workspace % 16 == 0;
    const long long threads = vec ? mn / 4 : mn;
    dim3 grid((unsigned) ((threads + 255) / 256), (unsigned) p.batch, 1);
    if (f16 && vec) hipLaunchKernelGGL((gemm_reduce_partials_kernel<_Float16, 4>), grid, dim3(256), 0, stream, p, split);
    else if (f16) hipLaunchKernelGGL((gemm_reduce_partials_kernel<_Float16, 1>), grid, dim3(256), 0, stream, p, split);
    else if (vec) hipLaunchKernelGGL((gemm_reduce_partials_kernel<float, 4>), grid, dim3(256), 0, stream, p, split);
    else hipLaunchKernelGGL((gemm_reduce_partials_kernel<float, 1>), grid, dim3(256), 0, stream, p, split);
    return (int) hipGetLastError();
}

// Tiny products: one wave per result element, lanes along K, a butterfly over the lanes, and the epilogue of the tiled
// kernels (f16: the product, and each sum with an addend, rounded to f16 like separate operations would round them).
template <typename T>
__global__ __launch_bounds__(256) void gemm_dot_kernel(GemmParams p) {
    const long long result = ((long long) blockIdx.x * 256 + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (result >= (long long) p.batch * p.m * p.n) return;  // (a whole wave at a time)
    const int col = (int) (result % p.n), row = (int) (result / p.n % p.m), bz = (int) (result / p.n / p.m);
    const T *a = (const T *) p.a + bz * p.a_sb + (long long) row * p.a_sm;
    const T *b = (const T *) p.b + bz * p.b_sb + (long long) col * p.b_sn;
    float acc = 0.0f;
    for (int k = lane; k < p.k; k += 64) acc += (float) a[(long long) k * p.a_sk] * (float) b[(long long) k * p.b_sk];
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) acc += __shfl_xor(acc, m, 64);
    if (lane != 0) return;
    T r = (T) acc;
    if (p.addend) r = (T) ((float) r + (float) ((const T *) p.addend)[bz * p.d_sb + (long long) row * p.d_sm + (long long) col * p.d_sn]);
    if (p.addend2) r = (T) ((float) r + (float) ((const T *) p.addend2)[bz * p.d2_sb + (long long) row * p.d2_sm + (long long) col * p.d2_sn]);
    if (p.relu) r = r > (T) 0 ? r : (T) 0;
    ((T *) p.c)[bz * p.c_sb + (long long) row * p.c_sm + (long long) col * p.c_sn] = r;
}

int launch_gemm_dot(const GemmLaunchPlan &lp, bool f16, ihipStream_t *stream) {
    const GemmParams &p = lp.p;
    if (p.addend2 != nullptr && p.addend == nullptr) return (int) hipErrorInvalidValue;
    const long long results = (long long) p.batch * p.m * p.n;
    const dim3 grid((unsigned) ((results * 64 + 255) / 256)), block(256);
    if (f16) hipLaunchKernelGGL((gemm_dot_kernel<_Float16>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_dot_kernel<float>), grid, block, 0, stream, p);
    return (int) hipGetLastError();
}

int launch_gemm_f32(const GemmLaunchPlan &lp, ihipStream_t *stream) {
    const GemmParams &p = lp.p;
    if (p.batch <= 0 || p.m <= 0 || p.n <= 0) return 0;
    if (lp.dot) return launch_gemm_dot(lp, false, stream);
    const int t = lp.small_tile ? 64 : 128;
    const int groups = p.groups > 1 ? p.groups : 1;
    if (groups > GEMM_MAX_GROUPS || (groups > 1 && (lp.split_k > 1 || p.addend || lp.swapped))) return (int) hipErrorInvalidValue;
    if (p.addend2 != nullptr && p.addend == nullptr) return (int) hipErrorInvalidValue;
    const long long tiles = (long long) ((p.m + t - 1) / t) * ((p.n + t - 1) / t) * groups;
    if (tiles > 0x7fffffffll || p.batch > 65535 || (long long) p.m * p.n > 0x7fffffffll * 256) return (int) hipErrorInvalidConfiguration;
    if (lp.split_k > 1 && p.workspace == nullptr) return (int) hipErrorInvalidValue;
    dim3 grid((unsigned) tiles, (unsigned) p.batch, (unsigned) lp.split_k);
    const int a_mode = pick_mode(p.a, p.a_sm, p.a_sk, p.a_sb, p.batch);
    int b_mode = pick_mode(groups > 1 ? p.b_group[0] : p.b, p.b_sn, p.b_sk, p.b_sb, p.batch);
    for (int g = 1; g < groups; g++) {  // the loader that every operand of the group allows
        const int mode = pick_mode(p.b_group[g], p.b_sn, p.b_sk, p.b_sb, p.batch);
        if (mode != b_mode) b_mode = Scalar;
    }
    bool direct = false;
    int e = launch_gemm_f32_direct(lp, stream, &direct);
    if (e != 0) return e;
    if (direct) {
    } else if (lp.small_tile && lp.bk == 64) launch_gemm_a<1, 64>(a_mode, b_mode, grid, stream, p, lp.k_chunk);
    else if (lp.small_tile) launch_gemm_a<1, 16>(a_mode, b_mode, grid, stream, p, lp.k_chunk);
    else launch_gemm_a<2, 16>(a_mode, b_mode, grid, stream, p, lp.k_chunk);
    e = (int) hipGetLastError();
    if (e == 0 && lp.split_k > 1) e = launch_gemm_reduce_partials(p, lp.split_k, false, stream);
    return e;
}

// Sums the partial results [split][image][channel][position] of a convolution that split its input channels and applies
// residual, bias and activation in the order the unsplit store does. VEC = 4: every thread owns four neighbouring
// positions (out_h * out_w a multiple of 4).
template <int VEC>
__global__ __launch_bounds__(256) void conv_reduce_partials_kernel(ConvParams p) {
    const long long ohw = (long long) p.out_h * p.out_w, total = (long long) p.batch * p.out_c * ohw;
    const long long e = ((long long) blockIdx.x * 256 + threadIdx.x) * VEC;
    if (e >= total) return;
    typedef float Vec __attribute__((ext_vector_type(VEC)));
    Vec parts[4], sum;
    for (int j = 0; j < VEC; j++) sum[j] = 0.0f;
    for (int s0 = 0; s0 < p.splits; s0 += 4) {  // four requests in flight, added in the order of the slices
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (s0 + i < p.splits) parts[i] = *(const Vec *) (p.workspace + (long long) (s0 + i) * total + e);
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (s0 + i < p.splits) sum += parts[i];
    }
    const int channel = (int) ((e / ohw) % p.out_c);
    if (p.res) sum += *(const Vec *) (p.res + e);
    if (p.bias) {
        const float b = p.bias[channel * p.bias_stride];
        for (int j = 0; j < VEC; j++) sum[j] += b;
    }
    if (p.relu)
        for (int j = 0; j < VEC; j++) sum[j] = fmaxf(sum[j], 0.0f);
    *(Vec *) (p.output + e) = sum;
}

// Sums the partial tiles of the shared tiles of a launch with a tail split (tiles from `tail_head` on; the partial
// results lie where a launch that splits all of its tiles would put them, [part][image][channel][position]) and
// applies residual, bias and activation in the order the unsplit store does. One workgroup per 64 positions of a
// tile (blockIdx.y: the second half of a tile of 128); VEC neighbouring positions per thread (out_h * out_w a
// multiple of VEC).
template <int VEC>
__global__ __launch_bounds__(256) void conv_sum_tail_kernel(ConvParams p) {
    const long long ohw = (long long) p.out_h * p.out_w, N = (long long) p.batch * ohw, total = N * p.out_c;
    const int tile = p.tail_tile;
    const int tiles_m = (p.out_c + tile - 1) / tile, tiles_n = (int) ((N + tile - 1) / tile);
    int tm, tn;
    tile_of_id(p.tail_head + (int) blockIdx.x, tiles_m, tiles_n, &tm, &tn);
    typedef float Vec __attribute__((ext_vector_type(VEC)));
    constexpr int COLS = 64 / VEC, ROWS = 256 / COLS;  // threads along the positions, channels per pass
    const int col = (threadIdx.x % COLS) * VEC, row0 = threadIdx.x / COLS;
    const long long pos = (long long) tn * tile + 64 * blockIdx.y + col;
    if (pos >= N) return;
    const long long img = pos / ohw, within = pos - img * ohw;
    for (int row = row0; row < tile; row += ROWS) {
        const int channel = tm * tile + row;
        if (channel >= p.out_c) break;
        const long long e = (img * p.out_c + channel) * ohw + within;
        Vec sum = *(const Vec *) (p.workspace + e);
        for (int part = 1; part < p.tail_parts; part++) sum += *(const Vec *) (p.workspace + (long long) part * total + e);
        if (p.res) sum += *(const Vec *) (p.res + e);
        if (p.bias) {
            const float b = p.bias[channel * p.bias_stride];
            for (int j = 0; j < VEC; j++) sum[j] += b;
        }
        if (p.relu)
            for (int j = 0; j < VEC; j++) sum[j] = fmaxf(sum[j], 0.0f);
        *(Vec *) (p.output + e) = sum;
    }
}

int conv_channel_split(const ConvParams &p) {
    const bool enabled = p.channel_split;
    const long long positions = (long long) p.batch * p.out_h * p.out_w;
    if (!enabled || positions <= 0 || p.out_c <= 0) return 1;
    // 64 x 64 tiles of four waves each, on 1024 SIMDs. The plane kernel keeps a SIMD busy with one wave, so it splits
    // while half of the SIMDs would be idle; the patch kernel waits for its gathers and gains up to three waves per
    // SIMD. Measured (us, unsplit -> split), 128 -> 128 channels on 8 x 8 boards: batch 16 28.9 -> 13.6, 32 -> 16.3,
    // 64 29.4 -> 22.6; 192 -> 192 on 19 x 19: batch 1 -> 18.5, batch 8 120 -> 54..61. Only K loops of 512 steps or
    // more are split, into slices of 16 channels or more, up to 16 of them.
    const long long tiles = ((positions + 63) / 64) * ((p.out_c + 63) / 64);
    const long long k = (long long) p.in_c * p.kernel_h * p.kernel_w;
    ConvParams shape_only = p;
    shape_only.input = shape_only.filter = nullptr;
    PlaneGeom geom;
    const long long target = plane_geometry(shape_only, 64, &geom) || plane_geometry_any(shape_only, 64, &geom) ? 1024 : 3072;
    // (the plane kernel also takes two parts when every compute unit has a tile but none has two: the ResNet tower at
    // batch 128, 256 tiles, 709 -> 687 us per evaluation with the parts summed inside the launch)
    const bool plane = target == 1024;
    if ((plane ? tiles * 4 > target : tiles * 4 * 2 > target) || k < 512) return 1;
    const long long most = std::min<long long>({16, std::max<long long>(plane ? 2 : 1, target / (tiles * 4)), p.in_c / 16});
    if (most < 2) return 1;
    // whole slices of CB channels per split, and no split without channels
    const int slices = (p.in_c + CB - 1) / CB;
    const int per_split = (int) ((slices + most - 1) / most);
    return (slices + per_split - 1) / per_split;
}

long long conv_tail_split(const ConvParams &p, int *parts, int *tile) {
    *parts = 1;
    if (tile) *tile = 64;
    const long long positions = (long long) p.batch * p.out_h * p.out_w;
    if (!p.channel_split || positions <= 0 || p.out_c <= 0 || p.kernel_h != 3 || conv_channel_split(p) > 1) return 0;
    ConvParams shape_only = p;
    shape_only.input = shape_only.filter = nullptr;
    PlaneGeom geom;
    if (!plane_geometry(shape_only, 64, &geom) && !(p.plane_any_width && plane_geometry_any(shape_only, 64, &geom))) return 0;
    // which tiles the launch picks (the same estimate as in launch_conv_f32)
    const long long small = ((positions + 63) / 64) * ((p.out_c + 63) / 64), big = ((positions + 127) / 128) * ((p.out_c + 127) / 128);
    const bool big_fits = plane_geometry(shape_only, 128, &geom) || (p.plane_any_width && plane_geometry_any(shape_only, 128, &geom));
    const bool big_wins = big_fits && (double) ((big * 4 + 1023) / 1024) * 4.0 * (big < 256 ? 1.2 : 1.0) <= (double) ((small * 4 + 1023) / 1024) * 1.1;
    const long long tiles = big_wins ? big : small, slices = (p.in_c + CB - 1) / CB;
    if (tile) *tile = big_wins ? 128 : 64;
    if (tiles > 0x7fffffffll / 8 || slices < 8) return tiles;
    // Tiles of 64 x 64: whole rounds of one tile per compute unit stay whole. Measured on 2 x 64 x 64 images, 320 input
    // channels (us by output channels): 256 112, 320 153, 384 154 - a compute unit with three tiles takes as long as if
    // all had three. Tiles of 128 x 128: a compute unit holds two, and what a round of 512 leaves over runs as a round
    // of its own (the tower convolution of a board game network, us per evaluation of 21 of them by batch size:
    // 1024 3487, 1536 6601, 2048 6912).
    const long long round = big_wins ? 512 : 256, rest = tiles % round;
    // (tiles of 128 x 128, one per compute unit or fewer: all in two parts, so that a compute unit has two workgroups
    // to overlap)
    if (big_wins && tiles >= 128 && tiles <= 256 && slices >= 8) {
        *parts = 2;
        return 0;
    }
    if (tiles < round || rest < round / 16 || rest > round / 2) return tiles;
    const long long most = std::min<long long>({4, round / rest, slices / 4});
    if (most < 2) return tiles;
    const long long per_part = (slices + most - 1) / most;
    *parts = (int) ((slices + per_part - 1) / per_part);
    return tiles - rest;
}

namespace {
// whether the kernel that keeps raw planes in LDS takes this convolution on tiles of 64 x 64 (shapes only)
bool plane_kernel_small_tiles(const ConvParams &p) {
    ConvParams shape_only = p;
    shape_only.input = shape_only.filter = nullptr;
    PlaneGeom geom;
    return plane_geometry(shape_only, 64, &geom) || (p.plane_any_width && plane_geometry_any(shape_only, 64, &geom));
}
}  // namespace

size_t conv_counter_bytes(const ConvParams &p) {
    const long long positions = (long long) p.batch * p.out_h * p.out_w;
    if (positions <= 0 || p.out_c <= 0) return 0;
    // A split of all tiles: only the plane kernel (on tiles of 64 x 64 then) sums inside the launch, and only up to four
    // parts: the last workgroup of a tile reads the parts one after the other, which with eight of them takes longer
    // than the second kernel (the ResNet tower, us per evaluation with the second kernel / summed inside: batch 1
    // 291 / 306, 8 316 / 343 with eight parts; 32 400 / 387 with four, 64 527 / 488 with two).
    if (const int splits = conv_channel_split(p); splits > 1)
        return splits <= 4 && plane_kernel_small_tiles(p) ? (size_t) (((positions + 63) / 64) * ((p.out_c + 63) / 64)) * sizeof(int) : 0;
    int parts = 1, tile = 64;
    const long long head = conv_tail_split(p, &parts, &tile);
    if (parts <= 1) return 0;
    return (size_t) (((positions + tile - 1) / tile) * ((p.out_c + tile - 1) / tile) - head) * sizeof(int);
}

size_t conv_workspace_bytes(const ConvParams &p) {
    const int splits = conv_channel_split(p);
    int tail_parts = 1;
    if (splits <= 1) conv_tail_split(p, &tail_parts);
    const int most = std::max(splits, tail_parts);
    if (most <= 1) return 0;
    // [part][image][channel][position] for the kernel that sums the parts; whole tiles per part and tile where the parts
    // are summed inside the launch
    const size_t plain = (size_t) most * p.batch * p.out_c * p.out_h * p.out_w * sizeof(float);
    int tile = 64;
    if (splits <= 1) conv_tail_split(p, &tail_parts, &tile);
    const size_t slots = conv_counter_bytes(p) / sizeof(int) * (size_t) most * tile * tile * sizeof(float);
    return std::max(plain, slots);
}

int launch_conv_f32(const ConvParams &params, ihipStream_t *stream) {
    ConvParams p = params;
    const long long positions = (long long) p.batch * p.out_h * p.out_w;
    if (positions <= 0 || p.out_c <= 0) return 0;
    p.splits = conv_channel_split(p);
    if (p.splits > 1) {
        if (!p.workspace) return (int) hipErrorInvalidValue;
        const int slices = (p.in_c + CB - 1) / CB;
        p.split_channels = (slices + p.splits - 1) / p.splits * CB;
    }
    const bool split = p.splits > 1;
    bool plane_sums_inside = false;
    auto sum_slices = [&]() {
        if (!split || plane_sums_inside) return (int) hipGetLastError();
        const long long total = (long long) p.batch * p.out_c * p.out_h * p.out_w;
        const bool vec = (p.out_h * p.out_w) % 4 == 0 && (uintptr_t) p.output % 16 == 0 && (!p.res || (uintptr_t) p.res % 16 == 0);
        const long long threads = vec ? total / 4 : total;
        const dim3 grid((unsigned) ((threads + 255) / 256)), block(256);
        if (vec) hipLaunchKernelGGL((conv_reduce_partials_kernel<4>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((conv_reduce_partials_kernel<1>), grid, block, 0, stream, p);
        return (int) hipGetLastError();
    };
    const long long big_tiles = ((positions + BN - 1) / BN) * ((p.out_c + BM - 1) / BM);
    if (positions > 0x7fffffffll || big_tiles > 0x7fffffffll / 4) return (int) hipErrorInvalidValue;
    if ((long long) p.out_c * p.out_h * p.out_w > 0x7fffffffll || (long long) p.in_c * p.in_h * p.in_w > 0x7fffffffll) return (int) hipErrorInvalidValue;
    // Plane kernel tiles (output channels x positions): 128 x 128 or 64 x 64, each wave owning 4 or 1 MFMA tiles of
    // the result. The waves of all workgroups spread over 1024 SIMDs and the launch takes about as long as the
    // busiest SIMD: rounds of waves x MFMA tiles per wave. The small tile costs a tenth more per MFMA tile (more LDS
    // reads and staged planes per flop) but rounds the work off better; the smaller estimate wins. Measured (us,
    // 128 x 128 / 64 x 64): 128 -> 128 channels on 8 x 8 images, batch 64 89 / 34, 256 94 / 55, 384 98 / 78,
    // 512 102 / 108, 768 176 / 156, 1024 189 / 206; 320 -> 320 on 2 x 64 x 64 228 / 183; 1280 -> 1280 on
    // 2 x 16 x 16 818 / 291. (128 x 64 tiles never won against both.)
    PlaneGeom geom;
    struct Variant { int bm, tn, id; double unit_cost; };
    static const Variant variants[2] = {{128, 128, 22, 4 * 1.00}, {64, 64, 11, 1 * 1.10}};
    const Variant *best = nullptr;
    double best_cost = 0.0;
    const bool any_enabled = p.plane_any_width;
    bool any_w = false;
    for (const Variant &v : variants) {
        if (split && v.id != 11) continue;  // (few tiles: the small one)
        // (5 x 5: 100 filter rows per slice for 128 channels leave LDS for one workgroup per compute unit; 64 x 64 tiles
        // run 101 TFLOP/s where 128 x 128 run 94, on 128 -> 128 channels at 32 x 32, 16 x 16 and 8 x 8 alike)
        if (p.kernel_h == 5 && v.id != 11) continue;
        const bool classic = plane_geometry(p, v.tn, &geom);
        if (!classic && !(any_enabled && plane_geometry_any(p, v.tn, &geom))) continue;
        const long long tiles = ((positions + v.tn - 1) / v.tn) * ((p.out_c + v.bm - 1) / v.bm);
        // (fewer big tiles than compute units: some of those idle, the others with a single workgroup that has nobody to
        // overlap its waits with; a fifth dearer. The ResNet tower at batch 448, us: 2110 on 224 big tiles, 1952 on 896
        // small ones, the last 128 of them shared)
        const double cost = (double) ((tiles * 4 + 1023) / 1024) * v.unit_cost * (v.id == 22 && tiles < 256 ? 1.2 : 1.0);
        if (!best || cost < best_cost) { best = &v; best_cost = cost; any_w = !classic; }
    }
    // a sparse last round of 64 x 64 tiles: its tiles shared by workgroups that take a slice of the input channels each
    long long tail_tiles = 0;
    if (best && !split && p.workspace) {
        int parts = 1, tile = 64;
        const long long head = conv_tail_split(params, &parts, &tile);
        // (only if the launch picked the tiles the plan was made for)
        if (parts > 1 && tile == best->tn) {
            const int slices = (p.in_c + CB - 1) / CB;
            p.tail_head = (int) head;
            p.tail_parts = parts;
            p.tail_channels = (slices + parts - 1) / parts * CB;
            p.tail_tile = tile;
            tail_tiles = ((positions + tile - 1) / tile) * ((p.out_c + tile - 1) / tile) - head;
        }
    }
    // (the plane kernel sums inside the launch when it has counters; the patch kernel never does)
    const bool sums_inside = best != nullptr && p.counters != nullptr;
    if (!best) p.counters = nullptr;
    plane_sums_inside = sums_inside;
    auto sum_tail = [&]() {
        if (tail_tiles == 0 || sums_inside) return (int) hipGetLastError();
        const bool vec = (p.out_h * p.out_w) % 4 == 0 && (uintptr_t) p.output % 16 == 0 && (uintptr_t) p.workspace % 16 == 0 &&
                         (!p.res || (uintptr_t) p.res % 16 == 0);
        const dim3 tail_grid((unsigned) tail_tiles, (unsigned) (p.tail_tile / 64));
        if (vec) hipLaunchKernelGGL((conv_sum_tail_kernel<4>), tail_grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((conv_sum_tail_kernel<1>), tail_grid, dim3(256), 0, stream, p);
        return (int) hipGetLastError();
    };
    if (best && any_w) {
        plane_geometry_any(p, best->tn, &geom);
        const long long tiles = ((positions + best->tn - 1) / best->tn) * ((p.out_c + best->bm - 1) / best->bm);
        const dim3 grid((unsigned) (tiles + tail_tiles * (p.tail_parts - 1)), (unsigned) p.splits), block(THREADS);
        const bool ragged = p.in_c % plane_slice_channels(p.kernel_h, p.kernel_w) != 0;
        const bool by4 = geom.by4 != 0;
        if (p.kernel_h == 5) {
            if (by4) hipLaunchKernelGGL((conv_plane_kernel<5, 5, 1, 1, false, 2>), grid, block, 0, stream, p, geom);
            else hipLaunchKernelGGL((conv_plane_kernel<5, 5, 1, 1, false, 1>), grid, block, 0, stream, p, geom);
            return sum_slices();
        }
        if (best->id == 22 && ragged && by4) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, true, 2>), grid, block, 0, stream, p, geom);
        else if (best->id == 22 && ragged) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, true, 1>), grid, block, 0, stream, p, geom);
        else if (best->id == 22 && by4) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, false, 2>), grid, block, 0, stream, p, geom);
        else if (best->id == 22) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, false, 1>), grid, block, 0, stream, p, geom);
        else if (ragged && by4) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, true, 2>), grid, block, 0, stream, p, geom);
        else if (ragged) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, true, 1>), grid, block, 0, stream, p, geom);
        else if (by4) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, false, 2>), grid, block, 0, stream, p, geom);
        else hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, false, 1>), grid, block, 0, stream, p, geom);
        return tail_tiles ? sum_tail() : sum_slices();
    }
    if (best) {
        plane_geometry(p, best->tn, &geom);
        const long long tiles = ((positions + best->tn - 1) / best->tn) * ((p.out_c + best->bm - 1) / best->bm);
        const dim3 grid((unsigned) (tiles + tail_tiles * (p.tail_parts - 1)), (unsigned) p.splits), block(THREADS);
        const bool ragged = p.in_c % plane_slice_channels(p.kernel_h, p.kernel_w) != 0;
        if (p.kernel_h == 5) {
            hipLaunchKernelGGL((conv_plane_kernel<5, 5, 1, 1, false>), grid, block, 0, stream, p, geom);
            return sum_slices();
        }
        if (best->id == 22 && ragged) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, true>), grid, block, 0, stream, p, geom);
        else if (best->id == 22) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 2, 2, false>), grid, block, 0, stream, p, geom);
        else if (ragged) hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, true>), grid, block, 0, stream, p, geom);
        else hipLaunchKernelGGL((conv_plane_kernel<3, 3, 1, 1, false>), grid, block, 0, stream, p, geom);
        return tail_tiles ? sum_tail() : sum_slices();
    }
    const long long K = (long long) p.in_c * p.kernel_h * p.kernel_w;
    const int a_mode = ((uintptr_t) p.filter % 16 == 0 && K % 4 == 0) ? VecK : Scalar;
    // the same estimate for the patch kernel: rounds of waves on 1024 SIMDs x MFMA tiles per wave (64 output channels on
    // 128 x 128 tiles would leave half of every tile empty)
    const long long small_tiles = ((positions + 63) / 64) * ((p.out_c + 63) / 64);
    const double big_cost = (double) ((big_tiles * 4 + 1023) / 1024) * 4.0, small_cost = (double) ((small_tiles * 4 + 1023) / 1024) * 1.1;
    if (split || big_tiles < small_tile_threshold() || small_cost < big_cost) {
        const long long tiles = small_tiles;
        launch_conv_t<1>(a_mode, dim3((unsigned) tiles, (unsigned) p.splits), stream, p);
    } else {
        launch_conv_t<2>(a_mode, dim3((unsigned) big_tiles), stream, p);
    }
    return sum_slices();
}

}  // namespace kn
