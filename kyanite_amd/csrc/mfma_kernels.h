// Host-side interface of the ahead-of-time compiled MFMA kernels (batched matrix multiply and fused convolution).
// They replace the library calls of the reference: cublasSgemm[StridedBatched] (kn-cuda-sys/src/wrapper/group.rs:107-171)
// and cudnnConvolutionBiasActivationForward (kn-cuda-sys/src/wrapper/operation.rs:157-240).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

struct ihipStream_t;

namespace kn {

// C[b, i, j] = sum_k A[b, i, k] * B[b, k, j]; element strides are arbitrary (zero batch stride = broadcast operand).
// The element type (float or _Float16, the same for all three matrices) is fixed by the launch function.
constexpr int GEMM_MAX_GROUPS = 4;

// Launch paths a caller may switch off (all on by default); part of the parameters, so that the plan made ahead of
// time and the launch see the same choice.
struct GemmTuning {
    bool direct = true;        // the kernels that load global -> LDS directly (off: every product stages through registers)
    bool split_k = true;       // workgroups that share a tile along K, of either kind
    bool tail_split = true;    // the split of just the last, sparse round of tiles inside one launch
    bool dot_products = true;  // one wave per result for products of up to 2^20 multiplications
    // The right operand is a weight that every evaluation reads once, out of more weights than the caches hold: the
    // direct kernel loads it with the non-temporal hint, so that its lines do not push the left operand's out. Measured:
    // a stand-alone stream with the matmul's access pattern 91 -> 87 us; the 512 token LLaMA decoder 564.4 -> 559.9 us
    // per step (alternating on one GPU); weights that do fit the last-level cache (a loop over one product) 5 to 15 %
    // SLOWER with it, 4096^3 4 % slower. Set by the planner from the size of the plan's constants and the rows of the
    // left operand.
    bool stream_b = false;
};

struct GemmParams {
    const void *a;
    const void *b;
    void *c;
    int batch, m, n, k;
    long long a_sb, a_sm, a_sk;
    long long b_sb, b_sk, b_sn;
    long long c_sb, c_sm, c_sn;
    // optional epilogue: C = act(A * B + D) with D addressed by element strides like C (zero = broadcast) and
    // act = max(., 0) when `relu` is set; for f16 the product and the sum are each rounded to f16, like separate
    // operations would
    const void *addend = nullptr;
    long long d_sb = 0, d_sm = 0, d_sn = 0;
    // a second operand of the same kind, added after the first (bias, then residual): C = act((A * B + D) + D2),
    // for f16 with a rounding after either sum; only together with `addend`
    const void *addend2 = nullptr;
    long long d2_sb = 0, d2_sm = 0, d2_sn = 0;
    int relu = 0;
    // Grouped launch: `groups` (up to GEMM_MAX_GROUPS) products A * B_g = C_g that share A, all shapes and all
    // strides, in one launch; b / c are then ignored in favour of b_group / c_group. Not combined with an addend
    // or a split of the K axis.
    int groups = 1;
    const void *b_group[4] = {nullptr, nullptr, nullptr, nullptr};
    void *c_group[4] = {nullptr, nullptr, nullptr, nullptr};
    // f32 scratch for partial products when the launch splits the K axis (`GemmLaunchPlan::workspace_bytes`
    // bytes, 256 byte aligned); may be null otherwise
    void *workspace = nullptr;
    // zero-filled ints that the launch hands back zero-filled (`GemmLaunchPlan::counter_bytes` bytes) when tiles
    // are shared between workgroups; may be null otherwise
    void *counters = nullptr;
    GemmTuning tuning;
    // Gated pair (f16, the kernel that loads global -> LDS directly, no groups, no addend, no split of K):
    // C = (G * sigmoid(G)) * U with G = A * B and U = A * B_pair, each product, the sigmoid and each multiplication
    // rounded to f16 like separate operations would. `n` counts VIRTUAL columns, two per column of C: the block of 32
    // virtual columns t holds the columns 16 t .. 16 t + 15 of G in its first half and those of U in its second, so
    // that the two factors of an element of C sit in one MFMA tile, 16 lanes apart. c_sm / c_sn address C itself
    // ([m, n / 2]); b_sn / b_sk address B and B_pair alike.
    int pair_op = 0;
    const void *b_pair = nullptr;
};
constexpr int GEMM_PAIR_SWIGLU = 1;

// How a matrix multiply is launched; a pure function of the shapes, strides and alignments, so the planner can ask
// for it ahead of time (to reserve the workspace) and the launch reproduces it.
struct GemmLaunchPlan {
    GemmParams p;            // operands swapped where needed so that the contiguous axis of C is the column axis
    bool swapped;            // whether they were
    bool small_tile;         // 64 x 64 workgroup tiles instead of 128 x 128
    bool tall_tile;          // f16 only: 256 x 128 workgroup tiles (8 waves)
    bool narrow_tile;        // f16 direct kernel only: 128 x 64 workgroup tiles
    bool wide_tile;          // f16 direct kernel only, together with tall_tile: 256 x 256 workgroup tiles
    bool mid_tile;           // f16 direct kernel only, together with tall_tile: 256 x 192 workgroup tiles
    bool skinny_tile;        // f32 direct kernel only: 32 x 128 workgroup tiles, for left operands of up to 32 rows
    bool dot;                // a product of up to 2^20 multiplications: one wave per result, no tiles, no MFMA
    bool direct;             // shapes and strides allow the kernel that loads global -> LDS directly
    int bk;                  // depth of a K slice
    int split_k;             // workgroups along K per output tile (1 = no split)
    int k_chunk;             // K elements per split, a multiple of bk
    // direct kernel (f16 and f32), one batch entry: the first `head_tiles` tiles are computed by one workgroup each,
    // every further tile by `tail_split` workgroups that take `tail_k_chunk` of K each and sum up inside the launch
    int head_tiles, tail_split, tail_k_chunk;
    size_t workspace_bytes;  // f32 scratch: split_k * batch * m * n * 4 when split_k > 1; one tile per sharing workgroup
    size_t counter_bytes;    // one int per shared tile
    double estimated_us;     // f16 direct kernel: what the cost model expects of the launch (0: no estimate)
};
GemmLaunchPlan plan_gemm_launch(const GemmParams &p, bool f16);
// the launch of a plan with `dot` set (both element types; `mfma_kernels.hip`)
int launch_gemm_dot(const GemmLaunchPlan &lp, bool f16, ihipStream_t *stream);
// "direct 256x128 bk64 head=256 tail_split=2x2048": kernel family, workgroup tile, slice depth and the splits
std::string describe_gemm_plan(const GemmLaunchPlan &lp, bool f16);
// whether `p.groups` products may share one launch: no operand swap, no K split, no epilogue
bool gemm_group_ok(const GemmParams &p, bool f16);


// out[n, ko, oy, ox] = act(sum_{c, fy, fx} in[n, c, oy*sy + fy - py, ox*sx + fx - px] * filter[ko, c, fy, fx]
//                          + bias[ko] + res[n, ko, oy, ox])
// Input, residual and output are dense NCHW, the filter is dense [K, C, kh, kw]; bias may be null (zero) and has
// element stride `bias_stride` between channels; res may be null.
struct ConvParams {
    const float *input;
    const float *filter;
    const float *bias;
    const float *res;
    float *output;
    int batch, in_c, in_h, in_w, out_c, out_h, out_w;
    int kernel_h, kernel_w, stride_y, stride_x, pad_y, pad_x;
    long long bias_stride;
    int relu;
    // f32 scratch of `conv_workspace_bytes` bytes (256 byte aligned) when the launch splits the input channels; may
    // be null otherwise
    float *workspace = nullptr;
    // `conv_counter_bytes` bytes of zero-filled ints that every launch hands back zero-filled: with them the kernel that
    // keeps raw planes in LDS sums the slices of a split inside the launch (the last workgroup to arrive at a tile adds
    // the parts up in their order and stores); without them (null) a second kernel does
    int *counters = nullptr;
    // filled in by the launch: slices of the input channels that are folded side by side, and channels per slice
    int splits = 1, split_channels = 0;
    // filled in by the launch: the tiles (of `tail_tile` x `tail_tile`) from `tail_head` on are each shared by
    // `tail_parts` workgroups that take `tail_channels` input channels each (conv_tail_split)
    int tail_head = 0, tail_parts = 1, tail_channels = 0, tail_tile = 64;
    // launch paths a caller may switch off
    bool channel_split = true;    // slices of the input channels folded side by side when the tiles are few
    bool plane_any_width = true;  // the plane kernel for 3 x 3 convolutions on images without a power-of-two width
};

// A convolution with few output tiles and many input channels (small batches of small boards) leaves most of the chip
// idle while every wave works through its K loop alone. The launch then folds `conv_channel_split` slices of the input
// channels side by side into f32 partial results and a second kernel sums them and applies bias, residual and
// activation. A function of the shapes alone, so that the planner can reserve the scratch ahead of time.
int conv_channel_split(const ConvParams &p);
// A tile count that leaves the last round of workgroups sparse (640 tiles of 64 x 64 on 256 compute units: two tiles
// each, and a third on half of them, which the other half waits for; 768 tiles of 128 x 128, of which a compute unit
// holds two at a time): the tiles of that round are each shared by `parts` workgroups that take a slice of the input
// channels and store f32 partial tiles, summed by a second, small kernel. Returns the number of tiles that stay whole
// (`parts` is 1 when nothing is split) and the edge of the tiles the launch picks (64 or 128). A function of the
// shapes alone, like conv_channel_split.
long long conv_tail_split(const ConvParams &p, int *parts, int *tile = nullptr);
size_t conv_workspace_bytes(const ConvParams &p);
size_t conv_counter_bytes(const ConvParams &p);

// O[b] = softmax(scale * Q[b] K[b]^T + mask[b]) V[b] with the softmax along the keys; Q is [batch, lq, dk],
// K [batch, lk, dk], V [batch, lk, dv], O [batch, lq, dv], mask [batch, lq, lk], with arbitrary element strides (batch,
// row, column in that order; zero stride = broadcast). The element type (float or _Float16) is fixed by the launch
// function; the f32 kernel takes no mask, the f16 kernel needs contiguous, 16 byte aligned rows of Q, K and V.
struct AttentionParams {
    const void *q;
    const void *k;
    const void *v;
    void *o;
    int batch, lq, lk, dk, dv;
    // batch entry z is (z / batch_inner, z % batch_inner); the `_sb` strides are those of the first index, the
    // `_sb2` strides those of the second (the mask is indexed by z itself)
    int batch_inner = 1;
    long long q_sb2 = 0, k_sb2 = 0, v_sb2 = 0, o_sb2 = 0;
    long long q_sb, q_sm, q_sk;
    long long k_sb, k_sn, k_sk;  // k_sn: between keys, k_sk: along dk
    long long v_sb, v_sk, v_sn;  // v_sk: between keys, v_sn: along dv
    long long o_sb, o_sm, o_sn;
    float scale;
    int has_scale = 1;  // f16: whether the scores are multiplied (and rounded) at all
    const void *mask = nullptr;
    long long m_sb = 0, m_sq = 0, m_sk = 0;
    int mask_vec = 0;  // rows of the mask are contiguous and 8 byte aligned
    // f16 kernel, optional: what the mask does to each block of 32 queries x ATTENTION_F16_BLOCK keys, one byte per
    // block, [mask batch (1 when m_sb is 0, else batch)][ceil(lq / 32)][ceil(lk / ATTENTION_F16_BLOCK)]:
    // 0 = has to be read and added, 1 = every entry is -inf (the block is not fetched or computed), 2 = every entry
    // is zero (the mask is not read). Known ahead of time where the mask is a constant.
    const void *block_class = nullptr;
    int o_vec = 0;  // set by the launcher: rows of O are contiguous and 16 byte aligned
};
constexpr int ATTENTION_F16_BLOCK = 32;
// the classes above for a mask given as f16 values on the host with element strides (batch, query, key); `batches` is
// 1 for a mask shared by all batch entries
std::vector<unsigned char> attention_f16_block_classes(const void *mask_f16, int batches, int lq, int lk, long long m_sb, long long m_sq, long long m_sk);
// widths the fused kernel is built for; other chains run as matmul, softmax, matmul
bool attention_supported(int dk, int dv);
bool attention_f16_supported(int dk, int dv);
// whether the launch takes the kernel whose workgroups own 128 queries and fetch every block of keys once
bool attention_f16_shares_keys(const AttentionParams &p);

// All return a hipError_t value (0 = success).
int launch_attention_f32(const AttentionParams &p, ihipStream_t *stream);
int launch_attention_f16(const AttentionParams &p, ihipStream_t *stream);
// (the plan is computed once per step, when the executor is built, from the operands at their final addresses)
int launch_gemm_f32(const GemmLaunchPlan &lp, ihipStream_t *stream);
// the kernel that loads global -> LDS directly, where `lp` (of an f32 product) and the alignment of the pointers allow
// it; `launched` tells whether it ran (the sum of split-K partial products is left to the caller)
int launch_gemm_f32_direct(const GemmLaunchPlan &lp, ihipStream_t *stream, bool *launched);
// f16 operands and result, f32 accumulation, one rounding (to nearest even) at the store
int launch_gemm_f16(const GemmLaunchPlan &lp, ihipStream_t *stream);
// second pass of a split-K launch: C = sum of the f32 partial products in the workspace (`p` already oriented)
int launch_gemm_reduce_partials(const GemmParams &p, int split, bool f16, ihipStream_t *stream);
int launch_conv_f32(const ConvParams &p, ihipStream_t *stream);
// zero `bytes` bytes (a multiple of 4, 4 byte aligned) with a kernel on `stream`
int launch_fill_zero(void *ptr, size_t bytes, ihipStream_t *stream);

}  // namespace kn
