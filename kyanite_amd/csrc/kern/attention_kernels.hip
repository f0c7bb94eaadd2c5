// Fused attention in f32 on the CDNA4 matrix cores: O = softmax(scale * Q K^T) V without the score matrix ever
// leaving the compute unit. It replaces the three launches that the reference plans for this chain (batched matmul,
// softmax, batched matmul: kn-cuda-eval/src/planner.rs:606-648 and :418-476), which move the [Lq, Lk] scores through
// memory four times.
//
// A workgroup of 4 waves owns 128 queries of one batch entry, a wave 32 of them, and walks the keys in blocks of 64
// that sit in LDS (K as [key][k], V as [key][dim], zero padded). Everything is computed transposed, keys (then dims)
// along the rows and queries along the columns of the 32 x 32 MFMA tiles:
//   S^T = K Q^T      A operand: a row of K from LDS, B operand: Q, held in registers for the whole kernel
//   O^T += V^T P^T   A operand: a column of V from LDS, B operand: P^T
// In this orientation a lane owns one query (column l % 32), so the softmax statistics of a row of the scores are
// per-lane values (plus one exchange between the two halves of the wave), and the accumulator registers of S^T are,
// as they are, B operands of the second product: register v of half h holds key 8 (v / 4) + 4 h + v % 4 of the
// tile, and the sum over keys may run in any order, so step v of the second product simply takes that key from V.
// The softmax is the usual running one: a reference value and a sum per query, the output rescaled when the
// reference moves.
//
// A width of V that is a little over a multiple of 32 (40 for the heads of a diffusion UNet) would leave most of its
// last 32-wide tile empty. Up to 16 such dims are computed with v_mfma_f32_4x4x1_16B_f32 instead: sixteen independent
// 4 x 4 outer products per instruction, one per group of 4 lanes, 4 dims of V against the 4 queries of those lanes.
// The B operand is again the lane's own register of P^T, the A operand one float of V per lane, and the result is
// the lane's own query: 4 accumulator registers per 4 dims, no exchange between lanes. 8 cycles per 4 dims where a
// 32 x 32 x 2 instruction takes 64 for 32.
#include <hip/hip_runtime.h>

#include <cmath>

#include "../mfma_kernels.h"

namespace kn {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int THREADS = 256;  // 4 waves
constexpr int BQ = 128;       // queries per workgroup
constexpr int BKEYS = 64;     // keys per block

// DK: width of Q and K (a multiple of 8); DVT: 32-wide tiles of V; R4: groups of 4 more dims of V after those tiles.
// Group g of them holds dims 32 DVT + R4 i + g, i < 4, so that a lane reads the R4 floats it feeds to the groups
// (its i is lane % 4) with one load.
// VEC: rows of Q, K and V are contiguous and 16 byte aligned (and dv is a multiple of 4), so they move as 128 bit
// vectors: a quarter of the load instructions, which is what the vector L1 of a compute unit, not the matrix cores,
// ran out of with 32 bit loads (busy 0.93 of the cycles of a 4096 x 4096 self-attention).
template <int DK, int DVT, int R4, bool VEC>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2))) void attention_f32_kernel(AttentionParams p) {
    constexpr int DV = 32 * DVT + 4 * R4, KS = DK + 4, VS = DV + 4, HALF = DK / 2;  // row strides that spread the LDS banks
    static_assert(DK % 8 == 0 && BKEYS * 4 == THREADS, "unsupported shape");
    __shared__ __attribute__((aligned(16))) float Ks[BKEYS][KS];
    __shared__ __attribute__((aligned(16))) float Vs[BKEYS][VS];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int bz = blockIdx.y;
    const int query = blockIdx.x * BQ + wave * 32 + c;
    const int bz1 = bz / p.batch_inner, bz2 = bz - bz1 * p.batch_inner;
    const float *kp = (const float *) p.k + bz1 * p.k_sb + bz2 * p.k_sb2, *vp = (const float *) p.v + bz1 * p.v_sb + bz2 * p.v_sb2;

    // Q^T operand: lane (query c, half h) holds k = h * HALF + t for step t, pre-multiplied by scale * log2(e) so
    // that the exponentials are plain exp2
    float qf[HALF];
    {
        const float factor = p.scale * 1.44269504088896340736f;
        const float *qp = (const float *) p.q + bz1 * p.q_sb + bz2 * p.q_sb2 + (long long) query * p.q_sm;
        if (VEC) {
#pragma unroll
            for (int t4 = 0; t4 < HALF / 4; t4++) {
                const floatx4 v = query < p.lq ? *(const floatx4 *) (qp + h * HALF + 4 * t4) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int u = 0; u < 4; u++) qf[4 * t4 + u] = v[u] * factor;
            }
        } else {
#pragma unroll
            for (int t = 0; t < HALF; t++) qf[t] = query < p.lq ? qp[(long long) (h * HALF + t) * p.q_sk] * factor : 0.0f;
        }
    }

    // Global -> register -> LDS: thread t moves elements t % 4, t % 4 + 4, ... of key t / 4 of the block, so that
    // one 32 bit offset per thread (and a wave-uniform base per step) addresses all of them. Strides are not
    // negative (the host checks).
    constexpr int K_PER_THREAD = DK / 4, V_PER_THREAD = DV / 4;
    const int my_key = threadIdx.x >> 2, sub = threadIdx.x & 3;
    const unsigned koff = (unsigned) (my_key * p.k_sn + sub * p.k_sk), voff = (unsigned) (my_key * p.v_sk + sub * p.v_sn);
    float kreg[VEC ? 1 : K_PER_THREAD], vreg[VEC ? 1 : V_PER_THREAD];
    // VEC: vector e of the block is 4 floats of key e / (width / 4); the last round of threads may have none
    constexpr int K_ROW4 = DK / 4, V_ROW4 = DV / 4;
    constexpr int K_ROUNDS = (BKEYS * K_ROW4 + THREADS - 1) / THREADS, V_ROUNDS = (BKEYS * V_ROW4 + THREADS - 1) / THREADS;
    floatx4 k4[VEC ? K_ROUNDS : 1], v4[VEC ? V_ROUNDS : 1];
    auto fetch = [&](int key0) {
        const float *kb = kp + (long long) key0 * p.k_sn, *vb = vp + (long long) key0 * p.v_sk;
        if (VEC) {
            const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int i = 0; i < K_ROUNDS; i++) {
                const int e = threadIdx.x + THREADS * i, key = e / K_ROW4, part = e - key * K_ROW4;
                const bool ok = (BKEYS * K_ROW4 % THREADS == 0 || e < BKEYS * K_ROW4) && key0 + key < p.lk;
                k4[i] = ok ? *(const floatx4 *) (kb + (unsigned) (key * (int) p.k_sn + 4 * part)) : zero;
            }
#pragma unroll
            for (int i = 0; i < V_ROUNDS; i++) {
                const int e = threadIdx.x + THREADS * i, key = e / V_ROW4, part = e - key * V_ROW4;
                const bool ok = (BKEYS * V_ROW4 % THREADS == 0 || e < BKEYS * V_ROW4) && key0 + key < p.lk && 4 * part < p.dv;
                v4[i] = ok ? *(const floatx4 *) (vb + (unsigned) (key * (int) p.v_sk + 4 * part)) : zero;
            }
            return;
        }
        const bool valid = key0 + my_key < p.lk;
#pragma unroll
        for (int i = 0; i < K_PER_THREAD; i++) kreg[i] = valid ? (kb + (long long) 4 * i * p.k_sk)[koff] : 0.0f;
#pragma unroll
        for (int i = 0; i < V_PER_THREAD; i++)
            vreg[i] = valid && 4 * i + sub < p.dv ? (vb + (long long) 4 * i * p.v_sn)[voff] : 0.0f;
    };
    auto stage = [&]() {
        if (VEC) {
#pragma unroll
            for (int i = 0; i < K_ROUNDS; i++) {
                const int e = threadIdx.x + THREADS * i, key = e / K_ROW4, part = e - key * K_ROW4;
                if (BKEYS * K_ROW4 % THREADS == 0 || e < BKEYS * K_ROW4) *(floatx4 *) &Ks[key][4 * part] = k4[i];
            }
#pragma unroll
            for (int i = 0; i < V_ROUNDS; i++) {
                const int e = threadIdx.x + THREADS * i, key = e / V_ROW4, part = e - key * V_ROW4;
                if (BKEYS * V_ROW4 % THREADS == 0 || e < BKEYS * V_ROW4) *(floatx4 *) &Vs[key][4 * part] = v4[i];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < K_PER_THREAD; i++) Ks[my_key][4 * i + sub] = kreg[i];
#pragma unroll
        for (int i = 0; i < V_PER_THREAD; i++) Vs[my_key][4 * i + sub] = vreg[i];
    };

    floatx16 oacc[DVT];
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[t][v] = 0.0f;
    floatx4 orem[R4 > 0 ? R4 : 1];  // [g][i]: dim 32 DVT + R4 i + g of the lane's own query, this half's share of the keys
#pragma unroll
    for (int g = 0; g < R4; g++) orem[g] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float row_max = -INFINITY, row_sum = 0.0f;  // row_sum: this half's share of the keys only

    fetch(0);
    for (int key0 = 0; key0 < p.lk; key0 += BKEYS) {
        stage();
        __syncthreads();
        if (key0 + BKEYS < p.lk) fetch(key0 + BKEYS);

        // scores of 2 x 32 keys against the wave's 32 queries
        floatx16 st[2];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) st[j][v] = 0.0f;
        // (LDS operands are requested one step before the MFMAs that use them, and the wave raises its priority
        // while it issues MFMAs; the scheduling barriers keep that order)
        {
            floatx4 a_next[2];
#pragma unroll
            for (int j = 0; j < 2; j++) a_next[j] = *(const floatx4 *) &Ks[32 * j + c][h * HALF];
#pragma unroll
            for (int t4 = 0; t4 < HALF / 4; t4++) {
                floatx4 a[2];
#pragma unroll
                for (int j = 0; j < 2; j++) a[j] = a_next[j];
                if (t4 + 1 < HALF / 4) {
#pragma unroll
                    for (int j = 0; j < 2; j++) a_next[j] = *(const floatx4 *) &Ks[32 * j + c][h * HALF + 4 * (t4 + 1)];
                }
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        st[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j][u], qf[4 * t4 + u], st[j], 0, 0, 0);
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (key0 + BKEYS > p.lk) {
            // keys past the end take no part
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    if (key0 + 32 * j + 8 * (v >> 2) + 4 * h + (v & 3) >= p.lk) st[j][v] = -INFINITY;
        }

        float block_max = st[0][0];
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) block_max = fmaxf(block_max, st[j][v]);
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32));
        // The reference of the exponentials follows the maximum lazily: it moves, and what has been summed so far is
        // scaled down, only when some query of the wave exceeds it by more than 2^8; until then the weights are up
        // to 256 instead of up to 1. (The first block always moves it, from -inf.)
        if (__any(block_max > row_max + 8.0f)) {
            const float new_max = fmaxf(row_max, block_max);
            const float alpha = __builtin_amdgcn_exp2f(row_max - new_max);  // 0 for the first block
            row_max = new_max;
            row_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DVT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) oacc[t][v] *= alpha;
#pragma unroll
            for (int g = 0; g < R4; g++) orem[g] *= alpha;
        }
        float block_sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                st[j][v] = __builtin_amdgcn_exp2f(st[j][v] - row_max);
                block_sum += st[j][v];
            }
        row_sum += block_sum;

        {
            // steps of the second product in groups of 4 keys (one per accumulator register v % 4)
            auto key_of = [&](int step) { return 32 * (step >> 4) + 8 * ((step & 15) >> 2) + 4 * h + (step & 3); };
            constexpr int VT = DVT + R4;  // the last R4: the lane's floats of the remaining dims
            float v_next[4][VT];
            auto read_v = [&](int step0) {
#pragma unroll
                for (int u = 0; u < 4; u++) {
#pragma unroll
                    for (int t = 0; t < DVT; t++) v_next[u][t] = Vs[key_of(step0 + u)][32 * t + c];
#pragma unroll
                    for (int g = 0; g < R4; g++) v_next[u][DVT + g] = Vs[key_of(step0 + u)][32 * DVT + R4 * (lane & 3) + g];
                }
            };
            read_v(0);
#pragma unroll
            for (int step0 = 0; step0 < 32; step0 += 4) {
                float vv[4][VT];
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int t = 0; t < VT; t++) vv[u][t] = v_next[u][t];
                if (step0 + 4 < 32) read_v(step0 + 4);
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int u = 0; u < 4; u++) {
#pragma unroll
                    for (int t = 0; t < DVT; t++)
                        oacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[u][t], st[(step0 + u) >> 4][(step0 + u) & 15], oacc[t], 0, 0, 0);
#pragma unroll
                    for (int g = 0; g < R4; g++)
                        orem[g] = __builtin_amdgcn_mfma_f32_4x4x1f32(vv[u][DVT + g], st[(step0 + u) >> 4][(step0 + u) & 15], orem[g], 0, 0, 0);
                }
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();  // the block has been consumed by every wave
    }

    row_sum += __shfl_xor(row_sum, 32);
    if (query < p.lq) {
        const float inv = 1.0f / row_sum;
        float *op = (float *) p.o + bz1 * p.o_sb + bz2 * p.o_sb2 + (long long) query * p.o_sm;
#pragma unroll
        for (int t = 0; t < DVT; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int d = 32 * t + 8 * (v >> 2) + 4 * h + (v & 3);
                if (d < p.dv) op[(long long) d * p.o_sn] = oacc[t][v] * inv;
            }
    }
    if (R4 > 0) {
        floatx4 total[R4 > 0 ? R4 : 1];
#pragma unroll
        for (int g = 0; g < R4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) total[g][i] = orem[g][i] + __shfl_xor(orem[g][i], 32);
        // both halves hold the sums now; half h stores groups g with g % 2 == h
        if (query < p.lq) {
            const float inv = 1.0f / row_sum;
            float *op = (float *) p.o + bz1 * p.o_sb + bz2 * p.o_sb2 + (long long) query * p.o_sm;
#pragma unroll
            for (int g = 0; g < R4; g++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int d = 32 * DVT + R4 * i + g;
                    if ((g & 1) == h && d < p.dv) op[(long long) d * p.o_sn] = total[g][i] * inv;
                }
        }
    }
}

}  // namespace

bool attention_supported(int dk, int dv) {
    return (dk == 32 || dk == 40 || dk == 64) && dv >= 1 && dv <= 64;
}

int launch_attention_f32(const AttentionParams &p, ihipStream_t *stream) {
    if (p.batch <= 0 || p.lq <= 0 || p.dv <= 0) return 0;
    if (!attention_supported(p.dk, p.dv) || p.lk <= 0 || p.batch > 65535 || p.batch_inner <= 0) return (int) hipErrorInvalidValue;
    const dim3 grid((unsigned) ((p.lq + BQ - 1) / BQ), (unsigned) p.batch), block(THREADS);
    // 32-wide tiles of V, and the groups of 4 dims after them (up to 16 dims; a second tile beyond that)
    const int tiles = p.dv > 48 ? 2 : 1;
    const int rem = p.dv > 32 && p.dv <= 48 ? (p.dv - 32 + 3) / 4 : 0;
    // rows that can move as 128 bit vectors
    auto rows_ok = [](const void *ptr, long long inner, long long row, long long b1, long long b2) {
        return inner == 1 && row % 4 == 0 && b1 % 4 == 0 && b2 % 4 == 0 && (uintptr_t) ptr % 16 == 0;
    };
    const bool vec = p.dv % 4 == 0 && rows_ok(p.q, p.q_sk, p.q_sm, p.q_sb, p.q_sb2) && rows_ok(p.k, p.k_sk, p.k_sn, p.k_sb, p.k_sb2) &&
                     rows_ok(p.v, p.v_sn, p.v_sk, p.v_sb, p.v_sb2);
#define KN_LAUNCH_ATTENTION_V(DK, VEC) \
    do { \
        if (tiles == 2) hipLaunchKernelGGL((attention_f32_kernel<DK, 2, 0, VEC>), grid, block, 0, stream, p); \
        else if (rem == 1) hipLaunchKernelGGL((attention_f32_kernel<DK, 1, 1, VEC>), grid, block, 0, stream, p); \
        else if (rem == 2) hipLaunchKernelGGL((attention_f32_kernel<DK, 1, 2, VEC>), grid, block, 0, stream, p); \
        else if (rem == 3) hipLaunchKernelGGL((attention_f32_kernel<DK, 1, 3, VEC>), grid, block, 0, stream, p); \
        else if (rem == 4) hipLaunchKernelGGL((attention_f32_kernel<DK, 1, 4, VEC>), grid, block, 0, stream, p); \
        else hipLaunchKernelGGL((attention_f32_kernel<DK, 1, 0, VEC>), grid, block, 0, stream, p); \
    } while (0)
#define KN_LAUNCH_ATTENTION(DK) \
    do { \
        if (vec) KN_LAUNCH_ATTENTION_V(DK, true); \
        else KN_LAUNCH_ATTENTION_V(DK, false); \
    } while (0)
    switch (p.dk) {
        case 32: KN_LAUNCH_ATTENTION(32); break;
        case 40: KN_LAUNCH_ATTENTION(40); break;
        default: KN_LAUNCH_ATTENTION(64); break;
    }
#undef KN_LAUNCH_ATTENTION
#undef KN_LAUNCH_ATTENTION_V
    return (int) hipGetLastError();
}

}  // namespace kn
