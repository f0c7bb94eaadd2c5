// Fused attention for f16 tensors on the CDNA4 matrix cores (v_mfma_f32_32x32x16_f16):
// O = softmax(scale * Q K^T + mask) V in one launch, with the roundings of the separate operations kept: the scores
// are rounded to f16 after the product, after the scaling and after the mask is added, exactly where the chain of
// matmul, mul, add, softmax would round them (kn-cuda-eval/src/planner.rs:606-648, :418-476 plan those launches);
// the softmax itself runs in f32 like the softmax kernel, the probabilities enter the second product as f16.
//
// Like the f32 kernel, everything is computed transposed so that a lane owns one query:
//   S^T = K Q^T      A operand: 8 consecutive k of a key row from LDS, B operand: Q, in registers
//   O^T += V^T P^T   A operand: 8 keys of one dim of V from LDS, B operand: P^T, straight from the S^T accumulators
// Register v of half h of a lane holds key 8 (v / 4) + 4 h + v % 4 of a 32-key tile, and an MFMA step takes 8 keys
// per half, so step s of the second product uses registers 8 s .. 8 s + 7, i.e. keys 16 s + 8 a + 4 h + b
// (a < 2, b < 4). V is stored in LDS transposed, [dim][slot], with slot = 16 s + 8 h + 4 a + b, so that those 8 keys
// are one 128 bit read.
#include <hip/hip_runtime.h>

#include <cmath>

#include "../mfma_kernels.h"

namespace kn {

namespace {

typedef _Float16 half_t;
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BKEYS = 32;  // keys per block: one MFMA tile
constexpr int WAVES = 4;   // waves per workgroup; they share 32 queries and take every fourth block of keys each

__device__ __forceinline__ float r16(float x) { return (float) (half_t) x; }

// position of a key of a block inside a row of the transposed V tile
__device__ __forceinline__ int slot_of_key(int key) {
    // key = 16 s + 8 a + 4 h + b  ->  16 s + 8 h + 4 a + b
    return (key & ~12) | ((key & 8) >> 1) | ((key & 4) << 1);
}

// DK: width of Q and K (a multiple of 16); DVT: 32-wide tiles that cover the width of V.
// A workgroup owns 32 queries of one batch entry. Its 4 waves split the keys: wave w walks blocks w, w + 4, ... of 32
// keys with a running softmax of its own, staging K and V in a private part of LDS (no workgroup barriers in the
// loop), and the four partial results (maximum, sum, unnormalised output) are merged through LDS at the end. That
// gives four times the waves of a one-wave-per-32-queries layout, which a prefill of a few hundred tokens needs to
// fill the chip, and lets every wave skip its own masked-out blocks.
template <int DK, int DVT>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_f16_kernel(AttentionParams p) {
    constexpr int DV = 32 * DVT, KS = DK + 8, VS = BKEYS + 8;
    constexpr int K_VECS = BKEYS * DK / 8 / 64;          // 128 bit loads of K per lane and block
    constexpr int V_ITEMS = (BKEYS / 2) * (DV / 8) / 64;  // (key pair, 8 dims) items of V per lane and block
    constexpr int STAGE_BYTES = (BKEYS * KS + DV * VS) * 2, MERGE_BYTES = (DV * 32 + 64) * 4;
    constexpr int WAVE_BYTES = ((STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES) + 15) / 16 * 16;
    static_assert(DK % 16 == 0 && K_VECS >= 1 && V_ITEMS >= 1, "unsupported shape");
    __shared__ __attribute__((aligned(16))) unsigned char lds[WAVES][WAVE_BYTES];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int bz = blockIdx.y;
    const int query = blockIdx.x * 32 + c;
    const int query_c = min(query, p.lq - 1);
    half_t (*Ks)[KS] = (half_t (*)[KS]) &lds[wave][0];
    half_t (*Vt)[VS] = (half_t (*)[VS]) &lds[wave][BKEYS * KS * 2];
    const int bz1 = bz / p.batch_inner, bz2 = bz - bz1 * p.batch_inner;
    const half_t *kp = (const half_t *) p.k + bz1 * p.k_sb + bz2 * p.k_sb2, *vp = (const half_t *) p.v + bz1 * p.v_sb + bz2 * p.v_sb2;
    const half_t *mp = p.mask ? (const half_t *) p.mask + bz * p.m_sb + (long long) query_c * p.m_sq : nullptr;

    // Q^T operand: lane (query c, half h) holds k = 16 t + 8 h .. + 7 for step t
    halfx8 qf[DK / 16];
    {
        const half_t *qp = (const half_t *) p.q + bz1 * p.q_sb + bz2 * p.q_sb2 + (long long) query_c * p.q_sm;
#pragma unroll
        for (int t = 0; t < DK / 16; t++) {
            qf[t] = *(const halfx8 *) (qp + 16 * t + 8 * h);
            if (query >= p.lq) qf[t] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    // global -> registers -> LDS. Element offsets inside a block of keys are the same for every block and kept as
    // 32 bit numbers (the host checks that they fit), the block's base pointer is wave-uniform; in a partial block
    // rows past the last key are read from the last key and zeroed when staged.
    halfx8 kreg[K_VECS], vreg[V_ITEMS][2];
    int koff[K_VECS], voff[V_ITEMS];
#pragma unroll
    for (int i = 0; i < K_VECS; i++) {
        const int e = lane + 64 * i, key = e / (DK / 8), part = e % (DK / 8);
        koff[i] = key * (int) p.k_sn + 8 * part;
    }
#pragma unroll
    for (int i = 0; i < V_ITEMS; i++) {
        const int e = lane + 64 * i, pair = e % (BKEYS / 2), part = e / (BKEYS / 2);
        voff[i] = 2 * pair * (int) p.v_sk + min(8 * part, (p.dv - 1) & ~7);  // dims past dv: any valid vector
    }
    halfx4 mreg[4];  // the mask of this lane's 16 scores
    auto fetch = [&](int key0) {
        const half_t *kb = kp + (long long) key0 * p.k_sn, *vb = vp + (long long) key0 * p.v_sk;
        if (key0 + BKEYS <= p.lk) {
#pragma unroll
            for (int i = 0; i < K_VECS; i++) kreg[i] = *(const halfx8 *) (kb + koff[i]);
#pragma unroll
            for (int i = 0; i < V_ITEMS; i++) {
                vreg[i][0] = *(const halfx8 *) (vb + voff[i]);
                vreg[i][1] = *(const halfx8 *) (vb + voff[i] + (int) p.v_sk);
            }
        } else {
            const int last = p.lk - 1 - key0;  // last valid row of the block
#pragma unroll
            for (int i = 0; i < K_VECS; i++) {
                const int key = (lane + 64 * i) / (DK / 8);
                kreg[i] = *(const halfx8 *) (kb + koff[i] - (key - min(key, last)) * (int) p.k_sn);
            }
#pragma unroll
            for (int i = 0; i < V_ITEMS; i++) {
                const int key = 2 * ((lane + 64 * i) % (BKEYS / 2));
#pragma unroll
                for (int u = 0; u < 2; u++)
                    vreg[i][u] = *(const halfx8 *) (vb + voff[i] + (min(key + u, last) - key) * (int) p.v_sk);
            }
        }
        if (mp) {
            if (p.mask_vec && key0 + BKEYS <= p.lk) {  // whole block, contiguous aligned rows
#pragma unroll
                for (int a = 0; a < 4; a++) mreg[a] = *(const halfx4 *) (mp + key0 + 8 * a + 4 * h);
            } else {
#pragma unroll
                for (int a = 0; a < 4; a++)
#pragma unroll
                    for (int b = 0; b < 4; b++)
                        mreg[a][b] = mp[(long long) min(key0 + 8 * a + 4 * h + b, p.lk - 1) * p.m_sk];
            }
        }
    };
    auto stage = [&](int key0) {
        const halfx8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        // a whole block of keys and all DV dims present (wave-uniform): nothing to zero
        const bool full = key0 + BKEYS <= p.lk && p.dv == DV;
#pragma unroll
        for (int i = 0; i < K_VECS; i++) {
            const int e = lane + 64 * i, key = e / (DK / 8), part = e % (DK / 8);
            *(halfx8 *) &Ks[key][8 * part] = full || key0 + key < p.lk ? kreg[i] : zero;
        }
#pragma unroll
        for (int i = 0; i < V_ITEMS; i++) {
            const int e = lane + 64 * i, pair = e % (BKEYS / 2), part = e / (BKEYS / 2);
            const int key = 2 * pair, slot = slot_of_key(key);  // the odd key sits in the next slot
            halfx8 v0 = vreg[i][0], v1 = vreg[i][1];
            if (!full) {
                if (!(key0 + key < p.lk && 8 * part < p.dv)) v0 = zero;
                if (!(key0 + key + 1 < p.lk && 8 * part < p.dv)) v1 = zero;
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
                halfx2 two;
                two[0] = v0[j];
                two[1] = v1[j];
                *(halfx2 *) &Vt[8 * part + j][slot] = two;
            }
        }
    };

    floatx16 oacc[DVT];
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[t][v] = 0.0f;
    float row_max = -INFINITY, row_sum = 0.0f;  // row_sum: this half's share of the keys only
    const float scale = p.scale;                // already an f16 value
    constexpr float LOG2E = 1.44269504088896340736f;

    const int first = wave * BKEYS, stride = WAVES * BKEYS;
    if (first < p.lk) fetch(first);
    for (int key0 = first; key0 < p.lk; key0 += stride) {
        halfx4 mv[4];
#pragma unroll
        for (int a = 0; a < 4; a++) mv[a] = mreg[a];
        // A block whose mask is -inf for every query of the wave (the upper triangle of a causal mask) adds exact
        // zeros to every sum: nothing to compute. (-inf + a finite score is -inf whatever the score.)
        bool dead = mp != nullptr;
        if (mp) {
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) dead = dead && (float) mv[a][b] == -INFINITY;
        }
        const bool skip = __all(dead);
        if (!skip) stage(key0);  // (the loaded registers are free again)
        if (key0 + stride < p.lk) fetch(key0 + stride);
        if (skip) continue;

        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.0f;
#pragma unroll
        for (int t = 0; t < DK / 16; t++) {
            const halfx8 a = *(const halfx8 *) &Ks[c][16 * t + 8 * h];
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[t], st, 0, 0, 0);
        }

        // the roundings of matmul -> * scale -> + mask, then the running softmax in f32
        float block_max = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            float s = r16(st[v]);
            if (p.has_scale) s = r16(s * scale);
            if (mp) s = r16(s + (float) mv[v >> 2][v & 3]);
            if (key0 + 8 * (v >> 2) + 4 * h + (v & 3) >= p.lk) s = -INFINITY;
            st[v] = s;
            block_max = fmaxf(block_max, s);
        }
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32));
        const float new_max = fmaxf(row_max, block_max);
        // a row that is masked out completely so far keeps zero weights instead of exp(-inf + inf)
        const float safe_max = new_max == -INFINITY ? 0.0f : new_max;
        const float alpha = __builtin_amdgcn_exp2f((row_max - safe_max) * LOG2E);
        row_max = new_max;
        float block_sum = 0.0f;
        halfx8 pv[2];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float e = __builtin_amdgcn_exp2f((st[v] - safe_max) * LOG2E);
            block_sum += e;
            pv[v >> 3][v & 7] = (half_t) e;
        }
        row_sum = row_sum * alpha + block_sum;
        if (!__all(alpha == 1.0f)) {  // the maximum of some query moved
#pragma unroll
            for (int t = 0; t < DVT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) oacc[t][v] *= alpha;
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
            halfx8 a[DVT];
#pragma unroll
            for (int t = 0; t < DVT; t++) a[t] = *(const halfx8 *) &Vt[32 * t + c][16 * s + 8 * h];
#pragma unroll
            for (int t = 0; t < DVT; t++) oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[t], pv[s], oacc[t], 0, 0, 0);
        }
    }

    // ---- merge the four partial results: every wave leaves its maximum, sum and output in its own part of LDS
    row_sum += __shfl_xor(row_sum, 32);
    float (*Of)[32] = (float (*)[32]) &lds[wave][0];
    float *stats = (float *) &lds[wave][DV * 32 * 4];  // [0..31] maxima, [32..63] sums
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) Of[32 * t + 8 * (v >> 2) + 4 * h + (v & 3)][c] = oacc[t][v];
    if (h == 0) {
        stats[c] = row_max;
        stats[32 + c] = row_sum;
    }
    __syncthreads();
    float weight[WAVES], total_max = -INFINITY, total_sum = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) total_max = fmaxf(total_max, ((const float *) &lds[w][DV * 32 * 4])[c]);
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
        const float *st_w = (const float *) &lds[w][DV * 32 * 4];
        weight[w] = __builtin_amdgcn_exp2f((st_w[c] - (total_max == -INFINITY ? 0.0f : total_max)) * LOG2E);
        total_sum += weight[w] * st_w[32 + c];
    }
    if (query < p.lq) {
        const float inv = 1.0f / total_sum;
        half_t *op = (half_t *) p.o + bz1 * p.o_sb + bz2 * p.o_sb2 + (long long) query * p.o_sm;
        // wave w, half h: dims (2 w + h) * DV / 8 ... + DV / 8
        constexpr int PER = DV / 8;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int d = (2 * wave + h) * PER + i;
            float x = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; w++) x += weight[w] * ((const float (*)[32]) &lds[w][0])[d][c];
            if (d < p.dv) op[(long long) d * p.o_sn] = (half_t) (x * inv);
        }
    }
}

template <int DK, int DVT>
void launch_waves(const AttentionParams &p, hipStream_t stream) {
    hipLaunchKernelGGL((attention_f16_kernel<DK, DVT>), dim3((unsigned) ((p.lq + 31) / 32), (unsigned) p.batch), dim3(64 * WAVES), 0, stream, p);
}

}  // namespace

bool attention_f16_supported(int dk, int dv) {
    return (dk == 64 || dk == 128) && dv >= 8 && dv <= 128 && dv % 8 == 0;
}

int launch_attention_f16(const AttentionParams &p, ihipStream_t *stream) {
    if (p.batch <= 0 || p.lq <= 0 || p.dv <= 0) return 0;
    if (!attention_f16_supported(p.dk, p.dv) || p.lk <= 0 || p.batch > 65535 || p.batch_inner <= 0) return (int) hipErrorInvalidValue;
    if (p.q_sb2 % 8 != 0 || p.k_sb2 % 8 != 0 || p.v_sb2 % 8 != 0) return (int) hipErrorInvalidValue;
    // the vector loads need contiguous, 16 byte aligned rows
    auto aligned = [](const void *ptr, long long batch_stride, long long row_stride) {
        return (uintptr_t) ptr % 16 == 0 && batch_stride % 8 == 0 && row_stride % 8 == 0;
    };
    if (p.q_sk != 1 || p.k_sk != 1 || p.v_sn != 1 || !aligned(p.q, p.q_sb, p.q_sm) || !aligned(p.k, p.k_sb, p.k_sn) ||
        !aligned(p.v, p.v_sb, p.v_sk))
        return (int) hipErrorInvalidValue;
    if (p.k_sn < 0 || p.k_sn > (1 << 20) || p.v_sk < 0 || p.v_sk > (1 << 20)) return (int) hipErrorInvalidValue;
    const int dvt = (p.dv + 31) / 32;
    if (p.dk == 64) {
        switch (dvt) {
            case 1: launch_waves<64, 1>(p, stream); break;
            case 2: launch_waves<64, 2>(p, stream); break;
            case 3: launch_waves<64, 3>(p, stream); break;
            default: launch_waves<64, 4>(p, stream); break;
        }
    } else {
        switch (dvt) {
            case 1: launch_waves<128, 1>(p, stream); break;
            case 2: launch_waves<128, 2>(p, stream); break;
            case 3: launch_waves<128, 3>(p, stream); break;
            default: launch_waves<128, 4>(p, stream); break;
        }
    }
    return (int) hipGetLastError();
}

}  // namespace kn
