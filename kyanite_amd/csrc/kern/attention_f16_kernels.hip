// Fused attention for f16 tensors on the CDNA4 matrix cores (v_mfma_f32_32x32x16_f16):
// O = softmax(scale * Q K^T + mask) V in one launch, with the roundings of the separate operations kept: the scores
// are rounded to f16 after the product, after the scaling and after the mask is added, exactly where the chain of
// matmul, mul, add, softmax would round them (kn-cuda-eval/src/planner.rs:606-648, :418-476 plan those launches);
// the softmax itself runs in f32 like the softmax kernel, the probabilities enter the second product as f16.
//
// Like the f32 kernel, everything is computed transposed so that a lane owns one query:
//   S^T = K Q^T      A operand: 8 consecutive k of a key row from LDS, B operand: Q, in registers
//   O^T += V^T P^T   A operand: 8 keys of one dim of V, B operand: P^T, straight from the S^T accumulators
// Register v of half h of a lane holds key 8 (v / 4) + 4 h + v % 4 of a 32-key tile, and an MFMA step takes 8 keys
// per half, so step s of the second product uses registers 8 s .. 8 s + 7, i.e. keys 16 s + 8 a + 4 h + b
// (a < 2, b < 4). K and V are both staged in LDS the way they lie in memory, one row per key; the A operand of the
// second product, which runs along the keys, is read with the transposing LDS load of gfx950 (ds_read_b64_tr_b16):
// 16 lanes hand in the addresses of 4 dims of 4 consecutive keys each and every lane gets the 4 keys of one dim.
//
// What bounds a prefill of a few hundred tokens is not arithmetic (a microsecond of it) but the number of 128 byte
// lines a compute unit requests from L2, of which it keeps about 64 in flight. So: rows are fetched whole (every
// line requested once per block), Q is fetched once per workgroup, blocks of keys that the mask removes are not
// fetched at all and neither is the mask where it is known to be zero.
#include <hip/hip_runtime.h>

#include <cmath>

#include "../mfma_kernels.h"

namespace kn {

namespace {

typedef _Float16 half_t;
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int BKEYS = ATTENTION_F16_BLOCK;  // keys per block: one MFMA tile
constexpr int WAVES = 4;   // waves per workgroup; they share 32 queries and take every fourth block of keys each

// the 4 keys (consecutive rows of the staged V) of one dim: see the head of the file
__device__ __forceinline__ halfx4 lds_read_transposed(const half_t *p) {
    return __builtin_bit_cast(halfx4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *) p));
}

// DK: width of Q and K (a multiple of 64); DVT: 32-wide tiles that cover the width of V.
// A workgroup owns 32 queries of one batch entry. Its 4 waves split the keys: wave w walks blocks w, w + 4, ... of 32
// keys with a running softmax of its own, staging K and V in a private part of LDS (no workgroup barriers in the
// loop), and the four partial results (maximum, sum, unnormalised output) are merged through LDS at the end. That
// gives four times the waves of a one-wave-per-32-queries layout, which a prefill of a few hundred tokens needs to
// fill the chip, and lets every wave skip its own masked-out blocks.
template <int DK, int DVT>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void attention_f16_kernel(AttentionParams p) {
    // Row strides in LDS. K rows are read 16 bytes per lane by 32 lanes with consecutive rows: 8 extra halves shift
    // consecutive rows by 4 banks. V rows are read 8 bytes per lane, 4 consecutive rows of 64 bytes at a time: the
    // stride is 64 or 192 bytes modulo 256, so that those 4 pieces cover all 64 banks once.
    constexpr int DV = 32 * DVT, KS = DK + 8, VS = (DV + 31) / 64 * 64 + 32;
    constexpr int KC = DK / 8, VC = DV / 8;      // 16 byte pieces per row
    constexpr int K_VECS = BKEYS * KC / 64;      // 128 bit loads of K per lane and block
    constexpr int V_VECS = BKEYS * VC / 64;      // and of V
    constexpr int Q_VECS = (32 / WAVES) * KC / 64;
    constexpr int OS = DV + 4;  // floats per query in the merge at the end
    constexpr int STAGE_BYTES = (BKEYS * KS + BKEYS * VS) * 2, MERGE_BYTES = (32 * OS + 64) * 4;
    constexpr int WAVE_BYTES = ((STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES) + 15) / 16 * 16;
    static_assert(DK % 64 == 0 && K_VECS >= 1 && V_VECS >= 1 && Q_VECS >= 1 && 64 % KC == 0 && 32 * KS * 2 <= WAVE_BYTES, "unsupported shape");
    __shared__ __attribute__((aligned(16))) unsigned char lds[WAVES][WAVE_BYTES];

    // (the wave index as a scalar: block base pointers then stay in scalar registers)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 31, h = lane >> 5;
    // Which 32 queries of which batch entry. Under a causal mask the last tile of queries has the most live key blocks
    // and the first has one; workgroups start in the order of their linear index and a compute unit holds two of them,
    // so the first half of the launch takes the later tiles of every batch entry, latest first, and the second half
    // the earlier ones: the two workgroups of a compute unit then carry about the same work together, and so do the
    // eight parts of the chip, which take workgroups in turn. Without a mask it is a harmless permutation.
    int tile = blockIdx.x, bz = blockIdx.y;
    {
        const int nt = gridDim.x, pairs = nt >> 1;
        if ((nt & 1) == 0) {
            int linear = bz * nt + tile;
            const int half_launch = pairs * (int) gridDim.y;
            const bool late = linear < half_launch;
            if (!late) linear -= half_launch;
            bz = linear / pairs;
            const int t = linear - bz * pairs;
            tile = late ? nt - 1 - t : t;
        }
    }
    const int query = tile * 32 + c;
    const int query_c = min(query, p.lq - 1);
    half_t (*Ks)[KS] = (half_t (*)[KS]) &lds[wave][0];
    half_t (*Vs)[VS] = (half_t (*)[VS]) &lds[wave][BKEYS * KS * 2];
    const int bz1 = bz / p.batch_inner, bz2 = bz - bz1 * p.batch_inner;
    const half_t *kp = (const half_t *) p.k + bz1 * p.k_sb + bz2 * p.k_sb2, *vp = (const half_t *) p.v + bz1 * p.v_sb + bz2 * p.v_sb2;
    const half_t *mp = p.mask ? (const half_t *) p.mask + bz * p.m_sb + (long long) query_c * p.m_sq : nullptr;

    // ---- the blocks of this wave and what the mask does to each: 0 = added as it is, 1 = removes the whole block
    // (every entry -inf: nothing to fetch or compute, all its terms are exact zeros), 2 = all zeros (nothing to add).
    // The launcher passes the classes where the mask is a constant; lane l keeps the class of the wave's block l.
    const int first = wave * BKEYS, stride = WAVES * BKEYS;
    const int n_blocks = first < p.lk ? (p.lk - first + stride - 1) / stride : 0;
    int class_of_block = mp ? 0 : 2;
    if (p.block_class) {
        const int key_blocks = (p.lk + BKEYS - 1) / BKEYS, kb = wave + WAVES * lane;
        const unsigned char *row = (const unsigned char *) p.block_class + ((long long) (p.m_sb ? bz : 0) * gridDim.x + tile) * key_blocks;
        class_of_block = kb < key_blocks ? row[kb] : 1;
    }
    auto block_class = [&](int i) { return __builtin_amdgcn_readlane(class_of_block, i & 63); };
    auto next_live = [&](int i) {
        while (i < n_blocks && block_class(i) == 1) i++;
        return i;
    };

    // ---- Q: every wave fetches 8 of the 32 rows, whole lines at a time; they go through the part of LDS that wave 0
    // stages K in later. The loads are issued here and picked up after the first block of keys has been requested,
    // so that the two round trips to memory overlap.
    const char *qb = (const char *) ((const half_t *) p.q + bz1 * p.q_sb + bz2 * p.q_sb2);
    const unsigned q_row = (unsigned) p.q_sm * 2;
    halfx8 qreg[Q_VECS];
#pragma unroll
    for (int i = 0; i < Q_VECS; i++) {
        const int e = lane + 64 * i, row = (32 / WAVES) * wave + e / KC, part = e % KC;
        qreg[i] = *(const halfx8 *) (qb + ((unsigned) min(tile * 32 + row, p.lq - 1) * q_row + 16 * part));
    }

    // ---- global -> registers -> LDS. The block's base pointer is wave-uniform and the lanes' offsets inside a block
    // are the same for every block, 32 bit numbers (the host checks that they fit); in a partial block rows past
    // the last key are read from the last key, and the rows of V among them are zeroed when staged.
    halfx8 kreg[K_VECS], vreg[V_VECS];
    const unsigned k_row = (unsigned) p.k_sn * 2, v_row = (unsigned) p.v_sk * 2;
    unsigned koff[K_VECS], voff[V_VECS];  // in bytes
#pragma unroll
    for (int i = 0; i < K_VECS; i++) {
        const int e = lane + 64 * i;
        koff[i] = (unsigned) (e / KC) * k_row + 16 * (e % KC);
    }
#pragma unroll
    for (int i = 0; i < V_VECS; i++) {
        const int e = lane + 64 * i;
        voff[i] = (unsigned) (e / VC) * v_row + 2 * min(8 * (e % VC), (p.dv - 1) & ~7);  // dims past dv: any valid vector
    }
    // the mask of this lane's 16 scores; a whole block with contiguous, aligned rows arrives as keys 16 h .. 16 h + 15
    // of the lane's query and is put in order later (see `mask_in_order`)
    uintx4 mraw[2];
    const unsigned moff = (unsigned) (query_c * (int) p.m_sq + 16 * h) * 2;  // vector loads only (the host checks the range)
    const char *mbase = p.mask ? (const char *) ((const half_t *) p.mask + bz * p.m_sb) : nullptr;
    auto mask_as_rows = [&](int key0) { return p.mask_vec == 2 && key0 + BKEYS <= p.lk; };
    auto fetch = [&](int i) {
        const int key0 = first + i * stride;
        const char *kb = (const char *) (kp + (long long) key0 * p.k_sn), *vb = (const char *) (vp + (long long) key0 * p.v_sk);
        if (key0 + BKEYS <= p.lk) {
#pragma unroll
            for (int j = 0; j < K_VECS; j++) kreg[j] = *(const halfx8 *) (kb + koff[j]);
#pragma unroll
            for (int j = 0; j < V_VECS; j++) vreg[j] = *(const halfx8 *) (vb + voff[j]);
        } else {
            const int last = p.lk - 1 - key0;  // last valid row of the block
#pragma unroll
            for (int j = 0; j < K_VECS; j++) {
                const int key = (lane + 64 * j) / KC;
                kreg[j] = *(const halfx8 *) (kb + (koff[j] - (unsigned) (key - min(key, last)) * k_row));
            }
#pragma unroll
            for (int j = 0; j < V_VECS; j++) {
                const int key = (lane + 64 * j) / VC;
                vreg[j] = *(const halfx8 *) (vb + (voff[j] - (unsigned) (key - min(key, last)) * v_row));
            }
        }
        if (block_class(i) == 0) {
            if (mask_as_rows(key0)) {
                const char *mb = mbase + 2 * key0;
                mraw[0] = *(const uintx4 *) (mb + moff);
                mraw[1] = *(const uintx4 *) (mb + (moff + 16));
            } else {
                halfx4 m[4];
#pragma unroll
                for (int a = 0; a < 4; a++)
#pragma unroll
                    for (int b = 0; b < 4; b++)
                        m[a][b] = mp[(long long) min(key0 + 8 * a + 4 * h + b, p.lk - 1) * p.m_sk];
                mraw[0] = uintx4{__builtin_bit_cast(uint2, m[0]).x, __builtin_bit_cast(uint2, m[0]).y, __builtin_bit_cast(uint2, m[1]).x, __builtin_bit_cast(uint2, m[1]).y};
                mraw[1] = uintx4{__builtin_bit_cast(uint2, m[2]).x, __builtin_bit_cast(uint2, m[2]).y, __builtin_bit_cast(uint2, m[3]).x, __builtin_bit_cast(uint2, m[3]).y};
            }
        }
    };
    // Keys 16 h .. 16 h + 15 of the query, as 8 registers d0 .. d7 of two keys each, become the keys of the lane's
    // scores, 8 a + 4 h + b: half 0 keeps d0 d1 d4 d5 and needs the same four of the other half's, half 1 keeps
    // d2 d3 d6 d7 and needs those of half 0. v_permlane32_swap(x, y) exchanges the upper half of x with the lower half
    // of y, so swapping (d0, d2) leaves keys 8 a + 4 h + {0, 1} for a = 0 in the first and for a = 2 in the second.
    auto mask_in_order = [&](int key0, halfx4 (&mv)[4]) {
        uint2 m[4];
        if (mask_as_rows(key0)) {
            const auto s0 = __builtin_amdgcn_permlane32_swap(mraw[0][0], mraw[0][2], false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(mraw[0][1], mraw[0][3], false, false);
            const auto s2 = __builtin_amdgcn_permlane32_swap(mraw[1][0], mraw[1][2], false, false);
            const auto s3 = __builtin_amdgcn_permlane32_swap(mraw[1][1], mraw[1][3], false, false);
            m[0] = uint2{s0[0], s1[0]};
            m[2] = uint2{s0[1], s1[1]};
            m[1] = uint2{s2[0], s3[0]};
            m[3] = uint2{s2[1], s3[1]};
        } else {
            m[0] = uint2{mraw[0][0], mraw[0][1]};
            m[1] = uint2{mraw[0][2], mraw[0][3]};
            m[2] = uint2{mraw[1][0], mraw[1][1]};
            m[3] = uint2{mraw[1][2], mraw[1][3]};
        }
#pragma unroll
        for (int a = 0; a < 4; a++) mv[a] = __builtin_bit_cast(halfx4, m[a]);
    };
    auto stage = [&](int key0) {
        const halfx8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        const bool full = key0 + BKEYS <= p.lk;  // wave-uniform
#pragma unroll
        for (int j = 0; j < K_VECS; j++) {
            const int e = lane + 64 * j;
            *(halfx8 *) &Ks[e / KC][8 * (e % KC)] = kreg[j];
        }
#pragma unroll
        for (int j = 0; j < V_VECS; j++) {
            const int e = lane + 64 * j, key = e / VC;
            *(halfx8 *) &Vs[key][8 * (e % VC)] = full || key0 + key < p.lk ? vreg[j] : zero;
        }
    };

    int i = next_live(0);
    if (i < n_blocks) fetch(i);

    // ---- Q into LDS, and from there each lane's operand: lane (query c, half h) holds k = 16 t + 8 h .. + 7 for step t
    halfx8 qf[DK / 16];
    {
        half_t (*Qs)[KS] = (half_t (*)[KS]) &lds[0][0];
#pragma unroll
        for (int j = 0; j < Q_VECS; j++) {
            const int e = lane + 64 * j, row = (32 / WAVES) * wave + e / KC, part = e % KC;
            *(halfx8 *) &Qs[row][8 * part] = qreg[j];
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < DK / 16; t++) {
            qf[t] = *(const halfx8 *) &Qs[c][16 * t + 8 * h];
            if (query >= p.lq) qf[t] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
        }
        __syncthreads();
    }

    floatx16 oacc[DVT];
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[t][v] = 0.0f;
    float row_max = -INFINITY, row_sum = 0.0f;  // row_max: the reference of the exponentials; row_sum: this half's share of the keys only
    const float scale = p.scale;                // already an f16 value
    constexpr float LOG2E = 1.44269504088896340736f;
    // the lane's corner of the transposed reads of V: 16 lanes cover 4 keys x 16 dims, lane s of them hands in the
    // address of dims 4 (s % 4) .. + 3 of key s / 4; the groups are (dims 0-15, 16-31) x (keys of half 0, half 1)
    const half_t *v_corner = &Vs[4 * h + (lane & 15) / 4][16 * ((lane >> 4) & 1) + 4 * (lane & 3)];

    while (i < n_blocks) {
        const int key0 = first + i * stride, cls = block_class(i), i_next = next_live(i + 1);
        halfx4 mv[4];
        bool skip = false;
        if (cls == 0) {
            mask_in_order(key0, mv);
            // A block whose mask is -inf for every query of the wave (the upper triangle of a causal mask) adds exact
            // zeros to every sum: nothing to compute. (-inf + a finite score is -inf whatever the score.)
            unsigned differs = 0;  // from -inf (0xfc00), two values at a time
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const uint2 bits = __builtin_bit_cast(uint2, mv[a]);
                differs |= (bits.x ^ 0xfc00fc00u) | (bits.y ^ 0xfc00fc00u);
            }
            skip = __all(differs == 0);
        }
        if (!skip) stage(key0);  // (the loaded registers are free again)
        if (i_next < n_blocks) fetch(i_next);
        i = i_next;
        if (skip) continue;

        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.0f;
#pragma unroll
        for (int t = 0; t < DK / 16; t++) {
            const halfx8 a = *(const halfx8 *) &Ks[c][16 * t + 8 * h];
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[t], st, 0, 0, 0);
        }

        // The roundings of matmul -> * scale -> + mask, in f16 arithmetic, two scores per instruction, with the same
        // results as f32 arithmetic rounded to f16: the product of two f16 values is exact in f32, and so is their sum
        // unless one is below a quarter of the other's last place, where either way of rounding returns the larger one.
        halfx2 sh[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            floatx2 two;
            two[0] = st[2 * j];
            two[1] = st[2 * j + 1];
            sh[j] = __builtin_convertvector(two, halfx2);
        }
        if (p.has_scale) {
            halfx2 scale2;
            scale2[0] = scale2[1] = (half_t) scale;
#pragma unroll
            for (int j = 0; j < 8; j++) sh[j] = sh[j] * scale2;
        }
        if (cls == 0) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                halfx2 m;
                m[0] = mv[j >> 1][2 * (j & 1)];
                m[1] = mv[j >> 1][2 * (j & 1) + 1];
                sh[j] = sh[j] + m;
            }
        }
        if (key0 + BKEYS > p.lk) {  // the last, partial block of keys
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (key0 + 8 * (v >> 2) + 4 * h + (v & 3) >= p.lk) sh[v >> 1][v & 1] = (half_t) -INFINITY;
        }
        // the running softmax in f32
        float block_max = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            st[v] = (float) sh[v >> 1][v & 1];
            block_max = fmaxf(block_max, st[v]);
        }
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32));
        // The reference value of the exponentials follows the maximum lazily: it moves (and the sums so far are
        // scaled down) only when some query's scores exceed it by more than 2^8 in the exponentials; until then the
        // weights of this wave are up to 256 instead of up to 1, which f16 weights and f32 sums hold as well, and the
        // merge at the end is told the reference, not the maximum. (The first live block of a query always moves it,
        // from -inf.)
        constexpr float SLACK = 8.0f / LOG2E;
        if (__any(block_max > row_max + SLACK)) {
            const float new_max = fmaxf(row_max, block_max);
            // a row that is masked out completely so far keeps zero weights instead of exp(-inf + inf)
            const float alpha = __builtin_amdgcn_exp2f((row_max - (new_max == -INFINITY ? 0.0f : new_max)) * LOG2E);
            row_max = new_max;
            row_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DVT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) oacc[t][v] *= alpha;
        }
        const float minus_ref = (row_max == -INFINITY ? 0.0f : -row_max) * LOG2E;
        float block_sum = 0.0f;
        halfx8 pv[2];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(st[v], LOG2E, minus_ref));
            block_sum += e;
            pv[v >> 3][v & 7] = (half_t) e;
        }
        row_sum += block_sum;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            halfx8 a[DVT];
#pragma unroll
            for (int t = 0; t < DVT; t++) {
                const halfx4 lo = lds_read_transposed(v_corner + (16 * s) * VS + 32 * t);
                const halfx4 hi = lds_read_transposed(v_corner + (16 * s + 8) * VS + 32 * t);
                a[t] = halfx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int t = 0; t < DVT; t++) oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[t], pv[s], oacc[t], 0, 0, 0);
        }
    }

    // ---- merge the four partial results: every wave leaves its maximum, sum and output in its own part of LDS, one
    // row of DV + 4 floats per query (rows 16 bytes apart modulo 256: 128 bit accesses of 16 lanes cover all banks)
    row_sum += __shfl_xor(row_sum, 32);
    typedef float floatx4 __attribute__((ext_vector_type(4)));
    float (*Of)[OS] = (float (*)[OS]) &lds[wave][0];
    float *stats = (float *) &lds[wave][32 * OS * 4];  // [0..31] maxima, [32..63] sums
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int a = 0; a < 4; a++)  // registers 4 a .. 4 a + 3: dims 32 t + 8 a + 4 h + (0 .. 3)
            *(floatx4 *) &Of[c][32 * t + 8 * a + 4 * h] = floatx4{oacc[t][4 * a], oacc[t][4 * a + 1], oacc[t][4 * a + 2], oacc[t][4 * a + 3]};
    if (h == 0) {
        stats[c] = row_max;
        stats[32 + c] = row_sum;
    }
    __syncthreads();
    float weight[WAVES], total_max = -INFINITY, total_sum = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) total_max = fmaxf(total_max, ((const float *) &lds[w][32 * OS * 4])[c]);
#pragma unroll
    for (int w = 0; w < WAVES; w++) {
        const float *st_w = (const float *) &lds[w][32 * OS * 4];
        weight[w] = __builtin_amdgcn_exp2f((st_w[c] - (total_max == -INFINITY ? 0.0f : total_max)) * LOG2E);
        total_sum += weight[w] * st_w[32 + c];
    }
    if (query < p.lq) {
        const float inv = 1.0f / total_sum;
        half_t *op = (half_t *) p.o + bz1 * p.o_sb + bz2 * p.o_sb2 + (long long) query * p.o_sm;
        // wave w, half h: dims (2 w + h) * DV / 8 ... + DV / 8
        constexpr int PER = DV / 8;
        const int d0 = (2 * wave + h) * PER;
        float x[PER];
#pragma unroll
        for (int j = 0; j < PER; j++) x[j] = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++)
#pragma unroll
            for (int j = 0; j < PER; j += 4) {
                const floatx4 part = *(const floatx4 *) &((const float (*)[OS]) &lds[w][0])[c][d0 + j];
#pragma unroll
                for (int u = 0; u < 4; u++) x[j + u] += weight[w] * part[u];
            }
        if (PER % 8 == 0 && p.o_sn == 1 && p.o_vec && d0 + PER <= p.dv) {
#pragma unroll
            for (int j = 0; j < PER; j += 8) {
                halfx8 out;
#pragma unroll
                for (int u = 0; u < 8; u++) out[u] = (half_t) (x[j + u] * inv);
                *(halfx8 *) (op + d0 + j) = out;
            }
        } else {
#pragma unroll
            for (int j = 0; j < PER; j++)
                if (d0 + j < p.dv) op[(long long) (d0 + j) * p.o_sn] = (half_t) (x[j] * inv);
        }
    }
}

// The same computation for long sequences, where the lines of K and V that the workgroups request bound the launch
// (32 heads of 2048 queries and keys under a causal mask: 104 us in the kernel above, which fetches every block of
// keys once per 32 queries). Here a workgroup owns 128 queries: wave w has queries 32 w .. 32 w + 31 of the tile, with
// a running softmax of its own over ALL blocks of keys, and the four waves fetch every block together, a quarter of
// its vectors each, into one of two LDS buffers: a block is requested once per 128 queries. One barrier per block:
// the block is staged into the buffer that nobody has read since the barrier before. A block is fetched when any
// of the four tiles of queries needs it; a wave whose own tile has it masked out only helps to stage it. The result
// of a query is complete in its wave, so there is no merge; it goes through LDS to be stored as whole rows.
template <int DK, int DVT>
// (width 64 fits the registers of three waves per SIMD without spilling, which long sequences use: 64 heads of 4096
// tokens 346 -> 267 us; width 128 would spill 40 registers there and take 1.7 times as long)
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(DK == 64 && DVT == 2 ? 3 : 2, DK == 64 && DVT == 2 ? 3 : 2)))
void attention_f16_shared_kernel(AttentionParams p) {
    constexpr int DV = 32 * DVT, KS = DK + 8, VS = (DV + 31) / 64 * 64 + 32;
    constexpr int KC = DK / 8, VC = DV / 8;                 // 16 byte pieces per row
    constexpr int THREADS = 64 * WAVES;
    constexpr int K_VECS = BKEYS * KC / THREADS;            // 128 bit loads of K per lane and block
    constexpr int V_VECS = BKEYS * VC / THREADS;            // and of V
    constexpr int Q_VECS = 32 * KC / 64;                    // of the wave's own 32 rows of Q
    constexpr int O_VECS = 32 * VC / 64;                    // 128 bit stores of the wave's 32 rows of the result
    constexpr int OS = DV + 8;                              // halves per row of the result in LDS
    constexpr int STAGE = BKEYS * KS + BKEYS * VS;          // halves per buffer
    constexpr int WAVE_ROWS = 32 * (KS > OS ? KS : OS);     // halves of a wave's own rows of Q, later of the result
    constexpr int LDS_HALVES = 2 * STAGE > WAVES * WAVE_ROWS ? 2 * STAGE : WAVES * WAVE_ROWS;
    static_assert(DK % 64 == 0 && BKEYS * KC % THREADS == 0 && BKEYS * VC % THREADS == 0 && 32 * VC % 64 == 0, "unsupported shape");
    __shared__ __attribute__((aligned(16))) half_t lds[LDS_HALVES];
    __shared__ unsigned long long needed_by[WAVES][4];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 31, h = lane >> 5;
    // (the order of the tiles under a causal mask: see the kernel above)
    int tile = blockIdx.x, bz = blockIdx.y;
    {
        const int nt = gridDim.x, pairs = nt >> 1;
        if ((nt & 1) == 0) {
            int linear = bz * nt + tile;
            const int half_launch = pairs * (int) gridDim.y;
            const bool late = linear < half_launch;
            if (!late) linear -= half_launch;
            bz = linear / pairs;
            const int t = linear - bz * pairs;
            tile = late ? nt - 1 - t : t;
        }
    }
    const int tile32 = tile * WAVES + wave, tiles32 = (p.lq + 31) / 32;
    const bool wave_has_queries = tile32 < tiles32;
    const int query = tile32 * 32 + c;
    const int query_c = min(query, p.lq - 1);
    const int bz1 = bz / p.batch_inner, bz2 = bz - bz1 * p.batch_inner;
    const half_t *kp = (const half_t *) p.k + bz1 * p.k_sb + bz2 * p.k_sb2, *vp = (const half_t *) p.v + bz1 * p.v_sb + bz2 * p.v_sb2;
    const half_t *mp = p.mask ? (const half_t *) p.mask + bz * p.m_sb + (long long) query_c * p.m_sq : nullptr;

    // ---- what the mask does to each block of keys for this wave's queries (lane l of register r: block 64 r + l),
    // and which blocks any wave of the workgroup needs
    const int n_blocks = (p.lk + BKEYS - 1) / BKEYS;
    int class_reg[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int kb = 64 * r + lane;
        int cls = mp ? 0 : 2;
        if (p.block_class && wave_has_queries && kb < n_blocks)
            cls = ((const unsigned char *) p.block_class)[((long long) (p.m_sb ? bz : 0) * tiles32 + tile32) * n_blocks + kb];
        class_reg[r] = wave_has_queries && kb < n_blocks ? cls : 1;
        const unsigned long long needs = __ballot(class_reg[r] != 1);
        if (lane == 0) needed_by[wave][r] = needs;
    }
    auto block_class = [&](int i) {
        const int r = i >> 6;
        const int reg = r == 0 ? class_reg[0] : r == 1 ? class_reg[1] : r == 2 ? class_reg[2] : class_reg[3];
        return __builtin_amdgcn_readlane(reg, i & 63);
    };

    // ---- Q: the wave's 32 rows, whole lines at a time, through the wave's own rows of LDS
    const char *qb = (const char *) ((const half_t *) p.q + bz1 * p.q_sb + bz2 * p.q_sb2);
    const unsigned q_row = (unsigned) p.q_sm * 2;
    halfx8 qreg[Q_VECS];
#pragma unroll
    for (int i = 0; i < Q_VECS; i++) {
        const int e = lane + 64 * i, row = e / KC, part = e % KC;
        qreg[i] = *(const halfx8 *) (qb + ((unsigned) min(tile32 * 32 + row, p.lq - 1) * q_row + 16 * part));
    }
    __syncthreads();  // (needed_by is written)
    unsigned long long needed[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        unsigned long long any = 0;
#pragma unroll
        for (int w = 0; w < WAVES; w++) any |= needed_by[w][r];
        needed[r] = ((unsigned long long) __builtin_amdgcn_readfirstlane((unsigned) (any >> 32)) << 32) | (unsigned) __builtin_amdgcn_readfirstlane((unsigned) any);
    }
    auto next_live = [&](int i) {
        while (i < n_blocks) {
            const int r = i >> 6;
            const unsigned long long bits = r == 0 ? needed[0] : r == 1 ? needed[1] : r == 2 ? needed[2] : needed[3];
            if ((bits >> (i & 63)) & 1) break;
            i++;
        }
        return i;
    };

    // ---- global -> registers -> LDS, a quarter of a block per wave
    halfx8 kreg[K_VECS], vreg[V_VECS];
    const unsigned k_row = (unsigned) p.k_sn * 2, v_row = (unsigned) p.v_sk * 2;
    unsigned koff[K_VECS], voff[V_VECS];  // in bytes
#pragma unroll
    for (int i = 0; i < K_VECS; i++) {
        const int e = (int) threadIdx.x + THREADS * i;
        koff[i] = (unsigned) (e / KC) * k_row + 16 * (e % KC);
    }
#pragma unroll
    for (int i = 0; i < V_VECS; i++) {
        const int e = (int) threadIdx.x + THREADS * i;
        voff[i] = (unsigned) (e / VC) * v_row + 2 * min(8 * (e % VC), (p.dv - 1) & ~7);  // dims past dv: any valid vector
    }
    uintx4 mraw[2];
    const unsigned moff = (unsigned) (query_c * (int) p.m_sq + 16 * h) * 2;
    const char *mbase = p.mask ? (const char *) ((const half_t *) p.mask + bz * p.m_sb) : nullptr;
    auto mask_as_rows = [&](int key0) { return p.mask_vec == 2 && key0 + BKEYS <= p.lk; };
    auto fetch = [&](int i) {
        const int key0 = i * BKEYS;
        const char *kb = (const char *) (kp + (long long) key0 * p.k_sn), *vb = (const char *) (vp + (long long) key0 * p.v_sk);
        if (key0 + BKEYS <= p.lk) {
#pragma unroll
            for (int j = 0; j < K_VECS; j++) kreg[j] = *(const halfx8 *) (kb + koff[j]);
#pragma unroll
            for (int j = 0; j < V_VECS; j++) vreg[j] = *(const halfx8 *) (vb + voff[j]);
        } else {
            const int last = p.lk - 1 - key0;  // last valid row of the block
#pragma unroll
            for (int j = 0; j < K_VECS; j++) {
                const int key = ((int) threadIdx.x + THREADS * j) / KC;
                kreg[j] = *(const halfx8 *) (kb + (koff[j] - (unsigned) (key - min(key, last)) * k_row));
            }
#pragma unroll
            for (int j = 0; j < V_VECS; j++) {
                const int key = ((int) threadIdx.x + THREADS * j) / VC;
                vreg[j] = *(const halfx8 *) (vb + (voff[j] - (unsigned) (key - min(key, last)) * v_row));
            }
        }
        if (block_class(i) == 0) {
            if (mask_as_rows(key0)) {
                const char *mb = mbase + 2 * key0;
                mraw[0] = *(const uintx4 *) (mb + moff);
                mraw[1] = *(const uintx4 *) (mb + (moff + 16));
            } else {
                halfx4 m[4];
#pragma unroll
                for (int a = 0; a < 4; a++)
#pragma unroll
                    for (int b = 0; b < 4; b++)
                        m[a][b] = mp[(long long) min(key0 + 8 * a + 4 * h + b, p.lk - 1) * p.m_sk];
                mraw[0] = uintx4{__builtin_bit_cast(uint2, m[0]).x, __builtin_bit_cast(uint2, m[0]).y, __builtin_bit_cast(uint2, m[1]).x, __builtin_bit_cast(uint2, m[1]).y};
                mraw[1] = uintx4{__builtin_bit_cast(uint2, m[2]).x, __builtin_bit_cast(uint2, m[2]).y, __builtin_bit_cast(uint2, m[3]).x, __builtin_bit_cast(uint2, m[3]).y};
            }
        }
    };
    // (the order of the mask's registers: see the kernel above)
    auto mask_in_order = [&](int key0, halfx4 (&mv)[4]) {
        uint2 m[4];
        if (mask_as_rows(key0)) {
            const auto s0 = __builtin_amdgcn_permlane32_swap(mraw[0][0], mraw[0][2], false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(mraw[0][1], mraw[0][3], false, false);
            const auto s2 = __builtin_amdgcn_permlane32_swap(mraw[1][0], mraw[1][2], false, false);
            const auto s3 = __builtin_amdgcn_permlane32_swap(mraw[1][1], mraw[1][3], false, false);
            m[0] = uint2{s0[0], s1[0]};
            m[2] = uint2{s0[1], s1[1]};
            m[1] = uint2{s2[0], s3[0]};
            m[3] = uint2{s2[1], s3[1]};
        } else {
            m[0] = uint2{mraw[0][0], mraw[0][1]};
            m[1] = uint2{mraw[0][2], mraw[0][3]};
            m[2] = uint2{mraw[1][0], mraw[1][1]};
            m[3] = uint2{mraw[1][2], mraw[1][3]};
        }
#pragma unroll
        for (int a = 0; a < 4; a++) mv[a] = __builtin_bit_cast(halfx4, m[a]);
    };
    auto stage = [&](int key0, half_t *buffer) {
        half_t (*Ks)[KS] = (half_t (*)[KS]) buffer;
        half_t (*Vs)[VS] = (half_t (*)[VS]) (buffer + BKEYS * KS);
        const halfx8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        const bool full = key0 + BKEYS <= p.lk;
#pragma unroll
        for (int j = 0; j < K_VECS; j++) {
            const int e = (int) threadIdx.x + THREADS * j;
            *(halfx8 *) &Ks[e / KC][8 * (e % KC)] = kreg[j];
        }
#pragma unroll
        for (int j = 0; j < V_VECS; j++) {
            const int e = (int) threadIdx.x + THREADS * j, key = e / VC;
            *(halfx8 *) &Vs[key][8 * (e % VC)] = full || key0 + key < p.lk ? vreg[j] : zero;
        }
    };

    int i = next_live(0);
    if (i < n_blocks) fetch(i);

    // ---- Q into LDS, and from there each lane's operand: lane (query c, half h) holds k = 16 t + 8 h .. + 7 for step t
    halfx8 qf[DK / 16];
    {
        half_t (*Qs)[KS] = (half_t (*)[KS]) (lds + wave * WAVE_ROWS);
#pragma unroll
        for (int j = 0; j < Q_VECS; j++) {
            const int e = lane + 64 * j;
            *(halfx8 *) &Qs[e / KC][8 * (e % KC)] = qreg[j];
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < DK / 16; t++) {
            qf[t] = *(const halfx8 *) &Qs[c][16 * t + 8 * h];
            if (query >= p.lq) qf[t] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
        }
        __syncthreads();  // (the buffers of K and V lie over these rows)
    }

    floatx16 oacc[DVT];
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[t][v] = 0.0f;
    float row_max = -INFINITY, row_sum = 0.0f;
    const float scale = p.scale;
    constexpr float LOG2E = 1.44269504088896340736f;
    // the lane's corner of the transposed reads of V inside a buffer (see the kernel above)
    const int v_corner = BKEYS * KS + (4 * h + (lane & 15) / 4) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    int parity = 0;
    while (i < n_blocks) {
        const int key0 = i * BKEYS, cls = block_class(i), i_next = next_live(i + 1);
        half_t *buffer = lds + parity * STAGE;
        parity ^= 1;
        halfx4 mv[4];
        bool skip = cls == 1;
        if (cls == 0) {
            mask_in_order(key0, mv);
            unsigned differs = 0;  // from -inf (0xfc00), two values at a time
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const uint2 bits = __builtin_bit_cast(uint2, mv[a]);
                differs |= (bits.x ^ 0xfc00fc00u) | (bits.y ^ 0xfc00fc00u);
            }
            skip = __all(differs == 0);
        }
        stage(key0, buffer);
        if (i_next < n_blocks) fetch(i_next);
        i = i_next;
        __syncthreads();
        if (skip) continue;

        const half_t (*Ks)[KS] = (const half_t (*)[KS]) buffer;
        floatx16 st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.0f;
        // (all of the block's K operands are requested before the first MFMA: one LDS round trip ahead of the chain
        // instead of one per pair of MFMAs, which is what the compiler makes of the plain loop; 2 % here, and a
        // loss in the kernel above, whose waves do not wait for each other)
        halfx8 ka[DK / 16];
#pragma unroll
        for (int t = 0; t < DK / 16; t++) ka[t] = *(const halfx8 *) &Ks[c][16 * t + 8 * h];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < DK / 16; t++) st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[t], qf[t], st, 0, 0, 0);
        // the roundings of matmul -> * scale -> + mask in f16 arithmetic (see the kernel above)
        halfx2 sh[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            floatx2 two;
            two[0] = st[2 * j];
            two[1] = st[2 * j + 1];
            sh[j] = __builtin_convertvector(two, halfx2);
        }
        if (p.has_scale) {
            halfx2 scale2;
            scale2[0] = scale2[1] = (half_t) scale;
#pragma unroll
            for (int j = 0; j < 8; j++) sh[j] = sh[j] * scale2;
        }
        if (cls == 0) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                halfx2 m;
                m[0] = mv[j >> 1][2 * (j & 1)];
                m[1] = mv[j >> 1][2 * (j & 1) + 1];
                sh[j] = sh[j] + m;
            }
        }
        if (key0 + BKEYS > p.lk) {  // the last, partial block of keys
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (key0 + 8 * (v >> 2) + 4 * h + (v & 3) >= p.lk) sh[v >> 1][v & 1] = (half_t) -INFINITY;
        }
        // the running softmax in f32, its reference following the maximum lazily (see the kernel above)
        float block_max = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            st[v] = (float) sh[v >> 1][v & 1];
            block_max = fmaxf(block_max, st[v]);
        }
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32));
        constexpr float SLACK = 8.0f / LOG2E;
        if (__any(block_max > row_max + SLACK)) {
            const float new_max = fmaxf(row_max, block_max);
            const float alpha = __builtin_amdgcn_exp2f((row_max - (new_max == -INFINITY ? 0.0f : new_max)) * LOG2E);
            row_max = new_max;
            row_sum *= alpha;
#pragma unroll
            for (int t = 0; t < DVT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) oacc[t][v] *= alpha;
        }
        const float minus_ref = (row_max == -INFINITY ? 0.0f : -row_max) * LOG2E;
        float block_sum = 0.0f;
        halfx8 pv[2];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(st[v], LOG2E, minus_ref));
            block_sum += e;
            pv[v >> 3][v & 7] = (half_t) e;
        }
        row_sum += block_sum;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            halfx8 a[DVT];
#pragma unroll
            for (int t = 0; t < DVT; t++) {
                const halfx4 lo = lds_read_transposed(buffer + v_corner + (16 * s) * VS + 32 * t);
                const halfx4 hi = lds_read_transposed(buffer + v_corner + (16 * s + 8) * VS + 32 * t);
                a[t] = halfx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
#pragma unroll
            for (int t = 0; t < DVT; t++) oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[t], pv[s], oacc[t], 0, 0, 0);
        }
    }

    // ---- the result: normalised, rounded, through the wave's own rows of LDS into whole rows of O
    row_sum += __shfl_xor(row_sum, 32);
    const float inv = 1.0f / row_sum;
    __syncthreads();  // (every wave is done with the buffers of K and V)
    half_t (*Os)[OS] = (half_t (*)[OS]) (lds + wave * WAVE_ROWS);
#pragma unroll
    for (int t = 0; t < DVT; t++)
#pragma unroll
        for (int a = 0; a < 4; a++) {  // registers 4 a .. 4 a + 3: dims 32 t + 8 a + 4 h + (0 .. 3)
            halfx4 out;
#pragma unroll
            for (int u = 0; u < 4; u++) out[u] = (half_t) (oacc[t][4 * a + u] * inv);
            *(halfx4 *) &Os[c][32 * t + 8 * a + 4 * h] = out;
        }
    __syncthreads();
    half_t *ob = (half_t *) p.o + bz1 * p.o_sb + bz2 * p.o_sb2;
#pragma unroll
    for (int j = 0; j < O_VECS; j++) {
        const int e = lane + 64 * j, row = e / VC, d0 = 8 * (e % VC), q = tile32 * 32 + row;
        if (q >= p.lq || d0 >= p.dv) continue;
        const halfx8 out = *(const halfx8 *) &Os[row][d0];
        half_t *op = ob + (long long) q * p.o_sm;
        if (p.o_sn == 1 && p.o_vec) {
            *(halfx8 *) (op + d0) = out;
        } else {
#pragma unroll
            for (int u = 0; u < 8; u++) op[(long long) (d0 + u) * p.o_sn] = out[u];
        }
    }
}

template <int DK, int DVT>
void launch_waves(const AttentionParams &p, hipStream_t stream) {
    hipLaunchKernelGGL((attention_f16_kernel<DK, DVT>), dim3((unsigned) ((p.lq + 31) / 32), (unsigned) p.batch), dim3(64 * WAVES), 0, stream, p);
}

template <int DK, int DVT>
void launch_shared(const AttentionParams &p, hipStream_t stream) {
    hipLaunchKernelGGL((attention_f16_shared_kernel<DK, DVT>), dim3((unsigned) ((p.lq + 127) / 128), (unsigned) p.batch), dim3(64 * WAVES), 0, stream, p);
}

}  // namespace

bool attention_f16_supported(int dk, int dv) {
    return (dk == 64 || dk == 128) && dv >= 8 && dv <= 128 && dv % 8 == 0;
}

// The kernel whose workgroups own 128 queries takes four times fewer lines of K and V through the caches, and per
// block of keys a wave of it does four times the work between two barriers. It wins from two workgroups per compute
// unit on (causal, width 128, us: 32 heads of 2048 tokens 100.7 -> 75.8, of 4096 295.8 -> 231.2; 64 heads of 1024
// 64.7 -> 43.5, of 2048 183.9 -> 111.9; 16 x 4096 queries on 77 keys 16.6 -> 9.1) and loses below (32 heads of 1024
// tokens 35.3 -> 39.8, of 512 14.8 -> 21.8). Its staging needs the width of V in tiles of 32 to be 2 or 4.
bool attention_f16_shares_keys(const AttentionParams &p) {
    const int dvt = (p.dv + 31) / 32;
    // (a wave of it keeps what the mask does to each block of keys in four registers, a lane per block)
    if ((dvt != 2 && dvt != 4) || p.lk > 256 * ATTENTION_F16_BLOCK) return false;
    return (long long) ((p.lq + 127) / 128) * p.batch >= 512;
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
    // rows inside a block of keys, and the queries of a batch entry, are addressed with 32 bit byte offsets
    if (p.k_sn < 0 || p.k_sn > (1 << 20) || p.v_sk < 0 || p.v_sk > (1 << 20)) return (int) hipErrorInvalidValue;
    if (p.q_sm < 0 || (long long) p.lq * p.q_sm >= (1ll << 30)) return (int) hipErrorInvalidValue;
    AttentionParams q = p;
    // whole rows of the mask are loaded 32 bytes per lane, addressed with 32 bit byte offsets inside a batch entry
    q.mask_vec = 0;
    if (p.mask && p.mask_vec && p.m_sk == 1 && p.m_sq >= 0 && p.m_sq % 8 == 0 && p.m_sb % 8 == 0 && (uintptr_t) p.mask % 16 == 0 &&
        (long long) p.lq * p.m_sq + p.lk < (1ll << 30))
        q.mask_vec = 2;
    // rows of the result can be stored 16 bytes at a time
    q.o_vec = p.o_sn == 1 && (uintptr_t) p.o % 16 == 0 && p.o_sb % 8 == 0 && p.o_sb2 % 8 == 0 && p.o_sm % 8 == 0;
    // block classes are indexed by at most 64 blocks per wave
    if (!p.mask || p.lk > 64 * 4 * ATTENTION_F16_BLOCK) q.block_class = nullptr;
    const int dvt = (p.dv + 31) / 32;
    if (attention_f16_shares_keys(p)) {
        if (p.dk == 64) {
            if (dvt == 2) launch_shared<64, 2>(q, stream);
            else launch_shared<64, 4>(q, stream);
        } else {
            if (dvt == 2) launch_shared<128, 2>(q, stream);
            else launch_shared<128, 4>(q, stream);
        }
        return (int) hipGetLastError();
    }
    if (p.dk == 64) {
        switch (dvt) {
            case 1: launch_waves<64, 1>(q, stream); break;
            case 2: launch_waves<64, 2>(q, stream); break;
            case 3: launch_waves<64, 3>(q, stream); break;
            default: launch_waves<64, 4>(q, stream); break;
        }
    } else {
        switch (dvt) {
            case 1: launch_waves<128, 1>(q, stream); break;
            case 2: launch_waves<128, 2>(q, stream); break;
            case 3: launch_waves<128, 3>(q, stream); break;
            default: launch_waves<128, 4>(q, stream); break;
        }
    }
    return (int) hipGetLastError();
}

}  // namespace kn
