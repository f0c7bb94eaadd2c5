// Launch decisions for the MFMA matrix multiply kernels: operand orientation, tile size, slice depth and the split
// of the K axis. Kept apart from the kernels so that the planner can reserve the split-K workspace in the arena.
#include <cstdlib>
#include <sstream>

#include "mfma_kernels.h"

#include <algorithm>

namespace kn {

namespace {

int env_int(const char *name, int fallback) {
    const char *env = getenv(name);
    return env && *env ? atoi(env) : fallback;
}

}  // namespace

GemmLaunchPlan plan_gemm_launch(const GemmParams &params, bool f16) {
    GemmLaunchPlan lp{};
    GemmParams p = params;
    // put the axis of C that is contiguous in memory on the MFMA column (lane) axis: D^T = B^T * A^T
    auto mag = [](long long x) { return x < 0 ? -x : x; };
    if (mag(p.c_sm) < mag(p.c_sn)) {
        GemmParams q = p;
        q.a = p.b; q.b = p.a;
        q.m = p.n; q.n = p.m;
        q.a_sb = p.b_sb; q.a_sm = p.b_sn; q.a_sk = p.b_sk;
        q.b_sb = p.a_sb; q.b_sk = p.a_sk; q.b_sn = p.a_sm;
        q.c_sm = p.c_sn; q.c_sn = p.c_sm;
        q.d_sm = p.d_sn; q.d_sn = p.d_sm;
        q.d2_sm = p.d2_sn; q.d2_sn = p.d2_sm;
        p = q;
        lp.swapped = true;
    }
    lp.p = p;
    lp.split_k = 1;
    lp.k_chunk = p.k;
    lp.tail_split = 1;
    lp.tail_k_chunk = p.k;
    if (p.batch <= 0 || p.m <= 0 || p.n <= 0) return lp;

    // 128 x 128 tiles unless there are too few of them to fill the chip. Measured thresholds: f32 344 tiles run
    // 534 us on 64 x 64 tiles against 597 us, 512 tiles 734 us against 662 us; f16 344 tiles 112 us against 85 us,
    // 128 tiles 47 us against 56 us. An output no wider than 64 would leave most of a 128 wide tile unused
    // (16 x [4096 x 4096] x [4096 x 40] in f32: 450 us on 64 x 64 tiles against 682 us).
    const long long threshold = f16 ? 256 : 512;
    static const int split_enabled = env_int("KNHIP_SPLIT_K", 1);
    const int groups = p.groups > 1 ? p.groups : 1;
    const long long big_blocks = (long long) ((p.m + 127) / 128) * ((p.n + 127) / 128) * p.batch * groups;
    const bool narrow = p.m <= 64 || p.n <= 64;
    // With a long K axis and too few tiles, 128 x 128 tiles split along K keep the higher arithmetic intensity
    // per byte fetched from L2 and still fill the chip.
    // A handful of tiles leaves the chip idle while every workgroup walks all of K at one slice per memory round
    // trip, so there K is split from 256 on (154 x 320 x 768 in f32: 41 us unsplit).
    const long long small_blocks = (long long) ((p.m + 63) / 64) * ((p.n + 63) / 64) * p.batch * groups;
    const bool few_tiles = small_blocks < 64;
    const bool can_split = split_enabled && (p.k >= 1024 || (few_tiles && p.k >= 256));
    lp.small_tile = narrow || (big_blocks < threshold && !(can_split && p.k >= 2048 && big_blocks < 256));
    // f16 with so few tiles that the K axis gets split anyway: 256 x 128 tiles (8 waves), which fetch a quarter
    // fewer bytes from L2 per flop and halve the partial products per split. Measured (us, 128 x 128 against
    // 256 x 128): 512 x 4096 x 4096 43 / 38, 512 x 4096 x 11008 89 / 75; without a split they do not pay:
    // 512 x 11008 x 4096 82 / 87, 8192^3 1454 / 1439.
    constexpr int tall_below = 128;
    const long long tall_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 127) / 128) * p.batch * groups;
    const bool tall_fits = !lp.small_tile && p.m >= 256 && (p.m + 255) / 256 * 256 - p.m <= p.m / 8;
    lp.tall_tile = f16 && groups == 1 && tall_fits && can_split && p.k >= 2048 && tall_blocks < tall_below;
    // Both operands with K contiguous in whole 16 byte vectors and K in whole slices of 64: given aligned
    // pointers, the launch takes the kernel that loads global -> LDS directly. There the tall tiles run on a ring
    // of three stages and also pay without a split, as long as they still fill the chip. Measured with weights
    // that come from memory, not from cache (us, 128 x 128 on two stages against 256 x 128 on three):
    // 512 x 22016 x 4096 147 / 133, 512 x 12288 x 4096 93 / 72, 4096^3 152 / 144; 512 x 4096 x 4096 53 / 59.
    // (In f32 the same kernel walks K in slices of 32 and has 128 x 128 and 64 x 64 tiles.)
    const int vec = f16 ? 8 : 4;
    // (row strides: positive and small enough for the 32 bit byte offsets that the kernel keeps per lane within a tile)
    constexpr long long max_row_stride = 1ll << 21;
    lp.direct = p.k > 0 && p.k % (8 * vec) == 0 && p.a_sk == 1 && p.b_sk == 1 && p.a_sm % vec == 0 && p.b_sn % vec == 0 &&
                p.a_sm > 0 && p.b_sn > 0 && p.a_sm < max_row_stride && p.b_sn < max_row_stride &&
                (p.batch <= 1 || (p.a_sb % vec == 0 && p.b_sb % vec == 0));
    if (f16 && lp.direct && tall_fits && tall_blocks >= 128) lp.tall_tile = true;
    // Direct kernel only: 128 x 64 tiles on a ring of four stages, where 128 x 128 tiles leave compute units
    // without a workgroup and K is too short for a split to pay (512 x 4096 x 4096: 29 us against 39 us on
    // 256 x 128 tiles split in four; 512 x 4096 x 11008: 84 us against 69 us).
    const long long narrow_blocks = (long long) ((p.m + 127) / 128) * ((p.n + 63) / 64) * p.batch * groups;
    lp.narrow_tile = f16 && lp.direct && !narrow && p.m > 64 && big_blocks < 256 && narrow_blocks >= 192 &&
                     p.k < 8192;
    if (lp.narrow_tile) lp.small_tile = lp.tall_tile = false;
    // Direct kernel only: 256 x 256 tiles (8 waves of 128 x 64) where they still give every compute unit a
    // workgroup. The LDS bounds this kernel, and they need the least LDS traffic per flop: 256 KB per slice of 64
    // for twice the work of a 256 x 128 tile with its 176 KB (8192^3: 1191 -> 1030 us, 4096^3: 166 -> 139 us).
    // Between the two sit 256 x 192 tiles (216 KB per slice for one and a half times the work). Among the three
    // the plan takes the one with the least estimated LDS time: rounds of workgroups on 256 compute units (a last
    // sparse round counts as one split in two) x LDS clocks per slice. 2 x 512 x 11008 x 4096 in one launch:
    // 344 tiles of 256 x 128 are 1.6 rounds of 2750 clocks, 232 tiles of 256 x 192 one round of 3375.
    const long long wide_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 255) / 256) * p.batch * groups;
    const long long mid_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 191) / 192) * p.batch * groups;
    if (f16 && lp.direct && lp.tall_tile) {
        auto lds_time = [&](long long tiles, double clocks) {
            const long long full = tiles / 256, rest = tiles % 256;
            double rounds = (double) full;
            if (rest > 0) rounds += full > 0 && rest <= 128 && p.batch == 1 && p.k >= 1024 ? 0.6 : 1.0;
            return rounds * clocks;
        };
        auto fits = [&](int width) { return p.n >= width && (p.n + width - 1) / width * width - p.n <= p.n / 8; };
        const double t_tall = lds_time(tall_blocks, 2750.0);
        const double t_mid = fits(192) ? lds_time(mid_blocks, 3375.0) : 1e30;
        const double t_wide = fits(256) && wide_blocks >= 256 ? lds_time(wide_blocks, 4000.0) : 1e30;
                lp.wide_tile = t_wide <= t_tall && t_wide <= t_mid;
        lp.mid_tile = !lp.wide_tile && t_mid < t_tall;
    }
    long long blocks = lp.small_tile ? small_blocks : big_blocks;
    if (lp.tall_tile) blocks = tall_blocks;
    if (lp.narrow_tile) blocks = narrow_blocks;
    if (lp.wide_tile) blocks = wide_blocks;
    if (lp.mid_tile) blocks = mid_blocks;
    if (f16) lp.bk = lp.small_tile || lp.tall_tile || lp.narrow_tile ? 64 : 128;
    else if (lp.direct) lp.bk = 32;
    else lp.bk = lp.small_tile && (p.k >= 2048 || (p.k >= 256 && small_blocks < 512)) ? 64 : 16;

    // A tile count that leaves the last round of workgroups mostly idle: the direct kernel splits the tiles of just
    // that round along K and sums the parts inside the launch, so that the round is short instead of sparse.
    // 344 tiles on 256 compute units run as one full round and 88 tiles in two halves each, instead of a second
    // round on a third of the chip (512 x 11008 x 4096 twice in one launch: 137 us -> 119 us). The partial tiles
    // pass between workgroups with accesses that bypass the L2 caches, which costs more than the second launch
    // of a plain split; so a launch with less than one round of tiles keeps that (512 x 4096 x 11008: 69 us
    // against 82 us).
    static const int tail_enabled = env_int("KNHIP_TAIL_SPLIT", 1);
    if (lp.direct && p.batch == 1 && tail_enabled && split_enabled) {
        const long long slots = 256 * (lp.tall_tile || lp.narrow_tile ? 1 : 2);
        const long long full = blocks / slots * slots, rest = blocks - full;
        long long s = rest > 0 ? slots / rest : 1;
        if (s > p.k / 512) s = p.k / 512;
        if (s > 16) s = 16;
        if (full > 0 && rest * 100 < slots * 85 && s >= 2 && blocks <= 0x3fffffff) {
            long long chunk = (p.k + s - 1) / s;
            chunk = (chunk + 63) / 64 * 64;
            s = (p.k + chunk - 1) / chunk;
            const int tm = lp.tall_tile ? 256 : (lp.small_tile ? 64 : 128), tn = lp.small_tile || lp.narrow_tile ? 64 : (lp.wide_tile ? 256 : (lp.mid_tile ? 192 : 128));
            const unsigned long long bytes = (unsigned long long) rest * s * tm * tn * 4ull;
            if (s >= 2 && bytes <= (256ull << 20)) {
                lp.head_tiles = (int) full;
                lp.tail_split = (int) s;
                lp.tail_k_chunk = (int) chunk;
                lp.workspace_bytes = (size_t) bytes;
                lp.counter_bytes = (size_t) rest * 4;
                return lp;
            }
        }
    }

    const long long split_below = lp.tall_tile ? 128 : 256, split_target = lp.tall_tile ? 256 : 512;
    if (can_split && blocks < split_below && groups == 1 && !lp.narrow_tile) {
        const int min_chunk = few_tiles ? 128 : (f16 ? 512 : 256);  // K elements a split should at least cover
        long long s = (split_target + blocks - 1) / blocks;
        if (s > p.k / min_chunk) s = p.k / min_chunk;
        if (s > 1) {
            long long chunk = (p.k + s - 1) / s;
            chunk = (chunk + lp.bk - 1) / lp.bk * lp.bk;
            s = (p.k + chunk - 1) / chunk;
            const unsigned long long bytes = (unsigned long long) s * p.batch * p.m * p.n * 4ull;
            if (s > 1 && bytes <= (256ull << 20)) {
                lp.split_k = (int) s;
                lp.k_chunk = (int) chunk;
                lp.workspace_bytes = (size_t) bytes;
            }
        }
    }
    return lp;
}

std::string describe_gemm_plan(const GemmLaunchPlan &lp, bool f16) {
    std::ostringstream ss;
    int tm = lp.small_tile ? 64 : 128, tn = tm;
    if (lp.tall_tile) tm = 256;
    if (lp.narrow_tile) tn = 64;
    if (lp.direct && f16) {
        if (lp.wide_tile) tn = 256;
        if (lp.mid_tile) tn = 192;
    } else if (lp.narrow_tile) {
        tm = tn = 64;
    }
    ss << (lp.direct ? "direct " : "staged ") << tm << "x" << tn << " bk" << lp.bk;
    if (lp.split_k > 1) ss << " split_k=" << lp.split_k << "x" << lp.k_chunk;
    if (lp.tail_split > 1) ss << " head=" << lp.head_tiles << " tail_split=" << lp.tail_split << "x" << lp.tail_k_chunk;
    return ss.str();
}

std::vector<unsigned char> attention_f16_block_classes(const void *mask_f16, int batches, int lq, int lk, long long m_sb, long long m_sq, long long m_sk) {
    const uint16_t *m = (const uint16_t *) mask_f16;
    const int q_tiles = (lq + 31) / 32, key_blocks = (lk + ATTENTION_F16_BLOCK - 1) / ATTENTION_F16_BLOCK;
    std::vector<unsigned char> classes((size_t) batches * q_tiles * key_blocks);
    for (int b = 0; b < batches; b++)
        for (int qt = 0; qt < q_tiles; qt++)
            for (int kb = 0; kb < key_blocks; kb++) {
                // queries past lq repeat the last query in the kernel and keys past lk are dropped there: neither counts
                bool all_neg_inf = true, all_zero = true;
                for (int q = 32 * qt; q < std::min(lq, 32 * qt + 32); q++)
                    for (int k = ATTENTION_F16_BLOCK * kb; k < std::min(lk, ATTENTION_F16_BLOCK * (kb + 1)); k++) {
                        const uint16_t bits = m[b * m_sb + q * m_sq + k * m_sk];
                        all_neg_inf &= bits == 0xfc00;
                        all_zero &= (bits & 0x7fff) == 0;  // +0 or -0: adding either leaves every score's value
                    }
                classes[((size_t) b * q_tiles + qt) * key_blocks + kb] = all_neg_inf ? 1 : all_zero ? 2 : 0;
            }
    return classes;
}

bool gemm_group_ok(const GemmParams &p, bool f16) {
    if (p.groups < 2 || p.groups > GEMM_MAX_GROUPS || p.addend != nullptr || p.relu) return false;
    auto mag = [](long long x) { return x < 0 ? -x : x; };
    if (mag(p.c_sm) < mag(p.c_sn)) return false;  // the launch would swap the operands
    // A grouped launch never splits K. Where even all products together leave the chip short of tiles, separate
    // launches that split K are faster.
    GemmParams wide = p;
    wide.groups = 1;
    wide.n = p.n * p.groups;
    return plan_gemm_launch(wide, f16).split_k == 1;
}

}  // namespace kn
