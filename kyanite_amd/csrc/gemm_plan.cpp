// Launch decisions for the MFMA matrix multiply kernels: operand orientation, tile size, slice depth and the split
// of the K axis. Kept apart from the kernels so that the planner can reserve the split-K workspace in the arena.
#include <cstdlib>
#include <sstream>

#include "mfma_kernels.h"

#include <algorithm>

namespace kn {

namespace {

// ---- Cost model of the f16 kernel that loads global -> LDS directly.
//
// What a compute unit can do per slice of 64 along K is bounded by the 128 byte lines it can request - it keeps
// about 64 of them in flight, so a line costs latency / 64 of its time, whoever asked for it - and by its matrix
// cores. A workgroup with a TM x TN tile asks for TM + TN lines per slice and issues TM * TN * 64 multiply-adds; a
// launch is as slow as the busiest compute unit: rounds of workgroups, each round its slices plus a fixed cost
// (first slice's round trip, epilogue), plus the pass that sums the parts when K is split. The constants were fitted
// (least squares on log time) to 780 timings of forced tile / split combinations over 38 shapes from 1 x 4096 x 4096
// to 8192 x 8192 x 1024 with weights that do not stay in cache; the model's choice is within 1.5 % of the best
// measured combination on average and 15 % at worst, where the thresholds it replaces were 10 % and 53 % off.
struct F16Tile {
    int tm, tn;
    int per_cu;          // workgroups of this tile a compute unit holds at a time
    double ns_per_line;  // fitted; 1.8 to 2.6 ns = 4.5 to 6 cycles: the 300 to 400 cycles of a request over 64 in flight
};
constexpr int F16_TILES = 6;
const F16Tile f16_tiles[F16_TILES] = {
    {64, 64, 2, 1.998}, {128, 64, 1, 1.849}, {128, 128, 2, 2.572}, {256, 128, 1, 2.196}, {256, 192, 1, 2.396}, {256, 256, 1, 2.590},
};
enum { TILE_SMALL = 0, TILE_NARROW = 1, TILE_PLAIN = 2, TILE_TALL = 3, TILE_MID = 4, TILE_WIDE = 5 };
constexpr double MFMA_EFFICIENCY = 0.745;    // of 2500 TFLOP/s: what the matrix cores sustain on real data
constexpr double WORKGROUP_FIXED_US = 3.26;  // per round: first round trip to memory, epilogue ...
constexpr double WORKGROUP_TILE_US = 1.53;   // ... and the part of it that grows with the tile (per 128 x 128 outputs)
constexpr double LAUNCH_US = 1.14;
constexpr double SHARED_CU_FACTOR = 0.87;    // two workgroups on a compute unit overlap a little of each other's waits
constexpr double SUM_PASS_US = 2.31, SUM_PASS_US_PER_MB = 0.255;  // the pass that sums split-K parts
constexpr int COMPUTE_UNITS = 256;

// parts of the last, sparse round of tiles (0: the round is not split), see plan_gemm_launch
int tail_parts(long long blocks, long long slots, int k) {
    const long long full = blocks / slots * slots, rest = blocks - full;
    long long s = rest > 0 ? slots / rest : 1;
    if (s > k / 512) s = k / 512;
    if (s > 16) s = 16;
    if (!(full > 0 && rest * 100 < slots * 85 && s >= 2 && blocks <= 0x3fffffff)) return 0;
    long long chunk = (k + s - 1) / s;
    chunk = (chunk + 63) / 64 * 64;
    s = (k + chunk - 1) / chunk;
    return s >= 2 ? (int) s : 0;
}

double estimate_f16_direct_us(const GemmParams &p, int groups, int tile, int split, bool tail_allowed) {
    const F16Tile &t = f16_tiles[tile];
    const long long tiles = (long long) ((p.m + t.tm - 1) / t.tm) * ((p.n + t.tn - 1) / t.tn) * groups * p.batch;
    long long chunk = p.k;
    if (split > 1) chunk = ((p.k + split - 1) / split + 63) / 64 * 64;
    const long long parts = (p.k + chunk - 1) / chunk, workgroups = tiles * parts;
    const double slices = (double) chunk / 64.0;
    const double mfma_us = (double) t.tm * t.tn * 64 * 2 / (2500e12 / COMPUTE_UNITS * MFMA_EFFICIENCY) * 1e6;
    const double fixed_us = WORKGROUP_FIXED_US + WORKGROUP_TILE_US * t.tm * t.tn / 16384.0;
    auto round_us = [&](long long per_cu, double slices_here) {
        double per_slice = std::max((double) per_cu * (t.tm + t.tn) * t.ns_per_line * 1e-3, (double) per_cu * mfma_us);
        if (per_cu > 1) per_slice *= SHARED_CU_FACTOR;
        return slices_here * per_slice + fixed_us;
    };
    const long long capacity = (long long) COMPUTE_UNITS * t.per_cu;
    const long long full = workgroups / capacity, rest = workgroups % capacity;
    double us = LAUNCH_US + (double) full * round_us(t.per_cu, slices);
    if (rest > 0) {
        const long long per_cu = (rest + COMPUTE_UNITS - 1) / COMPUTE_UNITS;
        const int tail = tail_allowed && parts == 1 && p.batch == 1 ? tail_parts(tiles, capacity, p.k) : 0;
        // a round split into `tail` parts of K: measured at 0.78 of a whole round for two parts and at 0.46 for
        // eight (the parts pass f32 tiles through memory and the last one to arrive reads them all)
        us += tail ? round_us(per_cu, slices) * (1.0 / tail + 0.26 + 0.01 * tail) : round_us(per_cu, slices);
    }
    if (parts > 1) us += SUM_PASS_US + SUM_PASS_US_PER_MB * (double) p.batch * p.m * p.n * (4.0 * parts + 4.0) / 1e6;
    return us;
}

// In how many parts the f32 kernel that loads global -> LDS directly splits K when its tiles do not fill the chip.
// f32 has a sixteenth of the MFMA rate of f16, so these launches are bound by the matrix cores of the busiest compute
// unit: workgroups spread evenly, so that unit works through ceil(workgroups / 256) of them, each over its part of K
// (time per element of K: the MFMA rate at the 0.76 of the peak that 128 x 128 tiles reach and 0.66 for the tiles of
// 4096 results). The parts that count are those that put a whole number of workgroups on every unit, not as many
// workgroups as there are places: 86 tiles in 6 parts are 516 workgroups, and the four beyond 2 x 256 made 3 x 704
// of K the longest path where 5 parts have 2 x 832 (128 x 11008 x 4096: 141 us). The pass that sums the parts and
// what the memory has to deliver in any case are the other two terms.
long long f32_direct_parts(const GemmParams &p, long long blocks, bool tile_of_4096, long long most) {
    const double us_per_k = tile_of_4096 ? 64.0 * 64 * 2 / (256 * 2400.0) / 0.66 : 128.0 * 128 * 2 / (256 * 2400.0) / 0.76;
    const double results = (double) p.batch * p.m * p.n;
    const double memory_us = 4.0 * ((double) p.batch * p.k * (p.m + p.n) + results) / 5.0e6;
    long long best = 1;
    double best_us = 0.0;
    for (long long s = 1; s <= std::min(most, 16ll); s++) {
        long long chunk = ((p.k + s - 1) / s + 31) / 32 * 32;
        const long long parts = (p.k + chunk - 1) / chunk;
        if (parts != s || 4.0 * s * results > (double) (256ull << 20)) continue;
        const long long per_unit = (blocks * s + COMPUTE_UNITS - 1) / COMPUTE_UNITS;
        // (a stream of weights runs the faster the more workgroups ask for it, up to two per compute unit:
        // 8 x 4096 x 11008 in 7 parts 40.3 us, in 16 parts 38.6 us)
        const double asking = std::min(1.0, 0.8 + 0.2 * (double) (blocks * s) / (2.0 * COMPUTE_UNITS));
        double us = std::max((double) per_unit * ((double) chunk * us_per_k + 1.5), memory_us / asking);
        if (s > 1) us += 3.0 + 4.0 * (s + 1) * results / 3.0e6;
        if (best_us == 0.0 || us < best_us) best_us = us, best = s;
    }
    return best;
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
        p.tuning.stream_b = false;  // (the weight is the left operand now)
    }
    lp.p = p;
    lp.split_k = 1;
    lp.k_chunk = p.k;
    lp.tail_split = 1;
    lp.tail_k_chunk = p.k;
    if (p.batch <= 0 || p.m <= 0 || p.n <= 0) return lp;
    // A product this small is a chain of memory round trips whichever way it is tiled, and a 64 x 64 tile spends its
    // MFMAs on rows and columns that do not exist (the value head's 1 x 1 x 256 took 15.7 us, the 32 x 64 x 128 of a
    // 1 x 1 convolution on one board 12.1 us): one wave per result instead, lanes along K.
    const bool dot_enabled = p.tuning.dot_products;
    if (dot_enabled && p.groups <= 1 && !p.pair_op && p.k > 0 && (long long) p.batch * p.m * p.n * p.k <= (1ll << 20) && (long long) p.batch * p.m * p.n <= 16384) {
        lp.dot = true;
        lp.small_tile = true;
        lp.bk = 64;
        return lp;
    }

    // 128 x 128 tiles unless there are too few of them to fill the chip. Measured thresholds: f32 344 tiles run
    // 534 us on 64 x 64 tiles against 597 us, 512 tiles 734 us against 662 us; f16 344 tiles 112 us against 85 us,
    // 128 tiles 47 us against 56 us. An output no wider than 64 would leave most of a 128 wide tile unused
    // (16 x [4096 x 4096] x [4096 x 40] in f32: 450 us on 64 x 64 tiles against 682 us).
    const long long threshold = f16 ? 256 : 512;
    const bool split_enabled = p.tuning.split_k;
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
    // f32 with enough tiles either way: the tile that multiplies less padding wins, the small one counted 15 % dearer
    // per flop (320 columns are 2.5 tiles of 128: q, k and v of the UNet block in one launch 70.8 -> 50 us)
    if (!f16 && !lp.small_tile && (double) small_blocks * (64 * 64) * 1.15 < (double) big_blocks * (128 * 128)) lp.small_tile = true;
    // f16 with so few tiles that the K axis gets split anyway: 256 x 128 tiles (8 waves), which fetch a quarter
    // fewer bytes from L2 per flop and halve the partial products per split. Measured (us, 128 x 128 against
    // 256 x 128): 512 x 4096 x 4096 43 / 38, 512 x 4096 x 11008 89 / 75; without a split they do not pay:
    // 512 x 11008 x 4096 82 / 87, 8192^3 1454 / 1439.
    constexpr int tall_below = 128;
    const long long tall_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 127) / 128) * p.batch * groups;
    const bool tall_fits = !lp.small_tile && p.m >= 256 && (p.m + 255) / 256 * 256 - p.m <= p.m / 8;
    lp.tall_tile = f16 && groups == 1 && tall_fits && can_split && p.k >= 2048 && tall_blocks < tall_below;
    // Both operands with K contiguous in whole 16 byte vectors and K in whole slices of 64 (f32: 32): given aligned
    // pointers, the launch takes the kernel that loads global -> LDS directly. In f32 that kernel has the 128 x 128
    // and 64 x 64 tiles chosen above; in f16 it has six tiles, chosen below.
    const int vec = f16 ? 8 : 4;
    // (row strides: positive and small enough for the 32 bit byte offsets that the kernel keeps per lane within a tile)
    constexpr long long max_row_stride = 1ll << 21;
    lp.direct = p.tuning.direct && p.k > 0 && p.k % (8 * vec) == 0 && p.a_sk == 1 && p.b_sk == 1 && p.a_sm % vec == 0 && p.b_sn % vec == 0 &&
                p.a_sm > 0 && p.b_sn > 0 && p.a_sm < max_row_stride && p.b_sn < max_row_stride &&
                (p.batch <= 1 || (p.a_sb % vec == 0 && p.b_sb % vec == 0));
    const long long narrow_blocks = (long long) ((p.m + 127) / 128) * ((p.n + 63) / 64) * p.batch * groups;
    const long long wide_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 255) / 256) * p.batch * groups;
    const long long mid_blocks = (long long) ((p.m + 255) / 256) * ((p.n + 191) / 192) * p.batch * groups;
    // The direct f16 kernel takes tile and split from the cost model (estimate_f16_direct_us): the cheapest of
    // 64 x 64, 128 x 64, 128 x 128, 256 x 128, 256 x 192 and 256 x 256 tiles with K in 1 to 16 parts. On the shapes of
    // a 512 token LLaMA layer that is 256 x 192 for gate + up (232 tiles: one round), 256 x 128 for q + k + v,
    // 256 x 128 with K in four parts for down, 128 x 64 for o - what sweeps over those shapes had arrived at before -
    // and on shapes nobody swept it is what the thresholds it replaces were not: 256 x 4096 x 4096 22 us instead of
    // 30 us, 512 x 512 x 4096 13 / 20, 768 x 768 x 3072 16 / 20, 8192 x 320 x 1280 20 / 25, 512 x 32000 x 4096 166 / 187.
    const bool tail_enabled = p.tuning.tail_split;
    int model_split = 0;
    if (f16 && lp.direct) {
        int best_tile = TILE_SMALL, best_split = 1;
        double best_us = 0.0;
        static const int split_choices[] = {1, 2, 3, 4, 6, 8, 12, 16};
        for (int tile = 0; tile < F16_TILES; tile++) {
            const F16Tile &t = f16_tiles[tile];
            if ((t.tm == 256 && p.m <= 128) || (tile == TILE_NARROW && p.m <= 64)) continue;
            for (int split : split_choices) {
                if (split > 1) {
                    const unsigned long long bytes = (unsigned long long) split * p.batch * p.m * p.n * 4ull;
                    if (!split_enabled || groups > 1 || p.pair_op || p.k / split < 256 || bytes > (256ull << 20)) continue;
                }
                const double us = estimate_f16_direct_us(p, groups, tile, split, tail_enabled && split_enabled);
                if (best_us == 0.0 || us < best_us) {
                    best_us = us;
                    best_tile = tile;
                    best_split = split;
                }
            }
        }
        lp.small_tile = best_tile == TILE_SMALL;
        lp.narrow_tile = best_tile == TILE_NARROW;
        lp.tall_tile = best_tile >= TILE_TALL;
        lp.mid_tile = best_tile == TILE_MID;
        lp.wide_tile = best_tile == TILE_WIDE;
        lp.estimated_us = best_us;
        model_split = best_split;
    }
    // f32 under a left operand of up to 32 rows: a pass over the weights in which a 64 row tile would spend its MFMAs
    // (which f32 has 16 times fewer of than f16) mostly on rows that do not exist; 32 x 128 tiles halve them per byte
    // of weights
    // (8 x 11008 x 4096: 76.7 -> 44.1 us, 8 x 4672 x 8192: 60.7 -> 37.0 us)
    lp.skinny_tile = !f16 && lp.direct && groups == 1 && p.m <= 32 && p.n >= 128;
    if (lp.skinny_tile) lp.small_tile = false;
    long long blocks = lp.small_tile ? small_blocks : big_blocks;
    if (lp.skinny_tile) blocks = (long long) ((p.m + 31) / 32) * ((p.n + 127) / 128) * p.batch;
    if (lp.tall_tile) blocks = tall_blocks;
    if (lp.narrow_tile) blocks = narrow_blocks;
    if (lp.wide_tile) blocks = wide_blocks;
    if (lp.mid_tile) blocks = mid_blocks;
    if (f16) lp.bk = lp.small_tile || lp.tall_tile || lp.narrow_tile ? 64 : 128;
    else if (lp.direct) lp.bk = 32;
    // (a handful of tiles is a chain of memory round trips, one per slice: deep slices from 64 on)
    else lp.bk = lp.small_tile && (p.k >= 2048 || (p.k >= 256 && small_blocks < 512) || (p.k >= 64 && few_tiles)) ? 64 : 16;

    // A tile count that leaves the last round of workgroups mostly idle: the direct kernel splits the tiles of just
    // that round along K and sums the parts inside the launch, so that the round is short instead of sparse.
    // 344 tiles on 256 compute units run as one full round and 88 tiles in two halves each, instead of a second
    // round on a third of the chip (512 x 11008 x 4096 twice in one launch: 137 us -> 119 us). The partial tiles
    // pass between workgroups with accesses that bypass the L2 caches, which costs more than the second launch
    // of a plain split; so a launch with less than one round of tiles keeps that (512 x 4096 x 11008: 69 us
    // against 82 us).
    if (lp.direct && p.batch == 1 && tail_enabled && split_enabled && model_split <= 1 && !lp.skinny_tile) {
        const long long slots = 256 * (lp.tall_tile || lp.narrow_tile ? 1 : 2);
        const long long full = blocks / slots * slots, rest = blocks - full;
        const int parts = tail_parts(blocks, slots, p.k);
        if (parts >= 2) {
            long long chunk = (p.k + parts - 1) / parts;
            chunk = (chunk + 63) / 64 * 64;
            const int tm = lp.tall_tile ? 256 : (lp.small_tile ? 64 : 128), tn = lp.small_tile || lp.narrow_tile ? 64 : (lp.wide_tile ? 256 : (lp.mid_tile ? 192 : 128));
            const unsigned long long bytes = (unsigned long long) rest * parts * tm * tn * 4ull;
            if (bytes <= (256ull << 20)) {
                lp.head_tiles = (int) full;
                lp.tail_split = parts;
                lp.tail_k_chunk = (int) chunk;
                lp.workspace_bytes = (size_t) bytes;
                lp.counter_bytes = (size_t) rest * 4;
                return lp;
            }
        }
    }
    // A handful of tiles in a grouped f32 launch (which never splits K over gridDim.z): every tile is shared by
    // workgroups that take 128 or more of K each and sum inside the launch (head_tiles = 0). Two projections of a
    // context of 154 rows, 768 -> 320, were two launches that split K 6 ways plus their two summing passes, 25 us; a
    // workgroup per tile over all of K walks 24 slices at one memory round trip each, 41 us for one of them.
    if (!f16 && lp.direct && p.batch == 1 && groups > 1 && tail_enabled && split_enabled && few_tiles && !lp.skinny_tile && p.k >= 256 && !p.pair_op) {
        long long parts = std::min<long long>(p.k / 128, 16);
        long long chunk = ((p.k + parts - 1) / parts + 31) / 32 * 32;
        parts = (p.k + chunk - 1) / chunk;
        if (parts >= 2) {
            lp.head_tiles = 0;
            lp.tail_split = (int) parts;
            lp.tail_k_chunk = (int) chunk;
            const long long tile = lp.small_tile ? 64 : 128;
            lp.workspace_bytes = (size_t) (blocks * parts * tile * tile * 4);
            lp.counter_bytes = (size_t) blocks * 4;
            return lp;
        }
    }
    if (f16 && lp.direct) {
        if (model_split > 1) {
            long long chunk = (p.k + model_split - 1) / model_split;
            chunk = (chunk + lp.bk - 1) / lp.bk * lp.bk;
            const long long parts = (p.k + chunk - 1) / chunk;
            if (parts > 1) {
                lp.split_k = (int) parts;
                lp.k_chunk = (int) chunk;
                lp.workspace_bytes = (size_t) ((unsigned long long) parts * p.batch * p.m * p.n * 4ull);
            }
        }
        return lp;
    }

    const long long split_below = lp.tall_tile ? 128 : 256, split_target = lp.tall_tile ? 256 : 512;
    // (a product of a few thousand multiplications is one short workgroup: a second launch to sum parts costs more)
    const bool tiny = (long long) p.batch * p.m * p.n * p.k < (1ll << 18);
    if (can_split && blocks < split_below && groups == 1 && !lp.narrow_tile && !tiny && !p.pair_op) {
        const int min_chunk = few_tiles ? 128 : (f16 ? 512 : 256);  // K elements a split should at least cover
        long long s = (split_target + blocks - 1) / blocks;
        if (s > p.k / min_chunk) s = p.k / min_chunk;
        if (!f16 && lp.direct) s = f32_direct_parts(p, blocks, lp.small_tile || lp.skinny_tile, p.k / min_chunk);
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
    if (lp.dot) return "a wave per result";
    int tm = lp.small_tile ? 64 : 128, tn = tm;
    if (lp.tall_tile) tm = 256;
    if (lp.narrow_tile) tn = 64;
    if (lp.direct && f16) {
        if (lp.wide_tile) tn = 256;
        if (lp.mid_tile) tn = 192;
    } else if (lp.narrow_tile) {
        tm = tn = 64;
    }
    if (lp.skinny_tile) tm = 32, tn = 128;
    ss << (lp.direct ? "direct " : "staged ") << tm << "x" << tn << " bk" << lp.bk;
    if (lp.p.pair_op) ss << " gated pairs";
    if (lp.direct && lp.p.tuning.stream_b) ss << " weights streamed";
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
    // A grouped launch never splits K. With the cost model (f16, the kernel that loads global -> LDS directly): one
    // launch if it is expected to take no longer than the products one by one, each on the tiles and the split of K it
    // would pick. (The rule below saw a split of K in the plan of all columns together for 384 rows against three
    // weights of 4096 x 4096 and left three launches of too few tiles each: a 384 token prefill of the two LLaMA
    // layers took 621 us, more than one of 512 tokens; 576 us as one launch. 256 tokens, which it had as one launch and
    // a pair, are 3 % slower as one launch of three.)
    GemmParams one = p;
    one.groups = 1;
    const GemmLaunchPlan single = plan_gemm_launch(one, f16), grouped = plan_gemm_launch(p, f16);
    if (single.estimated_us > 0.0 && grouped.estimated_us > 0.0) return grouped.estimated_us <= p.groups * single.estimated_us;
    // Otherwise: where even all products together leave the chip short of tiles, separate launches that split K are
    // faster.
    // (a handful of f32 tiles: the grouped launch shares every tile between workgroups along K)
    if (grouped.tail_split > 1 && grouped.head_tiles == 0) return true;
    GemmParams wide = p;
    wide.groups = 1;
    wide.n = p.n * p.groups;
    return plan_gemm_launch(wide, f16).split_k == 1;
}

}  // namespace kn
