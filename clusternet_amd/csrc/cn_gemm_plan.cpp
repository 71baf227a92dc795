// Host-side work decomposition for the fp32 GEMM kernels (pure function, no HIP calls).
//
// The output is cut into tiles of 128 rows and 128 or 256 columns, two workgroups per compute unit
// either way (of 64 rows where K would otherwise be cut into sixteen chunks and more), or, when it has no more than
// 64 rows or is small altogether, into tiles of 32 rows and 128 columns: a 128-row tile would spend most of its matrix-core work on rows that do not exist, while a 32-row
// tile leaves such a product to what it is bound by, the one pass over B; and a small product becomes four
// times as many workgroups.  The batches this library serves are skinny (M = 128), so tiles alone cannot fill 256
// compute units; K is therefore cut into `splits` chunks, every (chunk, tile) pair becomes one
// workgroup, and a second kernel adds the chunk results in a fixed order (deterministic, no
// atomics).  Chunks are ordered chunk-major so that workgroups running at the same time walk the
// same K range and share the A panel in L2.
//
// Tile width.  A 256-column tile fetches the A tile once per 256 output columns and reads less from
// LDS per flop, and halves the number of work units (and their fill / write-out overheads); a
// 128-column tile gives twice as many work units and wins when the problem would otherwise not fill
// the machine or would leave a round mostly empty.
#include "cn_internal.h"

namespace cn {

namespace {

struct Choice {
    double cost;
    int splits;
    int64_t ips;
};

// Cost in units of "32 k of a 128 x 128 tile on a compute unit shared by two workgroups".
// `iter_cost` is the cost of one pipeline stage of this tile width in that unit; a last, partial
// round that leaves every workgroup a compute unit of its own runs at `alone` of that.
Choice best_split(int64_t tiles, int64_t k_iters, int64_t cus, double iter_cost, int64_t max_splits,
                  double out_bytes) {
    const double unit_seconds = 2.0 * 4096.0 / 2.4e9;
    const double unit_overhead = 6.0;  // pipeline fill + C write-out
    const double alone = 0.6;
    const int64_t slots = cus * 2;
    Choice best{0.0, 1, k_iters};
    for (int64_t s = 1; s <= max_splits; ++s) {
        int64_t ips = (k_iters + s - 1) / s;
        int64_t eff = (k_iters + ips - 1) / ips;
        if (eff != s && s != 1) continue;  // same decomposition as a smaller s
        int64_t units = tiles * eff;
        const int64_t full = units / slots, rest = units % slots;
        double cost = (double)full * ((double)ips * iter_cost + unit_overhead);
        if (rest) cost += (double)ips * iter_cost * (rest <= cus ? alone : 1.0) + unit_overhead;
        if (eff > 1) cost += (double)(eff + 1) * out_bytes / 4.0e12 / unit_seconds + 3.0;
        if (s == 1 || cost < best.cost) best = Choice{cost, (int)eff, ips};
    }
    return best;
}

int64_t split_limit(int64_t k_iters, int min_iters, double out_bytes, size_t workspace_bytes) {
    int64_t m = k_iters / min_iters;
    if (m > 64) m = 64;
    if (out_bytes > 0) {
        int64_t by_ws = (int64_t)((double)workspace_bytes / out_bytes);
        if (by_ws < m) m = by_ws;
    }
    return m < 1 ? 1 : m;
}

}  // namespace

GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes, int force_tile_n, bool a_along_k) {
    GemmPlan p;
    p.tile_m = kTileM;
    p.tiles_m = (M + kTileM - 1) / kTileM;
    const int64_t cus = num_cu > 0 ? num_cu : 1;
    const double out_bytes = (double)M * (double)N * 4.0;
    const int64_t tiles_n128 = (N + 127) / 128, tiles_n256 = (N + 255) / 256;
    int64_t it128 = (K + gemm_tile_k(128) - 1) / gemm_tile_k(128), it256 = (K + gemm_tile_k(256) - 1) / gemm_tile_k(256);
    if (it128 < 1) it128 = 1;
    if (it256 < 1) it256 = 1;

    // A product too small to fill the machine with 128-row tiles even at the deepest split also takes the small
    // tile: four times as many, lighter workgroups (measured: 128 x 1024 x 784 in 9.7 us instead of 18.5 us,
    // 784 x 1024 x 128 in 5.6 us instead of 11.8 us).
    const bool small = p.tiles_m * tiles_n128 * split_limit(it128, 4, out_bytes, workspace_bytes) < cus * 2;
    if (force_tile_n == kTileMLow || force_tile_n == kTileMMid || (force_tile_n == 0 && (M <= kLowTileMaxRows || small))) {
        // A stage of the 32 x 128 tile moves 20 KB for a quarter of the unit's flops: it costs what its
        // loads cost, about a third of the unit; the 64 x 128 tile, for 33 .. 64 rows, half of the unit.
        const bool mid = force_tile_n == kTileMMid || (force_tile_n == 0 && !small && M > kTileMLow);
        p.tile_m = mid ? kTileMMid : kTileMLow;
        p.tiles_m = (M + p.tile_m - 1) / p.tile_m;
        const Choice c = best_split(p.tiles_m * tiles_n128, it128, cus, mid ? 0.55 : 0.35, split_limit(it128, 4, out_bytes, workspace_bytes), out_bytes);
        p.tile_n = 128;
        p.tiles_n = tiles_n128;
        p.k_iters = it128;
        p.splits = c.splits;
        p.iters_per_split = c.ips;
        p.units = p.tiles_m * p.tiles_n * p.splits;
        return p;
    }

    // a chunk is at least 128 k deep
    Choice narrow = best_split(p.tiles_m * tiles_n128, it128, cus, 1.0, split_limit(it128, 4, out_bytes, workspace_bytes), out_bytes);
    // One 16-deep stage of a 128 x 256 tile is as many flops as the unit.  Measured per flop the wide
    // tile is within 1 % of the narrow one on streaming shapes (its lower traffic buys a little clock),
    // so the choice is left to what the model sees: fewer, longer work units and rounding of rounds.
    const double kWideGain = 1.0;
    Choice wide = best_split(p.tiles_m * tiles_n256, it256, cus, kWideGain, split_limit(it256, 8, out_bytes, workspace_bytes), out_bytes);
    bool use_wide = wide.cost < narrow.cost;
    if (force_tile_n == 128) use_wide = false;
    if (force_tile_n == 256) use_wide = true;
    const Choice &c = use_wide ? wide : narrow;
    p.tile_n = use_wide ? 256 : 128;
    p.tiles_n = use_wide ? tiles_n256 : tiles_n128;
    p.k_iters = use_wide ? it256 : it128;
    p.splits = c.splits;
    p.iters_per_split = c.ips;
    // A product cut into sixteen and more chunks of K spends a noticeable part of its time on the chunk sum (sixteen
    // planes of the result written and read back).  Tiles of 64 rows with half as many chunks are as many work units
    // of the same length and halve the planes: 128 x 4096 x 8192 in 75.9 us instead of 78.8, 128 x 4096 x 4096 in 42.9
    // instead of 45.2 (with eight chunks the two are level: 128 x 8192 x 4096 73.1 against 74.5, 128 x 8192 x 8192
    // 142.0 against 139.7).
    // Only an even number of chunks halves into the same number of work units (an odd one would add units, and with
    // them a round: 128 x 3000 x 40000 went from 21 chunks on 504 units to 11 on 528 and from 248 us to 378).
    // With A stored k by m (Tdot) the 64-row tile reads 256-byte pieces of A and loses what the planes save (128 x 4096 x
    // 8192: 77.7 us against 75.2), so the rule is for A stored m by k.
    if (force_tile_n == 0 && a_along_k && !use_wide && p.splits >= 16 && p.splits % 2 == 0) {
        p.tile_m = kTileMMid;
        p.tiles_m = (M + kTileMMid - 1) / kTileMMid;
        const int64_t half = p.splits / 2;
        p.iters_per_split = (p.k_iters + half - 1) / half;
        p.splits = (int)((p.k_iters + p.iters_per_split - 1) / p.iters_per_split);
    }
    p.units = p.tiles_m * p.tiles_n * p.splits;
    return p;
}

}  // namespace cn

static void report(const cn::GemmPlan &p, int64_t out[8]);

extern "C" void cn_host_plan_gemm_rows_along_k(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes,
                                               int force_tile_n, int64_t out[8]) {
    report(cn::plan_gemm(M, N, K, num_cu, workspace_bytes, force_tile_n, true), out);
}

extern "C" void cn_host_plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes,
                                  int force_tile_n, int64_t out[8]) {
    report(cn::plan_gemm(M, N, K, num_cu, workspace_bytes, force_tile_n, false), out);
}

static void report(const cn::GemmPlan &p, int64_t out[8]) {
    out[0] = p.tiles_m;
    out[1] = p.tiles_n;
    out[2] = p.k_iters;
    out[3] = p.splits;
    out[4] = p.iters_per_split;
    out[5] = p.units;
    out[6] = p.tile_n;
    out[7] = p.tile_m;
}
