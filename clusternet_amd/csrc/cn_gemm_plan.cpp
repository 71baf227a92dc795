// Host-side work decomposition for the fp32 GEMM kernels (pure function, no HIP calls).
//
// The output is cut into tiles of 128 rows and 128 or 256 columns.  The batches this library
// serves are skinny (M = 128), so tiles alone cannot fill 256 compute units; K is therefore cut
// into `splits` chunks, every (chunk, tile) pair becomes one workgroup, and a second kernel adds
// the chunk results in a fixed order (deterministic, no atomics).  Chunks are ordered chunk-major
// so that workgroups running at the same time walk the same K range and share the A panel in L2.
//
// Tile width.  A 256-column tile (8 wavefronts, one workgroup per compute unit) fetches the A tile
// once per 256 output columns instead of once per 128; on streaming shapes the saved L2 -> LDS
// traffic is worth about 7 % of throughput because the part runs power-limited.  A 128-column tile
// (4 wavefronts, two workgroups per compute unit) gives twice as many work units and wins when the
// problem is too small to fill the machine otherwise.
#include "cn_internal.h"

namespace cn {

namespace {

struct Choice {
    double cost;
    int splits;
    int64_t ips;
};

// Cost in units of "one K iteration (32 deep) of a compute unit's worth of tiles": a 256-wide
// workgroup owns its compute unit, two 128-wide workgroups share one, so the unit is the same.
// `alone_iter` is the cost of an iteration in a last, partial round that leaves every workgroup a
// compute unit of its own (only possible with two workgroups per unit).
Choice best_split(int64_t tiles, int64_t k_iters, int64_t slots, double per_iter, double alone_iter,
                  int64_t alone_limit, int64_t max_splits, double out_bytes) {
    const double iter_seconds = 2.0 * 4096.0 / 2.4e9;
    const double unit_overhead = 6.0;  // pipeline fill + C write-out
    Choice best{0.0, 1, k_iters};
    for (int64_t s = 1; s <= max_splits; ++s) {
        int64_t ips = (k_iters + s - 1) / s;
        int64_t eff = (k_iters + ips - 1) / ips;
        if (eff != s && s != 1) continue;  // same decomposition as a smaller s
        int64_t units = tiles * eff;
        const int64_t full = units / slots, rest = units % slots;
        double cost = (double)full * ((double)ips * per_iter + unit_overhead);
        if (rest) cost += (double)ips * (rest <= alone_limit ? alone_iter : per_iter) + unit_overhead;
        if (eff > 1) cost += (double)(eff + 1) * out_bytes / 4.0e12 / iter_seconds + 3.0;
        if (s == 1 || cost < best.cost) best = Choice{cost, (int)eff, ips};
    }
    return best;
}

}  // namespace

GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes, int force_tile_n) {
    GemmPlan p;
    p.tiles_m = (M + kTileM - 1) / kTileM;
    p.k_iters = (K + kTileK - 1) / kTileK;
    if (p.k_iters < 1) p.k_iters = 1;
    const int64_t cus = num_cu > 0 ? num_cu : 1;
    const double out_bytes = (double)M * (double)N * 4.0;

    int64_t max_splits = p.k_iters / 4;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 64) max_splits = 64;
    if (out_bytes > 0) {
        int64_t by_ws = (int64_t)((double)workspace_bytes / out_bytes);
        if (by_ws < max_splits) max_splits = by_ws;
    }
    if (max_splits < 1) max_splits = 1;

    const int64_t tiles_n128 = (N + 127) / 128, tiles_n256 = (N + 255) / 256;
    Choice narrow = best_split(p.tiles_m * tiles_n128, p.k_iters, cus * 2, 1.0, 0.6, cus, max_splits, out_bytes);
    Choice wide = best_split(p.tiles_m * tiles_n256, p.k_iters, cus, 0.93, 0.93, 0, max_splits, out_bytes);
    // Measured on MI355X: the wide tile is slower on every shape tried (81.6 % against 83.7 % of peak
    // on 128 x 40000 x 100000, 86 % against 90 % on 4096^3), so it is only used on request.
    bool use_wide = false;
    (void)wide;
    if (force_tile_n == 128) use_wide = false;
    if (force_tile_n == 256) use_wide = true;
    const Choice &c = use_wide ? wide : narrow;
    p.tile_n = use_wide ? 256 : 128;
    p.tiles_n = use_wide ? tiles_n256 : tiles_n128;
    p.splits = c.splits;
    p.iters_per_split = c.ips;
    p.units = p.tiles_m * p.tiles_n * p.splits;
    return p;
}

}  // namespace cn

extern "C" void cn_host_plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes,
                                  int force_tile_n, int64_t out[7]) {
    cn::GemmPlan p = cn::plan_gemm(M, N, K, num_cu, workspace_bytes, force_tile_n);
    out[0] = p.tiles_m;
    out[1] = p.tiles_n;
    out[2] = p.k_iters;
    out[3] = p.splits;
    out[4] = p.iters_per_split;
    out[5] = p.units;
    out[6] = p.tile_n;
}
