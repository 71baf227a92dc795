// Host-side work decomposition for the fp32 GEMM kernels (pure function, no HIP calls).
//
// The output is cut into tiles of one of four geometries (rows x columns): 128 x 128, 128 x 256, 64 x 128 or 32 x 128,
// two workgroups per compute unit for each.  The batches this library serves are skinny (M = 128), so tiles alone cannot
// fill 256 compute units; K is therefore cut into `splits` chunks, every (chunk, tile) pair becomes one workgroup, and a
// second kernel adds the chunk results in a fixed order (deterministic, no atomics).  Chunks are ordered chunk-major so
// that workgroups running at the same time walk the same K range and share the A panel in L2.
//
// One cost model decides both the geometry and the split: rounds of resident workgroups, each costing its stages plus a
// fixed part, a last partial round that runs faster when its workgroups have a compute unit to themselves, and the chunk
// sum.  Its six kinds of constants are microseconds measured on this part (a least-squares fit over forty shapes times
// four geometries, 9 % rms); tests/test_gpu_planner.py times the planned form of those shapes against every forced
// geometry and fails when a rule change leaves one more than 7 % behind the best.
//   128 x 256  fetches the A tile once per 256 output columns and reads less from LDS per flop: 2.5 % faster per flop
//              than 128 x 128 on streaming shapes, half as many, longer work units
//   128 x 128  twice as many work units: wins when the wide tile would leave a round mostly empty
//   64 x 128   half the flops per stage at 52 % of the time: mid-size products, and products whose K would otherwise be
//              cut into sixteen and more chunks (half the planes to write and add)
//   32 x 128   a quarter of the flops at 30 % of the time: products of a handful of rows (a 128-row tile would spend
//              most of its matrix-core work on rows that do not exist) and small products (four times as many workgroups)
#include "cn_internal.h"

namespace cn {

namespace {

struct Geometry {
    int tile_m, tile_n;
    int min_iters;     // a chunk is at least this many stages (128 k) deep
    double stage_us;   // one pipeline stage of a workgroup that shares its compute unit with another
    double unit_us;    // per work unit: first stage's latency, write-out, start of the workgroup
};
// 256 compute units at the clock the part holds under this load.
constexpr Geometry kGeometries[] = {{128, 128, 4, 3.91, 2.3}, {128, 256, 8, 3.81, 3.4}, {64, 128, 4, 2.03, 2.0}, {32, 128, 4, 1.18, 1.25}};
constexpr double kAlone = 0.57;            // a stage of a workgroup that has its compute unit to itself, relative to stage_us
constexpr double kLaunchUs = 3.3;          // a launch
constexpr double kChunkSumUs = 4.9;        // the second kernel ...
constexpr double kChunkSumUsPerMB = 0.17;  // ... and what it moves: (chunks + 1) planes at 6 TB/s (52 us for the 287 MB of the README product)
constexpr double kPlaneWriteUsPerMB = 0.15; // what writing the chunk planes costs the product itself (128 x 100000 x 8192: nine planes of 51 MB
                                           // instead of five cost 40 us more than the rounds they even out save)
constexpr double kRowsAlongMPenalty = 1.10;  // 64- and 32-row tiles of an A stored k by m read it in short pieces

struct Choice {
    double cost;
    int splits;
    int64_t ips;
};

Choice best_split(int64_t tiles, int64_t k_iters, int64_t cus, double stage_us, double unit_us, int64_t max_splits,
                  double out_bytes) {
    const int64_t slots = cus * 2;
    Choice best{0.0, 1, k_iters};
    for (int64_t s = 1; s <= max_splits; ++s) {
        int64_t ips = (k_iters + s - 1) / s;
        int64_t eff = (k_iters + ips - 1) / ips;
        if (eff != s && s != 1) continue;  // same decomposition as a smaller s
        int64_t units = tiles * eff;
        const int64_t full = units / slots, rest = units % slots;
        double cost = kLaunchUs + (double)full * ((double)ips * stage_us + unit_us);
        if (rest) cost += (double)ips * stage_us * (rest <= cus ? kAlone : 1.0) + unit_us;
        if (eff > 1) cost += kChunkSumUs + (kChunkSumUsPerMB * (double)(eff + 1) + kPlaneWriteUsPerMB * (double)eff) * out_bytes / 1.0e6;
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
    const int64_t cus = num_cu > 0 ? num_cu : 1;
    const double out_bytes = (double)M * (double)N * 4.0;
    GemmPlan best;
    double best_cost = 0.0;
    bool have = false;
    for (const Geometry &g : kGeometries) {
        // force_tile_n: 128 / 256 name the width of the 128-row tile, 32 / 64 the rows of the 128-wide one
        const int name = g.tile_m == kTileM ? g.tile_n : g.tile_m;
        if (force_tile_n != 0 && force_tile_n != name) continue;
        if (force_tile_n == 0) {
            // a tile taller than twice the product only multiplies rows that do not exist
            if (g.tile_m > kTileMLow && M <= g.tile_m / 2) continue;
        }
        const int64_t tiles_m = (M + g.tile_m - 1) / g.tile_m, tiles_n = (N + g.tile_n - 1) / g.tile_n;
        int64_t k_iters = (K + gemm_tile_k(g.tile_n) - 1) / gemm_tile_k(g.tile_n);
        if (k_iters < 1) k_iters = 1;
        const double stage_us = g.stage_us * ((g.tile_m < kTileM && !a_along_k) ? kRowsAlongMPenalty : 1.0);
        const Choice c = best_split(tiles_m * tiles_n, k_iters, cus, stage_us, g.unit_us,
                                    split_limit(k_iters, g.min_iters, out_bytes, workspace_bytes), out_bytes);
        if (!have || c.cost < best_cost) {
            have = true;
            best_cost = c.cost;
            best.tile_m = g.tile_m;
            best.tile_n = g.tile_n;
            best.tiles_m = tiles_m;
            best.tiles_n = tiles_n;
            best.k_iters = k_iters;
            best.splits = c.splits;
            best.iters_per_split = c.ips;
            best.units = tiles_m * tiles_n * c.splits;
        }
    }
    return best;
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
