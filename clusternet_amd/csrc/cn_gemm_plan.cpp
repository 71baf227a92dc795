// Host-side work decomposition for the fp32 GEMM kernels (pure function, no HIP calls).
//
// The output is cut into 128 x 128 tiles.  The batches this library serves are skinny (M = 128),
// so tiles alone cannot fill 256 compute units; K is therefore cut into `splits` chunks, every
// (chunk, tile) pair becomes one workgroup, and a second kernel adds the chunk results in a fixed
// order (deterministic, no atomics).  Chunks are ordered chunk-major so that workgroups running at
// the same time walk the same K range and share the A panel in L2.
#include "cn_internal.h"

namespace cn {

GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes) {
    GemmPlan p;
    p.tiles_m = (M + kTileM - 1) / kTileM;
    p.tiles_n = (N + kTileN - 1) / kTileN;
    p.k_iters = (K + kTileK - 1) / kTileK;
    if (p.k_iters < 1) p.k_iters = 1;
    const int64_t tiles = p.tiles_m * p.tiles_n;
    const int64_t slots = (int64_t)(num_cu > 0 ? num_cu : 1) * 2;  // two workgroups per CU

    // Cost model in units of "one K iteration of one workgroup sharing its CU with another".
    const double iter_seconds = 2.0 * 4096.0 / 2.4e9;
    const double unit_overhead = 6.0;  // pipeline fill + C write-out
    const double out_bytes = (double)M * (double)N * 4.0;

    int64_t max_splits = p.k_iters / 4;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 64) max_splits = 64;
    if (out_bytes > 0) {
        int64_t by_ws = (int64_t)((double)workspace_bytes / out_bytes);
        if (by_ws < max_splits) max_splits = by_ws;
    }
    if (max_splits < 1) max_splits = 1;

    double best_cost = 0;
    int64_t best_ips = p.k_iters;
    int best_splits = 1;
    for (int64_t s = 1; s <= max_splits; ++s) {
        int64_t ips = (p.k_iters + s - 1) / s;
        int64_t eff = (p.k_iters + ips - 1) / ips;
        if (eff != s && s != 1) continue;  // same decomposition as a smaller s
        int64_t units = tiles * eff;
        int64_t waves = (units + slots - 1) / slots;
        double cost = (double)waves * ((double)ips + unit_overhead);
        if (eff > 1) cost += (double)(eff + 1) * out_bytes / 4.0e12 / iter_seconds + 3.0;
        if (s == 1 || cost < best_cost) {
            best_cost = cost;
            best_ips = ips;
            best_splits = (int)eff;
        }
    }
    p.splits = best_splits;
    p.iters_per_split = best_ips;
    p.units = tiles * p.splits;
    return p;
}

}  // namespace cn

extern "C" void cn_host_plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes,
                                  int64_t out[6]) {
    cn::GemmPlan p = cn::plan_gemm(M, N, K, num_cu, workspace_bytes);
    out[0] = p.tiles_m;
    out[1] = p.tiles_n;
    out[2] = p.k_iters;
    out[3] = p.splits;
    out[4] = p.iters_per_split;
    out[5] = p.units;
}
