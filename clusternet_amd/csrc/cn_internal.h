// Internal declarations shared by the translation units of libcnhip.  Not part of the C-ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/cnhip.h"
#include "../../include/cnhip_hooks.h"

namespace cn {

// ---- error plumbing -------------------------------------------------------------------------
void set_error(const char *fmt, ...);
cn_status hip_fail(hipError_t e, const char *what, const char *file, int line);

#define CN_HIP(call)                                                         \
    do {                                                                     \
        hipError_t cn_e_ = (call);                                           \
        if (cn_e_ != hipSuccess) return cn::hip_fail(cn_e_, #call, __FILE__, __LINE__); \
    } while (0)

// The 126-entry codebook (exact bit patterns of the reference's table file).
void host_table(float out[126]);

// ---- per-device state ------------------------------------------------------------------------
constexpr int kTileQueues = 32;  // ticket counters of the streaming kernels, each on a 128-byte line of its own
constexpr int kTileQueueWords = kTileQueues * 32;
// Host-side table: the first kTileQueues distinct keys get slots 0, 1, ... for good; later ones get -1.
struct StreamSlots {
    const void *owner[kTileQueues] = {};
    int used = 0;
    int slot_for(const void *key) {
        for (int i = 0; i < used; ++i)
            if (owner[i] == key) return i;
        if (used == kTileQueues) return -1;
        owner[used] = key;
        return used++;
    }
};
struct Context {
    bool ready = false;
    int device = -1;
    int num_cu = 0;
    float *table = nullptr;          // 126 floats
    struct XStep *xsteps = nullptr;  // the steps of the code function (cn_xlut.h), found once at init
    int xstep_count = 0;
    struct XEntry *quotient_table = nullptr;  // the encoder's table for precision 1 (cn_encode_table.h), built once at init
    void *workspace = nullptr;       // split-K partial sums
    size_t workspace_bytes = 0;
    uint32_t *reduce_scratch = nullptr;  // per-workgroup partial results + ticket counters
    uint32_t *tickets = nullptr;         // running maximum and arrival count of the max reductions (kTicketWords words)
    double *sum_scratch = nullptr;       // per-workgroup partial sums (1024 doubles)
    uint32_t *tile_queue = nullptr;      // ticket counters of the streaming kernels (kTileQueueWords words, left at 0)
    StreamSlots tile_queue_owners;       // which launch stream holds which counter
    // The counter a kernel launched on `stream` draws its tiles from, or NULL: take the form that does not draw.  A
    // counter belongs to one stream for good, so the kernels that share it are ordered by that stream, each finding the 0
    // its predecessor left.  NULL while the stream is being captured (a graph would carry the counter into replays that
    // nothing orders against later launches) and when more streams than counters have asked.
    uint32_t *tile_counter_for(hipStream_t stream);
};
constexpr int kMaxDevices = 16;
constexpr int kReduceSlots = 4096;
// Max reductions: a running maximum and an arrival count per group of kTicketGroup workgroups and one pair for
// the groups, every pair on a 128-byte line of its own, all left at 0.
constexpr int kTicketGroup = 8;
constexpr int kTicketStride = 32;
constexpr int kTicketWords = (1 + kReduceSlots / kTicketGroup) * kTicketStride;

// A kernel's attributes (its dynamic LDS limit) are set per device: one flag per device for a call site.
struct OncePerDevice {
    bool done[kMaxDevices] = {};
    bool first(int device) {
        if (device < 0 || device >= kMaxDevices) return true;
        const bool was = done[device];
        done[device] = true;
        return !was;
    }
};

// Test switch (cn_host_reduction_fences): nonzero makes the single-launch reductions order their partial results
// with a release fence per workgroup instead of by data dependence.
extern int g_reduction_fences;

// Returns the context of the current device, initialising it on first use.
cn_status current_context(Context **out);
// The context of `device` if it is initialised, else NULL (never initialises, never allocates).
Context *ready_context(int device);

// Bytes of split-K workspace cn_init allocates (CNHIP_WORKSPACE_MB, default 1 GiB), and the figure the planner
// sees on `device`: the context's if it is initialised, else what initialisation would allocate.
size_t default_workspace_bytes();
size_t planning_workspace_bytes(int device);

// What a product needs from its surroundings: where its K-chunk partial sums go, how much of that there is, and
// the workspace size the planner is told (two entry points that plan with the same figure give the same bits).
struct GemmEnv {
    int device;
    int num_cu;
    void *workspace;
    size_t workspace_bytes;
    size_t plan_bytes;
    const float *table;  // codebook, fused variant only
};
// The partial-sum array that is part of the library's device image (cn_gemm_f32_noalloc): resolves its address
// on `device`, which must be the current device.  No allocation.
cn_status gemm_static_setup(int device);

// ---- GEMM planning (host, pure function; exported for tests) ---------------------------------
struct GemmPlan {
    int tile_m;          // output tile is tile_m x tile_n: 128 x 128, 128 x 256, or 32 x 128 / 64 x 128 for a handful of rows
    int tile_n;
    int64_t tiles_m, tiles_n, k_iters;
    int splits;          // number of K chunks (1 = write C directly)
    int64_t iters_per_split;
    int64_t units;       // tiles_m * tiles_n * splits = grid size
};
// force_tile_n: 0 = choose, 128 or 256 = use that tile width, 32 / 64 = use the 32 x 128 / 64 x 128 tile.
// C = sum of `splits` M x N planes held at the start of the workspace (ascending order); optional max |C|.
cn_status add_chunk_planes(const void *planes, int num_cu, int splits, int64_t M, int64_t N, float *C, int64_t ldc,
                           uint32_t *amax, hipStream_t st);

// The product on 8-bit weights for up to 1024 rows (cn_gemm_w8_rows.hip): number of K chunks if it applies, else 0;
// with more than one chunk the planes land at the start of `workspace` for add_chunk_planes.
int gemm_w8_rows_splits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W, int64_t ldw,
                        float scale, const float *C, int64_t ldc, int num_cu, size_t workspace_bytes);
cn_status gemm_w8_rows(int splits, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W, int64_t ldw,
                       float scale, float *C, int64_t ldc, const float *table, void *workspace, int device, hipStream_t st);

// The product in one launch for shapes too small to fill the chip with tiles (cn_gemm_small.hip): a workgroup per
// 32 x 32 block of the result, K split among its wavefronts.
constexpr int64_t kSmallMaxBlocks = 256;           // of 32 x 32 results: a workgroup per compute unit (288 of them lost to the tiled kernel: 18.0 us against 11.6)
constexpr int64_t kSmallMaxWork = (int64_t)1 << 28;  // M * N * K; half of it where the blocks are 16 x 16
bool gemm_small_applies(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                        int64_t ldb);
// amax: NULL, or a word that starts at 0 and receives the bit pattern of max |C|.
cn_status gemm_small(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                     int64_t ldb, float *C, int64_t ldc, uint32_t *amax, hipStream_t st);

// a_along_k: A is stored m by k (dot, dotT), which lets products with many K chunks take 64-row tiles.
GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, int num_cu, size_t workspace_bytes, int force_tile_n, bool a_along_k);

constexpr int kTileM = 128;
constexpr int kTileMLow = 32;      // rows of the tile for products with a handful of rows or little work
constexpr int kTileMMid = 64;      // rows of the tile for products of 33 .. 64 rows
constexpr int kLowTileMaxRows = 64;  // largest M that takes one of the two unasked
// K depth of one pipeline stage for a tile width (iters in a GemmPlan count these).
constexpr int gemm_tile_k(int tile_n) { return tile_n == 256 ? 16 : 32; }

}  // namespace cn
