// fp32 GEMM for gfx950 on the matrix cores: C = op(A) op(B), row-major, alpha 1, beta 0, and the
// fused variant whose B operand is 8-bit codes.
//
// One kernel template, gemm_kernel<A_KC, B_KIND, TN, TM>, 256 lanes = 4 wavefronts, at least two workgroups
// per compute unit, in three geometries (TM x TN output tiles):
//   128 x 128 output tile 128 x 128, wavefronts 2 x 2, each 64 x 64 = 2 x 2 blocks of
//             v_mfma_f32_32x32x2_f32 (64 accumulators per lane); K advances 32 per stage through two
//             LDS stages (64 KiB)
//   128 x 256 output tile 128 x 256, wavefronts 1 x 4, each 128 x 64 = 4 x 2 blocks (128 accumulators
//             per lane); K advances 16 per stage through two LDS stages (48 KiB).  The A
//             tile is fetched once per 256 output columns and every B fragment read from LDS feeds four
//             MFMAs instead of two: less L2 -> LDS and LDS -> register traffic per flop, which matters
//             because the part runs power-limited on realistic data
//   32 x 128  for products with no more than 32 rows (a batch of 32 against 8-bit weights) and for products
//             too small to fill the machine with larger tiles (64 x 128, two blocks per wavefront, for 33 to
//             64 rows): wavefronts
//             1 x 4, one 32 x 32 block each; K advances 32 per stage through three LDS stages (60 KiB), two of
//             them in flight.  A 128-row tile would spend
//             three quarters of its MFMAs on rows that do not exist; with this one such a product costs
//             its pass over B
// Common to both:
//   * one barrier per stage; the global loads of the next stage are issued before the MFMAs of the
//     current one; the barrier sits eight MFMAs before the end of a stage
//   * fp32 tiles go from global memory straight into LDS with buffer_load_dwordx4 ... lds, 1 KiB
//     per wavefront instruction: no staging registers, no LDS store instructions.  An operand
//     whose memory is contiguous along k (A of dot/dotT, B of dotT) sits in LDS as [index][k], its
//     16-byte columns XOR-swizzled by the row (applied on the global-address side), and feeds four
//     MFMAs per 16-byte LDS read; an operand contiguous along its row/column index (A of Tdot, B
//     of dot/Tdot) sits as [k][index] and is read one value per MFMA with conflict-free 4-byte
//     LDS reads
//   * rows or columns of a ragged tile that lie outside the matrix are loaded like any other: they
//     only ever feed outputs outside the matrix, which are not stored, and the buffer descriptor's
//     range check turns addresses past the end of the matrix into zeros instead of memory accesses
//   * 8-bit codes of the fused variant are read in coalesced 4-byte words along n, expanded through
//     a 256-entry LDS table (the decode table of the stand-alone decompression kernel, bit for bit)
//     and stored as fp32 into the same [k][n] LDS image, so the MFMA side does not change
//   * the last, partial K stage and operands that do not allow 16-byte loads take a predicated
//     register path (zero-filled) into the same LDS images
//   * K may be split into chunks (one workgroup per chunk and tile); chunk results go to a
//     workspace and a second kernel adds them in a fixed order
//   * block ids are remapped so that the workgroups an XCD receives (ids congruent mod 8) cover a
//     contiguous range of work units and share their A/B panels in that XCD's L2
//   * global addresses are a uniform buffer descriptor (scalar registers) plus a 32-bit per-lane
//     byte offset, which is why leading dimensions are limited to 2^22 elements.
#include <mutex>

#include "cn_internal.h"

namespace cn {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

// Buffer descriptor with its origin at `p`, no stride, no range check (for accesses that are
// individually predicated).  0x00020000 = 32-bit untyped data format.
__device__ __forceinline__ rsrc_t make_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, 0xffffffff, 0x00020000);
}

constexpr int NT = 256;  // lanes per workgroup
constexpr int NW = 4;    // wavefronts per workgroup
constexpr int kNumXcd = 8;
constexpr int kPersistentFromRounds = 3;   // rounds of resident workgroups from which an unsplit product keeps its workgroups ...
constexpr int kPersistentMaxStages = 32;   // ... if a tile has no more stages than this

// What the B operand is.
enum BKind { B_IC = 0 /* fp32 [k][n] */, B_KC = 1 /* fp32 [n][k] */, B_CODES = 2 /* uint8 [k][n] */ };

// Geometry of a tile width: wavefront grid WM x WN, FM x FN 32 x 32 blocks per wavefront, K depth
// of a stage, LDS stages.
template <int TM, int TN> struct Geo;
template <> struct Geo<128, 128> { static constexpr int WM = 2, WN = 2, FM = 2, FN = 2, BK = 32, NST = 2; };
template <> struct Geo<128, 256> { static constexpr int WM = 1, WN = 4, FM = 4, FN = 2, BK = 16, NST = 2; };
template <> struct Geo<32, 128> { static constexpr int WM = 1, WN = 4, FM = 1, FN = 1, BK = 32, NST = 3; };
template <> struct Geo<64, 128> { static constexpr int WM = 1, WN = 4, FM = 2, FN = 1, BK = 32, NST = 3; };
static_assert(gemm_tile_k(128) == Geo<128, 128>::BK && gemm_tile_k(256) == Geo<128, 256>::BK &&
                  gemm_tile_k(128) == Geo<kTileMLow, 128>::BK && gemm_tile_k(128) == Geo<kTileMMid, 128>::BK &&
                  kTileM == 128 && kTileMLow == 32 && kTileMMid == 64,
              "planner and kernel disagree");

struct GemmArgs {
    const float *A;
    const void *B;       // float (plain) or uint8_t codes (fused)
    float *C;
    float *partial;      // [splits][M][N] when splits > 1
    int64_t M, N, K, lda, ldb, ldc;
    int64_t tiles_n, tiles, k_iters, iters_per_split;
    uint32_t units;
    int splits;
    int vec_a, vec_b;    // operand base and leading dimension allow 16-byte (fp32) / 4-byte (codes) loads
    float scale;         // fused: decode scale
    const float *table;  // fused: 126-entry codebook
    uint32_t *amax;      // optional: receives max |C| as the bit pattern of a non-negative float
    uint32_t *tile_counter;  // persistent form: the counter its workgroups draw their tiles from (0 between kernels), or NULL
    int units_in_order;  // work units in block-id order (one window of C in flight) instead of a contiguous slice per XCD
    int wide_store;      // the destination of the write-out (C, or the partial planes) allows 16-byte stores
    // What the write-out does instead of storing C when the kernel is instantiated with an epilogue (whole tiles
    // only, K not split): bias + maxout over epi_pool consecutive columns into epi_out / epi_arg_out (M x N / pool),
    // or the expansion of the product (M x N) to the winners' columns epi_arg_in names, into epi_out (M x N pool).
    const float *epi_bias;
    const float *epi_arg_in;
    float *epi_out;
    float *epi_arg_out;
    int epi_pool;
};
enum Epilogue { EPI_NONE = 0, EPI_BIAS_MAXOUT = 1, EPI_EXPAND = 2 };

// max over the wavefront of a non-negative float's bit pattern, then one atomic per wavefront.
// Bit patterns of non-negative floats order like the floats, so the unsigned maximum is exact and
// independent of the order of the updates.
__device__ __forceinline__ void publish_absmax(uint32_t v, uint32_t *amax) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
        v = o > v ? o : v;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(amax, v);
}

// LDS image of one operand tile (ROWS index values x BK k; ROWS = 128 for A, TN for B):
//   KC (memory [index][k]): float offset lds_offset(index, k / 4) + k % 4   (swizzled 16-byte columns)
//   IC (memory [k][index]): float offset k * ROWS + index
// The swizzle makes the 16-byte reads of consecutive rows at one k quad hit different 16-byte bank groups, for
// eight consecutive rows over 128 bytes of banks and for sixteen over 256 bytes (the LDS of this part serves
// 16-byte reads sixteen lanes at a time: with a swizzle that only separated eight rows, the counters showed a
// third of the LDS cycles of the 64-byte-row tile as bank conflicts).  Rows are 128 bytes (BK 32) or 64 bytes
// (BK 16) apart.
template <int BK>
__device__ __forceinline__ int swizzle_of(int row) {
    return BK == 32 ? ((row & 7) ^ ((row >> 3) & 3)) : (((row >> 1) & 3) ^ ((row >> 3) & 1));
}
template <int BK>
__device__ __forceinline__ int lds_offset(int row, int quad) {
    return row * BK + ((quad ^ swizzle_of<BK>(row)) << 2);
}

// ---- direct global -> LDS loads ------------------------------------------------------------------
// A wavefront fills a tile 1 KiB at a time: block b = 4 j + wave is 256 / BK consecutive rows of a KC
// tile or 256 / ROWS consecutive k rows of an IC tile; lane l supplies bytes 16 l .. 16 l + 15 of it.
template <bool KC, int ROWS, int BK>
struct DirectLoader {
    static constexpr int J = ROWS * BK / 256 / NW;  // blocks per wavefront
    uint32_t off[J];  // byte offset of this lane's 16 bytes of block 4 j + wave from the tile corner
    __device__ __forceinline__ void init(int64_t ld, int wave) {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int blk = NW * j + wave;
            if (KC) {
                constexpr int kQuads = BK / 4;  // lanes per row: 8 or 4
                const int row = blk * (64 / kQuads) + lane / kQuads;
                const int quad = (lane % kQuads) ^ swizzle_of<BK>(row);
                off[j] = (uint32_t)((row * ld + 4 * quad) * 4);
            } else {
                constexpr int kLanesPerRow = ROWS / 4;  // 32 or 64
                const int k = blk * (64 / kLanesPerRow) + lane / kLanesPerRow;
                off[j] = (uint32_t)((k * ld + 4 * (lane % kLanesPerRow)) * 4);
            }
        }
    }
    // The loads are written as inline assembly on purpose: the compiler's wait-count insertion
    // treats every LDS read that follows a compiler-visible LDS-writing load as dependent on it and
    // would wait for the whole next stage before the first MFMA of the current one.  Completion is
    // awaited explicitly (vmcnt) before the barrier that publishes the stage.
    // `limit` = bytes from the corner to the end of the matrix: the descriptor's range check makes
    // every access at or beyond it return zero instead of touching memory.
    __device__ __forceinline__ void issue(const void *corner, uint32_t limit, float *lds_stage, int wave) const {
        const uint64_t addr = reinterpret_cast<uint64_t>(corner);
        const u32x4 rsrc = {(uint32_t)addr, (uint32_t)(addr >> 32) & 0xffffu, limit, 0x00020000u};
        const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(
            (__attribute__((address_space(3))) float *)lds_stage) + (uint32_t)wave * 1024u;
#pragma unroll
        for (int j = 0; j < J; ++j)
            asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                         :
                         : "s"(lds0 + (uint32_t)(j * NW) * 1024u), "v"(off[j]), "s"(rsrc)
                         : "memory", "m0");
    }
};

// ---- predicated register paths (partial K stage, unaligned operands) ---------------------------------
// KC operand of ROWS rows: lane t covers k quad t % (BK / 4) of rows t / (BK / 4) + RB j.
template <int ROWS, int BK>
struct GuardedKC {
    static constexpr int KQ = BK / 4, RB = NT / KQ, J = ROWS / RB;
    static_assert(J <= 4, "register staging holds four vectors");
    uint32_t off[J];
    uint32_t ok;  // bit j: row of load j is inside the matrix
    int kfirst;
    __device__ __forceinline__ void init(int64_t ld, int64_t index0, int64_t indices) {
        const int kq = threadIdx.x % KQ, rb = threadIdx.x / KQ;
        kfirst = 4 * kq;
        ok = 0;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            off[j] = (uint32_t)(((rb + RB * j) * ld + 4 * kq) * 4);
            if (index0 + rb + RB * j < indices) ok |= 1u << j;
        }
    }
    __device__ __forceinline__ void load(rsrc_t base, int64_t kleft, f32x4 (&reg)[4]) const {
#pragma unroll
        for (int j = 0; j < J; ++j) {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (ok & (1u << j)) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (kfirst + e < kleft)
                        v[e] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(base, off[j] + 4 * e, 0, 0));
            }
            reg[j] = v;
        }
    }
    __device__ __forceinline__ void store(float *__restrict__ lds, const f32x4 (&reg)[4]) const {
        const int kq = threadIdx.x % KQ, rb = threadIdx.x / KQ;
#pragma unroll
        for (int j = 0; j < J; ++j) *reinterpret_cast<f32x4 *>(lds + lds_offset<BK>(rb + RB * j, kq)) = reg[j];
    }
};

// IC operand of ROWS indices, fp32 or codes: lane t covers indices 4 (t % (ROWS / 4)) .. + 3 of
// k rows t / (ROWS / 4) + KR r.
template <int ROWS, int BK>
struct GuardedIC {
    static constexpr int CQ = ROWS / 4, KR = NT / CQ, R = BK / KR;
    static_assert(R <= 4, "register staging holds four vectors");
    uint32_t off[R];  // byte offsets for an element size of `elem`
    uint32_t ok;      // bit e: index 4 cq + e is inside the matrix
    __device__ __forceinline__ void init(int64_t ld, int64_t index0, int64_t indices, int elem) {
        const int cq = threadIdx.x % CQ, kr = threadIdx.x / CQ;
        ok = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) off[r] = (uint32_t)(((kr + KR * r) * ld + 4 * cq) * elem);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (index0 + 4 * cq + e < indices) ok |= 1u << e;
    }
    __device__ __forceinline__ void load(rsrc_t base, int64_t kleft, f32x4 (&reg)[4]) const {
        const int kr = threadIdx.x / CQ;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (kr + KR * r < kleft) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (ok & (1u << e))
                        v[e] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(base, off[r] + 4 * e, 0, 0));
            }
            reg[r] = v;
        }
    }
    __device__ __forceinline__ void store(float *__restrict__ lds, const f32x4 (&reg)[4]) const {
        const int cq = threadIdx.x % CQ, kr = threadIdx.x / CQ;
#pragma unroll
        for (int r = 0; r < R; ++r) *reinterpret_cast<f32x4 *>(lds + (kr + KR * r) * ROWS + 4 * cq) = reg[r];
    }
    // Codes: four per 32-bit word.  `whole` = aligned words inside the matrix and inside K.
    __device__ __forceinline__ void load_codes(rsrc_t base, int64_t kleft, bool whole, uint32_t (&reg)[4]) const {
        const int kr = threadIdx.x / CQ;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (whole) {
                reg[r] = __builtin_amdgcn_raw_buffer_load_b32(base, off[r], 0, 0);
            } else {
                uint32_t w = 0;
                if (kr + KR * r < kleft) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (ok & (1u << e))
                            w |= (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(base, off[r] + e, 0, 0) << (8 * e);
                }
                reg[r] = w;
            }
        }
    }
    // Expand through the decode table.  Rows at or beyond K must contribute exactly zero whatever
    // code 0 decodes to; columns beyond N only reach outputs that are not stored.
    __device__ __forceinline__ void store_codes(float *__restrict__ lds, const float *__restrict__ lut,
                                                const uint32_t (&reg)[4], int64_t kleft, int r_begin = 0,
                                                int r_end = R) const {
        const int cq = threadIdx.x % CQ, kr = threadIdx.x / CQ;
#pragma unroll
        for (int r = r_begin; r < r_end; ++r) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = lut[(reg[r] >> (8 * e)) & 0xffu];
            if (kr + KR * r >= kleft) v = f32x4{0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<f32x4 *>(lds + (kr + KR * r) * ROWS + 4 * cq) = v;
        }
    }
};

template <bool A_KC, int B_KIND, int TN, int TM, int EPI = EPI_NONE>
__global__ __launch_bounds__(NT, 2) void gemm_kernel(GemmArgs g) {
    using G = Geo<TM, TN>;
    constexpr int BM = TM;
    constexpr bool B_IS_KC = (B_KIND == B_KC);
    constexpr bool kCodes = (B_KIND == B_CODES);
    constexpr int BN = TN, BK = G::BK, NST = G::NST, FM = G::FM, FN = G::FN;
    constexpr int kGroups = BK / 8;      // groups of 8 k per stage, 4 FM FN MFMAs each
    constexpr int kAStage = BM * BK;     // floats of one A stage
    constexpr int kBStage = TN * BK;     // floats of one B stage
    static_assert(G::WM * G::WN == NW && G::WM * FM * 32 == BM && G::WN * FN * 32 == TN, "geometry");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *sA = smem;                                  // [NST][kAStage]
    float *sB = smem + NST * kAStage;                  // [NST][kBStage]
    float *sLut = smem + NST * (kAStage + kBStage);    // [256], fused only

    // Work unit of this workgroup.  Hardware hands consecutive block ids to the XCDs round-robin;
    // give XCD x the x-th contiguous slice of the unit range (or, units_in_order, take the block id itself).
    const uint32_t bid = blockIdx.x, U = g.units;
    const uint32_t xcd = bid % kNumXcd, idx = bid / kNumXcd;
    const uint32_t per = U / kNumXcd, rem = U % kNumXcd;
    const uint32_t unit = g.units_in_order ? bid : xcd * per + (xcd < rem ? xcd : rem) + idx;
    // 32-bit unit arithmetic, then pinned to scalar registers: everything derived from these
    // (tile corners, buffer descriptors) must stay wave-uniform.
    const uint32_t tiles32 = (uint32_t)g.tiles, tiles_n32 = (uint32_t)g.tiles_n;
    const uint32_t split_v = unit / tiles32, tile_v = unit - split_v * tiles32;
    // Tiles of 128 rows go row of tiles by row of tiles (neighbours share their A panel; the B panels of a
    // chunk are shared through the L2 and the Infinity Cache).  The 32-row tiles of a product are few in m and
    // there to be cheap in B traffic, so there the tiles of one B panel are neighbours.
    uint32_t tm_v, tn_v;
    if (TM == kTileM) {
        tm_v = tile_v / tiles_n32;
        tn_v = tile_v - tm_v * tiles_n32;
    } else {
        const uint32_t tiles_m32 = tiles32 / tiles_n32;
        tn_v = tile_v / tiles_m32;
        tm_v = tile_v - tn_v * tiles_m32;
    }
    const int64_t split = __builtin_amdgcn_readfirstlane((int)split_v);
    const int64_t tm = __builtin_amdgcn_readfirstlane((int)tm_v);
    const int64_t tn = __builtin_amdgcn_readfirstlane((int)tn_v);
    const int64_t m0 = tm * BM, n0 = tn * BN;
    const int it0 = (int)(split * g.iters_per_split);
    int it1 = it0 + (int)g.iters_per_split;
    if (it1 > (int)g.k_iters) it1 = (int)g.k_iters;

    if (kCodes) {
        // decode table, built exactly as the stand-alone decompression kernel builds it
        const int t = threadIdx.x;
        if (t < 126) {
            float v = g.table[t] * g.scale;
            sLut[t] = v;
            sLut[t + 128] = -v;
        } else if (t == 126) {
            sLut[126] = g.scale;
            sLut[127] = g.scale;
            sLut[254] = g.scale;
            sLut[255] = -g.scale;
        }
        __syncthreads();
    }

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave_m = wave / G::WN, wave_n = wave % G::WN;
    const int half = lane >> 5, l32 = lane & 31;
    int row_a[FM], row_b[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) row_a[i] = wave_m * (32 * FM) + i * 32 + l32;
#pragma unroll
    for (int i = 0; i < FN; ++i) row_b[i] = wave_n * (32 * FN) + i * 32 + l32;

    f32x16 acc[FM][FN];
#pragma unroll
    for (int mi = 0; mi < FM; ++mi)
#pragma unroll
        for (int ni = 0; ni < FN; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    const float *Bf = reinterpret_cast<const float *>(g.B);
    const uint8_t *Bc = reinterpret_cast<const uint8_t *>(g.B);
    // One past the last element that may be read, as an element offset from the matrix base.  An
    // index-contiguous operand is read in aligned groups of four, hence the round-up.
    const int64_t end_a = A_KC ? (g.M - 1) * g.lda + g.K : (g.K - 1) * g.lda + ((g.M + 3) & ~(int64_t)3);
    const int64_t end_b = B_IS_KC ? (g.N - 1) * g.ldb + g.K : (g.K - 1) * g.ldb + ((g.N + 3) & ~(int64_t)3);

    DirectLoader<A_KC, BM, BK> da;
    DirectLoader<B_IS_KC, TN, BK> db;
    da.init(g.lda, wave);
    if (!kCodes) db.init(g.ldb, wave);
    GuardedKC<BM, BK> ga_kc;
    GuardedKC<TN, BK> gb_kc;
    GuardedIC<BM, BK> ga_ic;
    GuardedIC<TN, BK> gb_ic;
    if (A_KC) ga_kc.init(g.lda, m0, g.M); else ga_ic.init(g.lda, m0, g.M, 4);
    if (B_IS_KC) gb_kc.init(g.ldb, n0, g.N); else gb_ic.init(g.ldb, n0, g.N, kCodes ? 1 : 4);

    // Corner addresses of stage `it` (uniform across the workgroup).
    auto corner_a = [&](int it) { return A_KC ? g.A + m0 * g.lda + (int64_t)it * BK : g.A + (int64_t)it * BK * g.lda + m0; };
    auto corner_b = [&](int it) { return B_IS_KC ? Bf + n0 * g.ldb + (int64_t)it * BK : Bf + (int64_t)it * BK * g.ldb + n0; };
    auto corner_c = [&](int it) { return Bc + (int64_t)it * BK * g.ldb + n0; };
    auto limit_of = [](const float *base, int64_t end, const float *corner) {
        const int64_t bytes = (end - (corner - base)) * 4;
        return bytes <= 0 ? 0u : (bytes > 0xffffffffLL ? 0xffffffffu : (uint32_t)bytes);
    };

    // Fragments of one group of 8 k.  MFMA s (0..3) of the group consumes k = 8 g + 4 h + s from lane
    // half h on both operands, i.e. the k order inside a stage is permuted identically for A and B.
    auto load_frag = [&](const float *pa, const float *pb, int gq, f32x4 (&a)[FM], f32x4 (&b)[FN]) {
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (A_KC) {
                a[i] = *reinterpret_cast<const f32x4 *>(pa + lds_offset<BK>(row_a[i], 2 * gq + half));
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) a[i][s] = pa[(8 * gq + 4 * half + s) * BM + row_a[i]];
            }
        }
#pragma unroll
        for (int i = 0; i < FN; ++i) {
            if (B_IS_KC) {
                b[i] = *reinterpret_cast<const f32x4 *>(pb + lds_offset<BK>(row_b[i], 2 * gq + half));
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) b[i][s] = pb[(8 * gq + 4 * half + s) * TN + row_b[i]];
            }
        }
    };
    auto mfma_steps = [&](const f32x4 (&a)[FM], const f32x4 (&b)[FN], int s_begin, int s_end) {
#pragma unroll
        for (int s = s_begin; s < s_end; ++s)
#pragma unroll
            for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                for (int ni = 0; ni < FN; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi][s], b[ni][s], acc[mi][ni], 0, 0, 0);
    };
    // MFMA steps of the last group that are issued behind the barrier: eight MFMAs.
    constexpr int kTailFrom = FM * FN >= 2 ? 4 - 8 / (FM * FN) : 0;

    // Stages [it0, it_direct) use the direct loads (operands allow 16-byte / 4-byte accesses and the
    // stage lies inside K); the rest, if any, goes through predicated registers.
    // A ragged tile of codes (columns beyond N) is read byte by byte under conditions: predicated path.
    const bool whole_n = (n0 + BN <= g.N);
    int it_direct = it0;
    if (g.vec_a && g.vec_b && (!kCodes || whole_n)) {
        const int full = (int)(g.K / BK);
        it_direct = it1 < full ? it1 : full;
        if (it_direct < it0) it_direct = it0;
    }

    auto issue_stage = [&](int it, int slot) {
        da.issue(corner_a(it), limit_of(g.A, end_a, corner_a(it)), sA + slot * kAStage, wave);
        if (!kCodes) db.issue(corner_b(it), limit_of(Bf, end_b, corner_b(it)), sB + slot * kBStage, wave);
    };
    f32x4 a0[FM], b0[FN], a1[FM], b1[FN];
    // The MFMAs of one stage up to the last eight.  Fragment reads are left to the compiler's schedule
    // (just ahead of their MFMAs; the other workgroup on the compute unit covers their latency); the
    // register sets alternate.  The barrier that publishes the next stage sits eight MFMAs before the
    // end of a stage so that it is waited for in their shadow.
    auto stage_head = [&](const float *pa, const float *pb) {
        if (kGroups == 4) {
            load_frag(pa, pb, 0, a0, b0); mfma_steps(a0, b0, 0, 4);
            load_frag(pa, pb, 1, a1, b1); mfma_steps(a1, b1, 0, 4);
            load_frag(pa, pb, 2, a0, b0); mfma_steps(a0, b0, 0, 4);
            load_frag(pa, pb, 3, a1, b1); mfma_steps(a1, b1, 0, kTailFrom);
        } else {
            load_frag(pa, pb, 0, a0, b0); mfma_steps(a0, b0, 0, 4);
            load_frag(pa, pb, 1, a1, b1); mfma_steps(a1, b1, 0, kTailFrom);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // The same with a set of codes expanded into the LDS stage `pn` in four parts between the MFMA groups,
    // where the table look-ups and LDS stores cost nothing: the matrix pipe is busy anyway.
    auto stage_head_expanding = [&](const float *pa, const float *pb, float *pn, const uint32_t (&rc)[4]) {
        static_assert(!kCodes || GuardedIC<TN, BK>::R == 4, "four parts");
        if (kGroups == 4) {
            load_frag(pa, pb, 0, a0, b0); mfma_steps(a0, b0, 0, 4);         gb_ic.store_codes(pn, sLut, rc, BK, 0, 1);
            load_frag(pa, pb, 1, a1, b1); mfma_steps(a1, b1, 0, 4);         gb_ic.store_codes(pn, sLut, rc, BK, 1, 2);
            load_frag(pa, pb, 2, a0, b0); mfma_steps(a0, b0, 0, 4);         gb_ic.store_codes(pn, sLut, rc, BK, 2, 3);
            load_frag(pa, pb, 3, a1, b1); mfma_steps(a1, b1, 0, kTailFrom); gb_ic.store_codes(pn, sLut, rc, BK, 3, 4);
        } else {
            load_frag(pa, pb, 0, a0, b0); mfma_steps(a0, b0, 0, 4);         gb_ic.store_codes(pn, sLut, rc, BK, 0, 2);
            load_frag(pa, pb, 1, a1, b1); mfma_steps(a1, b1, 0, kTailFrom); gb_ic.store_codes(pn, sLut, rc, BK, 2, 4);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    if (NST == 2 && !kCodes && it0 < it_direct) {
        issue_stage(it0, 0);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the stage has landed in LDS
        __syncthreads();
        int slot = 0;
        for (int it = it0; it < it_direct; ++it) {
            const int slot_next = slot ^ 1;
            if (it + 1 < it_direct) issue_stage(it + 1, slot_next);  // lands in the other stage while this one is consumed
            stage_head(sA + slot * kAStage, sB + slot * kBStage);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // stage it + 1 has landed
            __syncthreads();
            mfma_steps(a1, b1, kTailFrom, 4);
            __builtin_amdgcn_sched_barrier(0);
            slot = slot_next;
        }
    }

    if (NST == 2 && kCodes && it0 < it_direct) {
        // Codes are requested two stages ahead into two register sets that alternate, and the set of stage
        // it + 1 is expanded into the other LDS stage between the MFMA groups of stage it.  The A tile of stage
        // it + 1 is requested right behind the barrier that frees its LDS stage.  Code loads past the last
        // stage get a range of zero bytes instead of being skipped (straight-line code, see the three-stage
        // loop below); what they "decode" lands in a stage that is not read again.
        constexpr int kCodeLoads = GuardedIC<TN, BK>::R;
        auto codes_ahead = [&](int it, uint32_t (&rc)[4]) {
            // the descriptor is the same for every lane: say so, or each load is wrapped in a loop over lanes
            const uint64_t corner = reinterpret_cast<uint64_t>(corner_c(it));
            const uint64_t uniform = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(corner >> 32)) << 32) |
                                     (uint32_t)__builtin_amdgcn_readfirstlane((int)corner);
            const int range = __builtin_amdgcn_readfirstlane(it < it_direct ? -1 : 0);
            const rsrc_t codes_of_stage = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<uint8_t *>(uniform), 0, range, 0x00020000);
            gb_ic.load_codes(codes_of_stage, BK, true, rc);
        };
        auto issue_a = [&](int it, int slot) {
            da.issue(corner_a(it), limit_of(g.A, end_a, corner_a(it)), sA + slot * kAStage, wave);
        };
        uint32_t rc_even[4], rc_odd[4];
        codes_ahead(it0, rc_even);
        codes_ahead(it0 + 1, rc_odd);
        issue_a(it0, 0);
        gb_ic.store_codes(sB, sLut, rc_even, BK);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (it0 + 1 < it_direct) issue_a(it0 + 1, 1);
        int slot = 0;
        // rc_ready holds the codes of stage it + 1, rc_next receives those of stage it + 2
        auto step = [&](int it, uint32_t (&rc_ready)[4], uint32_t (&rc_next)[4]) {
            const int slot_next = slot ^ 1;
            const float *pa = sA + slot * kAStage, *pb = sB + slot * kBStage;
            float *pn = sB + slot_next * kBStage;
            codes_ahead(it + 2, rc_next);
            stage_head_expanding(pa, pb, pn, rc_ready);
            // the A tile of stage it + 1 has landed: only the code loads of stage it + 2 are younger
            __builtin_amdgcn_s_waitcnt(0x0f70 | kCodeLoads);
            __syncthreads();
            if (it + 2 < it_direct) issue_a(it + 2, slot);  // every wavefront is done reading this stage
            mfma_steps(a1, b1, kTailFrom, 4);
            __builtin_amdgcn_sched_barrier(0);
            slot = slot_next;
        };
        int it = it0;
        for (int pairs = (it_direct - it0) >> 1; pairs > 0; --pairs, it += 2) {
            step(it, rc_odd, rc_even);
            step(it + 1, rc_even, rc_odd);
        }
        if ((it_direct - it0) & 1) step(it, rc_odd, rc_even);
        __builtin_amdgcn_s_waitcnt(0x0f70);
    }

    if (NST == 3 && it0 < it_direct) {
        // Three LDS stages, two in flight: a tile of few rows has little to compute per stage, so what
        // bounds it is how much of B is on its way.  Codes are held in two register sets, the one of
        // stage it + 1 being expanded into LDS while the one of stage it + 2 is still arriving.
        // Every step issues the same kStageLoads load instructions, past the last stage with a range of
        // zero bytes (such loads return zeros and touch no memory): straight-line code, so that the waits
        // can count.  "At most kStageLoads outstanding" then means that everything but the newest stage
        // has arrived.
        constexpr int kStageLoads = DirectLoader<A_KC, BM, BK>::J + (kCodes ? GuardedIC<TN, BK>::R : DirectLoader<B_IS_KC, TN, BK>::J);
        static_assert(kStageLoads < 16, "wait-count immediate");
        auto issue_ahead = [&](int it, int slot, uint32_t (&rc)[4]) {
            const bool live = it < it_direct;
            da.issue(corner_a(it), live ? limit_of(g.A, end_a, corner_a(it)) : 0u, sA + slot * kAStage, wave);
            if (kCodes) {
                const rsrc_t codes_of_stage = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(corner_c(it)), 0,
                                                                                live ? 0xffffffff : 0, 0x00020000);
                gb_ic.load_codes(codes_of_stage, BK, true, rc);
            } else {
                db.issue(corner_b(it), live ? limit_of(Bf, end_b, corner_b(it)) : 0u, sB + slot * kBStage, wave);
            }
        };
        uint32_t rc_even[4], rc_odd[4];
        issue_ahead(it0, 0, rc_even);
        issue_ahead(it0 + 1, 1, rc_odd);
        if (kCodes) gb_ic.store_codes(sB, sLut, rc_even, BK);
        __builtin_amdgcn_s_waitcnt(0x0f70 | kStageLoads);
        __syncthreads();
        int slot = 0;
        // rc_next receives the codes of stage it + 2, rc_ready holds those of stage it + 1
        auto step = [&](int it, uint32_t (&rc_ready)[4], uint32_t (&rc_next)[4]) {
            const int slot1 = slot == 2 ? 0 : slot + 1, slot2 = slot1 == 2 ? 0 : slot1 + 1;
            issue_ahead(it + 2, slot2, rc_next);  // into the stage that was consumed last
            if (kCodes) stage_head_expanding(sA + slot * kAStage, sB + slot * kBStage, sB + slot1 * kBStage, rc_ready);
            else        stage_head(sA + slot * kAStage, sB + slot * kBStage);
            __builtin_amdgcn_s_waitcnt(0x0f70 | kStageLoads);  // stage it + 1 has landed
            __syncthreads();
            mfma_steps(a1, b1, kTailFrom, 4);
            __builtin_amdgcn_sched_barrier(0);
            slot = slot1;
        };
        // whole pairs of steps in the loop, so that the register sets are in the same state every time
        // round; an odd stage at the end on its own
        int it = it0;
        for (int pairs = (it_direct - it0) >> 1; pairs > 0; --pairs, it += 2) {
            step(it, rc_odd, rc_even);
            step(it + 1, rc_even, rc_odd);
        }
        if ((it_direct - it0) & 1) step(it, rc_odd, rc_even);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // the zero-range loads behind the last stage
        __syncthreads();
    }

    if (it_direct < it1) {
        // Predicated path: global -> registers (zero-filled outside the matrix) -> LDS, stage in
        // flight while the previous one is consumed.  Same LDS images as above, stages 0 and 1.
        f32x4 ra[4], rb[4];
        uint32_t rc[4];
        auto fetch = [&](int it) {
            const int64_t kleft = g.K - (int64_t)it * BK;
            if (A_KC) ga_kc.load(make_rsrc(corner_a(it)), kleft, ra); else ga_ic.load(make_rsrc(corner_a(it)), kleft, ra);
            if (kCodes)       gb_ic.load_codes(make_rsrc(corner_c(it)), kleft, false, rc);
            else if (B_IS_KC) gb_kc.load(make_rsrc(corner_b(it)), kleft, rb);
            else              gb_ic.load(make_rsrc(corner_b(it)), kleft, rb);
        };
        auto stash = [&](int it, int buf) {
            const int64_t kleft = g.K - (int64_t)it * BK;
            if (A_KC) ga_kc.store(sA + buf * kAStage, ra); else ga_ic.store(sA + buf * kAStage, ra);
            if (kCodes)       gb_ic.store_codes(sB + buf * kBStage, sLut, rc, kleft);
            else if (B_IS_KC) gb_kc.store(sB + buf * kBStage, rb);
            else              gb_ic.store(sB + buf * kBStage, rb);
        };
        fetch(it_direct);
        stash(it_direct, 0);
        __syncthreads();
        int buf = 0;
        for (int it = it_direct; it < it1; ++it) {
            const bool more = (it + 1 < it1);
            if (more) fetch(it + 1);
            const float *pa = sA + buf * kAStage, *pb = sB + buf * kBStage;
            f32x4 a[FM], b[FN];
#pragma unroll
            for (int gq = 0; gq < kGroups; ++gq) {
                load_frag(pa, pb, gq, a, b);
                mfma_steps(a, b, 0, 4);
            }
            if (more) stash(it + 1, buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

    // Write-out.  Accumulator r of a lane holds row 8 (r / 4) + 4 half + (r % 4), column l32 of its
    // 32 x 32 block: for a fixed r the 32 lanes of a half write 128 contiguous bytes.
    float *dst;
    int64_t ldd;
    if (g.splits > 1) { dst = g.partial + (int64_t)split * g.M * g.N; ldd = g.N; }
    else              { dst = g.C; ldd = g.ldc; }
    const bool want_amax = (g.amax != nullptr) && (g.splits == 1);  // with chunks the reduction does it
    uint32_t amax = 0;
    if (g.wide_store && m0 + BM <= g.M && n0 + BN <= g.N) {
        // Whole tile inside the matrix: every 32 x 32 block goes through a wavefront-private patch of LDS (the
        // stages are no longer read: the last barrier of the loops is behind every wavefront) and leaves as
        // 16-byte stores, four per lane and block instead of sixteen 4-byte ones.  Rows are padded to 36
        // floats so that the two lane halves, four rows apart, fall into different banks.
        constexpr int kPatchLd = 36;
        float *patch = smem + wave * (32 * kPatchLd);
        const int prow = lane >> 3, pcol = (lane & 7) * 4;
#pragma unroll
        for (int mi = 0; mi < FM; ++mi)
#pragma unroll
            for (int ni = 0; ni < FN; ++ni) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    patch[(8 * (r >> 2) + 4 * half + (r & 3)) * kPatchLd + l32] = acc[mi][ni][r];
                    const uint32_t bits = __float_as_uint(acc[mi][ni][r]) & 0x7fffffffu;
                    amax = bits > amax ? bits : amax;
                }
                if (EPI == EPI_NONE) {
                    float *corner = dst + (m0 + wave_m * (32 * FM) + mi * 32) * ldd + n0 + wave_n * (32 * FN) + ni * 32 + pcol;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(patch + (prow + 8 * k) * kPatchLd + pcol);
                        // the result itself is not read again soon; the partial planes are, by the chunk sum
                        if (g.splits == 1) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(corner + (int64_t)(prow + 8 * k) * ldd));
                        else               *reinterpret_cast<f32x4 *>(corner + (int64_t)(prow + 8 * k) * ldd) = v;
                    }
                } else {
                    // The lane holds four consecutive columns of a row: the pools of 2 or 4 columns that the bias
                    // and the maximum go over, or the four pooled units whose error is spread to their winners,
                    // lie inside its own 16 bytes.  Same operations, in the same order, as the kernels that would
                    // follow the stored product (add_row_vector then maxout; expand_to_maxout_grad).
                    const int64_t col = n0 + wave_n * (32 * FN) + ni * 32 + pcol;
                    const int pool = g.epi_pool;
                    f32x4 bias4 = {0.f, 0.f, 0.f, 0.f};
                    if (EPI == EPI_BIAS_MAXOUT) bias4 = *reinterpret_cast<const f32x4 *>(g.epi_bias + col);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int64_t row = m0 + wave_m * (32 * FM) + mi * 32 + prow + 8 * k;
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(patch + (prow + 8 * k) * kPatchLd + pcol);
                        if (EPI == EPI_BIAS_MAXOUT) {
                            const f32x4 z = {v.x + bias4.x, v.y + bias4.y, v.z + bias4.z, v.w + bias4.w};
                            const int64_t at = row * (g.N / pool) + col / pool;
                            if (pool == 2) {
                                float b0 = z.x, b1 = z.z;
                                int a0 = 0, a1 = 0;
                                if (b0 < z.y) { b0 = z.y; a0 = 1; }
                                if (b1 < z.w) { b1 = z.w; a1 = 1; }
                                typedef float f32x2 __attribute__((ext_vector_type(2)));
                                __builtin_nontemporal_store(f32x2{b0, b1}, reinterpret_cast<f32x2 *>(g.epi_out + at));
                                __builtin_nontemporal_store(f32x2{(float)(col + a0), (float)(col + 2 + a1)},
                                                            reinterpret_cast<f32x2 *>(g.epi_arg_out + at));
                            } else if (pool == 4) {
                                float b = z.x;
                                int a = 0;
                                if (b < z.y) { b = z.y; a = 1; }
                                if (b < z.z) { b = z.z; a = 2; }
                                if (b < z.w) { b = z.w; a = 3; }
                                g.epi_out[at] = b;
                                g.epi_arg_out[at] = (float)(col + a);
                            } else {  // pool 1: every column its own winner
                                __builtin_nontemporal_store(z, reinterpret_cast<f32x4 *>(g.epi_out + at));
                                __builtin_nontemporal_store(f32x4{(float)col, (float)(col + 1), (float)(col + 2), (float)(col + 3)},
                                                            reinterpret_cast<f32x4 *>(g.epi_arg_out + at));
                            }
                        } else {
                            const f32x4 winner = *reinterpret_cast<const f32x4 *>(g.epi_arg_in + row * g.N + col);
                            float *to = g.epi_out + (row * g.N + col) * pool;
                            if (pool == 2) {
                                f32x4 lo, hi;
                                lo.x = ((int64_t)winner.x == col * 2 + 0) ? v.x : 0.0f;
                                lo.y = ((int64_t)winner.x == col * 2 + 1) ? v.x : 0.0f;
                                lo.z = ((int64_t)winner.y == col * 2 + 2) ? v.y : 0.0f;
                                lo.w = ((int64_t)winner.y == col * 2 + 3) ? v.y : 0.0f;
                                hi.x = ((int64_t)winner.z == col * 2 + 4) ? v.z : 0.0f;
                                hi.y = ((int64_t)winner.z == col * 2 + 5) ? v.z : 0.0f;
                                hi.z = ((int64_t)winner.w == col * 2 + 6) ? v.w : 0.0f;
                                hi.w = ((int64_t)winner.w == col * 2 + 7) ? v.w : 0.0f;
                                __builtin_nontemporal_store(lo, reinterpret_cast<f32x4 *>(to));
                                __builtin_nontemporal_store(hi, reinterpret_cast<f32x4 *>(to + 4));
                            } else if (pool == 4) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const int64_t c0 = (col + e) * 4;
                                    const int64_t w = (int64_t)winner[e];
                                    const f32x4 o = {w == c0 ? v[e] : 0.0f, w == c0 + 1 ? v[e] : 0.0f, w == c0 + 2 ? v[e] : 0.0f,
                                                     w == c0 + 3 ? v[e] : 0.0f};
                                    __builtin_nontemporal_store(o, reinterpret_cast<f32x4 *>(to + 4 * e));
                                }
                            } else {  // pool 1
                                const f32x4 o = {(int64_t)winner.x == col ? v.x : 0.0f, (int64_t)winner.y == col + 1 ? v.y : 0.0f,
                                                 (int64_t)winner.z == col + 2 ? v.z : 0.0f, (int64_t)winner.w == col + 3 ? v.w : 0.0f};
                                __builtin_nontemporal_store(o, reinterpret_cast<f32x4 *>(to));
                            }
                        }
                    }
                }
            }
    } else if (EPI == EPI_NONE) {  // a kernel with an epilogue is only launched on whole tiles
#pragma unroll
        for (int mi = 0; mi < FM; ++mi)
#pragma unroll
            for (int ni = 0; ni < FN; ++ni) {
                const int64_t col = n0 + wave_n * (32 * FN) + ni * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t row = m0 + wave_m * (32 * FM) + mi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    if (row < g.M && col < g.N) {
                        dst[row * ldd + col] = acc[mi][ni][r];
                        const uint32_t bits = __float_as_uint(acc[mi][ni][r]) & 0x7fffffffu;
                        amax = bits > amax ? bits : amax;
                    }
                }
            }
    }
    if (want_amax) publish_absmax(amax, g.amax);
}

// ---- unsplit products of many short tiles: persistent workgroups ------------------------------------------------
// A product whose K is not split and short (the weight gradient of a wide layer: K is the batch) and whose tiles are
// many more than the chip holds at once spends a good part of every tile outside the matrix pipe: a workgroup is
// started, works out its addresses, waits for its first stage, and at the end writes 128 KB out.  Here two workgroups
// per compute unit stay for the whole product and draw their tiles from a counter: the stages of consecutive tiles form
// one pipeline (the load issued during a tile's last stage is the first stage of the next tile), fragment reads run a
// group of 8 k ahead of the MFMAs, and a tile is written out straight from the accumulators while its successor's
// first stage is already in LDS.  Whole K stages and 16-byte operands only (the host checks; ragged tiles at the border of
// C are written element by element); same MFMA order per tile as gemm_kernel, so the same bits.
template <bool A_KC, bool B_IS_KC, int TN>
__global__ __launch_bounds__(NT, 2) void gemm_persistent_kernel(GemmArgs g) {
    using G = Geo<128, TN>;
    constexpr int BM = 128, BN = TN, BK = G::BK, FM = G::FM, FN = G::FN;
    constexpr int kGroups = BK / 8;
    constexpr int kAStage = BM * BK, kBStage = TN * BK;
    static_assert(G::NST == 2, "two LDS stages");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *sA = smem;
    float *sB = smem + 2 * kAStage;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave_m = wave / G::WN, wave_n = wave % G::WN;
    const int half = lane >> 5, l32 = lane & 31;
    int row_a[FM], row_b[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) row_a[i] = wave_m * (32 * FM) + i * 32 + l32;
#pragma unroll
    for (int i = 0; i < FN; ++i) row_b[i] = wave_n * (32 * FN) + i * 32 + l32;

    f32x16 acc[FM][FN];
    auto clear = [&]() {
#pragma unroll
        for (int mi = 0; mi < FM; ++mi)
#pragma unroll
            for (int ni = 0; ni < FN; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;
    };
    clear();

    const float *Bf = reinterpret_cast<const float *>(g.B);
    const int64_t end_a = A_KC ? (g.M - 1) * g.lda + g.K : (g.K - 1) * g.lda + ((g.M + 3) & ~(int64_t)3);
    const int64_t end_b = B_IS_KC ? (g.N - 1) * g.ldb + g.K : (g.K - 1) * g.ldb + ((g.N + 3) & ~(int64_t)3);
    DirectLoader<A_KC, BM, BK> da;
    DirectLoader<B_IS_KC, TN, BK> db;
    da.init(g.lda, wave);
    db.init(g.ldb, wave);
    // The stage to be requested next: corner addresses of its A and B pieces and the bytes from each corner to the end
    // of its matrix (the descriptor's range: rows of a ragged tile that lie outside the matrix read zeros instead of
    // memory).  Kept as running values, a few scalar additions per stage: the loop has nothing else to work out.
    const float *next_a, *next_b;
    int64_t left_a, left_b;
    constexpr int64_t kOne = 1;
    const int64_t step_a = A_KC ? (int64_t)BK : (int64_t)BK * g.lda, step_b = B_IS_KC ? (int64_t)BK : (int64_t)BK * g.ldb;
    auto first_stage_of = [&](int64_t m0, int64_t n0) {
        next_a = A_KC ? g.A + m0 * g.lda : g.A + m0;
        next_b = B_IS_KC ? Bf + n0 * g.ldb : Bf + n0;
        left_a = (end_a - (next_a - g.A)) * 4;  // positive: the corner of a tile lies inside its matrix
        left_b = (end_b - (next_b - Bf)) * 4;
    };
    // Requests that stage into LDS stage `slot` and moves on to the one behind it; not `live`: the same loads with a
    // range of zero bytes (they touch no memory), so that the code is straight-line and its waits can count.
    auto issue_next = [&](int slot, bool live) {
        const uint32_t la = !live ? 0u : ((uint64_t)left_a >> 32) != 0 ? 0xffffffffu : (uint32_t)left_a;
        const uint32_t lb = !live ? 0u : ((uint64_t)left_b >> 32) != 0 ? 0xffffffffu : (uint32_t)left_b;
        da.issue(next_a, la, sA + slot * kAStage, wave);
        db.issue(next_b, lb, sB + slot * kBStage, wave);
        next_a += step_a; left_a -= step_a * 4;
        next_b += step_b; left_b -= step_b * 4;
        (void)kOne;
    };
    auto load_frag = [&](const float *pa, const float *pb, int gq, f32x4 (&a)[FM], f32x4 (&b)[FN]) {
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (A_KC) {
                a[i] = *reinterpret_cast<const f32x4 *>(pa + lds_offset<BK>(row_a[i], 2 * gq + half));
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) a[i][s] = pa[(8 * gq + 4 * half + s) * BM + row_a[i]];
            }
        }
#pragma unroll
        for (int i = 0; i < FN; ++i) {
            if (B_IS_KC) {
                b[i] = *reinterpret_cast<const f32x4 *>(pb + lds_offset<BK>(row_b[i], 2 * gq + half));
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) b[i][s] = pb[(8 * gq + 4 * half + s) * TN + row_b[i]];
            }
        }
    };
    auto mfma_steps = [&](const f32x4 (&a)[FM], const f32x4 (&b)[FN], int s_begin, int s_end) {
#pragma unroll
        for (int s = s_begin; s < s_end; ++s)
#pragma unroll
            for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                for (int ni = 0; ni < FN; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi][s], b[ni][s], acc[mi][ni], 0, 0, 0);
    };
    constexpr int kTailFrom = 4 - 8 / (FM * FN);
    // Fragment reads run one group of 8 k ahead of the MFMAs, in two register sets that alternate: on entry to a stage
    // the first set holds (or is receiving) group 0, requested behind the barrier that published the stage, in the
    // shadow of the previous stage's last eight MFMAs.  A wavefront that has its SIMD to itself (its neighbour of the
    // other workgroup is writing a tile out) then waits for LDS once per stage at most, not once per handful of MFMAs.
    f32x4 a0[FM], b0[FN], a1[FM], b1[FN];
    static_assert(kGroups == 2 || kGroups == 4, "two register sets, even number of groups");
    auto stage_head = [&](const float *pa, const float *pb) {
        load_frag(pa, pb, 1, a1, b1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(a0, b0, 0, 4);
        if (kGroups == 4) {
            __builtin_amdgcn_sched_barrier(0);
            load_frag(pa, pb, 2, a0, b0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_steps(a1, b1, 0, 4);
            __builtin_amdgcn_sched_barrier(0);
            load_frag(pa, pb, 3, a1, b1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_steps(a0, b0, 0, 4);
        }
        mfma_steps(a1, b1, 0, kTailFrom);
        __builtin_amdgcn_sched_barrier(0);
    };
    // Behind the barrier: group 0 of the stage just published, then the last eight MFMAs of the stage before it.
    auto stage_tail = [&](const float *pa_next, const float *pb_next) {
        load_frag(pa_next, pb_next, 0, a0, b0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(a1, b1, kTailFrom, 4);
        __builtin_amdgcn_sched_barrier(0);
    };
    const uint32_t tiles_n32 = (uint32_t)g.tiles_n;
    const int iters = (int)g.k_iters;
    // Block ids are dealt round-robin to the eight XCDs, each with an L2 of its own.  Where the tile columns and the grid
    // divide by eight, an XCD keeps to an eighth of the tile columns (its slice of B stays in its L2, every slab of A is
    // fetched once per XCD) and draws from a counter of its own, the word of the stream's counter line that carries its
    // number; otherwise all workgroups share word 0 and the tiles run row-major over the whole result.  The 100000 x 8192
    // x 128 gradient product fetched 1.40 GB through the fabric with one counter (its operands are 55 MB: B, 4 MB, the
    // size of an L2, was pushed out again and again by the tiles of every other column), 0.41 GB with eight: A once per
    // XCD.  The time is the same; the fabric carries a gigabyte less beside the 3.3 GB of stores.
    const bool by_xcd = g.tile_counter != nullptr && tiles_n32 % kNumXcd == 0 && gridDim.x % kNumXcd == 0;
    const uint32_t groups = by_xcd ? kNumXcd : 1, group = by_xcd ? blockIdx.x % kNumXcd : 0;
    const uint32_t U = g.units / groups, workgroups = gridDim.x / groups, columns = tiles_n32 / groups;  // of this group
    auto corner_of = [&](uint32_t unit, int64_t &m0, int64_t &n0) {  // `unit` counts inside the group
        const uint32_t tm = unit / columns, tn = group * columns + (unit - tm * columns);
        m0 = (int64_t)__builtin_amdgcn_readfirstlane((int)tm) * BM;
        n0 = (int64_t)__builtin_amdgcn_readfirstlane((int)tn) * BN;
    };
    uint32_t amax = 0;

    // The first tile of a workgroup is its block id (the grid is never larger than the number of tiles); the others
    // are drawn from a counter, whichever workgroup is free taking the next one: two workgroups that share the SIMDs of
    // a compute unit do not advance at the same pace, and with a fixed share of the tiles the slower ones would finish
    // long after the faster.  Lane 0 draws the next tile at the top of the current one; the ticket travels during the
    // tile's first stage, is handed to the other wavefronts through LDS at that stage's barrier, and is needed in the
    // last stage, where the next tile's first stage is requested (so tiles of a single stage do not draw).  Every
    // workgroup draws until its first ticket past the last tile, so exactly U tickets are drawn, and whoever holds
    // the last of them puts the counter back to 0 (nobody draws after it).  Without a counter: tiles bid, bid + grid, ...
    uint32_t *ticket_slot = reinterpret_cast<uint32_t *>(smem + 2 * (kAStage + kBStage));
    // The counter's address passes through a register the compiler knows nothing about: a plain atomic on a uniform
    // address is rewritten into a reduction over the wavefront whose result is waited for on the spot, and the point
    // here is that nobody waits for the ticket.
    uint32_t *counter = g.tile_counter;
    const bool drawing = g.tile_counter != nullptr && iters >= 2;
    if (drawing) {
        uint32_t opaque_zero;
        asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
        counter += opaque_zero + group;
    }
    uint32_t drawn = 0;  // lane 0: the raw ticket on its way (tile = the group's workgroups + ticket)
    uint32_t unit = blockIdx.x / groups;
    int64_t m0, n0;
    corner_of(unit, m0, n0);
    first_stage_of(m0, n0);
    issue_next(0, true);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    load_frag(sA, sB, 0, a0, b0);
    int slot = 0;
    for (;;) {
        if (drawing && threadIdx.x == 0) drawn = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t unit_next = unit + workgroups;
        // all stages but the last: the stage requested is the next one of this tile
        for (int it = 1; it < iters; ++it) {
            issue_next(slot ^ 1, true);
            stage_head(sA + slot * kAStage, sB + slot * kBStage);
            // the next stage has landed (and the stores of the tile before this one have been acknowledged, and the
            // ticket has come back)
            __builtin_amdgcn_s_waitcnt(0x0f70);
            if (drawing && it == 1 && threadIdx.x == 0) {
                if (drawn == U - 1u) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *ticket_slot = drawn + workgroups;
            }
            __syncthreads();
            slot ^= 1;
            stage_tail(sA + slot * kAStage, sB + slot * kBStage);
        }
        // the last stage: the stage requested is the first of the next tile.  The slot is not written again before
        // the first barrier of the next tile's second stage, which lies behind this read for every wavefront.
        if (drawing) unit_next = (uint32_t)__builtin_amdgcn_readfirstlane((int)*ticket_slot);
        const bool more = unit_next < U;
        int64_t m1 = m0, n1 = n0;
        if (more) corner_of(unit_next, m1, n1);
        first_stage_of(m1, n1);
        issue_next(slot ^ 1, more);
        stage_head(sA + slot * kAStage, sB + slot * kBStage);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        slot ^= 1;
        stage_tail(sA + slot * kAStage, sB + slot * kBStage);  // the next tile's first stage (stale data if there is none)
        // Write-out.  Accumulator r of a lane is row 8 (r / 4) + 4 half + (r % 4), column l32 of its 32 x 32 block: for a
        // fixed r the 32 lanes of a half write 128 contiguous bytes.  A whole tile leaves as 4-byte stores straight from
        // the accumulators: the lane's part of the address is one register for the whole tile, the row's part travels in
        // a scalar register, so a store reads two vector registers and nothing passes through LDS (a pass through LDS
        // patches, which turns the 128 stores of a wavefront into 32 of 16 bytes, cost this product more than it saved:
        // a tile is only eight stages long).
        const bool want_amax = g.amax != nullptr;
        if (m0 + BM <= g.M && n0 + BN <= g.N) {
            const rsrc_t out = make_rsrc(g.C + m0 * g.ldc + n0);
            const uint32_t ldc_bytes = (uint32_t)g.ldc * 4u;
            const uint32_t mine = (uint32_t)(4 * half) * ldc_bytes + (uint32_t)(wave_n * (32 * FN) + l32) * 4u;
            // the row's offset is a running scalar (kept opaque, or the compiler works out all 64 ahead and parks them
            // in a vector register for want of scalar ones); the two blocks of a row differ by an immediate
            uint32_t row_bytes = (uint32_t)(wave_m * (32 * FM)) * ldc_bytes;
#pragma unroll
            for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        asm volatile("" : "+s"(row_bytes));
#pragma unroll
                        for (int ni = 0; ni < FN; ++ni) {
                            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[mi][ni][4 * q + i]), out, mine + (uint32_t)(ni * 32 * 4),
                                                                  row_bytes, 2 /* nt */);
                        }
                        row_bytes += ldc_bytes;
                    }
                    row_bytes += 4u * ldc_bytes;  // the other lane half's four rows
                }
            if (want_amax) {
#pragma unroll
                for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                    for (int ni = 0; ni < FN; ++ni)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const uint32_t bits = __float_as_uint(acc[mi][ni][r]) & 0x7fffffffu;
                            amax = bits > amax ? bits : amax;
                        }
            }
        } else {
#pragma unroll
            for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                for (int ni = 0; ni < FN; ++ni) {
                    const int64_t col = n0 + wave_n * (32 * FN) + ni * 32 + l32;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int64_t row = m0 + wave_m * (32 * FM) + mi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                        if (row < g.M && col < g.N) {
                            g.C[row * g.ldc + col] = acc[mi][ni][r];
                            const uint32_t bits = __float_as_uint(acc[mi][ni][r]) & 0x7fffffffu;
                            amax = bits > amax ? bits : amax;
                        }
                    }
                }
        }
        if (!more) break;
        clear();
        unit = unit_next;
        m0 = m1;
        n0 = n1;
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // the zero-range loads behind the last stage
    if (g.amax != nullptr) publish_absmax(amax, g.amax);
}

// C[m][n] = sum over chunks of partial[chunk][m][n], chunks added in ascending order.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial, int splits,
                                                            int64_t M, int64_t N, float *__restrict__ C,
                                                            int64_t ldc, int vec, uint32_t *amax_out) {
    const int64_t plane = M * N;
    uint32_t amax = 0;
    if (vec) {
        const int64_t nq = N / 4, total = M * nq;
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
             i += (int64_t)gridDim.x * blockDim.x) {
            const int64_t m = i / nq, q = i % nq;
            const float *src = partial + m * N + 4 * q;
            f32x4 s = *reinterpret_cast<const f32x4 *>(src);
            int c = 1;
            // eight planes requested before the first is added: the order of the additions stays, the
            // memory latencies overlap
            for (; c + 8 <= splits; c += 8) {
                f32x4 t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) t[u] = *reinterpret_cast<const f32x4 *>(src + (c + u) * plane);
#pragma unroll
                for (int u = 0; u < 8; ++u) s += t[u];
            }
            for (; c < splits; ++c) s += *reinterpret_cast<const f32x4 *>(src + c * plane);
            *reinterpret_cast<f32x4 *>(C + m * ldc + 4 * q) = s;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t bits = __float_as_uint(s[e]) & 0x7fffffffu;
                amax = bits > amax ? bits : amax;
            }
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < plane;
             i += (int64_t)gridDim.x * blockDim.x) {
            const int64_t m = i / N, n = i % N;
            float s = partial[i];
            int c = 1;
            for (; c + 8 <= splits; c += 8) {
                float t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) t[u] = partial[i + (c + u) * plane];
#pragma unroll
                for (int u = 0; u < 8; ++u) s += t[u];
            }
            for (; c < splits; ++c) s += partial[i + c * plane];
            C[m * ldc + n] = s;
            const uint32_t bits = __float_as_uint(s) & 0x7fffffffu;
            amax = bits > amax ? bits : amax;
        }
    }
    if (amax_out) publish_absmax(amax, amax_out);
}

// The chunk sum with the bias and maxout of the forward pass behind it: out, argmax = maxout(sum of planes +
// bias) over `pool` consecutive columns.  The planes are added in ascending order and the bias last, so the
// values compared are those of the chunk sum followed by add_row_vector.
__global__ __launch_bounds__(256) void splitk_reduce_bias_maxout_kernel(const float *__restrict__ partial, int splits,
                                                                        int64_t M, int64_t N, const float *__restrict__ bias,
                                                                        int pool, float *__restrict__ out,
                                                                        float *__restrict__ argmax) {
    const int64_t plane = M * N, oc = N / pool, total = M * oc;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / oc, o = i % oc;
        const float *src = partial + r * N + o * pool;
        float best = 0.0f;
        int arg = 0;
        for (int p = 0; p < pool; ++p) {
            float s = src[p];
            int c = 1;
            for (; c + 8 <= splits; c += 8) {
                float t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) t[u] = src[p + (c + u) * plane];
#pragma unroll
                for (int u = 0; u < 8; ++u) s += t[u];
            }
            for (; c < splits; ++c) s += src[p + c * plane];
            const float z = s + bias[o * pool + p];
            if (p == 0 || best < z) { best = z; arg = p; }
        }
        out[i] = best;
        argmax[i] = (float)(o * pool + arg);
    }
}

// The chunk sum with the backward step of a maxout layer behind it: out (M x N pool) receives the summed error
// of a pooled unit in its winner's column and zero in the others.
__global__ __launch_bounds__(256) void splitk_reduce_expand_kernel(const float *__restrict__ partial, int splits, int64_t M,
                                                                   int64_t N, const float *__restrict__ argmax, int pool,
                                                                   float *__restrict__ out) {
    const int64_t plane = M * N, cols = N * pool, total = M * cols;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / cols, c = i % cols, o = c / pool;
        float v = 0.0f;
        if ((int64_t)argmax[r * N + o] == c) {
            const float *src = partial + r * N + o;
            float s = src[0];
            for (int k = 1; k < splits; ++k) s += src[k * plane];
            v = s;
        }
        out[i] = v;
    }
}

__global__ void set_word_kernel(uint32_t *p, uint32_t value) {
    if (threadIdx.x == 0) *p = value;
}

__global__ __launch_bounds__(256) void zero_matrix_kernel(float *__restrict__ C, int64_t M, int64_t N, int64_t ldc) {
    const int64_t total = M * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x)
        C[(i / N) * ldc + (i % N)] = 0.0f;
}

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// C = sum of the `splits` M x N planes at `planes`, added in ascending order;
// optionally also max |C| (see publish_absmax).
cn_status add_chunk_planes(const void *planes, int num_cu, int splits, int64_t M, int64_t N, float *C, int64_t ldc,
                           uint32_t *amax, hipStream_t st) {
    int vec = (N % 4 == 0) && (ldc % 4 == 0) && aligned(C, 16);
    int64_t work = vec ? M * (N / 4) : M * N;
    int64_t blocks = (work + 255) / 256;
    int64_t cap = (int64_t)num_cu * 8;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0, st,
                       (const float *)planes, splits, M, N, C, ldc, vec, amax);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

template <bool A_KC, int B_KIND, int TN, int TM, int EPI = EPI_NONE>
static cn_status launch_tile(const GemmArgs &args, int device, hipStream_t st) {
    using G = Geo<TM, TN>;
    // the stages, the decode table of the fused variant, and at least the four write-out patches
    size_t lds = (size_t)(G::NST * (TM + TN) * G::BK + (B_KIND == B_CODES ? 256 : 0)) * sizeof(float);
    if (lds < NW * 32 * 36 * sizeof(float)) lds = NW * 32 * 36 * sizeof(float);
    static OncePerDevice configured;
    if (configured.first(device)) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<A_KC, B_KIND, TN, TM, EPI>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    hipLaunchKernelGGL((gemm_kernel<A_KC, B_KIND, TN, TM, EPI>), dim3(args.units), dim3(NT), lds, st, args);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

template <bool A_KC, int B_KIND>
static cn_status launch(const GemmArgs &args, const GemmPlan &plan, int device, hipStream_t st) {
    if (plan.tile_m == kTileMLow) return launch_tile<A_KC, B_KIND, 128, kTileMLow>(args, device, st);
    if (plan.tile_m == kTileMMid) return launch_tile<A_KC, B_KIND, 128, kTileMMid>(args, device, st);
    return plan.tile_n == 256 ? launch_tile<A_KC, B_KIND, 256, kTileM>(args, device, st)
                              : launch_tile<A_KC, B_KIND, 128, kTileM>(args, device, st);
}

template <bool A_KC, bool B_IS_KC, int TN>
static cn_status launch_persistent_tile(const GemmArgs &args, int num_cu, int device, hipStream_t st) {
    using G = Geo<128, TN>;
    const size_t lds = (size_t)(2 * (128 + TN) * G::BK + 4) * sizeof(float);  // the stages and the ticket word
    static OncePerDevice configured;
    if (configured.first(device)) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_persistent_kernel<A_KC, B_IS_KC, TN>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    const uint32_t slots = (uint32_t)num_cu * 2u;
    hipLaunchKernelGGL((gemm_persistent_kernel<A_KC, B_IS_KC, TN>), dim3(args.units < slots ? args.units : slots), dim3(NT), lds, st, args);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

template <bool A_KC, bool B_IS_KC>
static cn_status launch_persistent(const GemmArgs &args, int tile_n, int num_cu, int device, hipStream_t st) {
    return tile_n == 256 ? launch_persistent_tile<A_KC, B_IS_KC, 256>(args, num_cu, device, st)
                         : launch_persistent_tile<A_KC, B_IS_KC, 128>(args, num_cu, device, st);
}

static int g_force_tile_n = 0;
static bool g_wide_store = true;
static bool g_w8_rows = true;  // test hook: false keeps the tiled kernel for every product on 8-bit weights
static bool g_small = true;    // test hook: false keeps the tiled kernel for small products too
static bool g_persistent = true;  // test hook: false starts a workgroup per tile for every product
// Which kernel family the last product took and how many K chunks it had (test hook cn_host_last_gemm_kernel).
enum { kTookNone = 0, kTookTiled = 1, kTookSmall = 2, kTookW8Rows = 3, kTookPersistent = 4 };
static int g_last_kernel = kTookNone, g_last_splits = 0;
static bool g_epilogue_in_kernel = true;  // test hook: false sends every fused product through the workspace

// What follows the product instead of its delivery: bias and maxout (the forward pass of a maxout layer; `bias`
// given, out and argmax M x N / pool), or the expansion of a pooled error to the winners' columns (its backward
// pass; `bias` NULL, `argmax` M x N is read, out M x N pool).  All contiguous.
struct BiasMaxout {
    const float *bias;
    int pool;
    float *out, *argmax;
};

// `env` = NULL: the current device's context (initialised on first use) supplies the workspace.
static cn_status gemm_impl(int ta, int tb, bool w8, int64_t M, int64_t N, int64_t K, const float *A,
                           int64_t lda, const void *B, int64_t ldb, float scale, float *C, int64_t ldc,
                           float *absmax_out, void *stream, const BiasMaxout *then = nullptr,
                           const GemmEnv *given = nullptr) {
    const char *who = given ? "gemm_f32_noalloc"
                            : then ? (then->bias ? "gemm_f32_bias_maxout" : "gemm_f32_expand_maxout_grad") : (w8 ? "gemm_f32_w8" : "gemm_f32");
    auto finish_from = [&](const float *product) -> cn_status {  // `product` M x N contiguous
        if (then->bias) return cn_bias_maxout_f32(product, N, then->bias, M, N, then->pool, then->out, then->argmax, stream);
        return cn_expand_to_maxout_grad_f32(product, then->argmax, M, N, then->pool, then->out, stream);
    };
    if (M < 0 || N < 0 || K < 0) { set_error("%s: negative dimension", who); return CN_ERR_SHAPE; }
    if (lda < (ta ? M : K) || ldb < (tb ? K : N) || ldc < N) {
        set_error("%s: leading dimension too small (lda %lld, ldb %lld, ldc %lld for M %lld N %lld K %lld)",
                  who, (long long)lda, (long long)ldb, (long long)ldc, (long long)M, (long long)N, (long long)K);
        return CN_ERR_SHAPE;
    }
    if (lda > (1 << 22) || ldb > (1 << 22)) {
        set_error("%s: leading dimensions above 2^22 elements are not supported", who);
        return CN_ERR_SHAPE;
    }
    if ((M == 0 || N == 0) && !absmax_out) return CN_OK;
    if ((M > 0 && N > 0) && ((!C && !then) || (K > 0 && (!A || !B)))) { set_error("%s: NULL operand", who); return CN_ERR_NULL; }
    cn_status s = CN_OK;
    GemmEnv from_context;
    Context *context = nullptr;
    if (!given) {
        Context *c;
        s = current_context(&c);
        if (s != CN_OK) return s;
        from_context = GemmEnv{c->device, c->num_cu, c->workspace, c->workspace_bytes, c->workspace_bytes, c->table};
        context = c;
    }
    const GemmEnv *ctx = given ? given : &from_context;
    hipStream_t st = (hipStream_t)stream;
    // The maximum is accumulated with atomics from +0.0 (|C| >= 0); an empty C reports -1.0f, the start
    // value of the reference's reduction, like cn_absmax_f32.
    uint32_t *amax = reinterpret_cast<uint32_t *>(absmax_out);
    if (amax) {
        hipLaunchKernelGGL(set_word_kernel, dim3(1), dim3(64), 0, st, amax, (M == 0 || N == 0) ? 0xbf800000u : 0u);
        CN_HIP(hipGetLastError());
    }
    if (M == 0 || N == 0) return CN_OK;
    if (K == 0) {
        if (then) {
            if ((size_t)M * (size_t)N * sizeof(float) > ctx->workspace_bytes) { set_error("%s: product does not fit the workspace", who); return CN_ERR_WORKSPACE; }
            C = (float *)ctx->workspace;
            ldc = N;
        }
        hipLaunchKernelGGL(zero_matrix_kernel, dim3(ctx->num_cu * 4), dim3(256), 0, st, C, M, N, ldc);
        CN_HIP(hipGetLastError());
        if (then) return finish_from(C);
        return CN_OK;
    }
    if (w8 && !then && g_w8_rows && g_force_tile_n == 0) {
        // up to 1024 rows: the kernel that decodes straight into the matrix instruction's registers
        const int chunks = gemm_w8_rows_splits(M, N, K, A, lda, (const uint8_t *)B, ldb, scale, C, ldc, ctx->num_cu, ctx->workspace_bytes);
        if (chunks > 1 || (chunks == 1 && !amax)) {
            g_last_kernel = kTookW8Rows; g_last_splits = chunks;
            s = gemm_w8_rows(chunks, M, N, K, A, lda, (const uint8_t *)B, ldb, scale, C, ldc, ctx->table, ctx->workspace, ctx->device, st);
            if (s != CN_OK) return s;
            if (chunks > 1) return add_chunk_planes(ctx->workspace, ctx->num_cu, chunks, M, N, C, ldc, amax, st);
            return CN_OK;
        }
    }
    if (!w8 && g_small && g_force_tile_n == 0 && gemm_small_applies(ta, tb, M, N, K, A, lda, (const float *)B, ldb)) {
        // too small to fill the chip with tiles: one launch, and for every entry point the same one, so that the
        // calls that fuse something behind the product keep giving the bits of the separate calls
        if (then) {
            if ((size_t)M * (size_t)N * sizeof(float) > ctx->workspace_bytes) { set_error("%s: product does not fit the workspace", who); return CN_ERR_WORKSPACE; }
            C = (float *)ctx->workspace;
            ldc = N;
        }
        g_last_kernel = kTookSmall; g_last_splits = 1;
        s = gemm_small(ta, tb, M, N, K, A, lda, (const float *)B, ldb, C, ldc, amax, st);
        if (s != CN_OK) return s;
        return then ? finish_from(C) : CN_OK;
    }
    GemmPlan plan = plan_gemm(M, N, K, ctx->num_cu, ctx->plan_bytes, g_force_tile_n, !ta);
    // K not split, whole 128-row tiles and pools of 1, 2 or 4: bias + maxout, or the expansion, happen in the
    // product's own write-out and the product never exists in memory (dot for the forward pass, dotT for the
    // backward one; the other transpositions go through the workspace like ragged shapes).
    const bool in_write_out =
        then && g_epilogue_in_kernel && !w8 && plan.splits == 1 && plan.tile_m == kTileM && M % kTileM == 0 && N % plan.tile_n == 0 &&
        (then->pool == 1 || then->pool == 2 || then->pool == 4) && !ta && (then->bias ? !tb : tb) && aligned(then->out, 16) &&
        aligned(then->argmax, 16) && (!then->bias || aligned(then->bias, 16));
    if (then && plan.splits == 1 && !in_write_out) {
        // no chunk sum to fold into: the product goes to the workspace and one pass over it follows
        if ((size_t)M * (size_t)N * sizeof(float) > ctx->workspace_bytes) {
            set_error("%s: product does not fit the workspace", who);
            return CN_ERR_WORKSPACE;
        }
        C = (float *)ctx->workspace;
        ldc = N;
    }
    if (plan.units <= 0 || plan.units > 0x7fffffffLL) {
        set_error("%s: %lld work units exceed the launch limit", who, (long long)plan.units);
        return CN_ERR_SHAPE;
    }
    if (plan.splits > 1 && (size_t)plan.splits * (size_t)M * (size_t)N * sizeof(float) > ctx->workspace_bytes) {
        set_error("%s: the %d K-chunks of this %lld x %lld product need %zu bytes of partial sums, %zu are there%s", who,
                  plan.splits, (long long)M, (long long)N, (size_t)plan.splits * (size_t)M * (size_t)N * sizeof(float),
                  ctx->workspace_bytes, given ? " (the limit of this entry point; cn_gemm_f32 serves larger products)" : "");
        return CN_ERR_WORKSPACE;
    }
    GemmArgs a;
    a.A = A; a.B = B; a.C = C; a.partial = (float *)ctx->workspace;
    a.M = M; a.N = N; a.K = K; a.lda = lda; a.ldb = ldb; a.ldc = ldc;
    a.tiles_n = plan.tiles_n; a.tiles = plan.tiles_m * plan.tiles_n;
    a.k_iters = plan.k_iters; a.iters_per_split = plan.iters_per_split;
    a.units = (uint32_t)plan.units; a.splits = plan.splits;
    // An unsplit product is dominated by its own write-out more often than by operand re-use across tiles: its tiles
    // go out in block-id order, which keeps the part of C in flight in one window (100000 x 8192 x 128: 1.77 ms against
    // 1.80 ms; 4096^3 and 8192 x 8192 x 512: 0.5 % faster).  Split products keep a slice per XCD (B panels re-used in its L2).
    a.units_in_order = plan.splits == 1 ? 1 : 0;
    a.vec_a = aligned(A, 16) && (lda % 4 == 0);
    a.vec_b = w8 ? (aligned(B, 4) && (ldb % 4 == 0)) : (aligned(B, 16) && (ldb % 4 == 0));
    a.scale = scale; a.table = ctx->table;
    a.amax = amax;
    a.tile_counter = nullptr;
    a.wide_store = g_wide_store && (plan.splits > 1 ? (N % 4 == 0 && (M * N) % 4 == 0)
                                                     : (aligned(C, 16) && ldc % 4 == 0));
    a.epi_bias = nullptr; a.epi_arg_in = nullptr; a.epi_out = nullptr; a.epi_arg_out = nullptr; a.epi_pool = 1;
    if (in_write_out) {
        g_last_kernel = kTookTiled; g_last_splits = 1;
        a.wide_store = 1;  // the tiles leave through the LDS patch whatever C would have allowed
        a.epi_pool = then->pool;
        a.epi_out = then->out;
        if (then->bias) { a.epi_bias = then->bias; a.epi_arg_out = then->argmax; }
        else            { a.epi_arg_in = then->argmax; }
        if (then->bias)
            return plan.tile_n == 256 ? launch_tile<true, B_IC, 256, kTileM, EPI_BIAS_MAXOUT>(a, ctx->device, st)
                                      : launch_tile<true, B_IC, 128, kTileM, EPI_BIAS_MAXOUT>(a, ctx->device, st);
        return plan.tile_n == 256 ? launch_tile<true, B_KC, 256, kTileM, EPI_EXPAND>(a, ctx->device, st)
                                  : launch_tile<true, B_KC, 128, kTileM, EPI_EXPAND>(a, ctx->device, st);
    }

    // K not split and short, 128-row tiles, several rounds of them, whole K stages, 16-byte operands and a result that
    // 32-bit offsets reach: the workgroups stay and draw their tiles (100000 x 8192 x 128: 1.61 ms against 1.74 ms; from
    // about 64 stages per tile on there is nothing left to gain and the workgroup per tile is ahead by a percent).
    bool persistent = g_persistent && !w8 && !then && plan.splits == 1 && plan.tile_m == kTileM &&
                      plan.units >= (int64_t)ctx->num_cu * 2 * kPersistentFromRounds && plan.k_iters <= kPersistentMaxStages &&
                      a.vec_a && a.vec_b && K % gemm_tile_k(plan.tile_n) == 0 && ldc <= (1 << 22);
    if (persistent) {
        // its workgroups draw their tiles: without a counter (the stream is being captured, or the library has no context
        // yet and may not create one) the workgroup per tile stays
        if (!context) context = ready_context(ctx->device);
        a.tile_counter = context ? context->tile_counter_for(st) : nullptr;
        persistent = a.tile_counter != nullptr;
    }
    g_last_kernel = persistent ? kTookPersistent : kTookTiled;
    g_last_splits = plan.splits;
    if (persistent) {
        if (!ta && !tb)     s = launch_persistent<true, false>(a, plan.tile_n, ctx->num_cu, ctx->device, st);
        else if (ta && !tb) s = launch_persistent<false, false>(a, plan.tile_n, ctx->num_cu, ctx->device, st);
        else if (!ta && tb) s = launch_persistent<true, true>(a, plan.tile_n, ctx->num_cu, ctx->device, st);
        else                s = launch_persistent<false, true>(a, plan.tile_n, ctx->num_cu, ctx->device, st);
        return s;
    }
    if (w8)              s = launch<true, B_CODES>(a, plan, ctx->device, st);
    else if (!ta && !tb) s = launch<true, B_IC>(a, plan, ctx->device, st);
    else if (ta && !tb)  s = launch<false, B_IC>(a, plan, ctx->device, st);
    else if (!ta && tb)  s = launch<true, B_KC>(a, plan, ctx->device, st);
    else                 s = launch<false, B_KC>(a, plan, ctx->device, st);
    if (s != CN_OK) return s;

    if (then) {
        if (plan.splits == 1) return finish_from(C);
        const int64_t work = then->bias ? M * (N / then->pool) : M * N * then->pool;
        const int64_t blocks = (work + 255) / 256, cap = (int64_t)ctx->num_cu * 8;
        const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
        if (then->bias)
            hipLaunchKernelGGL(splitk_reduce_bias_maxout_kernel, grid, dim3(256), 0, st, (const float *)ctx->workspace,
                               plan.splits, M, N, then->bias, then->pool, then->out, then->argmax);
        else
            hipLaunchKernelGGL(splitk_reduce_expand_kernel, grid, dim3(256), 0, st, (const float *)ctx->workspace, plan.splits,
                               M, N, (const float *)then->argmax, then->pool, then->out);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (plan.splits > 1) return add_chunk_planes(ctx->workspace, ctx->num_cu, plan.splits, M, N, C, ldc, amax, st);
    return CN_OK;
}

// ---- the product for callers that must not allocate ----------------------------------------------------------
// Its K-chunk partial sums go to an array that is part of the library's device image instead of the workspace that
// cn_init allocates.  In host code the array's name stands for the symbol, not for a device address: the address
// is asked for once per device (every device holds its own copy) and only that pointer is ever handed to a kernel.
constexpr size_t kStaticPartialBytes = (size_t)64 << 20;
static __device__ __align__(256) float scratch[kStaticPartialBytes / sizeof(float)];

struct StaticPartials {
    float *ptr = nullptr;
    int num_cu = 0;
};
static StaticPartials g_static[kMaxDevices];
static std::mutex g_static_mutex;

cn_status gemm_static_setup(int device) {
    if (device < 0 || device >= kMaxDevices) { set_error("device %d out of range", device); return CN_ERR_NO_DEVICE; }
    std::lock_guard<std::mutex> lock(g_static_mutex);
    StaticPartials &sp = g_static[device];
    if (sp.ptr) return CN_OK;
    float *ptr = nullptr;
    CN_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
    int cus = 0;
    CN_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    if (!ptr || cus <= 0) { set_error("gemm_f32_noalloc: the partial-sum array could not be located on device %d", device); return CN_ERR_HIP; }
    sp.num_cu = cus;
    sp.ptr = ptr;
    return CN_OK;
}

}  // namespace cn

using namespace cn;

extern "C" {

// Test hook: 0 = write every tile with 4-byte stores.
void cn_host_gemm_wide_store(int enabled) { g_wide_store = enabled != 0; }

// Test hook: 0 = bias + maxout and the maxout expansion never run inside the product's write-out.
void cn_host_gemm_w8_rows(int enabled) { g_w8_rows = enabled != 0; }
void cn_host_gemm_small(int enabled) { g_small = enabled != 0; }
void cn_host_gemm_persistent(int enabled) { g_persistent = enabled != 0; }
int cn_host_last_gemm_kernel(int *splits) {
    if (splits) *splits = g_last_splits;
    return g_last_kernel;
}
void cn_host_gemm_epilogue_in_kernel(int enabled) { g_epilogue_in_kernel = enabled != 0; }

// Test and tuning hook: 0 = let the planner choose the tile, 128 / 256 = force that width of the 128-row
// tile, 32 / 64 = force the 32 x 128 / 64 x 128 tile.
void cn_host_force_gemm_tile_n(int tile_n) {
    g_force_tile_n = (tile_n == 128 || tile_n == 256 || tile_n == kTileMLow || tile_n == kTileMMid) ? tile_n : 0;
}

cn_status cn_gemm_f32(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                      const float *B, int64_t ldb, float *C, int64_t ldc, void *stream) {
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, C, ldc, nullptr, stream);
}

cn_status cn_gemm_f32_noalloc(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                              const float *B, int64_t ldb, float *C, int64_t ldc, void *stream) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
        set_error("gemm_f32_noalloc: no usable HIP device (%s)", e == hipSuccess ? "index out of range" : hipGetErrorString(e));
        return CN_ERR_NO_DEVICE;
    }
    if (!g_static[device].ptr) {  // first call on this device without cn_init: locate the array now
        cn_status s = gemm_static_setup(device);
        if (s != CN_OK) return s;
    }
    const GemmEnv env{device, g_static[device].num_cu, g_static[device].ptr, kStaticPartialBytes,
                      planning_workspace_bytes(device), nullptr};
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, C, ldc, nullptr, stream, nullptr, &env);
}

cn_status cn_gemm_f32_absmax(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A,
                             int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc, float *absmax_out,
                             void *stream) {
    if (!absmax_out) { set_error("gemm_f32_absmax: NULL output for the maximum"); return CN_ERR_NULL; }
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, C, ldc, absmax_out, stream);
}

cn_status cn_gemm_f32_bias_maxout(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                                  const float *B, int64_t ldb, const float *bias, int pool, float *out, float *argmax,
                                  void *stream) {
    if (pool < 1 || N % (pool > 0 ? pool : 1) != 0) {
        set_error("gemm_f32_bias_maxout: columns are not a multiple of the pool size");
        return CN_ERR_SHAPE;
    }
    if (M > 0 && N > 0 && (!bias || !out || !argmax)) { set_error("gemm_f32_bias_maxout: NULL pointer"); return CN_ERR_NULL; }
    const BiasMaxout then{bias, pool, out, argmax};
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, nullptr, N, nullptr, stream, &then);
}

cn_status cn_gemm_f32_expand_maxout_grad(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A,
                                         int64_t lda, const float *B, int64_t ldb, const float *argmax, int pool, float *out,
                                         void *stream) {
    if (pool < 1) { set_error("gemm_f32_expand_maxout_grad: pool size below 1"); return CN_ERR_SHAPE; }
    if (M > 0 && N > 0 && (!argmax || !out)) { set_error("gemm_f32_expand_maxout_grad: NULL pointer"); return CN_ERR_NULL; }
    const BiasMaxout then{nullptr, pool, out, const_cast<float *>(argmax)};
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, nullptr, N, nullptr, stream, &then);
}

cn_status cn_gemm_f32_w8(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W,
                         int64_t ldw, float scale, float *C, int64_t ldc, void *stream) {
    return gemm_impl(0, 0, true, M, N, K, A, lda, W, ldw, scale, C, ldc, nullptr, stream);
}

}  // extern "C"
