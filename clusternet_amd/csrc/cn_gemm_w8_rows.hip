// C = A . decode(W8) for products of up to 1024 rows, gfx950.
//
// With few rows the product is one pass over the codes: 16.8 MB for a 4096 x 4096 layer, against 67 MB for
// fp32 weights.  The tiled kernel (cn_gemm.hip) decodes a stage of codes into LDS, waits at a barrier and reads
// the values back as matrix fragments: three LDS operations per weight and a barrier between decode and use,
// which left it slower than the fp32 product it should beat (24 us against 20 us at 32 x 4096 x 4096).
//
// Here a wavefront decodes straight into the registers the matrix instruction reads:
//   * a workgroup of eight wavefronts owns 128 columns of 32 or 64 rows of the result and one chunk of K; each wavefront takes a
//     contiguous eighth of the chunk and all 128 columns, so no weight is shared between wavefronts and nothing
//     of B passes through LDS except the 1 KB decode table;
//   * lane (h, i) of a wavefront loads, for a group of 8 k, the four code words W[k0 + 4h + j][n0 + 4i .. 4i + 3],
//     j = 0 .. 3: a half-wavefront reads 128 contiguous bytes of a row of W.  Byte b of word j is the B operand of
//     v_mfma_f32_32x32x2_f32 number (j, b): that instruction sums over the k pair {k0 + j, k0 + 4 + j} and its 32
//     columns are n0 + 4i + b, i = 0 .. 31, so the four accumulator blocks b = 0 .. 3 interleave by column and a lane
//     ends up holding four consecutive columns of every row it owns;
//   * A comes from memory (it is small and stays in the L2) as one 16-byte load per lane and group, A[i][k0 + 4h .. + 3];
//   * the eight partial tiles of a workgroup meet in LDS (128 KB) and are summed in wavefront order by all 512 lanes;
//     the K chunks of different workgroups go to planes that splitk_reduce_kernel adds in chunk order, as for every
//     split product.  Both orders are fixed, so the result does not depend on scheduling.
#include "cn_internal.h"

namespace cn {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int kCols = 128;     // columns of a workgroup
constexpr size_t lds_bytes(int waves) { return (size_t)(waves * 32 * kCols + 256) * sizeof(float); }

struct RowsArgs {
    const float *A;
    const uint8_t *W;
    float *out;            // planes [splits][M][N] (out_ld = N, plane = M N) or C itself (splits == 1)
    const float *table;
    int64_t lda, ldw, out_ld, plane;
    int64_t M, N;
    int64_t groups;        // K / 8
    float scale;
    int splits, tiles_n, tiles_m;
};

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint32_t bytes) {
    // 0x00020000: 32-bit untyped data; accesses at or beyond `bytes` read zero
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// FM blocks of 32 rows per workgroup (row tiles of 32 FM rows), kAhead groups of 8 k whose loads are in flight, kWaves
// wavefronts that share the workgroup's chunk of K.
template <int FM, int kAhead, int kWaves>
__global__ __launch_bounds__(kWaves * 64) void gemm_w8_rows_kernel(RowsArgs g) {
    constexpr int kLanes = kWaves * 64;
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *lut = smem + kWaves * 32 * kCols;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    // decode table, built exactly as the stand-alone decompression kernel builds it
    if (tid < 126) {
        const float v = g.table[tid] * g.scale;
        lut[tid] = v;
        lut[tid + 128] = -v;
    } else if (tid == 126) {
        lut[126] = g.scale;
        lut[127] = g.scale;
        lut[254] = g.scale;
        lut[255] = -g.scale;
    }
    // row tiles of one column tile and chunk are neighbours: they read the same codes at the same time
    const unsigned column_unit = blockIdx.x / (unsigned)g.tiles_m;
    const int tm = __builtin_amdgcn_readfirstlane((int)(blockIdx.x % (unsigned)g.tiles_m));
    const int split = __builtin_amdgcn_readfirstlane((int)(column_unit / (unsigned)g.tiles_n));
    const int tn = __builtin_amdgcn_readfirstlane((int)(column_unit % (unsigned)g.tiles_n));
    const int64_t n0 = (int64_t)tn * kCols, m0 = (int64_t)tm * 32 * FM;
    // the groups of 8 k are dealt to the wavefronts of all chunks in contiguous, nearly equal runs
    const int64_t parts = (int64_t)g.splits * kWaves, part = (int64_t)split * kWaves + wave;
    const int64_t g0 = __builtin_amdgcn_readfirstlane((int)(g.groups * part / parts));
    const int64_t g1 = __builtin_amdgcn_readfirstlane((int)(g.groups * (part + 1) / parts));
    const int count = (int)(g1 - g0);

    // A: up to the last element of row M - 1, so that rows at or beyond M read zero and nothing past the matrix is
    // touched; W: this wavefront's rows, its 128 columns
    const rsrc_t ra = make_rsrc(g.A, (uint32_t)(((g.M - 1) * g.lda + g.groups * 8) * (int64_t)sizeof(float)));
    const int64_t cols_here = g.N - n0 < kCols ? g.N - n0 : kCols;
    const rsrc_t rw = make_rsrc(g.W + g0 * 8 * g.ldw + n0, count > 0 ? (uint32_t)((count * 8 - 1) * g.ldw + cols_here) : 0u);
    const uint32_t a_lane = (uint32_t)((m0 + l32) * g.lda * (int64_t)sizeof(float)) + 16u * half;
    const uint32_t a_block = (uint32_t)(32 * g.lda * (int64_t)sizeof(float));
    const uint32_t w_lane = (uint32_t)(4 * half * g.ldw) + 4u * l32;
    const uint32_t w_row = (uint32_t)g.ldw;

    uint32_t c[kAhead][4];
    f32x4 a[kAhead][FM];
    auto request = [&](int slot, int i) {  // group g0 + i; a request beyond the run reads the last group again (unused)
        i = i < count ? i : (count > 0 ? count - 1 : 0);
        const uint32_t w_base = __builtin_amdgcn_readfirstlane((int)((uint32_t)i * 8u * w_row));
        const uint32_t a_base = __builtin_amdgcn_readfirstlane((int)((uint32_t)((g0 + i) * 8 * (int64_t)sizeof(float))));
#pragma unroll
        for (int j = 0; j < 4; ++j) c[slot][j] = __builtin_amdgcn_raw_buffer_load_b32(rw, w_lane + j * w_row, w_base, 0);
#pragma unroll
        for (int mi = 0; mi < FM; ++mi) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(ra, a_lane + mi * a_block, a_base, 0);
            a[slot][mi] = f32x4{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
        }
    };
#pragma unroll
    for (int d = 0; d < kAhead; ++d) request(d, d);

    f32x16 acc[FM][4];
#pragma unroll
    for (int mi = 0; mi < FM; ++mi)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][b][r] = 0.0f;
    __syncthreads();  // the decode table is there

    for (int i = 0; i < count; i += kAhead) {
#pragma unroll
        for (int d = 0; d < kAhead; ++d) {
            if (i + d >= count) break;
            float bv[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = c[d][j];
                bv[j][0] = lut[w & 0xffu];
                bv[j][1] = lut[(w >> 8) & 0xffu];
                bv[j][2] = lut[(w >> 16) & 0xffu];
                bv[j][3] = lut[w >> 24];
            }
            f32x4 av[FM];
#pragma unroll
            for (int mi = 0; mi < FM; ++mi) av[mi] = a[d][mi];
            request(d, i + d + kAhead);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mi = 0; mi < FM; ++mi)
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[mi][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[mi][j], bv[j][b], acc[mi][b], 0, 0, 0);
        }
    }

    // The partial tiles of the workgroup's wavefronts: through LDS, summed in wavefront order.  Accumulator r of a lane holds
    // row 8 (r / 4) + 4 half + (r % 4) of its block; its four blocks are four consecutive columns, 4 l32 .. 4 l32 + 3.
    float *mine = smem + wave * 32 * kCols;
    float *dst = g.out + (g.splits > 1 ? (int64_t)split * g.plane : 0);
#pragma unroll
    for (int mi = 0; mi < FM; ++mi) {
        if (mi > 0) __syncthreads();  // the block before has been read
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * half + (r & 3);
            *reinterpret_cast<f32x4 *>(mine + row * kCols + 4 * l32) =
                f32x4{acc[mi][0][r], acc[mi][1][r], acc[mi][2][r], acc[mi][3][r]};
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 32 * kCols / 4 / kLanes; ++q) {
            const int f = tid + q * kLanes, row = f >> 5, col = (f & 31) * 4;
            f32x4 s = *reinterpret_cast<const f32x4 *>(smem + row * kCols + col);
#pragma unroll
            for (int w = 1; w < kWaves; ++w) s = s + *reinterpret_cast<const f32x4 *>(smem + w * 32 * kCols + row * kCols + col);
            const int64_t m = m0 + mi * 32 + row, n = n0 + col;
            if (m < g.M && n < g.N) *reinterpret_cast<f32x4 *>(dst + m * g.out_ld + n) = s;
        }
    }
}

}  // namespace

// Products of more rows than this stay with the tiled kernel of cn_gemm.hip: every 64-row tile decodes the codes it
// needs by itself, and from about 2000 rows on that costs more than a tile's barriers (4096 x 4096 weights: 42.6 us
// against 50.1 us at 128 rows, 134.5 against 142.6 at 512, 267 against 272 at 1024, 530 against 519 at 2048).
constexpr int64_t kRowsUpto = 1024;

// Whether the product takes this kernel, and if so how many K chunks (0 = no): whole 16-byte and 4-byte accesses, a
// finite scale (rows and groups outside a wavefront's run are multiplied by zero), offsets that fit 32 bits.
// Row tiles of 32 rows for up to 32 rows, of 64 rows beyond (tiles of 128 rows would need 256 accumulator registers
// per lane; the compiler spills them); eight wavefronts per workgroup.
static int rows_per_tile(int64_t M) { return M <= 32 ? 32 : 64; }
static int waves_for(int64_t) { return 8; }

int gemm_w8_rows_splits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W, int64_t ldw,
                        float scale, const float *C, int64_t ldc, int num_cu, size_t workspace_bytes) {
    auto aligned_to = [](const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; };
    if (M < 1 || M > kRowsUpto || N < 4 || K < 64 || N % 4 != 0 || K % 8 != 0) return 0;
    if (!aligned_to(A, 16) || lda % 4 != 0 || !aligned_to(W, 4) || ldw % 4 != 0) return 0;
    if (!(scale == scale) || scale - scale != 0.0f) return 0;  // NaN or infinite
    if ((uint64_t)K * (uint64_t)ldw >= (1ull << 31) || (uint64_t)M * (uint64_t)lda * 4 >= (1ull << 31)) return 0;
    const int64_t tiles_n = (N + kCols - 1) / kCols, tiles_m = (M + rows_per_tile(M) - 1) / rows_per_tile(M), groups = K / 8;
    // one workgroup per compute unit; a wavefront wants at least four groups
    int64_t splits = (num_cu + tiles_n * tiles_m - 1) / (tiles_n * tiles_m);
    if (splits > groups / (waves_for(M) * 4)) splits = groups / (waves_for(M) * 4);
    if (splits < 1) splits = 1;
    while (splits > 1 && (size_t)splits * (size_t)M * (size_t)N * sizeof(float) > workspace_bytes) --splits;
    if (splits == 1 && (!aligned_to(C, 16) || ldc % 4 != 0)) return 0;
    if (tiles_n * tiles_m * splits > 0x7fffffffLL) return 0;
    return (int)splits;
}

cn_status gemm_w8_rows(int splits, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W, int64_t ldw,
                       float scale, float *C, int64_t ldc, const float *table, void *workspace, int device, hipStream_t st) {
    RowsArgs g;
    g.A = A; g.W = W; g.table = table;
    g.lda = lda; g.ldw = ldw;
    g.M = M; g.N = N; g.groups = K / 8; g.scale = scale;
    g.splits = splits; g.tiles_n = (int)((N + kCols - 1) / kCols);
    g.tiles_m = (int)((M + rows_per_tile(M) - 1) / rows_per_tile(M));
    if (splits > 1) { g.out = (float *)workspace; g.out_ld = N; g.plane = M * N; }
    else            { g.out = C; g.out_ld = ldc; g.plane = 0; }
    static OncePerDevice configured;
    if (configured.first(device)) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_w8_rows_kernel<1, 4, 8>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(8)));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_w8_rows_kernel<2, 4, 8>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(8)));
    }
    const dim3 grid((unsigned)(g.tiles_n * g.tiles_m * splits));
    if (M <= 32)      hipLaunchKernelGGL((gemm_w8_rows_kernel<1, 4, 8>), grid, dim3(512), lds_bytes(8), st, g);
    else              hipLaunchKernelGGL((gemm_w8_rows_kernel<2, 4, 8>), grid, dim3(512), lds_bytes(8), st, g);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // namespace cn
