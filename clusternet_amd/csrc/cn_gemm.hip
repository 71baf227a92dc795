// fp32 GEMM for gfx950 on the matrix cores: C = op(A) op(B), row-major, alpha 1, beta 0.
//
// One kernel template covers dot (N,N), Tdot (T,N), dotT (N,T) and the fused variant whose B
// operand is 8-bit codes.  Structure:
//   * workgroup = 256 lanes = 4 wavefronts in a 2 x 2 arrangement, output tile 128 x 128,
//     each wavefront owns 64 x 64 = 2 x 2 blocks of v_mfma_f32_32x32x2_f32 (64 accumulators/lane)
//   * K advances 32 at a time through two LDS stages (global -> registers -> LDS, one barrier per
//     stage); both operands sit in LDS as [row][k] with k contiguous, so every lane fetches the
//     four k values of a block row with one 16-byte LDS read and feeds four MFMAs from it
//   * the operand whose memory is contiguous along k (A of dot/dotT, B of dotT) is copied as is;
//     the operand contiguous along its row/column index (B of dot/Tdot, A of Tdot) is read in
//     coalesced 16-byte pieces along that index and transposed 4 x 4 in registers on its way in
//   * 16-byte LDS columns are XOR-swizzled by the row number so that neither the transposing
//     writes nor the MFMA-side reads pile up on one bank group
//   * K may be split into chunks (one workgroup per chunk and tile); chunk results go to a
//     workspace and a second kernel adds them in a fixed order
//   * block ids are remapped so that the workgroups an XCD receives (ids congruent mod 8) cover a
//     contiguous range of work units and share their A/B panels in that XCD's L2.
#include "cn_internal.h"

namespace cn {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = kTileM, BN = kTileN, BK = kTileK;
constexpr int kGemmThreads = 256;
constexpr int kStageFloats = 128 * BK;  // one operand, one stage
constexpr int kNumXcd = 8;

struct GemmArgs {
    const float *A;
    const void *B;       // float (plain) or uint8_t codes (fused)
    float *C;
    float *partial;      // [splits][M][N] when splits > 1
    int64_t M, N, K, lda, ldb, ldc;
    int64_t tiles_n, tiles, k_iters, iters_per_split;
    uint32_t units;
    int splits;
    int vec_a, vec_b;    // operand base and leading dimension allow 16-byte (A, B) / 4-byte (codes) loads
    float scale;         // fused: decode scale
    const float *table;  // fused: 126-entry codebook
};

__device__ __forceinline__ int swizzle_of(int row) { return (row & 7) ^ ((row >> 3) & 3); }
__device__ __forceinline__ int lds_offset(int row, int quad) {
    return row * BK + ((quad ^ swizzle_of(row)) << 2);
}

// ---- global -> register loaders ----------------------------------------------------------------
// "kc": operand stored [index][k] (k contiguous).  Lane t covers k quad (t & 7) of rows
// (t >> 3) + 32 j, j = 0..3.
__device__ __forceinline__ void load_kc(const float *__restrict__ P, int64_t ld, int64_t row0,
                                        int64_t rows, int64_t k0, int64_t K, bool fast, f32x4 (&reg)[4]) {
    const int kq = threadIdx.x & 7, rb = threadIdx.x >> 3;
    const int64_t gk = k0 + 4 * kq;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t gr = row0 + rb + 32 * j;
        const float *src = P + gr * ld + gk;
        if (fast) {
            reg[j] = *reinterpret_cast<const f32x4 *>(src);
        } else {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (gr < rows) {
                if (gk + 0 < K) v.x = src[0];
                if (gk + 1 < K) v.y = src[1];
                if (gk + 2 < K) v.z = src[2];
                if (gk + 3 < K) v.w = src[3];
            }
            reg[j] = v;
        }
    }
}

__device__ __forceinline__ void store_kc(float *__restrict__ lds, const f32x4 (&reg)[4]) {
    const int kq = threadIdx.x & 7, rb = threadIdx.x >> 3;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        *reinterpret_cast<f32x4 *>(lds + lds_offset(rb + 32 * j, kq)) = reg[j];
}

// "ic": operand stored [k][index] (index contiguous).  Lane t covers indices 4 (t & 31) .. +3 of
// k rows 4 (t >> 5) .. +3.
__device__ __forceinline__ void load_ic(const float *__restrict__ P, int64_t ld, int64_t col0,
                                        int64_t cols, int64_t k0, int64_t K, bool fast, f32x4 (&reg)[4]) {
    const int cq = threadIdx.x & 31, kq = threadIdx.x >> 5;
    const int64_t gc = col0 + 4 * cq;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int64_t gk = k0 + 4 * kq + r;
        const float *src = P + gk * ld + gc;
        if (fast) {
            reg[r] = *reinterpret_cast<const f32x4 *>(src);
        } else {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (gk < K) {
                if (gc + 0 < cols) v.x = src[0];
                if (gc + 1 < cols) v.y = src[1];
                if (gc + 2 < cols) v.z = src[2];
                if (gc + 3 < cols) v.w = src[3];
            }
            reg[r] = v;
        }
    }
}

__device__ __forceinline__ void store_ic(float *__restrict__ lds, const f32x4 (&reg)[4]) {
    const int cq = threadIdx.x & 31, kq = threadIdx.x >> 5;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        f32x4 v = {reg[0][t], reg[1][t], reg[2][t], reg[3][t]};
        *reinterpret_cast<f32x4 *>(lds + lds_offset(4 * cq + t, kq)) = v;
    }
}

// Fused variant: B is [k][n] 8-bit codes; same lane layout as load_ic, four codes per 32-bit word.
__device__ __forceinline__ void load_codes(const uint8_t *__restrict__ W, int64_t ld, int64_t col0,
                                           int64_t cols, int64_t k0, int64_t K, bool fast, uint32_t (&reg)[4]) {
    const int cq = threadIdx.x & 31, kq = threadIdx.x >> 5;
    const int64_t gc = col0 + 4 * cq;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int64_t gk = k0 + 4 * kq + r;
        const uint8_t *src = W + gk * ld + gc;
        if (fast) {
            reg[r] = *reinterpret_cast<const uint32_t *>(src);
        } else {
            // out-of-range positions take code 0 with a zero multiplier on the A side being
            // impossible, so they must decode to exactly 0: mark them and zero after decoding
            uint32_t w = 0;
            if (gk < K) {
                if (gc + 0 < cols) w |= (uint32_t)src[0];
                if (gc + 1 < cols) w |= (uint32_t)src[1] << 8;
                if (gc + 2 < cols) w |= (uint32_t)src[2] << 16;
                if (gc + 3 < cols) w |= (uint32_t)src[3] << 24;
            }
            reg[r] = w;
        }
    }
}

__device__ __forceinline__ void store_codes(float *__restrict__ lds, const float *__restrict__ lut,
                                            const uint32_t (&reg)[4], int64_t col0, int64_t cols,
                                            int64_t k0, int64_t K, bool fast) {
    const int cq = threadIdx.x & 31, kq = threadIdx.x >> 5;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        f32x4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float d = lut[(reg[r] >> (8 * t)) & 0xffu];
            if (!fast && (k0 + 4 * kq + r >= K || col0 + 4 * cq + t >= cols)) d = 0.0f;
            v[r] = d;
        }
        *reinterpret_cast<f32x4 *>(lds + lds_offset(4 * cq + t, kq)) = v;
    }
}

// ---- one K stage of MFMAs ----------------------------------------------------------------------
// Within each group of 8 k values, MFMA s (0..3) consumes k = 8 g + 4 h + s from lane half h on
// both operands, i.e. the k order inside a stage is permuted identically for A and B.
__device__ __forceinline__ void mfma_stage(const float *__restrict__ sA, const float *__restrict__ sB,
                                           const int (&row_a)[2], const int (&row_b)[2], int half,
                                           f32x16 (&acc)[2][2]) {
#pragma unroll
    for (int g = 0; g < BK / 8; ++g) {
        f32x4 a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            a[i] = *reinterpret_cast<const f32x4 *>(sA + lds_offset(row_a[i], 2 * g + half));
            b[i] = *reinterpret_cast<const f32x4 *>(sB + lds_offset(row_b[i], 2 * g + half));
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi][s], b[ni][s], acc[mi][ni], 0, 0, 0);
    }
}

template <bool A_KC, bool B_KC, bool W8>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *sA = smem;                       // [2][kStageFloats]
    float *sB = smem + 2 * kStageFloats;    // [2][kStageFloats]
    float *sLut = smem + 4 * kStageFloats;  // [256], fused only

    // Work unit of this workgroup.  Hardware hands consecutive block ids to the XCDs round-robin;
    // give XCD x the x-th contiguous slice of the unit range.
    const uint32_t bid = blockIdx.x, U = g.units;
    const uint32_t xcd = bid % kNumXcd, idx = bid / kNumXcd;
    const uint32_t per = U / kNumXcd, rem = U % kNumXcd;
    const uint32_t unit = xcd * per + (xcd < rem ? xcd : rem) + idx;

    const int64_t split = unit / g.tiles;
    const int64_t tile = unit % g.tiles;
    const int64_t tm = tile / g.tiles_n, tn = tile % g.tiles_n;
    const int64_t m0 = tm * BM, n0 = tn * BN;
    const int64_t it0 = split * g.iters_per_split;
    int64_t it1 = it0 + g.iters_per_split;
    if (it1 > g.k_iters) it1 = g.k_iters;

    if (W8) {
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

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    int row_a[2], row_b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        row_a[i] = wave_m * 64 + i * 32 + l32;
        row_b[i] = wave_n * 64 + i * 32 + l32;
    }

    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    const bool inner_m = (m0 + BM <= g.M), inner_n = (n0 + BN <= g.N);
    const uint8_t *Wc = reinterpret_cast<const uint8_t *>(g.B);
    const float *Bf = reinterpret_cast<const float *>(g.B);

    f32x4 ra[4], rb[4];
    uint32_t rc[4];
    auto fetch = [&](int64_t it) {
        const int64_t k0 = it * BK;
        const bool inner_k = (k0 + BK <= g.K);
        if (A_KC) load_kc(g.A, g.lda, m0, g.M, k0, g.K, g.vec_a && inner_m && inner_k, ra);
        else      load_ic(g.A, g.lda, m0, g.M, k0, g.K, g.vec_a && inner_m && inner_k, ra);
        if (W8)        load_codes(Wc, g.ldb, n0, g.N, k0, g.K, g.vec_b && inner_n && inner_k, rc);
        else if (B_KC) load_kc(Bf, g.ldb, n0, g.N, k0, g.K, g.vec_b && inner_n && inner_k, rb);
        else           load_ic(Bf, g.ldb, n0, g.N, k0, g.K, g.vec_b && inner_n && inner_k, rb);
    };
    auto stash = [&](int64_t it, int buf) {
        const int64_t k0 = it * BK;
        if (A_KC) store_kc(sA + buf * kStageFloats, ra);
        else      store_ic(sA + buf * kStageFloats, ra);
        if (W8)        store_codes(sB + buf * kStageFloats, sLut, rc, n0, g.N, k0, g.K,
                                   g.vec_b && inner_n && (k0 + BK <= g.K));
        else if (B_KC) store_kc(sB + buf * kStageFloats, rb);
        else           store_ic(sB + buf * kStageFloats, rb);
    };

    if (it0 < it1) {
        fetch(it0);
        stash(it0, 0);
        __syncthreads();
        int buf = 0;
        for (int64_t it = it0; it < it1; ++it) {
            const bool more = (it + 1 < it1);
            if (more) fetch(it + 1);
            mfma_stage(sA + buf * kStageFloats, sB + buf * kStageFloats, row_a, row_b, half, acc);
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
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int64_t col = n0 + wave_n * 64 + ni * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t row = m0 + wave_m * 64 + mi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (row < g.M && col < g.N) dst[row * ldd + col] = acc[mi][ni][r];
            }
        }
}

// C[m][n] = sum over chunks of partial[chunk][m][n], chunks added in ascending order.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial, int splits,
                                                            int64_t M, int64_t N, float *__restrict__ C,
                                                            int64_t ldc, int vec) {
    const int64_t plane = M * N;
    if (vec) {
        const int64_t nq = N / 4, total = M * nq;
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
             i += (int64_t)gridDim.x * blockDim.x) {
            const int64_t m = i / nq, q = i % nq;
            const float *src = partial + m * N + 4 * q;
            f32x4 s = *reinterpret_cast<const f32x4 *>(src);
            for (int c = 1; c < splits; ++c) s += *reinterpret_cast<const f32x4 *>(src + c * plane);
            *reinterpret_cast<f32x4 *>(C + m * ldc + 4 * q) = s;
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < plane;
             i += (int64_t)gridDim.x * blockDim.x) {
            const int64_t m = i / N, n = i % N;
            float s = partial[i];
            for (int c = 1; c < splits; ++c) s += partial[i + c * plane];
            C[m * ldc + n] = s;
        }
    }
}

__global__ __launch_bounds__(256) void zero_matrix_kernel(float *__restrict__ C, int64_t M, int64_t N, int64_t ldc) {
    const int64_t total = M * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x)
        C[(i / N) * ldc + (i % N)] = 0.0f;
}

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

template <bool A_KC, bool B_KC, bool W8>
static cn_status launch(const GemmArgs &args, hipStream_t st) {
    const size_t lds = (size_t)(4 * kStageFloats + (W8 ? 256 : 0)) * sizeof(float);
    static bool configured = false;
    if (!configured) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<A_KC, B_KC, W8>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    hipLaunchKernelGGL((gemm_kernel<A_KC, B_KC, W8>), dim3(args.units), dim3(kGemmThreads), lds, st, args);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

static cn_status gemm_impl(int ta, int tb, bool w8, int64_t M, int64_t N, int64_t K, const float *A,
                           int64_t lda, const void *B, int64_t ldb, float scale, float *C, int64_t ldc,
                           void *stream) {
    const char *who = w8 ? "gemm_f32_w8" : "gemm_f32";
    if (M < 0 || N < 0 || K < 0) { set_error("%s: negative dimension", who); return CN_ERR_SHAPE; }
    if (lda < (ta ? M : K) || ldb < (tb ? K : N) || ldc < N) {
        set_error("%s: leading dimension too small (lda %lld, ldb %lld, ldc %lld for M %lld N %lld K %lld)",
                  who, (long long)lda, (long long)ldb, (long long)ldc, (long long)M, (long long)N, (long long)K);
        return CN_ERR_SHAPE;
    }
    if (M == 0 || N == 0) return CN_OK;
    if (!C || (K > 0 && (!A || !B))) { set_error("%s: NULL operand", who); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    if (K == 0) {
        hipLaunchKernelGGL(zero_matrix_kernel, dim3(ctx->num_cu * 4), dim3(256), 0, st, C, M, N, ldc);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    GemmPlan plan = plan_gemm(M, N, K, ctx->num_cu, ctx->workspace_bytes);
    if (plan.units <= 0 || plan.units > 0x7fffffffLL) {
        set_error("%s: %lld work units exceed the launch limit", who, (long long)plan.units);
        return CN_ERR_SHAPE;
    }
    if (plan.splits > 1 && (size_t)plan.splits * (size_t)M * (size_t)N * sizeof(float) > ctx->workspace_bytes) {
        set_error("%s: split-K workspace too small", who);
        return CN_ERR_WORKSPACE;
    }
    GemmArgs a;
    a.A = A; a.B = B; a.C = C; a.partial = (float *)ctx->workspace;
    a.M = M; a.N = N; a.K = K; a.lda = lda; a.ldb = ldb; a.ldc = ldc;
    a.tiles_n = plan.tiles_n; a.tiles = plan.tiles_m * plan.tiles_n;
    a.k_iters = plan.k_iters; a.iters_per_split = plan.iters_per_split;
    a.units = (uint32_t)plan.units; a.splits = plan.splits;
    a.vec_a = aligned(A, 16) && (lda % 4 == 0);
    a.vec_b = w8 ? (aligned(B, 4) && (ldb % 4 == 0)) : (aligned(B, 16) && (ldb % 4 == 0));
    a.scale = scale; a.table = ctx->table;

    if (w8)             s = launch<true, false, true>(a, st);
    else if (!ta && !tb) s = launch<true, false, false>(a, st);
    else if (ta && !tb)  s = launch<false, false, false>(a, st);
    else if (!ta && tb)  s = launch<true, true, false>(a, st);
    else                 s = launch<false, true, false>(a, st);
    if (s != CN_OK) return s;

    if (plan.splits > 1) {
        int vec = (N % 4 == 0) && (ldc % 4 == 0) && aligned(C, 16);
        int64_t work = vec ? M * (N / 4) : M * N;
        int64_t blocks = (work + 255) / 256;
        int64_t cap = (int64_t)ctx->num_cu * 8;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0, st,
                           (const float *)ctx->workspace, plan.splits, M, N, C, ldc, vec);
        CN_HIP(hipGetLastError());
    }
    return CN_OK;
}

}  // namespace cn

using namespace cn;

extern "C" {

cn_status cn_gemm_f32(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                      const float *B, int64_t ldb, float *C, int64_t ldc, void *stream) {
    return gemm_impl(trans_a != 0, trans_b != 0, false, M, N, K, A, lda, B, ldb, 1.0f, C, ldc, stream);
}

cn_status cn_gemm_f32_w8(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const uint8_t *W,
                         int64_t ldw, float scale, float *C, int64_t ldc, void *stream) {
    return gemm_impl(0, 0, true, M, N, K, A, lda, W, ldw, scale, C, ldc, stream);
}

}  // extern "C"
