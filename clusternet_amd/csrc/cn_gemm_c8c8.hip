// Both operands as 8-bit codes: C += decodeA(A) decodeB(B), the product of the reference's dot8bit and
// dot8bit_shared (source/clusterNet.cpp:1409-1431 -> source/basicOps.cu:1455-1472 -> kDot8bit,
// source/clusterKernels.cu:1717-1762, and kDot8bit_shared, :1764-1843).  Both of those expand each operand through a
// 256-entry table of its own in shared memory, whose special codes are not the codec's (and mix the two precisions
// up, :1731-1738); the tables here are built the same way, entry by entry.
//
// One launch, nothing staged in memory: a workgroup owns a 32 x 32 block of C and its wavefronts split K among
// themselves.  A lane reads the four codes of its row of A (one word where the alignment allows) and of its column of
// B for every group of eight k, expands them through the tables in LDS straight into the operand registers of
// v_mfma_f32_32x32x2_f32, and the wavefronts' shares meet in LDS and are added in ascending order of k, so the result
// does not depend on scheduling.  The products of a k at or beyond K are exactly zero.
#include "cn_internal.h"

namespace cn {

namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

struct C8Args {
    const uint8_t *A, *B;
    float *C;
    int64_t M, N, K, lda, ldb, ldc;
    int tiles_m;
    int a_words;  // rows of A start on 4-byte boundaries: four codes along k are one word
    float precision_a, precision_b;
    const float *table;  // the 126-entry codebook
};

constexpr int kAhead = 4;  // groups of eight k whose codes are in flight together (twice that with the next step's)

struct Codes {
    uint32_t a[kAhead], b[kAhead];  // code s of the group in byte s
};

template <int kWaves>
__global__ __launch_bounds__(kWaves * 64) void gemm_c8c8_kernel(C8Args a) {
    __shared__ float lut_a[256], lut_b[256];
    __shared__ float part[kWaves][16][64];
    const int t = threadIdx.x;
    {   // source/clusterKernels.cu:1725-1739, statement by statement
        const float pa = a.precision_a, pb = a.precision_b;
        if (t < 126) {
            const float v = a.table[t];
            lut_a[t] = v * pa;
            lut_a[t + 128] = -(v * pa);
            lut_b[t] = v * pb;
            lut_b[t + 128] = -(v * pb);
        } else if (t == 126) {
            lut_a[126] = 0.0f;
            lut_b[126] = 0.0f;
            lut_a[127] = pa;
            lut_b[127] = -pa;
            lut_a[254] = -0.0f;
            lut_b[254] = -0.0f;
            lut_a[255] = pb;
            lut_b[255] = -pb;
        }
    }
    __syncthreads();

    // Lane (sub, i), sub = lane / 32, supplies A[i][k] and B[k][i] for the instruction's k = sub; a group is four
    // instructions and eight k, instruction s taking k0 + 4 sub + s from the lanes of `sub`.  Accumulator r of lane
    // (sub, j) is row (r / 4) * 8 + 4 sub + r % 4, column j of the block.
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int sub = lane >> 5, idx = lane & 31;
    const int64_t tm = blockIdx.x % a.tiles_m, tn = blockIdx.x / a.tiles_m;
    const int64_t m0 = tm * 32, n0 = tn * 32;
    const int64_t row = m0 + idx < a.M ? m0 + idx : a.M - 1;  // lanes past the edge read the last row; nothing of theirs is stored
    const int64_t col = n0 + idx < a.N ? n0 + idx : a.N - 1;
    const uint8_t *arow = a.A + row * a.lda;
    const uint8_t *bcol = a.B + col;
    const int total = (int)((a.K + 7) / 8);
    const int each = (total + kWaves - 1) / kWaves;
    const int g_begin = wave * each < total ? wave * each : total;
    const int g_end = g_begin + each < total ? g_begin + each : total;

    f32x16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    auto request = [&](int g, Codes &c) {
#pragma unroll
        for (int q = 0; q < kAhead; ++q) {
            const int64_t k = (int64_t)(g + q < g_end ? g + q : g) * 8 + 4 * sub;  // past the slice: the first group again, unused
            if (a.a_words && k + 4 <= a.K) {
                c.a[q] = *reinterpret_cast<const uint32_t *>(arow + k);
            } else {
                uint32_t w = 0;
#pragma unroll
                for (int s = 0; s < 4; ++s) w |= (uint32_t)arow[k + s < a.K ? k + s : a.K - 1] << (8 * s);
                c.a[q] = w;
            }
            uint32_t w = 0;
#pragma unroll
            for (int s = 0; s < 4; ++s) w |= (uint32_t)bcol[(k + s < a.K ? k + s : a.K - 1) * a.ldb] << (8 * s);
            c.b[q] = w;
        }
    };
    auto consume = [&](int g, const Codes &c) {
#pragma unroll
        for (int q = 0; q < kAhead; ++q) {
            const int64_t k = (int64_t)(g + q) * 8 + 4 * sub;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bool live = g + q < g_end && k + s < a.K;
                const float x = lut_a[(c.a[q] >> (8 * s)) & 0xffu], y = lut_b[(c.b[q] >> (8 * s)) & 0xffu];
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(live ? x : 0.0f, live ? y : 0.0f, acc, 0, 0, 0);
            }
        }
    };
    if (g_begin < g_end) {
        Codes even, odd;
        request(g_begin, even);
        for (int g = g_begin;; g += 2 * kAhead) {
            if (g + kAhead < g_end) request(g + kAhead, odd);
            consume(g, even);
            if (g + kAhead >= g_end) break;
            if (g + 2 * kAhead < g_end) request(g + 2 * kAhead, even);
            consume(g + kAhead, odd);
            if (g + 2 * kAhead >= g_end) break;
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave][r][lane] = acc[r];
    __syncthreads();
#pragma unroll
    for (int o = 0; o < (1024 + kWaves * 64 - 1) / (kWaves * 64); ++o) {
        const int at = t + o * kWaves * 64;
        if (at < 1024) {
            const int r = at >> 6, ln = at & 63;
            float sum = part[0][r][ln];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) sum += part[w][r][ln];
            const int64_t out_row = m0 + (r >> 2) * 8 + 4 * (ln >> 5) + (r & 3), out_col = n0 + (ln & 31);
            if (out_row < a.M && out_col < a.N) {
                float *c = a.C + out_row * a.ldc + out_col;
                *c = *c + sum;
            }
        }
    }
}

}  // namespace

extern "C" {

cn_status cn_gemm_c8c8_add(int64_t M, int64_t N, int64_t K, const uint8_t *A, int64_t lda, const uint8_t *B, int64_t ldb,
                           float precision_a, float precision_b, float *C, int64_t ldc, void *stream) {
    if (M < 0 || N < 0 || K < 0) { set_error("gemm_c8c8_add: negative dimension"); return CN_ERR_SHAPE; }
    if (lda < K || ldb < N || ldc < N) { set_error("gemm_c8c8_add: leading dimension too small"); return CN_ERR_SHAPE; }
    if (M == 0 || N == 0 || K == 0) return CN_OK;  // an empty sum adds nothing
    if (!A || !B || !C) { set_error("gemm_c8c8_add: NULL pointer"); return CN_ERR_NULL; }
    const int64_t tiles_m = (M + 31) / 32, tiles = tiles_m * ((N + 31) / 32);
    if (tiles > 0x7fffffffLL) { set_error("gemm_c8c8_add: more than 2^31 blocks of 32 x 32"); return CN_ERR_SHAPE; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    C8Args a{A, B, C, M, N, K, lda, ldb, ldc, (int)tiles_m,
             (reinterpret_cast<uintptr_t>(A) & 3u) == 0 && lda % 4 == 0 ? 1 : 0, precision_a, precision_b, ctx->table};
    // enough k per wavefront to be worth a wavefront
    if ((K + 7) / 8 >= 32) hipLaunchKernelGGL(gemm_c8c8_kernel<8>, dim3((unsigned)tiles), dim3(512), 0, st, a);
    else                   hipLaunchKernelGGL(gemm_c8c8_kernel<4>, dim3((unsigned)tiles), dim3(256), 0, st, a);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // extern "C"

}  // namespace cn
