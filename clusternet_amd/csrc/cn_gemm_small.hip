// Products that are too small to fill the chip with tiles: one launch, no LDS staging, no second kernel.
//
// The tiled kernel serves a product like 128 x 1024 x 784 (a layer of the reference's MNIST test network,
// source/clusterNet.cpp:230-298 on tests/testSuite.cu's shapes) as 160 workgroups on K chunks plus a kernel that adds
// the chunks: 10 us, nearly all of it latencies one behind the other (launch, first stage, barrier per stage, second
// launch, the planes' round trip).  Here a workgroup owns one 32 x 32 (or 16 x 16) block of the result and its wavefronts split K
// among themselves: every wavefront loads its slice of both operands straight into the registers the matrix
// instruction reads (all loads of a step in flight at once), accumulates its share of the block, the shares meet in LDS
// and are added in ascending order of the slices, which makes the result independent of scheduling.
#include "cn_internal.h"

namespace cn {

namespace {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

struct SmallArgs {
    const float *A, *B;
    float *C;
    int64_t M, N, K, lda, ldb, ldc;
    int tiles_m;
    uint32_t *amax;  // if not NULL: receives max |C| by atomicMax on the bit patterns (the word starts at 0)
};

constexpr int kGroupsAhead = 4;  // groups whose loads are in flight together (twice that with the next step's)

// The matrix instruction for a block of kBlock x kBlock results: 32 -> v_mfma_f32_32x32x2_f32 (lanes in 2 k-halves, 16
// accumulators per lane), 16 -> v_mfma_f32_16x16x4_f32 (lanes in 4 k-quarters, 4 accumulators).  Lane (sub, i), sub =
// lane / kBlock, supplies A[i][k] and B[k][i] for the instruction's k = sub.  A group takes four instructions and
// covers 4 * kSub k: instruction s consumes k0 + 4 sub + s from the lanes of `sub`, for both operands, so an operand
// that is contiguous along k is read as one 16-byte vector per lane and group.  Accumulator r of lane (sub, j) is row
// (r / 4) * 4 kSub + 4 sub + r % 4, column j of the block.
template <int kBlock>
struct Mfma {
    static constexpr int kSub = 64 / kBlock;
    static constexpr int kGroupK = 4 * kSub;
    static constexpr int kAcc = kBlock * kBlock / 64;
    typedef float acc_t __attribute__((ext_vector_type(kAcc)));
    static __device__ __forceinline__ acc_t run(float x, float y, acc_t acc) {
        if constexpr (kBlock == 32) return __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc, 0, 0, 0);
        else                        return __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, acc, 0, 0, 0);
    }
};

// kAlongK: the operand's memory is [index][k] (k contiguous): A of dot and dotT, B of dotT.  Else [k][index].
template <bool kAlongK, int kGroupK>
struct Slice {
    f32x4_t v[kGroupsAhead];
    // `index`: the lane's row of A (column of B), clamped into the matrix; k0: first k of the first group; groups past
    // `groups` repeat the first one's addresses (their values are not used).
    __device__ __forceinline__ void load(const float *base, int64_t ld, int64_t index, int64_t k0, int groups, int sub) {
#pragma unroll
        for (int g = 0; g < kGroupsAhead; ++g) {
            const int64_t k = k0 + (g < groups ? kGroupK * g : 0) + 4 * sub;
            if (kAlongK) {
                v[g] = *reinterpret_cast<const f32x4_t *>(base + index * ld + k);
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) v[g][s] = base[(k + s) * ld + index];
            }
        }
    }
};

template <int kBlock, int kWaves, bool kAAlongK, bool kBAlongK>
__global__ __launch_bounds__(kWaves * 64) void gemm_small_kernel(SmallArgs a) {
    using I = Mfma<kBlock>;
    __shared__ float part[kWaves][I::kAcc][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int sub = lane / kBlock, idx = lane % kBlock;
    const int64_t tm = blockIdx.x % a.tiles_m, tn = blockIdx.x / a.tiles_m;
    const int64_t m0 = tm * kBlock, n0 = tn * kBlock;
    const int64_t row = m0 + idx < a.M ? m0 + idx : a.M - 1;  // lanes past the edge read the last row; nothing of theirs is stored
    const int64_t col = n0 + idx < a.N ? n0 + idx : a.N - 1;
    // this wavefront's groups
    const int total = (int)(a.K / I::kGroupK);
    const int each = (total + kWaves - 1) / kWaves;
    const int g_begin = wave * each < total ? wave * each : total;
    const int g_end = g_begin + each < total ? g_begin + each : total;

    typename I::acc_t acc;
#pragma unroll
    for (int r = 0; r < I::kAcc; ++r) acc[r] = 0.0f;

    // two register sets, named so that every index is a constant: the next step's loads are in flight while this
    // step's instructions run
    typedef Slice<kAAlongK, I::kGroupK> SliceA;
    typedef Slice<kBAlongK, I::kGroupK> SliceB;
    SliceA a_even, a_odd;
    SliceB b_even, b_odd;
    auto request = [&](int g, SliceA &sa, SliceB &sb) {
        const int left = g_end - g;
        const int groups = left < kGroupsAhead ? left : kGroupsAhead;
        sa.load(a.A, a.lda, row, (int64_t)g * I::kGroupK, groups, sub);
        sb.load(a.B, a.ldb, col, (int64_t)g * I::kGroupK, groups, sub);
    };
    auto consume = [&](int g, const SliceA &sa, const SliceB &sb) {
        const int left = g_end - g;
#pragma unroll
        for (int q = 0; q < kGroupsAhead; ++q) {
            const bool live = q < left;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float x = live ? sa.v[q][s] : 0.0f;
                const float y = live ? sb.v[q][s] : 0.0f;
                acc = I::run(x, y, acc);
            }
        }
    };
    if (g_begin < g_end) {
        request(g_begin, a_even, b_even);
        for (int g = g_begin;; g += 2 * kGroupsAhead) {
            if (g + kGroupsAhead < g_end) request(g + kGroupsAhead, a_odd, b_odd);
            consume(g, a_even, b_even);
            if (g + kGroupsAhead >= g_end) break;
            if (g + 2 * kGroupsAhead < g_end) request(g + 2 * kGroupsAhead, a_even, b_even);
            consume(g + kGroupsAhead, a_odd, b_odd);
            if (g + 2 * kGroupsAhead >= g_end) break;
        }
    }
#pragma unroll
    for (int r = 0; r < I::kAcc; ++r) part[wave][r][lane] = acc[r];
    __syncthreads();
    constexpr int kOutputs = kBlock * kBlock, kLanes = kWaves * 64;
    uint32_t largest = 0;
#pragma unroll
    for (int o = 0; o < (kOutputs + kLanes - 1) / kLanes; ++o) {
        const int at = (int)threadIdx.x + o * kLanes;
        if (at < kOutputs) {
            const int r = at >> 6, ln = at & 63;
            float sum = part[0][r][ln];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) sum += part[w][r][ln];
            const int64_t out_row = m0 + (r >> 2) * (4 * I::kSub) + 4 * (ln / kBlock) + (r & 3), out_col = n0 + (ln % kBlock);
            if (out_row < a.M && out_col < a.N) {
                a.C[out_row * a.ldc + out_col] = sum;
                const uint32_t bits = __float_as_uint(sum) & 0x7fffffffu;
                largest = bits > largest ? bits : largest;
            }
        }
    }
    if (a.amax) {  // the same for every lane
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t other = (uint32_t)__shfl_xor((int)largest, off, 64);
            largest = other > largest ? other : largest;
        }
        if (lane == 0 && largest) atomicMax(a.amax, largest);
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Fewer 32 x 32 blocks than this: 16 x 16 blocks instead, four times as many workgroups for the same product.
constexpr int64_t kFineBlocksBelow = 192;

inline bool fine_blocks(int64_t M, int64_t N, int64_t K) {
    return ((M + 31) / 32) * ((N + 31) / 32) < kFineBlocksBelow && K % 16 == 0;
}

template <int kBlock, bool kAAlongK, bool kBAlongK>
cn_status launch_small(const SmallArgs &a, int64_t tiles, hipStream_t st) {
    // enough k per wavefront to be worth a wavefront: four groups and more each
    const int64_t groups = a.K / Mfma<kBlock>::kGroupK;
    if (groups >= 64)      hipLaunchKernelGGL((gemm_small_kernel<kBlock, 16, kAAlongK, kBAlongK>), dim3((unsigned)tiles), dim3(1024), 0, st, a);
    else if (groups >= 32) hipLaunchKernelGGL((gemm_small_kernel<kBlock, 8, kAAlongK, kBAlongK>), dim3((unsigned)tiles), dim3(512), 0, st, a);
    else                   hipLaunchKernelGGL((gemm_small_kernel<kBlock, 4, kAAlongK, kBAlongK>), dim3((unsigned)tiles), dim3(256), 0, st, a);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

template <int kBlock>
cn_status launch_block(int ta, int tb, SmallArgs a, hipStream_t st) {
    a.tiles_m = (int)((a.M + kBlock - 1) / kBlock);
    const int64_t tiles = (int64_t)a.tiles_m * ((a.N + kBlock - 1) / kBlock);
    if (!ta && !tb) return launch_small<kBlock, true, false>(a, tiles, st);
    if (ta && !tb)  return launch_small<kBlock, false, false>(a, tiles, st);
    if (!ta && tb)  return launch_small<kBlock, true, true>(a, tiles, st);
    return launch_small<kBlock, false, true>(a, tiles, st);
}

}  // namespace

// Whether the product is one for this kernel: K in whole groups of 8, operands that are contiguous along k readable
// as 16-byte vectors, and few enough blocks and little enough work that latency, not the chip, is the limit.  Measured
// against the tiled kernel with its chunk sum, replayed from a graph: 128 x 1024 x 784 7.0 us against 9.9 us, its
// dotT 9.9 against 10.9, 128 x 10 x 1024 4.6 against 11.5, 128 x 1024 x 80 3.2 against 6.2, 256 x 1024 x 1024 9.9
// against 12.3, 128 x 4096 x 512 10.7 against 13.5; beyond the bounds the tiled kernel is ahead (784 x 1024 x 128: 6.3
// against 5.9; 1024 x 1024 x 256: 9.8 against 8.3; 32 x 4096 x 2048 in 16 x 16 blocks: 24 against 13).
bool gemm_small_applies(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                        int64_t ldb) {
    if (K < 32 || K % 8 != 0) return false;
    const int64_t blocks = ((M + 31) / 32) * ((N + 31) / 32);
    if (blocks > kSmallMaxBlocks) return false;
    if (M * N * K > (fine_blocks(M, N, K) ? kSmallMaxWork / 2 : kSmallMaxWork)) return false;
    if (!ta && !(aligned16(A) && lda % 4 == 0)) return false;
    if (tb && !(aligned16(B) && ldb % 4 == 0)) return false;
    return true;
}

cn_status gemm_small(int ta, int tb, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                     int64_t ldb, float *C, int64_t ldc, uint32_t *amax, hipStream_t st) {
    SmallArgs a{A, B, C, M, N, K, lda, ldb, ldc, 0, amax};
    if (fine_blocks(M, N, K)) return launch_block<16>(ta, tb, a, st);
    return launch_block<32>(ta, tb, a, st);
}

}  // namespace cn
