// Sparse (CSR) x dense products for gfx950 and the conversion from dense storage.
//
// The input batch of the reference's large configuration is 2 % dense.  A dense product streams the
// weight matrix once and spends 50x the necessary flops doing so; the products below are bound by
// the same stream (or by writing the result) and do no wasted arithmetic.  S is an R x C matrix in
// CSR form (row_ptr[R + 1], col_idx[nnz] ascending within a row, vals[nnz]), 32-bit indices.
//
//   csr_gemm        out[R x N] = S B: every output row gathers the B rows of its nonzeros, four columns
//                   per lane, accumulators in registers.  Three kernels by shape: many rows (one
//                   workgroup per row and 1024 columns), few long rows (one wavefront per row and
//                   256-column strip, a strip per XCD; optionally with bias and maxout in the write-out),
//                   and many short rows (blocks of 16 rows, loads requested rows ahead) for the passes
//                   that never store the product: its maximum, its 8-bit codes, and the weight update
//   csr_transpose   CSR(S) -> CSR(S^T), for the products with the transposed sparse operand
//   csr_from_dense, csr_to_dense   the conversions
//
// With X the 128 x 100000 batch:  X W = CSR(X) W and X^T E = CSR(X^T) E.
// Sums run over the nonzeros in ascending order with a rounded product and a rounded addition per
// term, so the results are reproducible to the bit.
#include <type_traits>

#include "cn_internal.h"
#include "cn_encode_table.h"

namespace cn {

namespace {

constexpr int kT = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---- dense -> CSR ----------------------------------------------------------------------------------
// counts[i] = number of nonzeros of row i of op(A); op = identity or transpose.  A value is a nonzero
// when it compares unequal to 0 (so -0.0 is dropped and NaN is kept).
// A row is cut into segments of kSegment columns so that a short, wide matrix still fills the machine.
constexpr int64_t kSegment = 4096;

// counts[r * segments + g] = nonzeros of columns [g kSegment, (g + 1) kSegment) of row r; one workgroup
// per (row, segment).
template <bool kVec>  // kVec: every row segment starts on a 16-byte boundary
__global__ __launch_bounds__(kT) void count_segments_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                            int64_t lda, int64_t segments, int32_t *__restrict__ counts) {
    __shared__ int partial[kT / 64];
    for (int64_t unit = blockIdx.x; unit < rows * segments; unit += gridDim.x) {
        const int64_t r = unit / segments, j0 = (unit % segments) * kSegment;
        const int64_t j1 = (j0 + kSegment < cols) ? j0 + kSegment : cols;
        const float *row = A + r * lda;
        int c = 0;
        int64_t j = j0 + threadIdx.x;
        if (kVec) {
            const f32x4 *v4 = reinterpret_cast<const f32x4 *>(row + j0);
            const int nv = (int)((j1 - j0) >> 2);
            for (int i = threadIdx.x; i < nv; i += kT) {
                const f32x4 v = v4[i];
                c += ((v.x != 0.0f) ? 1 : 0) + ((v.y != 0.0f) ? 1 : 0) + ((v.z != 0.0f) ? 1 : 0) + ((v.w != 0.0f) ? 1 : 0);
            }
            j = j0 + 4 * (int64_t)nv + threadIdx.x;
        }
        for (; j < j1; j += kT) c += (row[j] != 0.0f) ? 1 : 0;
        for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = c;
        __syncthreads();
        if (threadIdx.x == 0) counts[unit] = partial[0] + partial[1] + partial[2] + partial[3];
        __syncthreads();
    }
}

// row_ptr[r] = offset of the first segment of row r; row_ptr[rows] = offsets[rows * segments].
__global__ __launch_bounds__(kT) void row_ptr_from_segments_kernel(const int32_t *__restrict__ offsets, int64_t rows,
                                                                   int64_t segments, int32_t *__restrict__ row_ptr) {
    for (int64_t r = (int64_t)blockIdx.x * kT + threadIdx.x; r <= rows; r += (int64_t)gridDim.x * kT)
        row_ptr[r] = offsets[r * segments];
}

__global__ __launch_bounds__(kT) void count_cols_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                        int64_t lda, int32_t *__restrict__ counts) {
    // one thread per column of A (consecutive threads read consecutive addresses)
    for (int64_t j = (int64_t)blockIdx.x * kT + threadIdx.x; j < cols; j += (int64_t)gridDim.x * kT) {
        int c = 0;
        for (int64_t r = 0; r < rows; ++r) c += (A[r * lda + j] != 0.0f) ? 1 : 0;
        counts[j] = c;
    }
}

__global__ __launch_bounds__(kT) void zero_counts_kernel(int32_t *__restrict__ counts, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x; i < n; i += (int64_t)gridDim.x * kT) counts[i] = 0;
}

// row_ptr[0 .. n] = exclusive prefix sums of counts[0 .. n - 1]; counts == row_ptr is allowed (a tile is
// read completely before it is written); *total = row_ptr[n].  One workgroup walks the array in tiles
// of 256 with coalesced accesses; a tile is scanned by shuffles inside each wavefront and a four-entry
// table across wavefronts.
__global__ __launch_bounds__(kT) void scan_kernel(const int32_t *counts, int64_t n, int32_t *row_ptr,
                                                  int64_t *__restrict__ total) {
    // Sums are carried in 64 bits throughout: the entries may themselves be sums of blocks (up to 2^24 each), so a
    // tile of 256 can pass 2^31, and *total must stay exact for the callers that refuse more than 2^31 - 1 nonzeros.
    __shared__ long long wave_sum[kT / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int64_t carry = 0;
    for (int64_t i0 = 0; i0 < n; i0 += kT) {
        const int64_t i = i0 + threadIdx.x;
        const long long c = (i < n) ? counts[i] : 0;
        long long inc = c;  // inclusive scan within the wavefront
        for (int off = 1; off < 64; off <<= 1) {
            const long long up = __shfl_up(inc, off, 64);
            if (lane >= off) inc += up;
        }
        if (lane == 63) wave_sum[wave] = inc;
        __syncthreads();
        long long before = 0;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        const long long tile_total = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
        if (i < n) row_ptr[i] = (int32_t)(carry + before + inc - c);
        carry += tile_total;
        __syncthreads();
    }
    if (threadIdx.x == 0) { row_ptr[n] = (int32_t)carry; *total = carry; }
}

// Prefix sums of a long array in three launches: sums of blocks of kScanBlock elements, their prefix
// sums (scan_kernel), then every block scans itself from its offset.
constexpr int64_t kScanBlock = 4096;

__global__ __launch_bounds__(kT) void block_sums_kernel(const int32_t *__restrict__ counts, int64_t n,
                                                        int32_t *__restrict__ sums) {
    // A block's sum is carried in 64 bits and stored as at most INT32_MAX: a block that large makes the total reach
    // INT32_MAX, which every caller refuses, instead of wrapping round to a small number that would pass.
    __shared__ long long partial[kT / 64];
    const int64_t i0 = (int64_t)blockIdx.x * kScanBlock;
    const int64_t i1 = (i0 + kScanBlock < n) ? i0 + kScanBlock : n;
    long long c = 0;
    for (int64_t i = i0 + threadIdx.x; i < i1; i += kT) c += counts[i];
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        const long long sum = partial[0] + partial[1] + partial[2] + partial[3];
        sums[blockIdx.x] = sum > 0x7fffffffLL ? 0x7fffffff : (int32_t)sum;
    }
}

__global__ __launch_bounds__(kT) void block_scan_kernel(const int32_t *counts, int64_t n,
                                                        const int32_t *__restrict__ block_offsets, int32_t *row_ptr,
                                                        const int64_t *__restrict__ total) {
    __shared__ int wave_sum[kT / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t b0 = (int64_t)blockIdx.x * kScanBlock;
    const int64_t b1 = (b0 + kScanBlock < n) ? b0 + kScanBlock : n;
    int64_t carry = block_offsets[blockIdx.x];
    for (int64_t i0 = b0; i0 < b1; i0 += kT) {
        const int64_t i = i0 + threadIdx.x;
        const int c = (i < b1) ? counts[i] : 0;
        int inc = c;
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(inc, off, 64);
            if (lane >= off) inc += up;
        }
        if (lane == 63) wave_sum[wave] = inc;
        __syncthreads();
        int before = 0;
        for (int w = 0; w < wave; ++w) before += wave_sum[w];
        const int tile_total = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
        if (i < b1) row_ptr[i] = (int32_t)(carry + before + inc - c);
        carry += tile_total;
        __syncthreads();
    }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) row_ptr[n] = (int32_t)*total;
}

// CSR of A: one workgroup per (row, segment), columns compacted in ascending order from the
// segment's offset.  A thread owns sixteen consecutive columns (four 16-byte loads when kVec says that
// every row segment starts on a 16-byte boundary), counts its nonzeros, takes its place from a scan over the
// workgroup and writes them out in order: one pass and two barriers per segment.
static_assert(kSegment == 16 * kT, "a thread owns sixteen columns of a segment");
template <bool kVec>
__global__ __launch_bounds__(kT) void fill_segments_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                           int64_t lda, int64_t segments,
                                                           const int32_t *__restrict__ offsets,
                                                           int32_t *__restrict__ col_idx, float *__restrict__ vals) {
    __shared__ int wave_count[kT / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t unit = blockIdx.x; unit < rows * segments; unit += gridDim.x) {
        const int64_t r = unit / segments, s0 = (unit % segments) * kSegment;
        const int64_t s1 = (s0 + kSegment < cols) ? s0 + kSegment : cols;
        const float *row = A + r * lda;
        const int64_t mine = s0 + 16 * (int64_t)threadIdx.x;
        const int base = offsets[unit];
        float v[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int64_t j = mine + 4 * q;
            if (kVec && j + 4 <= s1) {
                const f32x4 x = *reinterpret_cast<const f32x4 *>(row + j);
                v[4 * q] = x.x; v[4 * q + 1] = x.y; v[4 * q + 2] = x.z; v[4 * q + 3] = x.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[4 * q + e] = (j + e < s1) ? row[j + e] : 0.0f;
            }
        }
        uint32_t keep = 0;
#pragma unroll
        for (int e = 0; e < 16; ++e) keep |= (v[e] != 0.0f) ? (1u << e) : 0u;
        const int count = __popc(keep);
        int inc = count;  // inclusive scan within the wavefront
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(inc, off, 64);
            if (lane >= off) inc += up;
        }
        if (lane == 63) wave_count[wave] = inc;
        __syncthreads();
        int at = base + inc - count;
        for (int w = 0; w < wave; ++w) at += wave_count[w];
#pragma unroll
        for (int e = 0; e < 16; ++e)
            if (keep & (1u << e)) {
                col_idx[at] = (int32_t)(mine + e);
                vals[at] = v[e];
                ++at;
            }
        __syncthreads();
    }
}

// CSR of A^T: one thread per column of A walks the rows in ascending order.
__global__ __launch_bounds__(kT) void fill_cols_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                       int64_t lda, const int32_t *__restrict__ row_ptr,
                                                       int32_t *__restrict__ col_idx, float *__restrict__ vals) {
    for (int64_t j = (int64_t)blockIdx.x * kT + threadIdx.x; j < cols; j += (int64_t)gridDim.x * kT) {
        int32_t at = row_ptr[j];
        for (int64_t r = 0; r < rows; ++r) {
            const float v = A[r * lda + j];
            if (v != 0.0f) { col_idx[at] = (int32_t)r; vals[at] = v; ++at; }
        }
    }
}

// ---- out = S B (gather) ---------------------------------------------------------------------------------
// A workgroup owns a block of 1024 columns (4 per lane) and walks a range of output rows.  The
// nonzeros of a row are taken eight at a time while eight are left: indices and values first, then the
// eight B rows, then the eight multiply-adds in order.
constexpr int kGather = 8;

template <bool kVector>
__global__ __launch_bounds__(kT) void csr_gemm_kernel(int64_t R, int64_t N, const int32_t *__restrict__ row_ptr,
                                                      const int32_t *__restrict__ col_idx,
                                                      const float *__restrict__ vals, const float *__restrict__ B,
                                                      int64_t ldb, float *__restrict__ out, int64_t ldo,
                                                      int64_t col_blocks, uint32_t *amax_out) {
    uint32_t amax = 0;  // bit patterns of |x| order like |x|
    const int64_t cb = blockIdx.x % col_blocks, rg = blockIdx.x / col_blocks, row_groups = gridDim.x / col_blocks;
    const int64_t n = cb * 1024 + 4 * (int64_t)threadIdx.x;
    for (int64_t r = rg; r < R; r += row_groups) {
        const int32_t j0 = row_ptr[r], j1 = row_ptr[r + 1];
        if (kVector) {
            if (n >= N) continue;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            int32_t j = j0;
            for (; j + kGather <= j1; j += kGather) {
                int32_t c[kGather];
                float v[kGather];
                f32x4 b[kGather];
#pragma unroll
                for (int u = 0; u < kGather; ++u) { c[u] = col_idx[j + u]; v[u] = vals[j + u]; }
#pragma unroll
                for (int u = 0; u < kGather; ++u) b[u] = *reinterpret_cast<const f32x4 *>(B + (int64_t)c[u] * ldb + n);
#pragma unroll
                for (int u = 0; u < kGather; ++u) acc = acc + v[u] * b[u];
            }
            for (; j < j1; ++j) {
                const float v = vals[j];
                const f32x4 b = *reinterpret_cast<const f32x4 *>(B + (int64_t)col_idx[j] * ldb + n);
                acc = acc + v * b;
            }
            if (out) __builtin_nontemporal_store(acc, reinterpret_cast<f32x4 *>(out + r * ldo + n));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t bits = __float_as_uint(acc[e]) & 0x7fffffffu;
                amax = bits > amax ? bits : amax;
            }
        } else {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int32_t j = j0; j < j1; ++j) {
                const float v = vals[j];
                const float *b = B + (int64_t)col_idx[j] * ldb + n;
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) acc[e] = acc[e] + v * b[e];
            }
            for (int e = 0; e < 4; ++e)
                if (n + e < N) {
                    if (out) out[r * ldo + n + e] = acc[e];
                    const uint32_t bits = __float_as_uint(acc[e]) & 0x7fffffffu;
                    amax = bits > amax ? bits : amax;
                }
        }
    }
    if (amax_out) {  // uniform over the launch; every lane of every wave arrives here
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)amax, off, 64);
            amax = o > amax ? o : amax;
        }
        if ((threadIdx.x & 63) == 0) atomicMax(amax_out, amax);
    }
}

// ---- rows with few nonzeros, software-pipelined ------------------------------------------------------
// The weight gradient X^T E has 100000 rows of two or three nonzeros each; one row is a chain of four
// dependent memory accesses (row pointers, nonzeros, rows of B, then the arithmetic), and a loop that walks
// it row by row is bound by that latency.  Here a wavefront owns 256 columns (four per lane) of a block
// of 16 consecutive rows and runs the block as straight-line code:
//   * the row pointers of the block and its first 64 nonzeros sit in vector registers, one entry per
//     lane, loaded a whole block ahead and handed to the scalar side with v_readlane;
//   * the B rows of row u + 1 (four loads; what a shorter row does not need reads one fixed cache line)
//     and the weights of row u + 8 are requested while row u is summed, encoded and written, into register
//     rings that the unrolled code indexes statically; the requests run on into the next block.
// Every load is issued unconditionally in a fixed number per row, so each wait counts exactly the loads
// issued after the one it needs.  Rows with more than four nonzeros, and rows of a block beyond its first
// 64 nonzeros, take what is missing from memory as the plain kernel does.  The sums run in the same order
// as there.
//   form 1: max |S B| only            2: codes of S B            3: codes and w += alpha * decode(codes)
//        4: codes and RMSprop with weight update on decode(codes)  (alpha = multiplier of the mean squares)
//        5, 6: what 3 and 4 do, with producing and streaming wavefronts (below)
constexpr int kRowThreads = 256;
// The codes-only form (2) needs no ring of weights and fits four wavefronts per SIMD: it runs 512 threads
// on one encoder table, two workgroups per compute unit (0.66 ms instead of 0.77 ms on the first-layer gradient).
// Forms 3 and 4, which stream the weights as well, gain nothing from that (1.73 ms against 1.69 ms) and keep 256.
template <int kForm> constexpr int row_threads() { return kForm >= 5 ? 1024 : kForm == 2 ? 512 : kRowThreads; }
// Forms 5 and 6 are forms 3 and 4 with the work split between the sixteen wavefronts of one workgroup per compute
// unit.  A wavefront that does everything waits for its B rows (from the L2, a row ahead) with the same in-order
// counter that its weight loads and its stores run on: each such wait also waits for every older weight load and
// store, so the weights are never more than two rows ahead in effect, whatever the ring holds.  (Measured on the
// first-layer gradient, 819.2 M elements: 1.71 ms; without the stores 1.08, without the weight loads 1.16, both
// gone 0.86; taking the encoder out changed nothing.)  Here twelve wavefronts produce codes exactly as form 2 does
// and leave each 16 x 256 patch of codes in LDS as well; four wavefronts take the patches of the round before
// (three each), read the weights sixteen rows ahead, add the decoded values and write; their waits see nothing but
// their own stream.  One barrier per round, the patches are double-buffered.  1.58 ms (RMSprop: 2.71 against
// 2.93).  The two halves do not overlap fully: the producers alone take 0.88 ms, the streaming wavefronts alone
// 1.10 (6.0 TB/s, what that mix of loads and stores reaches), and neither other splits (8 + 8, 10 + 5, 12 + 3,
// 12 + 2) nor B rows two ahead came closer; the producers' B rows come out of an L2 that the streams keep busy.
constexpr int kProducers = 12, kStreamers = 4, kPerStreamer = kProducers / kStreamers;
constexpr int kPatchWords = 16 * 64;  // a patch of codes: 16 rows, one word (four codes) per lane
static_assert(kProducers % kStreamers == 0 && (kProducers + kStreamers) * 64 == 1024, "sixteen wavefronts");
constexpr int kRowBlock = 16;  // rows per block
constexpr int kBAhead = 1;     // B values are requested this many rows ahead
constexpr int kBRing = 2 * kBAhead;
constexpr int kFixed = 4;      // B rows requested ahead per row

typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kRowAuxNt = 2;  // cache policy bit of the buffer instructions: nt
__device__ __forceinline__ rsrc_t row_rsrc(const void *base, uint32_t bytes) {
    // 0x00020000: 32-bit untyped data; accesses at or beyond `bytes` read zero and write nothing
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ f32x4 as_f32x4(u32x4 v) {
    return f32x4{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
}
__device__ __forceinline__ u32x4 as_u32x4(f32x4 v) {
    return u32x4{__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
}

// A 16-byte store whose row offset travels in a scalar register.  The compiler guards the two wait states between
// such a store and a vector instruction that overwrites its data registers only when the scalar offset is a
// constant; with a register there the next instruction may overwrite the data before the store has read it, and on
// this hardware the store then wrote the new contents now and then (seen as single wrong words, the first of a
// lane's four, under full memory load).  Here the data registers stay alive across two wait states.
__device__ __forceinline__ void store_row_b128(u32x4 data, rsrc_t r, uint32_t lane_offset, uint32_t row_offset) {
    __builtin_amdgcn_raw_buffer_store_b128(data, r, lane_offset, row_offset, kRowAuxNt);
    asm volatile("s_nop 1" ::"v"(data) : "memory");  // ordered behind the store, and the data registers are its operands
}

struct RowBlockMeta {
    int rp;    // lane l: row_ptr[first row + l], l <= 16
    int c;     // lane l: column index of the block's nonzero l
    float v;   // lane l: its value
};

template <int kForm>
__global__ __launch_bounds__(row_threads<kForm>(), kForm == 2 ? 4 : 1) void csr_rows_kernel(
    int64_t R, int64_t N, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
    const float *__restrict__ vals, const float *__restrict__ B, int64_t ldb, int64_t col_blocks, uint32_t *amax_out,
    const float *__restrict__ precision_ptr, uint8_t *__restrict__ codes, float *__restrict__ w, int64_t ldw, float alpha,
    float *__restrict__ rms, float rate, const XStep *__restrict__ steps, int step_count, const float *__restrict__ table,
    uint32_t b_bytes) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    EncodeShared &sh = *reinterpret_cast<EncodeShared *>(smem_raw);
    float *dlut = reinterpret_cast<float *>(smem_raw + sizeof(EncodeShared));  // decode table times alpha
    uint32_t *patches = reinterpret_cast<uint32_t *>(smem_raw + sizeof(EncodeShared) + 256 * sizeof(float));  // [2][kProducers][16][64]
    constexpr bool kPaired = kForm >= 5;
    constexpr int kMode = kPaired ? 2 : kForm;  // what this wavefront's rows do; the paired forms' producers are form 2
    constexpr int kWaves = kPaired ? kProducers : row_threads<kForm>() / 64;  // wavefronts that take units
    const int t = threadIdx.x;
    float precision = 0.0f;
    bool exact_only = false;
    const float rms_multiplier = alpha, one_minus = 1.0f - alpha;  // kMode 4 only
    if (kMode >= 2) {
        precision = *precision_ptr;
        exact_only = !build_table(sh, steps, step_count, precision, table);
        if (kForm == 4 || kForm == 6) alpha = 1.0f;  // RMSprop takes the decoded gradient itself; `alpha` then carries the multiplier
        if (t < 126) {
            const float v = table[t] * precision;
            dlut[t] = alpha * v;
            dlut[t + 128] = alpha * (-v);
        } else if (t == 126) {
            dlut[126] = alpha * precision;
            dlut[127] = alpha * precision;
            dlut[254] = alpha * precision;
            dlut[255] = alpha * (-precision);
        }
        __syncthreads();
    }
    const uint32_t first = xlut_first(precision);
    auto encode = [&](float v) -> uint32_t {
        if (exact_only) return encode_exact(v, precision, sh.slot);
        const uint32_t bits = __float_as_uint(v);
        return xlut_code(bits, sh.lut[xlut_index(bits & 0x7fffffffu, first)]);
    };

    const int lane = t & 63;
    // the wavefront's number as a scalar: what follows from it (the unit, its buffer descriptors) then lives in scalar
    // registers, and no buffer instruction has to be wrapped in a loop over the lanes' descriptors
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int32_t nnz = row_ptr[R];
    const int32_t last = nnz > 0 ? nnz - 1 : 0;
    const int64_t row_blocks = (R + kRowBlock - 1) / kRowBlock;
    const int64_t units = row_blocks * col_blocks;
    const int64_t unit_stride = (int64_t)gridDim.x * kWaves;
    uint32_t amax = 0;

    auto load_rp = [&](int64_t row0) -> int {
        int64_t k = row0 + lane;
        if (k > R) k = R;
        return row_ptr[k];
    };
    auto load_nz = [&](int rp, int &c, float &v) {
        int j = __builtin_amdgcn_readlane(rp, 0) + lane;
        if (j > last) j = last;
        c = nnz > 0 ? col_idx[j] : 0;
        v = nnz > 0 ? vals[j] : 0.0f;
    };

    const int64_t unit_first = (int64_t)blockIdx.x * kWaves + wave;
    const uint32_t b_row_bytes = (uint32_t)(ldb * (int64_t)sizeof(float));  // B spans less than 4 GiB on this path
    const char *Bbytes = reinterpret_cast<const char *>(B);
    // Everything a row touches is addressed through buffer descriptors: the part of an address that is the same for all
    // lanes (the row) travels in a scalar register, the lane's part is computed once per unit, and no row spends vector
    // instructions on 64-bit pointer arithmetic.
    const rsrc_t rb = row_rsrc(B, b_bytes);
    const uint32_t w_row_bytes = (uint32_t)(ldw * (int64_t)sizeof(float));
    // Where a unit lives: computed once per unit, the rows then only add multiples of the leading dimensions.
    struct UnitPos {
        int64_t row0;
        int rows;           // rows of the block inside the matrix (1 .. 16)
        bool live;          // the lane's four columns exist
        uint32_t lane_off;  // byte offset of the lane's columns inside a row of B (column 0 for idle lanes)
        rsrc_t rw, rr, rc;  // the unit's 16 x 256 patch of the weights, the running mean squares (RMSprop) and the codes
        uint32_t w_lane;    // byte offset of the lane's columns inside a row of those patches (column 0 for idle lanes)
    };
    auto locate = [&](int64_t unit) -> UnitPos {
        UnitPos p;
        const uint32_t rb = (uint32_t)unit / (uint32_t)col_blocks, cb = (uint32_t)unit - rb * (uint32_t)col_blocks;
        p.row0 = (int64_t)rb * kRowBlock;
        const int64_t left = R - p.row0;
        p.rows = left < kRowBlock ? (int)left : kRowBlock;
        const int64_t n = (int64_t)cb * 256 + 4 * (int64_t)lane;
        p.live = n < N;
        const int64_t nc = p.live ? n : 0;
        p.lane_off = (uint32_t)(nc * (int64_t)sizeof(float));
        const int64_t c0 = (int64_t)cb * 256, cols_here = N - c0 < 256 ? N - c0 : 256;
        p.w_lane = p.live ? (uint32_t)(4 * lane) : 0u;
        if (kForm >= 3) p.rw = row_rsrc(w + p.row0 * ldw + c0, (uint32_t)(((p.rows - 1) * ldw + cols_here) * (int64_t)sizeof(float)));
        if (kForm == 4 || kForm == 6) p.rr = row_rsrc(rms + p.row0 * ldw + c0, (uint32_t)(((p.rows - 1) * ldw + cols_here) * (int64_t)sizeof(float)));
        if (kMode >= 2) p.rc = row_rsrc(codes + p.row0 * N + c0, (uint32_t)((p.rows - 1) * N + cols_here));
        return p;
    };
    struct Ready {  // block metadata with what every request needs precomputed
        int rp, jb0;
        float v;
        uint32_t row_off;  // lane l: byte offset of the B row of the block's nonzero l
    };
    auto prepare = [&](const RowBlockMeta &m) -> Ready {
        Ready r;
        r.rp = m.rp;
        r.jb0 = __builtin_amdgcn_readlane(m.rp, 0);
        r.v = m.v;
        r.row_off = (uint32_t)m.c * b_row_bytes;
        return r;
    };
    // B rows of row u of a block: one v_readlane, one add and the load per request
    auto request_b = [&](const Ready &m, uint32_t lane_off, int u, f32x4 (&dst)[kFixed]) {
        const int q0 = __builtin_amdgcn_readlane(m.rp, u) - m.jb0, q1 = __builtin_amdgcn_readlane(m.rp, u + 1) - m.jb0;
        const int qend = q1 < 64 ? q1 : 64;
#pragma unroll
        for (int s2 = 0; s2 < kFixed; ++s2) {
            // a request beyond the row's nonzeros (or the cached 64) is still issued, so that the number of
            // loads per row is fixed, but all lanes then read the first 16 bytes of B: one cache line
            const bool real = q0 + s2 < qend;
            const uint32_t row = (uint32_t)__builtin_amdgcn_readlane((int)m.row_off, (q0 + s2) & 63);
            dst[s2] = as_f32x4(__builtin_amdgcn_raw_buffer_load_b128(rb, real ? lane_off : 0u, real ? row : 0u, 0));
        }
    };
    auto request_w = [&](const UnitPos &p, int u, f32x4 &dst, f32x4 &dst2) {
        const int uu = u < p.rows ? u : p.rows - 1;
        const uint32_t row = (uint32_t)uu * w_row_bytes;
        dst = as_f32x4(__builtin_amdgcn_raw_buffer_load_b128(p.rw, 4u * p.w_lane, row, kRowAuxNt));
        if (kMode == 4) dst2 = as_f32x4(__builtin_amdgcn_raw_buffer_load_b128(p.rr, 4u * p.w_lane, row, kRowAuxNt));
    };

    if constexpr (kPaired) {
        if (wave >= kProducers) {  // a streaming wavefront: the patches its three producers left a round ago
            constexpr bool kRms = kForm == 6;
            constexpr int kDepth = kRms ? 8 : 16;  // rows requested ahead (of the weights, and of the mean squares)
            const int s = wave - kProducers;
            const int64_t rounds = (units + unit_stride - 1) / unit_stride;
            const int64_t mine = (int64_t)blockIdx.x * kProducers + s * kPerStreamer;
            auto patch_at = [&](int64_t round, int j) -> UnitPos {
                const int64_t unit = round * unit_stride + mine + j;
                if (unit < units) return locate(unit);
                UnitPos p;  // beyond the last unit: loads give zero and stores go nowhere
                p.row0 = 0;
                p.rows = 0;
                p.live = false;
                p.lane_off = 0;
                p.w_lane = 0;
                p.rw = row_rsrc(w, 0);
                p.rr = row_rsrc(w, 0);
                p.rc = row_rsrc(codes, 0);
                return p;
            };
            auto request = [&](const UnitPos &p, int u, f32x4 &dw, f32x4 &dr) {
                int uu = u < p.rows ? u : p.rows - 1;
                uu = uu < 0 ? 0 : uu;
                const uint32_t row = (uint32_t)uu * w_row_bytes;
                dw = as_f32x4(__builtin_amdgcn_raw_buffer_load_b128(p.rw, 4u * p.w_lane, row, kRowAuxNt));
                if (kRms) dr = as_f32x4(__builtin_amdgcn_raw_buffer_load_b128(p.rr, 4u * p.w_lane, row, kRowAuxNt));
            };
            f32x4 sw[kDepth], sr[kRms ? kDepth : 1];
            UnitPos pos = patch_at(0, 0);
#pragma unroll
            for (int u = 0; u < kDepth; ++u) request(pos, u, sw[u], sr[kRms ? u : 0]);
            __syncthreads();  // round 0: the producers' first patches
            for (int64_t round = 1; round <= rounds; ++round) {
                const uint32_t *left = patches + (((round - 1) & 1) * kProducers + s * kPerStreamer) * kPatchWords + lane;
                for (int j = 0; j < kPerStreamer; ++j) {
                    const UnitPos nxt = j + 1 < kPerStreamer ? patch_at(round - 1, j + 1) : patch_at(round, 0);
                    // The loads and stores of a row are issued whatever the row is, so that every wait counts exactly
                    // what was issued behind the load it needs; a store that must not happen gets an offset beyond
                    // the patch and is dropped.
                    const uint32_t lane_bytes = pos.live ? 16u * (uint32_t)lane : 0xffffffffu;
#pragma unroll
                    for (int u = 0; u < kRowBlock; ++u) {
                        const uint32_t c = left[j * kPatchWords + u * 64];
                        const float g[4] = {dlut[c & 255u], dlut[(c >> 8) & 255u], dlut[(c >> 16) & 255u], dlut[c >> 24]};
                        f32x4 wv = sw[u % kDepth];
                        const uint32_t at = u < pos.rows ? lane_bytes : 0xffffffffu;
                        if (kRms) {  // kRMSprop_with_weight_update on the decoded gradient, operation by operation
                            f32x4 rv = sr[u % kDepth];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float r2 = (rms_multiplier * rv[e]) + ((g[e] * g[e]) * one_minus);
                                const float step = rate * (g[e] / (sqrtf(r2) + 1.0e-08f));
                                rv[e] = r2;
                                wv[e] = wv[e] - step;
                            }
                            store_row_b128(as_u32x4(rv), pos.rr, at, (uint32_t)u * w_row_bytes);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) wv[e] = wv[e] + g[e];
                        }
                        store_row_b128(as_u32x4(wv), pos.rw, at, (uint32_t)u * w_row_bytes);
                        if (u + kDepth < kRowBlock)
                            request(pos, u + kDepth, sw[u % kDepth], sr[kRms ? u % kDepth : 0]);
                        else
                            request(nxt, u + kDepth - kRowBlock, sw[u % kDepth], sr[kRms ? u % kDepth : 0]);
                    }
                    pos = nxt;
                }
                __syncthreads();  // the patches of this round are complete, those of the round before are free
            }
            return;
        }
    }
    int64_t round = 0;  // paired forms: rounds this wavefront has produced
    f32x4 b[kBRing][kFixed];
    constexpr int kWRing = kMode == 4 ? 4 : 8;  // weights (and mean squares) this many rows ahead
    f32x4 wr[kWRing], rr[kMode == 4 ? kWRing : 1];
    RowBlockMeta next;  // of the unit after the current one: loaded while the current one is worked on
    UnitPos pos_next = locate(unit_first < units ? unit_first : 0);
    next.rp = load_rp(pos_next.row0);
    load_nz(next.rp, next.c, next.v);
    if (unit_first < units) {  // the first unit's early requests; later units get theirs from the unit before
        if (kMode >= 3) {
#pragma unroll
            for (int u = 0; u < kWRing; ++u) request_w(pos_next, u, wr[u], rr[kMode == 4 ? u : 0]);
        }
        const Ready first_ready = prepare(next);
#pragma unroll
        for (int u = 0; u < kBAhead; ++u) request_b(first_ready, pos_next.lane_off, u, b[u]);
    }
    for (int64_t unit = unit_first; unit < units; unit += unit_stride) {
        const UnitPos pos = pos_next;
        const Ready m = prepare(next);
        pos_next = locate(unit + unit_stride < units ? unit + unit_stride : unit);
        next.rp = load_rp(pos_next.row0);
        Ready m_next = m;  // replaced once the next block's nonzeros are requested (row 8)
#pragma unroll
        for (int u = 0; u < kRowBlock; ++u) {
            if (u + kBAhead < kRowBlock)
                request_b(m, pos.lane_off, u + kBAhead, b[(u + kBAhead) % kBRing]);
            else
                request_b(m_next, pos_next.lane_off, u + kBAhead - kRowBlock, b[(u + kBAhead) % kBRing]);
            const int j0 = __builtin_amdgcn_readlane(m.rp, u), j1 = __builtin_amdgcn_readlane(m.rp, u + 1);
            const int count = j1 - j0, q0 = j0 - m.jb0;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            int32_t j = j0;
            if (q0 + (count < kFixed ? count : kFixed) <= 64) {  // the requested B values are the row's first ones
#pragma unroll
                for (int s2 = 0; s2 < kFixed; ++s2)
                    if (s2 < count) {
                        const float v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(m.v), q0 + s2));
                        acc = acc + v * b[u % kBRing][s2];
                    }
                j = j0 + (count < kFixed ? count : kFixed);
            }
            if (j < j1) {
                const float *Bl = reinterpret_cast<const float *>(Bbytes + pos.lane_off);
                for (; j + kGather <= j1; j += kGather) {
                    int32_t c[kGather];
                    float v[kGather];
                    f32x4 bb[kGather];
#pragma unroll
                    for (int k = 0; k < kGather; ++k) { c[k] = col_idx[j + k]; v[k] = vals[j + k]; }
#pragma unroll
                    for (int k = 0; k < kGather; ++k) bb[k] = *reinterpret_cast<const f32x4 *>(Bl + (int64_t)c[k] * ldb);
#pragma unroll
                    for (int k = 0; k < kGather; ++k) acc = acc + v[k] * bb[k];
                }
                for (; j < j1; ++j) {
                    const float v = vals[j];
                    const f32x4 bb = *reinterpret_cast<const f32x4 *>(Bl + (int64_t)col_idx[j] * ldb);
                    acc = acc + v * bb;
                }
            }
            if (u < pos.rows) {  // wave-uniform
                if (kMode == 1) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t bits = __float_as_uint(acc[e]) & 0x7fffffffu;
                        amax = bits > amax ? bits : amax;
                    }
                } else {
                    const uint32_t c0 = encode(acc.x), c1 = encode(acc.y), c2 = encode(acc.z), c3 = encode(acc.w);
                    const uint32_t four = c0 | (c1 << 8) | (c2 << 16) | (c3 << 24);
                    if (pos.live) __builtin_amdgcn_raw_buffer_store_b32(four, pos.rc, pos.w_lane, (uint32_t)u * (uint32_t)N, kRowAuxNt);
                    if (kPaired) patches[((round & 1) * kProducers + wave) * kPatchWords + u * 64 + lane] = four;
                    if (kMode == 4) {  // kRMSprop_with_weight_update on the decoded gradient, operation by operation
                        f32x4 wv = wr[u % kWRing], rv = rr[u % kWRing];
                        const float g[4] = {dlut[c0], dlut[c1], dlut[c2], dlut[c3]};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float r2 = (rms_multiplier * rv[e]) + ((g[e] * g[e]) * one_minus);
                            const float step = rate * (g[e] / (sqrtf(r2) + 1.0e-08f));
                            rv[e] = r2;
                            wv[e] = wv[e] - step;
                        }
                        if (pos.live) {
                            store_row_b128(as_u32x4(rv), pos.rr, 4u * pos.w_lane, (uint32_t)u * w_row_bytes);
                            store_row_b128(as_u32x4(wv), pos.rw, 4u * pos.w_lane, (uint32_t)u * w_row_bytes);
                        }
                    }
                    if (kMode == 3) {
                        f32x4 wv = wr[u % kWRing];
                        wv.x = wv.x + dlut[c0];
                        wv.y = wv.y + dlut[c1];
                        wv.z = wv.z + dlut[c2];
                        wv.w = wv.w + dlut[c3];
                        if (pos.live)
                            store_row_b128(as_u32x4(wv), pos.rw, 4u * pos.w_lane, (uint32_t)u * w_row_bytes);
                    }
                }
            }
            if (kMode >= 3) {
                if (u + kWRing < kRowBlock)
                    request_w(pos, u + kWRing, wr[u % kWRing], rr[kMode == 4 ? u % kWRing : 0]);
                else
                    request_w(pos_next, u + kWRing - kRowBlock, wr[u % kWRing], rr[kMode == 4 ? u % kWRing : 0]);
            }
            if (u == kRowBlock / 2) {  // the next block's row pointers were requested at the top
                load_nz(next.rp, next.c, next.v);
            }
            if (u == kRowBlock - kBAhead - 1) m_next = prepare(next);
        }
        if (kPaired) {
            __syncthreads();  // this round's patches are complete
            ++round;
        }
    }
    if (kPaired) {  // a wavefront with a unit less than the others, and the round in which only the streamers work
        const int64_t rounds = (units + unit_stride - 1) / unit_stride;
        for (; round <= rounds; ++round) __syncthreads();
    }
    if (kMode == 1) {  // every lane of every wave arrives here
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)amax, off, 64);
            amax = o > amax ? o : amax;
        }
        if (lane == 0) atomicMax(amax_out, amax);
    }
}

// ---- max |S B| with B in LDS ------------------------------------------------------------------------------
// csr_rows_kernel reads every B row it needs from the L2: 8.4 GB for the first-layer gradient, which is
// what bounds its max-only pass (20 TB/s out of the L2).  When B has at most 128 rows (the batch), a strip of
// 256 columns of it is 128 KB: a workgroup of sixteen wavefronts loads one strip into LDS and every wavefront
// runs blocks of 16 rows against it.  The B values then cost an LDS read per wavefront and nonzero, nothing
// has to be requested ahead, and the nonzeros of a row are simply looped over: 0.30 ms instead of 0.42 ms.
// (Reading a fixed four values per row from LDS a row ahead, as csr_rows_kernel does from memory, is slower,
// 0.375 ms: the LDS reads are what the kernel is made of, and a row has 2.6 nonzeros on average.)
// The fused passes do not take this route: with the encoder table in LDS as well only 128-column strips fit,
// two columns per lane, the per-row work per element doubles, and they measured 1.83 ms against 1.66 ms.
constexpr int kLdsThreads = 1024;
constexpr int kLdsStrip = 256;    // columns per workgroup, four per lane
constexpr int kLdsMaxRows = 128;  // rows of B that fit

__global__ __launch_bounds__(kLdsThreads) void csr_rows_max_lds_kernel(
    int64_t R, int Cc, int64_t N, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
    const float *__restrict__ vals, const float *__restrict__ B, int64_t ldb, int strips, int parts, uint32_t *amax_out) {
    extern __shared__ __attribute__((aligned(16))) float estrip[];  // [Cc][256]
    const int t = threadIdx.x;
    const int strip = blockIdx.x % strips, part = blockIdx.x / strips;
    for (int idx = t; idx < Cc * kLdsStrip; idx += kLdsThreads) {
        const int i = idx / kLdsStrip, c = idx % kLdsStrip;
        const int64_t col = (int64_t)strip * kLdsStrip + c;
        estrip[idx] = col < N ? B[(int64_t)i * ldb + col] : 0.0f;  // columns beyond N give zeros, which cannot win
    }
    __syncthreads();

    const int lane = t & 63, wave = t >> 6;
    const float *elane = estrip + 4 * lane;
    const int32_t nnz = row_ptr[R];
    const int32_t last = nnz > 0 ? nnz - 1 : 0;
    const int64_t row_blocks = (R + kRowBlock - 1) / kRowBlock;
    const int64_t rb_stride = (int64_t)parts * (kLdsThreads / 64);
    uint32_t amax = 0;

    auto load_rp = [&](int64_t rb) -> int {
        int64_t k = rb * kRowBlock + lane;
        if (k > R) k = R;
        return row_ptr[k];
    };
    auto load_nz_at = [&](int j0, int &c, float &v) {  // nonzeros j0 .. j0 + 63, one per lane
        int j = j0 + lane;
        if (j > last) j = last;
        c = nnz > 0 ? col_idx[j] : 0;
        v = nnz > 0 ? vals[j] : 0.0f;
    };

    const int64_t rb_first = (int64_t)part * (kLdsThreads / 64) + wave;
    RowBlockMeta next;  // of the block after the current one: loaded while the current one is worked on
    next.rp = load_rp(rb_first < row_blocks ? rb_first : 0);
    load_nz_at(__builtin_amdgcn_readlane(next.rp, 0), next.c, next.v);
    for (int64_t rb = rb_first; rb < row_blocks; rb += rb_stride) {
        const RowBlockMeta m = next;
        next.rp = load_rp(rb + rb_stride < row_blocks ? rb + rb_stride : rb);
        // the nonzeros at hand: 64 of them starting at chunk_base, one per lane
        int chunk_base = __builtin_amdgcn_readlane(m.rp, 0);
        int cur_c = m.c;
        float cur_v = m.v;
#pragma unroll
        for (int u = 0; u < kRowBlock; ++u) {  // rows beyond R have no nonzeros and contribute |0|
            const int j0 = __builtin_amdgcn_readlane(m.rp, u), j1 = __builtin_amdgcn_readlane(m.rp, u + 1);
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            for (int j = j0; j < j1; ++j) {
                if (j - chunk_base >= 64) {  // wave-uniform and rare: fetch the next 64 nonzeros now
                    chunk_base = j;
                    load_nz_at(j, cur_c, cur_v);
                }
                const int i = __builtin_amdgcn_readlane(cur_c, j - chunk_base);
                const float x = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cur_v), j - chunk_base));
                const f32x4 b = *reinterpret_cast<const f32x4 *>(elane + i * kLdsStrip);
                acc = acc + x * b;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t bits = __float_as_uint(acc[e]) & 0x7fffffffu;
                amax = bits > amax ? bits : amax;
            }
            if (u == kRowBlock / 2) load_nz_at(__builtin_amdgcn_readlane(next.rp, 0), next.c, next.v);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {  // every lane of every wave arrives here
        const uint32_t o = (uint32_t)__shfl_xor((int)amax, off, 64);
        amax = o > amax ? o : amax;
    }
    if (lane == 0) atomicMax(amax_out, amax);
}

__global__ void preset_word_kernel(uint32_t *p, uint32_t value) {
    if (threadIdx.x == 0) *p = value;
}

// ---- few long rows: narrow column strips, one XCD per strip ---------------------------------------------
// A batch of 128 rows with 2000 nonzeros each touches 92 % of the rows of B, every one of them two or three
// times.  Whether the second use finds the data in the L2 depends on how much is fetched in between:
// the rows walk their nonzeros at about the same pace, some 2000 rows of B apart, so a B row comes back
// after about 2000 other rows have been read.  With 1024 columns per workgroup that is 8 MB, twice an XCD's
// L2.  Here a wavefront takes one row and a strip of 256 columns (1 KB of a B row) with forty B rows in
// flight, and all rows of a strip run on one XCD (workgroup index mod 8).  Measured on the 128 x 100000
// batch against 100000 x 8192 weights: 0.86 ms instead of 1.06 ms (0.90 ms with sixteen in flight, when
// 6.7 GB were fetched instead of 7.55 GB; holding an XCD to one strip at a time brought that to 5.1 GB but
// left too few loads in flight to gain).
// Sums and results as in csr_gemm_kernel.
constexpr int kStripColumns = 256;
// Forty B rows in flight per wavefront.  That takes 215 registers, so a SIMD holds two wavefronts and an XCD
// works on two strips at a time instead of four: deeper queues and a smaller working set in its L2 (0.86 ms
// against 0.90 ms with sixteen in flight and every workgroup resident; 32 at the same occupancy is slower
// than either, 56 and more spill).  What a multiple of forty leaves over goes eight at a time.
constexpr int kStripGather = 40;
constexpr int kStripGatherTail = 8;

// kPool 0: out = S B (and optionally max |out|).  kPool 2 or 4: out = maxout(S B + bias) over kPool
// consecutive columns, argmax = the winner's column as a float (first maximum wins): what add_row_vector
// and maxout give, formed on the lane's four columns before anything is written.
template <int kPool>
__global__ __launch_bounds__(kT) void csr_gemm_strip_kernel(int64_t R, int64_t N, const int32_t *__restrict__ row_ptr,
                                                            const int32_t *__restrict__ col_idx,
                                                            const float *__restrict__ vals, const float *__restrict__ B,
                                                            int64_t ldb, float *__restrict__ out, int64_t ldo,
                                                            int64_t strips, int64_t row_quads, uint32_t *amax_out,
                                                            const float *__restrict__ bias, float *__restrict__ argmax,
                                                            int64_t lda) {
    uint32_t amax = 0;
    const int64_t xcd = blockIdx.x % 8, local = blockIdx.x / 8;
    // an XCD takes neighbouring strips, so that the two it has in flight read neighbouring kilobytes of the same
    // B rows (0.82 ms instead of 0.845 ms with its strips eight apart)
    const int64_t strip = xcd * ((strips + 7) / 8) + (local / row_quads);
    const int64_t r = (local % row_quads) * 4 + (threadIdx.x >> 6);
    const int64_t n = strip * kStripColumns + 4 * (int64_t)(threadIdx.x & 63);
    if (strip < strips && r < R && n < N) {
        const int32_t j0 = row_ptr[r], j1 = row_ptr[r + 1];
        const float *Bn = B + n;
        f32x4 acc = 0.0f;
        int32_t j = j0;
        for (; j + kStripGather <= j1; j += kStripGather) {
            int32_t c[kStripGather];
            float v[kStripGather];
            f32x4 b[kStripGather];
#pragma unroll
            for (int u = 0; u < kStripGather; ++u) { c[u] = col_idx[j + u]; v[u] = vals[j + u]; }
#pragma unroll
            for (int u = 0; u < kStripGather; ++u) b[u] = *reinterpret_cast<const f32x4 *>(Bn + (int64_t)c[u] * ldb);
#pragma unroll
            for (int u = 0; u < kStripGather; ++u) acc = acc + v[u] * b[u];
        }
        for (; j + kStripGatherTail <= j1; j += kStripGatherTail) {
            int32_t c[kStripGatherTail];
            float v[kStripGatherTail];
            f32x4 b[kStripGatherTail];
#pragma unroll
            for (int u = 0; u < kStripGatherTail; ++u) { c[u] = col_idx[j + u]; v[u] = vals[j + u]; }
#pragma unroll
            for (int u = 0; u < kStripGatherTail; ++u) b[u] = *reinterpret_cast<const f32x4 *>(Bn + (int64_t)c[u] * ldb);
#pragma unroll
            for (int u = 0; u < kStripGatherTail; ++u) acc = acc + v[u] * b[u];
        }
        for (; j < j1; ++j) {
            const float v = vals[j];
            const f32x4 b = *reinterpret_cast<const f32x4 *>(Bn + (int64_t)col_idx[j] * ldb);
            acc = acc + v * b;
        }
        if constexpr (kPool == 0) {
            if (out) __builtin_nontemporal_store(acc, reinterpret_cast<f32x4 *>(out + r * ldo + n));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t bits = __float_as_uint(acc[e]) & 0x7fffffffu;
                amax = bits > amax ? bits : amax;
            }
        } else {
            const f32x4 bv = *reinterpret_cast<const f32x4 *>(bias + n);
            const float z[4] = {acc[0] + bv[0], acc[1] + bv[1], acc[2] + bv[2], acc[3] + bv[3]};
            constexpr int kOut = 4 / kPool;
            float best[kOut], arg[kOut];
#pragma unroll
            for (int o = 0; o < kOut; ++o) {
                best[o] = z[o * kPool];
                int a = 0;
#pragma unroll
                for (int p = 1; p < kPool; ++p)
                    if (best[o] < z[o * kPool + p]) { best[o] = z[o * kPool + p]; a = p; }
                arg[o] = (float)(n + o * kPool + a);
            }
#pragma unroll
            for (int o = 0; o < kOut; ++o) {
                out[r * ldo + n / kPool + o] = best[o];
                argmax[r * lda + n / kPool + o] = arg[o];
            }
        }
    }
    if (kPool == 0 && amax_out) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)amax, off, 64);
            amax = o > amax ? o : amax;
        }
        if ((threadIdx.x & 63) == 0) atomicMax(amax_out, amax);
    }
}

// ---- product -> codes -> update, without the product ever reaching memory -------------------------------
// codes = compression_8bit(S B, *precision) and, if w is given, w += alpha * decompression_8bit(codes) (or
// RMSprop with weight update on the decoded values): the weight gradient of the first layer, its 8-bit
// codes for the exchange and the update of the weights in one pass that writes one byte per element and
// reads and writes the weights once.  Recomputing a row of S B costs its few nonzeros; the precision
// (max |S B|) comes from a first pass that stores nothing.  Every value is computed, encoded and decoded
// exactly as by csr_gemm, compress and decompress_axpy.
// This kernel is the plain form for operands that do not allow 16-byte accesses: one element at a time, row
// after row; csr_rows_kernel below is the one that is tuned.
constexpr int kCodedThreads = 512;

__global__ __launch_bounds__(kCodedThreads) void csr_gemm_coded_kernel(
    int64_t R, int64_t N, const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col_idx,
    const float *__restrict__ vals, const float *__restrict__ B, int64_t ldb, int64_t col_blocks,
    const float *__restrict__ precision_ptr, uint8_t *__restrict__ codes, float *__restrict__ w, int64_t ldw, float alpha,
    float *__restrict__ rms, float rate, const XStep *__restrict__ steps, int step_count, const float *__restrict__ table) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    EncodeShared &sh = *reinterpret_cast<EncodeShared *>(smem_raw);
    float *dlut = reinterpret_cast<float *>(smem_raw + sizeof(EncodeShared));  // decode table times alpha
    const float rms_multiplier = alpha, one_minus = 1.0f - alpha;  // with rms: RMSprop on the decoded gradient
    if (rms) alpha = 1.0f;
    const float precision = *precision_ptr;
    const bool exact_only = !build_table(sh, steps, step_count, precision, table);
    const int t = threadIdx.x;
    if (t < 126) {
        const float v = table[t] * precision;
        dlut[t] = alpha * v;
        dlut[t + 128] = alpha * (-v);
    } else if (t == 126) {
        dlut[126] = alpha * precision;
        dlut[127] = alpha * precision;
        dlut[254] = alpha * precision;
        dlut[255] = alpha * (-precision);
    }
    __syncthreads();
    const uint32_t first = xlut_first(precision);
    auto encode = [&](float v) -> uint32_t {
        if (exact_only) return encode_exact(v, precision, sh.slot);
        const uint32_t bits = __float_as_uint(v);
        return xlut_code(bits, sh.lut[xlut_index(bits & 0x7fffffffu, first)]);
    };

    const int64_t cb = blockIdx.x % col_blocks, rg = blockIdx.x / col_blocks, row_groups = gridDim.x / col_blocks;
    const int slot = t >> 8;
    const int64_t n = cb * 1024 + 4 * (int64_t)(t & 255);
    for (int64_t r = rg * 2 + slot; r < R; r += row_groups * 2) {
        const int32_t j0 = row_ptr[r], j1 = row_ptr[r + 1];
        {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int32_t j = j0; j < j1; ++j) {
                const float v = vals[j];
                const float *b = B + (int64_t)col_idx[j] * ldb + n;
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) acc[e] = acc[e] + v * b[e];
            }
            for (int e = 0; e < 4; ++e)
                if (n + e < N) {
                    const uint32_t c = encode(acc[e]);
                    codes[r * N + n + e] = (uint8_t)c;
                    if (rms) {
                        const float g = dlut[c];
                        const float r2 = (rms_multiplier * rms[r * ldw + n + e]) + ((g * g) * one_minus);
                        const float step = rate * (g / (sqrtf(r2) + 1.0e-08f));
                        rms[r * ldw + n + e] = r2;
                        w[r * ldw + n + e] = w[r * ldw + n + e] - step;
                    } else if (w) {
                        w[r * ldw + n + e] = w[r * ldw + n + e] + dlut[c];
                    }
                }
        }
    }
}

// ---- CSR(S) -> CSR(S^T) ------------------------------------------------------------------------------------
// Transposition as a counting sort whose result does not depend on scheduling and needs no sorting afterwards.
// The rows of S are cut into `blocks` blocks of `rows_per_block` consecutive rows; cursor[c * blocks + b] counts the
// nonzeros of column c inside block b, and after a prefix sum over that array (column-major: all blocks of column 0,
// then of column 1, ...) holds where block b's part of result row c starts.  One workgroup per block then walks its
// rows in ascending order, a barrier between rows, so that every result row comes out in ascending column (= source
// row) order whatever the lengths of its parts; within one source row the columns are distinct, so its nonzeros
// take their places without atomics.  A result row of any length costs what its nonzeros cost.
__global__ __launch_bounds__(kT) void transpose_count_kernel(int64_t R, const int32_t *__restrict__ row_ptr,
                                                             const int32_t *__restrict__ col_idx, int64_t blocks,
                                                             int64_t rows_per_block, int32_t *__restrict__ cursor) {
    for (int64_t r = blockIdx.x; r < R; r += gridDim.x) {
        const int64_t b = r / rows_per_block;
        for (int32_t j = row_ptr[r] + threadIdx.x; j < row_ptr[r + 1]; j += kT) atomicAdd(&cursor[(int64_t)col_idx[j] * blocks + b], 1);
    }
}

__global__ __launch_bounds__(kT) void transpose_row_ptr_kernel(const int32_t *__restrict__ cursor, int64_t Cc, int64_t blocks,
                                                               int32_t *__restrict__ t_row_ptr) {
    for (int64_t c = (int64_t)blockIdx.x * kT + threadIdx.x; c <= Cc; c += (int64_t)gridDim.x * kT) t_row_ptr[c] = cursor[c * blocks];
}

__global__ __launch_bounds__(kT) void transpose_fill_kernel(int64_t R, const int32_t *__restrict__ row_ptr,
                                                            const int32_t *__restrict__ col_idx,
                                                            const float *__restrict__ vals, int64_t blocks,
                                                            int64_t rows_per_block, int32_t *cursor,
                                                            int32_t *__restrict__ out_col, float *__restrict__ out_val) {
    for (int64_t b = blockIdx.x; b < blocks; b += gridDim.x) {
        const int64_t r_end = (b + 1) * rows_per_block < R ? (b + 1) * rows_per_block : R;
        for (int64_t r = b * rows_per_block; r < r_end; ++r) {
            for (int32_t j = row_ptr[r] + threadIdx.x; j < row_ptr[r + 1]; j += kT) {
                // an atomic, so that a row that names a column twice (the layout does not forbid it) still gives both
                // entries a place of their own; entries of different columns never meet on a slot
                const int32_t at = atomicAdd(&cursor[(int64_t)col_idx[j] * blocks + b], 1);
                out_col[at] = (int32_t)r;
                out_val[at] = vals[j];
            }
            __syncthreads();  // the next row of the block sees the places this one took
        }
    }
}

// out = dense form of S: zero fill, then one workgroup per row writes its nonzeros.
__global__ __launch_bounds__(kT) void csr_to_dense_kernel(int64_t R, int64_t Cc, const int32_t *__restrict__ row_ptr,
                                                          const int32_t *__restrict__ col_idx,
                                                          const float *__restrict__ vals, float *__restrict__ out,
                                                          int64_t ldo) {
    for (int64_t r = blockIdx.x; r < R; r += gridDim.x) {
        for (int64_t j = threadIdx.x; j < Cc; j += kT) out[r * ldo + j] = 0.0f;
        __syncthreads();
        for (int32_t j = row_ptr[r] + threadIdx.x; j < row_ptr[r + 1]; j += kT) out[r * ldo + col_idx[j]] = vals[j];
        __syncthreads();
    }
}

// row_ptr[0 .. n] = exclusive prefix sums of counts[0 .. n - 1] (in place allowed), *total_dev = their sum.
cn_status exclusive_scan(Context *ctx, const int32_t *counts, int64_t n, int32_t *row_ptr, int64_t *total_dev,
                         hipStream_t st) {
    const int64_t blocks = (n + kScanBlock - 1) / kScanBlock;
    if (blocks <= 2 || blocks + 1 > kReduceSlots) {  // the scratch holds kReduceSlots words before its counter
        hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kT), 0, st, counts, n, row_ptr, total_dev);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    int32_t *sums = reinterpret_cast<int32_t *>(ctx->reduce_scratch);
    hipLaunchKernelGGL(block_sums_kernel, dim3((unsigned)blocks), dim3(kT), 0, st, counts, n, sums);
    CN_HIP(hipGetLastError());
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kT), 0, st, sums, blocks, sums, total_dev);
    CN_HIP(hipGetLastError());
    hipLaunchKernelGGL(block_scan_kernel, dim3((unsigned)blocks), dim3(kT), 0, st, counts, n, sums, row_ptr, total_dev);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status check_csr_args(const char *who, int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr,
                         const int32_t *col_idx, const float *vals, const float *B, int64_t ldb, const float *out,
                         int64_t ldo) {
    if (R < 0 || Cc < 0 || N < 0) { set_error("%s: negative dimension", who); return CN_ERR_SHAPE; }
    if (ldb < N || (out && ldo < N)) { set_error("%s: leading dimension too small", who); return CN_ERR_SHAPE; }
    if (R > 0x7fffffffLL || Cc > 0x7fffffffLL) { set_error("%s: more than 2^31 rows or columns", who); return CN_ERR_SHAPE; }
    if (!row_ptr) { set_error("%s: NULL row pointers", who); return CN_ERR_NULL; }
    (void)col_idx; (void)vals; (void)B; (void)out;
    return CN_OK;
}

}  // namespace

}  // namespace cn

using namespace cn;

extern "C" {

cn_status cn_csr_from_dense_f32(const float *A, int64_t rows, int64_t cols, int64_t lda, int transpose,
                                int32_t *row_ptr, int32_t *col_idx, float *vals, int64_t capacity,
                                int64_t *nnz_host, void *stream) {
    if (rows < 0 || cols < 0 || lda < cols) { set_error("csr_from_dense_f32: bad dimensions"); return CN_ERR_SHAPE; }
    if (!row_ptr || !nnz_host || (rows > 0 && cols > 0 && !A)) { set_error("csr_from_dense_f32: NULL pointer"); return CN_ERR_NULL; }
    if (rows > 0x7fffffffLL || cols > 0x7fffffffLL) { set_error("csr_from_dense_f32: dimension above 2^31"); return CN_ERR_SHAPE; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int64_t out_rows = transpose ? cols : rows;
    int64_t *total_dev = reinterpret_cast<int64_t *>(ctx->sum_scratch);  // 8 bytes of the reduction scratch
    const int wide = ctx->num_cu * 8;
    const int64_t segments = (cols + kSegment - 1) / kSegment;
    const int64_t units = rows * segments;
    const bool vec_rows = aligned(A, 16) && lda % 4 == 0;  // segments start at multiples of 4096 columns
    int32_t *offsets = reinterpret_cast<int32_t *>(ctx->workspace);  // per (row, segment), transpose == 0 only
    if (!transpose && (size_t)(units + 1) * sizeof(int32_t) > ctx->workspace_bytes) {
        set_error("csr_from_dense_f32: matrix too large for the workspace");
        return CN_ERR_WORKSPACE;
    }
    if (rows > 0 && cols > 0 && transpose) {
        const int64_t blocks = (cols + kT - 1) / kT;
        hipLaunchKernelGGL(count_cols_kernel, dim3((unsigned)(blocks < wide ? blocks : wide)), dim3(kT), 0, st, A, rows, cols,
                           lda, row_ptr);
        CN_HIP(hipGetLastError());
        { cn_status sc = exclusive_scan(ctx, row_ptr, out_rows, row_ptr, total_dev, st); if (sc != CN_OK) return sc; }
    } else if (rows > 0 && cols > 0) {
        hipLaunchKernelGGL(vec_rows ? count_segments_kernel<true> : count_segments_kernel<false>,
                           dim3((unsigned)(units < wide ? units : wide)), dim3(kT), 0, st, A, rows, cols, lda, segments, offsets);
        CN_HIP(hipGetLastError());
        { cn_status sc = exclusive_scan(ctx, offsets, units, offsets, total_dev, st); if (sc != CN_OK) return sc; }
        const int64_t blocks = (rows + kT) / kT;
        hipLaunchKernelGGL(row_ptr_from_segments_kernel, dim3((unsigned)(blocks < wide ? blocks : wide)), dim3(kT), 0, st, offsets,
                           rows, segments, row_ptr);
        CN_HIP(hipGetLastError());
    } else {
        hipLaunchKernelGGL(zero_counts_kernel, dim3(wide), dim3(kT), 0, st, row_ptr, out_rows + 1);
        CN_HIP(hipGetLastError());
        hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kT), 0, st, row_ptr, (int64_t)0, row_ptr, total_dev);
        CN_HIP(hipGetLastError());
    }
    CN_HIP(hipMemcpyAsync(nnz_host, total_dev, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    CN_HIP(hipStreamSynchronize(st));
    if (*nnz_host >= 0x7fffffffLL) { set_error("csr_from_dense_f32: 2^31 - 1 nonzeros or more"); return CN_ERR_SHAPE; }
    if (*nnz_host > capacity) {
        set_error("csr_from_dense_f32: %lld nonzeros do not fit the capacity of %lld", (long long)*nnz_host, (long long)capacity);
        return CN_ERR_WORKSPACE;
    }
    if (*nnz_host == 0) return CN_OK;
    if (!col_idx || !vals) { set_error("csr_from_dense_f32: NULL output arrays"); return CN_ERR_NULL; }
    if (transpose) {
        const int64_t blocks = (cols + kT - 1) / kT;
        hipLaunchKernelGGL(fill_cols_kernel, dim3((unsigned)(blocks < wide ? blocks : wide)), dim3(kT), 0, st, A, rows, cols,
                           lda, row_ptr, col_idx, vals);
    } else {
        hipLaunchKernelGGL(vec_rows ? fill_segments_kernel<true> : fill_segments_kernel<false>,
                           dim3((unsigned)(units < wide ? units : wide)), dim3(kT), 0, st, A, rows, cols, lda, segments, offsets,
                           col_idx, vals);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

static bool g_strip_kernel = true;  // the test hooks below switch these kernels off to compare
static int g_rows_per_cu = 0;  // tuning hook: workgroups per compute unit of the fused row passes, 0 = their own figure
static bool g_lds_rows = true;
static bool g_paired_rows = true;  // fused update passes: producing and streaming wavefronts (forms 5, 6) instead of forms 3, 4

static cn_status csr_gemm(const char *who, int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                          const float *vals, const float *B, int64_t ldb, float *out, int64_t ldo, float *absmax_out,
                          void *stream) {
    cn_status s = check_csr_args(who, R, Cc, N, row_ptr, col_idx, vals, B, ldb, out, ldo);
    if (s != CN_OK) return s;
    Context *ctx;
    s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    uint32_t *amax = reinterpret_cast<uint32_t *>(absmax_out);
    if (amax) {  // 0, or -1.0f for an empty result as the abs-max pass reports it
        hipLaunchKernelGGL(preset_word_kernel, dim3(1), dim3(64), 0, st, amax, (R == 0 || N == 0) ? 0xbf800000u : 0u);
        CN_HIP(hipGetLastError());
    }
    if (R == 0 || N == 0) return CN_OK;
    if (!out && !amax) { set_error("%s: NULL output", who); return CN_ERR_NULL; }
    if (!out && g_lds_rows && Cc > 0 && Cc <= kLdsMaxRows) {  // maximum only, B strip in LDS
        const int lds_rows = (int)(Cc * kLdsStrip * sizeof(float));
        static OncePerDevice lds_configured;
        if (lds_configured.first(ctx->device)) {
            CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_max_lds_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMaxRows * kLdsStrip * (int)sizeof(float)));
        }
        const int64_t strips = (N + kLdsStrip - 1) / kLdsStrip;
        if (strips > 0x7fffffLL) { set_error("%s: too many columns", who); return CN_ERR_SHAPE; }
        int64_t parts = (int64_t)ctx->num_cu / strips;  // one workgroup per compute unit
        if (parts < 1) parts = 1;
        const int64_t row_blocks = (R + kRowBlock - 1) / kRowBlock;
        const int64_t most_parts = (row_blocks + kLdsThreads / 64 - 1) / (kLdsThreads / 64);
        if (parts > most_parts) parts = most_parts;
        hipLaunchKernelGGL(csr_rows_max_lds_kernel, dim3((unsigned)(strips * parts)), dim3(kLdsThreads), lds_rows, st, R, (int)Cc, N,
                           row_ptr, col_idx, vals, B, ldb, (int)strips, (int)parts, amax);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (!out && Cc > 0 && Cc * ldb < (1LL << 30) && aligned(B, 16) && ldb % 4 == 0 && N % 4 == 0) {  // maximum only: the pipelined row kernel
        const int64_t cblocks = (N + 255) / 256;
        const int64_t units = ((R + kRowBlock - 1) / kRowBlock) * cblocks;
        const int64_t per_wg = kRowThreads / 64;
        int64_t grid = (int64_t)ctx->num_cu * 5;
        if (grid > (units + per_wg - 1) / per_wg) grid = (units + per_wg - 1) / per_wg;
        hipLaunchKernelGGL(csr_rows_kernel<1>, dim3((unsigned)grid), dim3(kRowThreads), 0, st, R, N, row_ptr, col_idx, vals, B, ldb,
                           cblocks, amax, (const float *)nullptr, (uint8_t *)nullptr, (float *)nullptr, (int64_t)0, 0.0f,
                           (float *)nullptr, 0.0f, (const XStep *)nullptr, 0, (const float *)nullptr,
                           (uint32_t)(((Cc - 1) * ldb + N) * (int64_t)sizeof(float)));
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    const int64_t col_blocks = (N + 1023) / 1024;
    int64_t row_groups = ((int64_t)ctx->num_cu * 8 + col_blocks - 1) / col_blocks;
    if (row_groups > R) row_groups = R;
    const bool vec = aligned(B, 16) && ldb % 4 == 0 && N % 4 == 0 && (!out || (aligned(out, 16) && ldo % 4 == 0));
    // few rows, so that all rows of a strip run side by side on one XCD (four per compute unit, num_cu / 8
    // units), and enough columns to give every XCD a strip
    const int64_t row_quads = (R + 3) / 4;
    if (vec && g_strip_kernel && row_quads <= ctx->num_cu / 8 && N >= 8 * kStripColumns) {
        const int64_t strips = (N + kStripColumns - 1) / kStripColumns;
        const int64_t grid = ((strips + 7) / 8) * row_quads * 8;
        hipLaunchKernelGGL(csr_gemm_strip_kernel<0>, dim3((unsigned)grid), dim3(kT), 0, st, R, N, row_ptr, col_idx, vals, B, ldb, out,
                           ldo, strips, row_quads, amax, (const float *)nullptr, (float *)nullptr, (int64_t)0);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    if (vec)
        hipLaunchKernelGGL(csr_gemm_kernel<true>, dim3((unsigned)(col_blocks * row_groups)), dim3(kT), 0, st, R, N, row_ptr,
                           col_idx, vals, B, ldb, out, ldo, col_blocks, amax);
    else
        hipLaunchKernelGGL(csr_gemm_kernel<false>, dim3((unsigned)(col_blocks * row_groups)), dim3(kT), 0, st, R, N, row_ptr,
                           col_idx, vals, B, ldb, out, ldo, col_blocks, amax);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

void cn_host_csr_strip_kernel(int enabled) { g_strip_kernel = enabled != 0; }

// Test hook: the exclusive prefix sums the CSR builders use, on a caller's counts.
cn_status cn_host_exclusive_scan(const int32_t *counts_device, int64_t n, int32_t *sums_device, int64_t *total_host) {
    if (n < 0 || !total_host || (n > 0 && !counts_device) || !sums_device) { set_error("host_exclusive_scan: bad argument"); return CN_ERR_ARG; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    int64_t *total_dev = reinterpret_cast<int64_t *>(ctx->sum_scratch);
    s = exclusive_scan(ctx, counts_device, n, sums_device, total_dev, (hipStream_t)0);
    if (s != CN_OK) return s;
    CN_HIP(hipMemcpy(total_host, total_dev, sizeof(int64_t), hipMemcpyDeviceToHost));
    return CN_OK;
}
void cn_host_csr_rows_workgroups_per_cu(int per_cu) { g_rows_per_cu = per_cu > 0 ? per_cu : 0; }
void cn_host_csr_lds_rows(int enabled) { g_lds_rows = enabled != 0; }
void cn_host_csr_paired_rows(int enabled) { g_paired_rows = enabled != 0; }

cn_status cn_csr_gemm_f32(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                          const float *vals, const float *B, int64_t ldb, float *out, int64_t ldo, void *stream) {
    return csr_gemm("csr_gemm_f32", R, Cc, N, row_ptr, col_idx, vals, B, ldb, out, ldo, nullptr, stream);
}

cn_status cn_csr_gemm_bias_maxout_f32(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                                      const float *vals, const float *B, int64_t ldb, const float *bias, int pool, float *out,
                                      float *argmax, void *stream) {
    if (pool < 1 || N % (pool > 0 ? pool : 1) != 0) { set_error("csr_gemm_bias_maxout_f32: columns are not a multiple of the pool size"); return CN_ERR_SHAPE; }
    cn_status s = check_csr_args("csr_gemm_bias_maxout_f32", R, Cc, N, row_ptr, col_idx, vals, B, ldb, nullptr, 0);
    if (s != CN_OK) return s;
    if (R == 0 || N == 0) return CN_OK;
    if (!bias || !out || !argmax) { set_error("csr_gemm_bias_maxout_f32: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int64_t pooled = N / pool;
    const int64_t row_quads = (R + 3) / 4;
    const bool in_kernel = (pool == 2 || pool == 4) && g_strip_kernel && row_quads <= ctx->num_cu / 8 && N >= 8 * kStripColumns &&
                           aligned(B, 16) && ldb % 4 == 0 && N % 4 == 0 && aligned(bias, 16);
    if (in_kernel) {
        const int64_t strips = (N + kStripColumns - 1) / kStripColumns;
        const int64_t grid = ((strips + 7) / 8) * row_quads * 8;
        if (pool == 2)
            hipLaunchKernelGGL(csr_gemm_strip_kernel<2>, dim3((unsigned)grid), dim3(kT), 0, st, R, N, row_ptr, col_idx, vals, B, ldb, out,
                               pooled, strips, row_quads, (uint32_t *)nullptr, bias, argmax, pooled);
        else
            hipLaunchKernelGGL(csr_gemm_strip_kernel<4>, dim3((unsigned)grid), dim3(kT), 0, st, R, N, row_ptr, col_idx, vals, B, ldb, out,
                               pooled, strips, row_quads, (uint32_t *)nullptr, bias, argmax, pooled);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    // any other shape: the product into the workspace, then bias and maxout in one pass over it
    if ((size_t)R * (size_t)N * sizeof(float) > ctx->workspace_bytes) {
        set_error("csr_gemm_bias_maxout_f32: product does not fit the workspace");
        return CN_ERR_WORKSPACE;
    }
    float *z = reinterpret_cast<float *>(ctx->workspace);
    s = csr_gemm("csr_gemm_bias_maxout_f32", R, Cc, N, row_ptr, col_idx, vals, B, ldb, z, N, nullptr, stream);
    if (s != CN_OK) return s;
    return cn_bias_maxout_f32(z, N, bias, R, N, pool, out, argmax, stream);
}

cn_status cn_csr_gemm_f32_absmax(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                                 const float *vals, const float *B, int64_t ldb, float *out, int64_t ldo,
                                 float *absmax_out, void *stream) {
    if (!absmax_out) { set_error("csr_gemm_f32_absmax: NULL absmax_out"); return CN_ERR_NULL; }
    return csr_gemm("csr_gemm_f32_absmax", R, Cc, N, row_ptr, col_idx, vals, B, ldb, out, ldo, absmax_out, stream);
}

static cn_status csr_gemm_coded(const char *who, int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr,
                                const int32_t *col_idx, const float *vals, const float *B, int64_t ldb,
                                const float *precision_device, uint8_t *codes, float *w, int64_t ldw, float alpha, float *rms,
                                float rate, void *stream) {
    if (R < 0 || Cc < 0 || N < 0) { set_error("%s: negative dimension", who); return CN_ERR_SHAPE; }
    if (ldb < N || (w && ldw < N)) { set_error("%s: leading dimension too small", who); return CN_ERR_SHAPE; }
    if (R > 0x7fffffffLL || Cc > 0x7fffffffLL) { set_error("%s: more than 2^31 rows or columns", who); return CN_ERR_SHAPE; }
    if (R == 0 || N == 0) return CN_OK;
    if (!row_ptr || !precision_device || !codes || (rms && !w)) { set_error("%s: NULL pointer", who); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int lds = (int)sizeof(EncodeShared) + 256 * (int)sizeof(float);
    const int lds_paired = lds + 2 * kProducers * kPatchWords * (int)sizeof(uint32_t);
    static OncePerDevice configured;
    if (configured.first(ctx->device)) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_gemm_coded_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_kernel<2>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_kernel<3>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_kernel<4>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_kernel<5>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds_paired));
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_rows_kernel<6>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds_paired));
    }
    const bool vec = Cc > 0 && Cc * ldb < (1LL << 30) && aligned(B, 16) && ldb % 4 == 0 && N % 4 == 0 && aligned(codes, 4) &&
                     (!w || (aligned(w, 16) && ldw % 4 == 0)) && (!rms || aligned(rms, 16));
    if (vec) {
        const int64_t col_blocks = (N + 255) / 256;
        const int64_t units = ((R + kRowBlock - 1) / kRowBlock) * col_blocks;
        const bool codes_only = !rms && !w;
        const bool paired = !codes_only && g_paired_rows;
        const int threads = paired ? row_threads<5>() : codes_only ? row_threads<2>() : kRowThreads;
        const int64_t per_wg = paired ? kProducers : threads / 64;
        // the encoder table allows three workgroups of 256 threads per compute unit, the registers two of 512;
        // a paired workgroup fills a compute unit
        int64_t grid = (int64_t)ctx->num_cu * (paired ? 1 : g_rows_per_cu > 0 ? g_rows_per_cu : (codes_only ? 2 : 3));
        if (grid > (units + per_wg - 1) / per_wg) grid = (units + per_wg - 1) / per_wg;
        auto kernel = paired ? (rms ? csr_rows_kernel<6> : csr_rows_kernel<5>)
                             : rms ? csr_rows_kernel<4> : (w ? csr_rows_kernel<3> : csr_rows_kernel<2>);
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3((unsigned)threads), paired ? lds_paired : lds, st, R, N, row_ptr, col_idx, vals, B, ldb, col_blocks,
                           (uint32_t *)nullptr, precision_device, codes, w, ldw, alpha, rms, rate, ctx->xsteps, ctx->xstep_count,
                           ctx->table, (uint32_t)(((Cc - 1) * ldb + N) * (int64_t)sizeof(float)));
    } else {
        const int64_t col_blocks = (N + 1023) / 1024;
        int64_t row_groups = ((int64_t)ctx->num_cu * 3 + col_blocks - 1) / col_blocks;
        if (row_groups > (R + 1) / 2) row_groups = (R + 1) / 2;
        hipLaunchKernelGGL(csr_gemm_coded_kernel, dim3((unsigned)(col_blocks * row_groups)), dim3(kCodedThreads), lds, st,
                           R, N, row_ptr, col_idx, vals, B, ldb, col_blocks, precision_device, codes, w, ldw, alpha, rms, rate,
                           ctx->xsteps, ctx->xstep_count, ctx->table);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_csr_gemm_coded_update(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                                   const float *vals, const float *B, int64_t ldb, const float *precision_device,
                                   uint8_t *codes, float *w, int64_t ldw, float alpha, void *stream) {
    return csr_gemm_coded("csr_gemm_coded_update", R, Cc, N, row_ptr, col_idx, vals, B, ldb, precision_device, codes, w, ldw,
                          alpha, nullptr, 0.0f, stream);
}

cn_status cn_csr_gemm_coded_rmsprop(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                                    const float *vals, const float *B, int64_t ldb, const float *precision_device,
                                    uint8_t *codes, float *rms, float *w, int64_t ld, float rms_multiplier,
                                    float learning_rate, void *stream) {
    if (!rms || !w) { set_error("csr_gemm_coded_rmsprop: NULL pointer"); return CN_ERR_NULL; }
    return csr_gemm_coded("csr_gemm_coded_rmsprop", R, Cc, N, row_ptr, col_idx, vals, B, ldb, precision_device, codes, w, ld,
                          rms_multiplier, rms, learning_rate, stream);
}

cn_status cn_csr_to_dense_f32(int64_t R, int64_t Cc, const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                              float *out, int64_t ldo, void *stream) {
    if (R < 0 || Cc < 0 || ldo < Cc) { set_error("csr_to_dense_f32: bad dimensions"); return CN_ERR_SHAPE; }
    if (R == 0 || Cc == 0) return CN_OK;
    if (!row_ptr || !out) { set_error("csr_to_dense_f32: NULL pointer"); return CN_ERR_NULL; }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int64_t wide = (int64_t)ctx->num_cu * 8;
    hipLaunchKernelGGL(csr_to_dense_kernel, dim3((unsigned)(R < wide ? R : wide)), dim3(kT), 0, st, R, Cc, row_ptr, col_idx, vals,
                       out, ldo);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_csr_transpose(int64_t R, int64_t Cc, int64_t nnz, const int32_t *row_ptr, const int32_t *col_idx,
                           const float *vals, int32_t *t_row_ptr, int32_t *t_col_idx, float *t_vals,
                           int32_t *scratch, void *stream) {
    if (R < 0 || Cc < 0 || nnz < 0 || R > 0x7fffffffLL || Cc > 0x7fffffffLL || nnz > 0x7fffffffLL) {
        set_error("csr_transpose: bad dimensions");
        return CN_ERR_SHAPE;
    }
    (void)scratch;  // kept in the signature; the transposition counts in the library's workspace
    if (!row_ptr || !t_row_ptr || (nnz > 0 && (!col_idx || !vals || !t_col_idx || !t_vals))) {
        set_error("csr_transpose: NULL pointer");
        return CN_ERR_NULL;
    }
    Context *ctx;
    cn_status s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int wide = ctx->num_cu * 8;
    int64_t *total_dev = reinterpret_cast<int64_t *>(ctx->sum_scratch);
    if (nnz == 0 || R == 0 || Cc == 0) {
        hipLaunchKernelGGL(zero_counts_kernel, dim3(wide), dim3(kT), 0, st, t_row_ptr, Cc + 1);
        CN_HIP(hipGetLastError());
        return CN_OK;
    }
    // as many row blocks as a cursor array of about four million entries allows (a scan of that size is a few
    // microseconds); one block per row where that fits
    constexpr int64_t kCursorEntries = (int64_t)4 << 20;
    int64_t blocks = R;
    if (blocks * Cc > kCursorEntries) blocks = kCursorEntries / Cc > 1 ? kCursorEntries / Cc : 1;
    const int64_t rows_per_block = (R + blocks - 1) / blocks;
    blocks = (R + rows_per_block - 1) / rows_per_block;
    const int64_t entries = Cc * blocks;
    if ((size_t)(entries + 1) * sizeof(int32_t) > ctx->workspace_bytes) {
        set_error("csr_transpose: %lld columns need a cursor array beyond the workspace", (long long)Cc);
        return CN_ERR_WORKSPACE;
    }
    int32_t *cursor = reinterpret_cast<int32_t *>(ctx->workspace);
    hipLaunchKernelGGL(zero_counts_kernel, dim3(wide), dim3(kT), 0, st, cursor, entries + 1);
    CN_HIP(hipGetLastError());
    hipLaunchKernelGGL(transpose_count_kernel, dim3((unsigned)(R < wide ? R : wide)), dim3(kT), 0, st, R, row_ptr, col_idx, blocks,
                       rows_per_block, cursor);
    CN_HIP(hipGetLastError());
    { cn_status sc = exclusive_scan(ctx, cursor, entries, cursor, total_dev, st); if (sc != CN_OK) return sc; }
    hipLaunchKernelGGL(transpose_row_ptr_kernel, dim3(wide), dim3(kT), 0, st, cursor, Cc, blocks, t_row_ptr);
    CN_HIP(hipGetLastError());
    hipLaunchKernelGGL(transpose_fill_kernel, dim3((unsigned)(blocks < 65535 * 16 ? blocks : 65535 * 16)), dim3(kT), 0, st, R, row_ptr,
                       col_idx, vals, blocks, rows_per_block, cursor, t_col_idx, t_vals);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

}  // extern "C"
