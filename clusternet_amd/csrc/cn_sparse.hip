// Sparse (CSR) x dense products for gfx950 and the conversion from dense storage.
//
// The input batch of the reference's large configuration is 2 % dense.  A dense product streams the
// weight matrix once and spends 50x the necessary flops doing so; the products below are bound by
// the same stream (or by writing the result) and do no wasted arithmetic.  S is an R x C matrix in
// CSR form (row_ptr[R + 1], col_idx[nnz] ascending within a row, vals[nnz]), 32-bit indices.
//
//   csr_gemm      out[R x N] = S B     every output row gathers the B rows of its nonzeros
//                                       (bound by writing out; B should be small enough to stay in L2)
//   csr_gemm_tn   out[C x N] = S^T B   B is streamed once, row k of B is scattered into the output rows
//                                       named by row k of S; the output (C <= 128 rows per pass) is
//                                       accumulated in LDS; the R rows may be split into chunks whose
//                                       partial outputs are added in a fixed order
//
// With X the 128 x 100000 batch and S = CSR(X^T):  X W = S^T W (csr_gemm_tn) and X^T E = S E (csr_gemm).
// Sums run over the nonzeros in ascending order with a rounded product and a rounded addition per
// term, so csr_gemm is reproducible to the bit and csr_gemm_tn is once the chunking is fixed.
#include "cn_internal.h"

namespace cn {

namespace {

constexpr int kT = 256;
typedef float f32x4 __attribute__((ext_vector_type(4)));

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---- dense -> CSR ----------------------------------------------------------------------------------
// counts[i] = number of nonzeros of row i of op(A); op = identity or transpose.  A value is a nonzero
// when it compares unequal to 0 (so -0.0 is dropped and NaN is kept).
__global__ __launch_bounds__(kT) void count_rows_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                        int64_t lda, int32_t *__restrict__ counts) {
    // one workgroup per row of A
    __shared__ int partial[kT / 64];
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        int c = 0;
        for (int64_t j = threadIdx.x; j < cols; j += kT) c += (A[r * lda + j] != 0.0f) ? 1 : 0;
        for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = c;
        __syncthreads();
        if (threadIdx.x == 0) counts[r] = partial[0] + partial[1] + partial[2] + partial[3];
        __syncthreads();
    }
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

// row_ptr[0 .. n] = exclusive prefix sums of counts[0 .. n - 1] (in place: counts == row_ptr is allowed
// because every thread reads its run before any thread writes); *total = row_ptr[n].  One workgroup.
__global__ __launch_bounds__(kT) void scan_kernel(const int32_t *counts, int64_t n, int32_t *row_ptr,
                                                  int64_t *__restrict__ total) {
    __shared__ int64_t sums[kT];
    const int64_t per = (n + kT - 1) / kT;
    const int64_t lo = (int64_t)threadIdx.x * per, hi = (lo + per < n) ? lo + per : n;
    int64_t s = 0;
    for (int64_t i = lo; i < hi; ++i) s += counts[i];
    sums[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t run = 0;
        for (int i = 0; i < kT; ++i) { const int64_t v = sums[i]; sums[i] = run; run += v; }
        *total = run;
    }
    __syncthreads();
    int64_t run = sums[threadIdx.x];
    for (int64_t i = lo; i < hi; ++i) {
        const int32_t c = counts[i];
        row_ptr[i] = (int32_t)run;
        run += c;
    }
    __syncthreads();
    if (threadIdx.x == 0) row_ptr[n] = (int32_t)*total;
}

// CSR of A: one workgroup per row, columns compacted in ascending order.
__global__ __launch_bounds__(kT) void fill_rows_kernel(const float *__restrict__ A, int64_t rows, int64_t cols,
                                                       int64_t lda, const int32_t *__restrict__ row_ptr,
                                                       int32_t *__restrict__ col_idx, float *__restrict__ vals) {
    __shared__ int wave_count[kT / 64];
    __shared__ int base;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        if (threadIdx.x == 0) base = row_ptr[r];
        __syncthreads();
        for (int64_t j0 = 0; j0 < cols; j0 += kT) {
            const int64_t j = j0 + threadIdx.x;
            const float v = (j < cols) ? A[r * lda + j] : 0.0f;
            const bool keep = v != 0.0f;
            const unsigned long long mask = __ballot(keep);
            const int before = __popcll(mask & ((1ull << lane) - 1ull));
            if (lane == 0) wave_count[wave] = __popcll(mask);
            __syncthreads();
            int offset = base + before;
            for (int w = 0; w < wave; ++w) offset += wave_count[w];
            if (keep) { col_idx[offset] = (int32_t)j; vals[offset] = v; }
            __syncthreads();
            if (threadIdx.x == 0) base += wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
            __syncthreads();
        }
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
// A workgroup owns a block of 1024 columns (4 per lane) and walks a range of output rows.
template <bool kVector>
__global__ __launch_bounds__(kT) void csr_gemm_kernel(int64_t R, int64_t N, const int32_t *__restrict__ row_ptr,
                                                      const int32_t *__restrict__ col_idx,
                                                      const float *__restrict__ vals, const float *__restrict__ B,
                                                      int64_t ldb, float *__restrict__ out, int64_t ldo,
                                                      int64_t col_blocks) {
    const int64_t cb = blockIdx.x % col_blocks, rg = blockIdx.x / col_blocks, row_groups = gridDim.x / col_blocks;
    const int64_t n = cb * 1024 + 4 * (int64_t)threadIdx.x;
    for (int64_t r = rg; r < R; r += row_groups) {
        const int32_t j0 = row_ptr[r], j1 = row_ptr[r + 1];
        if (kVector) {
            if (n >= N) continue;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            for (int32_t j = j0; j < j1; ++j) {
                const float v = vals[j];
                const f32x4 b = *reinterpret_cast<const f32x4 *>(B + (int64_t)col_idx[j] * ldb + n);
                acc = acc + v * b;
            }
            __builtin_nontemporal_store(acc, reinterpret_cast<f32x4 *>(out + r * ldo + n));
        } else {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int32_t j = j0; j < j1; ++j) {
                const float v = vals[j];
                const float *b = B + (int64_t)col_idx[j] * ldb + n;
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) acc[e] = acc[e] + v * b[e];
            }
            for (int e = 0; e < 4; ++e)
                if (n + e < N) out[r * ldo + n + e] = acc[e];
        }
    }
}

// ---- out = S^T B (scatter into LDS) -----------------------------------------------------------------------
// A workgroup owns 256 output columns (one per lane), up to 128 output rows [c0, c0 + 128) and a range
// of S rows.  acc[c][lane] lives in LDS; lane t only ever touches column t, so no atomics are needed.
constexpr int kScatterRows = 128;
constexpr int kScatterCols = 256;

__global__ __launch_bounds__(kT) void csr_gemm_tn_kernel(int64_t R, int64_t Cc, int64_t N,
                                                         const int32_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col_idx,
                                                         const float *__restrict__ vals, const float *__restrict__ B,
                                                         int64_t ldb, float *__restrict__ out, int64_t ldo,
                                                         float *__restrict__ partial, int64_t col_blocks,
                                                         int64_t row_blocks, int splits, int64_t rows_per_split) {
    extern __shared__ __attribute__((aligned(16))) float acc[];  // [kScatterRows][kScatterCols]
    const int64_t cb = blockIdx.x % col_blocks;
    const int64_t rb = (blockIdx.x / col_blocks) % row_blocks;
    const int64_t split = blockIdx.x / (col_blocks * row_blocks);
    const int64_t n = cb * kScatterCols + threadIdx.x;
    const int32_t c0 = (int32_t)(rb * kScatterRows);
    const bool live = n < N;
    for (int c = 0; c < kScatterRows; ++c) acc[c * kScatterCols + threadIdx.x] = 0.0f;
    const int64_t k0 = split * rows_per_split;
    const int64_t k1 = (k0 + rows_per_split < R) ? k0 + rows_per_split : R;
    constexpr int kAhead = 8;  // B values in flight per lane
    for (int64_t kb = k0; kb < k1; kb += kAhead) {
        float b[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u)
            b[u] = (live && kb + u < k1) ? __builtin_nontemporal_load(B + (kb + u) * ldb + n) : 0.0f;
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            if (kb + u >= k1) break;
            const int32_t j0 = row_ptr[kb + u], j1 = row_ptr[kb + u + 1];
            for (int32_t j = j0; j < j1; ++j) {
                const int32_t c = col_idx[j] - c0;
                if (c < 0 || c >= kScatterRows) continue;
                float *cell = acc + c * kScatterCols + threadIdx.x;
                *cell = *cell + vals[j] * b[u];
            }
        }
    }
    if (!live) return;
    const int64_t rows_here = (Cc - c0 < kScatterRows) ? Cc - c0 : kScatterRows;
    if (splits > 1) {
        float *plane = partial + split * Cc * N;
        for (int64_t c = 0; c < rows_here; ++c) plane[(c0 + c) * N + n] = acc[c * kScatterCols + threadIdx.x];
    } else {
        for (int64_t c = 0; c < rows_here; ++c) out[(c0 + c) * ldo + n] = acc[c * kScatterCols + threadIdx.x];
    }
}

cn_status check_csr_args(const char *who, int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr,
                         const int32_t *col_idx, const float *vals, const float *B, int64_t ldb, const float *out,
                         int64_t ldo) {
    if (R < 0 || Cc < 0 || N < 0) { set_error("%s: negative dimension", who); return CN_ERR_SHAPE; }
    if (ldb < N || ldo < N) { set_error("%s: leading dimension too small", who); return CN_ERR_SHAPE; }
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
    if (rows > 0 && cols > 0) {
        if (transpose) {
            const int64_t blocks = (cols + kT - 1) / kT;
            hipLaunchKernelGGL(count_cols_kernel, dim3((unsigned)(blocks < wide ? blocks : wide)), dim3(kT), 0, st, A, rows,
                               cols, lda, row_ptr);
        } else {
            hipLaunchKernelGGL(count_rows_kernel, dim3((unsigned)(rows < wide ? rows : wide)), dim3(kT), 0, st, A, rows, cols,
                               lda, row_ptr);
        }
        CN_HIP(hipGetLastError());
    } else if (out_rows > 0) {
        hipLaunchKernelGGL(zero_counts_kernel, dim3(wide), dim3(kT), 0, st, row_ptr, out_rows);
        CN_HIP(hipGetLastError());
    }
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kT), 0, st, row_ptr, out_rows, row_ptr, total_dev);
    CN_HIP(hipGetLastError());
    CN_HIP(hipMemcpyAsync(nnz_host, total_dev, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    CN_HIP(hipStreamSynchronize(st));
    if (*nnz_host > 0x7fffffffLL) { set_error("csr_from_dense_f32: more than 2^31 nonzeros"); return CN_ERR_SHAPE; }
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
        hipLaunchKernelGGL(fill_rows_kernel, dim3((unsigned)(rows < wide ? rows : wide)), dim3(kT), 0, st, A, rows, cols, lda,
                           row_ptr, col_idx, vals);
    }
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_csr_gemm_f32(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                          const float *vals, const float *B, int64_t ldb, float *out, int64_t ldo, void *stream) {
    cn_status s = check_csr_args("csr_gemm_f32", R, Cc, N, row_ptr, col_idx, vals, B, ldb, out, ldo);
    if (s != CN_OK) return s;
    if (R == 0 || N == 0) return CN_OK;
    if (!out) { set_error("csr_gemm_f32: NULL output"); return CN_ERR_NULL; }
    Context *ctx;
    s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int64_t col_blocks = (N + 1023) / 1024;
    int64_t row_groups = ((int64_t)ctx->num_cu * 8 + col_blocks - 1) / col_blocks;
    if (row_groups > R) row_groups = R;
    const bool vec = aligned(B, 16) && aligned(out, 16) && ldb % 4 == 0 && ldo % 4 == 0 && N % 4 == 0;
    if (vec)
        hipLaunchKernelGGL(csr_gemm_kernel<true>, dim3((unsigned)(col_blocks * row_groups)), dim3(kT), 0, st, R, N, row_ptr,
                           col_idx, vals, B, ldb, out, ldo, col_blocks);
    else
        hipLaunchKernelGGL(csr_gemm_kernel<false>, dim3((unsigned)(col_blocks * row_groups)), dim3(kT), 0, st, R, N, row_ptr,
                           col_idx, vals, B, ldb, out, ldo, col_blocks);
    CN_HIP(hipGetLastError());
    return CN_OK;
}

cn_status cn_csr_gemm_tn_f32(int64_t R, int64_t Cc, int64_t N, const int32_t *row_ptr, const int32_t *col_idx,
                             const float *vals, const float *B, int64_t ldb, float *out, int64_t ldo, int splits,
                             void *stream) {
    cn_status s = check_csr_args("csr_gemm_tn_f32", R, Cc, N, row_ptr, col_idx, vals, B, ldb, out, ldo);
    if (s != CN_OK) return s;
    if (Cc == 0 || N == 0) return CN_OK;
    if (!out) { set_error("csr_gemm_tn_f32: NULL output"); return CN_ERR_NULL; }
    Context *ctx;
    s = current_context(&ctx);
    if (s != CN_OK) return s;
    hipStream_t st = (hipStream_t)stream;
    const int64_t col_blocks = (N + kScatterCols - 1) / kScatterCols;
    const int64_t row_blocks = (Cc + kScatterRows - 1) / kScatterRows;
    if (splits <= 0) {  // enough workgroups for one per compute unit, chunks at least 256 rows deep
        int64_t want = ((int64_t)ctx->num_cu + col_blocks * row_blocks - 1) / (col_blocks * row_blocks);
        int64_t most = R / 256;
        if (want > most) want = most;
        if (want > 64) want = 64;
        splits = (int)(want < 1 ? 1 : want);
    }
    if (splits > 1 && (size_t)splits * (size_t)Cc * (size_t)N * sizeof(float) > ctx->workspace_bytes) {
        size_t fit = ctx->workspace_bytes / ((size_t)Cc * (size_t)N * sizeof(float));
        splits = (int)(fit < 1 ? 1 : fit);
    }
    int64_t rows_per_split = (R + splits - 1) / splits;
    if (rows_per_split < 1) rows_per_split = 1;
    splits = (int)((R + rows_per_split - 1) / rows_per_split);
    if (splits < 1) splits = 1;
    const size_t lds = (size_t)kScatterRows * kScatterCols * sizeof(float);
    static bool configured = false;
    if (!configured) {
        CN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&csr_gemm_tn_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    const int64_t grid = col_blocks * row_blocks * splits;
    if (grid > 0x7fffffffLL) { set_error("csr_gemm_tn_f32: too many workgroups"); return CN_ERR_SHAPE; }
    hipLaunchKernelGGL(csr_gemm_tn_kernel, dim3((unsigned)grid), dim3(kT), lds, st, R, Cc, N, row_ptr, col_idx, vals, B, ldb,
                       out, ldo, (float *)ctx->workspace, col_blocks, row_blocks, splits, rows_per_split);
    CN_HIP(hipGetLastError());
    if (splits > 1) return add_chunk_planes(ctx, splits, Cc, N, out, ldo, nullptr, st);
    return CN_OK;
}

}  // extern "C"
