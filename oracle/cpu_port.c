/* TEST INFRASTRUCTURE ONLY: the multi-threaded CPU port timed as the cpu_baseline of the bench.
 *
 * Same arithmetic as oracle.c (which see for the reference lines each routine follows), arranged
 * to use all host cores: the codec loops are the literal per-element procedure of
 * source/clusterKernels.cu:1135-1232 spread over OpenMP threads, the GEMM is the fp32 product of
 * source/clusterNet.cpp:404-461 cache-blocked over output columns.  Never a product path.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

void cn_oracle_compress_literal(const float *x, float precision, size_t n, uint8_t *codes,
                                int sliver_rule);
void cn_oracle_decompress(const uint8_t *codes, float precision, size_t n, float *out);
float cn_oracle_absmax(const float *x, size_t n);

int cn_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void cn_oracle_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

#define CHUNK ((size_t)1 << 16)

void cn_port_compress(const float *x, float precision, size_t n, uint8_t *codes) {
    size_t chunks = (n + CHUNK - 1) / CHUNK;
#pragma omp parallel for schedule(static)
    for (size_t c = 0; c < chunks; ++c) {
        size_t b = c * CHUNK, e = b + CHUNK < n ? b + CHUNK : n;
        cn_oracle_compress_literal(x + b, precision, e - b, codes + b, 0);
    }
}

void cn_port_decompress(const uint8_t *codes, float precision, size_t n, float *out) {
    size_t chunks = (n + CHUNK - 1) / CHUNK;
#pragma omp parallel for schedule(static)
    for (size_t c = 0; c < chunks; ++c) {
        size_t b = c * CHUNK, e = b + CHUNK < n ? b + CHUNK : n;
        cn_oracle_decompress(codes + b, precision, e - b, out + b);
    }
}

float cn_port_absmax(const float *x, size_t n) {
    size_t chunks = (n + CHUNK - 1) / CHUNK;
    float best = -1.0f;
#pragma omp parallel for schedule(static) reduction(max : best)
    for (size_t c = 0; c < chunks; ++c) {
        size_t b = c * CHUNK, e = b + CHUNK < n ? b + CHUNK : n;
        float v = cn_oracle_absmax(x + b, e - b);
        if (v > best) best = v;
    }
    return best;
}

/* C[M x N] = op(A) op(B) (+ C if `accumulate`), row-major, fp32 accumulation: ClusterNet::dot / Tdot / dotT
 * (source/clusterNet.cpp:230-298,404-461).  trans_a: A stored K x M; trans_b: B stored N x K.  Threads own column
 * panels of 256; with B stored K x N, K is walked in slabs of 128 so the A slab and the C panel stay in cache, and
 * the inner loop runs along a row of B; with B stored N x K an output is a dot product of two contiguous rows,
 * summed in eight interleaved partial sums. */
#define NB 256
#define KB 128
void cn_port_gemm(int trans_a, int trans_b, int accumulate, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                  const float *B, int64_t ldb, float *C, int64_t ldc) {
    int64_t panels = (N + NB - 1) / NB;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t p = 0; p < panels; ++p) {
        int64_t n0 = p * NB, nw = n0 + NB <= N ? NB : N - n0;
        if (!accumulate)
            for (int64_t m = 0; m < M; ++m) memset(C + m * ldc + n0, 0, (size_t)nw * sizeof(float));
        if (!trans_b) {
            for (int64_t k0 = 0; k0 < K; k0 += KB) {
                int64_t kw = k0 + KB <= K ? KB : K - k0;
                for (int64_t m = 0; m < M; ++m) {
                    float *restrict crow = C + m * ldc + n0;
                    for (int64_t k = 0; k < kw; ++k) {
                        float av = trans_a ? A[(k0 + k) * lda + m] : A[m * lda + k0 + k];
                        const float *restrict brow = B + (k0 + k) * ldb + n0;
                        for (int64_t n = 0; n < nw; ++n) crow[n] += av * brow[n];
                    }
                }
            }
        } else {
            for (int64_t m = 0; m < M; ++m)
                for (int64_t n = 0; n < nw; ++n) {
                    const float *restrict brow = B + (n0 + n) * ldb;
                    float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                    int64_t k = 0;
                    if (!trans_a) {
                        const float *restrict arow = A + m * lda;
                        for (; k + 8 <= K; k += 8)
                            for (int u = 0; u < 8; ++u) part[u] += arow[k + u] * brow[k + u];
                        for (; k < K; ++k) part[0] += arow[k] * brow[k];
                    } else {
                        for (; k < K; ++k) part[k & 7] += A[k * lda + m] * brow[k];
                    }
                    C[m * ldc + n0 + n] += ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
                }
        }
    }
}

void cn_port_gemm_nn(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                     int64_t ldb, float *C, int64_t ldc) {
    cn_port_gemm(0, 0, 0, M, N, K, A, lda, B, ldb, C, ldc);
}
