/* libcnhip: C-ABI of the MI355X (gfx950) implementation of clusterNet's matrix-multiply and
 * 8-bit codec path.
 *
 * Plain pointers and sizes only; every pointer named "device" is a HIP device address, every
 * `stream` is a hipStream_t passed as void* (NULL = the default stream, which is where the
 * reference runs everything).  All calls are asynchronous on `stream` unless stated otherwise.
 * Every function returns a cn_status; 0 is success.  The library never falls back to the CPU:
 * without a usable GPU, cn_init and every compute entry point return CN_ERR_NO_DEVICE.
 *
 * One stream at a time per device, as in the reference (one host thread, the default stream,
 * source/clusterNet.cpp:406-407), for every call that keeps partial results in per-device memory owned by
 * the library; calls that may run at the same time on one device (different streams without an ordering
 * between them) race on it silently:
 *   - the split-K workspace: every product that splits K, cn_csr_from_dense_f32, cn_csr_transpose, and the
 *     fused products (bias + maxout, maxout expansion) for the shapes they do not fuse;
 *   - the ticket lines and slots of the reductions: cn_absmax_f32, cn_max_f32, cn_sum_f32,
 *     cn_absmax_compress_8bit, and the products that also deliver max|C|;
 *   - the array of cn_gemm_f32_noalloc.
 * Kernels that draw their tiles from a counter (the streaming passes on tensors of 2^26 elements and more, the
 * persistent form of an unsplit product) may overlap: a counter is tied to one stream, and a call that is being
 * captured into a graph takes the form that does not draw, so replays may run beside eager calls.
 *
 * Storage convention: matrices are ROW-major with an explicit leading dimension (elements per
 * row).  The reference keeps device matrices column-major (source/basicOps.cu:14-33) and calls
 * cublasSgemm with lda = rows (source/clusterNet.cpp:459-461); a column-major M x K matrix is the
 * same bytes as a row-major K x M one, so a column-major caller obtains C = op(A) op(B) by asking
 * for C^T = op(B)^T op(A)^T, i.e. cn_gemm_f32(transB, transA, N, M, K, B, ldb, A, lda, C, ldc).
 */
#ifndef CNHIP_H
#define CNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int cn_status;
enum {
    CN_OK = 0,
    CN_ERR_NULL = 1,       /* a required pointer is NULL */
    CN_ERR_SHAPE = 2,      /* negative dimension, leading dimension too small, size mismatch */
    CN_ERR_NO_DEVICE = 3,  /* no HIP device / device index out of range */
    CN_ERR_HIP = 4,        /* a HIP runtime call failed; see cn_last_error() */
    CN_ERR_WORKSPACE = 5,  /* internal workspace too small for the request */
    CN_ERR_ARG = 6         /* any other invalid argument */
};

/* Human-readable name of a status code. */
const char *cn_status_string(cn_status s);
/* Text of the most recent failure on the calling thread ("" if none). */
const char *cn_last_error(void);

/* Prepares `device`: uploads the 126-entry codebook and the encoder's bucket table, allocates the
 * split-K workspace (size in MiB from the environment variable CNHIP_WORKSPACE_MB, default 1024).
 * Replaces the table upload of ClusterNet::init (source/clusterNet.cpp:73) and the lazy per-device
 * cuBLAS handle creation (source/clusterNet.cpp:413-426).  Idempotent.  Compute entry points call
 * it on first use for the current device, so calling it explicitly is optional.  Synchronous. */
cn_status cn_init(int device);
/* Frees everything cn_init allocated on every device.  Synchronous. */
cn_status cn_shutdown(void);
/* Number of compute units of the current device as seen by the library (0 before init). */
int cn_num_compute_units(void);

/* Device memory for hosts that have no allocator of their own (the C++ facade).  Replace the
 * cudaMalloc / cudaFree / cudaMemcpy calls inside the Matrix allocators and to_gpu / to_host
 * (source/basicOps.cu:14-88,214-262).  cn_memcpy_* are synchronous with respect to the host. */
cn_status cn_malloc(void **device_ptr, size_t bytes);
cn_status cn_free(void *device_ptr);
cn_status cn_memcpy_h2d(void *device_dst, const void *host_src, size_t bytes);
cn_status cn_memcpy_d2h(void *host_dst, const void *device_src, size_t bytes);
cn_status cn_memcpy_d2d(void *device_dst, const void *device_src, size_t bytes, void *stream);
cn_status cn_fill_f32(float *device_dst, float value, size_t n, void *stream);
cn_status cn_synchronize(void *stream);

/* Copies the 126 codebook magnitudes (ascending, in (0,1)) to host memory.
 * Replaces reading source/8bit_floats.hdf5 through read_hdf5 (source/util.cu:100-131). */
cn_status cn_table_get(float out_host[126]);

/* C[M x N] = op(A) op(B), fp32, alpha = 1, beta = 0 (C is overwritten, never read).
 *   trans_a == 0: A is stored M x K (lda >= K);  trans_a != 0: A is stored K x M (lda >= M).
 *   trans_b == 0: B is stored K x N (ldb >= N);  trans_b != 0: B is stored N x K (ldb >= K).
 *   C is stored M x N (ldc >= N).  M, N, K >= 0 (a zero dimension is a no-op; K == 0 zeroes C).
 * Replaces the cublasSgemm call of ClusterNet::dot(A,B,out,T1,T2) (source/clusterNet.cpp:404-461):
 * dot = (0,0), Tdot = (1,0), dotT = (0,1).  Uses the library's workspace when it splits K, so two
 * GEMMs must not run concurrently on different streams of one device. */
cn_status cn_gemm_f32(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                      const float *A_device, int64_t lda, const float *B_device, int64_t ldb,
                      float *C_device, int64_t ldc, void *stream);

/* cn_gemm_f32 for callers that cannot allocate device memory (a stream under HIP graph capture, a serving loop, a
 * harness that forbids hipMalloc); it has no counterpart in the reference.  Same arguments, same result bit for bit
 * (it splits K exactly as cn_gemm_f32 does on this device), but the partial sums of a split K go to a 64 MiB array
 * that is part of the library's device image, one copy per GPU, held until the process ends, and the call performs
 * no hipMalloc / hipFree, with or without a preceding cn_init.  A product whose K-chunks need more than 64 MiB of
 * partial sums (chunks x M x N x 4 bytes) is refused with CN_ERR_WORKSPACE and nothing is launched.  All calls on
 * one GPU share the array: calls that may overlap on one GPU (streams without an ordering between them) race on it.
 * The first call on a device looks the array's address up; make that call, or cn_init, outside a capture. */
cn_status cn_gemm_f32_noalloc(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                              const float *A_device, int64_t lda, const float *B_device, int64_t ldb,
                              float *C_device, int64_t ldc, void *stream);

/* cn_gemm_f32 that also writes max |C[i][j]| to *absmax_out_device, taken in the kernel's write-out
 * (or in the addition of the K chunks): the value equals cn_absmax_f32 over the result bit for bit
 * (-1.0f for an empty C) and saves that pass over C.  It fuses dot / Tdot with the max(abs(grad)) that
 * precedes every compression_8bit of a gradient (source/DeepNeuralNetwork.cpp:334-337,
 * source/basicOps.cu:810-822,1076-1081). */
cn_status cn_gemm_f32_absmax(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                             const float *A_device, int64_t lda, const float *B_device, int64_t ldb,
                             float *C_device, int64_t ldc, float *absmax_out_device, void *stream);

/* C[M x N] = A[M x K] decode(W[K x N], scale): W holds 8-bit codes (row-major, ldw >= N) that are
 * expanded inside the kernel with exactly the table of cn_decompress_8bit(scale).  No counterpart
 * in the reference; its relatives are dot8bit / dot8bit_shared (source/clusterNet.cpp:1409-1431,
 * source/clusterKernels.cu:1717-1843), which take both operands coded. */
cn_status cn_gemm_f32_w8(int64_t M, int64_t N, int64_t K, const float *A_device, int64_t lda,
                         const uint8_t *W_device, int64_t ldw, float scale, float *C_device,
                         int64_t ldc, void *stream);

/* C[M x N] += decodeA(A[M x K]) decodeB(B[K x N]), both operands 8-bit codes (row-major, lda >= K, ldb >= N), in one
 * launch with nothing staged in memory.  Replaces ClusterNet::dot8bit and dot8bit_shared (source/clusterNet.cpp:1409-1431
 * -> source/basicOps.cu:1455-1472 -> kDot8bit, source/clusterKernels.cu:1717-1762, and kDot8bit_shared, :1764-1843),
 * which add the product to `out`.  The two decode tables are those kernels' own, entry by entry (:1725-1739): entry
 * i < 126 is table[i] * precision of its operand and entry i + 128 its negative; code 126 decodes to 0 and 254 to -0 in
 * both; 127 gives precision_a in A and -precision_a in B, 255 gives precision_b in A and -precision_b in B.  The sum over
 * k runs in fp32 in the order of the matrix instructions, not one k after the other as in kDot8bit: results agree to
 * fp32 rounding of a K-term sum, and bit for bit where a row of A holds a single code that decodes to non-zero. */
cn_status cn_gemm_c8c8_add(int64_t M, int64_t N, int64_t K, const uint8_t *A_codes_device, int64_t lda,
                           const uint8_t *B_codes_device, int64_t ldb, float precision_a, float precision_b,
                           float *C_device, int64_t ldc, void *stream);

/* *out_device = max_i |x_i| (n == 0 gives -1, the start value of the reference's reduction; a NaN
 * input gives NaN).  One pass, no temporary.
 * Replaces the abs + max pair callers use to obtain `precision` (source/basicOps.cu:810-822 and
 * :1076-1081; call sites source/test.cu:2108-2109, source/DeepNeuralNetwork.cpp:218-222). */
cn_status cn_absmax_f32(const float *x_device, size_t n, float *out_device, void *stream);
/* *out_device = max(-1, max_i x_i): the reference's max (source/basicOps.cu:1076-1081), whose
 * reduction starts from -1.  NaN inputs are ordered by their bit pattern. */
cn_status cn_max_f32(const float *x_device, size_t n, float *out_device, void *stream);

/* codes[i] = 8-bit code of x[i] / precision, bit-exact with kCompression_8bit
 * (source/clusterKernels.cu:1163-1232; launcher source/basicOps.cu:1163-1168), flat over n
 * elements.  Inputs whose scaled magnitude falls in (0.99140614, 0.995703], for which the
 * reference reads a table slot it never wrote, encode as 125 / 253. */
cn_status cn_compress_8bit(const float *x_device, float precision, size_t n,
                           uint8_t *codes_device, void *stream);
/* Same, with precision read from device memory (e.g. the output of cn_absmax_f32), so that the
 * absmax -> compress sequence needs no host synchronisation. */
cn_status cn_compress_8bit_dp(const float *x_device, const float *precision_device, size_t n,
                              uint8_t *codes_device, void *stream);

/* *precision_out_device = max_i |x_i| and codes = the codes of x under that precision, in one call and without a
 * round trip to the host: the same bits as cn_absmax_f32 followed by cn_compress_8bit_dp.  The pair of calls in front
 * of every exchange of a gradient, max(abs(grad)) then compression_8bit (source/DeepNeuralNetwork.cpp:334-339,
 * source/test.cu:2108-2111).  Aligned tensors of up to 2^23 elements take one launch that does both phases (a bounded
 * wait across the resident grid between them, the tensor read once); everything else runs as those two kernels, one
 * behind the other on the stream.  cn_host_absmax_compress_single_launch pins either form. */
cn_status cn_absmax_compress_8bit(const float *x_device, size_t n, uint8_t *codes_device,
                                  float *precision_out_device, void *stream);

/* cn_compress_8bit followed by cn_decompress_8bit_axpy on its codes, in one pass: codes[i] as above and
 * y[i] += alpha * (decoded value of codes[i]).  A gradient's codes for the exchange and the own weight
 * update (source/Layer.cpp:365, 430-433) at 13 bytes per element instead of 5 + 9; same bits.  x, codes and y
 * must not overlap. */
cn_status cn_compress_8bit_axpy(const float *x_device, float precision, size_t n, uint8_t *codes_device,
                                float alpha, float *y_device, void *stream);
cn_status cn_compress_8bit_axpy_dp(const float *x_device, const float *precision_device, size_t n,
                                   uint8_t *codes_device, float alpha, float *y_device, void *stream);

/* out[i] = lut[codes[i]] with lut[c] = table[c] * precision, lut[c + 128] = -lut[c] (c < 126),
 * lut[126] = lut[127] = lut[254] = +precision, lut[255] = -precision: bit-exact with
 * kDecompression_8bit (source/clusterKernels.cu:1135-1160; launcher source/basicOps.cu:1172-1176).
 * Note that code 254 (emitted for near-zero inputs) decodes to +precision, as in the reference. */
cn_status cn_decompress_8bit(const uint8_t *codes_device, float precision, size_t n,
                             float *out_device, void *stream);
cn_status cn_decompress_8bit_dp(const uint8_t *codes_device, const float *precision_device,
                                size_t n, float *out_device, void *stream);

/* out[i] = lut[codes[i]] for a 256-entry fp32 table the caller keeps in device memory.  It is the table look-up that
 * the 8-bit products kDot8bit / kDot8bit_shared apply to both coded operands, each with a table of its own whose
 * special codes differ from the codec's (source/clusterKernels.cu:1722-1739, 1775-1792). */
cn_status cn_decode_8bit_lut(const uint8_t *codes_device, const float *lut256_device, size_t n, float *out_device,
                             void *stream);

/* ---- fused passes that follow the 8-bit exchange of a gradient ------------------------------- */

/* y[i] = y[i] + alpha * decode(codes[i]) in one pass (9 bytes per element instead of 17), decode as
 * in cn_decompress_8bit.  alpha = 1 replaces decompression_8bit followed by add, the accumulation of
 * the peers' gradients (source/Layer.cpp:430-431); alpha = -1 replaces decompression_8bit followed by
 * sub (source/DeepNeuralNetwork.cpp:338-339); alpha = -rate is a plain gradient step on coded
 * gradients.  The product alpha * decode is rounded before the addition, so the result equals
 * cn_decompress_8bit followed by cn_sgd_update_f32 / add / sub bit for bit. */
cn_status cn_decompress_8bit_axpy(const uint8_t *codes_device, float precision, float alpha, size_t n,
                                  float *y_device, void *stream);
cn_status cn_decompress_8bit_axpy_dp(const uint8_t *codes_device, const float *precision_device,
                                     float alpha, size_t n, float *y_device, void *stream);

/* RMSprop with weight update, RMSprop_with_weight_update (source/basicOps.cu:1192-1197, kernel
 * source/clusterKernels.cu:1305-1325), per element:
 *   rms = rms_multiplier * rms + grad * grad * (1 - rms_multiplier)
 *   w   = w - learning_rate * (grad / (sqrtf(rms) + 1e-8f))
 * every operation rounded to fp32 in that order.  The reference divides with fdividef, which CUDA
 * documents as accurate to 2 ulp; here the division is correctly rounded.  (The batch_size, momentum
 * and m arguments of the reference routine are unused by its kernel.) */
cn_status cn_rmsprop_update_f32(float *rms_device, const float *grad_device, float *w_device,
                                float rms_multiplier, float learning_rate, size_t n, void *stream);
/* Same with the gradient given as 8-bit codes (decode as in cn_decompress_8bit): one pass of 17
 * bytes per element instead of decompression (5) followed by the update (20). */
cn_status cn_rmsprop_update_w8(float *rms_device, const uint8_t *codes_device, float precision,
                               float *w_device, float rms_multiplier, float learning_rate, size_t n,
                               void *stream);
cn_status cn_rmsprop_update_w8_dp(float *rms_device, const uint8_t *codes_device,
                                  const float *precision_device, float *w_device, float rms_multiplier,
                                  float learning_rate, size_t n, void *stream);

/* ---- sparse (CSR) operands ----------------------------------------------------------------------
 * 32-bit zero-based indices, column indices ascending within a row: the layout of the reference's
 * sparse Matrix (ptr_rows, idx_cols, data; source/basicOps.cuh:25-42) and of cusparseSdense2csr. */

/* CSR of A (transpose = 0) or of A^T (transpose != 0; i.e. the CSC arrays of A), A row-major rows x cols.
 * row_ptr has rows + 1 (cols + 1) entries; col_idx and vals have room for `capacity` nonzeros.
 * *nnz_host receives the number of nonzeros (values that compare unequal to zero); the call
 * synchronises the stream to deliver it.  If it exceeds `capacity`, row_ptr is valid, nothing else is
 * written and the status is CN_ERR_WORKSPACE: call once with capacity 0 to size the arrays.
 * dense_to_sparse, source/clusterNet.cpp:1004-1032 (cusparseSnnz + cusparseSdense2csr). */
cn_status cn_csr_from_dense_f32(const float *A_device, int64_t rows, int64_t cols, int64_t lda, int transpose,
                                int32_t *row_ptr_device, int32_t *col_idx_device, float *vals_device,
                                int64_t capacity, int64_t *nnz_host, void *stream);

/* out[R x N] = S B with S an R x C CSR matrix and B a dense C x N matrix: every output row gathers the
 * rows of B named by its nonzeros, in ascending order, each term as a rounded product added to the
 * running sum (reproducible to the bit).  dot_sparse, source/clusterNet.cpp:301-401 (cusparseScsrmm2). */
cn_status cn_csr_gemm_f32(int64_t R, int64_t C, int64_t N, const int32_t *row_ptr_device,
                          const int32_t *col_idx_device, const float *vals_device, const float *B_device,
                          int64_t ldb, float *out_device, int64_t ldo, void *stream);

/* out, argmax [R x N/pool, contiguous] = maxout(S B + bias): cn_csr_gemm_f32, cn_add_row_vector_f32 and
 * cn_maxout_f32 in one call, the same values.  For a batch of few long rows (the first layer of the forward
 * pass, source/Layer.cpp:250-258) and pool 2 or 4 the bias and the maximum are taken in the product's write-out
 * and S B is never stored; other shapes go through the library's workspace. */
cn_status cn_csr_gemm_bias_maxout_f32(int64_t R, int64_t C, int64_t N, const int32_t *row_ptr_device,
                                      const int32_t *col_idx_device, const float *vals_device, const float *B_device,
                                      int64_t ldb, const float *bias_device, int pool, float *out_device,
                                      float *argmax_device, void *stream);

/* cn_csr_gemm_f32 that also writes max |out[i][j]| to *absmax_out_device (equal bit for bit to
 * cn_absmax_f32 over the result; -1.0f for an empty one): the sparse weight gradient X^T E followed by
 * the max(abs(grad)) in front of compression_8bit (source/Layer.cpp:318-321,
 * source/DeepNeuralNetwork.cpp:334-337) without a second pass over the gradient.  out_device may be
 * NULL: then only the maximum is produced and the product is not stored. */
cn_status cn_csr_gemm_f32_absmax(int64_t R, int64_t C, int64_t N, const int32_t *row_ptr_device,
                                 const int32_t *col_idx_device, const float *vals_device, const float *B_device,
                                 int64_t ldb, float *out_device, int64_t ldo, float *absmax_out_device, void *stream);

/* With G = S B (never stored): codes[R x N, contiguous] = the codes cn_compress_8bit_dp gives for G and
 * *precision_device, and, when w_device is not NULL, w += alpha * (what cn_decompress_8bit gives for those
 * codes) -- bit for bit the sequence cn_csr_gemm_f32, cn_compress_8bit_dp, cn_decompress_8bit_axpy_dp.
 * It is the first-layer weight gradient of a sparse batch, its 8-bit codes for the exchange and the
 * weight update (source/Layer.cpp:318-321, 365, 430-433; source/DeepNeuralNetwork.cpp:334-339) in one
 * pass that reads and writes the weights once and writes one byte per gradient element; take
 * *precision_device from cn_csr_gemm_f32_absmax with a NULL output. */
cn_status cn_csr_gemm_coded_update(int64_t R, int64_t C, int64_t N, const int32_t *row_ptr_device,
                                   const int32_t *col_idx_device, const float *vals_device, const float *B_device,
                                   int64_t ldb, const float *precision_device, uint8_t *codes_device,
                                   float *w_device, int64_t ldw, float alpha, void *stream);

/* Same with RMSprop in place of the plain update: codes as above, then rms and w as cn_rmsprop_update_w8
 * leaves them for those codes (rms and w share the leading dimension ld) -- bit for bit the sequence
 * cn_csr_gemm_f32, cn_compress_8bit_dp, cn_rmsprop_update_w8_dp (source/basicOps.cu:1192-1197 on the
 * round-tripped gradient), 17 bytes per element. */
cn_status cn_csr_gemm_coded_rmsprop(int64_t R, int64_t C, int64_t N, const int32_t *row_ptr_device,
                                    const int32_t *col_idx_device, const float *vals_device, const float *B_device,
                                    int64_t ldb, const float *precision_device, uint8_t *codes_device,
                                    float *rms_device, float *w_device, int64_t ld, float rms_multiplier,
                                    float learning_rate, void *stream);

/* out[R x C] = dense form of S (zeros elsewhere).  sparse_to_dense, source/clusterNet.cpp:1034-1063. */
cn_status cn_csr_to_dense_f32(int64_t R, int64_t C, const int32_t *row_ptr_device, const int32_t *col_idx_device,
                              const float *vals_device, float *out_device, int64_t ldo, void *stream);

/* CSR of S^T from the CSR of the R x C matrix S with nnz nonzeros (t_row_ptr: C + 1 entries, t_col_idx
 * and t_vals: nnz entries, column indices ascending within a row; a source row that names a column twice keeps both
 * entries, in no fixed order).  A counting sort over (column, block of rows) whose cursor array lives in the library's
 * split-K workspace (do not overlap it with a product on another stream): the result does not depend on scheduling, and a column of any number of nonzeros costs
 * what its nonzeros cost.  `scratch` is not used any more and may be NULL.  With it Tdot_sparse (the transposed operand of cusparseScsrmm2, source/clusterNet.cpp:304,307)
 * is cn_csr_gemm_f32 on the transposed arrays. */
cn_status cn_csr_transpose(int64_t R, int64_t C, int64_t nnz, const int32_t *row_ptr_device,
                           const int32_t *col_idx_device, const float *vals_device, int32_t *t_row_ptr_device,
                           int32_t *t_col_idx_device, float *t_vals_device, int32_t *scratch_device, void *stream);

/* ---- small kernels used around the path by its callers (row-major, flat where no shape is given).
 * They are not on the measured hot path; each names the reference routine it stands in for. */

/* out[c][r] = in[r][c] (out is cols x rows).  kTranspose, source/clusterKernels.cu:457-482, the
 * engine of to_col_major / to_row_major / T (source/basicOps.cu:91-137). */
cn_status cn_transpose_f32(const float *in_device, int64_t rows, int64_t cols, float *out_device,
                           void *stream);
/* out[i] = x[i] * mul + add.  scalarMul / scalarAdd, source/basicOps.cu:603-631. */
cn_status cn_affine_f32(const float *x_device, float mul, float add, size_t n, float *out_device,
                        void *stream);
/* out[i] = |x[i]|.  abs, source/basicOps.cu:810-822. */
cn_status cn_abs_f32(const float *x_device, size_t n, float *out_device, void *stream);
/* out[i] = a[i] - b[i].  sub, source/basicOps.cu:456-468. */
cn_status cn_sub_f32(const float *a_device, const float *b_device, size_t n, float *out_device,
                     void *stream);
/* *out_device = sum_i x[i], accumulated in fp64 in a fixed order.  sum, source/basicOps.cu:1070-1074. */
cn_status cn_sum_f32(const float *x_device, size_t n, float *out_device, void *stream);
/* w[i] -= rate * grad[i]: the plain gradient step of the training configuration (the reference's
 * fused optimisers, source/clusterKernels.cu:1306-1346, are outside this path). */
cn_status cn_sgd_update_f32(float *w_device, const float *grad_device, float rate, size_t n,
                            void *stream);
/* out[r][c] = A[r][c] + v[c].  addMatrixVector, source/basicOps.cu:966-974. */
cn_status cn_add_row_vector_f32(const float *A_device, const float *v_device, int64_t rows,
                                int64_t cols, float *out_device, void *stream);
/* out, argmax = maxout(op(A) op(B) + bias): cn_gemm_f32, cn_add_row_vector_f32 and cn_maxout_f32 as one call, the
 * forward pass of a maxout layer (source/Layer.cpp:256-258: dot, addMatrixVector, maxout).  Where the product is
 * summed over chunks of K, bias and maxout ride on that sum; where K is not split, the tiles are whole and the pool
 * is 1, 2 or 4, they happen in the product's own write-out; either way the product never reaches memory as a whole.
 * Other shapes pass through the library's workspace (CN_ERR_WORKSPACE if it does not fit).  out and argmax are
 * M x N / pool, contiguous; same bits as the three calls. */
cn_status cn_gemm_f32_bias_maxout(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A_device,
                                  int64_t lda, const float *B_device, int64_t ldb, const float *bias_device, int pool,
                                  float *out_device, float *argmax_device, void *stream);
/* out = expand_to_maxout_grad(op(A) op(B), argmax): cn_gemm_f32 and cn_expand_to_maxout_grad_f32 as one call, the
 * backward pass through a maxout layer (source/Layer.cpp:318-321 with source/basicOps.cu:1315-1321): the error of the
 * pooled units, M x N, lands in the winners' columns of out, M x N pool, zero elsewhere.  Rides on the chunk sum
 * like cn_gemm_f32_bias_maxout; same bits as the two calls. */
cn_status cn_gemm_f32_expand_maxout_grad(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K,
                                         const float *A_device, int64_t lda, const float *B_device, int64_t ldb,
                                         const float *argmax_device, int pool, float *out_device, void *stream);
/* out, argmax = maxout(A + v) as cn_add_row_vector_f32 followed by cn_maxout_f32 give them, in one pass and
 * without the sum in memory (A with leading dimension lda; out and argmax rows x cols/pool, contiguous).
 * The bias-and-maxout step behind every dot of the forward pass, source/Layer.cpp:256-258. */
cn_status cn_bias_maxout_f32(const float *A_device, int64_t lda, const float *v_device, int64_t rows, int64_t cols,
                             int pool, float *out_device, float *argmax_device, void *stream);
/* Maxout over `pool` consecutive columns: out and argmax are rows x cols/pool; argmax holds the
 * winner's absolute column index as a float, first maximum wins.  maxout,
 * source/basicOps.cu:1272-1299 (defined by the expectations of tests/basicOps_test.cu:580-610). */
cn_status cn_maxout_f32(const float *A_device, int64_t rows, int64_t cols, int pool,
                        float *out_device, float *argmax_device, void *stream);
/* out (rows x pooled_cols*pool) receives err at each winner's column and zero elsewhere.
 * expand_to_maxout_grad, source/basicOps.cu:1315-1321 (tests/basicOps_test.cu:612-638). */
cn_status cn_expand_to_maxout_grad_f32(const float *err_device, const float *argmax_device,
                                       int64_t rows, int64_t pooled_cols, int pool,
                                       float *out_device, void *stream);
/* Row-wise softmax with max subtraction.  softmax, source/basicOps.cu:1012-1018. */
cn_status cn_softmax_f32(const float *A_device, int64_t rows, int64_t cols, float *out_device,
                         void *stream);

/* Stopwatch on a stream: cn_timer_start records a start event and returns a handle;
 * cn_timer_stop records the stop event, waits for it, returns the elapsed milliseconds and
 * releases the handle.  tick / tock, source/util.cu:218-252. */
cn_status cn_timer_start(void **handle, void *stream);
cn_status cn_timer_stop(void *handle, void *stream, float *milliseconds);

#ifdef __cplusplus
}
#endif
#endif /* CNHIP_H */
