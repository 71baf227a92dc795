// Matrix descriptor and free functions of the clusterNet host API, restricted to what the
// matrix-multiply + 8-bit codec path and its tests touch, implemented over libcnhip (include/cnhip.h).
//
// Mirrors source/basicOps.cuh of the reference: same struct fields, same function names and
// argument meaning.  Differences a caller can observe:
//   * `size` is 64-bit (the reference's int overflows at 100000 x 40000, source/basicOps.cuh:30);
//   * device matrices are ROW-major (the reference transposes to column-major in to_gpu,
//     source/basicOps.cu:14-33); to_gpu / to_host are therefore plain copies, and to_col_major /
//     to_row_major / T are genuine transposes kept for callers that ask for them;
//   * errors that made the reference assert(0) or print-and-continue throw a const char*.
#ifndef CLUSTERNET_FACADE_BASICOPS_H
#define CLUSTERNET_FACADE_BASICOPS_H

#include <stddef.h>

typedef struct Matrix {
    int rows;
    int cols;
    size_t bytes;
    long long size;            // rows * cols
    float *data;               // device (or host, for matrices made by to_host / empty_cpu) fp32 payload
    int isDistributed;
    int cols_distributed;
    unsigned char *char_data;  // 8-bit codes (matrices made by empty_char)
    int isSparse;
    size_t ptr_bytes;
    size_t idx_bytes;
    int *ptr_rows;
    int *idx_cols;
} Matrix;

// Transpose flags of the private ClusterNet::dot overload (cublasOperation_t in the reference).
enum MatrixOp { OP_N = 0, OP_T = 1 };

// ---- allocation (source/basicOps.cu:162-170,214-262,345-407) --------------------------------
Matrix *empty(int rows, int cols);
Matrix *zeros(int rows, int cols);
Matrix *ones(int rows, int cols);
Matrix *fill_matrix(int rows, int cols, float fill_value);
void fill_matrix(Matrix *A, const float fill_value);
Matrix *empty_char(int rows, int cols);
Matrix *empty_cpu(int rows, int cols);
// Not in the reference, whose callers free by hand with cudaFree(m->data); free(m).
void free_matrix(Matrix *A);
void free_cpu_matrix(Matrix *A);

// ---- host <-> device and layout (source/basicOps.cu:14-137) ---------------------------------
Matrix *to_gpu(Matrix *A);
Matrix *to_host(Matrix *A);
Matrix *T(Matrix *A);
Matrix *to_col_major(Matrix *A);
void to_col_major(Matrix *A, Matrix *out);
Matrix *to_row_major(Matrix *A);

// ---- element-wise helpers used next to the path ----------------------------------------------
Matrix *scalarMul(Matrix *A, float a);                 // source/basicOps.cu:622-634
void scalarMul(Matrix *A, float a, Matrix *out);
Matrix *scalarAdd(Matrix *A, float a);                 // source/basicOps.cu:636-648
void scalarAdd(Matrix *A, float a, Matrix *out);
Matrix *sub(Matrix *A, Matrix *B);                     // source/basicOps.cu:460-468,574-580
void sub(Matrix *A, Matrix *B, Matrix *out);
Matrix *abs(Matrix *A);                                // source/basicOps.cu:810-822
void abs(Matrix *A, Matrix *out);
float max(Matrix *A);                                  // source/basicOps.cu:1076-1081
float sum(Matrix *A);                                  // source/basicOps.cu:1070-1074
// max(abs(A)) in one pass without the temporary (not in the reference).
float absmax(Matrix *A);

Matrix *addMatrixVector(Matrix *A, Matrix *v);         // source/basicOps.cu:966-974
void addMatrixVector(Matrix *A, Matrix *v, Matrix *out);
Matrix *softmax(Matrix *A);                            // source/basicOps.cu:1004-1018
void softmax(Matrix *A, Matrix *out);
Matrix **maxout(Matrix *A, int maxout_level);          // source/basicOps.cu:1272-1299: {values, argmax}
void maxout(Matrix *A, Matrix *out, Matrix *outargmax, int maxout_level);
void expand_to_maxout_grad(Matrix *error, Matrix *idx, Matrix *grad);  // source/basicOps.cu:1315-1321

// ---- codec launchers (source/basicOps.cu:1163-1176); `tbl_flt` is accepted and ignored, the
// table lives inside the library --------------------------------------------------------------
void compression_8bit(Matrix *tbl_flt, Matrix *A, float precision, Matrix *out);
void decompression_8bit(Matrix *tbl_flt, Matrix *A, float precision, Matrix *out);

// ---- the passes that follow the 8-bit exchange of a gradient -----------------------------------
// RMSprop_with_weight_update, source/basicOps.cu:1192-1197: same argument list; `m`, `batch_size`
// and `momentum` are unused, as in the reference's kernel.
void RMSprop_with_weight_update(Matrix *RMS, Matrix *grad, Matrix *w, Matrix *m, float RMS_multiplier,
                                float learning_rate, int batch_size, float momentum);
// Not in the reference: the same update reading the gradient as 8-bit codes (grad8->char_data), and
// out += alpha * decode(A) as one pass (decompression_8bit followed by add / sub / a scaled step,
// source/Layer.cpp:430-431, source/DeepNeuralNetwork.cpp:338-339).
void RMSprop_with_weight_update_from_8bit(Matrix *RMS, Matrix *grad8, float precision, Matrix *w,
                                          float RMS_multiplier, float learning_rate);
void decompression_8bit_axpy(Matrix *A, float precision, float alpha, Matrix *out);

// ---- shape checks (source/basicOps.cu:824-933) ----------------------------------------------
int blnFaultySizes(Matrix *A, Matrix *B, Matrix *C);
int blnFaultyMatrixProductSizes(Matrix *A, Matrix *B, Matrix *C, MatrixOp T1, MatrixOp T2);
int checkMatrixOperation(Matrix *A, Matrix *B, Matrix *C, MatrixOp T1, MatrixOp T2, int blnMatrixProduct);

// Throws the library's last error text if `status` is not 0 (internal helper, exposed for tests).
void cn_throw_on_error(int status);

#endif
