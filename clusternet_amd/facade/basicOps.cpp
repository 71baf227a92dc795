// Free functions of the clusterNet host API over libcnhip.  See basicOps.h.
#include "basicOps.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>

#include "cnhip.h"

void cn_throw_on_error(int status) {
    if (status == CN_OK) return;
    static thread_local std::string message;
    message = std::string(cn_status_string(status)) + ": " + cn_last_error();
    fprintf(stderr, "libcnhip error: %s\n", message.c_str());
    throw message.c_str();
}

static Matrix *new_descriptor(int rows, int cols, size_t elem_bytes) {
    if (rows < 0 || cols < 0) {
        printf("Error: matrix dimensions %ix%i are negative.\n", rows, cols);
        throw "Matrix *size error:\n";
    }
    Matrix *m = (Matrix *)malloc(sizeof(Matrix));
    memset(m, 0, sizeof(Matrix));
    m->rows = rows;
    m->cols = cols;
    m->size = (long long)rows * (long long)cols;
    m->bytes = (size_t)m->size * elem_bytes;
    return m;
}

Matrix *empty(int rows, int cols) {
    Matrix *m = new_descriptor(rows, cols, sizeof(float));
    void *p = nullptr;
    cn_throw_on_error(cn_malloc(&p, m->bytes));
    m->data = (float *)p;
    return m;
}

Matrix *empty_char(int rows, int cols) {
    Matrix *m = new_descriptor(rows, cols, sizeof(unsigned char));
    void *p = nullptr;
    cn_throw_on_error(cn_malloc(&p, m->bytes));
    m->char_data = (unsigned char *)p;
    return m;
}

Matrix *empty_cpu(int rows, int cols) {
    Matrix *m = new_descriptor(rows, cols, sizeof(float));
    m->data = (float *)malloc(m->bytes ? m->bytes : 1);
    return m;
}

void fill_matrix(Matrix *A, const float fill_value) {
    cn_throw_on_error(cn_fill_f32(A->data, fill_value, (size_t)A->size, nullptr));
}

Matrix *fill_matrix(int rows, int cols, float fill_value) {
    Matrix *m = empty(rows, cols);
    fill_matrix(m, fill_value);
    return m;
}

Matrix *zeros(int rows, int cols) { return fill_matrix(rows, cols, 0.0f); }
Matrix *ones(int rows, int cols) { return fill_matrix(rows, cols, 1.0f); }

void free_matrix(Matrix *A) {
    if (!A) return;
    cn_free(A->data);
    cn_free(A->char_data);
    free(A);
}

void free_cpu_matrix(Matrix *A) {
    if (!A) return;
    free(A->data);
    free(A->char_data);
    free(A);
}

Matrix *to_gpu(Matrix *A) {
    Matrix *out = empty(A->rows, A->cols);
    cn_throw_on_error(cn_memcpy_h2d(out->data, A->data, A->bytes));
    return out;
}

Matrix *to_host(Matrix *A) {
    if (A->char_data && !A->data) {
        Matrix *out = new_descriptor(A->rows, A->cols, sizeof(unsigned char));
        out->char_data = (unsigned char *)malloc(out->bytes ? out->bytes : 1);
        cn_throw_on_error(cn_memcpy_d2h(out->char_data, A->char_data, A->bytes));
        return out;
    }
    Matrix *out = empty_cpu(A->rows, A->cols);
    cn_throw_on_error(cn_memcpy_d2h(out->data, A->data, A->bytes));
    return out;
}

Matrix *T(Matrix *A) {
    Matrix *out = empty(A->cols, A->rows);
    cn_throw_on_error(cn_transpose_f32(A->data, A->rows, A->cols, out->data, nullptr));
    return out;
}

// Same dimensions, payload re-ordered column-major (the reference's device layout).
void to_col_major(Matrix *A, Matrix *out) {
    cn_throw_on_error(cn_transpose_f32(A->data, A->rows, A->cols, out->data, nullptr));
}

Matrix *to_col_major(Matrix *A) {
    Matrix *out = empty(A->rows, A->cols);
    to_col_major(A, out);
    return out;
}

// Inverse of to_col_major: the payload is read as cols x rows and transposed back.
Matrix *to_row_major(Matrix *A) {
    Matrix *out = empty(A->rows, A->cols);
    cn_throw_on_error(cn_transpose_f32(A->data, A->cols, A->rows, out->data, nullptr));
    return out;
}

static void require_same_shape(Matrix *A, Matrix *B, Matrix *C) {
    if (checkMatrixOperation(A, B, C, OP_N, OP_N, 0)) throw "Matrix *size error:\n";
}

void scalarMul(Matrix *A, float a, Matrix *out) {
    require_same_shape(A, A, out);
    cn_throw_on_error(cn_affine_f32(A->data, a, 0.0f, (size_t)A->size, out->data, nullptr));
}
Matrix *scalarMul(Matrix *A, float a) {
    Matrix *out = empty(A->rows, A->cols);
    scalarMul(A, a, out);
    return out;
}

void scalarAdd(Matrix *A, float a, Matrix *out) {
    require_same_shape(A, A, out);
    cn_throw_on_error(cn_affine_f32(A->data, 1.0f, a, (size_t)A->size, out->data, nullptr));
}
Matrix *scalarAdd(Matrix *A, float a) {
    Matrix *out = empty(A->rows, A->cols);
    scalarAdd(A, a, out);
    return out;
}

void sub(Matrix *A, Matrix *B, Matrix *out) {
    require_same_shape(A, B, out);
    cn_throw_on_error(cn_sub_f32(A->data, B->data, (size_t)A->size, out->data, nullptr));
}
Matrix *sub(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->rows, A->cols);
    sub(A, B, out);
    return out;
}

void abs(Matrix *A, Matrix *out) {
    require_same_shape(A, A, out);
    cn_throw_on_error(cn_abs_f32(A->data, (size_t)A->size, out->data, nullptr));
}
Matrix *abs(Matrix *A) {
    Matrix *out = empty(A->rows, A->cols);
    abs(A, out);
    return out;
}

static float read_scalar(float *device_value) {
    float v = 0.0f;
    cn_throw_on_error(cn_memcpy_d2h(&v, device_value, sizeof(float)));
    return v;
}

// The reference reduces with thrust from a start value of -1 (source/basicOps.cu:1076-1081).
float max(Matrix *A) {
    float *d = nullptr;
    cn_throw_on_error(cn_malloc((void **)&d, sizeof(float)));
    cn_throw_on_error(cn_max_f32(A->data, (size_t)A->size, d, nullptr));
    float v = read_scalar(d);
    cn_free(d);
    return v;
}

float absmax(Matrix *A) {
    float *d = nullptr;
    cn_throw_on_error(cn_malloc((void **)&d, sizeof(float)));
    cn_throw_on_error(cn_absmax_f32(A->data, (size_t)A->size, d, nullptr));
    float v = read_scalar(d);
    cn_free(d);
    return v;
}

float sum(Matrix *A) {
    float *d = nullptr;
    cn_throw_on_error(cn_malloc((void **)&d, sizeof(float)));
    cn_throw_on_error(cn_sum_f32(A->data, (size_t)A->size, d, nullptr));
    float v = read_scalar(d);
    cn_free(d);
    return v;
}

void addMatrixVector(Matrix *A, Matrix *v, Matrix *out) {
    require_same_shape(A, A, out);
    if (v->size != A->cols) {
        printf("Error: vector of size %lld added to a matrix with %i columns.\n", v->size, A->cols);
        throw "Matrix *size error:\n";
    }
    cn_throw_on_error(cn_add_row_vector_f32(A->data, v->data, A->rows, A->cols, out->data, nullptr));
}
Matrix *addMatrixVector(Matrix *A, Matrix *v) {
    Matrix *out = empty(A->rows, A->cols);
    addMatrixVector(A, v, out);
    return out;
}

void softmax(Matrix *A, Matrix *out) {
    require_same_shape(A, A, out);
    cn_throw_on_error(cn_softmax_f32(A->data, A->rows, A->cols, out->data, nullptr));
}
Matrix *softmax(Matrix *A) {
    Matrix *out = empty(A->rows, A->cols);
    softmax(A, out);
    return out;
}

void maxout(Matrix *A, Matrix *out, Matrix *outargmax, int maxout_level) {
    if (maxout_level < 1 || A->cols % maxout_level != 0 || out->rows != A->rows ||
        out->cols != A->cols / maxout_level || outargmax->rows != out->rows || outargmax->cols != out->cols) {
        printf("Error: maxout of level %i on a %ix%i matrix into %ix%i.\n", maxout_level, A->rows, A->cols,
               out->rows, out->cols);
        throw "Matrix *size error:\n";
    }
    cn_throw_on_error(cn_maxout_f32(A->data, A->rows, A->cols, maxout_level, out->data, outargmax->data, nullptr));
}
Matrix **maxout(Matrix *A, int maxout_level) {
    if (maxout_level < 1 || A->cols % maxout_level != 0) throw "Matrix *size error:\n";
    Matrix **pair = (Matrix **)malloc(sizeof(Matrix *) * 2);
    pair[0] = empty(A->rows, A->cols / maxout_level);
    pair[1] = empty(A->rows, A->cols / maxout_level);
    maxout(A, pair[0], pair[1], maxout_level);
    return pair;
}

void expand_to_maxout_grad(Matrix *error, Matrix *idx, Matrix *grad) {
    if (error->cols == 0 || grad->cols % error->cols != 0 || grad->rows != error->rows ||
        idx->rows != error->rows || idx->cols != error->cols) {
        printf("Error: maxout gradient of a %ix%i error into %ix%i.\n", error->rows, error->cols, grad->rows,
               grad->cols);
        throw "Matrix *size error:\n";
    }
    cn_throw_on_error(cn_expand_to_maxout_grad_f32(error->data, idx->data, error->rows, error->cols,
                                                   grad->cols / error->cols, grad->data, nullptr));
}

void compression_8bit(Matrix * /*tbl_flt*/, Matrix *A, float precision, Matrix *out) {
    cn_throw_on_error(cn_compress_8bit(A->data, precision, (size_t)A->size, out->char_data, nullptr));
}

void decompression_8bit(Matrix * /*tbl_flt*/, Matrix *A, float precision, Matrix *out) {
    cn_throw_on_error(cn_decompress_8bit(A->char_data, precision, (size_t)A->size, out->data, nullptr));
}

void RMSprop_with_weight_update(Matrix *RMS, Matrix *grad, Matrix *w, Matrix * /*m*/, float RMS_multiplier,
                                float learning_rate, int /*batch_size*/, float /*momentum*/) {
    cn_throw_on_error(cn_rmsprop_update_f32(RMS->data, grad->data, w->data, RMS_multiplier, learning_rate,
                                            (size_t)RMS->size, nullptr));
}

void RMSprop_with_weight_update_from_8bit(Matrix *RMS, Matrix *grad8, float precision, Matrix *w,
                                          float RMS_multiplier, float learning_rate) {
    cn_throw_on_error(cn_rmsprop_update_w8(RMS->data, grad8->char_data, precision, w->data, RMS_multiplier,
                                           learning_rate, (size_t)RMS->size, nullptr));
}

void decompression_8bit_axpy(Matrix *A, float precision, float alpha, Matrix *out) {
    cn_throw_on_error(cn_decompress_8bit_axpy(A->char_data, precision, alpha, (size_t)A->size, out->data, nullptr));
}

// ---- shape checks: same rules and diagnostics as source/basicOps.cu:824-933 -------------------
int blnFaultySizes(Matrix *A, Matrix *B, Matrix *C) {
    bool ok = A->rows == B->rows && A->cols == B->cols && C->rows == A->rows && C->cols == A->cols;
    return ok ? 0 : 1;
}

static void logical_dims(Matrix *A, Matrix *B, MatrixOp T1, MatrixOp T2, int d[4]) {
    d[0] = T1 == OP_T ? A->cols : A->rows;
    d[1] = T1 == OP_T ? A->rows : A->cols;
    d[2] = T2 == OP_T ? B->cols : B->rows;
    d[3] = T2 == OP_T ? B->rows : B->cols;
}

int blnFaultyMatrixProductSizes(Matrix *A, Matrix *B, Matrix *C, MatrixOp T1, MatrixOp T2) {
    int d[4];
    logical_dims(A, B, T1, T2, d);
    bool ok = d[1] == d[2] && d[0] == C->rows && d[3] == C->cols;
    return ok ? 0 : 1;
}

int checkMatrixOperation(Matrix *A, Matrix *B, Matrix *C, MatrixOp T1, MatrixOp T2, int blnMatrixProduct) {
    if (blnMatrixProduct == 0) {
        if (!blnFaultySizes(A, B, C)) return 0;
        printf("Error: Faulty element-wise matrix operation: \n");
        if (A->rows != B->rows || A->cols != B->cols)
            printf("Matrix *A is of size %ix%i while Matrix *B is of size %ix%i.\n", A->rows, A->cols, B->rows, B->cols);
        else
            printf("Output Matrix *is of size %ix%i while the other matrices are of size %ix%i.\n", C->rows, C->cols,
                   B->rows, B->cols);
        return 1;
    }
    if (!blnFaultyMatrixProductSizes(A, B, C, T1, T2)) return 0;
    int d[4];
    logical_dims(A, B, T1, T2, d);
    printf("Error: Faulty dot product matrix operation:\n");
    if (d[1] != d[2])
        printf("Matrix *A is of size %ix%i while Matrix *B is of size %ix%i.\n", d[0], d[1], d[2], d[3]);
    else
        printf("Output Matrix *is of size %ix%i while Matrix *A and B have sizes %ix%i and %ix%i.\n", C->rows,
               C->cols, d[0], d[1], d[2], d[3]);
    return 1;
}
