// ClusterNet over libcnhip.  See clusterNet.h for what is kept from the reference and what is not.
#include "clusterNet.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include <random>
#include <vector>

#include "cnhip.h"

struct ClusterNet::State {
    std::mt19937_64 rng;
    std::map<std::string, void *> running;        // name -> stopwatch handle
    std::map<std::string, float> cumulative;      // name -> accumulated milliseconds
};

ClusterNet::ClusterNet() { init((int)time(0)); }
ClusterNet::ClusterNet(int seed) { init(seed); }
ClusterNet::ClusterNet(int, char **) { init((int)time(0)); }
ClusterNet::ClusterNet(int, char **, int seed) { init(seed); }
ClusterNet::ClusterNet(int, char **, int seed, bool) { init(seed); }

// Counterpart of ClusterNet::init (source/clusterNet.cpp:40-146): the table upload and handle
// creation happen inside cn_init; the rank topology collapses to a single rank.
void ClusterNet::init(int seed) {
    cn_throw_on_error(cn_init(0));
    m = std::make_shared<State>();
    m->rng.seed((unsigned long long)seed);
    MYRANK = 0;
    NODES = 1;
    MYGPUID = 0;
    MPI_SIZE = 1;
    GPU_COUNT = 1;
}

// Private worker of dot / Tdot / dotT (source/clusterNet.cpp:404-487): shape rule on the logical
// dimensions, diagnostic + throw on mismatch, then one GEMM with alpha 1, beta 0.
void ClusterNet::dot(Matrix *A, Matrix *B, Matrix *out, MatrixOp T1, MatrixOp T2) {
    if (checkMatrixOperation(A, B, out, T1, T2, 1) == 1) throw "Matrix *size error:\n";
    const long long M = out->rows, N = out->cols;
    const long long K = (T1 == OP_T) ? A->rows : A->cols;
    int status = cn_gemm_f32(T1 == OP_T, T2 == OP_T, M, N, K, A->data, A->cols, B->data, B->cols, out->data,
                             out->cols, nullptr);
    if (status != CN_OK) {
        printf("GEMM ERROR: Status %i (%s)\n", status, cn_last_error());
        throw "GEMM ERROR";
    }
}

void ClusterNet::dot(Matrix *A, Matrix *B, Matrix *out) { dot(A, B, out, OP_N, OP_N); }
void ClusterNet::Tdot(Matrix *A, Matrix *B, Matrix *out) { dot(A, B, out, OP_T, OP_N); }
void ClusterNet::dotT(Matrix *A, Matrix *B, Matrix *out) { dot(A, B, out, OP_N, OP_T); }

// The reference allocates with zeros(); beta is 0, so empty() is enough.
Matrix *ClusterNet::dot(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->rows, B->cols);
    dot(A, B, out);
    return out;
}
Matrix *ClusterNet::Tdot(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->cols, B->cols);
    Tdot(A, B, out);
    return out;
}
Matrix *ClusterNet::dotT(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->rows, B->rows);
    dotT(A, B, out);
    return out;
}

Matrix *ClusterNet::dotMPI(Matrix *A, Matrix *B) { return dot(A, B); }
Matrix *ClusterNet::TdotMPI(Matrix *A, Matrix *B) { return Tdot(A, B); }
Matrix *ClusterNet::dotTMPI(Matrix *A, Matrix *B) { return dotT(A, B); }
void ClusterNet::dotMPI(Matrix *A, Matrix *B, Matrix *out) { dot(A, B, out); }
void ClusterNet::TdotMPI(Matrix *A, Matrix *B, Matrix *out) { Tdot(A, B, out); }
void ClusterNet::dotTMPI(Matrix *A, Matrix *B, Matrix *out) { dotT(A, B, out); }

void ClusterNet::compression_8bit(Matrix *A, float precision, Matrix *out) {
    ::compression_8bit(nullptr, A, precision, out);
}
Matrix *ClusterNet::compression_8bit(Matrix *A, float precision) {
    Matrix *out = empty_char(A->rows, A->cols);
    ::compression_8bit(nullptr, A, precision, out);
    return out;
}
void ClusterNet::decompression_8bit(Matrix *A, float precision, Matrix *out) {
    ::decompression_8bit(nullptr, A, precision, out);
}
Matrix *ClusterNet::decompression_8bit(Matrix *A, float precision) {
    Matrix *out = empty(A->rows, A->cols);
    ::decompression_8bit(nullptr, A, precision, out);
    return out;
}

void ClusterNet::dot8bit_weights(Matrix *A, Matrix *B, float precisionB, Matrix *out) {
    if (checkMatrixOperation(A, B, out, OP_N, OP_N, 1) == 1) throw "Matrix *size error:\n";
    cn_throw_on_error(cn_gemm_f32_w8(out->rows, out->cols, A->cols, A->data, A->cols, B->char_data, B->cols,
                                     precisionB, out->data, out->cols, nullptr));
}
Matrix *ClusterNet::dot8bit_weights(Matrix *A, Matrix *B, float precisionB) {
    Matrix *out = empty(A->rows, B->cols);
    dot8bit_weights(A, B, precisionB, out);
    return out;
}

// out += decodeA(A) decodeB(B) with kDot8bit's own two tables (source/clusterKernels.cu:1725-1739): one launch.
void ClusterNet::dot8bit(Matrix *A, Matrix *B, float precisionA, float precisionB, Matrix *out) {
    if (checkMatrixOperation(A, B, out, OP_N, OP_N, 1) == 1) throw "Matrix *size error:\n";
    cn_throw_on_error(cn_gemm_c8c8_add(out->rows, out->cols, A->cols, A->char_data, A->cols, B->char_data, B->cols,
                                       precisionA, precisionB, out->data, out->cols, nullptr));
}
Matrix *ClusterNet::dot8bit(Matrix *A, Matrix *B, float precisionA, float precisionB) {
    Matrix *out = zeros(A->rows, B->cols);
    dot8bit(A, B, precisionA, precisionB, out);
    return out;
}
void ClusterNet::dot8bit_shared(Matrix *A, Matrix *B, float precisionA, float precisionB, Matrix *out) {
    dot8bit(A, B, precisionA, precisionB, out);
}
Matrix *ClusterNet::dot8bit_shared(Matrix *A, Matrix *B, float precisionA, float precisionB) {
    return dot8bit(A, B, precisionA, precisionB);
}

// ---- sparse operands -----------------------------------------------------------------------------
static void require_sparse(Matrix *A) {
    if (!A->isSparse) {
        printf("Error: the first operand must be a sparse matrix (dense_to_sparse).\n");
        throw "Matrix *size error:\n";
    }
}

static Matrix *sparse_shell(int rows, int cols, long long nnz) {
    Matrix *out = (Matrix *)calloc(1, sizeof(Matrix));
    out->rows = rows;
    out->cols = cols;
    out->size = nnz;
    out->bytes = (size_t)nnz * sizeof(float);
    out->idx_bytes = (size_t)nnz * sizeof(int);
    out->ptr_bytes = (size_t)(rows + 1) * sizeof(int);
    out->isSparse = 1;
    void *p = nullptr;
    cn_throw_on_error(cn_malloc(&p, out->ptr_bytes));
    out->ptr_rows = (int *)p;
    cn_throw_on_error(cn_malloc(&p, out->idx_bytes ? out->idx_bytes : 4));
    out->idx_cols = (int *)p;
    cn_throw_on_error(cn_malloc(&p, out->bytes ? out->bytes : 4));
    out->data = (float *)p;
    return out;
}

static void free_sparse(Matrix *A) {
    cn_free(A->data);
    cn_free(A->idx_cols);
    cn_free(A->ptr_rows);
    free(A);
}

Matrix *ClusterNet::dense_to_sparse(Matrix *A) {
    // first call sizes the arrays (capacity 0 reports the count), second call fills them
    void *ptr = nullptr;
    cn_throw_on_error(cn_malloc(&ptr, (size_t)(A->rows + 1) * sizeof(int)));
    int64_t nnz = 0;
    int status = cn_csr_from_dense_f32(A->data, A->rows, A->cols, A->cols, 0, (int *)ptr, nullptr, nullptr, 0, &nnz, nullptr);
    cn_free(ptr);
    if (status != CN_OK && status != CN_ERR_WORKSPACE) cn_throw_on_error(status);
    Matrix *out = sparse_shell(A->rows, A->cols, nnz);
    cn_throw_on_error(cn_csr_from_dense_f32(A->data, A->rows, A->cols, A->cols, 0, out->ptr_rows, out->idx_cols, out->data,
                                            nnz, &nnz, nullptr));
    return out;
}

Matrix *ClusterNet::sparse_to_dense(Matrix *A) {
    require_sparse(A);
    Matrix *out = empty(A->rows, A->cols);
    cn_throw_on_error(cn_csr_to_dense_f32(A->rows, A->cols, A->ptr_rows, A->idx_cols, A->data, out->data, out->cols, nullptr));
    return out;
}

void ClusterNet::dot_sparse(Matrix *A, Matrix *B, Matrix *out) {
    require_sparse(A);
    if (A->cols != B->rows || out->rows != A->rows || out->cols != B->cols) {
        printf("Error: dot_sparse %ix%i times %ix%i into %ix%i.\n", A->rows, A->cols, B->rows, B->cols, out->rows, out->cols);
        throw "Matrix *size error:\n";
    }
    cn_throw_on_error(cn_csr_gemm_f32(A->rows, A->cols, B->cols, A->ptr_rows, A->idx_cols, A->data, B->data, B->cols,
                                      out->data, out->cols, nullptr));
}

void ClusterNet::Tdot_sparse(Matrix *A, Matrix *B, Matrix *out) {
    require_sparse(A);
    if (A->rows != B->rows || out->rows != A->cols || out->cols != B->cols) {
        printf("Error: Tdot_sparse (%ix%i)^T times %ix%i into %ix%i.\n", A->rows, A->cols, B->rows, B->cols, out->rows, out->cols);
        throw "Matrix *size error:\n";
    }
    Matrix *At = sparse_shell(A->cols, A->rows, A->size);
    void *scratch = nullptr;
    cn_throw_on_error(cn_malloc(&scratch, (size_t)(A->cols > 0 ? A->cols : 1) * sizeof(int)));
    cn_throw_on_error(cn_csr_transpose(A->rows, A->cols, A->size, A->ptr_rows, A->idx_cols, A->data, At->ptr_rows, At->idx_cols,
                                       At->data, (int *)scratch, nullptr));
    cn_throw_on_error(cn_csr_gemm_f32(At->rows, At->cols, B->cols, At->ptr_rows, At->idx_cols, At->data, B->data, B->cols,
                                      out->data, out->cols, nullptr));
    cn_throw_on_error(cn_synchronize(nullptr));
    cn_free(scratch);
    free_sparse(At);
}

void ClusterNet::dotT_sparse(Matrix *A, Matrix *B, Matrix *out) {
    require_sparse(A);
    Matrix *Bt = T(B);
    dot_sparse(A, Bt, out);
    cn_throw_on_error(cn_synchronize(nullptr));
    free_matrix(Bt);
}

Matrix *ClusterNet::dot_sparse(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->rows, B->cols);
    dot_sparse(A, B, out);
    return out;
}
Matrix *ClusterNet::Tdot_sparse(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->cols, B->cols);
    Tdot_sparse(A, B, out);
    return out;
}
Matrix *ClusterNet::dotT_sparse(Matrix *A, Matrix *B) {
    Matrix *out = empty(A->rows, B->rows);
    dotT_sparse(A, B, out);
    return out;
}

static Matrix *upload(const std::vector<float> &host, int rows, int cols) {
    Matrix *out = empty(rows, cols);
    cn_throw_on_error(cn_memcpy_h2d(out->data, host.data(), out->bytes));
    return out;
}

Matrix *ClusterNet::rand(int rows, int cols) {
    std::vector<float> h((size_t)rows * cols);
    std::uniform_real_distribution<float> u(0.0f, 1.0f);
    for (float &v : h) v = u(m->rng);
    return upload(h, rows, cols);
}

Matrix *ClusterNet::randn(int rows, int cols) { return randn(rows, cols, 0.0f, 1.0f); }
Matrix *ClusterNet::randn(int rows, int cols, float mean, float std) {
    std::vector<float> h((size_t)rows * cols);
    std::normal_distribution<float> g(mean, std);
    for (float &v : h) v = g(m->rng);
    return upload(h, rows, cols);
}

// lower + u * range with the limits of kCreateRdmSqrtWeight_Logistic
// (source/clusterKernels.cu:126-138): +-4 sqrt(6 / (in + out)).
Matrix *ClusterNet::uniformSqrtWeight(int rows, int cols) {
    std::vector<float> h((size_t)rows * cols);
    std::uniform_real_distribution<float> u(0.0f, 1.0f);
    const float lower = -4.0f * sqrtf(6.0f / ((float)rows + cols));
    const float range = -2.0f * lower;
    for (float &v : h) v = lower + u(m->rng) * range;
    return upload(h, rows, cols);
}
Matrix *ClusterNet::distributed_uniformSqrtWeight(int rows, int cols) { return uniformSqrtWeight(rows, cols); }
Matrix *ClusterNet::distributed_zeros(int rows, int cols) { return zeros(rows, cols); }
Matrix *ClusterNet::distributed_ones(int rows, int cols) { return ones(rows, cols); }

void ClusterNet::tick() { tick("default"); }
void ClusterNet::tick(std::string name) {
    auto it = m->running.find(name);
    if (it != m->running.end()) {
        float ms = 0.0f;
        cn_throw_on_error(cn_timer_stop(it->second, nullptr, &ms));
        m->running.erase(it);
        m->cumulative[name] += ms;
    } else {
        void *h = nullptr;
        cn_throw_on_error(cn_timer_start(&h, nullptr));
        m->running[name] = h;
    }
}

float ClusterNet::tock() { return tock("default"); }
float ClusterNet::tock(std::string name) {
    auto c = m->cumulative.find(name);
    if (c != m->cumulative.end()) {
        float value = c->second;
        m->cumulative.erase(c);
        return value;
    }
    auto it = m->running.find(name);
    if (it == m->running.end()) {
        printf("Error for name: %s\n", name.c_str());
        throw "No tick event was registered for the name";
    }
    float ms = 0.0f;
    cn_throw_on_error(cn_timer_stop(it->second, nullptr, &ms));
    m->running.erase(it);
    return ms;
}
