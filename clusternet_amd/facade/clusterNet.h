// ClusterNet: the class callers of the reference hold (source/clusterNet.h:77-266), restricted to
// the matrix-multiply + 8-bit codec path and implemented over libcnhip on ONE MI355X.
//
// Kept from the reference: constructor overloads, method names, argument order and meaning,
// out-overloads that never allocate, value-returning overloads that allocate a Matrix the caller
// owns, `throw "Matrix *size error:\n"` on a shape mismatch, cheap by-value copies of the object
// (copies share state, nothing is released on destruction), everything on the default stream.
// Changed on purpose: there is no MPI; MYRANK is 0 and MPI_SIZE is 1, and dotMPI / TdotMPI /
// dotTMPI are the un-sharded product.  The value-returning Tdot of the reference reads
// out->isDistributed before `out` exists (source/clusterNet.cpp:248-249); here it does not.
#ifndef CLUSTERNET_FACADE_CLUSTERNET_H
#define CLUSTERNET_FACADE_CLUSTERNET_H

#include <map>
#include <memory>
#include <string>

#include "basicOps.h"

class ClusterNet {
public:
    ClusterNet();
    ClusterNet(int seed);
    ClusterNet(int argc, char *argv[]);
    ClusterNet(int argc, char *argv[], int seed);
    ClusterNet(int argc, char *argv[], int seed, bool useSameSeed);

    // C = A B, C = A^T B, C = A B^T (source/clusterNet.cpp:230-298)
    Matrix *dot(Matrix *A, Matrix *B);
    Matrix *Tdot(Matrix *A, Matrix *B);
    Matrix *dotT(Matrix *A, Matrix *B);
    void dot(Matrix *A, Matrix *B, Matrix *out);
    void Tdot(Matrix *A, Matrix *B, Matrix *out);
    void dotT(Matrix *A, Matrix *B, Matrix *out);
    // The sharded products of the reference (source/clusterNet.cpp:490-733); one rank, no exchange.
    Matrix *dotMPI(Matrix *A, Matrix *B);
    Matrix *TdotMPI(Matrix *A, Matrix *B);
    Matrix *dotTMPI(Matrix *A, Matrix *B);
    void dotMPI(Matrix *A, Matrix *B, Matrix *out);
    void TdotMPI(Matrix *A, Matrix *B, Matrix *out);
    void dotTMPI(Matrix *A, Matrix *B, Matrix *out);

    // 8-bit codec (source/clusterNet.cpp:1384-1406)
    Matrix *compression_8bit(Matrix *A, float precision);
    void compression_8bit(Matrix *A, float precision, Matrix *out);
    Matrix *decompression_8bit(Matrix *A, float precision);
    void decompression_8bit(Matrix *A, float precision, Matrix *out);
    // out = A decode(B codes, precisionB): the fused kernel that takes the place of the
    // dot8bit prototypes (source/clusterNet.cpp:1409-1431).  A is fp32, B is a char matrix.
    // The 8-bit products of the reference (source/clusterNet.h:146-149, source/clusterNet.cpp:1409-1431): A and B are
    // char matrices, out += decodeA(A) decodeB(B) in fp32.  As in kDot8bit (source/clusterKernels.cu:1717-1762) the
    // result is ADDED to what out holds, and each operand is decoded through that kernel's own table, whose special
    // codes are not the codec's: 126 -> 0 and 254 -> -0 on both sides, 127 -> precisionA (A) / -precisionA (B),
    // 255 -> precisionB (A) / -precisionB (B) -- the reference's literal, evidently mixed-up, assignments.  Here the
    // operands are decoded and multiplied on the matrix cores, so sums differ from the reference's sequential fp32
    // accumulation within the usual product tolerance; dot8bit_shared (tiles + atomicAdd in the reference, whose
    // order of additions is not defined) is the same computation.  The value-returning forms start from zeros of
    // A->rows x B->cols (the reference allocates A->rows x A->cols without clearing it).
    void dot8bit(Matrix *A, Matrix *B, float precisionA, float precisionB, Matrix *out);
    Matrix *dot8bit(Matrix *A, Matrix *B, float precisionA, float precisionB);
    void dot8bit_shared(Matrix *A, Matrix *B, float precisionA, float precisionB, Matrix *out);
    Matrix *dot8bit_shared(Matrix *A, Matrix *B, float precisionA, float precisionB);
    Matrix *dot8bit_weights(Matrix *A, Matrix *B, float precisionB);
    void dot8bit_weights(Matrix *A, Matrix *B, float precisionB, Matrix *out);

    // Sparse operands (source/clusterNet.cpp:301-401,1004-1063): A is a sparse Matrix as made by
    // dense_to_sparse (isSparse = 1; data = values, idx_cols, ptr_rows, size = number of nonzeros).
    Matrix *dense_to_sparse(Matrix *A);
    Matrix *sparse_to_dense(Matrix *A);
    Matrix *dot_sparse(Matrix *A, Matrix *B);    // A B
    Matrix *Tdot_sparse(Matrix *A, Matrix *B);   // A^T B
    Matrix *dotT_sparse(Matrix *A, Matrix *B);   // A B^T
    void dot_sparse(Matrix *A, Matrix *B, Matrix *out);
    void Tdot_sparse(Matrix *A, Matrix *B, Matrix *out);
    void dotT_sparse(Matrix *A, Matrix *B, Matrix *out);

    // Input generators of the test and benchmark harness (source/clusterNet.cpp:746-788,874-938).
    // Values come from a host-side generator seeded by the constructor, not from cuRAND.
    Matrix *rand(int rows, int cols);
    Matrix *randn(int rows, int cols);
    Matrix *randn(int rows, int cols, float mean, float std);
    Matrix *uniformSqrtWeight(int rows, int cols);              // +-4 sqrt(6 / (rows + cols))
    Matrix *distributed_uniformSqrtWeight(int rows, int cols);  // one rank: same as above
    Matrix *distributed_zeros(int rows, int cols);
    Matrix *distributed_ones(int rows, int cols);

    // Named stopwatches on the default stream (source/clusterNet.cpp:798-840): tick(name) starts,
    // tock(name) returns the milliseconds since the matching tick and adds them to the name's
    // running total, which a later tock of the same name keeps returning cumulatively.
    void tick(std::string name);
    void tick();
    float tock(std::string name);
    float tock();

    void shutdown_MPI() {}

    int MYRANK;
    int NODES;
    int MYGPUID;
    int MPI_SIZE;
    int GPU_COUNT;

private:
    struct State;
    std::shared_ptr<State> m;
    void init(int seed);
    void dot(Matrix *A, Matrix *B, Matrix *out, MatrixOp T1, MatrixOp T2);
};

#endif
