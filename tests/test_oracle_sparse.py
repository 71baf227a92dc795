"""Pins of the CPU checker's sparse routines: the CSR layout against scipy.sparse, the products
against the dense product of the densified operand (what the reference's own tests ask of its sparse
path, tests/clusterNet_test.cu:396-463), and the summation order against a direct loop."""
import numpy as np
import scipy.sparse as sp

import oracle


def _sparse(rng, rows, cols, density):
    A = rng.uniform(0, 1, (rows, cols)).astype(np.float32)
    return A * (rng.random((rows, cols)) < density)


def test_csr_layout_equals_scipy():
    rng = np.random.default_rng(1)
    for rows, cols, d in ((1, 1, 1.0), (7, 11, 0.3), (128, 1000, 0.02), (50, 3, 0.5), (4, 9, 0.0)):
        A = _sparse(rng, rows, cols, d)
        if A.size > 3:
            A.flat[1] = -0.0                       # negative zero is not stored
        for transpose in (False, True):
            M = A.T if transpose else A
            S = sp.csr_matrix(M)
            S.eliminate_zeros()
            S.sort_indices()
            row_ptr, col_idx, vals = oracle.csr_from_dense(A, transpose)
            assert np.array_equal(row_ptr, S.indptr) and np.array_equal(col_idx, S.indices)
            assert np.array_equal(vals.view(np.uint32), S.data.astype(np.float32).view(np.uint32))


def test_products_equal_dense_products():
    rng = np.random.default_rng(2)
    A = _sparse(rng, 37, 211, 0.05)
    B = rng.normal(0, 1, (211, 19)).astype(np.float32)
    E = rng.normal(0, 1, (37, 23)).astype(np.float32)
    csr = oracle.csr_from_dense(A)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.max(np.abs(oracle.csr_gemm(csr, B) - want)) < 1e-5
    # X^T E through the CSR of X^T, as the training step uses it
    want_t = A.T.astype(np.float64) @ E.astype(np.float64)
    csr_t = oracle.csr_from_dense(A, transpose=True)
    assert np.max(np.abs(oracle.csr_gemm(csr_t, E) - want_t)) < 1e-5


def test_summation_order_is_ascending_and_unfused():
    rng = np.random.default_rng(3)
    A = _sparse(rng, 5, 40, 0.4)
    B = rng.normal(0, 1, (40, 3)).astype(np.float32)
    got = oracle.csr_gemm(oracle.csr_from_dense(A), B)
    want = np.zeros((5, 3), np.float32)
    for r in range(5):
        for n in range(3):
            acc = np.float32(0)
            for c in range(40):
                if A[r, c] != 0:
                    acc = np.float32(acc + np.float32(A[r, c] * B[c, n]))
            want[r, n] = acc
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
