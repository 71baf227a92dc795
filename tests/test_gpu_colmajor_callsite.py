"""The reference keeps its device matrices column-major (to_gpu transposes, source/basicOps.cu:14-33) and hands
cublasSgemm the row counts as leading dimensions (source/clusterNet.cpp:459-461).  A maintainer who puts libcnhip under
that call site keeps the column-major buffers and swaps the operands:

    cn_gemm_f32(T2 == T, T1 == T, n, m, k, B->data, B->rows, A->data, A->rows, out->data, out->rows, stream)

This file stores A, B and out the way the reference's to_gpu does, issues exactly that call through the C-ABI for all
four (T1, T2), and compares the column-major result with the reference's known answers
(tests/clusterNet_test.cu:22-23,72-75,111-119,125-128,161-164) and with the CPU checker on ragged random cases."""
import ctypes

import numpy as np
import pytest

import oracle
from util import gemm_errors, gemm_tolerance

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


class ColMajorMatrix:
    """What the reference's Matrix is on the device: rows, cols and a column-major payload (element (i, j) at
    data[j * rows + i])."""

    def __init__(self, host_row_major, dev):
        import torch
        a = np.asarray(host_row_major, np.float32)
        self.rows, self.cols = a.shape
        # to_gpu: host row-major -> device column-major
        self.data = torch.from_numpy(np.ascontiguousarray(a.T).reshape(-1)).to(dev)

    def to_host(self):
        return self.data.cpu().numpy().reshape(self.cols, self.rows).T.copy()


def reference_call_site(A, B, out, T1, T2):
    """ClusterNet::dot(A, B, out, T1, T2) (source/clusterNet.cpp:404-487) with cublasSgemm replaced: the shape rule of
    checkMatrixOperation, then the operand swap."""
    import torch
    import clusternet_amd as cn
    a_rows, a_cols = (A.cols, A.rows) if T1 else (A.rows, A.cols)
    b_rows, b_cols = (B.cols, B.rows) if T2 else (B.rows, B.cols)
    assert a_cols == b_rows and a_rows == out.rows and b_cols == out.cols, "Matrix *size error"
    m, n, k = out.rows, out.cols, a_cols
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    status = cn.lib().cn_gemm_f32(int(T2), int(T1), n, m, k, B.data.data_ptr(), B.rows, A.data.data_ptr(), A.rows,
                                  out.data.data_ptr(), out.rows, stream)
    assert status == 0, status


def _run(dev, a, b, T1, T2):
    A, B = ColMajorMatrix(a, dev), ColMajorMatrix(b, dev)
    m = a.shape[1] if T1 else a.shape[0]
    n = b.shape[0] if T2 else b.shape[1]
    out = ColMajorMatrix(np.full((m, n), np.nan, np.float32), dev)
    reference_call_site(A, B, out, T1, T2)
    return out.to_host()


def test_reference_known_answers_through_the_swapped_call(dev):
    m1 = np.array([[0, 2, 3], [0, 0.83, 59.1387]], np.float32)
    m2 = np.array([[17, 0], [3, 4], [0, 0]], np.float32)
    f = lambda r: np.array(r, np.float32)
    np.testing.assert_allclose(_run(dev, m1, m2, False, False), f([[6, 8], [2.49, 3.32]]), rtol=1e-6)          # dot
    np.testing.assert_allclose(_run(dev, m1, m1, True, False),                                                   # Tdot
                               f([[0, 0, 0], [0, 4.6889, 55.085117], [0, 55.085117, 3506.385742]]), rtol=1e-6)
    np.testing.assert_allclose(_run(dev, m2, m2, True, False), f([[298, 12], [12, 16]]), rtol=1e-6)
    np.testing.assert_allclose(_run(dev, m1, m1, False, True), f([[13, 179.0761], [179.0761, 3498.074463]]), rtol=1e-6)  # dotT
    # both transposed: the reference holds no literal for it; (m2^T m1^T) = (m1 m2)^T
    np.testing.assert_allclose(_run(dev, m2, m1, True, True), f([[6, 8], [2.49, 3.32]]).T, rtol=1e-6)


@pytest.mark.parametrize("T1,T2", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("m,n,k", [(37, 129, 515), (128, 1024, 784), (130, 70, 33)])
def test_ragged_random_against_the_checker(dev, T1, T2, m, n, k):
    rng = np.random.default_rng(1000 * m + 10 * n + k + 2 * T1 + T2)
    a = rng.uniform(0, 1, (k, m) if T1 else (m, k)).astype(np.float32)
    b = rng.normal(0, 0.05, (n, k) if T2 else (k, n)).astype(np.float32)
    got = _run(dev, a, b, T1, T2)
    ref, refabs = oracle.gemm_with_abs(a, b, T1, T2)
    e1, e2 = gemm_errors(got, ref, refabs)
    assert got.shape == (m, n) and e1 <= gemm_tolerance(k) and e2 <= gemm_tolerance(k), (e1, e2)


def test_shape_rule_rejects_what_the_reference_rejects(dev):
    a, b = np.zeros((4, 5), np.float32), np.zeros((4, 6), np.float32)
    with pytest.raises(AssertionError):
        _run(dev, a, b, False, False)
    assert _run(dev, a, b, True, False).shape == (5, 6)
