"""cn_gemm_c8c8_add through the C-ABI: C += decodeA(A) decodeB(B) with both operands as 8-bit codes, the product of
ClusterNet::dot8bit / dot8bit_shared (source/clusterNet.cpp:1409-1431, kDot8bit source/clusterKernels.cu:1717-1762).
Checked against the CPU restatement of kDot8bit: the sums run in a different order (matrix instructions here, one k after
the other there), so the general case is held to the tolerance of the fp32 products (1e-4 of sum_k |a||b| + |out| up to
K = 4096); rows of A with a single code that decodes to non-zero, where no order exists, are held bit for bit."""
import ctypes

import numpy as np
import pytest

import oracle
from util import gemm_tolerance

pytestmark = pytest.mark.gpu
PA, PB = 0.75, 2.5


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("M,K,N", [(37, 150, 29), (128, 1000, 257), (33, 7, 65), (1, 1, 1), (64, 256, 64), (100, 2051, 40),
                                   (300, 96, 300), (32, 4096, 32)])
def test_against_the_restatement_of_kDot8bit(dev, M, K, N):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(M * 1000 + K + N)
    A = rng.integers(0, 256, (M, K)).astype(np.uint8)
    B = rng.integers(0, 256, (K, N)).astype(np.uint8)
    out0 = rng.normal(0, 0.5, (M, N)).astype(np.float32)
    want, mag = oracle.dot8bit(A, B, PA, PB, out0)
    out = _t(out0, dev)
    L.gemm_c8c8_add(_t(A, dev), _t(B, dev), PA, PB, out)
    got = out.cpu().numpy()
    err = float((np.abs(got.astype(np.float64) - want) / (mag + np.abs(out0))).max())
    assert err <= gemm_tolerance(K), (M, K, N, err)
    # a second call adds the product again
    L.gemm_c8c8_add(_t(A, dev), _t(B, dev), PA, PB, out)
    want2, _ = oracle.dot8bit(A, B, PA, PB, want)
    err2 = float((np.abs(out.cpu().numpy().astype(np.float64) - want2) / (2 * mag + np.abs(out0))).max())
    assert err2 <= gemm_tolerance(K), (M, K, N, err2)


@pytest.mark.parametrize("K,N", [(40, 33), (300, 70), (9, 5)])
def test_rows_with_one_nonzero_code_are_exact(dev, K, N):
    """Row m of A holds one code that decodes to non-zero (every special code and ordinary ones take a turn) among codes
    126 / 254, which decode to +0 / -0: each output is one fp32 product added to out once."""
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(K + N)
    B = rng.integers(0, 256, (K, N)).astype(np.uint8)
    B[0, :4] = (126, 127, 254, 255)
    A = np.where(rng.random((K, K)) < 0.5, 126, 254).astype(np.uint8)
    picks = np.array([127, 255, 3, 200, 125, 253] * (K // 6 + 1))[:K].astype(np.uint8)
    A[np.arange(K), np.arange(K)] = picks
    out0 = rng.normal(size=(K, N)).astype(np.float32)
    want, _ = oracle.dot8bit(A, B, PA, PB, out0)
    out = _t(out0, dev)
    L.gemm_c8c8_add(_t(A, dev), _t(B, dev), PA, PB, out)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_strided_and_unaligned_operands(dev):
    """Views with leading dimensions beyond the row length and a first operand that starts on an odd byte (its codes are
    then read one by one)."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(77)
    M, K, N = 45, 130, 50
    Abig = rng.integers(0, 256, (M, K + 7)).astype(np.uint8)
    Bbig = rng.integers(0, 256, (K, N + 14)).astype(np.uint8)
    obig = rng.normal(size=(M, N + 6)).astype(np.float32)
    A, B, out0 = Abig[:, 3:3 + K], Bbig[:, 5:5 + N], obig[:, 2:2 + N]
    want, mag = oracle.dot8bit(A, B, PA, PB, out0)
    od = _t(obig, dev)
    L.gemm_c8c8_add(_t(Abig, dev)[:, 3:3 + K], _t(Bbig, dev)[:, 5:5 + N], PA, PB, od[:, 2:2 + N])
    got = od.cpu().numpy()
    assert float((np.abs(got[:, 2:2 + N].astype(np.float64) - want) / (mag + np.abs(out0))).max()) <= gemm_tolerance(K)
    assert np.array_equal(got[:, :2], obig[:, :2]) and np.array_equal(got[:, 2 + N:], obig[:, 2 + N:])


def test_errors_and_empty_products(dev):
    import torch
    import clusternet_amd as cn
    lib = cn.lib()
    A = torch.zeros((4, 8), dtype=torch.uint8, device=dev)
    B = torch.zeros((8, 6), dtype=torch.uint8, device=dev)
    out = torch.full((4, 6), 1.25, device=dev)
    f = ctypes.c_float
    assert lib.cn_gemm_c8c8_add(4, 6, 8, A.data_ptr(), 7, B.data_ptr(), 6, f(1), f(1), out.data_ptr(), 6, None) == 2
    assert b"gemm_c8c8_add" in ctypes.c_char_p(lib.cn_last_error()).value
    assert lib.cn_gemm_c8c8_add(4, 6, 8, A.data_ptr(), 8, B.data_ptr(), 5, f(1), f(1), out.data_ptr(), 6, None) == 2
    assert lib.cn_gemm_c8c8_add(4, 6, 8, A.data_ptr(), 8, B.data_ptr(), 6, f(1), f(1), out.data_ptr(), 5, None) == 2
    assert lib.cn_gemm_c8c8_add(-1, 6, 8, A.data_ptr(), 8, B.data_ptr(), 6, f(1), f(1), out.data_ptr(), 6, None) == 2
    assert lib.cn_gemm_c8c8_add(4, 6, 8, None, 8, B.data_ptr(), 6, f(1), f(1), out.data_ptr(), 6, None) != 0
    for M, N, K in ((0, 6, 8), (4, 0, 8), (4, 6, 0)):   # nothing to add
        assert lib.cn_gemm_c8c8_add(M, N, K, A.data_ptr(), 8, B.data_ptr(), 6, f(1), f(1), out.data_ptr(), 6, None) == 0
    torch.cuda.synchronize()
    assert float(out.min()) == 1.25 and float(out.max()) == 1.25
