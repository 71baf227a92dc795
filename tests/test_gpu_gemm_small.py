"""Products too small to fill the chip with tiles (cn_gemm_small.hip), through the C-ABI, against the CPU checker.
Tolerance as for the tiled kernel: max relative error 1e-4 for K <= 4096, measured both against max|C_ref| and
element-wise against sum_k |a||b|."""
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


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _check(cn, dev, A, B, ta=False, tb=False):
    got = cn.gemm(_t(A, dev), _t(B, dev), ta, tb).cpu().numpy()
    Cref, Cabs = oracle.gemm_with_abs(A, B, ta, tb)
    K = A.shape[0] if ta else A.shape[1]
    e1, e2 = gemm_errors(got, Cref, Cabs)
    tol = gemm_tolerance(K)
    assert e1 <= tol and e2 <= tol, (A.shape, B.shape, ta, tb, e1, e2, tol)
    return got


@pytest.mark.parametrize("shape", [(128, 1024, 784), (128, 784, 1024), (784, 1024, 128), (33, 65, 64), (100, 1000, 800),
                                   (17, 19, 32), (31, 500, 40), (128, 10, 1024), (250, 260, 1000), (1, 1, 48),
                                   (512, 1024, 512), (90, 2047, 1024)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_small_products_in_one_launch(dev, shape, ta, tb):
    """Products too small to fill the chip with tiles take a kernel of their own (a workgroup per 32 x 32 or 16 x 16
    block of the result, K split among its wavefronts): against the CPU checker, with ragged edges in M and N, K in
    groups of 8 that are and are not groups of 16, every transposition, an output with a leading dimension of its own,
    the maximum of the result, and the same bits from the entry point that allocates nothing.  With the hook off the
    tiled kernel serves the same shapes to the same tolerance."""
    import torch
    import clusternet_amd as cn
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    A = rng.normal(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
    B = rng.normal(0, 1, (N, K) if tb else (K, N)).astype(np.float32)
    got = _check(cn, dev, A, B, ta, tb)
    At, Bt = _t(A, dev), _t(B, dev)
    big = torch.full((M, N + 9), float("nan"), device=dev)
    amax = torch.zeros(1, device=dev)
    cn.gemm(At, Bt, ta, tb, out=big[:, 5:5 + N], absmax_out=amax)
    assert np.array_equal(big[:, 5:5 + N].cpu().numpy().view(np.uint32), got.view(np.uint32))
    assert bool(torch.isnan(big[:, :5]).all()) and bool(torch.isnan(big[:, 5 + N:]).all())
    assert float(amax.cpu()[0]) == float(np.abs(got).max())
    out = torch.empty((M, N), device=dev)
    cn.gemm(At, Bt, ta, tb, out=out, noalloc=True)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), got.view(np.uint32))
    cn.lib().cn_host_gemm_small(0)
    try:
        _check(cn, dev, A, B, ta, tb)
    finally:
        cn.lib().cn_host_gemm_small(1)
