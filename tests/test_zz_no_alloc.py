"""cn_gemm_f32_noalloc, the product for callers that cannot allocate device memory: its K-chunk partial sums live
in an array that is part of the library's device image.  Checked through the C-ABI against cn_gemm_f32 bit for bit
(both split K the same way) and against the CPU checker within the GEMM tolerance, on two calls in a row that
share the array, the second on a smaller product, so that what the first call left behind would show."""
import ctypes

import numpy as np
import pytest

import oracle
from util import gemm_errors, gemm_tolerance

pytestmark = pytest.mark.gpu


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _pair(cn, dev, rng, M, N, K, ta, tb):
    import torch
    A = rng.uniform(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
    B = rng.uniform(-0.05, 0.05, (N, K) if tb else (K, N)).astype(np.float32)
    At, Bt = _t(A, dev), _t(B, dev)
    # the entry point under test goes first: in a fresh process its first call is the library's first call
    got = torch.full((M, N), float("nan"), device=dev)
    cn.gemm(At, Bt, ta, tb, out=got, noalloc=True)
    want = cn.gemm(At, Bt, ta, tb)
    return A, B, want.cpu().numpy(), got.cpu().numpy()


def test_two_calls_in_a_row_match_the_allocating_entry_point():
    import torch
    import clusternet_amd as cn
    dev = torch.device("cuda:0")
    L = cn.lib()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rng = np.random.default_rng(2024)
    # the first product splits K into many chunks (its partial sums fill most of the array's first megabytes),
    # the second is smaller in every dimension and splits K as well
    for (M, N, K, ta, tb) in ((128, 4096, 8192, False, False), (96, 1000, 1111, False, True), (64, 520, 3000, True, False)):
        out = (ctypes.c_int64 * 8)()
        L.cn_host_plan_gemm(M, N, K, cus, 1 << 30, 0, out)
        assert out[3] > 1, "the case is meant to split K (%d chunks planned)" % out[3]
        A, B, want, got = _pair(cn, dev, rng, M, N, K, ta, tb)
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), (M, N, K, ta, tb)
        ref, refabs = oracle.gemm_with_abs(A, B, ta, tb)
        e1, e2 = gemm_errors(got, ref, refabs)
        assert e1 <= gemm_tolerance(K) and e2 <= gemm_tolerance(K), (M, N, K, e1, e2)


def test_a_product_beyond_the_array_is_refused():
    import torch
    import clusternet_amd as cn
    from clusternet_amd._lib import CnError
    dev = torch.device("cuda:0")
    # 128 x 40000 x 100000 is cut into 13 chunks: 266 MB of partial sums against the array's 64 MiB
    M, N, K = 128, 40000, 100000
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = (ctypes.c_int64 * 8)()
    cn.lib().cn_host_plan_gemm(M, N, K, cus, 1 << 30, 0, out)
    assert out[3] * M * N * 4 > (64 << 20)
    A = torch.zeros((M, K), device=dev)
    B = torch.empty((K, N), device=dev)  # never read: the call is refused before any launch
    C = torch.full((M, N), 7.0, device=dev)
    with pytest.raises(CnError) as info:
        cn.gemm(A, B, out=C, noalloc=True)
    assert info.value.status == 5 and "partial sums" in str(info.value)
    assert float(C.min()) == 7.0 and float(C.max()) == 7.0
