"""cn_gemm_f32_noalloc, the product for callers that cannot allocate device memory: its K-chunk partial sums live
in an array that is part of the library's device image.  Checked through the C-ABI against cn_gemm_f32 bit for bit
(both split K the same way) and against the CPU checker within the GEMM tolerance, on calls in a row that share the
array, the later ones on smaller products, so that what an earlier call left behind would show.  That the call
allocates nothing is held two ways: free device memory is the same before and after, and a split-K call is captured
into a HIP graph (an allocation inside a capture fails it) and replayed against the eager bits.  The path on which the
entry point is the process's very first call into the library (no cn_init before it) runs in a child process, because
in this process other tests have long initialised the library."""
import ctypes
import os
import subprocess
import sys

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
    got = torch.full((M, N), float("nan"), device=dev)
    free_before = torch.cuda.mem_get_info()[0]
    cn.gemm(At, Bt, ta, tb, out=got, noalloc=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
    took = _took(cn)
    want = cn.gemm(At, Bt, ta, tb)
    assert _took(cn) == took, "the two entry points took different kernels"
    return A, B, want.cpu().numpy(), got.cpu().numpy(), took


TILED = 1


def _took(cn):
    splits = ctypes.c_int(0)
    return cn.lib().cn_host_last_gemm_kernel(ctypes.byref(splits)), splits.value


def test_two_calls_in_a_row_match_the_allocating_entry_point():
    import torch
    import clusternet_amd as cn
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(2024)
    # the first product splits K into many chunks (its partial sums fill most of the array's first megabytes), the
    # others are smaller in every dimension and split K as well; none of them is small enough for the one-launch
    # kernel, which has no partial sums (the third: K is not a multiple of 8)
    for (M, N, K, ta, tb) in ((128, 4096, 8192, False, False), (96, 1000, 1111, False, True), (64, 520, 3001, True, False)):
        A, B, want, got, took = _pair(cn, dev, rng, M, N, K, ta, tb)
        assert took[0] == TILED and took[1] > 1, "the case is meant to run on the tiled kernel with K split, it took %r" % (took,)
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


def test_a_split_product_can_be_captured_and_replayed():
    """Inside a stream capture hipMalloc is an error, so a capture that succeeds has allocated nothing.  The graph is
    replayed several times with eager products (which overwrite the partial-sum array) in between, and every replay
    must give the eager bits."""
    import torch
    import clusternet_amd as cn
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(77)
    M, N, K = 128, 2048, 8192
    A = _t(rng.uniform(0, 1, (M, K)).astype(np.float32), dev)
    B = _t(rng.uniform(-0.05, 0.05, (K, N)).astype(np.float32), dev)
    other_a = _t(rng.uniform(0, 1, (96, 4096)).astype(np.float32), dev)
    other_b = _t(rng.uniform(-1, 1, (4096, 1000)).astype(np.float32), dev)
    eager = torch.empty((M, N), device=dev)
    cn.gemm(A, B, out=eager, noalloc=True)  # also: the array's address is known before the capture starts
    assert _took(cn)[0] == TILED and _took(cn)[1] > 1
    torch.cuda.synchronize()
    out = torch.zeros((M, N), device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cn.gemm(A, B, out=out, noalloc=True)
    for replay in range(4):
        out.fill_(float("nan"))
        cn.gemm(other_a, other_b, noalloc=True)  # eager work on the same array between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), eager.view(torch.int32)), "replay %d differs from the eager result" % replay


_CHILD = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
import clusternet_amd as cn
import oracle
dev = torch.device("cuda:0")
rng = np.random.default_rng(3)
A = rng.uniform(0, 1, (128, 4096)).astype(np.float32)
B = rng.uniform(-0.05, 0.05, (4096, 1024)).astype(np.float32)
At, Bt = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
got = torch.full((128, 1024), float("nan"), device=dev)
cn.gemm(At, Bt, out=got, noalloc=True)          # the library's first call in this process: no cn_init before it
want = cn.gemm(At, Bt)                           # initialises the context; same plan, same bits
assert torch.equal(got.view(torch.int32), want.view(torch.int32)), "differs from cn_gemm_f32"
ref, refabs = oracle.gemm_with_abs(A, B)
err = float((np.abs(got.cpu().numpy() - ref) / np.maximum(refabs, 1e-300)).max())
assert err <= 1e-4, err
print("first call ok")
"""


def test_first_call_of_a_process_without_cn_init():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", _CHILD, root], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=280)
    assert proc.returncode == 0 and "first call ok" in proc.stdout, proc.stdout[-2000:]
