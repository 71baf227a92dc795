"""Kernels that draw their tiles from a counter (the streaming passes on tensors beyond the cache, the persistent
product) on several streams and under graph capture.  A counter is tied to the stream that first asked for one, so the
kernels on a counter are ordered by their stream; a call that is being captured gets no counter and takes the form that
walks its tiles in a fixed pattern, so a graph never carries a counter into its replays.  Overlapping work on two
streams, and graph replays beside eager calls, must give the bits of the same calls made one after the other, and every
counter must be back at zero afterwards.  (The reference is single-stream, source/clusterNet.cpp:406-407; this is the
library's own contract for callers that are not.)"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N = (1 << 26) + 4096 + 128  # beyond the size from which the passes draw their tiles; not a whole number of tiles


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


def test_two_streams_overlap(dev):
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    g = torch.Generator(device=dev).manual_seed(3)
    w0 = torch.rand(N, device=dev, generator=g)
    grad = torch.rand(N, device=dev, generator=g) - 0.5
    # one after the other on the current stream
    want_a, want_b = w0.clone(), torch.empty(N, device=dev)
    for _ in range(3):
        L.sgd_update(want_a, grad, 0.25)
    L.fill(want_b, 3.5)
    prec = float(cn.absmax(grad).cpu()[0])
    want_codes = cn.compression_8bit(grad, prec)
    torch.cuda.synchronize()
    # the same work on two streams at once, repeatedly
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    for rep in range(3):
        got_a, got_b = w0.clone(), torch.zeros(N, device=dev)
        got_codes = torch.zeros(N, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        with torch.cuda.stream(sa):
            for _ in range(3):
                L.sgd_update(got_a, grad, 0.25)
        with torch.cuda.stream(sb):
            L.fill(got_b, 3.5)
            cn.compression_8bit(grad, prec, got_codes)
        torch.cuda.synchronize()
        assert torch.equal(got_a.view(torch.int32), want_a.view(torch.int32)), rep
        assert torch.equal(got_b, want_b) and torch.equal(got_codes, want_codes), rep
    assert cn.lib().cn_host_tile_counters_in_use() == 0


def test_graph_replay_beside_eager_calls(dev):
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    g = torch.Generator(device=dev).manual_seed(4)
    w0 = torch.rand(N, device=dev, generator=g)
    grad = torch.rand(N, device=dev, generator=g) - 0.5
    want = w0.clone()
    L.sgd_update(want, grad, 0.5)
    torch.cuda.synchronize()
    captured_w = w0.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        L.sgd_update(captured_w, grad, 0.5)   # captured: the form that does not draw
    side = torch.cuda.Stream()
    for rep in range(4):
        captured_w.copy_(w0)
        eager_w = w0.clone()
        torch.cuda.synchronize()
        graph.replay()                        # on the current stream
        with torch.cuda.stream(side):
            L.sgd_update(eager_w, grad, 0.5)  # eager, drawing, at the same time
        torch.cuda.synchronize()
        assert torch.equal(captured_w.view(torch.int32), want.view(torch.int32)), rep
        assert torch.equal(eager_w.view(torch.int32), want.view(torch.int32)), rep
    assert cn.lib().cn_host_tile_counters_in_use() == 0


def test_persistent_product_under_capture_and_on_a_side_stream(dev):
    """The persistent product draws its tiles; captured, it runs as a workgroup per tile.  Same bits either way."""
    import ctypes
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(12)
    M, Nc, K = 20000, 8192, 128
    A = torch.from_numpy(rng.uniform(0, 1, (K, M)).astype(np.float32)).to(dev)
    B = torch.from_numpy(rng.normal(0, 0.01, (K, Nc)).astype(np.float32)).to(dev)
    want = cn.gemm(A, B, True, False)
    splits = ctypes.c_int(0)
    assert cn.lib().cn_host_last_gemm_kernel(ctypes.byref(splits)) == 4
    torch.cuda.synchronize()
    out = torch.zeros((M, Nc), device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cn.gemm(A, B, True, False, out=out)
    assert cn.lib().cn_host_last_gemm_kernel(ctypes.byref(splits)) == 1
    side = torch.cuda.Stream()
    for rep in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        with torch.cuda.stream(side):
            eager = cn.gemm(A, B, True, False)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), want.view(torch.int32)), rep
        assert torch.equal(eager.view(torch.int32), want.view(torch.int32)), rep
    assert cn.lib().cn_host_tile_counters_in_use() == 0
