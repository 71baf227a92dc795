"""Unsplit products of many short tiles (the weight gradient of a wide layer: K is the batch) run on workgroups that stay
and draw their tiles from a counter.  The form must give the bits of the form that starts a workgroup per tile, for every transposition,
ragged borders in M and N, one to many K stages, with and without the maximum; and both must agree with the CPU
checker.  Reference semantics: source/clusterNet.cpp:246-291,404-461 (Tdot / dotT / dot, alpha 1, beta 0)."""
import ctypes

import numpy as np
import pytest

import oracle
from util import gemm_errors, gemm_tolerance

pytestmark = pytest.mark.gpu

PERSISTENT, TILED = 4, 1


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


def _took(cn):
    splits = ctypes.c_int(0)
    return cn.lib().cn_host_last_gemm_kernel(ctypes.byref(splits)), splits.value


def _operands(rng, M, N, K, ta, tb, dev):
    import torch
    A = rng.uniform(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
    B = rng.normal(0, 0.01, (N, K) if tb else (K, N)).astype(np.float32)
    return A, B, torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)


# 128 x 256 tiles: at least three rounds of 512 resident workgroups
SHAPES = [(12800, 4096, 128), (12836, 4096, 64), (12800, 4000, 16), (6500, 8192, 48), (25000, 2048, 128), (3100, 16640, 32)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("ta,tb", [(True, False), (False, False), (False, True), (True, True)])
@pytest.mark.parametrize("tile_n", [256, 128])
def test_same_bits_as_a_workgroup_per_tile(dev, M, N, K, ta, tb, tile_n):
    import torch
    import clusternet_amd as cn
    if tile_n == 128 and K % 32:
        pytest.skip("a stage of the 128-wide tile is 32 deep: this K is not whole stages")
    rng = np.random.default_rng(M + N + K + 2 * ta + tb)
    A, B, At, Bt = _operands(rng, M, N, K, ta, tb, dev)
    L = cn.lib()
    L.cn_host_force_gemm_tile_n(tile_n)
    try:
        got = torch.full((M, N), float("nan"), device=dev)
        cn.gemm(At, Bt, ta, tb, out=got)
        assert _took(cn) == (PERSISTENT, 1)
        L.cn_host_gemm_persistent(0)
        want = torch.full((M, N), float("nan"), device=dev)
        cn.gemm(At, Bt, ta, tb, out=want)
        assert _took(cn) == (TILED, 1)
    finally:
        L.cn_host_gemm_persistent(1)
        L.cn_host_force_gemm_tile_n(0)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    # against the checker on a sample of rows that includes the first and last tile rows
    rows = np.unique(np.concatenate([np.arange(0, 3), np.arange(M - 3, M), rng.integers(0, M, 40)]))
    As = A[:, rows] if ta else A[rows]
    Cref, Cabs = oracle.gemm_with_abs(np.ascontiguousarray(As), B, ta, tb)
    e1, e2 = gemm_errors(got[torch.from_numpy(rows).to(dev)].cpu().numpy(), Cref, Cabs)
    assert e1 <= gemm_tolerance(K) and e2 <= gemm_tolerance(K), (e1, e2)


def test_with_the_maximum_and_a_padded_result(dev):
    """cn_gemm_f32_absmax on the persistent form: max|C| over all tiles, bit-equal to the abs-max of the stored result; the
    result has a leading dimension larger than N and the padding is left alone."""
    import torch
    import clusternet_amd as cn
    M, N, K = 12836, 4000, 128
    rng = np.random.default_rng(5)
    A, B, At, Bt = _operands(rng, M, N, K, True, False, dev)
    buf = torch.full((M, N + 8), -7.0, device=dev)
    out = buf[:, :N]
    mx = torch.zeros(1, device=dev)
    L = cn.lib()
    L.cn_host_force_gemm_tile_n(256)
    try:
        cn.gemm(At, Bt, True, False, out=out, absmax_out=mx)
        assert _took(cn) == (PERSISTENT, 1)
    finally:
        L.cn_host_force_gemm_tile_n(0)
    assert bool((buf[:, N:] == -7.0).all())
    assert float(mx.cpu()[0]) == float(out.abs().max().cpu())
    plain = cn.gemm(At, Bt, True, False)
    assert torch.equal(plain.view(torch.int32), out.contiguous().view(torch.int32))


def test_entry_point_that_allocates_nothing_and_an_unaligned_result(dev):
    """cn_gemm_f32_noalloc takes the same persistent form once the library is initialised (it borrows a counter, it does not
    create a context).  Same bits; here also with a result whose rows start at odd addresses (the write-out is 4-byte stores)."""
    import torch
    import clusternet_amd as cn
    M, N, K = 12836, 4096, 64
    rng = np.random.default_rng(6)
    A, B, At, Bt = _operands(rng, M, N, K, True, False, dev)
    want = cn.gemm(At, Bt, True, False)
    assert _took(cn) == (PERSISTENT, 1)
    buf = torch.full((M, N + 3), -7.0, device=dev)
    out = buf[:, 1:N + 1]
    cn.gemm(At, Bt, True, False, out=out, noalloc=True)
    assert _took(cn) == (PERSISTENT, 1)
    assert torch.equal(out.contiguous().view(torch.int32), want.view(torch.int32))
    assert bool((buf[:, 0] == -7.0).all()) and bool((buf[:, N + 1:] == -7.0).all())
    assert cn.lib().cn_host_tile_counters_in_use() == 0


def test_planner_takes_it_for_the_weight_gradient_shape(dev):
    """A slice of the training configuration's first-layer gradient (Tdot, K = 128, 8192 columns): the library's own plan
    is unsplit 128 x 256 tiles on persistent workgroups."""
    import clusternet_amd as cn
    rng = np.random.default_rng(9)
    A, B, At, Bt = _operands(rng, 20000, 8192, 128, True, False, dev)
    cn.gemm(At, Bt, True, False)
    assert _took(cn) == (PERSISTENT, 1)
    # operands that do not allow 16-byte loads, or a K that is not whole stages, keep the workgroup per tile
    cn.gemm(At, Bt[:, 1:], True, False)
    assert _took(cn)[0] == TILED
    cn.gemm(At[:120], Bt[:120], True, False)
    assert _took(cn)[0] == TILED
    # long tiles keep the workgroup per tile too (nothing to gain there)
    A2, B2, A2t, B2t = _operands(rng, 8192, 8192, 1024, False, False, dev)
    cn.gemm(A2t, B2t, False, False)
    assert _took(cn)[0] == TILED
    assert cn.lib().cn_host_tile_counters_in_use() == 0
