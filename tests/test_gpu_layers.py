"""The small kernels around the path and one maxout training step composed from the path's
operators, compared with the CPU checker."""
import numpy as np
import pytest

import oracle
from util import gemm_tolerance

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


def test_helpers_match_checker(dev):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(0)
    A = rng.normal(0, 1, (133, 1736)).astype(np.float32)
    v = rng.normal(0, 1, 1736).astype(np.float32)
    assert np.array_equal(L.add_row_vector(_t(A, dev), _t(v, dev)).cpu().numpy(), oracle.add_row_vector(A, v))
    assert np.array_equal(L.transpose(_t(A, dev)).cpu().numpy(), A.T)
    for pool in (2, 4, 8):
        out, arg = L.maxout(_t(A, dev), pool)
        wo, wa = oracle.maxout(A, pool)
        assert np.array_equal(out.cpu().numpy(), wo) and np.array_equal(arg.cpu().numpy(), wa)
        err = rng.normal(0, 1, wo.shape).astype(np.float32)
        g = L.expand_to_maxout_grad(_t(err, dev), arg, pool).cpu().numpy()
        assert np.array_equal(g, oracle.expand_to_maxout_grad(err, wa, pool))
    s = L.softmax(_t(A[:, :10].copy(), dev)).cpu().numpy()
    np.testing.assert_allclose(s, oracle.softmax(A[:, :10].copy()), rtol=2e-6, atol=1e-9)
    assert np.allclose(L.softmax(_t(np.zeros((7, 10), np.float32), dev)).cpu().numpy(), 0.1)
    B = rng.normal(0, 1, A.shape).astype(np.float32)
    assert np.array_equal(L.sub(_t(A, dev), _t(B, dev)).cpu().numpy(), A - B)
    w = _t(A, dev)
    L.sgd_update(w, _t(B, dev), 0.125)
    assert np.array_equal(w.cpu().numpy(), A - np.float32(0.125) * B)
    assert abs(float(L.reduce_sum(_t(A, dev)).cpu()[0]) - A.astype(np.float64).sum()) < 1e-2
    assert float(L.reduce_max(_t(A, dev)).cpu()[0]) == A.max()
    assert float(L.reduce_max(_t(-np.abs(A) - 2, dev)).cpu()[0]) == -1.0
    # ties in maxout: the first maximum wins
    T = np.array([[1, 1, 0, 2, 2, 2]], np.float32)
    out, arg = L.maxout(_t(T, dev), 3)
    assert arg.cpu().numpy().tolist() == [[0.0, 3.0]]


def test_flat_passes_on_ragged_sizes_and_unaligned_starts(dev):
    """sub and the plain update on 16-byte vectors where the arrays allow it and element by element where they do
    not: every size around a vector and a tile boundary, starts that are and are not 16-byte aligned, in place."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(4)
    A = rng.normal(0, 1, 70_000).astype(np.float32)
    B = rng.normal(0, 1, 70_000).astype(np.float32)
    At, Bt = _t(A, dev), _t(B, dev)
    for n in (1, 3, 4, 5, 1023, 1024, 4095, 4096, 4097, 16_385, 65_537):
        for oa, ob in ((0, 0), (4, 8), (1, 0), (0, 3), (2, 2)):
            got = L.sub(At[oa:oa + n], Bt[ob:ob + n]).cpu().numpy()
            assert np.array_equal(got, A[oa:oa + n] - B[ob:ob + n]), (n, oa, ob)
            w = At.clone()
            L.sgd_update(w[oa:oa + n], Bt[ob:ob + n], 0.375)
            want = A.copy()
            want[oa:oa + n] = A[oa:oa + n] - np.float32(0.375) * B[ob:ob + n]
            assert np.array_equal(w.cpu().numpy(), want), (n, oa, ob)


@pytest.mark.parametrize("rows,cols,pool", [(128, 8192, 2), (7, 12, 3), (33, 260, 4), (1, 2, 1), (5, 64, 64)])
def test_bias_and_maxout_in_one_pass_equal_the_two_kernels(dev, rows, cols, pool):
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(rows + cols)
    A = rng.normal(0, 1, (rows, cols + 3)).astype(np.float32)
    A[:, 1::2] = A[:, 0:-1:2][:, :A[:, 1::2].shape[1]]            # many ties between pool neighbours
    v = rng.normal(0, 0.1, cols).astype(np.float32)
    v[1::2] = v[0::2][:v[1::2].size]
    Ad = _t(A, dev)[:, :cols]                                        # leading dimension above the width
    out, arg = L.bias_maxout(Ad, _t(v, dev), pool)
    want_out, want_arg = L.maxout(L.add_row_vector(Ad.contiguous(), _t(v, dev)), pool)
    assert torch.equal(out.view(torch.int32), want_out.view(torch.int32)) and torch.equal(arg, want_arg)
    z = oracle.add_row_vector(np.ascontiguousarray(A[:, :cols]), v)
    h, a = oracle.maxout(z, pool)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), h.view(np.uint32)) and np.array_equal(arg.cpu().numpy(), a)


@pytest.mark.parametrize("M,N,K,pool", [(128, 8192, 4096, 2), (128, 1024, 784, 2), (32, 512, 4096, 4), (7, 12, 33, 3),
                                        (300, 260, 64, 2), (1, 2, 1, 1), (64, 4096, 100000, 2)])
def test_product_with_bias_and_maxout_equals_the_three_calls(dev, M, N, K, pool):
    """dot, add_row_vector and maxout as one call: where the product is summed over chunks of K the bias and
    the maxout ride on that sum, elsewhere the product passes through the workspace; the same bits either
    way, on every tile geometry."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev).manual_seed(M + N + K)
    A = torch.randn((M, K), device=dev, generator=gen)
    B = torch.randn((K, N), device=dev, generator=gen) * 0.05
    v = torch.randn(N, device=dev, generator=gen) * 0.1
    for force in (0, 32, 64, 128, 256):
        cn.lib().cn_host_force_gemm_tile_n(force)
        try:
            out, arg = L.dot_bias_maxout(A, B, v, pool)
            want_out, want_arg = L.maxout(L.add_row_vector(L.dot(A, B), v), pool)
        finally:
            cn.lib().cn_host_force_gemm_tile_n(0)
        assert torch.equal(out.view(torch.int32), want_out.view(torch.int32)), force
        assert torch.equal(arg, want_arg), force
    with pytest.raises(L.CnError):
        L.dot_bias_maxout(A, B, v[:-1] if N > 1 else torch.empty(0, device=dev), pool)
    assert cn.lib().cn_gemm_f32_bias_maxout(0, 0, 4, 6, 4, None, 4, None, 6, None, 4, None, None, None) == 2  # 6 % 4
    assert cn.lib().cn_gemm_f32_bias_maxout(0, 0, 4, 6, 4, None, 4, None, 6, None, 2, None, None, None) == 1  # NULL


@pytest.mark.parametrize("M,N,K,pool", [(128, 4096, 8192, 2), (128, 4096, 10, 2), (7, 5, 33, 3), (300, 130, 64, 4),
                                        (1, 1, 1, 1), (32, 512, 4096, 2)])
def test_product_with_expansion_equals_the_two_calls(dev, M, N, K, pool):
    """dotT and expand_to_maxout_grad as one call (the expansion rides on the chunk sum, or follows the product
    through the workspace): the same bits as the two calls on every tile geometry."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev).manual_seed(M * 3 + N + K)
    E = torch.randn((M, K), device=dev, generator=gen)
    W = torch.randn((N, K), device=dev, generator=gen) * 0.05
    winners = (torch.arange(N, device=dev) * pool)[None, :] + torch.randint(0, pool, (M, N), device=dev, generator=gen)
    argmax = winners.to(torch.float32)
    for force in (0, 32, 64, 128, 256):
        cn.lib().cn_host_force_gemm_tile_n(force)
        try:
            got = L.dotT_expand_to_maxout_grad(E, W, argmax, pool)
            want = L.expand_to_maxout_grad(L.dotT(E, W), argmax, pool)
        finally:
            cn.lib().cn_host_force_gemm_tile_n(0)
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), force
    assert cn.lib().cn_gemm_f32_expand_maxout_grad(0, 1, 4, 6, 4, None, 4, None, 4, None, 0, None, None) == 2
    assert cn.lib().cn_gemm_f32_expand_maxout_grad(0, 1, 4, 6, 4, None, 4, None, 4, None, 2, None, None) == 1


@pytest.mark.parametrize("M,N,K,pool", [(256, 512, 64, 2), (128, 1024, 100, 4), (384, 256, 33, 1), (2048, 4096, 64, 2),
                                        (1024, 2048, 120, 4)])
def test_bias_maxout_and_expansion_inside_the_write_out_of_an_unsplit_product(dev, M, N, K, pool):
    """Where K is not split and the tiles are whole, bias + maxout (forward, dot) and the expansion to the winners'
    columns (backward, dotT) happen in the product kernel's own write-out.  Same bits as the path through the
    workspace (the hook switches the write-out form off) and as the separate calls, on both 128-row tile widths;
    values against the CPU checker."""
    import ctypes
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    from util import gemm_errors
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    gen = torch.Generator(device=dev).manual_seed(M + 7 * N + K)
    A = torch.randn((M, K), device=dev, generator=gen)
    B = torch.randn((K, N), device=dev, generator=gen) * 0.05
    v = torch.randn(N, device=dev, generator=gen) * 0.1
    NE = N // 4                                   # pooled units of the backward case
    E = torch.randn((M, K), device=dev, generator=gen)
    W = torch.randn((NE, K), device=dev, generator=gen) * 0.05
    winners = (torch.arange(NE, device=dev) * pool)[None, :] + torch.randint(0, pool, (M, NE), device=dev, generator=gen)
    argmax = winners.to(torch.float32)
    try:
        for force in (128, 256, 0):
            plan = (ctypes.c_int64 * 8)()
            cn.lib().cn_host_plan_gemm(M, N, K, cus, 1 << 30, force, plan)
            assert plan[3] == 1, "the case is meant not to split K"
            cn.lib().cn_host_force_gemm_tile_n(force)
            results = []
            for in_kernel in (1, 0):
                cn.lib().cn_host_gemm_epilogue_in_kernel(in_kernel)
                out, arg = L.dot_bias_maxout(A, B, v, pool)
                back = L.dotT_expand_to_maxout_grad(E, W, argmax, pool)
                results.append((out, arg, back))
            for a, b in zip(results[0], results[1]):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), force
            want_out, want_arg = L.maxout(L.add_row_vector(L.dot(A, B), v), pool)
            assert torch.equal(results[0][0].view(torch.int32), want_out.view(torch.int32)) and torch.equal(results[0][1], want_arg)
            want_back = L.expand_to_maxout_grad(L.dotT(E, W), argmax, pool)
            assert torch.equal(results[0][2].view(torch.int32), want_back.view(torch.int32)), force
    finally:
        cn.lib().cn_host_gemm_epilogue_in_kernel(1)
        cn.lib().cn_host_force_gemm_tile_n(0)
    if M * N <= 1 << 20:
        C, Cabs = oracle.gemm_with_abs(A.cpu().numpy(), B.cpu().numpy())
        z = C.astype(np.float64) + v.cpu().numpy().astype(np.float64)[None, :]
        _maxout_against_checker(results[0][0].cpu().numpy(), results[0][1].cpu().numpy(), z, 1e-4 * float(Cabs.max()), pool)
        Cb, Cbabs = oracle.gemm_with_abs(E.cpu().numpy(), W.cpu().numpy(), False, True)
        at = np.take_along_axis(results[0][2].cpu().numpy(), winners.cpu().numpy(), axis=1)
        e1, e2 = gemm_errors(at, Cb, Cbabs)
        assert e1 <= 1e-4 and e2 <= 1e-4


def _maxout_against_checker(out, arg, z64, tol_abs, pool):
    """out / arg of a fused product + bias + maxout against the pre-activations z64 of the CPU checker (float64,
    M x N): the value is the maximum of its pool within the product tolerance, the stored winner lies in its pool and
    is a maximiser up to that tolerance, and the value is the pre-activation at the stored winner."""
    M, N = z64.shape
    groups = z64.reshape(M, N // pool, pool)
    best = groups.max(axis=2)
    assert np.all(np.abs(out.astype(np.float64) - best) <= tol_abs), float(np.abs(out - best).max())
    a = arg.astype(np.int64)
    base = (np.arange(N // pool, dtype=np.int64) * pool)[None, :]
    assert np.array_equal(arg, a.astype(np.float32)) and np.all(a >= base) and np.all(a < base + pool)
    at_winner = np.take_along_axis(z64, a.reshape(M, -1), axis=1).reshape(M, N // pool)
    assert np.all(best - at_winner <= 2 * tol_abs)
    assert np.all(np.abs(out.astype(np.float64) - at_winner) <= tol_abs)
    # where the pool has a clear winner (margin above the tolerance) the stored winner is that one
    if pool > 1:
        order = np.sort(groups, axis=2)
        clear = (order[:, :, -1] - order[:, :, -2]) > 2 * tol_abs
        assert np.array_equal(a[clear], (base + groups.argmax(axis=2))[clear])
        assert clear.mean() > 0.9


def test_forward_of_a_maxout_layer_against_the_checker_at_full_size(dev):
    """cn_gemm_f32_bias_maxout at the shapes of the training configuration, straight against the CPU checker (fp64
    product + bias + maxout) instead of against the unfused HIP calls: the second layer 128 x 8192 x 4096 in full,
    and a first layer at a quarter of its depth, 128 x 8192 x 25000, on 512 sampled pools."""
    import torch
    from clusternet_amd import _lib as L
    from util import gemm_tolerance
    rng = np.random.default_rng(2027)
    pool = 2
    M, N, K = 128, 8192, 4096
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.uniform(-0.022, 0.022, (K, N)).astype(np.float32)
    b = rng.normal(0, 0.05, N).astype(np.float32)
    out, arg = L.dot_bias_maxout(_t(A, dev), _t(W, dev), _t(b, dev), pool)
    C, Cabs = oracle.gemm_with_abs(A, W)
    z = C.astype(np.float64) + b.astype(np.float64)[None, :]
    tol = gemm_tolerance(K) * float(Cabs.max())
    _maxout_against_checker(out.cpu().numpy(), arg.cpu().numpy(), z, tol, pool)

    K = 25000
    A = (rng.uniform(0, 1, (M, K)) * (rng.uniform(0, 1, (M, K)) < 0.02)).astype(np.float32)
    W = rng.uniform(-0.0074, 0.0074, (K, N)).astype(np.float32)
    out, arg = L.dot_bias_maxout(_t(A, dev), _t(W, dev), _t(b, dev), pool)
    pools = np.sort(rng.choice(N // pool, 512, replace=False))
    cols = (pools[:, None] * pool + np.arange(pool)[None, :]).reshape(-1)
    C, Cabs = oracle.gemm_cols(A, W, cols)
    z = C + b.astype(np.float64)[cols][None, :]
    tol = gemm_tolerance(K) * float(Cabs.max())
    got_out = out.cpu().numpy()[:, pools]
    got_arg = arg.cpu().numpy()[:, pools]
    # renumber the sampled pools' winners into the sampled column space
    local = (got_arg.astype(np.int64) - (pools * pool)[None, :]) + (np.arange(pools.size) * pool)[None, :]
    _maxout_against_checker(got_out, local.astype(np.float32), z, tol, pool)


def test_backward_through_a_maxout_layer_against_the_checker_at_full_size(dev):
    """cn_gemm_f32_expand_maxout_grad at the training configuration's 128 x 4096 x 8192 (the input-gradient product
    of the second layer, scattered to the winners of the first), straight against the CPU checker."""
    import torch
    from clusternet_amd import _lib as L
    from util import gemm_errors, gemm_tolerance
    rng = np.random.default_rng(2028)
    pool = 2
    M, N, K = 128, 4096, 8192
    E = rng.normal(0, 0.01, (M, K)).astype(np.float32)
    W = rng.uniform(-0.022, 0.022, (N, K)).astype(np.float32)
    winners = (np.arange(N) * pool)[None, :] + rng.integers(0, pool, (M, N))
    argmax = winners.astype(np.float32)
    got = L.dotT_expand_to_maxout_grad(_t(E, dev), _t(W, dev), _t(argmax, dev), pool).cpu().numpy()
    C, Cabs = oracle.gemm_with_abs(E, W, False, True)
    assert got.shape == (M, N * pool)
    at = np.take_along_axis(got, winners, axis=1)
    e1, e2 = gemm_errors(at, C, Cabs)
    assert e1 <= gemm_tolerance(K) and e2 <= gemm_tolerance(K), (e1, e2)
    mask = np.ones_like(got, bool)
    np.put_along_axis(mask, winners, False, axis=1)
    assert np.all(got[mask].view(np.uint32) == 0)            # +0.0 everywhere else
    want = oracle.expand_to_maxout_grad(C.astype(np.float32), argmax, pool)
    assert np.array_equal(want != 0, (~mask) & (want != 0))   # the checker scatters to the same places


def _cpu_step(X, onehot, params, rate, pool):
    W1, b1, W2, b2, W3, b3 = params
    z1 = oracle.add_row_vector(oracle.gemm(X, W1), b1)
    h1, a1 = oracle.maxout(z1, pool)
    z2 = oracle.add_row_vector(oracle.gemm(h1, W2), b2)
    h2, a2 = oracle.maxout(z2, pool)
    p = oracle.softmax(oracle.add_row_vector(oracle.gemm(h2, W3), b3))
    e3 = p - onehot
    g3 = oracle.gemm(h2, e3, ta=True)
    e2 = oracle.expand_to_maxout_grad(oracle.gemm(e3, W3, tb=True), a2, pool)
    g2 = oracle.gemm(h1, e2, ta=True)
    e1 = oracle.expand_to_maxout_grad(oracle.gemm(e2, W2, tb=True), a1, pool)
    g1 = oracle.gemm(X, e1, ta=True)
    return p, (g1, g2, g3), (a1, a2)


def test_maxout_training_step_reduced_size(dev):
    """Same layer structure as the 100000 -> 4096 -> 4096 -> 10 configuration at 1/16 scale."""
    import torch
    from clusternet_amd import maxout_step as ms
    rng = np.random.default_rng(1)
    B, D, H, O, pool = 128, 6250, 256, 10, 2
    X = np.where(rng.random((B, D)) < 0.02, rng.random((B, D)), 0).astype(np.float32)
    lim = lambda i, o: np.sqrt(6.0 / (i + o))
    W1 = rng.uniform(-lim(D, 2 * H), lim(D, 2 * H), (D, 2 * H)).astype(np.float32)
    W2 = rng.uniform(-lim(H, 2 * H), lim(H, 2 * H), (H, 2 * H)).astype(np.float32)
    W3 = rng.uniform(-lim(H, O), lim(H, O), (H, O)).astype(np.float32)
    b1, b2, b3 = (rng.normal(0, 0.01, n).astype(np.float32) for n in (2 * H, 2 * H, O))
    y = rng.integers(0, O, B)
    onehot = np.eye(O, dtype=np.float32)[y]
    params = (W1, b1, W2, b2, W3, b3)
    p_ref, g_ref, args_ref = _cpu_step(X, onehot, params, 0.01, pool)

    dparams = tuple(_t(a, dev) for a in params)
    p, cache = ms.forward(_t(X, dev), dparams, pool)
    np.testing.assert_allclose(p.cpu().numpy(), p_ref, rtol=2e-4, atol=1e-7)
    # winners can only differ where two pool members are equal within rounding
    for a, a_ref in ((cache[1], args_ref[0]), (cache[3], args_ref[1])):
        assert (a.cpu().numpy() != a_ref).mean() < 1e-3
    grads = ms.backward(_t(X, dev), _t(onehot, dev), dparams, p, cache, pool)
    for g, gr, K in zip(grads, g_ref, (B, B, B)):
        err = np.abs(g.cpu().numpy() - gr).max() / np.abs(gr).max()
        assert err < 2e-3, err  # a flipped winner moves one error entry to the neighbouring column
    # gradient codec round trip on the device equals the checker's on the same gradient
    g1 = grads[0].clone()
    g8, codes, prec = ms.codec_round_trip(g1)
    g_host = grads[0].cpu().numpy()
    prec_h = oracle.absmax(g_host)
    assert float(prec.cpu()[0]) == prec_h
    want_codes = oracle.port_compress(g_host, prec_h)
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(g8.cpu().numpy().view(np.uint32), oracle.port_decompress(want_codes, prec_h).view(np.uint32))
    # the same batch as a sparse input: the first layer's products run on compressed rows and agree
    # with the dense ones to the product tolerance (different summation order, same terms)
    Xs = ms.sparse_input(_t(X, dev))
    assert Xs.csr.nnz == int((X != 0).sum()) and Xs.csr_t.rows == D
    p_s, cache_s = ms.forward(Xs, dparams, pool)
    np.testing.assert_allclose(p_s.cpu().numpy(), p.cpu().numpy(), rtol=2e-4, atol=1e-7)
    maxima = [torch.empty(1, device=dev) for _ in range(3)]
    grads_s = ms.backward(Xs, _t(onehot, dev), dparams, p, cache, pool, absmax_out=maxima)
    err = float((grads_s[0] - grads[0]).abs().max() / grads[0].abs().max())
    assert err < 1e-5, err
    assert float(maxima[0].cpu()[0]) == float(grads_s[0].abs().max())
    # the first layer's update straight from the error signal equals the one through the stored gradient
    e1_first = ms.backward(Xs, _t(onehot, dev), dparams, p, cache, pool, defer_first=True)[0]
    w_a, w_b = dparams[0].clone(), dparams[0].clone()
    codes_a, prec_a = ms.coded_sparse_update(w_a, Xs, e1_first, 0.01)
    codes_b, prec_b = ms.coded_update(w_b, grads_s[0].clone(), 0.01)
    assert float(prec_a.cpu()[0]) == float(prec_b.cpu()[0])
    assert torch.equal(codes_a.view(-1), codes_b.view(-1))
    assert torch.equal(w_a.view(torch.int32), w_b.view(torch.int32))
    # the full step runs and moves the weights by rate * decoded gradient
    before = dparams[4].clone()
    ms.step(_t(X, dev), _t(onehot, dev), dparams, 0.01, pool)
    assert float((dparams[4] - before).abs().max()) > 0
    # the sparse step is forward, backward and the three coded updates, nothing else
    pa = tuple(t.clone() for t in dparams)
    pb = tuple(t.clone() for t in dparams)
    ms.step(Xs, _t(onehot, dev), pb, 0.01, pool)
    p2, cache2 = ms.forward(Xs, pa, pool)
    e1_2, g2, g3 = ms.backward(Xs, _t(onehot, dev), pa, p2, cache2, pool, defer_first=True)
    ms.coded_sparse_update(pa[0], Xs, e1_2, 0.01)
    ms.coded_update(pa[2], g2, 0.01)
    ms.coded_update(pa[4], g3, 0.01)
    for a, b2 in zip(pa, pb):
        assert torch.equal(a.view(torch.int32), b2.view(torch.int32))


def test_maxout_training_step_full_size_properties(dev):
    """100000 -> 4096 -> 4096 -> 10 with pool 2 at batch 128: shapes, probabilities, the sparsity
    pattern of the expanded gradients, and sampled entries of the 100000 x 8192 weight gradient
    recomputed on the CPU."""
    import torch
    from clusternet_amd import maxout_step as ms
    g = torch.Generator(device=dev).manual_seed(3)
    B, D, H, O, pool = 128, 100000, 4096, 10, 2
    X = torch.rand((B, D), device=dev, generator=g)
    X = torch.where(torch.rand((B, D), device=dev, generator=g) < 0.02, X, torch.zeros_like(X))
    u = lambda r, c: (torch.rand((r, c), device=dev, generator=g) * 2 - 1) * float(np.sqrt(6.0 / (r + c)))
    params = (u(D, 2 * H), torch.zeros(2 * H, device=dev), u(H, 2 * H), torch.zeros(2 * H, device=dev),
              u(H, O), torch.zeros(O, device=dev))
    y = torch.randint(0, O, (B,), device=dev, generator=g)
    onehot = torch.nn.functional.one_hot(y, O).float()
    p, cache = ms.forward(X, params, pool)
    assert tuple(p.shape) == (B, O)
    assert float((p.sum(dim=1) - 1).abs().max()) < 1e-5 and float(p.min()) >= 0
    grads = ms.backward(X, onehot, params, p, cache, pool)
    assert [tuple(t.shape) for t in grads] == [(D, 2 * H), (H, 2 * H), (H, O)]
    # sampled columns of gW1 = X^T e1: recompute e1 on the device path, the product on the CPU
    e3 = p - onehot
    e2 = ms.L.expand_to_maxout_grad(ms.L.dotT(e3, params[4]), cache[3], pool)
    e1 = ms.L.expand_to_maxout_grad(ms.L.dotT(e2, params[2]), cache[1], pool)
    assert float((e1 != 0).float().mean()) <= 0.5 + 1e-6  # one winner per pool of two
    cols = np.array([0, 1, 4095, 8191, 777, 5000])
    Cref, Cabs = oracle.gemm_cols(X.cpu().numpy(), e1.cpu().numpy(), cols, ta=True)
    got = grads[0][:, torch.from_numpy(cols).to(dev)].cpu().numpy().astype(np.float64)
    assert (np.abs(got - Cref) / np.maximum(Cabs, 1e-300)).max() <= gemm_tolerance(B)
    # 8-bit round trip of the 3.28 GB gradient: decoded values stay within the codebook's step
    g1 = grads[0]
    prec = ms.L.absmax(g1)
    codes = ms.L.compression_8bit(g1, prec)
    dec = ms.L.decompression_8bit(codes, prec)
    pv = float(prec.cpu()[0])
    keep = codes != 254
    rel = ((dec - g1).abs() / pv)[keep]
    assert float(rel.max()) <= 0.0172 + 1e-6
    assert torch.equal(torch.sign(dec[keep]), torch.sign(g1[keep]))


def test_fill_on_every_path(dev):
    """cn_fill_f32 (zeros / ones of the reference): the element loop, a workgroup per tile and the form that draws its
    tiles; sizes round the tile borders, n % 4 tails, a start that is not 16-byte aligned, nothing written outside."""
    import torch
    from clusternet_amd import _lib as L
    for n in (1, 3, 5, 4097, (1 << 20) + 7, (1 << 22) + 32768 + 3, (1 << 26) + 5 * 32768 + 2):
        for off in (0, 1, 4):
            buf = torch.full((n + 16,), 7.0, device=dev)
            L.fill(buf[4 + off:4 + off + n], -0.375)
            assert float(buf[:4 + off].min()) == 7.0 and float(buf[:4 + off].max()) == 7.0, (n, off)
            assert float(buf[4 + off + n:].min()) == 7.0 and float(buf[4 + off + n:].max()) == 7.0, (n, off)
            got = buf[4 + off:4 + off + n]
            assert float(got.min()) == -0.375 and float(got.max()) == -0.375, (n, off)
            del buf
    assert L.lib().cn_host_tile_counters_in_use() == 0


def test_transpose_on_every_path(dev):
    """cn_transpose_f32: small matrices (32 x 32 tiles), whole and ragged 64 x 64 tiles, whole and ragged 128 x 128 tiles
    (a thousand of them and more), dimensions that are not multiples of four and starts that are not 16-byte aligned
    (element-wise tiles), against torch's transposition."""
    import torch
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(17)
    for r, c in ((1, 1), (3, 5), (63, 65), (64, 64), (128, 784), (1000, 1003), (260, 516), (4096, 4100), (516, 260),
                 (1024, 4096), (8192, 384), (4096, 4096), (5000, 4097), (128, 140000)):
        for off in (0, 1, 4):
            buf = torch.randn(r * c + 8, device=dev, generator=gen)
            A = buf[off:off + r * c].view(r, c)
            obuf = torch.full((r * c + 8,), 7.0, device=dev)
            out = obuf[off:off + r * c].view(c, r)
            L.transpose(A, out)
            assert torch.equal(out, A.t()), (r, c, off)
            assert float(obuf[:off].sum()) == 7.0 * off and float(obuf[off + r * c:].min()) == 7.0, (r, c, off)
    # beyond 2^26 elements a persistent grid draws 128 x 128 tiles from a counter: whole tiles, ragged ones on either edge,
    # twice in a row (the second call finds the counter as the first left it)
    for r, c in ((8320, 8200), (8200, 8320), (8192, 8192)):
        A = torch.randn((r, c), device=dev, generator=gen)
        out = torch.empty((c, r), device=dev)
        for _ in range(2):
            out.zero_()
            L.transpose(A, out)
            assert torch.equal(out, A.t()), (r, c)
        del A, out
    assert L.lib().cn_host_tile_counters_in_use() == 0
