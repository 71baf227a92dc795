"""Parity of the HIP fp32 GEMM kernels (dot / Tdot / dotT and the fused 8-bit-weight variant) with
the CPU checker, through the C-ABI.  Tolerance: max relative error 1e-4 for K <= 4096 and
1e-4 * sqrt(K / 4096) above, measured both against max|C_ref| and element-wise against
sum_k |a||b|; integer-valued and one-hot cases must be exact."""
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


@pytest.fixture(autouse=True, params=[128, 256, 32, 64, 0], ids=["tile128", "tile256", "tile32x128", "tile64x128", "planned"])
def tile_width(request, dev):
    """Every case runs on all four kernel geometries (128 x 128, 128 x 256, 32 x 128 and 64 x 128 output
    tiles) and once more with the planner's own choice."""
    import clusternet_amd as cn
    cn.lib().cn_host_force_gemm_tile_n(request.param)
    yield request.param
    cn.lib().cn_host_force_gemm_tile_n(0)


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


def test_reference_known_answers(dev):
    # literals of the reference's tests/clusterNet_test.cu:22-23,72-75,111-119,125-128,161-164;
    # the reference compares with ==, which sequential fp32 FMA meets; a matrix-core kernel may
    # differ in the last bit
    import clusternet_amd as cn
    m1 = np.array([[0, 2, 3], [0, 0.83, 59.1387]], np.float32)
    m2 = np.array([[17, 0], [3, 4], [0, 0]], np.float32)
    f = lambda r: np.array(r, np.float32)
    np.testing.assert_allclose(cn.dot(_t(m1, dev), _t(m2, dev)).cpu().numpy(), f([[6, 8], [2.49, 3.32]]), rtol=1e-6)
    np.testing.assert_allclose(cn.Tdot(_t(m1, dev), _t(m1, dev)).cpu().numpy(),
                               f([[0, 0, 0], [0, 4.6889, 55.085117], [0, 55.085117, 3506.385742]]), rtol=1e-6)
    np.testing.assert_allclose(cn.Tdot(_t(m2, dev), _t(m2, dev)).cpu().numpy(), f([[298, 12], [12, 16]]), rtol=1e-6)
    np.testing.assert_allclose(cn.dotT(_t(m1, dev), _t(m1, dev)).cpu().numpy(),
                               f([[13, 179.0761], [179.0761, 3498.074463]]), rtol=1e-6)


def test_all_ones_closed_forms_exact(dev):
    # tests/clusterNet_test.cu:338-394: 8783, 317 and 17 with exact equality
    import torch
    import clusternet_amd as cn
    ones = lambda r, c: torch.ones((r, c), dtype=torch.float32, device=dev)
    assert bool((cn.dot(ones(111, 8783), ones(8783, 317)) == 8783.0).all())
    out = cn.dotT(ones(17, 317), ones(8783, 317))
    assert tuple(out.shape) == (17, 8783) and bool((out == 317.0).all())
    out = ones(8783, 317)
    cn.dot(ones(8783, 17), ones(17, 317), out=out)
    assert bool((out == 17.0).all())
    # tests/clusterNet_test.cu:257-276: a constant product, every entry identical
    a = torch.full((200, 400), 0.3, dtype=torch.float32, device=dev)
    b = torch.full((400, 800), 1.0, dtype=torch.float32, device=dev) + 0.1748345
    c = cn.dot(a, b)
    assert tuple(c.shape) == (200, 800) and bool((c == c[0, 0]).all())
    assert abs(float(c[0, 0]) - 400 * 0.3 * 1.1748345) < 1e-3


def test_config1_mlp_layer(dev):
    import clusternet_amd as cn
    rng = np.random.default_rng(1)
    lim = np.sqrt(6.0 / (784 + 1024))
    A = rng.uniform(0, 1, (128, 784)).astype(np.float32)
    W = rng.uniform(-lim, lim, (784, 1024)).astype(np.float32)
    dC = rng.normal(0, 0.01, (128, 1024)).astype(np.float32)
    C = _check(cn, dev, A, W)                  # dot  -> 128 x 1024
    assert C.shape == (128, 1024)
    G = _check(cn, dev, A, dC, ta=True)        # Tdot -> 784 x 1024
    assert G.shape == (784, 1024)
    E = _check(cn, dev, dC, W, tb=True)        # dotT -> 128 x 784
    assert E.shape == (128, 784)


def test_config1_on_the_reference_mnist_batch(dev):
    """First layer of the reference's MNIST network on its own data file (tests/mnist_mini_X.hdf5 of
    the reference, 500 x 784 fp32 at byte 2144): real pixel rows are mostly exact zeros with runs of
    values in (0, 1], unlike the synthetic uniform batch."""
    import os
    import clusternet_amd as cn
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hdf5", "mnist_mini_X.hdf5")
    X = np.fromfile(path, dtype=np.float32, offset=2144, count=500 * 784).reshape(500, 784)
    rng = np.random.default_rng(6)
    lim = np.sqrt(6.0 / (784 + 1024))
    W = rng.uniform(-lim, lim, (784, 1024)).astype(np.float32)
    for lo in (0, 128, 372):                       # 372: the last, 128-row batch of the 500
        A = X[lo:lo + 128]
        C = _check(cn, dev, A, W)
        dC = (C * 0.01).astype(np.float32)
        _check(cn, dev, A, dC, ta=True)            # Tdot -> 784 x 1024
        _check(cn, dev, dC, W, tb=True)            # dotT -> 128 x 784
    _check(cn, dev, X, W)                          # all 500 rows: ragged in M


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (2, 2, 3), (128, 128, 32), (129, 130, 33),
                                   (64, 200, 31), (257, 100, 64), (100, 10, 4096), (200, 300, 1000),
                                   (128, 512, 8192), (37, 1029, 515), (1000, 4, 128)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_ragged_shapes_all_transposes(dev, shape, ta, tb):
    import clusternet_amd as cn
    M, N, K = shape
    rng = np.random.default_rng(M * 131 + N * 17 + K)
    A = rng.normal(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
    B = rng.normal(0, 1, (N, K) if tb else (K, N)).astype(np.float32)
    _check(cn, dev, A, B, ta, tb)


def test_identity_operand_is_exact(dev):
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(3)
    B = rng.normal(0, 1, (300, 517)).astype(np.float32)
    I = np.eye(300, dtype=np.float32)
    assert np.array_equal(cn.dot(_t(I, dev), _t(B, dev)).cpu().numpy(), B)
    assert np.array_equal(cn.Tdot(_t(I, dev), _t(B, dev)).cpu().numpy(), B)
    A = rng.normal(0, 1, (211, 300)).astype(np.float32)
    assert np.array_equal(cn.dot(_t(A, dev), _t(I, dev)).cpu().numpy(), A)
    assert np.array_equal(cn.dotT(_t(A, dev), _t(I, dev)).cpu().numpy(), A)
    # a permutation picks rows: the k index of every product lands where it should
    perm = rng.permutation(300)
    P = np.zeros((300, 300), np.float32)
    P[np.arange(300), perm] = 1
    assert np.array_equal(cn.dot(_t(P, dev), _t(B, dev)).cpu().numpy(), B[perm])


def test_strided_operands_and_output_overwrite(dev):
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(4)
    big_a = rng.normal(0, 1, (70, 203)).astype(np.float32)
    big_b = rng.normal(0, 1, (150, 99)).astype(np.float32)
    A, B = big_a[:, 3:153], big_b[:, 2:90]            # lda 203 > K 150, ldb 99 > N 88, odd offsets
    at, bt = _t(big_a, dev)[:, 3:153], _t(big_b, dev)[:, 2:90]
    out_big = torch.full((70, 120), float("nan"), dtype=torch.float32, device=dev)
    out = out_big[:, 5:93]
    cn.dot(at, bt, out=out)                           # beta = 0: NaNs in out must not leak
    Cref, Cabs = oracle.gemm_with_abs(np.ascontiguousarray(A), np.ascontiguousarray(B))
    e1, e2 = gemm_errors(out.cpu().numpy(), Cref, Cabs)
    assert e1 < 1e-4 and e2 < 1e-4
    assert bool(torch.isnan(out_big[:, :5]).all()) and bool(torch.isnan(out_big[:, 93:]).all())


@pytest.mark.parametrize("M,N,K,ta,tb", [(384, 512, 96, 0, 0), (640, 256, 128, 1, 0), (128, 1024, 4000, 0, 0),
                                         (300, 520, 64, 0, 1), (256, 260, 40, 1, 1)])
def test_wide_write_out_gives_the_same_bits(dev, M, N, K, ta, tb):
    """Tiles that lie inside the matrix leave through LDS as 16-byte stores, the others (and everything
    when the hook is off) as 4-byte stores: the same values either way, also in a padded output and with
    the maximum."""
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(M + N + K)
    A = _t(rng.normal(0, 1, (K, M) if ta else (M, K)).astype(np.float32), dev)
    B = _t(rng.normal(0, 1, (N, K) if tb else (K, N)).astype(np.float32), dev)
    big = torch.full((M, N + 12), float("nan"), device=dev)
    amax = torch.zeros(1, device=dev)
    wide = cn.gemm(A, B, bool(ta), bool(tb), out=big[:, 4:4 + N], absmax_out=amax).clone()
    assert bool(torch.isnan(big[:, :4]).all()) and bool(torch.isnan(big[:, 4 + N:]).all())
    cn.lib().cn_host_gemm_wide_store(0)
    try:
        narrow = cn.gemm(A, B, bool(ta), bool(tb))
    finally:
        cn.lib().cn_host_gemm_wide_store(1)
    assert torch.equal(wide.view(torch.int32), narrow.view(torch.int32))
    assert float(amax.cpu()[0]) == float(narrow.abs().max())


def test_shape_errors_are_reported(dev):
    import torch
    import clusternet_amd as cn
    a = torch.zeros((4, 5), device=dev)
    b = torch.zeros((6, 7), device=dev)
    with pytest.raises(cn.CnError):
        cn.dot(a, b)
    with pytest.raises(cn.CnError):
        cn.dot(a, torch.zeros((5, 7), device=dev), out=torch.zeros((4, 8), device=dev))
    L = cn.lib()
    assert L.cn_gemm_f32(0, 0, 4, 7, 5, a.data_ptr(), 4, b.data_ptr(), 7, a.data_ptr(), 7, None) == 2
    assert L.cn_gemm_f32(0, 0, 4, 7, 5, None, 5, b.data_ptr(), 7, a.data_ptr(), 7, None) == 1
    # K = 0 zeroes the output
    out = torch.full((4, 7), 3.0, device=dev)
    assert L.cn_gemm_f32(0, 0, 4, 7, 0, None, 1, None, 7, out.data_ptr(), 7, None) == 0
    assert bool((out == 0).all())


def test_linearity_and_transpose_identities_large(dev):
    """Size-independent properties on a K = 20000 product: dot(A, B1 + B2) = dot(A,B1) + dot(A,B2)
    up to rounding, Tdot(A^T stored, B) = dot(A, B), dotT(A, B^T stored) = dot(A, B)."""
    import torch
    import clusternet_amd as cn
    g = torch.Generator(device=dev).manual_seed(7)
    A = torch.rand((128, 20000), device=dev, generator=g)
    B1 = (torch.rand((20000, 1536), device=dev, generator=g) - 0.5) * 0.02
    B2 = (torch.rand((20000, 1536), device=dev, generator=g) - 0.5) * 0.02
    c1, c2, c12 = cn.dot(A, B1), cn.dot(A, B2), cn.dot(A, B1 + B2)
    scale = float(c12.abs().max())
    assert float((c12 - (c1 + c2)).abs().max()) / scale < gemm_tolerance(20000)
    ct = cn.Tdot(A.t().contiguous(), B1)
    cT = cn.dotT(A, B1.t().contiguous())
    assert float((ct - c1).abs().max()) / scale < gemm_tolerance(20000)
    assert float((cT - c1).abs().max()) / scale < gemm_tolerance(20000)


def test_config3_full_size_sampled_columns(dev, tile_width):
    """README workload on one GPU: 128x100000 . 100000x40000, then . 40000x20000 (source/clusterNet.cpp:404-461 on the
    un-sharded operands of README.md:22-32).  Recomputed on the CPU in fp64: all of out2, and of out1 all rows of at
    least 1024 columns: seven in each of its 157 tiles of 256 columns (every (K-chunk, tile) work unit of the product
    contributes to some checked entry), both columns either side of every tile border, and the corners."""
    import torch
    import clusternet_amd as cn
    thorough = tile_width == 0  # the library's own plan; a forced geometry gets a sample of 48 columns of each product
    g = torch.Generator(device=dev).manual_seed(11)
    batch = torch.rand((128, 100000), device=dev, generator=g)
    lim1, lim2 = float(np.sqrt(6.0 / 140000)), float(np.sqrt(6.0 / 60000))
    W1 = torch.empty((100000, 40000), device=dev)
    for r in range(0, 100000, 10000):
        W1[r:r + 10000] = (torch.rand((10000, 40000), device=dev, generator=g) * 2 - 1) * lim1
    W2 = (torch.rand((40000, 20000), device=dev, generator=g) * 2 - 1) * lim2
    out1 = cn.dot(batch, W1)
    out2 = cn.dot(out1, W2)
    assert tuple(out1.shape) == (128, 40000) and tuple(out2.shape) == (128, 20000)
    rng = np.random.default_rng(5)
    N1 = 40000
    borders = np.arange(256, N1, 256)
    cols = np.unique(np.concatenate([[0, 1, N1 - 2, N1 - 1], borders - 1, borders, borders - 129, borders - 128,
                                     (np.arange(157)[:, None] * 256 + rng.integers(0, 256, (157, 7))).ravel()]))
    cols = cols[(cols >= 0) & (cols < N1)]
    assert cols.size >= 1024
    if not thorough:
        cols = np.unique(np.concatenate([[0, 1, 127, 128, N1 - 129, N1 - 128, N1 - 1], rng.integers(0, N1, 41)]))
    idx = torch.from_numpy(cols).to(dev)
    Cref, Cabs = oracle.gemm_with_abs(batch.cpu().numpy(), W1[:, idx].contiguous().cpu().numpy())
    e1, e2 = gemm_errors(out1[:, idx].cpu().numpy(), Cref, Cabs)
    tol = gemm_tolerance(100000)
    assert e1 <= tol and e2 <= tol, ("out1", cols.size, e1, e2, tol)
    # every column got written: compare column sums against a torch matmul of a strided sample
    colsum_ref = batch.double() @ W1[:, ::397].double()
    assert float((out1[:, ::397].double() - colsum_ref).abs().max()) / float(colsum_ref.abs().max()) < tol
    del W1, Cref, Cabs
    if thorough:
        Cref, Cabs = oracle.gemm_with_abs(out1.cpu().numpy(), W2.cpu().numpy())
        got = out2.cpu().numpy()
    else:
        idx = torch.from_numpy(np.unique(np.concatenate([[0, 1, 127, 128, 19871, 19872, 19999], rng.integers(0, 20000, 41)]))).to(dev)
        Cref, Cabs = oracle.gemm_with_abs(out1.cpu().numpy(), W2[:, idx].contiguous().cpu().numpy())
        got = out2[:, idx].cpu().numpy()
    e1, e2 = gemm_errors(got, Cref, Cabs)
    tol = gemm_tolerance(40000)
    assert e1 <= tol and e2 <= tol, ("out2", e1, e2, tol)


def test_first_layer_input_gradient_full_size(dev, tile_width):
    """dotT 128 x 8192 . (100000 x 8192)^T -> 128 x 100000, the optional product of the training configuration that
    reads all of W1 (source/clusterNet.cpp:262-284): 1024 sampled columns and the borders of its tiles in fp64."""
    import torch
    import clusternet_amd as cn
    if tile_width != 0:
        pytest.skip("one run is enough: the library's own plan")
    g = torch.Generator(device=dev).manual_seed(12)
    E = torch.empty((128, 8192), device=dev).normal_(0.0, 0.01, generator=g)
    lim = float(np.sqrt(6.0 / 108192))
    W1 = (torch.rand((100000, 8192), device=dev, generator=g) * 2 - 1) * lim
    out = cn.dotT(E, W1)
    assert tuple(out.shape) == (128, 100000)
    rng = np.random.default_rng(8)
    borders = np.arange(256, 100000, 256)
    cols = np.unique(np.concatenate([[0, 1, 99998, 99999], borders[::8] - 1, borders[::8], rng.integers(0, 100000, 1024)]))
    idx = torch.from_numpy(cols).to(dev)
    Cref, Cabs = oracle.gemm_with_abs(E.cpu().numpy(), W1[idx].contiguous().cpu().numpy(), False, True)
    e1, e2 = gemm_errors(out[:, idx].cpu().numpy(), Cref, Cabs)
    tol = gemm_tolerance(8192)
    assert cols.size >= 1024 and e1 <= tol and e2 <= tol, (cols.size, e1, e2, tol)
    # every column written: a strided sample against torch in fp64
    ref = E.double() @ W1[::97].double().t()
    assert float((out[:, ::97].double() - ref).abs().max()) / float(ref.abs().max()) < tol


def test_fused_w8_decode_is_bit_identical(dev):
    import clusternet_amd as cn
    rng = np.random.default_rng(6)
    K, N = 300, 1000
    W = rng.integers(0, 256, (K, N), dtype=np.uint8)
    I = np.eye(K, dtype=np.float32)
    for scale in (1.0, 0.0371, 11.5):
        got = cn.gemm_w8(_t(I, dev), _t(W, dev), scale).cpu().numpy()
        want = oracle.decompress(W, scale)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), scale


@pytest.mark.parametrize("batch", [32, 128, 512])
def test_config4_fused_w8_gemm(dev, batch):
    import clusternet_amd as cn
    rng = np.random.default_rng(8 + batch)
    A = rng.normal(0, 1, (batch, 4096)).astype(np.float32)
    Wf = rng.normal(0, 1 / 64.0, (4096, 4096)).astype(np.float32)
    wt = _t(Wf, dev)
    scale_dev = cn.absmax(wt)
    scale = float(scale_dev.cpu()[0])
    codes_t = cn.compression_8bit(wt, scale)
    codes = codes_t.cpu().numpy()
    assert np.array_equal(codes, oracle.port_compress(Wf, scale))
    fused = cn.gemm_w8(_t(A, dev), codes_t, scale).cpu().numpy()
    Wd = oracle.decompress(codes, scale)
    Cref, Cabs = oracle.gemm_with_abs(A, Wd)
    e1, e2 = gemm_errors(fused, Cref, Cabs)
    assert e1 <= 1e-4 and e2 <= 1e-4, (e1, e2)
    # and it agrees with decompress-then-dot on the device to the same tolerance
    unfused = cn.dot(_t(A, dev), cn.decompression_8bit(codes_t, scale)).cpu().numpy()
    assert np.abs(unfused - fused).max() / np.abs(Cref).max() <= 1e-4


@pytest.mark.parametrize("shape", [(5, 7, 9), (130, 131, 65), (128, 1000, 30), (64, 4099, 257)])
def test_fused_w8_ragged(dev, shape):
    import clusternet_amd as cn
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.integers(0, 256, (K, N), dtype=np.uint8)
    got = cn.gemm_w8(_t(A, dev), _t(W, dev), 0.25).cpu().numpy()
    Cref, Cabs = oracle.gemm_with_abs(A, oracle.decompress(W, 0.25))
    e1, e2 = gemm_errors(got, Cref, Cabs)
    assert e1 <= 1e-4 and e2 <= 1e-4, (e1, e2)


@pytest.mark.parametrize("shape", [(1, 128, 64), (8, 132, 72), (31, 1000, 512), (32, 4096, 1024), (33, 260, 1024),
                                   (64, 4100, 264), (64, 8192, 4096), (65, 128, 4096), (200, 300, 512), (1024, 1024, 256)])
def test_fused_w8_few_rows(dev, shape):
    """Products of up to 1024 rows on 8-bit weights take a kernel of their own (codes decoded straight into the
    matrix instruction's registers, K dealt to the eight wavefronts of a workgroup and to chunks).  Against the CPU
    checker, against the tiled kernel it replaces there (the hook keeps it), with operands that sit inside wider
    arrays, and with one-hot rows, for which every output must be the decoded weight itself, bit for bit."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.integers(0, 256, (K, N), dtype=np.uint8)
    Cref, Cabs = oracle.gemm_with_abs(A, oracle.decompress(W, 0.25))
    At, Wt = _t(A, dev), _t(W, dev)
    got = cn.gemm_w8(At, Wt, 0.25).cpu().numpy()
    e1, e2 = gemm_errors(got, Cref, Cabs)
    assert e1 <= 1e-4 and e2 <= 1e-4, (e1, e2)
    try:
        L.lib().cn_host_gemm_w8_rows(0)
        tiled = cn.gemm_w8(At, Wt, 0.25).cpu().numpy()
    finally:
        L.lib().cn_host_gemm_w8_rows(1)
    assert np.abs(tiled - got).max() / np.abs(Cref).max() <= 1e-4
    # operands inside wider arrays (leading dimensions larger than the rows), output into a wider array too
    Aw = torch.zeros((M, K + 8), device=dev)
    Aw[:, 4:4 + K] = At
    Ww = torch.full((K, N + 12), 77, dtype=torch.uint8, device=dev)
    Ww[:, 8:8 + N] = Wt
    Cw = torch.full((M, N + 4), 7.0, device=dev)
    cn.gemm_w8(Aw[:, 4:4 + K], Ww[:, 8:8 + N], 0.25, out=Cw[:, :N])
    assert np.array_equal(Cw[:, :N].cpu().numpy().view(np.uint32), got.view(np.uint32))
    assert float(Cw[:, N:].min()) == 7.0 and float(Cw[:, N:].max()) == 7.0
    # one-hot rows: the product is a row of decoded weights
    ks = rng.integers(0, K, M)
    onehot = np.zeros((M, K), np.float32)
    onehot[np.arange(M), ks] = 1.0
    rows = cn.gemm_w8(_t(onehot, dev), Wt, 0.0371).cpu().numpy()
    want = oracle.decompress(W[ks], 0.0371)
    assert np.array_equal(rows.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape,ta,tb", [((128, 300, 64), False, False), ((1000, 257, 128), True, False),
                                          ((37, 1029, 515), False, True), ((128, 512, 8192), False, False),
                                          ((3, 5, 7), True, True), ((64, 64, 1), False, False)])
def test_gemm_with_absmax_output(dev, shape, ta, tb):
    """The maximum delivered by the product's write-out (or by the addition of K chunks) equals the
    stand-alone abs-max kernel over the result bit for bit, and the product itself is unchanged."""
    import torch
    import clusternet_amd as cn
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N)
    A = rng.normal(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
    B = rng.normal(0, 0.05, (N, K) if tb else (K, N)).astype(np.float32)
    At, Bt = _t(A, dev), _t(B, dev)
    plain = cn.gemm(At, Bt, ta, tb)
    m = torch.full((1,), 123.0, device=dev)
    fused = cn.gemm(At, Bt, ta, tb, absmax_out=m)
    assert torch.equal(plain.view(torch.int32), fused.view(torch.int32))
    want = cn.absmax(plain)
    assert torch.equal(m.view(torch.int32), want.view(torch.int32)), (float(m), float(want))
    assert float(m) == float(np.abs(plain.cpu().numpy()).max()) if plain.numel() else True


def test_gemm_with_absmax_output_strided_and_empty(dev):
    import torch
    import clusternet_amd as cn
    L = cn.lib()
    rng = np.random.default_rng(4)
    A = _t(rng.normal(0, 1, (128, 96)).astype(np.float32), dev)
    B = _t(rng.normal(0, 1, (96, 200)).astype(np.float32), dev)
    big = torch.full((128, 256), 1e9, device=dev)      # columns 200.. must not enter the maximum
    m = torch.empty(1, device=dev)
    cn.gemm(A, B, False, False, out=big[:, :200], absmax_out=m)
    assert float(m) == float(big[:, :200].abs().max()) and float(big[0, 200]) == 1e9
    assert L.cn_gemm_f32_absmax(0, 0, 0, 5, 3, None, 3, None, 5, None, 5, m.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert float(m) == -1.0
    assert L.cn_gemm_f32_absmax(0, 0, 4, 4, 4, A.data_ptr(), 96, B.data_ptr(), 200, big.data_ptr(), 256, None, None) == 1
