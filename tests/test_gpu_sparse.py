"""Parity of the sparse (CSR) path with the CPU checker through the C-ABI: layout, transposition and
product bit for bit (the product sums in the checker's order), and the products of the training step
within the GEMM tolerance of the fp64 dense product."""
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


@pytest.fixture(autouse=True, params=["b_in_lds", "b_from_l2", "whole_rows"])
def short_row_kernel(request, dev):
    """The max-only pass has two kernels (B strip in LDS when B has at most 128 rows, B from the L2
    otherwise), the passes that also update the weights two forms (a workgroup split into wavefronts that
    produce codes and wavefronts that stream the weights, or every wavefront on whole rows): every test runs
    with the library's choices, with the first kernel switched off, and with the split switched off."""
    from clusternet_amd import _lib as L
    L.lib().cn_host_csr_lds_rows(0 if request.param == "b_from_l2" else 1)
    L.lib().cn_host_csr_paired_rows(0 if request.param == "whole_rows" else 1)
    yield
    L.lib().cn_host_csr_lds_rows(1)
    L.lib().cn_host_csr_paired_rows(1)


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _sparse(rng, rows, cols, density):
    A = rng.uniform(0, 1, (rows, cols)).astype(np.float32)
    return A * (rng.random((rows, cols)) < density)


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("shape,density", [((1, 1), 1.0), ((7, 11), 0.3), ((128, 5000), 0.02), ((300, 257), 0.1),
                                           ((5, 1000), 0.0), ((128, 1024), 1.0), ((1000, 3), 0.5)])
@pytest.mark.parametrize("transpose", [False, True])
def test_csr_from_dense_matches_checker(dev, shape, density, transpose):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(shape[0] * 31 + shape[1])
    A = _sparse(rng, *shape, density)
    if A.size > 3:
        A.flat[1] = -0.0
    S = L.csr_from_dense(_t(A, dev), transpose)
    row_ptr, col_idx, vals = oracle.csr_from_dense(A, transpose)
    assert (S.rows, S.cols) == ((shape[1], shape[0]) if transpose else shape)
    assert np.array_equal(S.row_ptr.cpu().numpy(), row_ptr)
    assert np.array_equal(S.col_idx.cpu().numpy(), col_idx)
    assert np.array_equal(_bits(S.vals.cpu().numpy()), _bits(vals))


def test_csr_from_dense_of_a_strided_view_and_capacity_error(dev):
    import ctypes as C
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(5)
    big = _sparse(rng, 64, 300, 0.2)
    view = _t(big, dev)[:, 10:210]
    S = L.csr_from_dense(view)
    row_ptr, col_idx, vals = oracle.csr_from_dense(np.ascontiguousarray(big[:, 10:210]))
    assert np.array_equal(S.row_ptr.cpu().numpy(), row_ptr) and np.array_equal(S.col_idx.cpu().numpy(), col_idx)
    nnz = C.c_int64()
    rp = torch.empty(65, dtype=torch.int32, device=dev)
    ci = torch.empty(4, dtype=torch.int32, device=dev)
    va = torch.empty(4, dtype=torch.float32, device=dev)
    status = L.lib().cn_csr_from_dense_f32(view.data_ptr(), 64, 200, 300, 0, rp.data_ptr(), ci.data_ptr(), va.data_ptr(), 4,
                                           C.byref(nnz), None)
    assert status == 5 and nnz.value == vals.size and np.array_equal(rp.cpu().numpy(), row_ptr)


@pytest.mark.parametrize("R,Cc,N,density", [(37, 211, 19, 0.05), (1000, 128, 1024, 0.02), (300, 64, 4100, 0.1),
                                            (5, 9, 1, 0.5), (2048, 128, 8192, 0.02), (16, 40, 7, 0.0)])
def test_gather_product_is_bit_exact(dev, R, Cc, N, density):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(R + N)
    S_dense = _sparse(rng, R, Cc, density)
    B = rng.normal(0, 1, (Cc, N)).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    got = L.csr_gemm(S, _t(B, dev)).cpu().numpy()
    want = oracle.csr_gemm(oracle.csr_from_dense(S_dense), B)
    assert np.array_equal(_bits(got), _bits(want))
    # the variant that also reports max|out|: same product, and the maximum equals the abs-max pass
    import torch
    amax = torch.full((1,), 123.0, device=dev)
    got2 = L.csr_gemm(S, _t(B, dev), absmax_out=amax).cpu().numpy()
    assert np.array_equal(_bits(got2), _bits(want))
    assert float(amax.cpu()[0]) == float(oracle.absmax(want))


@pytest.mark.parametrize("R,Cc,N,density", [(128, 3000, 4096, 0.02), (100, 700, 2052, 0.1), (3, 50, 2048, 0.5),
                                            (128, 64, 8192, 1.0), (64, 500, 2820, 0.05), (128, 200, 4612, 0.03)])
def test_few_long_rows_take_the_strip_kernel_with_the_same_bits(dev, R, Cc, N, density):
    """Few rows and many columns run one column strip per L2 at a time; same sums, same bits, also with
    the maximum."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(R + N)
    S_dense = _sparse(rng, R, Cc, density)
    B = rng.normal(0, 1, (Cc, N)).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    amax = torch.zeros(1, device=dev)
    got = L.csr_gemm(S, _t(B, dev), absmax_out=amax)
    L.lib().cn_host_csr_strip_kernel(0)
    try:
        plain = L.csr_gemm(S, _t(B, dev))
    finally:
        L.lib().cn_host_csr_strip_kernel(1)
    assert torch.equal(got.view(torch.int32), plain.view(torch.int32))
    want = oracle.csr_gemm(oracle.csr_from_dense(S_dense), B)
    assert np.array_equal(_bits(got.cpu().numpy()), _bits(want))
    assert float(amax.cpu()[0]) == float(oracle.absmax(want))


@pytest.mark.parametrize("R,Cc,N,density,pool", [(128, 3000, 4096, 0.02, 2), (100, 700, 2048, 0.1, 4), (128, 300, 8192, 0.05, 2),
                                                 (37, 211, 18, 0.05, 3), (300, 64, 4100, 0.1, 2), (5, 9, 6, 0.5, 6)])
def test_product_bias_maxout_in_one_call_equals_the_three_kernels(dev, R, Cc, N, density, pool):
    """Few long rows take bias and maximum in the product's write-out, other shapes go through the
    workspace: either way the values and winners of csr_gemm, add_row_vector and maxout."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(R + N + pool)
    S_dense = _sparse(rng, R, Cc, density)
    B = rng.normal(0, 1, (Cc, N)).astype(np.float32)
    v = rng.normal(0, 0.1, N).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    out, arg = L.csr_gemm_bias_maxout(S, _t(B, dev), _t(v, dev), pool)
    want_out, want_arg = L.maxout(L.add_row_vector(L.csr_gemm(S, _t(B, dev)), _t(v, dev)), pool)
    assert torch.equal(out.view(torch.int32), want_out.view(torch.int32)) and torch.equal(arg, want_arg)
    z = oracle.add_row_vector(oracle.csr_gemm(oracle.csr_from_dense(S_dense), B), v)
    h, a = oracle.maxout(z, pool)
    assert np.array_equal(_bits(out.cpu().numpy()), _bits(h)) and np.array_equal(arg.cpu().numpy(), a)


def test_gather_product_absmax_of_an_empty_result(dev):
    import torch
    from clusternet_amd import _lib as L
    S = L.csr_from_dense(torch.zeros((0, 5), device=dev))
    amax = torch.full((1,), 123.0, device=dev)
    L.csr_gemm(S, torch.ones((5, 8), device=dev), absmax_out=amax)
    assert float(amax.cpu()[0]) == -1.0


@pytest.mark.parametrize("R,Cc,N,density", [(2000, 128, 1024, 0.02), (777, 64, 4100, 0.05), (37, 211, 19, 0.05),
                                            (5, 9, 1, 0.5), (301, 16, 2052, 0.0), (4096, 128, 8192, 0.02),
                                            (2005, 100, 8196, 0.03)])  # the last two: several rounds of a split workgroup
@pytest.mark.parametrize("with_update", [False, True])
def test_product_to_codes_and_update_equals_the_three_separate_calls(dev, R, Cc, N, density, with_update):
    """max|S B| without storing, then codes (and the weight update) straight from the recomputed product:
    bit for bit what csr_gemm, absmax, compression_8bit and decompression_8bit_axpy give, and what the
    CPU checker gives for the same sequence."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(R * 7 + N)
    S_dense = _sparse(rng, R, Cc, density)
    B = rng.normal(0, 0.01, (Cc, N)).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    Bd = _t(B, dev)
    G = L.csr_gemm(S, Bd)
    prec = L.csr_gemm_absmax(S, Bd)
    want_prec = L.absmax(G)
    assert float(prec.cpu()[0]) == float(want_prec.cpu()[0])
    want_codes = L.compression_8bit(G, want_prec)
    w0 = rng.normal(0, 0.05, (R, N)).astype(np.float32)
    w = _t(w0, dev) if with_update else None
    codes = L.csr_gemm_coded_update(S, Bd, prec, w=w, alpha=-0.01)
    assert torch.equal(codes, want_codes.view(R, N))
    # against the CPU checker on the checker's own product
    G_host = oracle.csr_gemm(oracle.csr_from_dense(S_dense), B)
    p_host = oracle.absmax(G_host)
    assert float(prec.cpu()[0]) == p_host
    if p_host > 0:
        assert np.array_equal(codes.cpu().numpy(), oracle.port_compress(G_host, p_host).reshape(R, N))
    if with_update:
        want_w = _t(w0, dev)
        L.decompression_8bit_axpy(want_codes, want_prec, -0.01, want_w)
        assert torch.equal(w.view(torch.int32), want_w.view(torch.int32))
        if p_host > 0:
            host_w = oracle.decompress_axpy(codes.cpu().numpy().reshape(-1), p_host, -0.01, w0.reshape(-1))
            assert np.array_equal(_bits(w.cpu().numpy().reshape(-1)), _bits(host_w))


@pytest.mark.parametrize("R,Cc,N,density", [(2000, 128, 1024, 0.02), (777, 64, 4100, 0.05), (37, 211, 19, 0.05),
                                            (301, 16, 2052, 0.0), (2005, 100, 8196, 0.03)])
def test_product_to_codes_and_rmsprop_equals_the_separate_calls(dev, R, Cc, N, density):
    """The RMSprop form: codes, running mean squares and weights bit for bit those of csr_gemm, absmax,
    compression_8bit and rmsprop_update on the codes; and those of the CPU checker."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(R * 5 + N)
    S_dense = _sparse(rng, R, Cc, density)
    B = rng.normal(0, 0.01, (Cc, N)).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    Bd = _t(B, dev)
    w0 = rng.normal(0, 0.05, (R, N)).astype(np.float32)
    r0 = rng.uniform(1e-6, 1e-3, (R, N)).astype(np.float32)
    G = L.csr_gemm(S, Bd)
    prec = L.csr_gemm_absmax(S, Bd)
    want_codes = L.compression_8bit(G, prec)
    want_w, want_r = _t(w0, dev), _t(r0, dev)
    L.rmsprop_update(want_r, want_codes, want_w, 0.9, 0.003, precision=prec)
    w, r = _t(w0, dev), _t(r0, dev)
    codes = L.csr_gemm_coded_rmsprop(S, Bd, prec, r, w, 0.9, 0.003)
    assert torch.equal(codes, want_codes.view(R, N))
    assert torch.equal(r.view(torch.int32), want_r.view(torch.int32))
    assert torch.equal(w.view(torch.int32), want_w.view(torch.int32))
    p_host = float(prec.cpu()[0])
    if p_host > 0:
        dec = oracle.port_decompress(codes.cpu().numpy().reshape(-1), p_host)
        host_r, host_w = oracle.rmsprop_update(r0.reshape(-1), dec, w0.reshape(-1), 0.9, 0.003)
        assert np.array_equal(_bits(r.cpu().numpy().reshape(-1)), _bits(host_r))
        assert np.array_equal(_bits(w.cpu().numpy().reshape(-1)), _bits(host_w))


def test_product_to_codes_takes_strided_operands(dev):
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(31)
    S_dense = _sparse(rng, 300, 40, 0.1)
    Bfull = rng.normal(0, 1, (40, 300)).astype(np.float32)
    S = L.csr_from_dense(_t(S_dense, dev))
    Bd = _t(Bfull, dev)[:, 8:208]
    wfull = torch.zeros((300, 256), device=dev)
    prec = L.csr_gemm_absmax(S, Bd)
    codes = L.csr_gemm_coded_update(S, Bd, prec, w=wfull[:, 16:216], alpha=1.0)
    G = L.csr_gemm(S, Bd.contiguous())
    assert torch.equal(codes, L.compression_8bit(G, prec).view(300, 200))
    assert torch.equal(wfull[:, 16:216], L.decompression_8bit(codes.view(-1), prec).view(300, 200))
    assert float(wfull[:, :16].abs().max()) == 0 and float(wfull[:, 216:].abs().max()) == 0


def test_csr_to_dense_restores_the_matrix(dev):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(12)
    for shape, density in (((128, 5000), 0.02), ((7, 11), 0.3), ((5, 1000), 0.0), ((64, 300), 1.0)):
        A = _sparse(rng, *shape, density)
        S = L.csr_from_dense(_t(A, dev))
        assert np.array_equal(_bits(L.csr_to_dense(S).cpu().numpy()), _bits(A))


@pytest.mark.parametrize("shape,density", [((1, 1), 1.0), ((7, 11), 0.3), ((128, 5000), 0.02), ((300, 257), 0.1),
                                           ((5, 1000), 0.0), ((64, 64), 1.0), ((1000, 3), 0.5)])
def test_csr_transpose_equals_csr_of_the_transpose(dev, shape, density):
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(shape[0] * 17 + shape[1])
    A = _sparse(rng, *shape, density)
    T = L.csr_transpose(L.csr_from_dense(_t(A, dev)))
    row_ptr, col_idx, vals = oracle.csr_from_dense(A, transpose=True)
    assert (T.rows, T.cols) == (shape[1], shape[0])
    assert np.array_equal(T.row_ptr.cpu().numpy(), row_ptr)
    assert np.array_equal(T.col_idx.cpu().numpy(), col_idx)
    assert np.array_equal(_bits(T.vals.cpu().numpy()), _bits(vals))


def test_csr_transpose_with_a_dense_column_and_long_rows(dev):
    """A column that every one of 60 000 rows uses, beside sparse ones, and a short wide matrix whose transposition
    has a hundred thousand short rows: the result rows come out in ascending column order whatever their length
    (a counting sort over blocks of rows; nothing is sorted afterwards), twice in a row with the same bits."""
    import scipy.sparse as sp
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(90)
    R, C = 60_000, 300
    A = (rng.uniform(0, 1, (R, C)) * (rng.uniform(0, 1, (R, C)) < 0.01)).astype(np.float32)
    A[:, 7] = rng.uniform(0.5, 1, R).astype(np.float32)       # fully dense column -> a result row of 60 000 entries
    A[::3, 123] = 2.0
    for M in (A, np.ascontiguousarray(A[:128].T), (rng.uniform(0, 1, (128, 100_000)) * (rng.uniform(0, 1, (128, 100_000)) < 0.02)).astype(np.float32)):
        S = L.csr_from_dense(_t(M, dev))
        want = sp.csr_matrix(M.T)
        want.sort_indices()
        for _ in range(2):
            T = L.csr_transpose(S)
            assert (T.rows, T.cols) == (M.shape[1], M.shape[0])
            assert np.array_equal(T.row_ptr.cpu().numpy(), want.indptr)
            assert np.array_equal(T.col_idx.cpu().numpy(), want.indices)
            assert np.array_equal(_bits(T.vals.cpu().numpy()), _bits(want.data.astype(np.float32)))


def test_more_than_2_to_31_nonzeros_are_refused_not_truncated(dev):
    """8.6 GB of ones: the count of nonzeros passes 2^31 - 1, which the 32-bit row pointers cannot hold.  The
    prefix sums carry 64 bits, so the count arrives exact and the call answers CN_ERR_SHAPE."""
    import ctypes
    import torch
    import clusternet_amd as cn
    rows, cols = 65_536, 32_800
    A = torch.ones((rows, cols), device=dev)
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device=dev)
    nnz = ctypes.c_int64(-1)
    status = cn.lib().cn_csr_from_dense_f32(A.data_ptr(), rows, cols, cols, 0, row_ptr.data_ptr(), None, None, 0, ctypes.byref(nnz), None)
    torch.cuda.synchronize()
    assert nnz.value == rows * cols and status == 2, (status, nnz.value, cn.lib().cn_last_error())
    del A
    torch.cuda.empty_cache()


def test_batch_products(dev):
    """The two products of the training step on a 2 % dense batch: X W = CSR(X) W and
    X^T E = CSR(X^T) E; against the dense kernels of this library, the fp64 product and the checker."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(8)
    X = _sparse(rng, 128, 6000, 0.02)
    W = rng.uniform(-0.01, 0.01, (6000, 2048)).astype(np.float32)
    E = rng.normal(0, 0.01, (128, 2048)).astype(np.float32)
    Xt, Wt, Et = _t(X, dev), _t(W, dev), _t(E, dev)
    Sx = L.csr_from_dense(Xt)
    S = L.csr_transpose(Sx)
    assert (S.rows, S.cols) == (6000, 128)
    fwd = L.csr_gemm(Sx, Wt).cpu().numpy()
    assert np.array_equal(_bits(fwd), _bits(oracle.csr_gemm(oracle.csr_from_dense(X), W)))
    ref = X.astype(np.float64) @ W.astype(np.float64)
    assert np.max(np.abs(fwd - ref)) <= gemm_tolerance(6000) * np.max(np.abs(ref))
    assert np.max(np.abs(fwd - cn.dot(Xt, Wt).cpu().numpy())) <= 2 * gemm_tolerance(6000) * np.max(np.abs(ref))
    grad = L.csr_gemm(S, Et).cpu().numpy()
    ref_g = X.T.astype(np.float64) @ E.astype(np.float64)
    assert np.max(np.abs(grad - ref_g)) <= gemm_tolerance(128) * np.max(np.abs(ref_g))
    assert np.array_equal(_bits(grad), _bits(oracle.csr_gemm(oracle.csr_from_dense(X, True), E)))


def test_shape_errors(dev):
    import torch
    from clusternet_amd import _lib as L
    S = L.csr_from_dense(torch.zeros((4, 5), device=dev))
    assert S.nnz == 0
    with pytest.raises(L.CnError):
        L.csr_gemm(S, torch.zeros((4, 3), device=dev))
    assert torch.equal(L.csr_gemm(S, torch.ones((5, 3), device=dev)), torch.zeros((4, 3), device=dev))
    T = L.csr_transpose(S)
    assert (T.rows, T.cols, T.nnz) == (5, 4, 0) and int(T.row_ptr.abs().sum()) == 0


def test_coded_entries_report_bad_arguments_and_handle_empty_matrices(dev):
    """Status codes of the fused entries through the C-ABI itself, and the all-zero matrix (every element
    encodes as 'zero', whose decoded value is +precision as in decompression_8bit)."""
    import ctypes
    import torch
    from clusternet_amd import _lib as L
    lib = L.lib()
    rng = np.random.default_rng(8)
    S = L.csr_from_dense(_t(_sparse(rng, 40, 16, 0.2), dev))
    B = torch.ones((16, 64), device=dev)
    prec = L.csr_gemm_absmax(S, B)
    codes = torch.empty((40, 64), dtype=torch.uint8, device=dev)
    w = torch.zeros((40, 64), device=dev)
    args = (40, 16, 64, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(), B.data_ptr(), 64)
    assert lib.cn_csr_gemm_coded_update(*args, None, codes.data_ptr(), w.data_ptr(), 64, 1.0, None) == 1       # NULL precision
    assert lib.cn_csr_gemm_coded_update(*args, prec.data_ptr(), None, w.data_ptr(), 64, 1.0, None) == 1        # NULL codes
    assert lib.cn_csr_gemm_coded_update(*args, prec.data_ptr(), codes.data_ptr(), w.data_ptr(), 32, 1.0, None) == 2  # ldw < N
    assert lib.cn_csr_gemm_coded_update(-1, 16, 64, *args[3:], prec.data_ptr(), codes.data_ptr(), None, 0, 1.0, None) == 2
    assert lib.cn_csr_gemm_coded_rmsprop(*args, prec.data_ptr(), codes.data_ptr(), None, w.data_ptr(), 64, 0.9, 0.1, None) == 1
    assert b"csr_gemm_coded_rmsprop" in ctypes.c_char_p(lib.cn_last_error()).value
    assert lib.cn_csr_gemm_f32_absmax(*args, None, 0, None, None) == 1                                          # nothing to produce
    # empty result: nothing is touched
    assert lib.cn_csr_gemm_coded_update(0, 16, 64, *args[3:], prec.data_ptr(), codes.data_ptr(), None, 0, 1.0, None) == 0
    # all-zero matrix with a positive precision: codes 254 throughout, weights move by alpha * precision
    Z = L.csr_from_dense(torch.zeros((40, 16), device=dev))
    one = torch.ones(1, device=dev)
    got = L.csr_gemm_coded_update(Z, B, one, w=w, alpha=0.5)
    assert int(got.min()) == 254 and int(got.max()) == 254
    assert torch.equal(w, torch.full((40, 64), 0.5, device=dev))


@pytest.mark.parametrize("seed", [5, 6])
def test_random_shapes_of_every_kernel_choice(dev, seed):
    """Shapes drawn at random over the three dispatch regimes (few long rows, many short rows, neither):
    product with maximum, maximum alone, bias + maxout in one call, codes with the weight update, each
    bit for bit against the checker."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(seed)
    for it in range(18):
        if it % 3 == 0:
            R, Cc = int(rng.integers(1, 129)), int(rng.integers(1, 1500))
            N = int(rng.choice([2048, 2052, 2304, 2820, 4100, 4612]))
            density = float(rng.choice([0.01, 0.05, 0.3]))
        elif it % 3 == 1:
            R, Cc, N = int(rng.integers(1, 3000)), int(rng.integers(1, 129)), int(rng.integers(1, 1200))
            density = float(rng.choice([0.0, 0.02, 0.1, 0.5]))
        else:
            R, Cc, N = int(rng.integers(1, 300)), int(rng.integers(1, 300)), int(rng.integers(1, 2500))
            density = float(rng.choice([0.02, 0.2]))
        case = "seed %d case %d: %d x %d times %d x %d, density %g" % (seed, it, R, Cc, Cc, N, density)
        S_dense = (rng.normal(0, 1, (R, Cc)) * (rng.random((R, Cc)) < density)).astype(np.float32)
        B = rng.normal(0, 1, (Cc, N)).astype(np.float32)
        S, Bd = L.csr_from_dense(_t(S_dense, dev)), _t(B, dev)
        want = oracle.csr_gemm(oracle.csr_from_dense(S_dense), B)
        peak = float(oracle.absmax(want))
        amax = torch.zeros(1, device=dev)
        got = L.csr_gemm(S, Bd, absmax_out=amax).cpu().numpy()
        assert np.array_equal(_bits(got), _bits(want)), case
        assert float(amax.cpu()[0]) == peak, case
        assert float(L.csr_gemm_absmax(S, Bd).cpu()[0]) == peak, case
        pools = [p for p in (2, 3, 4) if N % p == 0]
        if pools:
            pool = pools[it % len(pools)]
            v = rng.normal(0, 1, N).astype(np.float32)
            out, arg = L.csr_gemm_bias_maxout(S, Bd, _t(v, dev), pool)
            want_out, want_arg = oracle.maxout(oracle.add_row_vector(want, v), pool)
            assert np.array_equal(_bits(out.cpu().numpy()), _bits(want_out)), case
            assert np.array_equal(arg.cpu().numpy(), want_arg), case
        if peak > 0:
            w0 = rng.normal(0, 1, (R, N)).astype(np.float32)
            w = _t(w0.copy(), dev)
            codes = L.csr_gemm_coded_update(S, Bd, torch.full((1,), peak, device=dev), w=w, alpha=-0.01).cpu().numpy()
            want_codes = np.asarray(oracle.compress(want, np.float32(peak))).reshape(R, N)
            assert np.array_equal(codes, want_codes), case
            want_w = oracle.decompress_axpy(want_codes, np.float32(peak), np.float32(-0.01), w0)
            assert np.array_equal(_bits(w.cpu().numpy()), _bits(np.asarray(want_w).reshape(R, N))), case


@pytest.mark.parametrize("seed", [1, 2])
def test_dense_to_csr_on_random_shapes_strides_and_alignments(dev, seed):
    """The conversion reads rows with 16-byte loads when the base and the leading dimension allow it and
    element by element otherwise: shapes, paddings and one-element offsets drawn at random, segments that
    end inside a vector, each against the checker's arrays."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(100 + seed)
    for it in range(24):
        rows = int(rng.integers(1, 40))
        cols = int(rng.choice([1, 3, 4, 5, 63, 64, 255, 256, 257, 4095, 4096, 4097, 4100, 8191, 8192, 9001, 12289]))
        pad = int(rng.choice([0, 0, 1, 3, 4, 8]))
        shift = int(rng.choice([0, 0, 1, 2]))
        density = float(rng.choice([0.0, 0.01, 0.1, 0.6, 1.0]))
        case = "seed %d case %d: %d x %d, pad %d, shift %d, density %g" % (seed, it, rows, cols, pad, shift, density)
        A = (rng.normal(0, 1, (rows, cols)) * (rng.random((rows, cols)) < density)).astype(np.float32)
        A[rng.random((rows, cols)) < 0.01] = -0.0  # a negative zero is no nonzero
        store = torch.zeros(rows * (cols + pad) + shift, device=dev)
        view = store[shift:].view(rows, cols + pad)[:, :cols]
        view.copy_(_t(A, dev))
        for transpose in (False, True):
            S = L.csr_from_dense(view, transpose=transpose)
            rp, ci, va = oracle.csr_from_dense(A, transpose=transpose)
            assert np.array_equal(S.row_ptr.cpu().numpy(), rp), case
            assert np.array_equal(S.col_idx.cpu().numpy(), ci), case
            assert np.array_equal(_bits(S.vals.cpu().numpy()), _bits(va)), case


def test_prefix_sums_keep_their_total_in_64_bits(dev):
    """The CSR builders size their outputs from a prefix sum whose total decides whether the 32-bit row pointers can be
    used at all.  On synthetic counts: the prefix sums against numpy's on both forms of the scan (one workgroup; block
    sums, their scan, blocks), the total exact when it passes 2^31 (3e9 from entries of a million and from a million
    entries), and at least 2^31 - 1 when a single block of 4096 entries alone passes it, so that no overflow can
    wrap round to a small total that the callers would accept."""
    import ctypes as C
    import torch
    import clusternet_amd as cn
    L = cn.lib()
    L.cn_host_exclusive_scan.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.POINTER(C.c_int64)]
    L.cn_host_exclusive_scan.restype = C.c_int

    def scan(counts):
        c = torch.from_numpy(counts.astype(np.int32)).to(dev)
        out = torch.empty(counts.size + 1, dtype=torch.int32, device=dev)
        total = C.c_int64(-1)
        assert L.cn_host_exclusive_scan(c.data_ptr(), counts.size, out.data_ptr(), C.byref(total)) == 0
        return out.cpu().numpy(), total.value

    rng = np.random.default_rng(5)
    for n in (1, 255, 256, 257, 5000, 8192, 8193, 100_000, 1_000_003):
        counts = rng.integers(0, 2000, n)
        sums, total = scan(counts)
        want = np.concatenate([[0], np.cumsum(counts)])
        assert total == want[-1] and np.array_equal(sums, want.astype(np.int32)), n
    assert scan(np.full(3000, 1_000_000))[1] == 3_000_000_000          # one workgroup, entries of a million
    assert scan(np.full(1_000_000, 3000))[1] == 3_000_000_000          # a million entries through block sums
    assert scan(np.full(100_000, 600_000))[1] >= 2 ** 31 - 1           # every block of 4096 entries passes 2^31 by itself
    mixed = np.zeros(50_000, np.int64)
    mixed[10_000:14_096] = 600_000                                      # one such block among empty ones
    assert scan(mixed)[1] >= 2 ** 31 - 1
