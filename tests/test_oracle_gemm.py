"""Pins the CPU GEMM checker against the reference's own known-answer tests (no GPU needed).

Literals come from tests/clusterNet_test.cu of the reference: :22-23 (operands), :72-75 (dot),
:111-119 and :125-128 (Tdot), :161-164 (dotT), :257-276 (0.3 x 1.1748345 all-constant product),
:338-394 (all-ones closed forms 8783, 317, 17).  The reference compares with exact float
equality; sequential-k fp32 FMA accumulation reproduces every literal bit for bit.
"""
import numpy as np

import oracle

M1 = np.array([[0, 2, 3], [0, 0.83, 59.1387]], np.float32)
M2 = np.array([[17, 0], [3, 4], [0, 0]], np.float32)
f32 = lambda rows: np.array(rows, np.float32)


def test_reference_kats_exact_with_seqfma():
    assert np.array_equal(oracle.gemm(M1, M2, mode="seqfma"), f32([[6, 8], [2.49, 3.32]]))
    assert np.array_equal(oracle.gemm(M1, M1, ta=True, mode="seqfma"),
                          f32([[0, 0, 0], [0, 4.6889, 55.085117], [0, 55.085117, 3506.385742]]))
    assert np.array_equal(oracle.gemm(M2, M2, ta=True, mode="seqfma"), f32([[298, 12], [12, 16]]))
    assert np.array_equal(oracle.gemm(M1, M1, tb=True, mode="seqfma"),
                          f32([[13, 179.0761], [179.0761, 3498.074463]]))


def test_reference_kats_f64acc_within_one_ulp():
    for got, want in (
        (oracle.gemm(M1, M2), f32([[6, 8], [2.49, 3.32]])),
        (oracle.gemm(M1, M1, ta=True), f32([[0, 0, 0], [0, 4.6889, 55.085117],
                                           [0, 55.085117, 3506.385742]])),
        (oracle.gemm(M1, M1, tb=True), f32([[13, 179.0761], [179.0761, 3498.074463]])),
    ):
        np.testing.assert_allclose(got, want, rtol=1.2e-7, atol=0)


def test_all_ones_closed_forms():
    assert np.all(oracle.gemm(np.ones((111, 8783), np.float32), np.ones((8783, 317), np.float32)) == 8783.0)
    # dotT(m3 17x317, m1 8783x317) -> 17 x 8783 of 317
    assert np.all(oracle.gemm(np.ones((17, 317), np.float32), np.ones((8783, 317), np.float32), tb=True) == 317.0)
    assert np.all(oracle.gemm(np.ones((8783, 17), np.float32), np.ones((17, 317), np.float32)) == 17.0)


def test_constant_product():
    a = np.full((200, 400), 0.3, np.float32)
    b = np.full((400, 800), np.float32(1.0) + np.float32(0.1748345), np.float32)
    c = oracle.gemm(a, b)
    want = np.float32(400 * float(np.float32(0.3)) * float(b[0, 0]))
    assert c.shape == (200, 800) and np.all(c == want)


def test_transpose_identities_and_numpy_cross_check():
    rng = np.random.default_rng(0)
    A = rng.uniform(0, 1, (37, 53)).astype(np.float32)
    B = rng.normal(0, 1, (53, 29)).astype(np.float32)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    assert np.array_equal(oracle.gemm(A, B), want)
    assert np.array_equal(oracle.gemm(np.ascontiguousarray(A.T), B, ta=True), want)
    assert np.array_equal(oracle.gemm(A, np.ascontiguousarray(B.T), tb=True), want)
    np.testing.assert_allclose(oracle.gemm(A, B, mode="seqfma"), want, rtol=2e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.port_gemm_nn(A, B), want, rtol=2e-5, atol=1e-5)
    C, Cabs = oracle.gemm_with_abs(A, B)
    np.testing.assert_allclose(C, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-12)
    np.testing.assert_allclose(Cabs, np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64), rtol=1e-12)
    cols = np.array([0, 5, 28])
    Cc, _ = oracle.gemm_cols(A, B, cols)
    np.testing.assert_allclose(Cc, C[:, cols], rtol=1e-12)


def test_w8_gemm_is_gemm_of_decoded_weights():
    rng = np.random.default_rng(2)
    A = rng.normal(0, 1, (9, 40)).astype(np.float32)
    W = rng.integers(0, 256, (40, 13), dtype=np.uint8)
    assert np.array_equal(oracle.gemm_w8(A, W, 0.37), oracle.gemm(A, oracle.decompress(W, 0.37)))


def test_training_step_helpers_brute_force():
    rng = np.random.default_rng(4)
    A = rng.normal(0, 1, (7, 12)).astype(np.float32)
    v = rng.normal(0, 1, 12).astype(np.float32)
    assert np.array_equal(oracle.add_row_vector(A, v), A + v[None, :])
    for pool in (2, 3, 4):
        out, arg = oracle.maxout(A, pool)
        blocks = A.reshape(7, 12 // pool, pool)
        assert np.array_equal(out, blocks.max(axis=2))
        assert np.array_equal(arg, (blocks.argmax(axis=2) + np.arange(12 // pool)[None, :] * pool).astype(np.float32))
        err = rng.normal(0, 1, out.shape).astype(np.float32)
        g = oracle.expand_to_maxout_grad(err, arg, pool)
        want = np.zeros_like(A)
        for r in range(7):
            for o in range(12 // pool):
                want[r, int(arg[r, o])] = err[r, o]
        assert np.array_equal(g, want)
    s = oracle.softmax(np.zeros((5, 10), np.float32))
    assert np.allclose(s, 0.1)
    s = oracle.softmax(A)
    np.testing.assert_allclose(s.sum(axis=1), 1.0, rtol=1e-6)
    e = np.exp(A.astype(np.float64) - A.max(axis=1, keepdims=True))
    np.testing.assert_allclose(s, e / e.sum(axis=1, keepdims=True), rtol=1e-6)


def test_blocked_and_plain_loops_give_the_same_bits():
    """gemm_with_abs streams B by rows in blocks (B stored K x N); gemm_cols is the plain triple loop.  Every output adds its
    products in ascending k either way, so the fp64 results must agree bit for bit, also across block borders (8 rows,
    2048 columns) and for A stored K x M."""
    rng = np.random.default_rng(21)
    for M, N, K, ta in ((19, 2051, 300, False), (8, 4100, 33, True), (1, 1, 1, False)):
        A = rng.normal(size=(K, M) if ta else (M, K)).astype(np.float32)
        B = rng.normal(size=(K, N)).astype(np.float32)
        C, Cabs = oracle.gemm_with_abs(A, B, ta, False)
        P, Pabs = oracle.gemm_cols(A, B, np.arange(N), ta, False)
        assert np.array_equal(C.view(np.uint64), P.view(np.uint64)) and np.array_equal(Cabs.view(np.uint64), Pabs.view(np.uint64))


def test_cpu_port_gemm_all_transpositions_and_accumulation():
    """The multi-threaded port timed as the CPU baseline: every transposition against the fp64 yard-stick, and a product
    accumulated over row blocks of B (how the baseline streams a 16 GB weight matrix) against the product in one go."""
    rng = np.random.default_rng(33)
    M, N, K = 37, 700, 515
    for ta in (False, True):
        for tb in (False, True):
            A = rng.uniform(0, 1, (K, M) if ta else (M, K)).astype(np.float32)
            B = rng.normal(0, 0.05, (N, K) if tb else (K, N)).astype(np.float32)
            ref, refabs = oracle.gemm_with_abs(A, B, ta, tb)
            got = oracle.port_gemm(A, B, ta, tb)
            assert float((np.abs(got - ref) / refabs).max()) <= 1e-5, (ta, tb)
    A = rng.uniform(0, 1, (M, K)).astype(np.float32)
    B = rng.normal(0, 0.05, (K, N)).astype(np.float32)
    whole = oracle.port_gemm(A, B)
    acc = np.zeros((M, N), np.float32)
    for k0 in range(0, K, 128):   # the port's own K slabs: the accumulated product adds in the same order
        oracle.port_gemm(A[:, k0:k0 + 128], B[k0:k0 + 128], out=acc, accumulate=True, lda=K)
    assert np.array_equal(whole.view(np.uint32), acc.view(np.uint32))


def test_dot8bit_restatement_is_pinned_by_closed_forms():
    """The reference has no test of dot8bit / dot8bit_shared, so the restatement of kDot8bit
    (source/clusterKernels.cu:1717-1762) is held to what its source lines fix:
      * the special codes of the two tables, read off :1731-1738 (126 -> 0, 254 -> -0 in both; 127 -> precisionA in A and
        -precisionA in B; 255 -> precisionB in A and -precisionB in B), and the ordinary entries against the codec's
        decode table (same t[i] * precision, :1727-1730 against :1141-1146);
      * constant operands: K equal products, exact when they are powers of two;
      * a row of A with one code that decodes to non-zero among codes that decode to zero picks out a decoded row of B,
        scaled, bit for bit, and adds it to what out held;
      * linearity in out (out + P from zero equals out0 + P to one rounding) and the fp64 product of the decoded
        operands within the bound of a K-term fp32 sum."""
    pa, pb = 0.75, 2.5
    ta, tb = oracle.dot8bit_tables(pa, pb)
    assert ta[126] == 0 and not np.signbit(ta[126]) and tb[126] == 0 and not np.signbit(tb[126])
    assert ta[254] == 0 and np.signbit(ta[254]) and tb[254] == 0 and np.signbit(tb[254])
    assert (ta[127], tb[127], ta[255], tb[255]) == (np.float32(pa), np.float32(-pa), np.float32(pb), np.float32(-pb))
    la, lb = oracle.decode_lut(pa), oracle.decode_lut(pb)
    ordinary = np.r_[0:126, 128:254]
    assert np.array_equal(ta[ordinary].view(np.uint32), la[ordinary].view(np.uint32))
    assert np.array_equal(tb[ordinary].view(np.uint32), lb[ordinary].view(np.uint32))
    # constant operands: codes 127 (A: 0.75) and 255 (B: -2.5), K = 16 -> 16 * -1.875 = -30 exactly
    out, mag = oracle.dot8bit(np.full((3, 16), 127, np.uint8), np.full((16, 5), 255, np.uint8), pa, pb)
    assert np.all(out == np.float32(-30.0)) and np.all(mag == 30.0)
    # one-hot rows: row m of A holds code 127 (-> pa) at k = m and 126 / 254 (-> +0 / -0) elsewhere
    rng = np.random.default_rng(8)
    K, N = 40, 33
    B = rng.integers(0, 256, (K, N)).astype(np.uint8)
    A = np.where(rng.random((K, K)) < 0.5, 126, 254).astype(np.uint8)
    A[np.arange(K), np.arange(K)] = 127
    out0 = rng.normal(size=(K, N)).astype(np.float32)
    out, _ = oracle.dot8bit(A, B, pa, pb, out0)
    want = out0 + np.float32(pa) * tb[B]          # a single product and a single addition per output, both fp32
    assert np.array_equal(out.view(np.uint32), want.astype(np.float32).view(np.uint32))
    # general case against the fp64 product of the decoded operands
    M, K, N = 37, 150, 29
    A = rng.integers(0, 256, (M, K)).astype(np.uint8)
    B = rng.integers(0, 256, (K, N)).astype(np.uint8)
    out0 = rng.normal(size=(M, N)).astype(np.float32)
    out, mag = oracle.dot8bit(A, B, pa, pb, out0)
    ref = out0.astype(np.float64) + ta[A].astype(np.float64) @ tb[B].astype(np.float64)
    # the magnitudes are sums of the fp32 products: equal to the fp64 ones to the rounding of a product
    assert np.allclose(mag, np.abs(ta[A].astype(np.float64)) @ np.abs(tb[B].astype(np.float64)), rtol=2.0 ** -23)
    assert float((np.abs(out - ref) / (mag + np.abs(out0))).max()) <= K * 2.0 ** -24
    from_zero, _ = oracle.dot8bit(A, B, pa, pb)
    assert float((np.abs(out - (out0 + from_zero)) / (mag + np.abs(out0))).max()) <= K * 2.0 ** -24
