"""Parity of the fused update passes with the CPU checker and with the unfused kernels they replace,
through the C-ABI.  Everything here is bit-exact: each pass performs the same fp32 operations in
the same order as decompression followed by the element-wise step."""
import numpy as np
import pytest

import oracle

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("codec_form")]


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 1023, 4096, 4097, 1_000_003])
@pytest.mark.parametrize("alpha", [1.0, -1.0, -0.01])
def test_decompress_axpy_matches_checker(dev, n, alpha):
    import clusternet_amd as cn
    rng = np.random.default_rng(n + 7)
    codes = rng.integers(0, 256, n, dtype=np.uint8)
    y = rng.normal(0, 1, n).astype(np.float32)
    prec = 0.0371
    want = oracle.decompress_axpy(codes, prec, alpha, y)
    got = cn.decompression_8bit_axpy(_t(codes, dev), prec, alpha, _t(y, dev)).cpu().numpy()
    assert np.array_equal(_bits(got), _bits(want))


def test_decompress_axpy_equals_the_unfused_kernels_and_takes_device_precision(dev):
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    n = 8_388_608 + 5
    x = torch.randn(n, device=dev, generator=gen) * 0.02
    w = torch.randn(n, device=dev, generator=gen)
    prec = cn.absmax(x)                              # one-element device tensor
    codes = cn.compression_8bit(x, prec)
    rate = 0.0125
    w_ref = w.clone()
    L.sgd_update(w_ref, cn.decompression_8bit(codes, prec), rate)
    w_fused = cn.decompression_8bit_axpy(codes, prec, -rate, w.clone())
    assert torch.equal(w_ref.view(torch.int32), w_fused.view(torch.int32))
    acc = w.clone()
    acc_ref = acc + cn.decompression_8bit(codes, prec)   # accumulation of a peer's gradient
    cn.decompression_8bit_axpy(codes, float(prec.cpu()[0]), 1.0, acc)
    assert torch.equal(acc_ref.view(torch.int32), acc.view(torch.int32))
    # unaligned views take the scalar path
    w2 = w.clone()
    cn.decompression_8bit_axpy(codes[1:], prec, -rate, w2[1:])
    assert torch.equal(w2[1:].view(torch.int32), w_ref[1:].view(torch.int32)) and w2[0] == w[0]


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 1023, 4096, 4097, 1_000_003, 8_388_608 + 6, (1 << 26) + 2 * 16384 + 7])
@pytest.mark.parametrize("prec", [0.0371, 1e-30, 0.0])
def test_compress_axpy_is_compress_then_decompress_axpy(dev, n, prec):
    """Codes and updated array of the one-pass kernel against the two kernels it replaces and, for the
    sizes the checker finishes quickly, against the checker.  A precision of 1e-30 or 0 takes the
    encoder's search instead of its table.  The largest size is beyond the cache and takes the form that draws
    its tiles from a counter."""
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(n + 3)
    x = rng.normal(0, 0.01, n).astype(np.float32)
    if n > 8:
        x[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-38, -0.0371, 0.0371]
    y = rng.normal(0, 1, n).astype(np.float32)
    alpha = -0.0125
    xd, yd = _t(x, dev), _t(y, dev)
    want_codes = cn.compression_8bit(xd, prec)
    want_y = cn.decompression_8bit_axpy(want_codes, prec, alpha, yd.clone())
    got_y = yd.clone()
    got_codes = cn.compression_8bit_axpy(xd, prec, alpha, got_y)
    assert torch.equal(got_codes, want_codes)
    assert torch.equal(got_y.view(torch.int32), want_y.view(torch.int32))
    if n <= 1_000_003:
        host_codes = oracle.compress(x, prec)
        assert np.array_equal(got_codes.cpu().numpy(), host_codes)
        assert np.array_equal(_bits(got_y.cpu().numpy()), _bits(oracle.decompress_axpy(host_codes, prec, alpha, y)))
    # the precision on the device, and views that are not 16-byte aligned
    if n > 1:
        p_dev = torch.tensor([prec], dtype=torch.float32, device=dev)
        y2 = yd.clone()
        c2 = torch.zeros(n, dtype=torch.uint8, device=dev)
        cn.compression_8bit_axpy(xd[1:], p_dev, alpha, y2[1:], out=c2[1:])
        assert torch.equal(c2[1:], want_codes[1:]) and int(c2[0]) == 0
        assert torch.equal(y2[1:].view(torch.int32), want_y[1:].view(torch.int32))
        assert _bits(y2[:1].cpu().numpy())[0] == _bits(y[:1])[0]


def test_compress_axpy_rejects_null(dev):
    from clusternet_amd import _lib
    L = _lib.lib()
    assert L.cn_compress_8bit_axpy(None, 1.0, 4, None, 1.0, None, None) == 1
    assert L.cn_compress_8bit_axpy_dp(None, None, 4, None, 1.0, None, None) == 1
    assert L.cn_compress_8bit_axpy(None, 1.0, 0, None, 1.0, None, None) == 0


@pytest.mark.parametrize("n", [0, 1, 5, 4099, 1_000_003])
def test_rmsprop_update_matches_checker(dev, n):
    import clusternet_amd as cn
    rng = np.random.default_rng(n + 3)
    g = (rng.normal(0, 0.05, n) * (rng.random(n) < 0.9)).astype(np.float32)
    rms = rng.uniform(0, 0.01, n).astype(np.float32)
    rms[::7] = 0.0
    w = rng.normal(0, 0.05, n).astype(np.float32)
    for mult, lr in ((0.9, 0.003), (0.0, 0.1), (1.0, 0.01)):
        r_want, w_want = oracle.rmsprop_update(rms, g, w, mult, lr)
        r_t, w_t = _t(rms, dev), _t(w, dev)
        cn.rmsprop_update(r_t, _t(g, dev), w_t, mult, lr)
        assert np.array_equal(_bits(r_t.cpu().numpy()), _bits(r_want))
        assert np.array_equal(_bits(w_t.cpu().numpy()), _bits(w_want))


def test_rmsprop_update_on_codes_equals_decompress_then_update(dev):
    import torch
    import clusternet_amd as cn
    gen = torch.Generator(device=dev)
    gen.manual_seed(12)
    n = 4_194_304 + 3
    x = torch.randn(n, device=dev, generator=gen) * 0.02
    w = torch.randn(n, device=dev, generator=gen) * 0.05
    rms = torch.rand(n, device=dev, generator=gen) * 0.01
    prec = cn.absmax(x)
    codes = cn.compression_8bit(x, prec)
    r_ref, w_ref = rms.clone(), w.clone()
    cn.rmsprop_update(r_ref, cn.decompression_8bit(codes, prec), w_ref, 0.9, 0.003)
    for p in (prec, float(prec.cpu()[0])):
        r_f, w_f = rms.clone(), w.clone()
        cn.rmsprop_update(r_f, codes, w_f, 0.9, 0.003, precision=p)
        assert torch.equal(r_ref.view(torch.int32), r_f.view(torch.int32))
        assert torch.equal(w_ref.view(torch.int32), w_f.view(torch.int32))
    # and against the checker on a slice
    k = 100_000
    r_want, w_want = oracle.rmsprop_update(rms[:k].cpu().numpy(), oracle.decompress(codes[:k].cpu().numpy(), float(prec.cpu()[0])),
                                           w[:k].cpu().numpy(), 0.9, 0.003)
    assert np.array_equal(_bits(r_ref[:k].cpu().numpy()), _bits(r_want))
    assert np.array_equal(_bits(w_ref[:k].cpu().numpy()), _bits(w_want))


def test_null_and_size_errors(dev):
    import clusternet_amd as cn
    L = cn.lib()
    assert L.cn_decompress_8bit_axpy(None, 1.0, 1.0, 4, None, None) == 1
    assert L.cn_rmsprop_update_f32(None, None, None, 0.9, 0.1, 4, None) == 1
    assert L.cn_decompress_8bit_axpy(None, 1.0, 1.0, 0, None, None) == 0


def test_tensors_beyond_the_cache_take_drawn_tiles_and_give_the_same_bits(dev, codec_form):
    """From 2^26 elements on the update passes run as a persistent grid that draws its tiles from a counter.  Each is
    held to the same call made on pieces below that size (the workgroup-per-tile form, which the tests above hold to
    the CPU checker), on a size that ends in a partial tile and an n % 4 tail, twice in a row: the second call
    finds the counter as the first one left it."""
    if codec_form != "literal_for_small_tensors":
        pytest.skip("no compression in this test; one run is enough")
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    n = (1 << 26) + 3 * 4096 + 7
    cut = (1 << 25) + 4 * 1000  # pieces: 16-byte aligned starts, both below 2^26
    g = torch.randn(n, device=dev, generator=gen) * 0.02
    w0 = torch.randn(n, device=dev, generator=gen)
    r0 = torch.rand(n, device=dev, generator=gen)
    codes = torch.randint(0, 256, (n,), dtype=torch.uint8, device=dev, generator=gen)

    def pieces(fn, *arrays):
        for lo, hi in ((0, cut), (cut, n)):
            fn(*[a[lo:hi] for a in arrays])

    def same(a, b):
        return torch.equal(a.view(torch.int32), b.view(torch.int32))

    for _ in range(2):
        # flat passes
        w, ref = w0.clone(), w0.clone()
        L.sgd_update(w, g, 0.0125)
        pieces(lambda a, b: L.sgd_update(a, b, 0.0125), ref, g)
        assert same(w, ref)
        assert same(w, w0 - 0.0125 * g)
        out, ref = torch.empty_like(g), torch.empty_like(g)
        L.sub(w0, g, out)
        assert same(out, w0 - g)
        # decode + add
        w, ref = w0.clone(), w0.clone()
        cn.decompression_8bit_axpy(codes, 0.37, -0.5, w)
        pieces(lambda c, y: cn.decompression_8bit_axpy(c, 0.37, -0.5, y), codes, ref)
        assert same(w, ref)
        # RMSprop on a fp32 gradient and on codes
        for grad, prec in ((g, None), (codes, 0.37)):
            w, r, wref, rref = w0.clone(), r0.clone(), w0.clone(), r0.clone()
            cn.rmsprop_update(r, grad, w, 0.9, 0.001, precision=prec)
            pieces(lambda rr, gg, ww: cn.rmsprop_update(rr, gg, ww, 0.9, 0.001, precision=prec), rref, grad, wref)
            assert same(w, wref) and same(r, rref)
    assert L.lib().cn_host_tile_counters_in_use() == 0  # every kernel that drew tiles left its counter at zero
