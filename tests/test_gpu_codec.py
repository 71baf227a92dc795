"""Bit-exact parity of the HIP codec kernels with the CPU checker, through the C-ABI."""
import numpy as np
import pytest

import oracle
from util import cfg2_tensor

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


def _adversarial():
    t = oracle.table()
    pts = [t, np.nextafter(t, np.float32(0)), np.nextafter(t, np.float32(2))]
    mids = ((t[:-1].astype(np.float64) + t[1:].astype(np.float64)) / 2).astype(np.float32)
    for k in range(-3, 4):
        pts.append((mids.view(np.uint32).astype(np.int64) + k).astype(np.uint32).view(np.float32))
    for thr in (np.float32(0.0000015), np.float32(0.995703), np.float32(1.0), t[125]):
        b = int(np.array([thr]).view(np.uint32)[0])
        pts.append(np.arange(b - 8, b + 9, dtype=np.uint32).view(np.float32))
    pts.append(np.array([0.0, -0.0, 1e-45, 1e-38, 1.1754944e-38, 0.5, 0.25, 0.1, 0.01, 0.001, 0.993,
                         0.9957, 0.9958, 1.0, 1.5, 3e38, np.inf, np.nan], np.float32))
    x = np.concatenate([np.asarray(p, np.float32).reshape(-1) for p in pts])
    return np.concatenate([x, -x])


def test_absmax_matches_numpy(dev):
    import clusternet_amd as cn
    rng = np.random.default_rng(0)
    for n in (1, 2, 3, 5, 63, 64, 4095, 4096, 4097, 128 * 40000, 10_000_019):
        x = rng.normal(0, 1, n).astype(np.float32)
        got = float(cn.absmax(_t(x, dev)).cpu()[0])
        assert got == float(np.abs(x).max()) == oracle.absmax(x), n
    # unaligned start, empty input, NaN propagation, repeated calls reuse the scratch correctly
    x = rng.normal(0, 1, 100_001).astype(np.float32)
    xt = _t(x, dev)
    for off in (1, 2, 3):
        assert float(cn.absmax(xt[off:]).cpu()[0]) == float(np.abs(x[off:]).max())
    assert float(cn.absmax(xt[:0]).cpu()[0]) == -1.0
    x[777] = np.nan
    assert np.isnan(float(cn.absmax(_t(x, dev)).cpu()[0]))
    for _ in range(3):
        assert float(cn.absmax(xt).cpu()[0]) == oracle.absmax(xt.cpu().numpy())


def test_reductions_with_and_without_writer_fences(dev):
    """The single-launch reductions order a workgroup's partial result and its arrival count by a data dependence
    (the last workgroup acquires); cn_host_reduction_fences switches the writers to a release fence, the form the
    memory model prescribes.  Both forms must give the same bits, over grid sizes from one workgroup to the cap,
    and on repeated calls (every ticket word is put back to zero by the last to arrive)."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(123)
    x = rng.normal(0, 3, 6_000_011).astype(np.float32)
    xt = _t(x, dev)
    want_codes = {}
    try:
        for n in (1, 4096, 4097, 70_000, 1_000_003, 6_000_011, 1_000_000):
            want_max = float(np.abs(x[:n]).max())
            want_sum = None
            for per_cu in (0, 1, 3, 16):
                L.lib().cn_host_codec_workgroups_per_cu(per_cu)
                for fenced in (0, 1, 0):
                    L.lib().cn_host_reduction_fences(fenced)
                    assert float(cn.absmax(xt[:n]).cpu()[0]) == want_max, (n, per_cu, fenced)
                    assert float(L.reduce_max(xt[:n]).cpu()[0]) == max(float(x[:n].max()), -1.0), (n, per_cu, fenced)
                    got = float(L.reduce_sum(xt[:n]).cpu()[0])
                    want_sum = got if want_sum is None else want_sum
                    assert got == want_sum, (n, per_cu, fenced)
                    # abs-max -> compression as one launch shares the ticket lines and honours the same switch
                    if per_cu == 0 and n % 4 == 0:
                        L.lib().cn_host_absmax_compress_single_launch(1)
                        prec_out = torch.zeros(1, device=dev)
                        codes, _ = cn.absmax_compression_8bit(xt[:n], precision_out=prec_out)
                        L.lib().cn_host_absmax_compress_single_launch(-1)
                        assert float(prec_out.cpu()[0]) == want_max, (n, fenced)
                        if want_codes.get(n) is None:
                            want_codes[n] = oracle.compress(x[:n], want_max)
                        assert np.array_equal(codes.cpu().numpy(), want_codes[n]), (n, fenced)
            assert abs(want_sum - float(x[:n].astype(np.float64).sum())) <= 1e-6 * np.abs(x[:n]).astype(np.float64).sum()
    finally:
        L.lib().cn_host_reduction_fences(0)
        L.lib().cn_host_codec_workgroups_per_cu(0)
        L.lib().cn_host_absmax_compress_single_launch(-1)


def test_compress_config2_bit_exact(dev):
    import clusternet_amd as cn
    x = cfg2_tensor(np.random.default_rng(42))
    xt = _t(x, dev)
    prec_dev = cn.absmax(xt)
    prec = float(prec_dev.cpu()[0])
    assert prec == float(np.abs(x).max())
    want = oracle.compress(x, prec, 0)
    got = cn.compression_8bit(xt, prec).cpu().numpy()
    assert got.dtype == np.uint8 and got.shape == x.shape
    assert np.array_equal(got, want)
    # precision taken from device memory gives the same codes
    assert np.array_equal(cn.compression_8bit(xt, prec_dev).cpu().numpy(), want)
    # decompression, both ways of passing the precision
    back = cn.decompression_8bit(_t(want, dev), prec).cpu().numpy()
    assert np.array_equal(back.view(np.uint32), oracle.decompress(want, prec).view(np.uint32))
    back2 = cn.decompression_8bit(_t(want, dev), prec_dev).cpu().numpy()
    assert np.array_equal(back2.view(np.uint32), back.view(np.uint32))


@pytest.mark.parametrize("prec", [1.0, 0.1, 0.5, 2.0, 3.7, 1e-3, 1e3, -1.0, 1e-30, 1e30, 1e-42,
                                  0.0, float("inf"), float("nan")])
def test_compress_adversarial_inputs(dev, prec):
    import clusternet_amd as cn
    x = _adversarial()
    with np.errstate(all="ignore"):
        scale = np.float32(prec) if np.isfinite(prec) and prec != 0 else np.float32(1.0)
        xs = (x * scale).astype(np.float32)
        want = oracle.compress(xs, prec, 0)
    got = cn.compression_8bit(_t(xs, dev), prec).cpu().numpy()
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (prec, xs[bad[:5]], got[bad[:5]], want[bad[:5]])


def test_compress_sizes_and_alignment(dev):
    import clusternet_amd as cn
    rng = np.random.default_rng(5)
    base = rng.normal(0, 0.3, 70_000).astype(np.float32)
    bt = _t(base, dev)
    for n in (0, 1, 2, 3, 4, 5, 7, 255, 256, 1023, 1024, 4095, 4096, 4097, 16385, 65_537):
        for off in (0, 1, 2, 3):
            x = base[off:off + n]
            got = cn.compression_8bit(bt[off:off + n], 0.9).cpu().numpy()
            assert np.array_equal(got, oracle.compress(x, 0.9, 0)), (n, off)
    codes = rng.integers(0, 256, 70_000, dtype=np.uint8)
    ct = _t(codes, dev)
    for n in (0, 1, 3, 4, 5, 1023, 4096, 4099, 65_537):
        for off in (0, 1, 2, 3):
            got = cn.decompression_8bit(ct[off:off + n], 0.37).cpu().numpy()
            want = oracle.decompress(codes[off:off + n], 0.37)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n, off)


def test_decompress_every_code(dev):
    import clusternet_amd as cn
    codes = np.arange(256, dtype=np.uint8)
    for prec in (1.0, 0.1, 0.0234, 17.0, 1e-20, -2.0):
        got = cn.decompression_8bit(_t(codes, dev), prec).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), oracle.decode_lut(prec).view(np.uint32))
        assert got[254] == np.float32(prec)  # the "zero" code decodes to +precision


def test_compress_exhaustive_over_the_table_range(dev):
    """Every fp32 pattern from 2^-25 to just above 1, both signs, at precision 1."""
    import torch
    import clusternet_amd as cn
    lo, hi = 0x33000000, 0x3f900000
    step = 1 << 26
    for start in range(lo, hi, step):
        mags = np.arange(start, min(start + step, hi), dtype=np.uint32)
        want = oracle.port_compress(mags.view(np.float32), 1.0)
        xt = _t(mags.view(np.float32), dev)
        got = cn.compression_8bit(xt, 1.0)
        assert np.array_equal(got.cpu().numpy(), want), hex(start)
        neg = cn.compression_8bit(-xt, 1.0)
        expect_neg = torch.where(got == 254, got, got | 0x80)
        assert torch.equal(neg, expect_neg), hex(start)


def test_compress_random_precisions(dev):
    import clusternet_amd as cn
    rng = np.random.default_rng(77)
    for prec in list(rng.uniform(1e-4, 50, 6)) + [2.0 ** -40, 2.0 ** 40]:
        x = (np.exp(rng.uniform(np.log(1e-7), np.log(1.3), 2_000_000)) * prec).astype(np.float32)
        x *= rng.choice([-1.0, 1.0], x.size).astype(np.float32)
        got = cn.compression_8bit(_t(x, dev), float(prec)).cpu().numpy()
        assert np.array_equal(got, oracle.port_compress(x, float(prec))), prec


def test_compress_many_precisions_of_every_kind(dev):
    """Sixty precisions drawn over sixty decades, of either sign, exact powers of two and values next to the
    smallest normal number: each builds its own encoder table on the device (the steps of the code function
    are carried over from precision 1 through the division), and the codes of 2^18 inputs spread over the
    coded range must be those of the literal procedure."""
    import clusternet_amd as cn
    rng = np.random.default_rng(2026)
    n = 1 << 18
    for it in range(60):
        kind = it % 5
        if kind == 0:
            p = np.exp(rng.uniform(np.log(1e-30), np.log(1e30)))
        elif kind == 1:
            p = -np.exp(rng.uniform(np.log(1e-6), np.log(1e3)))
        elif kind == 2:
            p = 2.0 ** int(rng.integers(-100, 100))
        elif kind == 3:
            p = rng.uniform(0.001, 10)
        else:
            p = np.exp(rng.uniform(np.log(1e-38), np.log(1e-30)))
        p = float(np.float32(p))
        mag = np.exp(rng.uniform(np.log(1e-7), np.log(1.5), n)).astype(np.float32) * np.float32(abs(p))
        x = (mag * rng.choice(np.array([-1.0, 1.0], np.float32), n)).astype(np.float32)
        x[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, p]
        got = cn.compression_8bit(_t(x, dev), p).cpu().numpy()
        assert np.array_equal(got, oracle.compress(x, p)), p


def test_large_tensor_by_tiling(dev):
    """A 1.07e9-element tensor (4.3 GB) built by repeating a block whose codes are verified on the
    CPU: every repetition must carry the same codes, and decoding must repeat likewise."""
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(9)
    block = cfg2_tensor(rng, 1, 1 << 20).reshape(-1)
    block[123] = 0.75  # make sure max is not unique-position dependent
    prec = float(np.abs(block).max())
    want = oracle.port_compress(block, prec)
    reps = 1024
    big = _t(block, dev).repeat(reps)
    assert big.numel() == reps << 20
    assert float(cn.absmax(big).cpu()[0]) == prec
    codes = cn.compression_8bit(big, prec)
    wt = _t(want, dev)
    assert torch.equal(codes.view(reps, -1), wt.unsqueeze(0).expand(reps, -1))
    del big
    back = cn.decompression_8bit(codes, prec)
    bt = _t(oracle.decompress(want, prec), dev)
    assert torch.equal(back.view(reps, -1).view(torch.int32), bt.view(torch.int32).unsqueeze(0).expand(reps, -1))


def test_streaming_forms_ragged_sizes_offsets_and_fallback(dev):
    """Compression of 2^24 elements and more takes the streaming kernel, and decompression a workgroup per tile; in both
    the last tile is bounded by a buffer descriptor instead of a per-element test: sizes round a tile boundary, tails of 1 to 3
    elements, starts that are not 16-byte aligned (which fall back to the element-wise kernel), and a precision for
    which no table can be built (the literal procedure per element), all against the CPU checker."""
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(31)
    base_n = (1 << 24) + 12288 * 3 + 64
    mag = np.exp(rng.uniform(np.log(1e-7), np.log(1.3), base_n)).astype(np.float32)
    base = (mag * rng.choice(np.array([-1.0, 1.0], np.float32), base_n)).astype(np.float32)
    base[:5] = [0.0, -0.0, np.inf, -np.inf, np.nan]
    want_all = oracle.port_compress(base, 0.77)
    bt = _t(base, dev)
    ct = _t(want_all, dev)
    for n in (1 << 24, (1 << 24) + 1, (1 << 24) + 2, (1 << 24) + 3, (1 << 24) + 4, (1 << 24) + 12288 - 4,
              (1 << 24) + 12288, (1 << 24) + 12288 * 3 + 61):
        for off in (0, 4, 1):
            if off + n > base_n:
                continue
            got = cn.compression_8bit(bt[off:off + n], 0.77)
            assert torch.equal(got, ct[off:off + n]), ("compress", n, off)
            canary = torch.full((n + 8,), 7.0, device=dev)
            back = cn.decompression_8bit(ct[off:off + n], 0.77, out=canary[4:4 + n] if off != 1 else canary[1:1 + n])
            want = _t(oracle.decompress(want_all[off:off + n], 0.77), dev)
            assert torch.equal(back.view(torch.int32), want.view(torch.int32)), ("decompress", n, off)
            lo = 4 if off != 1 else 1
            assert float(canary[:lo].min()) == 7.0 and float(canary[lo + n:].max()) == 7.0 and float(canary[lo + n:].min()) == 7.0
    # codes written past the end would show here
    n = (1 << 24) + 5
    canary = torch.full((n + 64,), 0xAB, dtype=torch.uint8, device=dev)
    cn.compression_8bit(bt[:n], 0.77, out=canary[32:32 + n])
    assert torch.equal(canary[32:32 + n], ct[:n]) and int(canary[:32].min()) == 0xAB and int(canary[32 + n:].min()) == 0xAB
    # no table for these precisions: every element goes through the literal procedure
    small = base[:(1 << 24) + 7]
    for prec in (0.0, float("inf"), 1e-42):
        with np.errstate(all="ignore"):
            want = oracle.port_compress(small, prec)
        got = cn.compression_8bit(bt[:small.size], prec).cpu().numpy()
        assert np.array_equal(got, want), prec


def test_decode_through_a_given_table(dev):
    """cn_decode_8bit_lut: out[i] = lut[codes[i]] for any 256-entry table, on both kernels (a workgroup per tile, and
    element by element), ragged sizes and unaligned starts."""
    import torch
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(8)
    lut = rng.normal(0, 1, 256).astype(np.float32)
    lut[126], lut[254] = 0.0, -0.0
    codes = rng.integers(0, 256, (1 << 24) + 4103, dtype=np.uint8)
    ct, lt = _t(codes, dev), _t(lut, dev)
    for n in (0, 1, 5, 4096, 65_539, (1 << 24), (1 << 24) + 4103):
        for off in (0, 1, 4):
            if off + n > codes.size:
                continue
            got = L.decode_8bit_lut(ct[off:off + n], lt).cpu().numpy()
            assert np.array_equal(got.view(np.uint32), lut[codes[off:off + n]].view(np.uint32)), (n, off)


def test_absmax_and_compression_in_one_call(dev):
    """cn_absmax_compress_8bit against cn_absmax_f32 followed by cn_compress_8bit_dp and against the CPU checker, as
    the library picks by size, as the two kernels and as the single launch (cn_host_absmax_compress_single_launch): sizes on
    both sides of every dispatch boundary, unaligned starts, all-zero and NaN-bearing data, calls in a row, and with
    the single launch's wait for the rest of the grid cut to nothing, so that every workgroup that would have
    waited takes the maximum by itself."""
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(77)
    big = (1 << 26) + 8
    base = rng.normal(0, 0.02, big + 4).astype(np.float32)
    base[::101] *= 20
    bt = _t(base, dev)
    try:
        for single, spins in ((-1, -1), (0, -1), (1, -1), (1, 0), (1, -1)):
            L.lib().cn_host_absmax_compress_single_launch(single)
            L.lib().cn_host_absmax_compress_spin_limit(spins)
            for n, off in ((1, 0), (3, 0), (5, 4), (4096, 0), (4097, 0), (70_001, 0), (128 * 40000, 0), (128 * 40000, 1),
                           ((1 << 24) + 3, 4), (big, 0)):
                if spins == 0 and n > (1 << 23):
                    continue  # a workgroup on its own reads the whole tensor: keep that to small inputs
                x = bt[off:off + n]
                codes, prec = cn.absmax_compression_8bit(x)
                want_prec = cn.absmax(x)
                want = cn.compression_8bit(x, want_prec)
                assert torch.equal(prec.view(torch.int32), want_prec.view(torch.int32)), (spins, n, off)
                assert torch.equal(codes, want), (spins, n, off)
                if n <= 128 * 40000:
                    p = float(np.abs(base[off:off + n]).max())
                    assert float(prec.cpu()[0]) == p
                    assert np.array_equal(codes.cpu().numpy(), oracle.port_compress(base[off:off + n], p)), (spins, n, off)
            z = torch.zeros(10_000, device=dev)
            codes, prec = cn.absmax_compression_8bit(z)
            assert float(prec.cpu()[0]) == 0.0 and np.array_equal(codes.cpu().numpy(), oracle.compress(np.zeros(10_000, np.float32), 0.0))
            y = bt[:50_000].clone()
            y[12_345] = float("nan")
            codes, prec = cn.absmax_compression_8bit(y)
            assert np.isnan(float(prec.cpu()[0]))
            with np.errstate(all="ignore"):
                assert np.array_equal(codes.cpu().numpy(), oracle.compress(y.cpu().numpy(), float("nan")))
            codes, prec = cn.absmax_compression_8bit(bt[:0])
            assert float(prec.cpu()[0]) == -1.0 and codes.numel() == 0
    finally:
        L.lib().cn_host_absmax_compress_spin_limit(-1)
        L.lib().cn_host_absmax_compress_single_launch(-1)


def test_compression_beyond_the_cache_draws_its_tiles(dev, codec_form):
    """From 2^27 elements on compression runs one workgroup per compute unit that draws 49152-element tiles from a
    counter: sizes round a tile boundary, n % 4 tails and a start that is 16 bytes in, against the CPU checker, each
    size twice in a row (the second call finds the counter as the first one left it).  Once with the encoder the
    library takes at this size (the table built for the call's precision) and once with the table on the quotient."""
    if codec_form == "table_always":
        pytest.skip("the library's own choice at this size")
    import torch
    import clusternet_amd as cn
    rng = np.random.default_rng(77)
    tile = 1024 * 12 * 4
    first = 1 << 27
    base_n = first + 2 * tile + 16
    mag = np.exp(rng.uniform(np.log(1e-7), np.log(1.3), base_n)).astype(np.float32)
    base = (mag * rng.choice(np.array([-1.0, 1.0], np.float32), base_n)).astype(np.float32)
    want_all = oracle.port_compress(base, 0.77)
    bt, ct = _t(base, dev), _t(want_all, dev)
    for n in (first, first + 1, first + 3, first + tile - 4, first + tile, first + 2 * tile + 7):
        for off in (0, 4):
            for _ in range(2):
                canary = torch.full((n + 64,), 0xAB, dtype=torch.uint8, device=dev)
                cn.compression_8bit(bt[off:off + n], 0.77, out=canary[32:32 + n])
                assert torch.equal(canary[32:32 + n], ct[off:off + n]), (n, off)
                assert int(canary[:32].min()) == 0xAB and int(canary[32 + n:].min()) == 0xAB
    # a smaller tensor in between takes the other kernels and must not be disturbed by the counter
    got = cn.compression_8bit(bt[:1 << 20], 0.77)
    assert torch.equal(got, ct[:1 << 20])
    from clusternet_amd import _lib as L
    assert L.lib().cn_host_tile_counters_in_use() == 0  # every kernel that drew tiles left its counter at zero


def test_kernels_that_draw_tiles_replay_from_a_graph(dev, codec_form):
    """The kernels that draw their tiles leave their counter at zero, so a captured graph of them can be replayed:
    compression and the weight update beyond the cache, captured once, replayed three times with eager calls of the
    same kernels in between, every replay against the eager result."""
    if codec_form != "literal_for_small_tensors":
        pytest.skip("one run is enough")
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(21)
    n = (1 << 27) + 5 * 4096 + 3
    x = torch.randn(n, device=dev, generator=gen) * 0.02
    w0 = torch.randn(n, device=dev, generator=gen)
    want_codes = cn.compression_8bit(x, 0.11)
    want_w = w0.clone()
    L.sgd_update(want_w, x, 0.5)
    codes = torch.zeros(n, dtype=torch.uint8, device=dev)
    w = w0.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up on the capturing stream, as the capture API asks
        cn.compression_8bit(x, 0.11, out=codes)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cn.compression_8bit(x, 0.11, out=codes)
        L.sgd_update(w, x, 0.5)
    for _ in range(3):
        codes.zero_()
        w.copy_(w0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(codes, want_codes)
        assert torch.equal(w.view(torch.int32), want_w.view(torch.int32))
        # eager calls of the same kernels between the replays
        assert torch.equal(cn.compression_8bit(x, 0.11), want_codes)
        again = w0.clone()
        L.sgd_update(again, x, 0.5)
        assert torch.equal(again.view(torch.int32), want_w.view(torch.int32))


def test_kernels_that_draw_tiles_may_overlap_on_two_streams(dev, codec_form):
    """Launches take the library's ticket counters in turn, so two compressions of 2^27 elements and more issued on two streams
    (default priority) may run at the same time without drawing each other's tiles: both must give the codes of a
    compression that ran alone, over several rounds."""
    if codec_form != "literal_for_small_tensors":
        pytest.skip("one run is enough")
    import torch
    import clusternet_amd as cn
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(33)
    n = (1 << 27) + 12345 * 4
    xs = [torch.randn(n, device=dev, generator=gen) * 0.02 for _ in range(2)]
    want = [cn.compression_8bit(x, 0.09) for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.zeros(n, dtype=torch.uint8, device=dev) for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(4):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        for s, x, o in zip(streams, xs, outs):
            with torch.cuda.stream(s):
                cn.compression_8bit(x, 0.09, out=o)
        torch.cuda.synchronize()
        for o, w in zip(outs, want):
            assert torch.equal(o, w)
    assert L.lib().cn_host_tile_counters_in_use() == 0


def test_the_quotient_formed_in_double_precision_is_the_division(dev, codec_form):
    """The table on the quotient looks up (float)((double)x * (1.0 / (double)p)) where the literal procedure looks at x / p.
    On the device, over all 2^32 bit patterns of x, the two must agree in every bit (NaNs aside, and results below the
    normal range, which all have the code 254) for precisions of every kind: ordinary, negative, powers of two,
    significands of all ones or one above a power of two (the reciprocal's worst cases), tiny, huge, denormal, zero,
    infinite and NaN."""
    if codec_form != "table_on_the_quotient":
        pytest.skip("one run is enough")
    from clusternet_amd import _lib as L
    rng = np.random.default_rng(2024)
    bits = lambda b: float(np.array([b], np.uint32).view(np.float32)[0])
    precisions = [1.0, 0.1, 3.0, -0.37, 0.0234375, 2.0 ** -60, 2.0 ** 60, 1e-30, 1e30, 3e38, 1.2e-38, 1e-42, 1.4e-45,
                  bits(0x3fffffff), bits(0x3f800001), bits(0x3f7fffff), bits(0x40400001), bits(0x007fffff), bits(0x7f7fffff),
                  0.0, -0.0, float("inf"), float("nan")]
    precisions += [float(v) for v in np.exp(rng.uniform(np.log(1e-36), np.log(1e36), 40))]
    precisions += [float(v) for v in rng.uniform(1e-3, 2.0, 40).astype(np.float32)]
    for p in precisions:
        assert L.lib().cn_host_quotient_mismatches(p, 0, 1 << 32) == 0, p


def test_more_than_2_to_the_32_elements(dev, codec_form):
    """Element counts are size_t throughout: a tensor of 2^32 + 12293 elements (17 GB of fp32; the reference's int sizes
    stop at 2^31) through abs-max, compression and decompression.  Abs-max finds a value planted in the last element;
    the codes and the decoded values of the whole tensor equal, window by window (the start, both sides of element
    2^32, the end with its n % 4 tail), those of the windows processed on their own, which the other tests hold to
    the CPU checker."""
    if codec_form != "literal_for_small_tensors":
        pytest.skip("one run is enough")
    import torch
    import clusternet_amd as cn
    n = (1 << 32) + 3 * 4096 + 5
    free, _ = torch.cuda.mem_get_info()
    if free < 48 * (1 << 30):
        pytest.skip("needs 48 GB of device memory")
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    x = torch.empty(n, device=dev)
    piece = 1 << 28
    for lo in range(0, n, piece):  # filled piece by piece: the generator's own limits are not under test
        hi = min(lo + piece, n)
        x[lo:hi].normal_(0.0, 0.02, generator=gen)
    x[n - 1] = 7.25
    prec = cn.absmax(x)
    assert float(prec.cpu()[0]) == 7.25
    x[n - 1] = 0.01
    x[(1 << 32) + 1] = -0.3
    assert float(cn.absmax(x).cpu()[0]) == float(torch.maximum(x[:1 << 31].abs().max(), x[1 << 31:].abs().max()).cpu())
    p = 0.11
    codes = cn.compression_8bit(x, p)
    windows = [(0, 1 << 20), ((1 << 32) - (1 << 20), (1 << 32) + 4096 + 8), (n - (1 << 20) - 3, n)]
    for lo, hi in windows:
        lo -= lo % 4  # windows start 16-byte aligned, as the whole tensor does
        assert torch.equal(codes[lo:hi], cn.compression_8bit(x[lo:hi], p)), (lo, hi)
    del x
    back = cn.decompression_8bit(codes, p)
    for lo, hi in windows:
        lo -= lo % 4
        assert torch.equal(back[lo:hi].view(torch.int32), cn.decompression_8bit(codes[lo:hi], p).view(torch.int32)), (lo, hi)
    from clusternet_amd import _lib as L
    assert L.lib().cn_host_tile_counters_in_use() == 0


def test_one_launch_abs_max_and_compression_beside_a_product_on_another_stream(dev, codec_form):
    """The single launch waits inside the kernel for the rest of its grid.  With products that fill the chip running on
    another stream (default priority) part of that grid may not be resident when the first workgroups arrive: the
    wait is bounded, whoever gives up takes the maximum by itself, and the result is the one of a call that ran
    alone.  Products and codec share no scratch memory (the products' chunk planes against the codec's ticket lines)."""
    if codec_form != "literal_for_small_tensors":
        pytest.skip("one run is enough")
    import torch
    import clusternet_amd as cn
    gen = torch.Generator(device=dev)
    gen.manual_seed(8)
    n = 128 * 40000
    x = torch.randn(n, device=dev, generator=gen) * 0.02
    want_codes, want_prec = cn.absmax_compression_8bit(x)
    A = torch.randn((4096, 4096), device=dev, generator=gen)
    B = torch.randn((4096, 4096), device=dev, generator=gen)
    C = torch.empty((4096, 4096), device=dev)
    want_C = cn.dot(A, B)
    side, main = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(3):
        codes = torch.zeros(n, dtype=torch.uint8, device=dev)
        prec = torch.zeros(1, device=dev)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for _ in range(4):
                cn.dot(A, B, out=C)
        with torch.cuda.stream(main):
            for _ in range(8):
                cn.absmax_compression_8bit(x, out=codes, precision_out=prec)
        torch.cuda.synchronize()
        assert torch.equal(prec.view(torch.int32), want_prec.view(torch.int32))
        assert torch.equal(codes, want_codes)
        assert torch.equal(C.view(torch.int32), want_C.view(torch.int32))
