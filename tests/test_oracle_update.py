"""Pins of the CPU checker's fused update passes (decode + axpy, RMSprop with weight update) by
what the formulas fix: composition of already pinned pieces, closed forms at the multiplier's end
points, and an fp64 evaluation of the same expression."""
import numpy as np

import oracle


def test_decompress_axpy_is_decompress_then_scaled_add():
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 256, 100_003, dtype=np.uint8)
    y = rng.normal(0, 1, codes.size).astype(np.float32)
    for prec, alpha in ((0.37, 1.0), (0.37, -1.0), (2.5e-3, -0.01), (1.0, 0.333)):
        g = oracle.decompress(codes, prec)
        scaled = (np.float32(alpha) * g).astype(np.float32)       # rounded product first
        want = (y + scaled).astype(np.float32)
        got = oracle.decompress_axpy(codes, prec, alpha, y)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # alpha = 1 and -1 are the reference's add / sub after decompression_8bit
    g = oracle.decompress(codes, 0.5)
    assert np.array_equal(oracle.decompress_axpy(codes, 0.5, 1.0, y), y + g)
    assert np.array_equal(oracle.decompress_axpy(codes, 0.5, -1.0, y), y - g)
    # a gradient step on coded gradients: w - rate * g, product rounded first
    rate = np.float32(0.01)
    assert np.array_equal(oracle.decompress_axpy(codes, 0.5, -rate, y), (y - (rate * g).astype(np.float32)))


def test_rmsprop_closed_forms():
    rng = np.random.default_rng(2)
    n = 50_000
    g = rng.normal(0, 0.1, n).astype(np.float32)
    rms = rng.uniform(0, 0.01, n).astype(np.float32)
    w = rng.normal(0, 1, n).astype(np.float32)
    lr = np.float32(0.003)
    # multiplier 1: rms unchanged, step = lr * g / (sqrt(rms) + 1e-8)
    r1, w1 = oracle.rmsprop_update(rms, g, w, 1.0, lr)
    assert np.array_equal(r1, rms)
    step = (lr * (g / (np.sqrt(rms) + np.float32(1e-8))).astype(np.float32)).astype(np.float32)
    assert np.array_equal(w1, (w - step).astype(np.float32))
    # multiplier 0: rms = g * g, step = lr * g / (|g| + 1e-8) ~ lr * sign(g)
    r0, w0 = oracle.rmsprop_update(rms, g, w, 0.0, lr)
    assert np.array_equal(r0, (g * g).astype(np.float32))
    big = np.abs(g) > 1e-3
    assert np.allclose((w - w0)[big], lr * np.sign(g[big]), rtol=1e-4, atol=0)
    # zero gradient: the weights stay, rms decays
    rz, wz = oracle.rmsprop_update(rms, np.zeros(n, np.float32), w, 0.9, lr)
    assert np.array_equal(wz, w) and np.array_equal(rz, (np.float32(0.9) * rms).astype(np.float32))


def test_rmsprop_against_fp64_evaluation():
    rng = np.random.default_rng(3)
    n = 200_000
    g = (rng.normal(0, 0.05, n) * (rng.random(n) < 0.9)).astype(np.float32)
    rms = rng.uniform(0, 0.01, n).astype(np.float32)
    w = rng.normal(0, 0.05, n).astype(np.float32)
    mult, lr = 0.9, 0.003
    r, ww = oracle.rmsprop_update(rms, g, w, mult, lr)
    g64, r64, w64 = g.astype(np.float64), rms.astype(np.float64), w.astype(np.float64)
    m32 = float(np.float32(mult))
    om32 = float(np.float32(1.0) - np.float32(mult))
    rr = m32 * r64 + g64 * g64 * om32
    ws = w64 - float(np.float32(lr)) * g64 / (np.sqrt(rr) + float(np.float32(1e-8)))
    assert np.max(np.abs(r - rr) / np.maximum(rr, 1e-30)) < 4 * 2.0 ** -24
    # the step is a handful of fp32 roundings of a value of size <= lr / sqrt(1 - mult)
    assert np.max(np.abs(ww - ws)) < 8 * 2.0 ** -24 * (np.max(np.abs(w)) + lr / np.sqrt(1 - mult))
    # a dropped term or a swapped factor is far outside these bounds
    wrong = m32 * r64 + g64 * g64 * m32
    assert np.max(np.abs(r - wrong) / np.maximum(rr, 1e-30)) > 1e-3
