"""Pins the CPU checker for the 8-bit codec (no GPU needed).

The reference has no codec test vectors, so the checker is pinned by (1) the bytes of the
reference's table file, (2) agreement of two independent C formulations and a third pure-Python
walk of the search tree, (3) hand-traced inputs whose codes follow from the source text of
source/clusterKernels.cu:1163-1232 without running it, and (4) invariants of the procedure
(monotone rank, fixed points, error bound, sign symmetry).
"""
import hashlib
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
TABLE_SHA = "c2dbfffe982a2fc5430f56cbb44857fe8e6b610b4445f3dae2a64b0b6c977a37"
LOW = np.float32(0.0000015)
HIGH = np.float32(0.995703)


def golden_table():
    raw = open(os.path.join(HERE, "golden", "8bit_floats_table.bin"), "rb").read()
    return raw, np.frombuffer(raw, dtype="<f4")


def test_table_matches_fixture_and_hash():
    raw, t = golden_table()
    assert len(raw) == 504 and hashlib.sha256(raw).hexdigest() == TABLE_SHA
    assert oracle.table().tobytes() == raw


def test_table_matches_reference_file_when_mounted():
    path = "/root/reference/source/8bit_floats.hdf5"
    if not os.path.exists(path):
        pytest.skip("reference tree not mounted")
    ref = open(path, "rb").read()
    assert ref[2144:2648] == oracle.table().tobytes()


def test_table_structure():
    # six decades e = 6..1, each two half-decades [1,4.5]e-e and [4.5,10]e-e cut into 2^(6-e)
    # equal bins, entries are bin midpoints (up to fp32 noise)
    t = oracle.table().astype(np.float64)
    assert np.all(np.diff(t) > 0)
    expect = []
    for e in range(6, 0, -1):
        bins = 2 ** (6 - e)
        for lo, hi in ((1.0, 4.5), (4.5, 10.0)):
            w = (hi - lo) / bins
            expect += [(lo + (i + 0.5) * w) * 10.0 ** (-e) for i in range(bins)]
    assert len(expect) == 126
    np.testing.assert_allclose(t, np.array(expect), rtol=2e-6)


def py_walk(x, precision, slot126=1.0):
    """Third implementation: explicit descent of the 6-level search with numpy float32 scalars."""
    t = list(oracle.table()) + [np.float32(slot126), np.float32(0)]
    with np.errstate(all="ignore"):
        a = np.float32(x) / np.float32(precision)
    neg = bool(a < 0)
    if neg:
        a = -a
    if a < LOW:
        return 254
    if a > HIGH:
        return 255 if neg else 127
    lo, hi, p = 0, 125, 63
    for step in (32, 16, 8, 4, 2, 1):
        if a > t[p]:
            lo, p = p, p + step
        else:
            hi, p = p, p - step
    if lo == p:
        c = p if abs(np.float32(t[p] - a)) < np.float32(t[hi] - a) else hi
    else:
        c = p if np.float32(t[p] - a) < abs(np.float32(t[lo] - a)) else lo
    return (c | 0x80) if neg else c


def adversarial_inputs():
    t = oracle.table()
    pts = [t, np.nextafter(t, np.float32(0)), np.nextafter(t, np.float32(2))]
    mids = ((t[:-1].astype(np.float64) + t[1:].astype(np.float64)) / 2).astype(np.float32)
    for k in (-2, -1, 0, 1, 2):
        pts.append((mids.view(np.uint32) + np.uint32(k)).view(np.float32) if k >= 0
                   else (mids.view(np.uint32) - np.uint32(-k)).view(np.float32))
    for thr in (LOW, HIGH, np.float32(1.0), t[125]):
        b = np.array([thr]).view(np.uint32)[0]
        pts.append(np.arange(b - 4, b + 5, dtype=np.uint32).view(np.float32))
    pts.append(np.array([0.0, -0.0, 1e-45, 1e-38, 1.1754944e-38, 0.5, 0.25, 0.1, 0.01, 0.001,
                         0.993, 0.9957, 0.9958, 1.0, 1.5, 3e38], np.float32))
    x = np.concatenate([np.asarray(p, np.float32).reshape(-1) for p in pts])
    return np.concatenate([x, -x])


@pytest.mark.parametrize("rule", [0, 1])
def test_literal_equals_closed_form_adversarial(rule):
    x = adversarial_inputs()
    for prec in (1.0, 0.1, 0.5, 2.0, 3.7, 1e-3, 1e3):
        xs = (x * np.float32(prec)).astype(np.float32)
        a = oracle.compress(xs, prec, rule, "literal")
        b = oracle.compress(xs, prec, rule, "closed")
        assert np.array_equal(a, b), prec


def test_literal_equals_closed_form_random():
    rng = np.random.default_rng(7)
    n = 1_000_000
    logu = np.exp(rng.uniform(np.log(1e-7), np.log(1.2), n)).astype(np.float32)
    logu *= rng.choice([-1.0, 1.0], n).astype(np.float32)
    gauss = rng.normal(0, 0.3, n).astype(np.float32)
    for x in (logu, gauss):
        for prec in (1.0, 0.731, float(np.abs(x).max())):
            assert np.array_equal(oracle.compress(x, prec, 0, "literal"),
                                  oracle.compress(x, prec, 0, "closed"))


def test_c_equals_python_walk():
    x = adversarial_inputs()
    rng = np.random.default_rng(3)
    x = np.concatenate([x, rng.normal(0, 0.4, 3000).astype(np.float32)])
    got = oracle.compress(x, 1.0, 0)
    want = np.array([py_walk(v, 1.0) for v in x], np.uint8)
    assert np.array_equal(got, want)
    got1 = oracle.compress(x, 1.0, 1)
    want1 = np.array([py_walk(v, 1.0, slot126=0.0) for v in x], np.uint8)
    assert np.array_equal(got1, want1)


def test_hand_traced_codes():
    t = oracle.table()
    one = lambda v, p=1.0, r=0: int(oracle.compress(np.array([v], np.float32), p, r)[0])
    # thresholds: |a| < float(1.5e-6) is the "zero" code whatever the sign
    assert one(0.0) == 254 and one(-0.0) == 254 and one(1e-6) == 254 and one(-1e-6) == 254
    assert one(np.nextafter(LOW, np.float32(0))) == 254
    # a == 1.5e-6 is not below the threshold and lies under t[0]: q = 0, |t0-a| < t1-a -> code 0
    assert one(LOW) == 0
    # a > float(0.995703) saturates
    assert one(1.0) == 127 and one(-1.0) == 255 and one(7.0) == 127 and one(-7.0) == 255
    assert one(np.nextafter(HIGH, np.float32(2))) == 127
    # the never-written slot: rule 0 keeps 125/253, rule 1 yields 126/254
    assert one(HIGH) == 125 and one(-HIGH) == 253
    assert one(0.993) == 125 and one(0.993, r=1) == 126 and one(-0.993, r=1) == 254
    # an even entry is a fixed point; an odd entry p >= 3 is *not* above itself, so the search
    # settles on q = p - 1 and picks between q and q - 1: code p - 1
    for k in range(0, 126, 2):
        assert one(t[k]) == k and one(-t[k]) == (k | 0x80)
    for p in range(3, 126, 2):
        assert one(t[p]) == p - 1
    # t[1]: q = 0, candidates 0 and 1, |t0 - t1| < 0 is false -> 1
    assert one(t[1]) == 1
    # just above an odd entry p (q = p + 1): candidates p and p + 1, p is nearer
    for p in range(1, 124, 2):
        assert one(np.nextafter(t[p], np.float32(2))) == p
    # inputs in (t[q], t[q+1]] always map to q, even when q + 1 is nearer (the search never looks
    # at the upper odd neighbour)
    for q in range(2, 124, 2):
        assert one(np.nextafter(t[q + 1], np.float32(0))) == q
    # non-finite inputs by the literal comparisons
    assert one(np.nan) == 1 and one(np.inf) == 127 and one(-np.inf) == 255
    with np.errstate(all="ignore"):
        assert one(1.0, 0.0) == 127 and one(-1.0, 0.0) == 255 and one(0.0, 0.0) == 1
    # a negative precision flips the sign bit
    assert one(0.5, -1.0) == (one(0.5) | 0x80)


def test_rank_is_monotone_and_covers_expected_codes():
    # codes as a function of a > 0 never decrease (with 254 ordered below 0)
    a = np.sort(np.exp(np.random.default_rng(1).uniform(np.log(1e-7), np.log(1.1),
                                                         400_000)).astype(np.float32))
    c = oracle.compress(a, 1.0, 0).astype(np.int32)
    rank = np.where(c == 254, -1, c)
    assert np.all(np.diff(rank) >= 0)
    assert set(np.unique(c)) == set(range(0, 126)) | {127, 254}
    # sign symmetry
    cn = oracle.compress(-a, 1.0, 0).astype(np.int32)
    assert np.array_equal(np.where(c == 254, 254, c | 0x80), cn)


def test_decode_lut_closed_form():
    t = oracle.table()
    for prec in (1.0, 0.1, 0.0234, 17.0):
        lut = oracle.decode_lut(prec)
        p = np.float32(prec)
        assert np.array_equal(lut[:126], t * p)
        assert np.array_equal(lut[128:254], -(t * p))
        assert lut[126] == p and lut[127] == p and lut[254] == p and lut[255] == -p
        codes = np.arange(256, dtype=np.uint8)
        assert np.array_equal(oracle.decompress(codes, prec), lut)


def test_round_trip_error_bound():
    rng = np.random.default_rng(11)
    x = rng.normal(0, 0.02, 200_000).astype(np.float32)
    prec = float(np.abs(x).max())
    codes = oracle.compress(x, prec)
    y = oracle.decompress(codes, prec)
    a = np.abs(x) / prec
    keep = codes != 254  # the "zero" code decodes to +precision by the reference's table
    t = oracle.table().astype(np.float64)
    gaps = np.diff(np.concatenate([t, [1.0]]))
    idx = np.clip(np.searchsorted(t, a[keep]), 1, 125)
    bound = np.maximum(gaps[idx - 1], gaps[idx]) * prec
    err = np.abs(y[keep].astype(np.float64) - x[keep])
    assert np.all(err <= bound * 1.0001 + 1e-12)
    assert np.all(np.sign(y[keep]) == np.sign(x[keep]))
    assert np.all(y[~keep] == np.float32(prec))


def test_absmax():
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, 10_001).astype(np.float32)
    assert oracle.absmax(x) == float(np.abs(x).max())
    assert oracle.port_absmax(x) == float(np.abs(x).max())
    assert oracle.absmax(np.zeros(3, np.float32)) == 0.0
    assert oracle.absmax(np.array([-3.0, 2.0], np.float32)) == 3.0
    assert np.isnan(oracle.absmax(np.array([1.0, np.nan], np.float32)))


def test_port_equals_oracle():
    rng = np.random.default_rng(9)
    x = rng.normal(0, 0.1, 300_001).astype(np.float32)
    prec = oracle.absmax(x)
    c = oracle.compress(x, prec)
    assert np.array_equal(oracle.port_compress(x, prec), c)
    assert np.array_equal(oracle.port_decompress(c, prec), oracle.decompress(c, prec))
