"""The committed codec vectors (tests/golden/codec_vectors.bin + .json, written by make_codec_vectors.py): adversarial
inputs under five precisions with their codes for both readings of the reference's unwritten table slot, and the
decode tables.  The CPU tests hold the checker to the file (and the file to a pure-Python walk of the reference's
search, source/clusterKernels.cu:1163-1232); the GPU tests hold cn_compress_8bit / cn_decompress_8bit to it through
the C-ABI.  The library implements sliver rule 0 (codes 125 / 253)."""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))


def load():
    meta = json.load(open(os.path.join(HERE, "golden", "codec_vectors.json")))
    raw = open(os.path.join(HERE, "golden", "codec_vectors.bin"), "rb").read()
    assert len(raw) == meta["bytes"] and hashlib.sha256(raw).hexdigest() == meta["sha256"]
    n = meta["n"]
    x = np.frombuffer(raw, "<f4", n, 0)
    off = 4 * n
    sets = []
    for per in meta["precisions"]:
        p = np.array([int(per["precision_bits"], 16)], np.uint32).view(np.float32)[0]
        c0 = np.frombuffer(raw, np.uint8, n, off)
        c1 = np.frombuffer(raw, np.uint8, n, off + n)
        lut = np.frombuffer(raw, "<f4", 256, off + 2 * n)
        off += 2 * n + 1024
        with np.errstate(all="ignore"):
            xs = (x * p).astype(np.float32)
        sets.append((p, xs, c0, c1, lut))
    assert off == len(raw)
    return x, sets


def test_file_is_what_the_checker_computes():
    x, sets = load()
    assert len(sets) == 5 and x.size > 2000
    for p, xs, c0, c1, lut in sets:
        for form in ("literal", "closed"):
            assert np.array_equal(oracle.compress(xs, p, 0, form), c0), (p, form)
            assert np.array_equal(oracle.compress(xs, p, 1, form), c1), (p, form)
        assert np.array_equal(oracle.decode_lut(p).view(np.uint32), lut.view(np.uint32))


def test_file_against_a_python_walk_of_the_search():
    from test_oracle_codec import py_walk
    x, sets = load()
    for p, xs, c0, c1, lut in sets:
        pick = np.arange(0, xs.size, 3 if abs(p) == 1.0 else 11)
        assert [py_walk(v, p) for v in xs[pick]] == list(c0[pick]), p
        assert [py_walk(v, p, slot126=0.0) for v in xs[pick]] == list(c1[pick]), p


def test_the_two_rules_differ_only_in_the_sliver():
    x, sets = load()
    t125 = oracle.table()[125]
    for p, xs, c0, c1, lut in sets:
        with np.errstate(all="ignore"):
            a = np.abs(xs / np.float32(p))
        sliver = (a > t125) & (a <= np.float32(0.995703))
        assert sliver.any()
        assert np.array_equal(c0 != c1, sliver), p
        assert set(c0[sliver]) <= {125, 253} and set(c1[sliver]) <= {126, 254}


def test_decode_tables_follow_the_closed_form():
    x, sets = load()
    t = oracle.table()
    for p, xs, c0, c1, lut in sets:
        pos = (t * np.float32(p)).astype(np.float32)
        assert np.array_equal(lut[:126].view(np.uint32), pos.view(np.uint32))
        assert np.array_equal(lut[128:254].view(np.uint32), (-pos).view(np.uint32))
        assert all(lut[i] == np.float32(p) for i in (126, 127, 254)) and lut[255] == -np.float32(p)


@pytest.mark.gpu
@pytest.mark.usefixtures("codec_form")
def test_gpu_codes_equal_the_file():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    dev = torch.device("cuda:0")
    x, sets = load()
    for p, xs, c0, c1, lut in sets:
        got = cn.compression_8bit(torch.from_numpy(xs.copy()).to(dev), float(p)).cpu().numpy()
        assert np.array_equal(got, c0), ("precision", float(p), "first difference at", int(np.argmax(got != c0)))
        # also with the precision read from device memory
        pt = torch.tensor([float(p)], dtype=torch.float32, device=dev)
        got = cn.compression_8bit(torch.from_numpy(xs.copy()).to(dev), pt).cpu().numpy()
        assert np.array_equal(got, c0), float(p)


@pytest.mark.gpu
def test_gpu_decode_equals_the_file():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    dev = torch.device("cuda:0")
    x, sets = load()
    codes = torch.arange(256, dtype=torch.uint8, device=dev)
    for p, xs, c0, c1, lut in sets:
        got = cn.decompression_8bit(codes, float(p)).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), lut.view(np.uint32)), float(p)
        back = cn.decompression_8bit(torch.from_numpy(c0.copy()).to(dev), float(p)).cpu().numpy()
        assert np.array_equal(back.view(np.uint32), lut[c0].view(np.uint32)), float(p)
