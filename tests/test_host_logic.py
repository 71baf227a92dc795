"""Host-side logic of the library, checked without a GPU: the C-ABI loads and exports every
declared symbol, the encoder's bucket table reproduces the reference procedure for every fp32
pattern in range, the approximate-quotient fast path is never trusted where it could be wrong, and
the GEMM work decomposition covers K exactly."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import clusternet_amd as cn
import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    hdr = open(os.path.join(ROOT, "include", "cnhip.h")).read()
    names = set(re.findall(r"\b(cn_[a-z0-9_]+)\s*\(", hdr))
    assert {"cn_gemm_f32", "cn_gemm_f32_w8", "cn_compress_8bit", "cn_decompress_8bit",
            "cn_absmax_f32", "cn_init"} <= names
    L = cn.lib()
    for n in sorted(names):
        assert hasattr(L, n), n


def test_no_device_is_reported_not_hidden():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    L = cn.lib()
    assert L.cn_init(0) == 3  # CN_ERR_NO_DEVICE
    assert b"device" in L.cn_last_error()
    assert L.cn_gemm_f32(0, 0, 4, 4, 4, 16, 4, 16, 4, 16, 4, None) == 3
    assert L.cn_compress_8bit(16, 1.0, 4, 16, None) == 3
    # argument errors are detected before any device is needed
    assert L.cn_gemm_f32(0, 0, -1, 4, 4, 16, 4, 16, 4, 16, 4, None) == 2
    assert L.cn_gemm_f32(0, 0, 4, 4, 4, 16, 3, 16, 4, 16, 4, None) == 2
    assert L.cn_gemm_f32(0, 0, 0, 4, 4, None, 4, None, 4, None, 4, None) == 0


def test_product_table_equals_fixture():
    raw = open(os.path.join(ROOT, "tests", "golden", "8bit_floats_table.bin"), "rb").read()
    assert cn.table().tobytes() == raw


def _lookup(mags):
    L = cn.lib()
    mags = np.ascontiguousarray(mags, np.uint32)
    codes = np.empty(mags.size, np.uint8)
    near = np.empty(mags.size, np.uint8)
    L.cn_host_encode_lut_lookup_many.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
    assert L.cn_host_encode_lut_lookup_many(mags.ctypes.data, mags.size, codes.ctypes.data, near.ctypes.data) == 0
    return codes, near


def test_bucket_table_exhaustive_over_all_patterns_in_range():
    lo = int(np.array([1.0e-6], np.float32).view(np.uint32)[0])
    hi = int(np.array([1.01], np.float32).view(np.uint32)[0])
    step = 1 << 24
    for start in range(lo, hi, step):
        mags = np.arange(start, min(start + step, hi), dtype=np.uint32)
        codes, _ = _lookup(mags)
        want = oracle.compress(mags.view(np.float32), 1.0, 0)
        assert np.array_equal(codes, want), hex(start)
    # far outside the table: zero code below, saturation above (including infinity)
    far = np.array([0, 1, 0x00800000, lo - 1, hi + 5, 0x7f000000, 0x7f800000], np.uint32)
    codes, _ = _lookup(far)
    assert codes.tolist() == [254, 254, 254, 254, 127, 127, 127]


def test_fast_path_is_exact_wherever_it_is_trusted():
    """x * (1/p) stands in for x / p; wherever the table does not flag the element as near a
    boundary the code must equal the reference procedure's on the exact quotient."""
    rng = np.random.default_rng(123)
    t = oracle.table()
    edges = np.concatenate([t, (t[:-1] + t[1:]) / 2, [1.5e-6, 0.995703, 1.0]]).astype(np.float32)
    trusted = 0
    for p in [1.0, 0.1, 0.0234375, 3.0, 1e-5, 7.7e4] + list(rng.uniform(1e-3, 10, 6)):
        p = np.float32(p)
        r = np.float32(1.0) / p
        x = np.concatenate([
            np.exp(rng.uniform(np.log(1e-7), np.log(1.5), 400_000)).astype(np.float32) * p,
            # inputs whose quotient sits within a few ulps of every boundary candidate
            (np.repeat(edges, 41).view(np.uint32).astype(np.int64)
             + np.tile(np.arange(-20, 21), edges.size)).astype(np.uint32).view(np.float32) * p,
        ]).astype(np.float32)
        a0 = (x * r).astype(np.float32)
        codes, near = _lookup(a0.view(np.uint32) & np.uint32(0x7fffffff))
        want = oracle.compress(x, float(p), 0)
        ok = near == 0
        assert np.array_equal(codes[ok], want[ok]), float(p)
        trusted += int(ok.sum())
        assert near.mean() < 0.02
    assert trusted > 1_000_000


def test_gemm_plan_covers_k_and_fits_workspace():
    L = cn.lib()
    out = (C.c_int64 * 7)()
    rng = np.random.default_rng(0)
    shapes = [(128, 40000, 100000), (128, 20000, 40000), (128, 1024, 784), (784, 1024, 128),
              (128, 784, 1024), (100000, 8192, 128), (128, 4096, 4096), (2, 2, 3), (1, 1, 1),
              (128, 10, 4096), (5000, 5000, 31)]
    shapes += [tuple(int(v) for v in rng.integers(1, 3000, 3)) for _ in range(200)]
    for ws in (16 << 20, 1 << 30):
        for force in (0, 128, 256):
            for (M, N, K) in shapes:
                L.cn_host_plan_gemm(M, N, K, 256, ws, force, out)
                tm, tn, kit, splits, ips, units, tile_n = list(out)
                assert tile_n in (128, 256) and (force == 0 or tile_n == force)
                assert tm == -(-M // 128) and tn == -(-N // tile_n) and kit == max(1, -(-K // (32 if tile_n == 128 else 16)))
                assert splits >= 1 and units == tm * tn * splits
                assert ips * splits >= kit and ips * (splits - 1) < kit  # every chunk non-empty
                if splits > 1:
                    assert splits * M * N * 4 <= ws
    L.cn_host_plan_gemm(128, 40000, 100000, 256, 1 << 30, 128, out)
    assert list(out)[:6] == [1, 313, 3125, 13, 241, 4069]
