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
    inc = os.path.join(ROOT, "include")
    hdr = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    names = set(re.findall(r"\b(cn_[a-z0-9_]+)\s*\(", hdr))
    assert {"cn_gemm_f32", "cn_gemm_f32_w8", "cn_compress_8bit", "cn_decompress_8bit",
            "cn_absmax_f32", "cn_init"} <= names
    L = cn.lib()
    for n in sorted(names):
        assert hasattr(L, n), n
    # and nothing is exported that no header declares
    import shutil
    import subprocess
    if shutil.which("nm") is None:
        return
    out = subprocess.run(["nm", "-D", "--defined-only", L._name], capture_output=True, text=True, check=True).stdout
    exported = {l.split()[2] for l in out.splitlines() if len(l.split()) == 3 and l.split()[1] == "T" and l.split()[2].startswith("cn_")}
    assert exported <= names, sorted(exported - names)


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


def _encode_host(x, precision):
    """The encoder as the device runs it (per-call table, or the literal procedure where the table
    reports itself unusable), evaluated by the library's host build."""
    L = cn.lib()
    x = np.ascontiguousarray(x, np.float32)
    codes = np.empty(x.size, np.uint8)
    L.cn_host_xlut_encode_many.argtypes = [C.c_float, C.c_void_p, C.c_size_t, C.c_void_p]
    used_table = L.cn_host_xlut_encode_many(float(precision), x.ctypes.data, x.size, codes.ctypes.data)
    return codes, bool(used_table)


def test_encoder_table_exhaustive_at_precision_one():
    """Every fp32 pattern from 1e-6 to 1.01 and, sparsely strided, from 0 to NaN, both signs."""
    lo = int(np.array([1.0e-6], np.float32).view(np.uint32)[0])
    hi = int(np.array([1.01], np.float32).view(np.uint32)[0])
    step = 1 << 24
    for start in range(lo, hi, step):
        mags = np.arange(start, min(start + step, hi), dtype=np.uint32)
        for sign in (0, 0x80000000):
            x = (mags | np.uint32(sign)).view(np.float32)
            codes, used = _encode_host(x, 1.0)
            assert used
            assert np.array_equal(codes, oracle.port_compress(x, 1.0)), (hex(start), sign)
    with np.errstate(all="ignore"):
        sweep = np.arange(0, 1 << 32, 4099, dtype=np.uint64).astype(np.uint32).view(np.float32)
        codes, used = _encode_host(sweep, 1.0)
        assert used and np.array_equal(codes, oracle.compress(sweep, 1.0, 0))
    far = np.array([0, 1, 0x00800000, lo - 1, hi + 5, 0x7f000000, 0x7f800000, 0x7f800001, 0x7fc00000,
                    0x80000000, 0xff800000, 0xffc00000], np.uint32).view(np.float32)
    codes, _ = _encode_host(far, 1.0)
    assert codes.tolist() == [254, 254, 254, 254, 127, 127, 127, 1, 1, 254, 255, 1]


def test_encoder_table_over_precisions_and_step_neighbourhoods():
    """For ordinary, negative, tiny, huge and degenerate precisions: random inputs over the whole
    coded range, every pattern within 40 ulps of every step of the code function, and a strided
    sweep over all bit patterns.  Where the table is trusted it must equal the literal procedure;
    where it is not, the encoder must say so (and then runs the literal procedure itself)."""
    rng = np.random.default_rng(123)
    t = oracle.table()
    edges = np.concatenate([t, (t[:-1] + t[1:]) / 2, [1.5e-6, 0.995703, 1.0]]).astype(np.float32)
    trusted_precisions = 0
    with np.errstate(all="ignore"):
        sweep = np.arange(0, 1 << 32, 16411, dtype=np.uint64).astype(np.uint32).view(np.float32)
        precisions = [1.0, 0.1, 0.0234375, 3.0, 1e-5, 7.7e4, -1.0, -0.37, 2.0 ** -60, 2.0 ** 60, 1e-30, 1e30,
                      3e38, 1.2e-38, 1e-42, 0.0, -0.0, float("inf"), float("-inf"), float("nan")]
        precisions += list(rng.uniform(1e-3, 10, 6))
        for p in precisions:
            p32 = np.float32(p)
            scale = p32 if np.isfinite(p32) and p32 != 0 else np.float32(1.0)
            near = (np.repeat(edges, 81).view(np.uint32).astype(np.int64)
                    + np.tile(np.arange(-40, 41), edges.size)).astype(np.uint32).view(np.float32)
            x = np.concatenate([
                np.exp(rng.uniform(np.log(1e-7), np.log(1.5), 200_000)).astype(np.float32) * scale,
                -np.exp(rng.uniform(np.log(1e-7), np.log(1.5), 50_000)).astype(np.float32) * scale,
                near * scale, -near * scale, sweep,
            ]).astype(np.float32)
            codes, used = _encode_host(x, p)
            want = oracle.compress(x, float(p), 0)
            bad = np.nonzero(codes != want)[0]
            assert bad.size == 0, (p, used, x[bad[:4]], codes[bad[:4]], want[bad[:4]])
            trusted_precisions += int(used)
            if np.isfinite(p32) and 1e-30 <= abs(float(p32)) <= 1e30:
                assert used, p          # the table serves every precision a gradient can have
    assert trusted_precisions >= 18


def _encode_by_quotient_host(x, precision):
    L = cn.lib()
    x = np.ascontiguousarray(x, np.float32)
    codes = np.empty(x.size, np.uint8)
    L.cn_host_quotient_encode_many.argtypes = [C.c_float, C.c_void_p, C.c_size_t, C.c_void_p]
    assert L.cn_host_quotient_encode_many(float(precision), x.ctypes.data, x.size, codes.ctypes.data) == 1
    return codes


def test_encoder_on_the_quotient_equals_the_literal_procedure():
    """The table for precision 1 looked up at (float)((double)x * (1 / (double)p)) against the literal procedure (the CPU
    checker), for every kind of precision, with no exception: there is no precision for which this encoder steps
    aside.  Inputs: random values over the whole coded range, every pattern within 40 ulps of p times every step of
    the code function (where a quotient rounded the wrong way would change the code), a strided sweep over all
    bit patterns.  The precisions include ones whose significand is all ones or one above a power of two (the
    reciprocal's worst cases), denormal ones and the degenerate ones (0, inf, NaN)."""
    rng = np.random.default_rng(321)
    t = oracle.table()
    edges = np.concatenate([t, (t[:-1] + t[1:]) / 2, [1.5e-6, 0.995703, 1.0]]).astype(np.float32)
    bits = lambda b: float(np.array([b], np.uint32).view(np.float32)[0])
    with np.errstate(all="ignore"):
        sweep = np.arange(0, 1 << 32, 16411, dtype=np.uint64).astype(np.uint32).view(np.float32)
        precisions = [1.0, 0.1, 0.0234375, 3.0, 1e-5, 7.7e4, -1.0, -0.37, 2.0 ** -60, 2.0 ** 60, 1e-30, 1e30,
                      3e38, 1.2e-38, 1e-42, 1.4e-45, 0.0, -0.0, float("inf"), float("-inf"), float("nan"),
                      bits(0x3fffffff), bits(0x3f800001), bits(0x3f7fffff), bits(0x40400001), bits(0x007fffff), bits(0x7f7fffff)]
        precisions += list(np.exp(rng.uniform(np.log(1e-36), np.log(1e36), 30)))
        for p in precisions:
            p32 = np.float32(p)
            scale = p32 if np.isfinite(p32) and p32 != 0 else np.float32(1.0)
            near = (np.repeat(edges, 81).view(np.uint32).astype(np.int64)
                    + np.tile(np.arange(-40, 41), edges.size)).astype(np.uint32).view(np.float32)
            scaled = (near.astype(np.float64) * float(scale)).astype(np.float32)
            around = (np.repeat(scaled, 9).view(np.uint32).astype(np.int64) + np.tile(np.arange(-4, 5), scaled.size))
            around = np.clip(around, 0, 0x7f800000).astype(np.uint32).view(np.float32)
            x = np.concatenate([
                np.exp(rng.uniform(np.log(1e-7), np.log(1.5), 200_000)).astype(np.float32) * scale,
                -np.exp(rng.uniform(np.log(1e-7), np.log(1.5), 50_000)).astype(np.float32) * scale,
                around, -around, sweep,
            ]).astype(np.float32)
            codes = _encode_by_quotient_host(x, p)
            want = oracle.compress(x, float(p), 0)
            bad = np.nonzero(codes != want)[0]
            assert bad.size == 0, (p, x[bad[:4]], codes[bad[:4]], want[bad[:4]])


def test_encoder_table_shape():
    L = cn.lib()
    n = L.cn_host_xlut_entries()
    entries = np.zeros((n, 2), np.uint32)
    first = C.c_uint32()
    L.cn_host_xlut_build.argtypes = [C.c_float, C.c_void_p, C.POINTER(C.c_uint32)]
    assert L.cn_host_xlut_build(1.0, entries.ctypes.data, C.byref(first)) == 0
    assert n * 8 <= 48 * 1024                                  # two workgroups per CU keep it in LDS
    codes = entries[1:-1, 1]
    below, above = codes & 0xff, (codes >> 8) & 0xff
    steps = int((below != above).sum())
    assert 100 <= steps <= 260                                 # 254 -> 0 -> ... -> 125 -> 127 (a few codes never occur)
    assert entries[0, 1] == 0xfefefefe and (entries[-1, 1] & 0xff) == 127
    # negative side: same steps, sign bit on every code but 254
    nb, pb = (codes >> 16) & 0xff, below
    assert np.all(np.where(pb == 254, nb == 254, nb == (pb | 0x80)))


def test_gemm_plan_covers_k_and_fits_workspace():
    """Whatever the planner chooses: one of the four tile geometries, K covered by non-empty chunks, the chunk planes inside
    the workspace, a forced geometry respected, and no tile more than twice as tall as the product when it chooses itself."""
    L = cn.lib()
    out = (C.c_int64 * 8)()
    rng = np.random.default_rng(0)
    shapes = [(128, 40000, 100000), (128, 20000, 40000), (128, 1024, 784), (784, 1024, 128),
              (128, 784, 1024), (100000, 8192, 128), (128, 4096, 4096), (2, 2, 3), (1, 1, 1),
              (128, 10, 4096), (5000, 5000, 31)]
    shapes += [tuple(int(v) for v in rng.integers(1, 3000, 3)) for _ in range(200)]
    for ws in (16 << 20, 1 << 30):
        for force in (0, 128, 256, 32, 64):
            for fn in (L.cn_host_plan_gemm, L.cn_host_plan_gemm_rows_along_k):
                for (M, N, K) in shapes:
                    fn(M, N, K, 256, ws, force, out)
                    tm, tn, kit, splits, ips, units, tile_n, tile_m = list(out)
                    assert (tile_m, tile_n) in ((128, 128), (128, 256), (64, 128), (32, 128))
                    if force in (32, 64):
                        assert tile_m == force and tile_n == 128
                    elif force in (128, 256):
                        assert tile_m == 128 and tile_n == force
                    else:
                        assert tile_m == 32 or M > tile_m // 2
                    assert tm == -(-M // tile_m) and tn == -(-N // tile_n) and kit == max(1, -(-K // (32 if tile_n == 128 else 16)))
                    assert splits >= 1 and units == tm * tn * splits
                    assert ips * splits >= kit and ips * (splits - 1) < kit  # every chunk non-empty
                    if splits > 1:
                        assert splits * M * N * 4 <= ws
                        assert ips >= (8 if tile_n == 256 else 4)  # a chunk is at least 128 k deep
    L.cn_host_plan_gemm(128, 40000, 100000, 256, 1 << 30, 128, out)
    assert list(out)[:6] == [1, 313, 3125, 13, 241, 4069]


# (tile rows, tile columns, K chunks, stages per chunk) on 256 compute units with a 1 GiB workspace, as measured best or within
# 2 % of the best geometry on an MI355X (tests/test_gpu_planner.py holds the planner to that on the GPU; this freezes the
# answers so that a change of a rule or a constant shows up without one).
FROZEN_PLANS = {
    ("dot", 128, 1024, 784): (32, 128, 5, 5),
    ("Tdot", 784, 1024, 128): (32, 128, 1, 4),
    ("dotT", 128, 784, 1024): (32, 128, 8, 4),
    ("dot", 128, 40000, 100000): (128, 256, 13, 481),
    ("dot", 128, 20000, 40000): (128, 128, 13, 97),
    ("dot", 32, 4096, 4096): (32, 128, 8, 16),
    ("dot", 128, 4096, 4096): (64, 128, 8, 16),
    ("dot", 512, 4096, 4096): (64, 128, 2, 64),
    ("dot", 128, 8192, 100000): (128, 256, 16, 391),
    ("dot", 128, 8192, 4096): (64, 128, 4, 32),
    ("dot", 128, 10, 4096): (32, 128, 32, 4),
    ("Tdot", 100000, 8192, 128): (128, 256, 1, 8),
    ("Tdot", 4096, 8192, 128): (128, 256, 1, 8),
    ("Tdot", 4096, 10, 128): (32, 128, 1, 4),
    ("dotT", 128, 4096, 8192): (64, 128, 8, 32),
    ("dotT", 128, 4096, 10): (32, 128, 1, 1),
    ("dotT", 128, 100000, 8192): (128, 256, 5, 103),
    ("dot", 128, 3000, 40000): (128, 128, 21, 60),
    ("dot", 128, 8192, 8192): (64, 128, 4, 64),
    ("Tdot", 128, 8192, 4096): (128, 128, 8, 16),
    ("Tdot", 128, 4096, 8192): (128, 128, 16, 16),
    ("dot", 4096, 4096, 4096): (128, 256, 1, 256),
    ("dot", 8192, 8192, 512): (128, 256, 1, 32),
    ("dot", 32, 40000, 100000): (32, 128, 13, 241),
    ("dot", 64, 40000, 100000): (64, 128, 13, 241),
    ("dot", 256, 1024, 1024): (32, 128, 4, 8),
    ("Tdot", 3000, 3000, 300): (64, 128, 1, 10),
    ("dot", 500, 1024, 784): (32, 128, 2, 13),
    ("Tdot", 37, 1029, 515): (32, 128, 4, 5),
}


def test_plans_of_the_benchmark_shapes_are_the_measured_ones():
    L = cn.lib()
    out = (C.c_int64 * 8)()
    for (op, M, N, K), want in FROZEN_PLANS.items():
        (L.cn_host_plan_gemm if op == "Tdot" else L.cn_host_plan_gemm_rows_along_k)(M, N, K, 256, 1 << 30, 0, out)
        tm, tn, kit, splits, ips, units, tile_n, tile_m = list(out)
        assert (tile_m, tile_n, splits, ips) == want, (op, M, N, K, (tile_m, tile_n, splits, ips), want)


def test_tile_counters_are_tied_to_streams():
    """Kernels that draw their tiles from a counter may share one only if a stream orders them.  The table behind
    Context::tile_counter_for: a stream keeps the counter it was first given, 32 distinct streams get the 32 counters, a
    33rd gets none (its kernels walk their tiles in a fixed pattern), and the default stream (handle 0) is a stream like
    any other."""
    import ctypes
    L = cn.lib()
    keys = [0, 0x7f00, 0, 0x7f10, 0x7f00] + [0x9000 + 16 * i for i in range(40)] + [0x7f10, 0]
    arr = (ctypes.c_uint64 * len(keys))(*keys)
    out = (ctypes.c_int * len(keys))()
    L.cn_host_stream_slots(arr, len(keys), out)
    got = list(out)
    assert got[:5] == [0, 1, 0, 2, 1]
    assert got[5:5 + 29] == list(range(3, 32)) and got[5 + 29:5 + 40] == [-1] * 11
    assert got[-2:] == [2, 0]


def test_bench_refuses_more_than_one_gpu_before_touching_any():
    """The benchmark measures one GPU; asked for more it says so and exits, before it imports torch or the library."""
    import subprocess
    import sys
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0 and proc.stdout.strip() == ""
    assert "one GPU" in proc.stderr and "--gpus 2" in proc.stderr
