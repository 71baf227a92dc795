"""The planner's choice held against measurements.  For every shape below, the product as the library plans it
(tile geometry and K split from cn_host_plan_gemm's rules) is timed beside the same product with each tile geometry
forced (128 x 128, 128 x 256, 32 x 128, 64 x 128 output tiles; the K split is then planned for that geometry), and the
planned form may not be more than 7 % slower than the best of them.  Shapes: the products of the five benchmark
configurations (source/clusterNet.cpp:230-298 as called from source/Layer.cpp:256,327,334), the shapes the planner's own
rules were fitted on, and a ragged set.  Kernels of a few microseconds are timed replayed from a HIP graph (the host
cannot launch them as fast as they run), longer ones with an event pair round every call.  The table of the run is
written to planner_choice_table.txt in the directory CN_TEST_OUTPUT names (default: the run's output folder at the
top of the checkout)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GEOMETRIES = {"128x128": 128, "128x256": 256, "32x128": 32, "64x128": 64}
DOT, TDOT, DOTT = (False, False), (True, False), (False, True)

SHAPES = [
    # configuration 1: one 784 -> 1024 layer, batch 128
    ("cfg1 dot", 128, 1024, 784, DOT), ("cfg1 Tdot", 784, 1024, 128, TDOT), ("cfg1 dotT", 128, 784, 1024, DOTT),
    # configuration 3: the README pair
    ("cfg3 dot 1", 128, 40000, 100000, DOT), ("cfg3 dot 2", 128, 20000, 40000, DOT),
    # configuration 4: the fp32 product the fused 8-bit-weight product is compared with
    ("cfg4 batch 32", 32, 4096, 4096, DOT), ("cfg4 batch 128", 128, 4096, 4096, DOT), ("cfg4 batch 512", 512, 4096, 4096, DOT),
    # configuration 5: the maxout training step
    ("cfg5 fwd 1", 128, 8192, 100000, DOT), ("cfg5 fwd 2", 128, 8192, 4096, DOT), ("cfg5 fwd 3", 128, 10, 4096, DOT),
    ("cfg5 grad 1", 100000, 8192, 128, TDOT), ("cfg5 grad 2", 4096, 8192, 128, TDOT), ("cfg5 grad 3", 4096, 10, 128, TDOT),
    ("cfg5 back 2", 128, 4096, 8192, DOTT), ("cfg5 back 3", 128, 4096, 10, DOTT), ("cfg5 back 1", 128, 100000, 8192, DOTT),
    # shapes the planner's rules were fitted on
    ("128x3000x40000", 128, 3000, 40000, DOT), ("128x8192x8192", 128, 8192, 8192, DOT), ("128x8192x4096 Tdot", 128, 8192, 4096, TDOT),
    ("128x4096x8192 Tdot", 128, 4096, 8192, TDOT), ("4096^3", 4096, 4096, 4096, DOT), ("8192x8192x512", 8192, 8192, 512, DOT),
    ("32x40000x100000", 32, 40000, 100000, DOT), ("64x40000x100000", 64, 40000, 100000, DOT), ("256x1024x1024", 256, 1024, 1024, DOT),
    ("128x1024x80", 128, 1024, 80, DOT), ("16384x8192x1024", 16384, 8192, 1024, DOT), ("50000x4096x256 Tdot", 50000, 4096, 256, TDOT),
    # ragged
    ("129x130x33", 129, 130, 33, DOT), ("257x1000x640", 257, 1000, 640, DOT), ("100x10x4096", 100, 10, 4096, DOT),
    ("200x300x1000 dotT", 200, 300, 1000, DOTT), ("37x1029x515 Tdot", 37, 1029, 515, TDOT), ("1000x4x128", 1000, 4, 128, DOT),
    ("500x1024x784", 500, 1024, 784, DOT), ("640x5000x2000", 640, 5000, 2000, DOT), ("2000x2000x2000 dotT", 2000, 2000, 2000, DOTT),
    ("96x1000x1111 dotT", 96, 1000, 1111, DOTT), ("3000x3000x300 Tdot", 3000, 3000, 300, TDOT),
]


@pytest.fixture(scope="module")
def dev():
    import torch
    import clusternet_amd as cn
    cn.init(0)
    return torch.device("cuda:0")


def _time_us(torch, fn, rough_us):
    """Minimum over repetitions: of per-call event pairs for long kernels, of graph replays (ten calls each) for short ones."""
    if rough_us > 150.0:
        reps = 5 if rough_us > 2000.0 else 9
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for s, e in ev:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return min(s.elapsed_time(e) for s, e in ev) * 1e3
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(10):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(9)]
    for s, e in ev:
        s.record()
        graph.replay()
        e.record()
    torch.cuda.synchronize()
    return min(s.elapsed_time(e) for s, e in ev) * 1e2


def _rough_us(torch, fn):
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    fn()
    fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 500.0


def _measure(torch, cn, A, B, C, ta, tb):
    L = cn.lib()
    fn = lambda: cn.gemm(A, B, ta, tb, out=C)
    row = {}
    # the planned form is timed first and last (the first measurement of a shape meets cold caches and clocks on some boxes)
    for name, force in [("planned", 0)] + list(GEOMETRIES.items()) + [("planned", 0)]:
        L.cn_host_force_gemm_tile_n(force)
        t = _time_us(torch, fn, _rough_us(torch, fn))
        row[name] = min(t, row.get(name, t))
    L.cn_host_force_gemm_tile_n(0)
    return row


def test_planned_geometry_is_within_seven_percent_of_the_best(dev):
    import torch
    import clusternet_amd as cn
    L = cn.lib()
    g = torch.Generator(device=dev).manual_seed(2)
    lines = ["shape (M x N x K of C = op(A) op(B)) | planned us | 128x128 | 128x256 | 32x128 | 64x128 | planned / best"]
    late = []
    L.cn_host_gemm_small(0)  # the tiled kernel's geometries are what is compared; the one-launch kernel has its own line below
    try:
        for name, M, N, K, (ta, tb) in SHAPES:
            A = torch.rand((K, M) if ta else (M, K), device=dev, generator=g)
            B = (torch.rand((N, K) if tb else (K, N), device=dev, generator=g) - 0.5) * 0.02
            C = torch.empty((M, N), device=dev)
            row = _measure(torch, cn, A, B, C, ta, tb)
            best = min(row[k] for k in GEOMETRIES)
            if row["planned"] > 1.07 * best + 0.3:  # a second look before it counts: boxes have noisy moments
                again = _measure(torch, cn, A, B, C, ta, tb)
                row = {k: min(row[k], again[k]) for k in row}
                best = min(row[k] for k in GEOMETRIES)
            lines.append("%s: %d x %d x %d %s | %.1f | %.1f | %.1f | %.1f | %.1f | %.3f" %
                         (name, M, N, K, "Tdot" if ta else ("dotT" if tb else "dot"), row["planned"], row["128x128"], row["128x256"],
                          row["32x128"], row["64x128"], row["planned"] / best))
            if row["planned"] > 1.07 * best + 0.3:
                late.append(lines[-1])
            del A, B, C
        # the one-launch kernel for small products against the tiled kernel's plan, on the shapes it takes
        lines.append("")
        lines.append("one-launch kernel (products too small for tiles) | us | tiled kernel as planned us")
        for name, M, N, K, (ta, tb) in SHAPES:
            if M * N * K > (1 << 28):
                continue
            A = torch.rand((K, M) if ta else (M, K), device=dev, generator=g)
            B = (torch.rand((N, K) if tb else (K, N), device=dev, generator=g) - 0.5) * 0.02
            C = torch.empty((M, N), device=dev)
            fn = lambda: cn.gemm(A, B, ta, tb, out=C)
            L.cn_host_gemm_small(1)
            fn()
            took = L.cn_host_last_gemm_kernel(None)
            t_small = _time_us(torch, fn, 10.0)
            L.cn_host_gemm_small(0)
            t_tiled = _time_us(torch, fn, 10.0)
            lines.append("%s: %d x %d x %d | %.1f%s | %.1f" % (name, M, N, K, t_small, "" if took == 2 else " (tiled: the one-launch kernel does not take it)", t_tiled))
            if took == 2 and t_small > 1.07 * t_tiled + 0.3:
                late.append(lines[-1])
    finally:
        L.cn_host_gemm_small(1)
        L.cn_host_force_gemm_tile_n(0)
    out_dir = os.environ.get("CN_TEST_OUTPUT") or os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "planner_choice_table.txt"), "w") as f:
            f.write("\n".join(lines) + "\n")
    except OSError:
        pass
    assert not late, "planned form more than 7 % behind the best geometry:\n" + "\n".join(late)
