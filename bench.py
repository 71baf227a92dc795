#!/usr/bin/env python3
"""Benchmark of the matrix-multiply + 8-bit codec path on one MI355X.

A step is the README workload of the reference on ONE GPU, un-sharded and resident in HBM:
    out1 = batch(128 x 100000) . W1(100000 x 40000);  out2 = out1 . W2(40000 x 20000)
(fp32, ~19 GB, uniform inputs, synthetic).  `value` is (2*128*100000*40000 + 2*128*40000*20000)
FLOP divided by the wall time of a step.  The dominant kernel is the 128 x 40000 x 100000 dot; its
own duration is measured with events on the launch stream inside the timed steps and priced
against the fp32 matrix-core peak.  After the timed region the codec kernels (compression_8bit,
decompression_8bit, absmax) and the fused 8-bit-weight GEMM are measured on their own workloads and
reported under "extra"; the CPU port of the same arithmetic is timed on a bounded sample.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--only gemm|codec|fused|step|products] [--no-cpu] [--zero-operands]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBPS = 8000.0          # MI355X HBM3E peak

M, K1, N1, N2 = 128, 100000, 40000, 20000
FLOP1 = 2.0 * M * N1 * K1
FLOP2 = 2.0 * M * N2 * N1

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file (profiles/gemm_and_codec_kernels_hbm_traffic.txt): FETCH_SIZE 7956620 KiB x 2.0 (the factor
# that makes the same counter read 3276.8 MB on a 3276.8 MB device-to-device copy) + WRITE_SIZE
# 260000 KiB x 1.0.  Algorithmic bytes of the same launch: 16.07e9.
TRAFFIC_BYTES_GEMM1 = 7956620 * 1024 * 2.0 + 260000 * 1024 * 1.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_uniform(torch, shape, limit, dev, gen, chunk_rows=10000):
    out = torch.empty(shape, dtype=torch.float32, device=dev)
    for r in range(0, shape[0], chunk_rows):
        blk = out[r:r + chunk_rows]
        blk.uniform_(-limit, limit, generator=gen)
    return out


def event_pair(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_region(torch, fn, iters, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s, e = event_pair(torch)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters  # ms


def stats(ts):
    """mean, median and minimum of a list of times."""
    ts = sorted(ts)
    return {"mean": sum(ts) / len(ts), "median": ts[len(ts) // 2], "min": ts[0]}


def time_each(torch, fn, iters, warmup):
    """ms per call from an event pair round every call: {"mean", "median", "min"}.  For calls long enough that the gap
    a host launch leaves does not matter (tens of microseconds and more)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [event_pair(torch) for _ in range(iters)]
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return stats([s.elapsed_time(e) for s, e in ev])


def time_replayed(torch, fn, calls, replays, want_stats=False):
    """ms per call with the host out of the way: `calls` calls captured into one HIP graph, the graph
    replayed `replays` times between two events.  For kernels of a few microseconds, where the loop of
    time_region measures how fast Python can launch.  Every replay has its own event pair; the mean over the replays
    (or, want_stats, mean / median / min) is returned.  None if the capture is refused."""
    try:
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(calls):
                fn()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        ev = [event_pair(torch) for _ in range(replays)]
        for s, e in ev:
            s.record()
            graph.replay()
            e.record()
        torch.cuda.synchronize()
        st = stats([s.elapsed_time(e) / calls for s, e in ev])
        if want_stats:
            return st
        return st["mean"]
    except Exception:  # noqa: BLE001 - any refusal means "not measured this way"
        torch.cuda.synchronize()
        return None


def bench_gemm(torch, cn, dev, steps, warmup, zeros=False):
    gen = torch.Generator(device=dev).manual_seed(1234)
    if zeros:
        # same kernels, same schedule, no switching activity in the operands: separates what the code
        # can issue from what the part sustains under the power of real data
        batch = torch.zeros((M, K1), device=dev)
        W1 = torch.zeros((K1, N1), device=dev)
        W2 = torch.zeros((N1, N2), device=dev)
    else:
        batch = torch.rand((M, K1), device=dev, generator=gen)
        W1 = make_uniform(torch, (K1, N1), (6.0 / (K1 + N1)) ** 0.5, dev, gen)
        W2 = make_uniform(torch, (N1, N2), (6.0 / (N1 + N2)) ** 0.5, dev, gen)
    out1 = torch.empty((M, N1), device=dev)
    out2 = torch.empty((M, N2), device=dev)

    def step(ev=None):
        if ev is not None:
            ev[0].record()
        cn.dot(batch, W1, out1)
        if ev is not None:
            ev[1].record()
        cn.dot(out1, W2, out2)
        if ev is not None:
            ev[2].record()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        step(events[i])
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    g1 = stats([e[0].elapsed_time(e[1]) for e in events])
    g2 = stats([e[1].elapsed_time(e[2]) for e in events])
    pair = stats([e[0].elapsed_time(e[2]) for e in events])
    return {"wall_ms": wall_ms, "gemm1_ms": g1["mean"], "gemm2_ms": g2["mean"], "gemm1": g1, "gemm2": g2, "pair": pair,
            "tensors": (batch, W1, W2, out1, out2)}


def bench_codec(torch, cn, dev):
    """compression_8bit / decompression_8bit / absmax on the 100000 x 8192 gradient of the training
    configuration (819.2 M elements, 3.28 GB fp32) and on the 128 x 40000 round-trip tensor."""
    res = {}
    gen = torch.Generator(device=dev).manual_seed(99)
    for name, n, iters in (("grad_100000x8192", 100000 * 8192, 20), ("cfg2_128x40000", 128 * 40000, 200),
                           ("ref_microbench_5120x5120", 5120 * 5120, 100), ("layer_784x1024", 784 * 1024, 200)):
        x = torch.empty(n, device=dev).normal_(0.0, 0.02, generator=gen)
        idx = torch.randint(0, n, (n // 100,), device=dev, generator=gen)
        x[idx] = torch.empty(idx.numel(), device=dev).normal_(0.0, 0.5, generator=gen)
        del idx
        prec_t = cn.absmax(x)
        prec = float(prec_t.cpu()[0])
        codes = torch.empty(n, dtype=torch.uint8, device=dev)
        back = torch.empty(n, device=dev)
        warm = 3 if n >= 100000 * 8192 else 1000  # microsecond kernels: let the clocks come up first
        big = n >= 100000 * 8192
        if big:  # hundreds of microseconds per call: an event pair round every call
            st_abs = time_each(torch, lambda: cn.absmax(x, prec_t), iters, warm)
            st_c = time_each(torch, lambda: cn.compression_8bit(x, prec, codes), iters, warm)
            st_d = time_each(torch, lambda: cn.decompression_8bit(codes, prec, back), iters, warm)
            t_abs, t_c, t_d = st_abs["median"], st_c["median"], st_d["median"]
            how = "an event pair round every call, %d calls; figures from the median, mean and min beside it" % iters
        else:    # microseconds per call: back-to-back launches between two events (mean); medians under replayed_from_a_graph
            t_abs = time_region(torch, lambda: cn.absmax(x, prec_t), iters, warm)
            t_c = time_region(torch, lambda: cn.compression_8bit(x, prec, codes), iters, warm)
            t_d = time_region(torch, lambda: cn.decompression_8bit(codes, prec, back), iters, warm)
            how = "%d back-to-back calls between two events (mean); per-call medians and minima under replayed_from_a_graph" % iters
        t_copy = time_region(torch, lambda: back.copy_(x), iters, warm)
        res[name] = {
            "elements": n, "timing": how,
            "absmax_GBps": 4.0 * n / t_abs / 1e6, "absmax_us": t_abs * 1e3,
            "compress_GBps": 5.0 * n / t_c / 1e6, "compress_us": t_c * 1e3,
            "decompress_GBps": 5.0 * n / t_d / 1e6, "decompress_us": t_d * 1e3,
            "copy_GBps": 8.0 * n / t_copy / 1e6,
            "compress_frac_hbm_peak": 5.0 * n / t_c / 1e6 / PEAK_HBM_GBPS,
            "decompress_frac_hbm_peak": 5.0 * n / t_d / 1e6 / PEAK_HBM_GBPS,
            "absmax_frac_hbm_peak": 4.0 * n / t_abs / 1e6 / PEAK_HBM_GBPS,
        }
        if big:
            for key, st in (("absmax", st_abs), ("compress", st_c), ("decompress", st_d)):
                res[name][key + "_us_mean"] = st["mean"] * 1e3
                res[name][key + "_us_min"] = st["min"] * 1e3
        if n < 100000 * 8192:
            # small buffers: the kernels take a few microseconds, so also time them replayed from a graph
            replayed = {"absmax_us": time_replayed(torch, lambda: cn.absmax(x, prec_t), 20, 50),
                        "compress_us": time_replayed(torch, lambda: cn.compression_8bit(x, prec_t, codes), 20, 50),
                        "decompress_us": time_replayed(torch, lambda: cn.decompression_8bit(codes, prec_t, back), 20, 50),
                        "absmax_then_compress_us": time_replayed(
                            torch, lambda: (cn.absmax(x, prec_t), cn.compression_8bit(x, prec_t, codes)), 20, 50),
                        "absmax_compress_one_call_us": time_replayed(
                            torch, lambda: cn.absmax_compression_8bit(x, codes, prec_t), 20, 50)}
            # the one call pinned to each of its two forms (it picks by size)
            for label, mode in (("absmax_compress_two_kernels_us", 0), ("absmax_compress_single_launch_us", 1)):
                cn.lib().cn_host_absmax_compress_single_launch(mode)
                replayed[label] = time_replayed(torch, lambda: cn.absmax_compression_8bit(x, codes, prec_t), 20, 50)
            cn.lib().cn_host_absmax_compress_single_launch(-1)
            # the other encoders beside the one the library picks for this size (same bits)
            for label, which in (("compress_literal_us", 1), ("compress_table_on_quotient_us", 2), ("compress_own_table_us", 3)):
                if which == 1 and n > (8 << 20):
                    continue
                cn.lib().cn_host_codec_encoder(which)
                replayed[label] = time_replayed(torch, lambda: cn.compression_8bit(x, prec_t, codes), 20, 50)
                cn.lib().cn_host_codec_encoder(0)
            res[name]["replayed_from_a_graph"] = {k: (v * 1e3 if v is not None else None) for k, v in replayed.items()}
            for key, fn in (("absmax", lambda: cn.absmax(x, prec_t)), ("compress", lambda: cn.compression_8bit(x, prec_t, codes)),
                            ("decompress", lambda: cn.decompression_8bit(codes, prec_t, back))):
                st = time_replayed(torch, fn, 20, 50, want_stats=True)
                if st is not None:
                    res[name]["replayed_from_a_graph"][key + "_us_median_min"] = [st["median"] * 1e3, st["min"] * 1e3]
        if n >= 100000 * 8192:
            # movers that are not this library's: the runtime's device-to-device copy (above) and its fill, the latter a
            # pure write stream.  What access patterns reach on this part at all is in profiles/stream_patterns_sweep_819M_elements.txt.
            t_fill = time_region(torch, lambda: back.fill_(1.0), iters, warm)
            res[name]["fill_GBps"] = 4.0 * n / t_fill / 1e6
        del x, codes, back
    return res


def bench_cfg1(torch, cn, dev):
    """The reference's own small case: one 784 -> 1024 layer on a batch of 128 (forward product, weight
    gradient, input gradient; 0.2 GFLOP each).  Microsecond kernels, so timed replayed from a HIP graph where
    the capture is allowed, else launched one by one."""
    gen = torch.Generator(device=dev).manual_seed(11)
    A = torch.rand((128, 784), device=dev, generator=gen)
    W = make_uniform(torch, (784, 1024), (6.0 / (784 + 1024)) ** 0.5, dev, gen)
    dC = torch.empty((128, 1024), device=dev).normal_(0.0, 0.01, generator=gen)
    out = {}
    for name, fn, shape in (("dot_128x1024x784", lambda c: cn.gemm(A, W, False, False, out=c), (128, 1024)),
                            ("Tdot_784x1024x128", lambda c: cn.gemm(A, dC, True, False, out=c), (784, 1024)),
                            ("dotT_128x784x1024", lambda c: cn.gemm(dC, W, False, True, out=c), (128, 784))):
        C = torch.empty(shape, device=dev)
        st = time_replayed(torch, lambda: fn(C), 20, 50, want_stats=True)
        how = "replayed from a graph, 50 replays of 20 calls"
        if st is None:
            st, how = time_each(torch, lambda: fn(C), 200, 1000), "launched one by one"
        t = st["median"]
        out[name] = {"us": t * 1e3, "us_mean": st["mean"] * 1e3, "us_min": st["min"] * 1e3,
                     "TFLOPs": 2.0 * 128 * 784 * 1024 / t / 1e9, "timing": how + "; figures from the median"}
    return out


def bench_layout(torch, cn, dev):
    """The passes either side of the products: transposition (the reference's T / to_col_major, source/basicOps.cu:14-127)
    and fill (zeros / ones / fill), on the 100000 x 8192 weights; torch's own beside them as movers that are not this
    library's."""
    from clusternet_amd import _lib as L
    rows, cols = 100000, 8192
    n = rows * cols
    A = torch.empty((rows, cols), device=dev).normal_(0.0, 1.0)
    out = torch.empty((cols, rows), device=dev)
    res = {}
    t = time_region(torch, lambda: L.transpose(A, out), 20, 3)
    res["transpose_GBps"] = 8.0 * n / t / 1e6
    res["transpose_ms"] = t
    t = time_region(torch, lambda: out.copy_(A.t()), 10, 2)
    res["torch_transpose_GBps"] = 8.0 * n / t / 1e6
    t = time_region(torch, lambda: L.fill(out, 1.0), 20, 3)
    res["fill_GBps"] = 4.0 * n / t / 1e6
    t = time_region(torch, lambda: out.fill_(1.0), 20, 3)
    res["torch_fill_GBps"] = 4.0 * n / t / 1e6
    return res


def bench_fused(torch, cn, dev):
    """C = A . decode(W8) for A {32,128,512} x 4096, W 4096 x 4096: fused kernel against
    decompression_8bit followed by dot."""
    res = {}
    gen = torch.Generator(device=dev).manual_seed(7)
    W = torch.empty((4096, 4096), device=dev).normal_(0.0, 1.0 / 64.0, generator=gen)
    scale = float(cn.absmax(W).cpu()[0])
    codes = cn.compression_8bit(W, scale)
    Wd = torch.empty_like(W)
    for b in (32, 128, 512):
        A = torch.empty((b, 4096), device=dev).normal_(0.0, 1.0, generator=gen)
        C = torch.empty((b, 4096), device=dev)
        t_f = time_region(torch, lambda: cn.gemm_w8(A, codes, scale, C), 200, 5)

        def unfused():
            cn.decompression_8bit(codes, scale, Wd)
            cn.dot(A, Wd, C)
        t_u = time_region(torch, unfused, 200, 5)
        t_g = time_region(torch, lambda: cn.dot(A, Wd, C), 200, 5)
        res["batch%d" % b] = {"fused_us": t_f * 1e3, "decompress_plus_dot_us": t_u * 1e3,
                              "dot_fp32_only_us": t_g * 1e3, "speedup": t_u / t_f,
                              "fused_TFLOPs": 2.0 * b * 4096 * 4096 / t_f / 1e9,
                              "timing": "200 back-to-back calls between two events (mean); replayed: 50 replays of a graph of 20 calls, "
                                        "[median, min] per call"}
        for key, fn in (("fused", lambda: cn.gemm_w8(A, codes, scale, C)), ("decompress_plus_dot", unfused)):
            st = time_replayed(torch, fn, 20, 50, want_stats=True)
            if st is not None:
                res["batch%d" % b][key + "_us_replayed_median_min"] = [st["median"] * 1e3, st["min"] * 1e3]
        # these batches take the kernel that decodes into registers; the tiled kernel it replaces there, for comparison
        cn.lib().cn_host_gemm_w8_rows(0)
        res["batch%d" % b]["fused_tiled_kernel_us"] = time_region(torch, lambda: cn.gemm_w8(A, codes, scale, C), 200, 5) * 1e3
        cn.lib().cn_host_gemm_w8_rows(1)
    return res


def bench_step(torch, cn, dev):
    """Maxout training step of the reference's benchmark network at its full sizes (batch 128,
    100000 -> 8192 -> 8192 -> 10 with pool 2, 2 % dense input): forward, backward, 8-bit gradient round
    trip and update, phase by phase."""
    from clusternet_amd import maxout_step as ms
    from clusternet_amd import _lib as L
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    B, D, H, C, pool = 128, 100000, 8192, 10, 2
    X = torch.rand((B, D), device=dev, generator=gen)
    X = X * (torch.rand((B, D), device=dev, generator=gen) < 0.02)
    W1 = make_uniform(torch, (D, H), (6.0 / (D + H)) ** 0.5, dev, gen)
    W2 = make_uniform(torch, (H // pool, H), (6.0 / (H // pool + H)) ** 0.5, dev, gen)
    W3 = make_uniform(torch, (H // pool, C), (6.0 / (H // pool + C)) ** 0.5, dev, gen)
    b1 = torch.zeros(H, device=dev); b2 = torch.zeros(H, device=dev); b3 = torch.zeros(C, device=dev)
    params = (W1, b1, W2, b2, W3, b3)
    onehot = torch.zeros((B, C), device=dev)
    onehot[torch.arange(B, device=dev), torch.randint(0, C, (B,), device=dev, generator=gen)] = 1.0
    state = {}

    def fwd():
        state["p"], state["cache"] = ms.forward(X, params, pool)

    def bwd():
        state["grads"] = ms.backward(X, onehot, params, state["p"], state["cache"], pool)

    maxima = [torch.empty(1, device=dev) for _ in range(3)]

    def bwd_absmax():  # the gradient products also deliver max|gW|
        state["grads"] = ms.backward(X, onehot, params, state["p"], state["cache"], pool, absmax_out=maxima)

    def codec_update_given_max():
        for w, g, m in zip((W1, W2, W3), state["grads"], maxima):
            ms.coded_update(w, g, 1e-3, fused=True, prec=m)

    def codec_update():
        for w, g in zip((W1, W2, W3), state["grads"]):
            ms.coded_update(w, g, 1e-3, fused=True)

    def codec_update_unfused():
        for w, g in zip((W1, W2, W3), state["grads"]):
            ms.coded_update(w, g, 1e-3, fused=False, scratch=scratch[:g.numel()].view(g.shape))

    rms = [torch.full_like(w, 1e-4) for w in (W1, W2, W3)]
    scratch = torch.empty(W1.numel(), device=dev)  # where the unfused variants decode to

    def codec_rmsprop():
        for w, r, g in zip((W1, W2, W3), rms, state["grads"]):
            ms.coded_rmsprop_update(w, r, g, 0.9, 1e-3, fused=True)

    def codec_rmsprop_unfused():
        for w, r, g in zip((W1, W2, W3), rms, state["grads"]):
            ms.coded_rmsprop_update(w, r, g, 0.9, 1e-3, fused=False, scratch=scratch[:g.numel()].view(g.shape))

    def to_sparse():
        state["Xs"] = ms.sparse_input(X)

    def fwd_sparse():
        state["p"], state["cache"] = ms.forward(state["Xs"], params, pool)

    def bwd_absmax_sparse():
        state["grads"] = ms.backward(state["Xs"], onehot, params, state["p"], state["cache"], pool, absmax_out=maxima)

    def bwd_deferred_sparse():  # the first layer's gradient is left to first_layer_update below
        state["grads"] = ms.backward(state["Xs"], onehot, params, state["p"], state["cache"], pool, absmax_out=maxima,
                                     defer_first=True)
        state["e1"] = state["grads"][0]

    codes1 = torch.empty((D, H), dtype=torch.uint8, device=dev)

    def first_layer_update():  # max|X^T e1|, then codes + weight update from the recomputed gradient rows
        ms.coded_sparse_update(W1, state["Xs"], state["grads"][0], 1e-3, prec=maxima[0], codes=codes1)

    def first_layer_rmsprop():
        ms.coded_sparse_rmsprop_update(W1, rms[0], state["Xs"], state["e1"], 0.9, 1e-3, prec=maxima[0], codes=codes1)

    def other_layers_update():
        for w, g, m in zip((W2, W3), state["grads"][1:], maxima[1:]):
            ms.coded_update(w, g, 1e-3, fused=True, prec=m)

    out = {}
    for name, fn in (("sparse_input", to_sparse), ("forward_sparse", fwd_sparse),
                     ("backward_deferred_sparse", bwd_deferred_sparse),
                     ("first_layer_codes_and_update_sparse", first_layer_update),
                     ("other_layers_compress_and_update", other_layers_update),
                     ("backward_with_absmax_sparse", bwd_absmax_sparse),
                     ("forward", fwd), ("backward_with_absmax", bwd_absmax),
                     ("compress_and_update_given_absmax", codec_update_given_max),
                     ("backward", bwd), ("codec_and_update", codec_update),
                     ("codec_and_update_unfused", codec_update_unfused), ("codec_and_rmsprop", codec_rmsprop),
                     ("codec_and_rmsprop_unfused", codec_rmsprop_unfused),
                     ("first_layer_codes_and_rmsprop_sparse", first_layer_rmsprop)):
        st = time_each(torch, fn, 7, 2)
        out[name + "_ms"] = st["median"]
        out[name + "_ms_mean_min"] = [st["mean"], st["min"]]
    flop_f = 2.0 * B * (D * H + (H // pool) * H + (H // pool) * C)
    flop_b = flop_f + 2.0 * B * ((H // pool) * H + (H // pool) * C)
    elems = D * H + (H // pool) * H + (H // pool) * C
    out["forward_TFLOPs"] = flop_f / (out["forward_ms"] * 1e-3) / 1e12
    out["backward_TFLOPs"] = flop_b / (out["backward_ms"] * 1e-3) / 1e12
    out["codec_and_update_GBps"] = elems * (4 + 13) / (out["codec_and_update_ms"] * 1e-3) / 1e9
    out["codec_and_update_unfused_GBps"] = elems * (4 + 5 + 5 + 12) / (out["codec_and_update_unfused_ms"] * 1e-3) / 1e9
    out["codec_and_rmsprop_GBps"] = elems * (4 + 5 + 17) / (out["codec_and_rmsprop_ms"] * 1e-3) / 1e9
    out["codec_and_rmsprop_unfused_GBps"] = elems * (4 + 5 + 5 + 20) / (out["codec_and_rmsprop_unfused_ms"] * 1e-3) / 1e9
    out["step_ms"] = out["forward_ms"] + out["backward_with_absmax_ms"] + out["compress_and_update_given_absmax_ms"]
    out["step_sparse_ms"] = (out["sparse_input_ms"] + out["forward_sparse_ms"] + out["backward_with_absmax_sparse_ms"] +
                             out["compress_and_update_given_absmax_ms"])
    out["step_sparse_fused_ms"] = (out["sparse_input_ms"] + out["forward_sparse_ms"] + out["backward_deferred_sparse_ms"] +
                                   out["first_layer_codes_and_update_sparse_ms"] + out["other_layers_compress_and_update_ms"])
    out["step_unfused_ms"] = out["forward_ms"] + out["backward_ms"] + out["codec_and_update_unfused_ms"]
    out["timing"] = "an event pair round every call of a phase, 7 calls; figures from the median"
    out["note"] = ("bytes per gradient element: absmax 4, then codes and update in one pass 13 (unfused: compress 5 + "
                   "decompress 5 + update 12), or compress 5 + fused decode+RMSprop 17 (unfused 5 + 5 + 20); "
                   "the gradient GEMM of layer 1 is 100000 x 8192 x 128")
    return out


def bench_products(torch, cn, dev, zeros=False):
    """The backward products of the maxout training step one by one at their full shapes, each on its own (the step's
    phases above time several kernels together): the second layer's input gradient dotT 128 x 4096 x 8192, the first
    layer's weight gradient Tdot 100000 x 8192 x 128, and the first layer's input gradient dotT 128 x 100000 x 8192
    (reads all of W1).  Every call is timed by its own pair of events; mean, median and minimum are reported."""
    gen = torch.Generator(device=dev).manual_seed(21)
    B, D, H = 128, 100000, 8192
    if zeros:  # profiling aid, as for the README pair: what the code can issue, without the power of switching data
        X, E = torch.zeros((B, D), device=dev), torch.zeros((B, H), device=dev)
        W2, W1 = torch.zeros((H // 2, H), device=dev), torch.zeros((D, H), device=dev)
    else:
        X = torch.rand((B, D), device=dev, generator=gen)
        E = torch.empty((B, H), device=dev).normal_(0.0, 0.01, generator=gen)
        W2 = make_uniform(torch, (H // 2, H), (6.0 / (H // 2 + H)) ** 0.5, dev, gen)
        W1 = make_uniform(torch, (D, H), (6.0 / (D + H)) ** 0.5, dev, gen)
    out = {"operands": "all zero (profiling aid, not a result)"} if zeros else {}
    for name, a, b, ta, tb, shape, iters in (("dotT_128x4096x8192", E, W2, False, True, (B, H // 2), 200),
                                             ("Tdot_100000x8192x128", X, E, True, False, (D, H), 20),
                                             ("dotT_128x100000x8192", E, W1, False, True, (B, D), 20)):
        C = torch.empty(shape, device=dev)
        flop = 2.0 * C.shape[0] * C.shape[1] * (a.shape[0] if ta else a.shape[1])
        fn = lambda: cn.gemm(a, b, ta, tb, out=C)
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        ev = [event_pair(torch) for _ in range(iters)]
        for s, e in ev:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        ts = sorted(s.elapsed_time(e) for s, e in ev)
        mean, med, mn = sum(ts) / len(ts), ts[len(ts) // 2], ts[0]
        rec = {"mean_us": mean * 1e3, "median_us": med * 1e3, "min_us": mn * 1e3,
               "TFLOPs": flop / (med * 1e-3) / 1e12, "frac_mfma_peak": flop / (med * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
               "timing": "an event pair round every call, %d calls; TFLOPs from the median" % iters}
        if C.numel() * 4 < (64 << 20):
            t = time_replayed(torch, fn, 20, 20)
            if t is not None:
                rec["replayed_from_a_graph_us"] = t * 1e3
                rec["replayed_frac_mfma_peak"] = flop / (t * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS
        out[name] = rec
        del C
    return out


def describe_plan(cn, torch, m, n, k):
    """The decomposition the library plans for an m x n x k dot on this GPU, in words, from its own planner."""
    import ctypes
    out = (ctypes.c_int64 * 8)()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ws = (int(os.environ.get("CNHIP_WORKSPACE_MB", "1024")) << 20)
    cn.lib().cn_host_plan_gemm_rows_along_k(m, n, k, cus, ws, 0, out)
    tiles_m, tiles_n, k_iters, splits, ips, units, tile_n, tile_m = [int(v) for v in out]
    text = "gemm_kernel on %d x %d tiles, %d tiles x %d K-chunks = %d workgroups" % (tile_m, tile_n, tiles_m * tiles_n, splits, units)
    return text + (", followed by splitk_reduce_kernel over the %d planes" % splits if splits > 1 else ", K not split")


def cpu_baseline(torch, tensors):
    """The CPU port (oracle/cpu_port.c, all OpenMP threads) on the full README pair, once: out1 = batch . W1 with W1 (16 GB)
    brought to the host in blocks of 10000 rows and the product accumulated block by block, then out2 = out1 . W2.  Only the
    time inside the port's GEMM counts; the copies from the device do not."""
    import numpy as np
    import oracle
    batch, W1, W2 = tensors[0], tensors[1], tensors[2]
    A = batch.cpu().numpy()
    oracle.port_gemm(A[:, :1024].copy(), np.ones((1024, 512), np.float32))  # thread pool warm-up
    out1 = np.zeros((M, N1), np.float32)
    t1 = 0.0
    rows = 10000
    for r in range(0, K1, rows):
        blk = W1[r:r + rows].cpu().numpy()
        t0 = time.perf_counter()
        oracle.port_gemm(A[:, r:r + rows], blk, out=out1, accumulate=True, lda=K1)
        t1 += time.perf_counter() - t0
        del blk
    W2h = W2.cpu().numpy()
    t0 = time.perf_counter()
    out2 = oracle.port_gemm(out1, W2h)
    t2 = time.perf_counter() - t0
    # the port's result against the GPU's, as a plausibility check of what was timed (fp32 accumulation in another order)
    dev2 = float(np.abs(out2 - tensors[4].cpu().numpy()).max() / max(float(np.abs(out2).max()), 1e-30))
    return {"value": (FLOP1 + FLOP2) / (t1 + t2) / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": "the full README pair once: 128x100000 . 100000x40000 (W1 streamed to the host in blocks of %d rows, %.2f s in "
                      "the port's GEMM, %.3f TFLOP/s) then 128x40000 . 40000x20000 (%.2f s, %.3f TFLOP/s); copies from the device not "
                      "timed; max deviation of out2 from the GPU's %.1e of max|out2|"
                      % (rows, t1, FLOP1 / t1 / 1e12, t2, FLOP2 / t2 / 1e12, dev2)}


def cpu_codec_baseline():
    """The literal per-element codec loops on all OpenMP threads, 64 M elements."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(0)
    x = rng.normal(0.0, 0.02, 1 << 26).astype(np.float32)
    prec = oracle.port_absmax(x)
    t0 = time.perf_counter(); codes = oracle.port_compress(x, prec); tc = time.perf_counter() - t0
    t0 = time.perf_counter(); oracle.port_decompress(codes, prec); td = time.perf_counter() - t0
    return {"elements": x.size, "cores": oracle.num_threads(), "kind": "port",
            "compress_GBps": 5.0 * x.size / tc / 1e9, "decompress_GBps": 5.0 * x.size / td / 1e9}


def cpu_port_maxout_step():
    """The maxout training step of the fifth configuration on the host cores, once, composed from the CPU port's pieces the
    way the reference composes its kernels (dense batch; source/Layer.cpp:256-334, source/DeepNeuralNetwork.cpp:334-339):
    three products with bias and maxout (softmax at the end), the backward products with the maxout expansions, and for
    every weight gradient abs-max, compression_8bit, decompression_8bit and the update.  Products and codec run on all
    OpenMP threads; the helpers on 128-row matrices and the update (numpy) on one.  Only the step itself is timed, not
    the making of the 3.3 GB of weights."""
    import numpy as np
    import torch
    import oracle
    B, D, H, O, pool, rate = 128, 100000, 8192, 10, 2, 0.01
    g = torch.Generator().manual_seed(3)
    X = (torch.rand((B, D), generator=g) * (torch.rand((B, D), generator=g) < 0.02)).numpy()
    # the large weights: a cheap pattern instead of 819 M random numbers (their values do not matter to the time)
    W1 = np.empty((D, H), np.float32)
    W1[:] = ((np.arange(H, dtype=np.float32) % 17.0) - 8.0) * np.float32(0.001)
    W2 = ((torch.rand((H // pool, H), generator=g) - 0.5) * 0.05).numpy()
    W3 = ((torch.rand((H // pool, O), generator=g) - 0.5) * 0.05).numpy()
    b1, b2, b3 = np.zeros(H, np.float32), np.zeros(H, np.float32), np.zeros(O, np.float32)
    onehot = np.zeros((B, O), np.float32)
    onehot[np.arange(B), np.arange(B) % O] = 1.0
    t = {}

    def timed(name, fn):
        t0 = time.perf_counter()
        r = fn()
        t[name] = t.get(name, 0.0) + time.perf_counter() - t0
        return r

    def layer(x, W, b):
        return oracle.maxout(oracle.add_row_vector(oracle.port_gemm(x, W), b), pool)

    def forward():
        h1, a1 = layer(X, W1, b1)
        h2, a2 = layer(h1, W2, b2)
        return oracle.softmax(oracle.add_row_vector(oracle.port_gemm(h2, W3), b3)), (h1, a1, h2, a2)

    def backward(p, cache):
        h1, a1, h2, a2 = cache
        e3 = p - onehot
        gW3 = oracle.port_gemm(h2, e3, True, False)
        e2 = oracle.expand_to_maxout_grad(oracle.port_gemm(e3, W3, False, True), a2, pool)
        gW2 = oracle.port_gemm(h1, e2, True, False)
        e1 = oracle.expand_to_maxout_grad(oracle.port_gemm(e2, W2, False, True), a1, pool)
        return oracle.port_gemm(X, e1, True, False), gW2, gW3

    def update(w, grad):
        prec = oracle.port_absmax(grad.reshape(-1))
        dec = oracle.port_decompress(oracle.port_compress(grad.reshape(-1), prec), prec)
        np.multiply(dec, np.float32(rate), out=dec)
        np.subtract(w.reshape(-1), dec, out=w.reshape(-1))

    oracle.port_gemm(X[:, :1024].copy(), np.ones((1024, 512), np.float32))  # thread pool warm-up
    p, cache = timed("forward_s", forward)
    grads = timed("backward_s", lambda: backward(p, cache))
    for w, grad in zip((W1, W2, W3), grads):
        timed("codec_and_update_s", lambda: update(w, grad))
    total = sum(t.values())
    return dict(t, step_s=total, cores=oracle.num_threads(), kind="port",
                note="one step, host clock; dense 128 x 100000 batch with 2 % nonzeros, layers 100000 -> 8192 (pool 2) -> 8192 (pool 2) "
                     "-> 10; products and codec on all threads, helpers and the update on one")


def cpu_port_configs():
    """The CPU port on the other configurations, all OpenMP threads: the three products of the 784 -> 1024 layer (batch 128), the
    128 x 40000 round-trip tensor (abs-max, compression, decompression), and decompression of 4096 x 4096 weights followed by the
    product at batch 32 / 128 / 512.  Each timed as the best of a few repetitions (small workloads; the first pass pays for
    the threads and the caches)."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(1)

    def best(fn, reps):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return min(ts)

    out = {"cores": oracle.num_threads(), "kind": "port", "timing": "best of several repetitions, host clock"}
    A = rng.uniform(0, 1, (128, 784)).astype(np.float32)
    W = rng.uniform(-0.0576, 0.0576, (784, 1024)).astype(np.float32)
    dC = rng.normal(0, 0.01, (128, 1024)).astype(np.float32)
    flop = 2.0 * 128 * 784 * 1024
    for name, fn in (("dot_128x1024x784", lambda: oracle.port_gemm(A, W)), ("Tdot_784x1024x128", lambda: oracle.port_gemm(A, dC, True, False)),
                     ("dotT_128x784x1024", lambda: oracle.port_gemm(dC, W, False, True))):
        t = best(fn, 20)
        out["layer_784x1024_" + name] = {"us": t * 1e6, "TFLOPs": flop / t / 1e12}
    x = rng.normal(0.0, 0.02, 128 * 40000).astype(np.float32)
    x[::100] = rng.normal(0.0, 0.5, x[::100].size).astype(np.float32)
    prec = oracle.port_absmax(x)
    codes = oracle.port_compress(x, prec)
    out["round_trip_128x40000"] = {"absmax_us": best(lambda: oracle.port_absmax(x), 10) * 1e6,
                                   "compress_us": best(lambda: oracle.port_compress(x, prec), 10) * 1e6,
                                   "decompress_us": best(lambda: oracle.port_decompress(codes, prec), 10) * 1e6}
    Wq = rng.normal(0.0, 1.0 / 64.0, (4096, 4096)).astype(np.float32)
    scale = oracle.port_absmax(Wq)
    Wc = oracle.port_compress(Wq, scale)
    t_dec = best(lambda: oracle.port_decompress(Wc, scale), 5)
    Wd = oracle.port_decompress(Wc, scale)
    for b in (32, 128, 512):
        Ab = rng.normal(0.0, 1.0, (b, 4096)).astype(np.float32)
        t = best(lambda: oracle.port_gemm(Ab, Wd), 5)
        out["w8_gemm_batch%d" % b] = {"decompress_us": t_dec * 1e6, "dot_us": t * 1e6, "TFLOPs_of_the_pair": 2.0 * b * 4096 * 4096 / (t + t_dec) / 1e12}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--only", choices=["gemm", "codec", "fused", "step", "products"], default=None,
                    help="run one part only (for profiling); prints a reduced JSON line")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--zero-operands", action="store_true",
                    help="profiling aid: the two products run on all-zero operands (the line is marked; not a result)")
    ap.add_argument("--whole-rows", action="store_true",
                    help="profiling aid: the sparse first-layer update runs every wavefront on whole rows instead of "
                         "splitting a workgroup into code-producing and weight-streaming wavefronts (the line is marked)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build runs the un-sharded workload on a single "
                 "MI355X and has no multi-GPU path (--gpus %d refused)" % args.gpus)

    import torch
    import clusternet_amd as cn
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    cn.init(0)
    if args.whole_rows:
        cn.lib().cn_host_csr_paired_rows(0)

    line = {"metric": "fp32 GEMM TFLOP/s at 128x100000x40000 (%MFMA peak); 8-bit codec GB/s",
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic",
            "config": {"workload": "README dotMPI pair on one GPU, un-sharded: 128x100000 . 100000x40000 "
                                   "then 128x40000 . 40000x20000, fp32, resident in HBM"}}
    extra = {}

    def section(name, fn):
        """A side measurement must not cost the headline line: its failure is recorded in its place."""
        try:
            extra[name] = fn()
        except Exception as exc:  # noqa: BLE001
            extra[name] = {"error": "%s: %s" % (type(exc).__name__, exc)}
            try:
                torch.cuda.synchronize()
            except Exception:  # noqa: BLE001
                pass

    if args.only in (None, "gemm"):
        g = bench_gemm(torch, cn, dev, args.steps, args.warmup, zeros=args.zero_operands)
        if args.zero_operands:
            line["data"] = "all-zero operands (profiling aid, not a result)"
        line["value"] = (FLOP1 + FLOP2) / (g["wall_ms"] * 1e-3) / 1e12
        line["ms_per_step"] = g["wall_ms"]
        achieved = FLOP1 / (g["gemm1_ms"] * 1e-3) / 1e12
        line["ms_per_step_median"] = g["pair"]["median"]
        line["ms_per_step_min"] = g["pair"]["min"]
        line["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS,
                            "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                            "traffic": TRAFFIC_BYTES_GEMM1,
                            "traffic_source": "profiles/gemm_and_codec_kernels_hbm_traffic.txt (FETCH_SIZE x 2.0 + WRITE_SIZE of this "
                                              "launch; the file names the commit it was measured on); not re-measured by this run",
                            "kernel": "128x40000x100000: %s; both are inside the timed bracket" % describe_plan(cn, torch, M, N1, K1),
                            "avg_ms": g["gemm1_ms"], "median_ms": g["gemm1"]["median"], "min_ms": g["gemm1"]["min"],
                            "frac_at_median": FLOP1 / (g["gemm1"]["median"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS}
        extra["gemm2_128x20000x40000"] = {"ms": g["gemm2_ms"], "ms_median": g["gemm2"]["median"], "ms_min": g["gemm2"]["min"],
                                          "TFLOPs": FLOP2 / (g["gemm2_ms"] * 1e-3) / 1e12,
                                          "frac_mfma_peak": FLOP2 / (g["gemm2_ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                                          "kernel": describe_plan(cn, torch, M, N2, N1)}
        extra["readme_pair_ms_reference_unknown_hw"] = 117.704285
        section("cfg1_layer_128x784x1024", lambda: bench_cfg1(torch, cn, dev))
        if not args.no_cpu and args.only is None:
            line["cpu_baseline"] = cpu_baseline(torch, g["tensors"])
        del g
        torch.cuda.empty_cache()
    if args.only in (None, "codec"):
        section("codec", lambda: bench_codec(torch, cn, dev))
        torch.cuda.empty_cache()
        if not args.no_cpu and args.only is None and "error" not in extra["codec"]:
            extra["codec"]["cpu_port"] = cpu_codec_baseline()
            section("cpu_port_other_configs", cpu_port_configs)
            section("cpu_port_maxout_step", cpu_port_maxout_step)
    if args.only in (None, "codec"):
        section("layout_100000x8192", lambda: bench_layout(torch, cn, dev))
        torch.cuda.empty_cache()
    if args.only in (None, "fused"):
        section("fused_w8_gemm_4096x4096", lambda: bench_fused(torch, cn, dev))
    if args.only in (None, "products"):
        torch.cuda.empty_cache()
        section("maxout_step_backward_products", lambda: bench_products(torch, cn, dev, zeros=args.zero_operands))
    if args.only in (None, "step"):
        torch.cuda.empty_cache()
        section("maxout_step_128x100000_8192_8192_10", lambda: bench_step(torch, cn, dev))
    if args.whole_rows:
        line["data"] += "; sparse update passes on whole rows (profiling aid, not the library's choice)"
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
