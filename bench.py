#!/usr/bin/env python3
"""Benchmark of the MI355X array-op hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-suite] [--no-cpu] [--only parts]

Headline (the JSON line's `value`): f32 GEMM TFLOP/s at M=N=K=4096, C = A·B, operands seeded
U(-1,1) and resident in HBM before the timed region.  One step = one pass of the kernel; W untimed
launches, then exactly K launches between two stream synchronisations.

stdout carries exactly one line, a JSON object of a few KB (a reader that keeps only the tail of the
output still gets all of it):
  roofline     - the GEMM kernel against the fp32 matrix peak: `achieved` is the flop count divided
                 by the average launch duration of those K launches, from HIP events on the stream they
                 run on.  Beside it, flat: the median of per-launch event pairs (`achieved_median`),
                 the three forms at the headline size, the slowest form of each size of the GEMM sweep,
                 one GB/s figure of ALGORITHMIC bytes (against 8 TB/s) per bandwidth-bound op of the
                 metric, the slowest op of a GiB or more, and the two MLP training loops in steps/s;
  cpu_baseline - the CPU side on this host's cores: the oracle's sgemm (a restatement of the
                 reference's loops; `kind: port`) on one pass of the same 4096^3 product, the same
                 product through numpy's bundled OpenBLAS (the reference's CPU GEMM is a CBLAS sgemm),
                 and the two training loops in steps/s.
The full tables (every sweep entry, every op of the bandwidth suite with its times, the training
loops' variants, the CPU streaming ops) go to stderr as they are measured and, as JSON, to the file
named by --detail.  An untimed second of matrix-core load (`config.spin_up_s`) precedes the W
declared warm-up launches of the headline.
Bandwidth ops and sweep entries are timed as the median of per-launch HIP-event pairs over at least
20 launches after at least 5 warm-ups and 25 ms of untimed launches of the same op
(`config.op_warm_ms`); operands below 512 MiB have the caches swept (a read of a
1 GiB scratch) between launches, outside the event pair.  A per-launch pair contains the launch gap
(about 6 us: `fill of one element` in the list); the GEMM sweep therefore also reports the rate of
launches queued back to back inside one pair.  Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MATRIX_PEAK_TFLOPS = 157.3   # MI355X dense fp32 MFMA
# HBM-side bytes of one 4096^3 A*B launch, from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs of
# this program (profiles/hbm_traffic_gemm_and_bandwidth_suite.md): (646261.4 KiB x 2.0 + 65536 KiB x 1.0) x 1024,
# the factors being what the same counters read for the 1 GiB device copy of known size.  The read
# figure moves by +-15 % from run to run (557 000 to 768 000 KiB raw) with what the caches still hold.
# A counter run cannot happen inside this program; the figure is that profile's, not this run's.
GEMM_4096_TRAFFIC_BYTES = 868778845  # (391450.6 x 2.000 + 65536.0 x 1.000) KiB: FETCH_SIZE + WRITE_SIZE medians of the headline kernel, scaled by the 1 GiB copy
HBM_PEAK_GBS = 8000.0             # MI355X HBM3E
SEED = 0x51CED
MIN_ITERS, MIN_WARMUP = 20, 5
SPIN_UP_SECONDS = 1.0             # untimed load before the headline's declared warm-up launches
OP_WARM_MS = 25.0                 # untimed launches of an op before its per-launch pairs, at least this long
MAX_LINE_BYTES = 4096             # the result line stays well below what a log tail keeps
DETAIL_DEFAULT = os.path.join(ROOT, "bench_detail.json")
# the ops the metric names, as they appear in the one-line summary: (short key, entry of the suite)
COMPACT_OPS = [
    ("sum_rows 16384^2", "sum_rows [16384x16384]"), ("sum_cols 16384^2", "sum_cols [16384x16384]"),
    ("max_rows 16384^2", "max_rows [16384x16384]"), ("max_cols 16384^2", "max_cols [16384x16384]"),
    ("mean 2^28", "mean [2^28]"), ("transpose 16384^2", "transpose [16384x16384]"),
    ("sum_cols 1x2^28", "sum_cols [1x268435456] -> 1"), ("max_rows 2^28x1", "max_rows [268435456x1] -> 1"),
    ("softmax fwd 32768x4096", "softmax fwd [32768x4096]"), ("softmax bwd 32768x4096", "softmax bwd [32768x4096]"),
    ("softmax fwd 8192x16384", "softmax fwd [8192x16384]"), ("softmax bwd 8192x16384", "softmax bwd [8192x16384]"),
    ("softmax fwd 2^20x128", "softmax fwd [1048576x128]"), ("max_rows 32768x4096", "max_rows [32768x4096]"),
    ("sum_rows 32768x4096", "sum_rows [32768x4096]"), ("transpose 32768x4096", "transpose [32768x4096]"),
    ("ew chain 2^28", "ew_chain ((a+b)*c-d)^2^2 [2^28], hand-fused kernel"),
    ("copy 1 GiB", "device copy [1 GiB] (achievable line)"),
]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def timed(ctx, fn, steps, warmup):
    """(wall ms per step with a stream sync on both sides, HIP-event ms per launch averaged over the
    same launches)."""
    for _ in range(warmup):
        fn()
    ctx.sync()
    e0, e1 = ctx.event(), ctx.event()
    t0 = time.perf_counter()
    ctx.record(e0)
    for _ in range(steps):
        fn()
    ctx.record(e1)
    ctx.sync()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = ctx.elapsed_ms(e0, e1) / steps
    ctx.lib.slhip_event_destroy(e0)
    ctx.lib.slhip_event_destroy(e1)
    return wall, ev


def pair_times(ctx, fn, iters=MIN_ITERS, warmup=MIN_WARMUP, sweep=None):
    """HIP-event milliseconds of every one of `iters` launches of fn(), each between its own pair of
    events on the stream it runs on, after `warmup` untimed launches.  sweep: a 1 GiB scratch buffer
    that is read through between launches, outside the pairs, to push the operands out of L2 and the
    memory-side cache."""
    iters, warmup = max(iters, MIN_ITERS), max(warmup, MIN_WARMUP)
    for _ in range(warmup):
        fn()
    # ... and more of them until OP_WARM_MS have passed: setting up an entry's operands (allocation,
    # generation, a wait) lets the clocks drop, and five launches of a 0.1 ms kernel do not bring them
    # back - whichever entry came first after a change of shape measured 1-4 % low (3584^3: 133 TFLOP/s
    # as the first of the three forms, 137 as the last)
    t0 = time.perf_counter()
    ctx.sync()
    while (time.perf_counter() - t0) * 1e3 < OP_WARM_MS:
        for _ in range(8):
            fn()
        ctx.sync()
    ev = [(ctx.event(), ctx.event()) for _ in range(iters)]
    for a, b in ev:
        if sweep is not None:
            # a READ of the scratch: it pushes the operands out and leaves no dirty lines behind whose
            # write-back the timed kernel would have to wait for (a fill as the sweep costs a 64 MiB
            # read 4 us more than this)
            ctx.call("slhip_max", sweep.n - 1, sweep.ptr, sweep.view(sweep.n - 1, 1).ptr)
        ctx.record(a)
        fn()
        ctx.record(b)
    ctx.sync()
    ms = [ctx.elapsed_ms(a, b) for a, b in ev]
    for a, b in ev:
        ctx.lib.slhip_event_destroy(a)
        ctx.lib.slhip_event_destroy(b)
    return ms


def median_ms(ctx, fn, iters=MIN_ITERS, warmup=MIN_WARMUP, sweep=None):
    return statistics.median(pair_times(ctx, fn, iters, warmup, sweep))


def write_detail(path, detail):
    """The full tables (GEMM sweep, every op of the bandwidth suite, the training loops, the CPU side)
    as one JSON file; the directory is created if it is missing.  Returns the path, or None when it
    cannot be written (the tables have gone to stderr as they were measured either way)."""
    if not path:
        return None
    try:
        os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
        with open(path, "w") as f:
            json.dump(detail, f, indent=1)
        return path
    except OSError as e:
        log("detail not written:", e)
        return None


def spin_up(ctx, a, b, c, n, seconds=SPIN_UP_SECONDS):
    """Untimed: keep the matrix cores under the headline's own load until clocks and power state have
    settled (the first launches after an idle period run at about 2.0 instead of 2.4 GHz, and a lighter
    spin-up kernel, or operand set-up between spin-up and timing, left the first timed block 2-4 % slow
    in some runs).  Uses the A*Bt kernel on the headline's own operands, right before the headline's
    warm-up launches, so that a profile of this program attributes only the headline's own warm-up
    and timed launches to the headline A*B kernel."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            ctx.call("slhip_sgemm", 0, 1, n, n, n, a.ptr, b.ptr, c.ptr, 0.0)
        ctx.sync()


def bench_gemm(ctx, m, n, k, ta, tb, steps, warmup, beta=0.0, sweep=None, headline=False, back_to_back=False):
    a = ctx.uniform(m * k, -1, 1, 0, SEED)
    b = ctx.uniform(k * n, -1, 1, 1, SEED)
    c = ctx.zeros(m * n)
    fn = lambda: ctx.call("slhip_sgemm", ta, tb, m, n, k, a.ptr, b.ptr, c.ptr, beta)
    flop = 2.0 * m * n * k
    res = {}
    if headline:
        if m == n == k:
            spin_up(ctx, a, b, c, m)
        wall, ev = timed(ctx, fn, steps, warmup)
        res.update({"ms_wall": wall, "ms_kernel": ev, "tflops_wall": flop / wall / 1e9, "tflops_kernel": flop / ev / 1e9,
                    "frac_of_peak": flop / ev / 1e9 / FP32_MATRIX_PEAK_TFLOPS})
    med = median_ms(ctx, fn, steps, warmup)
    res.update({"ms_median": med, "tflops_median": flop / med / 1e9, "frac_median": flop / med / 1e9 / FP32_MATRIX_PEAK_TFLOPS})
    if back_to_back:
        # launches queued one behind the other inside ONE event pair: the launch gap of about 6 us
        # that every per-launch pair contains overlaps with the kernel before it
        _, ev = timed(ctx, fn, steps, warmup)
        res.update({"ms_back_to_back": ev, "tflops_back_to_back": flop / ev / 1e9})
    if sweep is not None:
        cold = median_ms(ctx, fn, steps, warmup, sweep)
        res.update({"ms_median_caches_swept": cold, "tflops_median_caches_swept": flop / cold / 1e9})
    for x in (a, b, c):
        x.free()
    return res


def shader_clock_mhz():
    """Best effort: the current shader clock from sysfs (the level marked '*' in pp_dpm_sclk); None
    where it cannot be read.  Reads files only: no other program is started from this process."""
    import glob
    import re
    best = None
    for path in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"):
        try:
            with open(path) as f:
                for line in f:
                    m = re.search(r"(\d+)\s*Mhz\s*\*", line, re.I)
                    if m:
                        best = max(best or 0, int(m.group(1)))
        except OSError:
            pass
    return best


def bw_entry(ctx, name, algo_bytes, fn, iters, sweep=None):
    ms = pair_times(ctx, fn, iters, MIN_WARMUP, sweep)
    med = statistics.median(ms)
    gbs = algo_bytes / med / 1e6
    e = {"op": name, "algorithmic_bytes": algo_bytes, "ms_median": med, "ms_min": min(ms), "ms_max": max(ms),
         "launches": len(ms), "caches_swept": sweep is not None, "GBps": gbs, "frac": gbs / HBM_PEAK_GBS}
    log(e)
    return e


def bench_bandwidth_suite(ctx, iters):
    out = []
    R = C = 16384
    n = R * C
    x = ctx.uniform(n, -10, 10, 0, SEED)
    vec_c, vec_r, one = ctx.empty(C), ctx.empty(R), ctx.empty(1)
    y = ctx.empty(n)
    add = lambda *a, **k: out.append(bw_entry(ctx, *a, **k))
    # config 4: reductions, mean and transpose on [16384 x 16384]
    for name, outbuf, olen in [("sum_rows", vec_c, C), ("sum_cols", vec_r, R), ("max_rows", vec_c, C),
                               ("max_cols", vec_r, R)]:
        add("%s [16384x16384]" % name, 4 * n + 4 * olen,
            lambda name=name, outbuf=outbuf: ctx.call("slhip_" + name, R, C, x.ptr, outbuf.ptr), iters)
    add("mean [2^28]", 4 * n + 4, lambda: ctx.call("slhip_mean", n, x.ptr, one.ptr), iters)
    add("transpose [16384x16384]", 8 * n, lambda: ctx.call("slhip_transpose", R, C, x.ptr, y.ptr, 0.0), iters)
    # config 4: the degenerate shapes of the same tensor - the reducing direction ...
    N1 = 1 << 28
    for name, rows, cols in [("sum_cols", 1, N1), ("sum_rows", N1, 1), ("max_cols", 1, N1), ("max_rows", N1, 1)]:
        add("%s [%dx%d] -> 1" % (name, rows, cols), 4 * n + 4,
            lambda name=name, rows=rows, cols=cols: ctx.call("slhip_" + name, rows, cols, x.ptr, one.ptr), iters)
    # ... and the copy direction (2^28 outputs), and the transposes of a vector
    for name, rows, cols in [("sum_rows", 1, N1), ("max_rows", 1, N1), ("sum_cols", N1, 1), ("max_cols", N1, 1)]:
        add("%s [%dx%d] -> 2^28" % (name, rows, cols), 8 * n,
            lambda name=name, rows=rows, cols=cols: ctx.call("slhip_" + name, rows, cols, x.ptr, y.ptr), iters)
    for rows, cols in [(1, N1), (N1, 1)]:
        add("transpose [%dx%d]" % (rows, cols), 8 * n,
            lambda rows=rows, cols=cols: ctx.call("slhip_transpose", rows, cols, x.ptr, y.ptr, 0.0), iters)
    # config 3: softmax forward / backward, [32768 x 4096] and the row-length sweep at 2^27 elements
    for rows, cols in [(32768, 4096), (1 << 20, 128), (1 << 17, 1024), (1 << 13, 16384)]:
        ne = rows * cols
        xs, g, s = x.view(0, ne), x.view(ne, ne), y.view(0, ne)
        xg = y.view(ne, ne)
        add("softmax fwd [%dx%d]" % (rows, cols), 8 * ne, lambda: ctx.call("slhip_softmax", rows, cols, xs.ptr, s.ptr), iters)
        add("softmax bwd [%dx%d]" % (rows, cols), 12 * ne,
            lambda: ctx.call("slhip_softmax_grad", rows, cols, xg.ptr, s.ptr, g.ptr, 0.0), iters)
        if cols == 4096:
            add("transpose [%dx%d]" % (rows, cols), 8 * ne,
                lambda: ctx.call("slhip_transpose", rows, cols, xs.ptr, s.ptr, 0.0), iters)
            for name, o1, olen in (("max_rows", vec_c.view(0, cols), cols), ("sum_rows", vec_c.view(0, cols), cols),
                                   ("max_cols", vec_r.view(0, R), rows), ("sum_cols", vec_r.view(0, R), rows)):
                if olen > o1.n:
                    o1 = y.view(ne, olen)
                add("%s [32768x4096]" % name, 4 * ne + 4 * olen,
                    lambda name=name, o1=o1: ctx.call("slhip_" + name, rows, cols, xs.ptr, o1.ptr), iters)
    # shapes off the beaten track, 2^27 elements each: rows of odd length, narrow and very wide matrices
    for rows, cols in [(4026, 33333), (522247, 257), (13421772, 10), (134, 1000000)]:
        ne = rows * cols
        xs = x.view(0, ne)
        ov = y.view(0, max(rows, cols))
        for name, olen in (("sum_rows", cols), ("max_rows", cols), ("sum_cols", rows)):
            add("%s [%dx%d]" % (name, rows, cols), 4 * ne + 4 * olen,
                lambda name=name: ctx.call("slhip_" + name, rows, cols, xs.ptr, ov.ptr), iters)
    # the other row-shaped ops on the narrow shapes (2^27 elements each): softmax and the fused loss on
    # short rows, transposes of narrow matrices, the broadcast-side gradients, the first-tie gradient
    # on few long rows
    ctx.call("slhip_fill", 1, 1.0, one.ptr)
    lrb = ctx.empty(13421772)
    for rows, cols in [(13421772, 10), (8388608, 16)]:
        ne = rows * cols
        xs, g, s, xg = x.view(0, ne), x.view(ne, ne), y.view(0, ne), y.view(ne, ne)
        lr = lrb.view(0, rows)
        add("softmax fwd [%dx%d]" % (rows, cols), 8 * ne, lambda: ctx.call("slhip_softmax", rows, cols, xs.ptr, s.ptr), iters)
        add("softmax bwd [%dx%d]" % (rows, cols), 12 * ne,
            lambda: ctx.call("slhip_softmax_grad", rows, cols, xg.ptr, s.ptr, g.ptr, 0.0), iters)
        add("softmax_cce [%dx%d]" % (rows, cols), 12 * ne + 4 * rows,
            lambda: ctx.call("slhip_softmax_cce", rows, cols, xs.ptr, g.ptr, s.ptr, lr.ptr), iters)
        add("softmax_cce_grad [%dx%d]" % (rows, cols), 12 * ne,
            lambda: ctx.call("slhip_softmax_cce_grad", rows, cols, s.ptr, g.ptr, xg.ptr, 0.0, one.ptr), iters)
    lrb.free()
    for rows, cols in [(13421772, 10), (10, 13421772), (128, 1 << 20), (1342177, 100)]:
        ne = rows * cols
        add("transpose [%dx%d]" % (rows, cols), 8 * ne,
            lambda rows=rows, cols=cols: ctx.call("slhip_transpose", rows, cols, x.ptr, y.ptr, 0.0), iters)
    for rows, cols in [(13421772, 10), (4026, 33333)]:
        ne = rows * cols
        lhs, g, lg = x.view(0, ne), x.view(ne, ne), y.view(0, ne)
        v, vg = y.view(ne, max(rows, cols)), y.view(ne + max(rows, cols), max(rows, cols))
        ctx.call("slhip_fill", max(rows, cols), 1.5, v.ptr)
        add("row_op_grad mul, rhs side [%dx%d]" % (rows, cols), 8 * ne + 12 * cols,
            lambda rows=rows, cols=cols: ctx.call("slhip_row_op_grad", 2, rows, cols, lhs.ptr, v.ptr, None, vg.ptr, g.ptr), iters)
        add("col_op_grad div, rhs side [%dx%d]" % (rows, cols), 8 * ne + 12 * rows,
            lambda rows=rows, cols=cols: ctx.call("slhip_col_op_grad", 3, rows, cols, lhs.ptr, v.ptr, None, vg.ptr, g.ptr), iters)
        add("add_row [%dx%d]" % (rows, cols), 8 * ne + 4 * cols,
            lambda rows=rows, cols=cols: ctx.call("slhip_add_row", rows, cols, lhs.ptr, v.ptr, lg.ptr), iters)
    rows, cols = 134, 1000000
    ne = rows * cols
    ctx.call("slhip_max_cols", rows, cols, x.ptr, vec_r.ptr)
    add("max_cols_grad [%dx%d]" % (rows, cols), 4 * ne + 16 * rows,
        lambda: ctx.call("slhip_max_cols_grad", rows, cols, vec_r.ptr, x.ptr, y.ptr, y.view(ne, rows).ptr), iters)
    # config 4: the elementwise chain on 2^28 elements per tensor: 4 reads + 1 write
    bb, cc, dd = ctx.uniform(n, -10, 10, 2, SEED), ctx.uniform(n, -10, 10, 3, SEED), ctx.uniform(n, -10, 10, 4, SEED)
    add("ew_chain ((a+b)*c-d)^2^2 [2^28], hand-fused kernel", 20 * n,
        lambda: ctx.call("slhip_ew_chain", n, x.ptr, bb.ptr, cc.ptr, dd.ptr, y.ptr), iters)
    for b in (bb, cc, dd):
        b.free()
    # the classifier's last layer (config 5): products with a side of 10, bound by HBM rather than by the
    # matrix cores; bytes = both operands and the result, each moved once.  64 MiB operands: caches swept
    sweep = ctx.empty(1 << 28)
    for m_, n_, k_, ta, tb, what in [(8192, 2048, 10, 0, 1, "A*Bt"), (2048, 10, 8192, 1, 0, "At*B"), (8192, 10, 2048, 0, 0, "A*B")]:
        a_, b_, c_ = x.view(0, m_ * k_), x.view(m_ * k_, k_ * n_), y.view(0, m_ * n_)
        add("gemm %s [%dx%dx%d]" % (what, m_, n_, k_), 4 * (m_ * k_ + k_ * n_ + m_ * n_),
            lambda: ctx.call("slhip_sgemm", ta, tb, m_, n_, k_, a_.ptr, b_.ptr, c_.ptr, 0.0), iters, sweep=sweep)
    # a head of 16 classes on a 1 GiB activation matrix: the tall-A kernel on the 32 x 32 x 2 instruction
    m_, n_, k_ = 16384, 16, 16384
    a_, b_, c_ = x.view(0, m_ * k_), y.view(0, k_ * n_), y.view(k_ * n_, m_ * n_)
    add("gemm A*B [%dx%dx%d]" % (m_, n_, k_), 4 * (m_ * k_ + k_ * n_ + m_ * n_),
        lambda: ctx.call("slhip_sgemm", 0, 0, m_, n_, k_, a_.ptr, b_.ptr, c_.ptr, 0.0), iters)
    # what a launch costs in this way of timing, and what a plain streaming kernel reaches on operands
    # of the head products' size (64 MiB) timed the same way: the lines those three stand against
    add("fill of one element (the launch floor of a per-launch event pair)", 4, lambda: ctx.call("slhip_fill", 1, 1.0, one.ptr), iters)
    n64 = 1 << 23
    add("device copy [64 MiB of traffic] (achievable line at the head products' size)", 8 * n64,
        lambda: ctx.call("slhip_memcpy_d2d", y.ptr, x.ptr, 4 * n64), iters, sweep=sweep)
    add("sum [64 MiB read] (achievable line for a reduction at that size)", 8 * n64,
        lambda: ctx.call("slhip_sum", 2 * n64, x.ptr, one.ptr), iters, sweep=sweep)
    sweep.free()
    add("device copy [1 GiB] (achievable line)", 8 * n, lambda: ctx.call("slhip_memcpy_d2d", y.ptr, x.ptr, 4 * n), iters)
    for b in (x, y, vec_c, vec_r, one):
        b.free()
    return out


def bench_tape_chain(ctx_unused, iters):
    """Config 4's chain written op by op against the host tape (add, mul, sub, pow 2, square), which
    fuses it into one launch where the intermediates have a single reader."""
    try:
        from sliced_amd import host
        return host.bench_chain(1 << 28, iters)
    except Exception as e:  # the host layer is optional for the kernel benchmark
        return {"skipped": "%s" % e}


def bench_mlp(steps_c5, steps_c1, graph=True):
    try:
        from sliced_amd import host
    except Exception as e:  # the host layer is optional for the kernel benchmark
        return {"skipped": "host layer not built: %s" % e}
    return host.bench_mlp(steps_c5, steps_c1, graph=graph)


def cpu_baseline(m, n, k):
    import oracle
    cores = oracle.max_threads()
    oracle.set_threads(cores)
    from sliced_amd import rng
    a = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)        # the very operands the GPU multiplies
    b = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
    oracle.gemm(64, 64, 64, a[:4096], b[:4096])        # load + warm
    t0 = time.perf_counter()
    oracle.gemm(m, n, k, a, b)
    dt = time.perf_counter() - t0
    res = {"value": 2.0 * m * n * k / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
           "sample": "one pass of the same %dx%dx%d product, oracle sgemm (sequential-k f32, no FMA), %.2f s, %d threads"
                     % (m, n, k, dt, cores)}
    oracle.set_threads(1)
    ms = 1024
    t0 = time.perf_counter()
    oracle.gemm(ms, ms, ms, a[:ms * ms], b[:ms * ms])
    dt1 = time.perf_counter() - t0
    res["single_thread_TFLOPs_at_1024"] = 2.0 * ms ** 3 / dt1 / 1e12
    res.update(cblas_row(m, n, k, a, b))
    res["ops"] = cpu_streaming_ops(oracle, cores)
    res["mlp"] = cpu_mlp_steps(oracle, cores)
    for loop, row in res["mlp"].items():
        if isinstance(row, dict):
            for key, v in row.items():
                if key.startswith("steps_per_s"):
                    res["%s %s" % (loop.split(" ")[0], key)] = v
    return res


def cblas_row(m, n, k, a, b):
    """The same product through a CBLAS sgemm - what the reference's CPU device calls
    (src/ops2/gemm/cpu_stack.rs:39 -> custos GenericBlas -> cblas_sgemm): numpy's f32 matmul runs on
    the OpenBLAS that numpy bundles, on as many threads as that library chooses to use."""
    A, B = a.reshape(m, k), b.reshape(k, n)
    np.matmul(A[:256], B)                               # load + warm the library's threads
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        np.matmul(A, B)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    threads, lib = None, "OpenBLAS bundled with numpy %s" % np.__version__
    try:
        from threadpoolctl import threadpool_info
        for info in threadpool_info():
            if info.get("user_api") == "blas":
                threads = info.get("num_threads")
                lib = "%s %s (numpy %s)" % (info.get("internal_api"), info.get("version"), np.__version__)
    except Exception:
        pass
    return {"cblas_TFLOPs": 2.0 * m * n * k / best / 1e12, "cblas_threads": threads,
            "cblas_sample": "best of 3 passes of the same %dx%dx%d f32 product, np.matmul -> cblas_sgemm of %s, %.3f s"
                            % (m, n, k, lib, best)}


def cpu_mlp_steps(oracle, cores):
    """Steps per second of the oracle's training loop (the reference's op sequence on the host) on the
    two MLP configurations: all 200 steps of the sine fit, a bounded sample of the classifier's steps
    (260 GFLOP each), on one thread (the reference's loops are single-threaded) and on every core."""
    try:
        from sliced_amd import host
    except Exception as e:  # configurations and seeded data live beside the host layer's bindings
        return {"skipped": "host layer not built: %s" % e}
    out = {}
    for name, cfg, steps_by_threads in (("C1 sine fit 1-64-64-1 batch 1024", host.C1, {1: 200, cores: 200}),
                                        ("C5 classifier 784-2048-2048-10 batch 8192", host.C5, {1: 2, cores: 6})):
        x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
        row = {}
        for th, steps in steps_by_threads.items():
            params = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
            oracle.set_threads(th)
            t0 = time.perf_counter()
            oracle.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, params, cfg["lr"], steps)
            row["steps_per_s_%d_thread%s" % (th, "" if th == 1 else "s")] = steps / (time.perf_counter() - t0)
            row["sample_steps_%d_thread%s" % (th, "" if th == 1 else "s")] = steps
        out[name] = row
    oracle.set_threads(1)
    return out


def cpu_streaming_ops(oracle, cores):
    """The bandwidth-bound ops on the host: GB/s of the same algorithmic bytes on a bounded sample
    ([8192 x 4096] = 128 MiB per tensor), once on one thread (the reference's loops are
    single-threaded) and once on every core."""
    rows, cols = 8192, 4096
    n = rows * cols
    rs = np.random.RandomState(2)
    x = rs.uniform(-10, 10, n).astype(np.float32)
    g = rs.standard_normal(n).astype(np.float32)
    s = oracle.softmax(rows, cols, x)
    cases = [("sum_rows", 4 * n, lambda: oracle.sum_rows(cols, x)), ("sum_cols", 4 * n, lambda: oracle.sum_cols(cols, x)),
             ("max_rows", 4 * n, lambda: oracle.max_rows(cols, x)), ("max_cols", 4 * n, lambda: oracle.max_cols(cols, x)),
             ("transpose", 8 * n, lambda: oracle.transpose(rows, cols, x)),
             ("softmax fwd", 8 * n, lambda: oracle.softmax(rows, cols, x)),
             ("softmax bwd", 12 * n, lambda: oracle.softmax_grad(rows, cols, s, g)),
             ("square (one elementwise op)", 8 * n, lambda: oracle.unary(oracle.SQUARE, x))]
    out = {"sample": "[%d x %d] f32 per tensor" % (rows, cols)}
    for name, nbytes, fn in cases:
        row = {}
        for label, th in (("GBps_1_thread", 1), ("GBps_%d_threads" % cores, cores)):
            oracle.set_threads(th)
            t0 = time.perf_counter()
            fn()
            row[label] = nbytes / (time.perf_counter() - t0) / 1e9
        out[name] = row
    oracle.set_threads(1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-suite", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-graph", action="store_true",
                    help="leave out the MLP variants that replay a recorded step (for runs under a kernel tracer, "
                         "which has crashed inside hipGraphLaunch; the kernels of a step are the same either way)")
    ap.add_argument("--size", type=int, default=4096)
    ap.add_argument("--detail", default=os.environ.get("SLICED_BENCH_DETAIL", DETAIL_DEFAULT),
                    help="file that receives the full tables as JSON ('' for none); stdout carries one short line")
    ap.add_argument("--only", default="", help="comma list of suite parts to run: gemm,sweep,bandwidth,chain,mlp")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus %d refused); the hot path has no "
              "multi-GPU leg" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from sliced_amd.device import Context
    ctx = Context(0)
    log("device:", ctx.name())
    M = N = K = args.size

    detail = {}
    head = bench_gemm(ctx, M, N, K, 0, 0, args.steps, args.warmup, headline=True)
    log("gemm A*B", head)
    detail["headline"] = head
    roof = {"bound": "mfma", "achieved": head["tflops_kernel"], "peak": FP32_MATRIX_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": head["frac_of_peak"], "traffic": GEMM_4096_TRAFFIC_BYTES if M == 4096 else None,
            "achieved_median": round(head["tflops_median"], 2)}
    detail["notes"] = {
        "traffic_source": "profiles/hbm_traffic_gemm_and_bandwidth_suite.md (rocprofv3 --pmc of this program, not this run)",
        "timing": "achieved: average over the timed launches; *_median and every op: median of per-launch "
                  "HIP-event pairs, >= %d launches after >= %d warm-ups and %g ms of untimed launches of the same op" % (MIN_ITERS, MIN_WARMUP, OP_WARM_MS)}
    # the clock while the matrix cores are busy: queue 0.3 s of launches, sample, then wait
    a, b, c = ctx.uniform(M * K, -1, 1, 0, SEED), ctx.uniform(K * N, -1, 1, 1, SEED), ctx.zeros(M * N)
    for _ in range(min(200, int(300 / max(head["ms_kernel"], 0.01)) + 1)):
        ctx.call("slhip_sgemm", 0, 0, M, N, K, a.ptr, b.ptr, c.ptr, 0.0)
    time.sleep(0.15)
    roof["sclk_mhz"] = shader_clock_mhz()
    ctx.sync()
    kernel_name = ctx.last_gemm_plan()
    for x in (a, b, c):
        x.free()
    log("sclk under load:", roof["sclk_mhz"], " plan:", kernel_name)
    parts = set(args.only.split(",")) if args.only else {"gemm", "sweep", "bandwidth", "chain", "mlp"}
    if args.no_suite:
        parts = set()
    iters = max(MIN_ITERS, args.steps)
    r1 = lambda v: round(v, 1)
    if "gemm" in parts:
        sweep_buf = ctx.empty(1 << 28)
        forms = {}
        for form, (ta, tb) in {"A*B": (0, 0), "A*Bt": (0, 1), "At*B": (1, 0)}.items():
            r = bench_gemm(ctx, M, N, K, ta, tb, iters, MIN_WARMUP, sweep=sweep_buf)
            forms[form] = r
            roof["TFLOPs %s" % form] = r1(r["tflops_median"])
            log(form, r)
        roof["TFLOPs A*B caches swept"] = r1(forms["A*B"]["tflops_median_caches_swept"])
        detail["gemm_forms"] = forms
        sweep_buf.free()
    if "sweep" in parts:
        sweep = {}
        for (m, n, k) in [(512,) * 3, (1024,) * 3, (2048,) * 3, (3584,) * 3, (4095,) * 3, (4608,) * 3, (8192,) * 3,
                          (8192, 2048, 784), (784, 2048, 8192)]:
            for form, (ta, tb) in {"A*B": (0, 0), "A*Bt": (0, 1), "At*B": (1, 0)}.items():
                r = bench_gemm(ctx, m, n, k, ta, tb, iters, MIN_WARMUP, back_to_back=True)
                key = "%dx%dx%d %s" % (m, n, k, form)
                sweep[key] = {"tflops": r["tflops_median"], "frac": r["frac_median"], "ms": r["ms_median"],
                              "tflops_back_to_back": r["tflops_back_to_back"], "ms_back_to_back": r["ms_back_to_back"]}
                log(key, sweep[key])
        detail["gemm_sweep"] = sweep
        # per size: the slowest of the three forms, per launch (median of event pairs)
        for size, label in (("512x512x512", "512^3"), ("1024x1024x1024", "1024^3"), ("2048x2048x2048", "2048^3"),
                            ("8192x8192x8192", "8192^3"), ("8192x2048x784", "8192x2048x784"), ("784x2048x8192", "784x2048x8192")):
            roof["TFLOPs %s min of forms" % label] = r1(min(v["tflops"] for kk, v in sweep.items() if kk.startswith(size + " ")))
    if "bandwidth" in parts:
        ops = bench_bandwidth_suite(ctx, iters)
        detail["ops"] = ops
        by_name = {e["op"]: e["GBps"] for e in ops}
        for short, name in COMPACT_OPS:
            if name in by_name:
                roof["GBps " + short] = int(round(by_name[name]))
        metric_ops = [e for e in ops if e["algorithmic_bytes"] >= (1 << 30) and not e["op"].startswith(("device copy", "gemm"))]
        worst = min(metric_ops, key=lambda e: e["GBps"])
        roof["GBps min over %d ops >= 1 GiB" % len(metric_ops)] = int(round(worst["GBps"]))
        roof["min op"] = worst["op"]
    ctx.close()
    if "chain" in parts:
        ch = bench_tape_chain(None, iters)
        log("tape chain", ch)
        detail["tape_chain"] = ch
        if "GBps_fused_tape" in ch:
            roof["GBps chain on the tape, fused"] = int(round(ch["GBps_fused_tape"]))
    if "mlp" in parts:
        mlp = bench_mlp(50, 200, graph=not args.no_graph)
        log(mlp)
        detail["mlp"] = mlp
        for cfg in ("C1", "C5"):
            rows = {loop: row["steps_per_s"] for loop, row in mlp.items()
                    if loop.startswith(cfg) and isinstance(row, dict) and "steps_per_s" in row}
            if rows:
                best = max(rows, key=rows.get)
                roof["steps/s %s" % cfg] = r1(rows[best])
                roof["steps/s %s variant" % cfg] = best[best.index("(") + 1:-1]

    cpu = None
    if not args.no_cpu:
        full = cpu_baseline(M, N, K)
        log("cpu", full)
        detail["cpu_baseline"] = full
        cpu = {key: full[key] for key in ("value", "unit", "cores", "kind", "sample", "cblas_TFLOPs", "cblas_threads") if key in full}
        for key, v in full.items():
            if key.startswith(("C1 steps_per_s", "C5 steps_per_s")):
                cpu[key] = round(v, 2)
        if isinstance(full.get("ops"), dict):
            for op in ("sum_rows", "max_cols", "transpose", "softmax fwd"):
                row = full["ops"].get(op)
                if isinstance(row, dict):
                    cpu["GBps " + op] = {kk.replace("GBps_", ""): round(v, 1) for kk, v in row.items()}

    line = {
        "metric": "f32 GEMM TFLOP/s @4096^3",
        "value": head["tflops_wall"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_wall"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "C2 standalone sgemm, M=N=K=%d, C = A*B, A and B ~ U(-1,1) seeded, beta=0" % M,
                   "kernel": kernel_name, "spin_up_s": SPIN_UP_SECONDS, "op_warm_ms": OP_WARM_MS},
        "roofline": roof,
        "cpu_baseline": cpu,
    }
    detail["line"] = line
    path = write_detail(args.detail, detail)
    if path:
        log("detail written to", path)
    text = json.dumps(line)
    if len(text) > MAX_LINE_BYTES:
        raise SystemExit("bench.py: the result line is %d bytes, above the %d that a reader of the last line can rely on"
                         % (len(text), MAX_LINE_BYTES))
    print(text, flush=True)


if __name__ == "__main__":
    main()
