#!/usr/bin/env python3
"""Benchmark of the MI355X array-op hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-suite] [--no-cpu]

Headline (the JSON line's `value`): f32 GEMM TFLOP/s at M=N=K=4096, C = A·B, operands seeded
U(-1,1) and resident in HBM before the timed region.  One step = one pass of the kernel.
The same line carries
  roofline     - the GEMM kernel against the fp32 matrix peak, from HIP-event timing of the same
                 launches on the stream they run on;
  cpu_baseline - the CPU oracle's sgemm (a restatement of the reference's CPU path) timed on this
                 host's cores on one pass of the same 4096^3 product;
  suite        - the other workloads of the metric: A·Bᵀ / Aᵀ·B, the reductions, softmax fwd/bwd,
                 transpose, the fused elementwise chain (GB/s of ALGORITHMIC bytes against 8 TB/s)
                 and MLP training steps/s.
Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import os
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
GEMM_4096_TRAFFIC_BYTES = int((646261.4 * 2.0 + 65536.0) * 1024)
HBM_PEAK_GBS = 8000.0             # MI355X HBM3E
SEED = 0x51CED


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def timed(ctx, fn, steps, warmup):
    """(wall ms per step with sync on both sides, HIP-event ms per launch)."""
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


def spin_up(ctx, seconds=0.4):
    """Untimed: keep the matrix cores busy until the clocks have ramped (the first launches after
    an idle period run at about 2.0 instead of 2.4 GHz).  Uses the At*B kernel so that a profile of
    this program attributes only the timed 4096^3 launches to the headline A*B kernel."""
    n = 2048
    a, b, c = ctx.uniform(n * n, -1, 1, 0, SEED), ctx.uniform(n * n, -1, 1, 1, SEED), ctx.zeros(n * n)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            ctx.call("slhip_sgemm", 1, 0, n, n, n, a.ptr, b.ptr, c.ptr, 0.0)
        ctx.sync()
    for x in (a, b, c):
        x.free()


def timed_cold(ctx, fn, steps, scratch):
    """HIP-event ms per launch with the caches (L2 and the 256 MiB memory-side cache) swept between
    launches by a fill of a 1 GiB scratch buffer; the sweep is outside the event pair."""
    e0, e1 = ctx.event(), ctx.event()
    total = 0.0
    for _ in range(steps):
        ctx.call("slhip_fill", scratch.n, 1.0, scratch.ptr)
        ctx.record(e0)
        fn()
        ctx.record(e1)
        total += ctx.elapsed_ms(e0, e1)
    ctx.lib.slhip_event_destroy(e0)
    ctx.lib.slhip_event_destroy(e1)
    return total / steps


def bench_gemm(ctx, m, n, k, ta, tb, steps, warmup, beta=0.0, cold_scratch=None):
    a = ctx.uniform(m * k, -1, 1, 0, SEED)
    b = ctx.uniform(k * n, -1, 1, 1, SEED)
    c = ctx.zeros(m * n)
    fn = lambda: ctx.call("slhip_sgemm", ta, tb, m, n, k, a.ptr, b.ptr, c.ptr, beta)
    wall, ev = timed(ctx, fn, steps, warmup)
    flop = 2.0 * m * n * k
    res = {"ms_wall": wall, "ms_kernel": ev, "tflops_wall": flop / wall / 1e9, "tflops_kernel": flop / ev / 1e9,
           "frac_of_peak": flop / ev / 1e9 / FP32_MATRIX_PEAK_TFLOPS}
    if cold_scratch is not None:
        cold = timed_cold(ctx, fn, max(5, steps // 2), cold_scratch)
        res["ms_kernel_caches_swept"] = cold
        res["tflops_kernel_caches_swept"] = flop / cold / 1e9
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


def bw_entry(name, algo_bytes, wall, ev):
    gbs = algo_bytes / ev / 1e6
    return {"op": name, "algorithmic_bytes": algo_bytes, "ms_wall": wall, "ms_kernel": ev, "GBps": gbs,
            "frac_of_hbm_peak": gbs / HBM_PEAK_GBS}


def bench_bandwidth_suite(ctx, steps, warmup):
    out = []
    R = C = 16384
    n = R * C
    x = ctx.uniform(n, -10, 10, 0, SEED)
    vec_c, vec_r, one = ctx.empty(C), ctx.empty(R), ctx.empty(1)
    y = ctx.empty(n)
    for name, outbuf, olen in [("sum_rows", vec_c, C), ("sum_cols", vec_r, R), ("max_rows", vec_c, C),
                               ("max_cols", vec_r, R)]:
        fn = lambda name=name, outbuf=outbuf: ctx.call("slhip_" + name, R, C, x.ptr, outbuf.ptr)
        w, e = timed(ctx, fn, steps, warmup)
        out.append(bw_entry("%s [16384x16384]" % name, 4 * n + 4 * olen, w, e))
        log(out[-1])
    w, e = timed(ctx, lambda: ctx.call("slhip_mean", n, x.ptr, one.ptr), steps, warmup)
    out.append(bw_entry("mean [2^28]", 4 * n + 4, w, e)); log(out[-1])
    w, e = timed(ctx, lambda: ctx.call("slhip_transpose", R, C, x.ptr, y.ptr, 0.0), steps, warmup)
    out.append(bw_entry("transpose [16384x16384]", 8 * n, w, e)); log(out[-1])
    # degenerate 1-D shapes of the same tensor
    N1 = 1 << 28
    for name, rows, cols, olen in [("sum_cols", 1, N1, 1), ("sum_rows", N1, 1, 1), ("max_cols", 1, N1, 1),
                                   ("max_rows", N1, 1, 1)]:
        fn = lambda name=name, rows=rows, cols=cols: ctx.call("slhip_" + name, rows, cols, x.ptr, one.ptr)
        w, e = timed(ctx, fn, steps, warmup)
        out.append(bw_entry("%s [%dx%d]" % (name, rows, cols), 4 * n + 4 * olen, w, e)); log(out[-1])
    # softmax forward / backward, [32768 x 4096] and the row-length sweep at 2^27 elements
    for rows, cols in [(32768, 4096), (1 << 20, 128), (1 << 17, 1024), (1 << 13, 16384)]:
        ne = rows * cols
        xs, g, s = x.view(0, ne), x.view(ne, ne), y.view(0, ne)
        xg = y.view(ne, ne)
        w, e = timed(ctx, lambda: ctx.call("slhip_softmax", rows, cols, xs.ptr, s.ptr), steps, warmup)
        out.append(bw_entry("softmax fwd [%dx%d]" % (rows, cols), 8 * ne, w, e)); log(out[-1])
        w, e = timed(ctx, lambda: ctx.call("slhip_softmax_grad", rows, cols, xg.ptr, s.ptr, g.ptr, 0.0), steps, warmup)
        out.append(bw_entry("softmax bwd [%dx%d]" % (rows, cols), 12 * ne, w, e)); log(out[-1])
        if cols == 4096:
            o1 = vec_c.view(0, cols)
            w, e = timed(ctx, lambda: ctx.call("slhip_max_rows", rows, cols, xs.ptr, o1.ptr), steps, warmup)
            out.append(bw_entry("max_rows [32768x4096]", 4 * ne + 4 * cols, w, e)); log(out[-1])
            w, e = timed(ctx, lambda: ctx.call("slhip_sum_rows", rows, cols, xs.ptr, o1.ptr), steps, warmup)
            out.append(bw_entry("sum_rows [32768x4096]", 4 * ne + 4 * cols, w, e)); log(out[-1])
    # shapes off the beaten track, 2^27 elements each: rows of odd length, narrow and very wide matrices
    for rows, cols in [(4026, 33333), (522247, 257), (13421772, 10), (134, 1000000)]:
        ne = rows * cols
        xs = x.view(0, ne)
        ov = y.view(0, max(rows, cols))
        for name, olen in (("sum_rows", cols), ("max_rows", cols), ("sum_cols", rows)):
            fn = lambda name=name: ctx.call("slhip_" + name, rows, cols, xs.ptr, ov.ptr)
            w, e = timed(ctx, fn, steps, warmup)
            out.append(bw_entry("%s [%dx%d]" % (name, rows, cols), 4 * ne + 4 * olen, w, e)); log(out[-1])
    # fused elementwise chain on 2^28 elements per tensor: 4 reads + 1 write
    bb, cc, dd = ctx.uniform(n, -10, 10, 2, SEED), ctx.uniform(n, -10, 10, 3, SEED), ctx.uniform(n, -10, 10, 4, SEED)
    w, e = timed(ctx, lambda: ctx.call("slhip_ew_chain", n, x.ptr, bb.ptr, cc.ptr, dd.ptr, y.ptr), steps, warmup)
    out.append(bw_entry("ew_chain ((a+b)*c-d)^2^2 [2^28]", 20 * n, w, e)); log(out[-1])
    # the classifier's last layer (config 5): products with a side of 10, bound by HBM rather than by the
    # matrix cores; bytes = both operands and the result, each moved once
    for m_, n_, k_, ta, tb, what in [(8192, 2048, 10, 0, 1, "A*Bt"), (2048, 10, 8192, 1, 0, "At*B"), (8192, 10, 2048, 0, 0, "A*B")]:
        a_, b_, c_ = x.view(0, m_ * k_), x.view(m_ * k_, k_ * n_), y.view(0, m_ * n_)
        w, e = timed(ctx, lambda: ctx.call("slhip_sgemm", ta, tb, m_, n_, k_, a_.ptr, b_.ptr, c_.ptr, 0.0), steps, warmup)
        out.append(bw_entry("gemm %s [%dx%dx%d]" % (what, m_, n_, k_), 4 * (m_ * k_ + k_ * n_ + m_ * n_), w, e)); log(out[-1])
    w, e = timed(ctx, lambda: ctx.call("slhip_memcpy_d2d", y.ptr, x.ptr, 4 * n), steps, warmup)
    out.append(bw_entry("device copy [1 GiB] (achievable line)", 8 * n, w, e)); log(out[-1])
    for b in (x, y, bb, cc, dd, vec_c, vec_r, one):
        b.free()
    return out


def bench_mlp(ctx, steps_c5, steps_c1):
    try:
        from sliced_amd import host
    except Exception as e:  # the host layer is optional for the kernel benchmark
        return {"skipped": "host layer not built: %s" % e}
    return host.bench_mlp(steps_c5, steps_c1)


def cpu_baseline(m, n, k):
    import oracle
    cores = oracle.max_threads()
    oracle.set_threads(cores)
    rs = np.random.RandomState(1)
    a = rs.uniform(-1, 1, m * k).astype(np.float32)
    b = rs.uniform(-1, 1, k * n).astype(np.float32)
    oracle.gemm(64, 64, 64, a[:4096], b[:4096])        # load + warm
    t0 = time.perf_counter()
    oracle.gemm(m, n, k, a, b)
    dt = time.perf_counter() - t0
    res = {"value": 2.0 * m * n * k / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
           "sample": "one pass of the same %dx%dx%d f32 product by the CPU oracle's blocked sgemm "
                     "(sequential-k f32, no FMA), %.2f s on %d threads" % (m, n, k, dt, cores)}
    oracle.set_threads(1)
    ms = 1024
    t0 = time.perf_counter()
    oracle.gemm(ms, ms, ms, a[:ms * ms], b[:ms * ms])
    dt1 = time.perf_counter() - t0
    res["single_thread_TFLOPs_at_1024"] = 2.0 * ms ** 3 / dt1 / 1e12
    res["ops"] = cpu_streaming_ops(oracle, cores)
    res["mlp"] = cpu_mlp_steps(oracle, cores)
    return res


def cpu_mlp_steps(oracle, cores):
    """Steps per second of the oracle's training loop (the reference's op sequence on the host) on the
    two MLP configurations: all 200 steps of the sine fit, a bounded sample of 2 steps of the
    classifier (260 GFLOP each), on one thread (the reference is single-threaded) and on every core."""
    try:
        from sliced_amd import host
    except Exception as e:  # configurations and seeded data live beside the host layer's bindings
        return {"skipped": "host layer not built: %s" % e}
    out = {}
    for name, cfg, steps_by_threads in (("C1 sine fit 1-64-64-1 batch 1024", host.C1, {1: 200, cores: 200}),
                                        ("C5 classifier 784-2048-2048-10 batch 8192", host.C5, {1: 1, cores: 2})):
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
    ap.add_argument("--size", type=int, default=4096)
    ap.add_argument("--only", default="", help="comma list of suite parts to run: gemm,sweep,bandwidth,mlp")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus %d refused); the hot path has no "
              "multi-GPU leg" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from sliced_amd.device import Context
    ctx = Context(0)
    log("device:", ctx.name())
    M = N = K = args.size

    spin_up(ctx)
    head = bench_gemm(ctx, M, N, K, 0, 0, args.steps, args.warmup)
    log("gemm NN", head)
    suite = {}
    # the clock while the matrix cores are busy: queue 0.3 s of launches, sample, then wait
    a, b, c = ctx.uniform(M * K, -1, 1, 0, SEED), ctx.uniform(K * N, -1, 1, 1, SEED), ctx.zeros(M * N)
    for _ in range(min(200, int(300 / max(head["ms_kernel"], 0.01)) + 1)):
        ctx.call("slhip_sgemm", 0, 0, M, N, K, a.ptr, b.ptr, c.ptr, 0.0)
    time.sleep(0.15)
    suite["shader_clock_mhz_under_gemm_load"] = shader_clock_mhz()
    ctx.sync()
    for x in (a, b, c):
        x.free()
    log("sclk under load:", suite["shader_clock_mhz_under_gemm_load"])
    parts = set(args.only.split(",")) if args.only else {"gemm", "sweep", "bandwidth", "mlp"}
    if args.no_suite:
        parts = set()
    if "gemm" in parts:
        scratch = ctx.empty(1 << 28)
        suite["gemm_4096"] = {"A*B": bench_gemm(ctx, M, N, K, 0, 0, args.steps, args.warmup, cold_scratch=scratch),
                              "A*Bt": bench_gemm(ctx, M, N, K, 0, 1, args.steps, args.warmup, cold_scratch=scratch),
                              "At*B": bench_gemm(ctx, M, N, K, 1, 0, args.steps, args.warmup, cold_scratch=scratch)}
        scratch.free()
        log(suite["gemm_4096"])
    if "sweep" in parts:
        sweep = {}
        for (m, n, k) in [(512,) * 3, (1024,) * 3, (2048,) * 3, (3584,) * 3, (4095,) * 3, (4608,) * 3, (8192,) * 3,
                          (8192, 2048, 784), (784, 2048, 8192)]:
            st = max(3, args.steps // 4) if m >= 8192 and k >= 8192 else args.steps
            for form, (ta, tb) in {"A*B": (0, 0), "A*Bt": (0, 1), "At*B": (1, 0)}.items():
                r = bench_gemm(ctx, m, n, k, ta, tb, st, 2)
                sweep["%dx%dx%d %s" % (m, n, k, form)] = {"tflops": r["tflops_kernel"], "frac": r["frac_of_peak"]}
                log(m, n, k, form, sweep["%dx%dx%d %s" % (m, n, k, form)])
        suite["gemm_sweep"] = sweep
    if "bandwidth" in parts:
        suite["bandwidth"] = bench_bandwidth_suite(ctx, max(5, args.steps // 2), 2)
    if "mlp" in parts:
        suite["mlp"] = bench_mlp(ctx, 50, 200)
        log(suite["mlp"])

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(M, N, K)
        log("cpu", cpu)

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
                   "kernel": "gemm_kernel<false,false,32,true,2,2>: 128x128 tiles, BK=32, v_mfma_f32_32x32x2_f32"},
        "roofline": {"bound": "mfma", "achieved": head["tflops_kernel"], "peak": FP32_MATRIX_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": head["frac_of_peak"],
                     "traffic": GEMM_4096_TRAFFIC_BYTES if M == 4096 else None},
        "cpu_baseline": cpu,
        "suite": suite,
    }
    print(json.dumps(line))
    ctx.close()


if __name__ == "__main__":
    main()
