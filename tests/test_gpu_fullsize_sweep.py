"""Parity at the remaining configured sizes: the GEMM sweep (1024^3, 2048^3, 8192^3 and the two
skinny backward shapes, each as A*B, A*B^T and A^T*B, the backward forms also accumulating into C),
the degenerate [1 x 2^28] / [2^28 x 1] shapes of transpose and the reductions, the reductions on
the softmax tensor [32768 x 4096], and max_rows with its all-ties gradient on [16384 x 16384] with
1 % of every column's maximum duplicated.

Every case compares the GPU result DIRECTLY with the CPU oracle's (the restatement of the
reference's loops) on the same seeded operands and records the worst deviation; the GEMMs are also
checked on sampled rows against an f64 product.  Operands come from the device generator, which is
bit-identical to the host generator (tests/test_gpu_parity.py)."""
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu
SEED = rng.DEFAULT_SEED


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


GEMM_SHAPES = [(1024, 1024, 1024), (2048, 2048, 2048), (8192, 8192, 8192), (8192, 2048, 784), (784, 2048, 8192)]


@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("form", ["A*B", "A*Bt", "At*B"])
def test_gemm_sweep_against_oracle(hip, orc, deviations, form, shape):
    """(M, N, K) of the sweep: |gpu - oracle| <= 1e-5 * sqrt(K) * (|A| |B|) for every element, the same
    against f64 on sampled rows, and for the two backward forms the accumulating variant
    (beta = 1, the OpenCL device's `+=`, src/ops2/gemm/grad/opencl.rs:20,33)."""
    m, n, k = shape
    c = hip.ctx()
    ta, tb = form == "At*B", form == "A*Bt"
    name = "gemm %s %dx%dx%d" % (form, m, n, k)
    say(name)
    da, db = c.uniform(m * k, -1, 1, 0, SEED), c.uniform(k * n, -1, 1, 1, SEED)
    dc = c.empty(m * n)
    a, b = da.numpy(), db.numpy()
    c.call("slhip_sgemm", int(ta), int(tb), m, n, k, da.ptr, db.ptr, dc.ptr, 0.0)
    got = dc.numpy()
    ref = (orc.Tgemm if ta else orc.gemmT if tb else orc.gemm)(m, n, k, a, b)
    A = a.reshape(k, m).T if ta else a.reshape(m, k)
    B = b.reshape(n, k).T if tb else b.reshape(k, n)
    scale = (np.abs(A) @ np.abs(B)).ravel().astype(np.float64)      # f32 BLAS is plenty for a scale
    # The contract's bar is 1e-5 * sqrt(K) (3e-4 .. 9e-4 here).  What is asserted is fifty to a
    # hundred times tighter: f32 accumulation on both sides leaves a few 1e-7 of |A||B|, while one
    # product dropped from one dot product is worth about 4/K of it (5e-4 .. 5e-3) - a lost k tail
    # or a missing chunk of a split cannot hide under this ceiling.
    tol = min(1e-5 * np.sqrt(k), 3e-6)
    deviations(name, "max |gpu-oracle| / (|A||B|), bar 1e-5*sqrt(K), asserted 3e-6", np.max(np.abs(got.astype(np.float64) - ref) / scale), tol)
    rows = np.unique(np.concatenate([rng.integers(48, m, tag=5, seed=SEED), [0, m - 1]]))
    exact = A[rows].astype(np.float64) @ B.astype(np.float64)
    srow = np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64)
    deviations(name, "max |gpu-f64| / (|A||B|), sampled rows", np.max(np.abs(got.reshape(m, n)[rows] - exact) / srow), tol)
    if ta or tb:
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        dc.upload(c0)
        c.call("slhip_sgemm", int(ta), int(tb), m, n, k, da.ptr, db.ptr, dc.ptr, 1.0)
        acc = dc.numpy().astype(np.float64)
        want = c0.astype(np.float64) + ref
        deviations(name + " beta=1", "max |gpu-(C0+oracle)| / (|A||B|+|C0|)",
                   np.max(np.abs(acc - want) / (scale + np.abs(c0))), tol)
    for z in (da, db, dc):
        z.free()


def test_degenerate_2_28_shapes_copy_and_reduce(hip, orc, deviations):
    """[1 x 2^28] and [2^28 x 1]: transpose is the same sequence of values; a reduction along the
    axis of length one returns its input (2^28 outputs); along the other axis it is the
    whole-buffer reduction.  One row (or column) with 1 % duplicates of its maximum."""
    c = hip.ctx()
    n = 1 << 28
    say("degenerate shapes on 2^28 elements")
    d = c.uniform(n, -10, 10, 0, SEED)
    x = d.numpy()
    x = rng.inject_row_max_ties(x, 1, n, 0.01)
    d.upload(x)
    out = c.empty(n)
    for rows, cols in ((1, n), (n, 1)):
        say("transpose", rows, cols)
        c.call("slhip_fill", n, 0.0, out.ptr)
        c.call("slhip_transpose", rows, cols, d.ptr, out.ptr, 0.0)
        assert np.array_equal(out.numpy(), x)
    # the copy direction: out has 2^28 entries, each the sum / max of one value
    for fn, rows, cols in (("slhip_sum_rows", 1, n), ("slhip_max_rows", 1, n), ("slhip_sum_cols", n, 1),
                           ("slhip_max_cols", n, 1)):
        say(fn, rows, cols, "-> 2^28 outputs")
        c.call("slhip_fill", n, 0.0, out.ptr)
        c.call(fn, rows, cols, d.ptr, out.ptr)
        assert np.array_equal(out.numpy(), x)
    # the same on a slice the oracle's loops finish quickly, against the oracle itself
    ns = 1 << 22
    xs = x[:ns]
    assert np.array_equal(orc.sum_rows(ns, xs), xs) and np.array_equal(orc.max_rows(ns, xs), xs)
    assert np.array_equal(orc.sum_cols(1, xs), xs) and np.array_equal(orc.max_cols(1, xs), xs)
    # the reducing direction: one output
    one = c.empty(1)
    m = float(x.max())
    absum = float(np.abs(x).sum(dtype=np.float64))
    tot = float(x.sum(dtype=np.float64))
    for fn, rows, cols in (("slhip_max_cols", 1, n), ("slhip_max_rows", n, 1)):
        c.call(fn, rows, cols, d.ptr, one.ptr)
        assert float(one.numpy()[0]) == m
    ref = float(orc.sum_cols(n, x)[0])        # the reference's sequential f32 sum of 2^28 values
    for fn, rows, cols in (("slhip_sum_cols", 1, n), ("slhip_sum_rows", n, 1)):
        c.call(fn, rows, cols, d.ptr, one.ptr)
        got = float(one.numpy()[0])
        deviations("%s [%dx%d]" % (fn[6:], rows, cols), "|gpu-f64| / sum|x|", abs(got - tot) / absum, 1e-6)
        # a sequential f32 sum of 2^28 terms, which is what the reference computes, is itself several
        # 1e-6 of sum|x| away from the exact sum: the direct deviation is the reference's rounding
        deviations("%s [%dx%d]" % (fn[6:], rows, cols), "|gpu-oracle| / sum|x|", abs(got - ref) / absum, 2e-5)
        deviations("%s [%dx%d]" % (fn[6:], rows, cols), "|oracle-f64| / sum|x| (the reference's own)", abs(ref - tot) / absum, 2e-5)
    for z in (d, out, one):
        z.free()


def test_reductions_on_the_softmax_tensor(hip, orc, deviations):
    """max_rows / sum_rows (and the per-row forms) on [32768 x 4096] ~ N(0, 9)."""
    rows, cols = 32768, 4096
    c = hip.ctx()
    say("reductions on [32768 x 4096]")
    x = rng.normal(rows * cols, 3.0, tag=0, seed=SEED)
    d = c.array(x)
    oc, orow = c.empty(cols), c.empty(rows)
    c.call("slhip_max_rows", rows, cols, d.ptr, oc.ptr)
    assert np.array_equal(oc.numpy(), orc.max_rows(cols, x))
    c.call("slhip_max_cols", rows, cols, d.ptr, orow.ptr)
    assert np.array_equal(orow.numpy(), orc.max_cols(cols, x))
    X = x.reshape(rows, cols)
    for fn, axis, out in (("slhip_sum_rows", 0, oc), ("slhip_sum_cols", 1, orow)):
        c.call(fn, rows, cols, d.ptr, out.ptr)
        got = out.numpy().astype(np.float64)
        ref = (orc.sum_rows if axis == 0 else orc.sum_cols)(cols, x)
        absum = np.abs(X).sum(axis, dtype=np.float64)
        exact = X.sum(axis, dtype=np.float64)
        deviations("%s [32768x4096]" % fn[6:], "max |gpu-oracle| / sum|x|", np.max(np.abs(got - ref) / absum), 1e-6)
        deviations("%s [32768x4096]" % fn[6:], "max |gpu-f64| / sum|x|", np.max(np.abs(got - exact) / absum), 1e-6)
    for z in (d, oc, orow):
        z.free()


def test_max_rows_and_its_gradient_with_column_ties_16384_squared(hip, orc):
    """1 % of every COLUMN's maximum duplicated down the column: max_rows is bit-exact and its
    gradient reaches every tied row (slice_max_rows_grad, src/ops2/max/grad/cpu.rs:40-55)."""
    R = C = 16384
    c = hip.ctx()
    say("max_rows / max_rows_grad 16384^2 with 1 % column ties")
    d = c.uniform(R * C, -10, 10, 0, SEED)
    x = rng.inject_col_max_ties(d.numpy(), R, C, 0.01)
    d.upload(x)
    out = c.empty(C)
    c.call("slhip_max_rows", R, C, d.ptr, out.ptr)
    mx = out.numpy()
    assert np.array_equal(mx, orc.max_rows(C, x))
    ties = (x.reshape(R, C) == mx[None, :]).sum(0)
    assert ties.min() >= 2 and ties.mean() >= 100          # the injection took: about 163 per column
    g = rng.normal(C, 1.0, tag=1, seed=SEED)
    dg, dxg = c.array(g), c.zeros(R * C)
    c.call("slhip_max_rows_grad", R, C, out.ptr, d.ptr, dxg.ptr, dg.ptr)
    got = dxg.numpy()
    want = orc.max_rows_grad(C, mx, x, np.zeros(R * C, np.float32), g)
    assert np.array_equal(got, want)
    assert np.count_nonzero(got) == int(ties[g != 0].sum())
    for z in (d, out, dg, dxg):
        z.free()
