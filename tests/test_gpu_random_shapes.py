"""Seeded sweep over random shapes: every kernel family against the oracle at sizes chosen to hit
the boundaries between code paths (vector tails, edge tiles, the wave-per-tile / tiled GEMM switch,
split-K, few-rows / few-columns transposes, register-resident / streaming softmax)."""
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu
SEED = rng.DEFAULT_SEED


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def pick_dim(r, hi):
    """A dimension biased towards path boundaries: small, near multiples of 4 / 32 / 128, or uniform."""
    kind = r.integers(0, 5)
    if kind == 0:
        return int(r.integers(1, 9))
    if kind == 1:
        return int(min(hi, max(1, 128 * r.integers(1, max(2, hi // 128 + 1)) + r.integers(-2, 3))))
    if kind == 2:
        return int(min(hi, max(1, 32 * r.integers(1, max(2, hi // 32 + 1)) + r.integers(-1, 2))))
    if kind == 3:
        return int(min(hi, 4 * r.integers(1, max(2, hi // 4 + 1))))
    return int(r.integers(1, hi + 1))


def test_random_gemm_shapes(hip, orc):
    r = np.random.default_rng(20240607)
    for case in range(70):
        m, n, k = pick_dim(r, 700), pick_dim(r, 700), pick_dim(r, 2100)
        ta, tb = [(0, 0), (0, 1), (1, 0)][case % 3]
        beta = float(r.integers(0, 2))
        say("gemm", case, m, n, k, ta, tb, beta)
        a = rng.uniform(m * k, -1, 1, tag=0, seed=SEED + case)
        b = rng.uniform(k * n, -1, 1, tag=1, seed=SEED + case)
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED + case)
        A = a.reshape(k, m).T if ta else a.reshape(m, k)
        B = b.reshape(n, k).T if tb else b.reshape(k, n)
        exact = (A.astype(np.float64) @ B.astype(np.float64)).ravel() + beta * c0
        bound = (1e-5 * np.sqrt(k) * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))).ravel() + 1e-6 * np.abs(c0) + 1e-30
        got = hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=beta)
        assert np.all(np.abs(got - exact) <= bound), (m, n, k, ta, tb, beta, float(np.max(np.abs(got - exact) / bound)))


def test_random_linear_fwd_shapes(hip, orc):
    r = np.random.default_rng(7)
    for case in range(20):
        m, k, n = pick_dim(r, 600), pick_dim(r, 900), pick_dim(r, 400)
        say("linear", case, m, k, n)
        x = rng.uniform(m * k, -1, 1, tag=0, seed=SEED + case)
        w = rng.uniform(k * n, -1, 1, tag=1, seed=SEED + case)
        bias = rng.uniform(n, -1, 1, tag=2, seed=SEED + case)
        h = hip.gemm(m, n, k, x, w)
        pre_ref = orc.add_row(m, n, h, bias)
        out, pre = hip.linear_fwd(m, k, n, x, w, bias, relu=True, want_pre_act=True)
        assert np.array_equal(pre, pre_ref) and np.array_equal(out, orc.unary(orc.RELU, pre_ref)), (m, k, n)


def test_random_matrix_op_shapes(hip, orc):
    r = np.random.default_rng(99)
    for case in range(60):
        rows, cols = pick_dim(r, 3000), pick_dim(r, 3000)
        if case % 10 == 0:
            rows, cols = pick_dim(r, 40), int(r.integers(16000, 70000))        # long rows: streaming softmax
        n = rows * cols
        say("matrix ops", case, rows, cols)
        x = rng.uniform(n, -4, 4, tag=0, seed=SEED + case)
        g = rng.normal(n, 1.0, tag=1, seed=SEED + case)
        X = x.reshape(rows, cols)
        # bit-exact families
        assert np.array_equal(hip.transpose(rows, cols, x), X.T.ravel())
        assert np.array_equal(hip.max_rows(cols, x), orc.max_rows(cols, x))
        assert np.array_equal(hip.max_cols(cols, x), orc.max_cols(cols, x))
        v = rng.uniform(cols, -1, 1, tag=2, seed=SEED + case)
        assert np.array_equal(hip.add_row(rows, cols, x, v), orc.add_row(rows, cols, x, v))
        gr = rng.normal(rows, 1.0, tag=3, seed=SEED + case)
        assert np.array_equal(hip.sum_cols_grad(cols, g.copy(), gr), orc.sum_cols_grad(cols, g.copy(), gr))
        assert np.array_equal(hip.sum_rows_grad(cols, g.copy(), v), orc.sum_rows_grad(cols, g.copy(), v))
        # sums
        for name, axis in (("sum_cols", 1), ("sum_rows", 0)):
            got = getattr(hip, name)(cols, x)
            exact = X.sum(axis, dtype=np.float64)
            assert np.all(np.abs(got - exact) <= 1e-6 * np.abs(X).astype(np.float64).sum(axis) + 1e-30), name
        # softmax forward / backward
        s = hip.softmax(rows, cols, x)
        sh = (X - X.max(1, keepdims=True)).astype(np.float32).astype(np.float64)
        P = np.exp(sh) / np.exp(sh).sum(1, keepdims=True)
        assert np.all(np.abs(s.reshape(rows, cols) - P) <= 1e-6 * P + 1e-37), (rows, cols)
        got = hip.softmax_grad(rows, cols, s, g)
        S, G = s.reshape(rows, cols).astype(np.float64), g.reshape(rows, cols).astype(np.float64)
        exact_b = S * (G - (S * G).sum(1, keepdims=True))
        bound = 1e-6 * (np.abs(S) * (np.abs(G) + (np.abs(S) * np.abs(G)).sum(1, keepdims=True))) + 1e-37
        assert np.all(np.abs(got.reshape(rows, cols) - exact_b) <= bound), (rows, cols)
        # the losses that ride the softmax kernels, and the cross-entropy as a row reduction
        t = np.zeros((rows, cols), np.float32)
        t[np.arange(rows), np.asarray(r.integers(0, cols, rows))] = 1.0
        p2, loss = hip.softmax_cce(rows, cols, x, t.ravel())
        assert np.all(np.abs(p2.reshape(rows, cols) - P) <= 1e-6 * P + 1e-37), (rows, cols)
        L = -np.log(np.sum(np.clip(P, 1e-7, 1 - 1e-7) * t, 1))
        assert np.all(np.abs(loss - L) <= 2e-6 * np.maximum(np.abs(L), 1.0)), (rows, cols)
        assert np.all(np.abs(hip.cce(rows, cols, s, t.ravel()) - L) <= 2e-6 * np.maximum(np.abs(L), 1.0)), (rows, cols)
        lg = hip.softmax_cce_grad(rows, cols, s, t.ravel(), np.zeros(n, np.float32), 0.0, 1.0)
        exact_l = (s.astype(np.float64) - t.ravel()) / rows
        assert np.all(np.abs(lg - exact_l) <= 2e-6 * (np.abs(s) + t.ravel()) / rows + 1e-37), (rows, cols)
        # broadcast-side gradients of the op-code broadcast ops (reduction kernels reading two matrices)
        lhs = rng.uniform(n, 0.5, 2.0, tag=4, seed=SEED + case)
        for kind, vlen, axis in (("row_op", cols, 0), ("col_op", rows, 1)):
            vv = rng.uniform(vlen, 0.5, 2.0, tag=5, seed=SEED + case)
            for op in (orc.MUL, orc.DIV):
                _, vg = getattr(hip, kind + "_grad")(op, cols, lhs, vv, None, np.zeros(vlen, np.float32), g)
                Lh, Gd = lhs.reshape(rows, cols).astype(np.float64), g.reshape(rows, cols).astype(np.float64)
                V = vv.astype(np.float64)[None, :] if kind == "row_op" else vv.astype(np.float64)[:, None]
                terms = (Lh if op == orc.MUL else -Lh / (V * V)) * Gd
                assert np.all(np.abs(vg - terms.sum(axis)) <= 2e-6 * np.abs(terms).sum(axis) + 1e-30), (kind, op, rows, cols)
        # first-tie gradient of the row maximum, bit-exact
        xt = rng.inject_row_max_ties(x.copy(), rows, cols, 0.05)
        mx = orc.max_cols(cols, xt)
        base = rng.normal(n, 1.0, tag=6, seed=SEED + case)
        assert np.array_equal(hip.max_cols_grad(cols, mx, xt, base.copy(), gr), orc.max_cols_grad(cols, mx, xt, base.copy(), gr))

