"""Pins the CPU oracle through what the mathematics fixes, for everything the reference's own
vectors leave open: closed forms, invariants, library routines (numpy in f64) and brute force on
small inputs.  Each check is chosen so that a plausible slip (a dropped term, a swapped operand,
a wrong index or sign) fails it."""
import numpy as np
import pytest

from sliced_amd import rng


def test_gemm_three_forms_against_f64_matmul(orc):
    for (m, n, k) in [(1, 1, 1), (3, 5, 7), (17, 9, 33), (64, 40, 129), (130, 257, 300)]:
        a = rng.uniform(m * k, -1, 1, tag=0, seed=m)
        b = rng.uniform(k * n, -1, 1, tag=1, seed=m)
        A, B = a.reshape(m, k).astype(np.float64), b.reshape(k, n).astype(np.float64)
        exact = A @ B
        tol = 1e-5 * np.sqrt(k) * (np.abs(A) @ np.abs(B)) + 1e-30
        # operands stored non-square and non-symmetric: a transposed-operand mix-up cannot pass
        assert np.all(np.abs(orc.gemm(m, n, k, a, b).reshape(m, n) - exact) <= tol)
        bt = np.ascontiguousarray(b.reshape(k, n).T).ravel()       # stored n x k
        assert np.all(np.abs(orc.gemmT(m, n, k, a, bt).reshape(m, n) - exact) <= tol)
        at = np.ascontiguousarray(a.reshape(m, k).T).ravel()       # stored k x m
        assert np.all(np.abs(orc.Tgemm(m, n, k, at, b).reshape(m, n) - exact) <= tol)
        assert np.allclose(orc.gemm_f64(0, 0, m, n, k, a, b).reshape(m, n), exact, rtol=1e-13, atol=1e-13)
        assert np.allclose(orc.gemm_f64(1, 0, m, n, k, at, b).reshape(m, n), exact, rtol=1e-13, atol=1e-13)
        assert np.allclose(orc.gemm_f64(0, 1, m, n, k, a, bt).reshape(m, n), exact, rtol=1e-13, atol=1e-13)
        # beta = 1 accumulates
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=m)
        acc = orc.gemm(m, n, k, a, b, c=c0.copy(), beta=1.0)
        assert np.all(np.abs(acc.reshape(m, n) - (exact + c0.reshape(m, n))) <= tol + 1e-6)


def test_gemm_is_sequential_in_k(orc):
    # the restated BLAS sums k in ascending order with f32 rounding after every product and add
    m, n, k = 3, 4, 50
    a = rng.uniform(m * k, -1, 1, tag=0)
    b = rng.uniform(k * n, -1, 1, tag=1)
    ref = np.zeros((m, n), np.float32)
    A, B = a.reshape(m, k), b.reshape(k, n)
    for kk in range(k):
        ref = (ref + (A[:, kk:kk + 1] * B[kk:kk + 1, :]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(orc.gemm(m, n, k, a, b).reshape(m, n), ref)


def test_gemm_grad_is_the_transposed_products(orc):
    m, k, n = 9, 5, 7
    lhs = rng.uniform(m * k, -1, 1, tag=0)
    rhs = rng.uniform(k * n, -1, 1, tag=1)
    g = rng.normal(m * n, 1.0, tag=2)
    lg, rg = np.zeros(m * k, np.float32), np.zeros(k * n, np.float32)
    orc.gemm_grad(m, k, n, lhs, rhs, lg, rg, g)
    G, L, R = g.reshape(m, n).astype(np.float64), lhs.reshape(m, k).astype(np.float64), rhs.reshape(k, n).astype(np.float64)
    assert np.allclose(lg.reshape(m, k), G @ R.T, rtol=1e-5, atol=1e-6)
    assert np.allclose(rg.reshape(k, n), L.T @ G, rtol=1e-5, atol=1e-6)
    # finite differences of <G, L R> with respect to one entry of each operand
    f = lambda L_, R_: np.sum(G * (L_ @ R_))
    eps = 1e-6
    Lp = L.copy(); Lp[2, 3] += eps
    assert abs((f(Lp, R) - f(L, R)) / eps - lg.reshape(m, k)[2, 3]) < 1e-4
    Rp = R.copy(); Rp[4, 1] += eps
    assert abs((f(L, Rp) - f(L, R)) / eps - rg.reshape(k, n)[4, 1]) < 1e-4
    # None = operand without requires_grad: skipped, the other side unchanged
    rg2 = np.zeros(k * n, np.float32)
    orc.gemm_grad(m, k, n, lhs, rhs, None, rg2, g)
    assert np.array_equal(rg, rg2)


def test_reductions_against_numpy_and_each_other(orc):
    rows, cols = 37, 53
    x = rng.uniform(rows * cols, -10, 10, tag=0)
    X = x.reshape(rows, cols)
    assert np.array_equal(orc.max_rows(cols, x), X.max(0))
    assert np.array_equal(orc.max_cols(cols, x), X.max(1))
    assert np.allclose(orc.sum_rows(cols, x), X.astype(np.float64).sum(0), rtol=0, atol=1e-3)
    assert np.allclose(orc.sum_cols(cols, x), X.astype(np.float64).sum(1), rtol=0, atol=1e-3)
    # reducing over rows is reducing over the columns of the transpose
    xt = orc.transpose(rows, cols, x)
    assert np.array_equal(orc.max_rows(cols, x), orc.max_cols(rows, xt))
    assert np.array_equal(orc.transpose(cols, rows, xt), x)
    # sequential left-to-right f32 order
    acc = np.float32(0)
    for v in X[5]:
        acc = np.float32(acc + v)
    assert orc.sum_cols(cols, x)[5] == acc
    acc = np.float32(0)
    for v in X[:, 7]:
        acc = np.float32(acc + v)
    assert orc.sum_rows(cols, x)[7] == acc
    assert orc.mean(np.full(1000, 0.375, np.float32)) == np.float32(0.375)
    assert np.array_equal(orc.mean_cols(cols, x), (orc.sum_cols(cols, x) / np.float32(cols)).astype(np.float32))
    assert np.array_equal(orc.mean_rows(cols, x), (orc.sum_rows(cols, x) / np.float32(rows)).astype(np.float32))


def test_max_grad_tie_rules_by_brute_force(orc):
    rows, cols = 6, 9
    x = rng.integers(rows * cols, 4, tag=0).astype(np.float32)      # many ties
    X = x.reshape(rows, cols)
    g_r = rng.normal(rows, 1.0, tag=1)
    g_c = rng.normal(cols, 1.0, tag=2)
    base = rng.normal(rows * cols, 1.0, tag=3)
    want = base.reshape(rows, cols).copy()
    for r in range(rows):                                            # first maximal column only
        want[r, int(np.argmax(X[r]))] += g_r[r]
    got = orc.max_cols_grad(cols, orc.max_cols(cols, x), x, base.copy(), g_r)
    assert np.array_equal(got.reshape(rows, cols), want)
    want = base.reshape(rows, cols).copy()
    for c in range(cols):                                            # every maximal row
        for r in range(rows):
            if X[r, c] == X[:, c].max():
                want[r, c] += g_c[c]
    got = orc.max_rows_grad(cols, orc.max_rows(cols, x), x, base.copy(), g_c)
    assert np.array_equal(got.reshape(rows, cols), want)


def test_softmax_closed_forms(orc):
    rows, cols = 11, 23
    x = rng.normal(rows * cols, 3.0, tag=0)
    g = rng.normal(rows * cols, 1.0, tag=1)
    s = orc.softmax(rows, cols, x)
    S = s.reshape(rows, cols).astype(np.float64)
    assert np.allclose(S.sum(1), 1.0, atol=1e-6)
    X = x.reshape(rows, cols).astype(np.float64)
    E = np.exp(X - X.max(1, keepdims=True))
    assert np.allclose(S, E / E.sum(1, keepdims=True), rtol=2e-6, atol=1e-12)
    # shifting a row by a constant does not change its softmax
    s2 = orc.softmax(rows, cols, (x.reshape(rows, cols) + np.float32(4.0)).ravel())
    assert np.allclose(s2, s, rtol=1e-5, atol=1e-9)
    # Jacobian form (the reference's literal algorithm) == closed form == J·g in f64
    jac = orc.softmax_grad_jacobian(rows, cols, s, g)
    closed = orc.softmax_grad(rows, cols, s, g)
    G = g.reshape(rows, cols).astype(np.float64)
    exact = np.stack([(np.diag(S[r]) - np.outer(S[r], S[r])) @ G[r] for r in range(rows)]).ravel()
    assert np.allclose(jac, exact, rtol=0, atol=2e-6)
    assert np.allclose(closed, exact, rtol=0, atol=2e-6)
    # finite difference of <g, softmax(x)> in one coordinate
    f = lambda Xm: np.sum(G * (np.exp(Xm - Xm.max(1, keepdims=True)) / np.exp(Xm - Xm.max(1, keepdims=True)).sum(1, keepdims=True)))
    Xp = X.copy(); Xp[3, 5] += 1e-6
    S64 = np.exp(X - X.max(1, keepdims=True)); S64 /= S64.sum(1, keepdims=True)
    exact64 = (S64 * (G - (S64 * G).sum(1, keepdims=True)))
    assert abs((f(Xp) - f(X)) / 1e-6 - exact64[3, 5]) < 1e-4
    assert abs(closed.reshape(rows, cols)[3, 5] - exact64[3, 5]) < 1e-5
    # accumulate form
    base = rng.normal(rows * cols, 1.0, tag=2)
    acc = orc.softmax_grad(rows, cols, s, g, x_grad=base.copy(), beta=1.0)
    assert np.allclose(acc, base + closed, rtol=0, atol=1e-6)
    assert np.max(np.abs(orc.softmax_grad(rows, cols, s, np.ones(rows * cols, np.float32)))) < 1e-6


def test_unary_and_binary_grads_by_finite_differences(orc):
    x = np.array([-2.5, -0.5, 0.75, 1.5, 3.0], np.float32)
    one = np.ones_like(x)
    for op, p, f in [(orc.SQUARE, 0.0, lambda v: v * v), (orc.POW, 3.0, lambda v: v ** 3), (orc.EXP, 0.0, np.exp),
                     (orc.SCALE, 0.37, lambda v: 0.37 * v), (orc.TANH, 0.0, np.tanh),
                     (orc.SIGMOID, 0.0, lambda v: 1.0 / (1.0 + np.exp(-v)))]:
        g = orc.unary_grad(op, x, np.zeros_like(x), one, p)
        x64 = x.astype(np.float64)
        fd = (f(x64 + 1e-6) - f(x64 - 1e-6)) / 2e-6
        assert np.allclose(g, fd, rtol=1e-4, atol=1e-5), op
        assert np.allclose(orc.unary(op, x, p), f(x64), rtol=1e-6)
    assert np.array_equal(orc.unary_grad(orc.RELU, np.array([-1, 0, 2], np.float32), np.zeros(3, np.float32),
                                         np.ones(3, np.float32)), [0, 1, 1])       # gradient at 0 is 1 (x >= 0)
    l, r = np.array([1.5, -2.0, 4.0], np.float32), np.array([0.5, 3.0, -1.25], np.float32)
    g = np.array([1.0, -2.0, 0.5], np.float32)
    for op, dl, dr in [(orc.ADD, g, g), (orc.SUB, g, -g), (orc.MUL, r * g, l * g), (orc.DIV, g / r, -l / (r * r) * g)]:
        lg, rg = orc.binary_ew_grad(op, l, r, np.zeros(3, np.float32), np.zeros(3, np.float32), g)
        assert np.allclose(lg, dl, rtol=1e-6) and np.allclose(rg, dr, rtol=1e-6), op
    # gradients accumulate
    lg, _ = orc.binary_ew_grad(orc.ADD, l, r, np.full(3, 10, np.float32), np.zeros(3, np.float32), g)
    assert np.array_equal(lg, 10 + g)


def test_row_op_and_loss_helpers(orc):
    rows, cols = 7, 5
    lhs = rng.uniform(rows * cols, -1, 1, tag=0)
    rhs = rng.uniform(cols, -1, 1, tag=1)
    assert np.array_equal(orc.add_row(rows, cols, lhs, rhs), (lhs.reshape(rows, cols) + rhs).ravel())
    g = rng.normal(rows * cols, 1.0, tag=2)
    lg, rg = orc.add_row_grad(rows, cols, np.full(rows * cols, 9, np.float32), np.full(cols, 1, np.float32), g)
    assert np.array_equal(lg, g)                                     # overwritten, not accumulated
    assert np.allclose(rg, 1 + g.reshape(rows, cols).sum(0), atol=1e-5)
    # cce of a one-hot target is -ln p[target]; its gradient is -(1/p)/rows at the target only
    cls = rng.integers(rows, cols, tag=3)
    t = orc.onehot(cols, cls.astype(np.float32))
    p = orc.softmax(rows, cols, rng.normal(rows * cols, 2.0, tag=4))
    P = p.reshape(rows, cols)
    assert np.allclose(orc.cce(rows, cols, p, t), -np.log(P[np.arange(rows), cls]), rtol=1e-6)
    gr = orc.cce_grad(rows, cols, p, t).reshape(rows, cols)
    want = np.zeros((rows, cols))
    want[np.arange(rows), cls] = -(1.0 / P[np.arange(rows), cls]) / rows
    assert np.allclose(gr, want, rtol=1e-6)
    pp = rng.uniform(20, -1, 1, tag=5)
    gg = rng.normal(20, 1.0, tag=6)
    assert np.array_equal(orc.sgd_step(pp.copy(), gg, 0.05), (pp - (gg * np.float32(0.05)).astype(np.float32)))


@pytest.mark.parametrize("by_row_index", [False, True], ids=["row_op", "col_op"])
def test_broadcast_op_grads_against_f64_and_finite_differences(orc, by_row_index):
    """row_op / col_op with a named op: forward against numpy broadcasting; gradients against the
    f64 chain rule and, for the broadcast side, a finite difference of sum(out * g)."""
    rows, cols = 6, 4
    lhs = rng.uniform(rows * cols, 0.5, 2.0, tag=0)
    v = rng.uniform(rows if by_row_index else cols, 0.5, 2.0, tag=1)
    g = rng.normal(rows * cols, 1.0, tag=2)
    L, G = lhs.reshape(rows, cols).astype(np.float64), g.reshape(rows, cols).astype(np.float64)
    bc = (lambda vec: vec.astype(np.float64)[:, None]) if by_row_index else (lambda vec: vec.astype(np.float64)[None, :])
    axis = 1 if by_row_index else 0
    fwd = orc.col_op if by_row_index else orc.row_op
    bwd = orc.col_op_grad if by_row_index else orc.row_op_grad
    fs = {orc.ADD: lambda a, b: a + b, orc.SUB: lambda a, b: a - b, orc.MUL: lambda a, b: a * b,
          orc.DIV: lambda a, b: a / b}
    for op, f in fs.items():
        assert np.allclose(fwd(op, cols, lhs, v).reshape(rows, cols), f(L, bc(v)), rtol=1e-6), op
        lg0, vg0 = rng.uniform(rows * cols, -1, 1, tag=3), rng.uniform(v.size, -1, 1, tag=4)
        lg, vg = bwd(op, cols, lhs, v, lg0.copy(), vg0.copy(), g)
        eps = 1e-6
        d_l = (f(L + eps, bc(v)) - f(L - eps, bc(v))) / (2 * eps)
        assert np.allclose(lg.reshape(rows, cols), lg0.reshape(rows, cols) + d_l * G, rtol=1e-4, atol=1e-5), op
        fd = np.zeros(v.size)
        for j in range(v.size):
            vp, vm = v.astype(np.float64).copy(), v.astype(np.float64).copy()
            vp[j] += eps; vm[j] -= eps
            fd[j] = (np.sum(f(L, bc(vp)) * G) - np.sum(f(L, bc(vm)) * G)) / (2 * eps)
        assert np.allclose(vg, vg0 + fd, rtol=1e-4, atol=1e-4), op
        # a NULL side is skipped
        lg2, _ = bwd(op, cols, lhs, v, lg0.copy(), None, g)
        assert np.array_equal(lg2, lg)
    if not by_row_index:   # the multiply-only restatement of the reference's own test agrees
        a = orc.mul_row_grad(cols, lhs, v, np.zeros(rows * cols, np.float32), np.zeros(cols, np.float32), g)
        b = orc.row_op_grad(orc.MUL, cols, lhs, v, np.zeros(rows * cols, np.float32), np.zeros(cols, np.float32), g)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_diagflat_and_onehot_gradients_pick_the_stored_entries(orc):
    n = 5
    x = rng.uniform(n, -1, 1, tag=0)
    d = orc.diagflat(x).reshape(n, n)
    assert np.array_equal(np.diag(d), x) and np.count_nonzero(d - np.diag(np.diag(d))) == 0
    og = rng.normal(n * n, 1.0, tag=1)
    assert np.array_equal(orc.diagflat_grad(np.ones(n, np.float32), og), 1 + np.diag(og.reshape(n, n)))
    cls = rng.integers(7, 4, tag=2).astype(np.float32)
    og = rng.normal(7 * 4, 1.0, tag=3)
    got = orc.onehot_grad(4, cls, np.zeros(7, np.float32), og)
    assert np.array_equal(got, og.reshape(7, 4)[np.arange(7), cls.astype(int)])


def _mlp_numpy_f64(kind, batch, d_in, d_h, d_out, x, t, params, lr, steps):
    """Independent f64 statement of the two training loops (explicit chain rule, no tape)."""
    W1, b1, W2, b2, W3, b3 = [p.astype(np.float64).copy() for p in params]
    W1, W2, W3 = W1.reshape(d_in, d_h), W2.reshape(d_h, d_h), W3.reshape(d_h, d_out)
    X, T = x.reshape(batch, d_in).astype(np.float64), t.reshape(batch, d_out).astype(np.float64)
    losses = []
    for _ in range(steps):
        h1 = X @ W1 + b1; a1 = np.maximum(h1, 0)
        h2 = a1 @ W2 + b2; a2 = np.maximum(h2, 0)
        o = a2 @ W3 + b3
        if kind == 0:
            d = o - T
            losses.append(np.sum(d * d) / d.size)
            go = 2 * d / d.size
        else:
            e = np.exp(o - o.max(1, keepdims=True)); p = e / e.sum(1, keepdims=True)
            losses.append(np.mean(-np.log(np.sum(np.clip(p, 1e-7, 1 - 1e-7) * T, 1))))
            gp = -(T / p) / batch
            go = p * (gp - np.sum(p * gp, 1, keepdims=True))
        gW3, gb3 = a2.T @ go, go.sum(0)
        gh2 = (go @ W3.T) * (h2 >= 0)
        gW2, gb2 = a1.T @ gh2, gh2.sum(0)
        gh1 = (gh2 @ W2.T) * (h1 >= 0)
        gW1, gb1 = X.T @ gh1, gh1.sum(0)
        for P, G in ((W1, gW1), (b1, gb1), (W2, gW2), (b2, gb2), (W3, gW3), (b3, gb3)):
            P -= lr * G
    return np.array(losses), [W1, b1, W2, b2, W3, b3]


@pytest.mark.parametrize("kind,dims,lr", [(0, (64, 1, 16, 1), 0.01), (1, (48, 12, 20, 5), 0.05)])
def test_oracle_training_loop_against_independent_f64_loop(orc, kind, dims, lr):
    from sliced_amd import host
    batch, d_in, d_h, d_out = dims
    x, t = host.mlp_data(kind, batch, d_in, d_out)
    params = host.mlp_init(kind, d_in, d_h, d_out)
    steps = 30
    want, want_p = _mlp_numpy_f64(kind, batch, d_in, d_h, d_out, x, t, params, lr, steps)
    p = [a.copy() for a in params]
    got = orc.mlp_train(kind, batch, d_in, d_h, d_out, x, t, p, lr, steps)
    assert want[-1] < want[0]
    assert np.max(np.abs(got - want) / np.abs(want)) < 2e-5
    for a, b in zip(p, want_p):
        assert np.allclose(a.ravel(), b.ravel(), rtol=0, atol=2e-5)


def test_host_rng_is_reproducible_and_in_range():
    a = rng.uniform(1000, -3, 5, tag=1)
    assert np.array_equal(a, rng.uniform(1000, -3, 5, tag=1))
    assert not np.array_equal(a, rng.uniform(1000, -3, 5, tag=2))
    assert a.min() >= -3 and a.max() < 5 and abs(a.mean() - 1.0) < 0.3
    n = rng.normal(200000, 3.0, tag=0)
    assert abs(n.mean()) < 0.05 and abs(n.std() - 3.0) < 0.05
    k = rng.integers(10000, 10, tag=1)
    assert k.min() == 0 and k.max() == 9
    x = rng.inject_row_max_ties(rng.uniform(40 * 300, -10, 10, tag=0), 40, 300, 0.01).reshape(40, 300)
    assert np.all((x == x.max(1, keepdims=True)).sum(1) >= 3)


def test_special_values_follow_ieee_and_the_documented_maximum(orc):
    """What the oracle does with NaN, infinities and signed zeros, pinned by what fixes it outside
    the oracle: `f32::max` is documented to return the other argument when one is NaN (so a maximum
    skips NaNs and is NaN only over nothing but NaN: numpy's fmax has the same rule); a sum is a
    chain of IEEE additions from +0 (NaN and inf - inf poison it, 0 + -0 is +0); softmax's shift by
    the row maximum turns a row holding +inf, or nothing but -inf, into NaN."""
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    x = np.array([[nan, 1, -inf, nan], [2, nan, -inf, nan], [-3, inf, -inf, nan]], np.float32)
    rows, cols = x.shape
    assert np.array_equal(orc.max_rows(cols, x.ravel()), np.fmax.reduce(x, axis=0), equal_nan=True)
    assert np.array_equal(orc.max_cols(cols, x.ravel()), np.fmax.reduce(x, axis=1), equal_nan=True)
    assert np.array_equal(orc.max_rows(cols, x.ravel()), np.array([2, inf, -inf, nan], np.float32), equal_nan=True)
    assert np.array_equal(orc.max_cols(cols, x.ravel()), np.array([1, 2, inf], np.float32), equal_nan=True)
    with np.errstate(invalid="ignore"):
        assert np.array_equal(orc.sum_rows(cols, x.ravel()), x.sum(axis=0), equal_nan=True)
        assert np.array_equal(orc.sum_cols(cols, x.ravel()), x.sum(axis=1), equal_nan=True)
    y = np.array([[1, inf, -inf], [-inf, -inf, -inf], [inf, -inf, 0], [0, 1, -inf]], np.float32)
    assert np.array_equal(orc.sum_cols(3, y.ravel()), np.array([nan, -inf, nan, -inf], np.float32), equal_nan=True)
    z = np.array([-0.0, -0.0, -0.0, -0.0], np.float32)
    for got in (orc.sum_rows(2, z), orc.sum_cols(2, z), orc.sum_rows(4, z), orc.sum_cols(1, z)):
        assert not np.signbit(got).any() and np.all(got == 0)
    s = orc.softmax(4, 3, y.ravel()).reshape(4, 3)
    assert np.isnan(s[0]).all() and np.isnan(s[1]).all() and np.isnan(s[2]).all()
    e = np.exp(np.float64(-1))
    assert np.allclose(s[3], [e / (1 + e), 1 / (1 + e), 0.0], rtol=1e-6, atol=0)
    # powf's corners, which a square root does not share
    got = orc.unary(orc.POW, np.array([-inf, -0.0, 0.0, inf, 4.0, -4.0], np.float32), 0.5)
    assert np.array_equal(got, np.array([inf, 0.0, 0.0, inf, 2.0, nan], np.float32), equal_nan=True)
    assert not np.signbit(got[1])
