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



# --------------------------------------------------------------------------- large random shapes
# Up to 2^27 elements per operand, where the host's choice between kernels changes with the size (the
# shifted-piece and chunk transposes, the tall and skinny GEMM kernels, long-row softmax, the two-stage
# reductions).  The operands come from the device generator and are checked against its values
# recomputed on the host (devgen.py) on windows, sampled rows and columns, and through the transpose of
# the transpose; views start 0..33 floats into their allocations.
BIG_CAP = (1 << 27) + 4096
SUB_OP, SCALE_OP = 1, 6   # SLHIP_SUB, SLHIP_SCALE


@pytest.fixture(scope="module")
def pool():
    from sliced_amd.device import Context
    ctx = Context(0)
    x = ctx.uniform(BIG_CAP + 64, -1, 1, 0, SEED)
    y, z = ctx.empty(BIG_CAP + 64), ctx.empty(BIG_CAP + 64)
    small = ctx.zeros(1 << 22)
    yield ctx, x, y, z, small
    for b in (x, y, z, small):
        b.free()
    ctx.close()


def near(r, base, spread=2):
    return max(1, int(base + r.integers(-spread, spread + 1)))


def pick_side(r, hi):
    k = r.integers(0, 7)
    if k == 0:
        return int(r.integers(1, 65))
    if k == 1:
        return near(r, int(r.choice([16, 32, 56, 57, 64, 128, 200, 201, 256, 512, 1024, 2048, 4096, 8192, 16384])))
    if k == 2:
        return near(r, 64 * int(r.integers(1, 400)))
    if k == 3:
        return near(r, 256 * int(r.integers(1, 200)), 17)
    if k == 4:
        return int(r.integers(1, 4000))
    if k == 5:
        return int(2 ** r.uniform(6, np.log2(hi)))
    return near(r, 1024 * int(r.integers(1, 64)), 1)


def test_random_large_transposes(pool):
    from devgen import host_values
    ctx, x, y, z, small = pool
    r = np.random.default_rng(4242)
    done = 0
    while done < 60:
        rows, cols = pick_side(r, 1 << 22), pick_side(r, 1 << 22)
        if r.integers(0, 3) == 0:
            cols = max(1, min(cols, BIG_CAP // max(rows, 1)))
            rows = max(1, min(int(2 ** r.uniform(20, 27)) // cols, 1 << 24))
        n = rows * cols
        if n > BIG_CAP:
            continue
        done += 1
        ox, oy = int(r.choice([0, 0, 1, 4, 5, 16, 17, 32])), int(r.choice([0, 0, 1, 3, 16, 17, 33]))
        xs, ys, zs = x.view(ox, n), y.view(oy, n), z.view(ox, n)
        say("large transpose", rows, cols, ox, oy)

        def want(start, m):
            o = np.arange(start, start + m, dtype=np.uint64)
            c, rr = o // np.uint64(rows), o % np.uint64(rows)
            return host_values(rr * np.uint64(cols) + c + np.uint64(ox), 0)

        ctx.call("slhip_transpose", rows, cols, xs.ptr, ys.ptr, 0.0)
        w = min(n, 4096)
        for start in (0, max(0, n // 2 - 1000), n - w):
            m = min(w, n - start)
            assert np.array_equal(ys.view(start, m).numpy(), want(start, m)), (rows, cols, ox, oy, start)
        ctx.call("slhip_transpose", cols, rows, ys.ptr, zs.ptr, 0.0)          # and back: every element
        ctx.call("slhip_ew_binary", SUB_OP, n, zs.ptr, xs.ptr, zs.ptr)
        ctx.call("slhip_max", n, zs.ptr, small.view(0, 1).ptr)
        ctx.call("slhip_ew_unary", SCALE_OP, -1.0, 0.0, n, zs.ptr, zs.ptr)
        ctx.call("slhip_max", n, zs.ptr, small.view(1, 1).ptr)
        assert np.all(small.view(0, 2).numpy() == 0.0), (rows, cols, ox, oy)
        ctx.call("slhip_transpose", rows, cols, xs.ptr, ys.ptr, 1.0)           # `Assign`: y = 2 x^T now
        for start in (0, n - w):
            assert np.array_equal(ys.view(start, w).numpy(), want(start, w) + want(start, w)), (rows, cols, ox, oy, start)


def test_random_large_products(pool):
    from devgen import host_values, host_range
    ctx, x, y, z, small = pool
    r = np.random.default_rng(777)
    ctx.call("slhip_rand_uniform", SEED, 1, -1.0, 1.0, 1 << 26, z.ptr)   # B comes from tag 1
    done = 0
    while done < 60:
        kind = r.integers(0, 4)
        if kind == 0:      # a tall A and a narrow B
            nn, k = int(r.integers(1, 40)), near(r, 4 * int(r.integers(16, 5000)), int(r.integers(0, 2)))
            m = max(1, min(int(2 ** r.uniform(18, 26)) // k, 1 << 21))
        elif kind == 1:    # few outputs, long k
            m, nn, k = int(r.integers(1, 300)), int(r.integers(1, 300)), int(2 ** r.uniform(8, 19))
        elif kind == 2:    # sides up to 5000 near the tile and vector boundaries
            m, nn, k = (min(pick_side(r, 4096), 5000) for _ in range(3))
        else:              # short k
            k, m, nn = int(r.integers(1, 20)), int(2 ** r.uniform(8, 20)), int(r.integers(1, 600))
        ta, tb = [(0, 0), (0, 1), (1, 0), (1, 1)][int(r.integers(0, 4))]
        if m * k > BIG_CAP or k * nn > (1 << 26) or m * nn > BIG_CAP:
            continue
        done += 1
        beta = float(r.integers(0, 2))
        say("large gemm", m, nn, k, ta, tb, beta)
        ctx.call("slhip_fill", m * nn, 0.25, y.ptr)
        ctx.call("slhip_sgemm", ta, tb, m, nn, k, x.ptr, z.ptr, y.ptr, beta)
        b = host_range(0, k * nn, 1)
        B = (b.reshape(nn, k).T if tb else b.reshape(k, nn)).astype(np.float64)
        for i in sorted(set([0, m - 1, m // 2] + [int(v) for v in r.integers(0, m, 5)])):
            if ta:
                a_row = host_values(np.arange(k, dtype=np.uint64) * np.uint64(m) + np.uint64(i), 0).astype(np.float64)
            else:
                a_row = host_range(i * k, k, 0).astype(np.float64)
            exact, scale = a_row @ B + beta * 0.25, np.abs(a_row) @ np.abs(B) + 0.25
            got = y.view(i * nn, nn).numpy()
            assert np.all(np.abs(got - exact) <= 3e-6 * scale + 1e-30), (m, nn, k, ta, tb, beta, i, ctx.last_gemm_plan())


def test_random_large_reductions_and_softmax(pool):
    from devgen import host_values, host_range
    ctx, x, y, z, small = pool
    r = np.random.default_rng(31337)
    done = 0
    while done < 50:
        rows, cols = pick_side(r, 1 << 22), pick_side(r, 1 << 22)
        if r.integers(0, 2) == 0:
            cols = max(1, min(cols, 1 << 20))
            rows = max(1, min(int(2 ** r.uniform(18, 27)) // cols, 1 << 24))
        n = rows * cols
        if n > BIG_CAP:
            continue
        done += 1
        ox = int(r.choice([0, 0, 1, 3, 4, 16]))
        xs = x.view(ox, n)
        say("large reductions / softmax", rows, cols, ox)
        pick_r = sorted(set([0, rows - 1, rows // 2] + [int(v) for v in r.integers(0, rows, 3)]))
        if rows <= (1 << 21):
            vr = small.view(0, rows)
            ctx.call("slhip_sum_cols", rows, cols, xs.ptr, vr.ptr)
            s = vr.numpy()
            ctx.call("slhip_max_cols", rows, cols, xs.ptr, vr.ptr)
            mx = vr.numpy()
            for i in pick_r:
                h = host_range(ox + i * cols, cols, 0)
                assert mx[i] == h.max(), (rows, cols, ox, i)
                assert abs(float(s[i]) - h.sum(dtype=np.float64)) <= 1e-6 * np.abs(h).sum(dtype=np.float64) + 1e-30, (rows, cols, ox, i)
        if cols <= (1 << 21):
            vc = small.view(1 << 21, cols)
            ctx.call("slhip_sum_rows", rows, cols, xs.ptr, vc.ptr)
            s = vc.numpy()
            ctx.call("slhip_max_rows", rows, cols, xs.ptr, vc.ptr)
            mx = vc.numpy()
            for c in sorted(set([0, cols - 1, cols // 2] + [int(v) for v in r.integers(0, cols, 3)])):
                h = host_values(np.arange(rows, dtype=np.uint64) * np.uint64(cols) + np.uint64(c + ox), 0)
                assert mx[c] == h.max(), (rows, cols, ox, c)
                assert abs(float(s[c]) - h.sum(dtype=np.float64)) <= 1e-6 * np.abs(h).sum(dtype=np.float64) + 1e-30, (rows, cols, ox, c)
        if cols >= 2:
            ys = y.view(int(r.choice([0, 1, 4])), n)
            ctx.call("slhip_softmax", rows, cols, xs.ptr, ys.ptr)
            ctx.call("slhip_softmax_grad", rows, cols, z.view(0, n).ptr, ys.ptr, x.view(ox + 1, n).ptr, 0.0)
            for i in pick_r:
                h = host_range(ox + i * cols, cols, 0).astype(np.float64)
                e = np.exp(h - h.max())
                ref = e / e.sum()
                got = ys.view(i * cols, cols).numpy()
                assert np.all(np.abs(got - ref) <= 2e-6 * ref + 1e-37), (rows, cols, ox, i)
                g, sg = host_range(ox + 1 + i * cols, cols, 0).astype(np.float64), got.astype(np.float64)
                bound = 2e-6 * (np.abs(sg) * (np.abs(g) + np.dot(np.abs(sg), np.abs(g)))) + 1e-37
                assert np.all(np.abs(z.view(i * cols, cols).numpy() - sg * (g - np.dot(sg, g))) <= bound), (rows, cols, ox, i)
