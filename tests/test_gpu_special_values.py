"""NaN, infinities, signed zeros and subnormals through the HIP path, against the oracle.

The reference folds `T::max` (src/ops2/max/cpu.rs:11-13, 37-54, 76-80) and plain `+=`
(src/ops2/sum/cpu.rs:86-90) over its slices, so what a NaN, an infinity or a subnormal does to a
result is fixed by IEEE arithmetic and by fmaxf: a NaN is skipped by a maximum unless nothing
else is there, poisons a sum, and an inf - inf inside softmax's shift turns the row into NaN.
The bars:
  * transpose and the maxima: the same values as the oracle's, NaN where it has NaN (the sign of
    a zero maximum is left open by fmaxf and is not compared);
  * sums, means, softmax: NaN and +-inf at exactly the oracle's positions, finite results within
    the bars of the ordinary parity tests;
  * subnormal operands and results are not flushed: elementwise ops bit for bit, sums and
    products within their bars measured on the subnormal scale.
"""
import sys
import warnings

import numpy as np
import pytest

from sliced_amd import numpy_api as dev

pytestmark = pytest.mark.gpu

SHAPES = [(7, 5), (64, 64), (300, 129), (33, 4096), (5000, 10), (1, 1000), (1000, 1), (2, 100003), (100001, 1),
          (1, 100001), (3, 1), (1, 3), (1, 1)]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def same_values(got, want):
    return np.array_equal(np.ravel(got), np.ravel(want), equal_nan=True)


def same_specials(got, want):
    got = np.asarray(got); want = np.asarray(want)
    special = ~np.isfinite(want)
    return np.array_equal(~np.isfinite(got), special) and same_values(got[special], want[special])


def sprinkled(rs, rows, cols):
    x = rs.uniform(-1, 1, rows * cols).astype(np.float32)
    idx = rs.choice(rows * cols, min(rows * cols, max(3, rows * cols // 50)), replace=False)
    k = len(idx) // 3
    x[idx[:k]] = np.nan
    x[idx[k:2 * k]] = np.inf
    x[idx[2 * k:]] = -np.inf
    x[0] = np.nan            # the reference's running maximum starts at the first element
    return x


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_nan_and_inf_land_where_the_reference_puts_them(hip, orc, shape):
    rows, cols = shape
    rs = np.random.RandomState(rows * 31 + cols)
    x = sprinkled(rs, rows, cols)
    say("sprinkled", shape)
    assert same_values(dev.max_rows(cols, x), orc.max_rows(cols, x))
    assert same_values(dev.max_cols(cols, x), orc.max_cols(cols, x))
    assert same_values(dev.max_all(x), orc.max_rows(1, x))
    got = dev.transpose(rows, cols, x)
    assert np.array_equal(got.view(np.uint32), orc.transpose(rows, cols, x).view(np.uint32))
    scale = np.abs(np.where(np.isfinite(x), x, 0)).astype(np.float64).reshape(rows, cols)
    for name, axis, div in [("sum_rows", 0, 1), ("sum_cols", 1, 1), ("mean_rows", 0, rows), ("mean_cols", 1, cols)]:
        got = getattr(dev, name)(cols, x)
        want = getattr(orc, name)(cols, x)
        assert same_specials(got, want), name
        fin = np.isfinite(want)
        # 1e-6 of sum|x| against the f64 sum, the bar of the ordinary parity tests; the oracle's
        # own sequential f32 sum is allowed its distance from the f64 sum on top
        exact = np.where(np.isfinite(x), x, 0).astype(np.float64).reshape(rows, cols).sum(axis=axis) / div
        bound = 1e-6 * scale.sum(axis=axis) / div + 1e-30
        assert np.all(np.abs(got[fin] - exact[fin]) <= bound[fin]), name
    got = dev.softmax(rows, cols, x)
    want = orc.softmax(rows, cols, x)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    with np.errstate(invalid="ignore", over="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)       # nanmax of a row of nothing but NaN
        x64 = x.astype(np.float64).reshape(rows, cols)
        e = np.exp(x64 - np.nanmax(x64, axis=1, keepdims=True))
        exact = (e / e.sum(axis=1, keepdims=True)).ravel()
    fin = ~np.isnan(want)
    assert not np.isnan(exact[fin]).any()
    assert np.all(np.abs(got[fin].astype(np.float64) - exact[fin]) <= 1e-6 * exact[fin] + 1e-37)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_a_maximum_over_nothing_but_nan_is_nan(hip, orc, shape):
    rows, cols = shape
    rs = np.random.RandomState(rows * 17 + cols)
    y = rs.uniform(-1, 1, rows * cols).astype(np.float32).reshape(rows, cols)
    y[rows // 2, :] = np.nan            # one whole row
    y[:, cols // 3] = np.nan            # one whole column
    if rows > 1:
        y[0, :] = -np.inf               # a row of -inf with one NaN in it: its maximum is -inf
        y[0, cols // 3] = np.nan
    y = y.ravel()
    say("all-NaN row and column", shape)
    got_r, want_r = dev.max_rows(cols, y), orc.max_rows(cols, y)
    got_c, want_c = dev.max_cols(cols, y), orc.max_cols(cols, y)
    assert np.isnan(want_r[cols // 3]) and np.isnan(want_c[rows // 2])
    assert same_values(got_r, want_r)
    assert same_values(got_c, want_c)
    z = np.full(rows * cols, np.nan, np.float32)
    assert np.isnan(dev.max_all(z)).all() and np.isnan(orc.max_rows(1, z)).all()
    assert np.isnan(dev.max_rows(cols, z)).all() and np.isnan(dev.max_cols(cols, z)).all()
    # softmax of a row of -inf, and of a row of NaN, is NaN throughout; the other rows are untouched
    got, want = dev.softmax(rows, cols, y), orc.softmax(rows, cols, y)
    assert np.array_equal(np.isnan(got), np.isnan(want))


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_signed_zeros(hip, orc, shape):
    rows, cols = shape
    rs = np.random.RandomState(rows + 3 * cols)
    z = np.where(rs.rand(rows * cols) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
    say("signed zeros", shape)
    assert same_values(dev.max_rows(cols, z), orc.max_rows(cols, z))
    assert same_values(dev.max_cols(cols, z), orc.max_cols(cols, z))
    got = dev.transpose(rows, cols, z)
    assert np.array_equal(got.view(np.uint32), orc.transpose(rows, cols, z).view(np.uint32))
    # a sum that starts at +0 never becomes -0 by adding zeros; the reference's starts there too
    neg = -np.abs(z)
    for name in ("sum_rows", "sum_cols"):
        got, want = getattr(dev, name)(cols, neg), getattr(orc, name)(cols, neg)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_subnormals_are_not_flushed(hip, orc, shape):
    rows, cols = shape
    rs = np.random.RandomState(rows * 5 + cols)
    d = rs.randint(1, 1 << 20, rows * cols).astype(np.uint32).view(np.float32).copy()
    assert np.all(d > 0) and np.all(d < np.finfo(np.float32).tiny)
    say("subnormals", shape)
    for name in ("max_rows", "max_cols"):
        got, want = getattr(dev, name)(cols, d), getattr(orc, name)(cols, d)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
    got = dev.transpose(rows, cols, d)
    assert np.array_equal(got.view(np.uint32), orc.transpose(rows, cols, d).view(np.uint32))
    exact = d.astype(np.float64).reshape(rows, cols)
    for name, axis in (("sum_rows", 0), ("sum_cols", 1)):
        got = getattr(dev, name)(cols, d).astype(np.float64)
        s = exact.sum(axis=axis)
        # sums of subnormals are exact until they pass 2^-126 * 2^24 / 2^23: every addend is a
        # multiple of the smallest subnormal, so only the bar of the ordinary tests is asked
        assert np.all(got > 0) and np.all(np.abs(got - s) <= 1e-6 * s), name
    e = d[::-1].copy()
    for op in (dev.ADD, dev.SUB, dev.MUL, dev.DIV):
        got, want = dev.binary_ew(op, d, e), orc.binary_ew(op, d, e)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), op
    big = rs.uniform(1e8, 1e9, rows * cols).astype(np.float32)
    got, want = dev.binary_ew(dev.MUL, d, big), orc.binary_ew(dev.MUL, d, big)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) and np.all(got > 0)
    a = np.full(rows * cols, 1e-20, np.float32); b = np.full(rows * cols, 3e-20, np.float32)
    got, want = dev.binary_ew(dev.MUL, a, b), orc.binary_ew(dev.MUL, a, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) and np.all(got > 0)
    # softmax of subnormal inputs: every shift is below half an ulp of 1, the row is uniform
    got, want = dev.softmax(rows, cols, d), orc.softmax(rows, cols, d)
    assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-6 * want)


GEMM_SHAPES = [(64, 64, 64), (128, 128, 128), (256, 256, 256), (33, 17, 100), (8, 2048, 512), (2048, 8, 512),
               (1, 512, 512), (512, 1, 512), (300, 10, 2048), (512, 512, 64), (1024, 1024, 96)]


@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("form", ["gemm", "gemmT", "Tgemm"])
def test_products_keep_subnormal_operands_and_results(hip, orc, form, shape):
    m, n, k = shape
    rs = np.random.RandomState(m + 7 * n + 13 * k)
    # subnormal A times B around 1e6: every product is a normal number a flush of A would lose
    a = rs.randint(1 << 10, 1 << 22, m * k).astype(np.uint32).view(np.float32).copy()
    b = rs.uniform(1e6, 1e7, k * n).astype(np.float32)
    say(form, shape, "subnormal A")
    got = getattr(dev, form)(m, n, k, a, b).astype(np.float64)
    say("   ", hip.ctx().last_gemm_plan())
    exact = orc.gemm_f64(form == "Tgemm", form == "gemmT", m, n, k, a, b).ravel()
    assert np.all(exact > 0)
    assert np.all(np.abs(got - exact) <= 1e-5 * np.sqrt(k) * exact)        # all terms positive: |A||B| is the result
    # tiny times tiny: the sum of k products of about 2e-42 is a subnormal result
    a2 = rs.uniform(1e-21, 2e-21, m * k).astype(np.float32)
    b2 = rs.uniform(1e-21, 2e-21, k * n).astype(np.float32)
    got = getattr(dev, form)(m, n, k, a2, b2).astype(np.float64)
    exact = orc.gemm_f64(form == "Tgemm", form == "gemmT", m, n, k, a2, b2).ravel()
    assert np.all(exact < np.finfo(np.float32).tiny) and np.all(exact > 0)
    # on the subnormal scale a rounding is an absolute 2^-150 per operation, not a relative one
    assert np.all(got > 0) and np.all(np.abs(got - exact) <= 1e-5 * np.sqrt(k) * exact + 2.0 ** -149 * (k + 1))


@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("form", ["gemm", "gemmT", "Tgemm"])
def test_products_spread_nan_and_inf_like_the_reference(hip, orc, form, shape):
    m, n, k = shape
    rs = np.random.RandomState(3 * m + 5 * n + k)
    a = rs.uniform(-1, 1, m * k).astype(np.float32)
    b = rs.uniform(0.5, 1, k * n).astype(np.float32)          # no zeros: inf * 0 would add NaNs of its own, which it also should
    a[rs.randint(m * k)] = np.nan
    a[rs.randint(m * k)] = np.inf
    b[rs.randint(k * n)] = -np.inf
    b[rs.randint(k * n)] = 0.0
    say(form, shape, "NaN and inf")
    got = getattr(dev, form)(m, n, k, a, b)
    want = getattr(orc, form)(m, n, k, a, b)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want))
    fin = np.isfinite(want)
    fa = np.where(np.isfinite(a), a, 0); fb = np.where(np.isfinite(b), b, 0)
    exact = orc.gemm_f64(form == "Tgemm", form == "gemmT", m, n, k, fa, fb).ravel()
    scale = orc.gemm_f64(form == "Tgemm", form == "gemmT", m, n, k, np.abs(fa), np.abs(fb)).ravel()
    assert np.all(np.abs(got[fin].astype(np.float64) - exact[fin]) <= 1e-5 * np.sqrt(k) * scale[fin])


def special_operand(rs, n, lo=-2.0, hi=2.0):
    x = rs.uniform(lo, hi, n).astype(np.float32)
    specials = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-40, -1e-40, 3e38, -3e38, 1.0, -1.0], np.float32)
    idx = rs.choice(n, min(n, max(len(specials), n // 20)), replace=False)
    x[idx] = specials[np.arange(len(idx)) % len(specials)]
    return x


def assert_same_outcome(got, want, what, rel=1e-6):
    got = np.asarray(got, np.float32).ravel(); want = np.asarray(want, np.float32).ravel()
    assert np.array_equal(np.isnan(got), np.isnan(want)), what
    assert np.array_equal(np.isposinf(got), np.isposinf(want)), what
    assert np.array_equal(np.isneginf(got), np.isneginf(want)), what
    fin = np.isfinite(want)
    g = got[fin].astype(np.float64); w = want[fin].astype(np.float64)
    assert np.all(np.abs(g - w) <= rel * np.abs(w) + 2.0 ** -149), what


UNARY = [("square", 0, 0.0, 0.0), ("pow 2.5", 1, 2.5, 0.0), ("pow 3", 1, 3.0, 0.0), ("pow 0.5", 1, 0.5, 0.0),
         ("pow -1", 1, -1.0, 0.0), ("relu", 2, 0.0, 0.0), ("exp", 3, 0.0, 0.0), ("clip", 4, -0.5, 0.75),
         ("neg_ln", 5, 0.0, 0.0), ("scale", 6, -3.5, 0.0), ("neg_div", 7, 2.0, 0.0)]


@pytest.mark.parametrize("case", UNARY, ids=[u[0].replace(" ", "_") for u in UNARY])
def test_unary_ops_on_special_operands(hip, orc, case):
    name, op, p, q = case
    rs = np.random.RandomState(op * 7 + int(p * 10) + 100)
    for n in (11, 1000, 100003):
        x = special_operand(rs, n)
        say(name, n)
        # the transcendental ops are within 1e-6 of the f64 value, so 2e-6 of each other
        assert_same_outcome(hip.unary(op, x, p, q), orc.unary(op, x, p, q), (name, n), rel=2e-6)
        if op in (4, 5, 7):       # no gradient in the reference
            continue
        g = special_operand(rs, n)
        xg_d = np.zeros(n, np.float32); xg_o = xg_d.copy()      # from zero: no cancellation against what is there
        hip.unary_grad(op, x, xg_d, g, p)
        orc.unary_grad(op, x, xg_o, g, p)
        assert_same_outcome(xg_d, xg_o, (name, "grad", n), rel=4e-6)


@pytest.mark.parametrize("op", [0, 1, 2, 3], ids=["add", "sub", "mul", "div"])
def test_binary_and_broadcast_ops_on_special_operands(hip, orc, op):
    rs = np.random.RandomState(op + 50)
    for rows, cols in [(7, 5), (300, 129), (33, 1024), (5000, 10)]:
        n = rows * cols
        l = special_operand(rs, n); r = special_operand(rs, n)
        say("binary", op, rows, cols)
        got, want = hip.binary_ew(op, l, r), orc.binary_ew(op, l, r)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))      # one IEEE operation: bit for bit
        row = special_operand(rs, cols); col = special_operand(rs, rows)
        got, want = hip.row_op(op, cols, l, row), orc.row_op(op, cols, l, row)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
        got, want = hip.col_op(op, cols, l, col), orc.col_op(op, cols, l, col)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
        # the gradients: a NaN or an inf in the upstream gradient reaches exactly the entries of the
        # broadcast side's gradient whose row or column holds it
        g = rs.uniform(-1, 1, n).astype(np.float32)
        g[rs.choice(n, 3, replace=False)] = [np.nan, np.inf, -np.inf]
        lf = rs.uniform(0.5, 2, n).astype(np.float32)
        for fn, side in (("row_op_grad", rs.uniform(0.5, 2, cols).astype(np.float32)),
                         ("col_op_grad", rs.uniform(0.5, 2, rows).astype(np.float32))):
            lg_d = np.zeros(n, np.float32); sg_d = np.zeros(side.size, np.float32)
            lg_o = np.zeros(n, np.float32); sg_o = np.zeros(side.size, np.float32)
            getattr(hip, fn)(op, cols, lf, side, lg_d, sg_d, g)
            getattr(orc, fn)(op, cols, lf, side, lg_o, sg_o, g)
            assert_same_outcome(lg_d, lg_o, (fn, "lhs"), rel=1e-6)
            assert np.array_equal(np.isnan(sg_d), np.isnan(sg_o)), fn
            assert np.array_equal(np.isposinf(sg_d), np.isposinf(sg_o)) and np.array_equal(np.isneginf(sg_d), np.isneginf(sg_o)), fn


def test_softmax_gradient_and_losses_on_special_operands(hip, orc):
    rs = np.random.RandomState(77)
    for rows, cols in [(7, 5), (64, 10), (33, 1000), (9, 4100)]:
        n = rows * cols
        logits = rs.uniform(-3, 3, n).astype(np.float32)
        probs = orc.softmax(rows, cols, logits)
        g = rs.uniform(-1, 1, n).astype(np.float32)
        for r, v in zip(rs.choice(rows, 3, replace=False), (np.nan, np.inf, -np.inf)):
            g[r * cols + rs.randint(cols)] = v
        say("softmax_grad", rows, cols)
        # a NaN or an inf in a row's upstream gradient turns that row of the result into NaN
        # (inf * p - p * sum is inf - inf) and leaves the others alone
        got, want = hip.softmax_grad(rows, cols, probs, g), orc.softmax_grad(rows, cols, probs, g)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isinf(got), np.isinf(want))
        # cross-entropy of predictions holding 0, 1, values outside [0, 1] and NaN (the reference
        # clips to [1e-7, 1 - 1e-7] first, src/ops2/... via fminf(fmaxf()): a NaN prediction becomes 1e-7)
        preds = rs.uniform(0, 1, n).astype(np.float32)
        preds[rs.choice(n, 5, replace=False)] = [0.0, 1.0, -0.5, 1.5, np.nan]
        targets = np.zeros(n, np.float32)
        targets.reshape(rows, cols)[np.arange(rows), rs.randint(0, cols, rows)] = 1.0
        assert_same_outcome(hip.cce(rows, cols, preds, targets), orc.cce(rows, cols, preds, targets), "cce", rel=2e-6)
        assert_same_outcome(hip.cce_grad(rows, cols, preds, targets), orc.cce_grad(rows, cols, preds, targets), "cce_grad", rel=2e-6)


def test_fused_chains_on_special_operands_equal_the_ops_one_by_one(hip):
    """A chain run as one launch keeps its intermediates in registers; NaN, inf, -0 and subnormals
    have to come out of it exactly as out of the same ops launched one after the other."""
    import test_gpu_fusion as fusion
    rs = np.random.RandomState(11)
    for name, (n_in, prog) in fusion.PROGRAMS.items():
        for n in (11, 1000, 4099):
            say("program", name, n)
            inputs = [special_operand(rs, n) for _ in range(n_in)]
            want = fusion.run_one_by_one(hip, inputs, prog)[4 + len(prog) - 1]
            got = hip.ew_program(inputs, prog)
            assert np.array_equal(got, want, equal_nan=True), name
            ok = ~np.isnan(want)
            assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32)), name      # the sign of a zero too
            g = special_operand(rs, n)
            grads0 = [np.zeros(n, np.float32) for _ in range(n_in)]
            want_g = fusion.grads_one_by_one(hip, inputs, grads0, prog, g)
            got_g = hip.ew_program_grad(inputs, grads0, prog, g)
            for j in range(n_in):
                assert np.array_equal(got_g[j], want_g[j], equal_nan=True), (name, j)


SET_SHAPES = [(1, 1, 1), (5, 10, 7), (64, 64, 64), (129, 127, 130), (300, 10, 2048), (1024, 64, 1), (1, 64, 1024),
              (64, 1, 1024), (512, 512, 512), (32, 32, 100003), (16, 3000, 500), (257, 17, 3333), (40, 72, 15),
              (96, 40, 8192), (16, 2048, 4096), (8, 4096, 2048), (4096, 16, 4096), (2048, 24, 8192), (1000, 1000, 256),
              (1, 2048, 2048), (2048, 2048, 96), (1100, 1100, 700)]


@pytest.mark.parametrize("shape", SET_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_beta_zero_overwrites_whatever_the_output_held(hip, shape):
    """beta = 0 is the reference's SET (src/ops2/gemm/cpu_stack.rs:39 hands BLAS beta = 0, which by
    the BLAS rule does not read C): an output full of NaN must come out as if it had held zeros,
    on every product kernel and every split / combine / transposed route behind the entry point."""
    m, n, k = shape
    rs = np.random.RandomState(m + 3 * n + 5 * k)
    a = rs.uniform(-1, 1, m * k).astype(np.float32)
    b = rs.uniform(-1, 1, k * n).astype(np.float32)
    nan_c = np.full(m * n, np.nan, np.float32)
    for ta, tb in ((0, 0), (0, 1), (1, 0), (1, 1)):
        say("sgemm", ta, tb, shape)
        clean = hip.sgemm(ta, tb, m, n, k, a, b, c=np.zeros(m * n, np.float32), beta=0.0)
        dirty = hip.sgemm(ta, tb, m, n, k, a, b, c=nan_c.copy(), beta=0.0)
        say("   ", hip.ctx().last_gemm_plan())
        assert np.isfinite(clean).all() and np.array_equal(clean, dirty)
    pre = rs.uniform(-1, 1, m * n).astype(np.float32)
    clean = hip.sgemm_relu_mask(0, 0, m, n, k, a, b, pre, c=np.zeros(m * n, np.float32))
    dirty = hip.sgemm_relu_mask(0, 0, m, n, k, a, b, pre, c=nan_c.copy())
    assert np.isfinite(clean).all() and np.array_equal(clean, dirty)
    # the gradient pair of a product and of a Linear layer (trait order m, k, n)
    g = rs.uniform(-1, 1, m * n).astype(np.float32)
    lg0, rg0 = hip.gemm_grad(m, k, n, a, b, np.zeros(m * k, np.float32), np.zeros(k * n, np.float32), g)
    lg1, rg1 = hip.gemm_grad(m, k, n, a, b, np.full(m * k, np.nan, np.float32), np.full(k * n, np.nan, np.float32), g)
    assert np.array_equal(lg0, lg1) and np.array_equal(rg0, rg1) and np.isfinite(lg0).all() and np.isfinite(rg0).all()
    z = lambda cnt: np.zeros(cnt, np.float32)
    f = lambda cnt: np.full(cnt, np.nan, np.float32)
    x0, w0, b0 = hip.linear_grad(m, k, n, a, b, g, x_grad=z(m * k), relu_pre=None, w_grad=z(k * n), bias_grad=z(n))
    # (the bias gradient always accumulates, as add_row_mut_grad does in the reference: src/ops2/row_op/grad/cpu.rs:42-50)
    x1, w1, b1 = hip.linear_grad(m, k, n, a, b, g, x_grad=f(m * k), relu_pre=None, w_grad=f(k * n), bias_grad=z(n))
    assert np.array_equal(x0, x1) and np.array_equal(w0, w1) and np.array_equal(b0, b1)
    assert np.isfinite(x0).all() and np.isfinite(w0).all() and np.isfinite(b0).all()


def test_set_semantics_of_the_other_ops_with_an_output_full_of_nan(hip):
    rs = np.random.RandomState(5)
    for rows, cols in [(7, 5), (300, 129), (1000, 4099), (5000, 10), (8191, 1025), (64, 100003)]:
        n = rows * cols
        x = rs.uniform(-3, 3, n).astype(np.float32)
        say("set semantics", rows, cols)
        clean = hip.transpose(rows, cols, x, out=np.zeros(n, np.float32), assign=False)
        dirty = hip.transpose(rows, cols, x, out=np.full(n, np.nan, np.float32), assign=False)
        assert np.array_equal(clean, dirty) and np.array_equal(clean.reshape(cols, rows), x.reshape(rows, cols).T)
        p = hip.softmax(rows, cols, x)
        g = rs.uniform(-1, 1, n).astype(np.float32)
        clean = hip.softmax_grad(rows, cols, p, g, x_grad=np.zeros(n, np.float32), beta=0.0)
        dirty = hip.softmax_grad(rows, cols, p, g, x_grad=np.full(n, np.nan, np.float32), beta=0.0)
        assert np.isfinite(clean).all() and np.array_equal(clean, dirty)
        t = np.zeros(n, np.float32)
        t.reshape(rows, cols)[np.arange(rows), rs.randint(0, cols, rows)] = 1.0
        clean = hip.softmax_cce_grad(rows, cols, p, t, np.zeros(n, np.float32), beta=0.0)
        dirty = hip.softmax_cce_grad(rows, cols, p, t, np.full(n, np.nan, np.float32), beta=0.0)
        assert np.isfinite(clean).all() and np.array_equal(clean, dirty)
