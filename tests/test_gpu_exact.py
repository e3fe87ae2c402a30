"""Oracle comparisons that cannot pass by accident: operands with small integer values.

Every partial sum of such operands is an integer below 2^24, which f32 holds exactly, so a sum or a
product has ONE right answer whatever the order of the additions - the reference's sequential
loops (src/ops2/sum/cpu.rs:78-90, src/ops2/mean/cpu.rs:34-49, the BLAS call of
src/ops2/gemm/cpu_stack.rs:39) and the device's trees, splits and matrix-core accumulators must agree
bit for bit.  A dropped term, a tile read twice, a lost k remainder or a partial result that is
combined wrongly changes the integer and fails `array_equal`; no tolerance is involved.

Sizes: the configured ones - [16384 x 16384], [1 x 2^28] / [2^28 x 1], [32768 x 4096], the whole
GEMM sweep in its three forms (also accumulating into C), and the two MLPs' layer shapes."""
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu
SEED = rng.DEFAULT_SEED


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def small_ints(n, half_width, tag, seed=SEED):
    """n values uniform in {-half_width .. half_width} as f32, from the seeded generator."""
    return (rng.integers(n, 2 * half_width + 1, tag=tag, seed=seed).astype(np.int64) - half_width).astype(np.float32)


@pytest.mark.parametrize("shape", [(16384, 16384), (32768, 4096), (4026, 33333), (522247, 257), (134, 1000000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_sums_and_means_of_small_integers_equal_the_oracle_bit_for_bit(hip, orc, shape):
    rows, cols = shape
    c = hip.ctx()
    say("integer-valued sums", rows, cols)
    x = small_ints(rows * cols, 8, tag=0)                 # |any partial sum| <= 8 * 2^20 < 2^24
    d = c.array(x)
    out_c, out_r = c.empty(cols), c.empty(rows)
    for fn, out, ref in (("slhip_sum_rows", out_c, orc.sum_rows), ("slhip_mean_rows", out_c, orc.mean_rows),
                         ("slhip_sum_cols", out_r, orc.sum_cols), ("slhip_mean_cols", out_r, orc.mean_cols)):
        c.call("slhip_fill", out.n, -1.0, out.ptr)
        c.call(fn, rows, cols, d.ptr, out.ptr)
        got, want = out.numpy(), ref(cols, x)
        assert np.array_equal(got, want), (fn, np.flatnonzero(got != want)[:5])
    # against integer arithmetic as well: the oracle is not its own witness
    X = x.reshape(rows, cols).astype(np.int64)
    c.call("slhip_sum_rows", rows, cols, d.ptr, out_c.ptr)
    c.call("slhip_sum_cols", rows, cols, d.ptr, out_r.ptr)
    assert np.array_equal(out_c.numpy().astype(np.int64), X.sum(0)) and np.array_equal(out_r.numpy().astype(np.int64), X.sum(1))
    for b in (d, out_c, out_r):
        b.free()


def test_whole_buffer_sums_of_2_28_small_integers_equal_the_oracle(hip, orc):
    """[1 x 2^28] and [2^28 x 1] in the reducing direction, `mean` and `sum` over 2^28 values in
    {-1, 0, 1}: the reference's sequential f32 sum never leaves the integers below 2^24 (the running
    sum of 2^28 such values stays within a few times 10^4)."""
    n = 1 << 28
    c = hip.ctx()
    say("integer-valued sums over 2^28 elements")
    x = small_ints(n, 1, tag=1)
    total = int(x.astype(np.int64).sum())
    walk_max = int(np.abs(np.cumsum(x[: 1 << 24].astype(np.int64))).max())
    assert abs(total) < (1 << 22) and walk_max < (1 << 22)
    d, one = c.array(x), c.empty(1)
    want_sum = orc.sum_cols(n, x)[0]
    assert int(want_sum) == total
    for fn, rows, cols in (("slhip_sum_cols", 1, n), ("slhip_sum_rows", n, 1)):
        c.call("slhip_fill", 1, -1.0, one.ptr)
        c.call(fn, rows, cols, d.ptr, one.ptr)
        assert one.numpy()[0] == want_sum, fn
    c.call("slhip_sum", n, d.ptr, one.ptr)
    assert one.numpy()[0] == orc.sum_all(x)
    c.call("slhip_mean", n, d.ptr, one.ptr)
    assert one.numpy()[0] == orc.mean(x) == np.float32(total) / np.float32(n)
    for fn, rows, cols in (("slhip_mean_cols", 1, n), ("slhip_mean_rows", n, 1)):
        c.call(fn, rows, cols, d.ptr, one.ptr)
        assert one.numpy()[0] == np.float32(total) / np.float32(n), fn
    d.free()
    one.free()


SWEEP = [(512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192),
         (8192, 2048, 784), (784, 2048, 8192)]
# the layer shapes of the two MLPs (forward, input gradient, weight gradient) and odd ones that take
# the edge, remainder, spread-tail, tall and skinny paths
LAYERS = [(8192, 10, 2048), (8192, 2048, 10), (2048, 10, 8192), (1024, 64, 64), (1024, 64, 1), (1024, 1, 64), (64, 64, 1024),
          (16384, 16, 16384), (4608, 4608, 1024), (3585, 3457, 1031), (1000, 777, 50), (257, 129, 4100), (70, 70, 100000)]


@pytest.mark.parametrize("shape", SWEEP + LAYERS, ids=lambda s: "x".join(map(str, s)))
def test_products_of_small_integers_equal_the_oracle_bit_for_bit(hip, orc, shape):
    """A, B in {-2 .. 2}: every product is an integer of magnitude <= 4 and every partial sum stays
    below 4 * K <= 2^19, so C = op(A) op(B) has one value in f32 whatever the order of the k loop:
    the three forms, and the backward forms accumulating into an integer-valued C, against the oracle
    and against an f64 product (exact for these integers) on sampled rows."""
    m, n, k = shape
    c = hip.ctx()
    a, b = small_ints(m * k, 2, tag=2), small_ints(k * n, 2, tag=3)
    da, db, dc = c.array(a), c.array(b), c.empty(m * n)
    c0 = small_ints(m * n, 100, tag=4)
    rows = np.unique(np.concatenate([rng.integers(16, m, tag=5, seed=SEED), [0, m - 1]]))
    for form, ta, tb in (("A*B", 0, 0), ("A*Bt", 0, 1), ("At*B", 1, 0)):
        say("integer-valued gemm", form, m, n, k)
        ref = (orc.Tgemm if ta else orc.gemmT if tb else orc.gemm)(m, n, k, a, b)
        A = a.reshape(k, m).T if ta else a.reshape(m, k)
        B = b.reshape(n, k).T if tb else b.reshape(k, n)
        assert np.array_equal(ref.reshape(m, n)[rows].astype(np.float64), A[rows].astype(np.float64) @ B.astype(np.float64))   # integers below 2^53: exact
        c.call("slhip_fill", m * n, -7.0, dc.ptr)
        c.call("slhip_sgemm", ta, tb, m, n, k, da.ptr, db.ptr, dc.ptr, 0.0)
        got = dc.numpy()
        assert np.array_equal(got, ref), (form, np.flatnonzero(got != ref)[:5])
        dc.upload(c0)
        c.call("slhip_sgemm", ta, tb, m, n, k, da.ptr, db.ptr, dc.ptr, 1.0)
        assert np.array_equal(dc.numpy(), c0 + ref), form + " beta=1"
    for z in (da, db, dc):
        z.free()


def test_linear_layer_on_small_integers_equals_the_oracle(hip, orc):
    """The fused Linear forward (product + bias + ReLU in the epilogue) and the fused backward of the
    classifier's first layer shape, on integer-valued operands: bit for bit the oracle's op sequence."""
    m, k, n = 8192, 784, 2048
    say("integer-valued linear layer", m, k, n)
    x, w, bias = small_ints(m * k, 2, tag=6), small_ints(k * n, 2, tag=7), small_ints(n, 50, tag=8)
    pre = orc.add_row(m, n, orc.gemm(m, n, k, x, w), bias)
    want = orc.unary(orc.RELU, pre)
    got = hip.linear_fwd(m, k, n, x, w, bias, relu=True)
    assert np.array_equal(got, want)
    g = small_ints(m * n, 2, tag=9)
    lg, rg = np.zeros(m * k, np.float32), np.zeros(k * n, np.float32)
    lg_r, rg_r = lg.copy(), rg.copy()
    hip.gemm_grad(m, k, n, x, w, lg, rg, g)
    orc.gemm_grad(m, k, n, x, w, lg_r, rg_r, g)
    assert np.array_equal(lg, lg_r) and np.array_equal(rg, rg_r)
    bg = hip.add_row_mut_grad(m, n, np.zeros(n, np.float32), g)
    assert np.array_equal(bg, orc.add_row_mut_grad(m, n, np.zeros(n, np.float32), g))
