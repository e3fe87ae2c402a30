"""The C++ host device layer (tape, gradient map, cache) on the GPU, driven the way the
reference's integration tests drive its devices: forward op, `backward()`, read `.grad()`.
Expected values are the reference's own (tests/*.rs); the training loops are compared with the
CPU oracle's loops step by step."""
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture()
def device():
    from sliced_amd import host
    d = host.HIP(0, cached=False)
    yield d
    d.close()


def eq(buf, expect):
    assert np.array_equal(buf.read(), np.asarray(expect, np.float32)), (buf.read(), expect)


# reference: tests/test_gemm.rs:4-43
def test_gemm(device):
    lhs = device.buffer([1, 2, 3, 4, 4, 5, 6, 5])
    rhs = device.buffer([1, 2, 3, 4, 5, 6])
    out = device.gemm(4, 2, 3, lhs, rhs)
    eq(out, [9, 12, 15, 19, 26, 33, 24, 33, 42, 26, 37, 48])
    out.backward()
    eq(lhs.grad(), [6, 15, 6, 15, 6, 15, 6, 15])
    eq(rhs.grad(), [14, 14, 14, 16, 16, 16])


def test_gemm_skips_operands_without_requires_grad(device):
    lhs = device.buffer([1, 2, 3, 4, 4, 5, 6, 5]).no_grad()
    rhs = device.buffer([1, 2, 3, 4, 5, 6])
    out = device.gemm(4, 2, 3, lhs, rhs)
    out.backward()
    assert not lhs.has_grad()            # src/ops2/gemm/grad/cpu_stack.rs:35
    eq(rhs.grad(), [14, 14, 14, 16, 16, 16])


# reference: tests/test_add.rs, test_sub.rs, test_mul.rs
def test_add_sub_mul(device):
    lhs, rhs = device.buffer([1, 2, 3, 4, 5]), device.buffer([6, 7, 8, 9, 10])
    out = device.add(lhs, rhs)
    eq(out, [7, 9, 11, 13, 15])
    out.backward()
    eq(lhs.grad(), [1] * 5)
    eq(rhs.grad(), [1] * 5)
    lhs, rhs = device.buffer([1, 2, 3, 4, 5]), device.buffer([6, 7, 8, 9, 10])
    out = device.sub(lhs, rhs)
    eq(out, [-5] * 5)
    out.backward()
    eq(lhs.grad(), [1] * 5)
    eq(rhs.grad(), [-1] * 5)
    lhs, rhs = device.buffer([1, 2, 3, 4, 5]), device.buffer([6, 7, 8, 9, 10])
    out = device.mul(lhs, rhs)
    eq(out, [6, 14, 24, 36, 50])
    out.backward()
    eq(lhs.grad(), [6, 7, 8, 9, 10])
    eq(rhs.grad(), [1, 2, 3, 4, 5])


# reference: tests/test_pow.rs, tests/test_square.rs, tests/matrix/relu.rs
def test_pow_square_relu(device):
    x = device.buffer([1, 2, 3, 4, 5])
    out = device.pow(x, 3.0)
    eq(out, [1, 8, 27, 64, 125])
    out.backward()
    eq(x.grad(), [3, 12, 27, 48, 75])
    x = device.buffer([1, 2, 3, 4, 5])
    out = device.square(x)
    eq(out, [1, 4, 9, 16, 25])
    out.backward()
    eq(x.grad(), [2, 4, 6, 8, 10])
    x = device.buffer([-1, -3, 2, 5, -1.3])
    out = device.relu(x)
    eq(out, [0, 0, 2, 5, 0])
    out.backward()
    eq(x.grad(), [0, 0, 1, 1, 0])


# reference: tests/test_row_op.rs:3-77
def test_row_op_and_row_op_mut(device):
    data = [-1, -3, 4, 5, 2, 2, 1, 5, -3, 2, 2, 4, 3, 2, -1]
    expect = [0, -1, 7, 9, 7, 3, 3, 8, 1, 7, 3, 6, 6, 6, 4]
    buf, row = device.buffer(data), device.buffer([1, 2, 3, 4, 5])
    out = device.add_row(3, 5, buf, row)
    eq(out, expect)
    out.backward()
    eq(row.grad(), [3] * 5)
    eq(buf.grad(), [1] * 15)
    buf, row = device.buffer(data), device.buffer([1, 2, 3, 4, 5])
    device.add_row_mut(3, 5, buf, row)
    eq(buf, expect)
    buf.backward()
    eq(row.grad(), [3] * 5)
    eq(buf.grad(), [1] * 15)


# reference: tests/test_sum_rows.rs, test_sum_cols.rs, test_max_rows.rs, test_max_cols.rs, test_mean.rs
def test_reductions_under_a_following_op(device):
    x = device.buffer([4, 2, 1, 3, 6, 1, 3, 1, 5, 4, 1, 1])
    rhs = device.buffer([1, 4, 2, 3])
    out = device.mul(device.sum_rows(4, x), rhs)
    out.backward()
    eq(x.grad(), [1, 4, 2, 3] * 3)
    eq(rhs.grad(), [15, 7, 5, 5])

    x = device.buffer([4, 2, 1, 3, 6, 1, 3, 1, 5, 4, 1, 1])
    rhs = device.buffer([1, 4, 2])
    out = device.mul(device.sum_cols(4, x), rhs)
    out.backward()
    eq(x.grad(), [1, 1, 1, 1, 4, 4, 4, 4, 2, 2, 2, 2])
    eq(rhs.grad(), [10, 11, 11])

    data = [-3, 2, 3, 1, 1, 5, -5, 4, -9, -2, -4, -1]
    x, rhs = device.buffer(data), device.buffer([2, 3, 4, 1])
    out = device.mul(device.max_rows(4, x), rhs)
    out.backward()
    eq(x.grad(), [0, 0, 4, 0, 2, 3, 0, 1, 0, 0, 0, 0])
    eq(rhs.grad(), [1, 5, 3, 4])

    x, rhs = device.buffer(data), device.buffer([1, 4, 2])
    mc = device.max_cols(3, 4, x)
    eq(mc, [3, 5, -1])
    out = device.add(mc, rhs)
    out.backward()
    eq(x.grad(), [0, 0, 1, 0, 0, 1, 0, 0, 0, 0, 0, 1])
    eq(rhs.grad(), [1, 1, 1])

    lhs = device.buffer([2, 3, 4])
    x = device.buffer([1, 4, 3, 2, 3, 5, 2, 1, 6, -2, 1, 4])
    out = device.sub(lhs, device.mean_rows(3, x))
    out.backward()
    eq(x.grad(), [-0.25] * 12)
    eq(lhs.grad(), [1, 1, 1])


# reference: tests/matrix/transpose.rs, tests/matrix/softmax.rs, tests/matrix/l2_norm_cols.rs
def test_transpose_softmax_l2norm(device):
    x = device.buffer([1, 2, 3, 4, 5, 6])
    xt = device.transpose(2, 3, x)
    eq(xt, [1, 4, 2, 5, 3, 6])
    y = device.buffer([-1, 1, 2, -5, -3, 2])
    out = device.mul(y, xt)
    out.backward()
    eq(x.grad(), [-1, 2, -3, 1, -5, 2])          # transpose(3, 2, y)

    x = device.buffer([1, 2, 3, 4, 5, 6])
    out = device.softmax(2, 3, x)
    assert np.max(np.abs(out.read() - np.array([0.09003057, 0.24472847, 0.66524096] * 2, np.float32))) < 1e-7
    out.backward()
    assert np.max(np.abs(x.grad().read())) < 1e-6

    x = device.buffer([1, 2, 3, 4, 5, 6, 7, 8])
    out = device.pow(device.sum_cols(4, device.square(x)), 0.5)
    out.backward()
    assert np.max(np.abs(x.grad().read()[:4] - np.array([0.1826, 0.3651, 0.5477, 0.7303], np.float32))) < 1e-2


# reference: tests/matrix/tanh.rs:12-31; sigmoid (src/matrix.rs:231-258) has no reference vector:
# closed form in f64
def test_tanh_sigmoid_on_the_tape(device):
    x = device.buffer([-1, -3, 2, 5, -1.3, 0])
    out = device.tanh(x)
    assert np.max(np.abs(out.read() - np.array([-0.7615942, -0.9950548, 0.9640276, 0.9999092, -0.8617231, 0.]))) < 1e-6
    out.backward()
    want = np.array([0.41997433, 0.009865999, 0.070650816, 0.00018155575, 0.25743324, 1.0])
    assert np.max(np.abs(x.grad().read() - want)) < 1e-6
    v = np.array([-2.0, -0.5, 0.0, 0.25, 3.0])
    x = device.buffer(v)
    out = device.sigmoid(x)
    s = 1 / (1 + np.exp(-v))
    assert np.max(np.abs(out.read() - s)) < 1e-6
    out.backward()
    assert np.max(np.abs(x.grad().read() - s * (1 - s))) < 1e-6


# reference: src/ops2/col_op/cpu.rs:56-72 (forward), src/ops2/col_op/grad/cpu.rs:97-161 (div grads),
# src/ops2/row_op/grad/cpu.rs:94-111 (mul grads), src/ops2/diagflat/grad/cpu.rs:44-60,
# src/ops2/onehot/grad/cpu.rs:18-38, tests/matrix/l2_norm_cols.rs
def test_col_op_row_op_diagflat_onehot_on_the_tape(device):
    from sliced_amd import host
    lhs = device.buffer([1, -1, 3, 4, 2, 2, 3, 4, 1, 1, 2, 0, 3, 3, -2])
    rhs = device.buffer([3, 2, 1])
    out = device.col_op(host.ADD, 3, 5, lhs, rhs)
    eq(out, [4, 2, 6, 7, 5, 4, 5, 6, 3, 3, 3, 1, 4, 4, -1])
    out.backward()                                  # runs (and clears) the tape
    eq(lhs.grad(), [1] * 15)
    eq(rhs.grad(), [5, 5, 5])

    lhs = device.buffer([1, 2, 3, 4, 5, 6])
    rhs = device.buffer([-3, 2])
    out = device.div_cols(2, 3, lhs, rhs)
    seed = device.buffer([1.4, 2.5, 3.3, 4, 5, 6])
    out.backward_with(seed)
    assert np.max(np.abs(lhs.grad().read() - np.array([1.4 / -3, 2.5 / -3, 3.3 / -3, 2, 2.5, 3]))) < 1e-6
    gf = lambda l, r: l / -(r * r)
    want = [gf(1, -3) * 1.4 + gf(2, -3) * 2.5 + gf(3, -3) * 3.3, gf(4, 2) * 4 + gf(5, 2) * 5 + gf(6, 2) * 6]
    assert np.max(np.abs(rhs.grad().read() - np.array(want))) < 1e-5

    # sub_cols: d/dlhs = 1, d/drhs = -1 summed over the row
    lhs = device.buffer([1, 2, 3, 4, 5, 6])
    rhs = device.buffer([0.5, -1])
    out = device.sub_cols(2, 3, lhs, rhs)
    eq(out, [0.5, 1.5, 2.5, 5, 6, 7])
    out.backward()
    eq(lhs.grad(), [1] * 6)
    eq(rhs.grad(), [-3, -3])

    # row_op multiply: lhs.grad = rhs[c] * g, rhs.grad[c] = sum_r lhs[r,c] * g[r,c]
    lhs = device.buffer([1, 2, 3, 4, 5, 6])
    rhs = device.buffer([2, -1, 0.5])
    out = device.row_op(host.MUL, 2, 3, lhs, rhs)
    eq(out, [2, -2, 1.5, 8, -5, 3])
    out.backward()
    eq(lhs.grad(), [2, -1, 0.5, 2, -1, 0.5])
    eq(rhs.grad(), [5, 7, 9])

    x = device.buffer([4, 5, 3, -3])
    d = device.diagflat(x)
    eq(d, [4, 0, 0, 0, 0, 5, 0, 0, 0, 0, 3, 0, 0, 0, 0, -3])
    d.backward_with(device.buffer([4, 1, 3, -3, 2, 5, 3, 1, 2, 6, 3, -3, 2, 7, 3, -3]))
    eq(x.grad(), [4, 5, 3, -3])

    cls = device.buffer([0, 1, 4, 3])
    oh = device.onehot(5, cls)
    eq(oh, [1, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 1, 0])
    oh.backward_with(device.buffer([2, -1, 3, 7, -2, 1, 3, 2, 4, 3, 3, -2, 3, -2, 1, 5, 6, -1, 4, 5]))
    eq(cls.grad(), [2, 3, 1, 4])

    x = device.buffer([1, 2, 3, 4, 5, 6, 7, 8])
    out = device.l2_norm_cols(2, 4, x)
    assert np.max(np.abs(out.read() - np.sqrt([30.0, 174.0]))) < 1e-5
    out.backward()
    assert np.max(np.abs(x.grad().read()[:4] - np.array([0.1826, 0.3651, 0.5477, 0.7303]))) < 1e-4


# reference: examples/chained_perf.rs:54-91 — cached device, the same chain every iteration
def test_cached_range_reuses_buffers_and_values():
    from sliced_amd import host
    dev = host.HIP(0, cached=True)
    n = 12345
    x, b = dev.buffer(np.full(n, 1.3, np.float32)), dev.buffer(np.full(n, 2.1, np.float32))
    ids = None
    for epoch in range(5):
        dev.begin_iteration()
        dev.zero_grad()                                # as the examples do at the top of every iteration
        squared = dev.square(x)
        add = dev.add(b, x)
        mul_b = dev.mul(add, b)
        mul = dev.mul(squared, x)
        out = dev.add(mul, mul_b)
        assert out.read()[0] == np.float32(9.336999)
        now = [t.id for t in (squared, add, mul_b, mul, out)]
        if ids is not None:
            assert now == ids                       # same call position -> same allocation
        ids = now
        out.backward()
        g = x.grad().read()
        # d/dx (x^3 + (b+x) b) = 3x^2 + b; the cached intermediates keep their ids and therefore
        # their gradient buffers, which zero_grad cleared
        assert abs(g[0] - (3 * 1.3 ** 2 + 2.1)) < 1e-4
    dev.zero_grad()
    assert np.all(x.grad().read() == 0)
    dev.close()


def test_linear_fused_matches_unfused_tape(device):
    m, k, n = 96, 40, 24
    x = rng.uniform(m * k, -1, 1, tag=0)
    w = rng.uniform(k * n, -1, 1, tag=1)
    b = rng.uniform(n, -1, 1, tag=2)
    res = []
    for fused in (False, True):
        xb, wb, bb = device.buffer(x), device.buffer(w), device.buffer(b)
        if fused:
            out = device.linear(m, k, n, xb, wb, bb, True)
        else:
            h = device.gemm(m, k, n, xb, wb)
            device.add_row_mut(m, n, h, bb)
            out = device.relu(h)
        out.backward()
        res.append([out.read(), xb.grad().read(), wb.grad().read(), bb.grad().read()])
    for a, c in zip(*res):
        assert np.array_equal(a, c)


def test_zero_grad_of_large_gradients_is_deferred_but_never_visible(device):
    """Gradients of 2^20 floats and more are zeroed when next read or accumulated into, and not at
    all when an op overwrites them first: whatever the order of calls, the values are those of
    an immediate fill."""
    n = (1 << 20) + 192
    xv = rng.uniform(n, -2, 2, tag=0)
    x = device.buffer(xv)
    device.square(x).backward()
    g = x.grad()                                       # handle kept across zero_grad
    assert np.array_equal(g.read(), 2 * xv)
    device.zero_grad()
    assert not g.read().any()                          # read through the old handle
    device.square(x).backward()                        # accumulating op: 0 + 2x, not 2x + 2x
    assert np.array_equal(x.grad().read(), 2 * xv)
    device.zero_grad()
    device.square(x).backward()
    device.square(x).backward()                        # second accumulation after one fill
    assert np.array_equal(x.grad().read(), 4 * xv)

    # overwriting op (gemm_grad with the default SET policy), then the accumulate policy
    m, k, nn = 2048, 512, 8
    a, b = device.buffer(rng.uniform(m * k, -1, 1, tag=1)), device.buffer(rng.uniform(k * nn, -1, 1, tag=2))
    device.gemm(m, k, nn, a, b).backward()
    first = a.grad().read()
    assert first.any()
    for _ in range(2):
        device.zero_grad()
        device.gemm(m, k, nn, a, b).backward()
        assert np.array_equal(a.grad().read(), first)
    device.set_grad_policy(gemm_beta=1.0)
    device.zero_grad()
    device.gemm(m, k, nn, a, b).backward()
    assert np.array_equal(a.grad().read(), first)      # 0 + v
    device.gemm(m, k, nn, a, b).backward()
    assert np.allclose(a.grad().read(), 2 * first, rtol=1e-6, atol=0)
    device.set_grad_policy()


def test_backward_seed_is_refilled_after_another_op_wrote_it():
    """backward() skips the fill of a seed gradient that still holds its ones; any other write to
    that gradient (here: the buffer feeds a further op in one iteration) brings the fill back."""
    from sliced_amd import host
    dev = host.HIP(0, cached=True)
    xv = rng.uniform(1000, 0.5, 1.5, tag=0)
    x = dev.buffer(xv)
    for epoch in range(6):
        dev.begin_iteration()
        dev.zero_grad()
        sq = dev.square(x)
        if epoch % 3 == 2:                              # sq is an inner node: its gradient is accumulated into
            dev.square(sq).backward()
            assert np.allclose(x.grad().read(), 4 * xv ** 3, rtol=1e-6, atol=0)
        else:                                           # sq is the loss: its gradient is the seed
            sq.backward()
            assert np.array_equal(x.grad().read(), 2 * xv)
            assert np.array_equal(sq.grad().read(), np.ones(1000, np.float32))
    dev.zero_grad()
    assert not sq.grad().read().any()
    dev.close()


def test_relu_grad_fused_into_the_next_layers_input_gradient(device):
    # two fused Linear+ReLU layers and a plain one: with the ReLU gradients riding in the next
    # layer's input-gradient GEMM every gradient keeps its bits
    m, d0, d1, d2, d3 = 192, 40, 96, 72, 10
    x = rng.uniform(m * d0, -1, 1, tag=0)
    ws = [rng.uniform(a * b, -0.5, 0.5, tag=10 + i) for i, (a, b) in enumerate([(d0, d1), (d1, d2), (d2, d3)])]
    bs = [rng.uniform(b, -0.5, 0.5, tag=20 + i) for i, b in enumerate([d1, d2, d3])]
    res = []
    try:
        for fuse in (False, True):
            device.set_fuse_relu_grad(fuse)
            xb = device.buffer(x)
            wb = [device.buffer(w) for w in ws]
            bb = [device.buffer(b) for b in bs]
            h1 = device.linear(m, d0, d1, xb, wb[0], bb[0], True)
            h2 = device.linear(m, d1, d2, h1, wb[1], bb[1], True)
            out = device.linear(m, d2, d3, h2, wb[2], bb[2], False)
            out.backward()
            res.append([out.read(), xb.grad().read()] + [w.grad().read() for w in wb] + [b.grad().read() for b in bb])
    finally:
        device.set_fuse_relu_grad(False)
    assert np.abs(res[0][1]).max() > 0
    for a, c in zip(*res):
        assert np.array_equal(a, c)


def test_relu_mask_kept_as_bits_gives_the_same_gradients(device):
    """Layers of 2^22 outputs and more keep their ReLU mask as bits when the policy allows it: the
    gradients equal those of the float path up to the order in which the GEMM plans add (the bit
    kernels run whole tiles unsplit) and the few mask bits that order decides, and a ReLU output that feeds something else than a fused
    Linear takes the unpacking elementwise gradient."""
    m, d0, d1, d2, d3 = 2048, 64, 2048, 2080, 10
    x = rng.uniform(m * d0, -1, 1, tag=0)
    ws = [rng.uniform(a * b, -0.1, 0.1, tag=10 + i) for i, (a, b) in enumerate([(d0, d1), (d1, d2), (d2, d3)])]
    bs = [rng.uniform(b, -0.5, 0.5, tag=20 + i) for i, b in enumerate([d1, d2, d3])]
    res = []
    try:
        device.set_fuse_relu_grad(True)
        for bits in (False, True):
            device.set_relu_bits(bits)
            for tail in ("linear", "square"):
                xb = device.buffer(x)
                wb = [device.buffer(w) for w in ws]
                bb = [device.buffer(b) for b in bs]
                h1 = device.linear(m, d0, d1, xb, wb[0], bb[0], True)
                h2 = device.linear(m, d1, d2, h1, wb[1], bb[1], True)
                out = device.linear(m, d2, d3, h2, wb[2], bb[2], False) if tail == "linear" else device.square(h2)
                out.backward()
                res.append([out.read(), xb.grad().read()] + [w.grad().read() for w in wb[:2]] + [b.grad().read() for b in bb[:2]])
    finally:
        device.set_fuse_relu_grad(False)
        device.set_relu_bits(False)
    for ref, got in ((res[0], res[2]), (res[1], res[3])):
        assert np.abs(ref[1]).max() > 0
        for a, c in zip(ref, got):
            # the two paths add in different orders, so a pre-activation within rounding of zero may
            # land on the other side of it: a handful of mask bits, each worth one term of a sum
            scale = np.abs(a).max()
            off = np.abs(a - c) > 1e-3 * scale          # three chained products of K up to 2080: 1e-5 * sqrt(K) each
            assert off.mean() <= 1e-3 and np.max(np.abs(a - c)) <= 5e-2 * scale, (off.mean(), np.max(np.abs(a - c)), scale)


def test_errors_surface_as_exceptions(device):
    from sliced_amd import host
    a = device.buffer([1, 2, 3])
    with pytest.raises(host.HostError):
        device.gemm(2, 2, 2, a, a)              # length != rows*cols
    with pytest.raises(host.HostError):
        a.grad()                                 # no gradient was ever written


def test_self_products_are_differentiable(device, orc):
    """x*x, x+x, x-x: both gradient terms land in the one gradient, lhs term first
    (slice_binary_grad, src/ops2/binary_ew/grad/cpu_stack.rs:55-58)."""
    xv = np.array([1, -2, 3, 0.5, -7], np.float32)
    for op, name, want in ((device.mul, "mul", 2 * xv), (device.add, "add", np.full(5, 2, np.float32)),
                           (device.sub, "sub", np.zeros(5, np.float32))):
        say("self", name)
        x = device.buffer(xv)
        out = op(x, x)
        out.backward()
        lg, rg = np.zeros(5, np.float32), np.zeros(5, np.float32)
        code = {"add": orc.ADD, "sub": orc.SUB, "mul": orc.MUL}[name]
        orc.binary_ew_grad(code, xv, xv, lg, rg, np.ones(5, np.float32))
        eq(x.grad(), lg + rg)
        eq(x.grad(), want)


def test_relu_output_with_two_readers_keeps_its_own_gradient(device):
    """With the ReLU gradient folded into the next layer's input-gradient GEMM switched on, a ReLU
    output that a second op reads as well must still collect that op's term: the fold is taken
    only for a single reader, and both settings give the same gradients."""
    m, d0, d1, d2 = 160, 48, 96, 80
    x = rng.uniform(m * d0, -1, 1, tag=0)
    w1, w2 = rng.uniform(d0 * d1, -0.5, 0.5, tag=1), rng.uniform(d1 * d2, -0.5, 0.5, tag=2)
    b1, b2 = rng.uniform(d1, -0.5, 0.5, tag=3), rng.uniform(d2, -0.5, 0.5, tag=4)
    res = []
    try:
        for fuse in (False, True):
            device.set_fuse_relu_grad(fuse)
            device.set_grad_policy(gemm_beta=1.0)           # accumulate, so both readers' terms add up
            xb, w1b, w2b, b1b, b2b = (device.buffer(v) for v in (x, w1, w2, b1, b2))
            h1 = device.linear(m, d0, d1, xb, w1b, b1b, True)
            y = device.linear(m, d1, d2, h1, w2b, b2b, False)   # reader 1: a fused Linear
            s = device.square(h1)                                # reader 2
            ys = device.sum_cols(d2, y)
            ss = device.sum_cols(d1, s)
            tot = device.add(ys, ss)
            tot.backward()
            res.append([h1.grad().read(), xb.grad().read(), w1b.grad().read(), b1b.grad().read()])
    finally:
        device.set_fuse_relu_grad(False)
        device.set_grad_policy()
    h1g = res[1][0]
    # h1.grad holds both terms: 2*h1 from the square and the rows of W2 summed from the Linear
    assert np.abs(h1g).max() > 0
    for a, c in zip(*res):
        assert np.array_equal(a, c)


def test_failed_backward_leaves_no_tape_behind(device):
    from sliced_amd import host
    a, b = device.buffer([1, 2, 3]), device.buffer([4, 5, 6])
    out = device.mul(a, b)
    device.release(a)                        # the closure on the tape now names a buffer that is gone
    with pytest.raises(host.HostError):
        out.backward()
    assert device.tape_len() == 0
    c, d = device.buffer([1, 2, 3]), device.buffer([4, 5, 6])
    out2 = device.mul(c, d)
    out2.backward()                          # must not replay the stale closure
    eq(c.grad(), [4, 5, 6])
    eq(d.grad(), [1, 2, 3])


def test_repeated_backward_with_manual_descent(device, orc):
    """tests/test_combination.rs:5-23: a hundred times square(x) -> backward -> x.grad *= 0.1 ->
    x -= x.grad -> clear the gradient.  Every step against the oracle's unary op and gradient, bit
    for bit; the sum of squares falls by 0.8^2 a step."""
    xv = np.array([10, -10, 10, -5, 6, 3, 1], np.float32)
    x = device.buffer(xv)
    ref = xv.copy()
    sums = []
    for i in range(100):
        squared = device.square(x)
        sq_ref = orc.unary(orc.SQUARE, ref)
        assert np.array_equal(squared.read(), sq_ref), i
        sums.append(float(sq_ref.sum()))
        squared.backward()
        g_ref = orc.unary_grad(orc.SQUARE, ref, np.zeros_like(ref), np.ones_like(ref))
        assert np.array_equal(x.grad().read(), g_ref), i
        device.sgd_step(x, 0.1)                  # x -= x.grad * 0.1: the two assign loops of the test
        ref = orc.sgd_step(ref, g_ref, 0.1)
        assert np.array_equal(x.read(), ref), i
        device.zero_grad()                       # x_grad.clear()
        eq(x.grad(), np.zeros(7))
        assert device.tape_len() == 0
    assert all(b < a for a, b in zip(sums, sums[1:]))
    assert abs(sums[-1] / sums[0] - 0.64 ** 99) < 1e-5 * 0.64 ** 99 * 100


def test_repeated_backward_with_manual_descent_through_pow(device, orc):
    """tests/matrix/min_fn.rs:3-23: the same loop with `x.pow(2.)` in place of `square`; powf is not
    pinned to the last ulp between libm and the device (1e-6 relative per step), the descent is."""
    xv = np.array([10, -10, 10, -5, 6, 3, 1], np.float32)
    x = device.buffer(xv)
    ref = xv.copy()
    first = last = None
    for i in range(100):
        p2 = device.pow(x, 2.0)
        want = orc.unary(orc.POW, ref, 2.0)
        got = p2.read()
        assert np.all(np.abs(got - want) <= 1e-6 * np.abs(want) + 1e-37), i
        first = float(want.sum()) if first is None else first
        last = float(want.sum())
        p2.backward()
        g_ref = orc.unary_grad(orc.POW, ref, np.zeros_like(ref), np.ones_like(ref), 2.0)
        g = x.grad().read()
        assert np.all(np.abs(g - g_ref) <= 1e-6 * np.abs(g_ref) + 1e-37), i
        device.sgd_step(x, 0.1)
        ref = orc.sgd_step(ref, g_ref, 0.1)
        assert np.all(np.abs(x.read() - ref) <= 2e-6 * np.abs(ref) + 1e-37), i
        # the next step starts from the device's own x on both sides, so roundings do not pile up
        ref = x.read().copy()
        device.zero_grad()
    assert last < first * 1e-15


def test_matrix_rand_fills_from_the_seeded_stream(device):
    """Matrix::rand(lo, hi) (src/matrix.rs:266-271): in range, and the very numbers the host-side
    generator gives for the same seed and tag."""
    from sliced_amd import host
    rows, cols = 37, 53
    b = device.zeros(rows * cols)
    device.matrix_rand(b, rows, cols, -0.25, 0.75, tag=5)
    got = b.read()
    assert got.min() >= -0.25 and got.max() < 0.75 and len(np.unique(got)) > rows * cols // 2
    assert np.array_equal(got, rng.uniform(rows * cols, -0.25, 0.75, tag=5))
    with pytest.raises(host.HostError):
        device.matrix_rand(b, rows, cols + 1, 0.0, 1.0)   # the view's length assert (src/matrix/impl_from.rs:7-10)


# --------------------------------------------------------------------------- training loops
def loss_parity(got, ref, tol):
    rel = np.abs(got - ref) / np.maximum(np.abs(ref), 1e-30)
    return rel.max()


def test_whole_step_kernels_train_the_sine_fit_like_the_oracle(orc):
    """Config 1 with every step as two launches (slhip_mlp3_mse_step): per-step loss within 1e-4
    relative of the oracle's loop over all 200 steps, the trained parameters beside the oracle's, and
    a second run bit-identical to the first."""
    from sliced_amd import host
    cfg = host.C1
    x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    p_ref = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    runs = []
    for _ in range(2):
        p_gpu = [a.copy() for a in p_ref]
        got, _ = host.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_gpu, cfg["lr"],
                                cfg["steps"], 0, True, whole_step=True)
        runs.append((got, p_gpu))
    ref = orc.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_ref, cfg["lr"], cfg["steps"])
    got, p_gpu = runs[0]
    worst = loss_parity(got, ref, 1e-4)
    say("C1 whole-step worst relative loss deviation", worst, "loss", ref[0], "->", ref[-1], "gpu", got[0], "->", got[-1])
    assert worst <= 1e-4
    for a, b in zip(p_gpu, p_ref):
        assert np.max(np.abs(a - b)) <= 1e-4 * max(1.0, np.max(np.abs(b)))
    assert np.array_equal(runs[0][0], runs[1][0])
    for a, b in zip(runs[0][1], runs[1][1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("dims", [(1024, 1, 64, 1), (37, 3, 50, 2), (1, 8, 64, 8), (4099, 2, 7, 3), (256, 1, 1, 1), (9, 5, 33, 1)],
                         ids=lambda d: "-".join(map(str, d)))
def test_whole_step_against_the_oracles_step(hip, orc, dims):
    """One and three steps of slhip_mlp3_mse_step on odd sizes (fewer hidden units than lanes, several
    inputs and outputs, batches that are no multiple of 4 or 8) against the oracle's training loop:
    the loss, the updated parameters, and the gradients as (old - new) / lr says they must be."""
    batch, d_in, d_h, d_out = dims
    x = rng.uniform(batch * d_in, -2, 2, tag=0)
    t = rng.uniform(batch * d_out, -1, 1, tag=1)
    shapes = [d_in * d_h, d_h, d_h * d_h, d_h, d_h * d_out, d_out]
    p0 = [rng.uniform(n, -0.25, 0.25, tag=10 + i) for i, n in enumerate(shapes)]
    lr = 0.02
    p_ref = [a.copy() for a in p0]
    ref_losses = orc.mlp_train(0, batch, d_in, d_h, d_out, x, t, p_ref, lr, 3)
    p_gpu = [a.copy() for a in p0]
    for step in range(3):
        before = [a.copy() for a in p_gpu]
        loss, grads = hip.mlp3_mse_step(batch, d_in, d_h, d_out, x, t, p_gpu, lr)
        # (the first step sees identical parameters; later ones the two sides' own, a rounding apart)
        assert abs(loss - ref_losses[step]) <= (2e-6 if step == 0 else 1e-5) * abs(ref_losses[step]) + 1e-30, (step, loss, ref_losses[step])
        for b, a, g in zip(before, p_gpu, grads):
            assert np.array_equal(a, b - g * np.float32(lr))       # value -= grad * lr, the gradient handed out
    for a, b, n in zip(p_gpu, p_ref, ("W1", "b1", "W2", "b2", "W3", "b3")):
        assert np.max(np.abs(a - b)) <= 5e-6 * max(1.0, np.max(np.abs(b))), n
    # without gradient buffers: the same parameters
    p_again = [a.copy() for a in p0]
    for step in range(3):
        hip.mlp3_mse_step(batch, d_in, d_h, d_out, x, t, p_again, lr, with_grads=False)
    for a, b in zip(p_again, p_gpu):
        assert np.array_equal(a, b)


def test_whole_step_refuses_layers_it_does_not_serve(hip):
    c = hip.ctx()
    z = c.zeros(1 << 16)
    args = lambda d_in, d_h, d_out: (4, d_in, d_h, d_out, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, None, 0.1, z.ptr)
    assert c.lib.slhip_mlp3_mse_step(c.h, *args(1, 65, 1)) == -1
    assert b"64 hidden units" in c.lib.slhip_last_error_string()
    assert c.lib.slhip_mlp3_mse_step(c.h, *args(9, 64, 1)) == -1
    assert c.lib.slhip_mlp3_mse_step(c.h, *args(1, 64, 9)) == -1
    assert c.lib.slhip_mlp3_mse_step(c.h, 0, 1, 64, 1, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, z.ptr, None, 0.1, z.ptr) == -1
    z.free()


@pytest.mark.parametrize("fused", [False, True], ids=["op-by-op", "fused-linear"])
def test_sine_mlp_loss_curve_matches_oracle(orc, fused):
    """Config 1: batch 1024, 1-64-64-1, MSE, SGD lr 0.01, 200 steps; per-step loss within 1e-4 rel."""
    from sliced_amd import host
    cfg = host.C1
    say("C1", "fused" if fused else "unfused")
    x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    p_ref = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    p_gpu = [a.copy() for a in p_ref]
    ref = orc.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_ref, cfg["lr"],
                        cfg["steps"])
    got, _ = host.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_gpu, cfg["lr"],
                            cfg["steps"], 0, fused)
    assert ref[-1] < ref[0]                       # it trains
    worst = loss_parity(got, ref, 1e-4)
    say("C1 worst relative loss deviation", worst, "loss", ref[0], "->", ref[-1])
    assert worst <= 1e-4
    for a, b in zip(p_gpu, p_ref):
        assert np.max(np.abs(a - b)) <= 1e-4 * max(1.0, np.max(np.abs(b)))


@pytest.mark.parametrize("fused", [False, True], ids=["op-by-op", "fused-linear"])
def test_classifier_mlp_loss_curve_matches_oracle(orc, fused):
    """Config 5: batch 8192, 784-2048-2048-10, softmax cross-entropy, SGD lr 0.05, 50 steps."""
    from sliced_amd import host
    cfg = host.C5
    say("C5", "fused" if fused else "unfused")
    x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    p_ref = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    p_gpu = [a.copy() for a in p_ref]
    global _C5_REF
    try:
        ref = _C5_REF
    except NameError:
        ref = _C5_REF = orc.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_ref,
                                      cfg["lr"], cfg["steps"])
    got, _ = host.mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, p_gpu, cfg["lr"],
                            cfg["steps"], 0, fused)
    worst = loss_parity(got, ref, 1e-4)
    say("C5 worst relative loss deviation", worst, "loss", ref[0], "->", ref[-1])
    assert np.all(np.isfinite(got))
    assert worst <= 1e-4


@pytest.mark.parametrize("name,steps", [("C1", 200), ("C5", 12)])
def test_recorded_step_replays_match_the_eager_loop(orc, name, steps):
    """One training step recorded as a graph and replayed: the loss curve and the trained
    parameters are bit-identical to the eager loop (same kernels in the same order), which the
    tests above hold to the oracle; C1 is compared with the oracle here as well."""
    from sliced_amd import host
    cfg = host.C1 if name == "C1" else host.C5
    say(name, "recorded step,", steps, "steps")
    x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    p0 = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    args = (cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t)
    p_eager = [a.copy() for a in p0]
    eager, _ = host.mlp_train(*args, p_eager, cfg["lr"], steps, 0, True)
    for warmup in (0, 3):     # the recording happens inside / before the timed steps
        p_graph = [a.copy() for a in p0]
        info = {}
        got, _ = host.mlp_train(*args, p_graph, cfg["lr"], steps - warmup, warmup, True, graph=True, info=info)
        say(name, "kernels per recorded step:", info["graph_nodes"])
        assert info["graph_nodes"] > 10
        assert np.array_equal(got, eager[warmup:])
        for a, b in zip(p_graph, p_eager):
            assert np.array_equal(a, b)
    if name == "C1":
        p_ref = [a.copy() for a in p0]
        ref = orc.mlp_train(*args, p_ref, cfg["lr"], steps)
        assert loss_parity(eager, ref, 1e-4) <= 1e-4


@pytest.mark.parametrize("name,steps", [("C1", 200), ("C5", 50)])
def test_fused_loss_training_matches_oracle_and_its_own_replay(orc, name, steps):
    """Fused Linear + fused loss kernels: per-step loss within 1e-4 of the oracle's op-by-op loop;
    the replayed recording bit-identical to the eager run of the same kernels."""
    from sliced_amd import host
    cfg = host.C1 if name == "C1" else host.C5
    say(name, "fused loss,", steps, "steps")
    x, t = host.mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    p0 = host.mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    args = (cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t)
    global _C5_REF
    if name == "C5" and "_C5_REF" in globals():
        ref = _C5_REF
    else:
        ref = orc.mlp_train(*args, [a.copy() for a in p0], cfg["lr"], steps)
        if name == "C5":
            _C5_REF = ref
    p_eager = [a.copy() for a in p0]
    eager, _ = host.mlp_train(*args, p_eager, cfg["lr"], steps, 0, True, fused_loss=True)
    worst = loss_parity(eager, ref, 1e-4)
    say(name, "fused loss: worst relative loss deviation", worst)
    assert np.all(np.isfinite(eager)) and worst <= 1e-4
    p_graph = [a.copy() for a in p0]
    info = {}
    got, _ = host.mlp_train(*args, p_graph, cfg["lr"], steps, 0, True, graph=True, info=info, fused_loss=True)
    say(name, "kernels per recorded step:", info["graph_nodes"])
    assert np.array_equal(got, eager)
    for a, b in zip(p_graph, p_eager):
        assert np.array_equal(a, b)
