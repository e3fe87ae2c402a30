"""Elementwise chains as one launch: the program kernels through the C ABI against the same ops
run one by one (bit for bit) and against the CPU oracle, and the host tape with elementwise fusion
switched on against the same tape with it off: values, leaf gradients, number of kernels in a
recording, and the cases where a fused-away intermediate is needed after all.

Reference shapes: examples/chained_perf.rs:86-91 (square, add, mul, mul, add -> 9.336999) and the
blanket wrappers src/ops.rs:20-187 that put each of these ops on the tape."""
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu
SEED = rng.DEFAULT_SEED
ADD, SUB, MUL, DIV = 0, 1, 2, 3
SQUARE, POW, RELU, EXP, CLIP, NEG_LN, SCALE, NEG_DIV, TANH, SIGMOID = range(10)
U, NOGRAD = 0x10, 0x1


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_one_by_one(hip, inputs, prog):
    """The program evaluated with one slhip_ew_binary / slhip_ew_unary call per instruction."""
    regs = {j: np.asarray(x, np.float32) for j, x in enumerate(inputs)}
    for i, ins in enumerate(prog):
        op, s0, s1, flags, p, q = tuple(ins) + (0,) * (6 - len(ins))
        if op & U:
            regs[4 + i] = hip.unary(op & 0xF, regs[s0], p, q)
        else:
            regs[4 + i] = hip.binary_ew(op, regs[s0], regs[s1])
    return regs


def grads_one_by_one(hip, inputs, grads0, prog, out_grad):
    """Gradients through one slhip_ew_*_grad call per instruction, last instruction first; the
    intermediates' gradients start from zero, the inputs' from grads0."""
    regs = run_one_by_one(hip, inputs, prog)
    adj = {k: np.zeros_like(v) for k, v in regs.items()}
    for j, g in enumerate(grads0):
        adj[j] = np.array(g, np.float32, copy=True)
    adj[4 + len(prog) - 1] = np.asarray(out_grad, np.float32)
    for i in reversed(range(len(prog))):
        op, s0, s1, flags, p, q = tuple(prog[i]) + (0,) * (6 - len(prog[i]))
        if flags & NOGRAD:
            continue
        g = adj[4 + i]
        if op & U:
            adj[s0] = hip.unary_grad(op & 0xF, regs[s0], adj[s0], g, p)
        elif s0 == s1:
            adj[s0], _ = hip.binary_ew_grad(op, regs[s0], regs[s1], adj[s0], None, g)
            _, adj[s0] = hip.binary_ew_grad(op, regs[s0], regs[s1], None, adj[s0], g)
        else:
            adj[s0], adj[s1] = hip.binary_ew_grad(op, regs[s0], regs[s1], adj[s0], adj[s1], g)
    return [adj[j] for j in range(len(inputs))]


C4_CHAIN = [(ADD, 0, 1), (MUL, 4, 2), (SUB, 5, 3), (U | POW, 6, 6, 0, 2.0), (U | SQUARE, 7, 7)]
CHAINED_PERF = [(U | SQUARE, 0, 0), (ADD, 1, 0), (MUL, 5, 1), (MUL, 4, 0), (ADD, 7, 6)]      # inputs: x, b
PROGRAMS = {
    "c4 chain": (4, C4_CHAIN),
    "chained_perf": (2, CHAINED_PERF),
    "single add": (2, [(ADD, 0, 1)]),
    "single tanh": (1, [(U | TANH, 0, 0)]),
    "x*x then x+x": (1, [(MUL, 0, 0), (ADD, 4, 4)]),
    "div and sigmoid": (3, [(DIV, 0, 1), (U | SIGMOID, 4, 4), (SUB, 5, 2), (U | SCALE, 6, 6, 0, 0.25)]),
    "eight ops": (4, [(ADD, 0, 1), (MUL, 4, 2), (U | TANH, 5, 5), (SUB, 6, 3), (U | RELU, 7, 7), (MUL, 8, 4),
                      (U | POW, 9, 9, 0, 3.0), (ADD, 10, 0)]),
    "exp stops the gradient": (2, [(ADD, 0, 1), (U | EXP, 4, 4, NOGRAD), (MUL, 5, 0)]),
    "clip, no gradient": (2, [(U | CLIP, 0, 0, NOGRAD, -1.0, 2.0), (MUL, 4, 1)]),
    "sqrt and relu": (2, [(U | SQUARE, 0, 0), (U | POW, 4, 4, 0, 0.5), (U | RELU, 1, 1), (ADD, 5, 6)]),
}


@pytest.mark.parametrize("name", list(PROGRAMS))
def test_program_equals_the_ops_one_by_one(hip, orc, name):
    n_in, prog = PROGRAMS[name]
    for n in (1, 3, 4, 7, 1000, 4099, 1 << 18):
        say("program", name, n)
        scale = 2.0 if "eight" in name or "exp" in name else 10.0
        inputs = [rng.uniform(n, -scale, scale, tag=j, seed=SEED + n) for j in range(n_in)]
        want = run_one_by_one(hip, inputs, prog)[4 + len(prog) - 1]
        got = hip.ew_program(inputs, prog)
        assert np.array_equal(got, want, equal_nan=True), name
        # the gradient: input gradients that already hold something, a random upstream gradient
        g = rng.normal(n, 1.0, tag=9, seed=SEED)
        grads0 = [rng.uniform(n, -1, 1, tag=20 + j, seed=SEED) for j in range(n_in)]
        want_g = grads_one_by_one(hip, inputs, grads0, prog, g)
        got_g = hip.ew_program_grad(inputs, grads0, prog, g)
        for j in range(n_in):
            assert np.array_equal(got_g[j], want_g[j], equal_nan=True), (name, j)
    # and against the CPU restatement of the reference for the two chains of its examples
    if name == "c4 chain":
        a, b, c, d = inputs
        t = orc.binary_ew(orc.SUB, orc.binary_ew(orc.MUL, orc.binary_ew(orc.ADD, a, b), c), d)
        ref = orc.unary(orc.SQUARE, orc.unary(orc.POW, t, 2.0))
        assert np.all(np.abs(got - ref) <= 1e-6 * np.abs(ref) + 1e-37)
    if name == "chained_perf":
        x, b = np.full(123412, 1.3, np.float32), np.full(123412, 2.1, np.float32)
        out = hip.ew_program([x, b], prog)
        assert np.all(out == np.float32(9.336999))        # examples/chained_perf.rs:91


def random_program(r):
    """A well-formed program of 2..8 instructions over 1..4 inputs: any earlier value may be read any
    number of times (or never), exp and clip carry NOGRAD, now and then so does another op."""
    n_in = int(r.integers(1, 5))
    n_ops = int(r.integers(2, 9))
    prog = []
    for i in range(n_ops):
        avail = list(range(n_in)) + [4 + k for k in range(i)]
        # the newest value most of the time, so that chains form, but not always
        pick = lambda: int(avail[-1] if i and r.random() < 0.5 else avail[int(r.integers(0, len(avail)))])
        if r.random() < 0.5:
            op = int(r.integers(0, 4))
            prog.append((op, pick(), pick(), NOGRAD if r.random() < 0.1 else 0))
        else:
            op = int(r.choice([SQUARE, POW, RELU, EXP, CLIP, SCALE, TANH, SIGMOID]))
            s = pick()
            flags = NOGRAD if op in (EXP, CLIP) or r.random() < 0.1 else 0
            p, q = {POW: (3.0, 0.0), CLIP: (-0.5, 0.75), SCALE: (-1.75, 0.0)}.get(op, (0.0, 0.0))
            prog.append((U | op, s, s, flags, p, q))
    return n_in, prog


@pytest.mark.parametrize("seed", range(24))
def test_random_programs_equal_the_ops_one_by_one(hip, seed):
    """Values die, share registers and are needed again on the way back in every pattern a random
    program produces: result and every input gradient bit for bit the ops run one by one."""
    r = np.random.default_rng(1000 + seed)
    n_in, prog = random_program(r)
    n = 4099
    say("random program", seed, n_in, prog)
    inputs = [rng.uniform(n, -1.5, 1.5, tag=j, seed=SEED + seed) for j in range(n_in)]
    want = run_one_by_one(hip, inputs, prog)[4 + len(prog) - 1]
    assert np.array_equal(hip.ew_program(inputs, prog), want, equal_nan=True)
    g = rng.normal(n, 1.0, tag=9, seed=SEED)
    grads0 = [rng.uniform(n, -1, 1, tag=20 + j, seed=SEED) for j in range(n_in)]
    want_g = grads_one_by_one(hip, inputs, grads0, prog, g)
    got_g = hip.ew_program_grad(inputs, grads0, prog, g)
    for j in range(n_in):
        assert np.array_equal(got_g[j], want_g[j], equal_nan=True), j


def test_program_skips_null_gradients_and_validates(hip):
    n = 1000
    a, b = rng.uniform(n, -1, 1, tag=0), rng.uniform(n, -1, 1, tag=1)
    g = rng.uniform(n, -1, 1, tag=2)
    only_b = hip.ew_program_grad([a, b], [None, np.zeros(n, np.float32)], [(MUL, 0, 1)], g)
    assert only_b[0] is None and np.array_equal(only_b[1], a * g)
    import ctypes as C
    c = hip.ctx()
    da, out = c.array(a), c.empty(n)
    ptrs = (C.c_void_p * 1)(da.ptr)
    bad_src = hip.ew_insn([(ADD, 0, 5)])                 # reads a register at or above its own
    bad_op = hip.ew_insn([(U | 11, 0, 0)])
    no_grad = hip.ew_insn([(U | CLIP, 0, 0, 0, 0.0, 1.0)])
    nine = hip.ew_insn([(U | SQUARE, 0, 0)] * 9)
    call = lambda code, k: c.lib.slhip_ew_program(c.h, n, 1, C.cast(ptrs, C.c_void_p), k, code.ctypes.data, out.ptr)
    assert call(bad_src, 1) == -1 and call(bad_op, 1) == -1 and call(nine, 9) == -1
    assert call(hip.ew_insn([(U | SQUARE, 0, 0)]), 0) == -1
    gp = (C.c_void_p * 1)(out.ptr)
    rc = c.lib.slhip_ew_program_grad(c.h, n, 1, C.cast(ptrs, C.c_void_p), C.cast(gp, C.c_void_p), 1, no_grad.ctypes.data, da.ptr)
    assert rc == -1 and b"no gradient" in c.lib.slhip_last_error_string()
    two = (C.c_void_p * 2)(da.ptr, da.ptr)
    gg = (C.c_void_p * 2)(out.ptr, out.ptr)
    code = hip.ew_insn([(ADD, 0, 1)])
    assert c.lib.slhip_ew_program_grad(c.h, n, 2, C.cast(two, C.c_void_p), C.cast(gg, C.c_void_p), 1, code.ctypes.data, da.ptr) == -4
    da.free()
    out.free()


# ------------------------------------------------------------------------------ the host tape
@pytest.fixture()
def device():
    from sliced_amd import host
    d = host.HIP(0, cached=False)
    yield d
    d.close()


@pytest.fixture()
def cached_device():
    """`HIP::<Autograd<Cached<Base>>>`: the second pass over an op sequence gets the first pass's buffers,
    which is what a recording needs (it must not allocate)."""
    from sliced_amd import host
    d = host.HIP(0, cached=True)
    yield d
    d.close()


def test_chained_perf_runs_as_one_kernel(cached_device):
    """examples/chained_perf.rs:54-91 with elementwise fusion on: the five ops, written one by one,
    land in a recording as ONE kernel and give the example's asserted value."""
    device = cached_device
    n = 123412
    x, b = device.buffer(np.full(n, 1.3, np.float32)), device.buffer(np.full(n, 2.1, np.float32))
    device.set_fuse_elementwise(True)
    device.enable_tape(False)
    for epoch in range(2):                       # `for epoch in device.range(..)`: pass 0 fills the cache
        device.begin_iteration()
        if epoch == 1:
            device.record_begin()
        squared = device.square(x)
        add = device.add(b, x)
        mul_b = device.mul(add, b)
        mul = device.mul(squared, x)
        out = device.add(mul, mul_b)
        assert device.deferred() == 5
        if epoch == 1:
            nodes = device.record_end()
        else:
            device.run()
    assert nodes == 1
    got = out.read()
    assert got[0] == np.float32(9.336999) and np.all(got == got[0])
    # the same through Matrix methods (the cache hands out the same five buffers again)
    device.enable_tape(True)
    device.begin_iteration()
    out2 = device.matrix_chain(1, 1, n, x, b)
    assert np.array_equal(out2.read(), got)
    # and its gradients against the op-by-op tape
    out2.backward()
    gx, gb = x.grad().read(), b.grad().read()
    device.set_fuse_elementwise(False)
    x2, b2 = device.buffer(np.full(n, 1.3, np.float32)), device.buffer(np.full(n, 2.1, np.float32))
    device.matrix_chain(1, 1, n, x2, b2).backward()
    assert np.array_equal(gx, x2.grad().read()) and np.array_equal(gb, b2.grad().read())
    assert abs(gx[0] - (3 * 1.3 ** 2 + 2.1)) < 1e-5 and abs(gb[0] - (1.3 + 2 * 2.1)) < 1e-5


def test_c4_chain_through_matrix_ops_is_bit_identical_and_one_kernel(orc):
    from sliced_amd import host
    n = (1 << 20) + 3
    vals = [rng.uniform(n, -10, 10, tag=1 + j, seed=SEED) for j in range(4)]
    res = {}
    for fuse in (False, True):
        device = host.HIP(0, cached=True)
        device.set_fuse_elementwise(fuse)
        bufs = [device.buffer(v) for v in vals]
        device.enable_tape(False)
        device.begin_iteration()
        device.matrix_chain(0, 1, n, *bufs)      # pass 0 fills the cache
        device.run()
        device.begin_iteration()
        device.record_begin()
        device.matrix_chain(0, 1, n, *bufs)
        nodes = device.record_end()
        device.enable_tape(True)
        device.begin_iteration()
        out = device.matrix_chain(0, 1, n, *bufs)
        out.backward()
        res[fuse] = (out.read(), [b.grad().read() for b in bufs], nodes)
        device.close()
    assert res[False][2] == 5 and res[True][2] == 1
    assert np.array_equal(res[True][0], res[False][0])
    for a, b in zip(res[True][1], res[False][1]):
        assert np.array_equal(a, b)
    a, b, c, d = vals
    t = orc.binary_ew(orc.SUB, orc.binary_ew(orc.MUL, orc.binary_ew(orc.ADD, a, b), c), d)
    ref = orc.unary(orc.SQUARE, orc.unary(orc.POW, t, 2.0))
    assert np.all(np.abs(res[True][0] - ref) <= 1e-6 * np.abs(ref) + 1e-37)
    # d out / d d = -4 t^3
    assert np.allclose(res[True][1][3], -4.0 * t.astype(np.float64) ** 3, rtol=1e-5)


def test_fused_tape_equals_the_eager_tape_on_assorted_graphs(device):
    """Chains longer than a program, more inputs than a program takes, a result with two readers, ops
    that are not elementwise in the middle, self products: values and every leaf gradient bit for bit."""
    n = 5000
    v = [rng.uniform(n, -1.5, 1.5, tag=j, seed=SEED) for j in range(7)]

    def graph(dev, leaf):
        t = dev.add(leaf[0], leaf[1])
        for k in range(11):                                   # 12 ops in a row over few inputs
            t = dev.mul(t, leaf[k % 3]) if k % 2 else dev.tanh(t)
        w = dev.add(dev.add(dev.add(dev.add(dev.add(leaf[0], leaf[1]), leaf[2]), leaf[3]), leaf[4]), leaf[5])  # 6 inputs
        shared = dev.sub(t, w)                                # two readers below
        p = dev.square(shared)
        q = dev.mul(shared, leaf[6])
        r = dev.add(p, q)
        s = dev.sum_cols(50, r)                               # not elementwise: ends the chain
        s2 = dev.mul(s, s)                                    # a self product after it
        return dev.sum_cols(100, s2), [t, w, shared, p, q, r, s, s2]

    res = {}
    for fuse in (False, True):
        device.set_fuse_elementwise(fuse)
        leaf = [device.buffer(x) for x in v]
        out, mids = graph(device, leaf)
        out.backward()
        res[fuse] = ([out.read()] + [m.read() for m in mids], [l.grad().read() for l in leaf])
    for a, b in zip(res[True][0], res[False][0]):
        assert np.array_equal(a, b)
    for a, b in zip(res[True][1], res[False][1]):
        assert np.array_equal(a, b)


def test_intermediate_needed_after_its_chain_ran(device):
    """t = a + b feeds only u = t * c, so the chain keeps t in registers.  Reading t afterwards computes
    it; a later op that reads t gets its value, and the gradient that op leaves for t flows on to a
    and b although t's own gradient step had been folded into the chain."""
    from sliced_amd import host
    n = 777
    av, bv, cv, dv = (rng.uniform(n, -2, 2, tag=j, seed=SEED) for j in range(4))
    res = {}
    for fuse in (False, True):
        device.set_fuse_elementwise(fuse)
        a, b, c, d = (device.buffer(x) for x in (av, bv, cv, dv))
        t = device.add(a, b)
        u = device.mul(t, c)
        y1 = device.sum_cols(n, u)               # flushes: with fusion on, t never reaches memory
        if fuse:
            assert np.array_equal(t.read(), av + bv)   # computed on demand
        z = device.mul(t, d)                     # a second reader of t, after the fact
        y2 = device.sum_cols(n, z)
        tot = device.add(y1, y2)
        tot.backward()
        res[fuse] = [x.grad().read() for x in (a, b, c, d)] + [t.grad().read()]
    for got, want in zip(res[True], res[False]):
        assert np.array_equal(got, want)
    assert np.array_equal(res[True][0], cv + dv)
    # a fused-away intermediate that nothing else reads has no gradient buffer
    device.set_fuse_elementwise(True)
    a, b, c = (device.buffer(x) for x in (av, bv, cv))
    t = device.add(a, b)
    u = device.mul(t, c)
    u.backward()
    assert np.array_equal(a.grad().read(), cv)
    with pytest.raises(host.HostError):
        t.grad()
    device.set_fuse_elementwise(False)


@pytest.mark.parametrize("root", ["exp", "clip", "tape off at the root"])
def test_chain_under_a_root_without_gradient_keeps_the_intermediates_gradient_steps(device, root):
    """t = a * b feeds u = exp(t) (or clip, or an op issued with the tape off): u carries no gradient,
    so the fused chain has no closure of its own.  A later reader of t (a product with W) leaves a
    gradient for t, and t's own gradient step must still carry it on to a and b, as it does op by op."""
    m, k, n = 24, 16, 8
    av, bv = rng.uniform(m * k, -1, 1, tag=0, seed=SEED), rng.uniform(m * k, -1, 1, tag=1, seed=SEED)
    wv = rng.uniform(k * n, -1, 1, tag=2, seed=SEED)
    res = {}
    for fuse in (False, True):
        device.set_fuse_elementwise(fuse)
        a, b, w = (device.buffer(x) for x in (av, bv, wv))
        t = device.mul(a, b)
        if root == "exp":
            u = device.exp(t)
        elif root == "clip":
            u = device.clip(t, -0.5, 0.5)
        else:
            device.enable_tape(False)
            u = device.square(t)
            device.enable_tape(True)
        us = u.read()                            # flushes the chain: with fusion on, t stays in registers
        v = device.gemm(m, k, n, t, w)           # the later reader of t
        v.backward()
        res[fuse] = [us, v.read(), t.grad().read(), a.grad().read(), b.grad().read(), w.grad().read()]
    device.set_fuse_elementwise(False)
    for got, want in zip(res[True], res[False]):
        assert np.array_equal(got, want)
    tg = np.ones((m, n), np.float32) @ wv.reshape(k, n).T
    assert np.allclose(res[True][3].reshape(m, k), tg * bv.reshape(m, k), rtol=1e-5, atol=1e-6)
    assert np.abs(res[True][3]).max() > 0


def test_release_of_a_chains_input_computes_the_intermediates_that_read_it(device):
    """t = a + b is kept in registers by the chain t * c; releasing a afterwards must not leave t
    uncomputable: it is given its value at the release."""
    n = 300
    av, bv, cv = (rng.uniform(n, -2, 2, tag=j, seed=SEED) for j in range(3))
    device.set_fuse_elementwise(True)
    a, b, c = (device.buffer(x) for x in (av, bv, cv))
    t = device.add(a, b)
    u = device.mul(t, c)
    assert np.array_equal(u.read(), (av + bv) * cv)
    device.release(a)
    junk = device.buffer(np.full(n, 99.0, np.float32))   # may take a's memory
    assert np.array_equal(t.read(), av + bv)
    assert junk.read()[0] == 99.0
    device.set_fuse_elementwise(False)


def test_fusion_in_a_cached_loop_with_inplace_updates():
    """The sine fit's loss chain (sub, square, sum, scale) in a cached loop with SGD updates in
    between: deferred ops see every update, and the cache hands the same buffers out again."""
    from sliced_amd import host
    n = 4096
    xv, yv = rng.uniform(n, -1, 1, tag=0, seed=SEED), rng.uniform(n, -1, 1, tag=1, seed=SEED)
    curves = {}
    for fuse in (False, True):
        dev = host.HIP(0, cached=True)
        dev.set_fuse_elementwise(fuse)
        w = dev.buffer(xv.copy())
        y = dev.buffer(yv).no_grad()
        losses = []
        for it in range(6):
            dev.begin_iteration()
            dev.zero_grad()
            d = dev.sub(w, y)
            q = dev.square(d)
            s = dev.sum_cols(n, q)
            loss = dev._un(host.SCALE, s, 1.0 / n)
            loss.backward()
            losses.append(loss.read()[0])
            dev.sgd_step(w, 0.1)
        curves[fuse] = (np.array(losses), w.read())
        dev.close()
    assert np.array_equal(curves[True][0], curves[False][0])
    assert np.array_equal(curves[True][1], curves[False][1])
    assert curves[True][0][-1] < curves[True][0][0]
