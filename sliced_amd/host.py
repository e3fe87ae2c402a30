"""Python handles onto the C++ host device layer (libsliced_host.so): a `HIP` device with the
reference's op names, `Buffer`s with `.backward()` / `.grad()`, and the two training loops.

The classes only forward to C++; the tape, the gradient map, the call-position cache and every
kernel launch live in the native libraries.  A test written against this module reads like the
reference's own integration tests (tests/test_gemm.rs etc.):

    device = HIP()
    lhs = device.buffer([1, 2, 3, 4, 4, 5, 6, 5]); rhs = device.buffer([1, 2, 3, 4, 5, 6])
    out = device.gemm(4, 2, 3, lhs, rhs)
    out.backward()
    lhs.grad().read()
"""
import ctypes as C
import os

import numpy as np

from . import _lib, rng

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsliced_host.so")

ADD, SUB, MUL, DIV = 0, 1, 2, 3
SQUARE, POW, RELU, EXP, CLIP, NEG_LN, SCALE, NEG_DIV, TANH, SIGMOID = range(10)
SUM_ROWS, SUM_COLS, MAX_ROWS, MAX_COLS, MEAN_ROWS, MEAN_COLS = range(6)

_h = None


class HostError(RuntimeError):
    pass


def lib():
    global _h
    if _h is None:
        _lib.load()  # libsliced_hip.so first: the host library links against it
        if not os.path.exists(LIB_PATH):
            raise HostError("%s not found: build it first (python -m sliced_amd.build)" % LIB_PATH)
        _h = C.CDLL(LIB_PATH)
        _h.slh_last_error.restype = C.c_char_p
        _h.slh_tape_len.restype = C.c_size_t
        _h.slh_deferred.restype = C.c_size_t
    return _h


def _ck(rc):
    if rc != 0:
        raise HostError(lib().slh_last_error().decode())


_u64, _sz, _f = C.c_uint64, C.c_size_t, C.c_float


class Buffer:
    def __init__(self, dev, bid):
        self.dev, self.id = dev, bid

    def __len__(self):
        n = _sz()
        _ck(lib().slh_buffer_len(self.dev.h, _u64(self.id), C.byref(n)))
        return n.value

    def read(self):
        out = np.empty(len(self), np.float32)
        _ck(lib().slh_buffer_read(self.dev.h, _u64(self.id), out.ctypes.data_as(C.POINTER(_f))))
        return out

    def require_grad(self):
        _ck(lib().slh_require_grad(self.dev.h, _u64(self.id), 1))
        return self

    def no_grad(self):
        _ck(lib().slh_require_grad(self.dev.h, _u64(self.id), 0))
        return self

    def grad(self):
        g = _u64()
        _ck(lib().slh_grad(self.dev.h, _u64(self.id), C.byref(g)))
        return Buffer(self.dev, g.value)

    def has_grad(self):
        return bool(lib().slh_has_grad(self.dev.h, _u64(self.id)))

    def backward(self):
        _ck(lib().slh_backward(self.dev.h, _u64(self.id)))

    def backward_with(self, seed):
        _ck(lib().slh_backward_with(self.dev.h, _u64(self.id), _u64(seed.id)))


class HIP:
    """`HIP::<Autograd<Cached<Base>>>` (cached=True) or `HIP::<Autograd<Base>>`."""

    def __init__(self, ordinal=0, cached=False):
        self.h = C.c_void_p()
        _ck(lib().slh_device_new(ordinal, int(cached), C.byref(self.h)))

    def close(self):
        if self.h:
            lib().slh_device_free(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def _out(self, fn, *args):
        o = _u64()
        _ck(fn(self.h, *args, C.byref(o)))
        return Buffer(self, o.value)

    def set_grad_policy(self, gemm_beta=0.0, softmax_beta=0.0, transpose_beta=0.0):
        _ck(lib().slh_set_grad_policy(self.h, _f(gemm_beta), _f(softmax_beta), _f(transpose_beta)))

    def set_relu_bits(self, on):
        """With set_fuse_relu_grad: large fused Linear + ReLU layers keep their ReLU mask as bits."""
        _ck(lib().slh_set_relu_bits(self.h, C.c_int(1 if on else 0)))

    def set_fuse_relu_grad(self, on):
        """Fused Linear layers write their input gradient through the previous layer's ReLU gradient."""
        _ck(lib().slh_set_fuse_relu_grad(self.h, C.c_int(1 if on else 0)))

    def set_fuse_elementwise(self, on):
        """Elementwise ops are deferred; chains whose intermediates nothing else reads run as one kernel."""
        _ck(lib().slh_set_fuse_elementwise(self.h, C.c_int(1 if on else 0)))

    def run(self):
        """Launches whatever is deferred (the lazy device's `run()`)."""
        _ck(lib().slh_run(self.h))

    def deferred(self):
        return lib().slh_deferred(self.h)

    def enable_tape(self, on):
        _ck(lib().slh_enable_tape(self.h, C.c_int(1 if on else 0)))

    def ctx_handle(self):
        """The slhip context this device issues its ops on (for event timing on the same stream)."""
        p = C.c_void_p()
        _ck(lib().slh_device_ctx(self.h, C.byref(p)))
        return p

    def record_begin(self):
        _ck(lib().slh_record_begin(self.h))

    def record_end(self):
        """Ends the recording, runs it once, returns its number of kernel nodes."""
        n = _sz()
        _ck(lib().slh_record_end(self.h, C.byref(n)))
        return n.value

    def matrix_chain(self, which, rows, cols, a, b, c=None, d=None):
        """which 0: ((a+b)*c-d).pow(2).squared(); which 1: square(x)*x + (b+x)*b with x = a - written against Matrix."""
        c, d = c or a, d or a
        return self._out(lib().slh_matrix_chain, int(which), _sz(rows), _sz(cols), _u64(a.id), _u64(b.id), _u64(c.id), _u64(d.id))

    def matrix_rand(self, buf, rows, cols, lo, hi, seed=rng.DEFAULT_SEED, tag=0):
        """Matrix::rand(lo, hi) on a rows x cols view of buf (src/matrix.rs:266-271), seeded."""
        _ck(lib().slh_matrix_rand(self.h, _u64(buf.id), _sz(rows), _sz(cols), _f(lo), _f(hi), _u64(seed), _u64(tag)))

    def buffer(self, data):
        a = np.ascontiguousarray(data, dtype=np.float32).ravel()
        return self._out(lib().slh_buffer_from, a.ctypes.data_as(C.POINTER(_f)), _sz(a.size))

    def zeros(self, n):
        return self._out(lib().slh_buffer_zeros, _sz(n))

    def release(self, buf):
        """Frees a buffer and its gradient; closures on the tape that still name it will throw."""
        _ck(lib().slh_buffer_release(self.h, _u64(buf.id)))

    def begin_iteration(self):
        _ck(lib().slh_begin_iteration(self.h))

    def zero_grad(self):
        _ck(lib().slh_zero_grad(self.h))

    def tape_len(self):
        return lib().slh_tape_len(self.h)

    # ---- the op traits ------------------------------------------------------------------------
    def gemm(self, m, k, n, lhs, rhs):
        return self._out(lib().slh_gemm, _sz(m), _sz(k), _sz(n), _u64(lhs.id), _u64(rhs.id))

    def linear(self, m, k, n, x, w, bias, relu):
        return self._out(lib().slh_linear, _sz(m), _sz(k), _sz(n), _u64(x.id), _u64(w.id), _u64(bias.id), int(relu))

    def add_row(self, rows, cols, lhs, rhs):
        return self._out(lib().slh_add_row, _sz(rows), _sz(cols), _u64(lhs.id), _u64(rhs.id))

    def add_row_mut(self, rows, cols, lhs, rhs):
        _ck(lib().slh_add_row_mut(self.h, _sz(rows), _sz(cols), _u64(lhs.id), _u64(rhs.id)))

    def _bin(self, op, l, r):
        return self._out(lib().slh_binary, int(op), _u64(l.id), _u64(r.id))

    def add(self, l, r):
        return self._bin(ADD, l, r)

    def sub(self, l, r):
        return self._bin(SUB, l, r)

    def mul(self, l, r):
        return self._bin(MUL, l, r)

    def _un(self, op, x, p=0.0, q=0.0, with_grad=True):
        return self._out(lib().slh_unary, int(op), _f(p), _f(q), _u64(x.id), int(with_grad))

    def square(self, x):
        return self._un(SQUARE, x)

    def pow(self, x, rhs):
        return self._un(POW, x, rhs)

    def relu(self, x):
        return self._un(RELU, x)

    def tanh(self, x):
        return self._un(TANH, x)

    def sigmoid(self, x):
        return self._un(SIGMOID, x)

    def exp(self, x):
        return self._un(EXP, x, with_grad=False)

    def clip(self, x, lo, hi):
        return self._un(CLIP, x, lo, hi, with_grad=False)

    def row_op(self, op, rows, cols, lhs, rhs):
        return self._out(lib().slh_bcast_op, 0, int(op), _sz(rows), _sz(cols), _u64(lhs.id), _u64(rhs.id))

    def col_op(self, op, rows, cols, lhs, rhs):
        return self._out(lib().slh_bcast_op, 1, int(op), _sz(rows), _sz(cols), _u64(lhs.id), _u64(rhs.id))

    def sub_cols(self, rows, cols, lhs, rhs):
        return self.col_op(SUB, rows, cols, lhs, rhs)

    def div_cols(self, rows, cols, lhs, rhs):
        return self.col_op(DIV, rows, cols, lhs, rhs)

    def diagflat(self, x):
        return self._out(lib().slh_diagflat, _u64(x.id))

    def onehot(self, classes, cls):
        return self._out(lib().slh_onehot, _sz(classes), _u64(cls.id))

    def l2_norm_cols(self, rows, cols, x):
        """Matrix::l2_norm_cols (src/matrix.rs:337-355): squared().sum_cols().pow(1/2)."""
        return self.pow(self._red(SUM_COLS, cols, self.square(x), rows), 0.5)

    def mse_loss(self, x, y):
        return self._out(lib().slh_mse_loss, _u64(x.id), _u64(y.id))

    def softmax_cce_loss(self, rows, cols, logits, targets):
        return self._out(lib().slh_softmax_cce_loss, _sz(rows), _sz(cols), _u64(logits.id), _u64(targets.id))

    def transpose(self, rows, cols, x):
        return self._out(lib().slh_transpose, _sz(rows), _sz(cols), _u64(x.id))

    def softmax(self, samples, features, x):
        return self._out(lib().slh_softmax, _sz(samples), _sz(features), _u64(x.id))

    def _red(self, kind, cols, x, rows=None):
        rows = len(x) // cols if rows is None else rows
        return self._out(lib().slh_reduce, int(kind), _sz(rows), _sz(cols), _u64(x.id))

    def sum_rows(self, cols, x):
        return self._red(SUM_ROWS, cols, x)

    def sum_cols(self, cols, x):
        return self._red(SUM_COLS, cols, x)

    def max_rows(self, cols, x):
        return self._red(MAX_ROWS, cols, x)

    def max_cols(self, rows, cols, x):
        return self._red(MAX_COLS, cols, x, rows)

    def mean_rows(self, cols, x):
        return self._red(MEAN_ROWS, cols, x)

    def mean_cols(self, cols, x):
        return self._red(MEAN_COLS, cols, x)

    def mean(self, x):
        v = _f()
        _ck(lib().slh_mean(self.h, _u64(x.id), C.byref(v)))
        return np.float32(v.value)

    def sgd_step(self, p, lr):
        _ck(lib().slh_sgd_step(self.h, _u64(p.id), _f(lr)))


# ---------------------------------------------------------------------------- training loops
def mlp_init(kind, d_in, d_h, d_out, seed=rng.DEFAULT_SEED):
    """Seeded parameters: U(+-1/sqrt(fan_in)) for the sine fit, Kaiming-uniform U(+-sqrt(6/fan_in))
    for the classifier; biases zero (the reference zero-initialises them, examples/sine_net.rs:27)."""
    dims = [(d_in, d_h), (d_h, d_h), (d_h, d_out)]
    params = []
    for i, (fi, fo) in enumerate(dims):
        bound = (1.0 / np.sqrt(fi)) if kind == 0 else np.sqrt(6.0 / fi)
        params.append(rng.uniform(fi * fo, -bound, bound, tag=10 + i, seed=seed))
        params.append(np.zeros(fo, np.float32))
    return params


def mlp_data(kind, batch, d_in, d_out, seed=rng.DEFAULT_SEED):
    if kind == 0:
        x = rng.uniform(batch * d_in, -np.pi, np.pi, tag=0, seed=seed)
        return x, np.sin(x).astype(np.float32)
    x = rng.uniform(batch * d_in, 0.0, 1.0, tag=0, seed=seed)
    labels = rng.integers(batch, d_out, tag=1, seed=seed)
    t = np.zeros((batch, d_out), np.float32)
    t[np.arange(batch), labels] = 1.0          # slice_onehot, class count fixed at d_out
    return x, t.ravel()


def mlp_train(kind, batch, d_in, d_h, d_out, x, target, params, lr, steps, warmup=0, fused=False, ordinal=0,
              graph=False, info=None, fused_loss=False, whole_step=False):
    """Runs the C++ training loop on the GPU.  params (six float32 arrays) are updated in place.
    graph=True records one step as a HIP graph and replays it (losses are read once at the end).
    whole_step=True (the MSE loop with at most 64 hidden units) runs every step as two launches.
    Returns (losses[steps], seconds for the timed steps); info, a dict, receives graph_nodes."""
    losses = np.zeros(steps, np.float32)
    secs = C.c_double()
    nodes = C.c_size_t()
    p = lambda a: a.ctypes.data_as(C.POINTER(_f))
    x = np.ascontiguousarray(x, np.float32)
    target = np.ascontiguousarray(target, np.float32)
    _ck(lib().slh_mlp_train(ordinal, int(kind), _sz(batch), _sz(d_in), _sz(d_h), _sz(d_out), p(x), p(target),
                            *[p(a) for a in params], _f(lr), _sz(steps), _sz(warmup), int(bool(fused)) | (2 if graph else 0) | (4 if fused_loss else 0) | (8 if whole_step else 0),
                            p(losses), C.byref(secs), C.byref(nodes)))
    if info is not None:
        info["graph_nodes"] = nodes.value
    return losses, secs.value


def bench_chain(n, iters=20, warmup=5, with_backward=True):
    """The bandwidth suite's chain ((a+b)*c-d) -> pow 2 -> square on n elements per tensor, issued op by
    op against the tape (add, mul, sub, pow, square), once with every op launched as it is issued and
    once with elementwise fusion switched on (one kernel for the chain, one for its backward).  Times
    are medians of per-iteration HIP-event pairs on the device's own stream; GB/s of the 20
    algorithmic bytes per element (4 reads, 1 write) forward, of 52 (4 inputs, the seed, 4 gradients
    read and written) for forward + backward."""
    import statistics
    L = _lib.load()
    out = {"elements": n}
    for label, fuse in (("op_by_op_tape", False), ("fused_tape", True)):
        dev = HIP(0, cached=True)
        dev.set_fuse_elementwise(fuse)
        ctx = dev.ctx_handle()
        bufs = []
        for tag in range(4):
            b = dev.zeros(n)
            p = C.c_void_p()
            _ck(lib().slh_buffer_ptr(dev.h, _u64(b.id), C.byref(p)))
            _lib.check(L.slhip_rand_uniform(ctx, 0x51CED, tag + 1, -10.0, 10.0, n, p), "slhip_rand_uniform")
            bufs.append(b)
        a, b, c, d = bufs

        def chain():
            dev.begin_iteration()
            return dev.square(dev.pow(dev.sub(dev.mul(dev.add(a, b), c), d), 2.0))

        def timed(body):
            ms = []
            for it in range(warmup + iters):
                e0, e1 = C.c_void_p(), C.c_void_p()
                L.slhip_event_create(ctx, C.byref(e0)); L.slhip_event_create(ctx, C.byref(e1))
                L.slhip_event_record(ctx, e0)
                body()
                L.slhip_event_record(ctx, e1)
                t = C.c_float()
                _lib.check(L.slhip_event_elapsed_ms(e0, e1, C.byref(t)), "slhip_event_elapsed_ms")
                L.slhip_event_destroy(e0); L.slhip_event_destroy(e1)
                if it >= warmup:
                    ms.append(t.value)
            return statistics.median(ms)

        dev.enable_tape(False)
        fwd = timed(lambda: (chain(), dev.run()))
        out["ms_" + label] = fwd
        out["GBps_" + label] = 20.0 * n / fwd / 1e6
        if with_backward:
            dev.enable_tape(True)

            def step():
                dev.zero_grad()
                chain().backward()
            both = timed(step)
            out["ms_fwd_bwd_" + label] = both
            out["GBps_fwd_bwd_" + label] = (20.0 + 52.0) * n / both / 1e6
        dev.close()
    return out


C1 = dict(kind=0, batch=1024, d_in=1, d_h=64, d_out=1, lr=0.01, steps=200)
C5 = dict(kind=1, batch=8192, d_in=784, d_h=2048, d_out=10, lr=0.05, steps=50)


def run_config(cfg, fused, warmup=0, steps=None, graph=False, info=None, fused_loss=False, whole_step=False):
    steps = steps or cfg["steps"]
    x, t = mlp_data(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_out"])
    params = mlp_init(cfg["kind"], cfg["d_in"], cfg["d_h"], cfg["d_out"])
    losses, secs = mlp_train(cfg["kind"], cfg["batch"], cfg["d_in"], cfg["d_h"], cfg["d_out"], x, t, params,
                             cfg["lr"], steps, warmup, fused, graph=graph, info=info, fused_loss=fused_loss, whole_step=whole_step)
    return losses, secs, params


def bench_mlp(steps_c5=50, steps_c1=200, graph=True):
    """Steps per second of the two training loops in their four variants; graph=False leaves out the
    two that replay a recorded step."""
    out = {}
    for name, cfg, steps in (("C5 classifier 784-2048-2048-10 batch 8192", C5, steps_c5),
                             ("C1 sine fit 1-64-64-1 batch 1024", C1, steps_c1)):
        for fused, graph_variant, floss, label in ((False, False, False, "op by op"), (True, False, False, "fused linear"),
                                           (True, True, False, "fused linear, recorded step replayed"),
                                           (True, True, True, "fused linear and loss, recorded step replayed")):
            if graph_variant and not graph:
                continue
            info = {}
            losses, secs, _ = run_config(cfg, fused, warmup=5, steps=steps, graph=graph_variant, info=info, fused_loss=floss)
            out["%s (%s)" % (name, label)] = {
                "steps_per_s": steps / secs, "ms_per_step": 1e3 * secs / steps,
                "first_loss": float(losses[0]), "last_loss": float(losses[-1])}
            if graph_variant:
                out["%s (%s)" % (name, label)]["kernels_per_step"] = info["graph_nodes"]
    info = {}
    losses, secs, _ = run_config(C1, True, warmup=5, steps=steps_c1, info=info, whole_step=True)
    out["C1 sine fit 1-64-64-1 batch 1024 (whole step in two launches)"] = {
        "steps_per_s": steps_c1 / secs, "ms_per_step": 1e3 * secs / steps_c1, "first_loss": float(losses[0]),
        "last_loss": float(losses[-1]), "kernels_per_step": info["graph_nodes"]}
    flop_c5 = 259.8e9
    k = "C5 classifier 784-2048-2048-10 batch 8192 (fused linear)"
    out["C5_fused_TFLOPs"] = flop_c5 * out[k]["steps_per_s"] / 1e12
    return out
