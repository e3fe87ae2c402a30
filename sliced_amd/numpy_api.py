"""numpy-in / numpy-out facade over the C ABI, one function per reference slice function or
trait method (same names and argument meaning as the CPU oracle's front-end), so that a
parity test is the same call on both sides.  Every call uploads its operands, runs the HIP
kernels and downloads the result; nothing is computed on the host.
"""
import ctypes as C

import numpy as np

from .device import Context

ADD, SUB, MUL, DIV = 0, 1, 2, 3
SQUARE, POW, RELU, EXP, CLIP, NEG_LN, SCALE, NEG_DIV = range(8)

_ctx = None


def init(ordinal=0):
    global _ctx
    if _ctx is None:
        _ctx = Context(ordinal)
    return _ctx


def ctx():
    return init(0)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32).ravel()


_operand_offsets = None       # see operands_off_the_vector_grid()
_next_offset = 0


def operands_off_the_vector_grid(on):
    """With on=True every device buffer this facade creates starts 1, 2 or 3 floats (in turn) into
    its allocation instead of on the allocator's 256-byte grid: the library promises to take
    pointers that are only float-aligned, and this lets any test that goes through the facade ask
    for exactly that."""
    global _operand_offsets, _next_offset
    _operand_offsets = (1, 2, 3) if on else None
    _next_offset = 0


class _Scope:
    """Frees every device buffer created inside the with-block."""

    def __init__(self):
        self.c = ctx()
        self.bufs = []

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        for b in self.bufs:
            b.free()

    def _alloc(self, n, zero):
        global _next_offset
        off = 0
        if _operand_offsets:
            off = _operand_offsets[_next_offset % len(_operand_offsets)]
            _next_offset += 1
        pool = (self.c.zeros if zero else self.c.empty)(n + off)
        self.bufs.append(pool)
        return pool.view(off, n) if off else pool

    def up(self, a):
        if a is None:
            return None
        a = _f32(a)
        return self._alloc(a.size, False).upload(a)

    def zeros(self, n):
        return self._alloc(n, True)

    def empty(self, n):
        return self._alloc(n, False)


def _ptr(b):
    return b.ptr if b is not None else None


# ---- reductions -------------------------------------------------------------
def _reduce(name, rows, cols, x, outlen):
    with _Scope() as s:
        dx, do = s.up(x), s.empty(outlen)
        s.c.call(name, rows, cols, dx.ptr, do.ptr)
        return do.numpy()


def sum_rows(cols, x):
    x = _f32(x)
    return _reduce("slhip_sum_rows", x.size // cols, cols, x, cols)


def sum_rows_static(cols, x):
    """slhip_sum_rows_static: the same reduction with its partial sums in the library's static scratch array."""
    x = _f32(x)
    return _reduce("slhip_sum_rows_static", x.size // cols, cols, x, cols)


def sum_cols(cols, x):
    x = _f32(x)
    return _reduce("slhip_sum_cols", x.size // cols, cols, x, x.size // cols)


def max_rows(cols, x):
    x = _f32(x)
    return _reduce("slhip_max_rows", x.size // cols, cols, x, cols)


def max_cols(cols, x):
    x = _f32(x)
    return _reduce("slhip_max_cols", x.size // cols, cols, x, x.size // cols)


def mean_rows(cols, x):
    x = _f32(x)
    return _reduce("slhip_mean_rows", x.size // cols, cols, x, cols)


def mean_cols(cols, x):
    x = _f32(x)
    return _reduce("slhip_mean_cols", x.size // cols, cols, x, x.size // cols)


def _scalar(name, x):
    x = _f32(x)
    with _Scope() as s:
        dx, do = s.up(x), s.empty(1)
        s.c.call(name, x.size, dx.ptr, do.ptr)
        return do.numpy()[0]


def sum_all(x):
    return float(_scalar("slhip_sum", x))


def max_all(x):
    return float(_scalar("slhip_max", x))


def mean(x):
    return _scalar("slhip_mean", x)


def _bcast_grad(name, cols, x_grad, out_grad):
    with _Scope() as s:
        dg, do = s.up(x_grad), s.up(out_grad)
        s.c.call(name, x_grad.size // cols, cols, dg.ptr, do.ptr)
        x_grad[:] = dg.numpy()
    return x_grad


def sum_rows_grad(cols, x_grad, out_grad):
    return _bcast_grad("slhip_sum_rows_grad", cols, x_grad, out_grad)


def sum_cols_grad(cols, x_grad, out_grad):
    return _bcast_grad("slhip_sum_cols_grad", cols, x_grad, out_grad)


def mean_rows_grad(cols, x_grad, out_grad):
    return _bcast_grad("slhip_mean_rows_grad", cols, x_grad, out_grad)


def mean_cols_grad(cols, x_grad, out_grad):
    return _bcast_grad("slhip_mean_cols_grad", cols, x_grad, out_grad)


def _max_grad(name, cols, out, x, x_grad, out_grad):
    x = _f32(x)
    with _Scope() as s:
        d_out, dx, dg, dog = s.up(out), s.up(x), s.up(x_grad), s.up(out_grad)
        s.c.call(name, x.size // cols, cols, d_out.ptr, dx.ptr, dg.ptr, dog.ptr)
        x_grad[:] = dg.numpy()
    return x_grad


def max_rows_grad(cols, out, x, x_grad, out_grad):
    return _max_grad("slhip_max_rows_grad", cols, out, x, x_grad, out_grad)


def max_cols_grad(cols, out, x, x_grad, out_grad):
    return _max_grad("slhip_max_cols_grad", cols, out, x, x_grad, out_grad)


# ---- row op -------------------------------------------------------------------
def add_row(rows, cols, lhs, rhs, inplace=False):
    with _Scope() as s:
        dl, dr = s.up(lhs), s.up(rhs)
        do = dl if inplace else s.empty(rows * cols)
        s.c.call("slhip_add_row", rows, cols, dl.ptr, dr.ptr, do.ptr)
        return do.numpy()


def add_row_grad(rows, cols, lhs_grad, rhs_grad, out_grad):
    with _Scope() as s:
        dl, dr, dg = s.up(lhs_grad), s.up(rhs_grad), s.up(out_grad)
        s.c.call("slhip_add_row_grad", rows, cols, dl.ptr, dr.ptr, dg.ptr)
        lhs_grad[:] = dl.numpy()
        rhs_grad[:] = dr.numpy()
    return lhs_grad, rhs_grad


def add_row_mut_grad(rows, cols, rhs_grad, out_grad):
    with _Scope() as s:
        dr, dg = s.up(rhs_grad), s.up(out_grad)
        s.c.call("slhip_add_row_mut_grad", rows, cols, dr.ptr, dg.ptr)
        rhs_grad[:] = dr.numpy()
    return rhs_grad


# ---- elementwise ------------------------------------------------------------------
def binary_ew(op, l, r):
    l = _f32(l)
    with _Scope() as s:
        dl, dr, do = s.up(l), s.up(r), s.empty(l.size)
        s.c.call("slhip_ew_binary", int(op), l.size, dl.ptr, dr.ptr, do.ptr)
        return do.numpy()


def binary_ew_grad(op, l, r, lg, rg, g):
    l = _f32(l)
    with _Scope() as s:
        dl, dr, dlg, drg, dg = s.up(l), s.up(r), s.up(lg), s.up(rg), s.up(g)
        s.c.call("slhip_ew_binary_grad", int(op), l.size, dl.ptr, dr.ptr, _ptr(dlg), _ptr(drg), dg.ptr)
        if lg is not None:
            lg[:] = dlg.numpy()
        if rg is not None:
            rg[:] = drg.numpy()
    return lg, rg


def unary(op, x, p=0.0, q=0.0):
    x = _f32(x)
    with _Scope() as s:
        dx, do = s.up(x), s.empty(x.size)
        s.c.call("slhip_ew_unary", int(op), float(p), float(q), x.size, dx.ptr, do.ptr)
        return do.numpy()


def unary_grad(op, x, x_grad, out_grad, p=0.0):
    x = _f32(x)
    with _Scope() as s:
        dx, dg, dog = s.up(x), s.up(x_grad), s.up(out_grad)
        s.c.call("slhip_ew_unary_grad", int(op), float(p), x.size, dx.ptr, dg.ptr, dog.ptr)
        x_grad[:] = dg.numpy()
    return x_grad


EW_UNARY, EW_NOGRAD = 0x10, 0x1
INSN = np.dtype([("op", "u1"), ("src0", "u1"), ("src1", "u1"), ("flags", "u1"), ("p", "f4"), ("q", "f4")])


def ew_insn(prog):
    """[(op, src0, src1, flags, p, q), ...] -> the packed slhip_ew_insn array."""
    arr = np.zeros(len(prog), INSN)
    for i, t in enumerate(prog):
        t = tuple(t) + (0,) * (6 - len(t))
        arr[i] = t
    return arr


def _ptr_array(bufs):
    import ctypes as C
    arr = (C.c_void_p * len(bufs))(*[b.ptr if b is not None else None for b in bufs])
    return arr


def ew_program(inputs, prog):
    """slhip_ew_program: the program's result over the input arrays."""
    import ctypes as C
    ins = [_f32(x) for x in inputs]
    code = ew_insn(prog)
    with _Scope() as s:
        d = [s.up(x) for x in ins]
        out = s.empty(ins[0].size)
        ptrs = _ptr_array(d)
        s.c.call("slhip_ew_program", ins[0].size, len(d), C.cast(ptrs, C.c_void_p), len(code), code.ctypes.data, out.ptr)
        return out.numpy()


def ew_program_grad(inputs, grads, prog, out_grad):
    """slhip_ew_program_grad: grads[j] (None = skipped) after the call."""
    import ctypes as C
    ins = [_f32(x) for x in inputs]
    code = ew_insn(prog)
    with _Scope() as s:
        d = [s.up(x) for x in ins]
        g = [s.up(x) for x in grads]
        og = s.up(out_grad)
        ip, gp = _ptr_array(d), _ptr_array(g)
        s.c.call("slhip_ew_program_grad", ins[0].size, len(d), C.cast(ip, C.c_void_p), C.cast(gp, C.c_void_p), len(code),
                 code.ctypes.data, og.ptr)
        return [b.numpy() if b is not None else None for b in g]


def ew_chain(a, b, c, d):
    a = _f32(a)
    with _Scope() as s:
        da, db, dc, dd, do = s.up(a), s.up(b), s.up(c), s.up(d), s.empty(a.size)
        s.c.call("slhip_ew_chain", a.size, da.ptr, db.ptr, dc.ptr, dd.ptr, do.ptr)
        return do.numpy()


# ---- transpose / gemm -----------------------------------------------------------------
def transpose(rows, cols, a, out=None, assign=False):
    a = _f32(a)
    with _Scope() as s:
        da = s.up(a)
        do = s.up(out) if out is not None else s.empty(a.size)
        s.c.call("slhip_transpose", rows, cols, da.ptr, do.ptr, 1.0 if assign else 0.0)
        res = do.numpy()
    if out is not None:
        out[:] = res
        return out
    return res


def sgemm(ta, tb, m, n, k, a, b, c=None, beta=0.0):
    a, b = _f32(a), _f32(b)
    assert a.size == m * k and b.size == k * n, (a.size, b.size, m, n, k)
    with _Scope() as s:
        da, db = s.up(a), s.up(b)
        dc = s.up(c) if c is not None else s.empty(m * n)
        s.c.call("slhip_sgemm", int(ta), int(tb), m, n, k, da.ptr, db.ptr, dc.ptr, float(beta))
        res = dc.numpy()
    if c is not None:
        c[:] = res
        return c
    return res


def sgemm_relu_mask(ta, tb, m, n, k, a, b, pre, c=None, beta=0.0):
    """c = beta*c + (op(a)·op(b)) * (pre >= 0)."""
    a, b, pre = _f32(a), _f32(b), _f32(pre)
    assert a.size == m * k and b.size == k * n and pre.size == m * n
    with _Scope() as s:
        da, db, dp = s.up(a), s.up(b), s.up(pre)
        dc = s.up(c) if c is not None else s.empty(m * n)
        s.c.call("slhip_sgemm_relu_mask", int(ta), int(tb), m, n, k, da.ptr, db.ptr, dp.ptr, dc.ptr, float(beta))
        return dc.numpy()


TAIL_AUTO, TAIL_WHOLE, TAIL_SPREAD = 0, 1, 2


def gemm_tail_policy(policy):
    """How the tiled GEMM treats a partly filled last round of workgroups (a tuning knob)."""
    ctx().call("slhip_gemm_tail_policy", int(policy))


TILE_AUTO, TILE_128X128, TILE_64X64, TILE_128X128_WIDE = 0, 1, 3, 4


def gemm_tile_policy(policy):
    """The tile of C per workgroup of the tiled GEMM (a tuning knob)."""
    ctx().call("slhip_gemm_tile_policy", int(policy))


def gemm(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::gemm(m, n, k, a, b, c)."""
    return sgemm(0, 0, m, n, k, a, b, c, beta)


def gemmT(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::gemmT: c = a·bᵀ, b stored n×k."""
    return sgemm(0, 1, m, n, k, a, b, c, beta)


def Tgemm(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::Tgemm: c = aᵀ·b, a stored k×m."""
    return sgemm(1, 0, m, n, k, a, b, c, beta)


def gemm_grad(m, k, n, lhs, rhs, lhs_grad, rhs_grad, out_grad, beta=0.0):
    with _Scope() as s:
        dl, dr, dlg, drg, dg = s.up(lhs), s.up(rhs), s.up(lhs_grad), s.up(rhs_grad), s.up(out_grad)
        s.c.call("slhip_gemm_grad", m, k, n, dl.ptr, dr.ptr, _ptr(dlg), _ptr(drg), dg.ptr, float(beta))
        if lhs_grad is not None:
            lhs_grad[:] = dlg.numpy()
        if rhs_grad is not None:
            rhs_grad[:] = drg.numpy()
    return lhs_grad, rhs_grad


def linear_fwd(m, k, n, x, w, bias, relu=False, want_pre_act=False):
    with _Scope() as s:
        dx, dw, db, do = s.up(x), s.up(w), s.up(bias), s.empty(m * n)
        dp = s.empty(m * n) if want_pre_act else None
        s.c.call("slhip_linear_fwd", m, k, n, dx.ptr, dw.ptr, _ptr(db), int(relu), _ptr(dp), do.ptr)
        if want_pre_act:
            return do.numpy(), dp.numpy()
        return do.numpy()


def linear_grad(m, k, n, x, w, out_grad, x_grad=None, relu_pre=None, w_grad=None, bias_grad=None, beta=0.0):
    """The backward pass of a Linear layer (slhip_linear_grad): the gradients that are given (as their
    values before the call) come back updated in place, the others are skipped."""
    with _Scope() as s:
        dx, dw, dg = s.up(x), s.up(w), s.up(out_grad)
        dxg, dpre, dwg, dbg = s.up(x_grad), s.up(relu_pre), s.up(w_grad), s.up(bias_grad)
        s.c.call("slhip_linear_grad", m, k, n, dx.ptr, dw.ptr, _ptr(dxg), _ptr(dpre), _ptr(dwg), _ptr(dbg), dg.ptr, float(beta))
        for host, dev in ((x_grad, dxg), (w_grad, dwg), (bias_grad, dbg)):
            if host is not None:
                host[:] = dev.numpy().reshape(host.shape)
    return x_grad, w_grad, bias_grad


def linear_fwd_bits(m, k, n, x, w, bias):
    """relu(x·w + bias) and the packed mask (x·w + bias >= 0): uint32 [m][ceil(n / 32)]."""
    words = m * ((n + 31) // 32)
    with _Scope() as s:
        dx, dw, db, do, dbits = s.up(x), s.up(w), s.up(bias), s.empty(m * n), s.zeros(words)
        s.c.call("slhip_linear_fwd_bits", m, k, n, dx.ptr, dw.ptr, _ptr(db), dbits.ptr, do.ptr)
        return do.numpy(), dbits.numpy().view(np.uint32).reshape(m, -1)


def sgemm_relu_bits(ta, tb, m, n, k, a, b, bits, c=None, beta=0.0):
    """c = beta*c + (op(a)·op(b)) * bit."""
    with _Scope() as s:
        da, db = s.up(a), s.up(b)
        dbits = s.up(np.ascontiguousarray(bits, np.uint32).ravel().view(np.float32))
        dc = s.up(c) if c is not None else s.empty(m * n)
        s.c.call("slhip_sgemm_relu_bits", int(ta), int(tb), m, n, k, da.ptr, db.ptr, dbits.ptr, dc.ptr, float(beta))
        return dc.numpy()


def relu_grad_bits(rows, cols, bits, x_grad, out_grad):
    with _Scope() as s:
        dbits = s.up(np.ascontiguousarray(bits, np.uint32).ravel().view(np.float32))
        dx, dg = s.up(x_grad), s.up(out_grad)
        s.c.call("slhip_relu_grad_bits", rows, cols, dbits.ptr, dx.ptr, dg.ptr)
        return dx.numpy()


# ---- softmax & co ----------------------------------------------------------------------
def softmax(samples, features, x):
    with _Scope() as s:
        dx, do = s.up(x), s.empty(samples * features)
        s.c.call("slhip_softmax", samples, features, dx.ptr, do.ptr)
        return do.numpy()


def softmax_grad(samples, features, out, out_grad, x_grad=None, beta=0.0):
    with _Scope() as s:
        d_out, dg = s.up(out), s.up(out_grad)
        dx = s.up(x_grad) if x_grad is not None else s.zeros(samples * features)
        s.c.call("slhip_softmax_grad", samples, features, dx.ptr, d_out.ptr, dg.ptr, float(beta))
        res = dx.numpy()
    if x_grad is not None:
        x_grad[:] = res
        return x_grad
    return res


def _bcast_op(name, op, cols, lhs, rhs):
    lhs = _f32(lhs)
    with _Scope() as s:
        dl, dr, do = s.up(lhs), s.up(rhs), s.empty(lhs.size)
        s.c.call(name, int(op), lhs.size // cols, cols, dl.ptr, dr.ptr, do.ptr)
        return do.numpy()


def row_op(op, cols, lhs, rhs):
    return _bcast_op("slhip_row_op", op, cols, lhs, rhs)


def col_op(op, cols, lhs, rhs):
    return _bcast_op("slhip_col_op", op, cols, lhs, rhs)


def _bcast_op_grad(name, op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    lhs = _f32(lhs)
    with _Scope() as s:
        dl, dr, dg = s.up(lhs), s.up(rhs), s.up(out_grad)
        dlg, drg = s.up(lhs_grad), s.up(rhs_grad)
        s.c.call(name, int(op), lhs.size // cols, cols, dl.ptr, dr.ptr, dlg.ptr if dlg else None,
                 drg.ptr if drg else None, dg.ptr)
        if lhs_grad is not None:
            lhs_grad[:] = dlg.numpy()
        if rhs_grad is not None:
            rhs_grad[:] = drg.numpy()
    return lhs_grad, rhs_grad


def row_op_grad(op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    return _bcast_op_grad("slhip_row_op_grad", op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad)


def col_op_grad(op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    return _bcast_op_grad("slhip_col_op_grad", op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad)


def mul_row_grad(cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    return row_op_grad(2, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad)


def diagflat(x):
    x = _f32(x)
    with _Scope() as s:
        dx, do = s.up(x), s.empty(x.size * x.size)
        s.c.call("slhip_diagflat", x.size, dx.ptr, do.ptr)
        return do.numpy()


def diagflat_grad(x_grad, out_grad):
    with _Scope() as s:
        dx, dg = s.up(x_grad), s.up(out_grad)
        s.c.call("slhip_diagflat_grad", x_grad.size, dx.ptr, dg.ptr)
        x_grad[:] = dx.numpy()
    return x_grad


def mlp3_mse_step(batch, d_in, d_h, d_out, x, target, params, lr, with_grads=True):
    """slhip_mlp3_mse_step on host arrays: params (W1, b1, W2, b2, W3, b3) are updated in place;
    returns (loss, the six gradients or None)."""
    with _Scope() as s:
        dx, dt, dl = s.up(x), s.up(target), s.empty(1)
        dp = [s.up(p) for p in params]
        dg = [s.empty(p.size) for p in params] if with_grads else None
        garr = (C.c_void_p * 6)(*[g.ptr for g in dg]) if with_grads else None
        s.c.call("slhip_mlp3_mse_step", batch, d_in, d_h, d_out, dx.ptr, dt.ptr, *[p.ptr for p in dp], garr, float(lr), dl.ptr)
        for host, dev in zip(params, dp):
            host[:] = dev.numpy().reshape(host.shape)
        return dl.numpy()[0], ([g.numpy() for g in dg] if with_grads else None)


def mse(x, y):
    x = _f32(x)
    with _Scope() as s:
        dx, dy, do = s.up(x), s.up(y), s.empty(1)
        s.c.call("slhip_mse", x.size, dx.ptr, dy.ptr, do.ptr)
        return do.numpy()[0]


def mse_grad(x, y, x_grad, upstream=1.0):
    x = _f32(x)
    with _Scope() as s:
        dx, dy, dg, du = s.up(x), s.up(y), s.up(x_grad), s.up(np.array([upstream], np.float32))
        s.c.call("slhip_mse_grad", x.size, dx.ptr, dy.ptr, dg.ptr, du.ptr)
        x_grad[:] = dg.numpy()
    return x_grad


def softmax_cce(rows, cols, logits, targets, want_probs=True):
    """(probs, loss per row); probs is None when want_probs is False (the library then stores none)"""
    with _Scope() as s:
        dl, dt, do = s.up(logits), s.up(targets), s.empty(rows)
        dp = s.empty(rows * cols) if want_probs else None
        s.c.call("slhip_softmax_cce", rows, cols, dl.ptr, dt.ptr, _ptr(dp), do.ptr)
        return (dp.numpy() if want_probs else None), do.numpy()


def softmax_cce_grad(rows, cols, probs, targets, logits_grad, beta=0.0, upstream=1.0):
    with _Scope() as s:
        dp, dt, dg, du = s.up(probs), s.up(targets), s.up(logits_grad), s.up(np.array([upstream], np.float32))
        s.c.call("slhip_softmax_cce_grad", rows, cols, dp.ptr, dt.ptr, dg.ptr, float(beta), du.ptr)
        logits_grad[:] = dg.numpy()
    return logits_grad


def onehot_grad(highest_class, classes, classes_grad, out_grad):
    classes = _f32(classes)
    with _Scope() as s:
        dc, dcg, dg = s.up(classes), s.up(classes_grad), s.up(out_grad)
        s.c.call("slhip_onehot_grad", classes.size, highest_class, dc.ptr, dcg.ptr, dg.ptr)
        classes_grad[:] = dcg.numpy()
    return classes_grad


def onehot(highest_class, classes):
    classes = _f32(classes)
    with _Scope() as s:
        dc, do = s.up(classes), s.empty(classes.size * highest_class)
        s.c.call("slhip_onehot", classes.size, highest_class, dc.ptr, do.ptr)
        return do.numpy()


def cce(rows, cols, preds, targets):
    with _Scope() as s:
        dp, dt, do = s.up(preds), s.up(targets), s.empty(rows)
        s.c.call("slhip_cce", rows, cols, dp.ptr, dt.ptr, do.ptr)
        return do.numpy()


def cce_grad(rows, cols, preds, targets):
    with _Scope() as s:
        dp, dt, do = s.up(preds), s.up(targets), s.empty(rows * cols)
        s.c.call("slhip_cce_grad", rows, cols, dp.ptr, dt.ptr, do.ptr)
        return do.numpy()


def sgd_step(p, g, lr):
    with _Scope() as s:
        dp, dg = s.up(p), s.up(g)
        s.c.call("slhip_sgd_step", p.size, dp.ptr, dg.ptr, float(lr))
        p[:] = dp.numpy()
    return p


def rand_uniform(n, lo, hi, tag, seed):
    with _Scope() as s:
        b = s.c.uniform(n, lo, hi, tag, seed)
        s.bufs.append(b)
        return b.numpy()
