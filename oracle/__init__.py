"""numpy front-end of the CPU oracle (``liboracle.so``, built from oracle.cpp / mlp.cpp).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the shipped package never imports it.

Every wrapper keeps the argument meaning of the reference slice function it restates
(see the citations in oracle.cpp); arrays are float32, C-contiguous.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

ADD, SUB, MUL, DIV = 0, 1, 2, 3
SQUARE, POW, RELU, EXP, CLIP, NEG_LN, SCALE, NEG_DIV, TANH, SIGMOID = range(10)


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


_lib = None
_f = C.POINTER(C.c_float)
_d = C.POINTER(C.c_double)
_sz = C.c_size_t


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_sum.restype = C.c_float
        _lib.orc_max.restype = C.c_float
        _lib.orc_mean.restype = C.c_float
        _lib.orc_max_cols_grad.restype = C.c_int
        _lib.orc_mlp_train.restype = C.c_int
    return _lib


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_f)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    lib().orc_set_threads(int(n))


def max_threads():
    return int(lib().orc_max_threads())


# ---- reductions -----------------------------------------------------------
def sum_all(x):
    x = f32(x)
    return float(lib().orc_sum(_sz(x.size), _p(x)))


def mean(x):
    x = f32(x)
    return np.float32(lib().orc_mean(_sz(x.size), _p(x)))


def sum_rows(cols, x):
    x = f32(x).ravel()
    out = np.zeros(cols, np.float32)
    lib().orc_sum_rows2(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


def sum_cols(cols, x):
    x = f32(x).ravel()
    out = np.zeros(x.size // cols, np.float32)
    lib().orc_sum_cols(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


def max_rows(cols, x):
    x = f32(x).ravel()
    out = np.zeros(cols, np.float32)
    lib().orc_max_rows(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


def max_cols(cols, x):
    x = f32(x).ravel()
    out = np.zeros(x.size // cols, np.float32)
    lib().orc_max_cols(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


def mean_rows(cols, x):
    x = f32(x).ravel()
    out = np.zeros(cols, np.float32)
    lib().orc_mean_rows(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


def mean_cols(cols, x):
    x = f32(x).ravel()
    out = np.zeros(x.size // cols, np.float32)
    lib().orc_mean_cols(_sz(cols), _sz(x.size), _p(x), _p(out))
    return out


# ---- reduction grads (x_grad is updated in place and returned) -------------
def sum_rows_grad(cols, x_grad, out_grad):
    lib().orc_sum_rows_grad(_sz(cols), _sz(x_grad.size), _p(x_grad), _p(f32(out_grad)))
    return x_grad


def sum_cols_grad(cols, x_grad, out_grad):
    lib().orc_sum_cols_grad(_sz(cols), _sz(x_grad.size), _p(x_grad), _p(f32(out_grad)))
    return x_grad


def max_rows_grad(cols, out, x, x_grad, out_grad):
    lib().orc_max_rows_grad(_sz(cols), _sz(x.size), _p(f32(out)), _p(f32(x).ravel()), _p(x_grad),
                            _p(f32(out_grad)))
    return x_grad


def max_cols_grad(cols, out, x, x_grad, out_grad):
    rc = lib().orc_max_cols_grad(_sz(cols), _sz(x.size), _p(f32(out)), _p(f32(x).ravel()), _p(x_grad),
                                 _p(f32(out_grad)))
    if rc != 0:
        raise ValueError("Could not find maximum in gradient calculation")
    return x_grad


def mean_rows_grad(cols, x_grad, out_grad):
    lib().orc_mean_rows_grad(_sz(cols), _sz(x_grad.size), _p(x_grad), _p(f32(out_grad)))
    return x_grad


def mean_cols_grad(cols, x_grad, out_grad):
    lib().orc_mean_cols_grad(_sz(cols), _sz(x_grad.size), _p(x_grad), _p(f32(out_grad)))
    return x_grad


# ---- row / col ops ----------------------------------------------------------
def add_row(rows, cols, lhs, rhs):
    lhs = f32(lhs).ravel()
    out = np.empty_like(lhs)
    lib().orc_add_row(_sz(rows), _sz(cols), _p(lhs), _p(f32(rhs)), _p(out))
    return out


def add_row_grad(rows, cols, lhs_grad, rhs_grad, out_grad):
    lib().orc_add_row_grad(_sz(rows), _sz(cols), _p(lhs_grad), _p(rhs_grad), _p(f32(out_grad).ravel()))
    return lhs_grad, rhs_grad


def add_row_mut_grad(rows, cols, rhs_grad, out_grad):
    lib().orc_add_row_mut_grad(_sz(rows), _sz(cols), _p(rhs_grad), _p(f32(out_grad).ravel()))
    return rhs_grad


def mul_row_grad(cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    lib().orc_mul_row_grad(_sz(cols), _sz(lhs.size), _p(f32(lhs)), _p(f32(rhs)), _p(lhs_grad), _p(rhs_grad),
                           _p(f32(out_grad)))
    return lhs_grad, rhs_grad


def col_op(op, cols, lhs, rhs):
    lhs = f32(lhs).ravel()
    out = np.empty_like(lhs)
    lib().orc_col_op(int(op), _sz(cols), _sz(lhs.size), _p(lhs), _p(f32(rhs)), _p(out))
    return out


def row_op(op, cols, lhs, rhs):
    lhs = f32(lhs).ravel()
    out = np.empty_like(lhs)
    lib().orc_row_op(int(op), _sz(cols), _sz(lhs.size), _p(lhs), _p(f32(rhs)), _p(out))
    return out


def _bcast_op_grad(by_row_index, op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    lhs = f32(lhs).ravel()
    lib().orc_bcast_op_grad(by_row_index, int(op), _sz(cols), _sz(lhs.size), _p(lhs), _p(f32(rhs)),
                            _p(lhs_grad) if lhs_grad is not None else None,
                            _p(rhs_grad) if rhs_grad is not None else None, _p(f32(out_grad).ravel()))
    return lhs_grad, rhs_grad


def row_op_grad(op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    return _bcast_op_grad(0, op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad)


def col_op_grad(op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad):
    return _bcast_op_grad(1, op, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad)


# ---- elementwise ------------------------------------------------------------
def binary_ew(op, l, r):
    l, r = f32(l).ravel(), f32(r).ravel()
    out = np.empty_like(l)
    lib().orc_binary_ew(int(op), _sz(l.size), _p(l), _p(r), _p(out))
    return out


def binary_ew_grad(op, l, r, lg, rg, g):
    lib().orc_binary_ew_grad(int(op), _sz(l.size), _p(f32(l).ravel()), _p(f32(r).ravel()),
                             _p(lg) if lg is not None else None, _p(rg) if rg is not None else None,
                             _p(f32(g).ravel()))
    return lg, rg


def add_ew_grad(lg, rg, g):
    lib().orc_add_ew_grad(_sz(lg.size), _p(lg), _p(rg), _p(f32(g)))
    return lg, rg


def unary(op, x, p=0.0, q=0.0):
    x = f32(x).ravel()
    out = np.empty_like(x)
    lib().orc_unary(int(op), C.c_float(p), C.c_float(q), _sz(x.size), _p(x), _p(out))
    return out


def unary_grad(op, x, x_grad, out_grad, p=0.0):
    lib().orc_unary_grad(int(op), C.c_float(p), _sz(x.size), _p(f32(x).ravel()), _p(x_grad),
                         _p(f32(out_grad).ravel()))
    return x_grad


# ---- transpose / gemm ---------------------------------------------------------
def transpose(rows, cols, a, out=None, assign=False):
    a = f32(a).ravel()
    if out is None:
        out = np.zeros_like(a)
    lib().orc_transpose(_sz(rows), _sz(cols), _p(a), _p(out), int(assign))
    return out


def _gemm(fn, m, n, k, a, b, c, beta):
    a, b = f32(a).ravel(), f32(b).ravel()
    assert a.size == m * k and b.size == k * n, (a.size, b.size, m, n, k)
    if c is None:
        c = np.zeros(m * n, np.float32)
    fn(_sz(m), _sz(n), _sz(k), _p(a), _p(b), _p(c), C.c_float(beta))
    return c


def gemm(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::gemm(m, n, k, a, b, c): c[m×n] = a[m×k]·b[k×n]."""
    return _gemm(lib().orc_gemm, m, n, k, a, b, c, beta)


def gemmT(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::gemmT: c[m×n] = a[m×k]·bᵀ, b stored n×k."""
    return _gemm(lib().orc_gemmT, m, n, k, a, b, c, beta)


def Tgemm(m, n, k, a, b, c=None, beta=0.0):
    """GenericBlas::Tgemm: c[m×n] = aᵀ·b, a stored k×m."""
    return _gemm(lib().orc_Tgemm, m, n, k, a, b, c, beta)


def gemm_f64(ta, tb, m, n, k, a, b):
    a, b = f32(a).ravel(), f32(b).ravel()
    c = np.zeros(m * n, np.float64)
    lib().orc_gemm_f64(int(ta), int(tb), _sz(m), _sz(n), _sz(k), _p(a), _p(b), c.ctypes.data_as(_d))
    return c


def gemm_grad(m, k, n, lhs, rhs, lhs_grad, rhs_grad, out_grad, beta=0.0):
    """GemmGrad::gemm_grad with the trait's (m, k, n); None grads are skipped."""
    lib().orc_gemm_grad(_sz(m), _sz(k), _sz(n), _p(f32(lhs).ravel()), _p(f32(rhs).ravel()),
                        _p(lhs_grad) if lhs_grad is not None else None,
                        _p(rhs_grad) if rhs_grad is not None else None, _p(f32(out_grad).ravel()),
                        C.c_float(beta))
    return lhs_grad, rhs_grad


# ---- softmax & co -------------------------------------------------------------
def softmax(samples, features, x):
    x = f32(x).ravel()
    out = np.empty_like(x)
    lib().orc_softmax(_sz(samples), _sz(features), _p(x), _p(out))
    return out


def softmax_grad(samples, features, out, out_grad, x_grad=None, beta=0.0):
    out, out_grad = f32(out).ravel(), f32(out_grad).ravel()
    if x_grad is None:
        x_grad = np.zeros_like(out)
    lib().orc_softmax_grad(_sz(samples), _sz(features), _p(x_grad), _p(out), _p(out_grad), C.c_float(beta))
    return x_grad


def softmax_grad_jacobian(samples, features, out, out_grad):
    out, out_grad = f32(out).ravel(), f32(out_grad).ravel()
    x_grad = np.zeros_like(out)
    lib().orc_softmax_grad_jacobian(_sz(samples), _sz(features), _p(x_grad), _p(out), _p(out_grad))
    return x_grad


def diagflat(x):
    x = f32(x).ravel()
    out = np.zeros(x.size * x.size, np.float32)
    lib().orc_diagflat(_sz(x.size), _p(x), _p(out))
    return out


def diagflat_grad(x_grad, out_grad):
    lib().orc_diagflat_grad(_sz(x_grad.size), _p(x_grad), _p(f32(out_grad).ravel()))
    return x_grad


def onehot(highest_class, classes):
    classes = f32(classes).ravel()
    out = np.zeros(classes.size * highest_class, np.float32)
    lib().orc_onehot(_sz(highest_class), _sz(classes.size), _p(classes), _p(out))
    return out


def onehot_grad(highest_class, classes, classes_grad, out_grad):
    classes = f32(classes).ravel()
    lib().orc_onehot_grad(_sz(highest_class), _sz(classes.size), _p(classes), _p(classes_grad),
                          _p(f32(out_grad).ravel()))
    return classes_grad


def cce(rows, cols, preds, targets):
    out = np.zeros(rows, np.float32)
    lib().orc_cce(_sz(rows), _sz(cols), _p(f32(preds).ravel()), _p(f32(targets).ravel()), _p(out))
    return out


def cce_grad(rows, cols, preds, targets):
    out = np.zeros(rows * cols, np.float32)
    lib().orc_cce_grad(_sz(rows), _sz(cols), _p(f32(preds).ravel()), _p(f32(targets).ravel()), _p(out))
    return out


def sgd_step(p, g, lr):
    lib().orc_sgd_step(_sz(p.size), _p(p), _p(f32(g)), C.c_float(lr))
    return p


def mlp_train(kind, batch, d_in, d_h, d_out, x, target, params, lr, steps):
    """params = [W1, b1, W2, b2, W3, b3] float32 arrays, updated in place. Returns losses."""
    losses = np.zeros(steps, np.float32)
    rc = lib().orc_mlp_train(int(kind), _sz(batch), _sz(d_in), _sz(d_h), _sz(d_out), _p(f32(x).ravel()),
                             _p(f32(target).ravel()), *[_p(p) for p in params], C.c_float(lr), _sz(steps),
                             _p(losses))
    assert rc == 0
    return losses
