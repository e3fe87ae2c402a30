"""Replays the reference's own test vectors (tests/golden/reference_vectors.json) against a
backend: the CPU oracle (``import oracle``) or the HIP path (``sliced_amd.numpy_api``).

Both backends expose the same numpy-level functions, named after the reference's slice
functions / trait methods, so one runner serves both.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}
UN = {"square": 0, "pow": 1, "relu": 2, "exp": 3, "tanh": 8, "sigmoid": 9}


def load_cases():
    with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
        return json.load(f)["cases"]


def f32(a):
    return np.asarray(a, dtype=np.float32)


def check(got, expect, tol, what=""):
    got = np.asarray(got, dtype=np.float32).ravel()
    expect = f32(expect).ravel()
    assert got.shape == expect.shape, (what, got.shape, expect.shape)
    if tol == 0:
        assert np.array_equal(got, expect), f"{what}: {got} != {expect}"
    else:
        assert np.max(np.abs(got - expect)) <= tol, f"{what}: {got} vs {expect}"


class Unsupported(Exception):
    pass


def run_case(be, c):
    fn, tol = c["fn"], c["tol"]
    need = lambda name: getattr(be, name, None) or (_ for _ in ()).throw(Unsupported(name))

    if fn in ("sum_rows", "sum_cols", "max_rows", "max_cols", "mean_rows", "mean_cols"):
        check(need(fn)(c["cols"], f32(c["x"])), c["expect"], tol, c["name"])
    elif fn in ("sum_rows_grad", "sum_cols_grad", "mean_rows_grad", "mean_cols_grad"):
        xg = np.zeros(c["len"], np.float32)
        check(need(fn)(c["cols"], xg, f32(c["out_grad"])), c["expect"], tol, c["name"])
    elif fn in ("max_rows_grad", "max_cols_grad"):
        x = f32(c["x"])
        out = need(fn[:-5])(c["cols"], x)
        xg = np.zeros(x.size, np.float32)
        check(need(fn)(c["cols"], out, x, xg, f32(c["out_grad"])), c["expect"], tol, c["name"])
    elif fn == "add_row":
        check(need(fn)(c["rows"], c["cols"], f32(c["lhs"]), f32(c["rhs"])), c["expect"], tol, c["name"])
    elif fn == "add_row_grad":
        n = c["rows"] * c["cols"]
        lg, rg = np.zeros(n, np.float32), np.zeros(c["cols"], np.float32)
        lg, rg = need(fn)(c["rows"], c["cols"], lg, rg, f32(c["out_grad"]))
        check(lg, c["expect_lhs"], tol, c["name"])
        check(rg, c["expect_rhs"], tol, c["name"])
    elif fn == "add_row_mut_grad":
        rg = np.zeros(c["cols"], np.float32)
        check(need(fn)(c["rows"], c["cols"], rg, f32(c["out_grad"])), c["expect"], tol, c["name"])
    elif fn == "mul_row_grad":
        lhs = f32(c["lhs"])
        lg, rg = np.zeros(lhs.size, np.float32), np.zeros(c["cols"], np.float32)
        lg, rg = need(fn)(c["cols"], lhs, f32(c["rhs"]), lg, rg, f32(c["out_grad"]))
        check(lg, c["expect_lhs"], tol, c["name"])
        check(rg, c["expect_rhs"], tol, c["name"])
    elif fn == "col_op":
        check(need(fn)(OPS[c["op"]], c["cols"], f32(c["lhs"]), f32(c["rhs"])), c["expect"], tol, c["name"])
    elif fn == "col_op_grad":
        lhs = f32(c["lhs"])
        lg, rg = np.zeros(lhs.size, np.float32), np.zeros(lhs.size // c["cols"], np.float32)
        lg, rg = need(fn)(OPS[c["op"]], c["cols"], lhs, f32(c["rhs"]), lg, rg, f32(c["out_grad"]))
        if "expect_lhs" in c:
            check(lg, c["expect_lhs"], tol, c["name"])
        if "expect_rhs" in c:
            check(rg, c["expect_rhs"], tol, c["name"])
    elif fn == "diagflat_grad":
        check(need(fn)(np.zeros(c["n"], np.float32), f32(c["out_grad"])), c["expect"], tol, c["name"])
    elif fn == "onehot_grad":
        cls = f32(c["classes"])
        check(need(fn)(c["highest_class"], cls, np.zeros(cls.size, np.float32), f32(c["out_grad"])), c["expect"], tol,
              c["name"])
    elif fn == "binary_ew":
        check(need(fn)(OPS[c["op"]], f32(c["lhs"]), f32(c["rhs"])), c["expect"], tol, c["name"])
    elif fn == "binary_ew_with_grad":
        l, r = f32(c["lhs"]), f32(c["rhs"])
        check(need("binary_ew")(OPS[c["op"]], l, r), c["expect"], tol, c["name"])
        lg, rg = np.zeros_like(l), np.zeros_like(r)
        seed = np.ones_like(l)                       # backward() seeds the output grad with ones
        lg, rg = need("binary_ew_grad")(OPS[c["op"]], l, r, lg, rg, seed)
        check(lg, c["expect_lhs_grad"], tol, c["name"])
        check(rg, c["expect_rhs_grad"], tol, c["name"])
    elif fn == "unary_with_grad":
        x = f32(c["x"])
        check(need("unary")(UN[c["op"]], x, c["p"]), c["expect"], tol, c["name"])
        xg = np.zeros_like(x)
        check(need("unary_grad")(UN[c["op"]], x, xg, np.ones_like(x), c["p"]), c["expect_grad"], tol, c["name"])
    elif fn == "transpose":
        check(need(fn)(c["rows"], c["cols"], f32(c["x"])), c["expect"], tol, c["name"])
    elif fn == "transpose_mul_grad":
        # out = mul(y, T(x)); backward seeds ones: T(x).grad = y; x.grad = transpose_grad(y)
        rows, cols = c["rows"], c["cols"]
        x, y = f32(c["x"]), f32(c["y"])
        xt = need("transpose")(rows, cols, x)
        lg, rg = np.zeros_like(y), np.zeros_like(xt)
        need("binary_ew_grad")(OPS["mul"], y, xt, lg, rg, np.ones_like(y))
        xg = need("transpose")(cols, rows, rg)      # transpose_grad(cols, rows, x.grad, out.grad)
        expect = need("transpose")(cols, rows, y)
        check(xg, expect, tol, c["name"])
    elif fn == "gemm":
        check(need("gemm")(c["m"], c["n"], c["k"], f32(c["lhs"]), f32(c["rhs"])), c["expect"], tol, c["name"])
    elif fn == "gemm_with_grad":
        m, k, n = c["m"], c["k"], c["n"]
        lhs, rhs = f32(c["lhs"]), f32(c["rhs"])
        check(need("gemm")(m, n, k, lhs, rhs), c["expect"], tol, c["name"])
        lg, rg = np.zeros_like(lhs), np.zeros_like(rhs)
        need("gemm_grad")(m, k, n, lhs, rhs, lg, rg, np.ones(m * n, np.float32))
        check(lg, c["expect_lhs_grad"], tol, c["name"])
        check(rg, c["expect_rhs_grad"], tol, c["name"])
    elif fn == "Tgemm_eq":
        m, n, k = c["m"], c["n"], c["k"]
        a, b = f32(c["a"]), f32(c["b"])              # a stored k×m
        at = need("transpose")(k, m, a)
        check(need("Tgemm")(m, n, k, a, b), need("gemm")(m, n, k, at, b), tol, c["name"])
    elif fn == "gemmT_eq":
        m, n, k = c["m"], c["n"], c["k"]
        a, b = f32(c["a"]), f32(c["b"])              # b stored n×k
        bt = need("transpose")(n, k, b)
        check(need("gemmT")(m, n, k, a, b), need("gemm")(m, n, k, a, bt), tol, c["name"])
    elif fn == "softmax":
        check(need(fn)(c["samples"], c["features"], f32(c["x"])), c["expect"], tol, c["name"])
    elif fn == "softmax_grad":
        s = need("softmax")(c["samples"], c["features"], f32(c["x"]))
        check(need(fn)(c["samples"], c["features"], s, f32(c["out_grad"])), c["expect"], tol, c["name"])
        jac = getattr(be, "softmax_grad_jacobian", None)
        if jac is not None:
            check(jac(c["samples"], c["features"], s, f32(c["out_grad"])), c["expect"], tol, c["name"])
    elif fn == "diagflat":
        check(need(fn)(f32(c["x"])), c["expect"], tol, c["name"])
    elif fn == "onehot":
        check(need(fn)(c["highest_class"], f32(c["classes"])), c["expect"], tol, c["name"])
    elif fn == "reduce_then_binary_grad":
        x, rhs, cols = f32(c["x"]), f32(c["rhs"]), c["cols"]
        red = need(c["reduce"])(cols, x)
        lg, rg = np.zeros_like(red), np.zeros_like(rhs)
        need("binary_ew_grad")(OPS[c["op"]], red, rhs, lg, rg, np.ones_like(red))
        xg = np.zeros_like(x)
        if c["reduce"].startswith("max"):
            need(c["reduce"] + "_grad")(cols, red, x, xg, lg)
        else:
            need(c["reduce"] + "_grad")(cols, xg, lg)
        check(xg, c["expect_x_grad"], tol, c["name"])
        check(rg, c["expect_rhs_grad"], tol, c["name"])
    elif fn == "mean_rows_sub_grad":
        x, lhs, cols = f32(c["x"]), f32(c["lhs"]), c["cols"]
        mr = need("mean_rows")(cols, x)
        lg, rg = np.zeros_like(lhs), np.zeros_like(mr)
        need("binary_ew_grad")(OPS["sub"], lhs, mr, lg, rg, np.ones_like(lhs))
        xg = np.zeros_like(x)
        need("mean_rows_grad")(cols, xg, rg)
        check(xg, c["expect_x_grad"], tol, c["name"])
        check(lg, c["expect_lhs_grad"], tol, c["name"])
    elif fn == "l2_norm_cols_grad":
        rows, cols = c["rows"], c["cols"]
        x = f32(c["x"])
        sq = need("unary")(UN["square"], x)
        sc = need("sum_cols")(cols, sq)
        g_sc = need("unary_grad")(UN["pow"], sc, np.zeros_like(sc), np.ones_like(sc), 0.5)
        g_sq = need("sum_cols_grad")(cols, np.zeros_like(x), g_sc)
        g_x = need("unary_grad")(UN["square"], x, np.zeros_like(x), g_sq)
        check(g_x[:cols], c["expect_first_row"], tol, c["name"])
    elif fn == "chain5":
        n = 7
        x, b = np.full(n, c["x"], np.float32), np.full(n, c["b"], np.float32)
        squared = need("unary")(UN["square"], x)
        add = need("binary_ew")(OPS["add"], b, x)
        mul_b = need("binary_ew")(OPS["mul"], add, b)
        mul = need("binary_ew")(OPS["mul"], squared, x)
        out = need("binary_ew")(OPS["add"], mul, mul_b)
        check(out, np.full(n, c["expect"], np.float32), tol, c["name"])
    else:
        raise AssertionError("unknown golden fn " + fn)
