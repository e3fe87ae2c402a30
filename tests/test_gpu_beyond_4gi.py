"""Tensors of more than 2^32 elements (16 GiB and up) through the C ABI: every index computation on
the path has to be 64 bits wide.  The operands come from the device generator, whose value at any
index the host can recompute, so results are checked on windows (the first elements, the elements
either side of index 2^32, the last ones) against numpy on the same values, and through properties
that hold at any size (a reduction of the whole equals the reduction of its parts; a transpose
taken twice is the identity).  Bars as for the small shapes: bit-exact for data movement, maxima
and single-operation elementwise work, the summation bounds for sums, 1e-6 relative for softmax.

Needs about 50 GiB of device memory; skipped when the device has less free.
"""
import ctypes as C
import sys

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu

SEED = rng.DEFAULT_SEED
ROWS, COLS = 65553, 65536            # 2^32 + 17 * 2^16 elements
N = ROWS * COLS
ODD = 65537                          # ODD x ODD = 2^32 + 2^17 + 1 elements, both sides odd
LO, HI = -1.0, 1.0
TWO32 = 1 << 32
CAP = N + (1 << 23)                  # elements per buffer: every shape below fits
ADD, SUB, MUL = 0, 1, 2              # SLHIP_ADD .. (include/sliced_hip.h)
RELU, SCALE = 2, 6                   # SLHIP_RELU, SLHIP_SCALE


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


from devgen import host_values, host_range  # noqa: E402  (the generator's values at any index)


WINDOWS = [(0, 8192), (TWO32 - 4096, 8192), (N - 8192, 8192)]


@pytest.fixture(scope="module")
def big():
    from sliced_amd.device import Context
    rt = C.CDLL("libamdhip64.so.7")
    free, total = C.c_size_t(), C.c_size_t()
    ctx = Context(0)   # (the library's own runtime is initialised now)
    assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    if free.value < (56 << 30):
        ctx.close()
        pytest.skip("needs 56 GiB of free device memory, %d GiB are free" % (free.value >> 30))
    say("allocating three buffers of", CAP, "floats")
    x = ctx.uniform(CAP, LO, HI, 0, SEED)
    y = ctx.empty(CAP)
    z = ctx.empty(CAP)
    small = ctx.zeros(1 << 20)
    yield ctx, x, y, z, small
    for b in (x, y, z, small):
        b.free()
    ctx.close()


def test_generator_beyond_index_2_32(big):
    ctx, x, y, z, small = big
    for start, n in WINDOWS:
        say("generator window", start, n)
        assert np.array_equal(x.view(start, n).numpy(), host_range(start, n, 0))


def test_copy_fill_and_elementwise(big):
    ctx, x, y, z, small = big
    say("memcpy_d2d", N)
    ctx.call("slhip_memcpy_d2d", y.ptr, x.ptr, 4 * N)
    for start, n in WINDOWS:
        assert np.array_equal(y.view(start, n).numpy(), host_range(start, n, 0))
    say("ew_unary relu", N)
    ctx.call("slhip_ew_unary", RELU, 0.0, 0.0, N, x.ptr, z.ptr)
    for start, n in WINDOWS:
        h = host_range(start, n, 0)
        assert np.array_equal(z.view(start, n).numpy(), (h >= 0).astype(np.float32) * h)
    say("ew_binary mul", N)
    ctx.call("slhip_ew_binary", MUL, N, x.ptr, z.ptr, y.ptr)
    for start, n in WINDOWS:
        h = host_range(start, n, 0)
        assert np.array_equal(y.view(start, n).numpy(), h * ((h >= 0).astype(np.float32) * h))
    say("fill", N)
    ctx.call("slhip_fill", N, 0.5, z.ptr)
    for start, n in WINDOWS:
        assert np.all(z.view(start, n).numpy() == np.float32(0.5))
    say("sgd_step", N)
    ctx.call("slhip_sgd_step", N, z.ptr, x.ptr, 0.25)   # z = 0.5 - 0.25 * x
    for start, n in WINDOWS:
        h = host_range(start, n, 0)
        assert np.array_equal(z.view(start, n).numpy(), np.float32(0.5) - np.float32(0.25) * h)
    say("ew_binary add, in place", N)
    ctx.call("slhip_ew_binary", ADD, N, z.ptr, x.ptr, z.ptr)
    for start, n in WINDOWS:
        h = host_range(start, n, 0)
        assert np.array_equal(z.view(start, n).numpy(), (np.float32(0.5) - np.float32(0.25) * h) + h)


def test_whole_buffer_reductions_equal_those_of_their_parts(big):
    ctx, x, y, z, small = big
    parts = [(0, 1 << 30), (1 << 30, 1 << 31), (3 << 30, N - (3 << 30))]
    say("sum / max / mean of", N)
    ctx.call("slhip_sum", N, x.ptr, small.view(0, 1).ptr)
    ctx.call("slhip_max", N, x.ptr, small.view(1, 1).ptr)
    ctx.call("slhip_mean", N, x.ptr, small.view(2, 1).ptr)
    for i, (s, n) in enumerate(parts):
        ctx.call("slhip_sum", n, x.view(s, n).ptr, small.view(8 + i, 1).ptr)
        ctx.call("slhip_max", n, x.view(s, n).ptr, small.view(16 + i, 1).ptr)
    r = small.view(0, 32).numpy()
    assert r[1] == max(r[16:19])
    # sum|x| is N / 2 for this generator to within a part in a thousand: the bound of the small shapes
    bound = 1e-6 * 0.5 * N
    psum = float(np.sum(r[8:11].astype(np.float64)))
    say("  sum", r[0], "parts", psum, "bound", bound)
    assert abs(float(r[0]) - psum) <= bound
    assert abs(float(r[2]) - psum / N) <= 1e-6 * 0.5
    # and the tail beyond 2^32 on its own, against the host
    tail = N - TWO32
    ctx.call("slhip_sum", tail, x.view(TWO32, tail).ptr, small.view(3, 1).ptr)
    h = host_range(TWO32, tail, 0)
    assert abs(float(small.view(3, 1).numpy()[0]) - h.sum(dtype=np.float64)) <= 1e-6 * np.abs(h).sum(dtype=np.float64)


def test_row_and_column_reductions(big):
    ctx, x, y, z, small = big
    vr, vc, vc2, vc3 = small.view(0, ROWS), small.view(1 << 17, COLS), small.view(2 << 17, COLS), small.view(3 << 17, COLS)
    top = 32768
    say("sum_cols / max_cols", ROWS, COLS)
    ctx.call("slhip_sum_cols", ROWS, COLS, x.ptr, vr.ptr)
    s = vr.numpy()
    ctx.call("slhip_max_cols", ROWS, COLS, x.ptr, vr.ptr)
    m = vr.numpy()
    for r in (0, 1, 32767, 65535, 65536, 65537, ROWS - 1):
        h = host_range(r * COLS, COLS, 0)
        assert m[r] == h.max(), r
        assert abs(float(s[r]) - h.sum(dtype=np.float64)) <= 1e-6 * np.abs(h).sum(dtype=np.float64), r
    ctx.call("slhip_sum", N, x.ptr, small.view(4 << 17, 1).ptr)
    assert abs(s.sum(dtype=np.float64) - float(small.view(4 << 17, 1).numpy()[0])) <= 2e-6 * 0.5 * N
    say("sum_rows / max_rows", ROWS, COLS)
    ctx.call("slhip_max_rows", ROWS, COLS, x.ptr, vc.ptr)
    ctx.call("slhip_max_rows", top, COLS, x.ptr, vc2.ptr)
    ctx.call("slhip_max_rows", ROWS - top, COLS, x.view(top * COLS, (ROWS - top) * COLS).ptr, vc3.ptr)
    assert np.array_equal(vc.numpy(), np.maximum(vc2.numpy(), vc3.numpy()))
    ctx.call("slhip_sum_rows", ROWS, COLS, x.ptr, vc.ptr)
    ctx.call("slhip_sum_rows", top, COLS, x.ptr, vc2.ptr)
    ctx.call("slhip_sum_rows", ROWS - top, COLS, x.view(top * COLS, (ROWS - top) * COLS).ptr, vc3.ptr)
    whole, parts = vc.numpy().astype(np.float64), vc2.numpy().astype(np.float64) + vc3.numpy().astype(np.float64)
    assert np.all(np.abs(whole - parts) <= 1e-6 * 0.5 * ROWS * 1.2)
    # a handful of columns against the host: column c is the elements c, c + COLS, ...
    for c in (0, 1, 4095, COLS - 1):
        h = host_values(np.arange(ROWS, dtype=np.uint64) * np.uint64(COLS) + np.uint64(c), 0)
        assert abs(whole[c] - h.sum(dtype=np.float64)) <= 1e-6 * np.abs(h).sum(dtype=np.float64), c
        ctx.call("slhip_max_rows", ROWS, COLS, x.ptr, vc2.ptr)
        assert vc2.numpy()[c] == h.max()
    say("add_row", ROWS, COLS)
    bias = host_range(5, COLS, 0)
    vc.upload(bias)
    ctx.call("slhip_add_row", ROWS, COLS, x.ptr, vc.ptr, y.ptr)
    for start, n in WINDOWS:
        cols = (np.arange(start, start + n) % COLS)
        assert np.array_equal(y.view(start, n).numpy(), host_range(start, n, 0) + bias[cols])


@pytest.mark.parametrize("shape", [(ROWS, COLS), (COLS, ROWS), (ODD, ODD), (4099, 1047937), (1047937, 4099), (429500001, 10), (10, 429500001)],
                         ids=lambda s: "%dx%d" % s)
def test_transpose(big, shape):
    ctx, x, y, z, small = big
    rows, cols = shape
    n = rows * cols
    assert n > TWO32 and n <= CAP
    say("transpose", rows, cols)
    ctx.call("slhip_transpose", rows, cols, x.ptr, y.ptr, 0.0)
    # windows of the result against the generator: out[c * rows + r] = x[r * cols + c]
    for start, m in [(0, 8192), (TWO32 - 4096, 8192), (n - 8192, 8192), (n // 2 - 333, 4096)]:
        o = np.arange(start, start + m, dtype=np.uint64)
        c, r = o // np.uint64(rows), o % np.uint64(rows)
        assert np.array_equal(y.view(start, m).numpy(), host_values(r * np.uint64(cols) + c, 0)), (start, m)
    # and back: the identity on every element, checked on the device (max |x - x''| = 0)
    ctx.call("slhip_transpose", cols, rows, y.ptr, z.ptr, 0.0)
    ctx.call("slhip_ew_binary", SUB, n, z.ptr, x.ptr, z.ptr)
    ctx.call("slhip_max", n, z.ptr, small.view(0, 1).ptr)
    ctx.call("slhip_ew_unary", SCALE, -1.0, 0.0, n, z.ptr, z.ptr)
    ctx.call("slhip_max", n, z.ptr, small.view(1, 1).ptr)
    d = small.view(0, 2).numpy()
    assert d[0] == 0.0 and d[1] == 0.0, d


def softmax_rows_f64(h):
    e = np.exp(h.astype(np.float64) - h.max(axis=1, keepdims=True).astype(np.float64))
    return e / e.sum(axis=1, keepdims=True)


@pytest.mark.parametrize("cols", [4096, 1048583, 10, 40007], ids=lambda c: "rows_of_%d" % c)
def test_softmax_and_its_gradient(big, cols):
    ctx, x, y, z, small = big
    rows = (TWO32 + 2 * cols) // cols + 3
    n = rows * cols
    assert n + 1 <= CAP
    say("softmax", rows, cols)
    ctx.call("slhip_softmax", rows, cols, x.ptr, y.ptr)
    pick = sorted({0, 1, TWO32 // cols - 1, TWO32 // cols, TWO32 // cols + 1, rows - 1})
    for r in pick:
        h = host_range(r * cols, cols, 0).reshape(1, cols)
        ref = softmax_rows_f64(h).ravel()
        got = y.view(r * cols, cols).numpy()
        assert np.all(np.abs(got - ref) <= 2e-6 * ref + 1e-37), (r, float(np.max(np.abs(got - ref) / ref)))
    say("softmax_grad", rows, cols)
    # upstream gradient: the input itself, shifted by one element (any values do)
    ctx.call("slhip_softmax_grad", rows, cols, z.ptr, y.ptr, x.view(1, n).ptr, 0.0)
    for r in pick:
        s = y.view(r * cols, cols).numpy().astype(np.float64)
        g = host_range(r * cols + 1, cols, 0).astype(np.float64)
        ref = s * (g - np.dot(s, g))
        got = z.view(r * cols, cols).numpy()
        bound = 2e-6 * (np.abs(s) * (np.abs(g) + np.dot(np.abs(s), np.abs(g)))) + 1e-37
        assert np.all(np.abs(got - ref) <= bound), r


def test_products_with_an_operand_beyond_2_32_elements(big):
    ctx, x, y, z, small = big
    # tall A (rows x 4096) times a narrow and a wider B; A^T * B with the same A stored K x M
    k = 4096
    m = TWO32 // k + 48
    for nn in (16, 10, 64):
        say("A * B", m, nn, k)
        b = rng.uniform(k * nn, -1, 1, 5, SEED)
        small.view(0, k * nn).upload(b)
        ctx.call("slhip_sgemm", 0, 0, m, nn, k, x.ptr, small.ptr, y.ptr, 0.0)
        B = b.reshape(k, nn).astype(np.float64)
        for r0 in (0, TWO32 // k - 8, m - 16):
            A = host_range(r0 * k, 16 * k, 0).reshape(16, k).astype(np.float64)
            got = y.view(r0 * nn, 16 * nn).numpy().reshape(16, nn)
            assert np.all(np.abs(got - A @ B) <= 3e-6 * (np.abs(A) @ np.abs(B))), (nn, r0)
    for nn in (16, 10, 64):
        say("At * B as the sum of two halves", k, nn, m)
        g = ctx.uniform(m * nn, -1, 1, 6, SEED)
        out = small.view(0, k * nn)
        ctx.call("slhip_sgemm", 1, 0, k, nn, m, x.ptr, g.ptr, out.ptr, 0.0)
        whole = out.numpy().astype(np.float64)
        half = m // 2
        ctx.call("slhip_sgemm", 1, 0, k, nn, half, x.ptr, g.ptr, out.ptr, 0.0)
        ctx.call("slhip_sgemm", 1, 0, k, nn, m - half, x.view(half * k, (m - half) * k).ptr, g.view(half * nn, (m - half) * nn).ptr,
                 out.ptr, 1.0)
        parts = out.numpy().astype(np.float64)
        # |A| |B| per element is about m / 4 for operands uniform in (-1, 1)
        assert np.all(np.abs(whole - parts) <= 3e-6 * 0.25 * m), float(np.max(np.abs(whole - parts)))
        # the last 4096 k on their own against the host (they lie beyond element 2^32 of A)
        last = 4096
        ctx.call("slhip_sgemm", 1, 0, k, nn, last, x.view((m - last) * k, last * k).ptr, g.view((m - last) * nn, last * nn).ptr,
                 out.ptr, 0.0)
        A = host_range((m - last) * k, last * k, 0).reshape(last, k).astype(np.float64)
        G = rng.raw_u24(last * nn, 6, SEED, start=(m - last) * nn).astype(np.float32) * np.float32(2.0 ** -24)
        G = (np.float32(-1) + np.float32(2) * G).astype(np.float32).reshape(last, nn).astype(np.float64)
        assert np.all(np.abs(out.numpy().reshape(k, nn) - A.T @ G) <= 3e-6 * (np.abs(A).T @ np.abs(G)))
        g.free()
    # a square-ish product whose A has more than 2^32 elements
    mm, nn, kk = 65552, 256, 65536
    say("A * B", mm, nn, kk)
    b = rng.uniform(kk * nn, -1, 1, 7, SEED)
    bb = ctx.array(b)
    ctx.call("slhip_sgemm", 0, 0, mm, nn, kk, x.ptr, bb.ptr, y.ptr, 0.0)
    B = b.reshape(kk, nn).astype(np.float64)
    for r0 in (0, 65535, mm - 2):
        A = host_range(r0 * kk, 2 * kk, 0).reshape(2, kk).astype(np.float64)
        got = y.view(r0 * nn, 2 * nn).numpy().reshape(2, nn)
        assert np.all(np.abs(got - A @ B) <= 3e-6 * (np.abs(A) @ np.abs(B))), r0
    bb.free()


def test_reduction_gradients_and_broadcast_ops(big):
    ctx, x, y, z, small = big
    vr, vc = small.view(0, ROWS), small.view(1 << 17, COLS)
    gr, gc = host_range(100, ROWS, 3), host_range(200, COLS, 3)
    small.view(2 << 17, ROWS).upload(gr)
    small.view(3 << 17, COLS).upload(gc)
    dgr, dgc = small.view(2 << 17, ROWS), small.view(3 << 17, COLS)
    row_of = lambda start, n: np.arange(start, start + n) // COLS
    col_of = lambda start, n: np.arange(start, start + n) % COLS
    say("sum_cols_grad / sum_rows_grad into a filled gradient", ROWS, COLS)
    ctx.call("slhip_fill", N, 0.5, y.ptr)
    ctx.call("slhip_sum_cols_grad", ROWS, COLS, y.ptr, dgr.ptr)
    for start, n in WINDOWS:
        assert np.array_equal(y.view(start, n).numpy(), np.float32(0.5) + gr[row_of(start, n)])
    ctx.call("slhip_fill", N, 0.5, y.ptr)
    ctx.call("slhip_sum_rows_grad", ROWS, COLS, y.ptr, dgc.ptr)
    for start, n in WINDOWS:
        assert np.array_equal(y.view(start, n).numpy(), np.float32(0.5) + gc[col_of(start, n)])
    say("max_cols_grad (first maximum of a row)", ROWS, COLS)
    ctx.call("slhip_max_cols", ROWS, COLS, x.ptr, vr.ptr)
    ctx.call("slhip_memset", y.ptr, 0, 4 * N)
    ctx.call("slhip_max_cols_grad", ROWS, COLS, vr.ptr, x.ptr, y.ptr, dgr.ptr)
    for r in (0, 65535, 65536, ROWS - 1):
        h = host_range(r * COLS, COLS, 0)
        want = np.zeros(COLS, np.float32)
        want[int(np.argmax(h))] = gr[r]
        assert np.array_equal(y.view(r * COLS, COLS).numpy(), want), r
    ctx.call("slhip_sum", N, y.ptr, small.view(5 << 17, 1).ptr)   # one entry per row and nothing else
    assert abs(float(small.view(5 << 17, 1).numpy()[0]) - gr.sum(dtype=np.float64)) <= 1e-6 * np.abs(gr).sum(dtype=np.float64)
    say("max_rows_grad (every maximum of a column)", ROWS, COLS)
    ctx.call("slhip_max_rows", ROWS, COLS, x.ptr, vc.ptr)
    m = vc.numpy()
    ctx.call("slhip_memset", y.ptr, 0, 4 * N)
    ctx.call("slhip_max_rows_grad", ROWS, COLS, vc.ptr, x.ptr, y.ptr, dgc.ptr)
    for start, n in WINDOWS:
        h = host_range(start, n, 0)
        c = col_of(start, n)
        assert np.array_equal(y.view(start, n).numpy(), np.where(h == m[c], gc[c], np.float32(0)))
    say("col_op sub / row_op mul and their gradients", ROWS, COLS)
    ctx.call("slhip_col_op", SUB, ROWS, COLS, x.ptr, dgr.ptr, y.ptr)
    for start, n in WINDOWS:
        assert np.array_equal(y.view(start, n).numpy(), host_range(start, n, 0) - gr[row_of(start, n)])
    ctx.call("slhip_row_op", MUL, ROWS, COLS, x.ptr, dgc.ptr, y.ptr)
    for start, n in WINDOWS:
        assert np.array_equal(y.view(start, n).numpy(), host_range(start, n, 0) * gc[col_of(start, n)])
    # row_op mul: lhs_grad += rhs[c] * g, rhs_grad[c] += sum_r lhs[r,c] * g[r,c]; with g = 1 the latter is sum_rows(x)
    ctx.call("slhip_fill", N, 1.0, y.ptr)
    ctx.call("slhip_memset", z.ptr, 0, 4 * N)
    ctx.call("slhip_memset", vc.ptr, 0, 4 * COLS)
    ctx.call("slhip_row_op_grad", MUL, ROWS, COLS, x.ptr, dgc.ptr, z.ptr, vc.ptr, y.ptr)
    for start, n in WINDOWS:
        assert np.array_equal(z.view(start, n).numpy(), gc[col_of(start, n)])
    rhs_grad = vc.numpy().astype(np.float64)
    ctx.call("slhip_sum_rows", ROWS, COLS, x.ptr, vc.ptr)
    assert np.all(np.abs(rhs_grad - vc.numpy().astype(np.float64)) <= 1e-6 * 0.5 * ROWS * 1.2)
    # col_op sub: lhs_grad += g, rhs_grad[r] -= sum_c g[r,c]; with g = x the latter is -sum_cols(x)
    ctx.call("slhip_memset", vr.ptr, 0, 4 * ROWS)
    ctx.call("slhip_col_op_grad", SUB, ROWS, COLS, x.ptr, dgr.ptr, None, vr.ptr, x.ptr)
    rhs_grad = vr.numpy().astype(np.float64)
    ctx.call("slhip_sum_cols", ROWS, COLS, x.ptr, vr.ptr)
    assert np.all(np.abs(rhs_grad + vr.numpy().astype(np.float64)) <= 1e-6 * 0.5 * COLS * 1.2)


def test_elementwise_chain_and_gradients(big):
    ctx, x, y, z, small = big
    say("ew_chain", N)
    # ((a + b) * c - d)^2, squared, with a = x, b = x shifted by 1, c = x shifted by 2, d = x shifted by 3
    n = N
    ctx.call("slhip_ew_chain", n, x.ptr, x.view(1, n).ptr, x.view(2, n).ptr, x.view(3, n).ptr, y.ptr)
    for start, m in WINDOWS:
        h = host_range(start, m + 3, 0)
        a, b, c, d = h[:m], h[1:m + 1], h[2:m + 2], h[3:m + 3]
        t = (a + b) * c - d
        t = t * t
        want = (t * t).astype(np.float64)
        assert np.all(np.abs(y.view(start, m).numpy() - want) <= 1e-6 * want), start   # (pow's last bit is the device library's)
    say("unary gradient (square) accumulating", N)
    SQUARE = 0
    ctx.call("slhip_fill", N, 0.25, z.ptr)
    ctx.call("slhip_ew_unary_grad", SQUARE, 0.0, N, x.ptr, z.ptr, x.view(1, N).ptr)   # z += 2 x * g
    for start, m in WINDOWS:
        h = host_range(start, m + 1, 0)
        want = np.float32(0.25) + (np.float32(2) * h[:m]) * h[1:m + 1]
        got = z.view(start, m).numpy()
        assert np.all(np.abs(got - want) <= 2.4e-7 * (0.25 + 2 * np.abs(h[:m] * h[1:m + 1]))), start
    say("binary gradient (mul) into both sides", N)
    ctx.call("slhip_memset", y.ptr, 0, 4 * N)
    ctx.call("slhip_memset", z.ptr, 0, 4 * N)
    ctx.call("slhip_ew_binary_grad", MUL, N, x.ptr, x.view(1, N).ptr, y.ptr, z.ptr, x.view(2, N).ptr)
    for start, m in WINDOWS:
        h = host_range(start, m + 2, 0)
        assert np.array_equal(y.view(start, m).numpy(), h[1:m + 1] * h[2:m + 2]), start
        assert np.array_equal(z.view(start, m).numpy(), h[:m] * h[2:m + 2]), start


@pytest.mark.parametrize("k", [32, 8, 1], ids=lambda k: "k%d" % k)
def test_product_with_a_result_beyond_2_32_elements(big, k):
    ctx, x, y, z, small = big
    m = nn = 65552
    say("A * B, A * Bt with", m * nn, "results, k =", k)
    a, b = host_range(0, m * k, 0), host_range(m * k, k * nn, 0)
    A = a.reshape(m, k).astype(np.float64)
    for tb in (0, 1):
        B = (b.reshape(nn, k).T if tb else b.reshape(k, nn)).astype(np.float64)
        ctx.call("slhip_sgemm", 0, tb, m, nn, k, x.ptr, x.view(m * k, k * nn).ptr, y.ptr, 0.0)
        for r in (0, 1, 65535, 65536, m - 1):           # row 65535 ends just short of element 2^32 of C
            got = y.view(r * nn, nn).numpy()
            want, scale = A[r] @ B, np.abs(A[r]) @ np.abs(B)
            assert np.all(np.abs(got - want) <= 3e-6 * scale), (k, tb, r)
