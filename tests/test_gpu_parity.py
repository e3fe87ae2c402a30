"""HIP path vs the CPU oracle, through the C ABI, on identical seeded inputs.

Bars (stated per test):
  * transpose, max_rows, max_cols and every op that is a single IEEE operation per element:
    bit-exact;
  * sums / means: |gpu - oracle| <= 1e-6 * sum|x| per output (the oracle's sequential f32 sum is
    itself off the exact sum by more than 1e-6 relative for long rows, so the bound is written on
    the backward-error scale), and |gpu - exact| <= the same bound;
  * softmax fwd/bwd, pow/exp/ln: 1e-6 relative per element against the f64 evaluation, and against
    the oracle with the oracle's own distance to the f64 evaluation added;
  * GEMM: |gpu - exact| <= 1e-5 * sqrt(K) * (|A|·|B|) elementwise.
"""
import ctypes as C
import sys

import numpy as np
import pytest

import golden_cases as gc
from sliced_amd import rng

pytestmark = pytest.mark.gpu

SEED = rng.DEFAULT_SEED


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


# --------------------------------------------------------------------------- golden vectors
CASES = gc.load_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"][:50] for c in CASES])
def test_hip_matches_reference_vector(hip, case):
    try:
        gc.run_case(hip, case)
    except gc.Unsupported as e:
        pytest.skip("not part of the device path: %s" % e)


# --------------------------------------------------------------------------- generator
def test_device_generator_is_bit_identical_to_host(hip):
    for n, lo, hi, tag in [(1, -1, 1, 0), (1000, -10, 10, 3), (1 << 20, 0, 1, 7), (12345, -3.5, 0.25, 9)]:
        say("rand_uniform", n, lo, hi, tag)
        d = hip.rand_uniform(n, lo, hi, tag, SEED)
        h = rng.uniform(n, lo, hi, tag, SEED)
        assert np.array_equal(d, h)


# --------------------------------------------------------------------------- GEMM
GEMM_SHAPES = [
    (1, 1, 1), (4, 3, 2), (5, 10, 7), (33, 65, 17), (64, 64, 64), (128, 128, 16), (128, 128, 128),
    (129, 127, 130), (256, 384, 200), (100, 10, 300), (300, 10, 2048), (1024, 64, 1), (1024, 1, 64),
    (1, 64, 1024), (64, 1, 1024), (384, 256, 784), (200, 136, 1000), (512, 512, 512),
    # one wave per 32x32 tile: k split over waves and over the grid, skinny sides, ragged edges
    (32, 32, 100003), (2000, 10, 1000), (40, 1000, 10), (16, 3000, 500), (31, 33, 4099), (96, 64, 64),
    # K off the multiples of 8 on that kernel: whole groups of 8 k, then one checked group of 1..7
    (257, 17, 3333), (17, 257, 3335), (100, 100, 1001), (48, 48, 9), (40, 72, 15), (70, 30, 8),
]


def gemm_operands(ta, tb, m, n, k):
    a = rng.uniform(m * k, -1, 1, tag=0, seed=SEED + m + 7 * n + 13 * k)
    b = rng.uniform(k * n, -1, 1, tag=1, seed=SEED + m + 7 * n + 13 * k)
    return a, b


def gemm_bound(ta, tb, m, n, k, a, b):
    A = a.reshape(k, m).T if ta else a.reshape(m, k)
    B = b.reshape(n, k).T if tb else b.reshape(k, n)
    exact = A.astype(np.float64) @ B.astype(np.float64)
    scale = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    return exact.ravel(), (1e-5 * np.sqrt(k) * scale + 1e-30).ravel()


@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("form", ["gemm", "gemmT", "Tgemm"])
def test_gemm_forms(hip, orc, shape, form):
    m, n, k = shape
    ta, tb = form == "Tgemm", form == "gemmT"
    say("gemm", form, m, n, k)
    a, b = gemm_operands(ta, tb, m, n, k)
    exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
    got = getattr(hip, form)(m, n, k, a, b)
    ref = getattr(orc, form)(m, n, k, a, b)
    assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
    assert np.all(np.abs(got - ref) <= bound)
    # beta = 1 accumulates into C (`Assign`)
    c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
    got1 = getattr(hip, form)(m, n, k, a, b, c=c0.copy(), beta=1.0)
    assert np.all(np.abs(got1 - (exact + c0)) <= bound + 1e-6 * np.abs(c0))


def test_gemm_split_k_and_large_tiles(hip, orc):
    # shapes whose tile grid is small enough that the K dimension is split
    for (m, n, k, ta, tb) in [(256, 256, 4096, 0, 0), (200, 136, 5000, 1, 0), (128, 384, 3000, 0, 1),
                              (784, 512, 2048, 1, 0)]:
        say("split-k gemm", m, n, k, ta, tb)
        a, b = gemm_operands(ta, tb, m, n, k)
        exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
        got = hip.sgemm(ta, tb, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        got1 = hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0)
        assert np.all(np.abs(got1 - (exact + c0)) <= bound + 1e-6 * np.abs(c0))


def test_gemm_spread_tail(hip, orc):
    # tile grids that do not fill the last round of workgroups: the k range of the last round's
    # tiles is spread over one more round, partial tiles are summed in a fixed order.  Forced here,
    # so that small shapes (a tail of 64 tiles, nothing but tail; edge tiles; k remainders; odd
    # leading dimensions) take the path, and compared with the whole-tile path as well.
    shapes = [(1000, 1000, 512, 0, 0), (1024, 1024, 1000, 1, 0), (640, 640, 4096, 0, 1), (999, 1001, 515, 0, 0),
              (129, 257, 4099, 1, 0), (2945, 3001, 290, 0, 1), (3000, 3000, 256, 0, 0), (3100, 2900, 321, 1, 0)]
    try:
        for (m, n, k, ta, tb) in shapes:
            say("spread gemm", m, n, k, ta, tb)
            a, b = gemm_operands(ta, tb, m, n, k)
            exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
            hip.gemm_tail_policy(hip.TAIL_SPREAD)
            got = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
            assert np.array_equal(got, hip.sgemm(ta, tb, m, n, k, a, b))  # same bits on every run
            c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
            got1 = hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0)
            assert np.array_equal(got1, got + c0)
            hip.gemm_tail_policy(hip.TAIL_WHOLE)
            whole = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - whole) <= 2 * bound)
            if not ta and not tb:  # the fused Linear epilogue on the spread path
                bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
                hip.gemm_tail_policy(hip.TAIL_SPREAD)
                out, pre = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
                pre_ref = orc.add_row(m, n, got, bias)
                assert np.array_equal(pre, pre_ref)
                assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
        # the default policy on a grid of 576 tiles with a long k
        hip.gemm_tail_policy(hip.TAIL_AUTO)
        m, n, k = 2945, 3001, 1024
        say("spread gemm, default policy", m, n, k)
        a, b = gemm_operands(0, 0, m, n, k)
        exact, bound = gemm_bound(0, 0, m, n, k, a, b)
        got = hip.sgemm(0, 0, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
    finally:
        hip.gemm_tail_policy(hip.TAIL_AUTO)


def test_gemm_skinny_kernels(hip, orc):
    """K <= 12 with a large result (vector-ALU kernel, rows of A staged in LDS) in all four forms with
    every epilogue, and A^T * B with N <= 16 and a long K (A streamed once, k split over workgroups
    and waves, partials combined in a fixed order): N in {1, 3, 10, 16} and between, K odd, K shorter
    and longer than a workgroup's chunk, M not a multiple of the 256 columns of a workgroup."""
    for (m, n, k, ta, tb) in [(1031, 260, 10, 0, 1), (4100, 64, 1, 0, 0), (1500, 512, 12, 1, 0), (2050, 1028, 7, 1, 1),
                              (8192, 2048, 10, 0, 1), (3000, 96, 4, 0, 1), (1111, 256, 9, 0, 0), (1024, 1024, 5, 0, 1),
                              (1400, 200, 11, 0, 1), (1400, 200, 8, 1, 1)]:
        say("short-K gemm", m, n, k, ta, tb)
        a, b = gemm_operands(ta, tb, m, n, k)
        exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
        got = hip.sgemm(ta, tb, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
        assert np.array_equal(hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre, c=c0.copy(), beta=1.0),
                              c0 + np.where(pre >= 0, got, 0 * got))
        if not ta and not tb:
            bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
            out, pre_act = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
            pre_ref = orc.add_row(m, n, got, bias)
            assert np.array_equal(pre_act, pre_ref)
            assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
    for (m, n, k) in [(2048, 10, 8192), (1028, 1, 4133), (1028, 3, 4133), (4100, 4, 1000), (4100, 13, 1030), (1024, 16, 5000),
                      (260, 8, 20000), (5000, 12, 900), (2052, 5, 2048), (1024, 9, 70000)]:
        say("narrow-N gemm", m, n, k)
        a, b = gemm_operands(1, 0, m, n, k)
        exact, bound = gemm_bound(1, 0, m, n, k, a, b)
        got = hip.sgemm(1, 0, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        assert np.array_equal(got, hip.sgemm(1, 0, m, n, k, a, b))          # same plan, same order of sums
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(1, 0, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(1, 0, m, n, k, a, b, pre, c=c0.copy(), beta=1.0),
                              c0 + np.where(pre >= 0, got, 0 * got))


def test_gemm_rows_narrow_kernel(hip, orc):
    """A * B with N <= 16 and a large row-major A (the classifier head's forward product): the
    sixteen-block matrix-instruction kernel.  N in {1, 3, 10, 16} and the sizes between, K a multiple
    of 4 that is not one of 64, shorter than a chunk, longer than one and than two, M not a multiple
    of 4 or of the workgroup's 32 rows, every epilogue, and a row of A that holds an inf (it must not
    leak into other rows through the zero padding)."""
    for (m, n, k) in [(8192, 10, 2048), (2049, 1, 2048), (4099, 3, 2052), (33000, 16, 260), (1030, 13, 4100), (2048, 8, 6148),
                      (4096, 5, 1024), (16385, 12, 256), (3001, 10, 2000), (70000, 2, 64 * 5 + 4),
                      # few long rows: the chunks of K shared out over several workgroups per row group
                      (2048, 1, 65536), (513, 10, 30000), (64, 16, 131072 + 4), (1000, 3, 8192)]:
        say("rows-narrow gemm", m, n, k)
        a, b = gemm_operands(0, 0, m, n, k)
        exact, bound = gemm_bound(0, 0, m, n, k, a, b)
        got = hip.sgemm(0, 0, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        assert np.all(np.abs(got - orc.gemm(m, n, k, a, b)) <= bound)
        assert np.array_equal(got, hip.sgemm(0, 0, m, n, k, a, b))          # same order of sums on every run
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(0, 0, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(0, 0, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
        bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
        out, pre_act = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
        pre_ref = orc.add_row(m, n, got, bias)
        assert np.array_equal(pre_act, pre_ref)
        assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
    m, n, k = 4100, 10, 1000
    a, b = gemm_operands(0, 0, m, n, k)
    a = a.copy()
    a[7 * k + 999] = np.inf          # the last element of row 7: the vector after it is another lane's padding
    got = hip.sgemm(0, 0, m, n, k, a, b).reshape(m, n)
    assert np.all(np.isinf(got[7])) and np.all(np.isfinite(np.delete(got, 7, axis=0)))


def test_gemm_tall_kernel(hip, orc):
    """A * B and A * Bt with a tall row-major A and 13..32 columns (8..12 with K >= 2048 and 2^24
    elements of A): the kernel whose waves own 32 rows each, on the 16 x 16 x 4 instruction up to 16
    columns and on the 32 x 32 x 2 one above.  M off the multiples of 32 and 128, K a multiple of 4 that
    is not one of 64, few rows with K split among workgroups and many rows without a split, every
    epilogue."""
    for (m, n, k, tb) in [(16384, 16, 1024, 0), (4100, 13, 4100, 0), (100000, 32, 260, 0), (513, 20, 40000, 0),
                          (8192, 31, 2048, 1), (1000, 17, 16388, 1), (65536, 10, 2048, 0), (131072 + 5, 8, 1024, 1),
                          (8200, 9, 4100, 1), (2049, 14, 2052, 0), (530, 12, 32772, 0)]:
        say("tall gemm", m, n, k, tb)
        a, b = gemm_operands(0, tb, m, n, k)
        exact, bound = gemm_bound(0, tb, m, n, k, a, b)
        got = hip.sgemm(0, tb, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        assert np.array_equal(got, hip.sgemm(0, tb, m, n, k, a, b))         # same order of sums on every run
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(0, tb, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(0, tb, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
        if not tb:
            bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
            out, pre_act = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
            pre_ref = orc.add_row(m, n, got, bias)
            assert np.array_equal(pre_act, pre_ref)
            assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
    m, n, k = 4100, 16, 4100
    a, b = gemm_operands(0, 0, m, n, k)
    a = a.copy()
    a[7 * k + k - 1] = np.inf            # the last element of row 7: it must stay in row 7
    got = hip.sgemm(0, 0, m, n, k, a, b).reshape(m, n)
    assert np.all(np.isinf(got[7])) and np.all(np.isfinite(np.delete(got, 7, axis=0)))


def test_gemm_transposed_tall_operand_with_narrow_b(hip, orc):
    """At * B and At * Bt with A stored K x M and 8..32 columns of B (the weight gradient of a narrow
    layer): the kernel that feeds both operands from global memory into the 16 x 16 x 4 instruction.
    M on and off the multiples of 64, K off the multiples of 4 and of a share, one share and many,
    beta and the mask epilogue; the same sums whichever way B is stored and on every run."""
    for (m, n, k) in [(2048, 10, 8192), (96, 16, 70001), (4096, 8, 1030), (64, 13, 65536), (65536, 9, 65), (8192, 12, 2048),
                      (1056, 11, 4099),
                      # 17..32 columns: the second block of 16 on the same loads of A
                      (2048, 17, 8192), (96, 32, 70001), (4096, 24, 1030), (64, 31, 65539), (8192, 20, 2048), (1056, 29, 4099)]:
        a, b = gemm_operands(1, 0, m, n, k)
        exact, bound = gemm_bound(1, 0, m, n, k, a, b)
        say("At*B, narrow B", m, n, k)
        got = hip.sgemm(1, 0, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        assert np.array_equal(got, hip.sgemm(1, 0, m, n, k, a, b))
        bt = np.ascontiguousarray(b.reshape(k, n).T).ravel()
        assert np.array_equal(got, hip.sgemm(1, 1, m, n, k, a, bt))
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(1, 0, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(1, 0, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
    m, n, k = 128, 16, 40000
    a, b = gemm_operands(1, 0, m, n, k)
    a = a.copy()
    a[(k - 1) * m + 77] = np.inf          # the last k of output row 77: it must stay in row 77
    got = hip.sgemm(1, 0, m, n, k, a, b).reshape(m, n)
    assert np.all(np.isinf(got[77])) and np.all(np.isfinite(np.delete(got, 77, axis=0)))


def test_gemm_narrow_b_stored_transposed(hip, orc):
    """A narrow B handed over as N x K (A*Bt, At*Bt with N <= 16): turned into K x N in the workspace
    and run through the narrow-N kernels; results within the GEMM bound, beta and the epilogues too."""
    for (m, n, k, ta) in [(8192, 10, 2048, 0), (2048, 10, 65536, 0), (16385, 16, 2052, 0), (4099, 3, 8200, 0),
                          (8192, 10, 4096, 1), (4096, 7, 8192, 1), (32768, 16, 1024, 1), (512, 2, 262144, 0)]:
        say("narrow B transposed", m, n, k, ta)
        a, b = gemm_operands(ta, 1, m, n, k)
        exact, bound = gemm_bound(ta, 1, m, n, k, a, b)
        got = hip.sgemm(ta, 1, m, n, k, a, b)
        assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
        bt = np.ascontiguousarray(b.reshape(n, k).T).ravel()
        if m * k >= 1 << 25:
            assert np.array_equal(got, hip.sgemm(ta, 0, m, n, k, a, bt))    # the same kernel, the same sums
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm(ta, 1, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_mask(ta, 1, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))


def test_gemm_with_a_row_vector_runs_as_matrix_times_column(hip, orc):
    """M = 1: the product is computed as op(B)^T * a through the narrow-N kernels; all four forms (the
    form of A is immaterial), beta, shapes that do and do not meet those kernels' conditions, and the
    epilogues that keep the plain route."""
    for (n, k) in [(4096, 2048), (4100, 4096), (1000, 999), (2048, 8192), (16, 100000), (300, 64)]:
        for ta, tb in ((0, 0), (0, 1), (1, 0), (1, 1)):
            say("row-vector gemm", n, k, ta, tb)
            a, b = gemm_operands(ta, tb, 1, n, k)
            exact, bound = gemm_bound(ta, tb, 1, n, k, a, b)
            got = hip.sgemm(ta, tb, 1, n, k, a, b)
            assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
            c0 = rng.uniform(n, -1, 1, tag=2, seed=SEED)
            assert np.all(np.abs(hip.sgemm(ta, tb, 1, n, k, a, b, c=c0.copy(), beta=1.0) - (exact + c0)) <= bound + 1e-6 * np.abs(c0))
        a, b = gemm_operands(0, 0, 1, n, k)
        exact, bound = gemm_bound(0, 0, 1, n, k, a, b)
        bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
        out, pre_act = hip.linear_fwd(1, k, n, a, b, bias, relu=True, want_pre_act=True)
        assert np.all(np.abs(pre_act - (exact + bias)) <= bound + 1e-6 * np.abs(bias))
        assert np.array_equal(out, orc.unary(orc.RELU, pre_act))


def test_gemm_few_rows_times_a_large_matrix(hip, orc):
    """2..32 rows times a matrix of 2^24 elements and more (a small batch through a wide layer): computed as
    C^T = op(B)^T * op(A)^T through the tall and narrow kernels and transposed into C.  All three forms and
    A^T * B^T, beta 0 and 1 (applied by the transpose), N and K off the vector and tile grids, the row
    counts 2..32 either side of the kernels' limits of 8 and 16, and what lies just outside the route (33 rows,
    a B just below 2^24 elements, another beta)."""
    cases = [(16, 4096, 4096, 0, 0), (10, 4099, 4100, 0, 0), (2, 8192, 4096, 0, 0), (7, 5000, 7001, 1, 0), (16, 2048, 8200, 1, 0),
             (3, 4096, 8192, 0, 1), (8, 4096, 4096, 0, 1), (17, 4099, 4101, 0, 1), (32, 2050, 8190, 0, 1), (5, 6000, 3000, 1, 1),
             (17, 4096, 4096, 0, 0), (33, 4096, 4096, 0, 1), (16, 4000, 4000, 0, 0), (2, 4096, 4096, 0, 1), (12, 16384, 1024, 0, 0),
             # the lower size limits of the forms: 2^23 elements of B for at most 16 rows against K x N, 2^22 for fewer than 8 stored K x M
             (16, 2048, 4096, 0, 0), (9, 4100, 2050, 1, 0), (4, 2048, 2048, 1, 0), (7, 1028, 4099, 1, 0), (16, 2048, 4096, 0, 1), (4, 2048, 2048, 0, 0)]
    for (m, n, k, ta, tb) in cases:
        a, b = gemm_operands(ta, tb, m, n, k)
        exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
        bound = bound * (3e-6 / (1e-5 * np.sqrt(k)))           # 3e-6 |A||B|, far inside the contract's bar
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        for beta in (0.0, 1.0, 0.5):
            say("few rows", m, n, k, ta, tb, beta)
            got = hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=beta)
            want = exact + beta * c0
            assert np.all(np.abs(got - want) <= bound + 1e-6 * np.abs(c0) + 1e-30), (m, n, k, ta, tb, beta, float(np.max(np.abs(got - want) / (bound + 1e-30))))


def test_gemm_small_tile(hip, orc):
    # 64 x 64 tiles (chosen by the cost model for products of a few hundred such tiles), forced here
    # so that edge tiles, rows of odd length, k remainders and the fused epilogues all run on them
    shapes = [(1000, 1000, 512, 0, 0), (1024, 1024, 1024, 0, 1), (999, 1001, 515, 1, 0), (640, 384, 300, 0, 0),
              (129, 257, 4099, 0, 1), (2048, 64, 777, 1, 0), (65, 2000, 333, 0, 0)]
    try:
        for (m, n, k, ta, tb) in shapes:
            say("small-tile gemm", m, n, k, ta, tb)
            a, b = gemm_operands(ta, tb, m, n, k)
            exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
            hip.gemm_tile_policy(hip.TILE_64X64)
            got = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
            c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
            assert np.array_equal(hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
            pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
            assert np.array_equal(hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
            if not ta and not tb:
                bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
                out, pre_act = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
                pre_ref = orc.add_row(m, n, got, bias)
                assert np.array_equal(pre_act, pre_ref)
                assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
            hip.gemm_tile_policy(hip.TILE_128X128)
            big = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - big) <= 2 * bound)
            # small tiles with their k ranges spread over the chip
            if (k + 31) // 32 >= 16:
                hip.gemm_tile_policy(hip.TILE_64X64)
                hip.gemm_tail_policy(hip.TAIL_SPREAD)
                sp = hip.sgemm(ta, tb, m, n, k, a, b)
                assert np.all(np.abs(sp - exact) <= bound), np.max(np.abs(sp - exact) / bound)
                assert np.array_equal(sp, hip.sgemm(ta, tb, m, n, k, a, b))
                assert np.array_equal(hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0), sp + c0)
                assert np.array_equal(hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre), np.where(pre >= 0, sp, 0 * sp))
                hip.gemm_tail_policy(hip.TAIL_AUTO)
        # the default policies on an output of one small tile and a long k
        hip.gemm_tile_policy(hip.TILE_AUTO)
        for (m, n, k, ta, tb) in [(64, 64, 200000, 1, 0), (60, 50, 70001, 0, 0), (64, 100, 50000, 0, 1)]:
            say("small-tile spread, default policy", m, n, k, ta, tb)
            a, b = gemm_operands(ta, tb, m, n, k)
            exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
            got = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
    finally:
        hip.gemm_tile_policy(hip.TILE_AUTO)
        hip.gemm_tail_policy(hip.TAIL_AUTO)


def test_gemm_eight_wave_tile(hip, orc):
    # The 128 x 128 tile on eight waves (chosen on its own when the tile grid gives a CU at most one
    # workgroup), forced here so that edge tiles, rows of odd length, k remainders, one to five k
    # tiles (the pipeline's prologue cases), k splits and the fused
    # epilogues all run on it.  With whole tiles and no k split it sums in the four-wave kernel's order.
    shapes = [(1000, 1000, 512, 0, 0), (1024, 1024, 1024, 0, 1), (999, 1001, 515, 1, 0), (640, 384, 300, 0, 0),
              (129, 257, 4099, 0, 1), (2048, 192, 777, 1, 0), (130, 2000, 333, 0, 0), (256, 256, 32, 0, 0),
              (256, 256, 64, 1, 0), (256, 384, 96, 0, 1), (256, 256, 130, 0, 0), (384, 256, 160, 1, 0),
              (2048, 2048, 2048, 0, 0)]
    try:
        for (m, n, k, ta, tb) in shapes:
            say("eight-wave gemm", m, n, k, ta, tb)
            a, b = gemm_operands(ta, tb, m, n, k)
            exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
            hip.gemm_tile_policy(hip.TILE_128X128_WIDE)
            hip.gemm_tail_policy(hip.TAIL_WHOLE)
            got = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.all(np.abs(got - exact) <= bound), np.max(np.abs(got - exact) / bound)
            c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
            assert np.array_equal(hip.sgemm(ta, tb, m, n, k, a, b, c=c0.copy(), beta=1.0), got + c0)
            pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
            assert np.array_equal(hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre), np.where(pre >= 0, got, 0 * got))
            if not ta and not tb:
                bias = rng.uniform(n, -1, 1, tag=3, seed=SEED)
                out, pre_act = hip.linear_fwd(m, k, n, a, b, bias, relu=True, want_pre_act=True)
                pre_ref = orc.add_row(m, n, got, bias)
                assert np.array_equal(pre_act, pre_ref)
                assert np.array_equal(out, orc.unary(orc.RELU, pre_ref))
            hip.gemm_tile_policy(hip.TILE_128X128)
            four = hip.sgemm(ta, tb, m, n, k, a, b)
            assert np.array_equal(got, four)       # the same k order per element, split or not
    finally:
        hip.gemm_tile_policy(hip.TILE_AUTO)
        hip.gemm_tail_policy(hip.TAIL_AUTO)


def test_sgemm_relu_mask_equals_gemm_then_relu_grad(hip, orc):
    # every kernel that has the epilogue: wave per tile, tiled, split K, spread tail
    shapes = [(64, 64, 64, 0, 1), (1024, 64, 64, 0, 1), (100, 37, 19, 0, 0), (256, 256, 4096, 0, 1), (640, 384, 300, 0, 1),
              (1000, 1000, 512, 1, 0), (515, 259, 1001, 0, 1)]
    try:
        for policy in (hip.TAIL_AUTO, hip.TAIL_SPREAD):
            hip.gemm_tail_policy(policy)
            for (m, n, k, ta, tb) in shapes:
                say("sgemm_relu_mask", policy, m, n, k, ta, tb)
                a, b = gemm_operands(ta, tb, m, n, k)
                pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
                pre[::7] = 0.0          # (0 >= 0) passes the gradient, like the reference's relu grad
                pre[3::11] = -0.0
                c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
                prod = hip.sgemm(ta, tb, m, n, k, a, b)
                masked = orc.unary_grad(orc.RELU, pre, np.zeros(m * n, np.float32), prod)   # 0 + (pre >= 0) * prod
                got = hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre)
                assert np.array_equal(got, masked)
                got1 = hip.sgemm_relu_mask(ta, tb, m, n, k, a, b, pre, c=c0.copy(), beta=1.0)
                assert np.array_equal(got1, c0 + masked)
    finally:
        hip.gemm_tail_policy(hip.TAIL_AUTO)


def test_gemm_grad_matches_oracle(hip, orc):
    for (m, k, n) in [(4, 2, 3), (70, 33, 19), (256, 128, 64), (1024, 64, 1), (1024, 1, 64)]:
        say("gemm_grad", m, k, n)
        lhs = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)
        rhs = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
        g = rng.normal(m * n, 1.0, tag=2, seed=SEED)
        lg_h, rg_h = np.zeros(m * k, np.float32), np.zeros(k * n, np.float32)
        lg_o, rg_o = lg_h.copy(), rg_h.copy()
        hip.gemm_grad(m, k, n, lhs, rhs, lg_h, rg_h, g)
        orc.gemm_grad(m, k, n, lhs, rhs, lg_o, rg_o, g)
        tol_l = 1e-5 * np.sqrt(n) * (np.abs(g.reshape(m, n)) @ np.abs(rhs.reshape(k, n)).T).ravel() + 1e-30
        tol_r = 1e-5 * np.sqrt(m) * (np.abs(lhs.reshape(m, k)).T @ np.abs(g.reshape(m, n))).ravel() + 1e-30
        assert np.all(np.abs(lg_h - lg_o) <= tol_l)
        assert np.all(np.abs(rg_h - rg_o) <= tol_r)
        # a NULL grad (operand without requires_grad) is skipped, the other side still written
        rg = np.zeros(k * n, np.float32)
        hip.gemm_grad(m, k, n, lhs, rhs, None, rg, g)
        assert np.array_equal(rg, rg_h)


def test_linear_fwd_fused_equals_gemm_bias_relu(hip, orc):
    for (m, k, n) in [(64, 1, 64), (130, 70, 50), (256, 784, 384), (1024, 64, 1), (300, 4096, 200)]:
        say("linear_fwd", m, k, n)
        x = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)
        w = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
        bias = rng.uniform(n, -1, 1, tag=2, seed=SEED)
        h = hip.gemm(m, n, k, x, w)
        pre_ref = orc.add_row(m, n, h, bias)          # same f32 add on the device's own product
        out_ref = orc.unary(orc.RELU, pre_ref)
        out, pre = hip.linear_fwd(m, k, n, x, w, bias, relu=True, want_pre_act=True)
        assert np.array_equal(pre, pre_ref)
        assert np.array_equal(out, out_ref)
        out2 = hip.linear_fwd(m, k, n, x, w, bias, relu=False)
        assert np.array_equal(out2, pre_ref)


def test_linear_grad_one_launch_equals_the_three_ops(hip, orc):
    """slhip_linear_grad: x.grad and w.grad carry the bits of slhip_sgemm / slhip_sgemm_relu_mask called on
    their own (small layers run both products in one launch, each with the plan of its own launch);
    the bias gradient is a sum in another order: within 1e-6 * sum|g| of the oracle's add_row_mut_grad.
    Shapes: the sine fit's three layers, ragged ones, one that needs the wave kernel's checked form,
    one too large for the single launch (it takes the three kernels in turn)."""
    for (m, k, n) in [(1024, 1, 64), (1024, 64, 64), (1024, 64, 1), (1000, 37, 13), (7, 5, 3), (33, 65, 31), (200, 96, 40),
                      (4096, 63, 17), (8192, 256, 10)]:
        for beta in (0.0, 1.0):
            for masked in (False, True):
                say("linear_grad", m, k, n, "beta", beta, "masked", masked)
                x = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)
                w = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
                g = rng.normal(m * n, 1.0, tag=2, seed=SEED)
                pre = rng.normal(m * k, 1.0, tag=3, seed=SEED) if masked else None
                xg0 = rng.uniform(m * k, -1, 1, tag=4, seed=SEED)
                wg0 = rng.uniform(k * n, -1, 1, tag=5, seed=SEED)
                bg0 = rng.uniform(n, -1, 1, tag=6, seed=SEED)
                xg, wg, bg = xg0.copy(), wg0.copy(), bg0.copy()
                hip.linear_grad(m, k, n, x, w, g, x_grad=xg, relu_pre=pre, w_grad=wg, bias_grad=bg, beta=beta)
                if masked:
                    xg_ref = hip.sgemm_relu_mask(0, 1, m, k, n, g, w, pre, c=xg0.copy(), beta=beta)
                else:
                    xg_ref = hip.sgemm(0, 1, m, k, n, g, w, c=xg0.copy(), beta=beta)
                wg_ref = hip.sgemm(1, 0, k, n, m, x, g, c=wg0.copy(), beta=beta)
                assert np.array_equal(xg, np.asarray(xg_ref).ravel())
                assert np.array_equal(wg, np.asarray(wg_ref).ravel())
                bg_ref = bg0.copy()
                orc.add_row_mut_grad(m, n, bg_ref, g)
                bound = 1e-6 * (np.abs(g.reshape(m, n)).sum(axis=0) + np.abs(bg0)) + 1e-30
                assert np.all(np.abs(bg - bg_ref) <= bound), np.abs(bg - bg_ref).max()
                exact = bg0.astype(np.float64) + g.reshape(m, n).astype(np.float64).sum(axis=0)
                assert np.all(np.abs(bg - exact) <= bound)
                # a layer whose input needs no gradient: only w.grad and the bias gradient
                wg2, bg2 = wg0.copy(), bg0.copy()
                hip.linear_grad(m, k, n, x, w, g, w_grad=wg2, bias_grad=bg2, beta=beta)
                assert np.array_equal(wg2, wg)
                assert np.array_equal(bg2, bg)
    with pytest.raises(Exception):
        hip.linear_grad(4, 4, 4, np.zeros(16, np.float32), np.zeros(16, np.float32), np.zeros(16, np.float32),
                        relu_pre=np.zeros(16, np.float32), w_grad=np.zeros(16, np.float32))


# --------------------------------------------------------------------------- reductions
RED_SHAPES = [(1, 1), (1, 5), (5, 1), (3, 4), (7, 13), (64, 64), (33, 1000), (1000, 33), (257, 4096), (4096, 257),
              (16, 40000), (40000, 16), (2, 300001), (300001, 2), (1, 1 << 20), (1 << 20, 1), (2048, 2048),
              (100, 10), (8192, 10), (5000, 128), (3, 70000),
              # many short rows whose length is not a power of two (LDS-staged contiguous-axis kernel),
              # odd and even row lengths through the flat strided-axis stages, few rows of great length
              (5000, 3), (4099, 10), (2000, 100), (1025, 127), (70000, 2), (30011, 7), (9001, 33), (20000, 258),
              (13, 300001), (9, 100002), (1500, 1001),
              # short rows a power of two long (the same LDS-staged kernel, several lanes per row)
              (3001, 64), (2100, 32), (5003, 8), (1100, 5), (1024, 4), (1029, 48)]


def sum_bound(x, rows, cols, axis):
    return 1e-6 * np.abs(x.reshape(rows, cols)).astype(np.float64).sum(axis=axis) + 1e-30


@pytest.mark.parametrize("shape", RED_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_reductions(hip, orc, shape):
    rows, cols = shape
    say("reductions", rows, cols)
    x = rng.uniform(rows * cols, -10, 10, tag=0, seed=SEED + rows)
    x64 = x.reshape(rows, cols).astype(np.float64)
    # max: bit-exact
    assert np.array_equal(hip.max_cols(cols, x), orc.max_cols(cols, x))
    assert np.array_equal(hip.max_rows(cols, x), orc.max_rows(cols, x))
    # sums
    # sums of small integers have one right answer in f32 whatever the order: the oracle's bits
    xi = (rng.integers(rows * cols, 17, tag=9, seed=SEED + rows) - 8).astype(np.float32)
    for name in ("sum_cols", "sum_rows", "mean_cols", "mean_rows"):
        assert np.array_equal(getattr(hip, name)(cols, xi), getattr(orc, name)(cols, xi)), name
    # sums of the U(-10, 10) data: within 1e-6 of sum|x| of the exact sum, and of the oracle's
    # sequential f32 sum directly where that sum is short enough to be that accurate itself
    got, ref = hip.sum_cols(cols, x), orc.sum_cols(cols, x)
    b = sum_bound(x, rows, cols, 1)
    assert np.all(np.abs(got - x64.sum(1)) <= b)
    if cols <= 64:
        assert np.all(np.abs(got - ref) <= b)
    got, ref = hip.sum_rows(cols, x), orc.sum_rows(cols, x)
    b = sum_bound(x, rows, cols, 0)
    assert np.all(np.abs(got - x64.sum(0)) <= b)
    if rows <= 64:
        assert np.all(np.abs(got - ref) <= b)
    # means
    got = hip.mean_cols(cols, x)
    assert np.all(np.abs(got - x64.mean(1)) <= sum_bound(x, rows, cols, 1) / cols + 1e-7 * np.abs(x64.mean(1)))
    got = hip.mean_rows(cols, x)
    assert np.all(np.abs(got - x64.mean(0)) <= sum_bound(x, rows, cols, 0) / rows + 1e-7 * np.abs(x64.mean(0)))
    # scalars
    tot = x64.sum()
    bt = 1e-6 * np.abs(x64).sum() + 1e-30
    assert abs(hip.sum_all(x) - tot) <= bt
    assert abs(float(hip.mean(x)) - tot / x.size) <= bt / x.size + 1e-7 * abs(tot / x.size)
    assert hip.max_all(x) == float(x.max())


def test_max_is_bit_exact_with_injected_ties_and_negatives(hip, orc):
    for rows, cols in [(200, 300), (64, 4096), (4096, 64)]:
        say("max ties", rows, cols)
        x = rng.uniform(rows * cols, -10, 10, tag=0, seed=SEED)
        x = rng.inject_row_max_ties(x, rows, cols, 0.01)
        assert np.array_equal(hip.max_cols(cols, x), orc.max_cols(cols, x))
        x = rng.inject_col_max_ties(x, rows, cols, 0.01)
        assert np.array_equal(hip.max_rows(cols, x), orc.max_rows(cols, x))
        xn = -np.abs(x) - 1.0  # all negative: the result must not be clamped at 0
        assert np.array_equal(hip.max_rows(cols, xn), orc.max_rows(cols, xn))
        assert np.array_equal(hip.max_cols(cols, xn), orc.max_cols(cols, xn))


def test_max_grads_tie_rules(hip, orc):
    # (the last three: few rows of great length, which several workgroups per row scan)
    for rows, cols in [(3, 4), (50, 200), (300, 40), (17, 5000), (2000, 1), (1, 2000), (3, 70001), (1, 300000),
                       (40, 65536)]:
        say("max grads", rows, cols)
        x = rng.uniform(rows * cols, -10, 10, tag=0, seed=SEED + cols)
        g_r = rng.normal(rows, 1.0, tag=1, seed=SEED)
        g_c = rng.normal(cols, 1.0, tag=2, seed=SEED)
        base = rng.normal(rows * cols, 1.0, tag=3, seed=SEED)
        # first tie only, along the contiguous axis
        xt = rng.inject_row_max_ties(x.copy(), rows, cols, 0.05)
        out = orc.max_cols(cols, xt)
        a = hip.max_cols_grad(cols, out, xt, base.copy(), g_r)
        b = orc.max_cols_grad(cols, out, xt, base.copy(), g_r)
        assert np.array_equal(a, b)
        # all ties, along the strided axis
        xt = rng.inject_col_max_ties(x.copy(), rows, cols, 0.05)
        out = orc.max_rows(cols, xt)
        a = hip.max_rows_grad(cols, out, xt, base.copy(), g_c)
        b = orc.max_rows_grad(cols, out, xt, base.copy(), g_c)
        assert np.array_equal(a, b)


def test_broadcast_grads_are_bit_exact(hip, orc):
    for rows, cols in [(3, 4), (5, 7), (128, 256), (1000, 10), (10, 1000), (513, 1028), (1234, 679), (3, 100003),
                       (100003, 3), (1, 1)]:
        say("broadcast grads", rows, cols)
        base = rng.normal(rows * cols, 1.0, tag=0, seed=SEED)
        g_r = rng.normal(rows, 1.0, tag=1, seed=SEED)
        g_c = rng.normal(cols, 1.0, tag=2, seed=SEED)
        for name, g in [("sum_rows_grad", g_c), ("sum_cols_grad", g_r), ("mean_rows_grad", g_c),
                        ("mean_cols_grad", g_r)]:
            a = getattr(hip, name)(cols, base.copy(), g)
            b = getattr(orc, name)(cols, base.copy(), g)
            assert np.array_equal(a, b), name


# --------------------------------------------------------------------------- softmax
SOFTMAX_SHAPES = [(2, 3), (1, 1), (7, 10), (8192, 10), (100, 128), (33, 130), (64, 1024), (17, 1000), (9, 4096),
                  (5, 4100), (3, 16384), (2, 16390), (2, 40000), (1000, 1), (50, 64), (50, 257),
                  # odd row lengths: the scalar tail of the vector paths, register-resident and streaming
                  (6, 7), (5, 5), (300, 1001), (3, 4099), (3, 16387), (2, 40003), (4, 100001), (700, 6789),
                  # 1025..2048 vectors per row: the forward pass runs 512 lanes there, the backward pass 1024
                  (5, 8192), (4, 4104), (3, 6000), (3, 8190), (3, 8196),
                  # rows of 16388..65536 floats held in registers, and few rows far longer than that, cut into segments
                  (3, 16388), (2, 16389), (2, 20000), (2, 20001), (2, 24577), (2, 32768), (2, 32771), (2, 32772), (2, 50257), (2, 65536), (2, 65539),
                  (1, 1048576), (3, 300001), (2, 262147), (7, 131072), (1, 131073),
                  # 257..448 vectors per row: the forward pass runs one wave per row with eight vectors a lane
                  (9, 1028), (9, 1030), (6, 1500), (5, 1792), (5, 1795), (5, 1796), (7, 1281),
                  # many short rows, not a power of two long: the LDS-staged kernels
                  (5000, 10), (1025, 100), (3000, 3), (1500, 159), (2000, 160), (1100, 161), (1030, 255), (1024, 129), (1500, 200), (1040, 254), (1027, 131), (4097, 37), (1024, 6),
                  # and short rows a power of two long, which take the same kernels
                  (3000, 16), (1100, 64), (5000, 2), (2049, 32), (1030, 8), (4100, 4), (1023, 16)]


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_softmax_forward_backward(hip, orc, shape):
    rows, cols = shape
    say("softmax", rows, cols)
    x = rng.normal(rows * cols, 3.0, tag=0, seed=SEED + cols)
    g = rng.normal(rows * cols, 1.0, tag=1, seed=SEED + cols)
    # exact value of the function both sides evaluate: the shifted logit x - max is an f32
    # subtraction in the reference (sub_cols) and on the device, so it is rounded to f32 here too;
    # exp, sum and division are then carried out in f64
    x2 = x.reshape(rows, cols)
    shifted = (x2 - x2.max(1, keepdims=True)).astype(np.float32).astype(np.float64)
    e = np.exp(shifted)
    exact = (e / e.sum(1, keepdims=True)).ravel()
    got, ref = hip.softmax(rows, cols, x), orc.softmax(rows, cols, x)
    rel = np.abs(got - exact) / np.maximum(np.abs(exact), 1e-30)
    assert rel.max() <= 1e-6, rel.max()
    if cols <= 64:     # the oracle's sequential sum of a short row is itself accurate: the direct bar
        assert np.all(np.abs(got - ref) <= 1e-6 * np.abs(ref) + 1e-37), np.max(np.abs(got - ref) / np.maximum(ref, 1e-37))
    assert np.all(np.abs(got.reshape(rows, cols).astype(np.float64).sum(1) - 1.0) <= 1e-6)
    # backward on the device's own forward output, SET and accumulate
    s64 = got.reshape(rows, cols).astype(np.float64)
    g64 = g.reshape(rows, cols).astype(np.float64)
    dot = (s64 * g64).sum(1, keepdims=True)
    exact_b = (s64 * (g64 - dot)).ravel()
    scale = (np.abs(s64) * (np.abs(g64) + (np.abs(s64) * np.abs(g64)).sum(1, keepdims=True))).ravel()
    bound = 1e-6 * scale + 1e-37          # cancellation in g - <s,g> is priced on the operands' scale
    gb = hip.softmax_grad(rows, cols, got, g)
    ob = orc.softmax_grad(rows, cols, got, g)
    assert np.all(np.abs(gb - exact_b) <= bound), np.max(np.abs(gb - exact_b) / bound)
    if cols <= 64:
        assert np.all(np.abs(gb - ob) <= bound), np.max(np.abs(gb - ob) / bound)
    base = rng.normal(rows * cols, 1.0, tag=2, seed=SEED)
    gacc = hip.softmax_grad(rows, cols, got, g, x_grad=base.copy(), beta=1.0)
    assert np.all(np.abs(gacc - (base + exact_b)) <= bound + 1e-6 * np.abs(base))


def test_softmax_grad_constant_seed_is_zero(hip):
    rows, cols = 64, 1000
    x = rng.normal(rows * cols, 3.0, tag=0, seed=SEED)
    s = hip.softmax(rows, cols, x)
    gz = hip.softmax_grad(rows, cols, s, np.ones(rows * cols, np.float32))
    assert np.max(np.abs(gz)) <= 1e-6


# --------------------------------------------------------------------------- transpose
TR_SHAPES = [(2, 3), (1, 7), (7, 1), (64, 64), (65, 63), (128, 256), (100, 300), (257, 129), (1024, 1024),
             (4, 4096), (4096, 4), (1000, 1000), (1, 1 << 18), (1 << 18, 1),
             # rows / columns of odd length on the vector paths, and the few-rows / few-columns kernels
             (4097, 4097), (1234, 679), (300, 1001), (1001, 300), (100000, 7), (7, 100000), (33, 1000), (1000, 33),
             (2, 5), (32, 70000), (259, 66),
             # the narrow-matrix kernel: chunk boundaries, sides 2..40, both directions, tiny and ragged long sides
             (70001, 2), (2, 70001), (30000, 31), (31, 30000), (9999, 40), (40, 9999), (5000, 16), (16, 5003), (41, 3000),
             (3000, 41), (3, 3), (40, 40), (17, 23),
             # the limits of the narrow kernels (56 columns in, 200 rows out) and what lies just beyond
             (5000, 56), (5001, 57), (200, 3001), (201, 3000), (224, 3001), (100, 8193), (128, 5000), (200, 41), (56, 57), (57, 56),
             (163, 9000), (9000, 55),
             # the 64 x 256 tile: tall matrices of 256 columns and more, whole tiles and ragged edges, and wide
             # ones of 64 / 128 / 192 rows; 128 KiB chunks: inputs of 57..128 columns off the 64-grid
             (2048, 512), (1100, 260), (4100, 257), (8200, 1023), (1025, 256), (64, 5000), (128, 1024), (192, 777), (64, 256),
             (128, 513), (2000, 100), (1700, 65), (3000, 127), (1600, 100), (2049, 128), (1919, 119), (330, 100),
             (4000, 200), (4200, 255), (700, 41), (9001, 140), (3300, 193), (5000, 256), (4095, 250),
             # narrow inputs whose output runs start off / on 64- and 128-byte boundaries (long sides odd, multiples
             # of 16 and of 32): shifted pieces with a halo, first and last chunks, pieces cut at both ends
             (50001, 100), (50016, 100), (50048, 100), (20001, 250), (20000, 250), (100003, 56), (100000, 33), (99984, 33),
             (17, 3), (31, 10), (33, 10), (8209, 10), (1647, 10), (1648, 10), (1649, 10), (3301, 10), (40007, 72), (5000001, 3),
             # tall matrices of 2048 columns: the mirrored tile (rows a multiple of 16) and the plain one beside it
             (8192, 2048), (8208, 2048), (8200, 2048), (8193, 2048),
             # 2^24 elements and more with output rows off the 64-byte grid: the 256 x 64 tile with pieces shifted
             # per output row (first and last tile rows, ragged tile columns, rows of odd length on both sides)
             (8200, 2049), (16385, 1031), (8209, 2100), (65521, 257), (8193, 2050), (8193, 2048), (16385, 1040),
             # the 128 x 128 tile with shifted pieces: shorter output rows and input pitches off the 64-byte grid
             (300, 140001), (4026, 4099), (1001, 20001), (257, 131073), (2050, 2051), (5000, 3001), (383, 16400),
             (16385, 1025)]


@pytest.mark.parametrize("shape", TR_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_transpose_bit_exact(hip, orc, shape):
    rows, cols = shape
    say("transpose", rows, cols)
    x = rng.uniform(rows * cols, -10, 10, tag=0, seed=SEED)
    got = hip.transpose(rows, cols, x)
    assert np.array_equal(got, orc.transpose(rows, cols, x))
    assert np.array_equal(got, x.reshape(rows, cols).T.ravel())
    assert np.array_equal(hip.transpose(cols, rows, got), x)           # involution
    base = rng.uniform(rows * cols, -1, 1, tag=1, seed=SEED)
    acc = hip.transpose(rows, cols, x, out=base.copy(), assign=True)   # `Assign` (+=)
    assert np.array_equal(acc, orc.transpose(rows, cols, x, out=base.copy(), assign=True))


@pytest.mark.parametrize("shape", [(50001, 100), (50016, 100), (8209, 10), (100003, 56), (64, 5000), (100, 8193), (1234, 679),
                                   (4096, 4100), (8208, 2048), (2048, 2049)],
                         ids=lambda s: "x".join(map(str, s)))
def test_transpose_between_views_off_the_allocation_grid(hip, orc, shape):
    """Input and output that start 1, 5, 16 and 17 floats into their allocations: no kernel may rely on
    the 256-byte alignment of a fresh buffer, and what lies around the output stays as it was."""
    rows, cols = shape
    n = rows * cols
    c = hip.ctx()
    x = rng.uniform(n, -10, 10, tag=0, seed=SEED)
    want = orc.transpose(rows, cols, x)
    pad = 64
    src, dst = c.empty(n + pad), c.empty(n + 2 * pad)
    for off in (1, 5, 16, 17):
        say("transpose into a view", rows, cols, off)
        src.view(off, n).upload(x)
        c.call("slhip_fill", n + 2 * pad, -3.0, dst.ptr)
        c.call("slhip_transpose", rows, cols, src.view(off, n).ptr, dst.view(pad + off, n).ptr, 0.0)
        got = dst.numpy()
        assert np.array_equal(got[pad + off:pad + off + n], want), off
        assert np.all(got[:pad + off] == -3.0) and np.all(got[pad + off + n:] == -3.0), off
        c.call("slhip_transpose", rows, cols, src.view(off, n).ptr, dst.view(pad + off, n).ptr, 1.0)
        assert np.array_equal(dst.numpy()[pad + off:pad + off + n], want + want), off
    src.free()
    dst.free()


# --------------------------------------------------------------------------- elementwise / row op
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 100003, 1 << 20])
def test_elementwise_ops(hip, orc, n):
    say("elementwise", n)
    a = rng.uniform(n, -10, 10, tag=1, seed=SEED)
    b = rng.uniform(n, -10, 10, tag=2, seed=SEED)
    c = rng.uniform(n, -10, 10, tag=3, seed=SEED)
    d = rng.uniform(n, -10, 10, tag=4, seed=SEED)
    g = rng.normal(n, 1.0, tag=5, seed=SEED)
    for op in (orc.ADD, orc.SUB, orc.MUL, orc.DIV):
        assert np.array_equal(hip.binary_ew(op, a, b), orc.binary_ew(op, a, b)), op
        lg, rg = rng.normal(n, 1.0, tag=6, seed=SEED), rng.normal(n, 1.0, tag=7, seed=SEED)
        lh, rh = hip.binary_ew_grad(op, a, b, lg.copy(), rg.copy(), g)
        lo, ro = orc.binary_ew_grad(op, a, b, lg.copy(), rg.copy(), g)
        if op == orc.DIV:   # 1/r and l/(r*r): the division may differ in the last place
            assert np.allclose(lh, lo, rtol=1e-6, atol=0) and np.allclose(rh, ro, rtol=1e-6, atol=1e-30)
        else:
            assert np.array_equal(lh, lo) and np.array_equal(rh, ro), op
        only_l, _ = hip.binary_ew_grad(op, a, b, lg.copy(), None, g)
        assert np.array_equal(only_l, lh)
    for op in (orc.SQUARE, orc.RELU):
        assert np.array_equal(hip.unary(op, a), orc.unary(op, a))
        xg = rng.normal(n, 1.0, tag=8, seed=SEED)
        assert np.array_equal(hip.unary_grad(op, a, xg.copy(), g), orc.unary_grad(op, a, xg.copy(), g))
    assert np.array_equal(hip.unary(orc.CLIP, a, -2.5, 3.0), orc.unary(orc.CLIP, a, -2.5, 3.0))
    assert np.array_equal(hip.unary(orc.SCALE, a, 0.37), orc.unary(orc.SCALE, a, 0.37))
    assert np.array_equal(hip.unary(orc.NEG_DIV, a, 8192.0), orc.unary(orc.NEG_DIV, a, 8192.0))
    # transcendental ops: 1e-6 relative against the f64 value
    a64 = a.astype(np.float64)
    for p in (2.0, 3.0, 0.5):
        base = np.abs(a64) if p == 0.5 else a64
        x32 = base.astype(np.float32)
        got = hip.unary(orc.POW, x32, p)
        assert np.all(np.abs(got - base ** p) <= 1e-6 * np.abs(base ** p) + 1e-37), p
        gg = hip.unary_grad(orc.POW, x32, np.zeros(n, np.float32), g, p)
        if p != 0.5:
            ex = p * base ** (p - 1) * g.astype(np.float64)
            assert np.all(np.abs(gg - ex) <= 2e-6 * np.abs(ex) + 1e-37), p
    small = (a * np.float32(0.5)).astype(np.float32)
    got = hip.unary(orc.EXP, small)
    assert np.all(np.abs(got - np.exp(small.astype(np.float64))) <= 1e-6 * np.exp(small.astype(np.float64)))
    pos = (np.abs(a) + np.float32(1e-3)).astype(np.float32)
    got = hip.unary(orc.NEG_LN, pos)
    ex = -np.log(pos.astype(np.float64))
    assert np.all(np.abs(got - ex) <= 1e-6 * np.abs(ex) + 1e-7)
    # fused chain ((a+b)*c - d) -> pow 2 -> square against the op-by-op oracle
    t = orc.binary_ew(orc.SUB, orc.binary_ew(orc.MUL, orc.binary_ew(orc.ADD, a, b), c), d)
    ref = orc.unary(orc.SQUARE, orc.unary(orc.POW, t, 2.0))
    got = hip.ew_chain(a, b, c, d)
    assert np.all(np.abs(got - ref) <= 1e-6 * np.abs(ref) + 1e-37)
    # sgd
    p0 = rng.uniform(n, -1, 1, tag=9, seed=SEED)
    assert np.array_equal(hip.sgd_step(p0.copy(), g, 0.05), orc.sgd_step(p0.copy(), g, 0.05))


def test_negative_base_integer_pow_is_finite(hip):
    x = np.array([-3.0, -0.5, 0.0, 2.0], np.float32)
    assert np.array_equal(hip.unary(1, x, 2.0), np.array([9.0, 0.25, 0.0, 4.0], np.float32))
    g = hip.unary_grad(1, x, np.zeros(4, np.float32), np.ones(4, np.float32), 2.0)
    assert np.array_equal(g, np.array([-6.0, -1.0, 0.0, 4.0], np.float32))


def test_row_op_and_bias_grad(hip, orc):
    for rows, cols in [(3, 5), (1, 9), (9, 1), (1024, 64), (1000, 10), (8192, 10), (300, 2048), (4097, 130),
                       (1234, 679), (7, 100003), (100003, 3), (2, 2), (1, 100000), (5, 4096), (3, 6)]:
        say("row op", rows, cols)
        lhs = rng.uniform(rows * cols, -10, 10, tag=0, seed=SEED)
        rhs = rng.uniform(cols, -10, 10, tag=1, seed=SEED)
        ref = orc.add_row(rows, cols, lhs, rhs)
        assert np.array_equal(hip.add_row(rows, cols, lhs, rhs), ref)
        assert np.array_equal(hip.add_row(rows, cols, lhs, rhs, inplace=True), ref)     # add_row_mut
        g = rng.normal(rows * cols, 1.0, tag=2, seed=SEED)
        rg0 = rng.normal(cols, 1.0, tag=3, seed=SEED)
        b = 1e-6 * (np.abs(g.reshape(rows, cols)).astype(np.float64).sum(0) + np.abs(rg0)) + 1e-30
        exact = g.reshape(rows, cols).astype(np.float64).sum(0) + rg0
        got = hip.add_row_mut_grad(rows, cols, rg0.copy(), g)
        assert np.all(np.abs(got - exact) <= b)
        lg, rg = hip.add_row_grad(rows, cols, np.full(rows * cols, 7.0, np.float32), rg0.copy(), g)
        assert np.array_equal(lg, g)                    # lhs_grad is overwritten, not accumulated
        assert np.all(np.abs(rg - exact) <= b)


def test_cce_and_onehot(hip, orc):
    rows, cols = 500, 10
    cls = rng.integers(rows, cols, tag=1, seed=SEED).astype(np.float32)
    t = hip.onehot(cols, cls)
    assert np.array_equal(t, orc.onehot(cols, cls))
    p = hip.softmax(rows, cols, rng.normal(rows * cols, 3.0, tag=0, seed=SEED))
    a, b = hip.cce(rows, cols, p, t), orc.cce(rows, cols, p, t)
    assert np.all(np.abs(a - b) <= 1e-6 * np.abs(b) + 1e-7)
    assert np.array_equal(hip.cce_grad(rows, cols, p, t), orc.cce_grad(rows, cols, p, t))


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 10), (257, 129), (4096, 33), (5, 70000), (2000, 2048),
                                   (5000, 1), (3000, 7), (1, 5000), (20000, 2), (1500, 64), (40, 4099)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("kind", ["row_op", "col_op"])
def test_broadcast_ops_with_op_code(hip, orc, shape, kind):
    """row_op / col_op: forward and the elementwise gradient are one IEEE operation (two for the
    gradient) per element: bit-exact; the broadcast-side gradient is a sum: 1e-6 of sum|terms|."""
    rows, cols = shape
    n = rows * cols
    lhs = rng.uniform(n, 0.5, 2.0, tag=0, seed=SEED)
    v = rng.uniform(rows if kind == "col_op" else cols, 0.5, 2.0, tag=1, seed=SEED)
    g = rng.normal(n, 1.0, tag=2, seed=SEED)
    for op in (orc.ADD, orc.SUB, orc.MUL, orc.DIV):
        say(kind, rows, cols, "op", op)
        assert np.array_equal(getattr(hip, kind)(op, cols, lhs, v), getattr(orc, kind)(op, cols, lhs, v))
        lg0 = rng.uniform(n, -1, 1, tag=3, seed=SEED)
        vg0 = rng.uniform(v.size, -1, 1, tag=4, seed=SEED)
        lg_h, vg_h = getattr(hip, kind + "_grad")(op, cols, lhs, v, lg0.copy(), vg0.copy(), g)
        lg_o, vg_o = getattr(orc, kind + "_grad")(op, cols, lhs, v, lg0.copy(), vg0.copy(), g)
        assert np.array_equal(lg_h, lg_o)
        # terms of the broadcast-side sum, in f64, for the bound
        L, G = lhs.reshape(rows, cols).astype(np.float64), g.reshape(rows, cols).astype(np.float64)
        V = v.astype(np.float64)[:, None] if kind == "col_op" else v.astype(np.float64)[None, :]
        dr = {orc.ADD: np.ones_like(L), orc.SUB: -np.ones_like(L), orc.MUL: L, orc.DIV: -L / (V * V)}[op] * G
        axis = 1 if kind == "col_op" else 0
        bound = 1e-6 * (np.abs(dr).sum(axis) + np.abs(vg0)) + 1e-30
        exact = vg0 + dr.sum(axis)
        assert np.all(np.abs(vg_h - exact) <= bound + 1e-6 * np.abs(exact))
        if (cols if kind == "col_op" else rows) <= 64:      # short sums: the oracle's own rounding is below the bar
            assert np.all(np.abs(vg_h - vg_o) <= bound + 1e-6 * np.abs(exact))
        # one side only
        lg1, _ = getattr(hip, kind + "_grad")(op, cols, lhs, v, lg0.copy(), None, g)
        assert np.array_equal(lg1, lg_o)


def test_tanh_sigmoid_diagflat_onehot_grad(hip, orc):
    x = rng.normal(100003, 2.0, tag=0, seed=SEED)
    g = rng.normal(x.size, 1.0, tag=1, seed=SEED)
    x64 = x.astype(np.float64)
    for op, f, df in [(orc.TANH, np.tanh, lambda v: 1 - np.tanh(v) ** 2),
                      (orc.SIGMOID, lambda v: 1 / (1 + np.exp(-v)), lambda v: np.exp(-v) / (1 + np.exp(-v)) ** 2)]:
        got, ref = hip.unary(op, x), orc.unary(op, x)
        assert np.all(np.abs(got - f(x64)) <= 1e-6 * np.abs(f(x64)) + 1e-37)
        assert np.all(np.abs(got - ref) <= 1e-6 * np.abs(ref) + 1e-37), np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-37))
        xg0 = rng.uniform(x.size, -1, 1, tag=2, seed=SEED)
        gg, gr = hip.unary_grad(op, x, xg0.copy(), g), orc.unary_grad(op, x, xg0.copy(), g)
        exact = xg0 + df(x64) * g
        # 1 - tanh(x)^2 cancels near |tanh| = 1: the reference's own formula carries an absolute
        # error of a few ulp(1) there, whoever evaluates it
        bound = (3e-7 + 2e-6 * np.abs(df(x64))) * np.abs(g) + 2e-6 * np.abs(xg0) + 1e-37
        assert np.all(np.abs(gg - exact) <= bound)
        assert np.all(np.abs(gg - gr) <= bound), np.max(np.abs(gg - gr) / bound)
    v = rng.uniform(300, -1, 1, tag=3, seed=SEED)
    assert np.array_equal(hip.diagflat(v), orc.diagflat(v))
    og = rng.normal(300 * 300, 1.0, tag=4, seed=SEED)
    assert np.array_equal(hip.diagflat_grad(np.ones(300, np.float32), og), orc.diagflat_grad(np.ones(300, np.float32), og))
    cls = rng.integers(5000, 10, tag=5, seed=SEED).astype(np.float32)
    og = rng.normal(5000 * 10, 1.0, tag=6, seed=SEED)
    assert np.array_equal(hip.onehot_grad(10, cls, np.ones(5000, np.float32), og),
                          orc.onehot_grad(10, cls, np.ones(5000, np.float32), og))


@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 1 << 20, 3000001])
def test_fused_mse_against_the_op_chain(hip, orc, n):
    """slhip_mse == sub, squared, sum over one row, mul by 1/n of the oracle; its gradient is the
    chain's own product ((x-y)*2)*((1/n)*1), bit for bit."""
    x = rng.uniform(n, -2, 2, tag=0, seed=SEED)
    y = rng.uniform(n, -2, 2, tag=1, seed=SEED)
    c = np.array([1.0 / n], np.float32)
    d = orc.binary_ew(orc.SUB, x, y)
    q = orc.unary(orc.SQUARE, d)
    ref = orc.binary_ew(orc.MUL, orc.sum_cols(n, q), c)[0]
    exact = np.sum(d.astype(np.float64) ** 2) / n
    got = hip.mse(x, y)
    assert abs(got - exact) <= 1e-6 * exact + 1e-37
    if n <= 1024:      # the oracle's sequential sum of a thousand squares is within the bar itself (of 4099: 1.3e-6 off)
        assert abs(got - ref) <= 1e-6 * exact + 1e-37, abs(got - ref) / exact
    xg0 = rng.uniform(n, -1, 1, tag=2, seed=SEED)
    for up in (1.0, -0.25):
        gs, _ = orc.binary_ew_grad(orc.MUL, np.zeros(1, np.float32), c, np.zeros(1, np.float32), np.zeros(1, np.float32),
                                   np.array([up], np.float32))                       # s.grad = c * upstream
        qg = orc.sum_cols_grad(n, np.zeros(n, np.float32), gs)
        dg = orc.unary_grad(orc.SQUARE, d, np.zeros(n, np.float32), qg)
        want, _ = orc.binary_ew_grad(orc.SUB, x, y, xg0.copy(), np.zeros(n, np.float32), dg)
        assert np.array_equal(hip.mse_grad(x, y, xg0.copy(), up), want)


@pytest.mark.parametrize("shape", [(1, 1), (7, 3), (8192, 10), (300, 1000), (5, 70001), (3000, 100), (70000, 7),
                                   (9000, 512), (1100, 4099)],  # the last two: softmax + cce as two kernels
                         ids=lambda s: "x".join(map(str, s)))
def test_fused_softmax_cross_entropy_against_the_op_chain(hip, orc, shape):
    rows, cols = shape
    n = rows * cols
    x = rng.normal(n, 3.0, tag=0, seed=SEED)
    cls = rng.integers(rows, cols, tag=1, seed=SEED)
    t = np.zeros((rows, cols), np.float32)
    t[np.arange(rows), cls] = 1.0
    t = t.ravel()
    p_ref = orc.softmax(rows, cols, x)
    loss_ref = orc.cce(rows, cols, p_ref, t)
    p, loss = hip.softmax_cce(rows, cols, x, t)
    X = x.reshape(rows, cols).astype(np.float64)
    sh = (x.reshape(rows, cols) - x.reshape(rows, cols).max(1, keepdims=True)).astype(np.float32).astype(np.float64)
    P = np.exp(sh) / np.exp(sh).sum(1, keepdims=True)
    assert np.all(np.abs(p.reshape(rows, cols) - P) <= 1e-6 * P + 1e-37)
    L = -np.log(np.sum(np.clip(P, 1e-7, 1 - 1e-7) * t.reshape(rows, cols), 1))
    assert np.all(np.abs(loss - L) <= 2e-6 * np.maximum(np.abs(L), 1.0))
    if cols <= 64:     # the oracle's probabilities come from short sequential sums: the direct bar
        assert np.all(np.abs(loss - loss_ref) <= 2e-6 * np.maximum(np.abs(L), 1.0)), np.max(np.abs(loss - loss_ref))
    # without a buffer for the probabilities: the same losses
    none, loss_only = hip.softmax_cce(rows, cols, x, t, want_probs=False)
    assert none is None and np.all(np.abs(loss_only - loss) <= 2e-6 * np.maximum(np.abs(L), 1.0))
    # gradient of mean_r loss_r wrt the logits: (p - t)/rows; the reference's chain is cce_grad
    # (unclipped p) pushed through softmax_grad
    for beta, up in ((0.0, 1.0), (1.0, 0.5)):
        lg0 = rng.uniform(n, -1, 1, tag=2, seed=SEED)
        got = hip.softmax_cce_grad(rows, cols, p, t, lg0.copy(), beta, up)
        exact = beta * lg0 + up * (p.astype(np.float64) - t) / rows
        bound = 2e-6 * (np.abs(p) + np.abs(t)) * abs(up) / rows + 1e-7 * np.abs(beta * lg0) + 1e-37
        assert np.all(np.abs(got - exact) <= bound)
    seed = orc.cce_grad(rows, cols, p_ref, t)
    if np.all(np.isfinite(seed)):                       # the chain divides by p: inf once a probability underflows
        chain = orc.softmax_grad(rows, cols, p_ref, seed)
        got = hip.softmax_cce_grad(rows, cols, p, t, np.zeros(n, np.float32))
        exact = (P - t.reshape(rows, cols)).ravel() / rows
        scale = (np.abs(P) + 1.0).ravel() / rows
        if cols <= 64:
            assert np.all(np.abs(got - chain) <= 4e-6 * scale), np.max(np.abs(got - chain) / scale)


def test_sgd_step_for_a_parameter_list_is_bit_exact(hip, orc):
    """Eleven tensors (two launches of up to eight), aligned and not, one of them long."""
    c = hip.ctx()
    lens = [1, 3, 64, 65, 1000, 4096, 10, 2048 * 10, 7, 300001, 129]
    pool_p, pool_g = c.empty(sum(lens) + 16), c.empty(sum(lens) + 16)
    p_host = rng.uniform(pool_p.n, -1, 1, tag=0, seed=SEED)
    g_host = rng.uniform(pool_g.n, -1, 1, tag=1, seed=SEED)
    pool_p.upload(p_host)
    pool_g.upload(g_host)
    offs, o = [], 1                                   # start one float in: the first tensors are not 16-byte aligned
    for n in lens:
        offs.append(o)
        o += n
    P = (C.c_void_p * len(lens))(*[pool_p.ptr + 4 * o for o in offs])
    G = (C.c_void_p * len(lens))(*[pool_g.ptr + 4 * o for o in offs])
    N = (C.c_size_t * len(lens))(*lens)
    c.call("slhip_sgd_step_multi", len(lens), P, G, N, 0.05)
    got = pool_p.numpy()
    want = p_host.copy()
    for o, n in zip(offs, lens):
        want[o:o + n] = orc.sgd_step(p_host[o:o + n].copy(), g_host[o:o + n], 0.05)
    assert np.array_equal(got, want)
    assert c.lib.slhip_sgd_step_multi(c.h, 0, P, G, N, 0.05) == -1
    pool_p.free()
    pool_g.free()


# --------------------------------------------------------------------------- views at odd offsets
@pytest.mark.parametrize("off", [1, 2, 3])
def test_operands_that_are_only_float_aligned(hip, orc, off):
    """Every operand sits `off` floats into its allocation (and outputs at a different offset): the
    vector paths must not assume 16-byte alignment.  Same bars as for aligned operands."""
    c = hip.ctx()
    rows, cols = 300, 1024
    n = rows * cols
    x = rng.uniform(n, -3, 3, tag=0, seed=SEED)
    g = rng.normal(n, 1.0, tag=1, seed=SEED)
    pool_x, pool_g = c.empty(n + 8), c.empty(n + 8)
    pool_o, pool_v = c.zeros(n + 8), c.zeros(max(rows, cols) + 8)
    dx, dg = pool_x.view(off, n), pool_g.view(off, n)
    oo = (off + 1) % 4
    do = pool_o.view(oo, n)
    dx.upload(x); dg.upload(g)
    vr, vc = pool_v.view(off, rows), pool_v.view(off, cols)
    say("offset", off)
    # reductions
    c.call("slhip_max_cols", rows, cols, dx.ptr, vr.ptr); assert np.array_equal(vr.numpy(), orc.max_cols(cols, x))
    c.call("slhip_max_rows", rows, cols, dx.ptr, vc.ptr); assert np.array_equal(vc.numpy(), orc.max_rows(cols, x))
    c.call("slhip_sum_cols", rows, cols, dx.ptr, vr.ptr)
    assert np.all(np.abs(vr.numpy() - x.reshape(rows, cols).sum(1, dtype=np.float64)) <= sum_bound(x, rows, cols, 1))
    c.call("slhip_sum_rows", rows, cols, dx.ptr, vc.ptr)
    assert np.all(np.abs(vc.numpy() - x.reshape(rows, cols).sum(0, dtype=np.float64)) <= sum_bound(x, rows, cols, 0))
    one = pool_v.view(off, 1)
    c.call("slhip_sum", n, dx.ptr, one.ptr)
    assert abs(float(one.numpy()[0]) - x.sum(dtype=np.float64)) <= 1e-6 * np.abs(x).sum(dtype=np.float64)
    # transpose, elementwise, bias row op: bit-exact
    c.call("slhip_transpose", rows, cols, dx.ptr, do.ptr, 0.0); assert np.array_equal(do.numpy(), orc.transpose(rows, cols, x))
    c.call("slhip_ew_binary", orc.MUL, n, dx.ptr, dg.ptr, do.ptr); assert np.array_equal(do.numpy(), orc.binary_ew(orc.MUL, x, g))
    c.call("slhip_ew_unary", orc.RELU, 0.0, 0.0, n, dx.ptr, do.ptr); assert np.array_equal(do.numpy(), orc.unary(orc.RELU, x))
    bias = x[:cols].copy()
    vc.upload(bias)
    c.call("slhip_add_row", rows, cols, dx.ptr, vc.ptr, do.ptr); assert np.array_equal(do.numpy(), orc.add_row(rows, cols, x, bias))
    c.call("slhip_memcpy_d2d", do.ptr, dx.ptr, 4 * n); assert np.array_equal(do.numpy(), x)
    # softmax forward / backward
    c.call("slhip_softmax", rows, cols, dx.ptr, do.ptr)
    s = do.numpy()
    ref = orc.softmax(rows, cols, x)
    assert np.all(np.abs(s - ref) <= 2e-6 * ref + 1e-37)
    c.call("slhip_softmax_grad", rows, cols, pool_x.view(oo, n).ptr, do.ptr, dg.ptr, 0.0)   # x's pool is free to overwrite now
    got = pool_x.view(oo, n).numpy()
    ob = orc.softmax_grad(rows, cols, s, g)
    S, G = s.reshape(rows, cols).astype(np.float64), g.reshape(rows, cols).astype(np.float64)
    bound = 2e-6 * (np.abs(S) * (np.abs(G) + (np.abs(S) * np.abs(G)).sum(1, keepdims=True))).ravel() + 1e-37
    assert np.all(np.abs(got - ob) <= bound)
    # GEMM, all forms, tiled and wave-per-tile sizes
    for (m, nn, k) in [(300, 256, 512), (96, 40, 64), (96, 40, 67), (300, 17, 1001)]:
        a = rng.uniform(m * k, -1, 1, tag=3, seed=SEED)
        b = rng.uniform(k * nn, -1, 1, tag=4, seed=SEED)
        da, db, dc = pool_x.view(off, m * k), pool_g.view(off, k * nn), pool_o.view(oo, m * nn)
        da.upload(a); db.upload(b)
        for ta, tb in ((0, 0), (0, 1), (1, 0)):
            c.call("slhip_sgemm", ta, tb, m, nn, k, da.ptr, db.ptr, dc.ptr, 0.0)
            exact, bound = gemm_bound(ta, tb, m, nn, k, a, b)
            assert np.all(np.abs(dc.numpy() - exact) <= bound), (m, nn, k, ta, tb)
    for z in (pool_x, pool_g, pool_o, pool_v):
        z.free()


# --------------------------------------------------------------------------- runtime
def test_context_on_a_callers_stream(hip, orc):
    """slhip_init_on_stream: ops run on a stream the caller created and still owns afterwards."""
    from sliced_amd import _lib
    rt = C.CDLL("libamdhip64.so")
    stream = C.c_void_p()
    assert rt.hipStreamCreate(C.byref(stream)) == 0
    lib = _lib.load()
    h = C.c_void_p()
    assert lib.slhip_init_on_stream(0, stream, C.byref(h)) == 0
    got = C.c_void_p()
    assert lib.slhip_stream(h, C.byref(got)) == 0 and got.value == stream.value
    assert lib.slhip_workspace_bytes(h) >= (64 << 20)
    name = C.create_string_buffer(64)
    assert lib.slhip_device_name(h, name, 64) == 0 and b"gfx950" in name.value
    n = 1000
    x = rng.uniform(n, -1, 1, tag=0, seed=SEED)
    dx, dy = C.c_void_p(), C.c_void_p()
    assert lib.slhip_malloc(h, 4 * n, C.byref(dx)) == 0 and lib.slhip_malloc(h, 4 * n, C.byref(dy)) == 0
    assert lib.slhip_memcpy_h2d(h, dx, x.ctypes.data, 4 * n) == 0
    assert lib.slhip_ew_unary(h, 0, 0.0, 0.0, n, dx, dy) == 0           # square, on the caller's stream
    assert rt.hipStreamSynchronize(stream) == 0                          # the caller waits on its own stream
    out = np.empty(n, np.float32)
    assert lib.slhip_memcpy_d2h(h, out.ctypes.data, dy, 4 * n) == 0
    assert np.array_equal(out, orc.unary(orc.SQUARE, x))
    assert lib.slhip_free(h, dx) == 0 and lib.slhip_free(h, dy) == 0
    assert lib.slhip_destroy(h) == 0
    assert rt.hipStreamQuery(stream) == 0                                # still a valid, idle stream
    assert rt.hipStreamDestroy(stream) == 0


def test_contexts_on_several_host_threads_do_not_disturb_each_other(hip):
    """Three contexts, each driven by its own host thread at the same time (ctypes releases the
    interpreter lock during a call), each with its own stream and workspace: a split-k product and
    a strided-axis sum (both keep partials in the workspace), a softmax, a transpose and a fused
    loss, thirty rounds each.  Every round of every thread equals, bit for bit, what one context
    computes alone: nothing in the library is shared between contexts but the error string, which
    is per thread."""
    import threading
    from sliced_amd.device import Context
    m, n, k = 96, 40, 8192                      # few tiles, long k: split over the grid, partials in the workspace
    rows, cols = 3000, 129

    def work(ctx, seed, rounds, out):
        a = ctx.array(rng.uniform(m * k, -1, 1, tag=0, seed=seed))
        b = ctx.array(rng.uniform(k * n, -1, 1, tag=1, seed=seed))
        x = ctx.array(rng.uniform(rows * cols, -4, 4, tag=2, seed=seed))
        cmat, colsum, soft, tr = ctx.empty(m * n), ctx.empty(cols), ctx.empty(rows * cols), ctx.empty(rows * cols)
        try:
            for _ in range(rounds):
                ctx.call("slhip_sgemm", 0, 0, m, n, k, a.ptr, b.ptr, cmat.ptr, 0.0)
                ctx.call("slhip_sum_rows", rows, cols, x.ptr, colsum.ptr)
                ctx.call("slhip_softmax", rows, cols, x.ptr, soft.ptr)
                ctx.call("slhip_transpose", rows, cols, soft.ptr, tr.ptr, 0.0)
                out.append((cmat.numpy(), colsum.numpy(), tr.numpy()))
                ctx.call("slhip_ew_unary", 6, 0.999, 0.0, rows * cols, x.ptr, x.ptr)      # the input moves on
        except Exception as e:                   # a failure in a thread has to reach the test
            out.append(e)
        for z in (a, b, x, cmat, colsum, soft, tr):
            z.free()

    seeds = [SEED + 1, SEED + 2, SEED + 3]
    alone = []
    for sd in seeds:
        res = []
        work(hip.ctx(), sd, 30, res)
        alone.append(res)
    ctxs = [Context(0) for _ in seeds]
    together = [[] for _ in seeds]
    threads = [threading.Thread(target=work, args=(c, sd, 30, res)) for c, sd, res in zip(ctxs, seeds, together)]
    say("three contexts on three threads")
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for c in ctxs:
        c.close()
    for res, ref in zip(together, alone):
        assert len(res) == len(ref) == 30 and not any(isinstance(r, Exception) for r in res + ref), [r for r in res if isinstance(r, Exception)]
        for got, want in zip(res, ref):
            for g, w in zip(got, want):
                assert np.array_equal(g, w)


# --------------------------------------------------------------------------- error behaviour
def test_invalid_arguments_return_status_not_crash(hip):
    c = hip.ctx()
    lib = c.lib
    x = c.zeros(16)
    assert lib.slhip_sum_rows(c.h, 0, 4, x.ptr, x.ptr) == -1            # zero rows
    assert lib.slhip_sum_rows(c.h, 1 << 40, 1 << 40, x.ptr, x.ptr) == -1  # rows*cols overflows
    assert lib.slhip_softmax(c.h, 4, 4, None, x.ptr) == -1              # null operand
    assert lib.slhip_sgemm(c.h, 0, 0, 2, 2, 2, x.ptr, x.ptr, x.ptr, 0.0) == -4   # C aliases A
    assert lib.slhip_transpose(c.h, 4, 4, x.ptr, x.ptr, 0.0) == -4
    assert lib.slhip_ew_unary(c.h, 99, 0.0, 0.0, 4, x.ptr, x.ptr) == -1
    assert lib.slhip_gemm_tail_policy(c.h, 7) == -1                      # unknown policies
    assert lib.slhip_gemm_tile_policy(c.h, 2) == -1 and lib.slhip_gemm_tile_policy(c.h, 5) == -1
    assert lib.slhip_gemm_tail_policy(c.h, 0) == 0 and lib.slhip_gemm_tile_policy(c.h, 0) == 0
    y = c.empty(16)
    assert lib.slhip_sgemm_relu_mask(c.h, 0, 0, 2, 2, 2, x.ptr, x.ptr, y.ptr, y.ptr, 0.0) == -4   # C aliases pre
    assert lib.slhip_sgemm_relu_bits(c.h, 0, 0, 2, 2, 2, x.ptr, x.ptr, y.ptr, y.ptr, 0.0) == -4   # C aliases the bits
    assert lib.slhip_sgemm_relu_bits(c.h, 0, 0, 2, 2, 2, x.ptr, x.ptr, None, y.ptr, 0.0) == -1
    assert lib.slhip_linear_fwd_bits(c.h, 2, 2, 2, x.ptr, x.ptr, None, y.ptr, y.ptr) == -4        # bits alias out
    assert lib.slhip_linear_fwd_bits(c.h, 2, 0, 2, x.ptr, x.ptr, None, y.ptr, x.ptr) == -1        # zero dimension
    assert lib.slhip_relu_grad_bits(c.h, 2, 2, None, y.ptr, x.ptr) == -1
    y.free()
    x.free()


# --------------------------------------------------------------------------- recorded sequences
def test_recorded_sequence_replays_like_eager_calls(hip, orc):
    """Record gemm (split-K) -> bias row op -> relu -> softmax -> column sums -> scaled copy once,
    replay it several times with eager work and waits in between, and compare every replay bit for
    bit with the same calls made eagerly on the same inputs."""
    c = hip.ctx()
    lib = c.lib
    m, k, n = 96, 1024, 40
    a0 = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)
    w = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
    bias = rng.uniform(n, -1, 1, tag=2, seed=SEED)
    da, dw, db = c.array(a0), c.array(w), c.array(bias)
    y, s, col, keep = c.empty(m * n), c.empty(m * n), c.zeros(n), c.zeros(n)

    def sequence():
        c.call("slhip_gemm", m, k, n, da.ptr, dw.ptr, y.ptr)
        c.call("slhip_add_row", m, n, y.ptr, db.ptr, y.ptr)
        c.call("slhip_ew_unary", 2, 0.0, 0.0, m * n, y.ptr, y.ptr)
        c.call("slhip_softmax", m, n, y.ptr, s.ptr)
        c.call("slhip_memset", col.ptr, 0, col.nbytes)
        c.call("slhip_sum_rows", m, n, s.ptr, col.ptr)
        c.call("slhip_memcpy_d2d", keep.ptr, col.ptr, col.nbytes)
        # the input moves on, so that every replay computes something new
        c.call("slhip_ew_unary", 6, 0.5, 0.0, m * k, da.ptr, da.ptr)

    eager = []
    for _ in range(4):
        sequence()
        eager.append((keep.numpy(), s.numpy()))
    da.upload(a0)

    c.call("slhip_graph_begin")
    # waiting or allocating calls are refused while recording, and leave the recording intact
    p = C.c_void_p()
    assert lib.slhip_malloc(c.h, 64, C.byref(p)) == -5
    assert lib.slhip_sync(c.h) == -5
    assert lib.slhip_memset(c.h, col.ptr, 1, 4) == -5
    assert lib.slhip_graph_begin(c.h) == -5
    sequence()
    g = C.c_void_p()
    c.call("slhip_graph_end", C.byref(g))
    nodes = C.c_size_t()
    assert lib.slhip_graph_node_count(g, C.byref(nodes)) == 0
    say("recorded nodes:", nodes.value)
    assert nodes.value >= 8
    # nothing ran while recording
    assert np.array_equal(da.numpy(), a0)
    none = C.c_void_p()
    assert lib.slhip_graph_end(c.h, C.byref(none)) == -5    # not recording any more

    scratch = c.empty(1 << 16)
    for i in range(4):
        c.call("slhip_graph_launch", g)
        # eager work on other buffers and a wait between the replays
        c.call("slhip_fill", scratch.n, float(i), scratch.ptr)
        c.sync()
        got_keep, got_s = keep.numpy(), s.numpy()
        assert np.array_equal(got_keep, eager[i][0]), i
        assert np.array_equal(got_s, eager[i][1]), i
        assert float(scratch.numpy()[-1]) == float(i)
    # against the oracle as well (first replay's inputs)
    ref = orc.softmax(m, n, orc.unary(orc.RELU, orc.add_row(m, n, orc.gemm(m, n, k, a0, w), bias)))
    assert np.max(np.abs(eager[0][1] - ref)) <= 1e-5
    assert lib.slhip_graph_destroy(g) == 0
    for z in (da, dw, db, y, s, col, keep, scratch):
        z.free()


def test_recording_holds_every_product_route_and_kernel_family(hip):
    """One recording with the products that take the library's side routes (a few rows times a large
    matrix, computed as the transposed product with a transposed combine; A^T B with 24 columns;
    split k with its combine; a grid with a spread tail; tall A; the wave-per-tile kernel), the
    transposes that stage more rows than they write, reductions that keep partials in the workspace,
    softmax on short, medium and two-sweep rows, the fused losses and a fused elementwise chain:
    three replays, eager work between them, each equal bit for bit to the same calls made eagerly.
    State that a route keeps on the context between its launches must not leak into a recording."""
    c = hip.ctx()
    lib = c.lib
    products = [(0, 0, 16, 2048, 4096), (0, 1, 8, 4096, 2048), (1, 0, 2048, 24, 8192), (0, 0, 96, 40, 8192),
                (0, 0, 1100, 1100, 700), (0, 0, 16384, 16, 2048), (0, 0, 40, 72, 15), (1, 0, 300, 10, 2048), (0, 1, 1, 2048, 2048)]
    mats = [(8191, 1025), (100003, 56), (64, 5000), (300, 129), (5000, 10), (9, 40000)]
    bufs = []

    def dev(n, tag):
        b = c.array(rng.uniform(n, -1, 1, tag=tag, seed=SEED + n % 1000))
        bufs.append(b)
        return b

    def out(n):
        b = c.zeros(n)
        bufs.append(b)
        return b

    P = [(ta, tb, m, n, k, dev(m * k, 0), dev(k * n, 1), out(m * n)) for ta, tb, m, n, k in products]
    M = [(r, cl, dev(r * cl, 2), out(r * cl), out(r * cl), out(cl), out(r), out(r * cl), out(r)) for r, cl in mats]
    outputs = [p[7] for p in P] + [b for mrow in M for b in mrow[3:]]

    def sequence():
        for ta, tb, m, n, k, a, b, cm in P:
            c.call("slhip_sgemm", ta, tb, m, n, k, a.ptr, b.ptr, cm.ptr, 0.0)
        for r, cl, x, tr, sm, colsum, rowmax, gr, loss in M:
            c.call("slhip_transpose", r, cl, x.ptr, tr.ptr, 0.0)
            c.call("slhip_softmax", r, cl, x.ptr, sm.ptr)
            c.call("slhip_sum_rows", r, cl, sm.ptr, colsum.ptr)
            c.call("slhip_max_cols", r, cl, x.ptr, rowmax.ptr)
            c.call("slhip_softmax_grad", r, cl, gr.ptr, sm.ptr, tr.ptr, 0.0)         # tr: any tensor of that size as upstream gradient
            c.call("slhip_softmax_cce", r, cl, x.ptr, sm.ptr, None, loss.ptr)        # sm as (soft) targets
            c.call("slhip_ew_unary", 6, 0.75, 0.0, r * cl, x.ptr, x.ptr)             # the input moves on
        for ta, tb, m, n, k, a, b, cm in P:
            c.call("slhip_ew_unary", 6, 0.9, 0.0, m * k, a.ptr, a.ptr)

    def snapshot():
        return [b.numpy() for b in outputs]

    inputs0 = [(p[5], p[5].numpy()) for p in P] + [(mrow[2], mrow[2].numpy()) for mrow in M]
    eager = []
    for _ in range(3):
        sequence()
        eager.append(snapshot())
    for b, h in inputs0:
        b.upload(h)
    for b in outputs:
        c.call("slhip_memset", b.ptr, 0, b.nbytes)
    c.call("slhip_graph_begin")
    sequence()
    g = C.c_void_p()
    c.call("slhip_graph_end", C.byref(g))
    scratch = c.empty(1 << 16)
    ea, eb, ec = dev(16 * 4096, 5), dev(4096 * 2048, 6), out(16 * 2048)
    for i in range(3):
        say("replay", i)
        c.call("slhip_graph_launch", g)
        c.call("slhip_fill", scratch.n, float(i), scratch.ptr)
        # an eager product on the same context between the replays: its route leaves its own state behind
        c.call("slhip_sgemm", 0, 0, 16, 2048, 4096, ea.ptr, eb.ptr, ec.ptr, 0.0)
        c.sync()
        got = snapshot()
        for j, (gv, ev) in enumerate(zip(got, eager[i])):
            assert np.array_equal(gv, ev, equal_nan=True), (i, j)
    assert lib.slhip_graph_destroy(g) == 0
    scratch.free()
    for z in bufs:
        z.free()


def test_relu_mask_as_bits_equals_the_float_mask(hip, orc):
    """slhip_linear_fwd_bits / slhip_sgemm_relu_bits / slhip_relu_grad_bits against the float forms
    (linear_fwd with pre-activations, sgemm_relu_mask, the relu gradient): the same values within the
    GEMM bound, a mask that agrees with the exact pre-activations wherever their sign is not within
    that bound of zero, and outputs that are zero exactly where the mask is clear."""
    # the last six: an output side of at most 32 or a short K, which the tile loads are not written for
    for (m, k, n) in [(256, 96, 128), (300, 70, 200), (129, 33, 97), (1024, 784, 2048), (520, 64, 36),
                      (300, 40, 1), (257, 70, 2), (130, 33, 3), (520, 64, 20), (20, 100, 200), (300, 8, 200)]:
        say("bit mask forward", m, k, n)
        x = rng.uniform(m * k, -1, 1, tag=0, seed=SEED)
        w = rng.uniform(k * n, -1, 1, tag=1, seed=SEED)
        bias = rng.uniform(n, -1, 1, tag=2, seed=SEED)
        out, bits = hip.linear_fwd_bits(m, k, n, x, w, bias)
        exact, bound = gemm_bound(0, 0, m, n, k, x, w)
        pre_ref = exact.reshape(m, n) + bias.astype(np.float64)
        out = out.reshape(m, n)
        unpacked = ((bits[:, np.arange(n) // 32] >> (np.arange(n) % 32).astype(np.uint32)) & 1).astype(bool)
        sure = np.abs(pre_ref) > bound.reshape(m, n) + 1e-6          # sign not in doubt
        assert np.array_equal(unpacked[sure], (pre_ref >= 0)[sure])
        assert np.all(np.abs(out - np.where(unpacked, pre_ref, 0)) <= bound.reshape(m, n) + 1e-6)
        assert np.all(out[~unpacked] == 0) and np.all(out[unpacked] >= 0)
        if n % 32:                                                    # bits beyond the last column stay clear
            assert not np.any(bits[:, -1] >> np.uint32(n % 32))
    for (m, n, k, ta, tb) in [(256, 128, 96, 0, 1), (300, 200, 70, 0, 1), (129, 97, 33, 0, 0), (1024, 2048, 512, 0, 1),
                              (1031, 260, 10, 0, 1), (4100, 64, 3, 1, 0), (2050, 1028, 7, 1, 1), (700, 512, 12, 0, 0),
                              (200, 130, 64, 1, 0), (140, 260, 40, 1, 1),
                              (300, 3, 40, 0, 0), (300, 1, 70, 0, 0), (3, 200, 40, 1, 0), (2, 130, 64, 1, 1),
                              (520, 20, 64, 0, 1), (1, 1, 33, 0, 0), (40, 2, 17, 1, 1)]:
        say("bit mask backward", m, n, k, ta, tb)
        a, b = gemm_operands(ta, tb, m, n, k)
        exact, bound = gemm_bound(ta, tb, m, n, k, a, b)
        pre = rng.uniform(m * n, -1, 1, tag=4, seed=SEED)
        keep = (pre >= 0).reshape(m, n)
        words = (n + 31) // 32
        bits = np.zeros((m, words), np.uint32)
        for c in range(n):
            bits[:, c // 32] |= keep[:, c].astype(np.uint32) << np.uint32(c % 32)
        got = hip.sgemm_relu_bits(ta, tb, m, n, k, a, b, bits)
        assert np.all(np.abs(got - np.where(keep.ravel(), exact, 0)) <= bound)
        assert np.all(got[~keep.ravel()] == 0)
        c0 = rng.uniform(m * n, -1, 1, tag=2, seed=SEED)
        assert np.array_equal(hip.sgemm_relu_bits(ta, tb, m, n, k, a, b, bits, c=c0.copy(), beta=1.0), c0 + got)
        g = rng.uniform(m * n, -1, 1, tag=5, seed=SEED)
        assert np.array_equal(hip.relu_grad_bits(m, n, bits, c0.copy(), g), c0 + np.where(keep.ravel(), g, 0 * g))
