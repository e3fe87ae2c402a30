"""slhip_sum_rows_static, the entry point that allocates nothing (its partial sums live in a
file-scope device array), against slhip_sum_rows through the C ABI: the same kernels, so the same
bits.  Two calls in a row share the array, the second on a smaller input; shapes cover the
one-kernel form, one and two streaming stages, rows of odd length, a single column and a single row.
This file is collected last on purpose, so that a failure here hides no other test."""
import ctypes as C

import numpy as np
import pytest

from sliced_amd import rng

pytestmark = pytest.mark.gpu
SEED = 0x51CED


def say(*a):
    print(*a, flush=True)


def test_static_scratch_variant_matches_sum_rows(hip, orc):
    shapes = [(8192, 4096), (2048, 1000), (16384, 2049), (300, 77), (1 << 20, 10), (64, 131072), (1 << 21, 1),
              (1, 5000), (4096, 64), (37, 3)]
    for i, (rows, cols) in enumerate(shapes):
        say("sum_rows_static", rows, cols)
        x = rng.uniform(rows * cols, -10, 10, tag=i, seed=SEED)
        want = hip.sum_rows(cols, x)
        got = hip.sum_rows_static(cols, x)
        assert np.array_equal(got, want), (rows, cols)
        # and against the CPU restatement of the reference, on the backward-error scale of a sum
        if rows * cols <= (1 << 24):
            ref = orc.sum_rows(cols, x)
            scale = np.abs(x.reshape(rows, cols).astype(np.float64)).sum(axis=0)
            assert np.all(np.abs(got.astype(np.float64) - ref) <= 2e-6 * scale + 1e-30), (rows, cols)


def test_two_calls_in_a_row_second_smaller(hip):
    """Back-to-back calls on one context share the scratch array; the second, smaller input must not
    see anything the first left there."""
    c = hip.ctx()
    big = rng.uniform(16384 * 4096, -10, 10, tag=20, seed=SEED)
    small = rng.uniform(2048 * 1000, -10, 10, tag=21, seed=SEED)
    want_big, want_small = hip.sum_rows(4096, big), hip.sum_rows(1000, small)
    dbig, dsmall = c.array(big), c.array(small)
    obig, osmall = c.empty(4096), c.empty(1000)
    say("static, 16384 x 4096 then 2048 x 1000, no wait in between")
    c.call("slhip_sum_rows_static", 16384, 4096, dbig.ptr, obig.ptr)
    c.call("slhip_sum_rows_static", 2048, 1000, dsmall.ptr, osmall.ptr)
    assert np.array_equal(obig.numpy(), want_big)
    assert np.array_equal(osmall.numpy(), want_small)
    for b in (dbig, dsmall, obig, osmall):
        b.free()


def test_static_variant_neither_uses_the_workspace_nor_allocates(hip):
    """The context workspace, where slhip_sum_rows keeps its partials, is filled with NaN before the
    call: a result that still has the bits of slhip_sum_rows did not pass through it.  Free device
    memory is the same before and after the calls."""
    c = hip.ctx()
    # free device memory as the HIP runtime the library itself runs on sees it (the library has loaded it:
    # this is the same instance, not a second runtime in the process)
    rt = C.CDLL("libamdhip64.so.7", mode=C.RTLD_GLOBAL)
    rt.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    rt.hipMemGetInfo.restype = C.c_int

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    rows, cols = 16384, 2049                    # two streaming stages: partials must live somewhere
    x = rng.uniform(rows * cols, -10, 10, tag=30, seed=SEED)
    want = hip.sum_rows(cols, x)
    dx, out = c.array(x), c.empty(cols)
    ws = C.c_void_p()
    c.call("slhip_workspace", C.byref(ws))
    ws_floats = c.lib.slhip_workspace_bytes(c.h) // 4
    assert ws.value and ws_floats >= (1 << 20)
    c.call("slhip_fill", ws_floats, float("nan"), ws.value)
    c.sync()
    free_bytes()                                # the first query sets the runtime's own bookkeeping up
    free0 = free_bytes()
    for _ in range(3):
        c.call("slhip_sum_rows_static", rows, cols, dx.ptr, out.ptr)
    c.sync()
    assert free_bytes() == free0
    got = out.numpy()
    assert not np.isnan(got).any() and np.array_equal(got, want)
    # the control: the workspace variant does read what the poisoned workspace holds only after
    # writing it, so it is still right - and leaves the NaNs overwritten
    assert np.array_equal(hip.sum_rows(cols, x), want)
    dx.free()
    out.free()


def test_static_variant_inside_a_recorded_sequence(hip):
    """The setting the entry point is for: between slhip_graph_begin and slhip_graph_end nothing may
    allocate.  The recording is replayed three times with eager work and waits in between; every
    replay gives the bits of the eager call."""
    c = hip.ctx()
    rows, cols = 8192, 1000
    x = rng.uniform(rows * cols, -10, 10, tag=31, seed=SEED)
    want = hip.sum_rows(cols, x)
    dx, out = c.array(x), c.empty(cols)
    c.call("slhip_graph_begin")
    try:
        c.call("slhip_sum_rows_static", rows, cols, dx.ptr, out.ptr)
    finally:
        g = C.c_void_p()
        c.call("slhip_graph_end", C.byref(g))
    for replay in range(3):
        say("replay", replay)
        c.call("slhip_fill", cols, -1.0, out.ptr)
        c.sync()
        c.call("slhip_graph_launch", g)
        assert np.array_equal(out.numpy(), want), replay
        other = rng.uniform(64 * 300, -1, 1, tag=40 + replay, seed=SEED)
        hip.sum_rows_static(300, other)              # an eager call shares the array between replays
    c.lib.slhip_graph_destroy(g)
    dx.free()
    out.free()


def test_static_variant_rejects_what_does_not_fit(hip):
    c = hip.ctx()
    x = c.zeros(2 * 131076)
    out = c.empty(131076)
    rc = c.lib.slhip_sum_rows_static(c.h, 2, 131076, x.ptr, out.ptr)
    assert rc == -3
    assert b"131072" in c.lib.slhip_last_error_string()
    assert c.lib.slhip_sum_rows_static(c.h, 0, 4, x.ptr, out.ptr) == -1
    assert c.lib.slhip_sum_rows_static(c.h, 2, 4, None, out.ptr) == -1
    x.free()
    out.free()
