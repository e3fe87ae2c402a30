"""Thin Python handle layer over the C ABI: a context (one HIP stream) and f32 device buffers.

This is plumbing for tests and benchmarks; all computation happens in libsliced_hip.so.
"""
import ctypes as C

import numpy as np

from . import _lib


class Buf:
    """A float32 device allocation owned by a Context."""

    __slots__ = ("ctx", "ptr", "n", "_owned")

    def __init__(self, ctx, ptr, n, owned=True):
        self.ctx, self.ptr, self.n, self._owned = ctx, ptr, int(n), owned

    @property
    def nbytes(self):
        return self.n * 4

    def numpy(self):
        out = np.empty(self.n, np.float32)
        self.ctx.call("slhip_memcpy_d2h", out.ctypes.data, self.ptr, self.nbytes)
        return out

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32).ravel()
        assert arr.size == self.n, (arr.size, self.n)
        self.ctx.call("slhip_memcpy_h2d", self.ptr, arr.ctypes.data, self.nbytes)
        return self

    def view(self, offset, n):
        """Sub-range sharing this allocation (offset and n in elements)."""
        assert 0 <= offset and offset + n <= self.n
        return Buf(self.ctx, self.ptr + 4 * offset, n, owned=False)

    def free(self):
        if self._owned and self.ptr:
            self.ctx.call("slhip_free", self.ptr)
            self.ptr = 0


class Context:
    def __init__(self, ordinal=0):
        self.lib = _lib.load()
        h = C.c_void_p()
        _lib.check(self.lib.slhip_init(ordinal, C.byref(h)), "slhip_init")
        self.h = h
        self._bufs = []

    def call(self, name, *args):
        rc = getattr(self.lib, name)(self.h, *args)
        _lib.check(rc, name)

    def name(self):
        b = C.create_string_buffer(128)
        self.call("slhip_device_name", b, 128)
        return b.value.decode()

    def last_gemm_plan(self):
        """Kernel and plan of the last product issued on this context, as text."""
        b = C.create_string_buffer(256)
        self.call("slhip_gemm_plan_describe", b, 256)
        return b.value.decode()

    def empty(self, n):
        p = C.c_void_p()
        self.call("slhip_malloc", int(n) * 4, C.byref(p))
        return Buf(self, p.value, n)

    def zeros(self, n):
        b = self.empty(n)
        self.call("slhip_memset", b.ptr, 0, b.nbytes)
        return b

    def array(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32).ravel()
        return self.empty(arr.size).upload(arr)

    def uniform(self, n, lo, hi, tag, seed):
        b = self.empty(n)
        self.call("slhip_rand_uniform", seed, tag, float(lo), float(hi), int(n), b.ptr)
        return b

    def sync(self):
        self.call("slhip_sync")

    # ---- HIP-event timing on the context's own stream
    def event(self):
        e = C.c_void_p()
        self.call("slhip_event_create", C.byref(e))
        return e

    def record(self, ev):
        self.call("slhip_event_record", ev)

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        _lib.check(self.lib.slhip_event_elapsed_ms(start, stop, C.byref(ms)), "slhip_event_elapsed_ms")
        return ms.value

    def time_ms(self, fn, iters, warmup=2):
        """Average milliseconds per call of fn() measured with HIP events on this stream."""
        for _ in range(warmup):
            fn()
        e0, e1 = self.event(), self.event()
        self.record(e0)
        for _ in range(iters):
            fn()
        self.record(e1)
        ms = self.elapsed_ms(e0, e1) / iters
        self.lib.slhip_event_destroy(e0)
        self.lib.slhip_event_destroy(e1)
        return ms

    def close(self):
        if self.h:
            self.lib.slhip_destroy(self.h)
            self.h = None
