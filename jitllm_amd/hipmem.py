"""Device memory, copies and event timing over the HIP runtime the C ABI uses.

Plumbing for tests and benchmarks: buffers are plain device allocations whose
addresses go to the *_dev entry points.  The runtime is the one libjlmi.so
resolved (jl_hip_runtime), so a process holds exactly one.
"""
import ctypes as C

import numpy as np

from . import _lib

_H2D, _D2H, _D2D = 1, 2, 3
_hip = None


def hip():
    global _hip
    if _hip is None:
        lib = _lib.load()
        lib.jl_hip_runtime.restype = C.c_char_p
        name = lib.jl_hip_runtime().decode()
        if not name:
            raise RuntimeError("no HIP runtime could be loaded")
        h = C.CDLL(name)
        h.hipGetErrorString.restype = C.c_char_p
        h.hipGetErrorString.argtypes = [C.c_int]
        h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        h.hipFree.argtypes = [C.c_void_p]
        h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        h.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        h.hipMemsetAsync.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]
        h.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        h.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        h.hipEventSynchronize.argtypes = [C.c_void_p]
        h.hipStreamSynchronize.argtypes = [C.c_void_p]
        h.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        h.hipEventDestroy.argtypes = [C.c_void_p]
        h.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        h.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        h.hipStreamDestroy.argtypes = [C.c_void_p]
        h.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        h.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        h.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        h.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        h.hipGraphExecDestroy.argtypes = [C.c_void_p]
        h.hipGraphDestroy.argtypes = [C.c_void_p]
        _hip = h
    return _hip


def check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what}: {hip().hipGetErrorString(rc).decode()}")


def synchronize():
    check(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")


def mem_info():
    free, total = C.c_size_t(), C.c_size_t()
    check(hip().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value, total.value


class DeviceArray:
    """A device allocation shaped like a numpy array."""

    def __init__(self, arr=None, shape=None, dtype=None, fill=None):
        if arr is not None:
            arr = np.ascontiguousarray(arr)
            shape, dtype = arr.shape, arr.dtype
        self.shape, self.dtype = tuple(np.atleast_1d(shape)) if np.isscalar(shape) else tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        check(hip().hipMalloc(C.byref(p), max(self.nbytes, 16)), "hipMalloc")
        self.ptr = p.value
        if arr is not None:
            self.put(arr)
        elif fill is not None:
            self.put(np.full(self.shape, fill, self.dtype))

    def put(self, arr):
        arr = np.ascontiguousarray(arr, self.dtype)
        assert arr.nbytes == self.nbytes
        check(hip().hipMemcpy(self.ptr, arr.ctypes.data, self.nbytes, _H2D), "hipMemcpy H2D")

    def get(self):
        out = np.empty(self.shape, self.dtype)
        check(hip().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, _D2H), "hipMemcpy D2H")
        return out

    def copy_from(self, other):
        assert other.nbytes == self.nbytes
        check(hip().hipMemcpy(self.ptr, other.ptr, self.nbytes, _D2D), "hipMemcpy D2D")

    def zero(self):
        check(hip().hipMemset(self.ptr, 0, self.nbytes), "hipMemset")

    def free(self):
        if getattr(self, "ptr", None):
            hip().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Event:
    def __init__(self):
        self.e = C.c_void_p()
        check(hip().hipEventCreate(C.byref(self.e)), "hipEventCreate")

    def record(self, stream):
        check(hip().hipEventRecord(self.e, stream), "hipEventRecord")

    def synchronize(self):
        check(hip().hipEventSynchronize(self.e), "hipEventSynchronize")

    def elapsed_ms(self, end):
        ms = C.c_float()
        check(hip().hipEventElapsedTime(C.byref(ms), self.e, end.e), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            hip().hipEventDestroy(self.e)
        except Exception:
            pass


class Stream:
    """A HIP stream of the caller's own (default priority), to pass where an entry point takes one."""

    def __init__(self):
        self.handle = C.c_void_p()
        check(hip().hipStreamCreate(C.byref(self.handle)), "hipStreamCreate")

    def synchronize(self):
        check(hip().hipStreamSynchronize(self.handle), "hipStreamSynchronize")

    def destroy(self):
        if self.handle:
            check(hip().hipStreamDestroy(self.handle), "hipStreamDestroy")
            self.handle = C.c_void_p()


class Gate:
    """Keeps a stream busy for a chosen time with the library's wait kernel (one wavefront
    watching the constant clock, no memory traffic).  Launches enqueued behind it pile up in the
    queue while it runs and then execute back to back, so a timed window measures the device
    and not the host's launch rate."""

    def __init__(self, dev):
        self.dev = dev

    def hold(self, stream, us):
        """Keep `stream` busy for at least `us` microseconds."""
        us = int(us) + 1
        while us > 0:
            self.dev.probe_dev(2, None, min(us, 100000), stream=stream)
            us -= 100000

    def free(self):
        pass


def timed_windows(enqueue, steps, stream, windows=9, gate=None, host_us=None):
    """Median over `windows` timed windows of `steps` launches each: (ms per step of the median
    window, every window's ms per step).  enqueue(i) enqueues step i on `stream`; the window is
    bracketed by HIP events recorded on that stream.  With a gate, the window is enqueued
    behind work that lasts 1.5 x the host's time to enqueue it (host_us per step, measured
    here over 32 untimed steps when not given) plus 100 us, so the whole window is queued
    before its first launch starts."""
    import time
    i = 0
    if gate is not None and host_us is None:
        t0 = time.perf_counter()
        for _ in range(32):
            enqueue(i)
            i += 1
        host_us = (time.perf_counter() - t0) * 1e6 / 32
        check(hip().hipStreamSynchronize(stream), "hipStreamSynchronize")
    per = []
    for _ in range(windows):
        e0, e1 = Event(), Event()
        if gate is not None:
            gate.hold(stream, 1.5 * steps * host_us + 100.0)
        e0.record(stream)
        for _ in range(steps):
            enqueue(i)
            i += 1
        e1.record(stream)
        e1.synchronize()
        per.append(e0.elapsed_ms(e1) / steps)
    return float(np.median(per)), per


class Graph:
    """A HIP graph captured from a stream: `with Graph.capture(stream) as g: <enqueue work>`,
    then g.launch(stream) replays the recorded launches with one submission."""

    _THREAD_LOCAL = 1  # hipStreamCaptureModeThreadLocal

    def __init__(self, stream):
        self.stream, self.graph, self.exe = stream, C.c_void_p(), C.c_void_p()

    @classmethod
    def capture(cls, stream):
        return cls(stream)

    def __enter__(self):
        check(hip().hipStreamBeginCapture(self.stream, self._THREAD_LOCAL), "hipStreamBeginCapture")
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = hip().hipStreamEndCapture(self.stream, C.byref(self.graph))
        if exc_type is None:
            check(rc, "hipStreamEndCapture")
            check(hip().hipGraphInstantiate(C.byref(self.exe), self.graph, None, None, 0), "hipGraphInstantiate")
        return False

    def launch(self, stream=None):
        check(hip().hipGraphLaunch(self.exe, stream if stream is not None else self.stream), "hipGraphLaunch")

    def __del__(self):
        try:
            if self.exe:
                hip().hipGraphExecDestroy(self.exe)
            if self.graph:
                hip().hipGraphDestroy(self.graph)
        except Exception:
            pass
