"""Minimal ctypes view of the HIP runtime the C-ABI library is linked against:
device buffers, copies, streams and events for callers that keep activations
resident in HBM (benchmarks, tests).  Using the very runtime instance that
libnative_hip.so loaded avoids a second HIP runtime in the process."""
import ctypes as C

import numpy as np

_rt = None

H2D, D2H = 1, 2


class HipRuntimeError(RuntimeError):
    pass


def rt():
    global _rt
    if _rt is None:
        from . import load_library
        load_library()  # pulls libamdhip64 in; CDLL below resolves to that same instance
        lib = C.CDLL("libamdhip64.so", mode=C.RTLD_GLOBAL)
        lib.hipGetErrorString.restype = C.c_char_p
        lib.hipGetErrorString.argtypes = [C.c_int]
        lib.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        lib.hipFree.argtypes = [C.c_void_p]
        lib.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        lib.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        lib.hipStreamCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
        lib.hipStreamSynchronize.argtypes = [C.c_void_p]
        lib.hipStreamDestroy.argtypes = [C.c_void_p]
        lib.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        lib.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        lib.hipEventSynchronize.argtypes = [C.c_void_p]
        lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        lib.hipEventDestroy.argtypes = [C.c_void_p]
        lib.hipSetDevice.argtypes = [C.c_int]
        lib.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        lib.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        lib.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        lib.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        lib.hipGraphExecDestroy.argtypes = [C.c_void_p]
        lib.hipGraphDestroy.argtypes = [C.c_void_p]
        _rt = lib
    return _rt


def check(code, what="HIP call"):
    if code != 0:
        raise HipRuntimeError(f"{what}: {rt().hipGetErrorString(code).decode()}")


class DeviceBuffer:
    def __init__(self, nbytes):
        self.nbytes = nbytes
        p = C.c_void_p()
        check(rt().hipMalloc(C.byref(p), max(nbytes, 1)), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        check(rt().hipMemcpy(b.ptr, a.ctypes.data, a.nbytes, H2D), "hipMemcpy H2D")
        return b

    def upload(self, a):
        """Overwrite the start of the buffer with the bytes of `a` (synchronous)."""
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        check(rt().hipMemcpy(self.ptr, a.ctypes.data, a.nbytes, H2D), "hipMemcpy H2D")

    def to_numpy(self, dtype, count=None):
        dt = np.dtype(dtype)
        n = self.nbytes // dt.itemsize if count is None else count
        out = np.empty(n, dt)
        check(rt().hipMemcpy(out.ctypes.data, self.ptr, n * dt.itemsize, D2H), "hipMemcpy D2H")
        return out

    def fill_byte(self, value):
        check(rt().hipMemset(self.ptr, value, self.nbytes), "hipMemset")

    def free(self):
        if self.ptr:
            rt().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        p = C.c_void_p()
        check(rt().hipStreamCreateWithFlags(C.byref(p), 1), "hipStreamCreate")  # non-blocking, default priority
        self.ptr = p.value

    def synchronize(self):
        check(rt().hipStreamSynchronize(self.ptr), "hipStreamSynchronize")

    def destroy(self):
        if self.ptr:
            rt().hipStreamDestroy(self.ptr)
            self.ptr = None


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(rt().hipEventCreate(C.byref(p)), "hipEventCreate")
        self.ptr = p.value

    def record(self, stream):
        check(rt().hipEventRecord(self.ptr, stream.ptr if stream else None), "hipEventRecord")

    def synchronize(self):
        check(rt().hipEventSynchronize(self.ptr), "hipEventSynchronize")

    def elapsed_ms(self, later):
        ms = C.c_float()
        check(rt().hipEventElapsedTime(C.byref(ms), self.ptr, later.ptr), "hipEventElapsedTime")
        return ms.value

    def destroy(self):
        if self.ptr:
            rt().hipEventDestroy(self.ptr)
            self.ptr = None


class Graph:
    """A stream capture of whatever `enqueue(stream)` launches, replayable with launch()."""

    def __init__(self, stream, enqueue):
        check(rt().hipStreamBeginCapture(stream.ptr, 0), "hipStreamBeginCapture")  # global mode
        try:
            enqueue(stream)
        finally:
            g = C.c_void_p()
            code = rt().hipStreamEndCapture(stream.ptr, C.byref(g))
        check(code, "hipStreamEndCapture")
        self.graph = g.value
        ex = C.c_void_p()
        check(rt().hipGraphInstantiate(C.byref(ex), self.graph, None, None, 0), "hipGraphInstantiate")
        self.exec = ex.value
        self.stream = stream

    def launch(self):
        check(rt().hipGraphLaunch(self.exec, self.stream.ptr), "hipGraphLaunch")

    def destroy(self):
        if self.exec:
            rt().hipGraphExecDestroy(self.exec)
            rt().hipGraphDestroy(self.graph)
            self.exec = self.graph = None


def device_synchronize():
    check(rt().hipDeviceSynchronize(), "hipDeviceSynchronize")
