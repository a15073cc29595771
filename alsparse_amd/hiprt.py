"""Minimal ctypes bindings of the HIP runtime: device buffers, copies, events.

Plumbing for tests and the benchmark only -- the library itself never goes
through Python.  Buffers are plain device pointers, exactly what the C API takes.
"""
import ctypes
import os

import numpy as np

_hip = None

H2D, D2H, D2D = 1, 2, 3


class HipError(RuntimeError):
    pass


def lib():
    global _hip
    if _hip is None:
        last = None
        for name in ("libamdhip64.so", "/opt/rocm/lib/libamdhip64.so", "libamdhip64.so.7"):
            try:
                _hip = ctypes.CDLL(name, mode=ctypes.RTLD_GLOBAL)
                break
            except OSError as e:  # pragma: no cover
                last = e
        if _hip is None:
            raise HipError("HIP runtime not found: %s" % last)
        _hip.hipGetErrorString.restype = ctypes.c_char_p
        _hip.hipGetErrorString.argtypes = [ctypes.c_int]
    return _hip


def check(err, what=""):
    if err != 0:
        raise HipError("%s failed: %s (%d)" % (what or "HIP call", lib().hipGetErrorString(err).decode(), err))


def device_count():
    n = ctypes.c_int(0)
    try:
        err = lib().hipGetDeviceCount(ctypes.byref(n))
    except HipError:
        return 0
    return n.value if err == 0 else 0


def set_device(i=0):
    check(lib().hipSetDevice(ctypes.c_int(i)), "hipSetDevice")


def synchronize():
    check(lib().hipDeviceSynchronize(), "hipDeviceSynchronize")


def mem_info():
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    check(lib().hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)), "hipMemGetInfo")
    return free.value, total.value


class DeviceArray:
    """A typed device allocation.  ``ptr`` is the raw device address."""

    def __init__(self, shape, dtype):
        self.shape = tuple(np.atleast_1d(shape).tolist()) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        check(lib().hipMalloc(ctypes.byref(p), ctypes.c_size_t(max(self.nbytes, 1))), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        d.copy_from(a)
        return d

    def copy_from(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.nbytes, self.nbytes)
        if self.nbytes:
            check(lib().hipMemcpy(ctypes.c_void_p(self.ptr), a.ctypes.data_as(ctypes.c_void_p),
                                  ctypes.c_size_t(self.nbytes), ctypes.c_int(H2D)), "hipMemcpy H2D")
        return self

    def copy_from_device(self, other):
        assert other.nbytes == self.nbytes
        if self.nbytes:
            check(lib().hipMemcpy(ctypes.c_void_p(self.ptr), ctypes.c_void_p(other.ptr),
                                  ctypes.c_size_t(self.nbytes), ctypes.c_int(D2D)), "hipMemcpy D2D")
        return self

    def fill_bytes(self, value=0):
        if self.nbytes:
            check(lib().hipMemset(ctypes.c_void_p(self.ptr), ctypes.c_int(value), ctypes.c_size_t(self.nbytes)), "hipMemset")
        return self

    def to_numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            check(lib().hipMemcpy(out.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(self.ptr),
                                  ctypes.c_size_t(self.nbytes), ctypes.c_int(D2H)), "hipMemcpy D2H")
        return out

    def c_ptr(self):
        return ctypes.c_void_p(self.ptr)

    def free(self):
        if getattr(self, "ptr", None):
            lib().hipFree(ctypes.c_void_p(self.ptr))
            self.ptr = None

    def __del__(self):  # best effort
        try:
            self.free()
        except Exception:
            pass


class Event:
    def __init__(self):
        self.ev = ctypes.c_void_p()
        check(lib().hipEventCreate(ctypes.byref(self.ev)), "hipEventCreate")

    def record(self, stream=None):
        check(lib().hipEventRecord(self.ev, ctypes.c_void_p(stream)), "hipEventRecord")

    def synchronize(self):
        check(lib().hipEventSynchronize(self.ev), "hipEventSynchronize")

    def elapsed_ms(self, later):
        ms = ctypes.c_float(0)
        check(lib().hipEventElapsedTime(ctypes.byref(ms), self.ev, later.ev), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            lib().hipEventDestroy(self.ev)
        except Exception:
            pass
