"""Minimal ctypes view of the HIP runtime: device memory, copies, streams and events.

Used by the Python-side callers of the C ABI (tests, bench) so that device
buffers can be handed to the sampler as plain pointers.
"""
import ctypes as C

import numpy as np

_lib = None

hipMemcpyHostToDevice = 1
hipMemcpyDeviceToHost = 2
hipMemcpyDeviceToDevice = 3


class HipError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL("libamdhip64.so")
        _lib.hipGetErrorString.restype = C.c_char_p
        _lib.hipGetErrorString.argtypes = [C.c_int]
        _lib.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _lib.hipFree.argtypes = [C.c_void_p]
        _lib.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _lib.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        _lib.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        _lib.hipStreamDestroy.argtypes = [C.c_void_p]
        _lib.hipStreamSynchronize.argtypes = [C.c_void_p]
        _lib.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        _lib.hipEventDestroy.argtypes = [C.c_void_p]
        _lib.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        _lib.hipEventSynchronize.argtypes = [C.c_void_p]
        _lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        _lib.hipGetDeviceCount.argtypes = [C.POINTER(C.c_int)]
        _lib.hipSetDevice.argtypes = [C.c_int]
    return _lib


def check(code, what="hip call"):
    if code != 0:
        raise HipError("%s failed: %s" % (what, lib().hipGetErrorString(code).decode()))


def device_count():
    n = C.c_int(0)
    try:
        if lib().hipGetDeviceCount(C.byref(n)) != 0:
            return 0
    except OSError:
        return 0
    return n.value


def set_device(i):
    check(lib().hipSetDevice(i), "hipSetDevice")


def synchronize():
    check(lib().hipDeviceSynchronize(), "hipDeviceSynchronize")


def mem_get_info():
    """(free, total) bytes of device memory on the current device."""
    free, total = C.c_size_t(0), C.c_size_t(0)
    check(lib().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value, total.value


class DeviceArray:
    """A typed device allocation; freed with the object."""

    def __init__(self, shape, dtype):
        self.shape = tuple(np.atleast_1d(shape).tolist()) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        check(lib().hipMalloc(C.byref(p), max(self.nbytes, 1)), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_host(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        d.upload(a)
        return d

    def upload(self, a):
        a = np.ascontiguousarray(a, self.dtype)
        assert a.nbytes == self.nbytes
        if self.nbytes:
            check(lib().hipMemcpy(self.ptr, a.ctypes.data, self.nbytes, hipMemcpyHostToDevice), "hipMemcpy H2D")

    def download(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            check(lib().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, hipMemcpyDeviceToHost), "hipMemcpy D2H")
        return out

    def zero(self):
        check(lib().hipMemset(self.ptr, 0, self.nbytes), "hipMemset")

    def free(self):
        if getattr(self, "ptr", None):
            lib().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self):
        p = C.c_void_p()
        check(lib().hipStreamCreate(C.byref(p)), "hipStreamCreate")
        self.ptr = p.value

    def synchronize(self):
        check(lib().hipStreamSynchronize(self.ptr), "hipStreamSynchronize")

    def __del__(self):
        try:
            if self.ptr:
                lib().hipStreamDestroy(self.ptr)
        except Exception:
            pass


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(lib().hipEventCreate(C.byref(p)), "hipEventCreate")
        self.ptr = p.value

    def record(self, stream=None):
        check(lib().hipEventRecord(self.ptr, stream.ptr if stream else None), "hipEventRecord")

    def synchronize(self):
        check(lib().hipEventSynchronize(self.ptr), "hipEventSynchronize")

    def elapsed_ms(self, end):
        ms = C.c_float(0)
        check(lib().hipEventElapsedTime(C.byref(ms), self.ptr, end.ptr), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().hipEventDestroy(self.ptr)
        except Exception:
            pass
