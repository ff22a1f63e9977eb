"""Minimal ctypes view of the HIP runtime: device buffers, a stream and events.

Plumbing for the benchmark and the device-pointer tests; the kernels are reached through
``liborangu_mi355x.so`` only.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

_hip = None

H2D, D2H = 1, 2


class HipError(RuntimeError):
    pass


def hip() -> C.CDLL:
    global _hip
    if _hip is None:
        L = C.CDLL("libamdhip64.so")
        L.hipGetErrorString.restype = C.c_char_p
        L.hipGetErrorString.argtypes = [C.c_int]
        L.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        L.hipFree.argtypes = [C.c_void_p]
        L.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        L.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        L.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        L.hipStreamDestroy.argtypes = [C.c_void_p]
        L.hipStreamSynchronize.argtypes = [C.c_void_p]
        L.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        L.hipEventDestroy.argtypes = [C.c_void_p]
        L.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        L.hipEventSynchronize.argtypes = [C.c_void_p]
        L.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        L.hipSetDevice.argtypes = [C.c_int]
        _hip = L
    return _hip


def check(rc: int, what: str):
    if rc != 0:
        raise HipError(f"{what}: {hip().hipGetErrorString(rc).decode()} ({rc})")


def set_device(i: int):
    check(hip().hipSetDevice(i), "hipSetDevice")


def device_synchronize():
    check(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")


def mem_get_info():
    """(free, total) bytes of the current device."""
    free, total = C.c_size_t(), C.c_size_t()
    check(hip().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value, total.value


class DeviceBuffer:
    def __init__(self, nbytes: int):
        self.nbytes = nbytes
        p = C.c_void_p()
        check(hip().hipMalloc(C.byref(p), max(nbytes, 1)), "hipMalloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        check(hip().hipMemcpy(b.ptr, a.ctypes.data, a.nbytes, H2D), "hipMemcpy H2D")
        return b

    def to_numpy(self, dtype, count: int) -> np.ndarray:
        out = np.empty(count, dtype)
        check(hip().hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, D2H), "hipMemcpy D2H")
        return out

    def fill(self, byte: int):
        """Sets every byte; complete on return (hipMemset runs on the null stream, which a library context's own
        stream does not wait for)."""
        check(hip().hipMemset(self.ptr, byte, self.nbytes), "hipMemset")
        device_synchronize()

    def free(self):
        if self.ptr:
            hip().hipFree(self.ptr)
            self.ptr = None


class Stream:
    def __init__(self):
        p = C.c_void_p()
        check(hip().hipStreamCreate(C.byref(p)), "hipStreamCreate")
        self.ptr = p.value

    def synchronize(self):
        check(hip().hipStreamSynchronize(self.ptr), "hipStreamSynchronize")

    def destroy(self):
        if self.ptr:
            hip().hipStreamDestroy(self.ptr)
            self.ptr = None


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(hip().hipEventCreate(C.byref(p)), "hipEventCreate")
        self.ptr = p.value

    def record(self, stream: Stream):
        check(hip().hipEventRecord(self.ptr, stream.ptr), "hipEventRecord")

    def synchronize(self):
        check(hip().hipEventSynchronize(self.ptr), "hipEventSynchronize")

    def elapsed_ms(self, end: "Event") -> float:
        ms = C.c_float()
        check(hip().hipEventElapsedTime(C.byref(ms), self.ptr, end.ptr), "hipEventElapsedTime")
        return float(ms.value)
