"""Minimal HIP runtime access for callers that hold device buffers themselves
(the `_dev` entry points, bench.py): hipMalloc / hipMemcpy / hipFree through
ctypes on the same libamdhip64 the kernel library is linked against.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import ffi

_rt = None
H2D, D2H, D2D = 1, 2, 3


def rt() -> C.CDLL:
    global _rt
    if _rt is None:
        ffi.load()  # pulls libamdhip64.so.7 into the process first
        _rt = C.CDLL("libamdhip64.so.7")
        _rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _rt.hipFree.argtypes = [C.c_void_p]
        _rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _rt.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        _rt.hipGetErrorString.restype = C.c_char_p
        _rt.hipGetErrorString.argtypes = [C.c_int]
        _rt.hipGetDeviceCount.argtypes = [C.POINTER(C.c_int)]
        _rt.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    return _rt


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {rt().hipGetErrorString(rc).decode()}")


def device_count() -> int:
    n = C.c_int(0)
    rc = rt().hipGetDeviceCount(C.byref(n))
    return n.value if rc == 0 else 0


def mem_free() -> int:
    """Free device memory in bytes (hipMemGetInfo) on the current device."""
    free, total = C.c_size_t(0), C.c_size_t(0)
    _check(rt().hipMemGetInfo(C.byref(free), C.byref(total)), "hipMemGetInfo")
    return free.value


def synchronize() -> None:
    _check(rt().hipDeviceSynchronize(), "hipDeviceSynchronize")


class DeviceArray:
    """A typed device allocation; freed when the object is collected."""

    def __init__(self, shape, dtype=np.float32, zero: bool = False):
        self.shape = tuple(np.atleast_1d(shape).tolist()) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        _check(rt().hipMalloc(C.byref(p), max(self.nbytes, 4)), "hipMalloc")
        self.ptr = p.value
        if zero:
            _check(rt().hipMemset(self.ptr, 0, self.nbytes), "hipMemset")

    @classmethod
    def from_host(cls, a: np.ndarray) -> "DeviceArray":
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        _check(rt().hipMemcpy(d.ptr, a.ctypes.data, a.nbytes, H2D), "hipMemcpy H2D")
        return d

    def to_host(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        _check(rt().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, D2H), "hipMemcpy D2H")
        return out

    def offset(self, elems: int) -> int:
        return self.ptr + elems * self.dtype.itemsize

    def free(self) -> None:
        if getattr(self, "ptr", None):
            rt().hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
