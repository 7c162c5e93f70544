"""DeviceTensor: the Python mirror of the reference's RAII float32 device buffer
(include/blackforge/backend/cuda/device_tensor.hpp:19-75), backed by the library's memory pool."""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import numpy as np

from . import capi


class Stream:
    """A HIP stream created through the C ABI (default priority)."""

    def __init__(self):
        h = ctypes.c_void_p()
        capi.call("bf_hip_stream_create", ctypes.byref(h))
        self.handle = h

    def synchronize(self):
        capi.call("bf_hip_stream_synchronize", self.handle)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                capi.call("bf_hip_stream_destroy", self.handle)
                self.handle = None
        except Exception:
            pass


class Event:
    def __init__(self):
        h = ctypes.c_void_p()
        capi.call("bf_hip_event_create", ctypes.byref(h))
        self.handle = h

    def record(self, stream: Optional[Stream] = None):
        capi.call("bf_hip_event_record", self.handle, stream.handle if stream else None)

    def synchronize(self):
        capi.call("bf_hip_event_synchronize", self.handle)

    def elapsed_ms(self, end: "Event") -> float:
        ms = ctypes.c_float()
        capi.call("bf_hip_event_elapsed_ms", self.handle, end.handle, ctypes.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                capi.call("bf_hip_event_destroy", self.handle)
                self.handle = None
        except Exception:
            pass


def _count(shape: Sequence[int]) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class DeviceTensor:
    """Owns a float32 buffer from the per-device pool; returned to the pool on destruction."""

    itemsize = 4

    def __init__(self, shape: Sequence[int], itemsize: int = 4):
        self.shape = tuple(int(d) for d in shape)
        self.itemsize = itemsize
        self._bytes = _count(self.shape) * itemsize
        ptr = ctypes.c_void_p()
        capi.call("bf_hip_pool_acquire", self._bytes, ctypes.byref(ptr))
        self.ptr = ptr

    # -- reference API ----------------------------------------------------------------------
    @staticmethod
    def fromHost(host) -> "DeviceTensor":
        host = np.ascontiguousarray(host, dtype=np.float32)
        t = DeviceTensor(host.shape)
        capi.call("bf_hip_memcpy_h2d", t.ptr, host.ctypes.data_as(ctypes.c_void_p), t._bytes)
        return t

    @staticmethod
    def zeros(shape: Sequence[int]) -> "DeviceTensor":
        t = DeviceTensor(shape)
        capi.call("bf_hip_fill_zero", t.ptr, t._bytes, None)
        return t

    def toHost(self) -> np.ndarray:
        dtype = np.float32 if self.itemsize == 4 else np.uint16
        out = np.empty(self.shape, dtype)
        capi.call("bf_hip_memcpy_d2h", out.ctypes.data_as(ctypes.c_void_p), self.ptr, self._bytes)
        return out

    def clone(self) -> "DeviceTensor":
        t = DeviceTensor(self.shape, self.itemsize)
        capi.call("bf_hip_memcpy_d2d", t.ptr, self.ptr, self._bytes, None)
        return t

    def reshaped(self, shape: Sequence[int]) -> "DeviceTensor":
        """Transfers the buffer to a tensor of another shape; this tensor becomes empty."""
        shape = tuple(int(d) for d in shape)
        if _count(shape) != self.elementCount():
            raise ValueError(f"reshaped: {self.shape} -> {shape} changes the element count")
        t = DeviceTensor.__new__(DeviceTensor)
        t.shape, t.itemsize, t._bytes, t.ptr = shape, self.itemsize, self._bytes, self.ptr
        self.ptr, self._bytes, self.shape = ctypes.c_void_p(), 0, (0,)
        return t

    def rank(self) -> int:
        return len(self.shape)

    def dim(self, axis: int) -> int:
        return self.shape[axis]

    def elementCount(self) -> int:
        return _count(self.shape)

    def data(self):
        return self.ptr

    def __del__(self):
        try:
            if getattr(self, "ptr", None) and self._bytes:
                capi.call("bf_hip_pool_release", self.ptr, self._bytes)
                self.ptr = None
        except Exception:
            pass
