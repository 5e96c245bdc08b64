"""Device buffers, streams and events over the library's own HIP runtime (no torch: loading
PyTorch's bundled HIP runtime next to the one this library links would put two runtimes in
one process)."""
import ctypes as C

import numpy as np

from . import _lib
from .plugin import _check


class DeviceArray:
    """A typed device buffer with numpy shape/dtype, filled from / read back to host arrays."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        _check(_lib.load().coeus_device_malloc(self.nbytes, C.byref(p)))
        self.ptr = p.value

    @classmethod
    def from_host(cls, a, dtype=None):
        a = np.ascontiguousarray(a, dtype=dtype)
        d = cls(a.shape, a.dtype)
        _check(_lib.load().coeus_memcpy_h2d(d.ptr, a.ctypes.data, d.nbytes))
        return d

    def to_host(self):
        out = np.empty(self.shape, dtype=self.dtype)
        _check(_lib.load().coeus_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def copy_from(self, other, stream=None):
        """Device-to-device copy of `other` (same byte size) into this array."""
        if other.nbytes != self.nbytes:
            raise ValueError("copy_from needs arrays of the same byte size")
        _check(_lib.load().coeus_device_copy(self.ptr, other.ptr, self.nbytes, stream))
        return self

    def zero_(self):
        _check(_lib.load().coeus_device_memset(self.ptr, 0, self.nbytes))
        return self

    def free(self):
        if getattr(self, "ptr", None):
            _lib.load().coeus_device_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def synchronize():
    _check(_lib.load().coeus_device_synchronize())


class Stream:
    def __init__(self):
        p = C.c_void_p()
        _check(_lib.load().coeus_stream_create(C.byref(p)))
        self.handle = p.value

    def synchronize(self):
        _check(_lib.load().coeus_stream_synchronize(self.handle))

    def __del__(self):
        try:
            if self.handle:
                _lib.load().coeus_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Event:
    def __init__(self):
        p = C.c_void_p()
        _check(_lib.load().coeus_event_create(C.byref(p)))
        self.handle = p.value

    def record(self, stream=None):
        _check(_lib.load().coeus_event_record(self.handle, stream.handle if stream else None))

    def synchronize(self):
        _check(_lib.load().coeus_event_synchronize(self.handle))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        _check(_lib.load().coeus_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                _lib.load().coeus_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass
