"""Device buffers for Python callers of the C ABI (tests, smoke check, benchmark).

A DeviceArray owns one allocation made through bidmat_malloc and knows its dtype and
element count; it converts from/to numpy through the library's copy entry points.
"""
import ctypes as C
import numpy as np

from . import hip_abi


class DeviceArray:
    def __init__(self, n, dtype):
        self.lib = hip_abi.load()
        self.dtype = np.dtype(dtype)
        self.n = int(n)
        self.nbytes = self.n * self.dtype.itemsize
        p = C.c_void_p()
        hip_abi.check(self.lib.bidmat_malloc(C.byref(p), self.nbytes), "bidmat_malloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.size, a.dtype)
        if a.size:
            hip_abi.check(d.lib.bidmat_memcpy_h2d(d.ptr, a.ctypes.data, a.nbytes), "h2d")
        return d

    @classmethod
    def zeros(cls, n, dtype=np.float32):
        d = cls(n, dtype)
        d.clear()
        return d

    def clear(self):
        if self.nbytes:
            hip_abi.check(self.lib.bidmat_memset(self.ptr, 0, self.nbytes), "memset")
        return self

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        assert a.size == self.n
        if a.size:
            hip_abi.check(self.lib.bidmat_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes), "h2d")
        return self

    def numpy(self, count=None):
        n = self.n if count is None else int(count)
        out = np.empty(n, dtype=self.dtype)
        if n:
            hip_abi.check(self.lib.bidmat_memcpy_d2h(out.ctypes.data, self.ptr, n * self.dtype.itemsize), "d2h")
        return out

    def free(self):
        if getattr(self, "ptr", None):
            self.lib.bidmat_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def device_available():
    """True when the library loads and reports at least one device."""
    try:
        lib = hip_abi.load()
    except (ImportError, OSError):
        return False
    n = C.c_int(0)
    return lib.bidmat_device_count(C.byref(n)) == 0 and n.value > 0
