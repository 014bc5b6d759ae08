"""Minimal device-memory plumbing over the HIP runtime (ctypes): enough to hand device arrays to the C ABIs of this
package without any other GPU library in the process.  The runtime is the one libpuct_hip.so / libmctsnc_hip.so are
linked against."""
import ctypes
import sys

import numpy as np

_hip = None
H2D, D2H = 1, 2


def hip():
    global _hip
    if _hip is None:
        from . import puct
        puct._lib()                                   # pulls in the HIP runtime the libraries use
        _hip = ctypes.CDLL("libamdhip64.so.7")
        vp = ctypes.c_void_p
        _hip.hipMalloc.argtypes = [ctypes.POINTER(vp), ctypes.c_size_t]
        _hip.hipFree.argtypes = [vp]
        _hip.hipMemcpy.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int]
        _hip.hipMemset.argtypes = [vp, ctypes.c_int, ctypes.c_size_t]
        _hip.hipEventCreate.argtypes = [ctypes.POINTER(vp)]
        _hip.hipEventRecord.argtypes = [vp, vp]
        _hip.hipEventDestroy.argtypes = [vp]
        _hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), vp, vp]
        _hip.hipGetErrorString.restype = ctypes.c_char_p
        _hip.hipGetErrorString.argtypes = [ctypes.c_int]
    return _hip


def check(code, what):
    if code != 0:
        raise RuntimeError(f"{what} failed: {hip().hipGetErrorString(code).decode()} ({code})")


def synchronize():
    check(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")


class DeviceArray:
    """A C-contiguous array in device memory with a numpy dtype and shape."""

    def __init__(self, source=None, shape=None, dtype=None):
        if source is not None:
            source = np.ascontiguousarray(source)
            shape, dtype = source.shape, source.dtype
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self._ptr = ctypes.c_void_p()
        check(hip().hipMalloc(ctypes.byref(self._ptr), max(self.nbytes, 1)), "hipMalloc")
        if source is not None and self.nbytes:
            check(hip().hipMemcpy(self._ptr, source.ctypes.data, self.nbytes, H2D), "hipMemcpy")

    def data_ptr(self):
        return self._ptr.value or 0

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            check(hip().hipMemcpy(out.ctypes.data, self._ptr, self.nbytes, D2H), "hipMemcpy")
        return out

    def copy_from(self, source):
        source = np.ascontiguousarray(source, dtype=self.dtype)
        if source.shape != self.shape:
            raise ValueError("shape mismatch")
        if self.nbytes:
            check(hip().hipMemcpy(self._ptr, source.ctypes.data, self.nbytes, H2D), "hipMemcpy")

    def free(self):
        ptr, self._ptr = self._ptr, ctypes.c_void_p()
        if ptr:
            hip().hipFree(ptr)

    def __del__(self):
        if sys.is_finalizing():   # the process is going away and the HIP runtime with it: nothing to give back
            return
        try:
            self.free()
        except Exception:
            pass


class Event:
    """A HIP event on the default stream (timing of the launches made through the C ABIs with a NULL stream)."""

    def __init__(self):
        self._ev = ctypes.c_void_p()
        check(hip().hipEventCreate(ctypes.byref(self._ev)), "hipEventCreate")

    def record(self):
        check(hip().hipEventRecord(self._ev, ctypes.c_void_p(0)), "hipEventRecord")

    def elapsed_ms(self, later):
        """Milliseconds from this event to `later` (both must have completed)."""
        ms = ctypes.c_float()
        check(hip().hipEventElapsedTime(ctypes.byref(ms), self._ev, later._ev), "hipEventElapsedTime")
        return float(ms.value)

    def __del__(self):
        if sys.is_finalizing():
            return
        try:
            if self._ev:
                hip().hipEventDestroy(self._ev)
        except Exception:
            pass
