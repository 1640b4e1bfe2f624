"""Device memory for tests that hand DEVICE pointers to the C-ABI: a few HIP runtime calls
through ctypes, on the runtime that libarboretum.so itself is linked against."""
import ctypes

import numpy as np

_hip = None


def hip():
    global _hip
    if _hip is None:
        import arboretum_amd  # noqa: F401  (loads libarboretum.so and with it the HIP runtime)
        lib = ctypes.CDLL("libamdhip64.so", mode=ctypes.RTLD_GLOBAL)
        lib.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        lib.hipFree.argtypes = [ctypes.c_void_p]
        lib.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        lib.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
        _hip = lib
    return _hip


def _ok(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed with HIP error %d" % (what, rc))


def free_device_bytes():
    """Free device memory as hipMemGetInfo reports it."""
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    _ok(hip().hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)), "hipMemGetInfo")
    return free.value


def synchronize():
    _ok(hip().hipDeviceSynchronize(), "hipDeviceSynchronize")


class DeviceArray:
    """A device buffer with the shape and dtype of a numpy array."""

    def __init__(self, host=None, shape=None, dtype=None, fill_byte=0):
        if host is not None:
            host = np.ascontiguousarray(host)
            shape, dtype = host.shape, host.dtype
        self.shape, self.dtype = tuple(np.atleast_1d(shape)) if not isinstance(shape, tuple) else shape, np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        _ok(hip().hipMalloc(ctypes.byref(p), max(self.nbytes, 256)), "hipMalloc")
        self.ptr = p.value
        if host is not None:
            _ok(hip().hipMemcpy(self.ptr, host.ctypes.data, self.nbytes, 1), "hipMemcpy H2D")
        else:
            _ok(hip().hipMemset(self.ptr, fill_byte, max(self.nbytes, 1)), "hipMemset")

    def get(self):
        synchronize()
        out = np.empty(self.shape, self.dtype)
        _ok(hip().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, 2), "hipMemcpy D2H")
        return out

    def __del__(self):
        if getattr(self, "ptr", None):
            hip().hipFree(self.ptr)
            self.ptr = None


class PinnedArray:
    """Pinned host memory (hipHostMalloc) seen as a numpy array."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        lib = hip()
        lib.hipHostMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t, ctypes.c_uint]
        lib.hipHostFree.argtypes = [ctypes.c_void_p]
        p = ctypes.c_void_p()
        _ok(lib.hipHostMalloc(ctypes.byref(p), max(self.nbytes, 256), 0), "hipHostMalloc")
        self.ptr = p.value
        buf = (ctypes.c_ubyte * self.nbytes).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype).reshape(self.shape)

    def __del__(self):
        if getattr(self, "ptr", None):
            self.array = None
            hip().hipHostFree(self.ptr)
            self.ptr = None
