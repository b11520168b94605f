"""Device buffers for tests that pass device pointers through the C ABI: a few HIP runtime calls via
ctypes on the runtime the library itself is linked against (so both see one HIP context)."""
import ctypes
import os

import numpy as np

_hip = None


def _rt():
    global _hip
    if _hip is None:
        _hip = ctypes.CDLL(os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib", "libamdhip64.so"))
        _hip.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        _hip.hipFree.argtypes = [ctypes.c_void_p]
        _hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        _hip.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
    return _hip


class DeviceArray:
    """a device copy of a numpy array (or zeros of its shape); .ptr is the device address"""

    def __init__(self, like: np.ndarray, zero: bool = False):
        self.shape, self.dtype, self.nbytes = like.shape, like.dtype, max(int(like.nbytes), 1)
        p = ctypes.c_void_p()
        assert _rt().hipMalloc(ctypes.byref(p), self.nbytes) == 0
        self.ptr = p.value
        if zero:
            assert _rt().hipMemset(self.ptr, 0, self.nbytes) == 0
        elif like.nbytes:
            src = np.ascontiguousarray(like)
            assert _rt().hipMemcpy(self.ptr, src.ctypes.data, src.nbytes, 1) == 0  # hipMemcpyHostToDevice

    def numpy(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        if out.nbytes:
            assert _rt().hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, 2) == 0  # hipMemcpyDeviceToHost
        return out

    def free(self):
        if self.ptr:
            _rt().hipFree(self.ptr)
            self.ptr = None
