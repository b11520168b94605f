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


def free_bytes() -> int:
    """free device memory as hipMemGetInfo reports it"""
    h = _rt()
    h.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert h.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return int(free.value)


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

    def set(self, a: np.ndarray):
        src = np.ascontiguousarray(a, dtype=self.dtype)
        assert src.nbytes == self.nbytes
        assert _rt().hipMemcpy(self.ptr, src.ctypes.data, src.nbytes, 1) == 0


class Stream:
    """a HIP stream of default priority, with capture into a graph"""

    def __init__(self):
        h = _rt()
        self.ptr = ctypes.c_void_p()
        h.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        assert h.hipStreamCreate(ctypes.byref(self.ptr)) == 0
        h.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
        h.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
        h.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
        h.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_size_t]
        h.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        h.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
        h.hipGraphDestroy.argtypes = [ctypes.c_void_p]
        h.hipStreamDestroy.argtypes = [ctypes.c_void_p]

    def sync(self):
        assert _rt().hipStreamSynchronize(self.ptr) == 0

    def capture(self, fn):
        """runs fn() with the stream capturing; returns a callable that replays the captured graph"""
        h = _rt()
        assert h.hipStreamBeginCapture(self.ptr, 0) == 0  # hipStreamCaptureModeGlobal
        try:
            fn()
        finally:
            graph = ctypes.c_void_p()
            rc = h.hipStreamEndCapture(self.ptr, ctypes.byref(graph))
        assert rc == 0 and graph.value
        exe = ctypes.c_void_p()
        assert h.hipGraphInstantiate(ctypes.byref(exe), graph, None, None, 0) == 0
        self._graphs = getattr(self, "_graphs", []) + [(exe, graph)]
        return lambda: h.hipGraphLaunch(exe, self.ptr)

    def destroy(self):
        h = _rt()
        for exe, graph in getattr(self, "_graphs", []):
            h.hipGraphExecDestroy(exe)
            h.hipGraphDestroy(graph)
        h.hipStreamDestroy(self.ptr)
