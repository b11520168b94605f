"""ctypes binding of libmi_qmm.so (the C ABI declared in include/mi_qmm.h).

Fails loudly when the library has not been built: nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes
import weakref
import os
import subprocess

import numpy as np
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI_QMM_LIB points at an alternative build of the library (e.g. an experimental variant)
LIB_PATH = os.environ.get("MI_QMM_LIB") or os.path.join(_HERE, "libmi_qmm.so")

F32, F16, Q4_0, Q5_0, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K, BF16, MXFP4 = 0, 1, 2, 6, 8, 12, 13, 14, 15, 30, 39
PLAIN_TYPES = (F32, F16, BF16)  # unquantized weight types: multiplied in their own type
SINGLE_ONLY_TYPES = PLAIN_TYPES + (Q5_K,)  # weight types that only mulmat / mulmat_multi multiply (no fused or expert forms)
HOST, DEVICE = 0, 1
PATH_AUTO, PATH_GEMV, PATH_GEMM, PATH_QUERY = 0, 1, 2, 3
# what PATH_QUERY returns (MI_QMM_ROUTE_*): the kernel a product takes
ROUTES = {1: "gemv_f32", 2: "deep_f32", 3: "gemm_blk32", 4: "gemm_f16", 5: "gemm_q6k", 6: "gemm_int8", 7: "skinny32",
          8: "skinny_deep", 9: "skinny_direct", 10: "skinny_rows_q4k", 11: "skinny_staged", 12: "skinny_rows_q6k", 13: "gemv",
          14: "plain_gemv", 15: "plain_gemm", 16: "plain_naive", 17: "plain_skinny"}
PRODUCE_NONE, PRODUCE_RMSNORM, PRODUCE_SWIGLU = 0, 1, 2
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_NOMEM, ERR_NODEVICE = 0, -1, -2, -3, -4, -5

NOALLOC_SCRATCH_BYTES = 16 << 20  # MI_QMM_NOALLOC_SCRATCH_BYTES

EXPORTS = [
    "mi_qmm_block_size", "mi_qmm_type_size", "mi_qmm_row_size", "mi_qmm_vec_dot_type",
    "mi_qmm_init", "mi_qmm_destroy", "mi_qmm_set_stream", "mi_qmm_sync", "mi_qmm_host_alloc", "mi_qmm_host_free",
    "mi_qmm_weight_upload", "mi_qmm_weight_free", "mi_qmm_weight_info",
    "mi_qmm_quantize_act", "mi_qmm_quantize_weights", "mi_qmm_mulmat", "mi_qmm_mulmat_path", "mi_qmm_mulmat_noalloc", "mi_qmm_scratch_freeze",
    "mi_qmm_mulmat_multi", "mi_qmm_mulmat_id", "mi_qmm_mulmat_id_multi",
    "mi_qmm_mulmat_produced", "mi_qmm_mulmat_id_produced", "mi_qmm_mulmat_swiglu", "mi_qmm_mulmat_id_swiglu", "mi_qmm_rms_norm", "mi_qmm_swiglu",
    "mi_qmm_act_create", "mi_qmm_act_free", "mi_qmm_act_quantize", "mi_qmm_mulmat_q8", "mi_qmm_mulmat_q8_multi",
    "mi_qmm_gguf_open", "mi_qmm_gguf_close", "mi_qmm_gguf_info", "mi_qmm_gguf_tensor", "mi_qmm_gguf_find_tensor",
    "mi_qmm_gguf_tensor_data", "mi_qmm_gguf_find_kv", "mi_qmm_gguf_kv", "mi_qmm_gguf_kv_int", "mi_qmm_gguf_kv_uint",
    "mi_qmm_gguf_kv_float", "mi_qmm_gguf_kv_bool", "mi_qmm_gguf_kv_string", "mi_qmm_gguf_upload",
    "mi_qmm_last_error", "mi_qmm_version", "mi_qmm_device_info",
]


class QmmError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"mi_qmm error {code}: {msg}")
        self.code = code


def build(verbose: bool = False) -> str:
    """Compile the HIP library in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8", "-B"]
    subprocess.run(cmd, check=True, stdout=None if verbose else subprocess.DEVNULL,
                   stderr=None if verbose else subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(there is no CPU fallback)")
    L = ctypes.CDLL(LIB_PATH)
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    L.mi_qmm_block_size.restype = i64; L.mi_qmm_block_size.argtypes = [ci]
    L.mi_qmm_type_size.restype = i64; L.mi_qmm_type_size.argtypes = [ci]
    L.mi_qmm_row_size.restype = i64; L.mi_qmm_row_size.argtypes = [ci, i64]
    L.mi_qmm_vec_dot_type.restype = ci; L.mi_qmm_vec_dot_type.argtypes = [ci]
    L.mi_qmm_init.restype = ci; L.mi_qmm_init.argtypes = [ci, ctypes.POINTER(vp)]
    L.mi_qmm_destroy.restype = None; L.mi_qmm_destroy.argtypes = [vp]
    L.mi_qmm_set_stream.restype = ci; L.mi_qmm_set_stream.argtypes = [vp, vp]
    L.mi_qmm_sync.restype = ci; L.mi_qmm_sync.argtypes = [vp]
    L.mi_qmm_weight_upload.restype = ci
    L.mi_qmm_weight_upload.argtypes = [vp, ci, vp, i64, i64, ci, ctypes.POINTER(vp)]
    L.mi_qmm_weight_free.restype = None; L.mi_qmm_weight_free.argtypes = [vp]
    L.mi_qmm_weight_info.restype = ci
    L.mi_qmm_weight_info.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(i64), ctypes.POINTER(i64),
                                     ctypes.POINTER(i64)]
    L.mi_qmm_quantize_act.restype = ci; L.mi_qmm_quantize_act.argtypes = [vp, ci, vp, i64, i64, vp, ci]
    L.mi_qmm_quantize_weights.restype = ci; L.mi_qmm_quantize_weights.argtypes = [vp, ci, vp, i64, i64, vp, ci]
    L.mi_qmm_mulmat.restype = ci; L.mi_qmm_mulmat.argtypes = [vp, vp, vp, i64, vp, ci]
    L.mi_qmm_mulmat_path.restype = ci; L.mi_qmm_mulmat_path.argtypes = [vp, vp, vp, i64, vp, ci, ci]
    L.mi_qmm_mulmat_noalloc.restype = ci; L.mi_qmm_mulmat_noalloc.argtypes = [vp, vp, vp, i64, vp]
    L.mi_qmm_scratch_freeze.restype = ci; L.mi_qmm_scratch_freeze.argtypes = [vp, ci]
    L.mi_qmm_act_create.restype = ci; L.mi_qmm_act_create.argtypes = [vp, ci, i64, i64, ctypes.POINTER(vp)]
    L.mi_qmm_act_free.restype = None; L.mi_qmm_act_free.argtypes = [vp]
    L.mi_qmm_act_quantize.restype = ci; L.mi_qmm_act_quantize.argtypes = [vp, vp, vp, i64, ci]
    L.mi_qmm_mulmat_q8.restype = ci; L.mi_qmm_mulmat_q8.argtypes = [vp, vp, vp, vp, ci, ci]
    L.mi_qmm_mulmat_q8_multi.restype = ci
    L.mi_qmm_mulmat_q8_multi.argtypes = [vp, ctypes.POINTER(vp), ci, vp, ctypes.POINTER(vp), ci]
    L.mi_qmm_mulmat_multi.restype = ci
    L.mi_qmm_mulmat_multi.argtypes = [vp, ctypes.POINTER(vp), ci, vp, i64, ctypes.POINTER(vp), ci]
    L.mi_qmm_mulmat_produced.restype = ci
    L.mi_qmm_mulmat_produced.argtypes = [vp, ctypes.POINTER(vp), ci, ci, vp, ctypes.c_float, vp, i64, ctypes.POINTER(vp), ci]
    L.mi_qmm_mulmat_id_produced.restype = ci
    L.mi_qmm_mulmat_id_produced.argtypes = [vp, vp, ci, ci, vp, ctypes.c_float, vp, ci, vp, ci, i64, vp, ci]
    L.mi_qmm_mulmat_id_swiglu.restype = ci
    L.mi_qmm_mulmat_id_swiglu.argtypes = [vp, vp, vp, ci, vp, ci, vp, ci, i64, vp, ci]
    L.mi_qmm_mulmat_swiglu.restype = ci
    L.mi_qmm_mulmat_swiglu.argtypes = [vp, vp, vp, ci, vp, ctypes.c_float, vp, i64, vp, ci]
    L.mi_qmm_rms_norm.restype = ci; L.mi_qmm_rms_norm.argtypes = [vp, vp, vp, ctypes.c_float, i64, i64, vp, ci]
    L.mi_qmm_swiglu.restype = ci; L.mi_qmm_swiglu.argtypes = [vp, vp, vp, i64, i64, vp, ci]
    L.mi_qmm_host_alloc.restype = vp; L.mi_qmm_host_alloc.argtypes = [vp, ctypes.c_size_t]
    L.mi_qmm_host_free.restype = None; L.mi_qmm_host_free.argtypes = [vp, vp]
    L.mi_qmm_mulmat_id_multi.restype = ci
    L.mi_qmm_mulmat_id_multi.argtypes = [vp, ctypes.POINTER(vp), ci, ci, vp, ci, vp, ci, i64, ctypes.POINTER(vp), ci]
    L.mi_qmm_mulmat_id.restype = ci
    L.mi_qmm_mulmat_id.argtypes = [vp, vp, ci, vp, ci, vp, ci, i64, vp, ci]
    P = ctypes.POINTER
    L.mi_qmm_gguf_open.restype = ci; L.mi_qmm_gguf_open.argtypes = [ctypes.c_char_p, P(vp)]
    L.mi_qmm_gguf_close.restype = None; L.mi_qmm_gguf_close.argtypes = [vp]
    L.mi_qmm_gguf_info.restype = ci; L.mi_qmm_gguf_info.argtypes = [vp, P(ci), P(i64), P(i64), P(i64), P(i64)]
    L.mi_qmm_gguf_tensor.restype = ci
    L.mi_qmm_gguf_tensor.argtypes = [vp, i64, P(ctypes.c_char_p), P(ci), P(ci), P(i64), P(i64), P(i64)]
    L.mi_qmm_gguf_find_tensor.restype = i64; L.mi_qmm_gguf_find_tensor.argtypes = [vp, ctypes.c_char_p]
    L.mi_qmm_gguf_tensor_data.restype = vp; L.mi_qmm_gguf_tensor_data.argtypes = [vp, i64]
    L.mi_qmm_gguf_find_kv.restype = i64; L.mi_qmm_gguf_find_kv.argtypes = [vp, ctypes.c_char_p]
    L.mi_qmm_gguf_kv.restype = ci; L.mi_qmm_gguf_kv.argtypes = [vp, i64, P(ctypes.c_char_p), P(ci), P(ci), P(i64)]
    L.mi_qmm_gguf_kv_int.restype = ci; L.mi_qmm_gguf_kv_int.argtypes = [vp, i64, i64, P(i64)]
    L.mi_qmm_gguf_kv_uint.restype = ci; L.mi_qmm_gguf_kv_uint.argtypes = [vp, i64, i64, P(ctypes.c_uint64)]
    L.mi_qmm_gguf_kv_float.restype = ci; L.mi_qmm_gguf_kv_float.argtypes = [vp, i64, i64, P(ctypes.c_double)]
    L.mi_qmm_gguf_kv_bool.restype = ci; L.mi_qmm_gguf_kv_bool.argtypes = [vp, i64, i64, P(ci)]
    L.mi_qmm_gguf_kv_string.restype = ci; L.mi_qmm_gguf_kv_string.argtypes = [vp, i64, i64, P(vp), P(i64)]
    L.mi_qmm_gguf_upload.restype = ci; L.mi_qmm_gguf_upload.argtypes = [vp, vp, i64, P(vp)]
    L.mi_qmm_last_error.restype = ctypes.c_char_p; L.mi_qmm_last_error.argtypes = []
    L.mi_qmm_version.restype = ctypes.c_char_p; L.mi_qmm_version.argtypes = []
    L.mi_qmm_device_info.restype = ci
    L.mi_qmm_device_info.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.c_char_p, ci]
    _lib = L
    return L


def last_error() -> str:
    return lib().mi_qmm_last_error().decode()


def _check(rc: int):
    if rc != 0:
        raise QmmError(rc, last_error())


def block_size(t: int) -> int:
    return int(lib().mi_qmm_block_size(t))


def type_size(t: int) -> int:
    return int(lib().mi_qmm_type_size(t))


def row_size(t: int, k: int) -> int:
    return int(lib().mi_qmm_row_size(t, k))


def vec_dot_type(t: int) -> int:
    return int(lib().mi_qmm_vec_dot_type(t))


def _ptr(a) -> ctypes.c_void_p:
    if a is None:
        return ctypes.c_void_p(None)
    if isinstance(a, np.ndarray):
        return ctypes.c_void_p(a.ctypes.data)
    return ctypes.c_void_p(int(a))  # raw device / host address


class Weight:
    """A weight tensor resident in HBM (mi_qmm_weight)."""

    def __init__(self, handle, ggml_type: int, k: int, m: int):
        self._h = handle
        self.type, self.k, self.m = ggml_type, k, m

    @property
    def device_bytes(self) -> int:
        nb = ctypes.c_int64()
        _check(lib().mi_qmm_weight_info(self._h, None, None, None, ctypes.byref(nb)))
        return nb.value

    @property
    def gguf_bytes(self) -> int:
        return row_size(self.type, self.k) * self.m

    def free(self):
        if self._h:
            lib().mi_qmm_weight_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Act:
    """Quantized activations resident on the device (mi_qmm_act), reusable across calls."""

    def __init__(self, handle, q8_type: int, k: int, n_max: int):
        self._h = handle
        self.type, self.k, self.n_max, self.n = q8_type, k, n_max, 0

    def free(self):
        if self._h:
            lib().mi_qmm_act_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    """One device + stream + scratch (mi_qmm_ctx)."""

    def __init__(self, device: int = 0):
        h = ctypes.c_void_p()
        _check(lib().mi_qmm_init(device, ctypes.byref(h)))
        self._h = h

    def close(self):
        if self._h:
            lib().mi_qmm_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def device_info(self):
        cus, mhz = ctypes.c_int(), ctypes.c_int()
        name = ctypes.create_string_buffer(128)
        _check(lib().mi_qmm_device_info(self._h, ctypes.byref(cus), ctypes.byref(mhz), name, 128))
        return {"compute_units": cus.value, "clock_mhz": mhz.value, "name": name.value.decode()}

    def set_stream(self, stream_ptr: int | None):
        _check(lib().mi_qmm_set_stream(self._h, ctypes.c_void_p(stream_ptr or None)))

    def sync(self):
        _check(lib().mi_qmm_sync(self._h))

    def host_array(self, shape, dtype=np.float32) -> np.ndarray:
        """a numpy array over page-locked host memory (freed when the array and its views are gone)"""
        n = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        p = lib().mi_qmm_host_alloc(self._h, n)
        if not p:
            raise QmmError(ERR_NOMEM, last_error())
        buf = (ctypes.c_uint8 * max(n, 1)).from_address(p)
        arr = np.frombuffer(buf, dtype=dtype, count=n // np.dtype(dtype).itemsize).reshape(shape)
        h = self._h
        weakref.finalize(buf, lambda: lib().mi_qmm_host_free(h, p))
        return arr

    def upload(self, ggml_type: int, gguf_bytes, k: int, m: int, location: int = HOST) -> Weight:
        if isinstance(gguf_bytes, np.ndarray):
            gguf_bytes = np.ascontiguousarray(gguf_bytes, dtype=np.uint8)
            rs = row_size(ggml_type, k)
            if rs >= 0 and gguf_bytes.size != rs * m:
                raise ValueError(f"weight bytes {gguf_bytes.size} != m*row_size = {rs * m}")
        h = ctypes.c_void_p()
        _check(lib().mi_qmm_weight_upload(self._h, ggml_type, _ptr(gguf_bytes), k, m, location, ctypes.byref(h)))
        return Weight(h, ggml_type, k, m)

    def quantize_weights(self, t: int, x: np.ndarray) -> np.ndarray:
        """f32 [m, k] -> uint8 [m, row_size(t, k)]: GGUF blocks of a weight type, encoded on the GPU"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        m, k = x.shape
        rb = row_size(t, k)
        out = np.empty((m, max(rb, 0)), dtype=np.uint8)
        _check(lib().mi_qmm_quantize_weights(self._h, t, _ptr(x), k, m, _ptr(out), HOST))
        return out

    def quantize_weights_device(self, t: int, x_ptr: int, k: int, m: int, out_ptr: int):
        _check(lib().mi_qmm_quantize_weights(self._h, t, ctypes.c_void_p(x_ptr), k, m, ctypes.c_void_p(out_ptr), DEVICE))

    def quantize_act(self, q8_type: int, x: np.ndarray) -> np.ndarray:
        """x f32 [n, k] -> uint8 [n, row_size] GGUF-layout Q8_0 / Q8_K blocks computed on the GPU."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        rs = row_size(q8_type, k)
        out = np.zeros((n, max(rs, 0)), dtype=np.uint8)
        _check(lib().mi_qmm_quantize_act(self._h, q8_type, _ptr(x), k, n, _ptr(out), HOST))
        return out

    def mulmat(self, w: Weight, x: np.ndarray, path: int = PATH_AUTO) -> np.ndarray:
        """x f32 [n, k] -> y f32 [n, m]; host arrays in and out."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        if k != w.k:
            raise ValueError(f"x has k={k}, weight has k={w.k}")
        y = np.empty((n, w.m), dtype=np.float32)
        _check(lib().mi_qmm_mulmat_path(self._h, w._h, _ptr(x), n, _ptr(y), HOST, path))
        return y

    def route(self, w: Weight, n: int) -> str:
        """name of the kernel mulmat takes for n f32 activation rows against w (nothing is launched)"""
        rc = lib().mi_qmm_mulmat_path(self._h, w._h, None, n, None, DEVICE, PATH_QUERY)
        if rc <= 0:
            raise QmmError(rc, last_error())
        return ROUTES[rc]

    def route_q8(self, w: Weight, act: "Act") -> str:
        """name of the kernel mulmat_q8 takes for these quantized activations against w (nothing is launched)"""
        rc = lib().mi_qmm_mulmat_q8(self._h, w._h, act._h, None, DEVICE, PATH_QUERY)
        if rc <= 0:
            raise QmmError(rc, last_error())
        return ROUTES[rc]

    def mulmat_device(self, w: Weight, x_ptr: int, n: int, y_ptr: int, path: int = PATH_AUTO):
        """device pointers in and out; queued on the ctx stream, returns without waiting."""
        _check(lib().mi_qmm_mulmat_path(self._h, w._h, ctypes.c_void_p(x_ptr), n, ctypes.c_void_p(y_ptr),
                                        DEVICE, path))

    def mulmat_noalloc_device(self, w: Weight, x_ptr: int, n: int, y_ptr: int):
        """mulmat_device through the entry point that never allocates (static device scratch of
        NOALLOC_SCRATCH_BYTES; larger calls raise)."""
        _check(lib().mi_qmm_mulmat_noalloc(self._h, w._h, ctypes.c_void_p(x_ptr), n, ctypes.c_void_p(y_ptr)))

    def scratch_freeze(self, frozen: bool = True):
        """while frozen, a call that would have to grow the ctx's scratch raises instead of reallocating
        (captured HIP graphs keep the old addresses)."""
        _check(lib().mi_qmm_scratch_freeze(self._h, 1 if frozen else 0))

    # ---- two-phase form -------------------------------------------------------------------------
    def act_create(self, q8_type: int, k: int, n_max: int) -> Act:
        h = ctypes.c_void_p()
        _check(lib().mi_qmm_act_create(self._h, q8_type, k, n_max, ctypes.byref(h)))
        return Act(h, q8_type, k, n_max)

    def act_quantize(self, act: Act, x, n: int | None = None, location: int = HOST):
        """x: numpy f32 [n, k] (HOST) or a device address with n given (DEVICE)."""
        if isinstance(x, np.ndarray):
            x = np.ascontiguousarray(x, dtype=np.float32)
            if x.ndim == 1:
                x = x[None, :]
            if x.shape[1] != act.k:
                raise ValueError(f"x has k={x.shape[1]}, act has k={act.k}")
            n = x.shape[0]
        _check(lib().mi_qmm_act_quantize(self._h, act._h, _ptr(x), n, location))
        act.n = n

    def mulmat_q8(self, w: Weight, act: Act, path: int = PATH_AUTO) -> np.ndarray:
        y = np.empty((act.n, w.m), dtype=np.float32)
        _check(lib().mi_qmm_mulmat_q8(self._h, w._h, act._h, _ptr(y), HOST, path))
        return y

    def mulmat_q8_device(self, w: Weight, act: Act, y_ptr: int, path: int = PATH_AUTO):
        _check(lib().mi_qmm_mulmat_q8(self._h, w._h, act._h, ctypes.c_void_p(y_ptr), DEVICE, path))

    def mulmat_multi(self, ws, x: np.ndarray):
        """several weights of one type and k against the same f32 activations; host arrays out"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        if any(w.k != k for w in ws):
            raise ValueError(f"x has k={k}, weights have k={[w.k for w in ws]}")
        ys = [np.empty((n, w.m), dtype=np.float32) for w in ws]
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[y.ctypes.data_as(ctypes.c_void_p) for y in ys])
        _check(lib().mi_qmm_mulmat_multi(self._h, wh, len(ws), x.ctypes.data_as(ctypes.c_void_p), n, yp, HOST))
        return ys

    def mulmat_multi_device(self, ws, x_ptr: int, n: int, y_ptrs):
        """device pointers; one launch (quantization included) for up to 4 weights when n <= 8"""
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[ctypes.c_void_p(int(p)) for p in y_ptrs])
        _check(lib().mi_qmm_mulmat_multi(self._h, wh, len(ws), ctypes.c_void_p(int(x_ptr)), n, yp, DEVICE))

    def mulmat_produced(self, ws, producer: int, aux, x: np.ndarray, eps: float = 0.0):
        """ws[i] . Q8(producer(x)): PRODUCE_RMSNORM with aux = norm weight [k] or None, PRODUCE_SWIGLU with
        aux = up [n, k]; host arrays out"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        if any(w.k != k for w in ws):
            raise ValueError(f"x has k={k}, weights have k={[w.k for w in ws]}")
        if aux is not None:
            aux = np.ascontiguousarray(aux, dtype=np.float32)
            want = (n, k) if producer == PRODUCE_SWIGLU else (k,)
            if producer == PRODUCE_SWIGLU and aux.ndim == 1:
                aux = aux[None, :]
            if aux.shape != want:
                raise ValueError(f"aux has shape {aux.shape}, the producer wants {want}")
        ys = [np.empty((n, w.m), dtype=np.float32) for w in ws]
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[y.ctypes.data_as(ctypes.c_void_p) for y in ys])
        _check(lib().mi_qmm_mulmat_produced(self._h, wh, len(ws), producer, _ptr(aux) if aux is not None else None,
                                            eps, x.ctypes.data_as(ctypes.c_void_p), n, yp, HOST))
        return ys

    def mulmat_produced_device(self, ws, producer: int, aux_ptr, x_ptr: int, n: int, y_ptrs, eps: float = 0.0):
        """device pointers; one launch for one activation row and up to 4 weights of one type"""
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[ctypes.c_void_p(int(p)) for p in y_ptrs])
        _check(lib().mi_qmm_mulmat_produced(self._h, wh, len(ws), producer,
                                            ctypes.c_void_p(int(aux_ptr)) if aux_ptr else None, eps,
                                            ctypes.c_void_p(int(x_ptr)), n, yp, DEVICE))

    def mulmat_swiglu(self, w_gate: Weight, w_up: Weight, x: np.ndarray, producer: int = PRODUCE_NONE, aux=None,
                      eps: float = 0.0) -> np.ndarray:
        """silu(w_gate . Q8(x')) * (w_up . Q8(x')) with x' = x or RMSNorm(x) (aux = norm weight or None)"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        if w_gate.k != k or w_up.k != k:
            raise ValueError(f"x has k={k}, weights have k={w_gate.k}, {w_up.k}")
        if aux is not None:
            aux = np.ascontiguousarray(aux, dtype=np.float32)
            if aux.shape != (k,):
                raise ValueError(f"aux has shape {aux.shape}, x has k={k}")
        h = np.empty((n, w_gate.m), dtype=np.float32)
        _check(lib().mi_qmm_mulmat_swiglu(self._h, w_gate._h, w_up._h, producer, _ptr(aux) if aux is not None else None,
                                          eps, _ptr(x), n, _ptr(h), HOST))
        return h

    def mulmat_swiglu_device(self, w_gate: Weight, w_up: Weight, x_ptr: int, n: int, h_ptr: int,
                             producer: int = PRODUCE_NONE, aux_ptr=None, eps: float = 0.0):
        _check(lib().mi_qmm_mulmat_swiglu(self._h, w_gate._h, w_up._h, producer,
                                          ctypes.c_void_p(int(aux_ptr)) if aux_ptr else None, eps,
                                          ctypes.c_void_p(int(x_ptr)), n, ctypes.c_void_p(int(h_ptr)), DEVICE))

    def rms_norm(self, x: np.ndarray, g, eps: float) -> np.ndarray:
        """(x / sqrt(mean(x^2) + eps)) * g per row; g f32 [k] or None"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None, :]
        n, k = x.shape
        if g is not None:
            g = np.ascontiguousarray(g, dtype=np.float32)
            if g.shape != (k,):
                raise ValueError(f"g has shape {g.shape}, x has k={k}")
        y = np.empty_like(x)
        _check(lib().mi_qmm_rms_norm(self._h, _ptr(x), _ptr(g) if g is not None else None, eps, k, n, _ptr(y), HOST))
        return y

    def swiglu(self, gate: np.ndarray, up: Optional[np.ndarray]) -> np.ndarray:
        """silu(gate) * up, f32 [n, k]; up None: silu(gate)"""
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        if up is not None:
            up = np.ascontiguousarray(up, dtype=np.float32)
            if gate.shape != up.shape:
                raise ValueError(f"gate {gate.shape} and up {up.shape} differ")
        g2 = gate.reshape(-1, gate.shape[-1])
        y = np.empty_like(g2)
        _check(lib().mi_qmm_swiglu(self._h, _ptr(g2), _ptr(up) if up is not None else None, g2.shape[1], g2.shape[0], _ptr(y), HOST))
        return y.reshape(gate.shape)

    def mulmat_id(self, w: Weight, n_expert: int, b: np.ndarray, ids: np.ndarray) -> np.ndarray:
        """w: n_expert stacked matrices uploaded as one weight of m = rows * n_expert; b: f32
        [tokens, b_cols, k]; ids: int32 [tokens, n_used] -> f32 [tokens, n_used, rows]."""
        b = np.ascontiguousarray(b, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        if b.ndim != 3 or ids.ndim != 2 or b.shape[0] != ids.shape[0] or b.shape[2] != w.k:
            raise ValueError(f"b {b.shape} / ids {ids.shape} do not fit [tokens, b_cols, k={w.k}] / [tokens, n_used]")
        t, n_used = ids.shape
        y = np.empty((t, n_used, w.m // max(n_expert, 1)), dtype=np.float32)  # the library rejects a ragged split
        _check(lib().mi_qmm_mulmat_id(self._h, w._h, n_expert, b.ctypes.data_as(ctypes.c_void_p), b.shape[1],
                                      ids.ctypes.data_as(ctypes.c_void_p), n_used, t,
                                      y.ctypes.data_as(ctypes.c_void_p), HOST))
        return y

    def mulmat_id_produced(self, w: Weight, n_expert: int, producer: int, aux, b: np.ndarray, ids: np.ndarray,
                           eps: float = 0.0) -> np.ndarray:
        """mulmat_id on producer(b): PRODUCE_SWIGLU with aux = up, shaped like b (the expert down projection), or
        PRODUCE_RMSNORM with aux = norm weight [k] or None"""
        b = np.ascontiguousarray(b, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        if b.ndim != 3 or ids.ndim != 2 or b.shape[0] != ids.shape[0] or b.shape[2] != w.k:
            raise ValueError(f"b {b.shape} / ids {ids.shape} do not fit [tokens, b_cols, k={w.k}] / [tokens, n_used]")
        if aux is not None:
            aux = np.ascontiguousarray(aux, dtype=np.float32)
            want = b.shape if producer == PRODUCE_SWIGLU else (w.k,)
            if aux.shape != want:
                raise ValueError(f"aux has shape {aux.shape}, the producer wants {want}")
        t, n_used = ids.shape
        y = np.empty((t, n_used, w.m // max(n_expert, 1)), dtype=np.float32)
        _check(lib().mi_qmm_mulmat_id_produced(self._h, w._h, n_expert, producer, _ptr(aux) if aux is not None else None,
                                               eps, _ptr(b), b.shape[1], _ptr(ids), n_used, t, _ptr(y), HOST))
        return y

    def mulmat_id_produced_device(self, w: Weight, n_expert: int, producer: int, aux_ptr, b_ptr: int, b_cols: int,
                                  ids_ptr: int, n_used: int, n_tokens: int, y_ptr: int, eps: float = 0.0):
        _check(lib().mi_qmm_mulmat_id_produced(self._h, w._h, n_expert, producer,
                                               ctypes.c_void_p(int(aux_ptr)) if aux_ptr else None, eps,
                                               ctypes.c_void_p(int(b_ptr)), b_cols, ctypes.c_void_p(int(ids_ptr)), n_used,
                                               n_tokens, ctypes.c_void_p(int(y_ptr)), DEVICE))

    def mulmat_id_swiglu(self, w_gate: Weight, w_up: Weight, n_expert: int, b: np.ndarray, ids: np.ndarray) -> np.ndarray:
        """silu(gate experts . Q8(b)) * (up experts . Q8(b)): f32 [tokens, n_used, rows]"""
        b = np.ascontiguousarray(b, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        if b.ndim != 3 or ids.ndim != 2 or b.shape[0] != ids.shape[0] or b.shape[2] != w_gate.k:
            raise ValueError(f"b {b.shape} / ids {ids.shape} do not fit [tokens, b_cols, k={w_gate.k}] / [tokens, n_used]")
        t, n_used = ids.shape
        h = np.empty((t, n_used, w_gate.m // max(n_expert, 1)), dtype=np.float32)
        _check(lib().mi_qmm_mulmat_id_swiglu(self._h, w_gate._h, w_up._h, n_expert, _ptr(b), b.shape[1], _ptr(ids), n_used, t,
                                             _ptr(h), HOST))
        return h

    def mulmat_id_swiglu_device(self, w_gate: Weight, w_up: Weight, n_expert: int, b_ptr: int, b_cols: int, ids_ptr: int,
                                n_used: int, n_tokens: int, h_ptr: int):
        _check(lib().mi_qmm_mulmat_id_swiglu(self._h, w_gate._h, w_up._h, n_expert, ctypes.c_void_p(int(b_ptr)), b_cols,
                                             ctypes.c_void_p(int(ids_ptr)), n_used, n_tokens, ctypes.c_void_p(int(h_ptr)),
                                             DEVICE))

    def mulmat_id_multi(self, ws, n_expert: int, b: np.ndarray, ids: np.ndarray):
        """several expert stacks against the same b and ids; host arrays out"""
        b = np.ascontiguousarray(b, dtype=np.float32)
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        if b.ndim != 3 or ids.ndim != 2 or b.shape[0] != ids.shape[0] or any(b.shape[2] != w.k for w in ws):
            raise ValueError(f"b {b.shape} / ids {ids.shape} do not fit [tokens, b_cols, k] / [tokens, n_used]")
        t, n_used = ids.shape
        ys = [np.empty((t, n_used, w.m // max(n_expert, 1)), dtype=np.float32) for w in ws]
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[y.ctypes.data_as(ctypes.c_void_p) for y in ys])
        _check(lib().mi_qmm_mulmat_id_multi(self._h, wh, len(ws), n_expert, b.ctypes.data_as(ctypes.c_void_p), b.shape[1],
                                            ids.ctypes.data_as(ctypes.c_void_p), n_used, t, yp, HOST))
        return ys

    def mulmat_id_multi_device(self, ws, n_expert: int, b_ptr: int, b_cols: int, ids_ptr: int, n_used: int,
                               n_tokens: int, y_ptrs):
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[ctypes.c_void_p(int(p)) for p in y_ptrs])
        _check(lib().mi_qmm_mulmat_id_multi(self._h, wh, len(ws), n_expert, ctypes.c_void_p(int(b_ptr)), b_cols,
                                            ctypes.c_void_p(int(ids_ptr)), n_used, n_tokens, yp, DEVICE))

    def mulmat_id_device(self, w: Weight, n_expert: int, b_ptr: int, b_cols: int, ids_ptr: int, n_used: int,
                         n_tokens: int, y_ptr: int):
        """device pointers; queued on the ctx's stream"""
        _check(lib().mi_qmm_mulmat_id(self._h, w._h, n_expert, ctypes.c_void_p(int(b_ptr)), b_cols,
                                      ctypes.c_void_p(int(ids_ptr)), n_used, n_tokens, ctypes.c_void_p(int(y_ptr)),
                                      DEVICE))

    def mulmat_q8_multi(self, ws, act: Act):
        """several weights against the same activations; host arrays out"""
        ys = [np.empty((act.n, w.m), dtype=np.float32) for w in ws]
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[y.ctypes.data for y in ys])
        _check(lib().mi_qmm_mulmat_q8_multi(self._h, wh, len(ws), act._h, yp, HOST))
        return ys

    def mulmat_q8_multi_device(self, ws, act: Act, y_ptrs):
        """device outputs; one launch for up to 4 weights of one type and k when n <= 8"""
        wh = (ctypes.c_void_p * len(ws))(*[w._h for w in ws])
        yp = (ctypes.c_void_p * len(ws))(*[ctypes.c_void_p(int(p)) for p in y_ptrs])
        _check(lib().mi_qmm_mulmat_q8_multi(self._h, wh, len(ws), act._h, yp, DEVICE))
