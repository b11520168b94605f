"""CPU oracle for the GGUF quantized-matmul path -- TEST INFRASTRUCTURE ONLY.

ctypes binding of ``oracle/ggml_ref.c`` (a scalar C restatement of the ggml CPU semantics).
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; the shipped library never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libggml_ref.so")

F32, F16, Q4_0, Q5_0, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K, BF16, MXFP4 = 0, 1, 2, 6, 8, 12, 13, 14, 15, 30, 39


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a second or two)."""
    src = os.path.join(_HERE, "ggml_ref.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libggml_ref.so"])
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.ref_block_size.restype = i64; L.ref_block_size.argtypes = [ci]
        L.ref_type_size.restype = i64; L.ref_type_size.argtypes = [ci]
        L.ref_row_size.restype = i64; L.ref_row_size.argtypes = [ci, i64]
        L.ref_fp32_to_fp16.restype = ctypes.c_uint16; L.ref_fp32_to_fp16.argtypes = [ctypes.c_float]
        L.ref_fp16_to_fp32.restype = ctypes.c_float; L.ref_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        L.ref_quantize.restype = ci; L.ref_quantize.argtypes = [ci, vp, vp, i64, i64, ci]
        L.ref_dequantize_row.restype = ci; L.ref_dequantize_row.argtypes = [ci, vp, vp, i64]
        L.ref_get_scale_min_k4.restype = None; L.ref_get_scale_min_k4.argtypes = [ci, vp, vp, vp]
        L.ref_unpack_scales_kmask.restype = None; L.ref_unpack_scales_kmask.argtypes = [vp, vp, vp]
        L.ref_fp32_to_bf16.restype = ctypes.c_uint16; L.ref_fp32_to_bf16.argtypes = [ctypes.c_float]
        L.ref_bf16_to_fp32.restype = ctypes.c_float; L.ref_bf16_to_fp32.argtypes = [ctypes.c_uint16]
        L.ref_e8m0_to_fp32_half.restype = ctypes.c_float; L.ref_e8m0_to_fp32_half.argtypes = [ctypes.c_uint8]
        for name in ("mxfp4_q8_0", "q5_0_q8_0", "q4_0_q8_0", "q8_0_q8_0", "q4_K_q8_K", "q5_K_q8_K", "q6_K_q8_K", "f32", "f16", "bf16"):
            f = getattr(L, "ref_vec_dot_" + name)
            f.restype = ctypes.c_float; f.argtypes = [i64, vp, vp]
        L.ref_vec_dot_type.restype = ci; L.ref_vec_dot_type.argtypes = [ci]
        L.ref_mul_mat.restype = ci
        L.ref_mul_mat.argtypes = [ci, vp, i64, i64, vp, i64, vp, vp, ci]
        L.ref_mul_mat_id.restype = ci
        L.ref_mul_mat_id.argtypes = [ci, vp, i64, i64, i64, vp, i64, vp, i64, i64, vp]
        L.ref_rms_norm.restype = None; L.ref_rms_norm.argtypes = [vp, vp, ctypes.c_float, i64, i64, vp]
        L.ref_qkx2_search.restype = ctypes.c_float
        L.ref_qkx2_search.argtypes = [ci, ci, vp, vp, vp, vp, ctypes.c_float, ctypes.c_float, ci]
        L.ref_qx_search.restype = ctypes.c_float; L.ref_qx_search.argtypes = [ci, ci, vp, vp]
        L.ref_swiglu.restype = None; L.ref_swiglu.argtypes = [vp, vp, i64, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def block_size(t: int) -> int:
    return int(lib().ref_block_size(t))


def type_size(t: int) -> int:
    return int(lib().ref_type_size(t))


def row_size(t: int, k: int) -> int:
    return int(lib().ref_row_size(t, k))


def vec_dot_type(t: int) -> int:
    return int(lib().ref_vec_dot_type(t))


def fp32_to_fp16(f: float) -> int:
    return int(lib().ref_fp32_to_fp16(f))


def fp32_to_bf16(f: float) -> int:
    return int(lib().ref_fp32_to_bf16(ctypes.c_float(f)))


def bf16_to_fp32(h: int) -> float:
    return float(lib().ref_bf16_to_fp32(h))


def fp16_to_fp32(h: int) -> float:
    return float(lib().ref_fp16_to_fp32(h))


def quantize(t: int, x: np.ndarray, nthreads: int = 1) -> np.ndarray:
    """x: f32 [rows, k] -> uint8 [rows, row_size(t, k)] of GGUF-layout blocks."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim == 1:
        x = x[None, :]
    rows, k = x.shape
    rb = row_size(t, k)
    if rb < 0:
        raise ValueError(f"k={k} is not a multiple of the block size of type {t}")
    out = np.zeros((rows, rb), dtype=np.uint8)
    if lib().ref_quantize(t, _p(x), _p(out), k, rows, nthreads) != 0:
        raise ValueError("ref_quantize failed")
    return out


def dequantize(t: int, blocks: np.ndarray, k: int) -> np.ndarray:
    """blocks: uint8 [rows, row_size] -> f32 [rows, k]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    if blocks.ndim == 1:
        blocks = blocks[None, :]
    rows = blocks.shape[0]
    assert blocks.shape[1] == row_size(t, k)
    out = np.empty((rows, k), dtype=np.float32)
    for r in range(rows):
        if lib().ref_dequantize_row(t, _p(blocks[r]), _p(out[r]), k) != 0:
            raise ValueError("ref_dequantize_row failed")
    return out


_DOTS = {MXFP4: "mxfp4_q8_0", Q5_0: "q5_0_q8_0", Q4_0: "q4_0_q8_0", Q8_0: "q8_0_q8_0", Q4_K: "q4_K_q8_K", Q5_K: "q5_K_q8_K", Q6_K: "q6_K_q8_K", F32: "f32", F16: "f16", BF16: "bf16"}


def vec_dot(wtype: int, k: int, wrow: np.ndarray, xqrow: np.ndarray) -> float:
    f = getattr(lib(), "ref_vec_dot_" + _DOTS[wtype])
    wrow = np.ascontiguousarray(wrow, dtype=np.uint8)
    xqrow = np.ascontiguousarray(xqrow, dtype=np.uint8)
    assert wrow.size == row_size(wtype, k) and xqrow.size == row_size(vec_dot_type(wtype), k)
    return float(f(k, _p(wrow), _p(xqrow)))


def mul_mat(wtype: int, w: np.ndarray, k: int, m: int, x: np.ndarray, nthreads: int = 1,
            return_xq: bool = False):
    """w: uint8 GGUF blocks of m rows; x: f32 [n, k] -> y f32 [n, m] (y[n, m] = dot(W_m, Q(x_n)))."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim == 1:
        x = x[None, :]
    n = x.shape[0]
    assert x.shape[1] == k and w.size == m * row_size(wtype, k)
    y = np.empty((n, m), dtype=np.float32)
    xq = np.zeros((n, row_size(vec_dot_type(wtype), k)), dtype=np.uint8)
    if lib().ref_mul_mat(wtype, _p(w), k, m, _p(x), n, _p(y), _p(xq), nthreads) != 0:
        raise ValueError("ref_mul_mat failed")
    return (y, xq) if return_xq else y


def mul_mat_id(wtype: int, w: np.ndarray, k: int, m: int, n_expert: int, b: np.ndarray, ids: np.ndarray):
    """w: uint8 GGUF blocks of n_expert stacked matrices of m rows; b: f32 [tokens, b_cols, k];
    ids: int32 [tokens, n_used] -> y f32 [tokens, n_used, m]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.float32)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    assert b.ndim == 3 and ids.ndim == 2 and b.shape[0] == ids.shape[0] and b.shape[2] == k
    assert w.size == n_expert * m * row_size(wtype, k)
    t, n_used = ids.shape
    y = np.empty((t, n_used, m), dtype=np.float32)
    rc = lib().ref_mul_mat_id(wtype, _p(w), k, m, n_expert, _p(b), b.shape[1], _p(ids), n_used, t, _p(y))
    if rc == -2:
        raise IndexError("expert id outside 0..n_expert-1")
    if rc != 0:
        raise ValueError("ref_mul_mat_id failed")
    return y


def rms_norm(x: np.ndarray, g, eps: float) -> np.ndarray:
    """x: f32 [n, k]; g: f32 [k] or None -> (x / sqrt(mean(x^2) + eps)) * g, row by row."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 2
    y = np.empty_like(x)
    if g is not None:
        g = np.ascontiguousarray(g, dtype=np.float32)
        assert g.shape == (x.shape[1],)
    lib().ref_rms_norm(_p(x), _p(g) if g is not None else None, eps, x.shape[1], x.shape[0], _p(y))
    return y


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(gate) * up, elementwise (f32)."""
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    up = np.ascontiguousarray(up, dtype=np.float32)
    assert gate.shape == up.shape
    y = np.empty_like(gate)
    lib().ref_swiglu(_p(gate), _p(up), gate.size, _p(y))
    return y


def qkx2_search(x: np.ndarray, weights: np.ndarray, nmax: int = 15, rmin: float = -1.0, rdelta: float = 0.1, nstep: int = 20):
    """The (scale, min) search of the Q4_K encoder on one group: returns (scale, min, levels) with min <= 0."""
    x = np.ascontiguousarray(x, np.float32); w = np.ascontiguousarray(weights, np.float32)
    assert x.ndim == 1 and x.shape == w.shape
    lv = np.zeros(x.size, np.uint8)
    neg_min = np.zeros(1, np.float32)
    sc = lib().ref_qkx2_search(x.size, nmax, _p(x), _p(w), _p(lv), _p(neg_min), rmin, rdelta, nstep)
    return float(sc), -float(neg_min[0]), lv


def qx_search(x: np.ndarray, nmax: int = 32):
    """The scale search of the Q6_K encoder on one group: returns (scale, signed levels)."""
    x = np.ascontiguousarray(x, np.float32)
    lv = np.zeros(x.size, np.int8)
    sc = lib().ref_qx_search(x.size, nmax, _p(x), _p(lv))
    return float(sc), lv.astype(np.int32) - nmax


def scale_min_k4(j: int, s12: np.ndarray):
    s12 = np.ascontiguousarray(s12, dtype=np.uint8)
    sc = np.zeros(1, np.uint8); m = np.zeros(1, np.uint8)
    lib().ref_get_scale_min_k4(j, _p(s12), _p(sc), _p(m))
    return int(sc[0]), int(m[0])


def unpack_scales_kmask(s12: np.ndarray):
    s12 = np.ascontiguousarray(s12, dtype=np.uint8)
    sc = np.zeros(8, np.uint8); m = np.zeros(8, np.uint8)
    lib().ref_unpack_scales_kmask(_p(s12), _p(sc), _p(m))
    return sc, m
