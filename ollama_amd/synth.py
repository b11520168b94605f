"""Synthetic GGUF weight blocks for benchmarks and smoke runs (numpy, host side, no GPU work).

These are simple *valid* encoders -- round-to-nearest on a per-sub-block min/max grid -- not the
iterative searches llama-quantize runs (make_qkx2_quants / make_qx_quants; reached in the product
through /root/reference/server/quantization.go:125-181).  Any valid block exercises the matmul path
identically: its cost and its arithmetic do not depend on how the scales were chosen.  Block layouts
are the ones in csrc/formats.h.
"""
from __future__ import annotations

import numpy as np

F32, F16, Q4_0, Q5_0, Q8_0, Q4_K, Q5_K, Q6_K, BF16, MXFP4 = 0, 1, 2, 6, 8, 12, 13, 14, 30, 39


def _f16_bytes(v: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(v.astype("<f2")).view(np.uint8).reshape(v.shape + (2,))


def encode_q8_0(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 32, 32)
    d = np.abs(b).max(axis=2) / np.float32(127)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[..., None] > 0, np.rint(b / d[..., None]), 0).clip(-127, 127).astype(np.int8)
    out = np.empty((m, k // 32, 34), np.uint8)
    out[..., 0:2] = _f16_bytes(d)
    out[..., 2:] = q.view(np.uint8)
    return out.reshape(m, -1)


def encode_q4_0(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 32, 32)
    idx = np.abs(b).argmax(axis=2)
    mx = np.take_along_axis(b, idx[..., None], axis=2)[..., 0]
    d = mx / np.float32(-8)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[..., None] != 0, np.rint(b / d[..., None]) + 8, 8).clip(0, 15).astype(np.uint8)
    out = np.empty((m, k // 32, 18), np.uint8)
    out[..., 0:2] = _f16_bytes(d)
    out[..., 2:] = q[..., :16] | (q[..., 16:] << 4)
    return out.reshape(m, -1)


def encode_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    return x.view(np.uint8).reshape(x.shape[0], -1)


def encode_f16(x: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(x, np.float32).astype(np.float16)
    return h.view(np.uint8).reshape(h.shape[0], -1)


def encode_bf16(x: np.ndarray) -> np.ndarray:
    """round to nearest even on the upper 16 bits"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    h = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return h.view(np.uint8).reshape(h.shape[0], -1)


def encode_mxfp4(x: np.ndarray) -> np.ndarray:
    """blocks of 32: the power-of-two scale that brings the largest magnitude to at most 6 (the largest E2M1 value),
    every element to the nearest E2M1 value; 17 bytes: the E8M0 scale byte, then low nibbles = elements 0..15, high
    nibbles = elements 16..31"""
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 32, 32).astype(np.float64)
    amax = np.abs(b).max(axis=2)
    with np.errstate(divide="ignore"):
        e = np.where(amax > 0, np.ceil(np.log2(np.maximum(amax, 1e-300) / 6.0)), -127).clip(-127, 127).astype(np.int64)
    grid = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6])
    v = np.abs(b) / (2.0 ** e)[..., None]
    code = np.abs(v[..., None] - grid).argmin(axis=-1).astype(np.uint8)
    code |= (b < 0).astype(np.uint8) << 3
    out = np.empty((m, k // 32, 17), np.uint8)
    out[..., 0] = (e + 127).astype(np.uint8)
    out[..., 1:] = code[..., :16] | (code[..., 16:] << 4)
    return out.reshape(m, -1)


def encode_q5_0(x: np.ndarray) -> np.ndarray:
    """as encode_q4_0 on 32 levels: d = (the element of largest magnitude) / -16, q = round(x / d) + 16 in 0..31; the fifth
    bits of the 32 elements in a little-endian 32-bit word"""
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 32, 32)
    idx = np.abs(b).argmax(axis=2)
    mx = np.take_along_axis(b, idx[..., None], axis=2)[..., 0]
    d = mx / np.float32(-16)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[..., None] != 0, np.rint(b / d[..., None]) + 16, 16).clip(0, 31).astype(np.uint8)
    out = np.empty((m, k // 32, 22), np.uint8)
    out[..., 0:2] = _f16_bytes(d)
    word = ((q >> 4).astype(np.uint64) << np.arange(32, dtype=np.uint64)).sum(axis=2).astype(np.uint32)
    out[..., 2:6] = word[..., None].view(np.uint8).reshape(m, k // 32, 4)
    out[..., 6:] = (q[..., :16] & 15) | ((q[..., 16:] & 15) << 4)
    return out.reshape(m, -1)


def encode_q4_K(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 256, 8, 32)
    lo = np.minimum(b.min(axis=3), 0)
    scale = (b.max(axis=3) - lo) / np.float32(15)
    mins = -lo
    d = (scale.max(axis=2) / np.float32(63)).astype(np.float16)
    dmin = (mins.max(axis=2) / np.float32(63)).astype(np.float16)
    df, dmf = d.astype(np.float32), dmin.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(df[..., None] > 0, np.rint(scale / df[..., None]), 0).clip(0, 63).astype(np.uint8)
        mn = np.where(dmf[..., None] > 0, np.rint(mins / dmf[..., None]), 0).clip(0, 63).astype(np.uint8)
        eff = df[..., None] * sc
        q = np.where(eff[..., None] > 0, np.rint((b + (dmf[..., None] * mn)[..., None]) / eff[..., None]), 0)
    q = q.clip(0, 15).astype(np.uint8)
    out = np.zeros((m, k // 256, 144), np.uint8)
    out[..., 0:2] = _f16_bytes(d)
    out[..., 2:4] = _f16_bytes(dmin)
    s = out[..., 4:16]
    for j in range(4):
        s[..., j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        s[..., j + 4] = (mn[..., j] & 63) | ((mn[..., j + 4] >> 4) << 6)
        s[..., j + 8] = (sc[..., j + 4] & 15) | ((mn[..., j + 4] & 15) << 4)
    qq = q.reshape(m, k // 256, 4, 2, 32)
    out[..., 16:] = (qq[..., 0, :] | (qq[..., 1, :] << 4)).reshape(m, k // 256, 128)
    return out.reshape(m, -1)


def encode_q5_K(x: np.ndarray) -> np.ndarray:
    """as encode_q4_K on a grid of 32 levels; the fifth bit of element l of sub-block j is bit j of qh[l]"""
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 256, 8, 32)
    lo = np.minimum(b.min(axis=3), 0)
    scale = (b.max(axis=3) - lo) / np.float32(31)
    mins = -lo
    d = (scale.max(axis=2) / np.float32(63)).astype(np.float16)
    dmin = (mins.max(axis=2) / np.float32(63)).astype(np.float16)
    df, dmf = d.astype(np.float32), dmin.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(df[..., None] > 0, np.rint(scale / df[..., None]), 0).clip(0, 63).astype(np.uint8)
        mn = np.where(dmf[..., None] > 0, np.rint(mins / dmf[..., None]), 0).clip(0, 63).astype(np.uint8)
        eff = df[..., None] * sc
        q = np.where(eff[..., None] > 0, np.rint((b + (dmf[..., None] * mn)[..., None]) / eff[..., None]), 0)
    q = q.clip(0, 31).astype(np.uint8)
    out = np.zeros((m, k // 256, 176), np.uint8)
    out[..., 0:2] = _f16_bytes(d)
    out[..., 2:4] = _f16_bytes(dmin)
    s = out[..., 4:16]
    for j in range(4):
        s[..., j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        s[..., j + 4] = (mn[..., j] & 63) | ((mn[..., j + 4] >> 4) << 6)
        s[..., j + 8] = (sc[..., j + 4] & 15) | ((mn[..., j + 4] & 15) << 4)
    hi = (q >> 4).astype(np.uint8)                                      # [m, nb, 8, 32]
    qh = np.zeros((m, k // 256, 32), np.uint8)
    for j in range(8):
        qh |= hi[..., j, :] << j
    out[..., 16:48] = qh
    qq = (q & 15).reshape(m, k // 256, 4, 2, 32)
    out[..., 48:] = (qq[..., 0, :] | (qq[..., 1, :] << 4)).reshape(m, k // 256, 128)
    return out.reshape(m, -1)


def encode_q6_K(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    b = x.reshape(m, k // 256, 16, 16)
    scale = np.abs(b).max(axis=3) / np.float32(31)
    d = (scale.max(axis=2) / np.float32(127)).astype(np.float16)
    df = d.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(df[..., None] > 0, np.rint(scale / df[..., None]), 0).clip(0, 127).astype(np.int8)
        eff = df[..., None] * sc
        q = np.where(eff[..., None] > 0, np.rint(b / eff[..., None]), 0).clip(-32, 31)
    e = (q + 32).astype(np.uint8).reshape(m, k // 256, 2, 4, 32)  # halves of 128, four runs of 32
    out = np.empty((m, k // 256, 210), np.uint8)
    ql = np.empty((m, k // 256, 2, 64), np.uint8)
    ql[..., 0:32] = (e[..., 0, :] & 15) | ((e[..., 2, :] & 15) << 4)
    ql[..., 32:64] = (e[..., 1, :] & 15) | ((e[..., 3, :] & 15) << 4)
    qh = (e[..., 0, :] >> 4) | ((e[..., 1, :] >> 4) << 2) | ((e[..., 2, :] >> 4) << 4) | ((e[..., 3, :] >> 4) << 6)
    out[..., 0:128] = ql.reshape(m, k // 256, 128)
    out[..., 128:192] = qh.reshape(m, k // 256, 64)
    out[..., 192:208] = sc.view(np.uint8)
    out[..., 208:210] = _f16_bytes(d)
    return out.reshape(m, -1)


ENCODERS = {Q4_0: encode_q4_0, Q5_0: encode_q5_0, Q8_0: encode_q8_0, Q4_K: encode_q4_K, Q5_K: encode_q5_K, Q6_K: encode_q6_K, MXFP4: encode_mxfp4,
            F32: encode_f32, F16: encode_f16, BF16: encode_bf16}


def weights(ggml_type: int, m: int, k: int, seed: int, std: float = 0.02, chunk_rows: int = 2048) -> np.ndarray:
    """N(0, std) weights drawn from ``seed`` and encoded to ``ggml_type``: uint8 [m, row_size]."""
    rng = np.random.default_rng(seed)
    enc = ENCODERS[ggml_type]
    parts = []
    for r0 in range(0, m, chunk_rows):
        r = min(chunk_rows, m - r0)
        parts.append(enc(rng.standard_normal((r, k), dtype=np.float32) * np.float32(std)))
    return np.concatenate(parts, axis=0)
