"""Independent numpy checkers for the GGUF block formats (test helper, not the oracle).

Written straight from the published block layouts (field order from the size formulas in
/root/reference/fs/ggml/ggml.go:450-473) with vectorised bit-field extraction, so that a wrong
index, shift or sign in the C oracle's loops disagrees with these.  Dequantizers return float64
so products with them are an fp64 brute-force statement of what each dot product must equal.
"""
from __future__ import annotations

import numpy as np

F32, Q4_0, Q5_0, Q8_0, Q4_K, Q5_K, Q6_K, Q8_K, MXFP4 = 0, 2, 6, 8, 12, 13, 14, 15, 39
BLOCK = {MXFP4: 32, Q5_0: 32, Q4_0: 32, Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256, Q8_K: 256}
BYTES = {MXFP4: 17, Q5_0: 22, Q4_0: 18, Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210, Q8_K: 292}


def _blocks(raw: np.ndarray, t: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    assert raw.size % BYTES[t] == 0
    return raw.reshape(-1, BYTES[t])


def _f16(b: np.ndarray) -> np.ndarray:
    """two little-endian bytes per row -> float64 via numpy's IEEE binary16"""
    return np.ascontiguousarray(b).view("<f2").astype(np.float64).reshape(-1)


def q4k_scales_mins(s12: np.ndarray):
    """[nb,12] uint8 -> (sc [nb,8], m [nb,8]) by plain bit-field extraction."""
    s = s12.astype(np.int64)
    sc = np.empty(s.shape[:-1] + (8,), np.int64)
    m = np.empty_like(sc)
    for j in range(4):
        sc[..., j] = s[..., j] & 63
        m[..., j] = s[..., j + 4] & 63
        sc[..., j + 4] = (s[..., j + 8] & 15) | ((s[..., j] >> 6) << 4)
        m[..., j + 4] = (s[..., j + 8] >> 4) | ((s[..., j + 4] >> 6) << 4)
    return sc, m


def q4_0_ints(raw):
    b = _blocks(raw, Q4_0)
    d = _f16(b[:, 0:2])
    qs = b[:, 2:18].astype(np.int64)
    q = np.concatenate([qs & 15, qs >> 4], axis=1) - 8  # elements 0..15 low nibbles, 16..31 high
    return d, q


def mxfp4_values(raw):
    """[nb, 32] float64 from the formats' definitions (OCP microscaling): E2M1 = sign, two exponent bits, one mantissa
    bit -- 0 and 0.5 at exponent 0, (1 + m / 2) 2^(exp - 1) above -- times the E8M0 scale 2^(e - 127)"""
    b = _blocks(raw, MXFP4)
    e = b[:, 0].astype(np.int64)
    nib = np.concatenate([b[:, 1:] & 15, b[:, 1:] >> 4], axis=1).astype(np.int64)   # elements 0..15, then 16..31
    sign = np.where(nib & 8, -1.0, 1.0)
    ex, man = (nib >> 1) & 3, nib & 1
    mag = np.where(ex == 0, man * 0.5, (1 + man / 2) * 2.0 ** (ex - 1))
    return sign * mag * (2.0 ** (e - 127))[:, None]


def q5_0_ints(raw):
    """(d, the 32 integers q - 16): nibbles as in Q4_0, bit i of the little-endian 32-bit word qh is the fifth bit of element i"""
    b = _blocks(raw, Q5_0)
    d = _f16(b[:, 0:2])
    qh = b[:, 2:6].astype(np.int64)
    word = qh[:, 0] | (qh[:, 1] << 8) | (qh[:, 2] << 16) | (qh[:, 3] << 24)
    bits = (word[:, None] >> np.arange(32)[None, :]) & 1
    nib = np.concatenate([b[:, 6:] & 15, b[:, 6:] >> 4], axis=1).astype(np.int64)
    return d, nib + 16 * bits - 16


def q8_0_ints(raw):
    b = _blocks(raw, Q8_0)
    return _f16(b[:, 0:2]), b[:, 2:34].view(np.int8).astype(np.int64)


def q4_K_ints(raw):
    b = _blocks(raw, Q4_K)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    sc, m = q4k_scales_mins(b[:, 4:16])
    qs = b[:, 16:144].astype(np.int64).reshape(-1, 4, 32)       # 4 chunks of 32 bytes
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32)  # sub-block 2c = low, 2c+1 = high
    return d, dmin, sc, m, q


def q5_K_ints(raw):
    """d, dmin, 6-bit scales and mins as for Q4_K; the 5-bit values: nibble + 16 * (bit j of qh[l]) for element l of
    sub-block j -- a bit-field statement written from the block layout, not from the C loops"""
    b = _blocks(raw, Q5_K)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    sc, m = q4k_scales_mins(b[:, 4:16])
    qh = b[:, 16:48].astype(np.int64)                                   # [nb, 32]
    qs = b[:, 48:176].astype(np.int64).reshape(-1, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32)
    bits = (qh[:, None, :] >> np.arange(8)[None, :, None]) & 1           # [nb, 8 sub-blocks, 32]
    return d, dmin, sc, m, q + 16 * bits


def q6_K_ints(raw):
    b = _blocks(raw, Q6_K)
    ql = b[:, 0:128].astype(np.int64).reshape(-1, 2, 64)
    qh = b[:, 128:192].astype(np.int64).reshape(-1, 2, 32)
    sc = b[:, 192:208].view(np.int8).astype(np.int64)
    d = _f16(b[:, 208:210])
    e = np.empty((b.shape[0], 2, 4, 32), np.int64)
    e[:, :, 0] = (ql[:, :, 0:32] & 15) | (((qh >> 0) & 3) << 4)
    e[:, :, 1] = (ql[:, :, 32:64] & 15) | (((qh >> 2) & 3) << 4)
    e[:, :, 2] = (ql[:, :, 0:32] >> 4) | (((qh >> 4) & 3) << 4)
    e[:, :, 3] = (ql[:, :, 32:64] >> 4) | (((qh >> 6) & 3) << 4)
    return d, sc, e.reshape(-1, 256) - 32


def q8_K_ints(raw):
    b = _blocks(raw, Q8_K)
    d = np.ascontiguousarray(b[:, 0:4]).view("<f4").astype(np.float64).reshape(-1)
    qs = b[:, 4:260].view(np.int8).astype(np.int64)
    bsums = np.ascontiguousarray(b[:, 260:292]).view("<i2").astype(np.int64)
    return d, qs, bsums


def dequant(t: int, raw) -> np.ndarray:
    """GGUF blocks -> float64 values, flat."""
    if t == Q4_0:
        d, q = q4_0_ints(raw)
        return (d[:, None] * q).reshape(-1)
    if t == Q8_0:
        d, q = q8_0_ints(raw)
        return (d[:, None] * q).reshape(-1)
    if t == MXFP4:
        return mxfp4_values(raw).reshape(-1)
    if t == Q5_0:
        d, q = q5_0_ints(raw)
        return (d[:, None] * q).reshape(-1)
    if t == Q4_K:
        d, dmin, sc, m, q = q4_K_ints(raw)
        w = (d[:, None] * sc)[:, :, None] * q - (dmin[:, None] * m)[:, :, None]
        return w.reshape(-1)
    if t == Q5_K:
        d, dmin, sc, m, q = q5_K_ints(raw)
        w = (d[:, None] * sc)[:, :, None] * q - (dmin[:, None] * m)[:, :, None]
        return w.reshape(-1)
    if t == Q6_K:
        d, sc, e = q6_K_ints(raw)
        w = d[:, None, None] * sc[:, :, None] * e.reshape(-1, 16, 16)
        return w.reshape(-1)
    if t == Q8_K:
        d, qs, _ = q8_K_ints(raw)
        return (d[:, None] * qs).reshape(-1)
    raise ValueError(t)


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    """numpy statement of the Q8_0 activation quantizer (fp32 arithmetic, half away from zero)."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    v = (x * idv[:, None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))).astype(np.int8)  # roundf
    out = np.empty((x.shape[0], 34), np.uint8)
    out[:, 0:2] = d.astype("<f2").view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def quantize_q8_K(x: np.ndarray) -> np.ndarray:
    """numpy statement of the Q8_K activation quantizer (first signed max, rne, bsums)."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, 256)
    nb = x.shape[0]
    idx = np.argmax(np.abs(x), axis=1)  # first occurrence of the maximum
    mx = x[np.arange(nb), idx]
    out = np.zeros((nb, 292), np.uint8)
    nz = mx != 0
    with np.errstate(divide="ignore", invalid="ignore"):
        iscale = (np.float32(-127.0) / mx).astype(np.float32)
        v = np.rint((x * iscale[:, None]).astype(np.float32))
        q = np.minimum(127, v)
        dd = (np.float32(1.0) / iscale).astype(np.float32)
    q = np.where(nz[:, None], q, 0).astype(np.int8)
    dd = np.where(nz, dd, np.float32(0)).astype("<f4")
    out[:, 0:4] = dd.view(np.uint8).reshape(-1, 4)
    out[:, 4:260] = q.view(np.uint8)
    bs = q.astype(np.int64).reshape(nb, 16, 16).sum(axis=2).astype("<i2")
    out[:, 260:292] = bs.view(np.uint8).reshape(nb, 32)
    return out.reshape(-1)


def matmul_f64(wtype: int, w_raw, k: int, m: int, xq_type: int, xq_raw, n: int) -> np.ndarray:
    """fp64 brute force: dequant(W) [m,k] against dequant(Q8(x)) [n,k] -> [n,m]."""
    W = dequant(wtype, w_raw).reshape(m, k)
    X = dequant(xq_type, xq_raw).reshape(n, k)
    return X @ W.T


def rel_err(y: np.ndarray, ref: np.ndarray, floor: float = 1e-2) -> float:
    """max over elements of |y-ref| / max(|ref|, floor*rms(ref)) -- the path's tolerance metric.

    Relative error is ill-posed where an output cancels to ~0, so the denominator is floored at
    1% of the output RMS.  (At a 0.1% floor the scalar oracle's own fp32 summation noise against
    exact arithmetic already reads 7e-4 at K=14336, i.e. the metric would measure the oracle.)
    The bar on this metric is 1e-3, which also bounds every absolute error by 1e-5*rms.
    """
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    if not ref.size:
        return 0.0
    rms = float(np.sqrt(np.mean(ref * ref)))
    den = np.maximum(np.abs(ref), floor * rms)
    den = np.where(den == 0, 1.0, den)
    return float(np.max(np.abs(y - ref) / den))
