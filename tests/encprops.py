"""What least squares and rounding fix about the K-quant weight encoders, checked in fp64 on the bytes of any encoder.

The encoders (ggml's quantize_row_q4_K_ref / quantize_row_q6_K_ref) search a small grid of candidate scales per group of
32 or 16 values, fit (scale, min) or scale to the candidate's levels by weighted least squares, keep the best, quantize
the group scales to 6 or 8 bits against the block's fp16 d / dmin and finally re-round every value against the stored
scales.  Nothing here needs the encoder's source: each check is a property the stored bytes must have.
"""
import numpy as np

import npref
import oracle


def _round_half_even(v):
    return np.rint(v)


def q4k_stored_bytes(x: np.ndarray, raw: np.ndarray, search=True):
    """x: f32 [rows][k]; raw: the rows' Q4_K bytes.  Raises AssertionError naming the first property that fails."""
    k = x.shape[1]
    xs = x.astype(np.float64).reshape(-1, 8, 32)                    # [block][sub-block][value]
    d, dmin, sc, mn, q = npref.q4_K_ints(raw.reshape(-1))
    nb = xs.shape[0]
    assert q.shape == (nb, 8, 32) and k % 256 == 0
    # the largest group scale (minimum) of a block takes code 63: d = max / 63
    live = d > 0
    assert np.all(sc[live].max(axis=1) == 63), "Q4_K: a block whose largest scale code is not 63"
    livem = dmin > 0
    assert np.all(mn[livem].max(axis=1) == 63), "Q4_K: a block whose largest min code is not 63"
    assert np.all(mn[~livem] == 0) or np.all(dmin[~livem] == 0)
    # every stored level is the nearest one for the stored scale and min (0..15, clamped at the ends)
    de = d[:, None] * sc                                            # [block][sub]
    dm = dmin[:, None] * mn
    on = de != 0
    t = (xs + dm[:, :, None]) / np.where(on, de, 1.0)[:, :, None]
    lo_ok = (q > 0) | (t <= 0.5 + 1e-4)
    hi_ok = (q < 15) | (t >= 14.5 - 1e-4)
    mid_ok = (q == 0) | (q == 15) | (np.abs(t - q) <= 0.5 + 1e-4)
    ok = (lo_ok & hi_ok & mid_ok) | ~on[:, :, None]
    assert ok.all(), f"Q4_K: {np.count_nonzero(~ok)} stored levels are not the nearest for the stored scale and min"
    if not search:
        return
    # the 6-bit codes are the group's searched (scale, min) against the block's maxima
    x32 = x.reshape(-1, 8, 32)
    for b in range(nb):
        s = np.zeros(8); m = np.zeros(8)
        for j in range(8):
            g = x32[b, j]
            av = np.sqrt(np.float32(np.cumsum(g * g, dtype=np.float32)[-1] / np.float32(32)))   # summed in order, like the encoder
            s[j], mj, _ = oracle.qkx2_search(g, (np.float32(av) + np.abs(g)).astype(np.float32))
            m[j] = -mj
        if s.max() > 0:
            assert np.all(np.abs(63.0 * s / s.max() - sc[b]) <= 0.5 + 1e-3), f"Q4_K block {b}: scale codes {sc[b]} for scales {s}"
            assert abs(d[b] - s.max() / 63.0) <= 2.0 ** -11 * d[b] + 2.0 ** -25
        if m.max() > 0:
            assert np.all(np.abs(63.0 * m / m.max() - mn[b]) <= 0.5 + 1e-3), f"Q4_K block {b}: min codes {mn[b]} for mins {m}"
            assert abs(dmin[b] - m.max() / 63.0) <= 2.0 ** -11 * dmin[b] + 2.0 ** -25


def q6k_stored_bytes(x: np.ndarray, raw: np.ndarray, search=True):
    """x: f32 [rows][k]; raw: the rows' Q6_K bytes."""
    xs = x.astype(np.float64).reshape(-1, 16, 16)
    d, sc, q = npref.q6_K_ints(raw.reshape(-1))
    nb = xs.shape[0]
    q = q.reshape(nb, 16, 16)
    live = d != 0
    # d = -(group scale of largest magnitude) / 128: that group's code is -128
    assert np.all(sc[live].min(axis=1) == -128), "Q6_K: a live block without the code -128"
    assert not sc[~live].any() and np.all(q[~live] == -32)          # an all-zero block is stored as zero bytes
    de = d[:, None] * sc
    on = de != 0
    t = xs / np.where(on, de, 1.0)[:, :, None]
    lo_ok = (q > -32) | (t <= -31.5 + 1e-4)
    hi_ok = (q < 31) | (t >= 30.5 - 1e-4)
    mid_ok = (q == -32) | (q == 31) | (np.abs(t - q) <= 0.5 + 1e-4)
    ok = (lo_ok & hi_ok & mid_ok) | ~on[:, :, None]
    assert ok.all(), f"Q6_K: {np.count_nonzero(~ok)} stored levels are not the nearest for the stored scale"
    if not search:
        return
    x16 = x.reshape(-1, 16, 16)
    for b in range(nb):
        s = np.array([oracle.qx_search(x16[b, j])[0] for j in range(16)])
        top = s[np.argmax(np.abs(s))]
        if abs(top) < 1e-15:
            assert d[b] == 0
            continue
        want = np.minimum(127, -128.0 * s / top)
        assert np.all(np.abs(np.minimum(want, 127.49) - sc[b]) <= 0.5 + 1e-3), f"Q6_K block {b}: codes {sc[b]} for scales {s}"
        assert abs(d[b] + top / 128.0) <= 2.0 ** -11 * abs(d[b]) + 2.0 ** -25   # fp16 rounding; half a subnormal step


# ---- the searches themselves -------------------------------------------------------------------------------------------
def _wls_scale_min(x, w, l):
    """fp64 weighted least squares of x ~ s*l + m with m <= 0 (the grid's offset is never positive)"""
    sw, sl, sl2, sx, sxl = w.sum(), (w * l).sum(), (w * l * l).sum(), (w * x).sum(), (w * l * x).sum()
    D = sw * sl2 - sl * sl
    if D <= 0:
        return None
    s, m = (sw * sxl - sx * sl) / D, (sl2 * sx - sl * sxl) / D
    if m > 0:
        s, m = sxl / sl2, 0.0
    return s, m


def _werr(x, w, l, s, m):
    return float((w * (s * l + m - x) ** 2).sum())


def qkx2_search_result(x, w, nmax=15, rmin=-1.0, rdelta=0.1, nstep=20):
    """Checks one group's result of the asymmetric search; returns 'flat', 'start' or 'fit' (which branch produced it)."""
    s, m, L = oracle.qkx2_search(x, w, nmax, rmin, rdelta, nstep)
    x64, w64, l64 = x.astype(np.float64), w.astype(np.float64), L.astype(np.float64)
    lo, hi = min(float(x.min()), 0.0), float(x.max())
    if hi == lo:
        assert s == 0.0 and m == lo and not L.any()
        return "flat"
    assert m <= 0.0 and L.max() <= nmax
    # the min/max start: levels of the grid that spans [lo, hi] exactly
    isc = np.float32(nmax) / (np.float32(hi) - np.float32(lo))
    l0 = np.clip(_round_half_even((isc * (x - np.float32(lo))).astype(np.float32)), 0, nmax).astype(np.float64)
    s0 = float(np.float32(1) / isc)
    e0 = _werr(x64, w64, l0, s0, lo)
    e = _werr(x64, w64, l64, s, m)
    floor = 1e-10 * float((w64 * x64 * x64).sum()) + 1e-30           # fp32 evaluation of an exact fit leaves this much
    assert e <= e0 * (1 + 1e-5) + floor, "the search returned a worse fit than its min/max start"
    kept_start = np.array_equal(l64, l0) and s == s0 and m == lo
    if not kept_start:
        fit = _wls_scale_min(x64, w64, l64)
        assert fit is not None
        tol = 2e-4 * max(abs(fit[0]), abs(fit[1]), 1e-30)
        assert abs(fit[0] - s) <= tol and abs(fit[1] - m) <= tol, f"(scale, min) = ({s}, {m}), least squares for the returned levels gives {fit}"
    # (The candidates after an improvement are laid out from the improved minimum, so which grids get tried depends on
    # the path of the search: "best of a fixed grid" is not a property of the result and is not asserted.)
    return "start" if kept_start else "fit"


def qx_search_result(x, nmax=32):
    """Checks one group's result of the symmetric search (weights x^2); returns the winning grid step or None."""
    s, l = oracle.qx_search(x, nmax)
    x64 = x.astype(np.float64)
    amax = np.abs(x64).max()
    if amax < 1e-15:
        assert s == 0.0 and np.all(l == -nmax)                      # raw level bytes 0; the scale 0 makes them moot
        return None
    w = x64 * x64
    top = x64[np.argmax(np.abs(x64))]
    assert l.min() >= -nmax and l.max() <= nmax - 1
    sxl, sl2 = (w * x64 * l).sum(), (w * l * l).sum()
    assert sl2 > 0 and abs(s - sxl / sl2) <= 1e-5 * abs(s), f"scale {s}, least squares for the returned levels gives {sxl / sl2}"
    assert np.sign(s) == -np.sign(top)                             # the value of largest magnitude sits at the level -nmax
    obj = sxl * sxl / sl2                                           # what least squares removes from sum w x^2
    won = None
    for i in range(-9, 10):
        isc = -(np.float32(nmax) + np.float32(0.1) * np.float32(i)) / np.float32(top)
        li = np.clip(_round_half_even((isc * x).astype(np.float32)), -nmax, nmax - 1).astype(np.float64)
        a, b = (w * x64 * li).sum(), (w * li * li).sum()
        if b > 0:
            assert obj >= a * a / b * (1 - 1e-4), f"grid step {i} fits better: {a * a / b} > {obj}"
            if np.array_equal(li, l) and won is None:
                won = i
    assert won is not None, "the returned levels belong to no step of the grid"
    return won
