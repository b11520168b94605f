"""Pins the CPU oracle (oracle/ggml_ref.c) before anything is compared against it.

The reference holds only size/id tables for this path (fs/ggml/ggml_test.go:163-213,
fs/ggml/type_test.go:68-115); those are checked from tests/golden/tensor_types.json.  Everything
numeric is pinned by what the mathematics fixes: numpy's IEEE binary16, closed-form known-answer
blocks, an independently written numpy statement of the formats (tests/npref.py), and fp64 brute
force of every dot product.  Each check is chosen so a dropped term, wrong sign/index/shift or a
transposed operand fails it.
"""
import json
import os

import numpy as np
import pytest

import npref
import oracle
from npref import Q4_0, Q4_K, Q6_K, Q8_0, Q8_K

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tensor_types.json")))
WTYPES = [Q4_0, Q8_0, Q4_K, Q6_K]


# ---- sizes (reference golden table) ---------------------------------------------------------
def test_sizes_match_reference_table():
    rows = {r["kind"]: r for r in GOLD["sizes"]}
    for t in (0, Q4_0, Q8_0, Q4_K, Q6_K, Q8_K):
        assert oracle.block_size(t) == rows[t]["block_size"]
        assert oracle.type_size(t) == rows[t]["type_size"]
    # row sizes quoted for the benchmark shapes
    assert oracle.row_size(Q4_0, 4096) == 2304 and oracle.row_size(Q8_0, 4096) == 4352
    assert oracle.row_size(Q4_K, 4096) == 2304 and oracle.row_size(Q6_K, 4096) == 3360
    assert oracle.row_size(Q4_K, 14336) == 8064 and oracle.row_size(Q6_K, 14336) == 11760
    assert oracle.row_size(Q8_K, 4096) == 4672 and oracle.row_size(Q8_K, 14336) == 16352
    bad = GOLD["row_not_multiple_of_block"]
    assert oracle.row_size(bad["kind"], bad["shape0"]) == -1


# ---- fp16 -------------------------------------------------------------------------------------
def test_fp16_to_fp32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_fp32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)  # NaN payloads do not survive the ctypes float return; NaN-ness must
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_fp32_to_fp16_rne_vs_numpy():
    rng = np.random.default_rng(7)
    # every half value, every midpoint between adjacent halves, +-1 ulp around midpoints, randoms
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (h[:-1] + h[1:]) / 2
    cand = np.concatenate([h, mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                           np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
                           [65504, 65519.99, 65520, 65536, 1e9, 2.0**-25, 2.0**-24, 5.96e-8, 2.98e-8,
                            2.9802326e-08, 0.0],
                           rng.standard_normal(20000) * 10.0 ** rng.integers(-8, 5, 20000)]).astype(np.float32)
    cand = np.concatenate([cand, -cand])
    with np.errstate(over="ignore"):
        want = cand.astype(np.float16).view(np.uint16)
    got = np.array([oracle.fp32_to_fp16(float(v)) for v in cand], dtype=np.uint16)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (cand[bad[:5]], got[bad[:5]], want[bad[:5]])


# ---- Q8_0 activation quantizer ---------------------------------------------------------------
def _q8_0(x):
    raw = oracle.quantize(Q8_0, np.asarray(x, np.float32).reshape(1, -1)).reshape(-1, 34)
    return raw[:, 0:2].copy().view(np.float16).reshape(-1), raw[:, 2:].view(np.int8)


def test_q8_0_known_answers():
    x = np.zeros(32, np.float32)
    x[:6] = [127, -127, 0, 1, -1, 64]
    d, q = _q8_0(x)
    assert d[0] == 1.0 and list(q[0][:6]) == [127, -127, 0, 1, -1, 64] and not q[0][6:].any()
    # constant block: q = +-127, d = fp16(|c|/127)
    d, q = _q8_0(np.full(32, -0.3, np.float32))
    assert (q == -127).all() and d[0] == np.float16(np.float32(0.3) / np.float32(127))
    # all-zero block
    d, q = _q8_0(np.zeros(32, np.float32))
    assert d[0] == 0 and not q.any()
    # halves round away from zero (roundf), not to even: amax 127 -> id 1
    x = np.zeros(32, np.float32); x[0] = 127; x[1:5] = [2.5, -2.5, 0.5, 3.5]
    _, q = _q8_0(x)
    assert list(q[0][1:5]) == [3, -3, 1, 4]


def test_q8_0_matches_numpy_statement():
    rng = np.random.default_rng(11)
    for scale in (1.0, 1e-3, 37.0, 1e-20, 3e4):
        x = (rng.standard_normal(32 * 257) * scale).astype(np.float32)
        assert np.array_equal(oracle.quantize(Q8_0, x).reshape(-1), npref.quantize_q8_0(x))
    d, q = _q8_0(rng.standard_normal(32 * 50).astype(np.float32))
    assert np.abs(q.astype(int)).max(axis=1).min() == 127  # the arg-max always maps to +-127


# ---- Q8_K activation quantizer ---------------------------------------------------------------
def _q8_K(x):
    raw = oracle.quantize(Q8_K, np.asarray(x, np.float32).reshape(1, -1)).reshape(-1)
    return npref.q8_K_ints(raw)


def test_q8_K_known_answers():
    # ramp j-128: max-magnitude element is -128 (first), iscale = +127/128 = 0.9921875
    x = np.arange(256, dtype=np.float32) - 128
    d, q, bs = _q8_K(x)
    assert d[0] == np.float32(1.0) / np.float32(0.9921875)
    want = np.minimum(127, np.rint((x * np.float32(0.9921875)).astype(np.float32)))
    assert np.array_equal(q[0], want) and q[0][0] == -127
    assert np.array_equal(bs[0], q[0].reshape(16, 16).sum(1))
    # single positive spike: q = -127 and d carries the sign
    x = np.zeros(256, np.float32); x[77] = 2.0
    d, q, bs = _q8_K(x)
    assert q[0][77] == -127 and q[0].sum() == -127 and d[0] == np.float32(1) / (np.float32(-127) / np.float32(2))
    assert bs[0][77 // 16] == -127 and bs[0].sum() == -127
    # tie +a before -a: the first wins, so +a -> -127 and -a -> +127
    x = np.zeros(256, np.float32); x[3] = 5.0; x[9] = -5.0
    d, q, _ = _q8_K(x)
    assert q[0][3] == -127 and q[0][9] == 127 and d[0] < 0
    x[3], x[9] = -5.0, 5.0
    d, q, _ = _q8_K(x)
    assert q[0][3] == -127 and q[0][9] == 127 and d[0] > 0
    # all-zero block is fully zero (d, qs, bsums)
    assert not oracle.quantize(Q8_K, np.zeros(256, np.float32)).any()


def test_q8_K_matches_numpy_statement_and_invariants():
    rng = np.random.default_rng(12)
    for scale in (1.0, 1e-4, 250.0):
        x = (rng.standard_normal(256 * 131) * scale).astype(np.float32)
        raw = oracle.quantize(Q8_K, x).reshape(-1)
        assert np.array_equal(raw, npref.quantize_q8_K(x))
        d, q, bs = npref.q8_K_ints(raw)
        assert q.min() >= -127 and q.max() <= 127
        assert np.array_equal(bs.sum(1), q.sum(1))
        err = np.abs(d[:, None] * q - x.reshape(-1, 256).astype(np.float64))
        assert (err <= np.abs(d)[:, None] * 0.5 * (1 + 1e-5)).all()


# ---- 6-bit scale / min unpack ------------------------------------------------------------------
def test_scale_min_unpack_formulations_agree():
    rng = np.random.default_rng(13)
    s = rng.integers(0, 256, (2000, 12), dtype=np.uint8)
    sc_np, m_np = npref.q4k_scales_mins(s)
    for i in range(len(s)):
        sc, m = oracle.unpack_scales_kmask(s[i])
        pairs = [oracle.scale_min_k4(j, s[i]) for j in range(8)]
        assert [p[0] for p in pairs] == list(sc) == list(sc_np[i])
        assert [p[1] for p in pairs] == list(m) == list(m_np[i])
    # each packed field is reachable: one sub-block at 63, the rest 0
    for j in range(8):
        s12 = np.zeros(12, np.uint8)
        if j < 4:
            s12[j] = 63
        else:
            s12[j + 4] = 0x0F; s12[j - 4] = 0xC0
        sc, m = oracle.unpack_scales_kmask(s12)
        assert list(sc) == [63 if i == j else 0 for i in range(8)] and not m.any()


# ---- dequantizers vs the independent numpy statement -----------------------------------------
@pytest.mark.parametrize("t", [Q4_0, Q8_0, Q4_K, Q6_K, Q8_K])
def test_dequant_random_bytes_matches_numpy(t):
    """random *bytes* (not encoder output) reach every bit pattern of every field"""
    rng = np.random.default_rng(100 + t)
    nb = 64
    raw = rng.integers(0, 256, (nb, npref.BYTES[t]), dtype=np.uint8)
    # keep fp16/fp32 scale fields finite and moderate
    h = rng.standard_normal(nb * 2).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if t in (Q4_0, Q8_0):
        raw[:, 0:2] = h[:, 0:2]
    elif t == Q4_K:
        raw[:, 0:4] = h
    elif t == Q6_K:
        raw[:, 208:210] = h[:, 0:2]
    else:
        raw[:, 0:4] = rng.standard_normal(nb).astype(np.float32).view(np.uint8).reshape(nb, 4)
    k = nb * npref.BLOCK[t]
    got = oracle.dequantize(t, raw.reshape(1, -1), k).reshape(-1).astype(np.float64)
    want = npref.dequant(t, raw)
    assert np.allclose(got, want, rtol=3e-7, atol=0)


# ---- dot products: fp64 brute force ------------------------------------------------------------
def _rand_blocks(t, nb, rng):
    raw = rng.integers(0, 256, (nb, npref.BYTES[t]), dtype=np.uint8)
    h = (rng.standard_normal(nb * 2) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if t in (Q4_0, Q8_0):
        raw[:, 0:2] = h[:, 0:2]
    elif t == Q4_K:
        raw[:, 0:4] = np.abs((rng.standard_normal(nb * 2) * 0.01)).astype(np.float16).view(np.uint8).reshape(nb, 4)
    elif t == Q6_K:
        raw[:, 208:210] = h[:, 0:2]
    return raw


@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("nb", [1, 3, 16])
def test_vec_dot_random_bytes_vs_fp64(t, nb):
    rng = np.random.default_rng(200 + t + nb)
    k = nb * 256
    w = _rand_blocks(t, k // npref.BLOCK[t], rng)
    x = rng.standard_normal(k).astype(np.float32)
    qt = oracle.vec_dot_type(t)
    xq = oracle.quantize(qt, x).reshape(-1)
    got = oracle.vec_dot(t, k, w.reshape(-1), xq)
    W = npref.dequant(t, w)
    X = npref.dequant(qt, xq)
    want = float(W @ X)
    scale = float(np.sqrt((W * W).sum() * (X * X).sum()))
    assert abs(got - want) <= 2e-6 * scale, (got, want)


def test_vec_dot_exact_integer_cases():
    """power-of-two scales and small integers: the answer is an exact integer."""
    rng = np.random.default_rng(5)
    one = np.float16(1.0).view(np.uint16)
    # Q8_0 x Q8_0, d = 1 on both sides -> plain int dot
    k = 128
    wq = rng.integers(-127, 128, k).astype(np.int8)
    w = np.zeros((k // 32, 34), np.uint8)
    w[:, 0:2] = np.array([one], np.uint16).view(np.uint8)
    w[:, 2:] = wq.view(np.uint8).reshape(-1, 32)
    x = rng.integers(-20, 21, k).astype(np.float32)
    x[::32] = 127  # amax = 127 -> d = 1, q = x
    xq = oracle.quantize(Q8_0, x).reshape(-1)
    assert oracle.vec_dot(Q8_0, k, w.reshape(-1), xq) == float(wq.astype(np.int64) @ x.astype(np.int64))
    # Q4_0 with d = 1: weights are (nibble - 8), low nibbles first then high nibbles
    nib = rng.integers(0, 16, k).astype(np.uint8).reshape(-1, 32)
    w4 = np.zeros((k // 32, 18), np.uint8)
    w4[:, 0:2] = np.array([one], np.uint16).view(np.uint8)
    w4[:, 2:] = nib[:, :16] | (nib[:, 16:] << 4)
    want = float((nib.astype(np.int64).reshape(-1) - 8) @ x.astype(np.int64))
    assert oracle.vec_dot(Q4_0, k, w4.reshape(-1), xq) == want
    # Q4_K: d = 1, dmin = 1, distinct scales/mins per sub-block (catches a swapped scale/min index)
    k = 256
    sc = np.array([1, 2, 3, 4, 5, 6, 7, 9]); mn = np.array([8, 7, 6, 5, 4, 3, 2, 1])
    s12 = np.zeros(12, np.uint8)
    for j in range(4):
        s12[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        s12[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        s12[j + 8] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    q = rng.integers(0, 16, 256).astype(np.uint8).reshape(4, 2, 32)
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([one], np.uint16).view(np.uint8); blk[2:4] = blk[0:2]
    blk[4:16] = s12
    blk[16:] = (q[:, 0, :] | (q[:, 1, :] << 4)).reshape(-1)
    x = rng.integers(-30, 31, 256).astype(np.float32); x[0] = -127  # iscale = 1 -> q8 = x, d = 1
    xq = oracle.quantize(Q8_K, x).reshape(-1)
    xi = x.astype(np.int64).reshape(8, 32)
    want = float(sum(sc[j] * int(q.reshape(8, 32)[j].astype(np.int64) @ xi[j]) - mn[j] * int(xi[j].sum())
                     for j in range(8)))
    assert oracle.vec_dot(Q4_K, k, blk, xq) == want
    # Q6_K: d = 1, distinct int8 scales (incl. negative) per 16
    scales = np.array([1, -2, 3, -4, 5, -6, 7, -8, 9, 10, -11, 12, 13, -14, 15, 16], np.int8)
    e = rng.integers(0, 64, 256).astype(np.uint8).reshape(2, 4, 32)
    blk = np.zeros(210, np.uint8)
    ql = np.zeros((2, 64), np.uint8); qh = np.zeros((2, 32), np.uint8)
    ql[:, 0:32] = (e[:, 0] & 15) | ((e[:, 2] & 15) << 4)
    ql[:, 32:64] = (e[:, 1] & 15) | ((e[:, 3] & 15) << 4)
    qh[:] = (e[:, 0] >> 4) | ((e[:, 1] >> 4) << 2) | ((e[:, 2] >> 4) << 4) | ((e[:, 3] >> 4) << 6)
    blk[0:128] = ql.reshape(-1); blk[128:192] = qh.reshape(-1)
    blk[192:208] = scales.view(np.uint8); blk[208:210] = np.array([one], np.uint16).view(np.uint8)
    ev = e.reshape(256).astype(np.int64) - 32
    want = float(sum(int(scales[g]) * int(ev[16 * g:16 * g + 16] @ x.astype(np.int64)[16 * g:16 * g + 16])
                     for g in range(16)))
    assert oracle.vec_dot(Q6_K, k, blk, xq) == want


# ---- mul_mat driver ----------------------------------------------------------------------------
@pytest.mark.parametrize("t", WTYPES)
def test_mul_mat_layout_and_brute_force(t):
    rng = np.random.default_rng(300 + t)
    k, m, n = 512, 7, 3  # m != n catches a transposed output
    w = oracle.quantize(t, (rng.standard_normal((m, k)) * 0.02).astype(np.float32))
    x = rng.standard_normal((n, k)).astype(np.float32)
    y1, xq = oracle.mul_mat(t, w, k, m, x, nthreads=1, return_xq=True)
    y3 = oracle.mul_mat(t, w, k, m, x, nthreads=3)
    assert y1.shape == (n, m) and np.array_equal(y1, y3)  # threading does not change results
    qt = oracle.vec_dot_type(t)
    assert np.array_equal(xq, oracle.quantize(qt, x))
    for ni in range(n):
        for mi in range(m):
            assert y1[ni, mi] == np.float32(oracle.vec_dot(t, k, w[mi], xq[ni]))
    want = npref.matmul_f64(t, w, k, m, qt, xq, n)
    assert npref.rel_err(y1, want) < 1e-5


@pytest.mark.parametrize("t", WTYPES)
def test_mul_mat_full_width_vs_fp64(t):
    """full K of the benchmark shapes, a slab of rows"""
    rng = np.random.default_rng(400 + t)
    k, m = (14336, 64) if t in (Q4_K, Q6_K) else (4096, 128)
    w = oracle.quantize(t, (rng.standard_normal((m, k)) * 0.02).astype(np.float32), nthreads=4)
    x = rng.standard_normal((2, k)).astype(np.float32)
    y, xq = oracle.mul_mat(t, w, k, m, x, nthreads=4, return_xq=True)
    want = npref.matmul_f64(t, w, k, m, oracle.vec_dot_type(t), xq, 2)
    assert npref.rel_err(y, want) < 2e-4  # what is left is the oracle's sequential fp32 summation


def test_mul_mat_rejects_bad_arguments():
    with pytest.raises(ValueError):
        oracle.quantize(Q4_0, np.zeros(31, np.float32))  # row not a multiple of the block
    L = oracle.lib()
    assert L.ref_mul_mat(3, None, 32, 1, None, 1, None, None, 1) == -1       # unsupported type
    assert L.ref_mul_mat(Q4_K, None, 128, 1, None, 1, None, None, 1) == -1   # k % 256 != 0
    assert L.ref_mul_mat(Q4_K, None, 256, 0, None, 0, None, None, 1) == 0    # empty is fine


# ---- mul_mat_id driver -------------------------------------------------------------------------
@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("b_cols", [1, 3])
def test_mul_mat_id_reduces_to_mul_mat_per_pair(t, b_cols):
    """every (token, slot) pair is mul_mat on that pair's expert alone with that pair's activation row;
    shapes chosen so that a swapped index (expert/slot/token, m/n_used) lands on a different value"""
    rng = np.random.default_rng(500 + t + b_cols)
    k, m, n_expert, n_used, tokens = 512, 5, 7, 3, 4
    w = oracle.quantize(t, (rng.standard_normal((n_expert * m, k)) * 0.02).astype(np.float32))
    b = rng.standard_normal((tokens, b_cols, k)).astype(np.float32)
    ids = rng.integers(0, n_expert, (tokens, n_used)).astype(np.int32)
    ids[0] = [6, 0, 6]  # the same expert twice in one token
    y = oracle.mul_mat_id(t, w, k, m, n_expert, b, ids)
    assert y.shape == (tokens, n_used, m)
    w3 = w.reshape(n_expert, m, -1)
    for ti in range(tokens):
        for i in range(n_used):
            want = oracle.mul_mat(t, w3[ids[ti, i]], k, m, b[ti, i % b_cols])
            assert np.array_equal(y[ti, i], want[0])


@pytest.mark.parametrize("t", WTYPES)
def test_mul_mat_id_vs_fp64_brute_force(t):
    rng = np.random.default_rng(520 + t)
    k, m, n_expert, n_used, tokens = 1024, 6, 4, 2, 3
    w = oracle.quantize(t, (rng.standard_normal((n_expert * m, k)) * 0.02).astype(np.float32))
    b = rng.standard_normal((tokens, n_used, k)).astype(np.float32)
    ids = np.array([[0, 3], [2, 2], [1, 0]], np.int32)
    y = oracle.mul_mat_id(t, w, k, m, n_expert, b, ids)
    qt = oracle.vec_dot_type(t)
    xq = oracle.quantize(qt, b.reshape(-1, k))
    full = npref.matmul_f64(t, w, k, n_expert * m, qt, xq, tokens * n_used).reshape(tokens, n_used, n_expert, m)
    want = np.stack([[full[ti, i, ids[ti, i]] for i in range(n_used)] for ti in range(tokens)])
    assert npref.rel_err(y, want) < 1e-5


def test_mul_mat_id_one_expert_is_mul_mat_and_bad_ids_are_rejected():
    rng = np.random.default_rng(540)
    k, m = 256, 9
    w = oracle.quantize(Q4_K, (rng.standard_normal((m, k)) * 0.02).astype(np.float32))
    b = rng.standard_normal((5, 1, k)).astype(np.float32)
    y = oracle.mul_mat_id(Q4_K, w, k, m, 1, b, np.zeros((5, 1), np.int32))
    assert np.array_equal(y[:, 0], oracle.mul_mat(Q4_K, w, k, m, b[:, 0]))
    for bad in (-1, 1):
        with pytest.raises(IndexError):
            oracle.mul_mat_id(Q4_K, w, k, m, 1, b, np.array([[0], [0], [bad], [0], [0]], np.int32))
    assert oracle.mul_mat_id(Q4_K, w, k, m, 1, b[:0], np.zeros((0, 1), np.int32)).shape == (0, 1, m)


# ---- weight encoders: error bounds, closed forms, and what least squares fixes about the K-quant searches
#      (bit-parity of Q4_K / Q6_K with llama-quantize stays unpinned: these catch slips of transcription, not of recall)
@pytest.mark.parametrize("t,bound", [(Q4_0, 0.14), (Q8_0, 0.008), (Q4_K, 0.10), (Q6_K, 0.03)])
def test_encoders_valid_blocks_and_error_bounds(t, bound):
    rng = np.random.default_rng(500 + t)
    k = 2048
    x = (rng.standard_normal((8, k)) * 0.02).astype(np.float32)
    raw = oracle.quantize(t, x)
    deq = npref.dequant(t, raw).reshape(8, k)
    rms = float(np.sqrt(np.mean((deq - x) ** 2)) / np.sqrt(np.mean(x.astype(np.float64) ** 2)))
    assert rms < bound, rms
    # zeros encode to blocks that decode to zeros
    z = oracle.quantize(t, np.zeros((1, k), np.float32))
    assert not npref.dequant(t, z).any()


def test_q4_0_and_q8_0_encoders_closed_form():
    # Q4_0: max-magnitude element (signed) maps to nibble 0 (value -8), d = max / -8
    x = np.linspace(-1, 0.9, 32).astype(np.float32)
    raw = oracle.quantize(Q4_0, x).reshape(-1)
    d, q = npref.q4_0_ints(raw)
    assert d[0] == np.float16(np.float32(-1) / np.float32(-8)) and q[0][0] == -8
    idv = np.float32(1) / (np.float32(-1) / np.float32(-8))
    want = np.minimum(15, (x * idv + np.float32(8.5)).astype(np.float32).astype(np.int8)).astype(np.int64) - 8
    assert np.array_equal(q[0], want)
    # Q8_0 weight encoder is the activation quantizer
    y = np.random.default_rng(3).standard_normal(64).astype(np.float32)
    assert np.array_equal(oracle.quantize(Q8_0, y).reshape(-1), npref.quantize_q8_0(y))


def _groups(rng, n, count):
    """groups of n values of the kinds a weight tensor holds: normal, one-sided, with an outlier, on a coarse grid"""
    for i in range(count):
        x = rng.standard_normal(n).astype(np.float32) * np.float32(0.02)
        kind = i % 6
        if kind == 1: x = np.abs(x) + np.float32(0.01)          # the fitted minimum would be positive: pulled to zero
        if kind == 2: x[rng.integers(n)] *= 30
        if kind == 3: x = -np.abs(x)
        if kind == 4: x = (np.rint(x * 50) / 50).astype(np.float32)
        if kind == 5: x *= np.float32(1000)
        yield x


def test_q4_K_search_returns_the_least_squares_fit_of_its_levels():
    """make_qkx2_quants as Q4_K calls it (32 values, 16 levels, weights av_x + |x|, 21 candidate grids): in fp64 the
    returned (scale, min) is the weighted least-squares optimum for the returned levels (with the minimum capped at
    zero), and never a worse fit than the min/max grid the search starts from.  A dropped term or a swapped sum in the
    normal equations fails the first, a wrong comparison the second."""
    import collections
    import encprops
    rng = np.random.default_rng(610)
    seen = collections.Counter()
    for x in _groups(rng, 32, 3000):
        av = np.sqrt(np.float32(np.cumsum(x * x, dtype=np.float32)[-1] / np.float32(32)))
        seen[encprops.qkx2_search_result(x, (av + np.abs(x)).astype(np.float32))] += 1
    assert seen["fit"] > 1000 and seen["start"] > 20, seen       # both ways out of the search were taken
    assert encprops.qkx2_search_result(np.zeros(32, np.float32), np.ones(32, np.float32)) == "flat"
    assert encprops.qkx2_search_result(np.full(32, -0.5, np.float32), np.ones(32, np.float32)) == "flat"   # stored as the minimum alone
    s, m, lv = oracle.qkx2_search(np.full(32, 0.5, np.float32), np.ones(32, np.float32))
    assert m == 0.0 and np.all(lv == 15) and abs(s * 15 - 0.5) < 1e-6       # positive constant: grid [0, 0.5], all at the top
    # other shapes of the same search: few values, few levels, no refinement steps
    for x in _groups(rng, 16, 300):
        encprops.qkx2_search_result(x, np.ones(16, np.float32), nmax=3, rmin=-0.5, rdelta=0.1, nstep=15)
        assert encprops.qkx2_search_result(x, np.abs(x) + np.float32(1e-3), nmax=31, nstep=0) in ("start", "flat")


def test_q6_K_search_returns_the_least_squares_scale_of_its_levels():
    """make_qx_quants as Q6_K calls it (16 values, levels -32..31, weights x^2, 19 candidate grids around -32/max): the
    returned scale is sum(w x l) / sum(w l^2) for the returned levels, the levels are those of one grid step, and no
    step removes more of sum(w x^2) -- the search's own criterion, evaluated in fp64."""
    import collections
    import encprops
    rng = np.random.default_rng(611)
    won = collections.Counter(encprops.qx_search_result(x) for x in _groups(rng, 16, 3000))
    assert len([i for i in won if i is not None]) >= 8, won        # the grid is really searched: many steps win somewhere
    assert encprops.qx_search_result(np.zeros(16, np.float32)) is None
    assert encprops.qx_search_result(np.full(16, 1e-16, np.float32)) is None   # below the threshold: stored as zeros
    # all values equal: every step rounds them to -32 (clamped) or -31; the scale is exactly x / l
    s, l = oracle.qx_search(np.full(16, 0.25, np.float32))
    assert len(set(l.tolist())) == 1 and l[0] in (-32, -31) and abs(s * l[0] - 0.25) < 1e-6


@pytest.mark.parametrize("scale", [0.02, 3.0, 1e-3])
def test_k_quant_encoders_stored_bytes_follow_from_the_searches(scale):
    """The blocks the encoders write: the largest group scale (min) takes the top code, d (dmin) is that scale over 63
    (Q6_K: the scale of largest magnitude takes -128), the other codes are the searched scales rounded against it, and
    every stored level is the nearest one for the scales as stored."""
    import encprops
    rng = np.random.default_rng(612)
    x = (rng.standard_normal((6, 2048)) * scale).astype(np.float32)
    x[1] *= (1 + 20 * (rng.random(2048) < 0.01)).astype(np.float32)
    x[2, :256] = 0; x[3] = np.abs(x[3]); x[4, 256:512] = -np.abs(x[4, 256:512]); x[5, 32:64] = 0
    encprops.q4k_stored_bytes(x, oracle.quantize(Q4_K, x))
    encprops.q6k_stored_bytes(x, oracle.quantize(Q6_K, x))


# ---- producers of the activations: RMSNorm, SwiGLU ------------------------------------------------

def test_rms_norm_closed_forms():
    """constant row c -> c / sqrt(c^2 + eps); one-hot row a*e_j -> a / sqrt(a^2/k + eps) at j, 0 elsewhere;
    eps = 0 makes the result invariant under scaling x; the weight multiplies elementwise afterwards"""
    k = 512
    for c, eps in ((3.0, 1e-5), (-0.25, 1e-6), (1.0, 0.5)):
        y = oracle.rms_norm(np.full((1, k), c, np.float32), None, eps)
        want = np.float32(c) * (np.float32(1) / np.sqrt(np.float32(np.float32(c) * np.float32(c)) + np.float32(eps)))
        assert np.all(y == want)
    x = np.zeros((1, k), np.float32); x[0, 77] = 4.0
    y = oracle.rms_norm(x, None, 1e-5)
    assert abs(y[0, 77] - 4.0 / np.sqrt(16.0 / k + 1e-5)) < 1e-5 and np.count_nonzero(y) == 1
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, k), dtype=np.float32)
    assert np.allclose(oracle.rms_norm(x, None, 0.0), oracle.rms_norm(4 * x, None, 0.0), rtol=1e-6)
    g = rng.standard_normal(k, dtype=np.float32)
    assert np.array_equal(oracle.rms_norm(x, g, 1e-5), oracle.rms_norm(x, None, 1e-5) * g)
    assert np.all(oracle.rms_norm(np.zeros((2, k), np.float32), g, 1e-5) == 0)


def test_rms_norm_against_fp64():
    rng = np.random.default_rng(6)
    for k in (32, 4096, 14336):
        x = (rng.standard_normal((4, k)) * rng.uniform(0.01, 30)).astype(np.float32)
        g = rng.standard_normal(k).astype(np.float32)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-5) * g
        got = oracle.rms_norm(x, g, 1e-5)
        assert np.max(np.abs(got - want) / (np.abs(want) + 1e-30)) < 1e-6
        # a dropped eps, a sum instead of a mean, or a missing square root would all miss by far more
        assert np.allclose(np.sqrt((oracle.rms_norm(x, None, 0.0).astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=1e-6)


def test_swiglu_identities_and_fp64():
    """silu(0) = 0, silu(v) - silu(-v) = v, silu(v) -> v for large v and -> 0 for very negative v;
    against an fp64 evaluation"""
    v = np.array([0.0, 1.0, -1.0, 0.5, 20.0, -20.0, 88.0, -88.0, 100.0, -100.0], np.float32)
    one = np.ones_like(v)
    s = oracle.swiglu(v, one)
    assert s[0] == 0 and s[8] == 100.0 and s[9] == 0.0 and abs(s[4] - 20.0) < 1e-6
    rng = np.random.default_rng(7)
    a = (rng.standard_normal(20000) * 4).astype(np.float32)
    u = rng.standard_normal(20000).astype(np.float32)
    ones = np.ones_like(a)
    assert np.allclose(oracle.swiglu(a, ones) - oracle.swiglu(-a, ones), a, rtol=0, atol=2e-6)
    want = a.astype(np.float64) / (1 + np.exp(-a.astype(np.float64))) * u
    got = oracle.swiglu(a, u)
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-30)) < 1e-6
    assert np.array_equal(oracle.swiglu(a, 2 * u), 2 * oracle.swiglu(a, u))  # linear in up (exact: power of two)
