"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same inputs.

Bars: quantized activation bytes bit-exact; fp32 outputs within 1e-3 on
|y-ref| / max(|ref|, 1e-2*rms(ref))  (see npref.rel_err for why the floor is 1% of the RMS).
"""
import ctypes

import numpy as np
import pytest

import npref
import oracle
from hipmem import DeviceArray, Stream
from npref import Q4_0, Q4_K, Q6_K, Q8_0, Q8_K
from ollama_amd import qmm

pytestmark = pytest.mark.gpu
TOL = 1e-3
WTYPES = [Q4_0, Q8_0, Q4_K, Q6_K]
NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _weights(t, m, k, seed, nthreads=16):
    rng = np.random.default_rng(seed)
    return oracle.quantize(t, (rng.standard_normal((m, k), dtype=np.float32) * np.float32(0.02)), nthreads=nthreads)


# ---- kernel 1: activation quantization, bit-exact ---------------------------------------------
@pytest.mark.parametrize("qt", [Q8_0, Q8_K])
@pytest.mark.parametrize("n,k", [(1, 256), (1, 4096), (3, 1024), (8, 4096), (1, 14336), (512, 4096), (5, 14336), (293, 14336), (4099, 256)])
def test_quantize_act_bit_exact(ctx, qt, n, k):
    rng = np.random.default_rng(n * 100003 + k + qt)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.quantize_act(qt, x)
    want = oracle.quantize(qt, x, nthreads=8)
    assert got.shape == want.shape
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} bytes differ"


@pytest.mark.parametrize("qt", [Q8_0, Q8_K])
def test_quantize_act_edge_cases_bit_exact(ctx, qt):
    rng = np.random.default_rng(99)
    k = 1024
    rows = []
    rows.append(np.zeros(k, np.float32))                                   # all-zero blocks
    r = np.zeros(k, np.float32); r[3] = 5.0; r[9] = -5.0; r[300] = -7.0; r[301] = 7.0   # ties, first wins
    rows.append(r)
    rows.append(np.full(k, -0.3, np.float32))                              # constant
    rows.append((np.arange(k, dtype=np.float32) - 512))                    # ramp with exact halves
    r = np.zeros(k, np.float32); r[::32] = 127; r[1::32] = 2.5; r[2::32] = -2.5; r[3::32] = 0.5
    rows.append(r)                                                         # x*id = k+0.5: roundf vs rint
    rows.append(rng.standard_normal(k).astype(np.float32) * np.float32(1e-30))   # tiny
    rows.append(rng.standard_normal(k).astype(np.float32) * np.float32(1e20))    # huge
    rows.append(rng.standard_normal(k).astype(np.float32) * np.float32(3e4))
    r = rng.standard_normal(k).astype(np.float32); r[:256] = 0; r[512:544] = 0    # zero blocks among live ones
    rows.append(r)
    rows.append(np.round(rng.standard_normal(k) * 40).astype(np.float32) / 2)    # many exact .5 products
    x = np.stack(rows)
    got = ctx.quantize_act(qt, x)
    want = oracle.quantize(qt, x)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"first differing (row, byte): {bad[:5].tolist()}"
    # the same rows as a batch large enough for the kernel that puts a Q8_K block on sixteen lanes (from 4096
    # blocks), shifted by one block per copy so that every edge block meets every position in a wave's group of four,
    # and with a row count that leaves the last group of four incomplete
    reps = 411
    big = np.concatenate([np.roll(x, 256 * i, axis=1) for i in range(reps)])[: reps * len(rows) - 1]
    big = np.ascontiguousarray(big[:, : k - 256])                            # 3 blocks per row: groups straddle rows
    got = ctx.quantize_act(qt, big)
    want = oracle.quantize(qt, big, nthreads=8)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"batch: first differing (row, byte): {bad[:5].tolist()}"


def test_quantize_act_empty_and_errors(ctx):
    assert ctx.quantize_act(Q8_K, np.zeros((0, 256), np.float32)).shape == (0, 292)
    with pytest.raises(qmm.QmmError) as e:
        ctx.quantize_act(Q8_K, np.zeros((1, 100), np.float32))
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError) as e:
        ctx.quantize_act(9, np.zeros((1, 32), np.float32))
    assert e.value.code == qmm.ERR_UNSUPPORTED


# ---- kernels 2/4: GEMV, small and ragged shapes ---------------------------------------------------
SMALL = [(256, 1), (256, 7), (512, 33), (1024, 100), (2048, 64), (2304, 5), (4096, 257), (6144, 31), (14336, 19),
         (28672, 3)]


@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("k,m", SMALL)
def test_gemv_small_shapes(ctx, t, k, m):
    w_raw = _weights(t, m, k, seed=k * 31 + m + t)
    W = ctx.upload(t, w_raw, k, m)
    rng = np.random.default_rng(k + m)
    for n in (1, 2, 3, 8):
        x = rng.standard_normal((n, k), dtype=np.float32)
        got = ctx.mulmat(W, x, path=qmm.PATH_GEMV)
        want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=8)
        assert got.shape == (n, m)
        err = npref.rel_err(got, want)
        assert err <= TOL, f"{NAMES[t]} k={k} m={m} n={n}: rel err {err}"
    W.free()


@pytest.mark.parametrize("t", WTYPES)
def test_gemv_every_column_count_and_groups(ctx, t):
    k, m = 1024, 96
    w_raw = _weights(t, m, k, seed=7 + t)
    W = ctx.upload(t, w_raw, k, m)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((19, k), dtype=np.float32)
    want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=8)
    for n in list(range(1, 10)) + [16, 17, 19]:   # > 8 runs in column groups of 8
        got = ctx.mulmat(W, x[:n], path=qmm.PATH_GEMV)
        assert npref.rel_err(got, want[:n]) <= TOL, n
    W.free()


@pytest.mark.parametrize("t", WTYPES)
def test_gemv_random_block_bytes(ctx, t):
    """weights made of random bytes reach every bit pattern of nibbles, 6-bit scales and high bits"""
    rng = np.random.default_rng(1234 + t)
    k, m = 2048, 40
    nb = m * k // npref.BLOCK[t]
    raw = rng.integers(0, 256, (nb, npref.BYTES[t]), dtype=np.uint8)
    h = np.abs(rng.standard_normal(nb * 2) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if t in (Q4_0, Q8_0):
        raw[:, 0:2] = h[:, 0:2]
    elif t == Q4_K:
        raw[:, 0:4] = h
    else:
        raw[:, 208:210] = h[:, 0:2]
    W = ctx.upload(t, raw.reshape(-1), k, m)
    x = rng.standard_normal((4, k), dtype=np.float32)
    got = ctx.mulmat(W, x, path=qmm.PATH_GEMV)
    want = oracle.mul_mat(t, raw.reshape(-1), k, m, x, nthreads=8)
    assert npref.rel_err(got, want) <= TOL
    # and against exact arithmetic: no worse than the oracle's own rounding noise by much
    xq = oracle.quantize(oracle.vec_dot_type(t), x)
    exact = npref.matmul_f64(t, raw.reshape(-1), k, m, oracle.vec_dot_type(t), xq, 4)
    assert npref.rel_err(got, exact) <= TOL
    W.free()


def test_mulmat_linearity_in_weights_rows(ctx):
    """size-independent property: rows are independent -- a row-permuted weight gives permuted outputs"""
    t, k, m = Q4_K, 4096, 512
    w_raw = _weights(t, m, k, seed=21)
    perm = np.random.default_rng(3).permutation(m)
    x = np.random.default_rng(4).standard_normal((2, k), dtype=np.float32)
    W1 = ctx.upload(t, w_raw, k, m)
    W2 = ctx.upload(t, w_raw[perm], k, m)
    y1, y2 = ctx.mulmat(W1, x), ctx.mulmat(W2, x)
    assert np.array_equal(y1[:, perm], y2)  # bit-identical: same lanes, same order per row
    W1.free(); W2.free()


# ---- the benchmark configurations at full size -----------------------------------------------------
def _config_case(ctx, t, m, k, ns, seed_w, seed_x):
    w_raw = _weights(t, m, k, seed=seed_w)
    W = ctx.upload(t, w_raw, k, m)
    assert W.gguf_bytes == w_raw.size
    rng = np.random.default_rng(seed_x)
    for n in ns:
        x = rng.standard_normal((n, k), dtype=np.float32)
        got = ctx.mulmat(W, x)
        want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=16)
        err = npref.rel_err(got, want)
        nrm = float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
        assert err <= TOL, f"{NAMES[t]} {m}x{k} n={n}: rel err {err}, normwise {nrm}"
        assert nrm <= 1e-5
        _check_against_exact_arithmetic(t, w_raw, k, m, x, got, f"{NAMES[t]} {m}x{k} n={n}")
    W.free()


def _check_against_exact_arithmetic(t, w_raw, k, m, x, got, what, max_rows=16384):
    """The GPU's integer block sums are exact, so against fp64 arithmetic on the same quantized operands it is
    held to the tighter floor, 1e-3 of the output RMS (the scalar oracle, whose sequential fp32 sums carry
    their own noise, binds the comparison above at the 1e-2 floor).  Large matrices: the first max_rows rows."""
    rows = min(m, max_rows)
    qt = qmm.vec_dot_type(t)
    n = x.shape[0]
    w_slab = np.ascontiguousarray(w_raw.reshape(m, -1)[:rows]).reshape(-1)
    exact = npref.matmul_f64(t, w_slab, k, rows, qt, oracle.quantize(qt, x, nthreads=8), n)
    err = npref.rel_err(got[:, :rows], exact, floor=1e-3)
    assert err <= TOL, f"{what}: rel err {err} against exact arithmetic at the 1e-3 floor"


def test_config1_q4_0_gemv(ctx):
    _config_case(ctx, Q4_0, 4096, 4096, [1], 1001, 2001)


def test_config2_q8_0_skinny(ctx):
    _config_case(ctx, Q8_0, 4096, 4096, [1, 2, 4, 8], 1002, 2002)


def test_config3_q4_K_ffn_gate_up(ctx):
    _config_case(ctx, Q4_K, 14336, 4096, [1], 1003, 2003)


def test_config3_q4_K_ffn_down(ctx):
    _config_case(ctx, Q4_K, 4096, 14336, [1], 1003, 2013)


def test_config4_q6_K_output_head(ctx):
    _config_case(ctx, Q6_K, 128256, 4096, [1, 8], 1004, 2004)


# ---- error behaviour -------------------------------------------------------------------------------------
def test_upload_and_mulmat_errors(ctx):
    with pytest.raises(qmm.QmmError) as e:
        ctx.upload(10, np.zeros(84, np.uint8), 256, 1)       # Q2_K is not on this path
    assert e.value.code == qmm.ERR_UNSUPPORTED
    with pytest.raises(qmm.QmmError) as e:
        ctx.upload(Q4_0, np.zeros(18, np.uint8), 31, 1)      # row not a multiple of the block
    assert e.value.code == qmm.ERR_INVALID
    W = ctx.upload(Q4_K, np.zeros(144, np.uint8), 256, 1)
    with pytest.raises(ValueError):
        ctx.mulmat(W, np.zeros((1, 512), np.float32))
    assert ctx.mulmat(W, np.zeros((0, 256), np.float32)).shape == (0, 1)
    assert not ctx.mulmat(W, np.ones((2, 256), np.float32)).any()   # zero weights -> zero outputs
    W.free()


# ---- two-phase form: quantize once, multiply by several weights --------------------------------------
def test_two_phase_matches_fused(ctx):
    k = 4096
    rng = np.random.default_rng(77)
    x = rng.standard_normal((3, k), dtype=np.float32)
    act = ctx.act_create(Q8_K, k, 8)
    ctx.act_quantize(act, x)
    for t, m in ((Q4_K, 300), (Q6_K, 129)):
        w_raw = _weights(t, m, k, seed=m)
        W = ctx.upload(t, w_raw, k, m)
        assert np.array_equal(ctx.mulmat_q8(W, act), ctx.mulmat(W, x))
        W.free()
    # a smaller batch afterwards reuses the same storage
    ctx.act_quantize(act, x[:1])
    w_raw = _weights(Q4_K, 64, k, seed=9)
    W = ctx.upload(Q4_K, w_raw, k, 64)
    assert np.array_equal(ctx.mulmat_q8(W, act), ctx.mulmat(W, x[:1]))
    # type / shape mismatches are rejected
    W8 = ctx.upload(Q8_0, _weights(Q8_0, 8, k, seed=1), k, 8)
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_q8(W8, act)
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError):
        ctx.act_quantize(act, np.zeros((9, k), np.float32))   # more rows than n_max
    W.free(); W8.free(); act.free()


def test_multi_weight_launch_matches_single(ctx):
    """gate+up (and q/k/v with different row counts) through one launch give the same bits as one
    launch per weight"""
    k = 4096
    rng = np.random.default_rng(31)
    for t in (Q4_K, Q8_0, Q6_K, Q4_0):
        ms = [1024, 300, 4096]
        raws = [_weights(t, m, k, seed=100 + m) for m in ms]
        Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
        act = ctx.act_create(qmm.vec_dot_type(t), k, 40)
        # 3, 4: Q4_K in one launch of the direct-load MFMA kernel; 6, 9, 12: K-quants in one launch of the staged
        # skinny kernel of their format (ragged M = 300 in the middle); 40: one GEMM launch (K-quants)
        for n in (1, 3, 4, 6, 9, 12, 40):
            x = rng.standard_normal((n, k), dtype=np.float32)
            ctx.act_quantize(act, x)
            want = [ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV if n <= 8 else qmm.PATH_AUTO) for W in Ws]
            got = ctx.mulmat_q8_multi(Ws, act)
            for y, wnt in zip(got, want):
                assert np.array_equal(y, wnt)
            # f32 activations in: the same bits as the two-phase calls
            for y, wnt in zip(ctx.mulmat_multi(Ws, x), want):
                assert np.array_equal(y, wnt)
        act.free()
        for W in Ws:
            W.free()


def test_multi_weight_launch_with_unequal_k_cuts_falls_back(ctx):
    """a large and a small matrix would cut K differently in launches of their own: the multi call must not
    join them, and gives the bits of the single calls"""
    k, ms = 4096, [14336, 1024]
    rng = np.random.default_rng(37)
    for t in (Q4_K, Q6_K, Q8_0):
        raws = [_weights(t, m, k, seed=300 + m + t) for m in ms]
        Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
        for n in (4, 7):
            x = rng.standard_normal((n, k), dtype=np.float32)
            want = [ctx.mulmat(W, x) for W in Ws]
            for y, wnt, raw, m in zip(ctx.mulmat_multi(Ws, x), want, raws, ms):
                assert np.array_equal(y, wnt)
                assert npref.rel_err(y, oracle.mul_mat(t, raw, k, m, x, nthreads=16)) < TOL
        for W in Ws:
            W.free()


@pytest.mark.parametrize("ms,k,ns", [([14336, 14336], 4096, (3, 8, 11, 16)), ([14336, 14336, 1000], 4096, (6,)),
                                     ([24600], 4096, (5,)), ([24592], 8192, (3,)), ([9000, 16000], 2048, (7,))])
def test_q4k_rows_kernel_alone_and_joint(ctx, ms, k, ns):
    """Q4_K at 3..16 columns on matrices with many rows (together from six 16-row groups per CU): the kernel with the
    activations resident in LDS, a wave per row group and whole K.  It restarts its accumulator where the general
    kernel would cut K for that matrix alone, so a joint launch gives the bits of the single launches (which take the
    general kernel below the row threshold: 14336, 1000, 9000 rows; K cut two, eight and three ways) -- and the
    oracle's numbers.  Ragged last row groups, K of 2048 / 4096 / 8192, one and two column sets."""
    rng = np.random.default_rng(8700 + sum(ms) + k)
    raws = [_weights(Q4_K, m, k, seed=8701 + m + i) for i, m in enumerate(ms)]
    Ws = [ctx.upload(Q4_K, r, k, m) for r, m in zip(raws, ms)]
    for n in ns:
        x = rng.standard_normal((n, k), dtype=np.float32)
        got = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        for y, W, raw, m in zip(got, Ws, raws, ms):
            assert npref.rel_err(y, oracle.mul_mat(Q4_K, raw, k, m, x, nthreads=16)) < TOL
            _check_against_exact_arithmetic(Q4_K, raw, k, m, x, y, f"Q4_K {m}x{k} n={n}", max_rows=2048)
            if len(Ws) > 1:
                assert np.array_equal(ctx.mulmat(W, x), y), (m, n)
        # a column's result does not depend on which other columns ride along
        again = ctx.mulmat_multi(Ws, x[::-1].copy()) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x[::-1].copy())]
        for y, z in zip(got, again):
            assert np.array_equal(z[::-1], y)
    for W in Ws:
        W.free()


@pytest.mark.parametrize("ms,k,ns", [([14336, 14336], 4096, (2, 3, 4, 8)), ([14336], 4096, (2, 5)), ([4096], 14336, (3, 4, 7, 8)),
                                     ([14330, 5000], 4096, (6,)), ([4100], 14336 + 256, (5,)), ([8192], 8192, (4, 8)),
                                     ([70000], 4096, (2, 3, 8)), ([40000, 33000], 2048, (2, 5)), ([131072 + 48], 1024, (8,)),
                                     ([8192], 4096, (5, 8)), ([6150, 5200], 4096, (6,)), ([2600], 8192, (7,)),
                                     ([4100], 28672, (2, 3, 4))])
def test_q4k_deep_kernel_few_columns_on_large_matrices(ctx, ms, k, ns):
    """Q4_K at 3..8 columns (from two on rows up to 4096) on matrices beyond 40 M weights, and at 5..8 columns from 20 M
    (8192 x 4096, 6150 and 5200 rows in one launch, 2600 x 8192): the kernel that loads weights straight into registers (a ring
    of four super-blocks per lane, quads of lanes on contiguous runs of a row, ds_bpermute into the MFMA operand order)
    with the activations resident in LDS -- quantized by the workgroups themselves when x comes as f32.  Shapes that
    take every cut of the launch: waves sharing a row group two and fourteen ways (gate + up, down), row groups of their
    own (70000 and 131120 rows: two row groups per wave in turn), a last piece of one super-block (K = 14592), ragged
    last row groups, two matrices of unequal size, rows of 28672 (their activations fit the LDS at up to four columns:
    the layout then holds four columns per super-block).  Against the oracle and exact arithmetic; the f32 form gives the bits
    of quantize-then-multiply; a joint launch gives the bits of the single ones; a column's result does not depend on
    which other columns ride along."""
    rng = np.random.default_rng(9100 + sum(ms) + k)
    raws = [_weights(Q4_K, m, k, seed=9101 + m + i) for i, m in enumerate(ms)]
    Ws = [ctx.upload(Q4_K, r, k, m) for r, m in zip(raws, ms)]
    act = ctx.act_create(Q8_K, k, 8)
    for n in ns:
        x = rng.standard_normal((n, k), dtype=np.float32)
        x[0, :256] = 0.0                                               # an all-zero block
        got = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        ctx.act_quantize(act, x)
        for y, W, raw, m in zip(got, Ws, raws, ms):
            rows = min(m, 6000)                                       # (the oracle on a slab of rows: the last ones)
            want = oracle.mul_mat(Q4_K, np.ascontiguousarray(raw[-rows:]), k, rows, x, nthreads=16)
            assert npref.rel_err(y[:, -rows:], want) < TOL, (m, n)
            _check_against_exact_arithmetic(Q4_K, raw, k, m, x, y, f"Q4_K {m}x{k} n={n}", max_rows=2048)
            assert np.array_equal(ctx.mulmat_q8(W, act), y), ("f32 != planes", m, n)
            if len(Ws) > 1:
                assert np.array_equal(ctx.mulmat(W, x), y), ("joint != alone", m, n)
        again = ctx.mulmat_multi(Ws, x[::-1].copy()) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x[::-1].copy())]
        for y, z in zip(got, again):
            assert np.array_equal(z[::-1], y), n
    act.free()
    for W in Ws:
        W.free()


@pytest.mark.parametrize("ms,k,ns", [([1], 256, (3, 5, 8)), ([7], 256, (3, 8)), ([16], 256, (4,)), ([33], 512, (3, 6)), ([100], 1024, (5,)),
                                     ([1000], 1024, (3, 8)), ([300], 2048, (4, 7)), ([4096], 4096, (3, 4, 5, 8)),
                                     ([4096, 1024, 1024], 4096, (3, 5, 8)), ([1030], 4096, (3, 8)), ([4096], 2048, (3, 8)),
                                     ([4100], 8192, (3, 5)), ([20000], 1024, (4, 8)), ([12288], 4096, (3, 8)), ([2048], 12288, (3,))])
def test_q4k_deep_kernel_on_small_products(ctx, ms, k, ns):
    """Q4_K at 3..8 columns on products small enough that the workgroups quantize f32 x themselves in three rounds: the
    same direct-load kernel.  Workgroups of a single wave (K up to 1024 with at most a row group per CU: the zero block
    of the LDS map is then one wave's to write), of two and four working waves filled up with helper waves that
    quantize their share of x and leave (4096 x 4096, the q + k + v launch, 4096 x 2048), of eight and twelve working
    waves with and without helpers (8192-long rows, 12288 x 4096), matrices of one row, of 7, of ragged last row
    groups.  Against the oracle and exact arithmetic; the f32 form gives the bits of quantize-then-multiply; a joint
    launch gives the bits of the single ones; a column's result does not depend on which other columns ride along."""
    rng = np.random.default_rng(9500 + sum(ms) + k)
    raws = [_weights(Q4_K, m, k, seed=9501 + m + i) for i, m in enumerate(ms)]
    Ws = [ctx.upload(Q4_K, r, k, m) for r, m in zip(raws, ms)]
    act = ctx.act_create(Q8_K, k, 8)
    for n in ns:
        assert all(ctx.route(W, n) == "deep_f32" for W in Ws), (ms, k, n)
        x = rng.standard_normal((n, k), dtype=np.float32)
        x[0, :256] = 0.0                                               # an all-zero block
        got = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        ctx.act_quantize(act, x)
        for y, W, raw, m in zip(got, Ws, raws, ms):
            assert ctx.route_q8(W, act) == "skinny_deep", (m, k, n)
            assert npref.rel_err(y, oracle.mul_mat(Q4_K, raw, k, m, x, nthreads=16)) < TOL, (m, n)
            _check_against_exact_arithmetic(Q4_K, raw, k, m, x, y, f"Q4_K {m}x{k} n={n}", max_rows=2048)
            assert np.array_equal(ctx.mulmat_q8(W, act), y), ("f32 != planes", m, n)
            if len(Ws) > 1:
                assert np.array_equal(ctx.mulmat(W, x), y), ("joint != alone", m, n)
        again = ctx.mulmat_multi(Ws, x[::-1].copy()) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x[::-1].copy())]
        for y, z in zip(got, again):
            assert np.array_equal(z[::-1], y), n
    act.free()
    for W in Ws:
        W.free()


@pytest.mark.parametrize("m,k,ns", [(4096, 14336, (3, 4, 5, 8)), (14336, 4096, (3, 6, 8)), (14330, 4096, (4, 7)), (4100, 14336 + 256, (5,)),
                                    (8192, 8192, (4, 8)), (40000, 2048, (4, 5)), (65536 + 48, 1024, (3, 8)),
                                    (4096, 4096, (3, 4, 8)), (6150, 4096, (3, 5)), (5120, 5120, (3, 4, 7)),
                                    (1, 256, (3, 5, 8)), (7, 256, (3, 8)), (33, 512, (4, 6)), (1000, 1024, (3, 8)), (300, 2048, (4, 7)),
                                    (1030, 4096, (3, 4, 5, 8)), (4096, 2048, (3, 8)), (20000, 1024, (4, 8)), (8200, 4096, (3, 4)),
                                    (2100, 28672, (2, 3, 4))])
def test_q6k_deep_kernel_few_columns_on_large_matrices(ctx, m, k, ns):
    """Q6_K at 4..8 columns on matrices from 16 Mi weights (three columns: from 20 Mi), and on the smaller ones whose
    f32 x the workgroups quantize themselves in two rounds (workgroups of a single wave; of one to eight working waves
    filled up with helper waves that quantize their share and leave; matrices of one row, of 7, ragged last row
    groups): the direct-load kernel on the Q6_K planes (low-nibble bytes,
    bit pairs, scales and row scales each loaded by the quad of lanes of a row, ds_bpermute into the MFMA operand order,
    the 6-bit quants multiplied as stored and the offset of 32 taken out with the block sums; one set of MFMAs up to
    four columns, two from five).  Waves sharing a row group fourteen and four ways (down, gate shape), row groups of
    their own (40000 and 65584 rows), a last piece of one super-block (K = 14592), ragged last row groups, blocks of
    random bytes.  Against the
    oracle and exact arithmetic; the f32 form (which quantizes in the kernel where that is two rounds at most) gives the
    bits of quantize-then-multiply; a column's result does not depend on which other columns ride along."""
    rng = np.random.default_rng(9300 + m + k)
    raw = _weights(Q6_K, m, k, seed=9301 + m)
    if m == 14336:      # blocks of random bytes: every pattern of nibbles, bit pairs and signed scales
        nb = m * k // 256
        raw = rng.integers(0, 256, (nb, 210), dtype=np.uint8)
        raw[:, 208:210] = np.abs(rng.standard_normal(nb) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
        raw = raw.reshape(m, -1)
    W = ctx.upload(Q6_K, raw, k, m)
    act = ctx.act_create(Q8_K, k, 8)
    for n in ns:
        assert ctx.route(W, n) in ("skinny_deep", "deep_f32"), (m, k, n)
        x = rng.standard_normal((n, k), dtype=np.float32)
        x[0, :256] = 0.0                                               # an all-zero block
        y = ctx.mulmat(W, x)
        ctx.act_quantize(act, x)
        rows = min(m, 6000)                                           # (the oracle on a slab of rows: the last ones)
        want = oracle.mul_mat(Q6_K, np.ascontiguousarray(raw[-rows:]), k, rows, x, nthreads=16)
        assert npref.rel_err(y[:, -rows:], want) < TOL, (m, n)
        _check_against_exact_arithmetic(Q6_K, raw, k, m, x, y, f"Q6_K {m}x{k} n={n}", max_rows=2048)
        assert ctx.route_q8(W, act) == "skinny_deep"
        assert np.array_equal(ctx.mulmat_q8(W, act), y), ("f32 != planes", m, n)
        assert np.array_equal(ctx.mulmat(W, x[::-1].copy())[::-1], y), n
    act.free()
    W.free()


@pytest.mark.parametrize("seed", [1, 2])
def test_deep_kernels_on_random_large_shapes(ctx, seed):
    """twelve seeded shapes per seed beyond 40 M weights -- K any multiple of 256 up to 16384, rows to match, 2..8
    columns, Q4_K and Q6_K in turn -- through the default routing: a slab of the first and of the last rows against the
    oracle, and where the deep kernels ran, the f32 form against quantize-then-multiply bit for bit"""
    rng = np.random.default_rng(9400 + seed)
    deep = 0
    for case in range(12):
        t = Q4_K if case % 2 == 0 else Q6_K
        k = 256 * int(rng.integers(2, 65))
        lo = (40 << 20) // k + 1
        m = int(rng.integers(lo, 3 * lo))
        n = int(rng.integers(2 if t == Q4_K else 3, 9))
        base = _weights(t, 512, k, seed=9401 + case)
        raw = np.ascontiguousarray(np.roll(np.tile(base.reshape(512, -1), (m // 512 + 1, 1))[:m], case, axis=0))
        W = ctx.upload(t, raw.reshape(-1), k, m)
        x = rng.standard_normal((n, k), dtype=np.float32)
        route = ctx.route(W, n)
        got = ctx.mulmat(W, x)
        for sl in (slice(0, 96), slice(m - 200, m)):
            want = oracle.mul_mat(t, np.ascontiguousarray(raw[sl]).reshape(-1), k, raw[sl].shape[0], x, nthreads=16)
            assert npref.rel_err(got[:, sl], want) < TOL, (NAMES[t], m, k, n, route)
        if route in ("skinny_deep", "deep_f32"):
            deep += 1
            act = ctx.act_create(Q8_K, k, n)
            ctx.act_quantize(act, x)
            assert np.array_equal(ctx.mulmat_q8(W, act), got), (NAMES[t], m, k, n, route)
            act.free()
        W.free()
    assert deep >= 8


@pytest.mark.parametrize("t,ms", [(Q4_K, [14336, 14336]), (Q4_K, [4096, 1024, 1024]), (Q4_K, [13824]), (Q6_K, [14336]), (Q4_K, [4100]),
                                  (Q4_K, [11008]), (Q6_K, [13830])])
def test_even_workgroup_plans_keep_the_bits(ctx, t, ms):
    """One and two f32 columns on rows of one K segment: the launch is planned with the same number of workgroups on
    every CU, their rows dealt out unevenly over the row groups (28672 rows: 512 workgroups of 56, some waves with four
    rows and some with three; several matrices in one launch keep within the even count).  A row's sum does not depend
    on the plan: the bits are those of the two-phase form, which is planned differently, and of each matrix alone;
    a slab of the last rows against the oracle."""
    k = 4096
    rng = np.random.default_rng(9500 + sum(ms) + t)
    raws = [_weights(t, m, k, seed=9501 + m + i) for i, m in enumerate(ms)]
    Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
    act = ctx.act_create(Q8_K, k, 2)
    for n in (1, 2):
        x = rng.standard_normal((n, k), dtype=np.float32)
        got = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        ctx.act_quantize(act, x)
        for y, W, raw, m in zip(got, Ws, raws, ms):
            if ctx.route(W, n) == "gemv_f32":
                assert np.array_equal(ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV), y), (m, n)
                assert np.array_equal(ctx.mulmat(W, x), y), (m, n)
            rows = min(m, 3000)
            want = oracle.mul_mat(t, np.ascontiguousarray(raw[-rows:]), k, rows, x, nthreads=16)
            assert npref.rel_err(y[:, -rows:], want) < TOL, (m, n)
    act.free()
    for W in Ws:
        W.free()


@pytest.mark.parametrize("t", WTYPES)
def test_in_kernel_quantization_gives_the_same_bits(ctx, t):
    """For n <= 8 the f32 entry points quantize x inside the GEMV's prologue.  The result must be
    bit-identical to quantizing with the stand-alone kernel (whose bytes are checked against the oracle
    above) and multiplying by the two-phase entry point -- i.e. the in-kernel quants are the same bits."""
    rng = np.random.default_rng(400 + t)
    blk = npref.BLOCK[t]
    ks = [blk, 4096, 14336] + ([2336, 96] if blk == 32 else [2304, 5120])   # 2336*n is not a multiple of 256
    for k in ks:
        ms = [37, 130]
        raws = [_weights(t, m, k, seed=k + m) for m in ms]
        Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
        act = ctx.act_create(qmm.vec_dot_type(t), k, 8)
        for n in (1, 2, 5, 8):
            x = rng.standard_normal((n, k), dtype=np.float32)
            x[0, : min(k, 256)] = 0.0                                 # an all-zero block
            ctx.act_quantize(act, x)
            want = [ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV) for W in Ws]
            for W, wnt in zip(Ws, want):
                assert np.array_equal(ctx.mulmat(W, x, path=qmm.PATH_GEMV), wnt), (k, n)
            got = ctx.mulmat_multi(Ws, x)
            for y, wnt in zip(got, want):
                assert np.array_equal(y, wnt), (k, n)
        # against the oracle as well, once per k
        x = rng.standard_normal((3, k), dtype=np.float32)
        got = ctx.mulmat_multi(Ws, x)
        for y, r, m in zip(got, raws, ms):
            assert npref.rel_err(y, oracle.mul_mat(t, r, k, m, x, nthreads=8)) <= TOL
        act.free()
        for W in Ws:
            W.free()


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
def test_in_kernel_q8_K_quantizer_edge_blocks_give_the_same_bits(ctx, t):
    """The decode prologue quantizes Q8_K blocks with sixteen lanes per block, the stand-alone kernel with a wave per
    block.  Blocks built to tell them apart: zeros; the same magnitude twice with opposite signs, first positive and
    first negative, in one lane's sixteen elements and lanes apart; the maximum in the very last element; huge and
    tiny magnitudes; products that land on .5; five blocks, so the last group of four is one block long."""
    k, m = 1280, 200
    w_raw = _weights(t, m, k, seed=91 + t)
    W = ctx.upload(t, w_raw, k, m)
    rng = np.random.default_rng(17)
    x = rng.standard_normal((2, k)).astype(np.float32)
    x[0, 0:256] = 0.0
    x[0, 256:512] *= 0.1; x[0, 256 + 7] = 3.0; x[0, 256 + 200] = -3.0
    x[0, 512:768] *= 0.1; x[0, 512 + 35] = -3.0; x[0, 512 + 36] = 3.0
    x[0, 768:1024] *= 0.1; x[0, 1023] = -2.5
    x[0, 1024:1280] = 1e-30; x[0, 1024 + 100] = 1e20
    x[1, 0:256] = np.arange(256, dtype=np.float32) - 127.5          # every product iscale * x a multiple of .5
    x[1, 256:512] = 0.0; x[1, 256 + 255] = -0.0
    x[1, 512:768] = 127.0; x[1, 512 + 16] = -127.0                   # first maximum positive, the other sign later
    x[1, 768:1024] = -1.0
    for n in (1, 2):
        act = ctx.act_create(Q8_K, k, n)
        ctx.act_quantize(act, x[:n])
        want = ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV)
        assert np.array_equal(ctx.mulmat(W, x[:n], path=qmm.PATH_GEMV), want), n
        assert np.all(np.isfinite(want))
        act.free()
    W.free()


@pytest.mark.parametrize("t,k", [(Q4_K, 14336), (Q4_K, 8192), (Q6_K, 4352), (Q4_0, 4096), (Q8_0, 4096), (Q8_0, 2080),
                                 (Q4_K, 5120), (Q6_K, 5120), (Q6_K, 14336), (Q4_0, 2560), (Q8_0, 5120),
                                 (Q4_K, 11008), (Q4_K, 8448), (Q6_K, 12544), (Q4_K, 16384), (Q6_K, 11008), (Q4_K, 28672)])
def test_long_rows_at_one_column(ctx, t, k):
    """One column, rows of several K segments (the waves of a workgroup cut K and combine through LDS): same
    bits as the two-phase path, call after call; row counts that do not fill the last workgroup, four
    weights in one launch, and the largest launch the f32 path takes (64 Ki rows).  The K-quant rows of three and four
    segments take the kernel whose waves wait for the other waves of their segment only (a count in LDS instead of a
    workgroup barrier) and whose last wave per row group adds the partial sums: last segments of one block (8448,
    12544), of eleven (11008), full ones (16384); 28672 is seven segments and two rounds of quantization."""
    rng = np.random.default_rng(900 + t + k)
    ms = [1, 31, 32, 33, 700]
    raws = [_weights(t, m, k, seed=k + m + t) for m in ms]
    Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
    act = ctx.act_create(qmm.vec_dot_type(t), k, 1)
    act3 = ctx.act_create(qmm.vec_dot_type(t), k, 3)
    for rep in range(3):
        x = rng.standard_normal((1, k), dtype=np.float32)
        ctx.act_quantize(act, x)
        want = [ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV) for W in Ws]
        for _ in range(3):
            for W, wnt in zip(Ws, want):
                assert np.array_equal(ctx.mulmat(W, x), wnt)
            for y, wnt in zip(ctx.mulmat_multi(Ws[1:], x), want[1:]):
                assert np.array_equal(y, wnt)
        assert npref.rel_err(want[4], oracle.mul_mat(t, raws[4], k, 700, x, nthreads=8)) <= TOL
        # the waves of a mostly empty last segment take rows side by side at one and two columns only: at three
        # columns every wave takes one row per load, and column 0 must come out with the same bits (not Q4_K: its
        # three-column products do not reproduce the one-column bits at any K, with or without a short last segment,
        # so they say nothing here; nor Q6_K rows short enough that three columns take the deep direct-load kernel)
        if t != Q4_K:
            x3 = np.concatenate([x, rng.standard_normal((2, k), dtype=np.float32)])
            ctx.act_quantize(act3, x3)
            assert t != Q6_K or (ctx.route_q8(Ws[4], act3) == "gemv") == (k > 10752)
            for W, wnt in zip(Ws, want):
                if t != Q6_K or ctx.route_q8(W, act3) == "gemv":
                    assert np.array_equal(ctx.mulmat_q8(W, act3, path=qmm.PATH_GEMV)[:1], wnt)
    act.free()
    act3.free()
    for W in Ws:
        W.free()
    if t == Q4_K and k == 8192:
        m = 65536
        raw = np.tile(_weights(t, 1024, k, seed=77).reshape(1024, -1), (m // 1024, 1)).reshape(-1)
        W = ctx.upload(t, raw, k, m)
        x = rng.standard_normal((1, k), dtype=np.float32)
        y = ctx.mulmat(W, x)
        assert np.array_equal(y[0, :1024], y[0, -1024:])                       # the rows repeat
        assert npref.rel_err(y[:, :1024], oracle.mul_mat(t, raw[: 1024 * qmm.row_size(t, k)], k, 1024, x, nthreads=8)) <= TOL
        W.free()


def test_results_do_not_depend_on_rows_per_wave(ctx):
    """A wave parks the totals of its rows in different lanes; every lane of the last 16 holds the wave
    total, but summed in a lane-dependent order.  The kernel must take one fixed lane's value, so that
    the same row gives the same bits whatever the launch geometry: a weight alone (2 rows per wave), as
    one of several tensors of a launch (4 rows per wave above 64 Ki rows in total) and with many columns
    (4 rows per wave)."""
    k = 1024
    rng = np.random.default_rng(5)
    raw = _weights(Q4_K, 48, k, seed=3)
    W = ctx.upload(Q4_K, raw, k, 48)
    big = ctx.upload(Q4_K, np.tile(_weights(Q4_K, 1024, k, seed=4).reshape(1024, -1), (66, 1)).reshape(-1), k, 67584)
    for n in (1, 4):
        x = rng.standard_normal((n, k), dtype=np.float32)
        act = ctx.act_create(Q8_K, k, 8)
        ctx.act_quantize(act, x)
        alone = ctx.mulmat_q8(W, act, path=qmm.PATH_GEMV)
        together = ctx.mulmat_q8_multi([big, W], act)[1]
        assert np.array_equal(alone, together), n
        assert np.array_equal(alone, ctx.mulmat(W, x, path=qmm.PATH_GEMV)), n
        act.free()
    W.free(); big.free()


def test_mulmat_multi_fallbacks_and_errors(ctx):
    k = 1024
    rng = np.random.default_rng(8)
    Ws = [ctx.upload(Q4_K, _weights(Q4_K, m, k, seed=m), k, m) for m in (40, 24, 8, 16, 32)]
    x = rng.standard_normal((12, k), dtype=np.float32)
    # five weights and twelve rows: falls back to one product per weight, same values
    got = ctx.mulmat_multi(Ws, x)
    for W, y in zip(Ws, got):
        assert np.array_equal(y, ctx.mulmat(W, x))
    W8 = ctx.upload(Q8_0, _weights(Q8_0, 8, k, seed=1), k, 8)
    got = ctx.mulmat_multi([Ws[0], W8], x[:1])                        # mixed types: per-weight products
    assert np.array_equal(got[0], ctx.mulmat(Ws[0], x[:1])) and np.array_equal(got[1], ctx.mulmat(W8, x[:1]))
    Wk = ctx.upload(Q4_K, _weights(Q4_K, 8, 2 * k, seed=2), 2 * k, 8)
    with pytest.raises(qmm.QmmError) as e:
        lib_ws = (ctypes.c_void_p * 2)(Ws[0]._h, Wk._h)                 # different k: rejected
        ys = [np.empty((1, 40), np.float32), np.empty((1, 8), np.float32)]
        yp = (ctypes.c_void_p * 2)(*[y.ctypes.data_as(ctypes.c_void_p) for y in ys])
        qmm._check(qmm.lib().mi_qmm_mulmat_multi(ctx._h, lib_ws, 2, x[:1].ctypes.data_as(ctypes.c_void_p), 1, yp,
                                                 qmm.HOST))
    assert e.value.code == qmm.ERR_INVALID
    for W in Ws + [W8, Wk]:
        W.free()


def test_randomized_shape_sweep(ctx):
    """seeded random (type, K, M, N) combinations through the default dispatch -- thin GEMV with and
    without in-kernel quantization, multi-segment rows, long-K kernel, column groups, GEMM tiles of
    both sizes, K slices -- against the oracle"""
    rng = np.random.default_rng(20240607)
    for case in range(28):
        t = int(rng.choice(WTYPES))
        blk = npref.BLOCK[t]
        k = int(rng.integers(1, 40 if blk == 256 else 160)) * blk
        if case % 7 == 3:
            k = int(rng.integers(33, 70)) * 256                       # long rows: several K segments, K slices
        m = int(rng.integers(1, 400))
        n = int(rng.choice([1, 1, 2, 3, 5, 8, 9, 17, 33, 64, 130]))
        w_raw = _weights(t, m, k, seed=case)
        W = ctx.upload(t, w_raw, k, m)
        x = rng.standard_normal((n, k), dtype=np.float32) * np.float32(rng.choice([1e-3, 1.0, 30.0]))
        got = ctx.mulmat(W, x)
        want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=8)
        err = npref.rel_err(got, want)
        assert got.shape == (n, m) and err <= TOL, f"case {case}: {NAMES[t]} k={k} m={m} n={n}: rel err {err}"
        W.free()


def test_randomized_shapes_through_the_large_matrix_kernels(ctx):
    """seeded random shapes where the kernels for large matrices take over: Q4_K on many rows at 3..16 columns, alone
    and several matrices in one call; Q6_K on 65536 rows and more at 2..8 columns; rows whose last K segment is at
    most half full at one and two columns (every format); two and three columns on large matrices -- against the
    oracle (weights tiled from 2048 encoded rows)"""
    rng = np.random.default_rng(20250131)

    def tiled(t, m, k, seed):
        base = min(m, 2048)
        return np.tile(_weights(t, base, k, seed).reshape(base, -1), ((m + base - 1) // base, 1))[:m].reshape(-1).copy()

    def check(t, ms, k, n, what):
        raws = [tiled(t, m, k, 7000 + i + m) for i, m in enumerate(ms)]
        Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
        x = rng.standard_normal((n, k), dtype=np.float32)
        got = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        for y, r, m in zip(got, raws, ms):
            err = npref.rel_err(y, oracle.mul_mat(t, r, k, m, x, nthreads=16))
            assert err <= TOL, f"{what}: {NAMES[t]} ms={ms} k={k} n={n}: rel err {err}"
        for W in Ws:
            W.free()

    for _ in range(3):
        ms = [int(rng.integers(9000, 30000)) for _ in range(int(rng.integers(1, 4)))]
        if sum((m + 15) // 16 for m in ms) < 1536:
            ms[0] += 26000
        check(Q4_K, ms, int(rng.choice([2048, 4096, 8192])), int(rng.integers(3, 17)), "many rows, Q4_K")
    for _ in range(2):
        check(Q6_K, [int(rng.integers(65536, 90000))], int(rng.choice([2048, 4096])), int(rng.integers(2, 9)), "many rows, Q6_K")
    for _ in range(8):
        t = int(rng.choice(WTYPES))
        blk, seg = (256, 4096) if t in (Q4_K, Q6_K) else (32, 2048)
        k = int(rng.integers(1, 5)) * seg + int(rng.integers(1, seg // blk // 2 + 1)) * blk
        check(t, [int(rng.integers(1, 6000))], k, int(rng.integers(1, 3)), "short last segment")
    for _ in range(4):
        t = int(rng.choice(WTYPES))
        check(t, [int(rng.integers(3000, 16000))], int(rng.choice([4096, 8192, 14336])), int(rng.integers(2, 4)), "two or three columns")


def test_randomized_products_through_every_route(ctx):
    """seeded random (type, rows, K, columns, number of matrices) over the whole range the entry points route on --
    one column to batch 512, a single block of K to 16384, one row to 40000, one to three matrices per call.  Every
    product against the oracle; and the three ways of asking for it give the same bits: several matrices in one
    call or one call each, f32 activations or activations quantized first (weights tiled from 1024 encoded rows)"""
    rng = np.random.default_rng(4242)
    cases = 0
    while cases < 70:
        t = int(rng.choice(WTYPES))
        blk = npref.BLOCK[t]
        kind = int(rng.integers(0, 3))
        k = (blk * int(rng.integers(1, 9)) if kind == 0 else
             int(rng.choice([2048, 4096, 5120, 8192, 11008 // blk * blk, 14336])) if kind == 1 else
             blk * int(rng.integers(1, 16384 // blk + 1)))
        n = int(rng.choice([1, 1, 2, 2, 3, 3, 4, 5, 6, 7, 8, 9, 12, 16, 17, 24, 31, 32, 33, 64, 65, 100, 128, 129, 200, 512]))
        ms = [int(np.exp(rng.uniform(0, np.log(40000))))]
        ms += [int(np.exp(rng.uniform(0, np.log(20000)))) for _ in range(int(rng.choice([0, 0, 0, 1, 2])))]
        while sum(ms) * k * n > 1.5e9 and n > 1:
            n = max(1, n // 2)
        if sum(ms) * k * n > 1.5e9:
            continue
        raws = []
        for i, m in enumerate(ms):
            base = min(m, 1024)
            w = _weights(t, base, k, 9000 + 7 * cases + i).reshape(base, -1)
            raws.append(np.concatenate([np.roll(w, j, axis=0) for j in range((m + base - 1) // base)], axis=0)[:m].reshape(-1).copy())
        Ws = [ctx.upload(t, r, k, m) for r, m in zip(raws, ms)]
        x = rng.standard_normal((n, k), dtype=np.float32) * np.float32(rng.choice([1.0, 1e-3, 30.0]))
        if rng.random() < 0.3:
            x[0, :blk] = 0.0
        what = f"{NAMES[t]} ms={ms} k={k} n={n}"
        joint = ctx.mulmat_multi(Ws, x) if len(Ws) > 1 else [ctx.mulmat(Ws[0], x)]
        single = [ctx.mulmat(W, x) for W in Ws]
        act = ctx.act_create(qmm.vec_dot_type(t), k, n)
        ctx.act_quantize(act, x)
        two_phase = [ctx.mulmat_q8(W, act) for W in Ws]
        for y, s1, s2, r, m in zip(joint, single, two_phase, raws, ms):
            err = npref.rel_err(y, oracle.mul_mat(t, r, k, m, x, nthreads=16))
            assert err <= TOL, f"{what}: rel err {err}"
            assert np.array_equal(y, s1), f"{what}: one call for several matrices and one call each differ"
            assert np.array_equal(s1, s2), f"{what}: f32 activations and activations quantized first differ"
        act.free()
        for W in Ws:
            W.free()
        cases += 1


def test_randomized_mulmat_id_sweep(ctx):
    """random types, expert counts, token counts, slots and activation rows per token across the decode, bucketed,
    matrix-core and expert-GEMM paths, against the oracle"""
    rng = np.random.default_rng(777)
    for case in range(36):
        t = int(rng.choice(WTYPES))
        blk = npref.BLOCK[t]
        k = int(rng.integers(1, 10 if blk == 256 else 60)) * blk
        m = int(rng.integers(1, 150))
        n_expert = int(rng.choice([1, 2, 5, 8, 16, 40]))
        n_used = int(rng.integers(1, min(n_expert, 8) + 1))
        tokens = int(rng.choice([1, 1, 2, 7, 20, 64, 150, 400]))
        b_cols = int(rng.choice([1, n_used]))
        wb = _weights(t, n_expert * m, k, seed=3000 + case)
        w = ctx.upload(t, wb, k, n_expert * m)
        b = rng.standard_normal((tokens, b_cols, k), dtype=np.float32)
        ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
        got = ctx.mulmat_id(w, n_expert, b, ids)
        want = oracle.mul_mat_id(t, wb, k, m, n_expert, b, ids)
        err = npref.rel_err(got, want)
        assert got.shape == (tokens, n_used, m) and err <= TOL, \
            f"case {case}: {NAMES[t]} k={k} m={m} E={n_expert} used={n_used} tokens={tokens} b_cols={b_cols}: {err}"
        w.free()


# ---- kernel 3: int8-MFMA GEMM ---------------------------------------------------------------------
@pytest.mark.parametrize("t", [Q4_K, Q6_K])
@pytest.mark.parametrize("k,m,n", [(256, 1, 1), (256, 32, 32), (512, 31, 33), (1024, 128, 128), (1024, 257, 200),
                                   (4096, 160, 65), (2304, 100, 7), (14336, 64, 40)])
def test_gemm_small_and_ragged_shapes(ctx, t, k, m, n):
    w_raw = _weights(t, m, k, seed=k + 7 * m + t)
    W = ctx.upload(t, w_raw, k, m)
    x = np.random.default_rng(k + n).standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(W, x, path=qmm.PATH_GEMM)
    want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=16)
    err = npref.rel_err(got, want)
    assert err <= TOL, f"{NAMES[t]} k={k} m={m} n={n}: rel err {err}"
    # the GEMV computes the same integers; only fp32 summation order differs
    assert npref.rel_err(got, ctx.mulmat(W, x, path=qmm.PATH_GEMV)) <= TOL
    W.free()


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
def test_gemm_random_block_bytes(ctx, t):
    """every nibble / 6-bit scale / high-bit / int8-scale pattern, incl. negative Q6_K scales"""
    rng = np.random.default_rng(4321 + t)
    k, m, n = 1024, 96, 48
    nb = m * k // 256
    raw = rng.integers(0, 256, (nb, npref.BYTES[t]), dtype=np.uint8)
    hbytes = np.abs(rng.standard_normal(nb * 2) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    if t == Q4_K:
        raw[:, 0:4] = hbytes
    else:
        raw[:, 208:210] = hbytes[:, 0:2]
    W = ctx.upload(t, raw.reshape(-1), k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(W, x, path=qmm.PATH_GEMM)
    want = oracle.mul_mat(t, raw.reshape(-1), k, m, x, nthreads=16)
    assert npref.rel_err(got, want) <= TOL
    W.free()


@pytest.mark.parametrize("name,t,m,k", [("q_proj", Q4_K, 4096, 4096), ("k_proj", Q4_K, 1024, 4096),
                                        ("ffn_gate", Q4_K, 14336, 4096), ("ffn_down", Q6_K, 4096, 14336)])
def test_config5_prefill_layer_batch512(ctx, name, t, m, k):
    """the Llama-3-8B-shaped layer of the prefill configuration at batch 512 (o = q shape, v = k shape,
    up = gate shape)"""
    w_raw = _weights(t, m, k, seed=1005 + m % 97)
    W = ctx.upload(t, w_raw, k, m)
    x = np.random.default_rng(2005).standard_normal((512, k), dtype=np.float32)
    got = ctx.mulmat(W, x)  # AUTO -> GEMM at n = 512
    want = oracle.mul_mat(t, w_raw, k, m, x, nthreads=16)
    err = npref.rel_err(got, want)
    nrm = float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
    assert err <= TOL and nrm <= 1e-5, f"{name}: rel err {err}, normwise {nrm}"
    _check_against_exact_arithmetic(t, w_raw, k, m, x, got, name, max_rows=4096)
    W.free()


# ---- kernel 3b: fp16-MFMA GEMM (Q4_K products with at least 192 output tiles of 256 x 128) ---------------------
@pytest.mark.parametrize("k,m,n", [(256, 6200, 1000), (512, 12300, 500), (1024, 3000, 2050), (2304, 49 * 256, 385),
                                   (4096, 14336, 512), (512, 49300, 70)])
def test_f16_gemm_ragged_shapes(ctx, k, m, n):
    """one super-block per row, rows and batches that end inside a tile, the gate shape, one tile column; through the one-call form
    and through an activation handle (same planes, same kernel, same bits)"""
    w_raw = _weights(Q4_K, m, k, seed=3 * k + m)
    W = ctx.upload(Q4_K, w_raw, k, m)
    x = np.random.default_rng(k + n).standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(W, x)
    rows = slice(0, m) if m * n * k <= 6200 * 1000 * 512 else np.r_[0:300, m // 2 - 150:m // 2 + 150, m - 300:m]
    sub = w_raw if isinstance(rows, slice) else np.ascontiguousarray(w_raw.reshape(m, -1)[rows]).reshape(-1)
    msub = m if isinstance(rows, slice) else len(rows)
    want = oracle.mul_mat(Q4_K, sub, k, msub, x, nthreads=16)
    err = npref.rel_err(got[:, rows], want)
    assert err <= TOL, f"k={k} m={m} n={n}: rel err {err}"
    # the int8 kernel computes the same integers
    assert npref.rel_err(got, ctx.mulmat(W, x, path=qmm.PATH_GEMM)) <= 1e-4
    act = ctx.act_create(Q8_K, k, n)
    ctx.act_quantize(act, x)
    assert np.array_equal(ctx.mulmat_q8(W, act), got)
    act.free()
    W.free()


def test_f16_gemm_random_block_bytes(ctx):
    """every nibble, 6-bit scale and 6-bit min pattern; activations that quantize to the extremes -127 and 127"""
    rng = np.random.default_rng(8642)
    k, m, n = 768, 6400, 1024
    nb = m * k // 256
    raw = rng.integers(0, 256, (nb, 144), dtype=np.uint8)
    raw[:, 0:4] = np.abs(rng.standard_normal(nb * 2) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    W = ctx.upload(Q4_K, raw.reshape(-1), k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    x[5] = np.where(rng.random(k) < 0.5, -3.0, 3.0)  # a row of +-max: every quant +-127
    x[6] = 0.0
    got = ctx.mulmat(W, x)
    want = oracle.mul_mat(Q4_K, raw.reshape(-1), k, m, x, nthreads=16)
    assert npref.rel_err(got, want) <= TOL
    assert not got[6].any()
    W.free()


def test_f16_gemm_largest_block_sums_stay_exact(ctx):
    """All scales 63, all nibbles 15, all activations equal: the super-block sums are the largest the format allows
    (63 * 15 * 127 * 256 > 2^24).  The result must still agree with exact arithmetic to fp32 rounding."""
    k, m, n = 512, 6400, 1024
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([2.0 ** -10], dtype=np.float16).view(np.uint8)   # d
    blk[2:4] = np.array([2.0 ** -12], dtype=np.float16).view(np.uint8)   # dmin
    blk[4:16] = 0xFF                                                     # scales and mins all 63
    blk[16:] = 0xFF
    raw = np.tile(blk, m * k // 256)
    W = ctx.upload(Q4_K, raw, k, m)
    x = np.ones((n, k), dtype=np.float32)
    x[1::2] = -1.0
    got = ctx.mulmat(W, x)
    # every quant is 127 (or -127) with d = 1/127 (or -1/127): per super-block d*63*15*127*256 - dmin*63*127*256
    per_sb = 2.0 ** -10 * 63 * 15 * 127 * 256 - 2.0 ** -12 * 63 * 127 * 256
    want = np.full((n, m), 2 * per_sb / 127.0)
    want[1::2] *= -1.0
    assert np.max(np.abs(got / want - 1.0)) <= 1e-6
    W.free()


# ---- kernel 3c: Q6_K GEMM with 256 x 128 tiles, one accumulator per tile, K slices -------------------------------
@pytest.mark.parametrize("k,m,n", [(1024, 6200, 1000), (4096, 3000, 600), (3328, 5000, 512), (14336, 4096, 512),
                                   (256 * 4, 128256, 512), (1024, 50000, 100)])
def test_q6k_gemm_tiles_and_slices(ctx, k, m, n):
    """no slices and ragged tiles; four slices; three uneven slices (4, 4 and 5 super-blocks); the ffn_down shape;
    the output head's rows; a batch that fills most of one 128-row tile column; one-call form == activation-handle form"""
    w_raw = _weights(Q6_K, m, k, seed=5 * k + m)
    W = ctx.upload(Q6_K, w_raw, k, m)
    x = np.random.default_rng(k + n + 1).standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(W, x)
    rows = slice(0, m) if m * n * k <= 6200 * 1000 * 1024 else np.r_[0:300, m // 2 - 150:m // 2 + 150, m - 300:m]
    sub = w_raw if isinstance(rows, slice) else np.ascontiguousarray(w_raw.reshape(m, -1)[rows]).reshape(-1)
    msub = m if isinstance(rows, slice) else len(rows)
    want = oracle.mul_mat(Q6_K, sub, k, msub, x, nthreads=16)
    err = npref.rel_err(got[:, rows], want)
    assert err <= TOL, f"k={k} m={m} n={n}: rel err {err}"
    assert npref.rel_err(got, ctx.mulmat(W, x, path=qmm.PATH_GEMM)) <= 1e-4  # the 128-row kernel: same integers, other fp32 order
    act = ctx.act_create(Q8_K, k, n)
    ctx.act_quantize(act, x)
    assert np.array_equal(ctx.mulmat_q8(W, act), got)
    act.free()
    W.free()


@pytest.mark.parametrize("ms,ns", [((4096, 1024, 1000), (1024, 1100, 512)), ((6144, 6400), (1024, 700))])
def test_fp16_gemm_takes_q_k_v_in_one_launch(ctx, ms, ns):
    """q, k and v of an attention block from batch 1024: too few 256-row tiles each (k and v: 4 x 8), enough together,
    so the multi entry points launch the fp16 kernel once over all three.  The bits are those of the single products
    (k and v alone run on the int8 kernel: same exact integer sums, same fp32 expressions), checked against the
    oracle on a sample; a batch too small for the joint launch (512) and a ragged one keep the rule too.  Second set: two
    matrices that each take the fp16 kernel alone (gate and up of a feed-forward block) in one launch."""
    k = 4096
    raws = [_weights(Q4_K, m, k, seed=880 + i) for i, m in enumerate(ms)]
    Ws = [ctx.upload(Q4_K, r, k, m) for r, m in zip(raws, ms)]
    rng = np.random.default_rng(88)
    try:
        for n in ns:
            x = rng.standard_normal((n, k), dtype=np.float32)
            act = ctx.act_create(Q8_K, k, n)
            ctx.act_quantize(act, x)
            alone = [ctx.mulmat_q8(W, act) for W in Ws]
            for got in (ctx.mulmat_q8_multi(Ws, act), ctx.mulmat_multi(Ws, x)):
                for y, wnt in zip(got, alone):
                    assert np.array_equal(y, wnt), n
            act.free()
            for raw, m, y in zip(raws, ms, alone):
                want = oracle.mul_mat(Q4_K, raw[-200:], k, 200, x[-24:], nthreads=16)
                assert npref.rel_err(y[-24:, -200:], want) < TOL
    finally:
        for W in Ws:
            W.free()


def test_gemm_k_slices_into_a_y_that_is_not_16_byte_aligned(ctx):
    """Products cut into K slices add their partial planes into the caller's y.  A device caller may pass y at any
    4-byte offset into a larger tensor: the sum then goes element by element, in the same slice order -- the bits of the
    aligned call.  ffn_down at batch 512 (Q6_K: four slices on the 256-row kernel) and a Q4_K product with few tiles and
    a long K (slices on the 128-row kernel)."""
    from hipmem import DeviceArray
    rng = np.random.default_rng(77)
    for t, m, k, n in ((Q6_K, 4096, 14336, 512), (Q4_K, 1024, 16384, 128)):
        raw = _weights(t, 512, k, seed=770 + t)
        raw = np.tile(raw, (m // 512, 1))
        W = ctx.upload(t, raw, k, m)
        x = rng.standard_normal((n, k), dtype=np.float32)
        dx = DeviceArray(x)
        buf = DeviceArray(np.empty(n * m + 8, np.float32), zero=True)
        try:
            ctx.mulmat_device(W, dx.ptr, n, buf.ptr)
            ctx.sync()
            aligned = buf.numpy()[: n * m].copy()
            ctx.mulmat_device(W, dx.ptr, n, buf.ptr + 4)
            ctx.sync()
            assert np.array_equal(buf.numpy()[1 : n * m + 1], aligned), NAMES[t]
            want = oracle.mul_mat(t, raw[:256], k, 256, x[:16], nthreads=16)
            assert npref.rel_err(aligned.reshape(n, m)[:16, :256], want) < TOL
        finally:
            dx.free(); buf.free(); W.free()


def test_q6k_gemm_random_block_bytes(ctx):
    """every ql / qh bit pattern and every int8 scale, negative ones and -128 included"""
    rng = np.random.default_rng(9753)
    k, m, n = 1024, 6400, 1024
    nb = m * k // 256
    raw = rng.integers(0, 256, (nb, 210), dtype=np.uint8)
    raw[:, 208:210] = np.abs(rng.standard_normal(nb) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
    raw[::7, 192] = 0x80  # scale -128
    W = ctx.upload(Q6_K, raw.reshape(-1), k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    x[5] = np.where(rng.random(k) < 0.5, -3.0, 3.0)
    got = ctx.mulmat(W, x)
    want = oracle.mul_mat(Q6_K, raw.reshape(-1), k, m, x, nthreads=16)
    assert npref.rel_err(got, want) <= TOL
    W.free()


def test_q6k_gemm_extreme_products_stay_exact(ctx):
    """all scales -128, all 6-bit values 0 (= -32), all activations equal: every product is the largest the format
    allows (+4096 * 127) and the super-block sums reach 256 * 4096 * 127 = 2^27; both digits and the shift carry it"""
    k, m, n = 512, 6400, 1024
    blk = np.zeros(210, dtype=np.uint8)
    blk[192:208] = 0x80
    blk[208:210] = np.array([2.0 ** -14], dtype=np.float16).view(np.uint8)
    raw = np.tile(blk, m * k // 256)
    W = ctx.upload(Q6_K, raw, k, m)
    x = np.ones((n, k), dtype=np.float32)
    x[1::2] = -1.0
    got = ctx.mulmat(W, x)
    # x = 1 quantizes to -127 with d = -1/127 (x = -1: -127 with d = 1/127): per super-block 2^-14 * 4096 * 256 = 64
    want = np.full((n, m), 2 * 64.0)
    want[1::2] *= -1.0
    assert np.max(np.abs(got / want - 1.0)) <= 1e-6
    W.free()


# ---- expert-indexed product (Tensor.MulmatID) ------------------------------------------------------
def _experts(t, n_expert, m, k, seed):
    return _weights(t, n_expert * m, k, seed)


@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("tokens,n_used,b_cols", [(1, 8, 1), (1, 8, 8), (2, 4, 4), (40, 4, 1), (33, 6, 6), (7, 5, 2)])
def test_mulmat_id_matches_oracle(ctx, t, tokens, n_used, b_cols):
    """decode (one pair per group, straight from ids) and batches (pairs bucketed by expert)"""
    rng = np.random.default_rng(7000 + t * 131 + tokens * 7 + n_used + b_cols)
    k, m, n_expert = 1024, 200, 12
    wb = _experts(t, n_expert, m, k, 7100 + t)
    w = ctx.upload(t, wb, k, n_expert * m)
    b = rng.standard_normal((tokens, b_cols, k), dtype=np.float32)
    ids = rng.integers(0, n_expert, (tokens, n_used)).astype(np.int32)
    got = ctx.mulmat_id(w, n_expert, b, ids)
    want = oracle.mul_mat_id(t, wb, k, m, n_expert, b, ids)
    assert got.shape == want.shape
    assert npref.rel_err(got, want) < TOL
    w.free()


@pytest.mark.parametrize("t,tokens", [(Q4_K, 3), (Q8_0, 3), (Q8_0, 24), (Q4_0, 24)])
def test_mulmat_id_equals_mulmat_on_the_expert_alone(ctx, t, tokens):
    """the streaming kernels (decode: one pair per group; Q4_0 / Q8_0 batches whose K is no multiple of 256:
    pairs bucketed by expert) give bit for bit what the plain one-column product gives on that expert's
    slice, whatever group a pair lands in"""
    rng = np.random.default_rng(7200 + t + tokens)
    k, m, n_expert, n_used = (2048 if tokens < 8 else 2080), 96, 6, 3
    wb = _experts(t, n_expert, m, k, 7201 + t)
    w = ctx.upload(t, wb, k, n_expert * m)
    b = rng.standard_normal((tokens, 1, k), dtype=np.float32)
    ids = rng.integers(0, n_expert, (tokens, n_used)).astype(np.int32)
    got = ctx.mulmat_id(w, n_expert, b, ids)
    w3 = wb.reshape(n_expert, m, -1)
    for e in range(n_expert):
        we = ctx.upload(t, w3[e], k, m)
        for ti, i in np.argwhere(ids == e):
            assert np.array_equal(got[ti, i], ctx.mulmat(we, b[ti, 0])[0])  # the decode GEMV, one column
        we.free()
    w.free()


def test_mulmat_id_on_the_matrix_cores(ctx):
    """K-quants from about two pairs per expert up (Q4_0 / Q8_0 with K a multiple of 256: from four): groups of
    16 pairs through the MFMA kernels; ragged expert height, experts that nobody picked, one expert picked by
    more than 16 pairs, ids outside the stack among device ids"""
    rng = np.random.default_rng(7250)
    for t, k, m, n_expert, tokens, n_used, b_cols in ((Q4_K, 1024, 72, 5, 40, 2, 1), (Q6_K, 512, 200, 9, 30, 4, 4),
                                                      (Q4_K, 2048, 33, 3, 64, 2, 2), (Q4_0, 1024, 72, 5, 40, 2, 1),
                                                      (Q8_0, 512, 200, 6, 30, 4, 4), (Q8_0, 256, 17, 3, 200, 2, 2),
                                                      (Q4_0, 2304, 50, 4, 33, 3, 1)):
        wb = _experts(t, n_expert, m, k, 7251 + t)
        w = ctx.upload(t, wb, k, n_expert * m)
        b = rng.standard_normal((tokens, b_cols, k), dtype=np.float32)
        ids = rng.integers(0, n_expert - 1, (tokens, n_used)).astype(np.int32)  # the last expert stays idle
        ids[: tokens // 2, 0] = 1                                                # a crowd on expert 1
        got = ctx.mulmat_id(w, n_expert, b, ids)
        assert npref.rel_err(got, oracle.mul_mat_id(t, wb, k, m, n_expert, b, ids)) < TOL
        # a pair's result does not depend on the other pairs of the call: same call, order of tokens reversed
        assert np.array_equal(ctx.mulmat_id(w, n_expert, b[::-1], ids[::-1])[::-1], got)
        bad = ids.copy()
        bad[0, 0] = n_expert
        bad[-1, -1] = -1
        db, dids = DeviceArray(b), DeviceArray(bad)
        dy = DeviceArray(np.zeros((tokens, n_used, m), np.float32), zero=True)
        ctx.mulmat_id_device(w, n_expert, db.ptr, b_cols, dids.ptr, n_used, tokens, dy.ptr)
        ctx.sync()
        out = dy.numpy()
        isbad = (bad < 0) | (bad >= n_expert)
        assert np.isnan(out[isbad]).all() and np.array_equal(out[~isbad], got[~isbad])
        for d in (db, dids, dy):
            d.free()
        w.free()


def test_mulmat_id_moe_decode_shape(ctx):
    """Qwen3-30B-A3B-like expert FFN: 128 experts, 8 used, gate 768x2048 then down 2048x768"""
    rng = np.random.default_rng(7300)
    n_expert, n_used = 128, 8
    for k, m, b_cols in ((2048, 768, 1), (768, 2048, 8)):
        wb = _experts(Q4_K, n_expert, m, k, 7301 + k)
        w = ctx.upload(Q4_K, wb, k, n_expert * m)
        b = rng.standard_normal((1, b_cols, k), dtype=np.float32)
        ids = rng.choice(n_expert, n_used, replace=False).astype(np.int32)[None, :]
        got = ctx.mulmat_id(w, n_expert, b, ids)
        assert npref.rel_err(got, oracle.mul_mat_id(Q4_K, wb, k, m, n_expert, b, ids)) < TOL
        w.free()


@pytest.mark.parametrize("t,n_expert,n_used,m,k", [
    (Q4_K, 8, 2, 4096, 14336),   # Mixtral-like down experts: rows of four segments, one workgroup per CU
    (Q4_K, 8, 2, 3000, 4096),    # rows of one segment, sixteen waves, a ragged last workgroup per expert
    (Q8_0, 6, 4, 2880, 2880),    # three segments, twelve waves
    (Q4_0, 6, 4, 2885, 2880),    # an odd number of rows per expert
    (Q6_K, 16, 4, 700, 2048),    # few rows: the eight-wave plan
])
def test_mulmat_id_decode_plans_on_large_experts(ctx, t, n_expert, n_used, m, k):
    """one and two tokens through experts large enough for every workgroup shape of the decode kernel: against the
    oracle on the last rows of each expert, and whole outputs against the plain product on the expert alone (1e-5)"""
    print(f"mulmat_id plan case t={t} experts={n_expert} m={m} k={k}", flush=True)
    rng = np.random.default_rng(7400 + m + k)
    rows = min(m, 512)
    base = _weights(t, rows, k, 7401 + t)
    one = np.tile(base, ((m + rows - 1) // rows, 1))[:m]
    wb = np.concatenate([np.roll(one, 5 * e, axis=0) for e in range(n_expert)])
    w = ctx.upload(t, wb, k, n_expert * m)
    try:
        for tokens in (1, 2):
            b = rng.standard_normal((tokens, 1, k), dtype=np.float32)
            ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
            got = ctx.mulmat_id(w, n_expert, b, ids)
            assert got.shape == (tokens, n_used, m)
            for tok in range(tokens):
                for slot in range(n_used):
                    e = int(ids[tok, slot])
                    ex = np.ascontiguousarray(wb[e * m:(e + 1) * m])
                    lo = m - 40  # the last rows of the expert: the ragged end of its last workgroup
                    want = oracle.mul_mat(t, np.ascontiguousarray(ex[lo:]), k, m - lo, b[tok], nthreads=4)
                    assert npref.rel_err(got[tok, slot, lo:][None, :], want) < TOL
                    if tok == 0 and slot < 2:
                        we = ctx.upload(t, ex, k, m)
                        assert npref.rel_err(got[tok, slot][None, :], ctx.mulmat(we, b[tok])) < 1e-5
                        we.free()
    finally:
        w.free()


def test_mulmat_id_device_ids_out_of_range_give_nan_host_ids_are_rejected(ctx):
    rng = np.random.default_rng(7400)
    k, m, n_expert = 512, 40, 4
    wb = _experts(Q8_0, n_expert, m, k, 7401)
    w = ctx.upload(Q8_0, wb, k, n_expert * m)
    for tokens in (1, 30):  # both the direct and the bucketed launch
        b = rng.standard_normal((tokens, 1, k), dtype=np.float32)
        ids = rng.integers(0, n_expert, (tokens, 2)).astype(np.int32)
        bad = ids.copy()
        bad[0, 1] = n_expert
        bad[-1, 0] = -1
        with pytest.raises(qmm.QmmError) as e:
            ctx.mulmat_id(w, n_expert, b, bad)
        assert e.value.code == qmm.ERR_INVALID
        db, dids = DeviceArray(b), DeviceArray(bad)
        dy = DeviceArray(np.zeros((tokens, 2, m), np.float32), zero=True)
        ctx.mulmat_id_device(w, n_expert, db.ptr, 1, dids.ptr, 2, tokens, dy.ptr)
        ctx.sync()
        got = dy.numpy()
        for d in (db, dids, dy):
            d.free()
        want = oracle.mul_mat_id(Q8_0, wb, k, m, n_expert, b, ids)
        isbad = (bad < 0) | (bad >= n_expert)
        assert np.isnan(got[isbad]).all()
        assert not np.isnan(got[~isbad]).any()
        assert npref.rel_err(got[~isbad], want[~isbad]) < TOL
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_id(w, 3, np.zeros((1, 1, k), np.float32), np.zeros((1, 1), np.int32))  # 160 rows / 3 experts
    assert e.value.code == qmm.ERR_INVALID
    assert ctx.mulmat_id(w, n_expert, np.zeros((0, 1, k), np.float32), np.zeros((0, 2), np.int32)).shape == (0, 2, m)
    w.free()


# ---- device pointers in and out ----------------------------------------------------------------------
@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("n", [1, 6, 48])
def test_device_pointers_give_the_same_bits_as_host_arrays(ctx, t, n):
    """MI_QMM_DEVICE: x and y stay on the device and the call only queues work on the ctx's stream"""
    rng = np.random.default_rng(7500 + t + n)
    k, m = 1024, 384
    wb = _weights(t, m, k, 7501 + t)
    wb2 = _weights(t, 128, k, 7502 + t)
    w, w2 = ctx.upload(t, wb, k, m), ctx.upload(t, wb2, k, 128)
    x = rng.standard_normal((n, k), dtype=np.float32)
    dx = DeviceArray(x)
    dy, dy2 = DeviceArray(np.zeros((n, m), np.float32), zero=True), DeviceArray(np.zeros((n, 128), np.float32), zero=True)
    ctx.mulmat_device(w, dx.ptr, n, dy.ptr)
    ctx.sync()
    assert np.array_equal(dy.numpy(), ctx.mulmat(w, x))
    for d in (dy, dy2):
        d.free()
    dy, dy2 = DeviceArray(np.zeros((n, m), np.float32), zero=True), DeviceArray(np.zeros((n, 128), np.float32), zero=True)
    ctx.mulmat_multi_device([w, w2], dx.ptr, n, [dy.ptr, dy2.ptr])
    ctx.sync()
    h, h2 = ctx.mulmat_multi([w, w2], x)
    assert np.array_equal(dy.numpy(), h) and np.array_equal(dy2.numpy(), h2)
    for d in (dx, dy, dy2):
        d.free()
    w.free()
    w2.free()


# ---- MFMA GEMM for the 32-element block formats -----------------------------------------------------
@pytest.mark.parametrize("t", [Q4_0, Q8_0])
@pytest.mark.parametrize("m,k,n", [(4096, 4096, 64), (1000, 1056, 70), (33, 32, 32), (257, 8192, 129), (64, 96, 1),
                                   (2, 2048, 200)])
def test_block32_gemm_matches_oracle(ctx, t, m, k, n):
    """full tiles; ragged M (also not a multiple of 4), N and a K of 33 blocks; one block; K cut between
    eight waves; one column and two rows through the forced GEMM path"""
    rng = np.random.default_rng(7600 + t + m + n)
    wb = _weights(t, m, k, 7601 + t + m)
    w = ctx.upload(t, wb, k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(w, x, path=qmm.PATH_GEMM)
    want = oracle.mul_mat(t, wb, k, m, x, nthreads=16)
    assert npref.rel_err(got, want) < TOL
    if n >= 32:
        assert np.array_equal(got, ctx.mulmat(w, x))  # what the automatic choice runs from 32 columns up
    w.free()


def test_block32_gemm_exact_integer_case(ctx):
    """weights and activations whose products and sums are exact in fp32: any misplaced operand byte,
    nibble or scale shows as a wrong integer"""
    k, m, n = 256, 96, 64
    rng = np.random.default_rng(7700)
    for t in (Q4_0, Q8_0):
        lim = 7 if t == Q4_0 else 127
        wi = rng.integers(-lim, lim + 1, (m, k)).astype(np.float32)
        wi[:, ::32] = -8 if t == Q4_0 else 127  # pins every block's scale to exactly 1.0
        xi = rng.integers(-127, 128, (n, k)).astype(np.float32)
        xi[:, 1::32] = 127
        wb = oracle.quantize(t, wi)
        assert np.array_equal(oracle.dequantize(t, wb, k), wi)
        w = ctx.upload(t, wb, k, m)
        got = ctx.mulmat(w, xi, path=qmm.PATH_GEMM)
        assert np.array_equal(got, (xi.astype(np.float64) @ wi.astype(np.float64).T).astype(np.float32))
        w.free()


def test_page_locked_host_buffers(ctx):
    """x and y in memory from mi_qmm_host_alloc behave like any other host memory"""
    rng = np.random.default_rng(7800)
    k, m, n = 1024, 256, 3
    wb = _weights(Q4_K, m, k, 7801)
    w = ctx.upload(Q4_K, wb, k, m)
    x = ctx.host_array((n, k))
    x[:] = rng.standard_normal((n, k), dtype=np.float32)
    y = ctx.host_array((n, m))
    rc = qmm.lib().mi_qmm_mulmat(ctx._h, w._h, ctypes.c_void_p(x.ctypes.data), n, ctypes.c_void_p(y.ctypes.data), qmm.HOST)
    assert rc == 0
    assert np.array_equal(y, ctx.mulmat(w, np.array(x)))
    assert ctx.host_array((0, 4)).shape == (0, 4)
    w.free()


# ---- skinny product on the matrix cores for the K-quants: both kernels ------------------------------
@pytest.mark.parametrize("t", [Q4_K, Q6_K])
@pytest.mark.parametrize("m,k,n", [(4096, 4096, 3), (1000, 1024, 4), (17, 256, 4), (9, 256, 3), (300, 2304, 19), (64, 8192, 4),
                                   (4096, 14336, 4), (1000, 1024, 7), (2048, 768, 3), (4096, 14336, 20), (14336, 4096, 19)])
def test_skinny_kquants_match_oracle(ctx, t, m, k, n):
    """3..31 columns through the C ABI's default routing: Q4_K at three and four columns of a small matrix
    takes the kernel that loads weights straight into the MFMA operands (ragged M, a single super-block,
    K cut one to sixteen ways, a second launch that starts at column 16), a large one and more columns
    the staged kernel; at 19 and 20 columns of a large matrix the second launch, of columns 16.., is one of the deep
    direct-load kernel"""
    rng = np.random.default_rng(8100 + t + m + n)
    wb = _weights(t, m, k, 8101 + t + m)
    w = ctx.upload(t, wb, k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(w, x)
    assert npref.rel_err(got, oracle.mul_mat(t, wb, k, m, x, nthreads=16)) < TOL
    if n <= 16:  # one launch: a column's result does not depend on which other columns ride along
        assert np.array_equal(ctx.mulmat(w, x[::-1].copy())[::-1], got)
    w.free()


@pytest.mark.parametrize("m,k,n", [(70003, 2048, 3), (66000, 4096, 8), (65617, 4096, 5), (65536, 2048, 8)])
def test_q6k_many_rows_few_columns(ctx, m, k, n):
    """Q6_K with 65536 rows and more, K of 2048 or 4096 and 3..8 columns (the output head at a few tokens) takes a
    kernel of its own: activations resident in LDS, a row group's scales fetched in whole lines.  Ragged last row
    group, both K sizes, every column set partly filled; a column's bits do not depend on the others, and are those
    the general kernel gives the column among sixteen."""
    rng = np.random.default_rng(8300 + m + n)
    wb = _weights(Q6_K, m, k, 8301 + m)
    w = ctx.upload(Q6_K, wb, k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(w, x)
    want = oracle.mul_mat(Q6_K, wb, k, m, x, nthreads=16)
    assert npref.rel_err(got, want) < TOL
    _check_against_exact_arithmetic(Q6_K, wb, k, m, x, got, f"Q6_K {m}x{k} n={n}", max_rows=4096)
    assert np.array_equal(ctx.mulmat(w, x[::-1].copy())[::-1], got)
    # the same columns among sixteen go through the general kernel (one wave per row group at this many rows: K uncut)
    x16 = np.concatenate([x, rng.standard_normal((16 - n, k), dtype=np.float32)])
    assert ctx.route(w, 16) == "skinny_staged"
    assert np.array_equal(ctx.mulmat(w, x16)[:n], got)
    w.free()


@pytest.mark.parametrize("n", [3, 4, 6])
def test_skinny_q4k_random_block_bytes(ctx, n):
    """random block bytes reach every bit pattern of nibbles and of the 6-bit scales and mins; compared
    with exact arithmetic on the quantized activations as well as with the oracle"""
    rng = np.random.default_rng(8200 + n)
    k, m = 2048, 40
    nb = m * k // 256
    raw = rng.integers(0, 256, (nb, 144), dtype=np.uint8)
    raw[:, 0:4] = np.abs(rng.standard_normal(nb * 2) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    W = ctx.upload(Q4_K, raw.reshape(-1), k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(W, x)
    assert npref.rel_err(got, oracle.mul_mat(Q4_K, raw.reshape(-1), k, m, x, nthreads=8)) <= TOL
    xq = oracle.quantize(Q8_K, x)
    assert npref.rel_err(got, npref.matmul_f64(Q4_K, raw.reshape(-1), k, m, Q8_K, xq, n)) <= TOL
    W.free()


# ---- skinny product on the matrix cores for the 32-element block formats ------------------------------
@pytest.mark.parametrize("t", [Q4_0, Q8_0])
@pytest.mark.parametrize("m,k,n", [(4096, 4096, 8), (1000, 1024, 5), (17, 256, 4), (300, 2304, 16), (64, 8192, 31),
                                   (4096, 14336, 7), (300, 14336, 2), (129, 9216, 3)])
def test_skinny32_matches_oracle(ctx, t, m, k, n):
    """4..31 columns, K a multiple of 256: ragged M, one 256-element step, K cut eight ways, two launches; rows
    longer than 8192 take this kernel from two columns"""
    rng = np.random.default_rng(7900 + t + m + n)
    wb = _weights(t, m, k, 7901 + t + m)
    w = ctx.upload(t, wb, k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(w, x)
    assert npref.rel_err(got, oracle.mul_mat(t, wb, k, m, x, nthreads=16)) < TOL
    # a column's result does not depend on which other columns ride along
    assert np.array_equal(ctx.mulmat(w, x[::-1].copy())[::-1], got)
    w.free()


@pytest.mark.parametrize("t,m,k,n", [(Q4_K, 14336, 4096, 2), (Q4_K, 4096, 14336, 2), (Q6_K, 4096, 14336, 2),
                                     (Q6_K, 4096, 14336, 3), (Q8_0, 14336, 4096, 3), (Q4_0, 14336, 4096, 2),
                                     (Q8_0, 4096, 14336, 2), (Q4_0, 4096, 14336, 3)])
def test_two_and_three_columns_on_large_matrices(ctx, t, m, k, n):
    """Two and three columns at the feed-forward shapes, through the default routing: the streaming kernel with the
    quantization of all columns in its prologue (K-quants at two columns, Q6_K at three from 32 MB, Q4_0 / Q8_0 with
    rows up to 8192), the matrix-core kernel for long rows of Q4_0 / Q8_0.  Against the oracle and, at the tighter
    floor, against exact arithmetic on the same quantized operands."""
    rng = np.random.default_rng(8500 + t + m + n)
    wb = _weights(t, m, k, 8501 + t + m)
    w = ctx.upload(t, wb, k, m)
    x = rng.standard_normal((n, k), dtype=np.float32)
    got = ctx.mulmat(w, x)
    assert npref.rel_err(got, oracle.mul_mat(t, wb, k, m, x, nthreads=16)) < TOL
    _check_against_exact_arithmetic(t, wb, k, m, x, got, f"{NAMES[t]} {m}x{k} n={n}", max_rows=2048)
    assert np.array_equal(ctx.mulmat(w, x[::-1].copy())[::-1], got)
    w.free()


def test_skinny32_exact_integer_case(ctx):
    """operands whose products and sums are exact in fp32: a misplaced byte, nibble, block sum or scale
    shows as a wrong integer"""
    k, m, n = 512, 48, 6
    rng = np.random.default_rng(7950)
    for t in (Q4_0, Q8_0):
        lim = 7 if t == Q4_0 else 127
        wi = rng.integers(-lim, lim + 1, (m, k)).astype(np.float32)
        wi[:, ::32] = -8 if t == Q4_0 else 127  # pins every block's scale to exactly 1.0
        xi = rng.integers(-127, 128, (n, k)).astype(np.float32)
        xi[:, 1::32] = 127
        wb = oracle.quantize(t, wi)
        w = ctx.upload(t, wb, k, m)
        got = ctx.mulmat(w, xi)
        assert np.array_equal(got, (xi.astype(np.float64) @ wi.astype(np.float64).T).astype(np.float32))
        w.free()


@pytest.mark.parametrize("t,tokens", [(Q4_K, 1), (Q8_0, 2), (Q4_K, 40), (Q4_0, 64)])
def test_mulmat_id_multi_equals_single_calls(ctx, t, tokens):
    """gate and up of an expert FFN in one call (decode: one launch) give the bits of two single calls;
    a third stack of another shape rides along on its own"""
    rng = np.random.default_rng(8000 + t + tokens)
    k, m, n_expert, n_used = 1024, 160, 10, 4
    raws = [_experts(t, n_expert, m, k, 8001 + i) for i in range(2)] + [_experts(t, n_expert, 48, k, 8003)]
    ws = [ctx.upload(t, r, k, r.shape[0]) for r in raws]
    b = rng.standard_normal((tokens, 1, k), dtype=np.float32)
    ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
    got = ctx.mulmat_id_multi(ws, n_expert, b, ids)
    for w, y, r in zip(ws, got, raws):
        assert np.array_equal(y, ctx.mulmat_id(w, n_expert, b, ids))
        assert npref.rel_err(y, oracle.mul_mat_id(t, r, k, r.shape[0] // n_expert, n_expert, b, ids)) < TOL
    with pytest.raises(qmm.QmmError):
        ctx.mulmat_id_multi(ws, n_expert, b, np.full((tokens, n_used), n_expert, np.int32))
    for w in ws:
        w.free()


@pytest.mark.parametrize("t,k,m,n_expert,tokens,n_used,b_cols", [(Q4_K, 1024, 200, 6, 64, 3, 1), (Q6_K, 512, 130, 4, 70, 2, 2),
                                                               (Q4_K, 2048, 768, 16, 128, 4, 1), (Q4_K, 256, 64, 3, 500, 1, 1),
                                                               (Q4_K, 256, 32, 40, 1100, 6, 1), (Q6_K, 512, 130, 2, 150, 2, 1),
                                                               (Q4_K, 256, 16, 8, 131100, 4, 1)])
def test_mulmat_id_expert_gemm(ctx, t, k, m, n_expert, tokens, n_used, b_cols):
    """sixteen pairs per expert and more: pairs sorted by expert, every expert's run through the tiled GEMM;
    an idle expert, a crowded one (several tiles), ragged expert height, ids outside the stack (device ids);
    tiles of 64 pairs, and of 128 from 96 pairs per expert; more pairs (524400) than the chunked sort takes, which
    one workgroup then sorts in several rounds of 8192"""
    rng = np.random.default_rng(8100 + t + tokens)
    wb = _experts(t, n_expert, m, k, 8101 + t)
    w = ctx.upload(t, wb, k, n_expert * m)
    b = rng.standard_normal((tokens, b_cols, k), dtype=np.float32)
    ids = rng.integers(0, max(n_expert - 1, 1), (tokens, n_used)).astype(np.int32)  # the last expert stays idle
    ids[: tokens // 2, 0] = 0                                                       # a crowd on expert 0
    got = ctx.mulmat_id(w, n_expert, b, ids)
    want = oracle.mul_mat_id(t, wb, k, m, n_expert, b, ids)
    assert npref.rel_err(got, want) < TOL
    assert np.array_equal(ctx.mulmat_id(w, n_expert, b[::-1].copy(), ids[::-1].copy())[::-1], got)
    bad = ids.copy()
    bad[1, 0] = n_expert
    bad[-1, -1] = -3
    db, dids = DeviceArray(b), DeviceArray(bad)
    dy = DeviceArray(np.zeros((tokens, n_used, m), np.float32), zero=True)
    ctx.mulmat_id_device(w, n_expert, db.ptr, b_cols, dids.ptr, n_used, tokens, dy.ptr)
    ctx.sync()
    out = dy.numpy()
    isbad = (bad < 0) | (bad >= n_expert)
    assert np.isnan(out[isbad]).all() and not np.isnan(out[~isbad]).any()
    assert np.array_equal(out[~isbad], got[~isbad])
    for d in (db, dids, dy):
        d.free()
    w.free()


def test_device_entry_points_replay_from_a_hip_graph():
    """Once the scratch buffers have their size, the device-pointer entry points only launch kernels, so a
    decode block can be captured on a caller's stream and replayed: gate and up behind RMSNorm in one launch,
    down behind SwiGLU, an expert product, a skinny product.  Every replay (with new inputs, and eager work
    in between) must give the eager result."""
    rng = np.random.default_rng(31)
    k, f, n_expert, n_used = 1024, 1536, 8, 2
    c = qmm.Context(0)
    st = Stream()
    c.set_stream(st.ptr.value)
    wg, wu = (c.upload(Q4_K, _weights(Q4_K, f, k, 310 + i), k, f) for i in range(2))
    wd = c.upload(Q6_K, _weights(Q6_K, k, f, 312), f, k)
    we = c.upload(Q4_K, _experts(Q4_K, n_expert, 64, k, 313), k, n_expert * 64)
    ws = c.upload(Q8_0, _weights(Q8_0, 200, k, 314), k, 200)
    x, g = DeviceArray(np.zeros((1, k), np.float32)), DeviceArray(rng.standard_normal(k).astype(np.float32))
    x5 = DeviceArray(np.zeros((5, k), np.float32))
    ids = DeviceArray(np.array([[3, 6]], np.int32))
    outs = {"gate": DeviceArray(np.zeros((1, f), np.float32)), "up": DeviceArray(np.zeros((1, f), np.float32)),
            "down": DeviceArray(np.zeros((1, k), np.float32)), "exp": DeviceArray(np.zeros((1, n_used, 64), np.float32)),
            "skinny": DeviceArray(np.zeros((5, 200), np.float32))}

    def block():
        c.mulmat_produced_device([wg, wu], qmm.PRODUCE_RMSNORM, g.ptr, x.ptr, 1, [outs["gate"].ptr, outs["up"].ptr], eps=1e-5)
        c.mulmat_produced_device([wd], qmm.PRODUCE_SWIGLU, outs["up"].ptr, outs["gate"].ptr, 1, [outs["down"].ptr])
        c.mulmat_id_device(we, n_expert, x.ptr, 1, ids.ptr, n_used, 1, outs["exp"].ptr)
        c.mulmat_device(ws, x5.ptr, 5, outs["skinny"].ptr)

    def fresh_inputs():
        x.set(rng.standard_normal((1, k)).astype(np.float32))
        x5.set(rng.standard_normal((5, k)).astype(np.float32))

    fresh_inputs()
    block()                      # sizes the scratch buffers (allocations are not capturable)
    st.sync()
    replay = st.capture(block)
    for _ in range(3):
        fresh_inputs()
        block()
        st.sync()
        eager = {n: d.numpy() for n, d in outs.items()}
        for d in outs.values():
            d.set(np.zeros(d.shape, np.float32))
        assert replay() == 0
        st.sync()
        for n, d in outs.items():
            assert np.array_equal(d.numpy(), eager[n]), n
    for w in (wg, wu, wd, we, ws):
        w.free()
    for d in [x, g, x5, ids] + list(outs.values()):
        d.free()
    c.close()
    st.destroy()


def test_calls_from_several_threads_each_with_its_own_ctx():
    """A Go caller's goroutines migrate between OS threads and several runners may share a process: contexts
    are independent (own stream, own scratch), a call re-asserts its device, and nothing but the error string is
    thread-local.  Four threads, each with its own ctx and weights, mixed entry points, against results
    computed beforehand on one thread."""
    import threading

    k, m, n_expert = 1024, 96, 4
    rng = np.random.default_rng(41)
    specs = []
    main = qmm.Context(0)
    for i, t in enumerate((Q4_K, Q6_K, Q8_0, Q4_0)):
        wb = _weights(t, m, k, 4100 + i)
        eb = _experts(t, n_expert, 32, k, 4200 + i)
        xs = [rng.standard_normal((n, k), dtype=np.float32) for n in (1, 5, 40)]
        ids = np.array([[1, 3]], np.int32)
        w, e = main.upload(t, wb, k, m), main.upload(t, eb, k, n_expert * 32)
        want = [main.mulmat(w, x) for x in xs] + [main.mulmat_id(e, n_expert, xs[0][None], ids)]
        w.free(); e.free()
        specs.append((t, wb, eb, xs, ids, want))
    main.close()
    errors = []

    def worker(spec):
        try:
            t, wb, eb, xs, ids, want = spec
            c = qmm.Context(0)
            w, e = c.upload(t, wb, k, m), c.upload(t, eb, k, n_expert * 32)
            for _ in range(20):
                got = [c.mulmat(w, x) for x in xs] + [c.mulmat_id(e, n_expert, xs[0][None], ids)]
                for a, b in zip(got, want):
                    if not np.array_equal(a, b):
                        raise AssertionError(f"type {t}: a result changed under concurrency")
            w.free(); e.free()
            c.close()
        except Exception as ex:  # noqa: BLE001 - reported to the main thread
            errors.append(repr(ex))

    threads = [threading.Thread(target=worker, args=(s,)) for s in specs]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors and not any(th.is_alive() for th in threads), errors


# ---- scratch that a captured graph points at must not move --------------------------------------
def test_frozen_scratch_refuses_to_grow_instead_of_reallocating():
    """A HIP graph captured after a warm-up call keeps the addresses of the ctx's scratch.  A later, larger
    eager call used to free and reallocate that scratch; frozen, it returns an error and the buffers stay."""
    k, m = 4096, 512
    c = qmm.Context(0)
    W = c.upload(Q4_K, _weights(Q4_K, m, k, 77), k, m)
    small = np.random.default_rng(5).standard_normal((4, k), dtype=np.float32)
    large = np.random.default_rng(6).standard_normal((600, k), dtype=np.float32)
    try:
        want = c.mulmat(W, small)          # warm-up: scratch sized for 4 rows
        c.scratch_freeze(True)
        with pytest.raises(qmm.QmmError) as e:
            c.mulmat(W, large)             # would have to grow the activation planes
        assert e.value.code == qmm.ERR_INVALID and "frozen" in str(e.value)
        assert np.array_equal(c.mulmat(W, small), want)   # the frozen size still works
        c.scratch_freeze(False)
        assert c.mulmat(W, large).shape == (600, m)       # growth allowed again
    finally:
        W.free()
        c.close()


# ---- exactly what bench.py times ---------------------------------------------------------------------
def test_the_benchmark_step_at_full_size(ctx):
    """bench.py's step on device pointers: gate and up (2 x 14336 x 4096, one launch through
    mi_qmm_mulmat_multi) and down (4096 x 14336, mi_qmm_mulmat), one f32 activation row each, against the oracle"""
    kf, mf = 4096, 14336
    raws = {"gate": _weights(Q4_K, mf, kf, 1003), "up": _weights(Q4_K, mf, kf, 1013), "down": _weights(Q4_K, kf, mf, 1023)}
    Ws = {n: ctx.upload(Q4_K, r, kf if n != "down" else mf, mf if n != "down" else kf) for n, r in raws.items()}
    rng = np.random.default_rng(2003)
    x = rng.standard_normal((1, kf), dtype=np.float32)
    h = rng.standard_normal((1, mf), dtype=np.float32)
    dx, dh = DeviceArray(x), DeviceArray(h)
    yg, yu = DeviceArray(np.empty((1, mf), np.float32), zero=True), DeviceArray(np.empty((1, mf), np.float32), zero=True)
    yd = DeviceArray(np.empty((1, kf), np.float32), zero=True)
    try:
        ctx.mulmat_multi_device([Ws["gate"], Ws["up"]], dx.ptr, 1, [yg.ptr, yu.ptr])
        ctx.mulmat_device(Ws["down"], dh.ptr, 1, yd.ptr)
        ctx.sync()
        for name, got, act, k, m in (("gate", yg.numpy(), x, kf, mf), ("up", yu.numpy(), x, kf, mf), ("down", yd.numpy(), h, mf, kf)):
            want = oracle.mul_mat(Q4_K, raws[name], k, m, act, nthreads=16)
            assert npref.rel_err(got, want) <= TOL, name
            _check_against_exact_arithmetic(Q4_K, raws[name], k, m, act, got, "bench " + name)
    finally:
        for b in (dx, dh, yg, yu, yd):
            b.free()
        for W in Ws.values():
            W.free()


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
@pytest.mark.parametrize("k,n", [(8192, 40), (14336, 128), (14336, 40)])
def test_multi_weight_gemm_keeps_the_k_cut_of_single_calls(ctx, t, k, n):
    """Long rows and few output tiles: a product asked for alone is cut into K slices, so a joint launch (which
    never slices) must not be taken for it -- the bits of a result may not depend on how it was asked for."""
    ms = [512, 256]
    Ws = [ctx.upload(t, _weights(t, m, k, seed=300 + m + k), k, m) for m in ms]
    act = ctx.act_create(qmm.vec_dot_type(t), k, n)
    x = np.random.default_rng(k + n).standard_normal((n, k), dtype=np.float32)
    try:
        ctx.act_quantize(act, x)
        want = [ctx.mulmat_q8(W, act) for W in Ws]
        for y, wnt in zip(ctx.mulmat_q8_multi(Ws, act), want):
            assert np.array_equal(y, wnt)
        for y, wnt in zip(ctx.mulmat_multi(Ws, x), want):
            assert np.array_equal(y, wnt)
    finally:
        act.free()
        for W in Ws:
            W.free()


def test_mulmat_id_rows_longer_than_the_streaming_limit_on_the_expert_gemm(ctx):
    """K above what the streaming kernels walk (32 segments): fine for the sorted expert GEMM, refused only where
    a call would fall to the streaming kernels"""
    t, n_expert, m, k = Q4_K, 2, 48, 131072 + 256
    raw = _experts(t, n_expert, m, k, 91)
    W = ctx.upload(t, raw, k, n_expert * m)
    rng = np.random.default_rng(92)
    tokens = 40  # 20 pairs per expert: the sorted GEMM
    x = rng.standard_normal((tokens, 1, k), dtype=np.float32)
    ids = (np.arange(tokens, dtype=np.int32) % n_expert).reshape(tokens, 1)
    try:
        got = ctx.mulmat_id(W, n_expert, x, ids)
        want = oracle.mul_mat_id(t, raw, k, m, n_expert, x, ids)
        assert npref.rel_err(got, want) <= TOL
        with pytest.raises(qmm.QmmError) as e:   # one pair: the streaming kernel, which cannot walk such a row
            ctx.mulmat_id(W, n_expert, x[:1], ids[:1])
        assert e.value.code == qmm.ERR_UNSUPPORTED
    finally:
        W.free()
