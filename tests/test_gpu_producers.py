"""GPU parity of the activation producers (RMSNorm, SwiGLU) and of the products fused with them, through
the C ABI, against the CPU oracle.

Bars: RMSNorm within 2 ulp of the oracle (the double-precision sum of squares is taken in a different
order, everything after it is the same correctly rounded fp32 arithmetic; in practice the bits agree);
SwiGLU within 1e-6 relative (the device expf is within 1 ulp of libm's); fused products within 1e-3 of the
oracle chain (the bar of the products themselves) and bit-identical to the library's own two-step path.
"""
import numpy as np
import pytest

import npref
import oracle
from hipmem import DeviceArray
from npref import Q4_0, Q4_K, Q6_K, Q8_0
from ollama_amd import qmm

pytestmark = pytest.mark.gpu
TOL = 1e-3
WTYPES = [Q4_0, Q8_0, Q4_K, Q6_K]


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _weights(t, m, k, seed):
    rng = np.random.default_rng(seed)
    return oracle.quantize(t, (rng.standard_normal((m, k), dtype=np.float32) * np.float32(0.02)), nthreads=16)


def _ulps(a, b):
    a = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    return np.abs(a - b).max() if a.size else 0


@pytest.mark.parametrize("n,k", [(1, 4), (1, 32), (3, 36), (1, 4096), (5, 14336), (2, 135168), (600, 128)])
@pytest.mark.parametrize("with_g", [True, False])
def test_rms_norm_matches_the_oracle(ctx, n, k, with_g):
    """rows shorter than a 256-element piece, rows that are no multiple of one, rows of more than 512 pieces"""
    rng = np.random.default_rng(k * 7 + n)
    x = (rng.standard_normal((n, k)) * rng.uniform(0.05, 20, (n, 1))).astype(np.float32)
    g = rng.standard_normal(k).astype(np.float32) if with_g else None
    for eps in (1e-5, 1e-6):
        got = ctx.rms_norm(x, g, eps)
        want = oracle.rms_norm(x, g, eps)
        assert _ulps(got, want) <= 2
        assert np.count_nonzero(got != want) <= got.size // 1000


def test_rms_norm_closed_forms_and_edges(ctx):
    k = 1024
    y = ctx.rms_norm(np.full((2, k), 3.0, np.float32), None, 1e-5)
    assert np.all(y == np.float32(3.0) * (np.float32(1) / np.sqrt(np.float32(9.0) + np.float32(1e-5))))
    assert np.all(ctx.rms_norm(np.zeros((1, k), np.float32), np.ones(k, np.float32), 1e-6) == 0)
    x = np.zeros((1, k), np.float32); x[0, 1000] = -2.0
    y = ctx.rms_norm(x, None, 0.0)
    assert np.count_nonzero(y) == 1 and abs(y[0, 1000] + np.sqrt(k)) < 1e-4
    assert ctx.rms_norm(np.zeros((0, k), np.float32), None, 1e-5).shape == (0, k)
    with pytest.raises(qmm.QmmError) as e:
        ctx.rms_norm(np.zeros((1, 6), np.float32), None, 1e-5)
    assert e.value.code == qmm.ERR_UNSUPPORTED
    with pytest.raises(qmm.QmmError) as e:
        ctx.rms_norm(np.zeros((1, 8), np.float32), None, -1.0)
    assert e.value.code == qmm.ERR_INVALID


def test_swiglu_matches_the_oracle(ctx):
    rng = np.random.default_rng(11)
    gate = (rng.standard_normal((7, 14336)) * 3).astype(np.float32)
    up = rng.standard_normal((7, 14336)).astype(np.float32)
    gate[0, :12] = [0.0, -0.0, 88.0, -88.0, 100.0, -100.0, 1e-30, -1e-30, 20.0, -20.0, 87.3, -87.3]
    got = ctx.swiglu(gate, up)
    want = oracle.swiglu(gate, up)
    assert np.all(np.isfinite(got))
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-30)) < 1e-6
    one = np.ones((1, 8), np.float32)
    v = np.array([[0.0, 100.0, -100.0, 1.0, -1.0, 30.0, -30.0, 0.5]], np.float32)
    s = ctx.swiglu(v, one)
    assert s[0, 0] == 0 and s[0, 1] == 100.0 and s[0, 2] == 0.0
    assert np.allclose(s[0, 3] - s[0, 4], 1.0, atol=1e-6) and np.allclose(s[0, 5] - s[0, 6], 30.0, atol=1e-5)
    assert ctx.swiglu(np.zeros((0, 8), np.float32), np.zeros((0, 8), np.float32)).shape == (0, 8)
    # the bare activation (no up): the same bits as gating with ones, and the closed form in fp64
    bare = ctx.swiglu(v, None)
    assert np.array_equal(bare, s)
    v64 = v.astype(np.float64)
    assert np.max(np.abs(bare - v64 / (1.0 + np.exp(-v64)))) <= 1e-6 * max(1.0, float(np.max(np.abs(v64))))


def _chain(t, wb, k, m, producer, aux, x, eps):
    xp = oracle.rms_norm(x, aux, eps) if producer == qmm.PRODUCE_RMSNORM else oracle.swiglu(x, aux)
    return oracle.mul_mat(t, wb, k, m, xp, nthreads=16)


def _two_step(ctx, ws, producer, aux, x, eps):
    xp = ctx.rms_norm(x, aux, eps) if producer == qmm.PRODUCE_RMSNORM else ctx.swiglu(x, aux)
    return ctx.mulmat_multi(ws, xp)


# decode: the GEMV produces x in its prologue.  Rows of one K segment, of several (down: 3.5), short rows that
# go 2 and 4 to a load, a Q8_0 row that is no multiple of 256, and a K too long for the prefetch registers
# (fused quantizer instead)
DECODE = [(Q4_K, 4096, 300), (Q4_K, 14336, 130), (Q6_K, 4096, 200), (Q6_K, 2048, 64), (Q4_K, 1024, 96), (Q4_K, 256, 40),
          (Q4_0, 4096, 128), (Q8_0, 4128, 70), (Q8_0, 512, 33), (Q4_0, 32, 5), (Q4_K, 24576, 48), (Q6_K, 14336, 77)]


@pytest.mark.parametrize("t,k,m", DECODE)
@pytest.mark.parametrize("producer", [qmm.PRODUCE_RMSNORM, qmm.PRODUCE_SWIGLU])
def test_decode_product_fused_with_its_producer(ctx, t, k, m, producer):
    rng = np.random.default_rng(t * 1000 + k + m + producer)
    wbs = [_weights(t, m, k, 4000 + t + k), _weights(t, m + 7, k, 4001 + t + k)]
    ws = [ctx.upload(t, wb, k, mm) for wb, mm in zip(wbs, (m, m + 7))]
    x = (rng.standard_normal((1, k)) * 1.7).astype(np.float32)
    aux = rng.standard_normal(k).astype(np.float32) if producer == qmm.PRODUCE_RMSNORM else rng.standard_normal((1, k)).astype(np.float32)
    got = ctx.mulmat_produced(ws, producer, aux, x, eps=1e-5)
    for y, wb, mm in zip(got, wbs, (m, m + 7)):
        assert npref.rel_err(y, _chain(t, wb, k, mm, producer, aux, x, 1e-5)) < TOL
    for y, y2 in zip(got, _two_step(ctx, ws, producer, aux, x, 1e-5)):
        assert np.array_equal(y, y2)
    if producer == qmm.PRODUCE_RMSNORM:  # the bare normalization
        got = ctx.mulmat_produced(ws[:1], producer, None, x, eps=1e-6)
        assert npref.rel_err(got[0], _chain(t, wbs[0], k, m, producer, None, x, 1e-6)) < TOL
        assert np.array_equal(got[0], ctx.mulmat_multi(ws[:1], ctx.rms_norm(x, None, 1e-6))[0])
    for w in ws:
        w.free()


# batches: fused quantizer (RMSNorm: row scales first), then the GEMV / skinny / GEMM kernels
@pytest.mark.parametrize("t,k,m,n", [(Q4_K, 4096, 200, 2), (Q4_K, 2048, 100, 5), (Q6_K, 1024, 130, 12), (Q4_K, 1024, 257, 70),
                                     (Q8_0, 1056, 90, 3), (Q4_0, 512, 64, 40), (Q8_0, 4096, 64, 9),
                                     # prefill sizes: the fused quantizer with sixteen lanes per block writes the fp16
                                     # planes too; the products run on the 256-row kernels (fp16 MFMA; Q6_K with K slices)
                                     (Q4_K, 2048, 12300, 512), (Q6_K, 3328, 5000, 512)])
@pytest.mark.parametrize("producer", [qmm.PRODUCE_RMSNORM, qmm.PRODUCE_SWIGLU])
def test_batch_product_fused_with_its_producer(ctx, t, k, m, n, producer):
    rng = np.random.default_rng(t * 1000 + k + m + n + producer)
    wb = _weights(t, m, k, 4100 + t + k)
    w = ctx.upload(t, wb, k, m)
    x = (rng.standard_normal((n, k)) * rng.uniform(0.2, 5, (n, 1))).astype(np.float32)
    aux = rng.standard_normal(k).astype(np.float32) if producer == qmm.PRODUCE_RMSNORM else rng.standard_normal((n, k)).astype(np.float32)
    got = ctx.mulmat_produced([w], producer, aux, x, eps=1e-5)[0]
    assert npref.rel_err(got, _chain(t, wb, k, m, producer, aux, x, 1e-5)) < TOL
    assert np.array_equal(got, _two_step(ctx, [w], producer, aux, x, 1e-5)[0])
    w.free()


def test_produced_weights_of_two_types_and_device_pointers(ctx):
    """gate (Q4_K) and a Q6_K matrix behind one RMSNorm; the same call on device pointers"""
    k, rng = 4096, np.random.default_rng(77)
    wbs = [_weights(Q4_K, 120, k, 4200), _weights(Q6_K, 90, k, 4201), _weights(Q8_0, 50, k, 4202)]
    ws = [ctx.upload(t, wb, k, m) for t, wb, m in zip((Q4_K, Q6_K, Q8_0), wbs, (120, 90, 50))]
    x = rng.standard_normal((1, k)).astype(np.float32)
    g = rng.standard_normal(k).astype(np.float32)
    got = ctx.mulmat_produced(ws, qmm.PRODUCE_RMSNORM, g, x, eps=1e-5)
    for y, t, wb, m in zip(got, (Q4_K, Q6_K, Q8_0), wbs, (120, 90, 50)):
        assert npref.rel_err(y, _chain(t, wb, k, m, qmm.PRODUCE_RMSNORM, g, x, 1e-5)) < TOL
    dx, dg = DeviceArray(x), DeviceArray(g)
    dys = [DeviceArray(np.zeros((1, m), np.float32), zero=True) for m in (120, 90, 50)]
    ctx.mulmat_produced_device(ws, qmm.PRODUCE_RMSNORM, dg.ptr, dx.ptr, 1, [d.ptr for d in dys], eps=1e-5)
    ctx.sync()
    for d, y in zip(dys, got):
        assert np.array_equal(d.numpy(), y)
    for d in [dx, dg] + dys:
        d.free()
    for w in ws:
        w.free()


def test_produced_errors(ctx):
    k = 256
    w = ctx.upload(Q4_K, _weights(Q4_K, 8, k, 1), k, 8)
    x = np.ones((1, k), np.float32)
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_produced([w], 7, None, x)
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_produced([w], qmm.PRODUCE_SWIGLU, None, x)
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_produced([w], qmm.PRODUCE_RMSNORM, None, x, eps=-1.0)
    assert e.value.code == qmm.ERR_INVALID
    assert ctx.mulmat_produced([w], qmm.PRODUCE_NONE, None, x)[0].shape == (1, 8)
    assert ctx.mulmat_produced([w], qmm.PRODUCE_RMSNORM, None, np.zeros((0, k), np.float32))[0].shape == (0, 8)
    w.free()


def test_randomized_produced_sweep(ctx):
    """random types, shapes, batch sizes, producers and weight counts against the oracle chain and the
    library's own two-step path"""
    rng = np.random.default_rng(20250)
    for case in range(40):
        t = int(rng.choice(WTYPES))
        blk = 256 if t in (Q4_K, Q6_K) else 32
        k = int(rng.integers(1, 24 if blk == 256 else 150)) * blk
        if case % 6 == 2:
            k = int(rng.integers(17, 60)) * 256
        n = int(rng.choice([1, 1, 1, 2, 3, 5, 8, 9, 33, 70]))
        ms = [int(rng.integers(1, 300)) for _ in range(int(rng.integers(1, 4)))]
        producer = int(rng.choice([qmm.PRODUCE_RMSNORM, qmm.PRODUCE_SWIGLU]))
        wbs = [_weights(t, m, k, 5000 + case + i) for i, m in enumerate(ms)]
        ws = [ctx.upload(t, wb, k, m) for wb, m in zip(wbs, ms)]
        x = (rng.standard_normal((n, k)) * float(rng.choice([1e-2, 1.0, 20.0]))).astype(np.float32)
        if producer == qmm.PRODUCE_RMSNORM:
            aux = rng.standard_normal(k).astype(np.float32) if case % 3 else None
        else:
            aux = rng.standard_normal((n, k)).astype(np.float32)
        eps = float(rng.choice([1e-5, 1e-6]))
        got = ctx.mulmat_produced(ws, producer, aux, x, eps=eps)
        two = _two_step(ctx, ws, producer, aux, x, eps)
        for y, y2, wb, m in zip(got, two, wbs, ms):
            err = npref.rel_err(y, _chain(t, wb, k, m, producer, aux, x, eps))
            assert y.shape == (n, m) and err < TOL, f"case {case}: type {t} k={k} m={m} n={n} producer {producer}: {err}"
            assert np.array_equal(y, y2), f"case {case}: type {t} k={k} m={m} n={n} producer {producer}"
        for w in ws:
            w.free()


def _experts(t, n_expert, m, k, seed):
    return _weights(t, n_expert * m, k, seed)


# the down projection of an expert feed-forward block: silu(gate) * up per slot, then the expert's matrix.
# Decode (in the prologue of the per-pair product), bucketed / matrix-core / expert-GEMM batches (fused
# quantizer), rows longer than the prefetch registers of the decode kernel.
@pytest.mark.parametrize("t,k,m,n_expert,tokens,n_used", [(Q4_K, 768, 200, 16, 1, 8), (Q4_K, 768, 64, 16, 3, 4), (Q6_K, 512, 96, 8, 2, 2),
                                                            (Q8_0, 352, 40, 6, 1, 3), (Q4_0, 2048, 33, 4, 2, 2), (Q4_K, 1024, 70, 4, 40, 2),
                                                            (Q4_K, 512, 64, 3, 300, 2), (Q8_0, 256, 50, 2, 30, 2), (Q4_K, 9216, 20, 4, 1, 2)])
def test_expert_down_projection_fused_with_swiglu(ctx, t, k, m, n_expert, tokens, n_used):
    rng = np.random.default_rng(6000 + t + k + tokens)
    wb = _experts(t, n_expert, m, k, 6001 + t + k)
    w = ctx.upload(t, wb, k, n_expert * m)
    gate = (rng.standard_normal((tokens, n_used, k)) * 2).astype(np.float32)
    up = rng.standard_normal((tokens, n_used, k)).astype(np.float32)
    ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
    got = ctx.mulmat_id_produced(w, n_expert, qmm.PRODUCE_SWIGLU, up, gate, ids)
    want = oracle.mul_mat_id(t, wb, k, m, n_expert, oracle.swiglu(gate, up), ids)
    assert npref.rel_err(got, want) < TOL
    assert np.array_equal(got, ctx.mulmat_id(w, n_expert, ctx.swiglu(gate, up), ids))
    w.free()


def test_expert_product_behind_rms_norm_and_errors(ctx):
    t, k, m, n_expert, n_used = Q4_K, 1024, 48, 8, 3
    rng = np.random.default_rng(61)
    wb = _experts(t, n_expert, m, k, 62)
    w = ctx.upload(t, wb, k, n_expert * m)
    g = rng.standard_normal(k).astype(np.float32)
    for tokens in (1, 50):
        x = rng.standard_normal((tokens, 1, k)).astype(np.float32)
        ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
        got = ctx.mulmat_id_produced(w, n_expert, qmm.PRODUCE_RMSNORM, g, x, ids, eps=1e-5)
        xn = oracle.rms_norm(x.reshape(tokens, k), g, 1e-5).reshape(tokens, 1, k)
        assert npref.rel_err(got, oracle.mul_mat_id(t, wb, k, m, n_expert, xn, ids)) < TOL
        assert np.array_equal(got, ctx.mulmat_id(w, n_expert, ctx.rms_norm(x.reshape(tokens, k), g, 1e-5).reshape(tokens, 1, k), ids))
    x = np.ones((1, 1, k), np.float32)
    ids = np.zeros((1, 1), np.int32)
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_id_produced(w, n_expert, qmm.PRODUCE_SWIGLU, None, x, ids)
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_id_produced(w, n_expert, 9, None, x, ids)
    assert e.value.code == qmm.ERR_INVALID
    assert np.array_equal(ctx.mulmat_id_produced(w, n_expert, qmm.PRODUCE_NONE, None, x, ids), ctx.mulmat_id(w, n_expert, x, ids))
    w.free()


# gate and up in one pass with the gating in the epilogue: rows of one K segment, of several (partials through
# LDS), short rows that go two and four to a load, ragged row counts; batches take the products and the gating
# kernel.  Always the bits of the separate calls.
@pytest.mark.parametrize("t,k,m", [(Q4_K, 4096, 300), (Q4_K, 4096, 14336), (Q4_K, 2048, 129), (Q4_K, 1024, 77), (Q4_K, 8192, 65),
                                   (Q4_K, 14336, 31), (Q6_K, 4096, 200), (Q6_K, 1280, 33), (Q4_0, 4096, 128), (Q4_0, 512, 19),
                                   (Q8_0, 1024, 70), (Q8_0, 4128, 45), (Q8_0, 256, 7), (Q4_K, 256, 1)])
@pytest.mark.parametrize("rms", [False, True])
def test_gate_and_up_with_the_gating_in_the_epilogue(ctx, t, k, m, rms):
    rng = np.random.default_rng(t * 100 + k + m)
    wbg, wbu = _weights(t, m, k, 7000 + k + m), _weights(t, m, k, 7001 + k + m)
    wg, wu = ctx.upload(t, wbg, k, m), ctx.upload(t, wbu, k, m)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32) if rms else None
    producer = qmm.PRODUCE_RMSNORM if rms else qmm.PRODUCE_NONE
    for n in (1, 3, 40):
        if n > 1 and m > 1000:
            continue
        x = (rng.standard_normal((n, k)) * 3).astype(np.float32)
        h = ctx.mulmat_swiglu(wg, wu, x, producer, g, eps=1e-5)
        xn = oracle.rms_norm(x, g, 1e-5) if rms else x
        want = oracle.swiglu(oracle.mul_mat(t, wbg, k, m, xn, nthreads=16), oracle.mul_mat(t, wbu, k, m, xn, nthreads=16))
        assert h.shape == (n, m) and npref.rel_err(h, want) < TOL, n
        yg, yu = ctx.mulmat_produced([wg, wu], producer, g, x, eps=1e-5) if rms else ctx.mulmat_multi([wg, wu], x)
        assert np.array_equal(h, ctx.swiglu(yg, yu)), n
    wg.free(); wu.free()


def test_mulmat_swiglu_errors_and_device_pointers(ctx):
    k, m = 512, 40
    wg, wu = ctx.upload(Q4_K, _weights(Q4_K, m, k, 1), k, m), ctx.upload(Q4_K, _weights(Q4_K, m, k, 2), k, m)
    w3 = ctx.upload(Q4_K, _weights(Q4_K, m + 1, k, 3), k, m + 1)
    w6 = ctx.upload(Q6_K, _weights(Q6_K, m, k, 4), k, m)
    x = np.random.default_rng(5).standard_normal((1, k)).astype(np.float32)
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_swiglu(wg, w3, x)
    assert e.value.code == qmm.ERR_INVALID
    with pytest.raises(qmm.QmmError) as e:
        ctx.mulmat_swiglu(wg, wu, x, qmm.PRODUCE_SWIGLU, None)
    assert e.value.code == qmm.ERR_INVALID
    # gate and up of different types: the products and the gating kernel
    h = ctx.mulmat_swiglu(wg, w6, x)
    yg, yu = ctx.mulmat_multi([wg, w6], x)
    assert np.array_equal(h, ctx.swiglu(yg, yu))
    assert ctx.mulmat_swiglu(wg, wu, np.zeros((0, k), np.float32)).shape == (0, m)
    want = ctx.mulmat_swiglu(wg, wu, x)
    for n in (1, 2):
        xs = np.repeat(x, n, axis=0)
        dx, dh = DeviceArray(xs), DeviceArray(np.zeros((n, m), np.float32), zero=True)
        ctx.mulmat_swiglu_device(wg, wu, dx.ptr, n, dh.ptr)
        ctx.sync()
        assert np.array_equal(dh.numpy(), np.repeat(want, n, axis=0))
        dx.free(); dh.free()
    for w in (wg, wu, w3, w6):
        w.free()


# gate and up of an expert block with the gating: decode sizes in one launch (rows of one segment, short rows
# two and four to a load, rows of several segments), batches through the two products and the gating kernel,
# stacks of different types, ids outside the stack
@pytest.mark.parametrize("t,k,m,n_expert,tokens,n_used,b_cols", [(Q4_K, 2048, 96, 16, 1, 8, 1), (Q4_K, 768, 200, 8, 2, 4, 4),
                                                                  (Q4_K, 4096, 33, 4, 1, 2, 1), (Q6_K, 1024, 70, 6, 3, 2, 1),
                                                                  (Q4_K, 8192, 20, 4, 1, 2, 1), (Q8_0, 352, 40, 6, 1, 3, 1),
                                                                  (Q4_0, 2048, 31, 4, 2, 2, 2), (Q4_K, 1024, 64, 4, 40, 2, 1),
                                                                  (Q4_K, 512, 64, 3, 300, 2, 1), (Q8_0, 256, 50, 2, 30, 2, 1)])
def test_expert_gate_and_up_with_the_gating(ctx, t, k, m, n_expert, tokens, n_used, b_cols):
    rng = np.random.default_rng(8000 + t + k + tokens)
    wbg, wbu = _experts(t, n_expert, m, k, 8001 + t + k), _experts(t, n_expert, m, k, 8002 + t + k)
    wg, wu = ctx.upload(t, wbg, k, n_expert * m), ctx.upload(t, wbu, k, n_expert * m)
    b = (rng.standard_normal((tokens, b_cols, k)) * 2).astype(np.float32)
    ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
    h = ctx.mulmat_id_swiglu(wg, wu, n_expert, b, ids)
    want = oracle.swiglu(oracle.mul_mat_id(t, wbg, k, m, n_expert, b, ids), oracle.mul_mat_id(t, wbu, k, m, n_expert, b, ids))
    assert h.shape == (tokens, n_used, m) and npref.rel_err(h, want) < TOL
    yg, yu = ctx.mulmat_id_multi([wg, wu], n_expert, b, ids)
    assert np.array_equal(h, ctx.swiglu(yg, yu))
    # ids outside the stack (device ids): NaN rows for those pairs, the others unchanged
    bad = ids.copy()
    bad[0, 0] = n_expert
    db, dids = DeviceArray(b), DeviceArray(bad)
    dh = DeviceArray(np.zeros((tokens, n_used, m), np.float32), zero=True)
    ctx.mulmat_id_swiglu_device(wg, wu, n_expert, db.ptr, b_cols, dids.ptr, n_used, tokens, dh.ptr)
    ctx.sync()
    out = dh.numpy()
    assert np.isnan(out[0, 0]).all() and np.array_equal(out.reshape(-1, m)[1:], h.reshape(-1, m)[1:])
    with pytest.raises(qmm.QmmError):
        ctx.mulmat_id_swiglu(wg, wu, n_expert, b, bad)
    for d in (db, dids, dh):
        d.free()
    wg.free(); wu.free()


def test_expert_gating_with_stacks_of_two_types(ctx):
    k, m, n_expert, n_used = 512, 48, 4, 2
    rng = np.random.default_rng(83)
    wbg, wbu = _experts(Q4_K, n_expert, m, k, 84), _experts(Q6_K, n_expert, m, k, 85)
    wg, wu = ctx.upload(Q4_K, wbg, k, n_expert * m), ctx.upload(Q6_K, wbu, k, n_expert * m)
    for tokens in (1, 20):
        b = rng.standard_normal((tokens, 1, k)).astype(np.float32)
        ids = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
        h = ctx.mulmat_id_swiglu(wg, wu, n_expert, b, ids)
        assert np.array_equal(h, ctx.swiglu(ctx.mulmat_id(wg, n_expert, b, ids), ctx.mulmat_id(wu, n_expert, b, ids)))
    wg.free(); wu.free()
