"""Mulmat on Q5_K weights through the C ABI against the oracle.  The library keeps a Q5_K tensor twice: as the blocks
themselves, which the streaming kernel multiplies at up to six activation rows (eight on small tensors), and as the Q4_K
tensor of rows twice as long that gives the same integer sums against [x | x], which every other Q4_K kernel serves."""
import numpy as np
import pytest

import npref
import oracle
from hipmem import DeviceArray
from ollama_amd import qmm, synth
from oracle import Q5_K, Q8_K

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _random_rows(m, k, seed):
    raw = np.random.default_rng(seed).integers(0, 256, (m, k // 256, 176), dtype=np.uint8)
    raw[..., 1] = (raw[..., 1] & 0x07) | 0x10   # d, dmin: small positive halves
    raw[..., 3] = (raw[..., 3] & 0x07) | 0x10
    return raw.reshape(m, -1)


# (rows, K, activation rows): the decode GEMV, the deep and staged kernels, the tiled GEMMs; the value projection and the
# down projection of an 8B model among them
SHAPES = [(64, 256, 1), (64, 256, 3), (100, 1024, 6), (100, 1024, 7), (4096, 14336, 2), (4096, 14336, 6), (2100, 4096, 7), (100, 1024, 1), (1024, 4096, 1), (1024, 4096, 2), (1024, 4096, 4), (1024, 4096, 8), (333, 2048, 16),
          (4096, 14336, 1), (512, 14336, 3), (1024, 4096, 40), (1024, 4096, 130), (4096, 4096, 512), (256, 512, 300)]


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_q5k_against_the_oracle(ctx, m, k, n):
    print(f"q5k case m={m} k={k} n={n}", flush=True)
    raw = synth.weights(Q5_K, m, k, seed=m + k) if m * k > (1 << 20) else _random_rows(m, k, seed=m + k + n)
    x = np.random.default_rng(n + k).standard_normal((n, k)).astype(np.float32)
    W = ctx.upload(Q5_K, raw, k, m)
    try:
        assert (W.type, W.k, W.m) == (Q5_K, k, m)
        y = ctx.mulmat(W, x)
        ref, xq = oracle.mul_mat(Q5_K, raw, k, m, x, nthreads=8, return_xq=True)
        assert npref.rel_err(y, ref) <= 1e-3
        if m * n <= 1 << 16:
            exact = npref.matmul_f64(Q5_K, raw, k, m, Q8_K, xq, n)
            assert npref.rel_err(y, exact, floor=1e-3) <= 1e-3
    finally:
        W.free()


def test_q5k_exact_integers(ctx):
    """unit scales: the outputs are integers, exactly -- low parts, fifth bits and mins all in place"""
    m, k, n = 48, 512, 2
    rng = np.random.default_rng(8)
    raw = _random_rows(m, k, seed=9).reshape(m, 2, 176)
    one = np.array([1.0], np.float16).view(np.uint8)
    raw[..., 0:2] = one
    raw[..., 2:4] = one
    x = rng.integers(-127, 128, (n, k)).astype(np.float32)
    x[:, 0], x[:, 256] = 127, -127
    W = ctx.upload(Q5_K, raw.reshape(m, -1), k, m)
    try:
        y = ctx.mulmat(W, x)
        d, dmin, sc, mn, q = npref.q5_K_ints(raw.reshape(-1))
        w_int = (sc[:, :, None] * q - mn[:, :, None]).reshape(m, k)
        assert np.array_equal(y, (x.astype(np.int64) @ w_int.T).astype(np.float32))
    finally:
        W.free()


def test_q5k_device_pointers_noalloc_joint_calls_and_refusals(ctx):
    m, k = 256, 2048
    raw = synth.weights(Q5_K, m, k, seed=3)
    W = ctx.upload(Q5_K, raw, k, m)
    Wq = ctx.upload(qmm.Q4_K, synth.weights(qmm.Q4_K, 64, k, seed=4), k, 64)
    try:
        for n in (1, 3, 5, 8, 70):
            x = np.random.default_rng(n).standard_normal((n, k)).astype(np.float32)
            want = ctx.mulmat(W, x)
            dx, dy = DeviceArray(x), DeviceArray(np.zeros((n, m), np.float32), zero=True)
            dz = DeviceArray(np.zeros((n, m), np.float32), zero=True)
            ctx.mulmat_device(W, dx.ptr, n, dy.ptr)
            ctx.mulmat_noalloc_device(W, dx.ptr, n, dz.ptr)
            ctx.sync()
            assert np.array_equal(dy.numpy(), want)
            assert npref.rel_err(dz.numpy(), want) <= 1e-3  # (the allocation-free call never cuts K: other order of sums)
            for d in (dx, dy, dz):
                d.free()
        x = np.random.default_rng(5).standard_normal((2, k)).astype(np.float32)
        y5, y4 = ctx.mulmat_multi([W, Wq], x)
        assert np.array_equal(y5, ctx.mulmat(W, x)) and np.array_equal(y4, ctx.mulmat(Wq, x))
        assert ctx.route(W, 1) == "gemv_f32" and ctx.route(W, 512) in ("gemm_int8", "gemm_f16")
        act = ctx.act_create(Q8_K, k, 2)
        ctx.act_quantize(act, x)
        for call in (lambda: ctx.mulmat_q8(W, act), lambda: ctx.mulmat_produced([W], qmm.PRODUCE_RMSNORM, None, x, 1e-5),
                     lambda: ctx.mulmat_swiglu(W, W, x[:1]), lambda: ctx.mulmat_swiglu(Wq, W, x[:1]),
                     lambda: ctx.mulmat_id(W, 2, x.reshape(2, 1, k), np.zeros((2, 1), np.int32))):
            with pytest.raises(qmm.QmmError) as e:
                call()
            assert e.value.code in (qmm.ERR_UNSUPPORTED, qmm.ERR_INVALID)
        act.free()
    finally:
        W.free()
        Wq.free()
