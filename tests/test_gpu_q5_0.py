"""Mulmat on Q5_0 weights through the C ABI against the oracle.  The library keeps such a tensor as the Q8_0 planes with the
same dot products (the 5-bit values minus 16 as int8 under the block's own scale), so every Q8_0 kernel serves it -- and
gives the oracle's bits where the Q8_0 kernels give them for Q8_0 weights."""
import numpy as np
import pytest

import npref
import oracle
from ollama_amd import qmm, synth
from oracle import Q5_0, Q8_0

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _random_rows(m, k, seed):
    raw = np.random.default_rng(seed).integers(0, 256, (m, k // 32, 22), dtype=np.uint8)
    raw[..., 1] = (raw[..., 1] & 0x07) | 0x10
    return raw.reshape(m, -1)


@pytest.mark.parametrize("m,k,n", [(64, 256, 1), (100, 96, 2), (512, 4096, 1), (512, 4096, 4), (300, 2080, 8), (256, 4096, 20),
                                   (1024, 4096, 130), (4096, 4096, 512)])
def test_q5_0_against_the_oracle(ctx, m, k, n):
    print(f"q5_0 case m={m} k={k} n={n}", flush=True)
    raw = _random_rows(m, k, seed=m + k + n) if m * k <= 1 << 22 else synth.weights(Q5_0, m, k, seed=m)
    x = np.random.default_rng(n + k).standard_normal((n, k)).astype(np.float32)
    W = ctx.upload(Q5_0, raw, k, m)
    try:
        assert (W.type, W.k, W.m) == (Q5_0, k, m)
        y = ctx.mulmat(W, x)
        ref, xq = oracle.mul_mat(Q5_0, raw, k, m, x, nthreads=8, return_xq=True)
        assert npref.rel_err(y, ref) <= 1e-3
        if m * n <= 1 << 16:
            assert npref.rel_err(y, npref.matmul_f64(Q5_0, raw, k, m, Q8_0, xq, n), floor=1e-3) <= 1e-3
    finally:
        W.free()


def test_q5_0_is_the_q8_0_product_of_its_integers(ctx):
    """the same bits as a Q8_0 weight holding q - 16 under the same scales, on the streaming kernel and on the matrix cores"""
    m, k = 128, 1024
    raw = _random_rows(m, k, seed=5)
    d, q = npref.q5_0_ints(raw.reshape(-1))
    as8 = np.empty((m * k // 32, 34), np.uint8)
    as8[:, 0:2] = raw.reshape(-1, 22)[:, 0:2]
    as8[:, 2:] = q.astype(np.int8).view(np.uint8)
    W5, W8 = ctx.upload(Q5_0, raw, k, m), ctx.upload(Q8_0, as8.reshape(m, -1), k, m)
    try:
        for n in (1, 8, 64):
            x = np.random.default_rng(n).standard_normal((n, k)).astype(np.float32)
            assert np.array_equal(ctx.mulmat(W5, x), ctx.mulmat(W8, x))
    finally:
        W5.free(); W8.free()
