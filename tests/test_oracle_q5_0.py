"""The oracle's Q5_0 functions and what pins them: the dequantizer against a bit-field statement written from the block
layout on random bytes and one-hot fifth bits, the dot product against fp64 brute force and exactly on integers."""
import numpy as np
import pytest

import npref
import oracle
from oracle import Q5_0, Q8_0


def _random_rows(m, nb, seed):
    raw = np.random.default_rng(seed).integers(0, 256, (m, nb, 22), dtype=np.uint8)
    raw[..., 1] &= 0x3F
    return raw.reshape(m, -1)


def test_sizes():
    assert oracle.block_size(Q5_0) == 32 and oracle.type_size(Q5_0) == 22 and oracle.vec_dot_type(Q5_0) == Q8_0


def test_dequantizer_on_random_bytes_and_one_hot_bits():
    raw = _random_rows(5, 6, seed=1)
    got = oracle.dequantize(Q5_0, raw, 6 * 32).astype(np.float64)
    assert np.array_equal(got, npref.dequant(Q5_0, raw).reshape(5, -1).astype(np.float32).astype(np.float64))
    blk = np.zeros(22, np.uint8)
    blk[0:2] = np.array([1.0], np.float16).view(np.uint8)
    for i in (0, 7, 15, 16, 24, 31):          # bit i of the little-endian word is element i: 16 - 16 = 0 there, -16 elsewhere
        b = blk.copy()
        b[2 + i // 8] = 1 << (i % 8)
        w = oracle.dequantize(Q5_0, b[None, :], 32).reshape(-1)
        want = np.full(32, -16.0)
        want[i] = 0.0
        assert np.array_equal(w, want), i


@pytest.mark.parametrize("nb", [1, 4, 128])
def test_dot_against_fp64_and_exact_integers(nb):
    k = 32 * nb
    raw = _random_rows(3, nb, seed=nb)
    rng = np.random.default_rng(10 + nb)
    x = rng.standard_normal((2, k)).astype(np.float32)
    y, xq = oracle.mul_mat(Q5_0, raw, k, 3, x, return_xq=True)
    want = npref.matmul_f64(Q5_0, raw, k, 3, Q8_0, xq, 2)
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()
    raw1 = raw.reshape(3, nb, 22).copy()
    raw1[..., 0:2] = np.array([1.0], np.float16).view(np.uint8)
    xi = rng.integers(-127, 128, (1, k)).astype(np.float32)
    xi[0, ::32] = 127
    got = oracle.mul_mat(Q5_0, raw1.reshape(3, -1), k, 3, xi)
    _, q = npref.q5_0_ints(raw1.reshape(-1))
    assert np.array_equal(got, (xi.astype(np.int64) @ q.reshape(3, k).T).astype(np.float32))
