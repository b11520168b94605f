"""The oracle's Q5_K functions and what pins them: the dequantizer against a bit-field statement written from the block
layout (random bytes: every bit pattern of every field), the dot product against fp64 brute force over those
dequantized values and against exact integers, the reduction to Q4_K when no fifth bit is set."""
import numpy as np
import pytest

import npref
import oracle
from ollama_amd import synth
from oracle import Q4_K, Q5_K, Q8_K


def _random_blocks(rows, nsb, seed):
    raw = np.random.default_rng(seed).integers(0, 256, (rows, nsb, 176), dtype=np.uint8)
    raw[..., 1] &= 0x3F  # d and dmin finite halves of moderate size
    raw[..., 3] &= 0x3F
    return raw.reshape(rows, -1)


def test_q5k_sizes():
    assert oracle.block_size(Q5_K) == 256 and oracle.type_size(Q5_K) == 176 and oracle.vec_dot_type(Q5_K) == Q8_K
    assert oracle.row_size(Q5_K, 4096) == 16 * 176 and oracle.row_size(Q5_K, 300) == -1


def test_q5k_dequantizer_on_random_bytes():
    raw = _random_blocks(6, 5, seed=1)
    got = oracle.dequantize(Q5_K, raw, 5 * 256).astype(np.float64)
    want = npref.dequant(Q5_K, raw).reshape(6, -1)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    # one-hot fifth bits: bit j of qh[l] is element 32 j + l
    blk = np.zeros(176, np.uint8)
    blk[0:2] = np.array([1.0], np.float16).view(np.uint8)       # d = 1, dmin = 0
    blk[4:8] = 1                                                  # scales of sub-blocks 0..3 = 1
    blk[8 + 4:8 + 8] = 1                                          # scales of sub-blocks 4..7 = 1 (low four bits)
    for j, l in ((0, 0), (3, 17), (7, 31), (4, 5)):
        b = blk.copy()
        b[16 + l] = 1 << j
        w = oracle.dequantize(Q5_K, b[None, :], 256).reshape(-1)
        want = np.zeros(256)
        want[32 * j + l] = 16
        assert np.array_equal(w, want), (j, l)


@pytest.mark.parametrize("nsb", [1, 3, 16])
def test_q5k_dot_against_fp64_brute_force(nsb):
    k = 256 * nsb
    raw = _random_blocks(4, nsb, seed=10 + nsb)
    x = np.random.default_rng(20 + nsb).standard_normal((3, k)).astype(np.float32) * 2
    y, xq = oracle.mul_mat(Q5_K, raw, k, 4, x, return_xq=True)
    want = npref.matmul_f64(Q5_K, raw, k, 4, Q8_K, xq, 3)
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()


def test_q5k_dot_exact_integers():
    """d = dmin = 1, distinct scales and mins per sub-block, unit activation scale: the result is an integer a swapped
    index, a dropped fifth bit or a wrong min would change"""
    rng = np.random.default_rng(3)
    k = 512
    raw = _random_blocks(1, 2, seed=4).reshape(2, 176)
    raw[:, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    raw[:, 2:4] = np.array([1.0], np.float16).view(np.uint8)
    x = rng.integers(-127, 128, (1, k)).astype(np.float32)
    x[0, 0], x[0, 256] = 127, -127                               # each block's largest: Q8_K keeps the integers, |d| = 1
    xq = oracle.quantize(Q8_K, x)
    d8, q8, _ = npref.q8_K_ints(xq)
    assert np.array_equal(np.abs(d8), [1.0, 1.0])
    got = oracle.vec_dot(Q5_K, k, raw.reshape(-1), xq.reshape(-1))
    d, dmin, sc, m, q = npref.q5_K_ints(raw.reshape(-1))
    y8 = (d8[:, None] * q8).reshape(2, 8, 32)
    want = float(((sc[:, :, None] * q - m[:, :, None]) * y8).sum())
    assert got == want


def test_q5k_without_fifth_bits_is_q4k():
    k, m = 1024, 7
    raw4 = synth.weights(Q4_K, m, k, seed=5).reshape(m, k // 256, 144)
    raw5 = np.zeros((m, k // 256, 176), np.uint8)
    raw5[..., 0:16] = raw4[..., 0:16]
    raw5[..., 48:] = raw4[..., 16:]
    x = np.random.default_rng(6).standard_normal((2, k)).astype(np.float32)
    assert np.array_equal(oracle.mul_mat(Q5_K, raw5.reshape(m, -1), k, m, x), oracle.mul_mat(Q4_K, raw4.reshape(m, -1), k, m, x))


def test_synthetic_q5k_blocks_reconstruct_their_input():
    x = (np.random.default_rng(7).standard_normal((3, 512)) * 0.02).astype(np.float32)
    raw = synth.encode_q5_K(x)
    back = oracle.dequantize(Q5_K, raw, 512)
    step = (x.reshape(3, 2, 8, 32).max(axis=3) - np.minimum(x.reshape(3, 2, 8, 32).min(axis=3), 0)) / 31
    assert np.abs(back - x).max() <= 1.6 * step.max()
    assert np.count_nonzero(raw.reshape(3, 2, 176)[..., 16:48])  # fifth bits are in use
