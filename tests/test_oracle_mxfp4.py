"""The oracle's MXFP4 functions and what pins them: the block layout by the reference's own converter
(/root/reference/convert/convert_gptoss.go:216-238, restated here as the byte shuffle it performs), the values by the
formats' definitions (OCP microscaling E2M1 and E8M0), the dot product by fp64 brute force and exact integers."""
import numpy as np
import pytest

import npref
import oracle
from ollama_amd import synth
from oracle import MXFP4, Q8_0

E2M1 = [0, 0.5, 1, 1.5, 2, 3, 4, 6]


def test_sizes_and_activation_type():
    assert oracle.block_size(MXFP4) == 32 and oracle.type_size(MXFP4) == 17 and oracle.vec_dot_type(MXFP4) == Q8_0


def test_every_code_and_every_scale():
    """all 16 codes under scales from one end of the range to the other: value = E2M1(code) * 2^(e - 127)"""
    for e in list(range(0, 250, 7)) + [1, 2, 103, 104, 127, 128, 251]:
        blk = np.zeros(17, np.uint8)
        blk[0] = e
        blk[1:] = np.arange(16, dtype=np.uint8) | (np.arange(15, -1, -1, dtype=np.uint8) << 4)
        w = oracle.dequantize(MXFP4, blk[None, :], 32).reshape(-1).astype(np.float64)
        codes = np.concatenate([np.arange(16), np.arange(15, -1, -1)])
        want = np.array([(-1 if c & 8 else 1) * E2M1[c & 7] for c in codes]) * 2.0 ** (e - 127)
        assert np.array_equal(w, want.astype(np.float32).astype(np.float64)), e
        assert np.array_equal(npref.dequant(MXFP4, blk).astype(np.float32), w.astype(np.float32))
    assert oracle.lib().ref_e8m0_to_fp32_half(0) == 2.0 ** -128 and oracle.lib().ref_e8m0_to_fp32_half(200) == 2.0 ** 72


def test_block_layout_is_what_the_reference_converter_writes():
    """the converter takes blocks whose byte i holds elements 2i (low nibble) and 2i + 1 (high nibble), shuffles every 16
    bytes so that byte p holds elements p (low) and p + 16 (high), and puts the scale byte in front"""
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 16, 32).astype(np.uint8)                 # the 32 elements of a block, in order
    hf = codes[0::2] | (codes[1::2] << 4)                            # the checkpoint's bytes
    tmp = np.zeros(16, np.uint8)
    for j in range(8):                                               # convert_gptoss.go:229-235
        a, b = int(hf[j]), int(hf[j + 8])
        tmp[2 * j] = (a & 0x0F) | ((b << 4) & 0xFF)
        tmp[2 * j + 1] = (a >> 4) | (b & 0xF0)
    blk = np.concatenate([[np.uint8(127)], tmp]).astype(np.uint8)    # scale byte first: 2^0
    w = oracle.dequantize(MXFP4, blk[None, :], 32).reshape(-1)
    want = np.array([(-1 if c & 8 else 1) * E2M1[c & 7] for c in codes], np.float32)
    assert np.array_equal(w, want)


@pytest.mark.parametrize("nb", [1, 4, 64])
def test_dot_against_fp64_and_exact_integers(nb):
    k = 32 * nb
    rng = np.random.default_rng(nb)
    raw = rng.integers(0, 256, (3, nb, 17), dtype=np.uint8)
    raw[..., 0] = rng.integers(110, 135, (3, nb))
    raw = raw.reshape(3, -1)
    x = rng.standard_normal((2, k)).astype(np.float32)
    y, xq = oracle.mul_mat(MXFP4, raw, k, 3, x, return_xq=True)
    want = npref.matmul_f64(MXFP4, raw, k, 3, Q8_0, xq, 2)
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()
    # scale 2^0 on the doubled values (e = 128), integer activations with block maximum 127: integers out
    raw3 = raw.reshape(3, nb, 17).copy()
    raw3[..., 0] = 128
    xi = rng.integers(-127, 128, (1, k)).astype(np.float32)
    xi[0, ::32] = 127
    got = oracle.mul_mat(MXFP4, raw3.reshape(3, -1), k, 3, xi)
    w = npref.dequant(MXFP4, raw3.reshape(-1)).reshape(3, k)
    assert np.array_equal(got, (xi.astype(np.float64) @ w.T).astype(np.float32))


def test_synthetic_blocks_reconstruct_their_input():
    x = (np.random.default_rng(2).standard_normal((4, 256)) * 0.02).astype(np.float32)
    back = oracle.dequantize(MXFP4, synth.encode_mxfp4(x), 256)
    amax = np.abs(x.reshape(4, 8, 32)).max(axis=2, keepdims=True)
    assert (np.abs(back - x).reshape(4, 8, 32) <= amax / 3 + 1e-12).all()   # E2M1 steps are at most a third of the top value
