"""The numpy weight generators used by bench.py / smoke(): blocks must be valid (decode through the
independent numpy statement of the formats and through the oracle's dequantizer identically) and
close to the values they encode."""
import time

import numpy as np
import pytest

import npref
import oracle
from ollama_amd import synth


@pytest.mark.parametrize("t,bound", [(2, 0.14), (8, 0.008), (12, 0.12), (14, 0.04)])
def test_synthetic_blocks_are_valid_and_close(t, bound):
    rng = np.random.default_rng(t)
    k, m = 1024, 16
    x = rng.standard_normal((m, k)).astype(np.float32) * np.float32(0.02)
    raw = synth.ENCODERS[t](x)
    assert raw.shape == (m, oracle.row_size(t, k)) and raw.dtype == np.uint8
    deq = npref.dequant(t, raw).reshape(m, k)
    assert np.allclose(oracle.dequantize(t, raw, k), deq, rtol=3e-7, atol=0)
    rel = float(np.sqrt(np.mean((deq - x) ** 2) / np.mean(x.astype(np.float64) ** 2)))
    assert rel < bound, rel
    z = synth.ENCODERS[t](np.zeros((1, k), np.float32))
    assert not npref.dequant(t, z).any()


def test_weights_deterministic_and_fast_enough():
    t0 = time.time()
    a = synth.weights(12, 512, 4096, seed=5)
    b = synth.weights(12, 512, 4096, seed=5)
    assert np.array_equal(a, b) and a.shape == (512, 2304)
    assert time.time() - t0 < 20
