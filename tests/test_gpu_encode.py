"""GPU weight encoders (mi_qmm_quantize_weights) against the CPU oracle's encoders: the same bytes.

The oracle's encoders restate ggml's scalar quantize_row_{q4_0,q8_0,q4_K,q6_K}_ref from recall (their bit-parity
with a compiled llama-quantize cannot be pinned offline: oracle/ggml_ref.h says so); what is pinned here is that the
GPU kernels keep every order of those sequential fp32 loops -- running sums, first maxima, the grid searches'
"strictly better" updates -- on blocks chosen to exercise each branch.
"""
import numpy as np
import pytest

import npref
import oracle
from hipmem import DeviceArray
from npref import Q4_0, Q4_K, Q6_K, Q8_0
from ollama_amd import qmm

pytestmark = pytest.mark.gpu
WTYPES = [Q4_0, Q8_0, Q4_K, Q6_K]
NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K"}


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _same_bytes(ctx, t, x, what):
    got = ctx.quantize_weights(t, x)
    want = oracle.quantize(t, x, nthreads=16)
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        rows = np.unique(bad[:, 0])
        raise AssertionError(f"{NAMES[t]} {what}: {len(bad)} bytes differ in {len(rows)} rows, first at row {bad[0][0]} byte {bad[0][1]}: "
                             f"gpu {got[tuple(bad[0])]} oracle {want[tuple(bad[0])]}")
    return got


@pytest.mark.parametrize("t", WTYPES)
@pytest.mark.parametrize("m,k", [(1, 256), (7, 4096), (3, 512), (33, 2304), (64, 14336)])
def test_random_rows_give_the_oracle_bytes(ctx, t, m, k):
    """weights like a model's (normal, 0.02), wide ones, and heavy tails; row counts that leave workgroups partly filled"""
    rng = np.random.default_rng(9100 + t + m + k)
    for scale, tail in ((0.02, False), (3.0, False), (0.02, True)):
        x = rng.standard_normal((m, k), dtype=np.float32) * np.float32(scale)
        if tail:
            x *= (1.0 + 20.0 * (rng.random((m, k), dtype=np.float32) < 0.01)).astype(np.float32)
        _same_bytes(ctx, t, x, f"{m}x{k} scale {scale} tail {tail}")


@pytest.mark.parametrize("t", WTYPES)
def test_edge_blocks_give_the_oracle_bytes(ctx, t):
    """one super-block (or eight 32-element blocks) per case: all zero; constant; positive only (the minimum is pulled to
    zero); negative only; one spike; magnitudes below the zero threshold of the Q6_K search and far above any weight;
    a ramp (many exact ties in the rounding); equal and opposite extremes (first maximum wins); a zero sub-block among
    live ones (its scale quantizes to zero and the search's own levels stay); blocks whose later sub-blocks dominate."""
    rng = np.random.default_rng(9200 + t)
    k = 256
    cases = []
    cases.append(np.zeros(k))
    cases.append(np.full(k, 0.37))
    cases.append(np.abs(rng.standard_normal(k)) + 0.5)
    cases.append(-np.abs(rng.standard_normal(k)) - 0.5)
    spike = np.zeros(k); spike[77] = -3.25; cases.append(spike)
    cases.append(rng.standard_normal(k) * 1e-17)
    cases.append(rng.standard_normal(k) * 1e-20)
    cases.append(rng.standard_normal(k) * 1e18)
    cases.append(np.linspace(-1.0, 1.0, k))
    cases.append(np.arange(k) * 0.5 - 31.75)
    pm = rng.standard_normal(k) * 0.1; pm[5] = 2.0; pm[9] = -2.0; pm[200] = -2.0; pm[201] = 2.0; cases.append(pm)
    hole = rng.standard_normal(k); hole[64:96] = 0.0; hole[16:32] = 0.0; cases.append(hole)
    grow = rng.standard_normal(k) * np.repeat(2.0 ** np.arange(8), 32); cases.append(grow)
    tiny_sub = rng.standard_normal(k); tiny_sub[128:160] *= 1e-6; tiny_sub[32:48] *= 1e-9; cases.append(tiny_sub)
    halves = np.round(rng.standard_normal(k) * 4) / 8.0; cases.append(halves)       # values on a coarse grid: rounding ties
    x = np.stack(cases).astype(np.float32)
    _same_bytes(ctx, t, x, "edge blocks")
    # the same blocks side by side in one row, and shifted by one sub-block
    row = x.reshape(1, -1)
    _same_bytes(ctx, t, row, "edge blocks in one row")
    _same_bytes(ctx, t, np.roll(row, 32, axis=1), "edge blocks shifted")


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
def test_k_quant_blocks_follow_from_least_squares_and_rounding(ctx, t):
    """The GPU encoders' own bytes, without comparing them to the oracle's: top codes, d / dmin, the scale codes against
    the searched group scales (the search being checked against fp64 least squares in the CPU suite), every level the
    nearest one for the stored scales."""
    import encprops
    rng = np.random.default_rng(9300 + t)
    for scale in (0.02, 3.0):
        x = (rng.standard_normal((8, 2048)) * scale).astype(np.float32)
        x[1] *= (1 + 20 * (rng.random(2048) < 0.01)).astype(np.float32)
        x[2, :256] = 0; x[3] = np.abs(x[3]); x[4, 256:512] = -np.abs(x[4, 256:512]); x[5, 32:64] = 0
        raw = ctx.quantize_weights(t, x)
        (encprops.q4k_stored_bytes if t == Q4_K else encprops.q6k_stored_bytes)(x, raw)


@pytest.mark.parametrize("t", WTYPES)
def test_device_pointers_and_the_product_on_encoded_weights(ctx, t):
    """device in, device out: the same bytes; uploaded, they multiply like the oracle's own encoding of the same rows"""
    rng = np.random.default_rng(9300 + t)
    m, k = 300, 4096
    x = rng.standard_normal((m, k), dtype=np.float32) * np.float32(0.05)
    dx = DeviceArray(x)
    dout = DeviceArray(np.empty((m, qmm.row_size(t, k)), np.uint8), zero=True)
    ctx.quantize_weights_device(t, dx.ptr, k, m, dout.ptr)
    ctx.sync()
    got = dout.numpy()
    dx.free(); dout.free()
    want = oracle.quantize(t, x, nthreads=16)
    assert np.array_equal(got, want)
    w = ctx.upload(t, got.reshape(-1), k, m)
    act = rng.standard_normal((3, k), dtype=np.float32)
    assert npref.rel_err(ctx.mulmat(w, act), oracle.mul_mat(t, want.reshape(-1), k, m, act, nthreads=16)) <= 1e-3
    w.free()
    # reconstruction error of the encoding itself, per type (a wrong scale or level shows here even if both sides agreed)
    back = oracle.dequantize(t, got, k)
    rel = float(np.sqrt(np.mean((back - x) ** 2)) / np.sqrt(np.mean(x ** 2)))
    assert rel < {Q4_0: 0.12, Q8_0: 0.01, Q4_K: 0.09, Q6_K: 0.02}[t], rel


def test_host_rows_beyond_one_staging_slab(ctx):
    """host arrays larger than the 64 MiB staging slab go through in several pieces: the same bytes as row by row"""
    rng = np.random.default_rng(9400)
    m, k = 5000, 4096  # 82 MB of f32: two slabs, the second one short
    x = rng.standard_normal((m, k), dtype=np.float32) * np.float32(0.03)
    for t in (Q8_0, Q4_K):
        got = ctx.quantize_weights(t, x)
        assert np.array_equal(got, oracle.quantize(t, x, nthreads=16))


def test_empty_and_argument_errors(ctx):
    assert ctx.quantize_weights(Q4_K, np.zeros((0, 256), np.float32)).shape == (0, 144)
    with pytest.raises(qmm.QmmError):
        ctx.quantize_weights(Q4_K, np.zeros((2, 100), np.float32))
    with pytest.raises(qmm.QmmError):
        ctx.quantize_weights(npref.Q8_K, np.zeros((2, 256), np.float32))
    dx = DeviceArray(np.zeros((2, 260), np.float32))
    dout = DeviceArray(np.zeros(2 * 144 + 8, np.uint8))
    with pytest.raises(qmm.QmmError, match="aligned"):
        ctx.quantize_weights_device(Q4_K, dx.ptr + 4, 256, 2, dout.ptr)
    with pytest.raises(qmm.QmmError, match="aligned"):
        ctx.quantize_weights_device(Q4_K, dx.ptr, 256, 2, dout.ptr + 2)
    dx.free(); dout.free()
