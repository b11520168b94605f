"""The entry point that allocates nothing (mi_qmm_mulmat_noalloc) against mi_qmm_mulmat, through the C ABI.

Same kernels, so the results are the same bits, except where mi_qmm_mulmat cuts K into slices for the tiled
GEMM (the no-allocation call never does): there the fp32 sums are added in another order and the parity bar
of the product applies (1e-3 on |y-ref| / max(|ref|, 1e-2*rms)).  Every case makes two calls in a row on the
same static scratch, the second with fewer rows, and both must match.
"""
import numpy as np
import pytest

import npref
from hipmem import DeviceArray, free_bytes
from npref import Q4_0, Q4_K, Q6_K, Q8_0
from ollama_amd import qmm, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _both(ctx, W, x):
    """(mi_qmm_mulmat, mi_qmm_mulmat_noalloc) on device pointers for activations x [n, k]"""
    n = x.shape[0]
    dx = DeviceArray(x)
    y0 = DeviceArray(np.empty((n, W.m), np.float32), zero=True)
    y1 = DeviceArray(np.empty((n, W.m), np.float32), zero=True)
    try:
        ctx.mulmat_device(W, dx.ptr, n, y0.ptr)
        ctx.mulmat_noalloc_device(W, dx.ptr, n, y1.ptr)
        ctx.sync()
        return y0.numpy(), y1.numpy()
    finally:
        dx.free(); y0.free(); y1.free()


# (type, m, k, first n, second n, bit-identical expected)
CASES = [
    (Q4_K, 1024, 4096, 1, 1, True),        # decode: in-kernel quantization, no scratch
    (Q4_K, 1024, 4096, 8, 3, True),        # skinny kernels on the static planes
    (Q6_K, 768, 2048, 16, 5, True),
    (Q4_0, 512, 4096, 8, 4, True),
    (Q8_0, 512, 4096, 40, 33, True),       # block-32 GEMM
    (Q4_K, 1536, 4096, 300, 130, True),    # tiled GEMM, rows past n in the last tile keep the first call's quants
    (Q6_K, 512, 14336, 512, 64, False),    # mi_qmm_mulmat may cut K here; the no-allocation call does not
    (Q4_K, 14336, 4096, 512, 200, True),   # fp16-MFMA GEMM: the fp16 planes carved out of the static scratch
    (Q6_K, 14336, 4096, 512, 200, False),  # Q6_K 256-row GEMM; at 200 columns mi_qmm_mulmat cuts K, this call does not
    (Q6_K, 4096, 14336, 512, 200, False),  # K slices would need workspace: falls back to the 128-row kernel without it
    (Q4_K, 14336, 4096, 4, 3, True),       # a few columns on a large matrix: the workgroups quantize x, no scratch
    (Q4_K, 4096, 14336, 8, 5, True),       # the same kernel on planes in the static scratch
    (1, 512, 4096, 8, 3, True),            # F16 weights at a few columns: no scratch (the activations are converted into LDS)
    (30, 384, 2048, 200, 64, True),        # BF16 on the tiles: the converted activations in the static scratch
    (0, 384, 2048, 200, 40, True),         # F32 on the tiles: no conversion, no scratch
    (13, 256, 2048, 70, 5, False),         # Q5_K: [x | x] at the end of the static scratch, the Q8_K planes in front of it
    (13, 1024, 4096, 6, 3, True),          # Q5_K at a few rows: the blocks as they are against Q8_K planes in the static scratch
    (39, 128, 2880, 40, 3, True),          # MXFP4 with rows padded to 3072: [x | 0] at the end of the static scratch
]


@pytest.mark.parametrize("t,m,k,n1,n2,same_bits", CASES)
def test_noalloc_matches_mulmat_on_two_calls_in_a_row(ctx, t, m, k, n1, n2, same_bits):
    W = ctx.upload(t, synth.weights(t, m, k, seed=41 + t), k, m)
    rng = np.random.default_rng(1000 * t + n1)
    try:
        for n in (n1, n2):
            print(f"noalloc case type={t} m={m} k={k} n={n}", flush=True)
            x = rng.standard_normal((n, k), dtype=np.float32)
            want, got = _both(ctx, W, x)
            assert np.isfinite(got).all()
            if same_bits:
                assert np.array_equal(got, want), f"n={n}: {np.count_nonzero(got != want)} values differ"
            else:
                assert npref.rel_err(got, want) <= 1e-3
    finally:
        W.free()


def test_noalloc_rejects_what_does_not_fit_and_allocates_nothing(ctx):
    k, m = 14336, 256
    W = ctx.upload(Q4_K, synth.weights(Q4_K, m, k, seed=7), k, m)
    n = 1024  # 1024 x 14336 Q8_K planes: about 20 MB, more than the static scratch holds
    dx = DeviceArray(np.zeros((n, k), np.float32))
    dy = DeviceArray(np.empty((n, m), np.float32), zero=True)
    try:
        with pytest.raises(qmm.QmmError) as e:
            ctx.mulmat_noalloc_device(W, dx.ptr, n, dy.ptr)
        assert e.value.code == qmm.ERR_UNSUPPORTED and "static scratch" in str(e.value)
        # with the ctx's own scratch frozen at its present size the call still works: it never touches it
        ctx.scratch_freeze(True)
        try:
            ctx.mulmat_noalloc_device(W, dx.ptr, 64, dy.ptr)
            ctx.sync()
            with pytest.raises(qmm.QmmError) as e2:   # the growable path would need a larger buffer now
                big = DeviceArray(np.zeros((4096, k), np.float32))
                bigy = DeviceArray(np.empty((4096, m), np.float32), zero=True)
                try:
                    ctx.mulmat_device(W, big.ptr, 4096, bigy.ptr)
                finally:
                    ctx.sync()
                    big.free(); bigy.free()
            assert e2.value.code == qmm.ERR_INVALID and "frozen" in str(e2.value)
        finally:
            ctx.scratch_freeze(False)
    finally:
        W.free(); dx.free(); dy.free()


def test_noalloc_on_a_fresh_ctx_with_frozen_scratch(ctx):
    """A ctx that has never multiplied holds no scratch at all; with its scratch frozen every attempt to reserve any
    fails.  mi_qmm_mulmat_noalloc must still run every kind of product -- streaming GEMV, the kernels for a few columns,
    the tiled GEMMs -- and the device's free memory must not move.  Expected values from the module's own ctx."""
    fresh = qmm.Context(0)
    try:
        fresh.scratch_freeze(True)
        shapes = [(Q4_K, 1024, 4096, (1, 8)), (Q6_K, 768, 2048, (16,)), (Q8_0, 512, 4096, (2, 40)), (Q4_K, 14336, 4096, (4, 300)),
                  (Q6_K, 4096, 14336, (512,))]
        for t, m, k, ns in shapes:
            raw = synth.weights(t, min(m, 1024), k, seed=90 + t)
            raw = np.tile(raw, ((m + raw.shape[0] - 1) // raw.shape[0], 1))[:m]
            W, Wf = ctx.upload(t, raw, k, m), fresh.upload(t, raw, k, m)
            rng = np.random.default_rng(17 * t + m)
            for n in ns:
                print(f"fresh frozen ctx: type={t} m={m} k={k} n={n}", flush=True)
                x = rng.standard_normal((n, k), dtype=np.float32)
                dx = DeviceArray(x)
                y0 = DeviceArray(np.empty((n, m), np.float32), zero=True)
                y1 = DeviceArray(np.empty((n, m), np.float32), zero=True)
                try:
                    ctx.mulmat_device(W, dx.ptr, n, y0.ptr)
                    ctx.sync()
                    before = free_bytes()
                    fresh.mulmat_noalloc_device(Wf, dx.ptr, n, y1.ptr)
                    fresh.sync()
                    assert free_bytes() == before, "device memory moved during mi_qmm_mulmat_noalloc"
                    assert npref.rel_err(y1.numpy(), y0.numpy()) <= 1e-3
                    with pytest.raises(qmm.QmmError):   # the growable path cannot even start on this ctx
                        fresh.mulmat_device(Wf, dx.ptr, max(n, 9), y1.ptr)
                finally:
                    fresh.sync()
                    dx.free(); y0.free(); y1.free()
            W.free(); Wf.free()
    finally:
        fresh.scratch_freeze(False)
        fresh.close()
