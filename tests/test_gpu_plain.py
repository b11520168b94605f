"""Mulmat on F32 / F16 / BF16 weights (the unquantized tensors of a GGUF file) through the C ABI, against the oracle.

The oracle adds fp32 products in double, the kernels in fp32: the comparison is the path's tolerance (1e-3 on
max |y - ref| / max(|ref|, 1e-2 rms)); observed differences are a few 1e-6.
"""
import numpy as np
import pytest

import npref
import oracle
from hipmem import DeviceArray
from ollama_amd import qmm
from oracle import BF16, F16, F32

pytestmark = pytest.mark.gpu

NAMES = {F32: "F32", F16: "F16", BF16: "BF16"}


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _weights(t, m, k, seed, scale=0.05):
    """random weights of type t as (bytes [m, row_size], the same values in f32)"""
    w = (np.random.default_rng(seed).standard_normal((m, k)) * scale).astype(np.float32)
    raw = oracle.quantize(t, w)  # conversion of the rows to the type: the tensor's bytes
    return raw, w


# (rows, K, activation rows): every kernel and both sides of each switch
#   matrix-core streaming kernel (1..16 columns, one to sixteen K segments per row group, ragged last segments and row
#   groups); vector-ALU streaming kernel where the activations do not fit the LDS, x in chunks; rounds with dead waves;
#   tiles of 128 x 32 and 128 x 128 with ragged edges; rows of 16-byte but not 64-byte multiples (8 columns per launch);
#   the feed-forward shapes at decode size, a prefill-sized product, long rows on the tiles; odd K (a wave per output)
SHAPES = [
    (512, 4096, 1), (512, 4096, 2), (515, 4096, 3), (77, 4096, 8), (1, 256, 1), (33, 64, 5), (5000, 2048, 16),
    (70000, 256, 2), (40, 4096 + 64, 7), (16, 64 * 9, 11),
    (256, 14336, 1), (256, 14336, 4), (200, 14336, 8), (96, 40960, 2),
    (512, 4096, 9), (300, 4096, 32), (515, 1024, 33), (130, 2048, 130), (1000, 512, 257),
    (14336, 4096, 1), (4096, 14336, 4), (2048, 4096, 128), (256, 14336, 64), (6200, 512, 1000),
    (64, 72, 3), (64, 72, 20), (50, 70, 1), (50, 70, 12), (9, 1, 2), (40, 1001, 3),
]


@pytest.mark.parametrize("t", [F32, F16, BF16], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_plain_weights_against_the_oracle(ctx, t, m, k, n):
    print(f"plain case type={NAMES[t]} m={m} k={k} n={n}", flush=True)
    raw, _ = _weights(t, m, k, seed=1000 + 7 * t + m + k)
    x = np.random.default_rng(2000 + n + k).standard_normal((n, k)).astype(np.float32)
    W = ctx.upload(t, raw, k, m)
    try:
        y = ctx.mulmat(W, x)
        ref = oracle.mul_mat(t, raw, k, m, x, nthreads=4)
        assert y.shape == ref.shape == (n, m)
        err = npref.rel_err(y, ref)
        assert err <= 1e-3, err
        assert err <= 3e-4, f"looser than this kernel has ever been: {err}"
    finally:
        W.free()


def _expected_route(t, m, k, n):
    row = k * (4 if t == F32 else 2)
    if n <= 16 and row % 64 == 0 and (256 + n * (row + 16) + 15) // 16 * 16 + 16384 <= 160 * 1024:
        return "plain_skinny"  # the converted activations fit the LDS
    if n <= 8 and row % 16 == 0:
        return "plain_gemv"
    if row % 64 == 0:
        return "plain_gemm"
    return "plain_gemv" if row % 16 == 0 else "plain_naive"


@pytest.mark.parametrize("t", [F32, F16, BF16], ids=lambda t: NAMES[t])
def test_plain_routes(ctx, t):
    for m, k, n in SHAPES:
        raw, _ = _weights(t, min(m, 8), k, seed=1)
        W = ctx.upload(t, np.tile(raw, ((m + 7) // 8, 1))[:m], k, m)
        try:
            assert ctx.route(W, n) == _expected_route(t, m, k, n), (m, k, n)
        finally:
            W.free()


@pytest.mark.parametrize("t", [F32, F16, BF16], ids=lambda t: NAMES[t])
def test_plain_small_integers_are_exact(ctx, t):
    """integers up to 256 are exact in all three types and every partial sum stays below 2^24: the results are the
    integer dot products whatever the order of the sums -- on the streaming kernel, the tiles and the wave per output"""
    rng = np.random.default_rng(77 + t)
    for m, k, n in ((70, 512, 3), (130, 256, 40), (20, 33, 2)):
        print(f"plain integers type={NAMES[t]} m={m} k={k} n={n}", flush=True)
        w = rng.integers(-15, 16, (m, k)).astype(np.float32)
        x = rng.integers(-256, 257, (n, k)).astype(np.float32)
        W = ctx.upload(t, oracle.quantize(t, w), k, m)
        try:
            y = ctx.mulmat(W, x)
            assert np.array_equal(y, (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))
        finally:
            W.free()


def test_f16_subnormal_weights_are_multiplied_not_flushed(ctx):
    """weights below the smallest normal half (6.1e-5) and activations that convert to subnormal halves: the matrix cores
    (1..16 columns and the tiles) and the vector-ALU kernel multiply them, none flushes them to zero"""
    m, k = 64, 1024
    w = (np.random.default_rng(3).standard_normal((m, k)) * 2e-6).astype(np.float32)
    raw = oracle.quantize(F16, w)
    assert np.count_nonzero(raw.view(np.uint16) & 0x7C00) == 0  # every weight is subnormal (or zero)
    W = ctx.upload(F16, raw, k, m)
    try:
        for n, scale in ((2, 1.0), (40, 1.0), (2, 1e-5)):
            x = (np.random.default_rng(4 + n).standard_normal((n, k)) * scale).astype(np.float32)
            ref = oracle.mul_mat(F16, raw, k, m, x)
            assert np.abs(ref).max() > 0
            for path in (qmm.PATH_AUTO, qmm.PATH_GEMV, qmm.PATH_GEMM):
                assert npref.rel_err(ctx.mulmat(W, x, path), ref) <= 1e-3, (n, scale, path)
    finally:
        W.free()


@pytest.mark.parametrize("t", [F32, F16, BF16], ids=lambda t: NAMES[t])
def test_plain_device_pointers_noalloc_and_forced_paths(ctx, t):
    m, k = 384, 2048
    raw, _ = _weights(t, m, k, seed=5 + t)
    W = ctx.upload(t, raw, k, m)
    try:
        for n in (1, 8, 9, 200):
            print(f"plain device type={NAMES[t]} n={n}", flush=True)
            x = np.random.default_rng(n).standard_normal((n, k)).astype(np.float32)
            want = ctx.mulmat(W, x)
            dx, dy = DeviceArray(x), DeviceArray(np.zeros((n, m), np.float32), zero=True)
            dz = DeviceArray(np.zeros((n, m), np.float32), zero=True)
            ctx.mulmat_device(W, dx.ptr, n, dy.ptr)
            ctx.mulmat_noalloc_device(W, dx.ptr, n, dz.ptr)
            ctx.sync()
            assert np.array_equal(dy.numpy(), want) and np.array_equal(dz.numpy(), want)
            # forced paths: the streaming kernel at any n, the tiles at any n
            ref = oracle.mul_mat(t, raw, k, m, x, nthreads=4)
            assert npref.rel_err(ctx.mulmat(W, x, qmm.PATH_GEMV), ref) <= 3e-4
            assert npref.rel_err(ctx.mulmat(W, x, qmm.PATH_GEMM), ref) <= 3e-4
            for d in (dx, dy, dz):
                d.free()
    finally:
        W.free()


def test_plain_noalloc_refuses_what_its_scratch_cannot_hold(ctx):
    m, k, n = 128, 8192, 2048  # 2048 x 8192 halves: 32 MiB of converted activations
    raw, _ = _weights(F16, m, k, seed=2)
    W = ctx.upload(F16, raw, k, m)
    dx, dy = DeviceArray(np.zeros((n, k), np.float32), zero=True), DeviceArray(np.zeros((n, m), np.float32), zero=True)
    try:
        with pytest.raises(qmm.QmmError) as e:
            ctx.mulmat_noalloc_device(W, dx.ptr, n, dy.ptr)
        assert e.value.code == qmm.ERR_UNSUPPORTED
        # F32 weights need no converted copy: the same shape goes through
        raw32, _ = _weights(F32, m, k, seed=2)
        W32 = ctx.upload(F32, raw32, k, m)
        ctx.mulmat_noalloc_device(W32, dx.ptr, n, dy.ptr)
        ctx.sync()
        assert not dy.numpy().any()
        W32.free()
    finally:
        W.free()
        dx.free()
        dy.free()


def test_plain_weights_in_joint_calls_and_where_they_are_refused(ctx):
    k = 1024
    raw16, _ = _weights(F16, 96, k, seed=11)
    rawbf, _ = _weights(BF16, 40, k, seed=12)
    Wa, Wb = ctx.upload(F16, raw16, k, 96), ctx.upload(BF16, rawbf, k, 40)
    from ollama_amd import synth
    rawq = synth.weights(qmm.Q4_K, 64, k, seed=13)
    Wq = ctx.upload(qmm.Q4_K, rawq, k, 64)
    try:
        x = np.random.default_rng(14).standard_normal((3, k)).astype(np.float32)
        ya, yq, yb = ctx.mulmat_multi([Wa, Wq, Wb], x)
        assert np.array_equal(ya, ctx.mulmat(Wa, x)) and np.array_equal(yb, ctx.mulmat(Wb, x))
        assert np.array_equal(yq, ctx.mulmat(Wq, x))
        for call in (lambda: ctx.mulmat_produced([Wa], qmm.PRODUCE_RMSNORM, None, x, 1e-5),
                     lambda: ctx.mulmat_swiglu(Wa, Wa, x[:1]),
                     lambda: ctx.mulmat_id(Wa, 2, x.reshape(3, 1, k), np.zeros((3, 1), np.int32))):
            with pytest.raises(qmm.QmmError) as e:
                call()
            assert e.value.code == qmm.ERR_UNSUPPORTED
    finally:
        for w in (Wa, Wb, Wq):
            w.free()


def test_python_mirror_multiplies_unquantized_weights_beside_quantized_ones():
    """one graph: an RMSNorm read by a Q4_K weight (folded into its launch) and by F16 / F32 / Q5_K weights (which need
    it in f32), at decode and prefill size"""
    from ollama_amd import ml, synth
    k = 1024
    rng = np.random.default_rng(21)
    raw_q = synth.weights(qmm.Q4_K, 64, k, seed=5)
    raw_h = oracle.quantize(F16, (rng.standard_normal((48, k)) * 0.05).astype(np.float32))
    raw_f = oracle.quantize(F32, (rng.standard_normal((10, k)) * 0.05).astype(np.float32))
    raw_5 = synth.weights(qmm.Q5_K, 33, k, seed=6)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    b = ml.Backend({"q.weight": (qmm.Q4_K, [k, 64], raw_q), "h.weight": (F16, [k, 48], raw_h), "r.weight": (F32, [k, 10], raw_f),
                    "v.weight": (qmm.Q5_K, [k, 33], raw_5),
                    "norm.weight": (F32, [k], g)})
    b.Load()
    try:
        for n in (1, 40):
            xs = rng.standard_normal((n, k)).astype(np.float32)
            ctx = b.NewContext()
            xn = ctx.FromFloats(xs.reshape(-1), k, n).RMSNorm(ctx, b.Get("norm.weight"), 1e-5)
            outs = {name: b.Get(name).Mulmat(ctx, xn) for name in ("q.weight", "h.weight", "r.weight", "v.weight")}
            ctx.Compute(*outs.values())
            want_x = oracle.rms_norm(xs, g, 1e-5)
            for name, t, raw, m in (("q.weight", qmm.Q4_K, raw_q, 64), ("h.weight", F16, raw_h, 48), ("r.weight", F32, raw_f, 10),
                                    ("v.weight", qmm.Q5_K, raw_5, 33)):
                want = oracle.mul_mat(t, raw, k, m, want_x)
                assert npref.rel_err(outs[name].Floats().reshape(n, m), want) <= 1e-3, (name, n)
            ctx.Close()
        with pytest.raises(TypeError):
            bad = ml.Backend({"e.weight": (F16, [k, 8, 2], oracle.quantize(F16, np.zeros((16, k), np.float32)))})
            bad.Load()
            c2 = bad.NewContext()
            bad.Get("e.weight").MulmatID(c2, c2.FromFloats(np.zeros(k, np.float32), k, 1, 1), c2.FromInts(np.zeros(1, np.int32), 1, 1))
    finally:
        b.Close()
