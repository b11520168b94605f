"""Mulmat and MulmatID on MXFP4 weights (the expert tensors of gpt-oss files) through the C ABI against the oracle.  The
library keeps such a tensor as the Q8_0 planes with the same dot products, so every Q8_0 kernel and entry point serves it."""
import numpy as np
import pytest

import npref
import oracle
from ollama_amd import qmm, synth
from oracle import MXFP4, Q8_0

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = qmm.Context(0)
    yield c
    c.close()


def _random_rows(m, k, seed, lo=110, hi=135):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, (m, k // 32, 17), dtype=np.uint8)
    raw[..., 0] = rng.integers(lo, hi, (m, k // 32))
    return raw.reshape(m, -1)


@pytest.mark.parametrize("m,k,n", [(64, 256, 1), (2880, 2880 // 32 * 32, 1), (512, 4096, 2), (512, 4096, 4), (300, 2048, 8),
                                   (256, 4096, 20), (1024, 4096, 130), (4096, 4096, 1), (5760, 2880 // 32 * 32, 512)])
def test_mxfp4_against_the_oracle(ctx, m, k, n):
    print(f"mxfp4 case m={m} k={k} n={n}", flush=True)
    raw = _random_rows(m, k, seed=m + k + n) if m * k <= 1 << 22 else synth.weights(MXFP4, m, k, seed=m)
    x = np.random.default_rng(n + k).standard_normal((n, k)).astype(np.float32)
    W = ctx.upload(MXFP4, raw, k, m)
    try:
        assert (W.type, W.k, W.m) == (MXFP4, k, m)
        y = ctx.mulmat(W, x)
        ref, xq = oracle.mul_mat(MXFP4, raw, k, m, x, nthreads=8, return_xq=True)
        assert np.array_equal(ctx.quantize_act(Q8_0, x), xq)
        assert npref.rel_err(y, ref) <= 1e-3
        if m * n <= 1 << 16:
            assert npref.rel_err(y, npref.matmul_f64(MXFP4, raw, k, m, Q8_0, xq, n), floor=1e-3) <= 1e-3
    finally:
        W.free()


def test_mxfp4_scales_at_the_edges_of_what_the_planes_hold(ctx):
    """e = 104 (a subnormal half), 113 / 114 (the last subnormal, the first normal), 143 (the largest half), 144 .. 146
    (the integers shifted instead): exact on every kernel; below 104 the matrix-core kernels see a zero block; above 146 the
    upload is refused"""
    k, m = 64, 16
    x = np.random.default_rng(1).integers(-127, 128, (2, k)).astype(np.float32)
    x[:, ::32] = 127
    x8 = np.tile(x, (4, 1))
    for e in (104, 105, 113, 114, 127, 128, 143, 144, 146):
        raw = _random_rows(m, k, seed=e).reshape(m, 2, 17)
        raw[..., 0] = e
        W = ctx.upload(MXFP4, raw.reshape(m, -1), k, m)
        y, y8 = ctx.mulmat(W, x), ctx.mulmat(W, x8)   # the streaming kernel (the tensor's own layout), the matrix cores (Q8_0 planes)
        W.free()
        w = npref.dequant(MXFP4, raw.reshape(-1)).reshape(m, k)
        assert np.array_equal(y, (x.astype(np.float64) @ w.T).astype(np.float32)), e   # integers times a power of two
        assert np.array_equal(y8, (x8.astype(np.float64) @ w.T).astype(np.float32)), e
    # below 104 the Q8_0 planes hold a zero block (weights under 7.2e-7); the streaming kernels read the tensor in its own
    # layout and still multiply it exactly
    raw = _random_rows(m, k, seed=3).reshape(m, 2, 17)
    raw[..., 0] = 100
    W = ctx.upload(MXFP4, raw.reshape(m, -1), k, m)
    w = npref.dequant(MXFP4, raw.reshape(-1)).reshape(m, k)
    assert ctx.route(W, 2) == "gemv_f32" and np.array_equal(ctx.mulmat(W, x), (x.astype(np.float64) @ w.T).astype(np.float32))
    x8 = np.tile(x, (4, 1))
    assert ctx.route(W, 8) == "skinny32" and not ctx.mulmat(W, x8).any()
    W.free()
    raw[3, 1, 0] = 147
    with pytest.raises(qmm.QmmError) as err:
        ctx.upload(MXFP4, raw.reshape(m, -1), k, m)
    assert err.value.code == qmm.ERR_UNSUPPORTED


def test_mxfp4_expert_stacks_and_joint_calls(ctx):
    """the entry points a Q8_0 weight goes through: the expert-indexed product (gpt-oss: 4 of 32 experts), the joint call,
    the two-phase form, the fused producers"""
    k, m, n_exp, n_used = 2880 // 32 * 32, 96, 8, 4
    raw = _random_rows(m * n_exp, k, seed=11)
    W = ctx.upload(MXFP4, raw, k, m * n_exp)
    try:
        for tokens in (1, 5, 70):
            rng = np.random.default_rng(tokens)
            b = rng.standard_normal((tokens, 1, k)).astype(np.float32)
            ids = np.stack([rng.permutation(n_exp)[:n_used] for _ in range(tokens)]).astype(np.int32)
            y = ctx.mulmat_id(W, n_exp, b, ids)
            ref = oracle.mul_mat_id(MXFP4, raw, k, m, n_exp, b, ids)
            assert npref.rel_err(y.reshape(ref.shape), ref) <= 1e-3, tokens
        x = np.random.default_rng(9).standard_normal((3, k)).astype(np.float32)
        W2 = ctx.upload(MXFP4, raw[:200], k, 200)
        W8 = ctx.upload(Q8_0, synth.weights(Q8_0, 64, k, seed=2), k, 64)
        ya, yb = ctx.mulmat_multi([W2, W8], x)
        assert np.array_equal(ya, ctx.mulmat(W2, x)) and np.array_equal(yb, ctx.mulmat(W8, x))
        # rows of 2880 are kept padded to 3072: the forms that read activations somebody else quantized are refused
        act = ctx.act_create(Q8_0, k, 3)
        ctx.act_quantize(act, x)
        for call in (lambda: ctx.mulmat_q8(W2, act), lambda: ctx.mulmat_produced([W2], qmm.PRODUCE_RMSNORM, None, x, 1e-5)):
            with pytest.raises(qmm.QmmError) as err:
                call()
            assert err.value.code == qmm.ERR_UNSUPPORTED
        act.free(); W2.free(); W8.free()
        # rows of whole 256-element steps: every entry point of a Q8_0 weight
        k2 = 2048
        raw2 = _random_rows(200, k2, seed=12)
        x2 = np.random.default_rng(10).standard_normal((3, k2)).astype(np.float32)
        W3 = ctx.upload(MXFP4, raw2, k2, 200)
        act = ctx.act_create(Q8_0, k2, 3)
        ctx.act_quantize(act, x2)
        assert np.array_equal(ctx.mulmat_q8(W3, act), ctx.mulmat(W3, x2))
        g = (1 + 0.1 * np.random.default_rng(4).standard_normal(k2)).astype(np.float32)
        yn, = ctx.mulmat_produced([W3], qmm.PRODUCE_RMSNORM, g, x2, 1e-5)
        want = oracle.mul_mat(MXFP4, raw2, k2, 200, oracle.rms_norm(x2, g, 1e-5))
        assert npref.rel_err(yn, want) <= 1e-3
        act.free(); W3.free()
    finally:
        W.free()


def test_python_mirror_on_a_gpt_oss_shaped_expert_block():
    """rows of 2880 (kept padded on the device): expert stacks through MulmatID at decode and prefill size, and a dense
    MXFP4 matrix beside a Q8_0 one reading the same activations"""
    from ollama_amd import ml
    k, m, n_exp, n_used = 2880, 64, 8, 4
    raw_e = _random_rows(m * n_exp, k, seed=21)
    raw_d = _random_rows(96, k, seed=22)
    raw_8 = synth.weights(Q8_0, 40, k, seed=23)
    b = ml.Backend({"blk.0.ffn_gate_up_exps.weight": (MXFP4, [k, m, n_exp], raw_e), "dense.weight": (MXFP4, [k, 96], raw_d),
                    "other.weight": (Q8_0, [k, 40], raw_8)})
    b.Load()
    try:
        assert b.Get("dense.weight").DType() == ml.DType.MXFP4
        for tokens in (1, 40):
            rng = np.random.default_rng(tokens)
            xs = rng.standard_normal((tokens, k)).astype(np.float32)
            ids = np.stack([rng.permutation(n_exp)[:n_used] for _ in range(tokens)]).astype(np.int32)
            ctx = b.NewContext()
            x = ctx.FromFloats(xs.reshape(-1), k, 1, tokens)
            e = b.Get("blk.0.ffn_gate_up_exps.weight").MulmatID(ctx, x, ctx.FromInts(ids.reshape(-1), n_used, tokens))
            x2 = ctx.FromFloats(xs.reshape(-1), k, tokens)
            d = b.Get("dense.weight").Mulmat(ctx, x2)
            o = b.Get("other.weight").Mulmat(ctx, x2)
            ctx.Compute(e, d, o)
            want_e = oracle.mul_mat_id(MXFP4, raw_e, k, m, n_exp, xs.reshape(tokens, 1, k), ids)
            assert npref.rel_err(e.Floats().reshape(want_e.shape), want_e) <= 1e-3
            assert npref.rel_err(d.Floats().reshape(tokens, 96), oracle.mul_mat(MXFP4, raw_d, k, 96, xs)) <= 1e-3
            assert npref.rel_err(o.Floats().reshape(tokens, 40), oracle.mul_mat(Q8_0, raw_8, k, 40, xs)) <= 1e-3
            ctx.Close()
    finally:
        b.Close()


def test_expert_stack_from_a_gguf_file(tmp_path):
    """a 3-D MXFP4 tensor [K, M, experts] in a file: opened by the C reader, uploaded from the mapping, multiplied by MulmatID"""
    from ollama_amd import gguf, ml
    k, m, n_exp, n_used, tokens = 2880, 32, 4, 2, 3
    raw_e = _random_rows(m * n_exp, k, seed=31)
    p = str(tmp_path / "experts.gguf")
    gguf.write_gguf(p, {"general.architecture": "gptoss"}, [("blk.0.ffn_down_exps.weight", MXFP4, [k, m, n_exp], raw_e.tobytes())])
    b = ml.Backend(p)
    b.Load()
    try:
        rng = np.random.default_rng(32)
        xs = rng.standard_normal((tokens, k)).astype(np.float32)
        ids = np.stack([rng.permutation(n_exp)[:n_used] for _ in range(tokens)]).astype(np.int32)
        ctx = b.NewContext()
        e = b.Get("blk.0.ffn_down_exps.weight").MulmatID(ctx, ctx.FromFloats(xs.reshape(-1), k, 1, tokens),
                                                        ctx.FromInts(ids.reshape(-1), n_used, tokens))
        ctx.Compute(e)
        want = oracle.mul_mat_id(MXFP4, raw_e, k, m, n_exp, xs.reshape(tokens, 1, k), ids)
        assert npref.rel_err(e.Floats().reshape(want.shape), want) <= 1e-3
        ctx.Close()
    finally:
        b.Close()
