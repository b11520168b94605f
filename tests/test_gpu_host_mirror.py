"""The host-side mirrors of the reference's ml.Backend / ml.Context / ml.Tensor interface
(/root/reference/ml/backend.go:16-33, 94-128, 130-153) driven the way a model's forward pass drives
them -- Get the weights, FromFloats the activations, Mulmat, Compute, Floats -- and checked against
the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

import npref
import oracle
from ollama_amd import qmm

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_python_mirror_layer_graph():
    from ollama_amd import ml

    k = 2048
    rng = np.random.default_rng(8)
    spec = {}
    raws = {}
    for name, t, m in [("blk.0.attn_q.weight", qmm.Q4_K, 2048), ("blk.0.attn_k.weight", qmm.Q4_K, 512),
                       ("blk.0.attn_v.weight", qmm.Q4_K, 512), ("blk.0.ffn_gate.weight", qmm.Q4_K, 1536),
                       ("blk.0.ffn_up.weight", qmm.Q4_K, 1536), ("blk.0.ffn_down.weight", qmm.Q6_K, 640),
                       ("output.weight", qmm.Q8_0, 1000), ("token_embd.weight", qmm.Q4_0, 96)]:
        raw = oracle.quantize(t, (rng.standard_normal((m, k), dtype=np.float32) * np.float32(0.02)), nthreads=8)
        spec[name] = (t, [k, m], raw)
        raws[name] = (t, m, raw)
    seen = []
    b = ml.Backend(spec)
    b.Load(progress=seen.append)
    assert seen and seen[-1] == 1.0
    assert b.Get("nope.weight") is None
    w = b.Get("output.weight")
    assert w.Shape() == [k, 1000] and w.DType() == ml.DType.Q80 and w.Dim(1) == 1000
    assert w.Stride(0) == 34 and w.Stride(1) == qmm.row_size(qmm.Q8_0, k)
    assert w.Bytes() == raws["output.weight"][2].tobytes()
    for n in (1, 5, 48):   # decode, skinny, prefill-sized (GEMM for the K-quants)
        ctx = b.NewContext()
        xv = rng.standard_normal((n, k), dtype=np.float32)
        x = ctx.FromFloats(xv.reshape(-1), k, n)
        outs = {name: b.Get(name).Mulmat(ctx, x) for name in spec}
        full = b.Get("blk.0.attn_q.weight").MulmatFullPrec(ctx, x)
        with pytest.raises(RuntimeError):
            outs["output.weight"].Floats()      # lazy until Compute
        ctx.Compute(*outs.values())
        for name, out in outs.items():
            t, m, raw = raws[name]
            assert out.Shape() == [m, n] and out.DType() == ml.DType.F32
            want = oracle.mul_mat(t, raw, k, m, xv, nthreads=8)
            assert npref.rel_err(out.Floats().reshape(n, m), want) <= 1e-3, (name, n)
        assert np.array_equal(full.Floats(), outs["blk.0.attn_q.weight"].Floats())
        ctx.Close()
    ctx = b.NewContext()
    with pytest.raises(ValueError):
        b.Get("output.weight").Mulmat(ctx, ctx.FromFloats(np.zeros(512, np.float32), 512, 1))
    with pytest.raises(TypeError):
        ctx.FromFloats(np.zeros(k, np.float32), k, 1).Mulmat(ctx, ctx.FromFloats(np.zeros(k, np.float32), k, 1))
    b.Close()


def test_python_mirror_ffn_block_with_producers():
    """x -> RMSNorm -> gate, up -> SILU(gate, up) -> down, the way a model's feed-forward block drives the
    interface (/root/reference/ml/backend.go:159, :180).  The norm and the gating run inside the products'
    quantization unless their values are asked for."""
    from ollama_amd import ml

    k, f = 1024, 1536
    rng = np.random.default_rng(18)
    mats = {"blk.0.ffn_gate.weight": (qmm.Q4_K, k, f), "blk.0.ffn_up.weight": (qmm.Q4_K, k, f),
            "blk.0.ffn_down.weight": (qmm.Q6_K, f, k)}
    spec, raws = {}, {}
    for name, (t, kk, m) in mats.items():
        raw = oracle.quantize(t, (rng.standard_normal((m, kk), dtype=np.float32) * np.float32(0.05)), nthreads=8)
        spec[name] = (t, [kk, m], raw)
        raws[name] = raw
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    spec["blk.0.ffn_norm.weight"] = (qmm.F32, [k], g)
    b = ml.Backend(spec)
    b.Load()
    assert np.array_equal(b.Get("blk.0.ffn_norm.weight").Floats(), g)
    for n in (1, 6, 40):
        xv = rng.standard_normal((n, k), dtype=np.float32)
        ctx = b.NewContext()
        x = ctx.FromFloats(xv.reshape(-1), k, n)
        h = x.RMSNorm(ctx, b.Get("blk.0.ffn_norm.weight"), 1e-5)
        gate = b.Get("blk.0.ffn_gate.weight").Mulmat(ctx, h)
        up = b.Get("blk.0.ffn_up.weight").Mulmat(ctx, h)
        act = gate.SILU(ctx, up)
        out = b.Get("blk.0.ffn_down.weight").Mulmat(ctx, act)
        ctx.Compute(out)
        # one row: norm, both products and the gating were one call, only the gated values exist; more rows: the
        # norm ran inside the quantization of gate / up and the gating inside that of down
        for lazy in ((h, gate, up) if n == 1 else (h, act)):
            with pytest.raises(RuntimeError):
                lazy.Floats()
        hv = oracle.rms_norm(xv, g, 1e-5)
        gv = oracle.mul_mat(qmm.Q4_K, raws["blk.0.ffn_gate.weight"], k, f, hv, nthreads=8)
        uv = oracle.mul_mat(qmm.Q4_K, raws["blk.0.ffn_up.weight"], k, f, hv, nthreads=8)
        actv = act.Floats().reshape(n, f) if n == 1 else oracle.swiglu(gate.Floats().reshape(n, f), up.Floats().reshape(n, f))
        assert npref.rel_err(actv, oracle.swiglu(gv, uv)) <= 1e-3
        # the oracle's down projection on the GPU's own gated values: isolates the last step
        want = oracle.mul_mat(qmm.Q6_K, raws["blk.0.ffn_down.weight"], f, k, actv, nthreads=8)
        assert npref.rel_err(out.Floats().reshape(n, k), want) <= 1e-3, n
        # and the whole chain on the CPU
        chain = oracle.mul_mat(qmm.Q6_K, raws["blk.0.ffn_down.weight"], f, k, oracle.swiglu(gv, uv), nthreads=8)
        assert npref.rel_err(out.Floats().reshape(n, k), chain) <= 2e-3, n
        # asking for the intermediate values gives the same result through the separate kernels
        ctx2 = b.NewContext()
        x2 = ctx2.FromFloats(xv.reshape(-1), k, n)
        h2 = x2.RMSNorm(ctx2, b.Get("blk.0.ffn_norm.weight"), 1e-5)
        gate2 = b.Get("blk.0.ffn_gate.weight").Mulmat(ctx2, h2)
        up2 = b.Get("blk.0.ffn_up.weight").Mulmat(ctx2, h2)
        act2 = gate2.SILU(ctx2, up2)
        out2 = b.Get("blk.0.ffn_down.weight").Mulmat(ctx2, act2)
        ctx2.Compute(h2, gate2, act2, out2)
        assert h2.Shape() == [k, n] and np.max(np.abs(h2.Floats().reshape(n, k) - hv)) < 1e-5
        assert npref.rel_err(gate2.Floats().reshape(n, f), gv) <= 1e-3
        assert np.array_equal(out2.Floats(), out.Floats())
        if n == 1:
            assert np.array_equal(act2.Floats(), act.Floats())
        # down reads the gating node alone (no gate / up pair to absorb): the gating runs inside its quantization
        ctx3 = b.NewContext()
        ga, ua = ctx3.FromFloats(gate2.Floats(), f, n), ctx3.FromFloats(up2.Floats(), f, n)
        a3 = ga.SILU(ctx3, ua)
        out3 = b.Get("blk.0.ffn_down.weight").Mulmat(ctx3, a3)
        ctx3.Compute(out3)
        with pytest.raises(RuntimeError):
            a3.Floats()
        assert np.array_equal(out3.Floats(), out.Floats())
        ctx3.Close()
        ctx.Close(); ctx2.Close()
    ctx = b.NewContext()
    # the bare activation SILU(ctx): an f32 node of its own, also in front of a product
    v = np.random.default_rng(3).standard_normal(k).astype(np.float32)
    bare = ctx.FromFloats(v, k, 1).SILU(ctx)
    ctx.Compute(bare)
    want = v.astype(np.float64) / (1.0 + np.exp(-v.astype(np.float64)))
    assert np.max(np.abs(bare.Floats() - want)) <= 1e-6
    with pytest.raises(TypeError):
        ctx.FromFloats(v, k, 1).SILU(ctx, bare, bare)
    with pytest.raises(ValueError):
        ctx.FromFloats(np.zeros(k, np.float32), k, 1).RMSNorm(ctx, ctx.FromFloats(np.zeros(8, np.float32), 8), 1e-5)
    b.Close()


def test_python_mirror_expert_graph(tmp_path):
    """a mixture-of-experts FFN the way a model drives it: router ids from FromInts, gate/up through
    MulmatID with one activation row per token, down with one row per used expert -- from a GGUF file
    whose expert tensors are 3-D"""
    from ollama_amd import gguf, ml

    k, ff, n_expert, n_used = 512, 384, 6, 3
    rng = np.random.default_rng(81)
    gate = oracle.quantize(qmm.Q4_K, rng.standard_normal((n_expert * ff, k), dtype=np.float32) * np.float32(0.02))
    down = oracle.quantize(qmm.Q8_0, rng.standard_normal((n_expert * k, ff), dtype=np.float32) * np.float32(0.02))
    up = oracle.quantize(qmm.Q4_K, rng.standard_normal((n_expert * ff, k), dtype=np.float32) * np.float32(0.02))
    path = str(tmp_path / "moe.gguf")
    gguf.write_gguf(path, {"general.architecture": "qwen3moe"},
                    [("blk.0.ffn_gate_exps.weight", qmm.Q4_K, [k, ff, n_expert], gate),
                     ("blk.0.ffn_up_exps.weight", qmm.Q4_K, [k, ff, n_expert], up),
                     ("blk.0.ffn_down_exps.weight", qmm.Q8_0, [ff, k, n_expert], down)])
    b = ml.Backend(path)
    b.Load()
    wg, wd = b.Get("blk.0.ffn_gate_exps.weight"), b.Get("blk.0.ffn_down_exps.weight")
    wu = b.Get("blk.0.ffn_up_exps.weight")
    assert wg.Shape() == [k, ff, n_expert] and wd.Shape() == [ff, k, n_expert]
    for tokens in (1, 9):
        ctx = b.NewContext()
        xv = rng.standard_normal((tokens, 1, k), dtype=np.float32)
        hv = rng.standard_normal((tokens, n_used, ff), dtype=np.float32)
        idv = np.stack([rng.choice(n_expert, n_used, replace=False) for _ in range(tokens)]).astype(np.int32)
        ids = ctx.FromInts(idv.reshape(-1), n_used, tokens)
        assert ids.DType() == ml.DType.I32
        xt = ctx.FromFloats(xv.reshape(-1), k, 1, tokens)
        g = wg.MulmatID(ctx, xt, ids)
        u = wu.MulmatID(ctx, xt, ids)      # same x and ids as gate: one call for both at Compute
        d = wd.MulmatID(ctx, ctx.FromFloats(hv.reshape(-1), ff, n_used, tokens), ids)
        assert g.Shape() == [ff, n_used, tokens] and d.Shape() == [k, n_used, tokens]
        ctx.Compute(g, u, d)
        assert npref.rel_err(g.Floats().reshape(tokens, n_used, ff),
                             oracle.mul_mat_id(qmm.Q4_K, gate, k, ff, n_expert, xv, idv)) <= 1e-3
        assert npref.rel_err(u.Floats().reshape(tokens, n_used, ff),
                             oracle.mul_mat_id(qmm.Q4_K, up, k, ff, n_expert, xv, idv)) <= 1e-3
        assert npref.rel_err(d.Floats().reshape(tokens, n_used, k),
                             oracle.mul_mat_id(qmm.Q8_0, down, ff, k, n_expert, hv, idv)) <= 1e-3
        # the whole expert block: down reads silu(gate) * up, which runs inside its quantization
        act = g.SILU(ctx, u)
        out = wd.MulmatID(ctx, act, ids)
        ctx.Compute(out)
        with pytest.raises(RuntimeError):
            act.Floats()
        av = oracle.swiglu(g.Floats().reshape(tokens, n_used, ff), u.Floats().reshape(tokens, n_used, ff))
        assert npref.rel_err(out.Floats().reshape(tokens, n_used, k),
                             oracle.mul_mat_id(qmm.Q8_0, down, ff, k, n_expert, av, idv)) <= 1e-3
        # the same block as one fresh graph: at one token gate, up and the gating are one call (the two products
        # are never materialized), with more tokens the gating runs inside the down experts' quantization
        ctx2 = b.NewContext()
        ids2 = ctx2.FromInts(idv.reshape(-1), n_used, tokens)
        x2 = ctx2.FromFloats(xv.reshape(-1), k, 1, tokens)
        g2, u2 = wg.MulmatID(ctx2, x2, ids2), wu.MulmatID(ctx2, x2, ids2)
        act2 = g2.SILU(ctx2, u2)
        out2 = wd.MulmatID(ctx2, act2, ids2)
        ctx2.Compute(out2)
        for lazy in ((g2, u2) if tokens == 1 else (act2,)):
            with pytest.raises(RuntimeError):
                lazy.Floats()
        assert np.array_equal(out2.Floats(), out.Floats())
        ctx2.Close()
        with pytest.raises(TypeError):
            wg.Mulmat(ctx, ctx.FromFloats(xv.reshape(-1), k, tokens))        # a stack is not a 2-D weight
        with pytest.raises(ValueError):
            wg.MulmatID(ctx, ctx.FromFloats(xv.reshape(-1), k, 1, tokens), ctx.FromInts([0], 1, 1) if tokens > 1
                        else ctx.FromInts([0, 1], 1, 2))                      # token counts differ
        ctx.Close()
    ctx = b.NewContext()
    bad = wg.MulmatID(ctx, ctx.FromFloats(np.zeros(k, np.float32), k, 1, 1), ctx.FromInts([n_expert], 1, 1))
    with pytest.raises(qmm.QmmError):
        ctx.Compute(bad)                                                      # ggml aborts on such an id
    b.Close()


def test_cpp_mirror_program():
    exe = os.path.join(ROOT, "tests", "cpp", "test_host_mirror")
    if not os.path.exists(exe):
        pytest.fail(f"{exe} is not built; run __graft_entry__.build()")
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(p.stdout, p.stderr)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    assert "host mirror: all ok" in p.stdout
