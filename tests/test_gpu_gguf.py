"""GGUF file -> resident weights -> Mulmat, on the GPU: the loader row of the path."""
import numpy as np
import pytest

import npref
import oracle
from ollama_amd import gguf, ml, qmm, synth

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _model_file(tmp_path):
    k = 1024
    tensors, raws = [], {}
    for name, t, m in (("blk.0.attn_q.weight", qmm.Q4_K, 96), ("blk.0.ffn_down.weight", qmm.Q6_K, 40),
                       ("blk.0.attn_k.weight", qmm.Q8_0, 33), ("output.weight", qmm.Q4_0, 50),
                       ("blk.0.attn_v.weight", qmm.Q5_K, 24), ("blk.1.attn_v.weight", qmm.Q5_0, 19), ("blk.0.dense_mx.weight", qmm.MXFP4, 21)):
        raw = synth.weights(t, m, k, seed=m).reshape(-1)
        raws[name] = (t, m, raw)
        tensors.append((name, t, [k, m], raw.tobytes()))
    norm = (1 + 0.05 * np.random.default_rng(9).standard_normal(k)).astype(np.float32)
    tensors.append(("blk.0.attn_norm.weight", 0, [k], norm.tobytes()))   # f32, 1-D: the operand of RMSNorm, kept on the host
    # unquantized 2-D tensors are weights of the path too (multiplied in their own type)
    rng = np.random.default_rng(10)
    for name, t, m in (("token_embd.weight", qmm.F32, 4), ("output_norm_proj.weight", qmm.F16, 24), ("mm.0.weight", qmm.BF16, 17)):
        raw = oracle.quantize(t, (rng.standard_normal((m, k)) * 0.05).astype(np.float32)).reshape(-1)
        raws[name] = (t, m, raw)
        tensors.append((name, t, [k, m], raw.tobytes()))
    tensors.append(("rope_freqs.weight", 26, [k, 2], np.zeros((2, k), np.int32).tobytes()))  # i32, 2-D: not on the path
    p = str(tmp_path / "model.gguf")
    gguf.write_gguf(p, {"general.architecture": "llama", "block_count": np.uint32(1)}, tensors)
    return p, k, raws


def test_upload_from_file_equals_upload_from_memory(tmp_path):
    p, k, raws = _model_file(tmp_path)
    ctx = qmm.Context(0)
    x = np.random.default_rng(3).standard_normal((3, k), dtype=np.float32)
    with gguf.File(p) as f:
        for name, (t, m, raw) in raws.items():
            assert np.array_equal(f.TensorBytes(name), raw)
            Wf = f.Upload(ctx, name)
            Wm = ctx.upload(t, raw, k, m)
            assert (Wf.type, Wf.k, Wf.m) == (t, k, m)
            assert np.array_equal(ctx.mulmat(Wf, x), ctx.mulmat(Wm, x))
            Wf.free(); Wm.free()
        with pytest.raises(qmm.QmmError) as e:
            f.Upload(ctx, "blk.0.attn_norm.weight")            # 1-D f32
        assert e.value.code == qmm.ERR_UNSUPPORTED
    ctx.close()


def test_backend_from_gguf_path(tmp_path):
    p, k, raws = _model_file(tmp_path)
    seen = []
    b = ml.Backend(p)
    b.Load(progress=seen.append)
    assert seen and seen[-1] == 1.0
    assert b.Get("rope_freqs.weight") is None and b.Get("nope") is None
    assert b.Get("output_norm_proj.weight").DType() == ml.DType.F16
    norm = b.Get("blk.0.attn_norm.weight")
    assert norm.Shape() == [k] and norm.DType() == ml.DType.F32 and abs(norm.Floats().mean() - 1) < 0.05
    ctx = b.NewContext()
    xs = np.random.default_rng(4).standard_normal((2, k), dtype=np.float32)
    x = ctx.FromFloats(xs.reshape(-1), k, 2)
    outs = {name: b.Get(name).Mulmat(ctx, x) for name in raws}
    normed = b.Get("blk.0.attn_q.weight").Mulmat(ctx, x.RMSNorm(ctx, norm, 1e-5))   # the file's norm in front of q
    ctx.Compute(normed, *outs.values())
    t, m, raw = raws["blk.0.attn_q.weight"]
    want = oracle.mul_mat(t, raw, k, m, oracle.rms_norm(xs, norm.Floats(), 1e-5), nthreads=4)
    assert npref.rel_err(normed.Floats().reshape(2, m), want) <= TOL
    for name, (t, m, raw) in raws.items():
        assert outs[name].Shape() == [m, 2]
        want = oracle.mul_mat(t, raw, k, m, xs, nthreads=4)
        assert npref.rel_err(outs[name].Floats().reshape(2, m), want) <= TOL, name
        assert b.Get(name).Bytes() == raw.tobytes()
    ctx.Close()
    b.Close()
