"""GGUF reader (C++ behind the C ABI) and writer.  The cases restate the reference's own tests as data:
/root/reference/fs/gguf/gguf_test.go:16-217 (TestRead on the file createBinFile builds),
/root/reference/fs/gguf/gguf_internal_test.go:11-122 (oversized string / array, row not a multiple of
the block, more than four dimensions, bad offset, missing tensor) and
/root/reference/fs/gguf/keyvalue_test.go (zero value on a kind mismatch).  No GPU needed."""
import json
import os
import struct

import numpy as np
import pytest

from ollama_amd import gguf, qmm

HERE = os.path.dirname(os.path.abspath(__file__))


def _reference_test_file(tmp_path):
    kv = {
        "general.architecture": "llama",
        "llama.block_count": np.uint32(8),
        "llama.embedding_length": np.uint32(3),
        "llama.attention.head_count": np.uint32(2),
        "llama.attention.head_count_kv": np.uint32(2),
        "llama.attention.key_length": np.uint32(3),
        "llama.rope.dimension_count": np.uint32(4),
        "llama.rope.freq_base": np.float32(10000.0),
        "llama.rope.freq_scale": np.float32(1.0),
        "llama.attention.layer_norm_rms_epsilon": np.float32(1e-6),
        "tokenizer.ggml.eos_token_id": np.uint32(0),
        "tokenizer.ggml.eos_token_ids": np.array([1, 2, 3], np.int32),
        "tokenizer.ggml.tokens": ["hello", "world"],
        "tokenizer.ggml.scores": np.array([0, 1], np.float32),
    }
    tensors = [("token_embd.weight", 0, [2, 3], bytes(4 * 2 * 3)), ("output.weight", 0, [3, 2], bytes(range(24)))]
    for i in range(8):
        for n in ("attn_q", "attn_k", "attn_v", "attn_output"):
            tensors.append((f"blk.{i}.{n}.weight", 0, [3, 3], bytes(4 * 3 * 3)))
    p = str(tmp_path / "ref.gguf")
    gguf.write_gguf(p, kv, tensors)
    return p, kv, tensors


def test_read_reference_test_file(tmp_path):
    p, kv, tensors = _reference_test_file(tmp_path)
    with gguf.File(p) as f:
        assert f.Version == 3 and f.Alignment == 32
        assert not f.KeyValue("does.not.exist").Valid()
        assert f.KeyValue("general.architecture").String() == "llama"
        t = f.TensorInfo("token_embd.weight")
        assert t.Name == "token_embd.weight" and t.Shape == [2, 3] and t.Type == 0
        assert f.KeyValue("block_count").Uint() == 8                      # architecture prefix added
        assert not f.KeyValue("llama.block_count").Valid()                 # ... to every key outside general./tokenizer.
        assert f.KeyValue("tokenizer.ggml.tokens").Strings() == ["hello", "world"]
        assert f.KeyValue("tokenizer.ggml.scores").Floats() == [0.0, 1.0]
        assert f.KeyValue("tokenizer.ggml.eos_token_ids").Ints() == [1, 2, 3]
        keys = [k.Key for k in f.KeyValues()]
        assert all(keys) and len(keys) == f.NumKeyValues() == 14
        assert sorted(keys) == sorted(kv)
        assert keys == sorted(keys)                                        # the writer sorts keys
        names = [t.Name for t in f.TensorInfos()]
        assert len(names) == f.NumTensors() == 34 and sorted(names) == sorted(n for n, *_ in tensors)
        assert names[0] == "blk.0.attn_k.weight" and names[-2:] == ["output.weight", "token_embd.weight"]
        t = f.TensorInfo("output.weight")
        assert t.Shape == [3, 2] and t.Type == 0 and t.NumBytes == 24
        assert f.TensorBytes("output.weight").tobytes() == bytes(range(24))
        # every tensor starts on an alignment boundary of the file
        for t in f.TensorInfos():
            assert (f.DataOffset + t.Offset) % 32 == 0
        assert f.DataOffset % 32 == 0


def test_value_kind_mismatch_gives_zero(tmp_path):
    p, _, _ = _reference_test_file(tmp_path)
    with gguf.File(p) as f:
        u = f.KeyValue("block_count")              # uint32
        assert u.Uint() == 8 and u.Int() == 0 and u.Float() == 0.0 and u.String() == "" and u.Bool() is False
        assert u.Ints() is None and u.Strings() is None
        s = f.KeyValue("general.architecture")     # string
        assert s.Uint() == 0 and s.Float() == 0.0
        a = f.KeyValue("tokenizer.ggml.eos_token_ids")   # []int32
        assert a.Ints() == [1, 2, 3] and a.Uints() is None and a.Floats() is None and a.Int() == 0
        fl = f.KeyValue("rope.freq_base")
        assert fl.Float() == 10000.0 and fl.Uint() == 0
        missing = f.KeyValue("nope")
        assert missing.Uint() == 0 and missing.String() == "" and missing.Strings() is None


def test_every_value_type_round_trips(tmp_path):
    kv = {"general.architecture": "t", "a.u8": np.uint8(200), "a.i8": np.int8(-5), "a.u16": np.uint16(60000),
          "a.i16": np.int16(-30000), "a.u32": np.uint32(4000000000), "a.i32": np.int32(-7), "a.u64": np.uint64(1 << 63),
          "a.i64": np.int64(-(1 << 62)), "a.f32": np.float32(0.1), "a.f64": np.float64(0.1), "a.true": True, "a.false": False,
          "a.str": "héllo", "a.empty": "", "a.bools": [True, False, True], "a.u64s": np.array([1, 1 << 40], np.uint64),
          "a.f64s": np.array([0.5, -2.0], np.float64), "a.strs": ["", "x", "yz"], "general.alignment": np.uint32(64)}
    p = str(tmp_path / "kinds.gguf")
    gguf.write_gguf(p, kv, [("w", 0, [4], bytes(16))])
    with gguf.File(p) as f:
        assert f.Alignment == 64 and f.DataOffset % 64 == 0
        g = f.KeyValue                     # "a.u8" is written and looked up as "t.a.u8"
        assert g("a.u8").Uint() == 200 and g("a.i8").Int() == -5 and g("a.u16").Uint() == 60000
        assert g("a.i16").Int() == -30000 and g("a.u32").Uint() == 4000000000 and g("a.i32").Int() == -7
        assert g("a.u64").Uint() == 1 << 63 and g("a.i64").Int() == -(1 << 62)
        assert g("a.f32").Float() == float(np.float32(0.1)) and g("a.f64").Float() == 0.1
        assert g("a.true").Bool() is True and g("a.false").Bool() is False
        assert g("a.str").String() == "héllo" and g("a.empty").String() == ""
        assert g("a.bools").Bools() == [True, False, True] and g("a.u64s").Uints() == [1, 1 << 40]
        assert g("a.f64s").Floats() == [0.5, -2.0] and g("a.strs").Strings() == ["", "x", "yz"]


def _raw(tmp_path, body: bytes):
    p = str(tmp_path / "raw.gguf")
    with open(p, "wb") as f:
        f.write(body)
    return p


def _s(x: str) -> bytes:
    return struct.pack("<Q", len(x)) + x.encode()


def _open_error(tmp_path, body):
    with pytest.raises(qmm.QmmError) as e:
        gguf.File(_raw(tmp_path, body))
    return str(e.value)


def test_rejects_what_the_reference_rejects(tmp_path):
    head = lambda nt, nkv: b"GGUF" + struct.pack("<IQQ", 3, nt, nkv)
    # more than four dimensions
    assert "dimensions" in _open_error(tmp_path, head(1, 0) + _s("bad.weight") + struct.pack("<I", 5))
    # offset beyond int64
    body = head(1, 0) + _s("bad.weight") + struct.pack("<IQIQ", 1, 1, 0, 0xFFFFFFFFFFFFFFFF)
    assert "offset" in _open_error(tmp_path, body)
    # data beyond the end of the file
    body = head(1, 0) + _s("w") + struct.pack("<IQIQ", 1, 1024, 0, 0)
    assert "exceeds file size" in _open_error(tmp_path, body + bytes(64))
    # string longer than 16 MiB, array longer than 64 Mi elements
    assert "string" in _open_error(tmp_path, head(0, 1) + struct.pack("<Q", (16 << 20) + 1) + bytes(32))
    body = head(0, 1) + _s("k") + struct.pack("<IIQ", gguf.ARRAY, gguf.STRING, (64 << 20) + 1)
    assert "array size" in _open_error(tmp_path, body + bytes(32))
    # row not a multiple of the block size (31 elements of Q4_0)
    body = head(1, 0) + _s("bad.weight") + struct.pack("<IQIQ", 1, 31, 2, 0)
    assert "bad.weight" in _open_error(tmp_path, body + bytes(64))
    # wrong magic, old version, truncated header, unknown value type
    assert "magic" in _open_error(tmp_path, b"gguf" + struct.pack("<IQQ", 3, 0, 0))
    assert "version" in _open_error(tmp_path, b"GGUF" + struct.pack("<IQQ", 1, 0, 0))
    assert _open_error(tmp_path, b"GGUF" + struct.pack("<I", 3))
    assert "type" in _open_error(tmp_path, head(0, 1) + _s("k") + struct.pack("<I", 99) + bytes(16))
    # counts that the file cannot hold (no giant allocation is attempted)
    assert "count" in _open_error(tmp_path, head(1 << 60, 0))
    with pytest.raises(qmm.QmmError):
        gguf.File(str(tmp_path / "does-not-exist.gguf"))
    # an empty file with a valid header opens; a missing tensor is "not found"
    with gguf.File(_raw(tmp_path, head(0, 0))) as f:
        assert f.NumTensors() == 0 and not f.TensorInfo("missing.weight").Valid()
        with pytest.raises(KeyError):
            f.TensorBytes("missing.weight")


def test_tensor_sizes_match_the_reference_table(tmp_path):
    """every type of the reference's TestTensorTypes table, one block's worth of elements per tensor"""
    golden = json.load(open(os.path.join(HERE, "golden", "tensor_types.json")))
    tensors = []
    for row in golden["sizes"]:
        tensors.append((f"t{row['kind']}", row["kind"], [row["block_size"] * 3, 2], bytes(row["type_size"] * 6)))
    p = str(tmp_path / "types.gguf")
    gguf.write_gguf(p, {"general.architecture": "x"}, tensors)
    with gguf.File(p) as f:
        for row in golden["sizes"]:
            t = f.TensorInfo(f"t{row['kind']}")
            assert t.Type == row["kind"] and t.NumBytes == row["type_size"] * 6, row


def test_expert_stack_tensors_and_array_buffers_round_trip(tmp_path):
    """3-D expert tensors (ne = [in, out, experts], /root/reference/convert/convert_gemma4.go:274-275) and
    tensor data handed over as a 2-D array of block rows: offsets count bytes, not rows"""
    rng = np.random.default_rng(3)
    a = rng.integers(0, 256, (6 * 4, 34 * 3), dtype=np.uint8)    # Q8_0 [96, 4, 6]: 24 rows of 3 blocks
    b = rng.integers(0, 256, (2 * 5, 144), dtype=np.uint8)       # Q4_K [256, 5, 2]
    p = str(tmp_path / "moe.gguf")
    gguf.write_gguf(p, {"general.architecture": "x"},
                    [("blk.0.ffn_down_exps.weight", qmm.Q8_0, [96, 4, 6], a), ("blk.0.ffn_up_exps.weight", qmm.Q4_K, [256, 5, 2], b)])
    with gguf.File(p) as f:
        ta, tb = f.TensorInfo("blk.0.ffn_down_exps.weight"), f.TensorInfo("blk.0.ffn_up_exps.weight")
        assert ta.Shape == [96, 4, 6] and ta.NumBytes == a.size and ta.Offset == 0
        assert tb.Shape == [256, 5, 2] and tb.NumBytes == b.size and tb.Offset == (a.size + 31) // 32 * 32
        assert f.TensorBytes(ta.Name).tobytes() == a.tobytes()
        assert f.TensorBytes(tb.Name).tobytes() == b.tobytes()


def test_hand_packed_file_pins_offsets_and_bytes(tmp_path):
    """A valid file packed field by field here (no writer of this repository involved, so a layout mistake shared
    by writer and reader cannot hide): two key-values, one of them a string array, general.alignment = 64, a Q4_K
    and an F32 tensor.  Layout per /root/reference/fs/gguf/gguf.go:54-110 (header, key-values, tensor infos, data
    offset = header end rounded up to the alignment) and :388-430 (a tensor's bytes start at data offset + its
    offset and run for its byte size)."""
    rng = np.random.default_rng(12)
    q4k = rng.integers(0, 256, 2 * 144, dtype=np.uint8).tobytes()          # 2 rows of 256 elements: 2 x 144 bytes
    f32 = np.arange(5, dtype="<f4").tobytes()                              # 5 floats: 20 bytes
    body = b"GGUF" + struct.pack("<I", 3) + struct.pack("<Q", 2) + struct.pack("<Q", 2)
    body += _s("general.alignment") + struct.pack("<I", 4) + struct.pack("<I", 64)                       # UINT32 64
    body += _s("tokenizer.ggml.tokens") + struct.pack("<I", 9) + struct.pack("<I", 8) + struct.pack("<Q", 3)
    body += _s("a") + _s("bc" * 16) + _s("")                                                             # ARRAY of STRING
    body += _s("blk.0.ffn_gate.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 256, 2) + struct.pack("<I", 12)
    body += struct.pack("<Q", 0)                                                                         # Q4_K at offset 0
    body += _s("output_norm.weight") + struct.pack("<I", 1) + struct.pack("<Q", 5) + struct.pack("<I", 0)
    body += struct.pack("<Q", 320)                                         # F32 at 320: 288 rounded up to 64
    header_len = len(body)
    data_offset = (header_len + 63) // 64 * 64
    assert data_offset != (header_len + 31) // 32 * 32                     # the non-default alignment matters here
    body += bytes(data_offset - header_len) + q4k + bytes(320 - 288) + f32
    with gguf.File(_raw(tmp_path, body)) as f:
        assert f.Version == 3 and f.Alignment == 64 and f.DataOffset == data_offset
        assert f.NumKeyValues() == 2 and f.NumTensors() == 2
        assert f.KeyValue("general.alignment").Uint() == 64
        assert f.KeyValue("tokenizer.ggml.tokens").Strings() == ["a", "bc" * 16, ""]
        g, n = f.TensorInfo("blk.0.ffn_gate.weight"), f.TensorInfo("output_norm.weight")
        assert (g.Type, g.Shape, g.Offset, g.NumBytes) == (12, [256, 2], 0, 288)
        assert (n.Type, n.Shape, n.Offset, n.NumBytes) == (0, [5], 320, 20)
        assert f.TensorBytes("blk.0.ffn_gate.weight").tobytes() == q4k
        assert f.TensorBytes("output_norm.weight").tobytes() == f32
        assert [t.Name for t in f.TensorInfos()] == ["blk.0.ffn_gate.weight", "output_norm.weight"]


def test_file_reader_knows_every_type_the_size_tables_know(tmp_path):
    """the reference's table of test rows ends at BF16 (30); its size formulas go on to MXFP4, NVFP4 and Q1_0
    (/root/reference/fs/ggml/ggml.go:427-436, 504-509).  A file that holds such tensors -- the expert tensors of a gpt-oss
    file are MXFP4 -- must open, with the sizes of the library's own tables."""
    kinds = [t for t in range(64) if qmm.type_size(t) > 0]
    assert {39, 40, 41} <= set(kinds)
    tensors = [(f"t{t}", t, [qmm.block_size(t) * 2, 3], bytes(qmm.type_size(t) * 6)) for t in kinds]
    p = str(tmp_path / "all_types.gguf")
    gguf.write_gguf(p, {"general.architecture": "x"}, tensors)
    with gguf.File(p) as f:
        for t in kinds:
            ti = f.TensorInfo(f"t{t}")
            assert ti.Type == t and ti.NumBytes == qmm.type_size(t) * 6, t
