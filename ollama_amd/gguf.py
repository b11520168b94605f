"""GGUF files: a writer that lays a file out the way the reference's writer does, and a reader that is a
thin wrapper over the C ABI (``mi_qmm_gguf_*``: mmap + parse in C++, tensors uploaded straight from
the mapping).

Writer: follows ``WriteGGUF`` (/root/reference/fs/ggml/gguf.go:620-687) -- magic "GGUF", version 3,
counts, key-values in sorted key order (keys outside ``general.`` / ``tokenizer.`` / ``adapter.`` get
the architecture prefix, :689-695), tensor infos sorted by (``blk.N.`` number, name) with offsets
padded to ``general.alignment`` (default 32), padding, data.  The value kinds are the ones the
reference writes (:706-747): numpy scalars select the integer / float width, ``bool``, ``str``, and
lists / arrays of those.

Reader: ``File`` mirrors ``gguf.Open`` / ``File.KeyValue`` / ``File.TensorInfo`` / ``File.TensorReader``
(/root/reference/fs/gguf/gguf.go:54-110, 332-351, 361-378, 390-430).
"""
from __future__ import annotations

import ctypes
import re
import struct
from typing import Any, Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np

from . import qmm

# GGUF value type ids (/root/reference/fs/gguf/gguf.go:23-37)
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)

_NP_KIND = {np.dtype(np.uint8): U8, np.dtype(np.int8): I8, np.dtype(np.uint16): U16, np.dtype(np.int16): I16,
            np.dtype(np.uint32): U32, np.dtype(np.int32): I32, np.dtype(np.float32): F32, np.dtype(np.bool_): BOOL,
            np.dtype(np.uint64): U64, np.dtype(np.int64): I64, np.dtype(np.float64): F64}


def _wstr(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _scalar_kind(v: Any) -> Tuple[int, bytes]:
    if isinstance(v, (bool, np.bool_)):
        return BOOL, struct.pack("<?", bool(v))
    if isinstance(v, str):
        return STRING, _wstr(v)
    if isinstance(v, np.generic):
        return _NP_KIND[v.dtype], v.tobytes()
    if isinstance(v, int):
        return I64, struct.pack("<q", v)
    if isinstance(v, float):
        return F64, struct.pack("<d", v)
    raise TypeError(f"improper type {type(v).__name__}")


def _value_bytes(v: Any) -> bytes:
    if isinstance(v, np.ndarray):
        return struct.pack("<IIQ", ARRAY, _NP_KIND[v.dtype], v.size) + np.ascontiguousarray(v).tobytes()
    if isinstance(v, (list, tuple)):
        if not v:
            raise TypeError("an empty list has no element type: pass a typed numpy array")
        kinds = [_scalar_kind(e) for e in v]
        if len({k for k, _ in kinds}) != 1:
            raise TypeError("array elements must share one type")
        return struct.pack("<IIQ", ARRAY, kinds[0][0], len(v)) + b"".join(b for _, b in kinds)
    k, b = _scalar_kind(v)
    return struct.pack("<I", k) + b


def _block_number(name: str) -> int:
    m = re.match(r"blk\.(\d+)\.", name)
    return int(m.group(1)) if m else (1 << 63) - 1


def write_gguf(path: str, kv: Dict[str, Any], tensors: Sequence[Tuple[str, int, Sequence[int], bytes]]) -> None:
    """tensors: (name, ggml type id, shape with dimension 0 contiguous, raw block bytes)."""
    arch = kv.get("general.architecture", "")
    if not arch:
        raise ValueError("architecture not set")
    alignment = int(kv.get("general.alignment", 32))
    out = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(kv)))
    for k in sorted(kv):
        kk = k if any(k.startswith(p) for p in (arch + ".", "general.", "adapter.", "tokenizer.")) else arch + "." + k
        out += _wstr(kk) + _value_bytes(kv[k])
    # raw may be any buffer (a 2-D numpy array of blocks included): its bytes are what counts
    ts = sorted(((n, kind, shape, bytes(raw)) for n, kind, shape, raw in tensors), key=lambda t: (_block_number(t[0]), t[0]))
    offsets, s = [], 0
    for name, kind, shape, raw in ts:
        offsets.append(s)
        out += _wstr(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", int(d)) for d in shape)
        out += struct.pack("<IQ", int(kind), s)
        s += len(raw)
        s += (alignment - s % alignment) % alignment
    out += b"\0" * ((alignment - len(out) % alignment) % alignment)
    base = len(out)
    with open(path, "wb") as f:
        f.write(out)
        for (name, kind, shape, raw), off in zip(ts, offsets):
            f.seek(base + off)
            f.write(raw)


class TensorInfo:
    def __init__(self, index: int, name: str, type_: int, shape: List[int], offset: int, nbytes: int):
        self.index, self.Name, self.Type, self.Shape, self.Offset, self.NumBytes = index, name, type_, shape, offset, nbytes

    def Valid(self) -> bool:
        return self.Name != ""


class KeyValue:
    """A key with its value; the accessors return zero values on a kind mismatch
    (/root/reference/fs/gguf/keyvalue.go:42-91)."""

    def __init__(self, f: Optional["File"], index: int):
        self._f, self._i = f, index
        self.Key, self.Type, self.ElemType, self.Count = "", -1, -1, 0
        if f is not None and index >= 0:
            key, t, et, n = ctypes.c_char_p(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int64()
            qmm._check(qmm.lib().mi_qmm_gguf_kv(f._h, index, ctypes.byref(key), ctypes.byref(t), ctypes.byref(et),
                                                ctypes.byref(n)))
            self.Key, self.Type, self.ElemType, self.Count = key.value.decode(), t.value, et.value, n.value

    def Valid(self) -> bool:
        return self.Key != ""

    def _get(self, fn, ctype, elem=-1):
        if not self.Valid():
            return ctype().value
        out = ctype()
        qmm._check(fn(self._f._h, self._i, elem, ctypes.byref(out)))
        return out.value

    def Int(self) -> int:
        return self._get(qmm.lib().mi_qmm_gguf_kv_int, ctypes.c_int64)

    def Uint(self) -> int:
        return self._get(qmm.lib().mi_qmm_gguf_kv_uint, ctypes.c_uint64)

    def Float(self) -> float:
        return self._get(qmm.lib().mi_qmm_gguf_kv_float, ctypes.c_double)

    def Bool(self) -> bool:
        return bool(self._get(qmm.lib().mi_qmm_gguf_kv_bool, ctypes.c_int))

    def _str(self, elem=-1) -> str:
        if not self.Valid():
            return ""
        p, n = ctypes.c_void_p(), ctypes.c_int64()
        qmm._check(qmm.lib().mi_qmm_gguf_kv_string(self._f._h, self._i, elem, ctypes.byref(p), ctypes.byref(n)))
        return ctypes.string_at(p.value, n.value).decode("utf-8") if n.value else ""

    def String(self) -> str:
        return self._str()

    def _elems(self, kinds, getter):
        if not self.Valid() or self.Type != ARRAY or self.ElemType not in kinds:
            return None
        return [getter(i) for i in range(self.Count)]

    def Ints(self):
        return self._elems((I8, I16, I32, I64), lambda i: self._get(qmm.lib().mi_qmm_gguf_kv_int, ctypes.c_int64, i))

    def Uints(self):
        return self._elems((U8, U16, U32, U64), lambda i: self._get(qmm.lib().mi_qmm_gguf_kv_uint, ctypes.c_uint64, i))

    def Floats(self):
        return self._elems((F32, F64), lambda i: self._get(qmm.lib().mi_qmm_gguf_kv_float, ctypes.c_double, i))

    def Bools(self):
        return self._elems((BOOL,), lambda i: bool(self._get(qmm.lib().mi_qmm_gguf_kv_bool, ctypes.c_int, i)))

    def Strings(self):
        return self._elems((STRING,), self._str)


class File:
    def __init__(self, path: str):
        h = ctypes.c_void_p()
        qmm._check(qmm.lib().mi_qmm_gguf_open(path.encode(), ctypes.byref(h)))
        self._h = h
        v, al, off, nkv, nt = ctypes.c_int(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        qmm._check(qmm.lib().mi_qmm_gguf_info(h, ctypes.byref(v), ctypes.byref(al), ctypes.byref(off), ctypes.byref(nkv),
                                              ctypes.byref(nt)))
        self.Version, self.Alignment, self.DataOffset = v.value, al.value, off.value
        self._nkv, self._nt = nkv.value, nt.value

    def NumKeyValues(self) -> int:
        return self._nkv

    def NumTensors(self) -> int:
        return self._nt

    def KeyValue(self, key: str) -> KeyValue:
        return KeyValue(self, qmm.lib().mi_qmm_gguf_find_kv(self._h, key.encode()))

    def KeyValues(self) -> Iterable[KeyValue]:
        return (KeyValue(self, i) for i in range(self._nkv))

    def _tensor(self, index: int) -> TensorInfo:
        if index < 0:
            return TensorInfo(-1, "", 0, [], 0, 0)
        name, t, nd = ctypes.c_char_p(), ctypes.c_int(), ctypes.c_int()
        dims, off, nb = (ctypes.c_int64 * 4)(), ctypes.c_int64(), ctypes.c_int64()
        qmm._check(qmm.lib().mi_qmm_gguf_tensor(self._h, index, ctypes.byref(name), ctypes.byref(t), ctypes.byref(nd),
                                                dims, ctypes.byref(off), ctypes.byref(nb)))
        return TensorInfo(index, name.value.decode(), t.value, list(dims[: nd.value]), off.value, nb.value)

    def TensorInfo(self, name: str) -> TensorInfo:
        return self._tensor(qmm.lib().mi_qmm_gguf_find_tensor(self._h, name.encode()))

    def TensorInfos(self) -> Iterable[TensorInfo]:
        return (self._tensor(i) for i in range(self._nt))

    def TensorBytes(self, name: str) -> np.ndarray:
        """the tensor's bytes, copied out of the mapping (the analogue of reading File.TensorReader to the end)"""
        t = self.TensorInfo(name)
        if not t.Valid() or t.NumBytes == 0:
            raise KeyError(f"tensor {name} not found")
        p = qmm.lib().mi_qmm_gguf_tensor_data(self._h, t.index)
        return np.frombuffer(ctypes.string_at(p, t.NumBytes), dtype=np.uint8)

    def Upload(self, ctx: "qmm.Context", name: str) -> "qmm.Weight":
        """tensor -> resident weight on ctx's GPU, straight from the mapping"""
        t = self.TensorInfo(name)
        if not t.Valid():
            raise KeyError(f"tensor {name} not found")
        h = ctypes.c_void_p()
        qmm._check(qmm.lib().mi_qmm_gguf_upload(ctx._h, self._h, t.index, ctypes.byref(h)))
        return qmm.Weight(h, t.Type, t.Shape[0], t.Shape[1] * (t.Shape[2] if len(t.Shape) == 3 else 1))

    def Close(self) -> None:
        if self._h:
            qmm.lib().mi_qmm_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.Close()
