"""Host-side mirror of the reference's tensor-backend interface for the Mulmat path.

Names, argument meaning and error behaviour follow /root/reference/ml/backend.go:
  Backend   :16-33   Load / Get(name) / NewContext / Close        (weights live here until Close)
  Context   :94-128  FromFloats / Compute / Close                 (tensors die with the context)
  Tensor    :130-153 Dim / Stride / Shape / DType / Bytes / Floats / Mulmat / MulmatFullPrec / MulmatID
            :159, :180 RMSNorm(ctx, weight, eps) / SILU(ctx, up): the producers of a product's activations
  DType     :404-412
The reference's tensor ops build a lazy graph and have no error returns: Mulmat records a node,
Compute runs it, and a failure is a panic -- here a raised exception.  Shapes are ggml's: dimension 0
is the contiguous one, a weight is [K, M], activations are [K, N], ``W.Mulmat(ctx, x)`` is [M, N].

Everything that computes goes through the C ABI (``ollama_amd.qmm``).  Compute groups the Mulmat
nodes of a graph by the ``x`` they read: decode-sized ones (N <= 8) of the same weight type run as one
multi-tensor launch that quantizes ``x`` in its prologue; larger ones share one quantization of ``x``.
An RMSNorm or SILU(up) node that only products read is never materialized: it becomes the producer of
those products' activations (``mi_qmm_mulmat_produced``).  ``gate.SILU(ctx, up)`` on two products of one
``x`` that nothing else reads runs as one call (``mi_qmm_mulmat_swiglu``) and the two products are never
materialized either.
"""
from __future__ import annotations

import enum
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import qmm


class DType(enum.IntEnum):  # /root/reference/ml/backend.go:404-412
    Other = 0
    F32 = 1
    F16 = 2
    Q80 = 3
    Q40 = 4
    I32 = 5
    MXFP4 = 6


I32 = 26  # ggml_type id of int32, /root/reference/fs/ggml/type.go:252-279
_GGML_TO_DTYPE = {qmm.F32: DType.F32, qmm.F16: DType.F16, qmm.Q8_0: DType.Q80, qmm.Q4_0: DType.Q40, qmm.MXFP4: DType.MXFP4, I32: DType.I32}


def _single_only(t: "Tensor") -> bool:
    """weights that only the plain product entry points multiply (mulmat, mulmat_multi; for padded MXFP4 stacks also
    mulmat_id): F32 / F16 / BF16, Q5_K, and MXFP4 / Q5_0 whose rows are no multiple of 256 (kept padded on the device)"""
    return t._type in qmm.SINGLE_ONLY_TYPES or (t._type in (qmm.MXFP4, qmm.Q5_0) and t.Dim(0) % 256 != 0)


class Tensor:
    """A node of the graph: a weight, an input, or a pending Mulmat result."""

    def __init__(self, shape: Sequence[int], ggml_type: int = qmm.F32):
        self._shape = [int(d) for d in shape]
        self._type = ggml_type
        self._weight: Optional[qmm.Weight] = None      # resident quantized weight
        self._raw: Optional[np.ndarray] = None          # GGUF bytes of a weight (kept for Bytes())
        self._data: Optional[np.ndarray] = None          # f32 values, flat in ggml order
        self._op: Optional[Tuple["Tensor", "Tensor"]] = None  # (W, x) of a pending Mulmat
        self._ids: Optional["Tensor"] = None             # third operand of a pending MulmatID
        self._prod: Optional[Tuple[int, "Tensor", Optional["Tensor"], float]] = None  # pending RMSNorm / SILU(up)
        self._absorbed = False                           # a product computed inside the SILU node that reads it

    # -- shape queries, /root/reference/ml/backend.go:131-135
    def Dim(self, n: int) -> int:
        return self._shape[n] if n < len(self._shape) else 1

    def Stride(self, n: int) -> int:
        """bytes between consecutive elements along dimension n (ggml nb[n])"""
        if self._type not in (qmm.F32, I32):
            row = qmm.row_size(self._type, self._shape[0])
            return qmm.type_size(self._type) if n == 0 else row * int(np.prod(self._shape[1:n], dtype=np.int64))
        return 4 * int(np.prod(self._shape[:n], dtype=np.int64))

    def Shape(self) -> List[int]:
        return list(self._shape)

    def DType(self) -> DType:
        return _GGML_TO_DTYPE.get(self._type, DType.Other)

    # -- data access, :138-140
    def Bytes(self) -> bytes:
        if self._raw is not None:
            return self._raw.tobytes()
        return self.Floats().tobytes()

    def Floats(self) -> np.ndarray:
        if self._data is None:
            raise RuntimeError("tensor has no data yet: call Context.Compute on it first")
        return self._data

    # -- the op, :151-152
    def Mulmat(self, ctx: "Context", t2: "Tensor") -> "Tensor":
        """self = W [K, M] (a weight from Backend.Get: block-quantized, or F32 / F16 / BF16), t2 = x [K, N] f32  ->
        [M, N] f32, lazily."""
        if self._weight is None:
            raise TypeError("Mulmat: the receiver must be a weight obtained from Backend.Get")
        if len(self._shape) != 2:
            raise TypeError(f"Mulmat: the weight must be 2-D, got {self.Shape()} (expert stacks go through MulmatID)")
        if t2._type != qmm.F32:
            raise TypeError("Mulmat: activations must be f32")
        if t2.Dim(0) != self.Dim(0):
            raise ValueError(f"Mulmat: inner dimensions differ: {self.Shape()} x {t2.Shape()}")
        out = Tensor([self.Dim(1)] + t2._shape[1:])
        out._op = (self, t2)
        ctx._nodes.append(out)
        return out

    def MulmatID(self, ctx: "Context", t2: "Tensor", ids: "Tensor") -> "Tensor":
        """self = expert stack [K, M, E], t2 = x [K, B, T] f32 (B = 1 or the number of used experts),
        ids = [n_used, T] int32  ->  [M, n_used, T] f32, lazily: slot i of token t goes through expert
        ids[i, t] with activation row i mod B of that token.  /root/reference/ml/backend.go:153"""
        if self._weight is None or len(self._shape) != 3:
            raise TypeError("MulmatID: the receiver must be a 3-D quantized expert stack obtained from Backend.Get")
        if self._type in qmm.SINGLE_ONLY_TYPES:
            raise TypeError("MulmatID: expert stacks must be of type Q4_0, Q8_0, Q4_K, Q6_K or MXFP4")
        if t2._type != qmm.F32 or ids._type != I32:
            raise TypeError("MulmatID: activations must be f32 and ids int32")
        if t2.Dim(0) != self.Dim(0):
            raise ValueError(f"MulmatID: inner dimensions differ: {self.Shape()} x {t2.Shape()}")
        if len(ids._shape) > 2 or len(t2._shape) > 3 or ids.Dim(1) != t2.Dim(2):
            raise ValueError(f"MulmatID: ids {ids.Shape()} and activations {t2.Shape()} disagree on the token count")
        out = Tensor([self.Dim(1), ids.Dim(0), ids.Dim(1)])
        out._op = (self, t2)
        out._ids = ids
        ctx._nodes.append(out)
        return out

    def MulmatFullPrec(self, ctx: "Context", t2: "Tensor") -> "Tensor":
        """The quantized path already accumulates block sums in exact integers and scales in fp32."""
        return self.Mulmat(ctx, t2)

    # -- the producers of a product's activations, :159 and :180
    def RMSNorm(self, ctx: "Context", weight: Optional["Tensor"], eps: float) -> "Tensor":
        """self = x [K, ...] f32, weight = [K] f32 or None  ->  (x / sqrt(mean(x^2) + eps)) * weight along
        dimension 0, lazily."""
        if self._type != qmm.F32 or (weight is not None and weight._type != qmm.F32):
            raise TypeError("RMSNorm: operands must be f32")
        if weight is not None and (weight._data is None or weight._data.size != self.Dim(0)):
            raise ValueError(f"RMSNorm: the weight must hold {self.Dim(0)} values")
        out = Tensor(self._shape)
        out._prod = (qmm.PRODUCE_RMSNORM, self, weight, float(eps))
        ctx._nodes.append(out)
        return out

    def SILU(self, ctx: "Context", *up: "Tensor") -> "Tensor":
        """self = gate, up[0] = up, both f32 of one shape  ->  silu(gate) * up, lazily (ggml's swiglu).  Without
        ``up``: the bare activation silu(self), an f32 node of its own (it is never folded into a product)."""
        if len(up) > 1:
            raise TypeError("SILU takes at most one operand")
        if self._type != qmm.F32 or (up and (up[0]._type != qmm.F32 or self._shape != up[0]._shape)):
            raise ValueError(f"SILU: gate {self.Shape()} and up must be f32 of one shape")
        out = Tensor(self._shape)
        out._prod = (qmm.PRODUCE_SWIGLU, self, up[0] if up else None, 0.0)
        ctx._nodes.append(out)
        return out


def tensors_ids(tensors) -> set:
    return {id(t) for t in tensors}


class Context:
    """Holds the tensors of one graph; Compute runs the pending Mulmat nodes."""

    def __init__(self, backend: "Backend"):
        self._b = backend
        self._nodes: List[Tensor] = []
        self._closed = False

    def FromFloats(self, s: Sequence[float], *shape: int) -> Tensor:
        arr = np.ascontiguousarray(s, dtype=np.float32).reshape(-1)
        if int(np.prod(shape, dtype=np.int64)) != arr.size:
            raise ValueError(f"FromFloats: {arr.size} values for shape {list(shape)}")
        t = Tensor(shape)
        t._data = arr
        return t

    def FromInts(self, s: Sequence[int], *shape: int) -> Tensor:
        arr = np.ascontiguousarray(s, dtype=np.int32).reshape(-1)
        if int(np.prod(shape, dtype=np.int64)) != arr.size:
            raise ValueError(f"FromInts: {arr.size} values for shape {list(shape)}")
        t = Tensor(shape, I32)
        t._data = arr
        return t

    def Forward(self, *tensors: Tensor) -> "Context":
        return self

    def Compute(self, *tensors: Tensor) -> None:
        """Run the pending nodes in the order they were recorded.  Producer nodes (RMSNorm, SILU) are
        materialized only when asked for here or read by something other than a Mulmat."""
        if self._closed:
            raise RuntimeError("Compute on a closed context")
        pending = [t for t in self._nodes if t._data is None and not t._absorbed and (t._op is not None or t._prod is not None)]
        c = self._b._ctx
        # producer nodes that must exist as f32: requested, or read by another producer
        needed = {id(t) for t in tensors}
        readers: Dict[int, List[Tensor]] = {}
        for t in pending:
            srcs = [s for s in (t._prod[1], t._prod[2]) if s is not None] if t._prod is not None else [t._op[1]]
            if t._prod is not None:
                needed.update(id(s) for s in srcs)
                if t._prod[0] == qmm.PRODUCE_SWIGLU and t._prod[2] is None:
                    needed.add(id(t))  # the bare silu is always an f32 node
            elif _single_only(t._op[0]):
                needed.update(id(s) for s in srcs)  # these weight types have no fused producers: x must exist as f32
            for s in srcs:
                readers.setdefault(id(s), []).append(t)
        # gate.SILU(up) on two pending products of one x that nothing else reads, at one activation row: one call
        # computes the gated result, the two products are never materialized.  (With more rows the gating is
        # better placed in the quantization of whatever reads it: the gated values then never exist in f32.)
        pair_of: Dict[int, Tensor] = {}
        for t in pending:
            if t._prod is None or t._prod[0] != qmm.PRODUCE_SWIGLU:
                continue
            gate, up = t._prod[1], t._prod[2]
            if not (gate in pending and up in pending and gate is not up and gate._op is not None and up._op is not None
                    and gate._ids is up._ids and gate._op[1] is up._op[1]
                    and not _single_only(gate._op[0]) and not _single_only(up._op[0])
                    and gate._op[0].Shape() == up._op[0].Shape() and id(gate) not in tensors_ids(tensors)
                    and id(up) not in tensors_ids(tensors) and readers.get(id(gate)) == [t] and readers.get(id(up)) == [t]):
                continue
            x = gate._op[1]
            # one activation row (one token for expert stacks): the single-launch form
            one = (gate._ids.Dim(1) if gate._ids is not None else int(np.prod(x._shape[1:], dtype=np.int64))) == 1
            if not one:
                continue
            pair_of[id(gate)] = pair_of[id(up)] = t
            if x._prod is not None and (x._prod[0] != qmm.PRODUCE_RMSNORM or gate._ids is not None):
                needed.add(id(x))  # only a norm in front of plain products runs inside the paired launch

        def rows(t: Tensor) -> np.ndarray:
            return t.Floats().reshape(-1, t.Dim(0))

        for t in pending:
            if t._data is not None:
                continue  # computed with an earlier node of its group
            if t._prod is not None:
                if id(t) in needed:
                    kind, src, aux, eps = t._prod
                    if kind == qmm.PRODUCE_RMSNORM:
                        t._data = c.rms_norm(rows(src), None if aux is None else aux.Floats(), eps).reshape(-1)
                    else:
                        t._data = c.swiglu(rows(src), None if aux is None else rows(aux)).reshape(-1)
                continue
            x = t._op[1]
            if t._absorbed:
                continue
            if id(t) in pair_of:
                silu = pair_of[id(t)]
                gate, up = silu._prod[1], silu._prod[2]
                if gate._ids is not None:
                    ids = gate._ids
                    tokens, n_used = ids.Dim(1), ids.Dim(0)
                    h = c.mulmat_id_swiglu(gate._op[0]._weight, up._op[0]._weight, gate._op[0].Dim(2),
                                           x.Floats().reshape(tokens, x.Dim(1), x.Dim(0)), ids._data.reshape(tokens, n_used))
                elif x._data is None and x._prod is not None and x._prod[0] == qmm.PRODUCE_RMSNORM:
                    _, src, aux, eps = x._prod  # the norm in front of gate and up runs in the same launch
                    h = c.mulmat_swiglu(gate._op[0]._weight, up._op[0]._weight, rows(src), qmm.PRODUCE_RMSNORM,
                                        None if aux is None else aux.Floats(), eps)
                else:
                    h = c.mulmat_swiglu(gate._op[0]._weight, up._op[0]._weight, rows(x))
                silu._data = h.reshape(-1)
                gate._absorbed = up._absorbed = True
                continue
            if t._ids is not None:
                # expert-indexed nodes that read the same x and ids (gate and up of an expert FFN) go out together
                ids = t._ids
                nodes = [u for u in pending if u._data is None and u._ids is ids and u._op[1] is x
                         and u._op[0].Dim(2) == t._op[0].Dim(2) and id(u) not in pair_of]
                tokens, n_used = ids.Dim(1), ids.Dim(0)
                idv = ids._data.reshape(tokens, n_used)
                if any(_single_only(u._op[0]) for u in nodes):
                    # stacks kept padded on the device (MXFP4 experts of K = 2880): one plain expert-indexed product each
                    b = x.Floats().reshape(tokens, x.Dim(1), x.Dim(0))
                    ys = [c.mulmat_id(u._op[0]._weight, t._op[0].Dim(2), b, idv) for u in nodes]
                elif x._data is None and x._prod is not None:
                    # x is a producer nobody needs in f32 (silu(gate) * up in front of the down experts)
                    kind, src, aux, eps = x._prod
                    b = src.Floats().reshape(tokens, x.Dim(1), x.Dim(0))
                    a = None if aux is None else (aux.Floats() if kind == qmm.PRODUCE_RMSNORM else aux.Floats().reshape(b.shape))
                    ys = [c.mulmat_id_produced(u._op[0]._weight, t._op[0].Dim(2), kind, a, b, idv, eps) for u in nodes]
                else:
                    b = x.Floats().reshape(tokens, x.Dim(1), x.Dim(0))
                    ys = c.mulmat_id_multi([u._op[0]._weight for u in nodes], t._op[0].Dim(2), b, idv)
                for u, y in zip(nodes, ys):
                    u._data = y.reshape(-1)  # [tokens][n_used][m] row-major == ggml [M, n_used, T]
                continue
            nodes = [u for u in pending if u._data is None and u._ids is None and u._op is not None and u._op[1] is x
                     and id(u) not in pair_of]
            for u in [u for u in nodes if _single_only(u._op[0])]:
                # F32 / F16 / BF16 / Q5_K weights: one product each
                u._data = c.mulmat(u._op[0]._weight, x.Floats().reshape(-1, x.Dim(0))).reshape(-1)
            nodes = [u for u in nodes if not _single_only(u._op[0])]
            if not nodes:
                continue
            if x._data is None and x._prod is not None:
                # x is a producer nobody needs in f32: it runs inside the products' own quantization
                kind, src, aux, eps = x._prod
                a = None if aux is None else (aux.Floats() if kind == qmm.PRODUCE_RMSNORM else rows(aux))
                ys = c.mulmat_produced([u._op[0]._weight for u in nodes], kind, a, rows(src), eps)
                for u, y in zip(nodes, ys):
                    u._data = y.reshape(-1)
                continue
            k = x.Dim(0)
            xs = rows(x)
            n = xs.shape[0]
            if n <= 8:
                # decode: the GEMV quantizes x itself; weights of one type share a launch, four at a time
                by_type: Dict[int, List[Tensor]] = {}
                for u in nodes:
                    by_type.setdefault(u._op[0]._type, []).append(u)
                for group in by_type.values():
                    for i in range(0, len(group), 4):
                        part = group[i:i + 4]
                        ys = c.mulmat_multi([u._op[0]._weight for u in part], xs)
                        for u, y in zip(part, ys):
                            u._data = y.reshape(-1)  # [n][m] row-major == ggml [M, N] with dim 0 contiguous
                continue
            # prefill: quantize once per (x, q8 type), then one product per weight
            by_q8: Dict[int, List[Tensor]] = {}
            for u in nodes:
                by_q8.setdefault(qmm.vec_dot_type(u._op[0]._type), []).append(u)
            for q8, group in by_q8.items():
                act = c.act_create(q8, k, n)
                try:
                    c.act_quantize(act, xs)
                    for u in group:
                        u._data = c.mulmat_q8(u._op[0]._weight, act).reshape(-1)
                finally:
                    act.free()

    def Close(self) -> None:
        self._nodes.clear()
        self._closed = True


class Backend:
    """Weights resident on one MI355X.  ``tensors`` is either the path of a GGUF file -- the model file
    ``ml.NewBackend(modelPath, params)`` receives, /root/reference/ml/backend.go:83 -- or a dict mapping a
    tensor name to (ggml_type, shape [K, M], block bytes), what fs/ggml hands out for a tensor
    (/root/reference/fs/ggml/gguf.go:281-308).  From a file, Load uploads every 2-D tensor (and every 3-D
    expert stack) of a type the Mulmat path multiplies (Q4_0, Q8_0, Q4_K, Q5_K, Q6_K; 2-D F32, F16 and BF16 too) straight
    from the file mapping and keeps 1-D f32 tensors (norm weights, the operand of RMSNorm) on the host; tensors of
    other types are outside this path and are skipped."""

    def __init__(self, tensors, device: int = 0):
        self._ctx = qmm.Context(device)
        self._tensors: Dict[str, Tensor] = {}
        self._spec = tensors
        self._loaded = False

    def Load(self, progress=None) -> None:
        if isinstance(self._spec, (str, bytes)):
            from . import gguf

            with gguf.File(self._spec if isinstance(self._spec, str) else self._spec.decode()) as f:
                infos = [t for t in f.TensorInfos()
                         if (len(t.Shape) in (2, 3) and qmm.vec_dot_type(t.Type) >= 0
                             and not (len(t.Shape) == 3 and t.Type in qmm.SINGLE_ONLY_TYPES))
                         or (len(t.Shape) == 1 and t.Type == qmm.F32)]
                for i, ti in enumerate(infos):
                    t = Tensor(ti.Shape, ti.Type)
                    t._raw = f.TensorBytes(ti.Name)
                    if ti.Type == qmm.F32 and len(ti.Shape) == 1:
                        t._data = np.frombuffer(t._raw, dtype=np.float32).copy()  # a norm weight: stays on the host
                    else:
                        t._weight = f.Upload(self._ctx, ti.Name)
                    self._tensors[ti.Name] = t
                    if progress:
                        progress((i + 1) / max(len(infos), 1))
            self._loaded = True
            return
        total = max(len(self._spec), 1)
        for i, (name, (ggml_type, shape, raw)) in enumerate(self._spec.items()):
            if ggml_type == qmm.F32 and len(shape) == 1:  # a norm weight: stays on the host
                t = Tensor(shape, ggml_type)
                t._data = np.ascontiguousarray(raw).view(np.float32).reshape(-1).copy()
                if t._data.size != int(shape[0]):
                    raise ValueError(f"{name}: {t._data.size} values for shape {list(shape)}")
                t._raw = t._data.view(np.uint8)
                self._tensors[name] = t
                continue
            if len(shape) not in (2, 3):
                raise ValueError(f"{name}: Mulmat takes 2-D weights and MulmatID 3-D expert stacks, got shape {list(shape)}")
            k, m = int(shape[0]), int(np.prod(shape[1:], dtype=np.int64))  # a stack is its experts' rows in a row
            raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
            t = Tensor(shape, ggml_type)
            t._weight = self._ctx.upload(ggml_type, raw, k, m)
            t._raw = raw
            self._tensors[name] = t
            if progress:
                progress((i + 1) / total)
        self._loaded = True

    def Get(self, name: str) -> Optional[Tensor]:
        return self._tensors.get(name)  # nil for an unknown name, like the reference

    def NewContext(self) -> Context:
        return Context(self)

    def BackendDevices(self):
        return [self._ctx.device_info()]

    def Close(self) -> None:
        for t in self._tensors.values():
            if t._weight is not None:
                t._weight.free()
        self._tensors.clear()
        self._ctx.close()
