"""PTIR (ptir.v0.4) program model, builder DSL and serde-JSON wire form.

Host-side mirror of the reference's IR types (crates/gpt-rs/src/backend/spec.rs:19-817)
and of its snippet DSL (crates/gpt-rs/src/ops/ptir/graph.rs).  A `FunctionBuilder`
records instructions in evaluation order with dense increasing value ids, exactly the
stream a backend's `run_program` receives (crates/gpt-rs/src/ops/graph/arena.rs:1014).

The JSON layout follows serde's defaults for the derive attributes in spec.rs:
externally tagged enums, unit variants as strings, newtypes as bare values.
"""
from __future__ import annotations

import json
import struct
from dataclasses import dataclass
from typing import Iterable, List, Optional, Sequence, Tuple, Union

import numpy as np

SPEC_VERSION = "ptir.v0.4"  # spec.rs:12

# dtype name (serde variant, spec.rs:21-41) -> storage bytes (spec.rs:105-118)
DTYPE_BYTES = {
    "I1": 1, "Si8": 1, "Ui8": 1, "Si16": 2, "Ui16": 2, "Bf16": 2, "F16": 2,
    "Si32": 4, "Ui32": 4, "F32": 4, "Si64": 8, "Ui64": 8, "F64": 8,
}
FLOAT_DTYPES = ("F32", "Bf16", "F16", "F64")


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit pattern (uint16). NaN stays NaN."""
    x = np.asarray(x, dtype=np.float32, order="C")
    u = x.reshape(-1).view(np.uint32)
    # uint32 arithmetic wraps only for negative NaNs, which the NaN fix-up below overrides
    rounded = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    out = rounded.astype(np.uint16).reshape(x.shape)
    nan = np.isnan(x)
    if np.any(nan):
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.reshape(-1).astype(np.uint32) << 16).view(np.float32).reshape(bits.shape)


@dataclass(frozen=True)
class TensorSpec:
    """spec.rs:210-232 (static shapes only: the LM path never emits dynamic dims)."""

    dtype: str
    dims: Tuple[int, ...]

    def __post_init__(self):
        object.__setattr__(self, "dims", tuple(int(d) for d in self.dims))
        if self.dtype not in DTYPE_BYTES and self.dtype not in ("Si4", "Ui4"):
            raise ValueError(f"unknown dtype {self.dtype}")

    @property
    def rank(self) -> int:
        return len(self.dims)

    def element_count(self) -> int:
        n = 1
        for d in self.dims:
            n *= d
        return n

    def byte_len(self) -> int:
        return self.element_count() * DTYPE_BYTES[self.dtype]

    def to_json(self):
        return {"dtype": self.dtype, "shape": {"dims": [{"Static": d} for d in self.dims]}}

    @staticmethod
    def from_json(obj) -> "TensorSpec":
        return TensorSpec(obj["dtype"], tuple(d["Static"] for d in obj["shape"]["dims"]))


@dataclass(frozen=True)
class TensorLiteral:
    """spec.rs:245-296: spec + row-major little-endian bytes."""

    spec: TensorSpec
    data: bytes

    def to_json(self):
        return {"spec": self.spec.to_json(), "bytes": list(self.data)}


def scalar_literal(dtype: str, value: float) -> TensorLiteral:
    """graph.rs:2278-2298: scalar literal already rounded to the tensor's dtype."""
    if dtype == "F32":
        data = struct.pack("<f", np.float32(value))
    elif dtype == "Bf16":
        data = struct.pack("<H", int(f32_to_bf16_bits(np.array([value], np.float32))[0]))
    elif dtype == "F16":
        data = np.array([value], np.float16).tobytes()
    elif dtype == "F64":
        data = struct.pack("<d", float(value))
    else:
        raise ValueError(f"scalar literal broadcast does not support dtype {dtype}")
    return TensorLiteral(TensorSpec(dtype, ()), data)


class Tensor:
    """SSA value handle inside one FunctionBuilder (graph.rs `Tensor`)."""

    __slots__ = ("fb", "id", "spec")

    def __init__(self, fb: "FunctionBuilder", vid: int, spec: TensorSpec):
        self.fb, self.id, self.spec = fb, vid, spec

    dtype = property(lambda self: self.spec.dtype)
    dims = property(lambda self: self.spec.dims)

    # -- elementwise -------------------------------------------------------
    def _binary(self, other, op: str) -> "Tensor":
        if not isinstance(other, Tensor):
            # graph.rs:1339-1345: tensor (lhs) op BroadcastTo(literal) (rhs)
            other = self.fb.emit({"BroadcastTo": {"result_shape": _shape_json(self.dims)}},
                                 [scalar_literal(self.dtype, other)], self.spec)
        if other.spec != self.spec:
            raise ValueError(f"elementwise {op}: operand specs differ {self.spec} vs {other.spec}")
        return self.fb.emit({"ElementwiseBinary": op}, [self, other], self.spec)

    def __add__(self, o): return self._binary(o, "Add")
    def __radd__(self, o): return self._binary(o, "Add")  # graph.rs:1879-1885: scalar+tensor swaps
    def __sub__(self, o): return self._binary(o, "Sub")
    def __mul__(self, o): return self._binary(o, "Mul")
    def __rmul__(self, o): return self._binary(o, "Mul")
    def __truediv__(self, o): return self._binary(o, "Div")
    def maximum(self, o): return self._binary(o, "Maximum")
    def minimum(self, o): return self._binary(o, "Minimum")

    def _unary(self, op: str) -> "Tensor":
        return self.fb.emit({"ElementwiseUnary": op}, [self], self.spec)

    def exp(self): return self._unary("Exp")
    def log(self): return self._unary("Log")
    def erf(self): return self._unary("Erf")
    def tanh(self): return self._unary("Tanh")
    def neg(self): return self._unary("Neg")
    def abs(self): return self._unary("Abs")
    def rsqrt(self): return self._unary("Rsqrt")
    def reciprocal(self): return self._unary("Reciprocal")
    def sqrt(self): return self.rsqrt().reciprocal()  # graph.rs:1564-1567

    # -- shape ops -----------------------------------------------------------
    def reshape(self, dims: Sequence[int]) -> "Tensor":
        dims = tuple(dims)
        out = TensorSpec(self.dtype, dims)
        if out.element_count() != self.spec.element_count():
            raise ValueError(f"reshape {self.dims} -> {dims}: element count differs")
        op = {"Reshape": {"new_shape": [{"Explicit": {"Static": d}} for d in dims]}}
        return self.fb.emit(op, [self], out)

    def transpose(self, perm: Sequence[int]) -> "Tensor":
        perm = list(perm)
        if sorted(perm) != list(range(self.spec.rank)):
            raise ValueError(f"transpose perm {perm} is not a permutation of rank {self.spec.rank}")
        out = TensorSpec(self.dtype, tuple(self.dims[p] for p in perm))
        return self.fb.emit({"Transpose": {"perm": perm}}, [self], out)

    def broadcast_to(self, dims: Sequence[int]) -> "Tensor":
        dims = tuple(dims)
        _check_broadcast(self.dims, dims)
        return self.fb.emit({"BroadcastTo": {"result_shape": _shape_json(dims)}}, [self],
                            TensorSpec(self.dtype, dims))

    def slice(self, starts: Sequence[int], sizes: Sequence[int]) -> "Tensor":
        starts, sizes = list(starts), list(sizes)
        if len(starts) != self.spec.rank or len(sizes) != self.spec.rank:
            raise ValueError("slice starts/sizes must match rank")
        for s, z, d in zip(starts, sizes, self.dims):
            if s + z > d:
                raise ValueError(f"slice [{s}, {s + z}) exceeds dim {d}")
        return self.fb.emit({"Slice": {"starts": starts, "sizes": sizes}}, [self],
                            TensorSpec(self.dtype, tuple(sizes)))

    @staticmethod
    def concat(axis: int, parts: Sequence["Tensor"]) -> "Tensor":
        first = parts[0]
        dims = list(first.dims)
        dims[axis] = sum(p.dims[axis] for p in parts)
        for p in parts:
            if p.dtype != first.dtype:
                raise ValueError("concat dtype mismatch")
            if any(a != b for i, (a, b) in enumerate(zip(p.dims, first.dims)) if i != axis):
                raise ValueError("concat shape mismatch off the concat axis")
        return first.fb.emit({"Concat": {"axis": axis}}, list(parts), TensorSpec(first.dtype, tuple(dims)))

    # -- reductions / linalg ---------------------------------------------------
    def _reduce(self, kind: str, axes: Sequence[int], keepdims: bool) -> "Tensor":
        axes = [a if a >= 0 else a + self.spec.rank for a in axes]
        if keepdims:
            dims = tuple(1 if i in axes else d for i, d in enumerate(self.dims))
        else:
            dims = tuple(d for i, d in enumerate(self.dims) if i not in axes)
        op = {"Reduce": {"kind": kind, "axes": axes, "keepdims": bool(keepdims),
                         "accum_dtype": None, "out_dtype": None}}  # graph.rs:1593-1652
        return self.fb.emit(op, [self], TensorSpec(self.dtype, dims))

    def reduce_sum(self, axes, keepdims=True): return self._reduce("Sum", axes, keepdims)
    def reduce_max(self, axes, keepdims=True): return self._reduce("Max", axes, keepdims)
    def reduce_min(self, axes, keepdims=True): return self._reduce("Min", axes, keepdims)

    def dot_general(self, rhs: "Tensor", batch: Sequence[int], contract_lhs: Sequence[int],
                    contract_rhs: Sequence[int], batch_rhs: Optional[Sequence[int]] = None,
                    out_dtype: Optional[str] = None) -> "Tensor":
        """DotGeneral; DotAttrs::default() (accum/out dtype None; docs/backend.md:104-115) unless `out_dtype` names
        the result dtype (DotGeneralSpec.out_dtype, spec.rs:354-361: accumulate in f32, cast to out_dtype).

        Output dims: batch, lhs free, rhs free (docs/backend.md:287-291).
        """
        batch_l = list(batch)
        batch_r = list(batch if batch_rhs is None else batch_rhs)
        cl, cr = list(contract_lhs), list(contract_rhs)
        if self.dtype != rhs.dtype:
            raise ValueError("dot_general dtype mismatch")
        for a, b in zip(batch_l, batch_r):
            if self.dims[a] != rhs.dims[b]:
                raise ValueError("dot_general: batch dimension mismatch")
        for a, b in zip(cl, cr):
            if self.dims[a] != rhs.dims[b]:
                raise ValueError("dot_general: dimension mismatch on contraction")
        out = [self.dims[a] for a in batch_l]
        out += [d for i, d in enumerate(self.dims) if i not in batch_l and i not in cl]
        out += [d for i, d in enumerate(rhs.dims) if i not in batch_r and i not in cr]
        op = {"DotGeneral": {"batch_lhs": batch_l, "batch_rhs": batch_r, "contract_lhs": cl,
                             "contract_rhs": cr, "accum_dtype": None, "out_dtype": out_dtype}}
        return self.fb.emit(op, [self, rhs], TensorSpec(out_dtype or self.dtype, tuple(out)))

    def matmul(self, rhs: "Tensor", out_dtype: Optional[str] = None) -> "Tensor":
        """functional::matmul (ops/functional/linalg.rs:53-127): 2-D or batched 3-D."""
        if self.spec.rank == 2 and rhs.spec.rank == 2:
            return self.dot_general(rhs, [], [1], [0], out_dtype=out_dtype)
        if self.spec.rank == 3 and rhs.spec.rank == 3:
            return self.dot_general(rhs, [0], [2], [1], out_dtype=out_dtype)
        raise ValueError("matmul expects rank-2 or rank-3 operands of equal rank")

    # -- indexing ------------------------------------------------------------
    def take(self, indices: "Tensor") -> "Tensor":
        if indices.dtype not in ("Si32", "Si64"):
            raise ValueError("take indices must be si32|si64")
        out = TensorSpec(self.dtype, tuple(indices.dims) + tuple(self.dims[1:]))
        return self.fb.emit("Take", [self, indices], out)

    def dynamic_slice(self, starts: "Tensor", sizes: Sequence[int]) -> "Tensor":
        sizes = list(sizes)
        return self.fb.emit({"DynamicSlice": {"sizes": sizes}}, [self, starts],
                            TensorSpec(self.dtype, tuple(sizes)))

    def dynamic_update_slice(self, update: "Tensor", starts: "Tensor", sizes: Sequence[int]) -> "Tensor":
        sizes = list(sizes)
        if tuple(sizes) != tuple(update.dims):
            raise ValueError("dynamic_update_slice sizes must equal the update shape")
        return self.fb.emit({"DynamicUpdateSlice": {"sizes": sizes}}, [self, update, starts], self.spec)

    # -- compare / select / cast -------------------------------------------------
    def compare(self, other: "Tensor", op: str) -> "Tensor":
        if other.spec != self.spec:
            raise ValueError("compare operand specs differ")
        return self.fb.emit({"Compare": {"op": op}}, [self, other], TensorSpec("I1", self.dims))

    def greater_equal(self, other): return self.compare(other, "GreaterEqual")

    @staticmethod
    def select(pred: "Tensor", on_true: "Tensor", on_false: "Tensor") -> "Tensor":
        if pred.dtype != "I1" or on_true.spec != on_false.spec or pred.dims != on_true.dims:
            raise ValueError("select operand mismatch")
        return pred.fb.emit("Select", [pred, on_true, on_false], on_true.spec)

    def cast(self, dtype: str) -> "Tensor":
        return self.fb.emit({"Cast": {"dtype": dtype}}, [self], TensorSpec(dtype, self.dims))


def _shape_json(dims: Iterable[int]):
    return {"dims": [{"Static": int(d)} for d in dims]}


def _check_broadcast(src: Tuple[int, ...], dst: Tuple[int, ...]):
    """docs/backend.md:70-79 right-aligned compatibility."""
    if len(src) > len(dst):
        raise ValueError(f"cannot broadcast {src} to {dst}")
    pad = (1,) * (len(dst) - len(src)) + tuple(src)
    for s, d in zip(pad, dst):
        if s != d and s != 1:
            raise ValueError(f"cannot broadcast {src} to {dst}")


class FunctionBuilder:
    """Records one PTIR function.  Parameter ids come first, then instruction ids."""

    def __init__(self, name: str = "main", dtype_scalar: str = "F32"):
        self.name = name
        self.params: List[Tensor] = []
        self.body: List[dict] = []
        self.results: List[Tensor] = []
        self._next = 0
        self.default_float = dtype_scalar

    def _fresh(self) -> int:
        v = self._next
        self._next += 1
        return v

    def param(self, dtype: str, dims: Sequence[int]) -> Tensor:
        t = Tensor(self, self._fresh(), TensorSpec(dtype, tuple(dims)))
        self.params.append(t)
        return t

    def emit(self, op, operands: Sequence[Union[Tensor, TensorLiteral]], out: TensorSpec) -> Tensor:
        vid = self._fresh()
        ops_json = []
        for o in operands:
            if isinstance(o, Tensor):
                if o.fb is not self:
                    raise ValueError("operand belongs to another function")
                ops_json.append({"Value": o.id})
            else:
                ops_json.append({"Literal": o.to_json()})
        self.body.append({"id": vid, "op": op, "operands": ops_json, "output": {"Tensor": out.to_json()}})
        return Tensor(self, vid, out)

    # session helpers ------------------------------------------------------------
    def scalar(self, value: float, dtype: Optional[str] = None) -> Tensor:
        """graph.rs:757-773: rank-0 BroadcastTo of an inline literal."""
        dtype = dtype or self.default_float
        spec = TensorSpec(dtype, ())
        return self.emit({"BroadcastTo": {"result_shape": _shape_json(())}}, [scalar_literal(dtype, value)], spec)

    def scalar_broadcast(self, value: float, dims: Sequence[int], dtype: Optional[str] = None) -> Tensor:
        """ops/ptir/mod.rs:16-22: scalar(value).broadcast_to(dims) -- two BroadcastTo ops."""
        return self.scalar(value, dtype).broadcast_to(dims)

    def iota(self, dims: Sequence[int], axis: int, dtype: str = "Si32") -> Tensor:
        op = {"Iota": {"shape": _shape_json(dims), "dtype": dtype, "axis": int(axis)}}
        return self.emit(op, [], TensorSpec(dtype, tuple(dims)))

    def constant(self, spec: TensorSpec, data: bytes) -> Tensor:
        return self.emit({"Constant": TensorLiteral(spec, data).to_json()}, [], spec)

    def custom_call(self, target: str, operands: Sequence[Tensor], out: TensorSpec, attrs=None) -> Tensor:
        return self.emit({"CustomCall": {"target": target, "attrs": attrs or {}}}, list(operands), out)

    def set_results(self, results: Sequence[Tensor]):
        self.results = list(results)

    def function_json(self):
        return {
            "name": self.name,
            "parameters": [{"Tensor": p.spec.to_json()} for p in self.params],
            "parameter_ids": [p.id for p in self.params],
            "results": [{"Tensor": r.spec.to_json()} for r in self.results],
            "body": self.body,
            "hints": [],
            "result_ids": [r.id for r in self.results],
        }


class Program:
    """spec.rs:748-857.  Holds the JSON text and a stable 64-bit key for plan caches."""

    def __init__(self, fb: FunctionBuilder):
        self.obj = {"spec_version": SPEC_VERSION, "entry": fb.name,
                    "functions": [fb.function_json()], "regions": []}
        self.param_specs = [p.spec for p in fb.params]
        self.result_specs = [r.spec for r in fb.results]
        self._json: Optional[bytes] = None
        self._key: Optional[int] = None

    @property
    def json_bytes(self) -> bytes:
        if self._json is None:
            self._json = json.dumps(self.obj, separators=(",", ":")).encode()
        return self._json

    @property
    def key(self) -> int:
        """FNV-1a over the JSON text: plays the role of PlanKey.hash (arena.rs:993)."""
        if self._key is None:
            h = 0xCBF29CE484222325
            data = self.json_bytes
            # chunked FNV keeps this cheap for multi-hundred-KB programs
            for i in range(0, len(data), 8):
                h ^= int.from_bytes(data[i:i + 8], "little")
                h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
            self._key = h or 1
        return self._key

    def instruction_count(self) -> int:
        return len(self.obj["functions"][0]["body"])
