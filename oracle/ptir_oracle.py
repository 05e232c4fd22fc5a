"""TEST INFRASTRUCTURE ONLY -- CPU oracle for PTIR programs.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module, and only as the checker.  The shipped backend never calls it.

A numpy restatement of the reference CPU interpreter
(crates/gpt-rs-backend-ref-cpu/src/cpu.rs), one function per `op_*`, interpreting the
same serde-JSON program text the HIP backend receives.  Summation-order-sensitive
loops (dot_general, reduce) and libm unary functions run in oracle/seqops.c so each
output sees the reference's exact sequence of f32 roundings.

Parity pinning status per op (what independent evidence each is checked against in
tests/test_oracle.py):
  * index ops (Slice/DynamicSlice/DynamicUpdateSlice/Concat/Transpose/Reshape/
    BroadcastTo/Iota/Compare/Select/Take/Cast): pinned by the reference-held vectors
    (crates/gpt-rs-backend-triton/tests/dynamic_ops_gpu.rs:35-104,
    crates/gpt-rs/tests/{graph_cache_stability,lazy_graph}.rs) and brute-force loops.
  * DotGeneral: pinned by [[1,2],[3,4]].[[5,6],[7,8]]=[19,22,43,50]
    (crates/gpt-rs-backend-tests/src/smoke.rs:12-24), by the reference C kernels built
    under oracle/_ref, and by float64 matmul.
  * Reduce/unary/binary and the functional sequences built from them: pinned by torch
    CPU (layer_norm, softmax, gelu, silu), the reference's own oracle
    (crates/gpt-rs-backend-tests/src/torch_parity/functional_ops.rs).
  * bf16 execution: parity unpinned -- the reference executes no bf16
    (crates/gpt-rs-backend-ref-cpu/src/cpu.rs:21-25); semantics defined here as
    "compute each op in f32, round each op OUTPUT to bf16 (RNE)", per
    docs/backend.md:99,104-115; a DotGeneral whose out_dtype is F32 keeps its f32 sums over
    bf16 operands (spec.rs:354-361).
  * gptrs.hip.* custom calls (weight-only int8/int4): parity unpinned BY THE REFERENCE -- it
    has no quantization scheme (docs/backend.md:620-632); closed form defined here.  The
    closed form itself is pinned against hand-written vectors (ties of both signs, zero
    columns and groups, clamping, the k = 127/128 group boundary, nibble order, one expected
    byte string) and against a pure-Python per-element loop (tests/test_oracle.py).
"""
from __future__ import annotations

import ctypes
import json
import os
import subprocess
from typing import Dict, List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class OracleError(Exception):
    """kind in {"spec", "unimplemented", "execution"} mirrors BackendError (spec.rs:1224-1228)."""

    def __init__(self, kind: str, message: str):
        super().__init__(f"{kind}: {message}")
        self.kind, self.message = kind, message


def build_seqops(force: bool = False) -> str:
    so = os.path.join(_HERE, "liboracle_seqops.so")
    src = os.path.join(_HERE, "seqops.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fno-fast-math", "-ffp-contract=off", "-fPIC", "-shared",
                               "-o", so, src, "-lm"])
    return so


def _lib():
    global _LIB
    if _LIB is None:
        lib = ctypes.CDLL(build_seqops())
        fp = ctypes.POINTER(ctypes.c_float)
        sz = ctypes.c_size_t
        lib.oracle_bmm_f32.argtypes = [fp, fp, fp, sz, sz, sz, sz]
        lib.oracle_reduce_f32.argtypes = [fp, fp, sz, sz, sz, ctypes.c_int]
        lib.oracle_unary_f32.argtypes = [fp, fp, sz, ctypes.c_int]
        for f in (lib.oracle_bmm_f32, lib.oracle_reduce_f32, lib.oracle_unary_f32):
            f.restype = None
        _LIB = lib
    return _LIB


def _fp(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


# Contractions of at least this many multiply-adds run through numpy's f32 matmul (a blocked BLAS sum) instead of the
# sequential-k loop of cpu.rs:2190-2236.  None (the default) keeps every dot on the reference's summation order.  Tests
# of full-size shapes (0.25 TFLOP for one Ministral layer at 1024 tokens) set it: the two orders differ by a few f32
# ulps of the sum, far inside the tolerances those tests state, and the sequential loop would take minutes.
BLAS_DOT_MIN_MACS = None


def _bmm(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """c[B,M,N] = a[B,M,K] . b[B,K,N] in f32."""
    B, M, K = a.shape
    N = b.shape[2]
    if BLAS_DOT_MIN_MACS is not None and B * M * K * N >= BLAS_DOT_MIN_MACS:
        return np.matmul(a, b).astype(np.float32, copy=False)
    c = np.empty((B, M, N), dtype=np.float32)
    _lib().oracle_bmm_f32(_fp(a), _fp(b), _fp(c), B, M, K, N)
    return c


# ----------------------------------------------------------------------------- tensors
NP_DTYPES = {"F32": np.float32, "Si32": np.int32, "I1": np.uint8, "Bf16": np.float32,
             "Si8": np.int8, "Ui8": np.uint8}
DTYPE_BYTES = {"F32": 4, "Si32": 4, "I1": 1, "Bf16": 2, "Si8": 1, "Ui8": 1}


def round_bf16(x: np.ndarray) -> np.ndarray:
    """f32 -> nearest-even bf16, returned as f32 (docs/backend.md:99)."""
    x = np.asarray(x, dtype=np.float32, order="C")
    u = x.reshape(-1).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).reshape(x.shape)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, np.float32(np.nan), out)
    return out


class OTensor:
    """dtype tag + numpy array.  Bf16 values are held as f32 that are bf16-representable."""

    __slots__ = ("dtype", "a")

    def __init__(self, dtype: str, a: np.ndarray):
        if dtype not in NP_DTYPES:
            raise OracleError("spec", f"dtype {dtype} unsupported")
        self.dtype = dtype
        self.a = np.asarray(a, dtype=NP_DTYPES[dtype], order="C")  # keeps rank 0

    @property
    def dims(self) -> Tuple[int, ...]:
        return tuple(self.a.shape)

    @staticmethod
    def from_bytes(dtype: str, dims: Sequence[int], data: bytes) -> "OTensor":
        dims = tuple(dims)
        n = int(np.prod(dims, dtype=np.int64)) if dims else 1
        if dtype not in DTYPE_BYTES:
            raise OracleError("spec", f"literal dtype {dtype} unsupported")
        if len(data) != n * DTYPE_BYTES[dtype]:
            raise OracleError("execution", "literal byte length mismatch")
        if dtype == "Bf16":
            bits = np.frombuffer(data, dtype="<u2").astype(np.uint32) << 16
            return OTensor(dtype, bits.view(np.float32).reshape(dims))
        arr = np.frombuffer(data, dtype=np.dtype(NP_DTYPES[dtype]).newbyteorder("<")).reshape(dims)
        return OTensor(dtype, arr)

    def to_bytes(self) -> bytes:
        if self.dtype == "Bf16":
            return (self.a.view(np.uint32) >> 16).astype("<u2").tobytes()
        return self.a.astype(np.dtype(NP_DTYPES[self.dtype]).newbyteorder("<")).tobytes()


def _spec(obj) -> Tuple[str, Tuple[int, ...]]:
    dims = []
    for d in obj["shape"]["dims"]:
        if "Static" not in d:
            raise OracleError("execution", f"dynamic dimension {d.get('Dynamic')} not supported at runtime")
        dims.append(int(d["Static"]))
    return obj["dtype"], tuple(dims)


def _is_float(dt: str) -> bool:
    return dt in ("F32", "Bf16")


def _finish(dtype: str, a: np.ndarray) -> OTensor:
    """Round an f32 result to the op's output dtype."""
    if dtype == "Bf16":
        a = round_bf16(a)
    return OTensor(dtype, a)


# ----------------------------------------------------------------------------- ops
def op_reshape(x: OTensor, out_dims) -> OTensor:                      # cpu.rs:644-678
    if int(np.prod(out_dims, dtype=np.int64)) != x.a.size:
        raise OracleError("execution", "reshape element count mismatch")
    return OTensor(x.dtype, x.a.reshape(out_dims))


def op_slice(x: OTensor, starts, sizes) -> OTensor:                   # cpu.rs:680-761
    if len(starts) != x.a.ndim or len(sizes) != x.a.ndim:
        raise OracleError("execution", "slice rank mismatch")
    for s, z, d in zip(starts, sizes, x.dims):
        if s + z > d:
            raise OracleError("execution", "slice exceeds bounds")
    idx = tuple(slice(s, s + z) for s, z in zip(starts, sizes))
    return OTensor(x.dtype, x.a[idx])


def _clamped_starts(starts: OTensor, dims, sizes) -> List[int]:       # cpu.rs:804-820
    if starts.dtype != "Si32":
        raise OracleError("execution", "dynamic_slice starts must be si32")
    if starts.a.ndim != 1 or starts.a.shape[0] != len(dims):
        raise OracleError("execution", "starts must be 1-D of length equal to rank")
    out = []
    for ax, (d, z) in enumerate(zip(dims, sizes)):
        if z > d:
            raise OracleError("execution", "dynamic_slice size exceeds dimension")
        s = int(starts.a[ax])
        out.append(min(max(s, 0), d - z))
    return out


def op_dynamic_slice(x: OTensor, starts: OTensor, sizes) -> OTensor:  # cpu.rs:763-873
    if len(sizes) != x.a.ndim:
        raise OracleError("execution", "dynamic_slice sizes length must match input rank")
    st = _clamped_starts(starts, x.dims, sizes)
    return OTensor(x.dtype, x.a[tuple(slice(s, s + z) for s, z in zip(st, sizes))])


def op_dynamic_update_slice(base: OTensor, upd: OTensor, starts: OTensor, sizes) -> OTensor:  # cpu.rs:875-1057
    if base.dtype != upd.dtype:
        raise OracleError("execution", "dynamic_update_slice dtype mismatch")
    if tuple(sizes) != upd.dims or len(sizes) != base.a.ndim:
        raise OracleError("execution", "dynamic_update_slice sizes must match update shape")
    st = _clamped_starts(starts, base.dims, sizes)
    out = base.a.copy()
    out[tuple(slice(s, s + z) for s, z in zip(st, sizes))] = upd.a
    return OTensor(base.dtype, out)


def op_transpose(x: OTensor, perm) -> OTensor:                        # cpu.rs:1059-1103
    if sorted(perm) != list(range(x.a.ndim)):
        raise OracleError("execution", "transpose perm invalid")
    return OTensor(x.dtype, np.transpose(x.a, perm))


def op_broadcast_to(x: OTensor, out_dims) -> OTensor:                 # cpu.rs:1105-1176
    try:
        return OTensor(x.dtype, np.broadcast_to(x.a, out_dims))
    except ValueError:
        raise OracleError("spec", f"cannot broadcast {x.dims} to {tuple(out_dims)}")


def op_cast(x: OTensor, dst: str) -> OTensor:                         # cpu.rs:1472-1583, docs/backend.md:96-102
    src = x.dtype
    a = x.a
    if src == dst:
        return OTensor(dst, a)
    if _is_float(src) and _is_float(dst):
        return _finish(dst, a.astype(np.float32))
    if src == "Si32" and _is_float(dst):
        return _finish(dst, a.astype(np.float32))
    if _is_float(src) and dst == "Si32":
        t = np.trunc(a.astype(np.float64))
        t = np.where(np.isnan(t), 0.0, t)
        t = np.clip(t, -2147483648.0, 2147483647.0)
        return OTensor(dst, t.astype(np.int64).astype(np.int32))
    if src == "I1" and dst == "Si32":
        return OTensor(dst, (a != 0).astype(np.int32))
    if src == "Si32" and dst == "I1":
        return OTensor(dst, (a != 0).astype(np.uint8))
    if src == "I1" and _is_float(dst):
        return OTensor(dst, (a != 0).astype(np.float32))
    if _is_float(src) and dst == "I1":
        return OTensor(dst, (a != 0.0).astype(np.uint8))
    raise OracleError("unimplemented", f"cast {src}->{dst}")


def op_take(x: OTensor, idx: OTensor) -> OTensor:                     # cpu.rs:1585-1648
    if x.a.ndim < 1:
        raise OracleError("execution", "take requires rank >= 1")
    if idx.dtype != "Si32":
        raise OracleError("execution", "take indices must be si32")
    if idx.a.size and (idx.a.min() < 0 or idx.a.max() >= x.a.shape[0]):
        raise OracleError("execution", "take index out of bounds")
    return OTensor(x.dtype, x.a[idx.a])


_BIN = {
    "Add": lambda a, b: a + b, "Sub": lambda a, b: a - b, "Mul": lambda a, b: a * b,
    "Div": lambda a, b: a / b,
    # Rust f32::max/min return the non-NaN operand (cpu.rs:1675-1676) == fmax/fmin
    "Maximum": np.fmax, "Minimum": np.fmin,
}


def op_binary(a: OTensor, b: OTensor, op: str) -> OTensor:            # cpu.rs:1650-1688
    if a.dtype != b.dtype or a.dims != b.dims:
        raise OracleError("execution", "elementwise size mismatch")
    if not _is_float(a.dtype):
        raise OracleError("execution", "elementwise binary only supports float tensors")
    with np.errstate(all="ignore"):
        r = _BIN[op](a.a, b.a).astype(np.float32)
    return _finish(a.dtype, r)


_UNARY_CODE = {"Neg": 0, "Abs": 1, "Exp": 2, "Log": 3, "Tanh": 4, "Erf": 5, "Rsqrt": 6, "Reciprocal": 7}


def op_unary(x: OTensor, op: str) -> OTensor:                         # cpu.rs:1690-1720
    if not _is_float(x.dtype):
        raise OracleError("execution", "elementwise unary only supports float tensors")
    y = np.empty_like(x.a)
    _lib().oracle_unary_f32(_fp(x.a), _fp(y), x.a.size, _UNARY_CODE[op])
    return _finish(x.dtype, y)


def op_reduce(x: OTensor, kind: str, axes, keepdims: bool) -> OTensor:  # cpu.rs:1722-1800
    if len(axes) != 1:
        raise OracleError("execution", "reduce currently supports single axis")
    if not keepdims:
        raise OracleError("execution", "reduce requires keepdims=true")
    if not _is_float(x.dtype):
        raise OracleError("execution", "reduce only supports float tensors")
    ax = axes[0]
    if ax >= x.a.ndim:
        raise OracleError("execution", "reduce axis out of range")
    dims = x.dims
    axis_len = dims[ax]
    inner = int(np.prod(dims[ax + 1:], dtype=np.int64))
    outer = int(np.prod(dims[:ax], dtype=np.int64))
    out_dims = dims[:ax] + (1,) + dims[ax + 1:]
    y = np.empty(out_dims, dtype=np.float32)
    _lib().oracle_reduce_f32(_fp(x.a), _fp(y), outer, axis_len, inner, {"Sum": 0, "Max": 1, "Min": 2}[kind])
    return _finish(x.dtype, y)


def op_dot_general(l: OTensor, r: OTensor, spec) -> OTensor:          # cpu.rs:2110-2236
    if l.dtype != r.dtype or not _is_float(l.dtype):
        raise OracleError("execution", "dot_general only supports float tensors of one dtype")
    for key in ("accum_dtype", "out_dtype"):
        if spec.get(key) not in (None, "F32") and not (key == "out_dtype" and spec.get(key) == l.dtype):
            raise OracleError("unimplemented", f"dot_general {key} override not supported")
    bl, br = sorted(spec["batch_lhs"]), sorted(spec["batch_rhs"])
    cl, cr = list(spec["contract_lhs"]), list(spec["contract_rhs"])
    lf = [i for i in range(l.a.ndim) if i not in bl and i not in cl]
    rf = [i for i in range(r.a.ndim) if i not in br and i not in cr]
    bshape = [l.dims[i] for i in bl]
    if bshape != [r.dims[i] for i in br]:
        raise OracleError("execution", "dot_general batch dimension mismatch")
    cshape = [l.dims[i] for i in cl]
    if cshape != [r.dims[i] for i in cr]:
        raise OracleError("execution", "dot_general contraction dimension mismatch")
    lshape, rshape = [l.dims[i] for i in lf], [r.dims[i] for i in rf]
    B = int(np.prod(bshape, dtype=np.int64))
    M = int(np.prod(lshape, dtype=np.int64))
    K = int(np.prod(cshape, dtype=np.int64))
    N = int(np.prod(rshape, dtype=np.int64))
    a = np.ascontiguousarray(np.transpose(l.a, bl + lf + cl).reshape(B, M, K))
    b = np.ascontiguousarray(np.transpose(r.a, br + cr + rf).reshape(B, K, N))
    c = _bmm(a, b)
    out_dtype = spec.get("out_dtype") or l.dtype
    return _finish(out_dtype, c.reshape(bshape + lshape + rshape))


_CMP = {"Less": np.less, "LessEqual": np.less_equal, "Equal": np.equal,
        "GreaterEqual": np.greater_equal, "Greater": np.greater, "NotEqual": np.not_equal}


def op_compare(a: OTensor, b: OTensor, op: str) -> OTensor:           # cpu.rs:2238-2271
    if a.dtype != b.dtype or a.dims != b.dims:
        raise OracleError("execution", "compare operand mismatch")
    return OTensor("I1", _CMP[op](a.a, b.a).astype(np.uint8))


def op_select(p: OTensor, t: OTensor, f: OTensor) -> OTensor:         # cpu.rs:2273-2294
    if p.dtype != "I1" or t.dtype != f.dtype or not (p.dims == t.dims == f.dims):
        raise OracleError("execution", "select dtype combination unsupported")
    return OTensor(t.dtype, np.where(p.a != 0, t.a, f.a))


def op_concat(xs: List[OTensor], axis: int) -> OTensor:               # cpu.rs:2296-2392
    if not xs:
        raise OracleError("execution", "concat expects at least one input")
    rank = xs[0].a.ndim
    axis = axis + rank if axis < 0 else axis
    if any(x.dtype != xs[0].dtype for x in xs):
        raise OracleError("execution", "concat dtype mismatch")
    try:
        return OTensor(xs[0].dtype, np.concatenate([x.a for x in xs], axis=axis))
    except ValueError as e:
        raise OracleError("execution", f"concat shape mismatch: {e}")


def op_iota(dims, dtype: str, axis: int) -> OTensor:                  # cpu.rs:2513-2546
    if dtype != "Si32":
        raise OracleError("execution", "iota only supports si32")
    shape = [1] * len(dims)
    shape[axis] = dims[axis]
    return OTensor(dtype, np.broadcast_to(np.arange(dims[axis], dtype=np.int32).reshape(shape), dims))


# -- build-defined extension ops (no counterpart in the reference) ---------------------
def quantize_int8_per_channel(w: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Weight-only int8, symmetric, one scale per OUTPUT channel (column of W[in,out]).

    s_n = bf16(max_k |W[k,n]| / 127) (1.0 when the column is all zero),
    q = clamp(rint(W / s_n), -127, 127) with round-half-even, computed in f32.
    """
    w = np.asarray(w, dtype=np.float32)
    amax = np.max(np.abs(w), axis=0)
    s = round_bf16((amax / np.float32(127.0)).astype(np.float32))
    s = np.where(s == 0, np.float32(1.0), s).astype(np.float32)
    q = np.clip(np.rint((w / s[None, :]).astype(np.float32)), -127, 127).astype(np.int8)
    return q, s


def quantize_int4_g128(w: np.ndarray, group: int = 128) -> Tuple[np.ndarray, np.ndarray]:
    """Weight-only int4, symmetric, groups of `group` along K (rows of W[in,out]) per column.

    s[g,n] = bf16(max |w| / 7) (1.0 for an all-zero group), q in [-7,7] (RNE),
    packed two per byte along K: byte[k/2, n] = (q[k] & 0xF) | ((q[k+1] & 0xF) << 4).
    """
    w = np.asarray(w, dtype=np.float32)
    K, N = w.shape
    if K % group or K % 2:
        raise OracleError("spec", "int4 packing needs K to be a multiple of the group size")
    wg = w.reshape(K // group, group, N)
    amax = np.max(np.abs(wg), axis=1)
    s = round_bf16((amax / np.float32(7.0)).astype(np.float32))
    s = np.where(s == 0, np.float32(1.0), s).astype(np.float32)
    q = np.clip(np.rint((wg / s[:, None, :]).astype(np.float32)), -7, 7).astype(np.int8).reshape(K, N)
    lo = (q[0::2] & 0xF).astype(np.uint8)
    hi = (q[1::2] & 0xF).astype(np.uint8)
    return (lo | (hi << 4)).astype(np.uint8), s


def dequantize_int8(q: np.ndarray, s: np.ndarray) -> np.ndarray:
    return (q.astype(np.float32) * s[None, :].astype(np.float32)).astype(np.float32)


def dequantize_int4_g128(packed: np.ndarray, s: np.ndarray, group: int = 128) -> np.ndarray:
    lo = (packed & 0xF).astype(np.int8)
    hi = (packed >> 4).astype(np.int8)
    lo = np.where(lo > 7, lo - 16, lo)
    hi = np.where(hi > 7, hi - 16, hi)
    K = packed.shape[0] * 2
    q = np.empty((K, packed.shape[1]), dtype=np.int8)
    q[0::2], q[1::2] = lo, hi
    sk = np.repeat(s.astype(np.float32), group, axis=0)
    return (q.astype(np.float32) * sk).astype(np.float32)


def _norm_call(target: str, attrs, ins: List[OTensor], out_dtype: str) -> OTensor:
    """gpt_rs.hip.layer_norm.v1 (x, gamma, beta) / gpt_rs.hip.rms_norm.v1 (x, gamma), attribute eps: what a front-end
    pass puts in place of the functional's instruction sequence (crates/gpt-rs/src/ops/functional/normalization.rs:
    123-217).  Defined as that sequence: the same operations in the same order through the same op_* functions, every
    intermediate in the tensor's dtype, so a program with the call computes bit for bit what the program with the
    sequence computes."""
    eps_attr = (attrs or {}).get("eps")
    if not isinstance(eps_attr, dict) or "value" not in eps_attr:
        raise OracleError("spec", f"{target}: attribute `eps` (F64) is missing")
    x = ins[0]
    dt, dims = x.dtype, tuple(x.a.shape)
    n = dims[-1]
    red = dims[:-1] + (1,)
    axis = len(dims) - 1

    def lit(v):   # scalar(v) broadcast to the reduced shape: a literal of the tensor's dtype (ops/ptir/graph.rs:2278-2298)
        a = np.full(red, np.float32(v), dtype=np.float32)
        return _finish(dt, a)

    inv_count = lit(np.float32(1.0) / np.float32(n))
    eps = lit(float(eps_attr["value"]))
    if target == "gpt_rs.hip.layer_norm.v1":
        if len(ins) != 3:
            raise OracleError("spec", f"{target}: expects (x, gamma, beta)")
        mean = op_binary(op_reduce(x, "Sum", [axis], True), inv_count, "Mul")
        centered = op_binary(x, op_broadcast_to(mean, dims), "Sub")
        var_mean = op_binary(op_reduce(op_binary(centered, centered, "Mul"), "Sum", [axis], True), inv_count, "Mul")
        inv_std = op_unary(op_binary(var_mean, eps, "Add"), "Rsqrt")
        normalized = op_binary(centered, op_broadcast_to(inv_std, dims), "Mul")
        out = op_binary(op_binary(normalized, op_broadcast_to(ins[1], dims), "Mul"), op_broadcast_to(ins[2], dims), "Add")
    else:
        if len(ins) != 2:
            raise OracleError("spec", f"{target}: expects (x, gamma)")
        mean_square = op_binary(op_reduce(op_binary(x, x, "Mul"), "Sum", [axis], True), inv_count, "Mul")
        inv_rms = op_unary(op_binary(mean_square, eps, "Add"), "Rsqrt")
        out = op_binary(op_binary(x, op_broadcast_to(inv_rms, dims), "Mul"), op_broadcast_to(ins[1], dims), "Mul")
    if out.dtype != out_dtype:
        raise OracleError("spec", f"{target}: the output has x's type")
    return out


def _custom_call(target: str, attrs, ins: List[OTensor], out_dtype: str, out_dims) -> OTensor:
    if target in ("gpt_rs.hip.layer_norm.v1", "gpt_rs.hip.rms_norm.v1"):
        return _norm_call(target, attrs, ins, out_dtype)
    if target == "gpt_rs.hip.dot_w8.v1":
        x, q, s = ins
        w = dequantize_int8(q.a, s.a)
    elif target == "gpt_rs.hip.dot_w4g128.v1":
        x, q, s = ins
        w = dequantize_int4_g128(q.a, s.a)
    elif target in ("gpt_rs.hip.quantize_w8_scales.v1", "gpt_rs.hip.quantize_w4g128_scales.v1"):
        (w,) = ins
        s = (quantize_int8_per_channel if "w8" in target else quantize_int4_g128)(w.a)[1]
        return _finish(out_dtype, s)           # bf16-representable either way: the store is exact
    elif target in ("gpt_rs.hip.quantize_w8.v1", "gpt_rs.hip.quantize_w4g128.v1"):
        w = ins[0]                              # the scales operand is by definition the scheme's own
        q = (quantize_int8_per_channel if "w8" in target else quantize_int4_g128)(w.a)[0]
        return OTensor(out_dtype, q)
    elif target == "gpt_rs.hip.dequantize_w8.v1":
        return _finish(out_dtype, dequantize_int8(ins[0].a, ins[1].a))
    elif target == "gpt_rs.hip.dequantize_w4g128.v1":
        return _finish(out_dtype, dequantize_int4_g128(ins[0].a, ins[1].a))
    else:
        raise OracleError("unimplemented", f"custom_call target {target}")
    # reference semantics for "dequantize + dot_general": f32 accumulate, output rounded
    a = np.ascontiguousarray(x.a, dtype=np.float32)
    wb = round_bf16(w) if x.dtype == "Bf16" else w
    wb = np.ascontiguousarray(wb, dtype=np.float32)
    return _finish(out_dtype, _bmm(a[None], wb[None])[0])


# ----------------------------------------------------------------------------- interpreter
def execute_instruction(instr, inputs: List[OTensor]) -> OTensor:     # cpu.rs:257-334
    out = instr["output"]
    if "Tensor" not in out:
        raise OracleError("execution", "tuple outputs are not supported")
    out_dtype, out_dims = _spec(out["Tensor"])
    op = instr["op"]
    if isinstance(op, str):
        name, attr = op, None
    else:
        (name, attr), = op.items()
    if name == "Constant":
        dt, dims = _spec(attr["spec"])
        res = OTensor.from_bytes(dt, dims, bytes(attr["bytes"]))
    elif name == "Reshape":
        res = op_reshape(inputs[0], out_dims)
    elif name == "Slice":
        res = op_slice(inputs[0], attr["starts"], attr["sizes"])
    elif name == "Transpose":
        res = op_transpose(inputs[0], attr["perm"])
    elif name == "BroadcastTo":
        res = op_broadcast_to(inputs[0], [d["Static"] for d in attr["result_shape"]["dims"]])
    elif name == "DotGeneral":
        if len(inputs) != 2:
            raise OracleError("execution", "dot_general expects two inputs")
        res = op_dot_general(inputs[0], inputs[1], attr)
    elif name == "ElementwiseBinary":
        if len(inputs) != 2:
            raise OracleError("execution", "elementwise binary expects 2 inputs")
        res = op_binary(inputs[0], inputs[1], attr)
    elif name == "ElementwiseUnary":
        res = op_unary(inputs[0], attr)
    elif name == "Reduce":
        res = op_reduce(inputs[0], attr["kind"], attr["axes"], attr["keepdims"])
    elif name == "Compare":
        res = op_compare(inputs[0], inputs[1], attr["op"])
    elif name == "Select":
        if len(inputs) != 3:
            raise OracleError("execution", "select expects three operands")
        res = op_select(*inputs)
    elif name == "Cast":
        res = op_cast(inputs[0], attr["dtype"])
    elif name == "Concat":
        res = op_concat(inputs, attr["axis"])
    elif name == "Take":
        if len(inputs) != 2:
            raise OracleError("execution", "take expects two operands")
        res = op_take(inputs[0], inputs[1])
    elif name == "Iota":
        dt, dims = attr["dtype"], [d["Static"] for d in attr["shape"]["dims"]]
        res = op_iota(dims, dt, attr["axis"])
    elif name == "DynamicSlice":
        res = op_dynamic_slice(inputs[0], inputs[1], attr["sizes"])
    elif name == "DynamicUpdateSlice":
        if len(inputs) != 3:
            raise OracleError("execution", "dynamic_update_slice expects (base, update, starts)")
        res = op_dynamic_update_slice(inputs[0], inputs[1], inputs[2], attr["sizes"])
    elif name == "CustomCall":
        res = _custom_call(attr["target"], attr.get("attrs", {}), inputs, out_dtype, out_dims)
    elif name == "StopGradient":
        res = inputs[0]
    else:
        raise OracleError("unimplemented", f"{name}: operation not supported in cpu portable backend")
    if res.dtype != out_dtype or res.dims != tuple(out_dims):
        raise OracleError("execution", f"{name}: result {res.dtype}{res.dims} != declared {out_dtype}{tuple(out_dims)}")
    return res


def run_program(program, entry_inputs: Sequence[OTensor]) -> List[OTensor]:  # cpu.rs:120-181
    if isinstance(program, (bytes, str)):
        program = json.loads(program)
    if program.get("spec_version", "ptir.v0.4") not in ("", "ptir.v0.4"):
        raise OracleError("spec", f"program spec version '{program['spec_version']}' does not match expected 'ptir.v0.4'")
    fn = next((f for f in program["functions"] if f["name"] == program["entry"]), None)
    if fn is None:
        raise OracleError("execution", "entry function not found")
    if len(fn["parameter_ids"]) != len(entry_inputs):
        raise OracleError("execution", "entry input arity mismatch")
    values: Dict[int, OTensor] = dict(zip(fn["parameter_ids"], entry_inputs))
    for instr in fn["body"]:
        ins = []
        for od in instr["operands"]:
            if "Value" in od:
                if od["Value"] not in values:
                    raise OracleError("execution", "operand value missing")
                ins.append(values[od["Value"]])
            elif "Literal" in od:
                dt, dims = _spec(od["Literal"]["spec"])
                ins.append(OTensor.from_bytes(dt, dims, bytes(od["Literal"]["bytes"])))
            else:
                raise OracleError("execution", "tuple operands not supported")
        values[instr["id"]] = execute_instruction(instr, ins)
    out = []
    for rid in fn["result_ids"]:
        if rid not in values:
            raise OracleError("execution", "missing function result value")
        out.append(values[rid])
    return out


def sample_temperature(logits_row: np.ndarray, temperature: float, random_u: float) -> int:
    """Temperature sampling of the reference's device path: Gumbel-max over a stateless per-index hash
    (crates/gpt-rs-backend-triton/src/kernels/sample_temperature_last_axis_f32.triton:24-72; seed from random_u as
    in runtime/sampling.rs:98-101).  All arithmetic in uint32 / float32 as there; ties -> smallest index."""
    row = np.asarray(logits_row, dtype=np.float32)
    bits = np.float32(random_u).view(np.uint32)
    seed = np.uint32((int(bits) * 747796405 + 2891336453) & 0xFFFFFFFF)
    x = np.arange(row.size, dtype=np.uint32) ^ seed
    x ^= x >> np.uint32(16)
    x = (x.astype(np.uint64) * np.uint64(0x7FEB352D)).astype(np.uint32)
    x ^= x >> np.uint32(15)
    x = (x.astype(np.uint64) * np.uint64(0x846CA68B)).astype(np.uint32)
    x ^= x >> np.uint32(16)
    u = (x.astype(np.float32) + np.float32(1.0)) * np.float32(1.0 / 4294967297.0)
    u = np.minimum(np.maximum(u, np.float32(1e-7)), np.float32(1.0) - np.float32(1e-7))
    gumbel = -np.log(-np.log(u, dtype=np.float32), dtype=np.float32)
    score = row * (np.float32(1.0) / np.float32(temperature)) + gumbel
    return int(np.argmax(score))


def argmax_first(logits_row: np.ndarray) -> int:
    """Greedy token: smallest index among maxima (docs/backend.md:270).  The host sampler
    (crates/gpt-rs/src/inference/sampler.rs:96-103) differs only on exact ties."""
    return int(np.argmax(logits_row))
