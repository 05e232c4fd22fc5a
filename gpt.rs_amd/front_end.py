"""The reference's optimizer between the functional emitters and `run_program`, restated.

Every program the reference hands to a backend has been through `PipelineOptimizer`
(crates/gpt-rs/src/backend/pipeline.rs:74-119):

    fixed point (2 rounds)   six canonicalisers
    [backend pre / legalize hooks]
    ParamOnlyFoldToParamPass
    [backend fuse hook]
    fixed point (4 rounds)   six canonicalisers, CSE, DCE
    [backend cleanup hook]

so what a backend's pattern matcher sees is not the emitters' instruction stream: identity reshapes / broadcasts /
transposes are gone, chains are collapsed, equal instructions are merged across layers, and every value computed from
exactly one Param and literals (`BroadcastTo(in)(gamma)`, a bias broadcast) has been executed once through
`run_program` and replaced by a derived Param input of the broadcast shape.  The model drivers run their programs
through `optimize` before the backend sees them, as the reference's arena does (ops/graph/arena.rs:744-922).

The passes follow, file by file:
  greedy driver + rewriter    backend/driver.rs:32-140, backend/rewriter.rs:110-225, backend/index.rs:95-190
  broadcast / reshape / transpose / slice / cast canonicalisers, elementwise simplification
                              backend/passes/{broadcast,reshape,transpose,slice,cast}_canonicalization.rs,
                              backend/passes/elementwise_simplification.rs
  CSE, DCE                    backend/passes/cse.rs:32-105, backend/passes/dce.rs:19-76
  ParamOnlyFoldToParam        backend/passes/param_only_fold_to_param.rs:24-160, optimizer/entry.rs:66-135

Value ids, instruction order and the order of parameters come out as the reference's do (a rewrite's new value takes
the next free id, a derived Param is appended): the reference's fixtures (crates/gpt-rs/tests/fixtures/*.lit) are
reproduced as text.  The integer value of a derived Param's stable id is NOT the reference's: it hashes bincode
serialisations (param_only_fold_to_param.rs:453-509) and this restatement hashes canonical JSON with the same FNV-1a
scheme; only uniqueness and stability reach a backend.
"""
from __future__ import annotations

import copy
import json
import math
import struct
from collections import deque
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

from .ptir import SPEC_VERSION, Program, TensorSpec

ARG, PARAM = "Arg", "Param"          # tensor/lazy_tensor.rs:10-13

PRE_ITERS, POST_ITERS = 2, 4          # env.rs:25-41 defaults


@dataclass
class EntryParam:
    """optimizer/entry.rs:9-15.  `stable_id` is the u128 as an int (None for an Arg without one)."""

    id: int
    type: dict
    role: str
    stable_id: Optional[int]


def stable_id_bytes(stable_id: int) -> bytes:
    return int(stable_id).to_bytes(16, "little")


# ------------------------------------------------------------------------------------------ op helpers
def op_name(op) -> str:
    return op if isinstance(op, str) else next(iter(op))


def op_attrs(op):
    return None if isinstance(op, str) else next(iter(op.values()))


def _static_dims(ty: dict) -> Tuple[int, ...]:
    return tuple(d["Static"] for d in ty["Tensor"]["shape"]["dims"])


def _value_operand(o) -> Optional[int]:
    return o["Value"] if "Value" in o else None


# ------------------------------------------------------------------------------------------ rewriter
class Rewriter:
    """ProgramRewriter + FunctionIndices (rewriter.rs, index.rs): def-use bookkeeping over one function's body.
    An instruction is identified by the value it defines."""

    def __init__(self, fn: dict):
        self.fn = fn
        self.types: Dict[int, dict] = dict(zip(fn["parameter_ids"], fn["parameters"]))
        self.inst: Dict[int, dict] = {}
        self.users: Dict[int, List[int]] = {}
        self.version: Dict[int, int] = {}
        max_value = 0
        for pid in fn["parameter_ids"]:
            max_value = max(max_value, pid)
        for ins in fn["body"]:
            self._index(ins)
            max_value = max(max_value, ins["id"])
        self.next_value = max_value + 1   # index.rs:95-113

    def _index(self, ins: dict):
        self.inst[ins["id"]] = ins
        self.types[ins["id"]] = ins["output"]
        self.version[ins["id"]] = 0
        for o in ins["operands"]:
            v = _value_operand(o)
            if v is not None:
                self.users.setdefault(v, []).append(ins["id"])

    def order(self) -> List[int]:
        return [ins["id"] for ins in self.fn["body"]]

    def contains(self, vid: int) -> bool:
        return vid in self.inst

    def users_of(self, vid: int) -> List[int]:
        return self.users.get(vid, [])

    def replace_all_uses(self, frm: int, to: int):
        """rewriter.rs:110-134."""
        if frm == to:
            return
        for user in list(dict.fromkeys(self.users.get(frm, []))):
            ins = self.inst[user]
            n = 0
            for o in ins["operands"]:
                if o.get("Value") == frm:
                    o["Value"] = to
                    n += 1
            self.users.setdefault(to, []).extend([user] * n)
            self.version[user] += 1
        self.users[frm] = []

    def replace_value(self, frm: int, to: int):
        """What every pattern does with its root: rewire the uses and the function results, erase the root."""
        self.replace_all_uses(frm, to)
        self.fn["result_ids"] = [to if r == frm else r for r in self.fn["result_ids"]]
        if frm in self.inst:
            self.erase(frm)

    def erase(self, vid: int):
        """rewriter.rs:137-153: only an instruction without users goes."""
        if self.users.get(vid):
            raise RuntimeError(f"erase of %{vid} with live uses")
        ins = self.inst.pop(vid)
        self.fn["body"].remove(ins)
        del self.version[vid]
        for o in ins["operands"]:
            v = _value_operand(o)
            if v is not None and vid in self.users.get(v, []):
                self.users[v].remove(vid)

    def insert_before(self, at: int, op, operands: List[dict], output: dict) -> int:
        """rewriter.rs:156-225: the new instruction defines the next free value id."""
        vid = self.next_value
        self.next_value += 1
        ins = {"id": vid, "op": op, "operands": operands, "output": output}
        self.fn["body"].insert(self.fn["body"].index(self.inst[at]), ins)
        self._index(ins)
        return vid


Pattern = Callable[[dict, Rewriter], bool]

SIDE_EFFECTS_DCE = ("ScatterAdd", "Cond", "While", "Scan", "RngUniform", "RngNormal")          # driver.rs:143-152, dce.rs:66-76
SIDE_EFFECTS_CSE = SIDE_EFFECTS_DCE + ("TopK", "Quantize", "Dequantize", "Requantize")             # cse.rs:11-25


def _greedy_dce(rw: Rewriter) -> int:
    """driver.rs:106-137: unused instructions go, last to first, until nothing changes."""
    removed = 0
    while True:
        n = 0
        for vid in reversed(rw.order()):
            if not rw.contains(vid) or op_name(rw.inst[vid]["op"]) in SIDE_EFFECTS_DCE:
                continue
            if vid in rw.fn["result_ids"]:
                continue
            if not rw.users_of(vid):
                rw.erase(vid)
                n += 1
        if n == 0:
            return removed
        removed += n


def apply_patterns_greedily(fn: dict, patterns: Dict[str, List[Pattern]]) -> Tuple[int, int]:
    """apply_patterns_and_fold_greedily (driver.rs:32-96): instructions are visited in body order, the first pattern
    that rewrites wins and the walk starts over; an (instruction, pattern) pair that failed is not tried again until
    the instruction's operands change.  Returns (rewrites applied, instructions removed as dead)."""
    rw = Rewriter(fn)
    work = deque(rw.order())
    failed: Dict[Tuple[int, int], int] = {}
    applied = 0
    while work:
        vid = work.popleft()
        if not rw.contains(vid):
            continue
        version = rw.version[vid]
        ins = rw.inst[vid]
        for idx, pat in enumerate(patterns.get(op_name(ins["op"]), ())):
            if failed.get((idx, vid)) == version:
                continue
            if pat(ins, rw):
                applied += 1
                for k in [k for k in failed if k[1] == vid]:
                    del failed[k]
                work = deque(rw.order())
                break
            failed[(idx, vid)] = version
    return applied, _greedy_dce(rw)


# ------------------------------------------------------------------------------------------ canonicalisers
def _single_value(ins: dict) -> Optional[int]:
    ops = ins["operands"]
    return ops[0]["Value"] if len(ops) == 1 and "Value" in ops[0] else None


def _eliminate_identity_broadcast(ins, rw):   # broadcast_canonicalization.rs:12-45
    src = _single_value(ins)
    if src is None or rw.types[src]["Tensor"]["shape"] != ins["output"]["Tensor"]["shape"]:
        return False
    rw.replace_value(ins["id"], src)
    return True


def _broadcast_compatible(frm: Sequence[int], to: Sequence[int]) -> bool:   # broadcast_canonicalization.rs:112-133
    if len(frm) > len(to):
        return False
    off = len(to) - len(frm)
    return all(f == 1 or f == to[i + off] for i, f in enumerate(frm))


def _collapse_broadcast_chain(ins, rw):   # broadcast_canonicalization.rs:48-110
    inner_v = _single_value(ins)
    inner = rw.inst.get(inner_v) if inner_v is not None else None
    if inner is None or op_name(inner["op"]) != "BroadcastTo":
        return False
    base = _single_value(inner)   # a literal operand ends the chain
    if base is None:
        return False
    if not _broadcast_compatible(_static_dims(rw.types[base]), _static_dims(ins["output"])):
        return False
    new = rw.insert_before(ins["id"], {"BroadcastTo": {"result_shape": copy.deepcopy(op_attrs(ins["op"])["result_shape"])}},
                           [{"Value": base}], copy.deepcopy(ins["output"]))
    rw.replace_value(ins["id"], new)
    return True


def _eliminate_identity_reshape(ins, rw):   # reshape_canonicalization.rs:16-45
    src = _single_value(ins)
    if src is None or rw.types[src]["Tensor"] != ins["output"]["Tensor"]:
        return False
    rw.replace_value(ins["id"], src)
    return True


def _collapse_reshape_chain(ins, rw):   # reshape_canonicalization.rs:48-122
    inner_v = _single_value(ins)
    inner = rw.inst.get(inner_v) if inner_v is not None else None
    if inner is None or op_name(inner["op"]) != "Reshape":
        return False
    base = _single_value(inner)
    if base is None:
        return False
    dims = _static_dims(ins["output"])
    if math.prod(_static_dims(rw.types[base])) != math.prod(dims):
        return False
    new = rw.insert_before(ins["id"], {"Reshape": {"new_shape": [{"Explicit": {"Static": d}} for d in dims]}},
                           [{"Value": base}], copy.deepcopy(ins["output"]))
    rw.replace_value(ins["id"], new)
    return True


def _eliminate_identity_transpose(ins, rw):   # transpose_canonicalization.rs:30-52
    perm = op_attrs(ins["op"])["perm"]
    src = _single_value(ins)
    if list(perm) != list(range(len(perm))) or src is None:
        return False
    rw.replace_value(ins["id"], src)
    return True


def _collapse_transpose_chain(ins, rw):   # transpose_canonicalization.rs:55-124
    inner_v = _single_value(ins)
    inner = rw.inst.get(inner_v) if inner_v is not None else None
    if inner is None or op_name(inner["op"]) != "Transpose":
        return False
    first, second = op_attrs(inner["op"])["perm"], op_attrs(ins["op"])["perm"]
    if len(first) != len(second) or any(a >= len(first) for a in second):
        return False
    composed = [first[a] for a in second]
    base = _single_value(inner)
    if base is None:
        return False
    if composed == list(range(len(composed))):
        rw.replace_value(ins["id"], base)
        return True
    new = rw.insert_before(ins["id"], {"Transpose": {"perm": composed}}, [{"Value": base}], copy.deepcopy(ins["output"]))
    rw.replace_value(ins["id"], new)
    return True


def _compose_slices(inner: dict, outer: dict) -> Optional[dict]:   # slice_canonicalization.rs:11-41
    if len(inner["starts"]) != len(outer["starts"]) or len(inner["sizes"]) != len(outer["sizes"]):
        return None
    starts, sizes = [], []
    for i_start, i_size, o_start, o_size in zip(inner["starts"], inner["sizes"], outer["starts"], outer["sizes"]):
        if o_start > i_size:
            return None
        new_start = i_start + o_start
        if new_start > i_start + i_size:
            return None
        if o_size > max(i_size - o_start, 0):
            return None
        starts.append(new_start)
        sizes.append(o_size)
    return {"starts": starts, "sizes": sizes}


def _collapse_slice_chain(ins, rw):   # slice_canonicalization.rs:83-124
    inner_v = _single_value(ins)
    inner = rw.inst.get(inner_v) if inner_v is not None else None
    if inner is None or op_name(inner["op"]) != "Slice":
        return False
    composed = _compose_slices(op_attrs(inner["op"]), op_attrs(ins["op"]))
    base = _single_value(inner)
    if composed is None or base is None:
        return False
    new = rw.insert_before(ins["id"], {"Slice": composed}, [{"Value": base}], copy.deepcopy(ins["output"]))
    rw.replace_value(ins["id"], new)
    return True


def _eliminate_redundant_cast(ins, rw):   # cast_canonicalization.rs:14-38
    src = _single_value(ins)
    if src is None or rw.types[src] != ins["output"]:
        return False
    rw.replace_value(ins["id"], src)
    return True


def _scalar_f32_from_literal(lit: dict) -> Optional[float]:   # elementwise_simplification.rs:16-35
    if lit["spec"]["dtype"] != "F32":
        return None
    dims = [d.get("Static") for d in lit["spec"]["shape"]["dims"]]
    if dims and not all(d in (0, 1) for d in dims):
        return None
    data = bytes(lit["bytes"])
    if len(data) != 4:
        return None
    return struct.unpack("<f", data)[0]


def _scalar_f32_from_value(vid: int, rw: Rewriter) -> Optional[float]:   # elementwise_simplification.rs:37-52
    ins = rw.inst.get(vid)
    if ins is None:
        return None
    name = op_name(ins["op"])
    if name == "Constant":
        return _scalar_f32_from_literal(op_attrs(ins["op"]))
    if name == "BroadcastTo" and len(ins["operands"]) == 1:
        o = ins["operands"][0]
        if "Value" in o:
            return _scalar_f32_from_value(o["Value"], rw)
        if "Literal" in o:
            return _scalar_f32_from_literal(o["Literal"])
    return None


def _simplify_elementwise_binary(ins, rw):   # elementwise_simplification.rs:92-184
    ops = ins["operands"]

    def side(i):
        if i >= len(ops):
            return None, None
        o = ops[i]
        if "Value" in o:
            return o["Value"], _scalar_f32_from_value(o["Value"], rw)
        if "Literal" in o:
            return None, _scalar_f32_from_literal(o["Literal"])
        return None, None

    (lhs, ls), (rhs, rs) = side(0), side(1)
    kind = op_attrs(ins["op"])
    pick = None
    if kind == "Add":
        if rs == 0.0 and lhs is not None:
            pick = lhs
        elif ls == 0.0 and rhs is not None:
            pick = rhs
    elif kind == "Sub":
        if rs == 0.0 and lhs is not None:
            pick = lhs
    elif kind == "Mul":
        if rs == 1.0 and lhs is not None:
            pick = lhs
        elif ls == 1.0 and rhs is not None:
            pick = rhs
        elif rs == 0.0 and rhs is not None:
            pick = rhs
        elif ls == 0.0 and lhs is not None:
            pick = lhs
    elif kind == "Div":
        if rs == 1.0 and lhs is not None:
            pick = lhs
    if pick is None:
        return False
    rw.replace_value(ins["id"], pick)
    return True


class GreedyPass:
    def __init__(self, name: str, patterns: Dict[str, List[Pattern]]):
        self.name, self.patterns = name, patterns

    def run(self, fn: dict, cx: "OptimizeContext") -> bool:
        applied, removed = apply_patterns_greedily(fn, self.patterns)
        return applied > 0 or removed > 0


def broadcast_canonicalization():
    return GreedyPass("broadcast-canonicalize", {"BroadcastTo": [_eliminate_identity_broadcast, _collapse_broadcast_chain]})


def reshape_canonicalization():
    return GreedyPass("reshape-canonicalize", {"Reshape": [_eliminate_identity_reshape, _collapse_reshape_chain]})


def transpose_canonicalization():
    return GreedyPass("transpose-canonicalize", {"Transpose": [_eliminate_identity_transpose, _collapse_transpose_chain]})


def slice_canonicalization():
    return GreedyPass("slice-canonicalize", {"Slice": [_collapse_slice_chain]})


def cast_canonicalization():
    return GreedyPass("cast-canonicalize", {"Cast": [_eliminate_redundant_cast]})


def elementwise_simplification():
    return GreedyPass("elementwise-simplify", {"ElementwiseBinary": [_simplify_elementwise_binary]})


def canonicalizers():
    """pipeline.rs:80-87, in this order."""
    return [broadcast_canonicalization(), reshape_canonicalization(), transpose_canonicalization(), slice_canonicalization(),
            cast_canonicalization(), elementwise_simplification()]


# ------------------------------------------------------------------------------------------ CSE / DCE
def _canon(obj) -> bytes:
    return json.dumps(obj, sort_keys=True, separators=(",", ":")).encode()


class CommonSubexpressionElimination:
    """cse.rs:32-105: a later instruction equal in (operation, operands, result type) to an earlier one is replaced by it."""

    name = "cse"

    def run(self, fn: dict, cx: "OptimizeContext") -> bool:
        rw = Rewriter(fn)
        seen: Dict[bytes, int] = {}
        changed = False
        for vid in rw.order():
            if not rw.contains(vid):
                continue
            ins = rw.inst[vid]
            if op_name(ins["op"]) in SIDE_EFFECTS_CSE:
                continue
            key = _canon([ins["op"], ins["operands"], ins["output"]])
            first = seen.get(key)
            if first is None:
                seen[key] = vid
            elif first != vid:
                rw.replace_value(vid, first)
                changed = True
        return changed


class DeadCodeElimination:
    """dce.rs:19-64: what no result (and no side-effecting instruction) reaches goes, entry parameters included
    (optimizer/entry.rs:107-135)."""

    name = "dce"

    def run(self, fn: dict, cx: "OptimizeContext") -> bool:
        defs = {ins["id"]: ins for ins in fn["body"]}
        work = list(fn["result_ids"]) + [ins["id"] for ins in fn["body"] if op_name(ins["op"]) in SIDE_EFFECTS_DCE]
        live = set()
        while work:
            v = work.pop()
            if v in live:
                continue
            live.add(v)
            ins = defs.get(v)
            if ins is not None:
                work.extend(o["Value"] for o in ins["operands"] if "Value" in o)
        before = len(fn["body"])
        fn["body"] = [ins for ins in fn["body"] if ins["id"] in live or op_name(ins["op"]) in SIDE_EFFECTS_DCE]
        cx.remove_params_by_live_set(fn, live)
        return len(fn["body"]) < before


# ------------------------------------------------------------------------------------------ param-only fold
FNV_INIT, FNV_PRIME, MASK64 = 0xCBF29CE484222325, 0x100000001B3, (1 << 64) - 1


def _fnv(h: int, data: bytes) -> int:
    for b in data:
        h = ((h ^ b) * FNV_PRIME) & MASK64
    return h


def _fnv_u64(h: int, v: int) -> int:
    return _fnv(h, (v & MASK64).to_bytes(8, "little"))


def _fnv_u128(h: int, v: int) -> int:
    return _fnv(h, int(v).to_bytes(16, "little"))


def _rotl64(v: int, r: int) -> int:
    return ((v << r) | (v >> (64 - r))) & MASK64


def _hash_literal(h: int, lit: dict) -> int:
    return _fnv(_fnv(_fnv(h, b"lit"), _canon(lit["spec"])), bytes(lit["bytes"]))


class OptimizeContext:
    """OptimizeContext + EntrySignature (optimizer/context.rs, optimizer/entry.rs)."""

    def __init__(self, backend, resolver, entry: List[EntryParam]):
        self.backend, self.resolver = backend, resolver
        self.entry = list(entry)
        self.failed_fold_keys = set()
        self.folds_run = 0          # subgraphs executed through run_program
        self.folds_reused = 0       # derived ids the resolver already held

    def param(self, vid: int) -> Optional[EntryParam]:
        for p in self.entry:
            if p.id == vid:
                return p
        return None

    def role_of(self, vid: int) -> Optional[str]:
        p = self.param(vid)
        return p.role if p else None

    def get_or_add_param(self, fn: dict, stable_id: int, ty: dict) -> Optional[int]:
        """entry.rs:66-105 for role Param: one entry parameter per stable id, a new one takes the next free id."""
        for p in self.entry:
            if p.role == PARAM and p.stable_id == stable_id:
                return p.id if p.type == ty else None
        vid = max([0] + fn["parameter_ids"] + [ins["id"] for ins in fn["body"]]) + 1
        fn["parameter_ids"].append(vid)
        fn["parameters"].append(copy.deepcopy(ty))
        self.entry.append(EntryParam(vid, copy.deepcopy(ty), PARAM, stable_id))
        return vid

    def remove_params_by_live_set(self, fn: dict, live):
        keep = [(i, t) for i, t in zip(fn["parameter_ids"], fn["parameters"]) if i in live]
        fn["parameter_ids"] = [i for i, _ in keep]
        fn["parameters"] = [t for _, t in keep]
        by_id = {p.id: p for p in self.entry}
        self.entry = [by_id[i] for i, _ in keep if i in by_id]


class ParamOnlyFoldToParam:
    """param_only_fold_to_param.rs:24-160.  A value is static when it depends on Param inputs and literals only.  A static
    value that a non-static instruction reads (or that is a result), whose leaves are exactly ONE Param, is computed once
    by `backend.run_program` on the subgraph with that Param as its only input, stored in the resolver under a derived
    stable id, and replaced in the function by a new Param input."""

    name = "param-only-fold-to-param"

    def run(self, fn: dict, cx: OptimizeContext) -> bool:
        if cx.resolver is None:
            return False
        total = False
        while True:
            defs = {ins["id"]: ins for ins in fn["body"]}
            types = dict(zip(fn["parameter_ids"], fn["parameters"]))
            types.update({ins["id"]: ins["output"] for ins in fn["body"]})
            memo: Dict[int, bool] = {}

            def is_static(v: int) -> bool:
                if v in memo:
                    return memo[v]
                if v in fn["parameter_ids"]:
                    memo[v] = cx.role_of(v) == PARAM
                    return memo[v]
                ins = defs.get(v)
                if ins is None:
                    memo[v] = False
                    return False
                flag = True
                for o in ins["operands"]:
                    if "Literal" in o:
                        continue
                    if "Value" in o and is_static(o["Value"]):
                        continue
                    flag = False
                    break
                memo[v] = flag
                return flag

            param_set = set(fn["parameter_ids"])
            dynamic_users = set()
            for ins in fn["body"]:
                if not is_static(ins["id"]):
                    dynamic_users.update(o["Value"] for o in ins["operands"] if "Value" in o)
            targets = [ins["id"] for ins in fn["body"]
                       if is_static(ins["id"]) and (ins["id"] in dynamic_users or ins["id"] in fn["result_ids"])]
            if not targets:
                break
            changed = False
            for target in targets:
                used = any(o.get("Value") == target for ins in fn["body"] for o in ins["operands"])
                if not used and target not in fn["result_ids"]:
                    continue
                desc = self._describe(fn, cx, defs, param_set, target)
                if desc is None:
                    continue
                leaf_ids, leaf_stable, inst_set, literal_hash = desc
                if len(leaf_stable) != 1:
                    continue
                dag_hash = self._dag_hash(fn, cx, defs, types, target)
                name = cx.backend.backend_name()
                derived = self._derived_id(name, dag_hash, literal_hash, leaf_stable)
                fail_key = _fnv_u64(_fnv(_fnv(FNV_INIT, b"ptir:fold_fail"), name.encode()), dag_hash)
                if fail_key in cx.failed_fold_keys:
                    continue
                if cx.resolver.get(stable_id_bytes(derived)) is not None:
                    cx.folds_reused += 1
                else:
                    leaf = cx.resolver.get(stable_id_bytes(leaf_stable[0]))
                    if leaf is None:
                        cx.failed_fold_keys.add(fail_key)
                        continue
                    sub = self._subgraph(fn, target, types, leaf_ids, inst_set)
                    try:
                        outs = cx.backend.run_program(sub, [leaf])
                    except Exception:
                        cx.failed_fold_keys.add(fail_key)
                        continue
                    if len(outs) != 1:
                        cx.failed_fold_keys.add(fail_key)
                        continue
                    cx.resolver.set(stable_id_bytes(derived), outs[0])
                    cx.folds_run += 1
                replacement = cx.get_or_add_param(fn, derived, types[target])
                if replacement is None:
                    continue
                if replacement != target:
                    for ins in fn["body"]:
                        for o in ins["operands"]:
                            if o.get("Value") == target:
                                o["Value"] = replacement
                    fn["result_ids"] = [replacement if r == target else r for r in fn["result_ids"]]
                changed = True
            if not changed:
                break
            total = True
        return total

    @staticmethod
    def _describe(fn, cx, defs, param_set, target):
        """describe_static_subgraph (param_only_fold_to_param.rs:224-315)."""
        inst_set, leaves = set(), set()
        lit_hash = [FNV_INIT]

        def dfs(v: int) -> bool:
            if v in param_set:
                if cx.role_of(v) == PARAM:
                    leaves.add(v)
                    return True
                return False
            ins = defs.get(v)
            if ins is None:
                return False
            if v in inst_set:
                return True
            inst_set.add(v)
            for o in ins["operands"]:
                if "Literal" in o:
                    lit_hash[0] = _hash_literal(lit_hash[0], o["Literal"])
                elif "Value" in o:
                    if not dfs(o["Value"]):
                        return False
                else:
                    return False
            return True

        if not dfs(target):
            return None
        leaf_ids = sorted(leaves)
        stable = []
        for v in leaf_ids:
            sid = cx.param(v).stable_id
            if sid is None:
                return None
            stable.append(sid)
        return leaf_ids, sorted(set(stable)), inst_set, lit_hash[0]

    @staticmethod
    def _dag_hash(fn, cx, defs, types, value) -> int:
        """dag_hash_value (param_only_fold_to_param.rs:393-451), with canonical JSON where the reference hashes bincode."""
        memo: Dict[int, int] = {}

        def rec(v: int) -> int:
            if v in memo:
                return memo[v]
            h = FNV_INIT
            if v in fn["parameter_ids"]:
                h = _fnv(h, b"param")
                p = cx.param(v)
                h = _fnv_u64(h, {ARG: 0, PARAM: 1}.get(p.role if p else None, 0))
                h = _fnv_u128(h, (p.stable_id or 0) if p else 0)
                h = _fnv(h, _canon(types[v]))
            elif v not in defs:
                h = _fnv(h, b"unknown")
            else:
                ins = defs[v]
                h = _fnv(_fnv(_fnv(h, b"inst"), _canon(ins["op"])), _canon(types[v]))
                for o in ins["operands"]:
                    if "Value" in o:
                        h = _fnv_u64(h, rec(o["Value"]))
                    elif "Literal" in o:
                        h = _hash_literal(h, o["Literal"])
            memo[v] = h
            return h

        return rec(value)

    @staticmethod
    def _derived_id(backend_name: str, dag_hash: int, literal_hash: int, leaf_stable: List[int]) -> int:
        """derived_param_id (param_only_fold_to_param.rs:453-477): two FNV-1a lanes, top bit set."""
        h1 = _fnv_u64(_fnv_u64(_fnv(_fnv(FNV_INIT, b"ptir:derived_param:lo"), backend_name.encode()), dag_hash), literal_hash)
        for leaf in leaf_stable:
            h1 = _fnv_u128(h1, leaf)
        h2 = _fnv(_fnv(FNV_INIT, b"ptir:derived_param:hi"), backend_name.encode())
        h2 = _fnv_u64(_fnv_u64(h2, _rotl64(dag_hash, 13)), _rotl64(literal_hash, 29))
        for leaf in reversed(leaf_stable):
            h2 = _fnv_u128(h2, leaf)
        return ((h2 << 64) | h1) | (1 << 127)

    @staticmethod
    def _subgraph(fn, target, types, leaf_ids, inst_set) -> Program:
        """build_subgraph_program (param_only_fold_to_param.rs:317-369): leaves first, then the instructions in body order,
        ids dense from 0."""
        mapping: Dict[int, int] = {}
        params, body = [], []
        for leaf in leaf_ids:
            mapping[leaf] = len(mapping)
            params.append(copy.deepcopy(types[leaf]))
        for ins in fn["body"]:
            if ins["id"] not in inst_set:
                continue
            operands = [{"Value": mapping[o["Value"]]} if "Value" in o else copy.deepcopy(o) for o in ins["operands"]]
            mapping[ins["id"]] = len(mapping)
            body.append({"id": mapping[ins["id"]], "op": copy.deepcopy(ins["op"]), "operands": operands, "output": copy.deepcopy(ins["output"])})
        sub = {"name": "param_only_fold", "parameters": params, "parameter_ids": list(range(len(params))),
               "results": [copy.deepcopy(types[target])], "body": body, "hints": [], "result_ids": [mapping[target]]}
        return program_from_function(sub, "param_only_fold")


# ------------------------------------------------------------------------------------------ pipeline
def program_from_function(fn: dict, entry: Optional[str] = None) -> Program:
    p = Program.__new__(Program)
    p.obj = {"spec_version": SPEC_VERSION, "entry": entry or fn["name"], "functions": [fn], "regions": []}
    p.param_specs = [TensorSpec.from_json(t["Tensor"]) for t in fn["parameters"]]
    p.result_specs = [TensorSpec.from_json(t["Tensor"]) for t in fn["results"]]
    p._json = None
    p._key = None
    return p


def run_passes(fn: dict, passes, cx: OptimizeContext) -> bool:
    changed = False
    for p in passes:
        changed |= bool(p.run(fn, cx))
    return changed


def _fixed_point(fn: dict, passes, cx: OptimizeContext, max_iters: int) -> bool:
    """pipeline.rs:166-183."""
    changed_any = False
    for _ in range(max(max_iters, 1)):
        if not run_passes(fn, passes, cx):
            break
        changed_any = True
    return changed_any


@dataclass
class OptimizedProgram:
    """What the arena keeps per plan (ops/graph/plan.rs): the program a backend runs and how its inputs are fed
    (arena.rs:1116-1170: Args positionally, Params by stable id)."""

    program: Program
    inputs: List[EntryParam]
    source_index: List[Optional[int]]   # position of each input in the unoptimised program, None for a derived Param
    folds_run: int
    folds_reused: int


def optimize(program: Program, roles: Sequence[str], stable_ids: Sequence[Optional[int]], backend, resolver,
             pre: Sequence = (), legalize: Sequence = (), fuse: Sequence = (), cleanup: Sequence = ()) -> OptimizedProgram:
    """PipelineOptimizer::new + optimize (pipeline.rs:74-145) on the entry function of `program`.  `pre`, `legalize`,
    `fuse`, `cleanup` are a backend pipeline's passes (BackendPipeline, pipeline.rs:60-65), run where the reference
    runs them."""
    fn = copy.deepcopy(program.obj["functions"][0])
    if len(roles) != len(fn["parameter_ids"]) or len(stable_ids) != len(fn["parameter_ids"]):
        raise ValueError("one role and one stable id (or None) per entry parameter")
    entry = [EntryParam(i, t, r, s) for i, t, r, s in zip(fn["parameter_ids"], fn["parameters"], roles, stable_ids)]
    original = list(fn["parameter_ids"])
    cx = OptimizeContext(backend, resolver, entry)
    _fixed_point(fn, canonicalizers(), cx, PRE_ITERS)
    run_passes(fn, list(pre) + list(legalize), cx)
    run_passes(fn, [ParamOnlyFoldToParam()], cx)
    run_passes(fn, list(fuse), cx)
    _fixed_point(fn, canonicalizers() + [CommonSubexpressionElimination(), DeadCodeElimination()], cx, POST_ITERS)
    run_passes(fn, list(cleanup), cx)
    # a result that was replaced by a value of the same type keeps its declared type
    out = program_from_function(fn, program.obj.get("entry"))
    return OptimizedProgram(out, list(cx.entry), [original.index(p.id) if p.id in original else None for p in cx.entry],
                            cx.folds_run, cx.folds_reused)


# ------------------------------------------------------------------------------------------ the hip backend's pipeline
NORM_TARGETS = {"layer_norm": "gpt_rs.hip.layer_norm.v1", "rms_norm": "gpt_rs.hip.rms_norm.v1"}


class HipNormFusionPass:
    """What `gpt-rs-backend-hip`'s BackendPipeline puts into `populate_pre` (crates/gpt-rs/src/backend/pipeline.rs:60-65,
    89-92), the route the reference's Triton backend takes for the same problem
    (crates/gpt-rs-backend-triton/src/optimizer/layer_norm_fusion.rs:30-97, pipeline.rs:15-21): ahead of the
    parameter-only fold, the instruction sequences of `functional::layer_norm` and `functional::rms_norm`
    (ops/functional/normalization.rs:123-217) are replaced by ONE CustomCall each, with gamma and beta themselves as
    operands, so the fold finds no broadcast of them to turn into a derived parameter.  The sequence's interior
    instructions go only where nothing else reads them (a program that also asks for the mean keeps it).

    The library does not need this pass: it plans a derived broadcast parameter as the broadcast it came from.  The pass
    is the second, explicit route, for a front end whose derived parameters lose that provenance (handles copied through
    the host, a resolver outside the library)."""

    name = "hip-norm-fusion"

    def run(self, fn: dict, cx: "OptimizeContext") -> bool:
        rw = Rewriter(fn)
        changed = False
        # roots last to first: a layer norm ends in an rms-norm-shaped tail over the centred row, and the larger sequence
        # has to claim its instructions first
        for vid in reversed(rw.order()):
            if not rw.contains(vid):
                continue
            ins = rw.inst[vid]
            if op_name(ins["op"]) != "ElementwiseBinary":
                continue
            m = self._layer_norm(rw, ins) if op_attrs(ins["op"]) == "Add" else (self._rms_norm(rw, ins) if op_attrs(ins["op"]) == "Mul" else None)
            if m is None:
                continue
            kind, operands, eps, interior = m
            call = {"CustomCall": {"target": NORM_TARGETS[kind], "attrs": {"eps": {"kind": "F64", "value": float(eps)},
                                                                             "axis": {"kind": "I64", "value": len(_static_dims(ins["output"])) - 1}}}}
            new = rw.insert_before(vid, call, [{"Value": v} for v in operands], copy.deepcopy(ins["output"]))
            rw.replace_value(vid, new)
            for dead in interior:   # last to first: an instruction goes once its readers have gone
                if rw.contains(dead) and not rw.users_of(dead) and dead not in fn["result_ids"]:
                    rw.erase(dead)
            changed = True
        return changed

    # -- matchers: every helper returns None when the shape of the graph is not the functional's
    @staticmethod
    def _def(rw, v, name, attr=None):
        ins = rw.inst.get(v)
        if ins is None or op_name(ins["op"]) != name:
            return None
        if attr is not None and op_attrs(ins["op"]) != attr:
            return None
        return ins

    @classmethod
    def _binary(cls, rw, v, kind):
        ins = cls._def(rw, v, "ElementwiseBinary", kind)
        if ins is None or len(ins["operands"]) != 2 or any("Value" not in o for o in ins["operands"]):
            return None
        return ins["operands"][0]["Value"], ins["operands"][1]["Value"]

    @classmethod
    def _bcast(cls, rw, v):
        ins = cls._def(rw, v, "BroadcastTo")
        return _single_value(ins) if ins is not None else None

    @classmethod
    def _scalar(cls, rw, v):
        """BroadcastTo(shape)(BroadcastTo([])(Literal)) (ops/ptir/mod.rs:16-22): the literal's value as float."""
        for _ in range(3):
            ins = cls._def(rw, v, "BroadcastTo")
            if ins is None or len(ins["operands"]) != 1:
                return None
            o = ins["operands"][0]
            if "Literal" in o:
                lit = o["Literal"]
                data = bytes(lit["bytes"])
                if lit["spec"]["dtype"] == "F32" and len(data) == 4:
                    return float(struct.unpack("<f", data)[0])
                if lit["spec"]["dtype"] == "Bf16" and len(data) == 2:
                    return float(struct.unpack("<f", b"\x00\x00" + data)[0])
                return None
            v = o["Value"]
        return None

    @classmethod
    def _reduce_sum_last(cls, rw, v):
        ins = cls._def(rw, v, "Reduce")
        if ins is None:
            return None
        a = op_attrs(ins["op"])
        src = _single_value(ins)
        if src is None or a["kind"] != "Sum" or not a["keepdims"] or list(a["axes"]) != [len(_static_dims(rw.types[src])) - 1]:
            return None
        return src

    @classmethod
    def _vector(cls, rw, v, n):
        src = cls._bcast(rw, v)
        if src is None or _static_dims(rw.types[src]) != (n,):
            return None
        return src

    def _rms_norm(self, rw, root):
        n = _static_dims(root["output"])[-1]
        ops = self._binary(rw, root["id"], "Mul")
        if ops is None:
            return None
        nrm, gb = ops
        gamma = self._vector(rw, gb, n)
        o2 = self._binary(rw, nrm, "Mul") if gamma is not None else None
        if o2 is None:
            return None
        x, irb = o2
        ir = self._bcast(rw, irb)
        t = self._def(rw, ir, "ElementwiseUnary", "Rsqrt") if ir is not None else None
        o3 = self._binary(rw, _single_value(t), "Add") if t is not None else None
        if o3 is None:
            return None
        ms, eb = o3
        eps = self._scalar(rw, eb)
        o4 = self._binary(rw, ms, "Mul")
        if eps is None or o4 is None:
            return None
        s, ic = o4
        inv_n = self._scalar(rw, ic)
        sq = self._reduce_sum_last(rw, s)
        o5 = self._binary(rw, sq, "Mul") if sq is not None else None
        if inv_n is None or o5 is None or o5 != (x, x) or rw.types[x] != root["output"]:
            return None
        if abs(inv_n * n - 1.0) > 1e-2:
            return None
        return "rms_norm", [x, gamma], eps, [nrm, gb, irb, ir, _single_value(t), eb, ms, ic, s, sq]

    def _layer_norm(self, rw, root):
        n = _static_dims(root["output"])[-1]
        ops = self._binary(rw, root["id"], "Add")
        if ops is None:
            return None
        t, bb = ops
        beta = self._vector(rw, bb, n)
        o1 = self._binary(rw, t, "Mul") if beta is not None else None
        if o1 is None:
            return None
        nrm, gb = o1
        gamma = self._vector(rw, gb, n)
        o2 = self._binary(rw, nrm, "Mul") if gamma is not None else None
        if o2 is None:
            return None
        cen, isb = o2
        istd = self._bcast(rw, isb)
        rs = self._def(rw, istd, "ElementwiseUnary", "Rsqrt") if istd is not None else None
        o3 = self._binary(rw, _single_value(rs), "Add") if rs is not None else None
        if o3 is None:
            return None
        vm, eb = o3
        eps = self._scalar(rw, eb)
        o4 = self._binary(rw, vm, "Mul")
        if eps is None or o4 is None:
            return None
        vs, ic = o4
        sq = self._reduce_sum_last(rw, vs)
        o5 = self._binary(rw, sq, "Mul") if sq is not None else None
        if self._scalar(rw, ic) is None or o5 is None or o5 != (cen, cen):
            return None
        o6 = self._binary(rw, cen, "Sub")
        if o6 is None:
            return None
        x, mb = o6
        mean = self._bcast(rw, mb)
        o7 = self._binary(rw, mean, "Mul") if mean is not None else None
        if o7 is None or self._scalar(rw, o7[1]) != self._scalar(rw, ic):
            return None
        s = o7[0]
        if self._reduce_sum_last(rw, s) != x or rw.types[x] != root["output"]:
            return None
        return "layer_norm", [x, gamma, beta], eps, [t, bb, gb, nrm, isb, istd, _single_value(rs), eb, vm, vs, sq, cen, mb, mean, o7[1], ic, s]


def hip_backend_pipeline() -> dict:
    """The passes of the hip backend's BackendPipeline by hook, as keyword arguments of `optimize`."""
    return {"pre": [HipNormFusionPass()]}
