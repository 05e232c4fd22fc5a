"""Text form of PTIR programs: the reference's `Display` for `Program` (crates/gpt-rs/src/backend/spec.rs:858-1069),

    program @entry (spec_version = ptir.v0.4) {
      func @entry {
        params:
          %0 : tensor<F32 x 2x3>
        body:
          %1 = Transpose(TransposeSpec { perm: [1, 0] })(%0) -> tensor<F32 x 3x2>
        results:
          %1 : tensor<F32 x 3x2>
      }
    }

where an instruction is `%id = <Debug of Operation>(<operands>) -> <type>` (spec.rs:992-1027) and a type is
`tensor<DTYPE x d0xd1...>` with `[]` for rank 0 (spec.rs:1029-1058).  `parse_program` reads that form back into a
`Program` (same JSON as the builders emit), `format_program` prints it; the operations covered are the ones the
reference's own reader of this form knows (crates/gpt-rs/tests/lit_support.rs:354-440): Constant, BroadcastTo,
ElementwiseBinary, ElementwiseUnary, Reshape, Transpose, Slice, Reduce.  `load_lit_cases` splits a `.lit` fixture
(lit_support.rs:32-96) into its META / EXPECTED / INPUT cases.
"""
from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, List, Tuple

from .ptir import SPEC_VERSION, Program, TensorSpec

_TYPE = re.compile(r"tensor<(\w+) x ([^>]*)>")


class PtirTextError(ValueError):
    pass


def _parse_type(s: str) -> TensorSpec:
    m = _TYPE.fullmatch(s.strip())
    if not m:
        raise PtirTextError(f"unsupported value type `{s}`")
    dims = m.group(2).strip()
    if dims == "[]":
        return TensorSpec(m.group(1), ())
    try:
        return TensorSpec(m.group(1), tuple(int(d) for d in dims.split("x")))
    except ValueError:
        raise PtirTextError(f"dynamic or malformed shape `{dims}`") from None


def _format_type(spec_json) -> str:
    dims = [str(d["Static"]) for d in spec_json["shape"]["dims"]]
    return "tensor<%s x %s>" % (spec_json["dtype"], "x".join(dims) if dims else "[]")


def _int_list(text: str, key: str) -> List[int]:
    m = re.search(re.escape(key) + r"[^\[]*\[([^\]]*)\]", text)
    if not m:
        raise PtirTextError(f"`{key}` list missing in `{text}`")
    return [int(v) for v in m.group(1).split(",") if v.strip()]


def _shape_json(dims):
    return {"dims": [{"Static": int(d)} for d in dims]}


def _parse_op(name: str, body: str):
    if name == "Reshape":
        return {"Reshape": {"new_shape": [{"Explicit": {"Static": int(v)}} for v in re.findall(r"Static\((\d+)\)", body)]}}
    if name == "Transpose":
        return {"Transpose": {"perm": _int_list(body, "perm")}}
    if name == "Slice":
        return {"Slice": {"starts": _int_list(body, "starts"), "sizes": _int_list(body, "sizes")}}
    if name == "BroadcastTo":
        return {"BroadcastTo": {"result_shape": _shape_json(re.findall(r"Static\((\d+)\)", body))}}
    if name in ("ElementwiseBinary", "ElementwiseUnary"):
        return {name: body.strip()}
    if name == "Constant":
        m = re.search(r"dtype: (\w+), shape: Shape \{ dims: \[([^\]]*)\] \} \}, bytes: \[([^\]]*)\]", body)
        if not m:
            raise PtirTextError(f"malformed Constant `{body}`")
        dims = re.findall(r"Static\((\d+)\)", m.group(2))
        data = [int(v) for v in m.group(3).split(",") if v.strip()]
        return {"Constant": {"spec": {"dtype": m.group(1), "shape": _shape_json(dims)}, "bytes": data}}
    if name == "Reduce":
        kind = re.search(r"kind: (\w+)", body)
        return {"Reduce": {"kind": kind.group(1), "axes": _int_list(body, "axes"), "keepdims": "keepdims: true" in body,
                           "accum_dtype": None, "out_dtype": None}}
    raise PtirTextError(f"unsupported op {name}")


def _format_op(op) -> str:
    (name, a), = op.items() if isinstance(op, dict) else ((op, None),)
    dim = lambda d: "Static(%d)" % d["Static"]  # noqa: E731
    ints = lambda v: "[" + ", ".join(str(int(x)) for x in v) + "]"  # noqa: E731
    if name == "Reshape":
        return "Reshape(ReshapeSpec { new_shape: [%s] })" % ", ".join("Explicit(%s)" % dim(d["Explicit"]) for d in a["new_shape"])
    if name == "Transpose":
        return "Transpose(TransposeSpec { perm: %s })" % ints(a["perm"])
    if name == "Slice":
        return "Slice(SliceSpec { starts: %s, sizes: %s })" % (ints(a["starts"]), ints(a["sizes"]))
    if name == "BroadcastTo":
        return "BroadcastTo(BroadcastToSpec { result_shape: Shape { dims: [%s] } })" % ", ".join(dim(d) for d in a["result_shape"]["dims"])
    if name in ("ElementwiseBinary", "ElementwiseUnary"):
        return "%s(%s)" % (name, a)
    if name == "Constant":
        return "Constant(TensorLiteral { spec: TensorSpec { dtype: %s, shape: Shape { dims: [%s] } }, bytes: %s })" % (
            a["spec"]["dtype"], ", ".join(dim(d) for d in a["spec"]["shape"]["dims"]), ints(a["bytes"]))
    if name == "Reduce":
        opt = lambda v: "None" if v is None else "Some(%s)" % v  # noqa: E731
        return "Reduce(ReduceSpec { kind: %s, axes: %s, keepdims: %s, accum_dtype: %s, out_dtype: %s })" % (
            a["kind"], ints(a["axes"]), "true" if a["keepdims"] else "false", opt(a.get("accum_dtype")), opt(a.get("out_dtype")))
    raise PtirTextError(f"unsupported op {name}")


def _split_call(rest: str) -> Tuple[str, str, str]:
    """`Name(<args>)(<operands>) -> type` / `Name(<args>) -> type` (no operands): name, args, operand text."""
    head, _, _ = rest.rpartition(" -> ")
    name = head[:head.index("(")]
    depth, i = 0, len(name)
    for i in range(len(name), len(head)):
        depth += head[i] == "("
        depth -= head[i] == ")"
        if depth == 0:
            break
    args, tail = head[len(name) + 1:i], head[i + 1:].strip()
    if tail and not (tail.startswith("(") and tail.endswith(")")):
        raise PtirTextError(f"malformed instruction `{rest}`")
    return name, args, tail[1:-1] if tail else ""


def program_from_obj(obj) -> Program:
    """A `Program` around an already assembled JSON object (one function, tensor parameters and results)."""
    p = Program.__new__(Program)
    fn = obj["functions"][0]
    p.obj = obj
    p.param_specs = [TensorSpec.from_json(t["Tensor"]) for t in fn["parameters"]]
    p.result_specs = [TensorSpec.from_json(t["Tensor"]) for t in fn["results"]]
    p._json = None
    p._key = None
    return p


def parse_program(text: str) -> Program:
    lines = [ln.strip() for ln in text.splitlines() if ln.strip()]
    m = re.fullmatch(r"program @(\S+) \(spec_version = (\S+)\) \{", lines[0]) if lines else None
    if not m:
        raise PtirTextError("missing `program @name (spec_version = ...) {` header")
    if m.group(2) != SPEC_VERSION:
        raise PtirTextError(f"unsupported spec version {m.group(2)}")
    entry = m.group(1)
    fm = re.fullmatch(r"func @(\S+) \{", lines[1]) if len(lines) > 1 else None
    if not fm:
        raise PtirTextError("missing `func @name {`")
    fn: Dict = {"name": fm.group(1), "parameters": [], "parameter_ids": [], "results": [], "body": [], "hints": [], "result_ids": []}
    section = None
    for ln in lines[2:]:
        if ln in ("params:", "body:", "results:"):
            section = ln[:-1]
            continue
        if ln == "}":
            continue
        if ln.startswith(("hints:", "region ")):
            raise PtirTextError("hints and regions are not supported")
        if section in ("params", "results"):
            b = re.fullmatch(r"%(\d+) : (.+)", ln)
            if not b:
                raise PtirTextError(f"malformed binding `{ln}`")
            spec = _parse_type(b.group(2))
            key = "parameter" if section == "params" else "result"
            fn[key + "s"].append({"Tensor": spec.to_json()})
            fn[key + "_ids"].append(int(b.group(1)))
        elif section == "body":
            b = re.fullmatch(r"%(\d+) = (.+)", ln)
            if not b or " -> " not in b.group(2):
                raise PtirTextError(f"malformed instruction `{ln}`")
            name, args, operands = _split_call(b.group(2))
            ops = []
            for o in (v.strip() for v in operands.split(",") if v.strip()):
                if not re.fullmatch(r"%\d+", o):
                    raise PtirTextError(f"unsupported operand `{o}`")   # literal operands print without their bytes
                ops.append({"Value": int(o[1:])})
            out = _parse_type(b.group(2).rpartition(" -> ")[2])
            fn["body"].append({"id": int(b.group(1)), "op": _parse_op(name, args), "operands": ops, "output": {"Tensor": out.to_json()}})
        else:
            raise PtirTextError(f"line outside a section: `{ln}`")
    return program_from_obj({"spec_version": SPEC_VERSION, "entry": entry, "functions": [fn], "regions": []})


def format_program(program: Program) -> str:
    obj = program.obj
    out = ["program @%s (spec_version = %s) {" % (obj["entry"], obj["spec_version"])]
    for fn in obj["functions"]:
        out.append("  func @%s {" % fn["name"])
        if fn["parameter_ids"]:
            out.append("    params:")
            out += ["      %%%d : %s" % (i, _format_type(t["Tensor"])) for i, t in zip(fn["parameter_ids"], fn["parameters"])]
        if fn["body"]:
            out.append("    body:")
            for ins in fn["body"]:
                ops = []
                for o in ins["operands"]:
                    if "Value" in o:
                        ops.append("%%%d" % o["Value"])
                    elif "Literal" in o:
                        s = o["Literal"]["spec"]
                        ops.append("literal(dtype=%s, shape=%s)" % (s["dtype"], _format_type(s).split(" x ")[1][:-1]))
                    else:
                        raise PtirTextError("tuple operands are not supported")
                call = _format_op(ins["op"]) + ("(%s)" % ", ".join(ops) if ops else "")
                out.append("      %%%d = %s -> %s" % (ins["id"], call, _format_type(ins["output"]["Tensor"])))
        if fn["result_ids"]:
            out.append("    results:")
            out += ["      %%%d : %s" % (i, _format_type(t["Tensor"])) for i, t in zip(fn["result_ids"], fn["results"])]
        out.append("  }")
    out.append("}")
    return "\n".join(out) + "\n"


@dataclass
class LitCase:
    name: str
    meta: str
    input: str
    expected: str


def load_lit_cases(path: str) -> List[LitCase]:
    """`META:` / `EXPECTED:` / `INPUT:` blocks closed by `run_test` (lit_support.rs:32-96)."""
    cases: List[LitCase] = []
    buf = {"meta": [], "expected": [], "input": []}
    cur = None
    with open(path) as f:
        for raw in f:
            ln = raw.rstrip()
            if ln in ("META:", "EXPECTED:", "INPUT:"):
                cur = ln[:-1].lower()
                buf[cur] = []
            elif ln == "run_test":
                cases.append(LitCase("case_%d" % (len(cases) + 1), "\n".join(buf["meta"]), "\n".join(buf["input"]) + "\n",
                                     "\n".join(buf["expected"]) + "\n"))
                cur = None
            elif cur is not None:
                buf[cur].append(ln)
    return cases
