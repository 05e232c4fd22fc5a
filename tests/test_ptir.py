"""CPU tests of the host-side PTIR emitter: the instruction sequences match what the reference's
functionals emit (the reference asserts the same with a RecordingBackend,
crates/gpt-rs/tests/functional_softmax.rs:15-130) and the JSON follows serde's encoding of
crates/gpt-rs/src/backend/spec.rs."""
import json

import numpy as np
import pytest

from gptrs_amd import functional as F
from gptrs_amd import models
from gptrs_amd.ptir import FunctionBuilder, Program, Tensor, TensorSpec, scalar_literal


def ops_of(fb):
    out = []
    for ins in fb.body:
        op = ins["op"]
        if isinstance(op, str):
            out.append(op)
        else:
            (name, attr), = op.items()
            if name in ("ElementwiseBinary", "ElementwiseUnary"):
                out.append(attr)
            elif name == "Reduce":
                out.append("Reduce" + attr["kind"])
            else:
                out.append(name)
    return out


def test_softmax_sequence():
    fb = FunctionBuilder()
    x = fb.param("F32", [2, 5])
    F.softmax_last_axis(x)
    assert ops_of(fb) == ["ReduceMax", "BroadcastTo", "Sub", "Exp", "ReduceSum", "BroadcastTo", "Div"]
    red = fb.body[0]["op"]["Reduce"]
    assert red == {"kind": "Max", "axes": [1], "keepdims": True, "accum_dtype": None, "out_dtype": None}


def test_layer_norm_sequence():  # ops/functional/normalization.rs:123-174
    fb = FunctionBuilder()
    x, g, b = fb.param("F32", [3, 8]), fb.param("F32", [8]), fb.param("F32", [8])
    F.layer_norm(x, g, b, 1e-5)
    assert ops_of(fb) == ["ReduceSum", "BroadcastTo", "BroadcastTo", "Mul", "BroadcastTo", "Sub", "Mul", "ReduceSum", "Mul",
                          "BroadcastTo", "BroadcastTo", "Add", "Rsqrt", "BroadcastTo", "Mul", "BroadcastTo", "BroadcastTo",
                          "Mul", "Add"]
    # 1/N is a pre-rounded f32 literal multiplier, not a divide
    lit = fb.body[1]["operands"][0]["Literal"]
    assert lit["spec"] == {"dtype": "F32", "shape": {"dims": []}}
    assert np.frombuffer(bytes(lit["bytes"]), "<f4")[0] == np.float32(1.0) / np.float32(8)


def test_rms_norm_gelu_swiglu_sequences():
    fb = FunctionBuilder()
    x, g = fb.param("F32", [3, 8]), fb.param("F32", [8])
    F.rms_norm(x, g, 1e-5)
    assert ops_of(fb) == ["Mul", "ReduceSum", "BroadcastTo", "BroadcastTo", "Mul", "BroadcastTo", "BroadcastTo", "Add", "Rsqrt",
                          "BroadcastTo", "Mul", "BroadcastTo", "Mul"]
    fb = FunctionBuilder()
    F.gelu(fb.param("F32", [4]))
    assert ops_of(fb) == ["BroadcastTo", "Mul", "BroadcastTo", "Div", "Erf", "BroadcastTo", "Add", "Mul"]
    div_lit = np.frombuffer(bytes(fb.body[2]["operands"][0]["Literal"]["bytes"]), "<f4")[0]
    assert div_lit == np.sqrt(np.float32(2.0))
    # tensor is always lhs, the literal broadcast rhs (graph.rs:1339-1345, 1879-1885)
    assert fb.body[1]["operands"] == [{"Value": 0}, {"Value": 1}]
    fb = FunctionBuilder()
    F.swiglu(fb.param("F32", [4]), fb.param("F32", [4]))
    assert ops_of(fb) == ["BroadcastTo", "Mul", "Exp", "BroadcastTo", "Add", "Div", "Mul"]


def test_decode_attention_contains_dynamic_ops_and_exports_caches():
    # crates/gpt-rs/tests/functional_softmax.rs:313-370 asserts the same presence
    cfg = F.AttentionConfig(32, 4, 2, 8)
    fb = FunctionBuilder()
    qkv = fb.param("F32", [1, cfg.total_projection_dim])
    ck, cv = fb.param("F32", [2, 16, 8]), fb.param("F32", [2, 16, 8])
    us, qs = fb.param("Si32", [3]), fb.param("Si32", [1])
    ctx, k2, v2 = F.attention_decode_cache(cfg, qkv, ck, cv, us, qs)
    ops = ops_of(fb)
    assert ops.count("DynamicUpdateSlice") == 2 and ops.count("DynamicSlice") == 1 and ops.count("DotGeneral") == 2
    assert "Iota" in ops and "Compare" in ops and "Select" in ops
    assert ctx.dims == (1, 32) and k2.dims == (2, 16, 8) and v2.dims == (2, 16, 8)
    dots = [i["op"]["DotGeneral"] for i in fb.body if isinstance(i["op"], dict) and "DotGeneral" in i["op"]]
    assert dots[0]["batch_lhs"] == [0] and dots[0]["contract_lhs"] == [2] and dots[0]["contract_rhs"] == [2]
    assert dots[1]["contract_lhs"] == [2] and dots[1]["contract_rhs"] == [1]
    with pytest.raises(ValueError):
        F.attention_decode_cache(cfg, fb.param("F32", [2, cfg.total_projection_dim]), ck, cv, us, qs)


def test_matmul_rejects_mismatches():  # torch_parity/matmul.rs:117-133
    fb = FunctionBuilder()
    with pytest.raises(ValueError, match="dimension mismatch"):
        fb.param("F32", [2, 3]).matmul(fb.param("F32", [4, 5]))
    with pytest.raises(ValueError, match="batch dimension mismatch"):
        fb.param("F32", [2, 3, 4]).matmul(fb.param("F32", [3, 4, 5]))
    with pytest.raises(ValueError):
        F.embedding_lookup(fb.param("F32", [8, 4]), fb.param("Si32", [2, 2]))


def test_json_wire_form():
    fb = FunctionBuilder("main")
    x = fb.param("F32", [2, 3])
    y = (x + 1.0).transpose([1, 0])
    fb.set_results([y])
    obj = json.loads(Program(fb).json_bytes)
    assert obj["spec_version"] == "ptir.v0.4" and obj["entry"] == "main" and obj["regions"] == []
    fn = obj["functions"][0]
    assert fn["parameter_ids"] == [0] and fn["result_ids"] == [3] and fn["hints"] == []
    assert fn["parameters"] == [{"Tensor": {"dtype": "F32", "shape": {"dims": [{"Static": 2}, {"Static": 3}]}}}]
    bcast, add, tr = fn["body"]
    assert bcast["op"] == {"BroadcastTo": {"result_shape": {"dims": [{"Static": 2}, {"Static": 3}]}}}
    assert bcast["operands"] == [{"Literal": {"spec": {"dtype": "F32", "shape": {"dims": []}}, "bytes": [0, 0, 128, 63]}}]
    assert add["op"] == {"ElementwiseBinary": "Add"} and add["operands"] == [{"Value": 0}, {"Value": 1}]
    assert tr["op"] == {"Transpose": {"perm": [1, 0]}} and tr["output"]["Tensor"]["shape"]["dims"] == [{"Static": 3}, {"Static": 2}]
    fb2 = FunctionBuilder()
    a = fb2.param("Si32", [4])
    t = fb2.param("F32", [8, 2]).take(a)
    assert fb2.body[-1]["op"] == "Take" and t.dims == (4, 2)


def test_bf16_scalar_literals_are_pre_rounded():
    lit = scalar_literal("Bf16", -1e9)
    assert len(lit.data) == 2
    bits = int.from_bytes(lit.data, "little")
    val = np.array([bits << 16], np.uint32).view(np.float32)[0]
    import torch
    assert val == torch.tensor(-1e9).to(torch.bfloat16).float().item() == -998244352.0  # nearest bf16 to -1e9


def test_program_key_is_stable_and_distinguishes_shapes():
    def build(n):
        fb = FunctionBuilder()
        fb.set_results([fb.param("F32", [n]) + 1.0])
        return Program(fb)
    assert build(4).key == build(4).key and build(4).key != build(5).key and build(4).key != 0


def test_model_program_shapes_and_result_order():
    class Recorder:
        """RecordingBackend (crates/gpt-rs-backend-tests/src/recording_backend.rs:9-76): records, executes nothing."""
        def __init__(self):
            self.params, self.program, self.inputs, self.donate = {}, None, None, None
        def backend_name(self):
            return "recording"
        def param_resolver(self):
            return self
        def get(self, sid):
            return self.params.get(bytes(sid))
        def set(self, sid, h):
            self.params[bytes(sid)] = h
        def materialize(self, spec, data):
            return ("h", spec)
        def run_program(self, program, inputs, donate=None):
            self.program, self.inputs, self.donate = program, inputs, donate
            return [("o", s) for s in program.result_specs]

    cfg = models.GptConfig(vocab_size=64, context_length=32, embed_dim=32, num_layers=2, num_heads=4, mlp_ratio=2)
    be = Recorder()
    m = models.Gpt.random(cfg, be, seed=0)
    caches = [None] * 2
    m.forward_with_decode_cache([1, 2, 3], 0, caches, None)
    # prefill: 2*L caches then logits for ALL rows (model/gpt.rs:735-736)
    assert [s.dims for s in be.program.result_specs] == [(4, 4, 8)] * 4 + [(3, 64)]
    assert caches[0].capacity == 4 and caches[0].len == 3
    m.forward_with_decode_cache([4], 3, caches, None)
    assert be.program.result_specs[-1].dims == (1, 64) and caches[1].len == 4
    # the old caches are donated, per-step scalars and weights are not
    n_args = 4
    assert be.donate[:n_args] == [False] * n_args and be.donate[n_args:n_args + 4] == [True] * 4 and not any(be.donate[n_args + 4:])
    # bucket grows to the next power of two (model/gpt.rs:940-943)
    m.forward_with_decode_cache([5], 4, caches, None)
    assert caches[0].capacity == 8
    with pytest.raises(ValueError):
        m.forward_with_decode_cache([5], 3, caches, None)  # cache length must match the offset
    with pytest.raises(ValueError):
        m.forward_with_decode_cache([999], 5, caches, None)


def test_decode_cache_capacity_policy():
    assert [models.decode_cache_capacity(n, 1024) for n in (1, 2, 3, 16, 17, 600, 1000, 5000)] == [1, 2, 4, 16, 32, 1024, 1024, 1024]
