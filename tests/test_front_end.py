"""The front end's optimizer passes (gpt.rs_amd/front_end.py) against the reference's own fixtures: every case of
tests/golden/lit/*.lit (the data files of crates/gpt-rs/tests/pass_lit_*.rs) is run through the passes its reference
test names, and the printed result must be the fixture's EXPECTED text, value ids and parameter order included."""
import glob
import os

import numpy as np
import pytest

from gptrs_amd import front_end as FE
from gptrs_amd import ptir_text as T
from gptrs_amd.ptir import TensorSpec
from oracle_backend import OracleBackend

LIT_DIR = os.path.join(os.path.dirname(__file__), "golden", "lit")

# the pass list of each fixture's reference test (crates/gpt-rs/tests/pass_lit_<name>.rs)
PASSES = {
    "dedup.lit": lambda: [FE.CommonSubexpressionElimination()],
    "elementwise.lit": lambda: [FE.elementwise_simplification()],
    "param_only_fold_to_param.lit": lambda: [FE.ParamOnlyFoldToParam(), FE.DeadCodeElimination()],
    "reshape.lit": lambda: [FE.reshape_canonicalization()],
    "slice.lit": lambda: [FE.slice_canonicalization()],
    "transpose.lit": lambda: [FE.transpose_canonicalization()],
}
CASES = [(os.path.basename(f), c) for f in sorted(glob.glob(os.path.join(LIT_DIR, "*.lit"))) for c in T.load_lit_cases(f)]


def _context(fn, meta, backend):
    """entry_signature_for_case (crates/gpt-rs/tests/lit_support.rs:139-210): roles and stable ids from the META block,
    an Arg and the value id where it is silent; every Param is materialised as zeros under its stable id."""
    roles, stable = [], []
    for line in meta.splitlines():
        line = line.strip()
        if line.startswith("roles:"):
            roles = [t for t in line[6:].replace(",", " ").split()]
        if line.startswith("stable_ids:"):
            stable = [int(t) for t in line[11:].replace(",", " ").split()]
    entry = []
    for idx, (pid, ty) in enumerate(zip(fn["parameter_ids"], fn["parameters"])):
        role = roles[idx] if idx < len(roles) else FE.ARG
        sid = stable[idx] if idx < len(stable) else pid
        if role == FE.PARAM:
            backend.param_resolver().set(FE.stable_id_bytes(sid), backend.materialize(TensorSpec.from_json(ty["Tensor"]), None))
        entry.append(FE.EntryParam(pid, ty, role, sid))
    return FE.OptimizeContext(backend, backend.param_resolver(), entry)


@pytest.mark.parametrize("name,case", CASES, ids=[f"{n}:{c.name}" for n, c in CASES])
def test_passes_reproduce_the_expected_text(name, case):
    prog = T.parse_program(case.input)
    fn = prog.obj["functions"][0]
    cx = _context(fn, case.meta, OracleBackend())
    changed = FE.run_passes(fn, PASSES[name](), cx)
    assert changed, "the reference test requires the pass to change the program"
    assert T.format_program(T.program_from_obj(prog.obj)).strip() == case.expected.strip()
    FE.Rewriter(fn)   # the def-use index builds: SSA holds


def test_fold_stores_the_subgraph_result_under_a_derived_id():
    """param_only_fold_to_param.lit, beyond the text: the derived Param holds Reshape[6](Transpose[1,0](%1)) of the
    leaf, its id has the top bit set (param_only_fold_to_param.rs:474-476), and a second fold of the same program finds
    it in the resolver instead of running the subgraph again."""
    case = T.load_lit_cases(os.path.join(LIT_DIR, "param_only_fold_to_param.lit"))[0]
    be = OracleBackend()
    leaf = np.arange(6, dtype=np.float32).reshape(2, 3)
    runs = []
    for _ in range(2):
        prog = T.parse_program(case.input)
        fn = prog.obj["functions"][0]
        cx = _context(fn, case.meta, be)
        be.param_resolver().set(FE.stable_id_bytes(1234), be.materialize(TensorSpec("F32", (2, 3)), leaf))
        FE.run_passes(fn, [FE.ParamOnlyFoldToParam(), FE.DeadCodeElimination()], cx)
        runs.append((cx.folds_run, cx.folds_reused))
        derived = [p for p in cx.entry if p.role == FE.PARAM]
        assert len(derived) == 1 and derived[0].id == 5 and derived[0].stable_id >> 127 == 1
        got = be.to_numpy(be.param_resolver().get(FE.stable_id_bytes(derived[0].stable_id)))
        assert np.array_equal(got, np.ascontiguousarray(leaf.T).reshape(6))
    assert runs == [(1, 0), (0, 1)]


def _layer_norm_program(rows, n):
    from gptrs_amd import functional as F
    from gptrs_amd.ptir import FunctionBuilder, Program
    fb = FunctionBuilder("main", "F32")
    x = fb.param("F32", [rows, n])
    g = fb.param("F32", [n])
    b = fb.param("F32", [n])
    out, *_ = F.layer_norm(x, g, b, 1e-5)
    out2, *_ = F.layer_norm(out, g, b, 1e-5)
    fb.set_results([out2])
    return Program(fb)


def test_pipeline_on_two_layer_norms():
    """The whole pipeline on what the models emit: gamma and beta broadcasts become ONE derived Param each (both norms
    share them after CSE of the derived inputs), the vectors themselves drop out of the signature, the scalar-literal
    broadcasts of the two norms merge, and the optimised program computes what the emitted one does."""
    be = OracleBackend()
    prog = _layer_norm_program(3, 8)
    rng = np.random.default_rng(0)
    x, g, b = (rng.standard_normal(s).astype(np.float32) for s in ((3, 8), (8,), (8,)))
    res = be.param_resolver()
    res.set(FE.stable_id_bytes(11), be.materialize(TensorSpec("F32", (8,)), g))
    res.set(FE.stable_id_bytes(12), be.materialize(TensorSpec("F32", (8,)), b))
    opt = FE.optimize(prog, [FE.ARG, FE.PARAM, FE.PARAM], [None, 11, 12], be, res)
    assert opt.folds_run == 2
    assert [p.role for p in opt.inputs] == [FE.ARG, FE.PARAM, FE.PARAM]
    assert opt.source_index == [0, None, None]
    assert [tuple(s.dims) for s in opt.program.param_specs] == [(3, 8), (3, 8), (3, 8)]
    body = opt.program.obj["functions"][0]["body"]
    bcasts_of_values = [i for i in body if FE.op_name(i["op"]) == "BroadcastTo" and "Value" in i["operands"][0]
                        and i["operands"][0]["Value"] in opt.program.obj["functions"][0]["parameter_ids"]]
    assert not bcasts_of_values
    # 2 x 19 emitted, 4 parameter broadcasts folded away, the second norm's 4 literal broadcasts (1/N, eps) merged with the first's
    assert prog.instruction_count() == 38 and len(body) == 30
    xin = be.materialize(TensorSpec("F32", (3, 8)), x)
    feeds = [xin] + [res.get(FE.stable_id_bytes(p.stable_id)) for p in opt.inputs[1:]]
    got = be.to_numpy(be.run_program(opt.program, feeds)[0])
    want = be.to_numpy(be.run_program(prog, [xin, res.get(FE.stable_id_bytes(11)), res.get(FE.stable_id_bytes(12))])[0])
    assert np.array_equal(got, want)


def test_broadcast_chain_over_a_literal_is_left_alone():
    """CollapseBroadcastChain needs a value under the inner broadcast (broadcast_canonicalization.rs:63-66): the
    scalar(...).broadcast_to(...) pairs of the emitters stay two instructions."""
    from gptrs_amd.ptir import FunctionBuilder, Program
    fb = FunctionBuilder("main", "F32")
    x = fb.param("F32", [2, 4])
    fb.set_results([x * fb.scalar_broadcast(3.0, [2, 4])])
    prog = Program(fb)
    be = OracleBackend()
    opt = FE.optimize(prog, [FE.ARG], [None], be, be.param_resolver())
    assert [FE.op_name(i["op"]) for i in opt.program.obj["functions"][0]["body"]] == ["BroadcastTo", "BroadcastTo", "ElementwiseBinary"]


# ------------------------------------------------------------------ the backend's fusion pass on the optimised stream
class _Recording:
    """RecordingBackend (crates/gpt-rs-backend-tests/src/recording_backend.rs:9-76): hands out handles, executes nothing."""

    def __init__(self):
        self.params = {}

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
        return [("o", s) for s in program.result_specs]


def _model(kind):
    from gptrs_amd import models
    be = _Recording()
    if kind == "gpt":
        m = models.Gpt(models.GptConfig(num_layers=2), be, "F32")
    elif kind == "ministral-f32-stream":
        m = models.Ministral(models.MinistralConfig(num_layers=2), be, "Bf16", "F32")
    else:
        m = models.Ministral(models.MinistralConfig(num_layers=2), be, "Bf16")
    for name, dims in m.expected_params().items():
        m.param_names.append(name)
        m.param_specs[name] = TensorSpec(m.param_dtype(name), dims)
        be.set(models.param_id(m.namespace, name), ("h", m.param_specs[name]))
    return m


@pytest.mark.parametrize("kind", ["gpt", "ministral", "ministral-f32-stream"])
@pytest.mark.parametrize("seq,decode,batch", [(1, True, 1), (64, False, 1), (1, True, 4), (1024, False, 1)])
def test_backend_fusion_is_the_same_on_the_optimised_stream(kind, seq, decode, batch):
    """What `gptrs_hip_run_program` makes of a model program must not depend on whether the program comes straight from
    the emitters or through the reference's optimizer: same fused instructions, same kernel families, at full model
    width (the kernel families depend on the shapes).  The derived parameters arrive as handles that remember the vector
    they were broadcast from, which `bcast_len` stands for here; a one-row decode program fuses the same without them."""
    from gptrs_amd import backend as B
    from gptrs_amd import models
    m = _model(kind)
    prog, layout = m._build(seq, 2048 if seq > 64 else 64, decode, batch, True)
    n_args, be = layout["n_args"], m.backend
    roles = [FE.ARG] * n_args + [FE.PARAM] * len(m.param_names)
    stable = [None] * n_args + [int.from_bytes(models.param_id(m.namespace, n), "little") for n in m.param_names]
    opt = FE.optimize(prog, roles, stable, be, be)
    assert opt.folds_run > 0 and opt.program.instruction_count() < prog.instruction_count()
    emitted = B.fusion_report(prog)
    lens = [0 if src is not None else spec.dims[-1] for src, spec in zip(opt.source_index, opt.program.param_specs)]
    assert B.fusion_report(opt.program, lens) == emitted
    assert not [line for line in emitted if line.split()[0] in ("ElementwiseBinary", "Reduce", "BroadcastTo", "Transpose", "Concat") and kind != "gpt"]
    if seq == 1 and batch == 1:
        assert B.fusion_report(opt.program, None) == emitted


@pytest.mark.parametrize("kind", ["gpt", "ministral", "ministral-f32-stream"])
@pytest.mark.parametrize("seq,decode,batch", [(1, True, 1), (64, False, 1), (1, True, 4)])
def test_backend_pipeline_route(kind, seq, decode, batch):
    """The second route through the optimizer: the hip backend's pre-pass turns every norm into a CustomCall ahead of the
    parameter-only fold, so no gain or shift is folded into a derived parameter (only bias broadcasts are), and the
    library's fusion of the result is what it makes of the emitted program -- without any provenance on the inputs but
    for the biases."""
    from gptrs_amd import backend as B
    from gptrs_amd import models
    m = _model(kind)
    prog, layout = m._build(seq, 64, decode, batch, True)
    n_args, be = layout["n_args"], m.backend
    roles = [FE.ARG] * n_args + [FE.PARAM] * len(m.param_names)
    stable = [None] * n_args + [int.from_bytes(models.param_id(m.namespace, n), "little") for n in m.param_names]
    opt = FE.optimize(prog, roles, stable, be, be, **FE.hip_backend_pipeline())
    body = opt.program.obj["functions"][0]["body"]
    calls = [FE.op_attrs(i["op"])["target"] for i in body if FE.op_name(i["op"]) == "CustomCall"]
    norms = 2 * 2 + 1
    assert len([t for t in calls if t in FE.NORM_TARGETS.values()]) == norms
    assert opt.folds_run == (0 if kind != "gpt" else 4 * 2)   # GPT-2: the four bias broadcasts of each block; Ministral has none
    lens = [0 if src is not None else spec.dims[-1] for src, spec in zip(opt.source_index, opt.program.param_specs)]
    assert B.fusion_report(opt.program, lens) == B.fusion_report(prog)
    if kind != "gpt":
        assert B.fusion_report(opt.program, None) == B.fusion_report(prog)


def test_norm_calls_compute_what_the_sequences_compute():
    """On the oracle the CustomCall is DEFINED as the functional's sequence: the program with the calls returns, bit for
    bit, what the emitted program returns (f32 and bf16); a program that also returns the mean keeps the instructions
    that produce it."""
    from gptrs_amd import functional as F
    from gptrs_amd.ptir import FunctionBuilder, Program
    for dtype in ("F32", "Bf16"):
        fb = FunctionBuilder("main", dtype)
        x, g, b, g2 = fb.param(dtype, [5, 24]), fb.param(dtype, [24]), fb.param(dtype, [24]), fb.param(dtype, [24])
        out, _, mean, _ = F.layer_norm(x, g, b, 1e-5)
        out2, *_ = F.rms_norm(out, g2, 1e-6)
        fb.set_results([out2, mean])
        prog = Program(fb)
        be = OracleBackend()
        fn = __import__("copy").deepcopy(prog.obj["functions"][0])
        cx = FE.OptimizeContext(be, be.param_resolver(), [FE.EntryParam(i, t, FE.ARG, None) for i, t in zip(fn["parameter_ids"], fn["parameters"])])
        assert FE.HipNormFusionPass().run(fn, cx)
        names = [FE.op_name(i["op"]) for i in fn["body"]]
        assert names.count("CustomCall") == 2 and "Reduce" in names, "the mean is a result: its reduction stays"
        opt = FE.program_from_function(fn, "main")
        rng = np.random.default_rng(3)
        arrays = [rng.standard_normal(s.dims).astype(np.float32) for s in prog.param_specs]
        from parity import oracle_run
        for got, want in zip(oracle_run(opt, arrays), oracle_run(prog, arrays)):
            assert np.array_equal(got, want)
