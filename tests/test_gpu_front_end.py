"""GPU: model programs that reach the backend through the reference's optimizer (gpt.rs_amd/front_end.py: canonicalisers,
parameter-only folds executed through `run_program` and stored in the backend's memo, CSE, DCE) run on the same fused
kernels, with the same launches and the same tokens, as the emitters' own instruction stream."""
import numpy as np
import pytest

from gptrs_amd import front_end as FE
from gptrs_amd import functional as F
from gptrs_amd import models
from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec
from oracle_backend import OracleBackend
from parity import assert_close

pytestmark = pytest.mark.gpu

MID_GPT = models.GptConfig(vocab_size=512, context_length=256, embed_dim=256, num_layers=2, num_heads=4, mlp_ratio=4)
MID_MINISTRAL = models.MinistralConfig(vocab_size=512, context_length=128, embed_dim=256, num_layers=2, num_heads=8,
                                       num_kv_heads=2, head_dim=32, ffn_dim=512, rotary_dim=32, rope_theta=1e6)
PROMPT = [3, 17, 42, 5, 99, 311, 8, 250, 1]


def _generate(be, make, front_end, n_new=8, counters=False, pipeline=False):
    """Tokens and per-step logits; with `counters` also (launches of the prefill, launches of a decode step, phases of
    the persistent launches of the decode steps, fused ops), with graph replay off so that every step counts."""
    m = make(be)
    m.front_end = front_end
    m.backend_pipeline = pipeline
    if counters:
        be.set_option("graphs", 0)
    try:
        f0 = be.counter("fused_ops") if counters else 0
        gen = models.Generator(m, PROMPT, kv_cache_capacity=64)
        prefill = be.counter("last_program_launches") if counters else 0
        p0 = be.counter("chain_phases") if counters else 0
        logits, toks = [be.to_numpy(gen.logits)[-1].copy()], []
        for _ in range(n_new):
            toks.append(gen.step())
            logits.append(be.to_numpy(gen.logits)[-1].copy())
        stats = (prefill, be.counter("last_program_launches"), be.counter("chain_phases") - p0, be.counter("fused_ops") - f0) if counters else None
    finally:
        if counters:
            be.set_option("graphs", 1)
    return toks, logits, stats


MAKERS = {
    "gpt-f32": lambda be: models.Gpt.random(MID_GPT, be, seed=3, dtype="F32", std=0.08),
    "ministral-f32": lambda be: models.Ministral.random(MID_MINISTRAL, be, seed=4, dtype="F32", std=0.08),
    "ministral-bf16": lambda be: models.Ministral.random(MID_MINISTRAL, be, seed=4, dtype="Bf16", std=0.08),
    "ministral-bf16-f32-stream": lambda be: models.Ministral.random(MID_MINISTRAL, be, seed=4, dtype="Bf16", std=0.08, residual_dtype="F32"),
}


@pytest.mark.parametrize("kind", list(MAKERS))
def test_decode_through_the_optimizer_is_the_same_computation(hip, kind):
    make = MAKERS[kind]
    t_raw, l_raw, s_raw = _generate(hip, make, False, counters=True)
    t_opt, l_opt, s_opt = _generate(hip, make, True, counters=True)
    # the same kernels in the same order: launches of the prefill and of a decode step, phases of the persistent launches
    assert s_opt[:3] == s_raw[:3], (s_raw, s_opt)
    assert s_opt[3] > 0
    assert t_opt == t_raw
    for a, b in zip(l_opt, l_raw):
        assert np.array_equal(a, b), "the optimised stream runs the same kernels on the same data"
    # the second route: the backend's own pre-pass hands the norms over as CustomCalls
    t_pipe, l_pipe, s_pipe = _generate(hip, make, True, counters=True, pipeline=True)
    assert s_pipe[:3] == s_raw[:3] and t_pipe == t_raw, (s_raw, s_pipe)
    for a, b in zip(l_pipe, l_raw):
        assert np.array_equal(a, b)
    if kind.endswith("f32") and "stream" not in kind:
        t_ref, l_ref, _ = _generate(OracleBackend(), make, True)
        assert t_opt == t_ref
        for a, e in zip(l_opt, l_ref):
            assert np.max(np.abs(a - e)) <= 1e-4 * float(np.abs(e).max()) + 5e-4


def test_oracle_runs_the_optimised_stream_to_the_same_values():
    """The optimizer must not change what a program computes: the oracle, which executes instruction by instruction,
    returns the same logits for the emitted program, for the optimised one and for the one whose norms the backend's
    pre-pass made CustomCalls (bit for bit: the same operations remain)."""
    runs = [_generate(OracleBackend(), MAKERS["ministral-f32"], fe, n_new=3, pipeline=pl) for fe, pl in ((False, False), (True, False), (True, True))]
    for t_b, l_b, _ in runs[1:]:
        assert runs[0][0] == t_b
        for a, b in zip(runs[0][1], l_b):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_norm_custom_calls_on_the_device(hip, dtype):
    """gpt_rs.hip.layer_norm.v1 / rms_norm.v1 as instructions of a program: fusion on and off against the oracle, whose
    definition of the calls is the functional's own sequence; a malformed call is a spec violation, not a crash."""
    from gptrs_amd.backend import BackendError
    from parity import check_program
    fb = FunctionBuilder("main", dtype)
    x, g, b, g2 = fb.param(dtype, [7, 96]), fb.param(dtype, [96]), fb.param(dtype, [96]), fb.param(dtype, [96])
    attrs = {"eps": {"kind": "F64", "value": 1e-5}, "axis": {"kind": "I64", "value": 1}}
    ln = fb.custom_call(FE.NORM_TARGETS["layer_norm"], [x, g, b], x.spec, attrs)
    out = fb.custom_call(FE.NORM_TARGETS["rms_norm"], [ln, g2], x.spec, attrs)
    fb.set_results([out, ln])
    rng = np.random.default_rng(5)
    arrays = [rng.standard_normal(s.dims).astype(np.float32) for s in Program(fb).param_specs]
    tol = dict(atol=5e-4, rtol=1e-4) if dtype == "F32" else dict(atol=4e-2, rtol=2e-2)
    check_program(hip, Program(fb), arrays, what="norm custom calls", **tol)
    bad = FunctionBuilder("main", dtype)
    x, g = bad.param(dtype, [7, 96]), bad.param(dtype, [95])
    bad.set_results([bad.custom_call(FE.NORM_TARGETS["rms_norm"], [x, g], x.spec, attrs)])
    with pytest.raises(BackendError) as err:
        hip.run_program(Program(bad), [hip.materialize(TensorSpec(dtype, (7, 96)), None), hip.materialize(TensorSpec(dtype, (95,)), None)])
    assert err.value.kind == "spec"


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("rows", [1, 5, 64])
def test_folded_gain_and_bias_inputs(hip, dtype, rows):
    """layer_norm -> linear with bias -> rms_norm over a [rows, 96] input, optimised against the HIP backend: gamma, beta,
    the bias and the RMS gain reach the program as derived parameters of the broadcast shape.  Values against the oracle
    running the emitted program; the fused kernels must have been chosen (4 launches or fewer); the derived handles
    hold no buffer until someone reads them, and read back as the broadcast."""
    n, n2 = 96, 64
    fb = FunctionBuilder("main", dtype)
    x = fb.param(dtype, [rows, n])
    g, b, w, bias, g2 = fb.param(dtype, [n]), fb.param(dtype, [n]), fb.param(dtype, [n, n2]), fb.param(dtype, [n2]), fb.param(dtype, [n2])
    h, *_ = F.layer_norm(x, g, b, 1e-5)
    y = F.linear(h, w, bias)
    out, *_ = F.rms_norm(y, g2, 1e-5)
    fb.set_results([out])
    prog = Program(fb)
    rng = np.random.default_rng(rows)
    arrays = [rng.standard_normal(s.dims).astype(np.float32) for s in prog.param_specs]
    from parity import oracle_run, to_bytes
    want = oracle_run(prog, arrays)[0]
    handles = [hip.materialize(s, to_bytes(a, s.dtype)) for s, a in zip(prog.param_specs, arrays)]
    res = hip.param_resolver()
    ids = [None] + [0x5000 + 16 * rows + i + (256 if dtype == "Bf16" else 0) for i in range(1, 6)]
    for sid, h in zip(ids[1:], handles[1:]):
        res.set(FE.stable_id_bytes(sid), h)
    before = hip.counter("bytes_allocated")
    opt = FE.optimize(prog, [FE.ARG] + [FE.PARAM] * 5, ids, hip, res)
    assert opt.folds_run == 4 and [tuple(s.dims) for s in opt.program.param_specs] == [(rows, n), (n, n2), (rows, n), (rows, n), (rows, n2), (rows, n2)]
    assert hip.counter("bytes_allocated") == before, "a folded broadcast is not materialised by the fold"
    feeds = [handles[0]] + [res.get(FE.stable_id_bytes(p.stable_id)) for p in opt.inputs[1:]]
    got = hip.to_numpy(hip.run_program(opt.program, feeds)[0])
    assert hip.counter("last_program_launches") <= 4
    tol = dict(atol=5e-4, rtol=1e-4) if dtype == "F32" else dict(atol=4e-2, rtol=2e-2)
    assert_close(got, want, what="optimised program", **tol)
    # the same through the generic kernels (fusion off reads the derived parameters' data, which exist from then on)
    hip.set_option("fusion", 0)
    try:
        plain = hip.to_numpy(hip.run_program(opt.program, feeds)[0])
    finally:
        hip.set_option("fusion", 1)
    assert_close(plain, want, what="optimised program, fusion off", **tol)
    gamma_b = hip.to_numpy(feeds[2])
    src = arrays[1] if dtype == "F32" else hip.to_numpy(handles[1])
    assert gamma_b.shape == (rows, n) and np.array_equal(gamma_b, np.broadcast_to(src, (rows, n)))


def test_fusion_report_matches_what_runs(hip):
    """The device-free report and the planner agree: the number of launches of a decode step is the number of lines."""
    from gptrs_amd import backend as B
    m = MAKERS["ministral-bf16"](hip)
    m.front_end = False
    gen = models.Generator(m, PROMPT, kv_cache_capacity=64)
    hip.set_option("graphs", 0)
    hip.set_option("chain", 0)
    try:
        gen.step()
        launches = hip.counter("last_program_launches")
    finally:
        hip.set_option("graphs", 1)
        hip.set_option("chain", 1)
    prog, _ = m._build(1, 64, True, 1, False)
    lines = B.fusion_report(prog)
    assert len(lines) == 2 + 5 * MID_MINISTRAL.num_layers and launches >= len(lines)
