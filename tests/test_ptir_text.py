"""The text form of PTIR programs (the reference's `Display`, crates/gpt-rs/src/backend/spec.rs:858-1069) against the
reference's own fixtures: tests/golden/lit/*.lit are the data files of crates/gpt-rs/tests/pass_lit_*.rs, each case an
optimizer INPUT and the EXPECTED program after the pass.  Checked here: the reader and the printer reproduce the
reference's printed text exactly, and INPUT and EXPECTED compute the same values (on the CPU oracle here, on the
device in the gpu-marked test), which is what the passes they document must preserve."""
import glob
import os
import re

import numpy as np
import pytest

from gptrs_amd import ptir_text as T
from parity import hip_run, oracle_run

LIT_DIR = os.path.join(os.path.dirname(__file__), "golden", "lit")
FIXTURES = sorted(glob.glob(os.path.join(LIT_DIR, "*.lit")))
CASES = [(os.path.basename(f), c) for f in FIXTURES for c in T.load_lit_cases(f)]
IDS = [f"{name}:{c.name}" for name, c in CASES]


def test_all_six_fixtures_are_present():
    assert [os.path.basename(f) for f in FIXTURES] == ["dedup.lit", "elementwise.lit", "param_only_fold_to_param.lit", "reshape.lit",
                                                       "slice.lit", "transpose.lit"]
    assert len(CASES) == 9


@pytest.mark.parametrize("name,case", CASES, ids=IDS)
def test_reader_and_printer_reproduce_the_reference_text(name, case):
    # EXPECTED is the reference printer's own output; INPUT is hand-written and may hold an empty `params:` line,
    # which the printer omits (spec.rs:880-893)
    assert T.format_program(T.parse_program(case.expected)) == case.expected
    want = re.sub(r" *params:\n(?= *body:)", "", case.input)
    assert T.format_program(T.parse_program(case.input)) == want


def _inputs_for(name, prog_in, prog_exp, seed):
    """Seeded arrays for INPUT's parameters; EXPECTED's parameters by id, a derived one computed from its definition."""
    rng = np.random.default_rng(seed)
    fn_in, fn_exp = prog_in.obj["functions"][0], prog_exp.obj["functions"][0]
    by_id = {}
    for vid, spec in zip(fn_in["parameter_ids"], prog_in.param_specs):
        by_id[vid] = (rng.uniform(0.5, 2.0, spec.dims)).astype(np.float32)   # positive: Rsqrt appears in the fixtures
    arrays_exp = []
    for vid, spec in zip(fn_exp["parameter_ids"], prog_exp.param_specs):
        if vid not in by_id:
            # param_only_fold_to_param.lit: %5 is the folded parameter-only chain Reshape[6](Transpose[1,0](%1))
            assert name == "param_only_fold_to_param.lit" and vid == 5
            by_id[vid] = np.ascontiguousarray(by_id[1].T).reshape(6)
        assert tuple(by_id[vid].shape) == tuple(spec.dims)
        arrays_exp.append(by_id[vid])
    return [by_id[v] for v in fn_in["parameter_ids"]], arrays_exp


@pytest.mark.parametrize("name,case", CASES, ids=IDS)
def test_input_and_expected_agree_on_the_oracle(name, case):
    p_in, p_exp = T.parse_program(case.input), T.parse_program(case.expected)
    a_in, a_exp = _inputs_for(name, p_in, p_exp, 7)
    got, want = oracle_run(p_exp, a_exp), oracle_run(p_in, a_in)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


@pytest.mark.gpu
@pytest.mark.parametrize("name,case", CASES, ids=IDS)
def test_fixture_programs_on_the_device(hip, name, case):
    p_in, p_exp = T.parse_program(case.input), T.parse_program(case.expected)
    a_in, a_exp = _inputs_for(name, p_in, p_exp, 8)
    want = oracle_run(p_in, a_in)
    for prog, arrays in ((p_in, a_in), (p_exp, a_exp)):
        got = hip_run(hip, prog, arrays)
        for g, w in zip(got, want):
            np.testing.assert_allclose(g, w, rtol=1e-6, atol=1e-6)


def test_reader_rejects_what_it_does_not_cover():
    ok = T.load_lit_cases(FIXTURES[0])[0].expected
    with pytest.raises(T.PtirTextError):
        T.parse_program(ok.replace("ptir.v0.4", "ptir.v0.3"))
    with pytest.raises(T.PtirTextError):
        T.parse_program(ok.replace("ElementwiseBinary(Add)", "DotGeneral(DotGeneralSpec { })"))
    with pytest.raises(T.PtirTextError):
        T.parse_program(ok.replace("tensor<F32 x 2>", "tensor<F32 x ?n>"))
    with pytest.raises(T.PtirTextError):
        T.parse_program("func @x {\n}\n")
