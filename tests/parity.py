"""Helpers shared by the parity tests: run one PTIR program on the HIP backend and on the CPU
oracle with identical inputs and compare (test infrastructure)."""
from __future__ import annotations

import json

import numpy as np

import __graft_entry__ as entry

entry.load_package()
from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec, f32_to_bf16_bits  # noqa: E402

po = entry.load_oracle()

# the reference suite's tolerance: |e - a| <= ATOL + RTOL * max(|e|, |a|)
# (crates/gpt-rs-backend-tests/src/torch_parity/common.rs:14-15, 286-299)
ATOL, RTOL = 5e-4, 1e-4


def to_bytes(arr: np.ndarray, dtype: str) -> bytes:
    if dtype == "Bf16":
        return f32_to_bf16_bits(np.asarray(arr, np.float32)).astype("<u2").tobytes()
    if dtype == "F32":
        return np.asarray(arr, dtype="<f4").tobytes()
    if dtype == "Si32":
        return np.asarray(arr, dtype="<i4").tobytes()
    if dtype == "I1":
        return np.asarray(arr, dtype=np.uint8).tobytes()
    if dtype == "Si8":
        return np.asarray(arr, dtype=np.int8).tobytes()
    if dtype == "Ui8":
        return np.asarray(arr, dtype=np.uint8).tobytes()
    raise ValueError(dtype)


def oracle_run(program: Program, arrays):
    ins = [po.OTensor.from_bytes(s.dtype, s.dims, to_bytes(a, s.dtype)) for s, a in zip(program.param_specs, arrays)]
    return [t.a for t in po.run_program(json.loads(program.json_bytes), ins)]


def hip_run(be, program: Program, arrays, donate=None):
    hs = [be.materialize(s, to_bytes(a, s.dtype)) for s, a in zip(program.param_specs, arrays)]
    outs = be.run_program(program, hs, donate)
    return [be.to_numpy(o) for o in outs]


def assert_close(actual, expected, atol=ATOL, rtol=RTOL, what=""):
    actual = np.asarray(actual)
    expected = np.asarray(expected)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    if actual.dtype.kind in "iub":
        assert np.array_equal(actual, expected), f"{what}: integer results differ"
        return
    a64, e64 = actual.astype(np.float64), expected.astype(np.float64)
    both_nan = np.isnan(a64) & np.isnan(e64)
    same_inf = np.isinf(a64) & np.isinf(e64) & (np.sign(a64) == np.sign(e64))
    diff = np.where(both_nan | same_inf, 0.0, np.abs(a64 - e64))
    tol = atol + rtol * np.maximum(np.abs(a64), np.abs(e64))
    tol = np.where(np.isfinite(tol), tol, 0.0)
    bad = ~(diff <= tol)
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, diff, -1)), diff.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} elements differ; worst at {idx}: "
                             f"actual {actual[idx]} expected {expected[idx]}")


def check_program(be, program: Program, arrays, atol=ATOL, rtol=RTOL, both_modes=True, what=""):
    """Runs `program` on the oracle and on HIP with the fusion pass off and on (the reference
    harness's two legs, torch_parity/harness.rs:494-511) and compares every result."""
    exp = oracle_run(program, arrays)
    modes = (0, 1) if both_modes else (1,)
    for fusion in modes:
        be.set_option("fusion", fusion)
        try:
            got = hip_run(be, program, arrays)
        finally:
            be.set_option("fusion", 1)
        assert len(got) == len(exp)
        for i, (g, e) in enumerate(zip(got, exp)):
            assert_close(g, e, atol, rtol, f"{what} result {i} (fusion={fusion})")
    return exp
