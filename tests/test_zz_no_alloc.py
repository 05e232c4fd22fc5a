"""The allocation-free sampling entry point, gptrs_hip_sample_decode_rows_into, against the existing
gptrs_hip_sample_decode_rows_begin / _wait on the same logits: integer results, so bit-exact.  Two calls in a row, the
second on a smaller input (the fixed device scratch keeps the first call's partials: nothing stale may be read), both
float dtypes, ties, and the size limit."""
import numpy as np
import pytest

from gptrs_amd.backend import BackendError
from gptrs_amd.ptir import TensorSpec, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _logits(hip, rows, vocab, dtype, seed):
    x = np.random.default_rng(seed).normal(0, 2, (rows, vocab)).astype(np.float32)
    x[rows // 2, 5] = x[rows // 2, vocab - 3] = 60.0                     # a tie: the smaller index wins
    data = x.tobytes() if dtype == "F32" else f32_to_bf16_bits(x).tobytes()
    return hip.materialize(TensorSpec(dtype, [rows, vocab]), data)


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_rows_into_matches_rows_begin(hip, dtype):
    allocated = None
    for call, (rows, vocab) in enumerate([(64, 131072), (3, 50257), (1, 700), (17, 131072)]):
        h = _logits(hip, rows, vocab, dtype, 10 + call)
        out = hip.materialize(TensorSpec("Si32", [rows]), np.full(rows, -7, np.int32))
        want = hip.sample_decode_rows_wait(hip.sample_decode_rows_begin(h), rows)
        hip.synchronize()
        before = hip.counter("bytes_allocated")
        hip.sample_decode_rows_into(h, out)
        assert hip.counter("bytes_allocated") == before, "the call went to the allocator"
        got = hip.to_numpy(out).tolist()
        assert got == want, f"call {call}: rows {rows} vocab {vocab}"
        assert got[rows // 2] == 5
        allocated = before if allocated is None else allocated


def test_rows_into_limits(hip):
    out = hip.materialize(TensorSpec("Si32", [65]), None)
    with pytest.raises(BackendError) as ei:
        hip.sample_decode_rows_into(_logits(hip, 65, 1000, "F32", 1), out)
    assert "exceed" in str(ei.value) and ei.value.kind == "execution"
    with pytest.raises(BackendError):                                    # output of the wrong length
        hip.sample_decode_rows_into(_logits(hip, 4, 1000, "F32", 1), hip.materialize(TensorSpec("Si32", [3]), None))
    with pytest.raises(BackendError):                                    # output of the wrong dtype
        hip.sample_decode_rows_into(_logits(hip, 4, 1000, "F32", 1), hip.materialize(TensorSpec("F32", [4]), None))
    # the backend still works after the refusals
    h = _logits(hip, 2, 1000, "F32", 2)
    o = hip.materialize(TensorSpec("Si32", [2]), None)
    hip.sample_decode_rows_into(h, o)
    assert hip.to_numpy(o).tolist() == hip.sample_decode_rows_wait(hip.sample_decode_rows_begin(h), 2)
