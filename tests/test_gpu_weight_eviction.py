"""GPU: a bf16 weight whose decode-chain copy exists is held twice; once no kernel of the programs that use it reads the
row-major form, the backend gives that form back ("evict_packed_weights", on by default) and rebuilds it, bit for
bit, from the packed copy whenever something asks for it: a read-back, a kernel family that has no copy yet, the
removal of the copies."""
import numpy as np
import pytest

from gptrs_amd import models

pytestmark = pytest.mark.gpu

CFG = models.MinistralConfig(vocab_size=512, context_length=128, embed_dim=256, num_layers=2, num_heads=8,
                             num_kv_heads=2, head_dim=32, ffn_dim=512, rotary_dim=32, rope_theta=1e6)
PROMPT = [3, 17, 42, 5, 99, 311, 8, 250, 1]
LINEARS = 5 * CFG.num_layers + 1   # w_qkv, w_out, w_gate, w_up, w_down per layer, and the head


def _make(be):
    return models.Ministral.random(CFG, be, seed=9, dtype="Bf16", std=0.08, residual_dtype="F32")


def _decode(be, m, n_new=6):
    gen = models.Generator(m, PROMPT, kv_cache_capacity=64)
    toks, logits = [], [be.to_numpy(gen.logits)[-1].copy()]
    for _ in range(n_new):
        toks.append(gen.step())
        logits.append(be.to_numpy(gen.logits)[-1].copy())
    return gen, toks, logits


def _weights(be, m):
    return {n: bytes(be.to_literal(m.param_handle(n))) for n in m.param_names}


def test_row_major_weights_leave_and_come_back_exactly(hip):
    hip.set_option("evict_packed_weights", 0)
    try:
        m0 = _make(hip)
        want = _weights(hip, m0)
        e0 = hip.counter("weights_evicted")
        _, toks0, logits0 = _decode(hip, m0)
        assert hip.counter("weights_evicted") == e0, "switched off"
        prompts = [PROMPT, PROMPT[::-1], PROMPT[2:] + PROMPT[:2]]
        rows0 = models.BatchGenerator(m0, prompts, kv_cache_capacity=64).generate(4)
        del m0
    finally:
        hip.set_option("evict_packed_weights", 1)

    m = _make(hip)
    e0, r0 = hip.counter("weights_evicted"), hip.counter("weights_restored")
    gen, toks, logits = _decode(hip, m)
    assert hip.counter("weights_evicted") - e0 == LINEARS, "every linear weight left once prefill and decode had their copies"
    assert hip.counter("weights_restored") == r0, "and nothing asked for one back while decoding"
    assert toks == toks0
    for a, b in zip(logits, logits0):
        assert np.array_equal(a, b), "the kernels read the same copies either way"

    # a read-back rebuilds the matrix from the packed copy (both matrices of the gate / up pair from their shared one)
    got = _weights(hip, m)
    assert hip.counter("weights_restored") - r0 == LINEARS
    for name in m.param_names:
        assert got[name] == want[name], f"{name} changed on its way through the packed copy"

    # the next step runs on the copies and lets the row-major forms go again
    e1 = hip.counter("weights_evicted")
    gen.step()
    assert hip.counter("weights_evicted") - e1 == LINEARS

    # a kernel family without a copy yet (several rows decoded at once) gets the matrices back to build its own
    built, r1 = hip.counter("derived_weights_built"), hip.counter("weights_restored")
    rows = models.BatchGenerator(m, prompts, kv_cache_capacity=64).generate(4)
    assert rows == rows0
    assert hip.counter("derived_weights_built") > built and hip.counter("weights_restored") > r1

    # removing the copies leaves every weight in place, and decoding starts over from there
    hip.set_option("drop_derived_weights", 1)
    assert _weights(hip, m) == want
    _, toks2, logits2 = _decode(hip, m)
    assert toks2 == toks0 and all(np.array_equal(a, b) for a, b in zip(logits2, logits0))


def test_a_replaced_weight_is_read_from_its_own_copies(hip):
    """set_param after the copies exist: the new values are what the next step reads and what a read-back returns."""
    m = _make(hip)
    _decode(hip, m, n_new=2)
    name = "blocks.0.attention.w_out"
    new = (np.random.default_rng(5).standard_normal(m.param_specs[name].dims) * 0.05).astype(np.float32)
    m.set_param(name, new, "Bf16")
    _, toks_a, logits_a = _decode(hip, m, n_new=3)
    back_a = bytes(hip.to_literal(m.param_handle(name)))
    del m
    hip.set_option("evict_packed_weights", 0)
    try:
        fresh = _make(hip)
        fresh.set_param(name, new, "Bf16")
        _, toks_b, logits_b = _decode(hip, fresh, n_new=3)
        back_b = bytes(hip.to_literal(fresh.param_handle(name)))
    finally:
        hip.set_option("evict_packed_weights", 1)
    assert toks_a == toks_b and all(np.array_equal(a, b) for a, b in zip(logits_a, logits_b))
    assert back_a == back_b


def test_a_weight_that_the_same_program_also_reads_stays(hip):
    """One tensor passed twice, once as the weight of a decode-shaped linear and once in a position that reads its
    storage (an elementwise add): it is not evicted (it would be rebuilt on every call), and both uses see its values."""
    from parity import FunctionBuilder, Program, to_bytes
    k, n = 1024, 1024
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((1, k)).astype(np.float32)
    fb = FunctionBuilder("main")
    a, b, c = fb.param("Bf16", [1, k]), fb.param("Bf16", [k, n]), fb.param("Bf16", [k, n])
    fb.set_results([a.matmul(b), c + c])
    prog = Program(fb)
    hw = hip.materialize(prog.param_specs[1], to_bytes(w, "Bf16"))
    hx = hip.materialize(prog.param_specs[0], to_bytes(x, "Bf16"))
    e0, r0 = hip.counter("weights_evicted"), hip.counter("weights_restored")
    for _ in range(3):
        y, d = hip.run_program(prog, [hx, hw, hw])
    assert hip.counter("weights_evicted") == e0 and hip.counter("weights_restored") == r0
    wb = hip.to_numpy(hw).astype(np.float32)
    assert np.array_equal(hip.to_numpy(d).astype(np.float32), 2.0 * wb), "doubling a bf16 value is exact"
    ref = hip.to_numpy(hx).astype(np.float32) @ wb
    assert np.allclose(hip.to_numpy(y).astype(np.float32), ref, rtol=2 ** -6, atol=2 ** -6 * float(np.abs(ref).max()))
    # alone, the same weight does leave once the decode copy exists
    fb2 = FunctionBuilder("main")
    a2, b2 = fb2.param("Bf16", [1, k]), fb2.param("Bf16", [k, n])
    fb2.set_results([a2.matmul(b2)])
    p2 = Program(fb2)
    y2 = hip.run_program(p2, [hx, hw])[0]
    assert hip.counter("weights_evicted") == e0 + 1, "the lone linear runs on the persistent launch, whose copy stands in for the matrix"
    assert np.array_equal(hip.to_numpy(y2), hip.to_numpy(y))
    assert bytes(hip.to_literal(hw)) == to_bytes(w, "Bf16"), "read back from the packed copy"
    assert hip.counter("weights_restored") == r0 + 1
