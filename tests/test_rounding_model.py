"""Pins oracle/rounding_model.py (a numpy restatement of the Ministral decoder with explicit bf16 rounding points):
(1) rounding off, it reproduces the PTIR oracle's F32 run of models.Ministral (prefill over all rows, decode over the
    cache) -- the model's arithmetic, independent of the PTIR emitters;
(2) rounding on, one-row steps reproduce the PTIR oracle running an F32 program in which every rounding point is an
    explicit Cast(Bf16) -> Cast(F32) pair around the functional;
(3) the one site (2) cannot express, probabilities rounded before P.V in a many-row attention, against a plain Python
    loop over a tiny head."""
import numpy as np
import pytest

from gptrs_amd import functional as F
from gptrs_amd import models
from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec, bf16_bits_to_f32, f32_to_bf16_bits
from oracle.rounding_model import MinistralRoundingModel, bf16_round
from oracle_backend import OracleBackend

TINY = models.MinistralConfig(vocab_size=64, context_length=32, embed_dim=16, num_layers=2, num_heads=4, num_kv_heads=2,
                              head_dim=4, ffn_dim=48, rotary_dim=4, rope_theta=10000.0)
MID = models.MinistralConfig(vocab_size=300, context_length=64, embed_dim=128, num_layers=2, num_heads=8, num_kv_heads=2,
                             head_dim=32, ffn_dim=256, rotary_dim=16, rope_theta=1e6)


def _weights(m, be):
    return {n: np.asarray(be.to_numpy(m.param_handle(n)), np.float32) for n in m.param_names}


def _rope(cfg):
    rc = F.RopeConfig(cfg.rotary_dim, cfg.rope_theta, cfg.rope_scaling)
    return lambda start, count: F.rotary_cos_sin_cache_slice(start, count, rc)


def test_bf16_round_is_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, 3.0e38, 1e-40, 0.0, -0.0, 1.0 + 2.0 ** -8 + 2.0 ** -20], np.float32)
    assert np.array_equal(bf16_round(x), bf16_bits_to_f32(f32_to_bf16_bits(x)))
    # 1 + 2^-8 is exactly between 1 and 1 + 2^-7: to even (1.0); 1 + 3 * 2^-8 to 1 + 2^-6
    assert bf16_round(np.array([1.00390625], np.float32))[0] == 1.0
    assert bf16_round(np.array([1.01171875], np.float32))[0] == np.float32(1.015625)
    rng = np.random.default_rng(0)
    y = rng.standard_normal(10000).astype(np.float32)
    assert np.array_equal(bf16_round(bf16_round(y)), bf16_round(y))
    assert np.max(np.abs(bf16_round(y) - y) / np.abs(y)) <= 2.0 ** -8


@pytest.mark.parametrize("cfg", [TINY, MID], ids=["tiny", "mid"])
def test_without_rounding_it_is_the_f32_model(cfg):
    be = OracleBackend()
    m = models.Ministral.random(cfg, be, seed=3, dtype="F32", std=0.2)
    rm = MinistralRoundingModel(cfg, _weights(m, be), _rope(cfg), rounding=False)
    prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab_size, 7)]
    caches, mine = [None] * cfg.num_layers, [None] * cfg.num_layers
    want = be.to_numpy(m.forward_with_decode_cache(prompt, 0, caches, 16))
    got = rm.forward(prompt, 0, mine, last_row_only=False)
    scale = float(np.abs(want).max())
    assert np.max(np.abs(got - want)) <= 1e-5 * scale
    for step, tok in enumerate([5, 9, 2]):
        want = be.to_numpy(m.forward_with_decode_cache([tok], 7 + step, caches, 16))
        got = rm.forward([tok], 7 + step, mine)
        assert np.max(np.abs(got - want)) <= 1e-5 * scale
    # the caches hold the same rows (K after RoPE)
    assert np.allclose(mine[0][0], be.to_numpy(caches[0].keys)[:, :10], rtol=1e-5, atol=1e-5)
    assert np.allclose(mine[1][1], be.to_numpy(caches[1].values)[:, :10], rtol=1e-5, atol=1e-5)


def _explicit_cast_program(cfg, capacity):
    """One decode step of a one-layer model as an F32 program whose rounding points are Cast pairs."""
    a = cfg.attention_config()
    d, half = cfg.embed_dim, cfg.rotary_dim // 2
    fb = FunctionBuilder("main", "F32")
    rb = lambda t: t.cast("Bf16").cast("F32")   # noqa: E731
    tok, cos, sin = fb.param("Si32", [1]), fb.param("F32", [1, half]), fb.param("F32", [1, half])
    upd, qst = fb.param("Si32", [3]), fb.param("Si32", [1])
    ck, cv = (fb.param("F32", [a.num_key_value_heads, capacity, a.kv_head_dim]) for _ in range(2))
    names = ["tok_embeddings.weight", "blocks.0.norm_1.gamma", "blocks.0.attention.w_qkv", "blocks.0.attention.w_out",
             "blocks.0.norm_2.gamma", "blocks.0.feed_forward.w_gate", "blocks.0.feed_forward.w_up", "blocks.0.feed_forward.w_down",
             "final_norm.gamma", "lm_head"]
    shapes = {"tok_embeddings.weight": (cfg.vocab_size, d), "blocks.0.norm_1.gamma": (d,), "blocks.0.attention.w_qkv": (d, a.total_projection_dim),
              "blocks.0.attention.w_out": (a.query_projection_dim, d), "blocks.0.norm_2.gamma": (d,),
              "blocks.0.feed_forward.w_gate": (d, cfg.ffn_dim), "blocks.0.feed_forward.w_up": (d, cfg.ffn_dim),
              "blocks.0.feed_forward.w_down": (cfg.ffn_dim, d), "final_norm.gamma": (d,), "lm_head": (d, cfg.vocab_size)}
    P = {n: fb.param("F32", shapes[n]) for n in names}
    x = F.embedding_lookup(P["tok_embeddings.weight"], tok)
    n1 = rb(F.rms_norm(x, P["blocks.0.norm_1.gamma"], cfg.eps)[0])
    qkv = rb(n1.matmul(P["blocks.0.attention.w_qkv"]))
    qkv = rb(F.apply_rope_qkv_packed(a, qkv, rb(cos), rb(sin)))
    ctx, k2, v2 = F.attention_decode_cache(a, qkv, ck, cv, upd, qst)
    h = rb(ctx).matmul(P["blocks.0.attention.w_out"]) + x
    n2 = rb(F.rms_norm(h, P["blocks.0.norm_2.gamma"], cfg.eps)[0])
    act = rb(F.swiglu(n2.matmul(P["blocks.0.feed_forward.w_gate"]), n2.matmul(P["blocks.0.feed_forward.w_up"])))
    out = act.matmul(P["blocks.0.feed_forward.w_down"]) + h
    logits = rb(F.rms_norm(out, P["final_norm.gamma"], cfg.eps)[0]).matmul(P["lm_head"])
    fb.set_results([k2, v2, logits])
    return Program(fb), names


@pytest.mark.parametrize("cfg", [TINY, MID], ids=["tiny", "mid"])
def test_rounding_points_of_one_row_steps(cfg):
    import dataclasses
    cfg = dataclasses.replace(cfg, num_layers=1)
    be = OracleBackend()
    m = models.Ministral.random(cfg, be, seed=4, dtype="F32", std=0.3, bf16_values=True)
    w = _weights(m, be)
    rope = _rope(cfg)
    rm = MinistralRoundingModel(cfg, w, rope, rounding=True, bf16_scale=False)   # (the F32 program below carries an f32 scale)
    cap = 8
    prog, names = _explicit_cast_program(cfg, cap)
    a = cfg.attention_config()
    mat = lambda spec, arr: be.materialize(spec, np.ascontiguousarray(arr))   # noqa: E731
    ck = cv = be.materialize(TensorSpec("F32", (a.num_key_value_heads, cap, a.kv_head_dim)), None)
    mine = [None]
    for pos, tok in enumerate([3, 11, 7, 1]):
        cos, sin = rope(pos, 1)
        args = [mat(TensorSpec("Si32", (1,)), np.array([tok], np.int32)), mat(TensorSpec("F32", cos.shape), cos), mat(TensorSpec("F32", sin.shape), sin),
                mat(TensorSpec("Si32", (3,)), np.array([0, pos, 0], np.int32)), mat(TensorSpec("Si32", (1,)), np.array([pos], np.int32)), ck, cv]
        ck, cv, logits = be.run_program(prog, args + [m.param_handle(n) for n in names])
        want = be.to_numpy(logits)
        got = rm.forward([tok], pos, mine)
        # the same roundings; what differs is f32 summation order and (e / l) . V against (e . V) / l, which can move a
        # value across a bf16 rounding boundary now and then (one bf16 ulp of one context element)
        scale = float(np.abs(want).max())
        assert np.max(np.abs(got - want)) <= 2e-3 * scale
        assert np.median(np.abs(got - want)) <= 2e-5 * scale
    assert np.array_equal(bf16_round(mine[0][0]), mine[0][0]), "cached K rows are bf16 values"
    # and rounding matters at this size: the model with the rounding points is measurably away from the one without
    plain = MinistralRoundingModel(cfg, w, rope, rounding=False)
    c2 = [None]
    for pos, tok in enumerate([3, 11, 7, 1]):
        ref = plain.forward([tok], pos, c2)
    assert np.max(np.abs(ref - got)) > 20 * np.max(np.abs(got - want))


def test_rounded_probabilities_of_a_many_row_attention():
    """_attend with round_p: per query row i, ctx = bf16(sum_j bf16(e_ij) v_j / sum_j e_ij), e_ij = exp(s_ij - max_j s_ij),
    keys j <= first_pos + i; written out as Python loops over one kv head with two query heads."""
    import dataclasses
    import math
    cfg = dataclasses.replace(TINY, num_heads=2, num_kv_heads=1, head_dim=4, embed_dim=8)
    rm = MinistralRoundingModel(cfg, {}, None, rounding=True)
    rng = np.random.default_rng(2)
    T, L, first = 3, 5, 2
    q = bf16_round(rng.standard_normal((T, 8)).astype(np.float32))
    K = bf16_round(rng.standard_normal((1, L, 4)).astype(np.float32))
    V = bf16_round(rng.standard_normal((1, L, 4)).astype(np.float32))
    got = rm._attend(q, K, V, first, round_p=True)
    f32 = np.float32
    for i in range(T):
        for h in range(2):
            s = [f32(sum(f32(q[i, 4 * h + d]) * f32(K[0, j, d]) for d in range(4))) * f32(0.5) for j in range(first + i + 1)]
            mx = max(s)
            e = [f32(math.exp(float(v - mx))) for v in s]
            l = f32(sum(e))
            for d in range(4):
                o = f32(sum(float(bf16_round(np.array([ej], f32))[0]) * float(V[0, j, d]) for j, ej in enumerate(e)))
                want = bf16_round(np.array([o / l], f32))[0]
                assert abs(float(got[i, 4 * h + d]) - float(want)) <= 2.0 ** -8 * abs(float(want)) + 1e-7
