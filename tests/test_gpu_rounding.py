"""GPU, Ministral-3B width: is the distance between the bf16 device pipeline and the F32 oracle rounding, or a kernel
error?  Three measurements answer it.

(a) The same layer entirely in F32 on the device (f32 matrix-core GEMMs, f32 prefill attention at 1024 positions, RoPE,
    grouped-query heads, SwiGLU, the f32 decode kernels) against the F32 oracle at the f32 bar: 1e-4 relative.
(b) The mixed-precision program bench.py times (bf16 weights and matmul operands, f32 residual stream and logits) against
    oracle/rounding_model.py, which computes in f32 and rounds to bf16 exactly where that program stores a bf16 tensor
    (pinned on the CPU in tests/test_rounding_model.py), STAGE BY STAGE: every fused kernel of a layer is run on the
    model's own input to that stage and must return the model's output of it.  A bf16 result may differ in a stray
    element by one bf16 ulp (an f32 sum that falls on the other side of a rounding boundary: a few in ten thousand), an
    f32 result by 2e-5 relative.  Stage by stage, because whole-model logits cannot be held that tight: a difference of
    1e-5 relative in front of a rounding point moves 1e-5 / 2^-8 = 0.3 % of its outputs by a whole ulp, each rounding
    point re-draws part of the rounding noise, and after a layer's seven rounding points two CORRECT bf16 pipelines are
    half a rounding-noise apart (measured below).  A dropped k-tile, a wrong head mapping or a stale cache row fails its
    stage by orders of magnitude.  Covered: an 8-token and a 1024-token prompt (the batched-decode kernels and the
    prefill GEMMs, prefill attention), a decode step behind them through the persistent launch and through one kernel
    per fused op, int8 and int4-g128 weights at 128 and at 8 rows (BASELINE configs[4] at batch 8).
(c) Whole-model logits, as statistics: device vs rounding model is no larger than rounding model vs the same model
    without rounding, and the latter reproduces on the CPU the 3-5e-2 by which the bf16 bar of 2e-2 is missed
    (tests/test_gpu_configs.py reports that miss as an expected failure): the miss is the roundings."""
import contextlib

import numpy as np
import pytest

from gptrs_amd import functional as F
from gptrs_amd import models
from gptrs_amd.ptir import FunctionBuilder, Program, TensorSpec, f32_to_bf16_bits
from oracle.rounding_model import MinistralRoundingModel, bf16_round
from oracle_backend import OracleBackend, po
from parity import assert_close

pytestmark = pytest.mark.gpu

FULL = dict(vocab_size=131072, context_length=4096, embed_dim=3072, num_heads=32, num_kv_heads=8, head_dim=128,
            ffn_dim=9216, rotary_dim=128, rope_theta=1e6)


@contextlib.contextmanager
def blas_dots(min_macs=1 << 27):
    old = po.BLAS_DOT_MIN_MACS
    po.BLAS_DOT_MIN_MACS = min_macs
    try:
        yield
    finally:
        po.BLAS_DOT_MIN_MACS = old


@contextlib.contextmanager
def option(hip, name, value, restore=1):
    hip.set_option(name, value)
    try:
        yield
    finally:
        hip.set_option(name, restore)


def _rope(cfg):
    rc = F.RopeConfig(cfg.rotary_dim, cfg.rope_theta, cfg.rope_scaling)
    return lambda start, count: F.rotary_cos_sin_cache_slice(start, count, rc)


def _host_weights(cfg, seed):
    """The f32 arrays (bf16-representable values) that models.Ministral.random(seed, dtype="Bf16") uploads."""
    ob = OracleBackend()
    m = models.Ministral.random(cfg, ob, seed=seed, dtype="F32", bf16_values=True)
    return {n: ob.to_numpy(m.param_handle(n)) for n in m.param_names}


def _err(what, got, ref):
    e = np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64))
    print(f"{what}: max {e.max():.5f} mean {e.mean():.6f} (max |ref| {np.abs(ref).max():.2f})")
    return float(e.max()), float(e.mean())


# ------------------------------------------------------------------------------------------------ (a)
def test_full_width_layer_in_f32_vs_oracle(hip):
    cfg = models.MinistralConfig(num_layers=1, **FULL)
    prompt = np.random.default_rng(6).integers(0, cfg.vocab_size, 1024).tolist()
    ob = OracleBackend()
    mo = models.Ministral.random(cfg, ob, seed=5, dtype="F32")
    with blas_dots():
        co = [None]
        ref = ob.to_numpy(mo.forward_with_decode_cache(prompt, 0, co, 1280, last_logits_only=True))[-1]
        tok = int(np.argmax(ref))
        dref = ob.to_numpy(mo.forward_with_decode_cache([tok], 1024, co, 1280))[-1]
    kr, vr = ob.to_numpy(co[0].keys)[:, :1025], ob.to_numpy(co[0].values)[:, :1025]
    del mo
    mh = models.Ministral.random(cfg, hip, seed=5, dtype="F32")
    ch = [None]
    got = hip.to_numpy(mh.forward_with_decode_cache(prompt, 0, ch, 1280, last_logits_only=True))[-1]
    dgot = hip.to_numpy(mh.forward_with_decode_cache([tok], 1024, ch, 1280))[-1]
    kc, vc = hip.to_numpy(ch[0].keys)[:, :1025], hip.to_numpy(ch[0].values)[:, :1025]
    for what, g, r in (("prefill 1024 logits", got, ref), ("decode logits", dgot, dref), ("K rows", kc, kr), ("V rows", vc, vr)):
        _err("f32 layer, " + what, g, r)
        assert_close(g, r, atol=1e-4 * float(np.abs(r).max()), rtol=1e-4, what=what)
    assert int(np.argmax(got)) == tok


def _effective_weights(hip, mh, scheme, exact_scales):
    """What the quantised kernels multiply by.  The many-row GEMM forms bf16(code * scale) on its way into LDS; the
    decode kernels accumulate x * code in f32 and apply the scale to the sum (code * scale unrounded)."""
    out = {}
    for name in mh.param_names:
        spec = mh.param_specs[name]
        if name.endswith(".s"):
            continue
        raw = hip.to_literal(mh.param_handle(name))
        if name.endswith(".q"):
            base = name[:-2]
            s = hip.to_numpy(mh.param_handle(base + ".s")).astype(np.float32)
            if scheme == "w8":
                wq = po.dequantize_int8(np.frombuffer(raw, np.int8).reshape(spec.dims), s)
            else:
                wq = po.dequantize_int4_g128(np.frombuffer(raw, np.uint8).reshape(spec.dims), s)
            out[base] = wq if exact_scales else bf16_round(wq)
        else:
            out[name] = hip.to_numpy(mh.param_handle(name)).astype(np.float32)
    return out



# ------------------------------------------------------------------------------------------------ (b)
BF16_ULP_REL = 2.0 ** -7      # one bf16 ulp is at most 2^-7 of the value


class Stages:
    """Runs the fused kernels of layer 0 one at a time on inputs taken from a rounding-model trace.  Weights are the device
    model's own handles (plain, or codes and scales)."""

    def __init__(self, hip, cfg, mh):
        self.hip, self.cfg, self.mh, self.a = hip, cfg, mh, cfg.attention_config()

    def up(self, arr, dtype):
        arr = np.ascontiguousarray(arr)
        if dtype == "Bf16":
            return self.hip.materialize(TensorSpec("Bf16", arr.shape), f32_to_bf16_bits(arr.astype(np.float32)).tobytes())
        if dtype == "Si32":
            return self.hip.materialize(TensorSpec("Si32", arr.shape), arr.astype(np.int32).tobytes())
        return self.hip.materialize(TensorSpec("F32", arr.shape), arr.astype(np.float32).tobytes())

    def run(self, build, acts, weights):
        """acts: [(array, dtype)], weights: parameter names (a quantised one contributes its codes and scales)."""
        fb = FunctionBuilder("main", "Bf16")
        ins = [fb.param(dt, np.shape(arr)) for arr, dt in acts]
        handles = [self.up(arr, dt) for arr, dt in acts]
        W = {}
        for name in weights:
            if name + ".q" in self.mh.param_specs:
                for part in (".q", ".s"):
                    sp = self.mh.param_specs[name + part]
                    W[name + part] = fb.param(sp.dtype, sp.dims)
                    handles.append(self.mh.param_handle(name + part))
            else:
                sp = self.mh.param_specs[name]
                W[name] = fb.param(sp.dtype, sp.dims)
                handles.append(self.mh.param_handle(name))
        res = build(fb, W, *ins)
        res = list(res) if isinstance(res, (list, tuple)) else [res]
        fb.set_results(res)
        return [self.hip.to_numpy(o) for o in self.hip.run_program(Program(fb), handles)]

    @staticmethod
    def lin(W, name, x, out_dtype=None):
        if name + ".q" in W:
            return F.linear_quantized(x, W[name + ".q"], W[name + ".s"], out_dtype=out_dtype)
        return F.linear(x, W[name], out_dtype=out_dtype)


def _same_bf16(what, got, ref, max_flips=3e-3, upstream=0.0):
    """bf16 results: the same values but for stray elements one bf16 ulp apart.  `upstream`: an absolute allowance for a
    stage that rounds INSIDE (a norm folded into its projection): one normalised element that fell on the other side of a
    rounding boundary shifts every output of its row by ulp(element) * |weight|."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    d = np.abs(got.astype(np.float64) - ref)
    flips = float(np.mean(got != ref))
    # one ulp of the value, or (a result near zero, the remainder of a cancelling sum) the f32 sums' own tolerance
    tol = BF16_ULP_REL * np.maximum(np.abs(got), np.abs(ref)) + 2e-5 * float(np.abs(ref).max())
    beyond = float(np.mean(d > tol + upstream))
    print(f"  {what}: {flips:.5f} of the elements differ, {beyond:.5f} by more than an ulp, max |diff| {d.max():.6f} (max |ref| {np.abs(ref).max():.3f})")
    worst = np.unravel_index(np.argmax(d - tol - upstream), d.shape)
    assert np.all(d <= tol + upstream), f"{what}: element {worst}: {got[worst]} vs {ref[worst]}"
    if max_flips is not None:
        assert flips <= max_flips, f"{what}: {flips:.4%} of the elements differ"
    assert beyond <= 2e-3, f"{what}: {beyond:.4%} of the elements are more than an ulp apart"


def _same_f32(what, got, ref, rel=2e-5, upstream=0.0):
    d = np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64))
    beyond = float(np.mean(d > rel * float(np.abs(ref).max())))
    print(f"  {what}: max |diff| {d.max():.2e}, {beyond:.5f} of the elements beyond {rel:g} relative (max |ref| {np.abs(ref).max():.3f})")
    assert d.max() <= rel * float(np.abs(ref).max()) + upstream, what
    assert beyond <= (0.0 if upstream == 0.0 else 0.15), what


def _check_stages(st: Stages, tr, x, pos0, rope, caches_before, rows_of_head, many_row_p=True, skip_attention=False):
    """Every stage of layer 0 for the call whose model trace is `tr` (x: the layer's f32 input rows)."""
    cfg, a, pre = st.cfg, st.a, "blocks.0."
    T = x.shape[0]
    g1, g2, gf = pre + "norm_1.gamma", pre + "norm_2.gamma", "final_norm.gamma"
    wqkv, wout, wg, wu, wd = (pre + n for n in ("attention.w_qkv", "attention.w_out", "feed_forward.w_gate", "feed_forward.w_up", "feed_forward.w_down"))
    (n1,) = st.run(lambda fb, W, x_: F.rms_norm(x_, W[g1], cfg.eps)[0].cast("Bf16"), [(x, "F32")], [g1])
    _same_bf16("normalised row", n1, tr[pre + "n1"])
    (qkv,) = st.run(lambda fb, W, x_: Stages.lin(W, wqkv, F.rms_norm(x_, W[g1], cfg.eps)[0].cast("Bf16")), [(x, "F32")], [g1, wqkv])
    # (weights N(0, 0.02): |w| < 0.12; one flipped normalised element moves its row's outputs by ulp(element) * |w|)
    up1 = BF16_ULP_REL * float(np.abs(tr[pre + "n1"]).max()) * 0.12
    _same_bf16("norm + qkv projection", qkv, tr[pre + "qkv"], upstream=up1)
    cos, sin = rope(pos0, T)
    if not skip_attention:
        if caches_before is None:
            (roped,) = st.run(lambda fb, W, q, c, s: F.apply_rope_qkv_packed(a, q, c, s), [(tr[pre + "qkv"], "Bf16"), (cos, "Bf16"), (sin, "Bf16")], [])
            _same_bf16("RoPE", roped, tr[pre + "qkv_rope"])
            (ctx,) = st.run(lambda fb, W, q: F.attention(a, q, None)[0], [(tr[pre + "qkv_rope"], "Bf16")], [])
            # The kernel rounds its probabilities to bf16 against a reference point that it moves lazily, the model against
            # the row maximum: two draws of the same rounding, each within 2^-9 of every term p_j v_j.  The bound is relative
            # to the terms (sum_j p_j |v_j|, from the model), not to their sum, which cancels.
            _same_bf16("many-row attention", ctx, tr[pre + "ctx"], max_flips=None if T > 64 else 3e-3, upstream=2.0 ** -8 * tr["attention_mass"])
        else:
            cap = 1280
            kb = np.zeros((a.num_key_value_heads, cap, a.kv_head_dim), np.float32)
            vb = np.zeros_like(kb)
            kb[:, :pos0], vb[:, :pos0] = caches_before[0], caches_before[1]
            ctx, k2, v2 = st.run(
                lambda fb, W, q, c, s, kc, vc, u, qs: F.attention_decode_cache(a, F.apply_rope_qkv_packed(a, q, c, s), kc, vc, u, qs),
                [(tr[pre + "qkv"], "Bf16"), (cos, "Bf16"), (sin, "Bf16"), (kb, "Bf16"), (vb, "Bf16"), (np.array([0, pos0, 0]), "Si32"), (np.array([pos0]), "Si32")], [])
            _same_bf16("RoPE + attention over the cache", ctx, tr[pre + "ctx"])
            qp, kp = a.query_projection_dim, a.key_value_projection_dim
            want_k = tr[pre + "qkv_rope"][:, qp:qp + kp].reshape(a.num_key_value_heads, a.kv_head_dim)
            assert np.array_equal(k2[:, pos0], want_k) and np.array_equal(k2[:, :pos0], kb[:, :pos0]), "appended K row / older rows"
            assert np.array_equal(v2[:, pos0], tr[pre + "qkv"][:, qp + kp:].reshape(a.num_key_value_heads, a.kv_head_dim))
    (h,) = st.run(lambda fb, W, c, x_: Stages.lin(W, wout, c, "F32") + x_, [(tr[pre + "ctx"], "Bf16"), (x, "F32")], [wout])
    _same_f32("out projection + residual", h, tr[pre + "h"])
    def pair(fb, W, h_):
        n2 = F.rms_norm(h_, W[g2], cfg.eps)[0].cast("Bf16")
        return F.swiglu(Stages.lin(W, wg, n2), Stages.lin(W, wu, n2))

    (act,) = st.run(pair, [(tr[pre + "h"], "F32")], [g2, wg, wu])
    # d(silu(g) u) <= |u| dg + |g| du with |g|, |u| below 8 at this width
    up2 = BF16_ULP_REL * float(np.abs(tr[pre + "n2"]).max()) * 0.12 * 16
    _same_bf16("norm + gate / up + SwiGLU", act, tr[pre + "act"], upstream=up2)
    (out,) = st.run(lambda fb, W, a_, h_: Stages.lin(W, wd, a_, "F32") + h_, [(tr[pre + "act"], "Bf16"), (tr[pre + "h"], "F32")], [wd])
    _same_f32("down projection + residual", out, tr[pre + "out"])
    last = tr[pre + "out"][rows_of_head]
    (logits,) = st.run(lambda fb, W, o: Stages.lin(W, "lm_head", F.rms_norm(o, W[gf], cfg.eps)[0].cast("Bf16"), "F32"), [(last, "F32")], [gf, "lm_head"])
    return logits, BF16_ULP_REL * float(np.abs(rm_norm_max(last)).max()) * 0.12


def rm_norm_max(rows):
    """Upper bound of the normalised rows' magnitude (gamma = 1): |x| / rms(x)."""
    rows = np.asarray(rows, np.float32)
    return np.abs(rows) / np.sqrt(np.mean(rows * rows, axis=-1, keepdims=True))


@pytest.mark.parametrize("prompt_len", [8, 1024])
def test_every_stage_of_a_layer_vs_the_rounding_model(hip, prompt_len):
    cfg = models.MinistralConfig(num_layers=1, **FULL)
    prompt = np.random.default_rng(6).integers(0, cfg.vocab_size, prompt_len).tolist()
    mh = models.Ministral.random(cfg, hip, seed=5, dtype="Bf16", residual_dtype="F32")
    w = {n: hip.to_numpy(mh.param_handle(n)).astype(np.float32) for n in mh.param_names}   # the device's weights, read back
    rope = _rope(cfg)
    rm = MinistralRoundingModel(cfg, w, rope, rounding=True)
    st = Stages(hip, cfg, mh)
    # the prompt
    rm.trace = {}
    cm = [None]
    want = rm.forward(prompt, 0, cm, last_row_only=True)
    x = w["tok_embeddings.weight"][np.asarray(prompt)]
    print(f"prompt of {prompt_len}:")
    logits, up = _check_stages(st, rm.trace, x, 0, rope, None, slice(prompt_len - 1, prompt_len))
    _same_f32("final norm + head", logits, want, upstream=up)
    # one decode step behind it: the persistent launch, then one kernel per fused op
    tok = int(np.argmax(want[-1]))
    before = (cm[0][0].copy(), cm[0][1].copy())
    rm.trace = {}
    want = rm.forward([tok], prompt_len, cm)
    x = w["tok_embeddings.weight"][[tok]]
    for chain in (1, 0):
        print(f"decode step at position {prompt_len}, chain={chain}:")
        with option(hip, "chain", chain):
            c0 = hip.counter("chain_launches")
            logits, up = _check_stages(st, rm.trace, x, prompt_len, rope, before, slice(0, 1))
            launched = hip.counter("chain_launches") - c0
            print(f"  persistent launches: {launched}")
            assert (launched > 0) == bool(chain)
        _same_f32("final norm + head", logits, want, upstream=up)


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
def test_quantised_stages_at_128_and_at_8_rows(hip, scheme):
    """BASELINE configs[4]: int8 per-channel and int4-g128 linears (lm_head included).  128 rows (eight 16-token prompts
    stacked: the matrix-core GEMM over the codes) and 8 rows (a batch-8 decode step: the batched decode kernel over the
    codes), every linear stage on the rounding model's input.  The rounding model multiplies by what the kernels multiply
    by: bf16(code * scale) in the many-row GEMM, which dequantises on its way into LDS; code * scale unrounded in the
    decode kernels, which scale the f32 sum of x * code."""
    cfg = models.MinistralConfig(num_layers=1, **FULL)
    B, T = 8, 16
    prompts = np.random.default_rng(8).integers(0, cfg.vocab_size, (B, T)).tolist()
    mh = models.Ministral.random(cfg, hip, seed=5, dtype="Bf16", residual_dtype="F32", quant=scheme)
    w_dec = _effective_weights(hip, mh, scheme, exact_scales=True)
    w_pre = _effective_weights(hip, mh, scheme, exact_scales=False)
    w_pre["lm_head"] = w_dec["lm_head"]     # the head of a many-row call runs on B rows: the decode kernel
    rope = _rope(cfg)
    st = Stages(hip, cfg, mh)
    pre, dec = MinistralRoundingModel(cfg, w_pre, rope), MinistralRoundingModel(cfg, w_dec, rope)
    # 128 rows: the traces of the eight sequences stacked (the linear stages do not mix rows)
    traces, caches, lasts = [], [], []
    for b in range(B):
        pre.trace = {}
        cm = [None]
        lasts.append(pre.forward(prompts[b], 0, cm))
        traces.append(pre.trace)
        caches.append(cm)
    stacked = {k: np.concatenate([t[k] for t in traces], axis=0) for k in traces[0]}
    x = np.concatenate([w_pre["tok_embeddings.weight"][np.asarray(p)] for p in prompts], axis=0)
    print(f"{scheme}, 128 rows:")
    head_rows = [b * T + T - 1 for b in range(B)]
    logits, up = _check_stages(st, stacked, x, 0, lambda s, c: rope(0, 1), None, head_rows, skip_attention=True)
    _same_f32("final norm + head", logits, np.concatenate(lasts, axis=0), upstream=up)
    # 8 rows: one decode step of every sequence
    toks = [int(np.argmax(l[-1])) for l in lasts]
    traces, wants = [], []
    for b in range(B):
        dec.trace = {}
        wants.append(dec.forward([toks[b]], T, caches[b]))
        traces.append(dec.trace)
    stacked = {k: np.concatenate([t[k] for t in traces], axis=0) for k in traces[0]}
    x = w_dec["tok_embeddings.weight"][np.asarray(toks)]
    print(f"{scheme}, 8 rows:")
    logits, up = _check_stages(st, stacked, x, T, lambda s, c: rope(T, 1), None, list(range(B)), skip_attention=True)
    _same_f32("final norm + head", logits, np.concatenate(wants, axis=0), upstream=up)


# ------------------------------------------------------------------------------------------------ (c)
@pytest.mark.parametrize("layers,prompt_len", [(1, 8), (4, 8), (1, 1024), (4, 1024)])
def test_whole_model_distance_is_the_rounding(hip, layers, prompt_len):
    """Logits of the whole program, as statistics (see the module text for why they cannot be tighter)."""
    cfg = models.MinistralConfig(num_layers=layers, **FULL)
    prompt = np.random.default_rng(6).integers(0, cfg.vocab_size, prompt_len).tolist()
    mh = models.Ministral.random(cfg, hip, seed=5, dtype="Bf16", residual_dtype="F32")
    w = {n: hip.to_numpy(mh.param_handle(n)).astype(np.float32) for n in mh.param_names}
    rm = MinistralRoundingModel(cfg, w, _rope(cfg), rounding=True)
    exact = MinistralRoundingModel(cfg, w, _rope(cfg), rounding=False)
    steps, cap = 3, (16 if prompt_len == 8 else 1280)
    all_rows = prompt_len == 8
    cm, ce = [None] * layers, [None] * layers
    model_rows = [rm.forward(prompt, 0, cm, last_row_only=not all_rows)]
    exact_rows = [exact.forward(prompt, 0, ce, last_row_only=not all_rows)]
    toks = []
    for s in range(steps):
        toks.append(int(np.argmax(model_rows[-1][-1])))
        model_rows.append(rm.forward([toks[-1]], prompt_len + s, cm))
        exact_rows.append(exact.forward([toks[-1]], prompt_len + s, ce))
    del exact, ce
    rounding = [_err(f"{layers} layer(s), prompt {prompt_len}, row {i} | rounding model vs the model without rounding", r, e)
                for i, (r, e) in enumerate(zip(model_rows, exact_rows))]
    for chain in (1, 0):
        with option(hip, "chain", chain):
            ch = [None] * layers
            before = hip.counter("chain_launches")
            rows = [hip.to_numpy(mh.forward_with_decode_cache(prompt, 0, ch, cap, last_logits_only=not all_rows))]
            for s in range(steps):
                rows.append(hip.to_numpy(mh.forward_with_decode_cache([toks[s]], prompt_len + s, ch, cap)))
            assert (hip.counter("chain_launches") > before) == bool(chain)
        kc, vc = hip.to_numpy(ch[0].keys)[:, :prompt_len + steps], hip.to_numpy(ch[0].values)[:, :prompt_len + steps]
        # layer 0 sees identical inputs on both sides: its cache rows are the model's but for stray ties
        assert np.mean(kc != cm[0][0]) < 2e-3 and np.mean(vc != cm[0][1]) < 2e-3
        for i, (g, r) in enumerate(zip(rows, model_rows)):
            what = f"{layers} layer(s), prompt {prompt_len}, chain={chain}, {'prefill' if i == 0 else 'decode step %d' % i}"
            mx, mean = _err(what + " | device vs rounding model", g, r)
            # two correct bf16 pipelines: no further apart than the pipeline is from exact arithmetic
            assert mean <= 1.1 * rounding[i][1] and mx <= 1.5 * rounding[i][0], what
            mx_e, mean_e = _err(what + " | device vs the model without rounding", g, exact_rows[i])
            assert mean_e <= 1.25 * rounding[i][1], what


