"""GPU parity of the persistent decode chain (one launch for a run of M = 1 bf16 linears and decode
attentions) against the CPU oracle, at the widths of the Ministral-3B-shaped decoder: several
words per lane and tile (K 3072..9216), several units per workgroup, RMSNorm prologue, SwiGLU pair,
bias + exact GELU, residual, and chains of dependent phases.

Reference: the oracle run in F32 on the same bf16-representable inputs (the reference's CPU backends
execute f32 only).  The chain keeps f32 inside a linear and rounds its output to bf16 once; the
per-op-rounded bf16 oracle is further away from f32 than the chain is (its RMSNorm scale alone is
rounded to 8 bits), so it is not the yardstick here.

Tolerances against the f32 oracle: rtol = 2^-8 (the one bf16 rounding of the result: half an ulp is
2^-9 .. 2^-8 of the value, depending on where in its binade it lies) plus an absolute term for the
inputs the kernel itself rounds to bf16 on the way (the normalised row, the intermediate vectors of a
multi-phase chain): about 4 sigma of the sum of K independent roundings, stated per test.  Against the
one-kernel-per-linear path of the same backend, whose rounding points are the same, only the f32
summation order differs, which now and then moves a result across a rounding boundary: one ulp,
rtol 2^-7, with a far smaller absolute term, which a dropped or doubled weight word (2 of K products)
exceeds."""
import numpy as np
import pytest

from parity import FunctionBuilder, Program, assert_close, hip_run, oracle_run
from gptrs_amd import functional as F
from gptrs_amd.ptir import f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def rnd(seed, shape, scale=1.0):
    return (np.random.default_rng(seed).uniform(-1.0, 1.0, size=shape) * scale).astype(np.float32)


def prog(build, param_specs):
    fb = FunctionBuilder("main")
    params = [fb.param(dt, dims) for dt, dims in param_specs]
    res = build(fb, *params)
    fb.set_results(list(res) if isinstance(res, (list, tuple)) else [res])
    return Program(fb)


def bf16_round(a):
    return (f32_to_bf16_bits(np.asarray(a, np.float32)).astype(np.uint32) << 16).view(np.float32)


HALF_ULP = 2.0 ** -8   # largest relative size of half a bf16 ulp: one rounding of an exact value
ULP = 2.0 ** -7        # largest relative size of one bf16 ulp: two roundings of nearly equal values


def _report(what, g, w):
    g, w = np.asarray(g, np.float64), np.asarray(w, np.float64)
    d = np.abs(g - w)
    print(f"{what}: max abs {d.max():.3e}, max beyond {HALF_ULP:.1e} rel {np.max(d - HALF_ULP * np.maximum(np.abs(g), np.abs(w))):.3e}, max |ref| {np.abs(w).max():.2f}")


def run_both(hip, build, specs, arrays, atol, atol_self, rtol=HALF_ULP):
    """chain on vs the f32 oracle, and chain on vs chain off (same backend, one kernel per linear)."""
    p = prog(build, [("Bf16", d) for d in specs])
    before = hip.counter("chain_launches")
    got = hip_run(hip, p, arrays)
    assert hip.counter("chain_launches") > before, "the program did not take the chain path"
    want = oracle_run(prog(build, [("F32", d) for d in specs]), [bf16_round(a) for a in arrays])
    hip.set_option("chain", 0)
    try:
        plain = hip_run(hip, p, arrays)
    finally:
        hip.set_option("chain", 1)
    for i, (g, w, q) in enumerate(zip(got, want, plain)):
        _report(f"result {i} vs oracle", g, w)
        _report(f"result {i} vs per-linear kernels", g, q)
        assert_close(g, w, atol=atol, rtol=rtol, what=f"result {i} vs oracle")
        assert_close(g, q, atol=atol_self, rtol=ULP, what=f"result {i} vs per-linear kernels")


@pytest.mark.parametrize("k,n", [(3072, 6144), (4096, 3072), (9216, 3072), (3072, 1000), (512, 40), (64, 12), (3072, 1001), (512, 41), (64, 13), (128, 7)])
def test_single_linear(hip, k, n):
    x, w = rnd(1, (1, k)), rnd(2, (k, n), 2.0 / np.sqrt(k))
    # inputs are exact in bf16: the result is the f32 dot rounded once
    run_both(hip, lambda fb, a, b: a.matmul(b), [[1, k], [k, n]], [x, w], 2e-5, 2e-5)


@pytest.mark.parametrize("k,n", [(3072, 6144), (1024, 256)])
def test_norm_linear(hip, k, n):
    x, g, w = rnd(3, (1, k), 3.0), rnd(4, (k,)) + 1.5, rnd(5, (k, n), 2.0 / np.sqrt(k))
    # the normalised row (|v| up to 4.3, rms 2) is rounded to bf16 as it is staged: K roundings of relative 2^-9 against
    # weights of rms 1.15 / sqrt(K) move a result by 3e-3 (sigma)
    run_both(hip, lambda fb, a, gm, b: F.rms_norm(a, gm, 1e-5)[0].matmul(b), [[1, k], [k], [k, n]], [x, g, w], 2e-2, 2e-3)


@pytest.mark.parametrize("k,n", [(3072, 9216), (256, 96)])
def test_swiglu_pair(hip, k, n):
    x, g = rnd(6, (1, k), 3.0), rnd(7, (k,)) + 1.5
    wg, wu = rnd(8, (k, n), 2.0 / np.sqrt(k)), rnd(9, (k, n), 2.0 / np.sqrt(k))

    def build(fb, a, gm, b, c):
        h = F.rms_norm(a, gm, 1e-5)[0]
        return F.swiglu(h.matmul(b), h.matmul(c))

    # as above for gate and up; silu(g) * u multiplies the effect by the other factor (|u|, |silu'| up to 7: results up
    # to 41), so it enters relative to the result as well
    run_both(hip, build, [[1, k], [k], [k, n], [k, n]], [x, g, wg, wu], 3e-2, 4e-3, rtol=ULP)


@pytest.mark.parametrize("k,n", [(9216, 3072), (768, 3072), (128, 64)])
def test_bias_gelu_residual(hip, k, n):
    x, w, b, r = rnd(10, (1, k)), rnd(11, (k, n), 2.0 / np.sqrt(k)), rnd(12, (n,)), rnd(13, (1, n))
    # the scalar literals of a bf16 program are bf16: its GELU divides by bf16(sqrt 2) = 1.4140625, which the linear kernel's
    # exact-erf epilogue (1.41421354) does not serve, so the GELU runs as its own kernel and the result carries three
    # roundings (linear + bias, GELU, residual add) against the f32 oracle's none
    run_both(hip, lambda fb, a, c, d, e: F.gelu(F.linear(a, c, d)) + e, [[1, k], [k, n], [n], [1, n]], [x, w, b, r], 2.5e-2, 2e-5)
    # bias and residual alone are absorbed: the f32 sum + bias + residual, rounded once
    run_both(hip, lambda fb, a, c, d, e: F.linear(a, c, d) + e, [[1, k], [k, n], [n], [1, n]], [x, w, b, r], 2e-5, 2e-5)


@pytest.mark.parametrize("d,f", [(3072, 9216), (256, 640)])
def test_block_tail_chain(hip, d, f):
    """out-proj (+residual) -> RMSNorm -> gate/up SwiGLU -> down (+residual) -> RMSNorm -> next
    projection: five dependent phases in one launch (model/ministral.rs:166-201)."""
    qp = d + d // 3 // 4 * 4
    ctx, x = rnd(20, (1, qp)), rnd(21, (1, d))
    wo, wg, wu = rnd(22, (qp, d), 2.0 / np.sqrt(qp)), rnd(23, (d, f), 2.0 / np.sqrt(d)), rnd(24, (d, f), 2.0 / np.sqrt(d))
    wd, wq = rnd(25, (f, d), 2.0 / np.sqrt(f)), rnd(26, (d, 2 * d), 2.0 / np.sqrt(d))
    g1, g2 = rnd(27, (d,)) + 1.5, rnd(28, (d,)) + 1.5

    def build(fb, c, xx, a_wo, a_wg, a_wu, a_wd, a_wq, a_g1, a_g2):
        h = c.matmul(a_wo) + xx
        n1 = F.rms_norm(h, a_g1, 1e-5)[0]
        ff = F.swiglu(n1.matmul(a_wg), n1.matmul(a_wu)).matmul(a_wd) + h
        return [F.rms_norm(ff, a_g2, 1e-5)[0].matmul(a_wq), ff]

    specs = [[1, qp], [1, d], [qp, d], [d, f], [d, f], [f, d], [d, 2 * d], [d], [d]]
    before = hip.counter("chain_phases")
    # four vectors are rounded to bf16 between the phases (h, the SwiGLU output, ff, the normalised rows)
    run_both(hip, build, specs, [ctx, x, wo, wg, wu, wd, wq, g1, g2], 6e-2, 1e-3)
    assert hip.counter("chain_phases") - before >= 4


@pytest.mark.parametrize("hq,hkv,dh,rope,cap", [(8, 2, 128, True, 2048), (4, 4, 64, False, 2048), (8, 1, 128, True, 2048), (4, 2, 256, False, 2048),
                                                (8, 2, 128, True, 128), (4, 4, 64, False, 96)])
def test_decode_attention_in_chain(hip, hq, hkv, dh, rope, cap):
    """projection -> (RoPE) -> attention_decode_cache -> out-projection as ONE launch: the attention takes
    two phases of the chain (per-chunk online softmax, then the merge).  Positions cover an empty cache,
    fewer positions than chunks, chunk boundaries, more positions per lane group than are requested
    ahead of the barrier, and the last slot; the updated caches must match as well (bit-exact when no
    RoPE touches the appended row)."""
    d = 256
    cfg = F.AttentionConfig(embed_dim=d, num_query_heads=hq, num_key_value_heads=hkv, head_dim=dh)
    tp, qp = cfg.total_projection_dim, cfg.query_projection_dim
    rcfg = F.RopeConfig(rotary_dim=dh, theta=10000.0) if rope else None
    x = rnd(30, (1, d))
    wqkv, wo = rnd(31, (d, tp), 2.0 / np.sqrt(d)), rnd(32, (qp, d), 2.0 / np.sqrt(qp))
    kc, vc = rnd(33, (hkv, cap, dh)), rnd(34, (hkv, cap, dh))

    def build(fb, a, w1, w2, k, v, us, qs, *cs):
        qkv = a.matmul(w1)
        if cs:
            qkv = F.apply_rope_qkv_packed(cfg, qkv, cs[0], cs[1])
        c, k2, v2 = F.attention_decode_cache(cfg, qkv, k, v, us, qs)
        return [c.matmul(w2), k2, v2]

    fspecs = [[1, d], [d, tp], [qp, d], [hkv, cap, dh], [hkv, cap, dh]]
    for pos in sorted({0, 5, 31, 32, min(100, cap - 2), (3 * cap) // 4, cap - 1}):
        us, qs = np.array([0, pos, 0], np.int32), np.array([pos], np.int32)
        arrays, ispecs = [x, wqkv, wo, kc, vc], [("Si32", [3]), ("Si32", [1])]
        extra, especs = [], []
        if rope:
            cos, sin = F.rotary_cos_sin_cache_slice(pos, 1, rcfg)
            extra, especs = [cos, sin], [list(cos.shape), list(sin.shape)]
        pb = prog(build, [("Bf16", s) for s in fspecs] + ispecs + [("Bf16", s) for s in especs])
        pf = prog(build, [("F32", s) for s in fspecs] + ispecs + [("F32", s) for s in especs])
        before = hip.counter("chain_phases")
        got = hip_run(hip, pb, arrays + [us, qs] + extra)
        # (a cache of at most 128 positions is one chunk per kv head: the attention is then one phase)
        assert hip.counter("chain_phases") - before == (3 if cap <= 128 else 4), "projection, attention and out-projection must share one launch"
        want = oracle_run(pf, [bf16_round(a) for a in arrays] + [us, qs] + [bf16_round(a) for a in extra])
        assert_close(got[0], want[0], atol=3e-2, rtol=2e-2, what=f"context projection at pos {pos}")
        for i in (1, 2):
            g, w = np.asarray(got[i], np.float32), np.asarray(want[i], np.float32)
            mask = np.ones(cap, bool)
            mask[pos] = False
            assert np.array_equal(g[:, mask], w[:, mask]), "cache rows other than the appended one must be untouched"
            assert_close(g[:, pos], w[:, pos], atol=2e-2, rtol=2e-2, what=f"appended row of cache {i} at pos {pos}")


def test_grid_barrier_gives_up_and_the_backend_goes_on(hip):
    """A grid barrier that cannot complete must end in an execution error, not in a hang: the host option
    "chain_stall_phase" makes every workgroup of the next launch expect one arrival more than the grid can deliver at that
    phase's barrier, so each control wave runs out of its (wall-clock) budget, raises the abort flag, and every wave leaves
    the kernel.  The error is reported at the next synchronisation; the launch after it runs the chain again and is right."""
    from gptrs_amd.backend import BackendError
    k = 1024
    x = rnd(60, (1, k))
    ws = [rnd(61 + i, (k, k), 2.0 / np.sqrt(k)) for i in range(3)]

    def build(fb, a, w0, w1, w2):
        return a.matmul(w0).matmul(w1).matmul(w2)

    specs = [[1, k]] + [[k, k]] * 3
    p = prog(build, [("Bf16", d) for d in specs])
    good = hip_run(hip, p, [x] + ws)[0]
    hip.set_option("chain_stall_phase", 1)
    launches = hip.counter("chain_launches")
    with pytest.raises(BackendError, match="grid barrier timed out"):
        hip_run(hip, p, [x] + ws)
    assert hip.counter("chain_launches") == launches + 1, "the stalled program must have taken the chain path"
    # the stall applies to one launch; the barrier counters were reset with the error
    before = hip.counter("chain_launches")
    again = hip_run(hip, p, [x] + ws)[0]
    assert hip.counter("chain_launches") == before + 1, "the chain must still be in use after a requested stall"
    assert np.array_equal(np.asarray(again), np.asarray(good))
    # phase 0 has no barrier to stall at: the value is refused instead of staying armed for ever
    with pytest.raises(BackendError):
        hip.set_option("chain_stall_phase", 0)
    # a stall that is armed while only one-phase launches run is consumed by the first launch that has a barrier, and
    # a launch without one runs normally meanwhile
    one = prog(lambda fb, a, w0: a.matmul(w0), [("Bf16", [1, k]), ("Bf16", [k, k])])
    want_one = hip_run(hip, one, [x, ws[0]])[0]
    hip.set_option("chain_stall_phase", 2)
    assert np.array_equal(np.asarray(hip_run(hip, one, [x, ws[0]])[0]), np.asarray(want_one))
    with pytest.raises(BackendError, match="a stall was requested"):
        hip_run(hip, p, [x] + ws)
    assert np.array_equal(np.asarray(hip_run(hip, p, [x] + ws)[0]), np.asarray(good))


@pytest.mark.parametrize("k,n", [(2560, 32768), (1536, 32768), (3072, 32776), (200, 4100)])
def test_padded_steps_and_missing_tiles_are_stable(hip, k, n):
    """Shapes whose tile streams end inside a j-step (K = 2560, 1536: the last step's upper waves hold nothing but padding;
    K = 200: a wave that is partly padding) or whose last unit lacks tiles (N = 32776 -> 8194 tiles = 2731 units + 1 tile;
    N = 4100 -> 1025 tiles), run many times: a wave asks for weights several steps ahead and tells by the count of its loads
    in flight which step has landed, which holds only while every load it issues returns in order.  (Loads that re-read
    cached words in place of padding did not, and whole units came out wrong now and then.)"""
    x, w = rnd(70, (1, k)), rnd(71, (k, n), 2.0 / np.sqrt(k))
    p = prog(lambda fb, a, b: a.matmul(b), [("Bf16", [1, k]), ("Bf16", [k, n])])
    hip.set_option("chain", 0)
    try:
        plain = np.asarray(hip_run(hip, p, [x, w])[0], np.float32)
    finally:
        hip.set_option("chain", 1)
    before = hip.counter("chain_launches")
    for rep in range(25):
        got = np.asarray(hip_run(hip, p, [x, w])[0], np.float32)
        assert_close(got, plain, atol=2e-5, rtol=ULP, what=f"run {rep} vs per-linear kernel")
    assert hip.counter("chain_launches") == before + 25


# ------------------------------------------------------------------------------ f32 phases (GPT-2)
def run_both_f32(hip, build, specs, arrays, atol=5e-4, rtol=1e-4, phases=1):
    """f32 program: chain on vs the oracle and vs chain off (the reference suite's f32 bar, 5e-4 + 1e-4 relative:
    only the order of the f32 sums differs)."""
    p = prog(build, [("F32", d) for d in specs])
    hip.set_option("chain_f32_min_kb", 0)   # (by default f32 phases that stream little keep their stand-alone kernels)
    try:
        before, ph0 = hip.counter("chain_launches"), hip.counter("chain_phases")
        got = hip_run(hip, p, arrays)
        assert hip.counter("chain_launches") > before, "the program did not take the chain path"
        assert hip.counter("chain_phases") - ph0 >= phases
    finally:
        hip.set_option("chain_f32_min_kb", 4096)
    want = oracle_run(p, arrays)
    hip.set_option("chain", 0)
    try:
        plain = hip_run(hip, p, arrays)
    finally:
        hip.set_option("chain", 1)
    for i, (g, w, q) in enumerate(zip(got, want, plain)):
        assert np.asarray(g).dtype == np.float32
        assert_close(g, w, atol=atol, rtol=rtol, what=f"result {i} vs oracle")
        assert_close(g, q, atol=atol, rtol=rtol, what=f"result {i} vs per-linear kernels")


@pytest.mark.parametrize("k,n", [(768, 2304), (768, 3072), (3072, 768), (768, 768), (200, 52), (4608, 64), (64, 12), (768, 50257), (200, 53), (64, 14), (64, 5)])
def test_f32_single_linear(hip, k, n):
    x, w = rnd(31, (1, k)), rnd(32, (k, n), 2.0 / np.sqrt(k))
    run_both_f32(hip, lambda fb, a, b: a.matmul(b), [[1, k], [k, n]], [x, w])


@pytest.mark.parametrize("k,n", [(768, 2304), (3072, 768), (100, 40)])
def test_f32_layer_norm_linear_bias(hip, k, n):
    x, g, bt = rnd(33, (1, k), 3.0) + 0.7, rnd(34, (k,)) + 1.5, rnd(35, (k,))
    w, b = rnd(36, (k, n), 2.0 / np.sqrt(k)), rnd(37, (n,))
    run_both_f32(hip, lambda fb, a, gm, be, c, d: F.linear(F.layer_norm(a, gm, be, 1e-5)[0], c, d),
                 [[1, k], [k], [k], [k, n], [n]], [x, g, bt, w, b])


@pytest.mark.parametrize("k,n", [(768, 3072), (3072, 768), (128, 64)])
def test_f32_bias_gelu_residual(hip, k, n):
    x, w, b, r = rnd(38, (1, k)), rnd(39, (k, n), 2.0 / np.sqrt(k)), rnd(40, (n,)), rnd(41, (1, n))
    run_both_f32(hip, lambda fb, a, c, d, e: F.gelu(F.linear(a, c, d)) + e, [[1, k], [k, n], [n], [1, n]], [x, w, b, r])
    run_both_f32(hip, lambda fb, a, c, d, e: F.linear(a, c, d) + e, [[1, k], [k, n], [n], [1, n]], [x, w, b, r])


@pytest.mark.parametrize("d", [768, 96])
def test_f32_block_tail_chain(hip, d):
    """out-proj (+bias, +residual) -> LayerNorm -> fc (+bias, GELU) -> proj (+bias, +residual) -> LayerNorm -> next qkv
    (+bias): the linears of a GPT-2 block behind its attention (model/gpt.rs:585-751), four dependent phases."""
    f = 4 * d
    ctx, x = rnd(50, (1, d)), rnd(51, (1, d))
    wo, bo = rnd(52, (d, d), 2.0 / np.sqrt(d)), rnd(53, (d,))
    wf, bf = rnd(54, (d, f), 2.0 / np.sqrt(d)), rnd(55, (f,))
    wp, bp = rnd(56, (f, d), 2.0 / np.sqrt(f)), rnd(57, (d,))
    wq, bq = rnd(58, (d, 3 * d), 2.0 / np.sqrt(d)), rnd(59, (3 * d,))
    g1, b1, g2, b2 = rnd(60, (d,)) + 1.5, rnd(61, (d,)), rnd(62, (d,)) + 1.5, rnd(63, (d,))

    def build(fb, c, xx, a_wo, a_bo, a_wf, a_bf, a_wp, a_bp, a_wq, a_bq, a_g1, a_b1, a_g2, a_b2):
        h = F.linear(c, a_wo, a_bo) + xx
        m = F.gelu(F.linear(F.layer_norm(h, a_g1, a_b1, 1e-5)[0], a_wf, a_bf))
        out = F.linear(m, a_wp, a_bp) + h
        return [F.linear(F.layer_norm(out, a_g2, a_b2, 1e-5)[0], a_wq, a_bq), out]

    specs = [[1, d], [1, d], [d, d], [d], [d, f], [f], [f, d], [d], [d, 3 * d], [3 * d], [d], [d], [d], [d]]
    run_both_f32(hip, build, specs, [ctx, x, wo, bo, wf, bf, wp, bp, wq, bq, g1, b1, g2, b2], atol=2e-3, rtol=1e-3, phases=4)


def test_f32_phases_that_stream_little_keep_their_kernels(hip):
    """The default policy: f32 linears join a persistent launch from 4 MiB of weights each on average."""
    x = rnd(80, (1, 768))
    small, big = rnd(81, (768, 768), 0.05), rnd(82, (768, 4096), 0.05)
    p_small = prog(lambda fb, a, b: a.matmul(b), [("F32", [1, 768]), ("F32", [768, 768])])
    p_big = prog(lambda fb, a, b: a.matmul(b), [("F32", [1, 768]), ("F32", [768, 4096])])
    before = hip.counter("chain_launches")
    hip_run(hip, p_small, [x, small])
    assert hip.counter("chain_launches") == before, "2.4 MB of f32 weights: stand-alone kernel"
    hip_run(hip, p_big, [x, big])
    assert hip.counter("chain_launches") == before + 1, "12.6 MB of f32 weights: persistent launch"


@pytest.mark.parametrize("hq,hkv,dh,cap", [(12, 12, 64, 128), (4, 4, 64, 1024), (8, 2, 128, 2048), (4, 1, 256, 256)])
def test_f32_decode_attention_in_chain(hip, hq, hkv, dh, cap):
    """f32 projection (+bias) -> attention_decode_cache over f32 caches -> out-projection (+bias) as ONE launch (the
    attention of a GPT-2 block, model/gpt.rs:585-751): context to the f32 bar against the oracle and against the
    stand-alone kernels, caches exact but for the appended row, which is a copy of the projection's output."""
    d = 192
    cfg = F.AttentionConfig(embed_dim=d, num_query_heads=hq, num_key_value_heads=hkv, head_dim=dh)
    tp, qp = cfg.total_projection_dim, cfg.query_projection_dim
    x = rnd(70, (1, d))
    wqkv, bqkv = rnd(71, (d, tp), 2.0 / np.sqrt(d)), rnd(72, (tp,))
    wo, bo = rnd(73, (qp, d), 2.0 / np.sqrt(qp)), rnd(74, (d,))
    kc, vc = rnd(75, (hkv, cap, dh)), rnd(76, (hkv, cap, dh))

    def build(fb, a, w1, b1, w2, b2, k, v, us, qs):
        c, k2, v2 = F.attention_decode_cache(cfg, F.linear(a, w1, b1), k, v, us, qs)
        return [F.linear(c, w2, b2), k2, v2]

    specs = [("F32", s) for s in [[1, d], [d, tp], [tp], [qp, d], [d], [hkv, cap, dh], [hkv, cap, dh]]] + [("Si32", [3]), ("Si32", [1])]
    p = prog(build, specs)
    for pos in sorted({0, 5, 31, 32, 100, cap // 2, cap - 1}):
        us, qs = np.array([0, pos, 0], np.int32), np.array([pos], np.int32)
        arrays = [x, wqkv, bqkv, wo, bo, kc, vc, us, qs]
        hip.set_option("chain_f32_min_kb", 0)
        try:
            before = hip.counter("chain_phases")
            got = hip_run(hip, p, arrays)
        finally:
            hip.set_option("chain_f32_min_kb", 4096)
        # a cache of at most 128 positions is one chunk per kv head: the attention is one phase
        assert hip.counter("chain_phases") - before == (3 if cap <= 128 else 4), "projection, attention and out-projection must share one launch"
        want = oracle_run(p, arrays)
        hip.set_option("chain", 0)
        try:
            plain = hip_run(hip, p, arrays)
        finally:
            hip.set_option("chain", 1)
        assert_close(got[0], want[0], atol=5e-4, rtol=1e-4, what=f"context projection at pos {pos}")
        assert_close(got[0], plain[0], atol=5e-4, rtol=1e-4, what=f"context projection at pos {pos} vs stand-alone kernels")
        for i in (1, 2):
            g, w = np.asarray(got[i]), np.asarray(want[i])
            mask = np.ones(cap, bool)
            mask[pos] = False
            assert np.array_equal(g[:, mask], w[:, mask]), "cache rows other than the appended one must be untouched"
            assert_close(g[:, pos], w[:, pos], atol=5e-4, rtol=1e-4, what=f"appended row of cache {i} at pos {pos}")
            assert np.array_equal(g[:, pos], np.asarray(plain[i])[:, pos]) or np.allclose(g[:, pos], np.asarray(plain[i])[:, pos], atol=5e-4)
