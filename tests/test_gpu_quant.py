"""GPU parity of the weight-only quantisation extension (int8 per output column, int4 in groups of 128).

The reference has no quantisation scheme (docs/backend.md:620-632 leaves Quantize/Dequantize
backend-defined, ref-cpu answers Unimplemented), so the yardstick is the oracle's closed form of the
scheme this build defines: codes and scales must match it bit for bit, and a quantised linear must match
"dequantise, then dot_general" as the oracle computes it, on every execution path of the backend (the
persistent decode chain for one bf16 row, the matrix-core kernels over the codes for 2..16 rows and for
prefill-sized inputs, the generic kernels otherwise), alone and under the epilogues the fusion pass folds into it."""
import numpy as np
import pytest

from parity import FunctionBuilder, Program, assert_close, hip_run, oracle_run, po
from gptrs_amd import functional as F
from gptrs_amd.ptir import f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def rnd(seed, shape, scale=1.0):
    return (np.random.default_rng(seed).uniform(-1.0, 1.0, size=shape) * scale).astype(np.float32)


def bf16_round(a):
    return (f32_to_bf16_bits(np.asarray(a, np.float32)).astype(np.uint32) << 16).view(np.float32)


def prog(build, param_specs):
    fb = FunctionBuilder("main")
    params = [fb.param(dt, dims) for dt, dims in param_specs]
    res = build(fb, *params)
    fb.set_results(list(res) if isinstance(res, (list, tuple)) else [res])
    return Program(fb)


def quantize(w, scheme):
    q, s = (po.quantize_int8_per_channel if scheme == "w8" else po.quantize_int4_g128)(w)
    return q, s


def code_spec(scheme, k, n):
    return ("Si8", [k, n]) if scheme == "w8" else ("Ui8", [k // 2, n])


def scale_dims(scheme, k, n):
    return [n] if scheme == "w8" else [k // 128, n]


# ---------------------------------------------------------------------------------- packing
def weights_with_corner_cases(seed, k, n):
    w = rnd(seed, (k, n), 0.05)
    w[:, 0] = 0.0                                   # all-zero column: scale 1, codes 0
    w[:, 1] = np.float32(0.001) * np.arange(k)      # monotone ramp: every code value appears
    w[::2, 2] *= -1.0
    if n > 3:                                       # ties: w / s exactly on .5 for s = 1/128
        w[:, 3] = (np.arange(k) % 254 - 127 + 0.5).astype(np.float32) / 128.0
    return w


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("scheme,k,n", [("w8", 96, 40), ("w8", 1024, 257), ("w4g128", 128, 8), ("w4g128", 512, 130)])
def test_codes_and_scales_bit_exact(hip, dtype, scheme, k, n):
    w = weights_with_corner_cases(40, k, n)
    if dtype == "Bf16":
        w = bf16_round(w)
    p = prog(lambda fb, a: list(F.quantize_weight(a, scheme)), [(dtype, [k, n])])
    q, s = hip_run(hip, p, [w])
    q_ref, s_ref = quantize(w, scheme)
    assert np.array_equal(np.asarray(s, np.float32), s_ref), "scales differ from the closed form"
    assert np.array_equal(q, q_ref), "codes differ from the closed form"
    oq, os_ = oracle_run(p, [w])
    assert np.array_equal(q, oq) and np.array_equal(np.asarray(s, np.float32), os_)


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("scheme,k,n", [("w8", 96, 40), ("w4g128", 256, 36)])
def test_dequantize_exact(hip, dtype, scheme, k, n):
    q, s = quantize(rnd(41, (k, n), 0.05), scheme)
    cs = code_spec(scheme, k, n)
    p = prog(lambda fb, a, b: F.dequantize_weight(a, b), [cs, (dtype, scale_dims(scheme, k, n))])
    (got,) = hip_run(hip, p, [q, s])
    (want,) = oracle_run(p, [q, s])
    assert np.array_equal(np.asarray(got, np.float32), want)


# ---------------------------------------------------------------------------------- linears
def run_linear(hip, build, specs, arrays, atol, rtol, expect_chain=None):
    """HIP (fusion on and off) against the oracle on the same program and inputs."""
    p = prog(build, specs)
    want = oracle_run(p, arrays)
    before = hip.counter("chain_launches")
    got = hip_run(hip, p, arrays)
    took_chain = hip.counter("chain_launches") > before
    if expect_chain is not None:
        assert took_chain == expect_chain, f"chain path taken: {took_chain}, expected {expect_chain}"
    hip.set_option("fusion", 0)
    try:
        plain = hip_run(hip, p, arrays)
    finally:
        hip.set_option("fusion", 1)
    for i, (g, w, q) in enumerate(zip(got, want, plain)):
        assert_close(g, w, atol=atol, rtol=rtol, what=f"result {i} vs oracle")
        assert_close(q, w, atol=atol, rtol=rtol, what=f"result {i} (fusion off) vs oracle")
    return took_chain


SHAPES = [(3072, 6144), (4096, 3072), (9216, 3072), (3072, 1000), (512, 40), (128, 12)]


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("k,n", SHAPES)
def test_decode_linear_bf16(hip, scheme, k, n):
    """One bf16 row: the persistent chain reads the codes directly."""
    x, w = bf16_round(rnd(1, (1, k))), rnd(2, (k, n), 2.0 / np.sqrt(k))
    q, s = quantize(w, scheme)
    specs = [("Bf16", [1, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))]
    run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x, q, s], 2e-2, 2e-2, expect_chain=True)


@pytest.mark.parametrize("scheme,k,n", [("w8", 3072, 32768), ("w4g128", 3072, 32768), ("w4g128", 2048, 155648)])
def test_decode_linear_wide(hip, scheme, k, n):
    """Vocabulary-sized outputs: many units per workgroup, and (last case) more int4 group scales per workgroup
    than one round of the cooperative staging loads."""
    x = bf16_round(rnd(14, (1, k)))
    w = np.random.default_rng(15).standard_normal((k, n), dtype=np.float32)
    w *= np.float32(0.02)
    q, s = quantize(w, scheme)
    del w
    specs = [("Bf16", [1, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))]
    p = prog(lambda fb, a, b, c: F.linear_quantized(a, b, c), specs)
    (want,) = oracle_run(p, [x, q, s])
    before = hip.counter("chain_launches")
    (got,) = hip_run(hip, p, [x, q, s])
    assert hip.counter("chain_launches") > before
    assert_close(got, want, atol=2e-2, rtol=2e-2, what="wide quantised decode linear")


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m,k,n", [(1, 256, 96), (5, 384, 40), (64, 512, 256), (200, 1024, 384)])
def test_linear_f32(hip, scheme, m, k, n):
    """f32 activations: dequantise + generic kernels; the reference suite's tolerance."""
    x, w = rnd(3, (m, k)), rnd(4, (k, n), 2.0 / np.sqrt(k))
    q, s = quantize(w, scheme)
    specs = [("F32", [m, k]), code_spec(scheme, k, n), ("F32", scale_dims(scheme, k, n))]
    run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x, q, s], 5e-4, 1e-4, expect_chain=False)


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m,k,n", [(128, 3072, 1024), (64, 512, 256), (7, 384, 40)])
def test_prefill_linear_bf16(hip, scheme, m, k, n):
    """Several bf16 rows: the MFMA GEMM over the k-grouped codes where it applies."""
    x, w = bf16_round(rnd(5, (m, k))), rnd(6, (k, n), 2.0 / np.sqrt(k))
    q, s = quantize(w, scheme)
    specs = [("Bf16", [m, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))]
    run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x, q, s], 3e-2, 2e-2, expect_chain=False)


def dequantize_host(q, s, scheme):
    """bf16(code * scale), the dequantiser's value (one f32 product, rounded to nearest even)."""
    if scheme == "w8":
        return bf16_round(q.astype(np.float32) * s.astype(np.float32)[None, :])
    lo = (q & 0xF).astype(np.int32)
    hi = (q >> 4).astype(np.int32)
    lo[lo > 7] -= 16
    hi[hi > 7] -= 16
    codes = np.empty((2 * q.shape[0], q.shape[1]), np.float32)
    codes[0::2], codes[1::2] = lo, hi
    return bf16_round(codes * np.repeat(s.astype(np.float32), 128, axis=0))


# 64 x 64 tiles (fewer than 128 tiles of 128 x 128): (128, 3072, 1024), (300, 1024, 3000), (17, 256, 40), (1024, 512, 200).
# 8-wave workgroups that split every tile's k-steps (128..256 tiles): (1024, 1024, 2048).  Tail split with tickets: 304
# tiles, the last 48 split four ways over 18 k tiles, so the second and fourth splits start in the middle of an int4
# scale group: (1024, 1152, 4860).  Plain 128 x 128 tiles, 512 of them: (1024, 3072, 8192).  Tail split at the
# gate / up / down width: (1024, 3072, 9216).
@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m,k,n", [(128, 3072, 1024), (300, 1024, 3000), (17, 256, 40), (1024, 512, 200),
                                   (1024, 1024, 2048), (1024, 1152, 4860), (1024, 3072, 8192), (1024, 3072, 9216)])
def test_prefill_codes_equal_dequantised_weights(hip, scheme, m, k, n):
    """The MFMA GEMM over the codes forms bf16(code * scale) on the way into LDS: its result must equal, BIT FOR BIT,
    the same GEMM over the dequantised matrix given as a plain bf16 weight (same kernel, same values, same order),
    with and without the SwiGLU pairing; every tile shape and split of the kernel, ragged M and N, zero and extreme
    columns.  The single-matrix GEMM is also checked against the oracle's "dequantise, then dot_general", and run
    twice: split tiles meet through tickets that every launch must leave at zero."""
    x = bf16_round(rnd(31, (m, k)))
    w = weights_with_corner_cases(32, k, n)
    w2 = rnd(33, (k, n), 2.0 / np.sqrt(k))
    (q, s), (q2, s2) = quantize(w, scheme), quantize(w2, scheme)
    cs_, ss_ = code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))
    built = hip.counter("derived_weights_built")
    (got,) = hip_run(hip, prog(lambda fb, a, b, c: F.linear_quantized(a, b, c), [("Bf16", [m, k]), cs_, ss_]), [x, q, s])
    assert hip.counter("derived_weights_built") == built + 1     # one copy: the codes (no dequantised matrix)
    # "same kernel": plain bf16 weights otherwise run on the LDS-direct GEMM, which sums in another order
    hip.set_option("gemm_lds_direct", 0)
    try:
        (want,) = hip_run(hip, prog(lambda fb, a, b: a.matmul(b), [("Bf16", [m, k]), ("Bf16", [k, n])]), [x, dequantize_host(q, s, scheme)])
    finally:
        hip.set_option("gemm_lds_direct", 1)
    assert np.array_equal(got, want), f"max diff {np.max(np.abs(got - want))}"
    (direct,) = hip_run(hip, prog(lambda fb, a, b: a.matmul(b), [("Bf16", [m, k]), ("Bf16", [k, n])]), [x, dequantize_host(q, s, scheme)])
    assert_close(direct, want, atol=1e-4 * np.sqrt(k), rtol=2.0 ** -7, what="LDS-direct GEMM vs register-staged GEMM")
    pq = prog(lambda fb, a, b, c: F.linear_quantized(a, b, c), [("Bf16", [m, k]), cs_, ss_])
    (again,) = hip_run(hip, pq, [x, q, s])
    assert np.array_equal(again, got), "a second launch of the same GEMM differs (tickets not returned to zero?)"
    po.BLAS_DOT_MIN_MACS, old_min = 1 << 27, po.BLAS_DOT_MIN_MACS
    try:
        (ref,) = oracle_run(pq, [x, q, s])
    finally:
        po.BLAS_DOT_MIN_MACS = old_min
    # both sides round an f32 sum to bf16: where the two summation orders straddle a rounding boundary, one ulp (2^-7)
    assert_close(got, ref, atol=1e-4 * np.sqrt(k), rtol=2.0 ** -7, what="quantised GEMM vs oracle")
    (gotp,) = hip_run(hip, prog(lambda fb, a, b, bs, c, cs: F.swiglu(F.linear_quantized(a, b, bs), F.linear_quantized(a, c, cs)),
                                [("Bf16", [m, k]), cs_, ss_, cs_, ss_]), [x, q, s, q2, s2])
    pair = prog(lambda fb, a, b, c: F.swiglu(a.matmul(b), a.matmul(c)), [("Bf16", [m, k]), ("Bf16", [k, n]), ("Bf16", [k, n])])
    pair_args = [x, dequantize_host(q, s, scheme), dequantize_host(q2, s2, scheme)]
    hip.set_option("gemm_lds_direct", 0)
    try:
        (wantp,) = hip_run(hip, pair, pair_args)
    finally:
        hip.set_option("gemm_lds_direct", 1)
    assert np.array_equal(gotp, wantp), f"pair: max diff {np.max(np.abs(gotp - wantp))}"
    (directp,) = hip_run(hip, pair, pair_args)
    # silu(g) * u of two sums that each differ by a rounding of the f32 accumulation order, then one bf16 rounding
    assert_close(directp, wantp, atol=2e-4 * np.sqrt(k), rtol=2.0 ** -6, what="LDS-direct pair vs register-staged pair")


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m,k,n", [(8, 3072, 6144), (8, 4096, 3072), (2, 9216, 3072), (16, 3072, 1000), (5, 512, 40), (8, 3072, 32768)])
def test_batched_decode_linear_bf16(hip, scheme, m, k, n):
    """2..16 bf16 rows: the matrix-core kernel streams the codes (biased codes are exact in bf16; the bias leaves through
    a second product against a column of ones), K split over workgroups where the layer has few column tiles."""
    x, w = bf16_round(rnd(21, (m, k))), rnd(22, (k, n), 2.0 / np.sqrt(k))
    q, s = quantize(w, scheme)
    specs = [("Bf16", [m, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))]
    built = hip.counter("derived_weights_built")
    run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x, q, s], 3e-2, 2e-2, expect_chain=False)
    assert hip.counter("derived_weights_built") > built        # the code copy in tile order, not the generic fallback
    # activations with a large common offset: the bias term 128 * sum(x) is then far larger than the result
    x2 = bf16_round(rnd(23, (m, k)) + 3.0)
    run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x2, q, s], 6e-2, 2e-2, expect_chain=False)


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m", [1, 8, 64])
def test_bias_gelu_residual(hip, scheme, m):
    k, n = 768, 3072
    x, w, b, r = bf16_round(rnd(10, (m, k))), rnd(11, (k, n), 2.0 / np.sqrt(k)), bf16_round(rnd(12, (n,))), bf16_round(rnd(13, (m, n)))
    q, s = quantize(w, scheme)
    specs = [("Bf16", [m, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n)), ("Bf16", [n]), ("Bf16", [m, n])]
    run_linear(hip, lambda fb, a, c, d, e, f: F.gelu(F.linear_quantized(a, c, d, e)) + f, specs, [x, q, s, b, r], 4e-2, 2e-2,
               expect_chain=(m == 1))


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
@pytest.mark.parametrize("m,k,n", [(1, 3072, 9216), (1, 256, 96), (64, 512, 256), (8, 3072, 9216), (16, 256, 96)])
def test_norm_swiglu_pair(hip, scheme, m, k, n):
    """RMSNorm -> gate / up -> SwiGLU: one phase of the chain (or one dual GEMM) over two quantised matrices."""
    x, g = bf16_round(rnd(6, (m, k), 3.0)), bf16_round(rnd(7, (k,)) + 1.5)
    qg, sg = quantize(rnd(8, (k, n), 2.0 / np.sqrt(k)), scheme)
    qu, su = quantize(rnd(9, (k, n), 2.0 / np.sqrt(k)), scheme)

    def build(fb, a, gm, b, bs, c, cs):
        h = F.rms_norm(a, gm, 1e-5)[0]
        return F.swiglu(F.linear_quantized(h, b, bs), F.linear_quantized(h, c, cs))

    cs_, ss_ = code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))
    run_linear(hip, build, [("Bf16", [m, k]), ("Bf16", [k]), cs_, ss_, cs_, ss_], [x, g, qg, sg, qu, su], 8e-2, 4e-2,
               expect_chain=(m == 1))


@pytest.mark.parametrize("scheme", ["w8", "w4g128"])
def test_block_tail_chain(hip, scheme):
    """out-proj (+residual) -> RMSNorm -> gate/up SwiGLU -> down (+residual) -> RMSNorm -> next projection with
    every matrix quantised: five dependent phases in one launch (model/ministral.rs:166-201)."""
    d, f = 256, 640
    qp = 384
    ctx, x = bf16_round(rnd(20, (1, qp))), bf16_round(rnd(21, (1, d)))
    mats = [rnd(22, (qp, d), 2.0 / np.sqrt(qp)), rnd(23, (d, f), 2.0 / np.sqrt(d)), rnd(24, (d, f), 2.0 / np.sqrt(d)),
            rnd(25, (f, d), 2.0 / np.sqrt(f)), rnd(26, (d, 2 * d), 2.0 / np.sqrt(d))]
    g1, g2 = bf16_round(rnd(27, (d,)) + 1.5), bf16_round(rnd(28, (d,)) + 1.5)
    arrays, specs = [ctx, x, g1, g2], [("Bf16", [1, qp]), ("Bf16", [1, d]), ("Bf16", [d]), ("Bf16", [d])]
    for w in mats:
        q, s = quantize(w, scheme)
        arrays += [q, s]
        specs += [code_spec(scheme, *w.shape), ("Bf16", scale_dims(scheme, *w.shape))]

    def build(fb, c, xx, a_g1, a_g2, wo, so, wg, sg, wu, su, wd, sd, wq, sq):
        h = F.linear_quantized(c, wo, so) + xx
        n1 = F.rms_norm(h, a_g1, 1e-5)[0]
        ff = F.linear_quantized(F.swiglu(F.linear_quantized(n1, wg, sg), F.linear_quantized(n1, wu, su)), wd, sd) + h
        return [F.linear_quantized(F.rms_norm(ff, a_g2, 1e-5)[0], wq, sq), ff]

    before = hip.counter("chain_phases")
    run_linear(hip, build, specs, arrays, 1e-1, 5e-2, expect_chain=True)
    assert hip.counter("chain_phases") - before >= 4


def test_chain_off_matches(hip):
    """The same quantised decode linear with the chain switched off runs the dequantise + generic path."""
    k, n = 1024, 512
    x, w = bf16_round(rnd(30, (1, k))), rnd(31, (k, n), 2.0 / np.sqrt(k))
    for scheme in ("w8", "w4g128"):
        q, s = quantize(w, scheme)
        specs = [("Bf16", [1, k]), code_spec(scheme, k, n), ("Bf16", scale_dims(scheme, k, n))]
        hip.set_option("chain", 0)
        try:
            run_linear(hip, lambda fb, a, b, c: F.linear_quantized(a, b, c), specs, [x, q, s], 2e-2, 2e-2, expect_chain=False)
        finally:
            hip.set_option("chain", 1)


def test_bad_operands_rejected(hip):
    """Shape and dtype rules of the extension targets; unknown targets stay Unimplemented (docs/backend.md:581-582)."""
    from gptrs_amd.backend import BackendError
    from gptrs_amd.ptir import TensorSpec
    k, n = 256, 16

    def dot(target, xs, qs, ss, out):
        def build(fb, a, b, c):
            return fb.custom_call(target, [a, b, c], TensorSpec(*out))
        return prog(build, [xs, qs, ss])

    cases = [
        dot("gpt_rs.hip.dot_w8.v1", ("F32", [2, k]), ("Si8", [k + 1, n]), ("F32", [n]), ("F32", [2, n])),      # K mismatch
        dot("gpt_rs.hip.dot_w8.v1", ("F32", [2, k]), ("Ui8", [k, n]), ("F32", [n]), ("F32", [2, n])),          # code dtype
        dot("gpt_rs.hip.dot_w8.v1", ("F32", [2, k]), ("Si8", [k, n]), ("Bf16", [n]), ("F32", [2, n])),         # scale dtype
        dot("gpt_rs.hip.dot_w4g128.v1", ("F32", [2, 192]), ("Ui8", [96, n]), ("F32", [1, n]), ("F32", [2, n])),  # K % 128
        dot("gpt_rs.hip.dot_w4g128.v1", ("F32", [2, k]), ("Ui8", [k // 2, n]), ("F32", [n]), ("F32", [2, n])),  # scale shape
    ]
    for p in cases:
        arrays = [np.zeros(s.dims, np.float32) for s in p.param_specs]
        with pytest.raises(BackendError) as ei:
            hip_run(hip, p, arrays)
        assert ei.value.kind == "execution"
    p = dot("gpt_rs.hip.no_such_op.v1", ("F32", [2, k]), ("Si8", [k, n]), ("F32", [n]), ("F32", [2, n]))
    with pytest.raises(BackendError) as ei:
        hip_run(hip, p, [np.zeros(s.dims, np.float32) for s in p.param_specs])
    assert ei.value.kind == "unimplemented"
