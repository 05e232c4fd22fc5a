"""GPU parity, op by op: every PTIR op the LM path emits, HIP vs the CPU oracle on identical
seeded inputs.  Integer / index ops must be bit-exact; float ops within the reference suite's
tolerance (5e-4 + 1e-4*max, torch_parity/common.rs:14-15).  Shapes follow the reference's
parity-case catalogue (crates/gpt-rs-backend-tests/src/lib.rs:99-261)."""
import numpy as np
import pytest

from parity import FunctionBuilder, Program, assert_close, check_program, hip_run, oracle_run, to_bytes
from gptrs_amd import functional as F
from gptrs_amd.ptir import Tensor, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def rng_uniform(seed, shape, lo=-1.0, hi=1.0):
    return np.random.default_rng(seed).uniform(lo, hi, size=shape).astype(np.float32)


def prog(build, param_specs):
    fb = FunctionBuilder("main")
    params = [fb.param(dt, dims) for dt, dims in param_specs]
    res = build(fb, *params)
    fb.set_results(list(res) if isinstance(res, (list, tuple)) else [res])
    return Program(fb)


# ------------------------------------------------------------------ reference-held vectors
def test_smoke_matmul_golden(hip):
    # crates/gpt-rs-backend-tests/src/smoke.rs:12-24
    p = prog(lambda fb, a, b: a.matmul(b), [("F32", [2, 2]), ("F32", [2, 2])])
    out = hip_run(hip, p, [np.array([[1, 2], [3, 4]], np.float32), np.array([[5, 6], [7, 8]], np.float32)])[0]
    assert out.reshape(-1).tolist() == [19.0, 22.0, 43.0, 50.0]


@pytest.mark.parametrize("start,expect", [(-3, [1, 2]), (9, [4, 5]), (2, [3, 4])])
def test_dynamic_slice_clamp_golden(hip, start, expect):
    # crates/gpt-rs-backend-triton/tests/dynamic_ops_gpu.rs:35-70
    p = prog(lambda fb, x, s: x.dynamic_slice(s, [2]), [("F32", [5]), ("Si32", [1])])
    out = hip_run(hip, p, [np.array([1, 2, 3, 4, 5], np.float32), np.array([start], np.int32)])[0]
    assert out.tolist() == [float(v) for v in expect]


def test_dynamic_slice_si32_golden(hip):
    p = prog(lambda fb, x, s: x.dynamic_slice(s, [2]), [("Si32", [5]), ("Si32", [1])])
    out = hip_run(hip, p, [np.array([10, 20, 30, 40, 50], np.int32), np.array([7], np.int32)])[0]
    assert out.tolist() == [40, 50]


@pytest.mark.parametrize("start,expect", [(-2, [99, 88, 12, 13, 14]), (8, [10, 11, 12, 99, 88])])
def test_dynamic_update_slice_clamp_golden(hip, start, expect):
    # crates/gpt-rs-backend-triton/tests/dynamic_ops_gpu.rs:72-104
    p = prog(lambda fb, x, u, s: x.dynamic_update_slice(u, s, [2]), [("F32", [5]), ("F32", [2]), ("Si32", [1])])
    out = hip_run(hip, p, [np.array([10, 11, 12, 13, 14], np.float32), np.array([99, 88], np.float32),
                           np.array([start], np.int32)])[0]
    assert out.tolist() == [float(v) for v in expect]


def test_scalar_broadcast_add_golden(hip):
    # crates/gpt-rs/tests/graph_cache_stability.rs:95-131, lazy_graph.rs:100-132
    x = np.array([1, 2, 3, 4], np.float32)
    assert hip_run(hip, prog(lambda fb, a: a + 1.0, [("F32", [4])]), [x])[0].tolist() == [2, 3, 4, 5]
    assert hip_run(hip, prog(lambda fb, a: a + 2.0, [("F32", [4])]), [x])[0].tolist() == [3, 4, 5, 6]
    p = prog(lambda fb, a, b: a + b, [("F32", [4]), ("F32", [4])])
    assert hip_run(hip, p, [np.array([2, 4, 6, 8], np.float32), np.ones(4, np.float32)])[0].tolist() == [3, 5, 7, 9]


def test_greedy_sample_golden(hip):
    # crates/gpt-rs-backend-triton/tests/decode_sampling.rs:6-20
    from gptrs_amd.ptir import TensorSpec
    h = hip.materialize(TensorSpec("F32", [1, 4]), np.array([[-1.0, 0.1, 2.5, 0.4]], np.float32))
    assert hip.sample_decode_token(h, temperature=0.0) == 2
    assert hip.supports_decode_sampling(0.0) and not hip.supports_decode_sampling(1.0, top_k=5)


# ------------------------------------------------------------------ layout / index ops (bit-exact)
@pytest.mark.parametrize("dtype", ["F32", "Bf16", "Si32"])
def test_layout_ops_exact(hip, dtype):
    r = np.random.default_rng(11)
    x = r.integers(-100, 100, size=(3, 4, 6)).astype(np.float32)

    def build(fb, a):
        s = a.slice([1, 0, 2], [2, 3, 4])
        t = a.transpose([2, 0, 1])
        rs = a.reshape([6, 12])
        c = Tensor.concat(1, [a, a.slice([0, 1, 0], [3, 2, 6])])
        b = a.slice([0, 0, 0], [3, 1, 6]).broadcast_to([2, 3, 4, 6])
        return [s, t, rs, c, b]

    check_program(hip, prog(build, [(dtype, [3, 4, 6])]), [x], atol=0, rtol=0)


def test_iota_compare_select_cast_exact(hip):
    def build(fb, x, y):
        i0 = fb.iota([5, 7], 0)
        i1 = fb.iota([5, 7], 1)
        ge = i0.greater_equal(i1)
        sel = Tensor.select(ge, x, y)
        return [i0, i1, ge, sel, ge.cast("Si32"), i1.cast("F32"), x.cast("Si32"), ge.cast("F32"), i0.compare(i1, "NotEqual")]

    x = rng_uniform(1, (5, 7), -300, 300)
    y = rng_uniform(2, (5, 7))
    check_program(hip, prog(build, [("F32", [5, 7]), ("F32", [5, 7])]), [x, y], atol=0, rtol=0)


def test_cast_saturation_and_nan(hip):
    x = np.array([1.9, -1.9, 3e9, -3e9, np.nan, 0.0, -0.0, 1e-30], np.float32)
    check_program(hip, prog(lambda fb, a: [a.cast("Si32"), a.cast("I1"), a.cast("Bf16")], [("F32", [8])]), [x], atol=0, rtol=0)


@pytest.mark.parametrize("vocab,embed,seq", [(64, 32, 16), (32, 8, 5), (32, 128, 8)])
def test_take_embedding_exact(hip, vocab, embed, seq):
    w = rng_uniform(3, (vocab, embed))
    idx = np.random.default_rng(4).integers(0, vocab, size=seq).astype(np.int32)
    idx[-1] = idx[0]  # duplicate indices
    check_program(hip, prog(lambda fb, t, i: F.embedding_lookup(t, i), [("F32", [vocab, embed]), ("Si32", [seq])]),
                  [w, idx], atol=0, rtol=0)


def test_take_out_of_range_is_an_execution_error(hip):
    from gptrs_amd.backend import BackendError
    p = prog(lambda fb, t, i: t.take(i), [("F32", [8, 4]), ("Si32", [2])])
    with pytest.raises(BackendError) as ei:
        hip_run(hip, p, [np.zeros((8, 4), np.float32), np.array([1, 8], np.int32)])
    assert ei.value.kind == "execution" and "out of bounds" in str(ei.value)


def test_dynamic_ops_rank3_exact(hip):
    base = rng_uniform(5, (4, 16, 8))
    upd = rng_uniform(6, (4, 1, 8))
    for pos in (0, 7, 15, 40, -3):
        st = np.array([0, pos, 0], np.int32)
        p = prog(lambda fb, b, u, s: [b.dynamic_update_slice(u, s, [4, 1, 8]), b.dynamic_slice(s, [4, 2, 8])],
                 [("F32", [4, 16, 8]), ("F32", [4, 1, 8]), ("Si32", [3])])
        check_program(hip, p, [base, upd, st], atol=0, rtol=0)


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_update_from_a_view_exact(hip, dtype):
    """DynamicUpdateSlice whose update is a Slice / Reshape / Transpose chain of another tensor: the fusion pass copies
    straight out of that tensor (the K / V rows of a packed projection go into the caches this way).  Bit-exact against
    the oracle, fusion on and off, including a chain whose reshape cannot be expressed as strides (merges transposed
    axes) and one whose intermediate value is also a result."""
    x = rng_uniform(11, (6, 20))
    if dtype == "Bf16":
        x = (f32_to_bf16_bits(x).astype(np.uint32) << 16).view(np.float32)
    base = np.zeros((3, 10, 4), np.float32)
    st = np.array([0, 2, 0], np.int32)
    specs = [(dtype, [6, 20]), (dtype, [3, 10, 4]), ("Si32", [3])]

    def heads(fb, a, b, s):          # columns 4..16 as 3 heads of 4, head-major
        u = a.slice([0, 4], [6, 12]).reshape([6, 3, 4]).transpose([1, 0, 2])
        return b.dynamic_update_slice(u, s, [3, 6, 4])

    def merged(fb, a, b, s):         # transpose, then a reshape that merges the transposed axes: needs a real copy
        u = a.slice([0, 0], [6, 12]).transpose([1, 0]).reshape([3, 6, 4])
        return b.dynamic_update_slice(u, s, [3, 6, 4])

    def shared(fb, a, b, s):         # the view is a result as well: it must still be materialised
        u = a.slice([0, 8], [6, 12]).reshape([6, 3, 4]).transpose([1, 0, 2])
        return [b.dynamic_update_slice(u, s, [3, 6, 4]), u]

    def split(fb, a, b, s):          # a reshape that splits the sliced axis after a transpose of the outer ones
        u = a.reshape([2, 3, 20]).transpose([1, 0, 2]).slice([0, 0, 4], [3, 2, 16]).reshape([3, 2, 4, 4]).reshape([3, 8, 4])
        return b.dynamic_update_slice(u, s, [3, 8, 4])

    for build in (heads, merged, shared, split):
        check_program(hip, prog(build, specs), [x, base, st], atol=0, rtol=0)

    # a view of the base itself, overlapping the rows it is written to: the view must be taken before the write
    own = rng_uniform(12, (3, 10, 4))
    if dtype == "Bf16":
        own = (f32_to_bf16_bits(own).astype(np.uint32) << 16).view(np.float32)

    def overlap(fb, b, s):
        return b.dynamic_update_slice(b.slice([0, 0, 0], [3, 6, 4]), s, [3, 6, 4])

    def overlap_reshaped(fb, b, s):
        flat = b.reshape([30, 4])
        u = flat.reshape([3, 10, 4]).slice([0, 1, 0], [3, 6, 4])
        return flat.reshape([3, 10, 4]).dynamic_update_slice(u, s, [3, 6, 4])

    for build in (overlap, overlap_reshaped):
        p = prog(build, [(dtype, [3, 10, 4]), ("Si32", [3])])
        check_program(hip, p, [own, st], atol=0, rtol=0)
        hs = [hip.materialize(sp, to_bytes(a, sp.dtype)) for sp, a in zip(p.param_specs, [own, st])]
        (got,) = hip.run_program(p, hs, [True, False])          # donated base: the update runs in place
        (want,) = oracle_run(p, [own, st])
        assert np.array_equal(hip.to_numpy(got), want)


# ------------------------------------------------------------------ float ops
MATMUL_SHAPES = [(1, 1, 1), (1, 5, 3), (4, 5, 1), (7, 13, 9), (33, 65, 31), (8, 1, 8), (1, 16, 17), (64, 128, 32)]


@pytest.mark.parametrize("m,k,n", MATMUL_SHAPES)
@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_matmul(hip, m, k, n, dtype):
    # torch_parity/matmul.rs:78-115
    a, b = rng_uniform(7, (m, k)), rng_uniform(8, (k, n))
    tol = dict(atol=5e-4, rtol=1e-4) if dtype == "F32" else dict(atol=2e-2, rtol=2e-2)
    check_program(hip, prog(lambda fb, x, y: x.matmul(y), [(dtype, [m, k]), (dtype, [k, n])]), [a, b], **tol)


@pytest.mark.parametrize("m,k,n", [(17, 64, 8), (100, 128, 72), (128, 192, 256), (300, 64, 200), (257, 320, 129)])
def test_prefill_linear_on_matrix_cores(hip, m, k, n):
    """bf16 linears with more than 16 rows and K % 64 == 0 run on the MFMA kernel over the k-grouped
    weight copy: plain matmul, bias + exact GELU + residual epilogue, and the SwiGLU pair.  Ragged M
    and N exercise the row clamp, the column padding and the store masks.  The oracle rounds every
    op to bf16, the fused kernel once at the end, hence the bf16-sized tolerance."""
    x = rng_uniform(40, (m, k))
    w, w2 = rng_uniform(41, (k, n)) / np.sqrt(k) * 2, rng_uniform(42, (k, n)) / np.sqrt(k) * 2
    b, r = rng_uniform(43, (n,)), rng_uniform(44, (m, n))
    tol = dict(atol=3e-2, rtol=3e-2)
    before = hip.counter("derived_weights_built")
    check_program(hip, prog(lambda fb, a, c: a.matmul(c), [("Bf16", [m, k]), ("Bf16", [k, n])]), [x, w], **tol)
    check_program(hip, prog(lambda fb, a, c, d, e: F.gelu(F.linear(a, c, d)) + e,
                            [("Bf16", [m, k]), ("Bf16", [k, n]), ("Bf16", [n]), ("Bf16", [m, n])]), [x, w, b, r], **tol)
    check_program(hip, prog(lambda fb, a, c, d: F.swiglu(a.matmul(c), a.matmul(d)),
                            [("Bf16", [m, k]), ("Bf16", [k, n]), ("Bf16", [k, n])]), [x, w, w2], **tol)
    assert hip.counter("derived_weights_built") - before >= 4  # the fused legs took the derived-weight path


@pytest.mark.parametrize("dtype", ["Bf16", "F32"])
@pytest.mark.parametrize("m,k,n,pair", [(1024, 1024, 4860, False), (1100, 512, 5120, False), (1024, 1024, 2430, True), (1024, 256, 4864, False),
                                        (1024, 768, 4860, False), (1024, 1536, 2430, True), (1030, 960, 8192, False),
                                        (1000, 512, 3072, False), (1000, 512, 3060, False), (1024, 512, 2432, True), (520, 64, 6144, False),
                                        (1000, 6144, 3072, False), (900, 6208, 3000, False)])
def test_prefill_linear_tail_tiles_split_over_k(hip, m, k, n, pair, dtype):
    """Launches of more than 256 tiles whose last round holds at most 128: those tiles are split 4 or 2 ways over k
    between workgroups that meet through a workspace and a ticket (304 tiles -> 48 x 4, 360 -> 104 x 2, the SwiGLU pair
    with 64 real columns per tile, and K = 256 with too few k tiles to split;
    further K and tile counts with and without a tail).  Unquantised bf16 runs on the LDS-direct kernel instead: these
    shapes take its 128 x 192 tiles, its 128 x 96 tiles (N = 3072 / 3060 at M = 1000), the pair whose two matrices are
    wave columns, ragged M, N that is and is not a multiple of 8 (16-byte and element-wise epilogues), K = 64 (fewer
    k tiles than the ring of staged tiles is deep), and 128 tiles of 128 x 192 split two ways over k with partial sums
    and tickets (K = 6144 / 6208 at N = 3072 / 3000; 97 k tiles split 48 + 49).  Checked against the oracle, and a second
    run (tickets must have returned to zero) must reproduce the first bit for bit."""
    x = rng_uniform(50, (m, k))
    w, w2 = rng_uniform(51, (k, n)) / np.sqrt(k) * 2, rng_uniform(52, (k, n)) / np.sqrt(k) * 2
    b, r = rng_uniform(53, (n,)), rng_uniform(54, (m, n))
    tol = dict(atol=3e-2, rtol=3e-2) if dtype == "Bf16" else dict(atol=5e-4, rtol=1e-4)
    if pair:
        p = prog(lambda fb, a, c, d: F.swiglu(a.matmul(c), a.matmul(d)), [(dtype, [m, k]), (dtype, [k, n]), (dtype, [k, n])])
        args = [x, w, w2]
    else:
        p = prog(lambda fb, a, c, d, e: F.gelu(F.linear(a, c, d)) + e, [(dtype, [m, k]), (dtype, [k, n]), (dtype, [n]), (dtype, [m, n])])
        args = [x, w, b, r]
    check_program(hip, p, args, both_modes=False, **tol)
    first, second = hip_run(hip, p, args)[0], hip_run(hip, p, args)[0]
    assert np.array_equal(first, second)


@pytest.mark.parametrize("b,m,k,n", [(1, 4, 5, 2), (2, 7, 13, 9), (8, 4, 8, 4), (3, 33, 65, 31)])
def test_matmul_batched(hip, b, m, k, n):
    a, c = rng_uniform(9, (b, m, k)), rng_uniform(10, (b, k, n))
    check_program(hip, prog(lambda fb, x, y: x.matmul(y), [("F32", [b, m, k]), ("F32", [b, k, n])]), [a, c])


def test_dot_general_attention_contractions(hip):
    q, kk, v = rng_uniform(1, (4, 3, 8)), rng_uniform(2, (4, 5, 8)), rng_uniform(3, (4, 5, 8))

    def build(fb, a, b, c):
        s = a.dot_general(b, [0], [2], [2])
        return [s, s.dot_general(c, [0], [2], [1])]

    check_program(hip, prog(build, [("F32", [4, 3, 8]), ("F32", [4, 5, 8]), ("F32", [4, 5, 8])]), [q, kk, v])


def test_dot_general_non_collapsible_operands(hip):
    # contraction over two non-adjacent lhs axes forces the repack path
    a, b = rng_uniform(1, (3, 4, 5)), rng_uniform(2, (3, 5, 6))
    p = prog(lambda fb, x, y: x.dot_general(y, [], [0, 2], [0, 1]), [("F32", [3, 4, 5]), ("F32", [3, 5, 6])])
    check_program(hip, p, [a, b])


@pytest.mark.parametrize("shape", [(3, 2, 4), (2, 1), (3, 2), (2, 7), (4, 128), (2, 3, 8), (2, 4, 32), (1, 3, 257), (4, 768)])
@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_softmax(hip, shape, dtype):
    x = rng_uniform(12, shape, -3, 3)
    tol = dict() if dtype == "F32" else dict(atol=1e-2, rtol=2e-2)
    check_program(hip, prog(lambda fb, a: F.softmax_last_axis(a), [(dtype, list(shape))]), [x], **tol)


def test_softmax_extreme_and_constant(hip):
    x = rng_uniform(13, (4, 16), -80, 80)
    check_program(hip, prog(lambda fb, a: F.softmax_last_axis(a), [("F32", [4, 16])]), [x], atol=5e-3, rtol=5e-3)
    c = np.full((2, 3, 17), 0.25, np.float32)
    out = check_program(hip, prog(lambda fb, a: F.softmax_last_axis(a), [("F32", [2, 3, 17])]), [c])
    assert np.allclose(out[0].sum(-1), 1.0, atol=1e-6)


@pytest.mark.parametrize("shape,lo,hi", [((6,), -1, 1), ((256,), -1, 1), ((4, 16), -1, 1), ((2, 3, 8), -1, 1), ((256,), -10, 10)])
def test_gelu(hip, shape, lo, hi):
    x = rng_uniform(14, shape, lo, hi)
    check_program(hip, prog(lambda fb, a: F.gelu(a), [("F32", list(shape))]), [x])


def test_silu_and_swiglu(hip):
    check_program(hip, prog(lambda fb, a: F.silu(a), [("F32", [3, 17])]), [rng_uniform(15, (3, 17), -40, 40)])
    g, u = rng_uniform(16, (5, 19), -10, 10), rng_uniform(17, (5, 19))
    check_program(hip, prog(lambda fb, a, b: F.swiglu(a, b), [("F32", [5, 19]), ("F32", [5, 19])]), [g, u])
    check_program(hip, prog(lambda fb, a, b: F.swiglu(a, b), [("Bf16", [5, 19]), ("Bf16", [5, 19])]), [g, u], atol=5e-2, rtol=2e-2)


@pytest.mark.parametrize("shape", [(3, 4), (2, 5, 8), (1, 16, 64), (2, 3, 4, 5)])
def test_add_bias(hip, shape):
    x, b = rng_uniform(18, shape), rng_uniform(19, (shape[-1],))
    check_program(hip, prog(lambda fb, a, c: F.add_bias(a, c), [("F32", list(shape)), ("F32", [shape[-1]])]), [x, b])


@pytest.mark.parametrize("shape,eps", [((2, 3, 4), 1e-5), ((2, 3, 1), 1e-5), ((2, 3, 13), 1e-5), ((2, 4, 256), 1e-5), ((1, 8), 1e-5),
                                       ((2, 3, 17), 1e-3), ((4, 768), 1e-5), ((3, 3072), 1e-5), ((2, 5000), 1e-5)])
def test_layer_norm_all_outputs(hip, shape, eps):
    # checks out, normalized, mean, inv_std like torch_parity/functional_ops.rs
    n = shape[-1]
    x, g, b = rng_uniform(20, shape), rng_uniform(21, (n,)), rng_uniform(22, (n,))
    p = prog(lambda fb, a, c, d: list(F.layer_norm(a, c, d, eps)), [("F32", list(shape)), ("F32", [n]), ("F32", [n])])
    check_program(hip, p, [x, g, b], atol=2e-3 if n == 1 else 5e-4)
    p1 = prog(lambda fb, a, c, d: F.layer_norm(a, c, d, eps)[0], [("F32", list(shape)), ("F32", [n]), ("F32", [n])])
    check_program(hip, p1, [x, g, b])


def test_layer_norm_constant_input_gives_beta(hip):
    x = np.full((2, 3, 17), 0.5, np.float32)
    g, b = rng_uniform(1, (17,)), rng_uniform(2, (17,))
    p = prog(lambda fb, a, c, d: F.layer_norm(a, c, d, 1e-5)[0], [("F32", [2, 3, 17]), ("F32", [17]), ("F32", [17])])
    out = check_program(hip, p, [x, g, b])[0]
    assert np.allclose(out, np.broadcast_to(b, out.shape), atol=1e-6)


@pytest.mark.parametrize("shape", [(2, 3, 4), (5, 16), (1, 3072), (8, 3072), (3, 24), (2, 8192), (2, 8200), (70, 1000)])
@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_rms_norm(hip, shape, dtype):
    n = shape[-1]
    x, g = rng_uniform(23, shape), rng_uniform(24, (n,))
    tol = dict() if dtype == "F32" else dict(atol=3e-2, rtol=2e-2)
    p = prog(lambda fb, a, c: F.rms_norm(a, c, 1e-5)[0], [(dtype, list(shape)), (dtype, [n])])
    check_program(hip, p, [x, g], **tol)


@pytest.mark.parametrize("hq,hkv,dh,rot,seq", [(4, 4, 8, 8, 5), (4, 2, 8, 4, 3), (8, 2, 16, 16, 1), (4, 1, 8, 6, 4)])
def test_rope_packed(hip, hq, hkv, dh, rot, seq):
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    cos, sin = F.rotary_cos_sin_cache_slice(3, seq, F.RopeConfig(rot, 10000.0))
    qkv = rng_uniform(25, (seq, cfg.total_projection_dim))
    p = prog(lambda fb, a, c, s: F.apply_rope_qkv_packed(cfg, a, c, s),
             [("F32", [seq, cfg.total_projection_dim]), ("F32", [seq, rot // 2]), ("F32", [seq, rot // 2])])
    out = check_program(hip, p, [qkv, cos, sin])[0]
    # rotation preserves the norm of each (first, second) pair; V passes through untouched
    assert np.array_equal(out[:, (hq + hkv) * dh:], qkv[:, (hq + hkv) * dh:])


@pytest.mark.parametrize("hq,hkv,dh,rot,seq", [(32, 8, 128, 128, 7), (4, 2, 16, 16, 33), (2, 1, 64, 64, 300), (4, 2, 16, 8, 3), (4, 4, 8, 8, 5)])
def test_rope_packed_bf16(hip, hq, hkv, dh, rot, seq):
    """bf16 rows: heads whose halves are multiples of 8 take the 16-byte kernel, the rest the element-wise one."""
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    cos, sin = F.rotary_cos_sin_cache_slice(5, seq, F.RopeConfig(rot, 10000.0))
    qkv = rng_uniform(27, (seq, cfg.total_projection_dim))
    p = prog(lambda fb, a, c, s: F.apply_rope_qkv_packed(cfg, a, c, s),
             [("Bf16", [seq, cfg.total_projection_dim]), ("Bf16", [seq, rot // 2]), ("Bf16", [seq, rot // 2])])
    check_program(hip, p, [qkv, cos, sin], atol=2e-2, rtol=2e-2)
    # V passes through bit for bit; the rotated part equals the f32 closed form of the bf16 inputs to one bf16 ulp
    r = lambda a: bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(a, np.float32)))
    out = np.asarray(hip_run(hip, p, [qkv, cos, sin])[0], np.float32)
    x, c, s_ = r(qkv), r(cos), r(sin)
    assert np.array_equal(out[:, (hq + hkv) * dh:], x[:, (hq + hkv) * dh:])
    h = rot // 2
    heads = x[:, :(hq + hkv) * dh].reshape(seq, hq + hkv, dh)
    want = heads.copy()
    want[:, :, :h] = heads[:, :, :h] * c[:, None, :] - heads[:, :, h:rot] * s_[:, None, :]
    want[:, :, h:rot] = heads[:, :, h:rot] * c[:, None, :] + heads[:, :, :h] * s_[:, None, :]
    got = out[:, :(hq + hkv) * dh].reshape(seq, hq + hkv, dh)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -7 + 1e-6)


@pytest.mark.parametrize("hq,hkv,dh,seq", [(3, 3, 2, 4), (2, 2, 4, 1), (4, 4, 8, 8), (4, 4, 1, 3), (4, 1, 4, 5), (4, 2, 8, 6), (8, 2, 16, 33)])
def test_attention_prefill(hip, hq, hkv, dh, seq):
    # torch_parity/attention.rs: seq4/embed6/H3, seq1 embed8 H2, seq8 embed32 H4, head_dim 1, MQA, GQA
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    qkv = rng_uniform(26, (seq, cfg.total_projection_dim))
    p = prog(lambda fb, a: list(F.attention(cfg, a, None)), [("F32", [seq, cfg.total_projection_dim])])
    check_program(hip, p, [qkv])


@pytest.mark.parametrize("m,k,n", [(2, 3072, 6144), (8, 4096, 3072), (8, 9216, 3072), (16, 3072, 1000), (5, 512, 40), (3, 64, 24),
                                   (8, 3072, 32768)])
def test_batched_decode_linear_on_matrix_cores(hip, m, k, n):
    """2..16 bf16 rows (batched decode): the 16x16x32 MFMA kernel over the 16-column tiled weight copy, plain and
    under bias + exact GELU + residual; reference = the f32 oracle on the same bf16-representable inputs."""
    r16 = lambda a: (f32_to_bf16_bits(np.asarray(a, np.float32)).astype(np.uint32) << 16).view(np.float32)  # noqa: E731
    x, w = r16(rng_uniform(50, (m, k))), r16(rng_uniform(51, (k, n)) * (2.0 / np.sqrt(k)))
    b, r = r16(rng_uniform(52, (n,))), r16(rng_uniform(53, (m, n)))
    for build, arrays, dims in [
        (lambda fb, a, c: a.matmul(c), [x, w], [[m, k], [k, n]]),
        (lambda fb, a, c, d, e: F.gelu(F.linear(a, c, d)) + e, [x, w, b, r], [[m, k], [k, n], [n], [m, n]]),
    ]:
        got = hip_run(hip, prog(build, [("Bf16", d) for d in dims]), arrays)[0]
        want = oracle_run(prog(build, [("F32", d) for d in dims]), arrays)[0]
        assert_close(got, want, atol=3e-2, rtol=2e-2, what=f"m={m} k={k} n={n}")


@pytest.mark.parametrize("m,k,n", [(8, 768, 2304), (16, 3072, 768), (16, 768, 50257), (5, 512, 40), (2, 64, 24), (3, 48, 16)])
def test_batched_decode_linear_f32_on_matrix_cores(hip, m, k, n):
    """2..16 f32 rows: the same kernel on v_mfma_f32_16x16x4_f32 (weights in groups of 4 k); the reference suite's
    tolerance (5e-4 + 1e-4 relative), plain, under LayerNorm + bias + exact GELU + residual, and as a SwiGLU pair."""
    x, w = rng_uniform(60, (m, k)), rng_uniform(61, (k, n)) * (2.0 / np.sqrt(k))
    b, r, g, be_ = rng_uniform(62, (n,)), rng_uniform(63, (m, n)), rng_uniform(64, (k,)) + 1.5, rng_uniform(65, (k,))
    w2 = rng_uniform(66, (k, n)) * (2.0 / np.sqrt(k))
    built = hip.counter("derived_weights_built")
    check_program(hip, prog(lambda fb, a, c: a.matmul(c), [("F32", [m, k]), ("F32", [k, n])]), [x, w])
    assert hip.counter("derived_weights_built") > built
    check_program(hip, prog(lambda fb, a, gm, bt, c, d, e: F.gelu(F.linear(F.layer_norm(a, gm, bt, 1e-5)[0], c, d)) + e,
                            [("F32", [m, k]), ("F32", [k]), ("F32", [k]), ("F32", [k, n]), ("F32", [n]), ("F32", [m, n])]), [x, g, be_, w, b, r])
    check_program(hip, prog(lambda fb, a, c, d: F.swiglu(a.matmul(c), a.matmul(d)), [("F32", [m, k]), ("F32", [k, n]), ("F32", [k, n])]),
                  [x, w, w2])


@pytest.mark.parametrize("m,k,n", [(8, 3072, 9216), (4, 256, 96), (16, 3072, 9216), (12, 512, 256)])
def test_batched_decode_norm_swiglu_on_matrix_cores(hip, m, k, n):
    r16 = lambda a: (f32_to_bf16_bits(np.asarray(a, np.float32)).astype(np.uint32) << 16).view(np.float32)  # noqa: E731
    x, g = r16(rng_uniform(54, (m, k)) * 3.0), r16(rng_uniform(55, (k,)) + 1.5)
    wg, wu = r16(rng_uniform(56, (k, n)) * (2.0 / np.sqrt(k))), r16(rng_uniform(57, (k, n)) * (2.0 / np.sqrt(k)))

    def build(fb, a, gm, c, d):
        h = F.rms_norm(a, gm, 1e-5)[0]
        return F.swiglu(h.matmul(c), h.matmul(d))

    dims = [[m, k], [k], [k, n], [k, n]]
    got = hip_run(hip, prog(build, [("Bf16", d) for d in dims]), [x, g, wg, wu])[0]
    want = oracle_run(prog(build, [("F32", d) for d in dims]), [x, g, wg, wu])[0]
    assert_close(got, want, atol=8e-2, rtol=4e-2, what=f"m={m} k={k} n={n}")


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
def test_temperature_sampling_matches_oracle(hip, dtype):
    """sample_decode_token with temperature > 0 (DecodeSampleRequest, spec.rs:1270-1284): the device kernel and the
    oracle restate the same Gumbel-max rule, so they must pick the same token whenever the two best scores are not
    within float noise of each other; the reference's own case (decode_sampling.rs:22-48) must land in range."""
    from parity import TensorSpec, po, to_bytes
    h = hip.materialize(TensorSpec("F32", [1, 4]), np.array([[0.1, 0.2, 0.3, 0.4]], np.float32).tobytes())
    assert 0 <= hip.sample_decode_token(h, temperature=0.8, random_u=0.42) < 4
    assert hip.sample_decode_token(h, temperature=0.8) is None                # no draw supplied: host sampler's job
    assert hip.sample_decode_token(h, temperature=0.8, top_k=2, random_u=0.42) is None
    rng = np.random.default_rng(8)
    agree = 0
    for case in range(24):
        vocab = int(rng.choice([5, 64, 1000, 50257, 131072]))
        rows = int(rng.integers(1, 4))
        logits = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
        if dtype == "Bf16":
            logits = (f32_to_bf16_bits(logits).astype(np.uint32) << 16).view(np.float32)
        temperature, u = float(rng.uniform(0.2, 1.5)), float(np.float32(rng.uniform(1e-6, 1 - 1e-6)))
        hh = hip.materialize(TensorSpec(dtype, [rows, vocab]), to_bytes(logits, dtype))
        got = hip.sample_decode_token(hh, temperature=temperature, random_u=u)
        want = po.sample_temperature(logits[-1], temperature, u)
        assert 0 <= got < vocab
        agree += got == want
    assert agree >= 23, f"device and oracle agree on {agree} of 24 draws"


@pytest.mark.parametrize("hq,hkv,dh,seq", [(4, 4, 32, 1), (4, 2, 32, 31), (8, 2, 32, 33), (4, 1, 64, 64), (12, 12, 64, 100),
                                           (8, 2, 128, 257), (32, 8, 128, 96), (8, 1, 64, 130)])
def test_attention_prefill_bf16_matrix_cores(hip, hq, hkv, dh, seq):
    """bf16 prefill attention on the MFMA kernel (head_dim 32/64/128; group sizes 1, 2, 4, 8; sequence lengths
    around the 32-row / 32-key tile edges) against the f32 oracle on the same bf16-representable input.  The kernel
    keeps f32 scores and sums and rounds the probabilities to bf16 for the P.V product; the result is stored as bf16."""
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    P = cfg.total_projection_dim
    qkv = rng_uniform(33, (seq, P))
    qkv = (f32_to_bf16_bits(qkv).astype(np.uint32) << 16).view(np.float32)
    got = hip_run(hip, prog(lambda fb, a: list(F.attention(cfg, a, None)), [("Bf16", [seq, P])]), [qkv])
    want = oracle_run(prog(lambda fb, a: list(F.attention(cfg, a, None)), [("F32", [seq, P])]), [qkv])
    assert_close(got[0], want[0], atol=1e-2, rtol=1e-2, what="context")
    for i in (1, 2):   # K and V in cache layout: pure copies
        assert np.array_equal(np.asarray(got[i], np.float32), want[i])


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("hq,hkv,dh,seq,clen", [(4, 2, 4, 3, 4), (3, 3, 2, 4, 1), (4, 4, 8, 1, 9), (4, 1, 4, 5, 70), (8, 2, 16, 33, 100),
                                                (12, 12, 64, 2, 130), (32, 8, 128, 5, 64)])
def test_attention_with_concat_cache(hip, dtype, hq, hkv, dh, seq, clen):
    """attention.rs:359-437 (`cache = Some`): new rows behind a growing cache, in one fused step (two launches: the
    combined caches, then the attention over them).  Context against the oracle's op-by-op evaluation; the combined caches
    are copies and must be exact; the fused row i equals what the prefill of all clen + seq rows gives at row clen + i."""
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    P = cfg.total_projection_dim
    r16 = (lambda a: a) if dtype == "F32" else (lambda a: (f32_to_bf16_bits(np.asarray(a, np.float32)).astype(np.uint32) << 16).view(np.float32))
    qkv_all = r16(rng_uniform(27, (clen + seq, P)))
    # the cache holds the K / V rows of the first clen tokens
    k_full = qkv_all[:, hq * dh:(hq + hkv) * dh].reshape(clen + seq, hkv, dh).transpose(1, 0, 2)
    v_full = qkv_all[:, (hq + hkv) * dh:].reshape(clen + seq, hkv, dh).transpose(1, 0, 2)
    ck, cv = np.ascontiguousarray(k_full[:, :clen]), np.ascontiguousarray(v_full[:, :clen])
    qkv = np.ascontiguousarray(qkv_all[clen:])
    build = lambda fb, a, k, v: list(F.attention(cfg, a, (k, v)))  # noqa: E731
    specs = lambda dt: [(dt, [seq, P]), (dt, [hkv, clen, dh]), (dt, [hkv, clen, dh])]  # noqa: E731
    fused0 = hip.counter("fused_ops")
    got = hip_run(hip, prog(build, specs(dtype)), [qkv, ck, cv])
    assert hip.counter("fused_ops") > fused0 and hip.counter("last_program_launches") == 2, "one fused step"
    want = oracle_run(prog(build, specs("F32")), [qkv, ck, cv])
    tol = dict() if dtype == "F32" else dict(atol=2e-2, rtol=2e-2)
    assert_close(got[0], want[0], what="context", **tol)
    assert np.array_equal(np.asarray(got[1], np.float32), k_full) and np.array_equal(np.asarray(got[2], np.float32), v_full)
    whole = oracle_run(prog(lambda fb, a: list(F.attention(cfg, a, None)), [("F32", [clen + seq, P])]), [qkv_all])
    assert_close(got[0], whole[0][clen:], what="rows of the whole prefill", **tol)
    # fusion off: the same program op by op, same results to the same bar
    hip.set_option("fusion", 0)
    try:
        plain = hip_run(hip, prog(build, specs(dtype)), [qkv, ck, cv])
    finally:
        hip.set_option("fusion", 1)
    assert_close(plain[0], want[0], what="context, op by op", **tol)


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("hq,hkv,dh,cap", [(4, 4, 8, 16), (4, 2, 8, 32), (8, 2, 16, 128), (12, 12, 64, 128), (32, 8, 128, 256), (4, 4, 1, 8), (6, 2, 4, 16),
                                           (8, 2, 128, 2048), (16, 2, 64, 1024), (4, 2, 64, 640), (24, 2, 64, 64)])
def test_attention_decode_cache(hip, dtype, hq, hkv, dh, cap):
    cfg = F.AttentionConfig(hq * dh, hq, hkv, dh)
    P = cfg.total_projection_dim
    specs = [(dtype, [1, P]), (dtype, [hkv, cap, dh]), (dtype, [hkv, cap, dh]), ("Si32", [3]), ("Si32", [1])]
    p = prog(lambda fb, a, k, v, us, qs: list(F.attention_decode_cache(cfg, a, k, v, us, qs)), specs)
    tol = dict() if dtype == "F32" else dict(atol=3e-2, rtol=3e-2)
    for pos in (0, 1, cap // 2, cap - 1):
        qkv = rng_uniform(30 + pos, (1, P))
        ck, cv = rng_uniform(31, (hkv, cap, dh)), rng_uniform(32, (hkv, cap, dh))
        # stale garbage beyond the valid length must not matter (capacity-independence)
        ck[:, pos + 1:], cv[:, pos + 1:] = 1e3, -1e3
        check_program(hip, p, [qkv, ck, cv, np.array([0, pos, 0], np.int32), np.array([pos], np.int32)], **tol)


def test_decode_equals_prefill_row(hip):
    # attention_prefill4_decode3 == full (crates/gpt-rs-backend-tests/src/lib.rs:231-232)
    cfg = F.AttentionConfig(32, 4, 2, 8)
    P, T, cap = cfg.total_projection_dim, 7, 16
    qkv = rng_uniform(40, (T, P))
    full = prog(lambda fb, a: list(F.attention(cfg, a, None)), [("F32", [T, P])])
    ctx_full, k_full, v_full = hip_run(hip, full, [qkv])
    dec = prog(lambda fb, a, k, v, us, qs: list(F.attention_decode_cache(cfg, a, k, v, us, qs)),
               [("F32", [1, P]), ("F32", [2, cap, 8]), ("F32", [2, cap, 8]), ("Si32", [3]), ("Si32", [1])])
    ck = np.zeros((2, cap, 8), np.float32)
    cv = np.zeros((2, cap, 8), np.float32)
    ck[:, :4], cv[:, :4] = k_full[:, :4], v_full[:, :4]
    for pos in range(4, T):
        ctx, ck, cv = hip_run(hip, dec, [qkv[pos:pos + 1], ck, cv, np.array([0, pos, 0], np.int32), np.array([pos], np.int32)])
        assert_close(ctx[0], ctx_full[pos], what=f"decode row {pos}")
    assert_close(ck[:, :T], k_full)


# ------------------------------------------------------------------ execute_instruction
def test_execute_instruction_single_ops(hip):
    """PortableBackend::execute_instruction (spec.rs:1317): one instruction, operands positional.  Take (the embedding
    gather, bit-exact), DotGeneral (the reference-held 2x2 vector, smoke.rs:12-24), DynamicUpdateSlice with a clamped
    start (dynamic_ops_gpu.rs:35-104), a literal operand, and an operand that repeats."""
    import json
    from gptrs_amd.backend import BackendError
    from gptrs_amd.ptir import TensorSpec

    def instr_of(build, specs):
        p = prog(build, specs)
        body = p.obj["functions"][0]["body"]
        return p, json.dumps(body[-1], separators=(",", ":")).encode()

    def mat(dtype, arr):
        arr = np.asarray(arr)
        return hip.materialize(TensorSpec(dtype, arr.shape), arr)

    # Take
    table = np.arange(40, dtype=np.float32).reshape(10, 4)
    idx = np.array([7, 0, 7, 9], np.int32)
    p, js = instr_of(lambda fb, t, i: t.take(i), [("F32", [10, 4]), ("Si32", [4])])
    out = hip.execute_instruction(js, [mat("F32", table), mat("Si32", idx)])
    assert np.array_equal(hip.to_numpy(out), oracle_run(p, [table, idx])[0]) and np.array_equal(hip.to_numpy(out), table[idx])
    # DotGeneral: [[1,2],[3,4]] . [[5,6],[7,8]] = [[19,22],[43,50]]
    a, b = np.array([[1, 2], [3, 4]], np.float32), np.array([[5, 6], [7, 8]], np.float32)
    p, js = instr_of(lambda fb, x, y: x.matmul(y), [("F32", [2, 2]), ("F32", [2, 2])])
    assert hip.to_numpy(hip.execute_instruction(js, [mat("F32", a), mat("F32", b)])).tolist() == [[19, 22], [43, 50]]
    # DynamicUpdateSlice, start 8 clamps to 3
    p, js = instr_of(lambda fb, base, u, s: base.dynamic_update_slice(u, s, [2]), [("F32", [5]), ("F32", [2]), ("Si32", [1])])
    base_h = mat("F32", np.array([10, 11, 12, 13, 14], np.float32))
    out = hip.execute_instruction(js, [base_h, mat("F32", np.array([99, 88], np.float32)), mat("Si32", np.array([8], np.int32))])
    assert hip.to_numpy(out).tolist() == [10, 11, 12, 99, 88] and hip.to_numpy(base_h).tolist() == [10, 11, 12, 13, 14]
    # a literal operand travels inside the JSON: BroadcastTo(Literal 1.0)
    p, js = instr_of(lambda fb, x: x + 1.0, [("F32", [4])])
    lit = json.dumps(p.obj["functions"][0]["body"][0], separators=(",", ":")).encode()
    assert hip.to_numpy(hip.execute_instruction(lit, [])).tolist() == [1, 1, 1, 1]
    # one value on both sides of a product
    p, js = instr_of(lambda fb, x: x * x, [("F32", [4])])
    h = mat("F32", np.array([1, 2, 3, 4], np.float32))
    assert hip.to_numpy(hip.execute_instruction(js, [h, h])).tolist() == [1, 4, 9, 16]
    with pytest.raises(BackendError):
        hip.execute_instruction(js, [h])              # fewer inputs than Value operands


# ------------------------------------------------------------------ error surface
def test_unknown_custom_call_is_unimplemented(hip):
    from gptrs_amd.backend import BackendError
    from gptrs_amd.ptir import TensorSpec
    p = prog(lambda fb, a: fb.custom_call("gpt_rs.nobody.knows.v1", [a], TensorSpec("F32", [4])), [("F32", [4])])
    with pytest.raises(BackendError) as ei:
        hip_run(hip, p, [np.zeros(4, np.float32)])
    assert ei.value.kind == "unimplemented"


def test_wrong_spec_version_and_arity(hip):
    from gptrs_amd.backend import BackendError
    from gptrs_amd.ptir import TensorSpec
    p = prog(lambda fb, a: a + 1.0, [("F32", [4])])
    js = p.json_bytes.replace(b"ptir.v0.4", b"ptir.v0.3")
    h = hip.materialize(TensorSpec("F32", [4]), np.zeros(4, np.float32))
    with pytest.raises(BackendError) as ei:
        hip.run_program_json(js, 0, [h], 1)
    assert ei.value.kind == "spec"
    with pytest.raises(BackendError) as ei:
        hip.run_program_json(p.json_bytes, 0, [h, h], 1)
    assert "arity" in str(ei.value)
    h2 = hip.materialize(TensorSpec("F32", [5]), np.zeros(5, np.float32))
    with pytest.raises(BackendError):
        hip.run_program_json(p.json_bytes, 0, [h2], 1)


def test_inputs_unchanged_without_donation(hip):
    from gptrs_amd.ptir import TensorSpec
    p = prog(lambda fb, b, u, s: b.dynamic_update_slice(u, s, [2]), [("F32", [5]), ("F32", [2]), ("Si32", [1])])
    base = hip.materialize(TensorSpec("F32", [5]), np.arange(5, dtype=np.float32))
    upd = hip.materialize(TensorSpec("F32", [2]), np.array([9, 9], np.float32))
    st = hip.materialize(TensorSpec("Si32", [1]), np.array([1], np.int32))
    out = hip.run_program(p, [base, upd, st])[0]
    assert hip.to_numpy(out).tolist() == [0, 9, 9, 3, 4]
    assert hip.to_numpy(base).tolist() == [0, 1, 2, 3, 4]
    # donated: the update happens in place and the input handle is consumed
    before = hip.counter("inplace_updates")
    out2 = hip.run_program(p, [base, upd, st], [True, False, False])[0]
    assert hip.to_numpy(out2).tolist() == [0, 9, 9, 3, 4]
    assert hip.counter("inplace_updates") == before + 1
    from gptrs_amd.backend import BackendError
    with pytest.raises(BackendError):
        hip.to_numpy(base)


def test_drop_derived_weights_frees_memory_and_results_stay(hip):
    """The re-ordered weight copies are built at first use and can be given back: a decode-shaped and a prefill-shaped
    linear over the same weight each build one, "drop_derived_weights" frees both (device bytes go down by at least their
    size), and the same programs give the same bits afterwards (the copies are rebuilt)."""
    from parity import FunctionBuilder, Program, hip_run
    k, n = 1024, 4096
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((k, n)) * 0.03).astype(np.float32)
    x1 = rng.standard_normal((1, k)).astype(np.float32)
    xm = rng.standard_normal((64, k)).astype(np.float32)

    def prog(m):
        fb = FunctionBuilder("main")
        a, b = fb.param("Bf16", [m, k]), fb.param("Bf16", [k, n])
        fb.set_results([a.matmul(b)])
        return Program(fb)

    from parity import to_bytes
    p1, pm = prog(1), prog(64)
    hw = hip.materialize(p1.param_specs[1], to_bytes(w, "Bf16"))
    h1 = hip.materialize(p1.param_specs[0], to_bytes(x1, "Bf16"))
    hm = hip.materialize(pm.param_specs[0], to_bytes(xm, "Bf16"))
    built = hip.counter("derived_weights_built")
    hip.set_option("evict_packed_weights", 0)   # so that the bytes counted below are those of the copies alone
    try:
        y1 = hip.to_numpy(hip.run_program(p1, [h1, hw])[0])
        ym = hip.to_numpy(hip.run_program(pm, [hm, hw])[0])
        assert hip.counter("derived_weights_built") == built + 2
        before = hip.counter("bytes_allocated")
        hip.set_option("drop_derived_weights", 1)
        after = hip.counter("bytes_allocated")
        assert before - after >= 2 * k * n * 2, f"two bf16 copies of {k} x {n} expected back, got {before - after} bytes"
        z1 = hip.to_numpy(hip.run_program(p1, [h1, hw])[0])
        zm = hip.to_numpy(hip.run_program(pm, [hm, hw])[0])
    finally:
        hip.set_option("evict_packed_weights", 1)
    assert hip.counter("derived_weights_built") == built + 4
    assert np.array_equal(np.asarray(y1), np.asarray(z1)) and np.array_equal(np.asarray(ym), np.asarray(zm))


@pytest.mark.parametrize("dtype", ["F32", "Bf16"])
@pytest.mark.parametrize("m,k,n", [(64, 3072, 768), (48, 1024, 200), (100, 2048, 64)])
def test_few_tile_gemm_splits_k_and_is_reproducible(hip, dtype, m, k, n):
    """A prefill-shaped linear with few 64 x 64 tiles splits every tile over k between workgroups (partial sums through a
    workspace, a ticket per tile, the last ticket adds them in split order): the result matches the oracle and two runs
    give the same bits whichever workgroup drew the last ticket."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    b = rng.standard_normal((n,)).astype(np.float32)
    if dtype == "Bf16":
        x, w, b = (bf16_bits_to_f32(f32_to_bf16_bits(a)) for a in (x, w, b))
    fb = FunctionBuilder("main")
    a, c, d = fb.param(dtype, [m, k]), fb.param(dtype, [k, n]), fb.param(dtype, [n])
    fb.set_results([F.linear(a, c, d)])
    p = Program(fb)
    (want,) = oracle_run(p, [x, w, b])
    (got,) = hip_run(hip, p, [x, w, b])
    (again,) = hip_run(hip, p, [x, w, b])
    assert np.array_equal(np.asarray(got), np.asarray(again)), "split-k sums must not depend on the arrival order"
    if dtype == "F32":
        assert_close(got, want, atol=2e-4, rtol=1e-4, what="few-tile f32 linear")
    else:
        assert_close(got, want, atol=1e-2, rtol=2.0 ** -7, what="few-tile bf16 linear")
