"""The host sampler (crates/gpt-rs/src/inference/sampler.rs:7-104) and the generation loop's use of it, on the CPU.

The reference has no test of its sampler and draws from `thread_rng()`, so nothing of its random stream can be pinned.
What the code fixes is checked against what the mathematics fixes: the arg-max rule of `Iterator::max_by` (last of equal
maxima), the top-k threshold (k-th largest value, ties kept) against a sort, the weights against a float64 softmax, the
fall-back cases, the draw against the inverse of the cumulative weights, and the frequencies of many draws against the
weights."""
import numpy as np
import pytest

import __graft_entry__ as entry

entry.load_package()
from gptrs_amd import models  # noqa: E402
from gptrs_amd.models import Sampler  # noqa: E402
from oracle_backend import OracleBackend  # noqa: E402


def test_argmax_is_the_last_of_equal_maxima():
    assert Sampler.argmax(np.array([1.0, 3.0, 2.0, 3.0, 0.0], np.float32)) == 3
    assert Sampler.argmax(np.array([5.0], np.float32)) == 0
    assert Sampler.argmax(np.zeros(7, np.float32)) == 6
    assert Sampler(0.0).sample(np.array([0.5, 2.0, 2.0], np.float32), np.random.default_rng(0)) == 2
    assert Sampler(-1.0, top_k=2).sample(np.array([4.0, 2.0, 1.0], np.float32), np.random.default_rng(0)) == 0
    with pytest.raises(ValueError, match="empty logits"):
        Sampler(1.0).sample(np.zeros(0, np.float32), np.random.default_rng(0))


@pytest.mark.parametrize("k", [1, 2, 3, 5, 8, 9, 50])
def test_top_k_threshold_against_a_sort(k):
    rng = np.random.default_rng(k)
    row = rng.standard_normal(9).astype(np.float32)
    row[4] = row[2]                       # a tie: both stay or both go
    s = Sampler(0.7, top_k=k)
    adj = s.adjusted(row)
    scaled = (row / np.float32(0.7)).astype(np.float32)
    if k >= row.size:
        assert np.array_equal(adj, scaled)
    else:
        kth = np.sort(scaled)[::-1][k - 1]
        assert np.array_equal(np.isfinite(adj), scaled >= kth)
        assert np.array_equal(adj[np.isfinite(adj)], scaled[scaled >= kth])
        assert np.isfinite(adj).sum() >= k
    assert Sampler(1.0, top_k=0).top_k == 1   # with_top_k: k.max(1)


def test_weights_are_the_softmax_of_the_kept_values():
    rng = np.random.default_rng(3)
    row = (3.0 * rng.standard_normal(1000)).astype(np.float32)
    for temp, k in [(1.0, None), (0.5, None), (2.0, 40), (0.8, 1)]:
        p = Sampler(temp, k).probabilities(row)
        x = row.astype(np.float64) / temp
        if k is not None:
            kth = np.sort(x)[::-1][k - 1]
            x = np.where(x < kth, -np.inf, x)
        want = np.exp(x - x.max())
        want /= want.sum()
        assert p.dtype == np.float32 and np.max(np.abs(p - want)) < 1e-6
        assert abs(float(p.sum(dtype=np.float64)) - 1.0) < 1e-4
        if k is not None:
            assert np.count_nonzero(p) == k


def test_fall_back_to_argmax_when_the_weights_do_not_sum():
    row = np.array([1.0, np.inf, 2.0], np.float32)          # inf - inf = nan in the shifted row
    assert Sampler(1.0).probabilities(row) is None
    assert Sampler(1.0).sample(row, np.random.default_rng(0)) == 1
    nan_row = np.array([np.nan, 1.0, 2.0], np.float32)
    assert Sampler(1.0).probabilities(nan_row) is None


def test_the_draw_inverts_the_cumulative_weights():
    row = np.log(np.array([0.1, 0.2, 0.3, 0.4], np.float64)).astype(np.float32)
    s = Sampler(1.0)
    cum = np.cumsum(s.probabilities(row), dtype=np.float32)

    class Fixed:
        def __init__(self, x): self.x = x
        def uniform(self, lo, hi): return self.x
    for x, want in [(0.0, 0), (0.05, 0), (float(cum[0]), 1), (0.25, 1), (0.31, 2), (0.61, 3), (0.999, 3)]:
        assert s.sample(row, Fixed(x)) == want, x


def test_frequencies_follow_the_weights():
    row = np.array([2.0, 1.0, 0.0, -1.0, 3.0, 0.5], np.float32)
    s = Sampler(0.9, top_k=4)
    p = s.probabilities(row).astype(np.float64)
    rng = np.random.default_rng(11)
    n = 40000
    counts = np.bincount([s.sample(row, rng) for _ in range(n)], minlength=row.size)
    assert counts[p == 0].sum() == 0
    # every frequency within five standard deviations of its expectation
    assert np.all(np.abs(counts - n * p) <= 5.0 * np.sqrt(n * p * (1 - p)) + 1e-9)


def test_decode_sample_request():
    rng = np.random.default_rng(5)
    assert Sampler(0.0).decode_sample_request(rng) == {"temperature": 0.0, "top_k": None, "random_u": None}
    assert Sampler(0.7, top_k=5).decode_sample_request(rng) is None and not Sampler(0.7, top_k=5).supports_backend_decode_sampling()
    eps = float(np.finfo(np.float32).eps)
    for _ in range(100):
        r = Sampler(0.7).decode_sample_request(rng)
        assert r["temperature"] == pytest.approx(0.7) and r["top_k"] is None and eps <= r["random_u"] < 1.0


TINY = models.GptConfig(vocab_size=48, context_length=32, embed_dim=16, num_layers=2, num_heads=2, mlp_ratio=2)


def test_generator_with_top_k_samples_on_the_host():
    be = OracleBackend()
    m = models.Gpt.random(TINY, be, seed=2, std=0.3)
    prompt = [3, 9, 4]
    greedy = models.Generator(m, prompt).generate(10)
    # k = 1 leaves one token with weight 1: the greedy continuation, whatever the draws
    assert models.Generator(m, prompt, temperature=0.8, top_k=1, seed=7).generate(10) == greedy
    g = models.Generator(m, prompt, temperature=1.5, top_k=5, seed=7)
    assert not g.device_sampling and not g.pipelined
    toks = g.generate(12)
    assert toks == models.Generator(m, prompt, temperature=1.5, top_k=5, seed=7).generate(12), "same seed, same tokens"
    assert toks != models.Generator(m, prompt, temperature=1.5, top_k=5, seed=8).generate(12)
    # every sampled token is one of the five most likely of its step
    g2 = models.Generator(m, prompt, temperature=1.5, top_k=5, seed=7)
    for t in toks:
        row = be.to_numpy(g2.logits)[-1]
        assert t in np.argsort(row)[::-1][:5]
        g2.step()
    with pytest.raises(ValueError, match="top-k is sampled on the host"):
        models.Generator(m, prompt, temperature=1.0, top_k=3, pipelined=True)


def test_generator_falls_back_to_the_host_sampler_when_the_backend_declines():
    class Declines(OracleBackend):
        def sample_decode_token(self, logits, temperature=0.0, top_k=None, random_u=None):
            return None
    m = models.Gpt.random(TINY, Declines(), seed=2, std=0.3)
    m_ref = models.Gpt.random(TINY, OracleBackend(), seed=2, std=0.3)
    assert models.Generator(m, [3, 9, 4]).generate(8) == models.Generator(m_ref, [3, 9, 4]).generate(8)
    assert len(models.Generator(m, [3, 9, 4], temperature=0.9, seed=1).generate(8)) == 8


def test_a_draw_that_rounds_up_to_the_total_never_picks_a_zero_weight_token():
    """WeightedIndex samples in [0, total) (sampler.rs:52-72): a uniform draw whose f32 rounding reaches `total` must not
    fall behind the last cumulative weight, where the clamp would pick the last index whatever its weight."""
    class Top:
        """A generator whose uniform draw is the largest double below `high`."""
        def uniform(self, low, high):
            return float(np.nextafter(high, low))

    s = Sampler(1.0, top_k=2)
    row = np.array([3.0, 2.5, -1.0, -2.0, -3.0], np.float32)   # top-2 masks the last three: their weight is exactly 0
    probs = s.probabilities(row)
    assert probs[-1] == 0.0 and probs[2] == 0.0
    assert s.sample(row, Top()) in (0, 1)
