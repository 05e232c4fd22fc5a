"""Weight streaming through `loader.load_model` (the reference's runtime/loader.rs:19-434) on the CPU oracle backend.

The four behavioural cases are the reference's own tests (crates/gpt-rs/tests/runtime_weight_streaming_loader.rs:294-381):
a backend that counts `materialize` calls, a one-layer GPT (vocab 32, context 16, width 8, two heads, mlp ratio 2), the
same four tokens forwarded twice, and the counts of the two forwards compared between runtime configurations.  The cache
itself (budget, pinning, eviction order) and the budget arithmetic are pinned against hand-worked cases."""
import numpy as np
import pytest

import __graft_entry__ as entry

entry.load_package()
from gptrs_amd import loader, models  # noqa: E402
from gptrs_amd.checkpoint import Checkpoint, Entry  # noqa: E402
from gptrs_amd.loader import (ParamHandleCache, SourceCacheConfig, WeightStreamingConfig, block_layer_index,  # noqa: E402
                              effective_cache_budget_bytes, effective_device_budget_bytes, prefetch_block_base_ids,
                              source_cache_config, validate_weight_streaming_config)
from oracle_backend import OracleBackend  # noqa: E402


class CountingBackend(OracleBackend):
    """runtime_weight_streaming_loader.rs:44-111: counts materialize calls."""

    def __init__(self):
        super().__init__()
        self.materialize_calls = 0

    def materialize(self, spec, data):
        self.materialize_calls += 1
        return super().materialize(spec, data)


SMALL = models.GptConfig(vocab_size=32, context_length=16, embed_dim=8, num_layers=1, num_heads=2, mlp_ratio=2)
TOKENS = [1, 2, 3, 4]


def save_small(tmp_path, ws: WeightStreamingConfig, name="m.bin", cfg=SMALL):
    m = models.Gpt.random(cfg, OracleBackend(), seed=7)
    path = str(tmp_path / name)
    m.save_checkpoint(path, "gpt", m.checkpoint_config(), runtime={"weight_streaming": ws.to_json()} if ws != WeightStreamingConfig() else None)
    return path, m


def run_case(tmp_path, ws: WeightStreamingConfig):
    """(materialize calls of the first forward, of the second) after load_model, as the reference's run_case."""
    path, _ = save_small(tmp_path, ws)
    be = CountingBackend()
    model = loader.load_model(be, path)
    deltas = []
    for _ in range(2):
        before = be.materialize_calls
        model.forward_with_decode_cache(TOKENS, 0, [None] * SMALL.num_layers)
        deltas.append(be.materialize_calls - before)
    return deltas[0], deltas[1], model


def test_default_runtime_avoids_streaming_reload_penalty_across_forwards(tmp_path):
    first, second, _ = run_case(tmp_path, WeightStreamingConfig())
    assert second <= first


def test_streaming_without_budget_reloads_more_than_default_runtime(tmp_path):
    _, default_second, _ = run_case(tmp_path, WeightStreamingConfig())
    first, second, model = run_case(tmp_path, WeightStreamingConfig(enabled=True))
    assert second >= first // 2, "a streamed second forward stays expensive without a cache budget"
    assert second > default_second
    assert second - default_second == len(model.param_names), "every parameter is loaded again, and nothing else"


def test_budget_and_host_cap_change_streaming_reload_behavior(tmp_path):
    _, no_cache_second, _ = run_case(tmp_path, WeightStreamingConfig(enabled=True))
    _, large_second, _ = run_case(tmp_path, WeightStreamingConfig(enabled=True, device_budget_bytes=1_000_000_000))
    _, host_second, _ = run_case(tmp_path, WeightStreamingConfig(enabled=True, device_budget_bytes=1_000_000_000, cache_budget_cap_bytes=1))
    assert large_second < no_cache_second, "a large device budget keeps the weights between forwards"
    assert host_second >= large_second, "a one-byte cache cap undoes that"
    assert host_second == no_cache_second


def test_prefetch_layers_reduce_streaming_first_forward_materialization(tmp_path):
    first, second, _ = run_case(tmp_path, WeightStreamingConfig(enabled=True))
    p_first, p_second, model = run_case(tmp_path, WeightStreamingConfig(enabled=True, prefetch_layers=1))
    assert p_first < first and p_second <= second
    n_block = sum(1 for n in model.param_names if n.startswith("blocks.0."))
    assert first - p_first == n_block, "exactly the tensors of blocks.0 were there before the first forward"


def test_streamed_model_computes_what_the_resident_model_computes(tmp_path):
    path, ref = save_small(tmp_path, WeightStreamingConfig(enabled=True, small_param_persist_threshold=64), "s.bin")
    want = ref.backend.to_numpy(ref.forward_with_decode_cache(TOKENS, 0, [None]))
    for be in (CountingBackend(),):
        m = loader.load_model(be, path)
        assert m._lazy and m._source.cache.cfg.small_param_persist_threshold == 64
        got = be.to_numpy(m.forward_with_decode_cache(TOKENS, 0, [None]))
        assert np.array_equal(got, want)
        # tensors of at most 64 bytes (the width-8 vectors: 32 bytes) are pinned after their first load
        pinned = {bid for bid, e in m._source.cache.entries.items() if e.pinned}
        small = {m._base_ids[n] for n in m.param_names if int(np.prod(m.param_specs[n].dims)) * 4 <= 64}
        assert pinned == small and small
        before = m._source.loads
        m.forward_with_decode_cache(TOKENS, 0, [None])
        assert m._source.loads - before == len(m.param_names) - len(small), "only the large tensors are loaded again"


def test_knobs_without_enabled_are_rejected(tmp_path):
    with pytest.raises(ValueError, match="enabled=false but streaming knobs are set"):
        validate_weight_streaming_config(WeightStreamingConfig(device_budget_bytes=10))
    with pytest.raises(ValueError, match=r"device_weights_percent must be in \[0.0, 1.0\]"):
        validate_weight_streaming_config(WeightStreamingConfig(enabled=True, device_weights_percent=1.5))
    validate_weight_streaming_config(WeightStreamingConfig(enabled=True, device_weights_percent=0.25, prefetch_layers=2))
    path, _ = save_small(tmp_path, WeightStreamingConfig())
    # a checkpoint whose runtime section sets a knob but not `enabled`
    m = models.Gpt.random(SMALL, OracleBackend(), seed=7)
    bad = str(tmp_path / "bad.bin")
    m.save_checkpoint(bad, "gpt", m.checkpoint_config(), runtime={"weight_streaming": {"enabled": False, "prefetch_layers": 1}})
    with pytest.raises(ValueError, match="streaming knobs are set"):
        loader.load_model(OracleBackend(), bad)
    with Checkpoint(path) as ck:
        assert ck.runtime is None


def E(name, nbytes, base_id=0):
    return Entry(name, base_id, (nbytes // 4,), 0, 0, 0, nbytes)


def test_budget_arithmetic():
    """loader.rs:342-368, 422-434 on hand-worked numbers: total 1000 bytes."""
    entries = [E("a", 400), E("b", 600)]
    ws = WeightStreamingConfig
    assert effective_device_budget_bytes(entries, ws(enabled=True)) is None
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_budget_bytes=700)) == 700
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_weights_percent=0.25)) == 250
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_weights_percent=1.0)) == 1000
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_weights_percent=0.0)) == 0
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_budget_bytes=100, device_weights_percent=0.5)) == 100
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_budget_bytes=900, device_weights_percent=0.5)) == 500
    # the percentage is an f32 in the reference: 0.3f32 = 0.300000011920929 -> floor(1000 * that) = 300
    assert effective_device_budget_bytes(entries, ws(enabled=True, device_weights_percent=0.3)) == 300
    assert effective_cache_budget_bytes(entries, ws(enabled=True, cache_budget_cap_bytes=50)) == 50
    assert effective_cache_budget_bytes(entries, ws(enabled=True, device_budget_bytes=700, cache_budget_cap_bytes=50)) == 50
    assert effective_cache_budget_bytes(entries, ws(enabled=True, device_budget_bytes=20, cache_budget_cap_bytes=50)) == 20
    assert effective_cache_budget_bytes(entries, ws(enabled=True)) is None


def test_block_layer_index_and_prefetch_ids():
    assert block_layer_index("blocks.0.attention.w_qkv") == 0
    assert block_layer_index("blocks.12.norm_1.gamma") == 12
    for name in ("tok_embeddings.weight", "blocks.x.w", "blocks.3", "blocks..w", "xblocks.1.w", "blocks.-1.w"):
        assert block_layer_index(name) is None
    entries = [E("blocks.0.w", 8, 11), E("blocks.1.w", 8, 12), E("blocks.2.w", 8, 13), E("lm_head", 8, 14)]
    assert prefetch_block_base_ids(entries, None) == set()
    assert prefetch_block_base_ids(entries, 0) == set()
    assert prefetch_block_base_ids(entries, 2) == {11, 12}
    cfg = source_cache_config(entries, WeightStreamingConfig(enabled=True, prefetch_layers=1))
    assert cfg.enabled and cfg.budget_bytes is None and cfg.prefetch_base_ids == {11}
    assert not source_cache_config(entries, WeightStreamingConfig(enabled=True)).enabled
    assert not source_cache_config(entries, WeightStreamingConfig()).enabled


def test_cache_budget_pinning_and_eviction_order():
    """loader.rs:47-161.  Budget 100 bytes, tensors 1..5 of 40 bytes, id 9 of 8 bytes pinned by the small-tensor rule."""
    c = ParamHandleCache(SourceCacheConfig(enabled=True, budget_bytes=100, small_param_persist_threshold=8))
    c.insert(9, 8, "h9")
    assert c.entries[9].pinned and c.cached_bytes == 8
    c.insert(1, 40, "h1")
    c.insert(2, 40, "h2")
    assert c.cached_bytes == 88
    assert c.get(1) == "h1"                      # 1 is now the more recently used of the two
    c.insert(3, 40, "h3")                        # 88 + 40 > 100: evicts 2 (least recently used, unpinned)
    assert set(c.entries) == {9, 1, 3} and c.cached_bytes == 88
    c.insert(4, 101, "h4")                       # larger than the budget: not cached at all
    assert 4 not in c.entries
    c.insert(3, 40, "h3b")                       # re-insert replaces the handle, keeps the bytes
    assert c.entries[3].handle == "h3b" and c.cached_bytes == 88
    assert c.get(7) is None
    # pinned bytes count against the budget: 8 pinned + 96 does not fit, so nothing is evicted for it either
    c.insert(5, 96, "h5")
    assert 5 not in c.entries and set(c.entries) == {9, 1, 3}
    # ties on last use go to the smaller id (only reachable through equal ticks; forced here)
    c.entries[1].last_used = c.entries[3].last_used = 5
    c.insert(6, 40, "h6")
    assert set(c.entries) == {9, 3, 6}
    # a disabled cache stores and returns nothing
    d = ParamHandleCache(SourceCacheConfig())
    d.insert(1, 4, "x")
    assert d.get(1) is None and not d.entries
    # without a budget only prefetched ids and small tensors are kept
    s = ParamHandleCache(SourceCacheConfig(enabled=True, small_param_persist_threshold=8, prefetch_base_ids={5}))
    s.insert(1, 40, "big")
    s.insert(2, 8, "small")
    s.insert(5, 4000, "prefetched")
    assert set(s.entries) == {2, 5} and all(e.pinned for e in s.entries.values())
