"""Model loading with weight streaming: the reference's `runtime::load_model`
(crates/gpt-rs/src/runtime/loader.rs:19-434).

A checkpoint's config may carry `runtime.weight_streaming` (model/config.rs:5-29).  Without it every tensor is
materialised once and lives in the backend's parameter memo, as `Gpt/Ministral.from_checkpoint` do.  With
`enabled: true` the model holds no handles of its own: every forward asks the `CheckpointParamSource` for each
parameter by its base id, the source reads the bytes out of the file mapping and materialises them, and a
`ParamHandleCache` decides what stays on the device between forwards:

* `device_budget_bytes` / `device_weights_percent` (the smaller of the two) and `cache_budget_cap_bytes` cap the bytes of
  cached handles (loader.rs:342-368, 422-434); the least recently used unpinned entry goes first, ties by the smaller
  base id (loader.rs:135-154);
* `small_param_persist_threshold`: tensors of at most that many bytes are cached and pinned (never evicted);
* `prefetch_layers = n`: the tensors of `blocks.0 .. blocks.(n-1)` are materialised when the model is opened and pinned
  (loader.rs:186-215, 392-420).

A streamed weight is a new device buffer each time it is loaded, so the backend's derived layouts of it are rebuilt as
well: streaming trades time for memory, as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Iterable, List, Optional, Set

import numpy as np

from .checkpoint import Checkpoint, CheckpointError, Entry
from .ptir import TensorSpec, bf16_bits_to_f32, f32_to_bf16_bits


@dataclass
class WeightStreamingConfig:
    """model/config.rs:5-18."""

    enabled: bool = False
    device_budget_bytes: Optional[int] = None
    device_weights_percent: Optional[float] = None
    cache_budget_cap_bytes: Optional[int] = None
    prefetch_layers: Optional[int] = None
    small_param_persist_threshold: Optional[int] = None

    @classmethod
    def from_runtime(cls, runtime: Optional[dict]) -> "WeightStreamingConfig":
        ws = (runtime or {}).get("weight_streaming") or {}
        known = {f: ws[f] for f in cls.__dataclass_fields__ if f in ws and ws[f] is not None}
        return cls(**known)

    def to_json(self) -> dict:
        out = {"enabled": bool(self.enabled)}
        for f in ("device_budget_bytes", "device_weights_percent", "cache_budget_cap_bytes", "prefetch_layers",
                  "small_param_persist_threshold"):
            if getattr(self, f) is not None:
                out[f] = getattr(self, f)
        return out


def validate_weight_streaming_config(cfg: WeightStreamingConfig) -> None:
    """loader.rs:322-340: knobs without `enabled` are an error, the percentage lies in [0, 1]."""
    has_knob = any(getattr(cfg, f) is not None for f in ("device_budget_bytes", "device_weights_percent",
                                                         "cache_budget_cap_bytes", "prefetch_layers",
                                                         "small_param_persist_threshold"))
    if not cfg.enabled and has_knob:
        raise ValueError("runtime.weight_streaming.enabled=false but streaming knobs are set; set "
                         "runtime.weight_streaming.enabled=true or clear streaming knobs")
    if cfg.device_weights_percent is not None and not (0.0 <= cfg.device_weights_percent <= 1.0):
        raise ValueError(f"runtime.weight_streaming.device_weights_percent must be in [0.0, 1.0], got {cfg.device_weights_percent}")


def effective_device_budget_bytes(entries: Iterable[Entry], cfg: WeightStreamingConfig) -> Optional[int]:
    """loader.rs:342-368: the explicit byte budget, capped by the percentage of the checkpoint's tensor bytes."""
    budget = cfg.device_budget_bytes
    if cfg.device_weights_percent is not None:
        total = sum(e.byte_len for e in entries)
        p = float(np.float32(cfg.device_weights_percent))   # the reference holds an f32 and widens it
        pb = total if p >= 1.0 else (0 if p <= 0.0 else int(np.floor(float(total) * p)))
        budget = pb if budget is None else min(budget, pb)
    return budget


def effective_cache_budget_bytes(entries: Iterable[Entry], cfg: WeightStreamingConfig) -> Optional[int]:
    """loader.rs:422-434: the smaller of the device budget and the cache cap, whichever are set."""
    device = effective_device_budget_bytes(list(entries), cfg)
    cap = cfg.cache_budget_cap_bytes
    if device is not None and cap is not None:
        return min(device, cap)
    return device if device is not None else cap


def block_layer_index(name: str) -> Optional[int]:
    """loader.rs:416-420: `blocks.<i>.rest` -> i."""
    if not name.startswith("blocks."):
        return None
    head, sep, _ = name[len("blocks."):].partition(".")
    if not sep or not head.isdigit() or not head.isascii():
        return None
    return int(head)


def base_id_of(entry: Entry) -> int:
    """The stored base id, or (stored 0 = "derive from the name", docs/formats.md) the reference's `base_param_id` of the
    name: the first 16 bytes of blake3(name), little endian (params.rs:29-37)."""
    if entry.base_id:
        return entry.base_id
    from .models import base_param_id
    return base_param_id(entry.name)


def prefetch_block_base_ids(entries: Iterable[Entry], prefetch_layers: Optional[int]) -> Set[int]:
    """loader.rs:392-414."""
    if not prefetch_layers:
        return set()
    out = set()
    for e in entries:
        layer = block_layer_index(e.name)
        if layer is not None and layer < prefetch_layers:
            out.add(base_id_of(e))
    return out


@dataclass
class SourceCacheConfig:
    """loader.rs:24-30."""

    enabled: bool = False
    budget_bytes: Optional[int] = None
    small_param_persist_threshold: Optional[int] = None
    prefetch_base_ids: Set[int] = field(default_factory=set)


def source_cache_config(entries: List[Entry], cfg: WeightStreamingConfig) -> SourceCacheConfig:
    """loader.rs:370-390."""
    if not cfg.enabled:
        return SourceCacheConfig()
    budget = effective_cache_budget_bytes(entries, cfg)
    pre = prefetch_block_base_ids(entries, cfg.prefetch_layers)
    return SourceCacheConfig(enabled=budget is not None or cfg.small_param_persist_threshold is not None or bool(pre),
                             budget_bytes=budget, small_param_persist_threshold=cfg.small_param_persist_threshold,
                             prefetch_base_ids=pre)


class ParamHandleCache:
    """loader.rs:32-161: handles by base id with a byte budget, pinning and least-recently-used eviction."""

    @dataclass
    class _Cached:
        handle: object
        bytes: int
        pinned: bool
        last_used: int

    def __init__(self, cfg: SourceCacheConfig):
        self.cfg = cfg
        self.entries: Dict[int, ParamHandleCache._Cached] = {}
        self.cached_bytes = 0
        self.usage_tick = 0

    def _next_tick(self) -> int:
        self.usage_tick = (self.usage_tick + 1) & 0xFFFFFFFFFFFFFFFF
        return self.usage_tick

    def get(self, base_id: int):
        if not self.cfg.enabled:
            return None
        tick = self._next_tick()
        e = self.entries.get(base_id)
        if e is None:
            return None
        e.last_used = tick
        return e.handle

    def should_cache(self, base_id: int, nbytes: int) -> bool:
        if base_id in self.cfg.prefetch_base_ids:
            return True
        if self.cfg.budget_bytes is not None:
            return True
        t = self.cfg.small_param_persist_threshold
        return t is not None and nbytes <= t

    def is_pinned(self, base_id: int, nbytes: int) -> bool:
        t = self.cfg.small_param_persist_threshold
        return base_id in self.cfg.prefetch_base_ids or (t is not None and nbytes <= t)

    def _evict_one_unpinned(self) -> bool:
        victims = [(e.last_used, bid) for bid, e in self.entries.items() if not e.pinned]
        if not victims:
            return False
        _, bid = min(victims)
        self.cached_bytes -= self.entries.pop(bid).bytes
        return True

    def insert(self, base_id: int, nbytes: int, handle) -> None:
        if not self.cfg.enabled or not self.should_cache(base_id, nbytes):
            return
        pinned = self.is_pinned(base_id, nbytes)
        touch = self._next_tick()
        existing = self.entries.get(base_id)
        if existing is not None:
            existing.handle = handle
            existing.last_used = touch
            return
        budget = self.cfg.budget_bytes
        if budget is not None:
            if nbytes > budget:
                return
            pinned_bytes = sum(e.bytes for e in self.entries.values() if e.pinned)
            if pinned_bytes + nbytes > budget:
                return
            while self.cached_bytes + nbytes > budget:
                if not self._evict_one_unpinned():
                    return
        self.cached_bytes += nbytes
        self.entries[base_id] = ParamHandleCache._Cached(handle, nbytes, pinned, self._next_tick())


class CheckpointParamSource:
    """loader.rs:19-236: `load(base_id)` = the cached handle, or the tensor's bytes out of the open checkpoint,
    materialised on the backend (in `dtype_of(name)`, the model's storage dtype for that tensor)."""

    def __init__(self, backend, checkpoint: Checkpoint, cache_cfg: SourceCacheConfig, dtype_of: Callable[[str], str]):
        self.backend = backend
        self.checkpoint = checkpoint
        self.dtype_of = dtype_of
        self.by_id: Dict[int, Entry] = {base_id_of(e): e for e in checkpoint.entries}
        self.cache = ParamHandleCache(cache_cfg)
        self.loads = 0
        if cache_cfg.enabled and cache_cfg.prefetch_base_ids:   # loader.rs:186-215
            for e in checkpoint.entries:
                bid = base_id_of(e)
                if bid in cache_cfg.prefetch_base_ids and self.cache.get(bid) is None:
                    self.cache.insert(bid, e.byte_len, self._materialize(e))

    def _materialize(self, e: Entry):
        arr = self.checkpoint.array(e.name)
        want = self.dtype_of(e.name)
        if e.dtype == "F32":
            host = np.asarray(arr, np.float32)
        elif e.dtype == "Bf16":
            host = bf16_bits_to_f32(np.asarray(arr))
        else:
            raise CheckpointError(f"tensor `{e.name}`: dtype {e.dtype} cannot feed a model parameter")
        data = host.astype("<f4").tobytes() if want == "F32" else f32_to_bf16_bits(host).astype("<u2").tobytes()
        self.loads += 1
        return self.backend.materialize(TensorSpec(want, e.dims), data)

    def load(self, base_id: int):
        h = self.cache.get(base_id)
        if h is not None:
            return h
        e = self.by_id.get(base_id)
        if e is None:
            raise CheckpointError(f"no tensor with base id {base_id:#034x} in the checkpoint")
        h = self._materialize(e)
        self.cache.insert(base_id, e.byte_len, h)
        return h


def load_model(backend, path: str, dtype: Optional[str] = None, **model_kwargs):
    """loader.rs:238-306: open the checkpoint, read its kind, config and `runtime.weight_streaming`, build the model.
    Not streaming: every parameter is loaded once into the backend's memo.  Streaming: the model resolves every
    parameter through the source at each forward.  The checkpoint stays open for the life of the model."""
    from . import models
    ck = Checkpoint(path)
    try:
        ws = WeightStreamingConfig.from_runtime(ck.runtime)
        validate_weight_streaming_config(ws)
        if ck.kind == "gpt":
            model = models.Gpt(models.Gpt.config_from_json(ck.config), backend, dtype or "F32")
        elif ck.kind == "ministral":
            model = models.Ministral(models.Ministral.config_from_json(ck.config), backend, dtype or "Bf16", **model_kwargs)
        else:
            raise CheckpointError(f"unsupported model kind '{ck.kind}'")
        expected = model.expected_params()
        for name, dims in expected.items():
            e = ck.entry(name)   # "missing tensor '<name>' in checkpoint"
            if tuple(e.dims) != tuple(dims):
                raise CheckpointError(f"tensor `{name}` has shape {list(e.dims)}, the model expects {list(dims)}")
        source = CheckpointParamSource(backend, ck, source_cache_config(ck.entries, ws), model.param_dtype)
        model.bind_param_source(source, {n: base_id_of(ck.entry(n)) for n in expected},
                                {n: TensorSpec(model.param_dtype(n), expected[n]) for n in expected}, lazy=ws.enabled)
        return model
    except Exception:
        ck.close()
        raise
