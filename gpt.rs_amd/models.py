"""GPT-2 and Ministral model drivers and the greedy Generator, generic over a backend.

Host-side mirror of crates/gpt-rs/src/model/{gpt,ministral}.rs, nn/layers/*.rs and
inference/{generate,sampler}.rs: each forward call captures the whole model into ONE
PTIR program (as the reference's lazy GraphArena does, ops/graph/arena.rs:340-375),
caches it by shape (plan cache, ops/graph/plan.rs:20-29) and hands it to
`backend.run_program`.  Weights are program inputs fed from the backend's parameter
memo; per-step scalars (token ids, positions, update_starts, query_start, RoPE rows)
are tiny uploads, exactly the reference's calling convention.

`backend` is any object with the PortableBackend surface (spec.rs:1287-1349):
materialize / to_literal / run_program / param_resolver / sample_decode_token.
"""
from __future__ import annotations

import itertools
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import functional as F
from .blake3 import blake3
from .ptir import FunctionBuilder, Program, Tensor, TensorSpec, bf16_bits_to_f32, f32_to_bf16_bits


def decode_cache_capacity(required_len: int, max_len: int) -> int:
    """model/gpt.rs:940-943: next power of two, capped at the context length."""
    bucket = 1
    while bucket < max(required_len, 1):
        bucket *= 2
    return min(bucket, max_len)


@dataclass
class DecodeKvCache:
    """ops/functional/attention.rs:100-126: fixed-capacity [Hkv, capacity, Dh] + active len."""

    keys: object
    values: object
    len: int
    capacity: int


def _np_to_bytes(arr: np.ndarray, dtype: str) -> bytes:
    if dtype == "Bf16":
        return f32_to_bf16_bits(np.asarray(arr, np.float32)).astype("<u2").tobytes()
    if dtype == "F32":
        return np.ascontiguousarray(arr, dtype="<f4").tobytes()
    if dtype == "Si32":
        return np.ascontiguousarray(arr, dtype="<i4").tobytes()
    raise ValueError(dtype)


def base_param_id(name: str) -> int:
    """crates/gpt-rs/src/params.rs:29-37: the first 16 bytes of blake3(name) as a little-endian u128."""
    if not name.isascii():
        raise ValueError(f"param name must be ASCII, got '{name}'")
    return int.from_bytes(blake3(name.encode("ascii"))[:16], "little")


def namespace_id(namespace: str) -> int:
    """The u128 a model instance is bound under.  The reference takes it from the model handle that `load_model` hands
    out (runtime/loader.rs: a counter per loaded model); here it is derived from the instance's label the same way a
    base id is derived from a name."""
    return int.from_bytes(blake3(b"gpt-rs:model-namespace:" + namespace.encode())[:16], "little")


def param_id(namespace: str, name: str) -> bytes:
    """Stable 16-byte parameter key, the reference's derivation (crates/gpt-rs/src/params.rs:39-48): the first 16 bytes of
    blake3("gpt-rs:param-key:v1" || namespace u128 LE || base id u128 LE), which read as a little-endian u128 are
    `ParamKey`; the memo of the C ABI is keyed by those 16 bytes."""
    msg = b"gpt-rs:param-key:v1" + namespace_id(namespace).to_bytes(16, "little") + base_param_id(name).to_bytes(16, "little")
    return blake3(msg)[:16]


class _ModelBase:
    """Shared plumbing: parameter registration, program cache, tiny uploads."""

    namespace = "model"

    _instances = itertools.count()

    def __init__(self, backend, dtype: str):
        self.backend = backend
        self.dtype = dtype
        # one memo namespace per model instance (the reference namespaces by model handle)
        self.namespace = f"{type(self).namespace}#{next(_ModelBase._instances)}"
        self.param_names: List[str] = []
        self.param_specs: Dict[str, TensorSpec] = {}
        self._programs: Dict[tuple, Tuple[Program, dict]] = {}
        self._param_handles: Optional[list] = None
        self._source = None                 # loader.CheckpointParamSource of a model opened by loader.load_model
        self._base_ids: Dict[str, int] = {}
        self._lazy = False                  # weight streaming: parameters are resolved through the source at every run
        # programs go through the reference's optimizer pipeline (front_end.py) before the backend sees them; False hands
        # the backend the emitters' instruction stream as it is captured
        self.front_end = True
        # with the front end on: also run the hip backend's own pipeline passes (front_end.hip_backend_pipeline: norms
        # become CustomCalls ahead of the parameter-only fold), the second route through the reference's optimizer
        self.backend_pipeline = False
        self._optimized: Dict[int, tuple] = {}

    # -- parameters ------------------------------------------------------------------
    def param_dtype(self, name: str) -> str:
        """Storage dtype of the parameter `name`."""
        return self.dtype

    def bind_param_source(self, source, base_ids: Dict[str, int], specs: Dict[str, TensorSpec], lazy: bool):
        """runtime/loader.rs:264-297: parameters come from `source` by base id.  Not lazy: each is loaded once and
        stored in the backend's memo under its stable id; lazy (`runtime.weight_streaming.enabled`): nothing is
        loaded here, every run asks the memo and then the source (`DeviceTensor::lazy_param`)."""
        self._source, self._lazy = source, bool(lazy)
        for name, spec in specs.items():
            if name not in self.param_specs:
                self.param_names.append(name)
            self.param_specs[name] = spec
            self._base_ids[name] = base_ids[name]
            if not lazy:
                self.backend.param_resolver().set(param_id(self.namespace, name), source.load(base_ids[name]))
        self._param_handles = None
        self._optimized.clear()

    def set_param(self, name: str, array: np.ndarray, dtype: Optional[str] = None):
        """runtime/loader.rs:234-239: materialize once, store under the stable id."""
        dtype = dtype or self.dtype
        spec = TensorSpec(dtype, array.shape)
        handle = self.backend.materialize(spec, _np_to_bytes(array, dtype))
        self.backend.param_resolver().set(param_id(self.namespace, name), handle)
        if name not in self.param_specs:
            self.param_names.append(name)
        self.param_specs[name] = spec
        self._param_handles = None
        self._optimized.clear()

    def set_param_bytes(self, name: str, spec: TensorSpec, data: bytes):
        handle = self.backend.materialize(spec, data)
        self.backend.param_resolver().set(param_id(self.namespace, name), handle)
        if name not in self.param_specs:
            self.param_names.append(name)
        self.param_specs[name] = spec
        self._param_handles = None
        self._optimized.clear()

    def set_param_handle(self, name: str, handle):
        """Register a tensor that already lives on the device."""
        self.backend.param_resolver().set(param_id(self.namespace, name), handle)
        if name not in self.param_specs:
            self.param_names.append(name)
        self.param_specs[name] = handle.spec
        self._param_handles = None
        self._optimized.clear()
        self._programs.clear()

    def drop_param(self, name: str):
        """Forget a parameter and release its device memory (the memo keeps a 1-element stand-in)."""
        spec = self.param_specs.pop(name)
        self.param_names.remove(name)
        stub = self.backend.materialize(TensorSpec(spec.dtype, [1]), None)
        self.backend.param_resolver().set(param_id(self.namespace, name), stub)
        self._param_handles = None
        self._optimized.clear()
        self._programs.clear()

    _quant_programs: Dict[tuple, Program] = {}

    def quantize_param(self, name: str, scheme: str):
        """Replace the matrix `name` by `name.q` (codes) and `name.s` (scales), quantised on the device
        (functional.quantize_weight); layers that find `name.q` read the codes directly."""
        spec = self.param_specs[name]
        key = (scheme, spec.dtype, tuple(spec.dims))
        prog = _ModelBase._quant_programs.get(key)
        if prog is None:
            fb = FunctionBuilder("main", spec.dtype)
            q, s = F.quantize_weight(fb.param(spec.dtype, spec.dims), scheme)
            fb.set_results([q, s])
            prog = _ModelBase._quant_programs[key] = Program(fb)
        q, s = self.backend.run_program(prog, [self.param_handle(name)])
        self.drop_param(name)
        self.set_param_handle(name + ".q", q)
        self.set_param_handle(name + ".s", s)

    # -- checkpoints -----------------------------------------------------------------
    def _load_tensors(self, ck, expected: Dict[str, tuple], dtype: Optional[str] = None):
        """Upload every expected tensor from an open checkpoint (checkpoint/loader.rs: by name, shape checked),
        one at a time out of the file mapping; `dtype` overrides the model's storage dtype."""
        from .checkpoint import CheckpointError
        for name, dims in expected.items():
            e = ck.entry(name)
            if tuple(e.dims) != tuple(dims):
                raise CheckpointError(f"tensor `{name}` has shape {list(e.dims)}, the model expects {list(dims)}")
            arr = ck.array(name)
            if e.dtype == "F32":
                host = np.asarray(arr, np.float32)
            elif e.dtype == "Bf16":
                host = bf16_bits_to_f32(np.asarray(arr))
            else:
                raise CheckpointError(f"tensor `{name}`: dtype {e.dtype} cannot feed a model parameter")
            self.set_param(name, host, dtype)

    def save_checkpoint(self, path: str, kind: str, config: Dict[str, object], runtime: Optional[Dict[str, object]] = None):
        """Write the parameters back as a GPTRSCHK v2 file (checkpoint/saver.rs), in their storage dtype."""
        from .checkpoint import write_checkpoint
        tensors, dtypes = {}, {}
        for name in self.param_names:
            spec = self.param_specs[name]
            if spec.dtype not in ("F32", "Bf16"):
                raise ValueError(f"parameter {name} of dtype {spec.dtype} has no checkpoint representation")
            raw = self.backend.to_literal(self.param_handle(name))
            if spec.dtype == "F32":
                tensors[name] = np.frombuffer(raw, "<f4").reshape(spec.dims)
            else:
                tensors[name] = np.frombuffer(raw, "<u2").reshape(spec.dims)
                dtypes[name] = "Bf16"
        write_checkpoint(path, kind, config, tensors, dtypes, runtime=runtime)

    def param_handle(self, name: str):
        h = self.backend.param_resolver().get(param_id(self.namespace, name))
        if h is None and self._source is not None and name in self._base_ids:
            h = self._source.load(self._base_ids[name])
        if h is None:
            raise KeyError(f"parameter {name} not materialized")
        return h

    def _declare_params(self, fb: FunctionBuilder) -> Dict[str, Tensor]:
        return {n: fb.param(self.param_specs[n].dtype, self.param_specs[n].dims) for n in self.param_names}

    def _upload_i32(self, values: Sequence[int]):
        arr = np.asarray(values, dtype=np.int32)
        return self.backend.materialize(TensorSpec("Si32", arr.shape), arr.tobytes())

    def _zeros(self, dims):
        return self.backend.materialize(TensorSpec(self.dtype, dims), None)

    def _run(self, program: Program, args: list, donate: Optional[list] = None):
        if self.front_end:
            return self._run_optimized(program, args, donate)
        if self._lazy:                    # streamed weights: resolved anew for every run, kept only by the source's cache
            params = [self.param_handle(n) for n in self.param_names]
        else:
            if self._param_handles is None:   # Param inputs are fed by stable id (arena.rs:1163-1168)
                self._param_handles = [self.param_handle(n) for n in self.param_names]
            params = self._param_handles
        don = None
        if donate is not None:
            don = list(donate) + [False] * len(params)
        return self.backend.run_program(program, list(args) + params, don)

    def _run_optimized(self, program: Program, args: list, donate: Optional[list] = None):
        """The reference's path from a captured graph to the backend: the program goes through the optimizer once
        (front_end.optimize: canonicalisers, parameter-only folds executed through the backend and stored in its memo
        under derived ids, CSE, DCE; ops/graph/arena.rs:744-922), the optimised program and its input roles are kept
        with the plan, and every run feeds Args positionally and Params by stable id (arena.rs:1116-1170)."""
        from . import front_end as FE
        n_args, names = len(args), self.param_names
        entry = self._optimized.get(program.key)
        if entry is None or entry[2] != tuple(names) or entry[3] != self.backend_pipeline:
            roles = [FE.ARG] * n_args + [FE.PARAM] * len(names)
            stable = [None] * n_args + [int.from_bytes(param_id(self.namespace, n), "little") for n in names]
            hooks = FE.hip_backend_pipeline() if self.backend_pipeline else {}
            opt = FE.optimize(program, roles, stable, self.backend, self.backend.param_resolver(), **hooks)
            entry = self._optimized[program.key] = (opt, {}, tuple(names), self.backend_pipeline)
        opt, held = entry[0], entry[1]
        inputs, don = [], []
        resolver = self.backend.param_resolver()
        for pos, (p, src) in enumerate(zip(opt.inputs, opt.source_index)):
            if p.role == FE.ARG:
                inputs.append(args[src])
                don.append(bool(donate[src]) if donate is not None else False)
                continue
            h = None if self._lazy and src is not None else held.get(pos)
            if h is None:
                if src is not None:
                    h = self.param_handle(names[src - n_args])
                else:
                    h = resolver.get(FE.stable_id_bytes(p.stable_id))
                    if h is None:
                        raise KeyError(f"derived parameter {p.stable_id:#x} is not in the backend's memo")
                held[pos] = h
            inputs.append(h)
            don.append(False)
        return self.backend.run_program(opt.program, inputs, don if donate is not None else None)


def _last_rows(hidden: Tensor, seq: int, batch: int) -> Tensor:
    """Row seq - 1 of each of the `batch` stacked sequences."""
    d = hidden.dims[1]
    rows = [hidden.slice([b * seq + seq - 1, 0], [1, d]) for b in range(batch)]
    return rows[0] if batch == 1 else Tensor.concat(0, rows)


# ================================================================================ GPT-2
@dataclass
class GptConfig:
    """model/gpt.rs GptConfig."""

    vocab_size: int = 50257
    context_length: int = 1024
    embed_dim: int = 768
    num_layers: int = 12
    num_heads: int = 12
    mlp_ratio: int = 4
    eps: float = 1e-5

    def attention_config(self) -> F.AttentionConfig:
        return F.AttentionConfig(self.embed_dim, self.num_heads, self.num_heads, self.embed_dim // self.num_heads)


class Gpt(_ModelBase):
    """model/gpt.rs: learned positions, pre-LN blocks with biases, final LN, lm_head[d,V]."""

    namespace = "gpt"

    def __init__(self, config: GptConfig, backend, dtype: str = "F32"):
        super().__init__(backend, dtype)
        self.config = config
        self.attn = config.attention_config()

    @classmethod
    def random(cls, config: GptConfig, backend, seed: int = 0, dtype: str = "F32", std: float = 0.02) -> "Gpt":
        """Shapes and constant inits of Gpt::random (model/gpt.rs:128-208); the random
        stream is numpy's PCG64, not Rust's StdRng."""
        m = cls(config, backend, dtype)
        rng = np.random.default_rng(seed)
        d, hid = config.embed_dim, config.embed_dim * config.mlp_ratio

        def rn(*shape):
            return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)

        m.set_param("tok_embeddings.weight", rn(config.vocab_size, d))
        m.set_param("pos_embeddings", rn(config.context_length, d))
        for i in range(config.num_layers):
            p = f"blocks.{i}."
            m.set_param(p + "ln_1.gamma", np.ones(d, np.float32))
            m.set_param(p + "ln_1.beta", np.zeros(d, np.float32))
            m.set_param(p + "attention.w_qkv", rn(d, 3 * d))
            m.set_param(p + "attention.b_qkv", np.zeros(3 * d, np.float32))
            m.set_param(p + "attention.w_out", rn(d, d))
            m.set_param(p + "attention.b_out", np.zeros(d, np.float32))
            m.set_param(p + "ln_2.gamma", np.ones(d, np.float32))
            m.set_param(p + "ln_2.beta", np.zeros(d, np.float32))
            m.set_param(p + "feed_forward.w_in", rn(d, hid))
            m.set_param(p + "feed_forward.b_in", np.zeros(hid, np.float32))
            m.set_param(p + "feed_forward.w_out", rn(hid, d))
            m.set_param(p + "feed_forward.b_out", np.zeros(d, np.float32))
        m.set_param("final_ln.gamma", np.ones(d, np.float32))
        m.set_param("final_ln.beta", np.zeros(d, np.float32))
        m.set_param("lm_head", rn(d, config.vocab_size))
        return m

    def expected_params(self) -> Dict[str, tuple]:
        """Names and shapes as Gpt::build_from_params reads them (model/gpt.rs:300-370)."""
        c = self.config
        d, hid = c.embed_dim, c.embed_dim * c.mlp_ratio
        out = {"tok_embeddings.weight": (c.vocab_size, d), "pos_embeddings": (c.context_length, d)}
        for i in range(c.num_layers):
            p = f"blocks.{i}."
            out.update({p + "ln_1.gamma": (d,), p + "ln_1.beta": (d,), p + "attention.w_qkv": (d, 3 * d),
                        p + "attention.b_qkv": (3 * d,), p + "attention.w_out": (d, d), p + "attention.b_out": (d,),
                        p + "ln_2.gamma": (d,), p + "ln_2.beta": (d,), p + "feed_forward.w_in": (d, hid),
                        p + "feed_forward.b_in": (hid,), p + "feed_forward.w_out": (hid, d), p + "feed_forward.b_out": (d,)})
        out.update({"final_ln.gamma": (d,), "final_ln.beta": (d,), "lm_head": (d, c.vocab_size)})
        return out

    @staticmethod
    def config_from_json(c) -> GptConfig:
        """GptConfig's serde form (model/gpt.rs)."""
        return GptConfig(vocab_size=int(c["vocab_size"]), context_length=int(c["context_length"]), embed_dim=int(c["embed_dim"]),
                         num_layers=int(c["num_layers"]), num_heads=int(c["num_heads"]), mlp_ratio=int(c.get("mlp_ratio", 4)))

    @classmethod
    def from_checkpoint(cls, path: str, backend, dtype: str = "F32") -> "Gpt":
        """runtime/loader.rs:19-241 for kind "gpt": config from the file, tensors streamed by name."""
        from .checkpoint import Checkpoint, CheckpointError
        with Checkpoint(path) as ck:
            if ck.kind != "gpt":
                raise CheckpointError(f"checkpoint holds a `{ck.kind}` model, not `gpt`")
            m = cls(cls.config_from_json(ck.config), backend, dtype)
            m._load_tensors(ck, m.expected_params())
        return m

    def checkpoint_config(self) -> Dict[str, object]:
        c = self.config
        return {"vocab_size": c.vocab_size, "context_length": c.context_length, "embed_dim": c.embed_dim,
                "num_layers": c.num_layers, "num_heads": c.num_heads, "mlp_ratio": c.mlp_ratio, "dropout": 0.0}

    @property
    def num_layers(self): return self.config.num_layers
    @property
    def context_length(self): return self.config.context_length

    # -- graph pieces ----------------------------------------------------------------
    def _block_tail(self, P, i, x, attn_ctx):
        p = f"blocks.{i}."
        eps = self.config.eps
        attn_out = F.linear(attn_ctx, P[p + "attention.w_out"], P[p + "attention.b_out"])
        residual = attn_out + x                               # model/gpt.rs:81-97: attn_output.add(x)
        normed2, *_ = F.layer_norm(residual, P[p + "ln_2.gamma"], P[p + "ln_2.beta"], eps)
        hidden = F.linear(normed2, P[p + "feed_forward.w_in"], P[p + "feed_forward.b_in"])
        act = F.gelu(hidden)
        ff = F.linear(act, P[p + "feed_forward.w_out"], P[p + "feed_forward.b_out"])
        return ff + residual

    def _build(self, seq: int, capacity: int, decode: bool, batch: int = 1, last_only: bool = False) -> Tuple[Program, dict]:
        """One program for the whole forward (model/gpt.rs:585-751).  last_only: the head runs on the last row of
        each sequence only (logits [batch, V] instead of [batch * seq, V])."""
        last_only = last_only and seq > 1
        key = (seq, capacity, decode, batch, last_only)
        if key in self._programs:
            return self._programs[key]
        cfg, L = self.config, self.config.num_layers
        hkv, dh = self.attn.num_key_value_heads, self.attn.kv_head_dim
        fb = FunctionBuilder("main", self.dtype)
        rows = seq * batch
        tok = fb.param("Si32", [rows])
        pos = fb.param("Si32", [rows])
        layout = {"args": ["tokens", "positions"]}
        if decode:
            upd = fb.param("Si32", [3])
            qst = fb.param("Si32", [1])
            layout["args"] += ["update_starts", "query_start"]
            caches = [[(fb.param(self.dtype, [hkv, capacity, dh]), fb.param(self.dtype, [hkv, capacity, dh]))
                       for _ in range(L)] for _ in range(batch)]
        else:
            start_zeros = fb.param("Si32", [3])
            layout["args"] += ["start_zeros"]
            bases = [[(fb.param(self.dtype, [hkv, capacity, dh]), fb.param(self.dtype, [hkv, capacity, dh]))
                      for _ in range(L)] for _ in range(batch)]
        layout["n_args"] = len(fb.params)
        P = self._declare_params(fb)

        tok_emb = F.embedding_lookup(P["tok_embeddings.weight"], tok)
        pos_emb = F.embedding_lookup(P["pos_embeddings"], pos)
        hidden = tok_emb + pos_emb
        new_caches = [[None] * L for _ in range(batch)]
        for i in range(L):
            p = f"blocks.{i}."
            normed, *_ = F.layer_norm(hidden, P[p + "ln_1.gamma"], P[p + "ln_1.beta"], cfg.eps)
            qkv = F.linear(normed, P[p + "attention.w_qkv"], P[p + "attention.b_qkv"])
            ctxs = []
            for b in range(batch):
                qkv_b = qkv if batch == 1 else qkv.slice([b * seq, 0], [seq, qkv.dims[1]])
                if decode:
                    ck, cv = caches[b][i]
                    ctx, k2, v2 = F.attention_decode_cache(self.attn, qkv_b, ck, cv, upd, qst)
                else:
                    ctx, k, v = F.attention(self.attn, qkv_b, None)
                    kb, vb = bases[b][i]
                    k2 = F.dynamic_update_slice_into(kb, k, start_zeros)   # model/gpt.rs:712-730
                    v2 = F.dynamic_update_slice_into(vb, v, start_zeros)
                new_caches[b][i] = (k2, v2)
                ctxs.append(ctx)
            ctx_all = ctxs[0] if batch == 1 else Tensor.concat(0, ctxs)
            hidden = self._block_tail(P, i, hidden, ctx_all)
        if last_only:
            hidden = _last_rows(hidden, seq, batch)
        normalized, *_ = F.layer_norm(hidden, P["final_ln.gamma"], P["final_ln.beta"], cfg.eps)
        logits = normalized.matmul(P["lm_head"])
        results = []
        for b in range(batch):
            for i in range(L):
                results += list(new_caches[b][i])
        results.append(logits)
        fb.set_results(results)
        prog = Program(fb)
        self._programs[key] = (prog, layout)
        return prog, layout

    # -- forward -----------------------------------------------------------------------
    def forward_with_decode_cache(self, tokens: Sequence[int], position_offset: int,
                                  caches: List[Optional[DecodeKvCache]], fixed_capacity: Optional[int] = None,
                                  last_logits_only: bool = False):
        """model/gpt.rs:585-751.  Returns the logits handle [T, V]; `caches` is updated in place.
        last_logits_only: the final norm and the lm_head run on the last position only and the handle is [1, V] (the
        reference computes every row, gpt.rs:735-736, and its generation loop reads the last)."""
        return self.forward_batch([list(tokens)], position_offset, [caches], fixed_capacity, last_logits_only=last_logits_only)

    def forward_decode_device_token(self, token_handle, position_offset: int, caches: List[Optional[DecodeKvCache]],
                                    fixed_capacity: Optional[int] = None):
        """One decode step whose token id is already on the device (a si32[1] handle, e.g.
        backend.decode_token_tensor()): the same program as forward_with_decode_cache([token], ...), without the
        host having to know the token yet.  An id outside the vocabulary raises at the next synchronising call."""
        return self.forward_batch([[None]], position_offset, [caches], fixed_capacity, token_handle=token_handle)

    def forward_batch(self, token_rows: List[List[int]], position_offset: int,
                      caches: List[List[Optional[DecodeKvCache]]], fixed_capacity: Optional[int] = None,
                      token_handle=None, last_logits_only: bool = False):
        """Independent sequences sharing the weights: row-stacked hidden states, one M=B*T
        GEMM per linear, per-sequence attention.  The reference has no batch dimension
        (ops/functional/attention.rs:189-203); with one row this is exactly its path."""
        cfg = self.config
        batch, seq = len(token_rows), len(token_rows[0])
        if seq == 0:
            raise ValueError("token sequence must contain at least one element")
        if any(len(r) != seq for r in token_rows):
            raise ValueError("all sequences of a batch must have equal length")
        total = position_offset + seq
        if total > cfg.context_length:
            raise ValueError(f"token sequence length {total} exceeds model context length {cfg.context_length}")
        if token_handle is None:
            for row in token_rows:
                for t in row:
                    if not 0 <= t < cfg.vocab_size:
                        raise ValueError(f"token index {t} out of range")
        elif seq != 1:
            raise ValueError("device tokens feed one step (one token per sequence)")
        if any(len(c) != cfg.num_layers for c in caches):
            raise ValueError(f"expected {cfg.num_layers} cache slots (one per layer)")
        if fixed_capacity is not None:
            if not 0 < fixed_capacity <= cfg.context_length or fixed_capacity < total:
                raise ValueError(f"decode cache capacity {fixed_capacity} invalid for sequence length {total}")
            capacity = fixed_capacity
        else:
            capacity = decode_cache_capacity(total, cfg.context_length)
        have = caches[0][0] is not None
        if have and caches[0][0].capacity < capacity:
            self._grow_caches(caches, capacity)
        if have and (seq != 1):
            raise ValueError("decode with an existing cache supports one token per sequence")
        L = cfg.num_layers
        prog, _ = self._build(seq, capacity, have, batch, last_logits_only)
        poss = [position_offset + j for _ in range(batch) for j in range(seq)]
        tok_arg = token_handle if token_handle is not None else self._upload_i32([t for row in token_rows for t in row])
        args = [tok_arg, self._upload_i32(poss)]
        if have:
            for c in caches:
                for slot in c:
                    if slot.len != position_offset:
                        raise ValueError(f"decode cache length {slot.len} must match position offset {position_offset}")
            args += [self._upload_i32([0, position_offset, 0]), self._upload_i32([position_offset])]
            kv = [h for c in caches for slot in c for h in (slot.keys, slot.values)]
        else:
            hkv, dh = self.attn.num_key_value_heads, self.attn.kv_head_dim
            args.append(self._upload_i32([0, 0, 0]))
            kv = [self._zeros([hkv, capacity, dh]) for _ in range(2 * L * batch)]
        donate = [False] * len(args) + [True] * len(kv)       # old caches are dropped (gpt.rs:738-747)
        outs = self._run(prog, args + kv, donate)
        it = iter(outs[:-1])
        for b in range(batch):
            for i in range(L):
                k, v = next(it), next(it)
                caches[b][i] = DecodeKvCache(k, v, total, capacity)
        return outs[-1]

    def _grow_caches(self, caches, capacity: int):
        """model/gpt.rs:626-657: copy each layer's cache into a larger zero buffer."""
        hkv, dh = self.attn.num_key_value_heads, self.attn.kv_head_dim
        old_cap = caches[0][0].capacity
        key = ("grow", old_cap, capacity)
        if key not in self._programs:
            fb = FunctionBuilder("main", self.dtype)
            base = fb.param(self.dtype, [hkv, capacity, dh])
            old = fb.param(self.dtype, [hkv, old_cap, dh])
            st = fb.param("Si32", [3])
            fb.set_results([F.dynamic_update_slice_into(base, old, st)])
            self._programs[key] = (Program(fb), {})
        prog = self._programs[key][0]
        st = self._upload_i32([0, 0, 0])
        for c in caches:
            for i, slot in enumerate(c):
                k = self.backend.run_program(prog, [self._zeros([hkv, capacity, dh]), slot.keys, st], [True, False, False])[0]
                v = self.backend.run_program(prog, [self._zeros([hkv, capacity, dh]), slot.values, st], [True, False, False])[0]
                c[i] = DecodeKvCache(k, v, slot.len, capacity)


# ================================================================================ Ministral
@dataclass
class MinistralConfig:
    """model/ministral.rs MinistralConfig."""

    vocab_size: int = 131072
    context_length: int = 4096
    embed_dim: int = 3072
    num_layers: int = 26
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    ffn_dim: int = 9216
    rotary_dim: int = 128
    rope_theta: float = 1e6
    eps: float = 1e-5
    rope_scaling: Optional[object] = None   # None | ("linear", factor) | functional.YarnScaling (rotary.rs:20-43)

    def attention_config(self) -> F.AttentionConfig:
        return F.AttentionConfig(self.embed_dim, self.num_heads, self.num_kv_heads, self.head_dim)


class Ministral(_ModelBase):
    """model/ministral.rs: RMSNorm, packed-QKV RoPE from host tables, GQA, SwiGLU, no biases,
    untied lm_head."""

    namespace = "ministral"

    def __init__(self, config: MinistralConfig, backend, dtype: str = "Bf16", residual_dtype: Optional[str] = None):
        """`residual_dtype="F32"` on a bf16 model keeps the residual stream, the norms and the logits in f32: the
        embedding rows are cast up, RMSNorm runs on f32 (what the reference's rms_norm requires,
        ops/functional/normalization.rs:183-217) and is cast to bf16 for the projection that follows, the two
        projections that feed a residual add (attention out, feed-forward down) and the lm_head leave their f32
        accumulator as f32 (DotGeneralSpec.out_dtype, spec.rs:354-361; docs/backend.md:104-115).  Matmul operands,
        RoPE, attention and the KV cache stay bf16.  Norm gains are then stored as f32."""
        super().__init__(backend, dtype)
        self.config = config
        self.attn = config.attention_config()
        self.rope = F.RopeConfig(config.rotary_dim, config.rope_theta, config.rope_scaling)
        if residual_dtype is not None and residual_dtype not in ("F32",):
            raise ValueError("residual_dtype must be None or 'F32'")
        self.residual_dtype = residual_dtype if (residual_dtype and residual_dtype != dtype) else None

    @property
    def norm_dtype(self) -> str:
        return self.residual_dtype or self.dtype

    @classmethod
    def random(cls, config: MinistralConfig, backend, seed: int = 0, dtype: str = "Bf16", std: float = 0.02,
               bf16_values: bool = False, quant: Optional[str] = None, residual_dtype: Optional[str] = None):
        """Shapes and constant inits of Ministral::random (model/ministral.rs:262-330).  Every
        tensor draws from its own numpy stream SeedSequence([seed, index]), so the weights do not
        depend on the order or the number of worker threads that generate them.  `bf16_values`
        rounds the draws to bf16-representable values whatever the storage dtype, so an f32
        model can be given exactly the weights of a bf16 one.  `quant` ("w8" / "w4g128") quantises
        every linear weight (projections, feed-forward, lm_head) as it arrives on the device."""
        from concurrent.futures import ThreadPoolExecutor
        m = cls(config, backend, dtype, residual_dtype)
        d, a = config.embed_dim, config.attention_config()
        plan = [("tok_embeddings.weight", (config.vocab_size, d), "randn")]
        for i in range(config.num_layers):
            p = f"blocks.{i}."
            plan += [(p + "norm_1.gamma", (d,), "ones"),
                     (p + "attention.w_qkv", (d, a.total_projection_dim), "randn"),
                     (p + "attention.w_out", (a.query_projection_dim, d), "randn"),
                     (p + "norm_2.gamma", (d,), "ones"),
                     (p + "feed_forward.w_gate", (d, config.ffn_dim), "randn"),
                     (p + "feed_forward.w_up", (d, config.ffn_dim), "randn"),
                     (p + "feed_forward.w_down", (config.ffn_dim, d), "randn")]
        plan += [("final_norm.gamma", (d,), "ones"), ("lm_head", (d, config.vocab_size), "randn")]

        def make(idx):
            name, shape, kind = plan[idx]
            if kind == "ones":
                return name, shape, m.norm_dtype, _np_to_bytes(np.ones(shape, np.float32), m.norm_dtype)
            else:
                arr = np.random.default_rng(np.random.SeedSequence([seed, idx])).standard_normal(shape, dtype=np.float32)
                arr *= np.float32(std)
                if bf16_values and dtype != "Bf16":
                    arr = bf16_bits_to_f32(f32_to_bf16_bits(arr))
            return name, shape, dtype, _np_to_bytes(arr, dtype)

        workers = max(1, min(16, (os.cpu_count() or 1)))
        with ThreadPoolExecutor(max_workers=workers) as ex:
            # bounded look-ahead keeps at most a few tensors of host memory in flight
            pending, nxt = [], 0
            while nxt < len(plan) or pending:
                while nxt < len(plan) and len(pending) < 2 * workers:
                    pending.append(ex.submit(make, nxt))
                    nxt += 1
                name, shape, dt, data = pending.pop(0).result()
                m.set_param_bytes(name, TensorSpec(dt, shape), data)
                if quant and len(shape) == 2 and name != "tok_embeddings.weight":
                    m.quantize_param(name, quant)
        return m

    def expected_params(self) -> Dict[str, tuple]:
        """Names and shapes as Ministral::build_from_params reads them (model/ministral.rs:360-425)."""
        c, a = self.config, self.attn
        d = c.embed_dim
        out = {"tok_embeddings.weight": (c.vocab_size, d)}
        for i in range(c.num_layers):
            p = f"blocks.{i}."
            out.update({p + "norm_1.gamma": (d,), p + "attention.w_qkv": (d, a.total_projection_dim),
                        p + "attention.w_out": (a.query_projection_dim, d), p + "norm_2.gamma": (d,),
                        p + "feed_forward.w_gate": (d, c.ffn_dim), p + "feed_forward.w_up": (d, c.ffn_dim),
                        p + "feed_forward.w_down": (c.ffn_dim, d)})
        out.update({"final_norm.gamma": (d,), "lm_head": (d, c.vocab_size)})
        return out

    @staticmethod
    def _scaling_from_json(js) -> Optional[object]:
        """RopeScaling's serde form: {"kind": "none" | "linear" | "yarn", ...} (ops/functional/rotary.rs:20-43)."""
        if not js or js.get("kind", "none") == "none":
            return None
        if js["kind"] == "linear":
            return ("linear", float(js["factor"]))
        if js["kind"] == "yarn":
            return F.YarnScaling(factor=float(js["factor"]), original_max_position_embeddings=js.get("original_max_position_embeddings"),
                                 mscale=js.get("mscale"), mscale_all_dim=js.get("mscale_all_dim"), beta_fast=js.get("beta_fast"),
                                 beta_slow=js.get("beta_slow"), truncate=bool(js.get("truncate", True)))
        raise ValueError(f"unknown rope scaling kind {js['kind']!r}")

    @classmethod
    def config_from_json(cls, c) -> MinistralConfig:
        """MinistralConfig's serde form (model/ministral.rs:13-30)."""
        from .checkpoint import CheckpointError
        head_dim = int(c["head_dim"]) if c.get("head_dim") else int(c["embed_dim"]) // int(c["num_heads"])
        if c.get("kv_head_dim") and int(c["kv_head_dim"]) != head_dim:
            raise CheckpointError("kv_head_dim different from head_dim is not supported")
        return MinistralConfig(vocab_size=int(c["vocab_size"]), context_length=int(c["context_length"]), embed_dim=int(c["embed_dim"]),
                               num_layers=int(c["num_layers"]), num_heads=int(c["num_heads"]), num_kv_heads=int(c["num_kv_heads"]),
                               head_dim=head_dim, ffn_dim=int(c["mlp_hidden_dim"]), rotary_dim=int(c["rotary_dim"]),
                               rope_theta=float(c["rope_theta"]), eps=float(c["rms_norm_eps"]),
                               rope_scaling=cls._scaling_from_json(c.get("rope_scaling")))

    def param_dtype(self, name: str) -> str:
        return self.norm_dtype if name.endswith(".gamma") else self.dtype

    @classmethod
    def from_checkpoint(cls, path: str, backend, dtype: str = "Bf16", quant: Optional[str] = None,
                        residual_dtype: Optional[str] = None) -> "Ministral":
        """runtime/loader.rs:19-241 for kind "ministral" (MinistralConfig, model/ministral.rs:13-30)."""
        from .checkpoint import Checkpoint, CheckpointError
        with Checkpoint(path) as ck:
            if ck.kind != "ministral":
                raise CheckpointError(f"checkpoint holds a `{ck.kind}` model, not `ministral`")
            m = cls(cls.config_from_json(ck.config), backend, dtype, residual_dtype)
            for name, dims in m.expected_params().items():
                m._load_tensors(ck, {name: dims}, m.norm_dtype if name.endswith(".gamma") else None)
                if quant and len(dims) == 2 and name != "tok_embeddings.weight":
                    m.quantize_param(name, quant)
        return m

    def checkpoint_config(self) -> Dict[str, object]:
        c = self.config
        out = {"vocab_size": c.vocab_size, "context_length": c.context_length, "embed_dim": c.embed_dim, "num_layers": c.num_layers,
               "num_heads": c.num_heads, "num_kv_heads": c.num_kv_heads, "head_dim": c.head_dim, "mlp_hidden_dim": c.ffn_dim,
               "rms_norm_eps": c.eps, "rope_theta": c.rope_theta, "rotary_dim": c.rotary_dim}
        sc = c.rope_scaling
        if sc is None:
            out["rope_scaling"] = {"kind": "none"}
        elif isinstance(sc, F.YarnScaling):
            out["rope_scaling"] = {k: v for k, v in dict(kind="yarn", factor=sc.factor, mscale=sc.mscale, mscale_all_dim=sc.mscale_all_dim,
                                                         beta_fast=sc.beta_fast, beta_slow=sc.beta_slow,
                                                         original_max_position_embeddings=sc.original_max_position_embeddings,
                                                         truncate=sc.truncate).items() if v is not None}
        else:
            out["rope_scaling"] = {"kind": "linear", "factor": sc[1]}
        return out

    QUANTIZABLE = ("attention.w_qkv", "attention.w_out", "feed_forward.w_gate", "feed_forward.w_up",
                   "feed_forward.w_down", "lm_head")

    def quantize(self, scheme: str):
        """Weight-only quantisation of every linear weight of a loaded model, in place."""
        for name in list(self.param_names):
            if name.endswith(self.QUANTIZABLE) and len(self.param_specs[name].dims) == 2:
                self.quantize_param(name, scheme)
        return self

    @property
    def num_layers(self): return self.config.num_layers
    @property
    def context_length(self): return self.config.context_length

    def _linear(self, P, name: str, x: Tensor, out_dtype: Optional[str] = None) -> Tensor:
        """nn/layers/linear.rs:50-71 without bias; quantised weights are read as codes and scales."""
        if name + ".q" in P:
            return F.linear_quantized(x, P[name + ".q"], P[name + ".s"], out_dtype=out_dtype)
        return F.linear(x, P[name], out_dtype=out_dtype)

    def _norm(self, x: Tensor, gamma: Tensor) -> Tensor:
        """RMSNorm in the residual stream's dtype, handed on in the matmul dtype."""
        out, *_ = F.rms_norm(x, gamma, self.config.eps)
        return out.cast(self.dtype) if self.residual_dtype else out

    def _build(self, seq: int, capacity: int, decode: bool, batch: int = 1, last_only: bool = False) -> Tuple[Program, dict]:
        last_only = last_only and seq > 1
        key = (seq, capacity, decode, batch, last_only)
        if key in self._programs:
            return self._programs[key]
        cfg, L = self.config, self.config.num_layers
        hkv, dh = self.attn.num_key_value_heads, self.attn.kv_head_dim
        half = cfg.rotary_dim // 2
        fb = FunctionBuilder("main", self.dtype)
        rows = seq * batch
        tok = fb.param("Si32", [rows])
        cos = fb.param(self.dtype, [seq, half])
        sin = fb.param(self.dtype, [seq, half])
        layout = {"args": ["tokens", "cos", "sin"]}
        if decode:
            upd = fb.param("Si32", [3])
            qst = fb.param("Si32", [1])
            caches = [[(fb.param(self.dtype, [hkv, capacity, dh]), fb.param(self.dtype, [hkv, capacity, dh]))
                       for _ in range(L)] for _ in range(batch)]
        else:
            start_zeros = fb.param("Si32", [3])
            bases = [[(fb.param(self.dtype, [hkv, capacity, dh]), fb.param(self.dtype, [hkv, capacity, dh]))
                      for _ in range(L)] for _ in range(batch)]
        layout["n_args"] = len(fb.params)
        P = self._declare_params(fb)

        rdt = self.residual_dtype   # None: every tensor in the model dtype
        hidden = F.embedding_lookup(P["tok_embeddings.weight"], tok)
        if rdt:
            hidden = hidden.cast(rdt)
        new_caches = [[None] * L for _ in range(batch)]
        for i in range(L):
            p = f"blocks.{i}."
            normed = self._norm(hidden, P[p + "norm_1.gamma"])
            qkv = self._linear(P, p + "attention.w_qkv", normed)
            ctxs = []
            for b in range(batch):
                qkv_b = qkv if batch == 1 else qkv.slice([b * seq, 0], [seq, qkv.dims[1]])
                qkv_b = F.apply_rope_qkv_packed(self.attn, qkv_b, cos, sin)   # ministral.rs:166-201
                if decode:
                    ck, cv = caches[b][i]
                    ctx, k2, v2 = F.attention_decode_cache(self.attn, qkv_b, ck, cv, upd, qst)
                else:
                    ctx, k, v = F.attention(self.attn, qkv_b, None)
                    kb, vb = bases[b][i]
                    k2 = F.dynamic_update_slice_into(kb, k, start_zeros)
                    v2 = F.dynamic_update_slice_into(vb, v, start_zeros)
                new_caches[b][i] = (k2, v2)
                ctxs.append(ctx)
            ctx_all = ctxs[0] if batch == 1 else Tensor.concat(0, ctxs)
            attn_out = self._linear(P, p + "attention.w_out", ctx_all, rdt)
            residual = attn_out + hidden
            normed2 = self._norm(residual, P[p + "norm_2.gamma"])
            gate = self._linear(P, p + "feed_forward.w_gate", normed2)     # nn/layers/feed_forward.rs GatedFeedForward
            up = self._linear(P, p + "feed_forward.w_up", normed2)
            act = F.swiglu(gate, up)
            ff = self._linear(P, p + "feed_forward.w_down", act, rdt)
            hidden = ff + residual
        if last_only:
            hidden = _last_rows(hidden, seq, batch)
        normalized = self._norm(hidden, P["final_norm.gamma"])
        logits = self._linear(P, "lm_head", normalized, rdt)
        results = []
        for b in range(batch):
            for i in range(L):
                results += list(new_caches[b][i])
        results.append(logits)
        fb.set_results(results)
        prog = Program(fb)
        self._programs[key] = (prog, layout)
        return prog, layout

    def forward_with_decode_cache(self, tokens, position_offset, caches, fixed_capacity=None, last_logits_only=False):
        """model/ministral.rs:613-766.  last_logits_only: see Gpt.forward_with_decode_cache."""
        return self.forward_batch([list(tokens)], position_offset, [caches], fixed_capacity, last_logits_only=last_logits_only)

    def forward_decode_device_token(self, token_handle, position_offset, caches, fixed_capacity=None):
        """See Gpt.forward_decode_device_token."""
        return self.forward_batch([[None]], position_offset, [caches], fixed_capacity, token_handle=token_handle)

    def forward_batch(self, token_rows, position_offset, caches, fixed_capacity=None, token_handle=None, last_logits_only=False):
        cfg = self.config
        batch, seq = len(token_rows), len(token_rows[0])
        if token_handle is not None and seq != 1:
            raise ValueError("device tokens feed one step (one token per sequence)")
        if seq == 0:
            raise ValueError("token sequence must contain at least one element")
        if any(len(r) != seq for r in token_rows):
            raise ValueError("all sequences of a batch must have equal length")
        total = position_offset + seq
        if total > cfg.context_length:
            raise ValueError(f"token sequence length {total} exceeds model context length {cfg.context_length}")
        if fixed_capacity is not None:
            if not 0 < fixed_capacity <= cfg.context_length or fixed_capacity < total:
                raise ValueError(f"decode cache capacity {fixed_capacity} invalid for sequence length {total}")
            capacity = fixed_capacity
        else:
            capacity = decode_cache_capacity(total, cfg.context_length)
        have = caches[0][0] is not None
        if have and caches[0][0].capacity < capacity:
            Gpt._grow_caches(self, caches, capacity)
        if have and seq != 1:
            raise ValueError("decode with an existing cache supports one token per sequence")
        L = cfg.num_layers
        prog, _ = self._build(seq, capacity, have, batch, last_logits_only)
        cos, sin = F.rotary_cos_sin_cache_slice(position_offset, seq, self.rope)   # ministral.rs:253-261
        half = cfg.rotary_dim // 2
        tok_arg = token_handle if token_handle is not None else self._upload_i32([t for row in token_rows for t in row])
        args = [tok_arg,
                self.backend.materialize(TensorSpec(self.dtype, [seq, half]), _np_to_bytes(cos, self.dtype)),
                self.backend.materialize(TensorSpec(self.dtype, [seq, half]), _np_to_bytes(sin, self.dtype))]
        if have:
            args += [self._upload_i32([0, position_offset, 0]), self._upload_i32([position_offset])]
            kv = [h for c in caches for slot in c for h in (slot.keys, slot.values)]
        else:
            hkv, dh = self.attn.num_key_value_heads, self.attn.kv_head_dim
            args.append(self._upload_i32([0, 0, 0]))
            kv = [self._zeros([hkv, capacity, dh]) for _ in range(2 * L * batch)]
        donate = [False] * len(args) + [True] * len(kv)
        outs = self._run(prog, args + kv, donate)
        it = iter(outs[:-1])
        for b in range(batch):
            for i in range(L):
                k, v = next(it), next(it)
                caches[b][i] = DecodeKvCache(k, v, total, capacity)
        return outs[-1]


# ================================================================================ BatchGenerator
class BatchGenerator:
    """Greedy generation for several independent sequences of equal prompt length at once (the reference decodes one
    sequence per model call; its batch is a host-side loop): rows stacked through `forward_batch`, one attention launch
    per layer for all of them.  On a backend with sample_decode_rows_begin / _wait the loop is pipelined like
    `Generator`: the tokens of step t stay on the device as the input of step t + 1, which is queued before the host
    has seen them; elsewhere the rows are arg-maxed on the host (sampler.rs:96-103, last maximum... first index wins
    here as on the device).  The context window does not slide: generation stops at the context length."""

    def __init__(self, model, prompts: Sequence[Sequence[int]], kv_cache_capacity: Optional[int] = None):
        if len(prompts) == 0 or len(prompts[0]) == 0:
            raise ValueError("prompts must be non-empty")
        if any(len(p) != len(prompts[0]) for p in prompts):
            raise ValueError("all prompts of a batch must have equal length")
        self.model = model
        self.batch = len(prompts)
        self.tokens = [list(p) for p in prompts]
        self.capacity = kv_cache_capacity
        self.caches = [[None] * model.num_layers for _ in prompts]
        self.pipelined = hasattr(model.backend, "sample_decode_rows_begin")
        self.logits = model.forward_batch(self.tokens, 0, self.caches, self.capacity, last_logits_only=True)
        self.processed_len = len(prompts[0])

    def step(self) -> List[int]:
        """Samples one token per sequence and runs the forward that consumes them."""
        be, B = self.model.backend, self.batch
        if self.processed_len >= self.model.context_length:
            raise ValueError("context length reached")
        if self.pipelined:
            ticket = be.sample_decode_rows_begin(self.logits)
            self.logits = self.model.forward_batch([[None]] * B, self.processed_len, self.caches, self.capacity,
                                                   token_handle=be.decode_rows_tensor(B))
            nxt = be.sample_decode_rows_wait(ticket, B)
        else:
            rows = be.to_numpy(self.logits)
            nxt = [int(np.argmax(rows[b])) for b in range(B)]
            self.logits = self.model.forward_batch([[t] for t in nxt], self.processed_len, self.caches, self.capacity)
        self.processed_len += 1
        for b in range(B):
            self.tokens[b].append(nxt[b])
        return nxt

    def generate(self, max_new_tokens: int) -> List[List[int]]:
        out = [[] for _ in range(self.batch)]
        for _ in range(max_new_tokens):
            for b, t in enumerate(self.step()):
                out[b].append(t)
        return out


# ================================================================================ host sampler
class Sampler:
    """The reference's host sampler (crates/gpt-rs/src/inference/sampler.rs:7-104): what a generation loop falls back to
    when the backend answers `Ok(None)` to sample_decode_token, and the only path for top-k (sampler.rs:74-76: a request
    with top_k is never offered to the backend).

    `sample(row, rng)`: temperature <= 0 -> arg-max (the LAST of equal maxima, as `Iterator::max_by` returns it).  Otherwise
    logits / temperature in f32; with top_k = k < len every value below the k-th largest becomes -inf (values equal to it
    stay); softmax with the maximum taken out; a sum that is not finite or not positive falls back to arg-max; the token is
    drawn from the cumulative f32 weights as `WeightedIndex` does (a uniform draw in [0, total), first cumulative weight
    above it).  The reference draws from `thread_rng()`, which no one can replay: `rng` is a numpy Generator here, so the
    distribution is the reference's and the stream is this implementation's own."""

    def __init__(self, temperature: float, top_k: Optional[int] = None):
        self.temperature = float(temperature)
        self.top_k = None if top_k is None else max(int(top_k), 1)   # with_top_k: k.max(1)

    @staticmethod
    def argmax(values: np.ndarray) -> int:
        v = np.asarray(values, np.float32).reshape(-1)
        if v.size == 0:
            return 0
        return int(v.size - 1 - np.argmax(v[::-1]))

    def adjusted(self, row: np.ndarray) -> np.ndarray:
        """logits / temperature with everything below the k-th largest value at -inf (sampler.rs:34-50)."""
        adj = (np.asarray(row, np.float32).reshape(-1) / np.float32(self.temperature)).astype(np.float32)
        k = self.top_k
        if k is not None and 0 < k < adj.size:
            kth = np.partition(adj, adj.size - k)[adj.size - k]
            adj = np.where(adj < kth, np.float32(-np.inf), adj).astype(np.float32)
        return adj

    def probabilities(self, row: np.ndarray) -> Optional[np.ndarray]:
        """The f32 weights the draw is made from; None where the reference falls back to arg-max."""
        adj = self.adjusted(row)
        with np.errstate(over="ignore", invalid="ignore"):
            probs = np.exp(adj - np.max(adj), dtype=np.float32)
            total = np.cumsum(probs, dtype=np.float32)[-1]   # the f32 running sum, in order, of `iter().sum()`
        if not np.isfinite(total) or total <= 0.0:
            return None
        return (probs * (np.float32(1.0) / total)).astype(np.float32)

    def sample(self, row: np.ndarray, rng: np.random.Generator) -> int:
        row = np.asarray(row, np.float32).reshape(-1)
        if row.size == 0:
            raise ValueError("cannot sample from empty logits")
        if self.temperature <= 0.0:
            return self.argmax(row)
        probs = self.probabilities(row)
        if probs is None or not np.all(np.isfinite(probs)):
            return self.argmax(row)
        cum = np.cumsum(probs, dtype=np.float32)
        total = cum[-1]
        if not total > 0.0:
            return self.argmax(row)
        # WeightedIndex draws in [0, total): the f32 rounding of the draw must not reach `total`, or the last index would
        # be picked even where its weight is zero (a token that top-k masked)
        x = min(np.float32(rng.uniform(0.0, float(total))), np.nextafter(total, np.float32(0.0)))
        return int(min(np.searchsorted(cum, x, side="right"), row.size - 1))

    def supports_backend_decode_sampling(self) -> bool:
        return self.top_k is None

    def decode_sample_request(self, rng: np.random.Generator) -> Optional[dict]:
        """sampler.rs:78-93: None with top-k; greedy; or the temperature with a uniform draw in [eps, 1 - eps)."""
        if not self.supports_backend_decode_sampling():
            return None
        if self.temperature <= 0.0:
            return {"temperature": 0.0, "top_k": None, "random_u": None}
        eps = float(np.finfo(np.float32).eps)
        return {"temperature": self.temperature, "top_k": None, "random_u": float(np.float32(rng.uniform(eps, 1.0 - eps)))}


# ================================================================================ Generator
class Generator:
    """Generation loop, greedy by default (crates/gpt-rs/src/inference/generate.rs:37-203).

    With `device_sampling` the token comes from backend.sample_decode_token (spec.rs:1333-1348)
    and only 8 bytes cross PCIe per step; otherwise, where the backend declines (`Ok(None)`), and always with `top_k`
    (sampler.rs:74-76), the last logits row is read back and the host `Sampler` draws the token.

    `pipelined` (default: on when the backend offers sample_decode_token_begin / _wait and sampling is on the
    device): a step queues the sampling of token t, then the forward of step t + 1 fed by the device copy of that
    token, and only then waits for token t, so the device never idles for the host round trip.  Same tokens as
    the unpipelined loop; an error of step t + 1's launch surfaces one step later.
    """

    def __init__(self, model, prompt: Sequence[int], kv_cache_capacity: Optional[int] = None,
                 device_sampling: bool = True, temperature: float = 0.0, seed: int = 0,
                 pipelined: Optional[bool] = None, last_logits_only: bool = True, top_k: Optional[int] = None):
        if len(prompt) == 0:
            raise ValueError("prompt must be non-empty")
        self.sampler = Sampler(temperature, top_k)
        if not self.sampler.supports_backend_decode_sampling():
            if pipelined:
                raise ValueError("pipelined generation needs device sampling: top-k is sampled on the host")
            device_sampling = False
        self.model = model
        self.tokens = list(prompt)
        self.capacity = kv_cache_capacity
        self.device_sampling = device_sampling
        # temperature > 0: the backend samples from softmax(logits / temperature) given a uniform draw per
        # step (DecodeSampleRequest.random_u, spec.rs:1270-1284; sampler.rs:83-93 draws it in (eps, 1 - eps))
        self.temperature = float(temperature)
        # the loop only ever samples from the last row: prefill runs the head on that row alone (`self.logits` is then
        # [1, V] after a prefill as after a decode step); False keeps every row as the reference's forward does
        self.last_logits_only = bool(last_logits_only)
        self._rng = np.random.default_rng(seed)
        can_pipeline = device_sampling and hasattr(model.backend, "sample_decode_token_begin") and \
            hasattr(model, "forward_decode_device_token")
        if pipelined and not can_pipeline:
            raise ValueError("pipelined generation needs device sampling and a backend with sample_decode_token_begin")
        self.pipelined = can_pipeline if pipelined is None else bool(pipelined)
        self.caches: List[Optional[DecodeKvCache]] = [None] * model.num_layers
        self.window_start = max(0, len(self.tokens) - model.context_length)
        context = self.tokens[self.window_start:]
        self.logits = self._prefill(context)
        self.processed_len = len(context)

    def _sample(self) -> int:
        be = self.model.backend
        if self.device_sampling:
            req = self.sampler.decode_sample_request(self._rng)
            if req is not None:
                state = self._rng.bit_generator.state
                tok = be.sample_decode_token(self.logits, temperature=req["temperature"], random_u=req["random_u"])
                if tok is not None:
                    return tok
                self._rng.bit_generator.state = state   # Ok(None): the host sampler draws instead
        row = be.to_numpy(self.logits)
        return self.sampler.sample(row[-1] if row.ndim == 2 else row, self._rng)

    def _prefill(self, context):
        if self.last_logits_only:
            return self.model.forward_with_decode_cache(context, 0, self.caches, self.capacity, last_logits_only=True)
        return self.model.forward_with_decode_cache(context, 0, self.caches, self.capacity)

    def _draw_u(self) -> float:
        eps = float(np.finfo(np.float32).eps)
        return float(np.float32(self._rng.uniform(eps, 1.0 - eps)))

    def _step_pipelined(self) -> Optional[int]:
        """Queue sampling + next forward, then wait for the token.  None: the backend declined (nothing queued)."""
        be = self.model.backend
        if self.temperature > 0.0:
            state = self._rng.bit_generator.state
            ticket = be.sample_decode_token_begin(self.logits, temperature=self.temperature, random_u=self._draw_u())
            if ticket is None:
                self._rng.bit_generator.state = state   # the unpipelined path draws again
                return None
        else:
            ticket = be.sample_decode_token_begin(self.logits, temperature=0.0)
            if ticket is None:
                return None
        self.logits = self.model.forward_decode_device_token(be.decode_token_tensor(), self.processed_len, self.caches,
                                                             self.capacity)
        self.processed_len += 1
        nxt = be.sample_decode_token_wait(ticket)
        self.tokens.append(nxt)
        return nxt

    def step(self) -> int:
        if self.pipelined and self.processed_len < self.model.context_length:
            nxt = self._step_pipelined()
            if nxt is not None:
                return nxt
        nxt = self._sample()
        self.tokens.append(nxt)
        if self.processed_len >= self.model.context_length:
            # generate.rs:127-134: slide the window and rebuild the caches
            self.caches = [None] * self.model.num_layers
            self.window_start = len(self.tokens) - self.model.context_length
            context = self.tokens[self.window_start:]
            self.logits = self._prefill(context)
            self.processed_len = len(context)
        else:
            self.logits = self.model.forward_with_decode_cache([nxt], self.processed_len, self.caches, self.capacity)
            self.processed_len += 1
        return nxt

    def step_final(self) -> int:
        nxt = self._sample()
        self.tokens.append(nxt)
        return nxt

    def generate(self, max_new_tokens: int) -> List[int]:
        out = []
        for i in range(max_new_tokens):
            out.append(self.step() if i + 1 < max_new_tokens else self.step_final())
        return out
