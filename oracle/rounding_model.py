"""TEST INFRASTRUCTURE ONLY -- a Ministral-shaped decoder written out in numpy with explicit rounding points.

Only tests/ may import this module, and only as a checker.  The shipped backend never calls it.

What it is for.  The PTIR oracle (oracle/ptir_oracle.py) executes a program instruction by instruction; run on an F32
program it is the reference's arithmetic (crates/gpt-rs-backend-ref-cpu/src/cpu.rs), and the distance of a bf16 device
result from it mixes two things: the roundings a bf16 pipeline must make, and any error of a kernel.  This module
separates them.  It computes the same model (crates/gpt-rs/src/model/ministral.rs:166-201, 613-766; functionals
ops/functional/{normalization.rs:183-217, rotary.rs:430-536, attention.rs:338-541, 657-779, activation.rs:141-162}) in
f32, and with `rounding=True` rounds to bf16 (round to nearest even) at exactly the places where the mixed-precision
program (bf16 weights and matmul operands, f32 residual stream, f32 norms, f32 logits) stores a bf16 tensor when every
functional is ONE kernel:

    normalised row        bf16((x * rsqrt(mean(x^2) + eps)) * gamma)           input of every projection
    packed q | k | v      bf16 of the f32 dot products
    rotated q, k          bf16(a * cos -/+ b * sin), cos / sin tables in bf16
    probabilities         bf16(exp(s - max)) before P.V (a matrix-core operand) in the many-row kernel;
                          f32 in the one-row kernel over the cache; the normaliser sums the unrounded ones
    context row           bf16(sum(p v) / sum(p))
    SwiGLU output         bf16((g / (1 + exp(-g))) * u) with g, u the f32 dot products
    nothing else          residual adds, out / down projections and logits stay f32

so that |device - this model| holds only summation order, exp / rsqrt ulps and the rare rounding tie that falls the
other way, while |this model - F32 oracle| is the rounding the pipeline cannot avoid.

Parity pinning: with `rounding=False` the model must reproduce the PTIR oracle's F32 run of the same weights
(tests/test_rounding_model.py: tiny and mid-size configurations, prefill and decode over the cache, 1e-5 relative);
with `rounding=True` on a one-layer configuration it must reproduce the PTIR oracle's bf16 run of a program written
with those rounding points as explicit Cast instructions (same test file).  The reference executes no bf16
(cpu.rs:21-25), so the rounding semantics themselves are this build's: "parity unpinned" by the reference.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np


def bf16_round(x: np.ndarray) -> np.ndarray:
    """f32 -> nearest bf16 (ties to even) -> f32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = ((u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)) << np.uint32(16)
    out = r.view(np.float32).reshape(x.shape)
    nan = np.isnan(x)
    return np.where(nan, np.float32(np.nan), out) if nan.any() else out


class MinistralRoundingModel:
    """`params`: name -> float32 array (checkpoint names of model/ministral.rs:376-422; matrices [in, out]);
    `rope(start, count) -> (cos, sin)` float32 tables [count, rotary_dim / 2] (the caller's, so that both sides read the
    same tables); `cfg` carries embed_dim, num_heads, num_kv_heads, head_dim, ffn_dim, rotary_dim, eps, num_layers."""

    def __init__(self, cfg, params: Dict[str, np.ndarray], rope: Callable[[int, int], Tuple[np.ndarray, np.ndarray]],
                 rounding: bool = True, bf16_scale: Optional[bool] = None, sites: Optional[Sequence[str]] = None):
        self.cfg, self.p, self.rope, self.rounding = cfg, params, rope, rounding
        # `sites`: round only at the named places ("norm", "qkv", "rope", "p", "ctx", "act"; None: all of them), to
        # see what each rounding point contributes
        self.sites = None if sites is None else set(sites)
        # the attention scale 1 / sqrt(head_dim) reaches a program as a scalar literal of the tensor's dtype
        # (crates/gpt-rs/src/ops/ptir/graph.rs:2278-2298): a bf16 value in a bf16 attention (default with rounding on)
        self.bf16_scale = rounding if bf16_scale is None else bf16_scale
        self.trace: Optional[Dict[str, np.ndarray]] = None   # set to a dict to collect every layer's intermediate tensors

    def _t(self, name: str, value: np.ndarray) -> np.ndarray:
        if self.trace is not None:
            self.trace[name] = value
        return value

    def _r(self, x, site: Optional[str] = None):
        on = self.rounding and (self.sites is None or site is None or site in self.sites)
        return bf16_round(x) if on else np.asarray(x, np.float32)

    def _norm(self, x: np.ndarray, gamma: np.ndarray) -> np.ndarray:
        n = x.shape[-1]
        ms = (x * x).sum(axis=-1, keepdims=True, dtype=np.float32) * np.float32(1.0 / n)
        inv = (np.float32(1.0) / np.sqrt(ms + np.float32(self.cfg.eps), dtype=np.float32)).astype(np.float32)
        return self._r((x * inv) * gamma.astype(np.float32), "norm")

    def _rope_rows(self, x: np.ndarray, heads: int, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
        """x [T, heads * Dh] -> rotate-half on the first rotary_dim of every head."""
        c = self.cfg
        T, dh, half = x.shape[0], c.head_dim, c.rotary_dim // 2
        xh = x.reshape(T, heads, dh).astype(np.float32)
        cs, sn = self._r(cos, "rope")[:, None, :], self._r(sin, "rope")[:, None, :]
        a, b = xh[:, :, :half], xh[:, :, half:2 * half]
        out = xh.copy()
        out[:, :, :half] = self._r(a * cs - b * sn, "rope")
        out[:, :, half:2 * half] = self._r(b * cs + a * sn, "rope")
        return out.reshape(T, heads * dh)

    def _attend(self, q: np.ndarray, K: np.ndarray, V: np.ndarray, first_pos: int, round_p: bool) -> np.ndarray:
        """q [T, Hq * Dh] at positions first_pos .., K / V [Hkv, L, Dh] holding positions 0 .. L - 1: causal GQA."""
        c = self.cfg
        T, hq, hkv, dh = q.shape[0], c.num_heads, c.num_kv_heads, c.head_dim
        g = hq // hkv
        L = K.shape[1]
        scale = np.float32(1.0) / np.sqrt(np.float32(dh))
        if self.bf16_scale:
            scale = bf16_round(np.array([scale], np.float32))[0]
        qh = q.reshape(T, hq, dh)
        ctx = np.empty((T, hq, dh), np.float32)
        mass = np.empty((T, hq, dh), np.float32) if self.trace is not None else None
        keys = np.arange(L)[None, :]
        visible = keys <= (first_pos + np.arange(T))[:, None]
        for h in range(hq):
            s = (qh[:, h, :] @ K[h // g].T).astype(np.float32) * scale
            s = np.where(visible, s, np.float32(-np.inf))
            e = np.exp(s - s.max(axis=1, keepdims=True), dtype=np.float32)
            l = e.sum(axis=1, keepdims=True, dtype=np.float32)
            pe = self._r(e, "p") if round_p else e
            ctx[:, h, :] = (pe @ V[h // g]).astype(np.float32) / l
            if mass is not None:
                mass[:, h, :] = (e @ np.abs(V[h // g])).astype(np.float32) / l
        if mass is not None:
            # sum_j p_j |v_j| per output: what a relative error of the probabilities is relative TO (the sum itself may cancel)
            self.trace["attention_mass"] = mass.reshape(T, hq * dh)
        return self._r(ctx.reshape(T, hq * dh), "ctx")

    def _block(self, i: int, x: np.ndarray, pos0: int, cache: Optional[Tuple[np.ndarray, np.ndarray]]):
        c, p = self.cfg, self.p
        pre = f"blocks.{i}."
        T = x.shape[0]
        hq, hkv, dh = c.num_heads, c.num_kv_heads, c.head_dim
        qp, kp = hq * dh, hkv * dh
        n1 = self._t(pre + "n1", self._norm(x, p[pre + "norm_1.gamma"]))
        qkv = self._t(pre + "qkv", self._r(n1 @ p[pre + "attention.w_qkv"], "qkv"))
        cos, sin = self.rope(pos0, T)
        q = self._rope_rows(qkv[:, :qp], hq, cos, sin)
        k = self._rope_rows(qkv[:, qp:qp + kp], hkv, cos, sin)
        v = qkv[:, qp + kp:]
        self._t(pre + "qkv_rope", np.concatenate([q, k, v], axis=1))
        k_new = k.reshape(T, hkv, dh).transpose(1, 0, 2)
        v_new = v.reshape(T, hkv, dh).transpose(1, 0, 2)
        if cache is None:
            K, V = k_new, v_new
        else:
            K, V = np.concatenate([cache[0], k_new], axis=1), np.concatenate([cache[1], v_new], axis=1)
        # many rows at once: the probabilities are a bf16 matrix-core operand; one row over the cache: they stay f32
        ctx = self._t(pre + "ctx", self._attend(q, K, V, pos0, round_p=self.rounding and T > 1))
        h = self._t(pre + "h", (ctx @ p[pre + "attention.w_out"]).astype(np.float32) + x)
        n2 = self._t(pre + "n2", self._norm(h, p[pre + "norm_2.gamma"]))
        gate = (n2 @ p[pre + "feed_forward.w_gate"]).astype(np.float32)
        up = (n2 @ p[pre + "feed_forward.w_up"]).astype(np.float32)
        act = self._t(pre + "act", self._r((gate / (np.float32(1.0) + np.exp(gate * np.float32(-1.0), dtype=np.float32))) * up, "act"))
        out = self._t(pre + "out", (act @ p[pre + "feed_forward.w_down"]).astype(np.float32) + h)
        return out, (np.ascontiguousarray(K), np.ascontiguousarray(V))

    def forward(self, tokens: Sequence[int], pos0: int, caches: List[Optional[Tuple[np.ndarray, np.ndarray]]],
                last_row_only: bool = True) -> np.ndarray:
        """Logits [rows, V] (rows = 1 with last_row_only) for `tokens` at positions pos0 ..; `caches` (one slot per
        layer, None before the first call) is updated in place with K, V [Hkv, positions so far, Dh]."""
        x = self.p["tok_embeddings.weight"][np.asarray(tokens, np.int64)].astype(np.float32)
        for i in range(self.cfg.num_layers):
            x, caches[i] = self._block(i, x, pos0, caches[i])
        if last_row_only:
            x = x[-1:]
        return (self._norm(x, self.p["final_norm.gamma"]) @ self.p["lm_head"]).astype(np.float32)
